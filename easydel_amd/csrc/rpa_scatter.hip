// Page scatter kernels: bit-exact copies of new K/V token rows into the paged cache.
#include "rpa_common.h"

namespace rpa {

// Copy `bytes` from src to dst with the whole block; 16-byte vectors when both are aligned.
__device__ __forceinline__ void block_copy(char* dst, const char* src, int64_t bytes) {
  const bool aligned = ((((uintptr_t)dst) | ((uintptr_t)src) | (uintptr_t)bytes) & 15) == 0;
  if (aligned) {
    const int64_t n = bytes >> 4;
    for (int64_t k = threadIdx.x; k < n; k += blockDim.x) ((uint4*)dst)[k] = ((const uint4*)src)[k];
  } else {
    for (int64_t k = threadIdx.x; k < bytes; k += blockDim.x) dst[k] = src[k];
  }
}

// Slice form.  One block per slice column.  A column's packed-token offset is the sum of the
// effective lengths of the columns before it (inactive and non-local columns count as zero),
// which the block recomputes with a strided sum: N is at most a few thousand.
__global__ __launch_bounds__(256) void scatter_slices_kernel(const char* __restrict__ new_kv,
                                                             const int32_t* __restrict__ si,
                                                             const int32_t* __restrict__ num_slices,
                                                             char* __restrict__ pages, int T, int N,
                                                             int64_t num_positions, int page_size,
                                                             int64_t row_bytes, int shard) {
  const int c = blockIdx.x;
  const int n_valid = num_slices[0];
  if (c >= n_valid) return;
  int64_t local_pages = num_positions / page_size;
  if (local_pages < 1) local_pages = 1;
  const int64_t page_base = (int64_t)shard * local_pages;

  auto floordiv = [](int64_t a, int64_t b) { int64_t q = a / b; return (a % b != 0 && ((a < 0) != (b < 0))) ? q - 1 : q; };
  auto eff_len = [&](int col) -> int {
    if (col >= n_valid) return 0;
    const int64_t lp = floordiv(si[col], page_size) - page_base;
    if (lp < 0 || lp >= local_pages) return 0;
    const int ln = si[2 * N + col];
    return ln > 0 ? ln : 0;
  };

  __shared__ int red[256];
  int partial = 0;
  for (int col = threadIdx.x; col < c; col += blockDim.x) partial += eff_len(col);
  red[threadIdx.x] = partial;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
    __syncthreads();
  }
  const int packed0 = red[0];
  const int ln = eff_len(c);
  if (ln == 0) return;

  const int64_t g = si[c];
  const int64_t gp = floordiv(g, page_size);
  const int64_t dst0 = (gp - page_base) * page_size + (g - gp * page_size);
  const int64_t src0 = si[N + c];
  for (int off = 0; off < ln; ++off) {
    if (packed0 + off >= T) break;  // beyond the packed prefix the reference can address
    const int64_t src = src0 + off;
    int64_t dst = dst0 + off;
    if (src < 0 || src >= T) continue;
    if (dst < 0) dst += num_positions;
    if (dst < 0 || dst >= num_positions) continue;
    block_copy(pages + dst * row_bytes, new_kv + src * row_bytes, row_bytes);
  }
}

// Ragged form.  One block per query token: find its sequence, then its slot in the sequence's pages.
__global__ __launch_bounds__(256) void scatter_ragged_kernel(const char* __restrict__ key,
                                                             const char* __restrict__ value,
                                                             char* __restrict__ pages,
                                                             const int32_t* __restrict__ context_lens,
                                                             const int32_t* __restrict__ block_tables,
                                                             const int32_t* __restrict__ qsl,
                                                             const int32_t* __restrict__ num_seqs, int S, int M, int P,
                                                             int page_size, int Hkv, int head_bytes, int row_bytes,
                                                             int64_t token_stride, int64_t page_stride) {
  // interleaved pages: V of a head one stored row (row_bytes >= head_bytes) behind its K, heads two rows apart
  scatter_token(key, value, pages, pages + row_bytes, context_lens, block_tables, qsl, min(num_seqs[0], S), M, P, page_size, Hkv,
                head_bytes, 2 * (int64_t)row_bytes, token_stride, page_stride, blockIdx.x, threadIdx.x, blockDim.x,
                row_bytes - head_bytes);
}

// ---- quantising ragged write ---------------------------------------------------------------------------
// Four scaled values -> four 8-bit codes in one dword: clamp to the code range, round to nearest even.
template <int KVT>
__device__ __forceinline__ uint32_t quant4(float a, float b, float c, float d) {
  if constexpr (KVT == RPA_FP8_E4M3) {
    const float q = 448.f;
    a = fminf(fmaxf(a, -q), q); b = fminf(fmaxf(b, -q), q); c = fminf(fmaxf(c, -q), q); d = fminf(fmaxf(d, -q), q);
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
    return (uint32_t)w;
  } else {
    const float q = 127.f;
    const int ia = (int)rintf(fminf(fmaxf(a, -q), q)), ib = (int)rintf(fminf(fmaxf(b, -q), q));
    const int ic = (int)rintf(fminf(fmaxf(c, -q), q)), id = (int)rintf(fminf(fmaxf(d, -q), q));
    return (uint32_t)(ia & 0xff) | ((uint32_t)(ib & 0xff) << 8) | ((uint32_t)(ic & 0xff) << 16) | ((uint32_t)(id & 0xff) << 24);
  }
}

template <int KVT>
__device__ __forceinline__ void decode4_codes(uint32_t w, float* f) {
  if constexpr (KVT == RPA_FP8_E4M3) {
    auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    f[0] = lo[0]; f[1] = lo[1]; f[2] = hi[0]; f[3] = hi[1];
  } else {
    f[0] = (float)(int8_t)(w & 0xff); f[1] = (float)(int8_t)((w >> 8) & 0xff);
    f[2] = (float)(int8_t)((w >> 16) & 0xff); f[3] = (float)(int8_t)(w >> 24);
  }
}

template <int SRC>
__device__ __forceinline__ void load4_src(const void* base, int64_t idx, float* f) {  // idx: element index, multiple of 4
  if constexpr (SRC == RPA_F32) {
    const float4 v = *(const float4*)((const float*)base + idx);
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
  } else {
    const uint2 v = *(const uint2*)((const uint16_t*)base + idx);
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  }
}

// One wave per (query token, combined head); only the wave of the first new token a sequence writes to a page
// works, and it handles all of that page's new tokens for its head:
//   old scale (0 if the page starts with these tokens) -> new scale = max(old, amax / qmax), 1 if that is 0
//   -> tokens already in the page re-coded if the scale grew -> new tokens coded -> scale stored.
// All arithmetic in float32, in this order, so that the codes can be checked bit for bit.
template <int SRC, int KVT>
__global__ __launch_bounds__(64) void scatter_ragged_quant_kernel(const void* __restrict__ key, const void* __restrict__ value,
                                                                  unsigned char* __restrict__ pages, float* __restrict__ scales,
                                                                  const int32_t* __restrict__ context_lens,
                                                                  const int32_t* __restrict__ block_tables,
                                                                  const int32_t* __restrict__ qsl,
                                                                  const int32_t* __restrict__ num_seqs, int S, int M, int P,
                                                                  int page_size, int Hkv, int D, int C, int Dp) {
  const int t = blockIdx.x, c = blockIdx.y, lane = threadIdx.x;
  const int n_live = min(num_seqs[0], S);  // never more than the rows the metadata arrays hold
  if (n_live <= 0 || t < qsl[0] || t >= qsl[n_live]) return;
  const int i = find_seq_wave(qsl, n_live, t);
  const int q0 = qsl[i], q_len = qsl[i + 1] - q0;
  const int ctx = context_lens[i];
  const int pos = ctx - q_len + (t - q0);
  if (pos < 0) return;
  const int first_pos = max(ctx - q_len, 0);
  if (pos != first_pos && pos % page_size != 0) return;  // another token's wave covers this one
  const int j = pos / page_size;
  if (j >= M) return;
  const int page = block_tables[(int64_t)i * M + j];
  if (page < 0 || page >= P) return;
  const int first = pos - j * page_size;
  const int n = min(ctx, (j + 1) * page_size) - pos;
  const float qmax = KVT == RPA_FP8_E4M3 ? 448.f : 127.f;
  const int D4 = D >> 2;
  const void* src = (c & 1) ? value : key;
  const int64_t src0 = ((int64_t)t * Hkv + (c >> 1)) * D;  // element index of the first new token's head row
  const int64_t src_row = (int64_t)Hkv * D;
  unsigned char* dst = pages + ((int64_t)page * page_size * C + c) * Dp;  // token row r of this head: dst + r*C*Dp
  const int64_t dst_row = (int64_t)C * Dp;  // stored rows are Dp >= D codes wide; the padding is written as zero codes

  float amax = 0.f;
  for (int idx = lane; idx < n * D4; idx += 64) {
    const int r = idx / D4, c4 = idx - r * D4;
    float f[4];
    load4_src<SRC>(src, src0 + r * src_row + c4 * 4, f);
    amax = fmaxf(amax, fmaxf(fmaxf(fabsf(f[0]), fabsf(f[1])), fmaxf(fabsf(f[2]), fabsf(f[3]))));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
  const float old_scale = first == 0 ? 0.f : scales[(int64_t)page * C + c];
  float new_scale = fmaxf(old_scale, amax / qmax);
  if (new_scale == 0.f) new_scale = 1.f;

  if (new_scale > old_scale && first > 0) {
    for (int idx = lane; idx < first * D4; idx += 64) {
      const int r = idx / D4, c4 = idx - r * D4;
      uint32_t* w = (uint32_t*)(dst + r * dst_row + c4 * 4);
      float f[4];
      decode4_codes<KVT>(*w, f);
      *w = quant4<KVT>((f[0] * old_scale) / new_scale, (f[1] * old_scale) / new_scale, (f[2] * old_scale) / new_scale,
                       (f[3] * old_scale) / new_scale);
    }
  }
  for (int idx = lane; idx < n * D4; idx += 64) {
    const int r = idx / D4, c4 = idx - r * D4;
    float f[4];
    load4_src<SRC>(src, src0 + r * src_row + c4 * 4, f);
    *(uint32_t*)(dst + (first + r) * dst_row + c4 * 4) = quant4<KVT>(f[0] / new_scale, f[1] / new_scale, f[2] / new_scale, f[3] / new_scale);
  }
  const int P4 = (Dp - D) >> 2;
  for (int idx = lane; idx < n * P4; idx += 64) {
    const int r = idx / P4, c4 = idx - r * P4;
    *(uint32_t*)(dst + (first + r) * dst_row + D + c4 * 4) = 0u;
  }
  if (lane == 0) scales[(int64_t)page * C + c] = new_scale;
}

int launch_scatter_ragged_quant(hipStream_t stream, const void* key, const void* value, void* pages, float* scales,
                                const int32_t* context_lens, const int32_t* block_tables, const int32_t* qsl,
                                const int32_t* num_seqs, int T, int S, int M, int P, int page_size, int Hkv, int D, int C,
                                int Dp, int src_dtype, int kv_dtype) {
  const dim3 grid(T, 2 * Hkv), block(64);
#define RPA_QSCATTER(SRC, KVT)                                                                                        \
  hipLaunchKernelGGL((scatter_ragged_quant_kernel<SRC, KVT>), grid, block, 0, stream, key, value, (unsigned char*)pages, \
                     scales, context_lens, block_tables, qsl, num_seqs, S, M, P, page_size, Hkv, D, C, Dp)
  if (src_dtype == RPA_F32 && kv_dtype == RPA_FP8_E4M3) RPA_QSCATTER(RPA_F32, RPA_FP8_E4M3);
  else if (src_dtype == RPA_F32 && kv_dtype == RPA_INT8) RPA_QSCATTER(RPA_F32, RPA_INT8);
  else if (src_dtype == RPA_BF16 && kv_dtype == RPA_FP8_E4M3) RPA_QSCATTER(RPA_BF16, RPA_FP8_E4M3);
  else if (src_dtype == RPA_BF16 && kv_dtype == RPA_INT8) RPA_QSCATTER(RPA_BF16, RPA_INT8);
  else return (int)hipErrorInvalidValue;
#undef RPA_QSCATTER
  return (int)hipGetLastError();
}

int launch_scatter_slices(hipStream_t stream, const void* new_kv, const int32_t* si, const int32_t* num_slices,
                          void* pages, int T, int N, int64_t num_positions, int page_size, int64_t row_bytes,
                          int shard) {
  hipLaunchKernelGGL(scatter_slices_kernel, dim3(N), dim3(256), 0, stream, (const char*)new_kv, si, num_slices,
                     (char*)pages, T, N, num_positions, page_size, row_bytes, shard);
  return (int)hipGetLastError();
}

int launch_scatter_ragged(hipStream_t stream, const void* key, const void* value, void* pages,
                          const int32_t* context_lens, const int32_t* block_tables, const int32_t* qsl,
                          const int32_t* num_seqs, int T, int S, int M, int P, int page_size, int Hkv, int D, int C,
                          int Dp, int elem_bytes) {
  const int head_bytes = D * elem_bytes, row_bytes = Dp * elem_bytes;
  const int64_t token_stride = (int64_t)C * row_bytes;
  hipLaunchKernelGGL(scatter_ragged_kernel, dim3(T), dim3(256), 0, stream, (const char*)key, (const char*)value,
                     (char*)pages, context_lens, block_tables, qsl, num_seqs, S, M, P, page_size, Hkv, head_bytes, row_bytes,
                     token_stride, token_stride * page_size);
  return (int)hipGetLastError();
}

}  // namespace rpa
