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

// Plain grid-stride copy of 16-byte vectors: the known-size kernel that calibrates HBM traffic counters.
__global__ __launch_bounds__(256) void calibration_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x; k < n16; k += stride) dst[k] = src[k];
}

int launch_calibration_copy(hipStream_t stream, void* dst, const void* src, size_t bytes) {
  hipLaunchKernelGGL(calibration_copy_kernel, dim3(4096), dim3(256), 0, stream, (const uint4*)src, (uint4*)dst, bytes >> 4);
  return (int)hipGetLastError();
}

// Read-only probe of the memory system: `workgroups` workgroups of eight waves (96 KiB of LDS each, so one per CU), every
// wave streaming its own contiguous share of the buffer with 16-byte loads, DEPTH instructions (KiB) in flight.
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
template <int DEPTH>
__global__ __launch_bounds__(512) void read_probe_kernel(const probe_u32x4* __restrict__ src, size_t kib_per_wave, uint32_t* __restrict__ sink) {
  __shared__ char occupy[98304];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const probe_u32x4* p = src + ((size_t)blockIdx.x * 8 + wave) * kib_per_wave * 64 + lane;
  probe_u32x4 acc = {0u, 0u, 0u, 0u};
  for (size_t c = 0; c + DEPTH <= kib_per_wave; c += DEPTH) {
    probe_u32x4 v[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) v[d] = __builtin_nontemporal_load(p + (c + d) * 64);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) acc ^= v[d];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[0] = occupy[lane];  // keeps the loads and the LDS alive
}

// Returns the bytes the launch reads (0: bad arguments): bytes / (8 workgroups) rounded down to whole rounds of loads.
size_t launch_read_probe(hipStream_t stream, const void* src, size_t bytes, int workgroups, int kib_in_flight_per_wave,
                         uint32_t* sink) {
  if (workgroups <= 0) return 0;
  size_t per = bytes / ((size_t)workgroups * 8) / 1024;
  per -= per % (size_t)(kib_in_flight_per_wave > 0 ? kib_in_flight_per_wave : 1);
  if (per == 0) return 0;
#define RPA_PROBE(D) hipLaunchKernelGGL(read_probe_kernel<D>, dim3(workgroups), dim3(512), 0, stream, (const probe_u32x4*)src, per, sink)
  switch (kib_in_flight_per_wave) {
    case 2: RPA_PROBE(2); break;
    case 4: RPA_PROBE(4); break;
    case 8: RPA_PROBE(8); break;
    case 16: RPA_PROBE(16); break;
    case 32: RPA_PROBE(32); break;
    default: return 0;
  }
#undef RPA_PROBE
  return hipGetLastError() == hipSuccess ? per * 1024 * 8 * (size_t)workgroups : 0;
}

// The same reader over pages: the buffer is cut into chunks of `chunk_kib` KiB, a workgroup visits its chunks in a
// scattered order (a multiplicative permutation of the chunk numbers, as a block table of a long-lived pool would hand
// them out), DEPTH KiB per wave in flight, i.e. DEPTH / (chunk_kib / 8) chunks per workgroup.  SPLIT says how the eight
// waves share a chunk: 0 contiguous eighths; 1 and 2 the decode kernel's own split -- the chunk is rows of 4 KiB (a
// token's keys and values of eight heads) and wave w reads bytes [512 w, 512 w + 512) of every row, two rows per
// instruction -- with non-temporal (1) or ordinary (2) loads.
template <int DEPTH, int SPLIT>
__global__ __launch_bounds__(512) void read_probe_paged_kernel(const probe_u32x4* __restrict__ src, uint32_t chunk_mask, uint32_t chunks_per_wg,
                                                               uint32_t kib_per_wave_chunk, uint32_t* __restrict__ sink) {
  __shared__ char occupy[98304];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t per = kib_per_wave_chunk;          // KiB of a chunk one wave reads (DEPTH is a multiple of it)
  const uint32_t group = DEPTH / per;               // chunks in flight per workgroup
  probe_u32x4 acc = {0u, 0u, 0u, 0u};
  for (uint32_t c = 0; c + group <= chunks_per_wg; c += group) {
    probe_u32x4 v[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const uint32_t step = c + (uint32_t)d / per;                                               // which of the workgroup's chunks
      const uint32_t chunk = ((blockIdx.x * chunks_per_wg + step) * 0x9E3779B1u) & chunk_mask;  // where it lies
      if constexpr (SPLIT == 0) {
        const probe_u32x4* p = src + ((size_t)chunk * 8 + wave) * per * 64 + lane;
        v[d] = __builtin_nontemporal_load(p + ((uint32_t)d % per) * 64);
      } else {
        const uint32_t row = 2 * ((uint32_t)d % per) + (lane >> 5);  // of the chunk's 2 per rows
        const probe_u32x4* p = src + (size_t)chunk * 8 * per * 64 + (size_t)row * 256 + wave * 32 + (lane & 31);
        if constexpr (SPLIT == 1) v[d] = __builtin_nontemporal_load(p);
        else v[d] = *p;
      }
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) acc ^= v[d];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[0] = occupy[lane];  // keeps the loads and the LDS alive
}

// Returns the bytes the launch reads (0: bad arguments).  The number of chunks in the buffer is rounded down to a power of
// two (the permutation needs one), each workgroup takes an equal share of them in whole groups.
size_t launch_read_probe_paged(hipStream_t stream, const void* src, size_t bytes, int workgroups, int kib_in_flight_per_wave,
                               int chunk_kib, int split, uint32_t* sink) {
  if (workgroups <= 0 || chunk_kib < 8 || (chunk_kib & 7) || kib_in_flight_per_wave <= 0 || split < 0 || split > 2) return 0;
  const uint32_t per = (uint32_t)chunk_kib / 8;
  if ((uint32_t)kib_in_flight_per_wave % per) return 0;
  size_t n_chunks = bytes / ((size_t)chunk_kib * 1024);
  if (n_chunks == 0) return 0;
  size_t pow2 = 1;
  while (pow2 * 2 <= n_chunks && pow2 < ((size_t)1 << 31)) pow2 *= 2;
  const uint32_t group = (uint32_t)kib_in_flight_per_wave / per;
  uint32_t per_wg = (uint32_t)(pow2 / (size_t)workgroups);
  per_wg -= per_wg % group;
  if (per_wg == 0) return 0;
#define RPA_PROBE_S(D, S)                                                                                                \
  hipLaunchKernelGGL((read_probe_paged_kernel<D, S>), dim3(workgroups), dim3(512), 0, stream, (const probe_u32x4*)src, \
                     (uint32_t)(pow2 - 1), per_wg, per, sink)
#define RPA_PROBE(D)                \
  if (split == 0) RPA_PROBE_S(D, 0); \
  else if (split == 1) RPA_PROBE_S(D, 1); \
  else RPA_PROBE_S(D, 2)
  switch (kib_in_flight_per_wave) {
    case 2: RPA_PROBE(2); break;
    case 4: RPA_PROBE(4); break;
    case 8: RPA_PROBE(8); break;
    case 16: RPA_PROBE(16); break;
    case 32: RPA_PROBE(32); break;
    default: return 0;
  }
#undef RPA_PROBE
#undef RPA_PROBE_S
  return hipGetLastError() == hipSuccess ? (size_t)per_wg * (size_t)chunk_kib * 1024 * (size_t)workgroups : 0;
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
