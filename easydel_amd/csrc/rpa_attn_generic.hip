// fp32 VALU ragged paged attention: one wavefront per (query token, query head).
//
// This is the full-precision kernel: fp32 queries (1e-5 parity), head sizes and page sizes the
// MFMA kernels do not cover, and fp32 KV pages.  Keys are processed 64 at a time: each lane
// scores one key (q broadcast from LDS, K row read straight from the page), the block max/sum
// run through cross-lane reductions, then the lanes switch to owning output dims for P.V.
#include "rpa_common.h"

namespace rpa {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

template <int QT, int KVT>
__global__ __launch_bounds__(64) void attn_generic_kernel(AttnParams p) {
  constexpr int kMaxD = 256;
  __shared__ float q_s[kMaxD];
  const int t = blockIdx.x, hq = blockIdx.y, lane = threadIdx.x;
  const int n_live = live_rows(p);
  if (n_live <= 0 || t < p.qsl[0] || t >= p.qsl[n_live]) return;
  const int i = find_seq_wave(p.qsl, n_live, t);
  const SeqPlan sp = seq_plan(p, i);
  if (!sp.live) return;
  if (p.mfma_path && sp.small_rows) return;  // the MFMA decode kernel owns these rows

  const int D = p.Dq;  // q / out row length; the pages are addressed through the strides
  const int h = hq / p.group;
  const int pos = sp.ctx - sp.q_len + (t - sp.q0);
  int k_hi = pos + 1;
  if (k_hi > sp.ctx) k_hi = sp.ctx;
  int k_lo = 0;
  if (p.window > 0 && pos - p.window + 1 > 0) k_lo = pos - p.window + 1;

  for (int d = lane; d < D; d += 64) q_s[d] = load_elem<QT>(p.q, ((int64_t)t * p.Hq + hq) * D + d);
  __syncthreads();

  constexpr int eb = ElemBytes<KVT>::v;
  const char* k_pages = (const char*)p.k_pages;
  const char* v_pages = (const char*)p.v_pages;
  const int32_t* bt = p.block_tables + (int64_t)i * p.M;
  const int64_t head_off = (int64_t)h * p.head_stride;
  (void)eb;

  float m = -INFINITY, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};

  for (int base = k_lo; base < k_hi; base += 64) {
    const int j = base + lane;
    float s = -INFINITY;
    float v_scale = 1.f;
    int64_t row = 0;  // byte offset of the key's (token, KV head) row inside the K pool; V has the same in its pool
    if (j < k_hi) {
      const int page = min(max(bt[j / p.page_size], 0), p.P - 1);
      row = (int64_t)page * p.page_stride + (int64_t)(j % p.page_size) * p.token_stride + head_off;
      const void* kp = k_pages + row;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(q_s[d], load_elem<KVT>(kp, d), dot);
      if (p.kv_scales) {
        dot *= p.kv_scales[(int64_t)page * p.C + 2 * h];
        v_scale = p.kv_scales[(int64_t)page * p.C + 2 * h + 1];
      }
      s = dot * p.scale;
      if (p.softcap > 0.f) s = p.softcap * tanhf(s / p.softcap);
    }
    const float bm = wave_max(s);
    const float m_new = fmaxf(m, bm);  // finite: lane 0 of every block holds a visible key
    const float pj = (j < k_hi) ? __expf(s - m_new) : 0.f;
    const float alpha = __expf(m - m_new);  // exp(-inf) = 0 on the first block
    l = l * alpha + wave_sum(pj);
    m = m_new;
#pragma unroll
    for (int k = 0; k < 4; ++k) acc[k] *= alpha;
    const float pv = pj * v_scale;
    const int n_keys = min(64, k_hi - base);
    for (int jj = 0; jj < n_keys; ++jj) {
      const float w = __shfl(pv, jj);
      const char* vrow = v_pages + (int64_t)__shfl((unsigned long long)row, jj);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int d = lane + 64 * k;
        if (d < D) acc[k] = fmaf(w, load_elem<KVT>(vrow, d), acc[k]);
      }
    }
  }
  if (p.sinks && l > 0.f) l += expf(p.sinks[hq] - m);  // attention sink: one more logit in the denominator only
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int d = lane + 64 * k;
    if (d < D) {
      store_out<QT>(p.out, ((int64_t)t * p.Hq + hq) * D + d, acc[k] * inv);
    }
  }
}

template <int QT>
static int launch_generic_q(hipStream_t stream, const AttnParams& p) {
  dim3 grid(p.T, p.Hq), block(64);
  switch (p.kv_dtype) {
    case RPA_F32: hipLaunchKernelGGL((attn_generic_kernel<QT, RPA_F32>), grid, block, 0, stream, p); break;
    case RPA_BF16: hipLaunchKernelGGL((attn_generic_kernel<QT, RPA_BF16>), grid, block, 0, stream, p); break;
    case RPA_FP8_E4M3: hipLaunchKernelGGL((attn_generic_kernel<QT, RPA_FP8_E4M3>), grid, block, 0, stream, p); break;
    case RPA_INT8: hipLaunchKernelGGL((attn_generic_kernel<QT, RPA_INT8>), grid, block, 0, stream, p); break;
    case RPA_F16: hipLaunchKernelGGL((attn_generic_kernel<QT, RPA_F16>), grid, block, 0, stream, p); break;
    default: return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

int launch_attn_generic(hipStream_t stream, const AttnParams& p) {
  if (p.Dq > 256) return (int)hipErrorInvalidValue;
  if (p.q_dtype == RPA_F32) return launch_generic_q<RPA_F32>(stream, p);
  if (p.q_dtype == RPA_F16) return launch_generic_q<RPA_F16>(stream, p);
  return launch_generic_q<RPA_BF16>(stream, p);
}

}  // namespace rpa
