// Split-K merge: combines the decode kernel's per-chunk partial outputs, and zero-fills the
// output rows of padded tokens so the whole [T, Hq, D] result is defined.
#include "rpa_common.h"

namespace rpa {

template <int QT>
__global__ __launch_bounds__(256) void attn_merge_kernel(AttnParams p) {
  const int t = blockIdx.x;
  const int n_live = p.num_seqs[0];
  const int D = p.D;
  const int units = p.Hq * (D / 4);  // D % 4 == 0 is checked by the host
  bool zero = false, merge = false;
  SeqPlan sp;
  if (n_live <= 0 || t < p.qsl[0] || t >= p.qsl[n_live]) {
    zero = true;
  } else {
    sp = seq_plan(p, find_seq(p.qsl, n_live, t));
    if (!sp.live) zero = true;
    else merge = p.mfma_path && sp.small_rows && sp.n_chunks > 1;
  }
  if (!zero && !merge) return;
  for (int u = threadIdx.x; u < units; u += blockDim.x) {
    const int hq = u / (D / 4), dv = u - hq * (D / 4);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (merge) {
      float m = -INFINITY;
      for (int c = 0; c < sp.n_chunks; ++c)
        m = fmaxf(m, p.part_ml[(((int64_t)c * p.T + t) * p.Hq + hq) * 2]);
      const float m_use = (m == -INFINITY) ? 0.f : m;
      float l = 0.f;
      for (int c = 0; c < sp.n_chunks; ++c) {
        const int64_t slot = ((int64_t)c * p.T + t) * p.Hq + hq;
        const float w = __builtin_amdgcn_exp2f(p.part_ml[slot * 2] - m_use);
        l += w * p.part_ml[slot * 2 + 1];
        const float4 o = ((const float4*)(p.part_o + slot * D))[dv];
        acc.x += w * o.x; acc.y += w * o.y; acc.z += w * o.z; acc.w += w * o.w;
      }
      const float inv = l > 0.f ? 1.f / l : 0.f;
      acc.x *= inv; acc.y *= inv; acc.z *= inv; acc.w *= inv;
    }
    const int64_t o = ((int64_t)t * p.Hq + hq) * D + dv * 4;
    if constexpr (QT == RPA_F32) {
      *(float4*)((float*)p.out + o) = acc;
    } else {
      uint2 r;
      r.x = (uint32_t)float_to_bf16_bits(acc.x) | ((uint32_t)float_to_bf16_bits(acc.y) << 16);
      r.y = (uint32_t)float_to_bf16_bits(acc.z) | ((uint32_t)float_to_bf16_bits(acc.w) << 16);
      *(uint2*)((uint16_t*)p.out + o) = r;
    }
  }
}

int launch_attn_merge(hipStream_t stream, const AttnParams& p) {
  if (p.q_dtype == RPA_F32) hipLaunchKernelGGL((attn_merge_kernel<RPA_F32>), dim3(p.T), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((attn_merge_kernel<RPA_BF16>), dim3(p.T), dim3(256), 0, stream, p);
  return (int)hipGetLastError();
}

}  // namespace rpa
