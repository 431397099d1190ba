// Split-K merge: combines the decode kernel's per-chunk partial outputs, and zero-fills the
// output rows of padded tokens so the whole [T, Hq, D] result is defined.
//
// One wavefront per (token, query head).  Lanes load the pieces' (max, sum) pairs, a cross-lane
// max gives the global max, each lane turns its pair into a weight; the partial rows are then
// accumulated with the weight broadcast from its lane, every lane owning D/64 output dims
// (coalesced row reads).
#include "rpa_common.h"

namespace rpa {


// NK: output dims per lane (D <= 64 * NK)
template <int QT, int NK>
__global__ __launch_bounds__(256, 8) void attn_merge_kernel(AttnParams p) {
  // partial rows in flight per wave: as many as leave the kernel within 64 registers, i.e. eight waves per SIMD
  constexpr int kUnroll = NK == 4 ? 2 : 4;
  const int lane = threadIdx.x & 63;
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);  // (token, head) index
  if (pair >= p.T * p.Hq) return;
  // the plan kernel has seen the whole batch: no padded token, no partial row -- nothing to do (a batch of prompts
  // whose row tiles are not cut would otherwise pay a look-up per row for nothing)
  if (p.mfma_path && p.plan[3] == 0) return;
  const int t = pair / p.Hq, hq = pair - t * p.Hq;
  const int n_live = live_rows(p);
  const int D = p.D;
  bool zero = false;
  int n_pieces = 0, part_row = 0;
  const float* part_o = p.part_o;
  const float* part_ml = p.part_ml;
  int64_t stride = (int64_t)p.t_dec_max * p.Hq;  // slots between consecutive pieces
  if (n_live <= 0 || t < p.qsl[0] || t >= p.qsl[n_live]) {
    zero = true;
  } else {
    const int i = find_seq_wave(p.qsl, n_live, t);  // one wave per (token, head): t is the same in all its lanes
    const SeqPlan sp = seq_plan(p, i);
    if (!sp.live) zero = true;
    else if (p.mfma_path && sp.small_rows) {
      n_pieces = decode_pieces(p.plan, i);
      part_row = p.plan[kPlanHeader + p.S + 1 + i] + (t - sp.q0);
    } else if (p.mfma_path && p.pre_max_chunks > 1) {  // prefill row tile split over key chunks
      const int row = (t - sp.q0) * p.group + hq % p.group;
      n_pieces = prefill_tile(p, sp, (row / pre_rows_of(p)) * pre_rows_of(p)).n_chunks;
      part_row = t;
      part_o = p.pre_o;
      part_ml = p.pre_ml;
      stride = (int64_t)p.T * p.Hq;
    }
  }
  const bool merge = n_pieces > 1;
  if (!zero && !merge) return;

  float acc[NK];  // dims lane, lane+64, ...
#pragma unroll
  for (int k = 0; k < NK; ++k) acc[k] = 0.f;
  float inv = 0.f;
  if (merge) {
    const int64_t slot0 = (int64_t)part_row * p.Hq + hq;
    float m = -INFINITY;
    for (int c = lane; c < n_pieces; c += 64) m = fmaxf(m, part_ml[(slot0 + c * stride) * 2]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    const float m_use = (m == -INFINITY) ? 0.f : m;
    float l = 0.f;
    for (int base = 0; base < n_pieces; base += 64) {
      const int c_mine = base + lane;
      float w_c = 0.f;
      if (c_mine < n_pieces) {
        const float2 ml = *(const float2*)(part_ml + (slot0 + c_mine * stride) * 2);
        w_c = __builtin_amdgcn_exp2f(ml.x - m_use);
        l += w_c * ml.y;
      }
      const int cnt = min(64, n_pieces - base);
      int c = 0;
      // A row with hundreds of pieces (one long sequence spread over the whole chip leaves a piece per workgroup) is
      // bound by the latency of these reads: kUnroll rows in flight at a time, accumulated in piece order as below.
      for (; c + kUnroll <= cnt; c += kUnroll) {
        float v[kUnroll][NK];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const float* row = part_o + (slot0 + (base + c + u) * stride) * D;
#pragma unroll
          for (int k = 0; k < NK; ++k) {
            const int d = lane + 64 * k;
            v[u][k] = (d < D) ? row[d] : 0.f;
          }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const float w = __shfl(w_c, c + u);
#pragma unroll
          for (int k = 0; k < NK; ++k) acc[k] = fmaf(w, v[u][k], acc[k]);
        }
      }
      for (; c < cnt; ++c) {
        const float w = __shfl(w_c, c);
        const float* row = part_o + (slot0 + (base + c) * stride) * D;
#pragma unroll
        for (int k = 0; k < NK; ++k) {
          const int d = lane + 64 * k;
          if (d < D) acc[k] = fmaf(w, row[d], acc[k]);
        }
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o);
    l = with_sink(p, hq, m_use, l);  // the pieces carry key sums only; the sink joins the denominator once, here
    inv = l > 0.f ? 1.f / l : 0.f;
  }
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int d = lane + 64 * k;
    if (d < p.Dq) store_out<QT>(p.out, ((int64_t)t * p.Hq + hq) * p.Dq + d, acc[k] * inv);  // partial rows are D wide, out rows Dq
  }
}

// The same for HPW neighbouring query heads of a token per wave (head size exactly 64 NK, Hq a multiple of HPW).  The
// partial rows of neighbouring heads are neighbours in memory, so the wave treats them as one row of HPW * D floats
// with a weight per head.  What bounds a row's merge is its chain of dependent loads (sequence look-up, plan, (max, sum)
// pairs, partial rows), not bytes: here one chain serves HPW rows.
template <int QT, int NK, int HPW>
__global__ __launch_bounds__(256, 4) void attn_merge_wide_kernel(AttnParams p) {
  constexpr int NKT = NK * HPW;  // floats per lane and piece
  constexpr int D = 64 * NK;
  constexpr int kUnroll = 32 / NKT;
  static_assert(NKT == 8, "eight floats per lane and four pieces in flight: 32 registers of loads per wave");
  const int lane = threadIdx.x & 63;
  const int groups = p.Hq / HPW;
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);  // (token, group of HPW heads) index
  if (pair >= p.T * groups) return;
  if (p.mfma_path && p.plan[3] == 0) return;  // nothing to merge or zero in this batch (see attn_merge_kernel)
  const int t = pair / groups, hq0 = (pair - t * groups) * HPW;
  const int n_live = live_rows(p);
  bool zero = false;
  int n_p[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) n_p[hh] = 0;
  int part_row = 0;
  const float* part_o = p.part_o;
  const float* part_ml = p.part_ml;
  int64_t stride = (int64_t)p.t_dec_max * p.Hq;  // slots between consecutive pieces
  if (n_live <= 0 || t < p.qsl[0] || t >= p.qsl[n_live]) {
    zero = true;
  } else {
    const int i = find_seq_wave(p.qsl, n_live, t);
    const SeqPlan sp = seq_plan(p, i);
    if (!sp.live) zero = true;
    else if (p.mfma_path && sp.small_rows) {
      const int n = decode_pieces(p.plan, i);
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) n_p[hh] = n;
      part_row = p.plan[kPlanHeader + p.S + 1 + i] + (t - sp.q0);
    } else if (p.mfma_path && p.pre_max_chunks > 1) {  // prefill row tiles split over key chunks
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {  // neighbouring heads can lie in different row tiles
        const int row = (t - sp.q0) * p.group + (hq0 + hh) % p.group;
        n_p[hh] = prefill_tile(p, sp, (row / pre_rows_of(p)) * pre_rows_of(p)).n_chunks;
      }
      part_row = t;
      part_o = p.pre_o;
      part_ml = p.pre_ml;
      stride = (int64_t)p.T * p.Hq;
    }
  }
  int n_max = 0;
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    if (n_p[hh] < 2) n_p[hh] = 0;  // a row in one piece was written by the kernel that computed it
    n_max = max(n_max, n_p[hh]);
  }
  if (!zero && n_max == 0) return;

  float acc[NKT];  // element lane + 64 k of the HPW * D floats: head k / NK
#pragma unroll
  for (int k = 0; k < NKT; ++k) acc[k] = 0.f;
  float inv[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) inv[hh] = 0.f;
  if (n_max > 0) {
    const int64_t slot0 = (int64_t)part_row * p.Hq + hq0;
    float m_use[HPW], l[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      float m = -INFINITY;
      for (int c = lane; c < n_p[hh]; c += 64) m = fmaxf(m, part_ml[(slot0 + hh + c * stride) * 2]);
      m_use[hh] = m;
      l[hh] = 0.f;
    }
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) m_use[hh] = fmaxf(m_use[hh], __shfl_xor(m_use[hh], o));
      if (m_use[hh] == -INFINITY) m_use[hh] = 0.f;
    }
    for (int base = 0; base < n_max; base += 64) {
      const int c_mine = base + lane;
      float w_c[HPW];
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {
        w_c[hh] = 0.f;
        if (c_mine < n_p[hh]) {
          const float2 ml = *(const float2*)(part_ml + (slot0 + hh + c_mine * stride) * 2);
          w_c[hh] = __builtin_amdgcn_exp2f(ml.x - m_use[hh]);
          l[hh] += w_c[hh] * ml.y;
        }
      }
      const int cnt = min(64, n_max - base);
      for (int c = 0; c < cnt; c += kUnroll) {
        float v[kUnroll][NKT];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const float* row = part_o + (slot0 + (int64_t)(base + c + u) * stride) * D;
#pragma unroll
          for (int k = 0; k < NKT; ++k) v[u][k] = (base + c + u < n_p[k / NK]) ? row[lane + 64 * k] : 0.f;  // never a piece nobody wrote
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          float w[HPW];
#pragma unroll
          for (int hh = 0; hh < HPW; ++hh) w[hh] = __shfl(w_c[hh], (c + u) & 63);  // zero past the head's pieces
#pragma unroll
          for (int k = 0; k < NKT; ++k) acc[k] = fmaf(w[k / NK], v[u][k], acc[k]);
        }
      }
    }
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      float lt = l[hh];
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) lt += __shfl_xor(lt, o);
      lt = with_sink(p, hq0 + hh, m_use[hh], lt);
      inv[hh] = lt > 0.f ? 1.f / lt : 0.f;
    }
  }
#pragma unroll
  for (int k = 0; k < NKT; ++k) {
    if (!zero && n_p[k / NK] == 0) continue;
    const int d = (lane + 64 * k) % D;  // dim inside head k / NK (partial rows are D wide, out rows Dq)
    if (d < p.Dq) store_out<QT>(p.out, ((int64_t)t * p.Hq + hq0 + k / NK) * p.Dq + d, acc[k] * inv[k / NK]);
  }
}

template <int QT>
static void launch_merge_q(hipStream_t stream, const AttnParams& p, int blocks) {
  if ((p.D == 64 || p.D == 128 || p.D == 256) && p.Hq % (512 / p.D) == 0) {  // eight floats per lane: 8, 4 or 2 heads per wave
    const int wide = (p.T * (p.Hq / (512 / p.D)) + 3) / 4;
    if (p.D == 64) hipLaunchKernelGGL((attn_merge_wide_kernel<QT, 1, 8>), dim3(wide), dim3(256), 0, stream, p);
    else if (p.D == 128) hipLaunchKernelGGL((attn_merge_wide_kernel<QT, 2, 4>), dim3(wide), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((attn_merge_wide_kernel<QT, 4, 2>), dim3(wide), dim3(256), 0, stream, p);
    return;
  }
  if (p.D <= 64) hipLaunchKernelGGL((attn_merge_kernel<QT, 1>), dim3(blocks), dim3(256), 0, stream, p);
  else if (p.D <= 128) hipLaunchKernelGGL((attn_merge_kernel<QT, 2>), dim3(blocks), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((attn_merge_kernel<QT, 4>), dim3(blocks), dim3(256), 0, stream, p);
}

int launch_attn_merge(hipStream_t stream, const AttnParams& p) {
  const int blocks = (p.T * p.Hq + 3) / 4;
  if (p.q_dtype == RPA_F32) launch_merge_q<RPA_F32>(stream, p, blocks);
  else if (p.q_dtype == RPA_F16) launch_merge_q<RPA_F16>(stream, p, blocks);
  else launch_merge_q<RPA_BF16>(stream, p, blocks);
  return (int)hipGetLastError();
}

}  // namespace rpa
