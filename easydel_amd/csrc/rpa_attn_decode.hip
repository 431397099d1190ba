// Split-K decode attention on MFMA: one wavefront per (sequence, KV head, key chunk).
//
// Serves sequences whose query rows for one KV head (q_len * group) fit one 16-row MFMA block:
// plain decode (q_len = 1) and short speculative / multi-token rows.  A workgroup holds WPB
// waves working on WPB adjacent KV heads of the same (sequence, chunk), so together they sweep
// whole token rows of a page; each wave streams its own K_h|V_h spans (contiguous in the
// [page][token][2*Hkv][D] layout) with 128-bit loads into registers one tile ahead, stages them
// in a wave-private swizzled LDS tile, and reads them back in MFMA operand order:
//     S^T[token][row] = K[token][:] . Q[row][:]          v_mfma_f32_16x16x32_bf16, k = head dim
//     O^T[dim][row]  += V^T[dim][token] . P^T[token][row] v_mfma_f32_16x16x16_bf16, k = tokens
// S^T's accumulator layout (lane = row, 4 tokens per lane) is exactly the B-operand layout of the
// second product, so probabilities never cross lanes; only the running max does (2 steps).
// fp8 / int8 pages are widened to bf16 (exactly) after the LDS read; their per-(page, head)
// scales fold into the score scale (K) and into P (V).
// No barriers: LDS tiles are wave-private and LDS operations of one wave execute in order.
#include "rpa_mfma.h"

namespace rpa {

template <int D, int KVT, int TT, int WPB>
__global__ __launch_bounds__(64 * WPB) void attn_decode_kernel(AttnParams p) {
  constexpr int EB = ElemBytes<KVT>::v;
  constexpr int RK = D * EB;           // bytes of one K (or V) row
  constexpr int HB = 2 * RK;           // K_h | V_h span of one token
  constexpr int NCH = RK / 16;         // 16-byte chunks per row
  constexpr int LPT = HB / 16;         // lanes covering one token's span
  constexpr int TPI = 64 / LPT;        // tokens per load instruction
  constexpr int NLD = TT / TPI;        // load instructions per tile
  constexpr int NS = TT / 16;          // 16-token sub-tiles per tile
  constexpr int DPL = D / 16;          // output dims per lane per accumulator register column
  constexpr int VB = DPL * EB;         // bytes of V one lane reads per token
  constexpr int NKK = D / 32;          // k-steps of the score MFMA
  static_assert(LPT <= 64 && TT % TPI == 0 && TT % 16 == 0, "tile shape");

  __shared__ __attribute__((aligned(16))) unsigned char lds_all[WPB * TT * HB];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int i = blockIdx.x;
  const int c = blockIdx.y;
  const int h = blockIdx.z * WPB + wave;
  if (h >= p.Hkv) return;
  const SeqPlan sp = seq_plan(p, i);
  if (!sp.live || !sp.small_rows || c >= sp.n_chunks) return;

  const int G = p.group;
  const int rows = sp.q_len * G;
  const int t_begin = sp.lo + c * sp.chunk;
  const int t_end = min(sp.hi, t_begin + sp.chunk);
  const int n_tiles = (t_end - t_begin + TT - 1) / TT;

  const int n = lane & 15;   // query row (column of S^T / O^T)
  const int g4 = lane >> 4;  // token group / k group

  // ---- per-lane row limits -------------------------------------------------------------
  const int r_tok = (n < rows) ? n / G : 0;           // padded rows shadow row 0 and are never stored
  const int r_head = (n < rows) ? n - r_tok * G : 0;
  const int pos = sp.ctx - sp.q_len + r_tok;
  const int row_hi = min(pos + 1, sp.ctx);            // exclusive
  const int row_lo = (p.window > 0) ? max(pos - p.window + 1, 0) : 0;
  const int vis_lo = (p.window > 0) ? max(sp.ctx - sp.q_len - p.window + 1, 0) : 0;  // lowest key any row sees

  // ---- Q as B operands -----------------------------------------------------------------
  bf16x8 qf[NKK];
  {
    const char* qrow = (const char*)p.q + ((int64_t)(sp.q0 + r_tok) * p.Hq + (h * G + r_head)) * D * 2;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      // bf16 pages: step kk covers dims 32kk + 8g4 + e.  8-bit pages: a 16-byte K chunk holds 16
      // dims, so steps (2j, 2j+1) cover dims 64j + 16g4 + 8b + e.
      const int d0 = (EB == 2) ? (kk * 32 + 8 * g4) : ((kk >> 1) * 64 + 16 * g4 + 8 * (kk & 1));
      u32x4 v = {0u, 0u, 0u, 0u};
      if (n < rows) v = *(const u32x4*)(qrow + d0 * 2);
      qf[kk] = __builtin_bit_cast(bf16x8, v);
    }
  }

  // ---- tile addressing -----------------------------------------------------------------
  unsigned char* lds_k = lds_all + wave * (TT * HB);
  unsigned char* lds_v = lds_k + TT * RK;
  const int sub = lane / LPT;
  const int c32 = lane % LPT;
  const bool is_v = c32 >= NCH;
  const int cc = is_v ? c32 - NCH : c32;
  const int32_t* bt = p.block_tables + (int64_t)i * p.M;
  const char* pages = (const char*)p.kv_pages;
  const int64_t lane_goff = (int64_t)h * HB + c32 * 16 + (int64_t)sub * p.token_stride;
  const int pg = p.page_size;

  u32x4 stage[NLD];
  auto page_of = [&](int tok) -> int {
    int pgid = bt[tok / pg];
    pgid = __builtin_amdgcn_readfirstlane(pgid);
    return min(max(pgid, 0), p.P - 1);
  };
  auto issue = [&](int tile, int page) {
    const int tb = t_begin + tile * TT;
    const char* base = pages + (int64_t)page * p.page_stride + (int64_t)(tb % pg) * p.token_stride + lane_goff;
#pragma unroll
    for (int u = 0; u < NLD; ++u) stage[u] = *(const u32x4*)(base + (int64_t)(u * TPI) * p.token_stride);
  };

  float m_run = -INFINITY, l_run = 0.f;
  f32x4 o_acc[DPL];
#pragma unroll
  for (int rt = 0; rt < DPL; ++rt) o_acc[rt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  int page_cur = page_of(t_begin);
  issue(0, page_cur);

  for (int tile = 0; tile < n_tiles; ++tile) {
    const int tb = t_begin + tile * TT;
    // ---- registers -> LDS (zero rows past the context end or left of every row's window, so stale
    //      or null-page bytes cannot reach P.V as 0 * NaN)
    if (tb + TT > sp.ctx || tb < vis_lo) {
#pragma unroll
      for (int u = 0; u < NLD; ++u) {
        const int tok = tb + u * TPI + sub;
        if (tok >= sp.ctx || tok < vis_lo) stage[u] = (u32x4){0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int u = 0; u < NLD; ++u) {
      const int tk = u * TPI + sub;
      unsigned char* dst = (is_v ? lds_v : lds_k) + tk * RK + ((cc ^ swz_key<RK>(tk)) << 4);
      *(u32x4*)dst = stage[u];
    }
    float k_scale = 1.f, v_scale = 1.f;
    if constexpr (EB == 1) {
      const float* sc = p.kv_scales + (int64_t)page_cur * p.C + 2 * h;
      k_scale = sc[0];
      v_scale = sc[1];
    }
    // ---- prefetch the next tile into registers ---------------------------------------------
    if (tile + 1 < n_tiles) {
      page_cur = page_of(tb + TT);
      issue(tile + 1, page_cur);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // ---- S^T = K . Q^T ----------------------------------------------------------------------
    f32x4 s_acc[NS];
#pragma unroll
    for (int st = 0; st < NS; ++st) {
      s_acc[st] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const int tk = st * 16 + n;  // this lane's A-operand row (token)
      const unsigned char* krow = lds_k + tk * RK;
      const int key = swz_key<RK>(tk);
      if constexpr (EB == 2) {
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
          const u32x4 a = *(const u32x4*)(krow + (((kk * 4 + g4) ^ key) << 4));
          s_acc[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), qf[kk], s_acc[st], 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int j = 0; j < NKK / 2; ++j) {
          const u32x4 a = *(const u32x4*)(krow + (((j * 4 + g4) ^ key) << 4));
          s_acc[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(codes8_to_bf16x8<KVT>(a[0], a[1]), qf[2 * j], s_acc[st], 0, 0, 0);
          s_acc[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(codes8_to_bf16x8<KVT>(a[2], a[3]), qf[2 * j + 1], s_acc[st], 0, 0, 0);
        }
      }
    }

    // ---- online softmax (log2 domain) -------------------------------------------------------
    float mx = -INFINITY;
#pragma unroll
    for (int st = 0; st < NS; ++st) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int tok = tb + st * 16 + 4 * g4 + j;
        float s = s_acc[st][j];
        if (p.softcap > 0.f) s = p.softcap * 1.4426950408889634f * fast_tanh(s * (p.scale * k_scale / p.softcap));
        else s *= p.scale_log2 * k_scale;
        s = (tok >= row_lo && tok < row_hi) ? s : -INFINITY;
        s_acc[st][j] = s;
        mx = fmaxf(mx, s);
      }
    }
    mx = xor32_max(xor16_max(mx));
    const float m_new = fmaxf(m_run, mx);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
    m_run = m_new;
    float psum = 0.f;
    uint32_t pfrag[NS][2];
#pragma unroll
    for (int st = 0; st < NS; ++st) {
      float pr[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pr[j] = __builtin_amdgcn_exp2f(s_acc[st][j] - m_use);
        psum += pr[j];
      }
      pfrag[st][0] = pack_bf16(pr[0] * v_scale, pr[1] * v_scale);
      pfrag[st][1] = pack_bf16(pr[2] * v_scale, pr[3] * v_scale);
    }
    l_run = l_run * alpha + psum;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int rt = 0; rt < DPL; ++rt) o_acc[rt] *= alpha;
    }

    // ---- O^T += V^T . P^T ---------------------------------------------------------------------
#pragma unroll
    for (int st = 0; st < NS; ++st) {
      const u32x2 pb2 = {pfrag[st][0], pfrag[st][1]};
      const s16x4 pb = __builtin_bit_cast(s16x4, pb2);
      if constexpr (EB == 2) {
        // raw[e][w]: token 4g4+e, dword w of this lane's DPL dims (2 dims per dword)
        uint32_t raw[4][DPL / 2];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int tk = st * 16 + 4 * g4 + e;
          const unsigned char* vrow = lds_v + tk * RK;
          const int key = swz_key<RK>(tk);
          if constexpr (VB >= 16) {
#pragma unroll
            for (int r = 0; r < VB / 16; ++r) {
              const u32x4 v = *(const u32x4*)(vrow + ((((n * VB) / 16 + r) ^ key) << 4));
              raw[e][4 * r + 0] = v[0]; raw[e][4 * r + 1] = v[1]; raw[e][4 * r + 2] = v[2]; raw[e][4 * r + 3] = v[3];
            }
          } else {  // VB == 8
            const u32x2 v = *(const u32x2*)(vrow + ((((n * VB) >> 4) ^ key) << 4) + ((n * VB) & 15));
            raw[e][0] = v[0]; raw[e][1] = v[1];
          }
        }
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) {
          const uint32_t sel = (rt & 1) ? 0x07060302u : 0x05040100u;
          const u32x2 a2 = {__builtin_amdgcn_perm(raw[1][rt >> 1], raw[0][rt >> 1], sel),
                            __builtin_amdgcn_perm(raw[3][rt >> 1], raw[2][rt >> 1], sel)};
          o_acc[rt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a2), pb, o_acc[rt], 0, 0, 0);
        }
      } else {
        float vf[4][DPL];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int tk = st * 16 + 4 * g4 + e;
          const unsigned char* vrow = lds_v + tk * RK;
          const int key = swz_key<RK>(tk);
          if constexpr (VB >= 16) {
#pragma unroll
            for (int r = 0; r < VB / 16; ++r) {
              const u32x4 v = *(const u32x4*)(vrow + ((((n * VB) / 16 + r) ^ key) << 4));
#pragma unroll
              for (int w = 0; w < 4; ++w) decode4<KVT>(v[w], &vf[e][16 * r + 4 * w]);
            }
          } else if constexpr (VB == 8) {
            const u32x2 v = *(const u32x2*)(vrow + ((((n * VB) >> 4) ^ key) << 4) + ((n * VB) & 15));
            decode4<KVT>(v[0], &vf[e][0]);
            decode4<KVT>(v[1], &vf[e][4]);
          } else {  // VB == 4
            const uint32_t v = *(const uint32_t*)(vrow + ((((n * VB) >> 4) ^ key) << 4) + ((n * VB) & 15));
            decode4<KVT>(v, &vf[e][0]);
          }
        }
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) {
          const u32x2 a2 = {pack_bf16(vf[0][rt], vf[1][rt]), pack_bf16(vf[2][rt], vf[3][rt])};
          o_acc[rt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a2), pb, o_acc[rt], 0, 0, 0);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }

  // ---- epilogue: lane (n, g4) holds dims [4*DPL*g4, 4*DPL*(g4+1)) of row n, ordered j*DPL + rt ----
  float l_tot = l_run + __shfl_xor(l_run, 16);
  l_tot += __shfl_xor(l_tot, 32);
  if (n >= rows) return;
  const int tok_out = sp.q0 + r_tok;
  const int head_out = h * G + r_head;
  const int d_base = 4 * DPL * g4;
  if (sp.n_chunks == 1) {
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    uint16_t* orow = (uint16_t*)p.out + ((int64_t)tok_out * p.Hq + head_out) * D + d_base;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int rt = 0; rt < DPL; rt += 2) {
        *(uint32_t*)(orow + j * DPL + rt) = pack_bf16(o_acc[rt][j] * inv, o_acc[rt + 1][j] * inv);
      }
    }
  } else {
    const int64_t slot = ((int64_t)c * p.T + tok_out) * p.Hq + head_out;
    float* prow = p.part_o + slot * D + d_base;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int rt = 0; rt < DPL; ++rt) prow[j * DPL + rt] = o_acc[rt][j];
    }
    if (g4 == 0) {
      p.part_ml[slot * 2 + 0] = m_run;
      p.part_ml[slot * 2 + 1] = l_tot;
    }
  }
}

template <int D, int KVT, int TT, int WPB>
static int launch_one(hipStream_t stream, const AttnParams& p) {
  dim3 grid(p.S, p.max_splits, (p.Hkv + WPB - 1) / WPB), block(64 * WPB);
  hipLaunchKernelGGL((attn_decode_kernel<D, KVT, TT, WPB>), grid, block, 0, stream, p);
  return (int)hipGetLastError();
}

template <int D, int KVT, int TT>
static int launch_wpb(hipStream_t stream, const AttnParams& p) {
  constexpr int tile_bytes = TT * 2 * D * ElemBytes<KVT>::v;
  if constexpr (tile_bytes * 8 <= 65536) {
    if (p.Hkv >= 8) return launch_one<D, KVT, TT, 8>(stream, p);
  }
  if (p.Hkv >= 4) return launch_one<D, KVT, TT, 4>(stream, p);
  if (p.Hkv >= 2) return launch_one<D, KVT, TT, 2>(stream, p);
  return launch_one<D, KVT, TT, 1>(stream, p);
}

template <int KVT>
static int launch_kvt(hipStream_t stream, const AttnParams& p) {
  constexpr int EB = ElemBytes<KVT>::v;
  const bool tt32 = (p.page_size % 32 == 0);
  switch (p.D) {
    case 64:
      return tt32 ? launch_wpb<64, KVT, 32>(stream, p) : launch_wpb<64, KVT, 16>(stream, p);
    case 128:
      if constexpr (EB == 1) return tt32 ? launch_wpb<128, KVT, 32>(stream, p) : launch_wpb<128, KVT, 16>(stream, p);
      else return launch_wpb<128, KVT, 16>(stream, p);
    case 256:
      return launch_wpb<256, KVT, 16>(stream, p);
    default:
      return (int)hipErrorInvalidValue;
  }
}

bool decode_supported(const AttnParams& p) {
  if (p.q_dtype != RPA_BF16 || p.kv_dtype == RPA_F32) return false;
  if (p.D != 64 && p.D != 128 && p.D != 256) return false;
  if (p.page_size % 16 != 0) return false;
  if (p.kv_dtype != RPA_BF16 && p.kv_scales == nullptr) return false;
  return true;
}

int launch_attn_decode(hipStream_t stream, const AttnParams& p) {
  switch (p.kv_dtype) {
    case RPA_BF16: return launch_kvt<RPA_BF16>(stream, p);
    case RPA_FP8_E4M3: return launch_kvt<RPA_FP8_E4M3>(stream, p);
    case RPA_INT8: return launch_kvt<RPA_INT8>(stream, p);
    default: return (int)hipErrorInvalidValue;
  }
}

}  // namespace rpa
