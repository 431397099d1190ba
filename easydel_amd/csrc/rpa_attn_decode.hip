// Split-K decode attention on MFMA, persistent and evenly split: one wavefront per KV head.
//
// Serves sequences whose query rows for one KV head (q_len * group) fit one or two 16-row MFMA blocks:
// plain decode (q_len = 1) and short speculative / multi-token rows.  The keys of all such
// sequences are laid end to end (a small plan kernel computes the prefix sums on the device); each
// of the resident workgroups takes one equal span of that stream, whatever sequence boundaries fall
// inside it, so every CU streams the same number of bytes and no launch-time shape depends on the
// batch.  A sequence cut by a span boundary leaves partial results that the merge kernel combines.
// A workgroup holds WPB waves working on WPB adjacent KV heads of the same keys, so together they
// sweep whole token rows of a page; each wave streams its own K_h|V_h spans (contiguous in the
// [page][token][2*Hkv][D] layout) with 128-bit loads into registers one tile ahead, stages them
// in a wave-private swizzled LDS tile, and reads them back in MFMA operand order:
//     S^T[token][row] = K[token][:] . Q[row][:]          v_mfma_f32_16x16x32_bf16, k = head dim
//     O^T[dim][row]  += V^T[dim][token] . P^T[token][row] v_mfma_f32_16x16x16_bf16, k = tokens
// S^T's accumulator layout (lane = row, 4 tokens per lane) is exactly the B-operand layout of the
// second product, so probabilities never cross lanes; only the running max does (2 steps).
// bf16 V operands come from transposing LDS reads (ds_read_b64_tr_b16); fp8 / int8 pages are widened
// to bf16 (exactly) after the LDS read.  Their per-(page, head) scales travel with the tile: the K scale
// folds into the score scale, and the accumulators are kept in units of the current page's V scale, so
// the probabilities stay exact softmax weights.
// LDS tiles are wave-private and LDS operations of one wave execute in order, so no barrier is needed for
// correctness; one every few tiles keeps the workgroup's waves on the same token rows, which keeps its
// outstanding loads inside the same DRAM rows.
#include <atomic>
#include <type_traits>

#include "rpa_attn_decode_dma.h"
#include "rpa_mfma.h"

namespace rpa {

// Per-workgroup piece of the flattened key stream: a token range of one sequence.
struct Piece {
  int i, q0, q_len, ctx;
  int part_row;        // row of the sequence's first query token in the partial buffers
  int t_begin, t_end;  // keys [t_begin, t_end) of sequence i
  int slot;            // which partial slot of the sequence this piece fills
  int single;          // the sequence lies in one piece: write the final output directly
  int flat_end;        // flat position where the piece ends
};

// Finds the sequence that holds flat position `pos` (searching upwards from i) and cuts the piece
// [pos, min(span_end, end of that sequence)) out of it.  pos < span_end <= W.
__device__ __forceinline__ Piece make_piece(const AttnParams& p, const int32_t* __restrict__ P, int i, int pos,
                                            int span_end, int Q) {
  int p1 = P[i + 1];
  while (p1 <= pos) {  // sequences without decode-class work have zero length
    ++i;
    p1 = P[i + 1];
  }
  const int p0 = P[i];
  const SeqPlan sp = seq_plan(p, i);
  Piece pc;
  pc.i = i; pc.q0 = sp.q0; pc.q_len = sp.q_len; pc.ctx = sp.ctx;
  pc.part_row = P[p.S + 1 + i];
  pc.flat_end = min(span_end, p1);
  pc.t_begin = sp.lo + (pos - p0);
  pc.t_end = min(sp.hi, sp.lo + (pc.flat_end - p0));
  const int j_first = p0 / Q;
  pc.slot = pos / Q - j_first;
  pc.single = (j_first == (p1 - 1) / Q);
  return pc;
}

// RB: 16-row blocks of query rows one wave carries (rows of a sequence for one KV head: q_len * group <= 16 * RB).
// Every K and V operand read from LDS feeds the MFMAs of all RB blocks.
// PACE: the workgroup counts its waves that have a tile's loads in flight (an LDS counter: up by one before a wave
// issues, down by one when its data has arrived), and a wave that finds kPaceCrowd or more of them pauses once, for
// kPacePause x 64 clocks, before it adds its own.  This memory system delivers more a little below saturation than
// with every wave pressing on it: bounding the requests in flight this way is worth 2.4 % on long bf16 streams
// (738.5 -> 721 us on the Llama-shaped decode batch, both builds run in one process; crowds of 3 to 5 and pauses
// of 512 to 1024 clocks all lie within 1 % of that; 8-bit pages and four-wave workgroups lose by it, so they are
// built without).  There is no loop and no waiting on another wave: the delay of a tile is bounded by the pause.
constexpr int kPaceCrowd = 4, kPacePause = 8;
template <int D, int KVT, int TT, int WPB, bool CAP, int RB, bool PACE>
__global__ __launch_bounds__(64 * WPB, 1) void attn_decode_kernel(AttnParams p) {
  constexpr int EB = ElemBytes<KVT>::v;
  constexpr int HT = KVT == RPA_F16 ? RPA_F16 : RPA_BF16;  // 16-bit float type of the MFMA operands
  using H = Half16<HT>;
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
  // Tiles in flight per wave (register staging buffers).  Two were measured slower than one on MI355X (780 vs
  // 766 us on the Llama-shaped decode batch) -- but as compiled, the DEPTH = 2 build never has two tiles in flight:
  // the compiler's waits before a tile's registers are first used (s_waitcnt vmcnt(n), n <= 6 throughout) also
  // drain the newer tile's loads.  A build that means it has to issue these loads and their waits itself.
  constexpr int DEPTH = 1;
  static_assert(LPT <= 64 && TT % TPI == 0 && TT % 16 == 0, "tile shape");

  __shared__ __attribute__((aligned(16))) unsigned char lds_all[WPB * TT * HB];
  __shared__ int s_inflight;  // PACE: waves of this workgroup with a tile's loads in flight
  if constexpr (PACE) {
    if (threadIdx.x == 0) s_inflight = 0;
    __syncthreads();
  }

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h = blockIdx.y * WPB + wave;
  if (h >= p.Hkv) return;

  // ---- this workgroup's span of the flattened key stream --------------------------------------
  const int32_t* __restrict__ plan = p.plan;
  const int W = plan[0], Q = plan[1];
  const int32_t* __restrict__ P = plan + kPlanHeader;
  if ((int64_t)blockIdx.x * Q >= W) return;
  const int span_begin = blockIdx.x * Q;
  const int span_end = min(W, span_begin + Q);

  const int G = p.group;
  const int n = lane & 15;   // query row (column of S^T / O^T)
  const int g4 = lane >> 4;  // token group / k group
  const int pg = p.page_size;

  // ---- tile addressing (independent of the piece) ---------------------------------------------
  unsigned char* lds_k = lds_all + wave * (TT * HB);
  unsigned char* lds_v = lds_k + TT * RK;
  const int sub = lane / LPT;
  const int c32 = lane % LPT;
  const bool is_v = c32 >= NCH;
  const int cc = is_v ? c32 - NCH : c32;
  // a lane fetches either K or V chunks, always: its pool and its offset inside a token row are fixed
  const char* pages = (const char*)(is_v ? p.v_pages : p.k_pages);
  const int64_t lane_goff = (int64_t)h * p.head_stride + cc * 16 + (int64_t)sub * p.token_stride;

  u32x4 stage[DEPTH][NLD];
  u32x2 sc_stage[DEPTH];  // (K scale, V scale) of the staged tile's page: fetched with the tile, in order behind it
  auto page_of = [&](int seq, int tok) -> int {
    int pgid = p.block_tables[(int64_t)seq * p.M + tok / pg];
    pgid = __builtin_amdgcn_readfirstlane(pgid);
    return min(max(pgid, 0), p.P - 1);
  };
  auto issue = [&](auto buf, int tb, int page) {  // buf: std::integral_constant, so the register array index is static
    constexpr int B = decltype(buf)::value;
    const char* base = pages + (int64_t)page * p.page_stride + (int64_t)(tb % pg) * p.token_stride + lane_goff;
    // Non-temporal loads: a decode step reads every cached key and value exactly once, and marked as a stream the pages
    // come out of HBM a tenth faster than through ordinary loads (the paged read probe shows the same gap without any
    // arithmetic: 89 % against 78 % of the peak for this very access pattern).
#pragma unroll
    for (int u = 0; u < NLD; ++u) stage[B][u] = __builtin_nontemporal_load((const u32x4*)(base + (int64_t)(u * TPI) * p.token_stride));
    // a vector load on purpose: a scalar load would be waited for together with the next LDS read
    if constexpr (EB == 1) {
      if (p.kv_scales) sc_stage[B] = *(const u32x2*)(p.kv_scales + (int64_t)page * p.C + 2 * h);
      else sc_stage[B] = (u32x2){0x3f800000u, 0x3f800000u};  // unscaled 8-bit pages: the codes are the values
    }
  };
  using Buf0 = std::integral_constant<int, 0>;
  using Buf1 = std::integral_constant<int, DEPTH - 1>;

  const float cap_out = p.softcap * 1.4426950408889634f;
  const float cap_in = CAP ? p.scale / p.softcap : 0.f;

  // short spans (small batches) are latency-bound from start to end: no pacing there
  const bool pace = PACE && p.decode_pace != 0 && Q >= 512;
  bool counted = false;
  auto enter = [&]() {
    if constexpr (PACE) {
      if (!pace) return;
      int seen = 0;
      if (lane == 0) seen = atomicAdd(&s_inflight, 1);
      seen = __builtin_amdgcn_readfirstlane(seen);
      counted = true;
      if (seen >= kPaceCrowd) __builtin_amdgcn_s_sleep(kPacePause);
    }
  };
  auto leave = [&]() {
    if constexpr (PACE) {
      if (!counted) return;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the tile has arrived
      if (lane == 0) atomicSub(&s_inflight, 1);
      counted = false;
    }
  };
  Piece cur = make_piece(p, P, plan[kPlanHeader + 2 * (p.S + 1) + blockIdx.x], span_begin, span_end, Q);
  int page_a = page_of(cur.i, cur.t_begin), page_b = 0;  // pages of the tiles in staging buffers 0 and 1
  enter();
  issue(Buf0{}, cur.t_begin, page_a);  // first tile in flight before anything else is set up

  for (;;) {
  const int rows = cur.q_len * G;
  const int t_begin = cur.t_begin;
  const int n_tiles = (cur.t_end - t_begin + TT - 1) / TT;

  // ---- per-lane row limits -------------------------------------------------------------
  int r_tok[RB], r_head[RB], row_hi[RB], row_lo[RB];  // this lane's row of block rb is row n + 16 rb of the sequence
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int nr = n + 16 * rb;
    r_tok[rb] = (nr < rows) ? nr / G : 0;               // padded rows shadow row 0 and are never stored
    r_head[rb] = (nr < rows) ? nr - r_tok[rb] * G : 0;
    const int pos = cur.ctx - cur.q_len + r_tok[rb];
    row_hi[rb] = min(pos + 1, cur.ctx);                 // exclusive
    row_lo[rb] = (p.window > 0) ? max(pos - p.window + 1, 0) : 0;
  }
  const int vis_lo = (p.window > 0) ? max(cur.ctx - cur.q_len - p.window + 1, 0) : 0;  // lowest key any row sees
  // keys every row sees: from the last row's window start to the first row's causal limit
  const int all_lo = (p.window > 0) ? max(cur.ctx - p.window, 0) : 0;
  const int all_hi = cur.ctx - cur.q_len + 1;

  // ---- Q as B operands -----------------------------------------------------------------
  u32x4 qf[RB][NKK];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const char* qrow = (const char*)p.q + ((int64_t)(cur.q0 + r_tok[rb]) * p.Hq + (h * G + r_head[rb])) * p.Dq * 2;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      // bf16 pages: step kk covers dims 32kk + 8g4 + e.  8-bit pages: a 16-byte K chunk holds 16
      // dims, so steps (2j, 2j+1) cover dims 64j + 16g4 + 8b + e.
      const int d0 = (EB == 2) ? (kk * 32 + 8 * g4) : ((kk >> 1) * 64 + 16 * g4 + 8 * (kk & 1));
      u32x4 v = {0u, 0u, 0u, 0u};
      if (n + 16 * rb < rows && d0 < p.Dq) v = *(const u32x4*)(qrow + d0 * 2);  // dims past Dq: zero padding
      qf[rb][kk] = v;
    }
  }

  // ---- the piece after this one (its first tile is prefetched during this piece's last tile) ---
  const bool has_next = cur.flat_end < span_end;
  Piece nxt = cur;
  int page_nxt = 0;
  if (has_next) {
    nxt = make_piece(p, P, cur.i + 1, cur.flat_end, span_end, Q);
    page_nxt = page_of(nxt.i, nxt.t_begin);
  }

  float m_run[RB], l_run[RB];
  float v_unit = 1.f;  // V scale the accumulators are currently expressed in (8-bit pages)
  f32x4 o_acc[RB][DPL];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    m_run[rb] = -INFINITY;
    l_run[rb] = 0.f;
#pragma unroll
    for (int rt = 0; rt < DPL; ++rt) o_acc[rb][rt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  // ---- registers -> LDS (zero rows past the context end or left of every row's window, so stale or
  //      null-page bytes cannot reach P.V as 0 * NaN)
  auto commit = [&](auto buf, int tb) {
    constexpr int B = decltype(buf)::value;
    if (tb + TT > cur.ctx || tb < vis_lo) {
#pragma unroll
      for (int u = 0; u < NLD; ++u) {
        const int tok = tb + u * TPI + sub;
        if (tok >= cur.ctx || tok < vis_lo) stage[B][u] = (u32x4){0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int u = 0; u < NLD; ++u) {
      const int tk = u * TPI + sub;
      unsigned char* dst = (is_v ? lds_v : lds_k) + tk * RK + ((cc ^ swz_key<RK>(tk)) << 4);
      *(u32x4*)dst = stage[B][u];
    }
  };

  auto compute = [&](int tb, float k_scale, float v_scale) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // ---- S^T = K . Q^T ----------------------------------------------------------------------
    f32x4 s_acc[RB][NS];
#pragma unroll
    for (int st = 0; st < NS; ++st) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) s_acc[rb][st] = (f32x4){0.f, 0.f, 0.f, 0.f};
      const int tk = st * 16 + n;  // this lane's A-operand row (token)
      const unsigned char* krow = lds_k + tk * RK;
      const int key = swz_key<RK>(tk);
      if constexpr (EB == 2) {
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
          const u32x4 a = *(const u32x4*)(krow + (((kk * 4 + g4) ^ key) << 4));
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
            s_acc[rb][st] = H::mfma32(a, qf[rb][kk], s_acc[rb][st]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < NKK / 2; ++j) {
          const u32x4 a = *(const u32x4*)(krow + (((j * 4 + g4) ^ key) << 4));
          const u32x4 a_lo = codes8_to_bf16x8<KVT>(a[0], a[1]), a_hi = codes8_to_bf16x8<KVT>(a[2], a[3]);
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            s_acc[rb][st] = H::mfma32(a_lo, qf[rb][2 * j], s_acc[rb][st]);
            s_acc[rb][st] = H::mfma32(a_hi, qf[rb][2 * j + 1], s_acc[rb][st]);
          }
        }
      }
    }

    // ---- online softmax (log2 domain) -------------------------------------------------------
    const float sc_mul = CAP ? cap_out : p.scale_log2 * k_scale;
    uint32_t pfrag[RB][NS][2];
    // The accumulators hold sum(p * v_code) in units of the current page's V scale, so P stays an exact
    // softmax weight in bf16; when the scale changes (a new page) they are converted once.
    float unit_mul = 1.f;
    if constexpr (EB == 1) {
      if (v_unit != v_scale) unit_mul = v_unit * __builtin_amdgcn_rcpf(v_scale);
      v_unit = v_scale;
    }
    const bool inside = tb >= all_lo && tb + TT <= all_hi;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      float alpha;
      if (inside)
        alpha = softmax_step<false, CAP, NS, HT>(s_acc[rb], sc_mul, cap_in * k_scale, tb, g4, row_lo[rb], row_hi[rb], m_run[rb], l_run[rb], pfrag[rb]);
      else
        alpha = softmax_step<true, CAP, NS, HT>(s_acc[rb], sc_mul, cap_in * k_scale, tb, g4, row_lo[rb], row_hi[rb], m_run[rb], l_run[rb], pfrag[rb]);
      const float o_mul = (EB == 1) ? alpha * unit_mul : alpha;
      if (__any(o_mul != 1.f)) {
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) o_acc[rb][rt] *= o_mul;
      }
    }

    // ---- O^T += V^T . P^T ---------------------------------------------------------------------
    // bf16 pages: ds_read_b64_tr_b16 hands each lane the key-major column it needs (inside a 16-lane group,
    // lane l addresses key 4g4 + l/4, dims d0 + 4(l%4).. and receives dim d0 + l of keys 4g4..4g4+3).
    // 8-bit pages: each lane reads 4 keys x 4 consecutive dims of codes and widens them while transposing.
#pragma unroll
    for (int st = 0; st < NS; ++st) {
      u32x2 pb[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const u32x2 pb2 = {pfrag[rb][st][0], pfrag[rb][st][1]};
        pb[rb] = pb2;
      }
      if constexpr (EB == 2) {
        const int tk = st * 16 + 4 * g4 + (n >> 2);
        const unsigned char* vrow = lds_v + tk * RK;
        const int key = swz_key<RK>(tk);
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) {
          const int off = rt * 32 + (n & 3) * 8;
          const unsigned char* ptr = vrow + (((off >> 4) ^ key) << 4) + (off & 15);
          const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)ptr);
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) o_acc[rb][rt] = H::mfma16(__builtin_bit_cast(u32x2, a), pb[rb], o_acc[rb][rt]);
        }
      } else {
        // lane (n, g4) reads DPL consecutive dims (DPL*n ..) of keys 4g4..4g4+3 and widens them; row tile rt
        // of this path therefore holds dims DPL*i + rt (any dim permutation works for O^T, see the epilogue)
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
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
            o_acc[rb][rt] = H::mfma16(a2, pb[rb], o_acc[rb][rt]);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  };

  // ---- tile loop: DEPTH tiles in flight; the next piece's first tile is issued into buffer 0 as soon as this
  //      piece no longer needs it, so the stream of loads never drains at a piece boundary
  if (DEPTH == 2 && n_tiles > 1) {
    page_b = page_of(cur.i, t_begin + TT);
    issue(Buf1{}, t_begin + TT, page_b);
  }
  for (int tile = 0; tile < n_tiles; tile += DEPTH) {
    const int tb = t_begin + tile * TT;
    // The waves of a workgroup read adjacent 512-byte spans of the same token rows; a barrier every few tiles
    // keeps them in step so each DRAM row is opened once (740 vs 764 us).  All waves of a workgroup walk the
    // same pieces and tiles, so every live wave reaches every barrier.
    leave();
    if (p.decode_sync > 0 && (tile & (p.decode_sync - 1)) == 0) __builtin_amdgcn_s_barrier();
    commit(Buf0{}, tb);
    float ks = 1.f, vs = 1.f;
    if constexpr (EB == 1) {
      ks = __uint_as_float(sc_stage[0][0]);
      vs = __uint_as_float(sc_stage[0][1]);
    }
    if (tile + DEPTH < n_tiles) {
      page_a = page_of(cur.i, tb + DEPTH * TT);
      enter();
      issue(Buf0{}, tb + DEPTH * TT, page_a);
    } else if (has_next) {
      page_a = page_nxt;
      enter();
      issue(Buf0{}, nxt.t_begin, page_nxt);
    }
    compute(tb, ks, vs);
    if constexpr (DEPTH == 2) {
      if (tile + 1 < n_tiles) {
        commit(Buf1{}, tb + TT);
        float ks_b = 1.f, vs_b = 1.f;
        if constexpr (EB == 1) {
          ks_b = __uint_as_float(sc_stage[DEPTH - 1][0]);
          vs_b = __uint_as_float(sc_stage[DEPTH - 1][1]);
        }
        if (tile + 3 < n_tiles) {
          page_b = page_of(cur.i, tb + 3 * TT);
          issue(Buf1{}, tb + 3 * TT, page_b);
        }
        compute(tb + TT, ks_b, vs_b);
      }
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------------
  // accumulator column j of row tile rt is dim 16rt + 4g4 + j (bf16 pages) or DPL*(4g4 + j) + rt (8-bit pages)
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float l_tot = l_run[rb] + __shfl_xor(l_run[rb], 16);
    l_tot += __shfl_xor(l_tot, 32);
    if (n + 16 * rb < rows) {
      const int tok_out = cur.q0 + r_tok[rb];
      const int head_out = h * G + r_head[rb];
      if (cur.single) {
        const float l_fin = with_sink(p, head_out, m_run[rb], l_tot);
        const float inv = (l_fin > 0.f ? 1.f / l_fin : 0.f) * v_unit;
        uint16_t* orow = (uint16_t*)p.out + ((int64_t)tok_out * p.Hq + head_out) * p.Dq;
        if constexpr (EB == 2) {
#pragma unroll
          for (int rt = 0; rt < DPL; ++rt) {
            const u32x2 w = {H::pack(o_acc[rb][rt][0] * inv, o_acc[rb][rt][1] * inv),
                             H::pack(o_acc[rb][rt][2] * inv, o_acc[rb][rt][3] * inv)};
            if (16 * rt + 4 * g4 < p.Dq) *(u32x2*)(orow + 16 * rt + 4 * g4) = w;
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int rt = 0; rt < DPL; rt += 2)
              if (DPL * (4 * g4 + j) + rt < p.Dq)
                *(uint32_t*)(orow + DPL * (4 * g4 + j) + rt) = H::pack(o_acc[rb][rt][j] * inv, o_acc[rb][rt + 1][j] * inv);
        }
      } else {
        const int64_t slot = ((int64_t)cur.slot * p.t_dec_max + cur.part_row + r_tok[rb]) * p.Hq + head_out;
        float* prow = p.part_o + slot * D;
        if constexpr (EB == 2) {
#pragma unroll
          for (int rt = 0; rt < DPL; ++rt) *(f32x4*)(prow + 16 * rt + 4 * g4) = o_acc[rb][rt];
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int rt = 0; rt < DPL; ++rt) prow[DPL * (4 * g4 + j) + rt] = o_acc[rb][rt][j] * v_unit;
        }
        if (g4 == 0) {
          p.part_ml[slot * 2 + 0] = m_run[rb];
          p.part_ml[slot * 2 + 1] = l_tot;
        }
      }
    }
  }
  if (!has_next) break;
  cur = nxt;
  }  // pieces
}

// One block: exclusive prefix sum of the 64-token-rounded key spans of the decode-class sequences
// (the flattened key stream), the per-workgroup span length Q, and each workgroup's first sequence.
// With new_k / new_v set (the fused write + attention call), the blocks after the first copy the new tokens' K/V
// rows into their page slots, one token per wavefront (16 per block): the two jobs do not depend on each other,
// and the attention kernels that follow on the stream see both.
constexpr int kScatterTokensPerBlock = 16;
__global__ __launch_bounds__(1024) void decode_plan_kernel(AttnParams p) {
  if (blockIdx.x > 0) {
    const int t = ((int)blockIdx.x - 1) * kScatterTokensPerBlock + (int)(threadIdx.x >> 6);
    if (t < p.T)
      scatter_token((const char*)p.new_k, (const char*)p.new_v, (char*)p.k_pages, (char*)p.v_pages, p.context_lens,
                    p.block_tables, p.qsl, live_rows(p), p.M, p.P, p.page_size, p.Hkv, p.Dq * elem_bytes_dev(p.kv_dtype),
                    p.head_stride, p.token_stride, p.page_stride, t, threadIdx.x & 63, 64, p.kv_pad_bytes);
    return;
  }
  __shared__ int part[1024], part2[1024];
  __shared__ int s_Q;
  int32_t* plan = p.plan;
  int32_t* P = plan + kPlanHeader;
  const int S = p.S, tid = threadIdx.x;
  const int per = (S + 1023) / 1024;
  const int i0 = min(S, tid * per), i1 = min(S, i0 + per);
  __shared__ int s_large, s_merge, s_reach, s_span_min, s_span_max, s_tiles, s_chunk;
  __shared__ unsigned long long s_work;
  if (tid == 0) {
    s_large = 0;
    s_reach = 0;
    s_work = 0;
    s_span_min = 0x7fffffff;
    s_span_max = 0;
    s_tiles = 0;
    // Does the merge kernel have anything to do?  Rows of padded tokens to zero ...
    const int n_live = live_rows(p);
    s_merge = (n_live <= 0 || p.qsl[0] > 0 || p.qsl[n_live] < p.T) ? 1 : 0;
  }
  __syncthreads();
  auto span_of = [&](int i, const SeqPlan& sp, int& toks) -> int {
    toks = 0;
    if (sp.live && !sp.small_rows) s_large = 1;  // benign race: every writer stores 1
    // ... rows of sequences with tokens but no context to zero, or partial rows of the decode kernel (any sequence of
    // its class may be cut by a span boundary); row tiles of the large-row kernel cut into key chunks are added below
    if (i < live_rows(p) && sp.q_len > 0 && (!sp.live || sp.small_rows)) s_merge = 1;
    if (!sp.live || !sp.small_rows) return 0;
    toks = sp.q_len;
    return (sp.hi - sp.lo + 63) & ~63;
  };
  // Large-row sequences ordered by the length of their workgroups, longest first (the keys an average row tile of
  // theirs visits over the chunks it is cut into): the large-row kernel's workgroups are dealt to the chip in grid
  // order, and the chip then idles for at most the shortest workgroup's time at the end, not the longest's.  One
  // sequence per thread, ranks by counting, once the chunk length is known.
  __shared__ int s_key[kMaxSortedSeqs], s_tiles_of[kMaxSortedSeqs], s_rank_tiles[kMaxSortedSeqs];
  const bool sorted = S <= kMaxSortedSeqs;
  int my_key = -1, my_tiles = 0;
  int sum = 0, tsum = 0, toks;
  unsigned long long work = 0;  // keys the large-row kernel visits per KV head, over its row tiles (an estimate)
  int reach = 0;                // a bound on the keys one of its row tiles visits
  int span_min = 0x7fffffff, span_max = 0, n_tiles = 0;  // of a sequence's average row tile
  const int pre_rows = pre_rows_of(p);
  for (int i = i0; i < i1; ++i) {
    const SeqPlan sp = seq_plan(p, i);
    sum += span_of(i, sp, toks);
    tsum += toks;
    if (sp.live && !sp.small_rows && sp.q_len > 0) {
      const int tile_reach = p.window > 0 ? min(sp.ctx, p.window + pre_rows / p.group + 64) : sp.ctx;
      const int tiles = (sp.q_len * p.group + pre_rows - 1) / pre_rows;
      const int span = max(min(tile_reach, sp.ctx - sp.q_len / 2), 1);  // causal: half the new keys on average
      work += (unsigned long long)tiles * (unsigned)span;
      reach = max(reach, tile_reach);
      span_min = min(span_min, span);
      span_max = max(span_max, span);
      n_tiles += tiles;
      my_key = span;
      my_tiles = tiles;
    }
  }
  if (sorted) {  // (per == 1: thread tid owns sequence tid)
    s_key[tid] = my_key;
    s_tiles_of[tid] = my_tiles;
    s_rank_tiles[tid] = 0;
  }
  if (work) atomicAdd(&s_work, work);
  if (reach) {
    atomicMax(&s_reach, reach);
    atomicMin(&s_span_min, span_min);
    atomicMax(&s_span_max, span_max);
    atomicAdd(&s_tiles, n_tiles);
  }
  part[tid] = sum;
  part2[tid] = tsum;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {  // inclusive Hillis-Steele scans
    const int v = (tid >= off) ? part[tid - off] : 0;
    const int v2 = (tid >= off) ? part2[tid - off] : 0;
    __syncthreads();
    part[tid] += v;
    part2[tid] += v2;
    __syncthreads();
  }
  int run = part[tid] - sum, trun = part2[tid] - tsum;
  for (int i = i0; i < i1; ++i) {
    P[i] = run;
    P[S + 1 + i] = min(trun, max(p.t_dec_max - 1, 0));
    run += span_of(i, seq_plan(p, i), toks);
    trun += toks;
  }
  const int W = part[1023];
  if (tid == 0) {
    P[S] = W;
    // span per workgroup: even split, but never so small that a sequence needs more than max_splits pieces
    int q = ((W + p.n_wg - 1) / p.n_wg + 63) & ~63;
    const int q_min = (((p.M * p.page_size + 64) + (p.max_splits - 2)) / (p.max_splits - 1) + 63) & ~63;
    q = max(max(q, q_min), 256);
    plan[0] = W;
    plan[1] = q;
    // Keys per split-K chunk of the large-row kernel.  Its workgroups are dealt to the chip in grid order as others
    // finish, so the last ones leave part of the chip idle for up to one chunk's time: about four chunks per resident
    // workgroup keep that within a few percent.  Row tiles of (nearly) one length need no more than a whole number
    // of rounds: they are cut into the fewest equal parts that give one, often not at all.
    long long chunk = (long long)1 << 30;
    if (p.pre_max_chunks > 1) {
      chunk = p.pre_chunk;
      if (p.pre_auto) {
        const int slots = max(pre_slots_of(p), 1);
        chunk = (long long)((s_work * (unsigned)p.Hkv / (unsigned)slots / 4 + 63) & ~63ull);
        if (s_tiles > 0 && 4ll * s_span_max <= 5ll * s_span_min) {
          const long long units = (long long)s_tiles * p.Hkv;
          int parts = 1;  // rounds * slots <= 1.08 units * parts
          while (parts < p.pre_max_chunks && ((units * parts + slots - 1) / slots) * slots * 100 > units * parts * 108) ++parts;
          chunk = parts == 1 ? (long long)1 << 30 : ((s_reach + parts - 1) / parts + 63) & ~63;
        }
      }
      chunk = min(max(chunk, (long long)kMinPrefillChunk), (long long)1 << 30);
      if (2ll * s_reach >= 3 * chunk) s_merge = 1;  // a row tile is cut in two from 1.5 chunks on (prefill_tile)
    }
    plan[2] = s_large;  // any sequence for the large-row (prefill) kernel?
    plan[3] = s_merge;  // anything for the merge kernel?
    plan[4] = (int)chunk;
    s_Q = q;
    s_chunk = (int)min(chunk, (long long)0x7fffffff);
  }
  __threadfence_block();
  __syncthreads();
  {
    int32_t* order = plan + kPlanHeader + 2 * (S + 1) + kMaxDecodeWgs;
    int32_t* tile_start = order + kMaxSortedSeqs;
    if (!sorted) {
      if (tid == 0) plan[5] = -1;
    } else if (s_large) {  // (uniform: written before the scans' barriers)
      // the key: the keys one workgroup of the sequence visits, i.e. its span over the number of chunks it is cut into
      // (prefill_tile's rule, on the sequence's average row tile)
      if (my_key >= 0) {
        const int target = s_chunk;
        const int n = min(max((int)(((int64_t)my_key + target / 2) / target), 1), p.pre_max_chunks);
        my_key = (my_key + n - 1) / n;
      }
      s_key[tid] = my_key;
      __syncthreads();
      int rank = 0, n_large = 0;
      for (int j = 0; j < S; ++j) {
        const int kj = s_key[j];
        n_large += kj >= 0;
        rank += (kj > my_key) || (kj == my_key && j < tid);
      }
      if (my_key >= 0) {
        order[rank] = tid;
        s_rank_tiles[rank] = my_tiles;
      }
      __syncthreads();
      if (tid <= n_large) {
        int start = 0;
        for (int r = 0; r < tid; ++r) start += s_rank_tiles[r];
        tile_start[tid] = start;
      }
      if (tid == 0) plan[5] = n_large;
    } else if (tid == 0) {
      plan[5] = 0;
    }
  }
  // first sequence of every workgroup: the last i with P[i] <= j*Q (the kernel then skips empty ones)
  const int Q = s_Q;
  for (int j = tid; j < p.n_wg; j += 1024) {
    const int64_t target = (int64_t)j * Q;
    if (target >= W) { plan[kPlanHeader + 2 * (S + 1) + j] = 0; continue; }
    // First among the threads' groups of `per` sequences, whose running sums are still in LDS (part[c] = the sum up
    // to and including group c; groups past S are empty and sit at W > target), then inside the group in the plan
    // itself: with up to 1024 sequences the search never leaves LDS.
    int clo = 0, chi = 1024;  // invariant: the sum before group clo is <= target; the answer's group is in [clo, chi)
    while (chi - clo > 1) {
      const int mid = (clo + chi) >> 1;
      if (part[mid - 1] <= target) clo = mid; else chi = mid;
    }
    int lo = clo * per, hi = min(S, lo + per);  // invariant: P[lo] <= target; answer in [lo, hi)
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (P[mid] <= target) lo = mid; else hi = mid;
    }
    plan[kPlanHeader + 2 * (S + 1) + j] = lo;
  }
}

// The kernel that serves these template arguments: the LDS-direct one where it applies and the call asks for it.
// It is built for bf16 / float16 pages (every head size, four or eight waves) and for 8-bit pages at head size 128 with eight waves.
template <int D, int KVT, int TT, int WPB>
constexpr bool kHasDecodeDma = (ElemBytes<KVT>::v == 2 && WPB >= 4 && TT == (D == 64 ? 32 : 16)) ||
                               (ElemBytes<KVT>::v == 1 && D == 128 && TT == 32 && WPB == 8);
template <int D, int KVT, int TT, int WPB, bool CAP, int RB>
static bool use_dma(const AttnParams& p) {
  if constexpr (kHasDecodeDma<D, KVT, TT, WPB>) return p.decode_dma != 0 && decode_dma_supported(p);
  else return false;
}

template <int D, int KVT, int TT, int WPB, bool CAP, int RB>
static int launch_rb(hipStream_t stream, AttnParams p) {
  constexpr bool PACE = ElemBytes<KVT>::v == 2 && WPB == 8;
  const bool dma = use_dma<D, KVT, TT, WPB, CAP, RB>(p);
  // persistent grid: as many workgroups as are resident at once, per KV-head group.  The figure belongs to the device
  // the call runs on; it is looked up once per device and kernel (a racing first call computes the same value).
  static std::atomic<int> resident_of[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return (int)hipGetLastError();
  if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
  int resident = resident_of[dev].load(std::memory_order_relaxed);
  if (resident == 0) {
    int cus = 0, per_cu = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return (int)hipGetLastError();
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_decode_kernel<D, KVT, TT, WPB, CAP, RB, PACE>, 64 * WPB, 0) != hipSuccess)
      return (int)hipGetLastError();
    resident = max(1, cus * max(1, per_cu));  // one workgroup per CU for either kernel (registers here, LDS there)
    resident_of[dev].store(resident, std::memory_order_relaxed);
  }
  const int head_groups = (p.Hkv + WPB - 1) / WPB;
  int n_wg = resident / head_groups;
  if (p.decode_wgs > 0) n_wg = p.decode_wgs;
  n_wg = max(1, min(n_wg, kMaxDecodeWgs));
  p.n_wg = n_wg;
  if (p.decode_which & 1) hipLaunchKernelGGL(decode_plan_kernel, dim3(p.new_k ? 1 + (p.T + kScatterTokensPerBlock - 1) / kScatterTokensPerBlock : 1), dim3(1024), 0, stream, p);
  if (p.decode_which & 2) {
    if constexpr (kHasDecodeDma<D, KVT, TT, WPB>) {
      if (dma) {
        hipLaunchKernelGGL((attn_decode_dma_kernel<D, KVT, TT, WPB, CAP, RB>), dim3(n_wg, head_groups), dim3(64 * WPB), 0, stream, p);
        return (int)hipGetLastError();
      }
    }
    hipLaunchKernelGGL((attn_decode_kernel<D, KVT, TT, WPB, CAP, RB, PACE>), dim3(n_wg, head_groups), dim3(64 * WPB), 0, stream, p);
  }
  return (int)hipGetLastError();
}

// Two row blocks per wave exist for bf16 pages up to head size 128 (beyond that the accumulators of the second block do
// not fit the registers of two waves per SIMD); decode_row_limit() below tells the callers which limit applies.
template <int D, int KVT, int TT, int WPB, bool CAP>
static int launch_cap(hipStream_t stream, const AttnParams& p) {
  if constexpr (ElemBytes<KVT>::v == 2 && D <= 128) {
    if (p.dec_rows > kRowBlock) return launch_rb<D, KVT, TT, WPB, CAP, 2>(stream, p);
  }
  return launch_rb<D, KVT, TT, WPB, CAP, 1>(stream, p);
}

template <int D, int KVT, int TT, int WPB>
static int launch_one(hipStream_t stream, const AttnParams& p) {
  return p.softcap > 0.f ? launch_cap<D, KVT, TT, WPB, true>(stream, p) : launch_cap<D, KVT, TT, WPB, false>(stream, p);
}

// Waves (KV heads) per workgroup: as many of 8 / 4 / 2 / 1 as there are heads and as LDS holds tiles for.
// (Four waves per workgroup with more workgroups per CU, and builds for 3 or 4 waves per SIMD, measured no
// faster on the Llama-shaped decode batch; the latter spill.)
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

// Most query rows per KV head (q_len * group) a sequence may have and still be served by the decode kernel, for a
// call with T query tokens over S sequence rows.  A call that cannot hold a multi-token row (T <= S leaves no room
// for one unless other rows are empty) keeps the one-block kernel, which is the faster one on single-token rows.
int decode_row_limit(int T, int S, int D, int kv_dtype) {
  if ((kv_dtype == RPA_BF16 || kv_dtype == RPA_F16) && D <= 128 && T > S) return 2 * kRowBlock;
  return kRowBlock;
}

bool decode_supported(const AttnParams& p) {
  // bf16 queries over bf16 / fp8 / int8 pages, or float16 queries over float16 pages (the MFMA operands of a kernel
  // are of one 16-bit type); float16 pages also need the LDS-direct prefill kernel (its page sizes and offset range,
  // and a call that has not switched it off): it is the only large-row kernel built for them
  if (p.kv_dtype == RPA_F32) return false;
  if (p.kv_dtype == RPA_F16 ? (p.q_dtype != RPA_F16 || !p.prefill_dma || !prefill_dma_supported(p)) : p.q_dtype != RPA_BF16) return false;
  if (p.D != 64 && p.D != 128 && p.D != 256) return false;
  if (p.Dq > p.D || p.Dq % 8 != 0) return false;  // a q row is read in 16-byte chunks, whole chunks inside or outside Dq
  if (p.page_size % 16 != 0) return false;
  if (!(p.scale > 0.f)) return false;  // the MFMA kernels take the running max before scaling
  return true;
}

int launch_attn_decode(hipStream_t stream, const AttnParams& p_in, int which) {
  AttnParams p = p_in;
  p.decode_which = which;
  switch (p.kv_dtype) {
    case RPA_BF16: return launch_kvt<RPA_BF16>(stream, p);
    case RPA_F16: return launch_kvt<RPA_F16>(stream, p);
    case RPA_FP8_E4M3: return launch_kvt<RPA_FP8_E4M3>(stream, p);
    case RPA_INT8: return launch_kvt<RPA_INT8>(stream, p);
    default: return (int)hipErrorInvalidValue;
  }
}

}  // namespace rpa
