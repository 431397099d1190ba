// Split-K decode attention with the K/V tiles moved global -> LDS by the load unit itself
// (global_load_lds_dwordx4), two tiles in flight per wave.  Included by rpa_attn_decode.hip.
//
// Same work split, plan, arithmetic and result layout as attn_decode_kernel: a workgroup takes one equal span of the
// flattened key stream, a wave one KV head and the <= 16 RB query rows that use it.  What differs is how a tile
// reaches LDS.  There a tile passes through registers (load, wait, ds_write), one tile ahead, and the waits are the
// compiler's, which drain every load in flight.  Here every lane hands the load unit one 16-byte global address and
// the unit writes the 64 lanes' chunks to 1 KiB of LDS in lane order; the XOR swizzle of the tile is applied on the
// global side (the lane for LDS chunk c' of row r fetches global chunk c' ^ key(r)).  No register is held while a
// tile is in flight and the kernel states its own waits (s_waitcnt vmcnt(n); loads complete in issue order), so a
// wave keeps two tiles, 16 KiB, in flight where the register kernel keeps 8 KiB: the K half and the V half of a tile
// live in rings of two slots each, K of tile t+2 is issued as soon as the scores of tile t have been computed, V of
// tile t+2 as soon as its P.V product has.  Rows of a tile that nobody may see (past the context, or left of every
// row's window) are not zeroed but fetched from a visible row of the same page, so a NaN in an unused cache slot
// cannot reach 0 x NaN; the mask gives their scores weight zero.
//
// 8-bit pages (fp8 / int8): the raw codes are what lands in LDS, 32 keys a tile; the compute side widens them after
// its LDS reads exactly as attn_decode_kernel does.  The two scales of a tile's page ride behind its K half as one
// more DMA (global_load_lds_dword) into a slot beside the ring, so they are there when the K half is.
//
// The issue side and the compute side walk the same sequence of pieces (token ranges of sequences inside the span),
// each with its own cursor; both read the plan, the lengths and the block table through the constant address space,
// so that these stay scalar loads (after the assembly statements above have "written memory" the compiler would
// otherwise demote them to vector loads and wait for everything in flight).
#pragma once
#include "rpa_mfma.h"

namespace rpa {

typedef const __attribute__((address_space(4))) int32_t* ConstI32;

// A piece as make_piece() cuts it, from constant-address-space metadata, plus the lowest key any of its rows sees.
struct DmaPiece {
  int i, q0, q_len, ctx, part_row, t_begin, t_end, slot, single, flat_end, vis_lo;
};

__device__ __forceinline__ DmaPiece make_piece_dma(const AttnParams& p, ConstI32 P, ConstI32 ctxs, ConstI32 qsl, int i, int pos,
                                                   int span_end, int Q) {
  int p1 = P[i + 1];
  while (p1 <= pos) {  // sequences without decode-class work have zero length
    ++i;
    p1 = P[i + 1];
  }
  const int p0 = P[i];
  DmaPiece pc;
  pc.i = i;
  pc.q0 = qsl[i];
  pc.q_len = qsl[i + 1] - pc.q0;
  pc.ctx = min(ctxs[i], p.M * p.page_size);  // as seq_plan(): never index past the block-table row
  const int first = pc.ctx - pc.q_len - p.window + 1;  // lowest key visible to the first query row, under a window
  pc.vis_lo = (p.window > 0 && first > 0) ? first : 0;
  const int lo = pc.vis_lo & ~63;
  pc.part_row = P[p.S + 1 + i];
  pc.flat_end = min(span_end, p1);
  pc.t_begin = lo + (pos - p0);
  pc.t_end = min(pc.ctx, lo + (pc.flat_end - p0));
  const int j_first = p0 / Q;
  pc.slot = pos / Q - j_first;
  pc.single = (j_first == (p1 - 1) / Q);
  return pc;
}

__device__ const float decode_dma_unit_scales[2] = {1.f, 1.f};  // what unscaled 8-bit pages read as their scales

template <int D, int KVT, int TT, int WPB, bool CAP, int RB>
__global__ __launch_bounds__(64 * WPB, 1) void attn_decode_dma_kernel(AttnParams p) {
  constexpr int EB = ElemBytes<KVT>::v;
  constexpr int HT = KVT == RPA_F16 ? RPA_F16 : RPA_BF16;  // 16-bit float type of the MFMA operands
  using H = Half16<HT>;
  constexpr int RK = D * EB;           // bytes of one K (or V) row
  constexpr int NCH = RK / 16;         // 16-byte chunks per row
  constexpr int RPI = 64 / NCH;        // rows one DMA instruction covers
  constexpr int NLH = TT / RPI;        // DMA instructions per half tile
  constexpr int NS = TT / 16;          // 16-token sub-tiles per tile
  constexpr int DPL = D / 16;          // output dims per lane per accumulator register column
  constexpr int NKK = D / 32;          // k-steps of the score MFMA
  constexpr int VB = DPL * EB;         // bytes of V one lane reads per token (8-bit pages)
  constexpr int HALF = TT * RK;        // bytes of the K (or V) rows of one tile
  constexpr int KN = 2, VN = 2;        // ring slots per wave
  constexpr int SCB = EB == 1 ? 256 : 0;  // bytes of a K slot's scale record (the two floats, repeated over the lanes)
  constexpr int KI = NLH + (EB == 1 ? 1 : 0), VI = NLH;  // DMA instructions of a K half (with its scales) and of a V half
  constexpr int WAVE_LDS = (KN + VN) * HALF + KN * SCB;
  static_assert(RPI >= 1 && TT % RPI == 0 && NCH <= 64, "tile shape");
  static_assert(2 * (KI + VI) <= 63, "the wait counter holds 63 loads");

  __shared__ __attribute__((aligned(1024))) unsigned char lds_all[WPB * WAVE_LDS];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int h = blockIdx.y * WPB + wave;
  if (h >= p.Hkv) return;

  ConstI32 plan = (ConstI32)(uintptr_t)p.plan;
  ConstI32 ctxs = (ConstI32)(uintptr_t)p.context_lens;
  ConstI32 qsl = (ConstI32)(uintptr_t)p.qsl;
  ConstI32 bt = (ConstI32)(uintptr_t)p.block_tables;
  const int W = plan[0], Q = plan[1];
  ConstI32 P = plan + kPlanHeader;
  if ((int64_t)blockIdx.x * Q >= W) return;
  const int span_begin = blockIdx.x * Q;
  const int span_end = min(W, span_begin + Q);

  const int G = p.group;
  const int n = lane & 15;   // query row (column of S^T / O^T)
  const int g4 = lane >> 4;  // token group / k group
  const int pg = p.page_size;

  // ---- LDS: per wave two K slots, two V slots, then (8-bit pages) the scale records of the K slots --------
  unsigned char* lds_wave = lds_all + wave * WAVE_LDS;
  const uint32_t lds_wave_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds_wave;

  // ---- DMA lane mapping: instruction u fills rows u RPI .. + RPI - 1; lane L sits at row + L / NCH, LDS chunk L % NCH
  const int dma_row0 = lane / NCH;
  const int dma_c = lane % NCH;
  // bf16 V rows are swizzled for their transposing reads; 8-bit V rows are read like K rows
  auto key_v = [](int row) { return EB == 2 ? swz_key_v<RK>(row) : swz_key<RK>(row); };
  uint32_t voff_k[NLH], voff_v[NLH];
#pragma unroll
  for (int u = 0; u < NLH; ++u) {
    const int row = u * RPI + dma_row0;
    voff_k[u] = (uint32_t)row * (uint32_t)p.token_stride + (uint32_t)((dma_c ^ swz_key<RK>(row)) << 4);
    voff_v[u] = (uint32_t)row * (uint32_t)p.token_stride + (uint32_t)((dma_c ^ key_v(row)) << 4);
  }
  const char* pages_k = (const char*)p.k_pages + (int64_t)h * p.head_stride;
  const char* pages_v = (const char*)p.v_pages + (int64_t)h * p.head_stride;

  // ---- issue side -------------------------------------------------------------------------------------------
  DmaPiece ip = make_piece_dma(p, P, ctxs, qsl, plan[kPlanHeader + 2 * (p.S + 1) + blockIdx.x], span_begin, span_end, Q);
  int i_tok = ip.t_begin;     // first token of the next tile to issue
  bool i_live = true;         // false once the span's last tile has been issued
  int i_ks = 0, i_vs = 0;     // ring slots the next K / V half goes to
  int n_issued = 0;           // half tiles issued so far: K(t) is number 2t, V(t) number 2t + 1
  int64_t i_off = 0;          // byte offset of the tile whose K half was issued last (its V half follows)
  auto load_page = [&]() -> int { return __builtin_amdgcn_readfirstlane(bt[(int64_t)ip.i * p.M + min(i_tok / pg, p.M - 1)]); };
  int i_page_raw = load_page();  // fetched one issue ahead, clamped when used: no issue waits for a load it has just made
  auto issue_half = [&](bool is_v, int slot) __attribute__((always_inline)) {
    const char* base = (is_v ? pages_v : pages_k) + i_off;
    const uint32_t lds = lds_wave_addr + (uint32_t)(((is_v ? KN : 0) + slot) * HALF);
    const bool edge = (i_tok + TT > ip.ctx) || (i_tok < ip.vis_lo);
    if (!edge) {
#pragma unroll
      for (int u = 0; u < NLH; ++u) dma16_nt(lds + u * 1024, is_v ? voff_v[u] : voff_k[u], base);
    } else {
#pragma unroll
      for (int u = 0; u < NLH; ++u) {  // rows nobody may see: a visible row's bytes (same page: pages hold whole 64-token groups)
        const int row = u * RPI + dma_row0;
        const int r = min(max(i_tok + row, ip.vis_lo), ip.ctx - 1) - i_tok;
        const uint32_t off = (uint32_t)r * (uint32_t)p.token_stride + (uint32_t)((dma_c ^ (is_v ? key_v(row) : swz_key<RK>(row))) << 4);
        dma16_nt(lds + u * 1024, off, base);
      }
    }
    ++n_issued;
  };
  auto issue_k = [&]() __attribute__((always_inline)) {
    if (!i_live) return;
    const int page = min(max(i_page_raw, 0), p.P - 1);
    i_off = (int64_t)page * p.page_stride + (int64_t)(i_tok % pg) * p.token_stride;
    issue_half(false, i_ks);
    if constexpr (EB == 1) {  // the page's (K scale, V scale) of this head, behind the K rows
      const float* sc = p.kv_scales ? p.kv_scales + (int64_t)page * p.C + 2 * h : decode_dma_unit_scales;
      dma4(lds_wave_addr + (uint32_t)((KN + VN) * HALF + i_ks * SCB), (uint32_t)((lane & 1) << 2), sc);
    }
    i_ks ^= 1;
  };
  auto issue_v = [&]() __attribute__((always_inline)) {
    if (!i_live) return;
    issue_half(true, i_vs);
    i_vs ^= 1;
    i_tok += TT;
    if (i_tok >= ip.t_end) {
      if (ip.flat_end < span_end) {
        ip = make_piece_dma(p, P, ctxs, qsl, ip.i + 1, ip.flat_end, span_end, Q);
        i_tok = ip.t_begin;
      } else {
        i_live = false;
      }
    }
    if (i_live) i_page_raw = load_page();
  };
  // Waits for half tile number j (a V half if is_v): every half issued after it may still be in flight, and halves
  // alternate K, V, K, ...
  auto wait_half = [&](auto is_v, int j) __attribute__((always_inline)) {
    constexpr int A = decltype(is_v)::value ? KI : VI, B = decltype(is_v)::value ? VI : KI;  // the next half's loads, and the one after
    const int later = n_issued - 1 - j;
    if (later >= 3) wait_loads<2 * A + B>();
    else if (later == 2) wait_loads<A + B>();
    else if (later == 1) wait_loads<A>();
    else wait_loads<0>();
  };
  const std::false_type k_half{};
  const std::true_type v_half{};

  issue_k();
  issue_v();
  if (p.decode_dma != 2) {  // 2: one tile ahead only (a measurement setting)
    issue_k();
    issue_v();
  }

  const float cap_out = p.softcap * 1.4426950408889634f;
  const float cap_in = CAP ? p.scale / p.softcap : 0.f;

  // ---- compute side ------------------------------------------------------------------------------------------
  DmaPiece cur = make_piece_dma(p, P, ctxs, qsl, plan[kPlanHeader + 2 * (p.S + 1) + blockIdx.x], span_begin, span_end, Q);
  int tg = 0;  // tiles computed so far in the span: tile tg lives in ring slots tg & 1
  for (;;) {
    const int rows = cur.q_len * G;
    const int t_begin = cur.t_begin;
    const int n_tiles = (cur.t_end - t_begin + TT - 1) / TT;

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
    // keys every row sees: from the last row's window start to the first row's causal limit
    const int all_lo = (p.window > 0) ? max(cur.ctx - p.window, 0) : 0;
    const int all_hi = cur.ctx - cur.q_len + 1;

    // ---- Q as B operands: step kk covers dims 32kk + 8g4 + e
    u32x4 qf[RB][NKK];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const char* qrow = (const char*)p.q + ((int64_t)(cur.q0 + r_tok[rb]) * p.Hq + (h * G + r_head[rb])) * p.Dq * 2;
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        // bf16 pages: step kk covers dims 32kk + 8g4 + e.  8-bit pages: a 16-byte K chunk holds 16 dims, so steps
        // (2j, 2j+1) cover dims 64j + 16g4 + 8b + e.
        const int d0 = (EB == 2) ? (kk * 32 + 8 * g4) : ((kk >> 1) * 64 + 16 * g4 + 8 * (kk & 1));
        u32x4 v = {0u, 0u, 0u, 0u};
        if (n + 16 * rb < rows && d0 < p.Dq) v = *(const u32x4*)(qrow + d0 * 2);  // dims past Dq: zero padding
        qf[rb][kk] = v;
      }
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

    for (int tile = 0; tile < n_tiles; ++tile, ++tg) {
      const int tb = t_begin + tile * TT;
      // The waves of a workgroup read adjacent spans of the same token rows; a barrier every few tiles keeps them in
      // step so each DRAM row is opened once.  All waves of a workgroup walk the same pieces and tiles.
      if (p.decode_sync > 0 && (tile & (p.decode_sync - 1)) == 0) __builtin_amdgcn_s_barrier();
      const unsigned char* lds_k = lds_wave + (tg & 1) * HALF;
      const unsigned char* lds_v = lds_wave + (KN + (tg & 1)) * HALF;

      // ---- S^T = K . Q^T ------------------------------------------------------------------------------------
      wait_half(k_half, 2 * tg);
      float k_scale = 1.f, v_scale = 1.f;
      if constexpr (EB == 1) {
        const float* sc = (const float*)(lds_wave + (KN + VN) * HALF + (tg & 1) * SCB);
        k_scale = sc[0];
        v_scale = sc[1];
      }
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
      // The scores are in registers: this K slot is free for tile tg + 2.  (Using the accumulators here makes the
      // compiler finish the LDS reads that feed them before the loads below are issued.)
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int st = 0; st < NS; ++st) asm volatile("" : "+v"(s_acc[rb][st]));
      if (p.decode_dma != 3) issue_k();

      // ---- online softmax (log2 domain) ---------------------------------------------------------------------
      const float sc_mul = CAP ? cap_out : p.scale_log2 * k_scale;
      uint32_t pfrag[RB][NS][2];
      // 8-bit pages: the accumulators hold sum(p * v_code) in units of the current page's V scale, so P stays an exact
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

      // ---- O^T += V^T . P^T: ds_read_b64_tr_b16 hands each lane the key-major column it needs ------------------
      wait_half(v_half, 2 * tg + 1);
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
          const int key = swz_key_v<RK>(tk);
#pragma unroll
          for (int rt = 0; rt < DPL; ++rt) {
            const int off = rt * 32 + (n & 3) * 8;
            const unsigned char* ptr = vrow + (((off >> 4) ^ key) << 4) + (off & 15);
            const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)ptr);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) o_acc[rb][rt] = H::mfma16(__builtin_bit_cast(u32x2, a), pb[rb], o_acc[rb][rt]);
          }
        } else {
          // lane (n, g4) reads DPL consecutive dims (DPL*n ..) of keys 4g4..4g4+3 and widens them; row tile rt of this
          // path therefore holds dims DPL*i + rt (any dim permutation works for O^T, see the epilogue)
          static_assert(EB == 2 || VB == 8 || VB == 4 || VB % 16 == 0, "V bytes per lane");
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
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) asm volatile("" : "+v"(o_acc[rb][rt]));
      if (p.decode_dma == 3) issue_k();  // a measurement setting: both halves of a tile asked for at the same moment
      issue_v();
    }

    // ---- epilogue: accumulator column j of row tile rt is dim 16rt + 4g4 + j (bf16 pages) or DPL (4g4 + j) + rt (8-bit)
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
    if (cur.flat_end >= span_end) break;
    cur = make_piece_dma(p, P, ctxs, qsl, cur.i + 1, cur.flat_end, span_end, Q);
  }  // pieces
}

// 16-bit or 8-bit pages whose size is a multiple of 64 tokens (a tile's unseen rows borrow a visible row of the same page,
// and the lowest visible key of a sequence lies in the 64-token group its first tile starts), four or more KV heads,
// and tiles that a 32-bit byte offset can address.
inline bool decode_dma_supported(const AttnParams& p) {
  return p.kv_dtype != RPA_F32 && p.page_size % 64 == 0 && p.Hkv >= 4 && (int64_t)64 * p.token_stride < ((int64_t)1 << 31);
}

}  // namespace rpa
