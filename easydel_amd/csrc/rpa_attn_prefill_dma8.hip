// MFMA prefill / chunked-prefill attention for 8-bit pages (fp8-e4m3 or int8 codes, with or without per-page scales),
// on the LDS-direct tile pipeline of attn_prefill_dma_kernel (rpa_attn_prefill_dma.hip).
//
// Work split, score / softmax / P.V arithmetic, software pipeline and the split over key chunks are those of
// attn_prefill_dma_kernel; see there.  The tiles it computes on are bf16 as there; what differs is where they come
// from.  The load unit (global_load_lds_dwordx4) moves the codes of a tile -- 32 rows of D bytes for K, as many for
// V -- into a ring in LDS, three tiles ahead, together with the two scales of the tile's page; each wave moves a
// quarter (an eighth at head size 256) of the rows and, two steps before the tile is needed, widens exactly those
// rows into the bf16 tile the whole workgroup then reads in MFMA operand order (the swizzle is applied by the write).
// A wave therefore waits only for loads of its own (s_waitcnt vmcnt(n), stated by the kernel) and the step keeps
// its single barrier.  Widening is exact (both code sets fit bf16); the K scale of a tile rides on its score scale, and
// the accumulators are kept in units of the current page's V scale (converted when the page changes), so that the
// probabilities stay exact softmax weights.
#include <type_traits>

#include "rpa_mfma.h"

namespace rpa {

// Two floats of ones: what unscaled 8-bit pages use in place of a page's (K scale, V scale).
__device__ const float ones2[2] = {1.f, 1.f};


template <int D, int KVT, int NW, int RB, bool CAP>
__global__ __launch_bounds__(64 * NW, 2) void attn_prefill_dma8_kernel(AttnParams p) {
  constexpr int TT = 32;                 // keys per tile
  constexpr int RKL = D * 2;             // bytes of one K (or V) row of a bf16 tile
  constexpr int RAW = D;                 // bytes of one K (or V) row of codes
  constexpr int CPR = RAW / 16;          // 16-byte chunks per row of codes
  constexpr int RPI = 64 / CPR;          // rows one DMA instruction covers
  static_assert(RPI * NW == TT, "one DMA instruction per wave moves its share of a half tile: the rows it later widens");
  constexpr int NS = TT / 16;            // 16-key sub-tiles per tile
  constexpr int DPL = D / 16;            // 16-dim row tiles of O^T
  constexpr int NKK = D / 32;            // k-steps of the score MFMA
  constexpr int ROWS = NW * RB * 16;
  constexpr float kMaxSlack = 8.f;       // how far a score may exceed the softmax reference before it is raised
  static_assert(ROWS == kPrefillRows, "merge kernel assumes this row-tile height");
  constexpr int HALF = TT * RKL;         // bytes of the K (or V) rows of one bf16 tile
  constexpr int RAWH = TT * RAW;         // bytes of the K (or V) rows of one tile of codes
  // bf16 tiles: K(t+2) is written while K(t+1) is read, V(t+2) while V(t+1) waits and V(t) is read, and V(t-1) may
  // still be read by a wave that lags: two K slots, four V slots.  Codes: a ring of RN tiles in flight, wave-private.
  constexpr int KN = 2, VN = 4, RN = 3;
  constexpr int kRawBase = (KN + VN) * HALF;
  constexpr int kScaleBase = kRawBase + RN * 2 * RAWH;  // per wave and ring slot 256 bytes: (K scale, V scale) of the tile's page

  __shared__ __attribute__((aligned(1024))) unsigned char lds_all[kScaleBase + NW * RN * 256];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g4 = lane >> 4;
  const int G = p.group;

  // ---- block -> (sequence, row tile, KV head, key chunk) ---------------------------------------------
  const int h = blockIdx.x % p.Hkv;
  const int n_slots = gridDim.x / (p.Hkv * p.pre_max_chunks);
  const int slot = (blockIdx.x / p.Hkv) % n_slots;
  const int chunk = blockIdx.x / (p.Hkv * n_slots);  // slowest: neighbouring blocks share a key chunk (L2 reuse)
  if (p.plan[2] == 0) return;  // the plan kernel saw no sequence with more than 16 rows per KV head
  if (wide_mode(p)) return;    // this batch's large rows are served from bf16 copies of their pages, by the 32x32-tile kernel
  const int n_live = live_rows(p);
  if (n_live <= 0) return;
  // sequence i starts at slot floor(qsl[i]*G/ROWS) + i; find the last sequence starting at or before `slot`
  int lo_i = 0, hi_i = n_live;
  while (hi_i - lo_i > 1) {
    const int mid = (lo_i + hi_i) >> 1;
    if ((int)(((int64_t)p.qsl[mid] * G) / ROWS) + mid <= slot) lo_i = mid; else hi_i = mid;
  }
  const int i = lo_i;
  const SeqPlan sp = seq_plan(p, i);
  if (!sp.live || sp.small_rows) return;
  const int tile_in_seq = slot - ((int)(((int64_t)sp.q0 * G) / ROWS) + i);
  const int rows_total = sp.q_len * G;
  const int R0 = tile_in_seq * ROWS;
  if (tile_in_seq < 0 || R0 >= rows_total) return;

  // ---- key range of the workgroup: one chunk of the row tile's range ----------------------------
  const PrefillTile pt = prefill_tile(p, sp, R0);
  if (pt.n_chunks == 0 && chunk == 0) {  // every row of the tile lies before position 0 and sees no key: zeros
    for (int e = tid; e < ROWS * (p.Dq / 4); e += 64 * NW) {
      const int row = R0 + e / (p.Dq / 4), d4 = e % (p.Dq / 4);
      if (row < rows_total)
        *(u32x2*)((uint16_t*)p.out + ((int64_t)(sp.q0 + row / G) * p.Hq + h * G + row % G) * p.Dq + 4 * d4) = (u32x2){0u, 0u};
    }
    return;
  }
  if (chunk >= pt.n_chunks) return;
  const int base_pos = sp.ctx - sp.q_len;  // position of the sequence's first query token
  const int vis_lo = pt.vis_lo;
  // the first tile must hold vis_lo, so that rows of it that nobody may see can borrow a visible row's address
  const int kv_lo = max(pt.kv_lo + chunk * pt.chunk_len, vis_lo & ~(TT - 1));
  const int kv_hi = (chunk == pt.n_chunks - 1) ? pt.kv_hi : pt.kv_lo + (chunk + 1) * pt.chunk_len;
  const int n_tiles = (kv_hi - kv_lo + TT - 1) / TT;
  const bool single = pt.n_chunks == 1;

  // ---- per row-block lane state --------------------------------------------------------------------
  int row_lo[RB], row_hi[RB];
  bool row_ok[RB];
  int out_tok[RB], out_head[RB];
  bf16x8 qf[RB][NKK];
  int wave_lo, wave_hi;          // keys every row of the wave sees: [max row_lo, min row_hi)
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = R0 + (wave * RB + rb) * 16 + n;
    row_ok[rb] = row < rows_total;
    const int r_tok = row_ok[rb] ? row / G : (rows_total - 1) / G;  // padded rows shadow the last row
    const int r_head = row_ok[rb] ? row - r_tok * G : 0;
    const int pos = base_pos + r_tok;
    row_hi[rb] = min(pos + 1, sp.ctx);
    row_lo[rb] = (p.window > 0) ? max(pos - p.window + 1, 0) : 0;
    out_tok[rb] = sp.q0 + r_tok;
    out_head[rb] = h * G + r_head;
    const char* qrow = (const char*)p.q + ((int64_t)out_tok[rb] * p.Hq + out_head[rb]) * p.Dq * 2;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok[rb] && kk * 32 + 8 * g4 < p.Dq) v = *(const u32x4*)(qrow + (kk * 32 + 8 * g4) * 2);  // dims past Dq: zero padding
      qf[rb][kk] = __builtin_bit_cast(bf16x8, v);
    }
  }
  // Use the query registers once here, so that the compiler waits for these loads now and not at their first use
  // inside the loop, where its wait would also cover every tile in flight.
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      u32x4 v = __builtin_bit_cast(u32x4, qf[rb][kk]);
      asm volatile("" : "+v"(v));
      qf[rb][kk] = __builtin_bit_cast(bf16x8, v);
    }
  {
    int lo_max = 0, hi_min = 0x7fffffff;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      lo_max = max(lo_max, row_lo[rb]);
      hi_min = min(hi_min, row_hi[rb]);
    }
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) {
      lo_max = max(lo_max, __shfl_xor(lo_max, o));
      hi_min = min(hi_min, __shfl_xor(hi_min, o));
    }
    wave_lo = __builtin_amdgcn_readfirstlane(lo_max);
    wave_hi = __builtin_amdgcn_readfirstlane(hi_min);
  }

  // ---- tile loads ------------------------------------------------------------------------------------
  // Wave w moves rows w RPI .. + RPI - 1 of the K codes of a tile with one DMA instruction (lane L: row + L / CPR,
  // chunk L % CPR, unswizzled: only this wave reads them back), the same rows of the V codes with a second, and
  // the two scales of the tile's page with a third (every lane fetches one of the two floats; they land in the
  // wave's own 256 bytes of the scale ring).  The block table is read through the constant address space: it does not
  // change while the kernel runs, and only so may the compiler keep these loads scalar after the assembly statements
  // have "written memory".
  typedef const __attribute__((address_space(4))) int32_t* ConstI32;
  ConstI32 bt = (ConstI32)(uintptr_t)(p.block_tables + (int64_t)i * p.M);
  const char* k_pages = (const char*)p.k_pages;
  const char* v_pages = (const char*)p.v_pages;
  const int pg = p.page_size;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds_all;
  const int dma_row = wave * RPI + lane / CPR;  // the tile row this lane moves, and later widens
  const int dma_chunk = lane % CPR;
  const uint32_t voff_raw = (uint32_t)dma_row * (uint32_t)p.token_stride + (uint32_t)(dma_chunk << 4);
  const uint32_t voff_scale = (uint32_t)(lane & 1) * 4u;
  int cur_idx = kv_lo / pg;
  int cur_off = kv_lo - cur_idx * pg;
  int cur_tb = kv_lo;
  int cur_rs = 0;    // ring slot of the tile the cursor is at
  int n_issued = 0;  // tiles issued so far
  auto load_page = [&](int idx) -> int { return __builtin_amdgcn_readfirstlane(bt[min(idx, p.M - 1)]); };
  int cur_page_raw = load_page(cur_idx);
  auto issue = [&]() __attribute__((always_inline)) {  // starts the DMA of the cursor's tile into its ring slot and advances the cursor
    const int cur_page = min(max(cur_page_raw, 0), p.P - 1);
    const int64_t tile_off = (int64_t)cur_page * p.page_stride + (int64_t)cur_off * p.token_stride + (int64_t)h * p.head_stride;
    const bool edge = (cur_tb + TT > sp.ctx) || (cur_tb < vis_lo);
    const uint32_t raw_lds = lds_base + kRawBase + (uint32_t)cur_rs * (2 * RAWH) + (uint32_t)wave * 1024u;
    uint32_t voff = voff_raw;
    if (edge) {  // keys nobody may see: any visible row's bytes
      const int r = min(max(cur_tb + dma_row, vis_lo), sp.ctx - 1) - cur_tb;
      voff = (uint32_t)r * (uint32_t)p.token_stride + (uint32_t)(dma_chunk << 4);
    }
    dma16(raw_lds, voff, k_pages + tile_off);
    dma16(raw_lds + RAWH, voff, v_pages + tile_off);
    const float* sc = p.kv_scales ? p.kv_scales + (int64_t)cur_page * p.C + 2 * h : nullptr;
    dma4(lds_base + kScaleBase + (uint32_t)(wave * RN + cur_rs) * 256u, voff_scale, sc ? (const void*)sc : (const void*)ones2);
    cur_tb += TT;
    cur_off += TT;
    if (cur_off >= pg) {
      cur_off -= pg;
      ++cur_idx;
    }
    cur_rs = (cur_rs == RN - 1) ? 0 : cur_rs + 1;
    cur_page_raw = load_page(cur_idx);
    ++n_issued;
  };
  // ---- codes -> bf16 tile: every wave widens the rows it moved (exactly: both code sets fit bf16) ------------------------
  int cv_rs = 0;  // ring slot of the next tile to widen
  auto convert = [&](int tau, float& k_scale_out, float& v_scale_out) __attribute__((always_inline)) {
    const int later = n_issued - 1 - tau;  // tiles issued after it, which may stay in flight (three instructions each)
    if (later >= 2) wait_loads<6>();
    else if (later == 1) wait_loads<3>();
    else wait_loads<0>();
    const unsigned char* raw = lds_all + kRawBase + cv_rs * (2 * RAWH) + wave * 1024 + lane * 16;
    const u32x4 ck = *(const u32x4*)raw;
    const u32x4 cv = *(const u32x4*)(raw + RAWH);
    const float2 sc = *(const float2*)(lds_all + kScaleBase + (wave * RN + cv_rs) * 256);
    k_scale_out = sc.x;
    v_scale_out = sc.y;
    unsigned char* krow = lds_all + (tau & (KN - 1)) * HALF + dma_row * RKL;
    unsigned char* vrow = lds_all + (KN + (tau & (VN - 1))) * HALF + dma_row * RKL;
    const int kkey = swz_key<RKL>(dma_row), vkey = swz_key_v<RKL>(dma_row);
#pragma unroll
    for (int e = 0; e < 2; ++e) {  // codes 8e .. 8e + 7 of the lane's sixteen: chunk 2 dma_chunk + e of the bf16 row
      *(u32x4*)(krow + (((2 * dma_chunk + e) ^ kkey) << 4)) = codes8_to_bf16x8<KVT>(ck[2 * e], ck[2 * e + 1]);
      *(u32x4*)(vrow + (((2 * dma_chunk + e) ^ vkey) << 4)) = __builtin_bit_cast(u32x4, codes8_to_bf16x8<KVT>(cv[2 * e], cv[2 * e + 1]));
    }
    cv_rs = (cv_rs == RN - 1) ? 0 : cv_rs + 1;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the codes are in registers: their ring slot may be refilled
    if (tau + RN < n_tiles) issue();
  };

  const float cap_out = p.softcap * 1.4426950408889634f;
  const float cap_in = CAP ? p.scale / p.softcap : 0.f;

  float m_run[RB];
  f32x4 l_acc[RB];  // row sums, replicated over the four elements (see soft_pv)
  f32x4 o_acc[RB][DPL];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    m_run[rb] = -INFINITY;
    l_acc[rb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int rt = 0; rt < DPL; ++rt) o_acc[rb][rt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  // ---- S^T = K . Q^T for every row block (K operands shared) ------------------------------------------
  // K operand i = (16-key sub-tile i / NKK, k-step i % NKK).  The first KPD operands of a tile are read a phase
  // early (k_prefetch, behind the PV MFMAs of the tile before), the rest KPD operands ahead of their MFMAs.
  constexpr int NKO = NS * NKK;
  constexpr int KPD = NKO < 4 ? NKO : 4;
  auto read_k = [&](const unsigned char* lds_k, int i) __attribute__((always_inline)) -> u32x4 {
    const int tk = (i / NKK) * 16 + n;
    return *(const u32x4*)(lds_k + tk * RKL + ((((i % NKK) * 4 + g4) ^ swz_key<RKL>(tk)) << 4));
  };
  auto k_prefetch = [&](const unsigned char* lds_k, u32x4 (&kp)[KPD]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < KPD; ++i) kp[i] = read_k(lds_k, i);
  };
  auto qk = [&](const unsigned char* lds_k, u32x4 (&kp)[KPD], f32x4 (&sa)[RB][NS]) __attribute__((always_inline)) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int st = 0; st < NS; ++st) sa[rb][st] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < NKO; ++i) {
      const u32x4 a = kp[i % KPD];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
        sa[rb][i / NKK] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), qf[rb][i % NKK], sa[rb][i / NKK], 0, 0, 0);
      if (i + KPD < NKO) kp[i % KPD] = read_k(lds_k, i + KPD);
    }
  };
  // ---- online softmax of the scores of tile tb ----------------------------------------------------------
  auto softmax = [&](auto mask_tag, f32x4 (&sa)[RB][NS], int tb, uint32_t (&pfrag)[RB][NS][2], float k_scale) __attribute__((always_inline)) {
    constexpr bool MASK = decltype(mask_tag)::value;
    const float sc_mul = CAP ? cap_out : p.scale_log2 * k_scale;  // the K scale of the tile's page rides on the score scale
    const float cap_in_k = cap_in * k_scale;
    // Soft cap and mask in place; each lane's maximum over its own 8 keys of the row.
    float lmx[RB];
    bool grow = false;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      lmx[rb] = -INFINITY;
#pragma unroll
      for (int st = 0; st < NS; ++st)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float sv = sa[rb][st][j];
          if constexpr (CAP) sv = fast_tanh(sv * cap_in_k);
          if constexpr (MASK) {
            const int tok = tb + st * 16 + 4 * g4 + j;
            sv = (tok >= row_lo[rb] && tok < row_hi[rb]) ? sv : -INFINITY;
          }
          sa[rb][st][j] = sv;
          lmx[rb] = fmaxf(lmx[rb], sv);
        }
      lmx[rb] *= sc_mul;  // sc_mul > 0: scaling commutes with the maximum
      grow |= lmx[rb] > m_run[rb] + kMaxSlack;
    }
    // The reference every probability of a row is taken against need not be the exact running maximum: any common
    // value works as long as exp2 stays in range, the quotient of the two accumulated sums does not depend on it.
    // It is raised -- the lanes of a row agree on the new maximum and everything accumulated so far is scaled down --
    // only when some key of the tile exceeds it by more than kMaxSlack (in log2 units, so probabilities stay below
    // 2^kMaxSlack).  After the first tiles of a sequence that is rare, and a tile then costs neither the lane
    // exchange nor a rescale.
    if (__any(grow)) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const float m_new = fmaxf(m_run[rb], xor32_max(xor16_max(lmx[rb])));
        const float m_use = (MASK && m_new == -INFINITY) ? 0.f : m_new;
        float alpha = __builtin_amdgcn_exp2f(m_run[rb] - m_use);
        m_run[rb] = m_new;
        // The multiplications below are opaque to the compiler, so it does not pad the distance this chip wants
        // between a transcendental instruction and a reader of its result; the padding is put here by hand.
        asm volatile("s_nop 1" : "+v"(alpha));
        // In place, through assembly: left to the compiler, the two arms of this branch meet in a second copy of the
        // accumulators, which costs their registers again and a move of each on every tile.
#pragma unroll
        for (int j = 0; j < 4; ++j) asm("v_mul_f32 %0, %1, %0" : "+v"(l_acc[rb][j]) : "v"(alpha));
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt)
#pragma unroll
          for (int j = 0; j < 4; ++j) asm("v_mul_f32 %0, %1, %0" : "+v"(o_acc[rb][rt][j]) : "v"(alpha));
      }
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const float m_use = (MASK && m_run[rb] == -INFINITY) ? 0.f : m_run[rb];
#pragma unroll
      for (int st = 0; st < NS; ++st) {
        float pr[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) pr[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(sa[rb][st][j], sc_mul, -m_use));
        pfrag[rb][st][0] = pack_bf16(pr[0], pr[1]);
        pfrag[rb][st][1] = pack_bf16(pr[2], pr[3]);
      }
    }
  };
  // ---- O^T += V^T . P^T, and the row sums ------------------------------------------------------------------
  auto pv = [&](uint32_t (&pfrag)[RB][NS][2], const unsigned char* lds_v) __attribute__((always_inline)) {
    // The row sums come from the matrix cores as well: a V^T tile of ones times P^T leaves, in every accumulator
    // element of column n, the sum of row n's probabilities over all 32 keys (as rounded to bf16, i.e. exactly the
    // weights the PV product uses).  Two MFMAs replace 16 additions per lane and the cross-lane sum at the end.
    {
      const u32x4 ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const u32x4 b4 = {pfrag[rb][0][0], pfrag[rb][0][1], pfrag[rb][1][0], pfrag[rb][1][1]};
        l_acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ones), __builtin_bit_cast(bf16x8, b4), l_acc[rb], 0, 0, 0);
      }
    }
    // ds_read_b64_tr_b16: inside a 16-lane group, lane l supplies the address of 4 consecutive bf16
    // (key 4g4 + l/4, dims d0 + 4(l%4)..) and receives the transposed column: for dim d0 + (l&15) the
    // values of keys 4g4..4g4+3, which is the A operand of the product with k = keys.
    const int tr_key = 4 * g4 + (n >> 2);          // key (within a 16-key sub-tile) this lane addresses
    const int tr_byte = (n & 3) * 8;               // byte offset of its 4 dims inside the 32-byte row-tile span
    // The V operands are read PD row tiles ahead of the MFMAs that use them: one row tile of MFMAs lasts 32 cycles,
    // an LDS read under load several times that, so a wave that reads just in time waits at every row tile.
    constexpr int PD = DPL < 4 ? DPL : 4;
    auto read_v = [&](int rt) -> u32x4 {
      const int off = rt * 32 + tr_byte;
      const unsigned char* lo = lds_v + tr_key * RKL + (((off >> 4) ^ swz_key_v<RKL>(tr_key)) << 4) + (off & 15);
      const unsigned char* hi = lds_v + (16 + tr_key) * RKL + (((off >> 4) ^ swz_key_v<RKL>(16 + tr_key)) << 4) + (off & 15);
      const u32x2 a_lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)lo));
      const u32x2 a_hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)hi));
      return (u32x4){a_lo[0], a_lo[1], a_hi[0], a_hi[1]};
    };
    __builtin_amdgcn_sched_barrier(0);  // keep the V operand reads out of the softmax: they would only pile up in registers
    u32x4 av[PD];
#pragma unroll
    for (int rt = 0; rt < PD; ++rt) av[rt] = read_v(rt);
#pragma unroll
    for (int rt = 0; rt < DPL; ++rt) {
      const u32x4 a4 = av[rt % PD];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const u32x4 b4 = {pfrag[rb][0][0], pfrag[rb][0][1], pfrag[rb][1][0], pfrag[rb][1][1]};
        o_acc[rb][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a4), __builtin_bit_cast(bf16x8, b4),
                                                                o_acc[rb][rt], 0, 0, 0);
      }
      if (rt + PD < DPL) av[rt % PD] = read_v(rt + PD);
    }
    // The order the scheduler must keep: PD row tiles of reads first, then a row tile of MFMAs and the next reads in turn.
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * PD, 0);
#pragma unroll
    for (int rt = 0; rt + PD < DPL; ++rt) {
      __builtin_amdgcn_sched_group_barrier(0x008, RB, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, RB * PD, 0);
  };
  // ---- pipeline ----------------------------------------------------------------------------------------
  // Step t: the matrix cores compute the scores of tile t+1 while the vector ALU does the softmax of tile t; then
  // every wave widens its rows of tile t+2 (whose codes it waits for itself: it moved them) and refills the ring slot;
  // behind the step's barrier tile t+2 is visible: its first K operands are read, and the P.V product of tile t runs.
  auto k_slot = [&](int tau) -> const unsigned char* { return lds_all + (tau & (KN - 1)) * HALF; };
  auto v_slot = [&](int tau) -> const unsigned char* { return lds_all + (KN + (tau & (VN - 1))) * HALF; };
  const std::true_type masked{};
  f32x4 s_cur[RB][NS], s_nxt[RB][NS];
  uint32_t pf[RB][NS][2];
  u32x4 kp[KPD];
  float ks0 = 1.f, ks1 = 1.f, ks2 = 1.f;  // K scales of tiles t, t+1, t+2
  float vs0 = 1.f, vs1 = 1.f, vs2 = 1.f;  // and their V scales
  float v_unit = 1.f;                      // the V scale the accumulators are currently expressed in
  // Before the P.V product of a tile whose page has another V scale the accumulators change units, in place (through
  // assembly, for the reason given at the softmax's rescale).
  auto to_unit = [&](float v_scale) __attribute__((always_inline)) {
    if (v_scale != v_unit) {  // the same in every lane
      float f = v_unit * __builtin_amdgcn_rcpf(v_scale);
      asm volatile("s_nop 1" : "+v"(f));
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt)
#pragma unroll
          for (int j = 0; j < 4; ++j) asm("v_mul_f32 %0, %1, %0" : "+v"(o_acc[rb][rt][j]) : "v"(f));
      v_unit = v_scale;
    }
  };
  {
    const int n_pro = min(n_tiles, RN);
    for (int k = 0; k < n_pro; ++k) issue();
  }
  convert(0, ks0, vs0);
  if (n_tiles > 1) convert(1, ks1, vs1);
  asm volatile("s_barrier" ::: "memory");
  k_prefetch(k_slot(0), kp);
  qk(k_slot(0), kp, s_cur);
  if (n_tiles > 1) k_prefetch(k_slot(1), kp);
  int t = 0;
  auto run = [&](auto mask_tag, int t_end) __attribute__((always_inline)) {
    for (; t < t_end; ++t) {  // t + 2 < n_tiles
      qk(k_slot(t + 1), kp, s_nxt);
      softmax(mask_tag, s_cur, kv_lo + t * TT, pf, ks0);
      convert(t + 2, ks2, vs2);
      asm volatile("s_barrier" ::: "memory");
      k_prefetch(k_slot(t + 2), kp);
      to_unit(vs0);
      pv(pf, v_slot(t));
      ks0 = ks1;
      ks1 = ks2;
      vs0 = vs1;
      vs1 = vs2;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int st = 0; st < NS; ++st) s_cur[rb][st] = s_nxt[rb][st];
    }
  };
  const int t_plain_lo = max(0, (wave_lo - kv_lo + TT - 1) / TT);  // first tile no row of the wave masks from below
  const int t_plain_hi = (wave_hi - kv_lo) / TT;                   // first tile some row of the wave masks from above
  run(masked, min(t_plain_lo, n_tiles - 2));
  run(std::false_type{}, min(t_plain_hi, n_tiles - 2));
  run(masked, n_tiles - 2);
  if (n_tiles > 1) {  // t = n_tiles - 2: the last scores; every tile is widened and visible
    qk(k_slot(t + 1), kp, s_nxt);
    softmax(masked, s_cur, kv_lo + t * TT, pf, ks0);
    to_unit(vs0);
    pv(pf, v_slot(t));
    ks0 = ks1;
    vs0 = vs1;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int st = 0; st < NS; ++st) s_cur[rb][st] = s_nxt[rb][st];
    ++t;
  }
  softmax(masked, s_cur, kv_lo + t * TT, pf, ks0);  // the last tile
  to_unit(vs0);
  pv(pf, v_slot(t));

  // ---- epilogue -----------------------------------------------------------------------------------------
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const float l_tot = l_acc[rb][0];
    if (row_ok[rb]) {
      if (single) {
        const float l_fin = with_sink(p, out_head[rb], m_run[rb], l_tot);
        const float inv = (l_fin > 0.f ? 1.f / l_fin : 0.f) * v_unit;
        uint16_t* orow = (uint16_t*)p.out + ((int64_t)out_tok[rb] * p.Hq + out_head[rb]) * p.Dq + 4 * g4;
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) {  // accumulator column j of row tile rt is dim 16rt + 4g4 + j
          const u32x2 w = {pack_bf16(o_acc[rb][rt][0] * inv, o_acc[rb][rt][1] * inv),
                           pack_bf16(o_acc[rb][rt][2] * inv, o_acc[rb][rt][3] * inv)};
          if (16 * rt + 4 * g4 < p.Dq) *(u32x2*)(orow + 16 * rt) = w;
        }
      } else {
        const int64_t pslot = ((int64_t)chunk * p.T + out_tok[rb]) * p.Hq + out_head[rb];
        float* prow = p.pre_o + pslot * D + 4 * g4;
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) *(f32x4*)(prow + 16 * rt) = o_acc[rb][rt] * v_unit;
        if (g4 == 0) {
          p.pre_ml[pslot * 2 + 0] = m_run[rb];
          p.pre_ml[pslot * 2 + 1] = l_tot;
        }
      }
    }
  }
}

template <int D, int KVT, int NW, int RB>
static int launch_dma8(hipStream_t stream, const AttnParams& p) {
  constexpr int ROWS = NW * RB * 16;
  const int64_t slots = ((int64_t)p.T * p.group) / ROWS + p.S;  // upper bound on row tiles of the batch
  const int64_t blocks = slots * p.Hkv * p.pre_max_chunks;
  if (blocks > 0x7fffffff) return (int)hipErrorInvalidValue;
  if (p.softcap > 0.f)
    hipLaunchKernelGGL((attn_prefill_dma8_kernel<D, KVT, NW, RB, true>), dim3((unsigned)blocks), dim3(64 * NW), 0, stream, p);
  else
    hipLaunchKernelGGL((attn_prefill_dma8_kernel<D, KVT, NW, RB, false>), dim3((unsigned)blocks), dim3(64 * NW), 0, stream, p);
  return (int)hipGetLastError();
}

// 8-bit pages whose size is a multiple of the 32-key tile, head sizes 128 and 256 (one DMA instruction per wave covers
// its share of a half tile), page rows that a 32-bit byte offset can address
bool prefill_dma8_supported(const AttnParams& p) {
  return (p.kv_dtype == RPA_FP8_E4M3 || p.kv_dtype == RPA_INT8) && p.page_size % 32 == 0 && (p.D == 128 || p.D == 256) &&
         (int64_t)32 * p.token_stride < ((int64_t)1 << 31);
}

int launch_attn_prefill_dma8(hipStream_t stream, const AttnParams& p) {
  const bool fp8 = p.kv_dtype == RPA_FP8_E4M3;
  switch (p.D) {
    case 128: return fp8 ? launch_dma8<128, RPA_FP8_E4M3, 4, 2>(stream, p) : launch_dma8<128, RPA_INT8, 4, 2>(stream, p);
    case 256: return fp8 ? launch_dma8<256, RPA_FP8_E4M3, 8, 1>(stream, p) : launch_dma8<256, RPA_INT8, 8, 1>(stream, p);
    default: return (int)hipErrorInvalidValue;
  }
}

}  // namespace rpa
