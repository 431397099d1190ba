// MFMA prefill / chunked-prefill attention for bf16 pages, K/V tiles moved global -> LDS by the
// load unit itself (global_load_lds_dwordx4) and the loop software-pipelined inside every wave.
//
// Same work split and arithmetic as attn_prefill_kernel (rpa_attn_prefill.hip): a workgroup owns 128
// query rows of one (sequence, KV head), each wave keeps RB 16-row blocks in registers and every wave
// reads the shared K/V tile in MFMA operand order.  What differs is how a tile reaches LDS and how a
// step is scheduled.  There the tile passes through registers (load, wait, ds_write), which costs
// staging registers, address and write instructions, and leaves one tile of prefetch; scores, softmax
// and PV product run one after the other.  Here every lane hands the load unit one 16-byte global
// address and the unit writes the 64 lanes' chunks to 1 KiB of LDS in lane order; the XOR swizzle of
// the tile is applied on the global side (lane for LDS chunk c' of row r fetches global chunk
// c' ^ key(r)).  No registers are held while a tile is in flight, so a tile is issued four steps before
// its last read, and the compute loop holds no global-memory instructions of its own.  Inside a step the
// scores of the next tile run on the matrix cores while the vector ALU does the softmax of this one.
//
// The loads are issued through inline assembly: the compiler then neither tracks them nor orders its
// own waits around them, and the kernel states its waits itself (s_waitcnt vmcnt(n) + s_barrier before a
// tile is read).  Every other global access of the kernel (queries before the loop, results after it)
// is ordinary code; the compiler's waits for those can only be stricter than needed, never weaker,
// because the counter retires loads in order.
#include <type_traits>

#include "rpa_mfma.h"

namespace rpa {

template <int D, int NW, int RB, bool CAP, int HT>
__global__ __launch_bounds__(64 * NW, 2) void attn_prefill_dma_kernel(AttnParams p) {
  using H = Half16<HT>;  // bf16, or half for float16 queries over float16 pages
  constexpr int TT = 32;                 // keys per tile
  constexpr int RKL = D * 2;             // bytes of one K (or V) row
  constexpr int CPR = RKL / 16;          // 16-byte chunks per row
  constexpr int RPI = 64 / CPR;          // rows one DMA instruction covers
  constexpr int NLH = TT / (RPI * NW);   // DMA instructions per wave per tile, for K and again for V
  static_assert(TT % (RPI * NW) == 0 && NLH >= 1, "the waves' DMA instructions tile the 32 rows exactly");
  static_assert(NLH == 1 || (RPI * NW) % 16 == 0, "a lane's swizzle key must not depend on the instruction");
  constexpr int NS = TT / 16;            // 16-key sub-tiles per tile
  constexpr int DPL = D / 16;            // 16-dim row tiles of O^T
  constexpr int NKK = D / 32;            // k-steps of the score MFMA
  constexpr int ROWS = NW * RB * 16;
  constexpr float kMaxSlack = 8.f;       // how far a score may exceed the softmax reference before it is raised
  static_assert(ROWS == kPrefillRows, "merge kernel assumes this row-tile height");
  constexpr int HALF = TT * RKL;         // bytes of the K (or V) rows of one tile
  // K of a tile is needed a step before its V (see the pipeline below), so the two halves live in rings of their
  // own: three K slots and five V slots hold everything between a tile's issue and its last read.
  constexpr int KN = 3, VN = 5;

  __shared__ __attribute__((aligned(1024))) unsigned char lds_all[(KN + VN) * HALF];

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
  u32x4 qf[RB][NKK];
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
      qf[rb][kk] = v;
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
      qf[rb][kk] = v;
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
  // DMA instruction u of wave w fills LDS rows (u NW + w) RPI .. + RPI - 1 of the K half, and again of the V
  // half; lane L sits at row + L / CPR, LDS chunk L % CPR, and fetches the global chunk that the swizzle maps there.
  // The block table is read through the constant address space: it does not change while the kernel runs, and
  // only so may the compiler keep these loads scalar after the assembly statements above have "written memory".
  typedef const __attribute__((address_space(4))) int32_t* ConstI32;
  ConstI32 bt = (ConstI32)(uintptr_t)(p.block_tables + (int64_t)i * p.M);
  const char* k_pages = (const char*)p.k_pages;
  const char* v_pages = (const char*)p.v_pages;
  const int pg = p.page_size;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds_all;
  const int dma_row = wave * RPI + lane / CPR;          // row for u = 0; instruction u adds u * NW * RPI
  const int dma_chunk = (lane % CPR) ^ swz_key<RKL>(dma_row);
  const int dma_chunk_v = (lane % CPR) ^ swz_key_v<RKL>(dma_row);  // the V half is swizzled for its transposing reads
  const uint32_t dma_wave_lds = (uint32_t)wave * 1024u;
  // issue cursor: the next tile to load (block-table column, token offset inside that page, page id)
  int cur_idx = kv_lo / pg;
  int cur_off = kv_lo - cur_idx * pg;
  int cur_tb = kv_lo;
  int cur_ks = 0, cur_vs = 0;  // ring slots of the tile the cursor is at
  // Lane offsets of an ordinary tile, loop-invariant; only a tile that holds keys nobody may see recomputes them.
  uint32_t voff_k[NLH], voff_v[NLH];
#pragma unroll
  for (int u = 0; u < NLH; ++u) {
    const uint32_t roff = (uint32_t)(dma_row + u * NW * RPI) * (uint32_t)p.token_stride;
    voff_k[u] = roff + (uint32_t)(dma_chunk << 4);
    voff_v[u] = roff + (uint32_t)(dma_chunk_v << 4);
  }
  // The page id of the cursor's tile is fetched one issue ahead and only clamped when it is used, so that no issue
  // waits for the scalar load it has just made.
  auto load_page = [&](int idx) -> int { return __builtin_amdgcn_readfirstlane(bt[min(idx, p.M - 1)]); };
  int cur_page_raw = load_page(cur_idx);
  auto issue = [&]() __attribute__((always_inline)) {  // starts the DMA of the cursor's tile into its ring slots and advances the cursor
    const int cur_page = min(max(cur_page_raw, 0), p.P - 1);
    const int64_t tile_off = (int64_t)cur_page * p.page_stride + (int64_t)cur_off * p.token_stride + (int64_t)h * p.head_stride;
    const char* base_k = k_pages + tile_off;
    const char* base_v = v_pages + tile_off;
    const bool edge = (cur_tb + TT > sp.ctx) || (cur_tb < vis_lo);
    const uint32_t k_lds = lds_base + (uint32_t)cur_ks * HALF + dma_wave_lds;
    const uint32_t v_lds = lds_base + (uint32_t)(KN + cur_vs) * HALF + dma_wave_lds;
    if (!edge) {
#pragma unroll
      for (int u = 0; u < NLH; ++u) {
        dma16(k_lds + u * NW * 1024, voff_k[u], base_k);  // K rows
        dma16(v_lds + u * NW * 1024, voff_v[u], base_v);  // V rows
      }
    } else {
#pragma unroll
      for (int u = 0; u < NLH; ++u) {  // keys nobody may see: any visible row's bytes
        const int r = min(max(cur_tb + dma_row + u * NW * RPI, vis_lo), sp.ctx - 1) - cur_tb;
        const uint32_t roff = (uint32_t)r * (uint32_t)p.token_stride;
        dma16(k_lds + u * NW * 1024, roff + (uint32_t)(dma_chunk << 4), base_k);
        dma16(v_lds + u * NW * 1024, roff + (uint32_t)(dma_chunk_v << 4), base_v);
      }
    }
    cur_tb += TT;
    cur_off += TT;
    if (cur_off >= pg) {
      cur_off -= pg;
      ++cur_idx;
    }
    cur_ks = (cur_ks == KN - 1) ? 0 : cur_ks + 1;
    cur_vs = (cur_vs == VN - 1) ? 0 : cur_vs + 1;
    cur_page_raw = load_page(cur_idx);
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
        sa[rb][i / NKK] = H::mfma32(a, qf[rb][i % NKK], sa[rb][i / NKK]);
      if (i + KPD < NKO) kp[i % KPD] = read_k(lds_k, i + KPD);
    }
  };
  // ---- online softmax of the scores of tile tb ----------------------------------------------------------
  auto softmax = [&](auto mask_tag, f32x4 (&sa)[RB][NS], int tb, uint32_t (&pfrag)[RB][NS][2]) __attribute__((always_inline)) {
    constexpr bool MASK = decltype(mask_tag)::value;
    const float sc_mul = CAP ? cap_out : p.scale_log2;
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
          if constexpr (CAP) sv = fast_tanh(sv * cap_in);
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
        pfrag[rb][st][0] = H::pack(pr[0], pr[1]);
        pfrag[rb][st][1] = H::pack(pr[2], pr[3]);
      }
    }
  };
  // ---- O^T += V^T . P^T, and the row sums ------------------------------------------------------------------
  auto pv = [&](uint32_t (&pfrag)[RB][NS][2], const unsigned char* lds_v) __attribute__((always_inline)) {
    // The row sums come from the matrix cores as well: a V^T tile of ones times P^T leaves, in every accumulator
    // element of column n, the sum of row n's probabilities over all 32 keys (as rounded to bf16, i.e. exactly the
    // weights the PV product uses).  Two MFMAs replace 16 additions per lane and the cross-lane sum at the end.
    {
      const u32x4 ones = {H::kOnes, H::kOnes, H::kOnes, H::kOnes};
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const u32x4 b4 = {pfrag[rb][0][0], pfrag[rb][0][1], pfrag[rb][1][0], pfrag[rb][1][1]};
        l_acc[rb] = H::mfma32(ones, b4, l_acc[rb]);
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
        o_acc[rb][rt] = H::mfma32(a4, b4, o_acc[rb][rt]);
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
  // Step t: (A) the matrix cores compute the scores of tile t+1 while the vector ALU does the softmax of tile t;
  // (B) the workgroup meets at the step's barrier, behind which tile t+2 is visible and the slots of K(t+1) and
  // V(t-1) are free: tile t+4 is issued into them and the first K operands of tile t+2 are read; (C) the PV product
  // of tile t runs, hiding the latency of those reads, so that the next step starts on the matrix cores at once.
  // (With the barrier at the head of the step every wave of the CU asked LDS for its K operands at the same moment
  // and waited for them with nothing else to do: a quarter of the kernel's time.)
  auto k_slot = [&](int sl) -> const unsigned char* { return lds_all + sl * HALF; };
  auto v_slot = [&](int sl) -> const unsigned char* { return lds_all + (KN + sl) * HALF; };
  const std::true_type masked{};
  f32x4 s_cur[RB][NS], s_nxt[RB][NS];
  uint32_t pf[RB][NS][2];
  u32x4 kp[KPD];
  issue();                   // tile 0
  if (n_tiles > 1) issue();  // tile 1
  if (n_tiles > 2) issue();  // tile 2
  if (n_tiles > 2) wait_loads_and_barrier<4 * NLH>();
  else if (n_tiles > 1) wait_loads_and_barrier<2 * NLH>();
  else wait_loads_and_barrier<0>();
  k_prefetch(k_slot(0), kp);
  qk(k_slot(0), kp, s_cur);
  if (n_tiles > 1) {
    if (n_tiles > 2) wait_loads_and_barrier<2 * NLH>();  // tile 1 has landed, and every wave is done with K slot 0
    else wait_loads_and_barrier<0>();
    if (n_tiles > 3) issue();  // tile 3
    k_prefetch(k_slot(1), kp);
  }
  int t = 0;
  int rd_k = 1, rd_v = 0;  // ring slots of K(t+1) and V(t)
  auto next_k = [&](int sl) { return sl == KN - 1 ? 0 : sl + 1; };
  // Steps [t, t_end) with or without the masking code.  Two variants side by side in one loop body (an if / else
  // around the step) make the compiler keep a second copy of every accumulator, so the choice is made per run of
  // steps instead: masked steps at the window's lower edge, unmasked ones, masked ones at the causal edge.
  // (Unrolling two steps per trip to alternate the score registers instead of copying them was tried: the
  // compiler then needs 50 more registers and spills.)
  auto run = [&](auto mask_tag, int t_end) __attribute__((always_inline)) {
    for (; t < t_end; ++t) {  // t + 2 < n_tiles
      qk(k_slot(rd_k), kp, s_nxt);
      softmax(mask_tag, s_cur, kv_lo + t * TT, pf);
      if (t + 3 < n_tiles) wait_loads_and_barrier<2 * NLH>();  // tile t+2 has landed; tile t+3 may still be in flight
      else wait_loads_and_barrier<0>();
      if (t + 4 < n_tiles) issue();
      rd_k = next_k(rd_k);
      k_prefetch(k_slot(rd_k), kp);
      pv(pf, v_slot(rd_v));
      rd_v = (rd_v == VN - 1) ? 0 : rd_v + 1;
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
  if (n_tiles > 1) {  // t = n_tiles - 2: the last scores; every tile has landed and is visible
    qk(k_slot(rd_k), kp, s_nxt);
    softmax(masked, s_cur, kv_lo + t * TT, pf);
    pv(pf, v_slot(rd_v));
    rd_v = (rd_v == VN - 1) ? 0 : rd_v + 1;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int st = 0; st < NS; ++st) s_cur[rb][st] = s_nxt[rb][st];
    ++t;
  }
  softmax(masked, s_cur, kv_lo + t * TT, pf);  // the last tile
  pv(pf, v_slot(rd_v));

  // ---- epilogue -----------------------------------------------------------------------------------------
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const float l_tot = l_acc[rb][0];
    if (row_ok[rb]) {
      if (single) {
        const float l_fin = with_sink(p, out_head[rb], m_run[rb], l_tot);
        const float inv = l_fin > 0.f ? 1.f / l_fin : 0.f;
        uint16_t* orow = (uint16_t*)p.out + ((int64_t)out_tok[rb] * p.Hq + out_head[rb]) * p.Dq + 4 * g4;
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) {  // accumulator column j of row tile rt is dim 16rt + 4g4 + j
          const u32x2 w = {H::pack(o_acc[rb][rt][0] * inv, o_acc[rb][rt][1] * inv),
                           H::pack(o_acc[rb][rt][2] * inv, o_acc[rb][rt][3] * inv)};
          if (16 * rt + 4 * g4 < p.Dq) *(u32x2*)(orow + 16 * rt) = w;
        }
      } else {
        const int64_t pslot = ((int64_t)chunk * p.T + out_tok[rb]) * p.Hq + out_head[rb];
        float* prow = p.pre_o + pslot * D + 4 * g4;
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) *(f32x4*)(prow + 16 * rt) = o_acc[rb][rt];
        if (g4 == 0) {
          p.pre_ml[pslot * 2 + 0] = m_run[rb];
          p.pre_ml[pslot * 2 + 1] = l_tot;
        }
      }
    }
  }
}

template <int D, int NW, int RB, int HT>
static int launch_dma(hipStream_t stream, const AttnParams& p) {
  constexpr int ROWS = NW * RB * 16;
  const int64_t slots = ((int64_t)p.T * p.group) / ROWS + p.S;  // upper bound on row tiles of the batch
  const int64_t blocks = slots * p.Hkv * p.pre_max_chunks;
  if (blocks > 0x7fffffff) return (int)hipErrorInvalidValue;
  if (p.softcap > 0.f)
    hipLaunchKernelGGL((attn_prefill_dma_kernel<D, NW, RB, true, HT>), dim3((unsigned)blocks), dim3(64 * NW), 0, stream, p);
  else
    hipLaunchKernelGGL((attn_prefill_dma_kernel<D, NW, RB, false, HT>), dim3((unsigned)blocks), dim3(64 * NW), 0, stream, p);
  return (int)hipGetLastError();
}

// bf16 (or float16) pages whose size is a multiple of the 32-key tile, and page rows that a 32-bit byte offset can address
bool prefill_dma_supported(const AttnParams& p) {
  return (p.kv_dtype == RPA_BF16 || p.kv_dtype == RPA_F16) && p.page_size % 32 == 0 && (p.D == 64 || p.D == 128 || p.D == 256) &&
         (int64_t)32 * p.token_stride < ((int64_t)1 << 31);
}

template <int HT>
static int launch_dma_d(hipStream_t stream, const AttnParams& p) {
  switch (p.D) {
    case 64: return launch_dma<64, 4, 2, HT>(stream, p);
    case 128: return launch_dma<128, 4, 2, HT>(stream, p);
    case 256: return launch_dma<256, 8, 1, HT>(stream, p);
    default: return (int)hipErrorInvalidValue;
  }
}

int launch_attn_prefill_dma(hipStream_t stream, const AttnParams& p) {
  return p.kv_dtype == RPA_F16 ? launch_dma_d<RPA_F16>(stream, p) : launch_dma_d<RPA_BF16>(stream, p);
}

}  // namespace rpa
