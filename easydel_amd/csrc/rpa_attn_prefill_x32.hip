// MFMA prefill / chunked-prefill attention for bf16 (or float16) pages on 32x32x16 tiles: one wave per SIMD, 64 query
// rows per wave, and a steady-state step whose instruction order and register files are written down, not left to the
// scheduler and the allocator.
//
// Why this shape.  A bf16 MFMA stream whose A operands come out of LDS sustains, on this chip, 65-78 % of the matrix
// peak with 16x16x32 tiles and two row blocks per operand (what attn_prefill_dma_kernel does), but 86 % with 32x32x16
// tiles and two 32-row blocks per operand, already with one wave per SIMD: a 32x32x16 MFMA occupies the pipe for 32
// cycles, takes the same 1 KiB operand, and leaves the issue port free for six vector instructions.  So a wave here
// owns 64 rows (row = (token, GQA head)) of one (sequence, KV head): Q as B operands (S^T = K Q^T) and the O^T
// accumulators stay in registers for the whole key range, every K and V operand read from LDS feeds two MFMAs, and a
// workgroup of four waves (256 rows) has a CU to itself.  With a single wave per SIMD nothing but the wave's own
// instruction order overlaps the matrix pipe with the softmax, so the step -- one block of 32 keys -- is
// software-pipelined over three blocks and its order is pinned (a sched_barrier after every MFMA slot):
//
//   step b :  MFMA slots 0..15   S(b+2) = K(b+2) Q^T       | vector: softmax of block b+1, half a pair of probabilities per slot
//             MFMA slots 16..19  row sums of P(b)            |
//             MFMA slots 20..35  O     += V(b)^T P(b)^T     | vector: the softmax goes on; row maxima of S(b+2)
//
// Operands are read four ahead of their MFMAs, across the phase and step boundaries.  The wave has 512 registers; which
// of them sit in the accumulation file is stated through the operand constraints of the MFMAs (issued as single
// assembly statements): O^T and Q live there (192 registers the vector ALU never touches), the scores are produced in
// ordinary registers because the vector ALU reads them next.  The compiler does not see into those statements, so the
// waits this chip wants between an MFMA and a vector instruction that reads its result are stated here as well: in the
// pinned step the first reader of a result comes at least sixteen MFMA slots behind its writer, everywhere else an
// explicit pause (mfma_settle) precedes the reader.
//
// Tiles travel global -> LDS through the load unit (global_load_lds_dwordx4) into one ring for K and one for V.  At head
// size 128 a tile is 64 keys (two steps), the rings hold four tiles each (128 KiB), K is requested four tiles and V three
// tiles ahead, and there is one barrier per tile.  At head size 256 a wave owns 32 rows (the O^T tile of 64 rows would
// not fit its registers), a tile is one block of 32 keys, the rings hold five tiles each (160 KiB: all of the CU's LDS),
// K is requested six and V four tiles ahead, and there is one barrier per step.
//
// Softmax as in attn_prefill_dma_kernel: probabilities are taken against a per-row reference that is only raised when a
// score exceeds it by more than kMaxSlack (log2 units); here the reference is kept at whole numbers, so that raising it
// scales what has been accumulated -- and the probabilities of the block still waiting for its PV product -- by a power
// of two, exactly.  Row sums come from the matrix cores (a tile of ones against P^T: four more MFMAs per step), so that
// they are the sums of the probabilities as rounded to 16 bits, the very weights of the PV product -- a row that one
// key dominates then comes out exact.  The vector ALU, the busier unit here, could not do it cheaper: the dot-product
// instruction that adds a packed pair (v_dot2) runs in the matrix pipe and waits for the MFMA in flight (measured: 52
// instead of 36 cycles per MFMA slot), and unpacking costs four instructions per pair.
//
// Tiles that need masking (the window's lower edge, the causal diagonal) and the first and the last two tiles of a key
// range run through the same two steps written plainly (phases one after the other, flags at run time); the pinned
// steps serve the unmasked middle.
#include <type_traits>

#include "rpa_mfma.h"

namespace rpa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

// The pause between an MFMA issued through an assembly statement and an instruction that reads its result (the
// compiler cannot place it): 32 wait states, more than the eight passes of a 32x32x16 MFMA plus the margin this chip asks for.
// The registers whose readers it protects are operands of the statement: that is what orders it behind the MFMAs that
// write them and ahead of the instructions that read them.
__device__ __forceinline__ void mfma_settle(f32x16 (&s)[2]) { asm volatile("s_nop 15\n\ts_nop 15" : "+v"(s[0]), "+v"(s[1])); }
__device__ __forceinline__ void mfma_settle(f32x16 (&s)[1]) { asm volatile("s_nop 15\n\ts_nop 15" : "+v"(s[0])); }
__device__ __forceinline__ void mfma_settle_acc(f32x16 (&o)[8], f32x16 (&l)[2]) {
  asm volatile("s_nop 15\n\ts_nop 15" : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]), "+a"(o[4]), "+a"(o[5]), "+a"(o[6]), "+a"(o[7]), "+a"(l[0]), "+a"(l[1]));
}
__device__ __forceinline__ void mfma_settle_acc(f32x16 (&o)[8], f32x16 (&l)[1]) {
  asm volatile("s_nop 15\n\ts_nop 15" : "+a"(o[0]), "+a"(o[1]), "+a"(o[2]), "+a"(o[3]), "+a"(o[4]), "+a"(o[5]), "+a"(o[6]), "+a"(o[7]), "+a"(l[0]));
}

template <int HT>
struct Wide16;
template <>
struct Wide16<RPA_BF16> {
  // S^T accumulation: result in ordinary registers, K operand in ordinary registers, Q operand in the accumulation file
  static __device__ __forceinline__ void mfma_s0(f32x16& acc, const u32x4& a, const u32x4& q) {
    asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(q));
  }
  static __device__ __forceinline__ void mfma_s(f32x16& acc, const u32x4& a, const u32x4& q) {
    asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(q));
  }
  // O^T accumulation: accumulator in the accumulation file, V and P operands in ordinary registers
  static __device__ __forceinline__ void mfma_o(f32x16& acc, const u32x4& a, const u32x4& b) {
    asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma_o0(f32x16& acc, const u32x4& a, const u32x4& b) {  // starts from zero
    asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&a"(acc) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ float lo_half(uint32_t w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi_half(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
  static __device__ __forceinline__ uint32_t scale_pair(uint32_t w, float a) {  // both halves times a
    return pack_bf16(lo_half(w) * a, hi_half(w) * a);
  }
};
template <>
struct Wide16<RPA_F16> {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ void mfma_s0(f32x16& acc, const u32x4& a, const u32x4& q) {
    asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(q));
  }
  static __device__ __forceinline__ void mfma_s(f32x16& acc, const u32x4& a, const u32x4& q) {
    asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(q));
  }
  static __device__ __forceinline__ void mfma_o(f32x16& acc, const u32x4& a, const u32x4& b) {
    asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma_o0(f32x16& acc, const u32x4& a, const u32x4& b) {
    asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&a"(acc) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ float lo_half(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[0]; }
  static __device__ __forceinline__ float hi_half(uint32_t w) { return (float)__builtin_bit_cast(f16x2, w)[1]; }
  static __device__ __forceinline__ uint32_t scale_pair(uint32_t w, float a) {
    return Half16<RPA_F16>::pack(lo_half(w) * a, hi_half(w) * a);
  }
};

// Swizzle of the V half of a tile for the transposing reads of 32x32x16 operands: one ds_read_b64_tr_b16 fetches, for
// each half of the wave, 64 contiguous bytes of four consecutive key rows; XOR-ing the 16-byte chunk index with four
// times the row number (mod 4) puts those four rows on distinct quarters of the banks.
template <int ROW_BYTES>
__device__ __forceinline__ int swz_key_v32(int tok) {
  constexpr int NCH = ROW_BYTES / 16;
  if constexpr (NCH >= 16) return (tok & 3) << 2;
  else if constexpr (NCH == 8) return (tok & 1) << 2;
  else return 0;
}

// KS: the pages are bf16 copies of scaled 8-bit pages (AttnParams::wide), bare codes.  A tile of 64 keys lies in one
// page: its scores are scaled by the page's K scale on top of the softmax scale; its probabilities are multiplied by
// the page's V scale (inside the exponent) before they are rounded for the PV product, and the row sums are taken per
// tile and divided by that scale in float32 as they join the running sums -- numerator and denominator then hold
// the same rounded weights, as with 16-bit pages.  (The scale rounded to 16 bits anywhere, in the values or in the
// operand of the row sums, is 2^-9 of an output: rows of a few keys then miss 2e-2 on outputs near 4.)
template <int D, int NW, int RB, int HT, bool CAP, bool KS = false>
__global__ __launch_bounds__(64 * NW) void attn_prefill_x32_kernel(AttnParams p) {
  using H = Half16<HT>;
  using W = Wide16<HT>;
  constexpr int BK = 32;                 // keys per block (what a step computes)
  constexpr int SPT = D <= 128 ? 2 : 1;  // steps per tile
  constexpr int TT = BK * SPT;           // keys per tile (what a barrier and a set of loads cover)
  constexpr int RKL = D * 2;             // bytes of one K (or V) row
  constexpr int CPR = RKL / 16;          // 16-byte chunks per row
  constexpr int RPI = 64 / CPR;          // rows one DMA instruction covers
  constexpr int NLH = TT / (RPI * NW);   // DMA instructions per wave per tile, for K and again for V
  static_assert(TT % (RPI * NW) == 0 && NLH >= 1, "the waves' DMA instructions tile the rows exactly");
  constexpr int NKK = D / 16;            // k-steps of the score MFMA = K operands per block
  constexpr int DB = D / 32;             // 32-dim blocks of O^T
  constexpr int NVO = DB * 2;            // V operands per block: (dim block, 16-key half)
  constexpr int ROWS = NW * RB * 32;
  constexpr float kMaxSlack = 8.f;
  constexpr int HALF = TT * RKL;         // bytes of the K (or V) rows of one tile
  constexpr int KN = SPT == 2 ? 4 : 5;   // ring slots (tiles), of K and again of V
  // The barrier with index u stands in front of step SPT u.  Behind it K tiles up to u + KNO are visible (the steps up to
  // the next barrier read as far as the first operands of block SPT u + SPT + 2) and V tiles up to u; K tiles below
  // u + 2 / SPT and V tiles below u will not be read again.  It requests the tiles that take the newest free slots:
  constexpr int KNO = (SPT + 2) / SPT;
  constexpr int KAH = 2 / SPT - 1 + KN;  // K of tile u + KAH ...
  constexpr int VAH = KN - 1;            // ... behind V of tile u + VAH
  constexpr int DQ = KAH - VAH;          // a tile's V rows are requested this many tiles behind its K rows
  constexpr int FLYB = KAH - KNO - 1;    // all requests of this many barriers may still be in flight at a barrier
  constexpr int U0 = -2 / SPT;           // the first barrier (step -2)
  static_assert(2 * KN * HALF <= 160 * 1024 && FLYB >= 1 && DQ >= 1 && 2 * FLYB * NLH <= 48, "ring sizes");
  constexpr int NQ = NKK * RB;           // MFMA slots of the score phase
  constexpr int NSUM = 2 * RB;           // MFMA slots of the row sums (ones x P^T, per row block and 16-key half)
  constexpr int NP = NVO * RB;           // MFMA slots of the PV phase
  constexpr int PD = 4;                  // operands read ahead
  constexpr int NPAIR = RB * 8;          // pairs of probabilities per lane and block
  constexpr int SPP = (NQ + NP) / NPAIR; // MFMA slots of the two products per pair of the softmax
  constexpr int MSP = NP / NPAIR;        // PV slots per three-way maximum
  static_assert(SPP * NPAIR == NQ + NP && MSP * NPAIR == NP && (SPP == 2 || SPP == 4), "the softmax is dealt out over the MFMA slots of the two products");
  static_assert(!CAP || SPP == 4, "the soft cap's stages take four slots per pair");
  static_assert(NKK >= PD && NVO >= PD, "the operand ring is shorter than either phase");
  constexpr int NG = SPT == 2 ? 1 : 2;   // half tiles a step requests: at two steps per tile V in the first, K in the second
  constexpr int NDI = NG * NLH;          // DMA instructions of a step: in the slots of the row sums ...
  constexpr int DSP = (NQ + NP) / NDI;   // where they outnumber the slots of the row sums: one per DSP slots of the two products

  __shared__ __attribute__((aligned(1024))) unsigned char lds_all[2 * KN * HALF];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j32 = lane & 31, hh = lane >> 5;  // row inside a 32-row block, half of the wave
  const int n = lane & 15;
  const int G = p.group;

  // ---- block -> (sequence, row tile, KV head, key chunk) ---------------------------------------------
  const int h = blockIdx.x % p.Hkv;
  const int n_slots = gridDim.x / (p.Hkv * p.pre_max_chunks);
  int slot = (blockIdx.x / p.Hkv) % n_slots;
  const int chunk = blockIdx.x / (p.Hkv * n_slots);
  if (p.plan[2] == 0) return;
  if constexpr (KS) {
    if (!wide_mode(p)) return;  // this batch stays with the kernel that reads the 8-bit pages
  }
  const int n_live = live_rows(p);
  if (n_live <= 0) return;
  // Slot -> (sequence, row tile): through the plan's longest-first order where the plan kernel made one (the grid deals
  // workgroups to the chip in this order), else sequence i starts at slot floor(qsl[i] G / ROWS) + i.
  int i, tile_in_seq;
  const int n_sorted = p.plan[5];
  if (n_sorted >= 0) {
    const int32_t* order = p.plan + kPlanHeader + 2 * (p.S + 1) + kMaxDecodeWgs;
    const int32_t* tile_start = order + kMaxSortedSeqs;
    if (n_sorted == 0) return;
    const int n_tiles_all = tile_start[n_sorted];
    // The chip deals consecutive workgroups round-robin to its CUs (measured: every CU gets the same number of them, and
    // the CUs' loads differ by what ranks a round apart differ by), so with the slots in longest-first order the same
    // CU would get the longest row tile of every round: from four rounds on (eight row tiles per CU and 4.7 % between
    // the busiest CU and the mean on the long-context prefill shape), every other whole round of slots is walked backwards.
    // Head size 128 only, where a CU holds two workgroups: with one workgroup per CU (head size 256) the plain
    // longest-first order measured 1 % faster.
    const int round = p.pre_slots / p.Hkv;  // slots per round of workgroups over the chip
    if (D <= 128 && round > 1 && p.pre_slots % p.Hkv == 0 && n_tiles_all >= 4 * round) {
      const int r = slot / round;
      if ((r & 1) && (r + 1) * round <= n_tiles_all) slot = r * round + (round - 1 - slot % round);
    }
    if (slot >= n_tiles_all) return;
    int lo_r = 0, hi_r = n_sorted;
    while (hi_r - lo_r > 1) {
      const int mid = (lo_r + hi_r) >> 1;
      if (tile_start[mid] <= slot) lo_r = mid; else hi_r = mid;
    }
    i = order[lo_r];
    tile_in_seq = slot - tile_start[lo_r];
  } else {
    int lo_i = 0, hi_i = n_live;
    while (hi_i - lo_i > 1) {
      const int mid = (lo_i + hi_i) >> 1;
      if ((int)(((int64_t)p.qsl[mid] * G) / ROWS) + mid <= slot) lo_i = mid; else hi_i = mid;
    }
    i = lo_i;
    tile_in_seq = slot - ((int)(((int64_t)p.qsl[i] * G) / ROWS) + i);
  }
  const SeqPlan sp = seq_plan(p, i);
  if (!sp.live || sp.small_rows) return;
  const int rows_total = sp.q_len * G;
  const int R0 = tile_in_seq * ROWS;
  if (tile_in_seq < 0 || R0 >= rows_total) return;

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
  const int base_pos = sp.ctx - sp.q_len;
  const int vis_lo = pt.vis_lo;
  const int kv_lo = max(pt.kv_lo + chunk * pt.chunk_len, vis_lo & ~63);
  const int kv_hi = (chunk == pt.n_chunks - 1) ? pt.kv_hi : pt.kv_lo + (chunk + 1) * pt.chunk_len;
  const int n_tiles = (kv_hi - kv_lo + TT - 1) / TT;
  const bool single = pt.n_chunks == 1;

  // ---- the page table ------------------------------------------------------------------------------
  // (Requested ahead of the query rows: the first tile loads wait for it.)
  // Block-table entries are held 64 columns at a time, one per lane, and picked with v_readlane: the loop then holds no
  // scalar memory load, whose out-of-order return would turn every wait for an LDS operand into a wait for all of them.
  const int32_t* bt_row = p.block_tables + (int64_t)i * p.M;
  int col_base = kv_lo / p.page_size;
  // (held as the page's offset in the pool in units of 256 bytes: ids clipped and multiplied once per 64 columns here,
  //  not once per tile in scalar arithmetic; a page is a multiple of 64 rows of 16 bytes or more, the pool is below 2^40 bytes)
  const uint32_t page_units = (uint32_t)(p.page_stride >> 8);
  const float sc_mul = p.scale_log2;
  // what a raw score is multiplied by first: the softmax scale in log2 units, or with a soft cap 2 log2(e) scale / cap
  // (the argument of the exponential the hyperbolic tangent is made of); KS: times the K scale of the score's page
  const float sc_unit = CAP ? (p.scale / p.softcap) * 2.8853900817779268f : sc_mul;
  int wide_first = 0;
  if constexpr (KS) wide_first = p.wide[2 + i];  // the sequence's copied pages follow one another: column c is page wide_first + c
  auto page_offsets = [&](int col0) -> uint32_t {
    if constexpr (KS) return (uint32_t)min(max(wide_first + col0 + lane, 0), p.P - 1) * page_units;
    else return (uint32_t)min(max(bt_row[min(col0 + lane, p.M - 1)], 0), p.P - 1) * page_units;
  };
  uint32_t pages_vec = page_offsets(col_base);
  // KS: beside them the score scale of each of the 64 columns (softmax scale x the K scale of the column's 8-bit page)
  // and the logarithm of its V scale; a tile's pair is taken when the tile is requested and queued until its steps.
  float sck_vec = sc_unit, lvs_vec = 0.f;
  auto page_scales = [&](int col0) __attribute__((always_inline)) {
    if (p.kv_scales != nullptr) {
      const int id = min(max(bt_row[min(col0 + lane, p.M - 1)], 0), p.src_P - 1);
      const float2 kv = *(const float2*)(p.kv_scales + (int64_t)id * p.C + 2 * h);
      sck_vec = sc_unit * fmaxf(kv.x, 1e-30f);
      lvs_vec = __builtin_amdgcn_logf(fmaxf(kv.y, 1e-30f));  // log2
    }
  };
  if constexpr (KS) page_scales(col_base);
  float kq[KAH + 1], lq[KAH + 1];  // after barrier u: kq[c], lq[c] belong to tile u + c
#pragma unroll
  for (int c = 0; c <= KAH; ++c) {
    kq[c] = sc_unit;
    lq[c] = 0.f;
  }
  int cur_col = col_base, cur_off = kv_lo - col_base * p.page_size, cur_tb = kv_lo;

  // ---- per row-block lane state --------------------------------------------------------------------
  int row_lo[RB], row_hi[RB];
  bool row_ok[RB];
  int out_tok[RB], out_head[RB];
  u32x4 qf[RB][NKK];
  int wave_lo, wave_hi;          // keys every row of the wave sees: [max row_lo, min row_hi)
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = R0 + (wave * RB + rb) * 32 + j32;
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
    for (int kk = 0; kk < NKK; ++kk) {  // B operand of k-step kk: dims 16 kk + 8 hh .. + 7 of the lane's row
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok[rb] && kk * 16 + 8 * hh < p.Dq) v = *(const u32x4*)(qrow + (kk * 16 + 8 * hh) * 2);
      qf[rb][kk] = v;
    }
  }
  {
    int lo_max = 0, hi_min = 0x7fffffff;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      lo_max = max(lo_max, row_lo[rb]);
      hi_min = min(hi_min, row_hi[rb]);
    }
#pragma unroll
    for (int o = 1; o < 32; o <<= 1) {
      lo_max = max(lo_max, __shfl_xor(lo_max, o));
      hi_min = min(hi_min, __shfl_xor(hi_min, o));
    }
    wave_lo = __builtin_amdgcn_readfirstlane(lo_max);
    wave_hi = __builtin_amdgcn_readfirstlane(hi_min);
  }

  // ---- tile loads ------------------------------------------------------------------------------------
  // Wave w moves rows [RW w, RW (w + 1)) of a tile's K rows, and again of its V rows, with NLH instructions of RPI rows
  // each into consecutive 1 KiB blocks of LDS: one m0 per half tile, the instruction offsets u KiB select the block.
  // (An instruction offset moves the global address as well: it is taken out of the lane offsets beforehand.)
  constexpr int RW = TT / NW;
  static_assert(RW == NLH * RPI && RW * RKL == NLH * 1024, "a wave's rows are whole DMA instructions");
  const char* k_base = (const char*)p.k_pages + (int64_t)h * p.head_stride;
  const char* v_base = (const char*)p.v_pages + (int64_t)h * p.head_stride;
  const uint32_t tok_stride = (uint32_t)p.token_stride;  // 64 rows of it fit 31 bits (the host checks)
  const int pg = p.page_size;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds_all;
  const uint32_t dma_wave_lds = (uint32_t)wave * (uint32_t)(RW * RKL);
  auto dma_row = [&](int u) -> int { return wave * RW + u * RPI + lane / CPR; };  // row of the tile instruction u of this lane's wave moves
  auto dma_chunk = [&](int u, bool is_v) -> int { return (lane % CPR) ^ (is_v ? swz_key_v32<RKL>(dma_row(u)) : swz_key<RKL>(dma_row(u))); };
  uint32_t voff_k[NLH], voff_v[NLH];
#pragma unroll
  for (int u = 0; u < NLH; ++u) {
    const uint32_t roff = (uint32_t)dma_row(u) * tok_stride - (uint32_t)(u * 1024);
    voff_k[u] = roff + (uint32_t)(dma_chunk(u, false) << 4);
    voff_v[u] = roff + (uint32_t)(dma_chunk(u, true) << 4);
  }
  // Descriptors of the tiles the cursor was last at, newest first: a tile's V rows are requested DQ tiles behind its K rows.
  struct TileDesc {
    int64_t off;
    bool edge;
    int tb;
    float sc, lv;  // KS: the tile's score scale and the logarithm of its V scale
  };
  TileDesc td[DQ];
#pragma unroll
  for (int j = 0; j < DQ; ++j) td[j] = TileDesc{0, false, 0, 0.f, 0.f};
  // The next 64 columns are fetched when the cursor is within `margin` columns of the end of the held ones.
  auto refill_pages = [&](int margin) __attribute__((always_inline)) {
    if (cur_col - col_base >= 64 - margin) {
      if constexpr (KS) {
        page_scales(cur_col);
        asm volatile("" : "+v"(sck_vec), "+v"(lvs_vec));
      }
      col_base = cur_col;
      pages_vec = page_offsets(col_base);
      asm volatile("" : "+v"(pages_vec));  // waited for here, once in 64 columns, not at the look-up every tile shares
    }
  };
  auto next_tile = [&](bool refill = true) __attribute__((always_inline)) {  // (also for tiles past the range: the cursor then only counts)
    if (refill) refill_pages(0);
    const uint64_t page_off = (uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)pages_vec, cur_col - col_base) << 8;
#pragma unroll
    for (int j = DQ - 1; j > 0; --j) td[j] = td[j - 1];
    td[0].off = (int64_t)(page_off + (uint32_t)cur_off * tok_stride);
    if constexpr (KS) {
      td[0].sc = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(sck_vec), (cur_col - col_base) & 63));
      td[0].lv = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(lvs_vec), (cur_col - col_base) & 63));
    }
    td[0].edge = (cur_tb + TT > sp.ctx) || (cur_tb < vis_lo);
    td[0].tb = cur_tb;
    cur_tb += TT;
    cur_off += TT;
    if (cur_off >= pg) {
      cur_off -= pg;
      ++cur_col;
    }
  };
  auto issue_half = [&](bool is_v, int slot, const TileDesc& t) __attribute__((always_inline)) {  // K or V rows of tile t into ring slot `slot`
    const char* base = (is_v ? v_base : k_base) + t.off;
    const uint32_t lds = lds_base + (uint32_t)((is_v ? KN : 0) + slot) * HALF + dma_wave_lds;
    if (!t.edge) {
      dma16_group<NLH>(lds, is_v ? voff_v : voff_k, base);
    } else {
#pragma unroll
      for (int u = 0; u < NLH; ++u) {  // keys nobody may see: any visible row's bytes
        const int r = min(max(t.tb + dma_row(u), vis_lo), sp.ctx - 1) - t.tb;
        dma16(lds + u * 1024, (uint32_t)r * tok_stride + (uint32_t)(dma_chunk(u, is_v) << 4), base);
      }
    }
  };

  // ---- registers of the pipeline -------------------------------------------------------------------------
  // Block b of the key range = (tile b / SPT, part b % SPT).  Scores and probabilities of block b live in buffer b % 2.
  f32x16 sa[2][RB];            // raw scores S^T: lane = row j32, register r = key 8 (r / 4) + 4 hh + r % 4 of the block
  u32x4 pb[2][RB][2];          // packed probabilities, as the two B operands (16 keys each) of the PV product
  f32x16 o_acc[RB][DB];        // O^T: lane = row j32, register r = dim 8 (r / 4) + 4 hh + r % 4 of the 32-dim block
  f32x16 l_acc[RB];            // row sums, from the matrix cores: every register of lane j32 holds the sum of row j32
  float m_ref[RB], lmx[RB];
  float m_neg[RB];             // what is added to a scaled score ahead of the exponential: -m_ref (with a soft cap: cap - m_ref)
  float thr[RB];               // (m_ref + slack) in units of the raw scores: what a block's maximum is compared with
  u32x4 ops[PD];               // operands read ahead of their MFMAs
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    m_ref[rb] = -INFINITY;
    thr[rb] = -INFINITY;
    m_neg[rb] = 0.f;
    {
      f32x16 z;
#pragma unroll
      for (int r = 0; r < 16; ++r) z[r] = 0.f;
      asm volatile("" : "+a"(z));
      l_acc[rb] = z;
    }
    lmx[rb] = -INFINITY;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      f32x16 z;
#pragma unroll
      for (int r = 0; r < 16; ++r) z[r] = 0.f;
      asm volatile("" : "+a"(z));
      o_acc[rb][db] = z;
    }
  }
  // Without a soft cap a probability is exp2(s sc_mul + m_neg).  With one, the capped score in log2 units is
  // cap_out tanh(s cap_in) = cap_out (1 - 2 / (exp2(s cap_in2) + 1)), so the probability is exp2(r cap_m2 + m_neg) with
  // r = 1 / (exp2(s cap_in2) + 1) and m_neg = cap_out - m_ref.  (The multiplication per score stays: queries scaled
  // ahead of the MFMAs and rounded back to 16 bits would save it, and move a score by 2^-9 of its terms -- measured at
  // four times the usual spread of scores: 3e-2 instead of 1.5e-2 max-abs against the oracle.)
  const float inv_sc = 1.f / sc_mul;
  const float cap_out = CAP ? p.softcap * 1.4426950408889634f : 0.f;
  const float cap_in = CAP ? p.scale / p.softcap : 0.f;
  const float cap_in2 = cap_in * 2.8853900817779268f;
  const float cap_m2 = -2.f * cap_out;
  // a raw score to log2 units (sc: what fast_step multiplies it by, cap_in2 or with KS cap_in2 x the page's K scale)
  auto capped = [&](float s, float sc) -> float { return cap_out * fast_tanh(KS ? s * sc * 0.34657359027997264f : s * cap_in); };
  auto prob = [&](float s, float mn, float sc) __attribute__((always_inline)) -> float {
    if constexpr (CAP) {
      const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(s * (KS ? sc : cap_in2)) + 1.f);
      return s == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(__builtin_fmaf(r, cap_m2, mn));  // a masked key is not the cap's lower end
    } else {
      return __builtin_amdgcn_exp2f(__builtin_fmaf(s, sc, mn));
    }
  };
  // KS: the queues move on by a tile (at a barrier, ahead of its request), and take the pair of the tile just described.
  auto queue_shift = [&]() __attribute__((always_inline)) {
    if constexpr (KS) {
#pragma unroll
      for (int c = 0; c < KAH; ++c) {
        kq[c] = kq[c + 1];
        lq[c] = lq[c + 1];
      }
    }
  };
  auto queue_put = [&](int c) __attribute__((always_inline)) {
    if constexpr (KS) {
      kq[c] = td[0].sc;
      lq[c] = td[0].lv;
    }
  };
  // KS: l_acc holds the row sums of one tile, in units of 1 / inv_cur; l_run the sums of the tiles before.  At a tile's
  // first step, ahead of its row-sum MFMAs (the first of which starts from zero), the tile before joins the running sums.
  float l_run[RB], inv_cur = 0.f;
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) l_run[rb] = 0.f;
  auto fold_tile = [&](float lv_new) __attribute__((always_inline)) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) l_run[rb] = __builtin_fmaf(l_acc[rb][0], inv_cur, l_run[rb]);
    inv_cur = __builtin_amdgcn_exp2f(-lv_new);
  };
  // The A operand of the row sums: ones, written to registers once, here.  (Left to the compiler it is rebuilt from
  // scalar registers right in front of the MFMA that reads it, and an MFMA issued through an assembly statement gets
  // no pause behind a vector instruction that writes one of its operands: it read the old register contents.)
  u32x4 ones = {H::kOnes, H::kOnes, H::kOnes, H::kOnes};
  asm volatile("" : "+v"(ones));

  // Lane addresses of the operand reads, relative to a ring slot.  K operand kk of a block: key j32 of the block, chunk 2 kk + hh.
  // V operand (db, s) of a block: two transposing reads; the lane addresses key 16 s + 4 hh (+ 8) + n / 4 of the block,
  // dims 32 db + 16 (lane / 16 % 2) + 4 (n % 4).
  uint32_t kaddr[NKK], vaddr[DB];
  auto set_lane_addrs = [&](int ln) __attribute__((always_inline)) {  // ln: the lane's number
    const int j = ln & 31, h2 = ln >> 5;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) kaddr[kk] = lds_base + (uint32_t)(j * RKL + (((2 * kk + h2) ^ swz_key<RKL>(j)) << 4));
    const int key = 4 * h2 + ((ln & 15) >> 2);
    const int byte0 = 32 * ((ln >> 4) & 1) + 8 * (ln & 3);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int off = 64 * db + byte0;
      vaddr[db] = lds_base + (uint32_t)(KN * HALF + key * RKL + ((((off >> 4) ^ swz_key_v32<RKL>(key))) << 4) + (off & 15));
    }
  };
  set_lane_addrs(lane);
  auto rv_at = [&](uint32_t a) __attribute__((always_inline)) -> u32x4 {  // one V operand: 16 keys x 32 dims, transposed on the way
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(uintptr_t)a));
    const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(uintptr_t)(a + 8 * RKL)));
    return (u32x4){lo[0], lo[1], hi[0], hi[1]};
  };

  // Raises the references of the rows whose new scores (maxima in lmx, raw) exceed them by more than the slack; what
  // has been accumulated, and the pending probabilities pend (relative to the old reference), are scaled to match.
  // sc: the scale of the scores the maxima were taken of (KS: thr is then in scaled units, the scores of two tiles having no common unit).
  auto check = [&](u32x4 (&pend)[RB][2], bool has_pending, float sc) __attribute__((always_inline)) {
    bool grow = false;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) grow |= (KS ? lmx[rb] * sc : lmx[rb]) > thr[rb];
    if (__builtin_expect(__any(grow), 0)) {  // rare: what the register allocator has to park, it parks around this block
      mfma_settle_acc(*(f32x16 (*)[RB * DB])o_acc, l_acc);  // the accumulators may still be on their way
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const float raw = xor32_max(lmx[rb]);
        const float mx = CAP ? (raw == -INFINITY ? -INFINITY : capped(raw, sc)) : raw * sc;
        const float m_new = fmaxf(m_ref[rb], ceilf(mx));
        float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_ref[rb] - m_new);  // a power of two, or 0
        m_ref[rb] = m_new;
        if constexpr (CAP) {  // the raw score whose capped value is m_new + slack, if there is one
          const float y = (m_new + kMaxSlack) / cap_out;
          const float ath = 0.5f * __logf((1.f + y) / (1.f - y));  // (KS: thr in units of raw score x sc)
          thr[rb] = (m_new == -INFINITY) ? -INFINITY : (y >= 0.999f ? INFINITY : (KS ? ath * 2.8853900817779268f : ath / cap_in));
          m_neg[rb] = (m_new == -INFINITY) ? 0.f : cap_out - m_new;
        } else {
          thr[rb] = KS ? m_new + kMaxSlack : (m_new + kMaxSlack) * inv_sc;
          m_neg[rb] = (m_new == -INFINITY) ? 0.f : -m_new;
        }
        asm volatile("s_nop 1" : "+v"(alpha));
        {
          f32x16 l = l_acc[rb];
          l[0] *= alpha;  // the register the epilogue reads; the others hold the same sum and are never read
          l_acc[rb] = l;
          if constexpr (KS) l_run[rb] *= alpha;
        }
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          f32x16 o = o_acc[rb][db];
#pragma unroll
          for (int r = 0; r < 16; ++r) o[r] *= alpha;
          o_acc[rb][db] = o;
        }
        if (has_pending) {
#pragma unroll
          for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int w = 0; w < 4; ++w) pend[rb][s][w] = W::scale_pair(pend[rb][s][w], alpha);
        }
      }
    }
  };

  // ---- the pinned step ---------------------------------------------------------------------------------------
  // PAR = (b + 1) % 2: the buffer of block b+1 (the other receives block b+2 and held block b).  ka: lane addresses of
  // the K operands of block b+2; kn: of the first PD operands of block b+3 (read at the end); va: lane addresses of the V
  // operands of block b.  dl / dv0, dv1 / dg: LDS address, lane offsets and global base of the NG half tiles the step requests.
  auto fast_step = [&](auto par_tag, auto&& ka, auto&& kn, auto&& va, auto&& in_slot, const uint32_t (&dl)[NG],
                       const uint32_t (&dv0)[NLH], const uint32_t (&dv1)[NLH], const char* const (&dg)[NG], const float sc, const float lv, auto first_tag) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_tag)::value;
    constexpr bool FIRST = decltype(first_tag)::value;  // KS: the step is the first of its tile
    float mn[RB];  // what the exponent adds to a scaled score (KS: the logarithm of the tile's V scale on top)
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) mn[rb] = KS ? m_neg[rb] + lv : m_neg[rb];
    f32x16 (&s_cur)[RB] = sa[PAR];              // S(b+1), consumed by the softmax
    f32x16 (&s_nxt)[RB] = sa[PAR ^ 1];          // S(b+2), produced
    u32x4 (&p_cur)[RB][2] = pb[PAR ^ 1];        // P(b), consumed by the PV product
    u32x4 (&p_nxt)[RB][2] = pb[PAR];            // P(b+1), produced
    auto rk = [&](uint32_t a) __attribute__((always_inline)) -> u32x4 { return *(const __attribute__((address_space(3))) u32x4*)(uintptr_t)a; };
    auto rv = [&](int o) __attribute__((always_inline)) -> u32x4 { return rv_at(va(o / 2) + (uint32_t)(16 * (o % 2) * RKL)); };
    auto dma = [&](int j) __attribute__((always_inline)) {  // m0 is set by a half tile's first request and kept for its others
      if (j % NLH == 0) dma16_at(dl[j / NLH], 0, j < NLH ? dv0[0] : dv1[0], dg[j / NLH]);
      else dma16_at_same_m0(j % NLH, j < NLH ? dv0[j % NLH] : dv1[j % NLH], dg[j / NLH]);
    };
    float xa = 0.f, xb = 0.f, ea = 0.f, eb = 0.f, fa = 0.f, fb = 0.f;  // softmax values in flight between slots
    float mx_part[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) mx_part[rb] = -INFINITY;
    // One MFMA slot; PH: 0 the scores, 1 between the products, 2 the PV product.  (A loop per phase: one loop over all
    // slots, each iteration holding the code of all three phases until it is unrolled, grows past what the compiler
    // unrolls in full, and the score registers it indexes then live in memory.)
    auto slot = [&](auto ph_tag, int k) __attribute__((always_inline)) {
      constexpr int PH = decltype(ph_tag)::value;
      // -- the MFMA of the slot: scores, then the row sums of block b (a V^T tile of ones against P^T leaves, in every
      //    accumulator register of lane j32, the sum of row j32's probabilities as rounded to 16 bits: exactly the weights
      //    the PV product uses), then the PV product; behind an operand's last MFMA, the read of the operand PD further on
      if constexpr (PH == 0) {
        const int g = k / RB, rb = k % RB;
        if (rb == 0 && g % 2 == 0) asm volatile("" ::"v"(ops[g % PD]), "v"(ops[(g + 1) % PD]));  // one wait for two operands
        if (g == 0) W::mfma_s0(s_nxt[rb], ops[g % PD], qf[rb][g]);
        else W::mfma_s(s_nxt[rb], ops[g % PD], qf[rb][g]);
        if (rb == RB - 1) {
          const int nx = g + PD;
          if (nx < NKK) ops[g % PD] = rk(ka(nx));
          else ops[g % PD] = rv(nx - NKK);
        }
      } else if constexpr (PH == 1) {
        const int e = k - NQ, rb = e % RB, sh = e / RB;
        if (KS && FIRST && sh == 0) W::mfma_o0(l_acc[rb], ones, p_cur[rb][sh]);
        else W::mfma_o(l_acc[rb], ones, p_cur[rb][sh]);
        // These slots carry no softmax and no operand read: the step's tile loads are requested from here on, where the
        // time the load unit takes to accept 1 KiB of addresses hides behind an MFMA.
        if (NDI <= NSUM && e < NDI) dma(e);
      } else {
        const int kk2 = k - NQ - NSUM, v = kk2 / RB, rb = kk2 % RB, db = v / 2, sh = v % 2, g = NKK + v;
        if (rb == 0 && g % 2 == 0) asm volatile("" ::"v"(ops[g % PD]), "v"(ops[(g + 1) % PD]));
        W::mfma_o(o_acc[rb][db], ops[g % PD], p_cur[rb][sh]);
        if (rb == RB - 1) {
          const int nx = g + PD;
          if (nx < NKK + NVO) ops[g % PD] = rv(nx - NKK);
          else ops[g % PD] = rk(kn(nx - NKK - NVO));  // the next step's first operands
        }
      }
      // The MFMA leads its slot: left free, the compiler moves a slot's pack ahead of it, directly behind the exponentials
      // of the slot before, where it needs a wait state of its own and then waits for their results.
      __builtin_amdgcn_sched_barrier(0);
      // -- the softmax of block b+1, on the slots of the two products: pair ip = (row block, register pair) owns SPP slots
      if constexpr (PH != 1) {
        const int ks = k < NQ ? k : k - NSUM;
        if (NDI > NSUM && ks % DSP == DSP - 1 && ks / DSP < NDI) dma(ks / DSP);  // more tile loads than row-sum slots: spread evenly
        const int ip = ks / SPP, st = ks % SPP;
        const int srb = ip / 8, sr2 = ip % 8;
        const int jp = ip - 1, prb = jp / 8, pr2 = jp % 8;  // the pair before
        if constexpr (!CAP) {
          // first the scaled differences of the pair, and the pair before packed (behind the two multiply-adds: they are
          // the distance an exponential wants from its reader); half the pair's slots on, the exponentials
          if (st == 0) {
            xa = __builtin_fmaf(s_cur[srb][2 * sr2], sc, mn[srb]);
            xb = __builtin_fmaf(s_cur[srb][2 * sr2 + 1], sc, mn[srb]);
            if (ip > 0) p_nxt[prb][pr2 / 4][pr2 % 4] = H::pack(ea, eb);
          } else if (st == SPP / 2) {
            ea = __builtin_amdgcn_exp2f(xa);
            eb = __builtin_amdgcn_exp2f(xb);
          }
        } else {
          // four stages, one slot each; the last exponentials and the packing of a pair ride on the first two slots of the next
          if (st == 0) {
            xa = s_cur[srb][2 * sr2] * (KS ? sc : cap_in2);
            xb = s_cur[srb][2 * sr2 + 1] * (KS ? sc : cap_in2);
            if (ip > 0) {
              fa = __builtin_amdgcn_exp2f(ea);
              fb = __builtin_amdgcn_exp2f(eb);
            }
          } else if (st == 1) {
            xa = __builtin_amdgcn_exp2f(xa);
            xb = __builtin_amdgcn_exp2f(xb);
            if (ip > 0) p_nxt[prb][pr2 / 4][pr2 % 4] = H::pack(fa, fb);
          } else if (st == 2) {
            xa += 1.f;
            xb += 1.f;
            xa = __builtin_amdgcn_rcpf(xa);
            xb = __builtin_amdgcn_rcpf(xb);
          } else {
            ea = __builtin_fmaf(xa, cap_m2, mn[srb]);
            eb = __builtin_fmaf(xb, cap_m2, mn[srb]);
          }
        }
        // (the last pair's stages have no reader inside the step: unpinned they gather behind its last MFMA)
        if (ip == NPAIR - 1) asm volatile("" : "+v"(xa), "+v"(xb), "+v"(ea), "+v"(eb));
      }
      // -- row maxima of S(b+2), whose MFMAs lie at least NSUM slots back: one three-way maximum per MSP PV slots
      if (PH == 2 && (k - NQ - NSUM) % MSP == 0) {
        const int e = (k - NQ - NSUM) / MSP, mrb = e / 8, mr2 = e % 8;
        mx_part[mrb] = __builtin_fmaxf(__builtin_fmaxf(mx_part[mrb], s_nxt[mrb][2 * mr2]), s_nxt[mrb][2 * mr2 + 1]);
        asm volatile("" : "+v"(mx_part[mrb]));  // in this slot: left free, the chain of maxima gathers behind the step's last MFMA
      }
      in_slot(k);  // what the caller wants done during this slot: the lane addresses of the steps to come
      __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int k = 0; k < NQ; ++k) slot(std::integral_constant<int, 0>{}, k);
#pragma unroll
    for (int k = NQ; k < NQ + NSUM; ++k) slot(std::integral_constant<int, 1>{}, k);
#pragma unroll
    for (int k = NQ + NSUM; k < NQ + NSUM + NP; ++k) slot(std::integral_constant<int, 2>{}, k);
    {  // the last pair
      constexpr int jp = NPAIR - 1, prb = jp / 8, pr2 = jp % 8;
      if constexpr (CAP) {
        ea = __builtin_amdgcn_exp2f(ea);
        eb = __builtin_amdgcn_exp2f(eb);
      }
      p_nxt[prb][pr2 / 4][pr2 % 4] = H::pack(ea, eb);
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) lmx[rb] = mx_part[rb];
  };

  // ---- the same step written plainly, with run-time flags ---------------------------------------------------------
  // do_qk: block b+2 exists; do_sm: block b+1 exists; do_pv: block b >= 0; next_k: block b+3 exists (its first operands
  // are read at the end); first: the first operands of block b+2 have not been read ahead.  kb2: first key of block b+2.
  // koff / nkoff / voff: byte offsets (slot and part) of blocks b+2 / b+3 in the K ring and of block b in the V ring.
  auto slow_step = [&](auto par_tag, uint32_t koff, uint32_t nkoff, uint32_t voff, bool do_qk, bool do_sm, bool do_pv, bool next_k, bool first, int kb2, float sc, float lv, bool first_of_tile) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_tag)::value;
    f32x16 (&s_cur)[RB] = sa[PAR];
    f32x16 (&s_nxt)[RB] = sa[PAR ^ 1];
    u32x4 (&p_cur)[RB][2] = pb[PAR ^ 1];
    u32x4 (&p_nxt)[RB][2] = pb[PAR];
    auto rk = [&](uint32_t off, int kk) __attribute__((always_inline)) -> u32x4 {
      return *(const __attribute__((address_space(3))) u32x4*)(uintptr_t)(kaddr[kk] + off);
    };
    auto rv = [&](int o) __attribute__((always_inline)) -> u32x4 { return rv_at(vaddr[o / 2] + voff + (uint32_t)(16 * (o % 2) * RKL)); };
    if (do_qk) {
      if (first) {
#pragma unroll
        for (int o = 0; o < PD; ++o) ops[o] = rk(koff, o);
      }
#pragma unroll
      for (int g = 0; g < NKK; ++g) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          if (g == 0) W::mfma_s0(s_nxt[rb], ops[g % PD], qf[rb][g]);
          else W::mfma_s(s_nxt[rb], ops[g % PD], qf[rb][g]);
        }
        if (g + PD < NKK) ops[g % PD] = rk(koff, g + PD);
      }
    }
    if (do_sm) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int r2 = 0; r2 < 8; ++r2) {
          const float e0 = prob(s_cur[rb][2 * r2], KS ? m_neg[rb] + lv : m_neg[rb], sc);
          const float e1 = prob(s_cur[rb][2 * r2 + 1], KS ? m_neg[rb] + lv : m_neg[rb], sc);
          p_nxt[rb][r2 / 4][r2 % 4] = H::pack(e0, e1);
        }
    }
    if (do_pv) {
      u32x4 (&vo)[PD] = ops;  // the K operands read ahead for the next step are read at the end of this one
#pragma unroll
      for (int o = 0; o < PD; ++o) vo[o] = rv(o);
#pragma unroll
      for (int sh = 0; sh < 2; ++sh)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {  // row sums of block b
          if (KS && first_of_tile && sh == 0) W::mfma_o0(l_acc[rb], ones, p_cur[rb][sh]);
          else W::mfma_o(l_acc[rb], ones, p_cur[rb][sh]);
        }
#pragma unroll
      for (int g = 0; g < NVO; ++g) {
        const int db = g / 2, s = g % 2;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          W::mfma_o(o_acc[rb][db], vo[g % PD], p_cur[rb][s]);
        }
        if (g + PD < NVO) vo[g % PD] = rv(g + PD);
      }
    }
    if (do_qk) {  // mask S(b+2) in place and take the row maxima
      mfma_settle(s_nxt);
      const bool plain = kb2 >= wave_lo && kb2 + BK <= wave_hi;  // no row of the wave masks a key of this block
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        float mx = -INFINITY;
        const int lo_rel = row_lo[rb] - kb2 - 4 * hh;
        const uint32_t span = (uint32_t)(row_hi[rb] - row_lo[rb]);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float sv = s_nxt[rb][r];
          if (!plain) {
            const int c = 8 * (r / 4) + (r % 4);
            sv = ((uint32_t)(c - lo_rel) < span) ? sv : -INFINITY;
            s_nxt[rb][r] = sv;
          }
          mx = fmaxf(mx, sv);
        }
        lmx[rb] = mx;
      }
    }
    if (next_k) {
#pragma unroll
      for (int o = 0; o < PD; ++o) ops[o] = rk(nkoff, o);
    }
  };

  // ---- the walk over the key range -------------------------------------------------------------------------
  // Step b (b = -2 .. n_blocks - 1): scores of block b+2, softmax of block b+1, PV product of block b.  Requests so far,
  // in order: K and V of the tiles the first barrier expects behind it, then per barrier V(u + VAH), K(u + KAH).
  const int n_blocks = SPT * n_tiles;
#pragma unroll
  for (int t = 0; t < U0 + KAH; ++t) {
    next_tile();
    queue_put(t - U0 + 1);  // (the first barrier moves the queues on by one)
    if (t < n_tiles) issue_half(false, t % KN, td[0]);
    if (t < U0 + VAH && t < n_tiles) issue_half(true, t % KN, td[0]);
  }
  // The query rows, requested at the top: from here on in the accumulation file.
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {  // waited for here, behind the first tile requests and not inside the loop; kept in the accumulation file from here on
      u32x4 v = qf[rb][kk];
      asm volatile("" : "+a"(v));
      qf[rb][kk] = v;
    }
  auto ring_off = [&](int x) -> uint32_t { return (uint32_t)(((x / SPT) % KN) * HALF + (x % SPT) * BK * RKL); };  // block x >= 0 in its ring
  auto head = [&](int u) __attribute__((always_inline)) {  // barrier u, written plainly
    // in flight may stay the requests of the FLYB barriers before, where they made them in full
    if (u - FLYB >= U0 && u - 1 + KAH < n_tiles) wait_loads_and_barrier<2 * FLYB * NLH>();
    else wait_loads_and_barrier<0>();
    const int vt = u + VAH, kt = u + KAH;
    if (vt < n_tiles) issue_half(true, vt % KN, td[DQ - 1]);
    queue_shift();
    next_tile();
    queue_put(KAH);
    if (kt < n_tiles) issue_half(false, kt % KN, td[0]);
  };
  auto slow_step_at = [&](auto par_tag, int b) __attribute__((always_inline)) {
    if (b % SPT == 0) head(b / SPT);  // (b is even wherever SPT is 2 and b is negative)
    const bool do_qk = b + 2 < n_blocks, do_sm = b + 1 >= 0 && b + 1 < n_blocks, do_pv = b >= 0 && b < n_blocks;
    const bool next_k = b + 3 < n_blocks, first = b == -2;
    constexpr int PAR = decltype(par_tag)::value;
    // KS: block b + 1 lies in the barrier's tile if b is even and there are two steps per tile, else in the next; block b in the barrier's
    constexpr int C1 = (SPT == 2 && PAR == 1) ? 0 : 1;
    const float sc = kq[C1], lv = lq[C1];
    const bool first_of_tile = SPT == 1 || PAR == 1;  // (b is even)
    if constexpr (KS) {
      if (first_of_tile && do_pv) {  // (a step past the last block issues no row sums: the last tile's stay for the epilogue)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) asm volatile("s_nop 15\n\ts_nop 15" : "+a"(l_acc[rb]));  // the row sums may still be on their way
        fold_tile(lq[0]);
      }
    }
    if (do_sm) check(pb[PAR ^ 1], do_pv, sc);
    slow_step(par_tag, ring_off(b + 2), ring_off(b + 3), ring_off(max(b, 0)), do_qk, do_sm, do_pv, next_k, first, kv_lo + (b + 2) * BK, sc, lv, first_of_tile);
  };
  // Pairs of steps (b, b + 1), b even, the pinned code may serve: b >= 0, the barriers whose requests may be in flight
  // were regular ones, blocks b+2 and b+3 exist and are unmasked for the whole wave ...
  const int b_fast_lo = max(0, (((wave_lo - kv_lo + BK - 1) / BK - 2 + 1) >> 1) << 1);
  // ... and the tiles its barriers request (with plain lane offsets) are not the one that straddles the end of the
  // context, whose rows past the end must not be fetched as they are.  Tiles past the key range may be requested: the
  // cursor has moved on into valid pages (the next chunk's keys, or whatever page the table names: ids are clipped),
  // the bytes land in ring slots nobody reads again, and the count of loads in flight stays what the barriers assume.
  // The plain steps do not request such tiles, so the plain barriers ahead of the first pinned one must all have had
  // real tiles to request.
  const int n_whole = min(n_tiles, (sp.ctx - kv_lo) / TT);  // tiles without a row past the context
  const int b_req_hi = n_whole == n_tiles ? 0x7ffffff0 : (SPT == 2 ? 2 * (n_whole - KAH) : n_whole - KAH - 1);
  const bool lead_in_full = b_fast_lo / SPT - 1 + KAH < n_tiles;
  const int b_fast_hi = lead_in_full ? max(b_fast_lo, min(min((wave_hi - kv_lo) / BK - 3, n_blocks - 3), b_req_hi)) : b_fast_lo;  // first even b behind them
  int b = -2;
  for (; b < b_fast_lo; b += 2) {
    slow_step_at(std::integral_constant<int, 1>{}, b);
    slow_step_at(std::integral_constant<int, 0>{}, b + 1);
  }
  // What the pinned loop reads but never writes is touched once here: should the compiler have parked any of it in
  // memory across the code above, its wait for the reload lands here and not inside the loop, where a wait on the
  // vector-memory counter would also wait for the tiles in flight.
#pragma unroll
  for (int u = 0; u < NLH; ++u) asm volatile("" : "+v"(voff_k[u]), "+v"(voff_v[u]));
  asm volatile("" : "+v"(pages_vec));
  if constexpr (KS) asm volatile("" : "+v"(sck_vec), "+v"(lvs_vec));
  if (b < b_fast_hi) {
    // Ring offsets of the tiles u .. u + KN - 1, u the index of the next barrier (r[c]: tile u + c), turned once per barrier.
    uint32_t r[KN];
#pragma unroll
    for (int c = 0; c < KN; ++c) r[c] = (uint32_t)(((b / SPT + c) % KN) * HALF);
    // Lane addresses the steps read their operands through: ring offset added.  A: K of tile u + KC (the tile whose
    // scores the barrier's steps take); VA: V of tile u.  Operands 8 k-steps, or 4 dim blocks, apart lie 256 bytes apart
    // whatever the lane's swizzle key, and the parts of a tile a constant apart: those fold into the instructions' offsets.
    // Each is moved on to the next barrier's ring slot behind its last use, by an addition pinned to a slot of the step:
    // computed at the head of a step, ahead of its first MFMA, the additions are time the matrix pipe stands idle.
    constexpr int KC = SPT == 2 ? 1 : 2;
    constexpr int NKA = NKK < 8 ? NKK : 8, NVA = DB < 4 ? DB : 4;
    static_assert(NKK % NKA == 0 && DB % NVA == 0 && NKA >= PD, "");
    uint32_t A[NKA], VA[NVA];
#pragma unroll
    for (int kk = 0; kk < NKA; ++kk) A[kk] = kaddr[kk] + r[KC];
#pragma unroll
    for (int db = 0; db < NVA; ++db) VA[db] = vaddr[db] + r[0];
    const uint32_t k_lds0 = lds_base + dma_wave_lds, v_lds0 = k_lds0 + (uint32_t)(KN * HALF);
    auto pinned_add = [&](uint32_t sgpr, uint32_t vgpr) __attribute__((always_inline)) -> uint32_t {
      uint32_t d;
      asm volatile("v_add_u32 %0, %1, %2" : "=v"(d) : "s"(sgpr), "v"(vgpr));
      return d;
    };
    // The last step of a barrier moves the addresses on: K once the step's own K operands are read (the row-sum slots on;
    // the operands read at its end are the next barrier's), V behind the last V operand.
    constexpr int K_UPD0 = NQ, K_UPD_SLOTS = NSUM + 4, V_UPD0 = NQ + NSUM + NP - 4;
    constexpr int K_PER = (NKA + K_UPD_SLOTS - 1) / K_UPD_SLOTS;
    auto move_on = [&](int k) __attribute__((always_inline)) {
#pragma unroll
      for (int kk = 0; kk < NKA; ++kk)
        if (k == K_UPD0 + kk / K_PER) A[kk] = pinned_add(r[(KC + 1) % KN] - r[KC], A[kk]);
#pragma unroll
      for (int db = 0; db < NVA; ++db)
        if (k == V_UPD0 + db) VA[db] = pinned_add(r[1 % KN] - r[0], VA[db]);
    };
    auto nothing = [&](int) __attribute__((always_inline)) {};

    // one barrier and the SPT steps behind it; PAR0: the buffer the first of them hands its softmax
    auto fast_trip = [&](auto par_tag) __attribute__((always_inline)) {
      constexpr int PAR0 = decltype(par_tag)::value;
      // visible now: K tiles up to u + KNO, V tiles up to u; in flight stay the requests of the FLYB barriers before
      wait_loads_and_barrier<2 * FLYB * NLH>();
      queue_shift();
      const float sc0 = kq[SPT == 2 ? 0 : 1], sc1 = kq[1];  // of blocks b + 1 and b + 2
      const float lv0 = lq[SPT == 2 ? 0 : 1], lv1 = lq[1];
      if constexpr (KS) fold_tile(lq[0]);  // (the row sums of the tile before were issued a whole PV phase ago)
      check(pb[PAR0 ^ 1], true, sc0);
      // this barrier's requests, made from inside its steps: V(u + VAH), described DQ tiles ago, and K(u + KAH)
      const char* v_ptr = v_base + td[DQ - 1].off;
      next_tile(false);
      queue_put(KAH);
      const char* k_ptr = k_base + td[0].off;
      const uint32_t v_lds = v_lds0 + r[VAH % KN];
      const uint32_t k_lds = k_lds0 + r[KAH % KN];
      if constexpr (SPT == 2) {
        constexpr uint32_t PART = BK * RKL;
        const uint32_t dl0[1] = {v_lds}, dl1[1] = {k_lds};
        const char* const dg0[1] = {v_ptr};
        const char* const dg1[1] = {k_ptr};
        fast_step(std::integral_constant<int, PAR0>{},
                  [&](int nx) { return A[nx]; }, [&](int o) { return A[o] + PART; }, [&](int db) { return VA[db]; }, nothing,
                  dl0, voff_v, voff_v, dg0, sc0, lv0, std::true_type{});
        check(pb[PAR0], true, sc1);
        fast_step(std::integral_constant<int, PAR0 ^ 1>{},
                  [&](int nx) { return A[nx] + PART; }, [&](int o) { return A[o]; }, [&](int db) { return VA[db] + PART; }, move_on,
                  dl1, voff_k, voff_k, dg1, sc1, lv1, std::false_type{});
      } else {
        const uint32_t dl0[2] = {v_lds, k_lds};
        const char* const dg0[2] = {v_ptr, k_ptr};
        fast_step(std::integral_constant<int, PAR0>{},
                  [&](int nx) { return A[nx % NKA] + (uint32_t)(256 * (nx / NKA)); }, [&](int o) { return A[o]; },
                  [&](int db) { return VA[db % NVA] + (uint32_t)(256 * (db / NVA)); }, move_on, dl0, voff_v, voff_k, dg0, sc0, lv0, std::true_type{});
      }
      const uint32_t r0 = r[0];
#pragma unroll
      for (int c = 0; c + 1 < KN; ++c) r[c] = r[c + 1];
      r[KN - 1] = r0;
    };
    for (; b < b_fast_hi; b += 2) {
      // No branch between the steps of an iteration: instructions of a pinned step must not find a later block to sink
      // into.  An iteration moves the cursor by at most one column (pages hold two tiles or more).
      refill_pages(1);
      fast_trip(std::integral_constant<int, 1>{});
      if constexpr (SPT == 1) fast_trip(std::integral_constant<int, 0>{});
    }
    // The plain steps behind read through the lane addresses without a ring offset again: made anew here (from a copy of the
    // lane number the compiler cannot see through), they take no registers across the loop.
    int ln = lane;
    asm volatile("" : "+v"(ln));
    set_lane_addrs(ln);
  }
  for (; b < n_blocks; b += 2) {
    slow_step_at(std::integral_constant<int, 1>{}, b);
    slow_step_at(std::integral_constant<int, 0>{}, b + 1);
  }

  // ---- epilogue -----------------------------------------------------------------------------------------
  // A lane holds 4-dim pieces of its own row: stored as they are, every store instruction would scatter 16- or 32-byte
  // pieces over 32 rows.  The rows go through the wave's share of the (now idle) rings instead and leave as whole rows,
  // 16 bytes per lane over consecutive lanes.  Rows narrower than the padded head (Dq < D) are stored piecewise.
  mfma_settle_acc(*(f32x16 (*)[RB * DB])o_acc, l_acc);
  const bool staged = p.Dq == D;
  constexpr int RS32 = D * 4 + 16, RS16 = D * 2 + 16;  // row strides of the staging area: 16 bytes of padding spread the rows over the banks
  static_assert(NW * 32 * RS32 <= 2 * KN * HALF, "the staging areas of the waves fit the rings");
  const uint32_t stage = lds_base + (uint32_t)wave * (uint32_t)(32 * RS32);
  if (staged) wait_loads_and_barrier<0>();  // every wave is through with the rings, and no tile is still on its way into them
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const float l_tot = KS ? __builtin_fmaf(l_acc[rb][0], inv_cur, l_run[rb]) : l_acc[rb][0];
    // where the lane's row goes: its index among the [T][Hq] rows of the output (or of a chunk's partial rows), -1: nowhere
    const int my_slot = row_ok[rb] ? out_tok[rb] * p.Hq + out_head[rb] : -1;
    if (single) {
      const float l_fin = with_sink(p, out_head[rb], m_ref[rb], l_tot);
      const float inv = l_fin > 0.f ? 1.f / l_fin : 0.f;
      if (!staged) {
        if (row_ok[rb]) {
          uint16_t* orow = (uint16_t*)p.out + (int64_t)my_slot * p.Dq + 4 * hh;
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const f32x16 o = o_acc[rb][db];
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {  // registers 4 q4 .. 4 q4 + 3 are dims 32 db + 8 q4 + 4 hh + 0..3
              const u32x2 w = {H::pack(o[4 * q4] * inv, o[4 * q4 + 1] * inv), H::pack(o[4 * q4 + 2] * inv, o[4 * q4 + 3] * inv)};
              if (32 * db + 8 * q4 + 4 * hh < p.Dq) *(u32x2*)(orow + 32 * db + 8 * q4) = w;
            }
          }
        }
      } else {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const f32x16 o = o_acc[rb][db];
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            const u32x2 w = {H::pack(o[4 * q4] * inv, o[4 * q4 + 1] * inv), H::pack(o[4 * q4 + 2] * inv, o[4 * q4 + 3] * inv)};
            *(__attribute__((address_space(3))) u32x2*)(uintptr_t)(stage + (uint32_t)(j32 * RS16 + (32 * db + 8 * q4 + 4 * hh) * 2)) = w;
          }
        }
        constexpr int CPRO = D * 2 / 16, RPIO = 64 / CPRO;  // 16-byte chunks per row, rows per store instruction
#pragma unroll
        for (int it = 0; it < 32 / RPIO; ++it) {
          const int r = it * RPIO + lane / CPRO, c = lane % CPRO;
          const u32x4 v = *(const __attribute__((address_space(3))) u32x4*)(uintptr_t)(stage + (uint32_t)(r * RS16 + c * 16));
          const int slot_r = __shfl(my_slot, r);
          if (slot_r >= 0) *(u32x4*)((char*)p.out + ((int64_t)slot_r * D) * 2 + c * 16) = v;
        }
      }
    } else {
      const int64_t pbase = (int64_t)chunk * p.T * p.Hq;
      if (!staged) {
        if (row_ok[rb]) {
          float* prow = p.pre_o + (pbase + my_slot) * D + 4 * hh;
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const f32x16 o = o_acc[rb][db];
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4)
              *(f32x4*)(prow + 32 * db + 8 * q4) = (f32x4){o[4 * q4], o[4 * q4 + 1], o[4 * q4 + 2], o[4 * q4 + 3]};
          }
        }
      } else {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const f32x16 o = o_acc[rb][db];
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4)
            *(__attribute__((address_space(3))) f32x4*)(uintptr_t)(stage + (uint32_t)(j32 * RS32 + (32 * db + 8 * q4 + 4 * hh) * 4)) =
                (f32x4){o[4 * q4], o[4 * q4 + 1], o[4 * q4 + 2], o[4 * q4 + 3]};
        }
        constexpr int CPRO = D * 4 / 16, RPIO = CPRO >= 64 ? 1 : 64 / CPRO;  // 16-byte chunks per row, rows per store instruction
        constexpr int IPR = CPRO >= 64 ? CPRO / 64 : 1;                        // store instructions per row where a row is wider than a wave
#pragma unroll
        for (int it = 0; it < 32 / RPIO * IPR; ++it) {
          const int r = IPR > 1 ? it / IPR : it * RPIO + lane / CPRO;
          const int c = IPR > 1 ? (it % IPR) * 64 + lane : lane % CPRO;
          const f32x4 v = *(const __attribute__((address_space(3))) f32x4*)(uintptr_t)(stage + (uint32_t)(r * RS32 + c * 16));
          const int slot_r = __shfl(my_slot, r);
          if (slot_r >= 0) *(f32x4*)((char*)p.pre_o + ((pbase + slot_r) * D) * 4 + c * 16) = v;
        }
      }
      if (row_ok[rb] && hh == 0) {
        p.pre_ml[(pbase + my_slot) * 2 + 0] = m_ref[rb];
        p.pre_ml[(pbase + my_slot) * 2 + 1] = l_tot;
      }
    }
  }
}

template <int D, int NW, int RB, int HT, bool CAP, bool KS = false>
static int launch_x32(hipStream_t stream, const AttnParams& p) {
  constexpr int ROWS = NW * RB * 32;
  if (p.pre_rows != ROWS) return (int)hipErrorInvalidValue;  // the plan and merge kernels are told this row-tile height
  const int64_t slots = ((int64_t)p.T * p.group) / ROWS + p.S;  // upper bound on row tiles of the batch
  const int64_t blocks = slots * p.Hkv * p.pre_max_chunks;
  if (blocks > 0x7fffffff) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL((attn_prefill_x32_kernel<D, NW, RB, HT, CAP, KS>), dim3((unsigned)blocks), dim3(64 * NW), 0, stream, p);
  return (int)hipGetLastError();
}

// Query rows one workgroup of this kernel owns at the call's shape, 0 where the kernel does not apply.  Served: bf16 or
// float16 pages of head size 128 without a soft cap (256 rows), bf16 pages of head size 256 with or without one (128
// rows); page sizes that are multiples of 64 tokens.
int prefill_x32_rows(const AttnParams& p) {
  if (p.page_size % 64 != 0 || (int64_t)64 * p.token_stride >= ((int64_t)1 << 31)) return 0;
  if (p.page_stride % 256 != 0 || (int64_t)p.P * (p.page_stride >> 8) >= ((int64_t)1 << 32)) return 0;  // page offsets are held in units of 256 bytes
  if (p.D == 128 && (p.kv_dtype == RPA_BF16 || p.kv_dtype == RPA_F16) && !(p.softcap > 0.f)) return 256;
  if (p.D == 256 && p.kv_dtype == RPA_BF16) return 128;
  return 0;
}

int launch_attn_prefill_x32(hipStream_t stream, const AttnParams& p) {
  if (p.wide != nullptr) {  // bf16 copies of 8-bit pages
    if ((p.D != 128 && p.D != 256) || p.kv_dtype != RPA_BF16 || (p.softcap > 0.f && p.D != 256)) return (int)hipErrorInvalidValue;
    if (p.D == 256) return p.softcap > 0.f ? launch_x32<256, 4, 1, RPA_BF16, true, true>(stream, p) : launch_x32<256, 4, 1, RPA_BF16, false, true>(stream, p);
    return launch_x32<128, 4, 2, RPA_BF16, false, true>(stream, p);
  }
  if (p.D == 256) return p.softcap > 0.f ? launch_x32<256, 4, 1, RPA_BF16, true>(stream, p) : launch_x32<256, 4, 1, RPA_BF16, false>(stream, p);
  if (p.kv_dtype == RPA_F16) return launch_x32<128, 4, 2, RPA_F16, false>(stream, p);
  return launch_x32<128, 4, 2, RPA_BF16, false>(stream, p);
}

}  // namespace rpa
