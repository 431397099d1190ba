// MFMA prefill / chunked-prefill attention over the paged cache.
//
// Serves sequences with more than 16 query rows per KV head (row = (query token, head of the GQA
// group), token-major).  A workgroup owns ROWS = NW*RB*16 consecutive rows of one (sequence, KV
// head): each of its NW waves keeps RB 16-row blocks (Q as MFMA B operands, O^T accumulators,
// running max / sum) in registers.  K/V tiles of TT keys are loaded once per workgroup with
// 128-bit loads, one tile ahead, into a double-buffered swizzled LDS tile (8-bit pages are
// widened to bf16 on the way in, so the compute path sees bf16 only); every wave then reads the
// tile in MFMA operand order and reuses each K / V operand for its RB row blocks:
//     S^T[key][row]  = K[key][:] . Q[row][:]            v_mfma_f32_16x16x32_bf16, k = head dim
//     O^T[dim][row] += V^T[dim][key] . P^T[key][row]    v_mfma_f32_16x16x32_bf16, k = 32 keys
// Causal and window limits are per row; key tiles wholly outside a workgroup's limits are never
// loaded, tiles wholly inside skip the masking code.  Block index -> (row tile, KV head) keeps the
// KV head fastest, so the row tiles of one (sequence, head) share an XCD and its L2.
#include "rpa_mfma.h"

namespace rpa {

template <int D, int KVT, int TT, int NW, int RB, bool CAP>
__global__ __launch_bounds__(64 * NW, 2) void attn_prefill_kernel(AttnParams p) {
  constexpr int EB = ElemBytes<KVT>::v;
  constexpr int RKL = D * 2;             // bytes of one K (or V) row in LDS (always bf16)
  constexpr int HBG = 2 * D * EB;        // K_h | V_h span of one token in global memory
  constexpr int LPTG = HBG / 16;         // 16-byte global chunks per token span
  constexpr int THREADS = 64 * NW;
  constexpr int NLD = (TT * LPTG + THREADS - 1) / THREADS;  // global loads per thread per tile
  constexpr bool FULL = (TT * LPTG) % THREADS == 0;         // every thread has NLD chunks of every tile
  constexpr int NS = TT / 16;            // 16-key sub-tiles per tile
  constexpr int DPL = D / 16;            // 16-dim row tiles of O^T
  constexpr int NKK = D / 32;            // k-steps of the score MFMA
  constexpr int ROWS = NW * RB * 16;
  static_assert(ROWS == kPrefillRows, "merge kernel assumes this row-tile height");
  constexpr int TILE_BYTES = TT * 2 * RKL;
  static_assert(NS == 1 || NS == 2, "tile is one or two 16-key sub-tiles");

  __shared__ __attribute__((aligned(16))) unsigned char lds_all[2 * TILE_BYTES];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g4 = lane >> 4;
  const int G = p.group;

  // ---- block -> (sequence, row tile, KV head) ---------------------------------------------------
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
  const int kv_lo = pt.kv_lo + chunk * pt.chunk_len;
  const int kv_hi = (chunk == pt.n_chunks - 1) ? pt.kv_hi : kv_lo + pt.chunk_len;
  const int n_tiles = (kv_hi - kv_lo + TT - 1) / TT;
  const bool single = pt.n_chunks == 1;

  // ---- per row-block lane state --------------------------------------------------------------------
  int row_lo[RB], row_hi[RB];
  bool row_ok[RB];
  int out_tok[RB], out_head[RB];
  bf16x8 qf[RB][NKK];
  int wave_lo, wave_hi;          // keys every row of the wave sees: [max row_lo, min row_hi)
  int wave_lo_min, wave_hi_max;  // keys some row of the wave sees: [min row_lo, max row_hi)
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
  {
    int lo_max = 0, hi_min = 0x7fffffff, lo_min = 0x7fffffff, hi_max = 0;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      lo_max = max(lo_max, row_lo[rb]);
      hi_min = min(hi_min, row_hi[rb]);
      lo_min = min(lo_min, row_lo[rb]);
      hi_max = max(hi_max, row_hi[rb]);
    }
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) {
      lo_max = max(lo_max, __shfl_xor(lo_max, o));
      hi_min = min(hi_min, __shfl_xor(hi_min, o));
      lo_min = min(lo_min, __shfl_xor(lo_min, o));
      hi_max = max(hi_max, __shfl_xor(hi_max, o));
    }
    wave_lo = __builtin_amdgcn_readfirstlane(lo_max);
    wave_hi = __builtin_amdgcn_readfirstlane(hi_min);
    wave_lo_min = __builtin_amdgcn_readfirstlane(lo_min);
    wave_hi_max = __builtin_amdgcn_readfirstlane(hi_max);
  }
  // a wave whose row blocks all lie past the sequence's rows only helps with the loads
  const bool wave_active = (R0 + wave * RB * 16) < rows_total;

  // ---- staging ---------------------------------------------------------------------------------------
  const int32_t* bt = p.block_tables + (int64_t)i * p.M;
  const char* k_pages = (const char*)p.k_pages;
  const char* v_pages = (const char*)p.v_pages;
  const int pg = p.page_size;
  int st_tok[NLD], st_cc[NLD];
  bool st_v[NLD], st_ok[NLD];
  int64_t st_off[NLD];
#pragma unroll
  for (int u = 0; u < NLD; ++u) {
    const int idx = u * THREADS + tid;
    st_ok[u] = FULL || idx < TT * LPTG;
    st_tok[u] = st_ok[u] ? idx / LPTG : 0;
    const int c = idx % LPTG;
    st_v[u] = c >= LPTG / 2;
    st_cc[u] = st_v[u] ? c - LPTG / 2 : c;
    st_off[u] = (int64_t)st_tok[u] * p.token_stride + (int64_t)h * p.head_stride + st_cc[u] * 16;
  }
  u32x4 stage[NLD];
  auto page_of = [&](int tok) -> int {
    int pgid = bt[tok / pg];
    pgid = __builtin_amdgcn_readfirstlane(pgid);
    return min(max(pgid, 0), p.P - 1);
  };
  auto issue = [&](int tb, int page) {
    const int64_t base = (int64_t)page * p.page_stride + (int64_t)(tb % pg) * p.token_stride;
#pragma unroll
    for (int u = 0; u < NLD; ++u)
      if (FULL || st_ok[u]) stage[u] = *(const u32x4*)((st_v[u] ? v_pages : k_pages) + base + st_off[u]);
  };
  auto commit = [&](int tb, unsigned char* buf) {  // registers -> LDS tile (zeroing keys nobody may see)
    const bool edge = (tb + TT > sp.ctx) || (tb < vis_lo);
#pragma unroll
    for (int u = 0; u < NLD; ++u) {
      if (!FULL && !st_ok[u]) continue;
      u32x4 v = stage[u];
      if (edge) {
        const int tok = tb + st_tok[u];
        if (tok >= sp.ctx || tok < vis_lo) v = (u32x4){0u, 0u, 0u, 0u};
      }
      unsigned char* row = buf + (st_v[u] ? TT * RKL : 0) + st_tok[u] * RKL;
      const int key = swz_key<RKL>(st_tok[u]);
      if constexpr (EB == 2) {
        *(u32x4*)(row + ((st_cc[u] ^ key) << 4)) = v;
      } else {  // 16 codes -> 16 bf16 = two LDS chunks
        *(u32x4*)(row + (((2 * st_cc[u]) ^ key) << 4)) = codes8_to_bf16x8<KVT>(v[0], v[1]);
        *(u32x4*)(row + (((2 * st_cc[u] + 1) ^ key) << 4)) = codes8_to_bf16x8<KVT>(v[2], v[3]);
      }
    }
  };

  const float cap_out = p.softcap * 1.4426950408889634f;
  const float cap_in = CAP ? p.scale / p.softcap : 0.f;

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

  int page_cur = page_of(kv_lo);
  issue(kv_lo, page_cur);
  commit(kv_lo, lds_all);
  __syncthreads();

  for (int tile = 0; tile < n_tiles; ++tile) {
    const int tb = kv_lo + tile * TT;
    unsigned char* lds_k = lds_all + (tile & 1) * TILE_BYTES;
    unsigned char* lds_v = lds_k + TT * RKL;
    float k_scale = 1.f, v_scale = 1.f;
    if constexpr (EB == 1) {
      if (p.kv_scales) {  // null: unscaled 8-bit pages, the codes are the values
        const float* sc = p.kv_scales + (int64_t)page_cur * p.C + 2 * h;
        k_scale = sc[0];
        v_scale = sc[1];
      }
    }
    const bool more = tile + 1 < n_tiles;
    if (more) {
      page_cur = page_of(tb + TT);
      issue(tb + TT, page_cur);
    }

    if (wave_active && tb < wave_hi_max && tb + TT > wave_lo_min) {
      // ---- S^T = K . Q^T for every row block (K operands shared) --------------------------------
      f32x4 s_acc[RB][NS];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int st = 0; st < NS; ++st) s_acc[rb][st] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int st = 0; st < NS; ++st) {
        const int tk = st * 16 + n;
        const unsigned char* krow = lds_k + tk * RKL;
        const int key = swz_key<RKL>(tk);
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
          const u32x4 a = *(const u32x4*)(krow + (((kk * 4 + g4) ^ key) << 4));
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
            s_acc[rb][st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), qf[rb][kk], s_acc[rb][st], 0, 0, 0);
        }
      }

      // ---- online softmax per row block -------------------------------------------------------------
      const bool inside = (tb >= wave_lo) && (tb + TT <= wave_hi);  // no row of the wave masks any key here
      const float sc_mul = CAP ? cap_out : p.scale_log2 * k_scale;
      const float cap_k = cap_in * k_scale;
      uint32_t pfrag[RB][NS][2];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        float alpha;
        if (inside) alpha = softmax_step<false, CAP, NS>(s_acc[rb], sc_mul, cap_k, tb, g4, row_lo[rb], row_hi[rb], m_run[rb], l_run[rb], pfrag[rb]);
        else alpha = softmax_step<true, CAP, NS>(s_acc[rb], sc_mul, cap_k, tb, g4, row_lo[rb], row_hi[rb], m_run[rb], l_run[rb], pfrag[rb]);
        // accumulators are kept in units of the current page's V scale (see the decode kernel)
        float o_mul = alpha;
        if constexpr (EB == 1) {
          if (v_unit != v_scale) o_mul = alpha * (v_unit * __builtin_amdgcn_rcpf(v_scale));
        }
        if (__any(o_mul != 1.f)) {
#pragma unroll
          for (int rt = 0; rt < DPL; ++rt) o_acc[rb][rt] *= o_mul;
        }
      }
      v_unit = v_scale;

      // ---- O^T += V^T . P^T (V operands shared by the row blocks) -----------------------------------
      // ds_read_b64_tr_b16: inside a 16-lane group, lane l supplies the address of 4 consecutive bf16
      // (key 4g4 + l/4, dims d0 + 4(l%4)..) and receives the transposed column: for dim d0 + (l&15) the
      // values of keys 4g4..4g4+3, which is the A operand of the product with k = keys.
      const int tr_key = 4 * g4 + (n >> 2);          // key (within a 16-key sub-tile) this lane addresses
      const int tr_byte = (n & 3) * 8;               // byte offset of its 4 dims inside the 32-byte row-tile span
#pragma unroll
      for (int rt = 0; rt < DPL; ++rt) {
        u32x2 a_lo, a_hi;
        {
          const int tk = tr_key;
          const int off = rt * 32 + tr_byte;
          const unsigned char* ptr = lds_v + tk * RKL + (((off >> 4) ^ swz_key<RKL>(tk)) << 4) + (off & 15);
          a_lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)ptr));
        }
        if constexpr (NS == 2) {
          const int tk = 16 + tr_key;
          const int off = rt * 32 + tr_byte;
          const unsigned char* ptr = lds_v + tk * RKL + (((off >> 4) ^ swz_key<RKL>(tk)) << 4) + (off & 15);
          a_hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)ptr));
          const u32x4 a4 = {a_lo[0], a_lo[1], a_hi[0], a_hi[1]};
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            const u32x4 b4 = {pfrag[rb][0][0], pfrag[rb][0][1], pfrag[rb][1][0], pfrag[rb][1][1]};
            o_acc[rb][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a4), __builtin_bit_cast(bf16x8, b4),
                                                                    o_acc[rb][rt], 0, 0, 0);
          }
        } else {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            const u32x2 b2 = {pfrag[rb][0][0], pfrag[rb][0][1]};
            o_acc[rb][rt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a_lo), __builtin_bit_cast(s16x4, b2),
                                                                      o_acc[rb][rt], 0, 0, 0);
          }
        }
      }
    }

    if (more) commit(tb + TT, lds_all + ((tile + 1) & 1) * TILE_BYTES);
    __syncthreads();
  }

  // ---- epilogue -----------------------------------------------------------------------------------------
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float l_tot = l_run[rb] + __shfl_xor(l_run[rb], 16);
    l_tot += __shfl_xor(l_tot, 32);
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

template <int D, int KVT, int TT, int NW, int RB>
static int launch_one(hipStream_t stream, const AttnParams& p) {
  constexpr int ROWS = NW * RB * 16;
  const int64_t slots = ((int64_t)p.T * p.group) / ROWS + p.S;  // upper bound on row tiles of the batch
  const int64_t blocks = slots * p.Hkv * p.pre_max_chunks;
  if (blocks > 0x7fffffff) return (int)hipErrorInvalidValue;
  if (p.softcap > 0.f)
    hipLaunchKernelGGL((attn_prefill_kernel<D, KVT, TT, NW, RB, true>), dim3((unsigned)blocks), dim3(64 * NW), 0, stream, p);
  else
    hipLaunchKernelGGL((attn_prefill_kernel<D, KVT, TT, NW, RB, false>), dim3((unsigned)blocks), dim3(64 * NW), 0, stream, p);
  return (int)hipGetLastError();
}

template <int KVT>
static int launch_kvt(hipStream_t stream, const AttnParams& p) {
  const bool tt32 = (p.page_size % 32 == 0);
  switch (p.D) {
    case 64: return tt32 ? launch_one<64, KVT, 32, 4, 2>(stream, p) : launch_one<64, KVT, 16, 4, 2>(stream, p);
    case 128: return tt32 ? launch_one<128, KVT, 32, 4, 2>(stream, p) : launch_one<128, KVT, 16, 4, 2>(stream, p);
    case 256: return tt32 ? launch_one<256, KVT, 32, 8, 1>(stream, p) : launch_one<256, KVT, 16, 8, 1>(stream, p);
    default: return (int)hipErrorInvalidValue;
  }
}

bool prefill_supported(const AttnParams& p) { return decode_supported(p); }

int launch_attn_prefill(hipStream_t stream, const AttnParams& p) {
  if (p.pre_x32) return launch_attn_prefill_x32(stream, p);  // chosen by the caller together with the row-tile height
  if (p.prefill_dma && prefill_dma_supported(p)) return launch_attn_prefill_dma(stream, p);
  if (p.prefill_dma && prefill_dma8_supported(p)) return launch_attn_prefill_dma8(stream, p);
  switch (p.kv_dtype) {
    case RPA_BF16: return launch_kvt<RPA_BF16>(stream, p);
    case RPA_FP8_E4M3: return launch_kvt<RPA_FP8_E4M3>(stream, p);
    case RPA_INT8: return launch_kvt<RPA_INT8>(stream, p);
    default: return (int)hipErrorInvalidValue;
  }
}

}  // namespace rpa
