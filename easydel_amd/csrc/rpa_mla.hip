// Multi-latent attention (MLA) over latent ragged pages: page write, MFMA kernel, fp32 kernel, merge.
//
// The cache holds one row per token, shared by every query head: [latent (lkv) | rope key (rope)], each part padded
// to a multiple of 128 elements.  For query row (token t, head h) at position pos the operation computes
//     s_j = scale * (q_nope[t][h] . latent_j + q_pe[t][h] . rope_j)      over the visible keys j
//     out[t][h] = sum_j softmax(s)_j * latent_j                          (lkv values; the caller applies the value
//                                                                         half of the up-projection afterwards)
// i.e. attention with one KV head, key width lkv + rope, value width lkv, and values that are a prefix of the keys.
//
// MFMA kernel (bf16, lkv = 512, rope = 64): a workgroup of eight waves owns 128 consecutive rows (row = (token,
// head), token-major) of one sequence and one chunk of its keys; every wave keeps one 16-row block in registers
// (Q as MFMA B operands: 18 k-steps of 32 = 72 registers; O^T accumulators: 32 tiles of 16 dims = 128 registers), two
// waves per SIMD.  Tiles of 32 keys x 576 elements go global -> LDS through the load unit (global_load_lds_dwordx4,
// no staging registers) into a ring of three slots, two tiles ahead of their use; the one tile serves all eight waves
// and both products:
//     S^T[key][row]  = K[key][:] . Q[row][:]            A = 16 keys x 32 dims read row-wise
//     O^T[dim][row] += V^T[dim][key] . P^T[key][row]    A = 16 dims x 32 keys read with the transposing LDS load
// Every matrix instruction takes one operand from LDS (1 KiB), which bounds the kernel: a compute unit's LDS delivers
// 128 B a clock against the 256 B a clock its four SIMDs could consume at full rate.  Two row blocks per wave would
// halve that, but their 256 accumulators and 144 query registers leave the compiler no working set in 512 registers
// (it spilled the queries); that variant needs hand-placed registers and is not built.
#include "rpa_mfma.h"
#include "rpa_mla.h"

namespace rpa {

namespace {

// ---- page write ------------------------------------------------------------------------------------------------
// One wavefront per query token: its latent row and rope key into the page slot of its position, padding zeroed.
template <typename E>
__device__ __forceinline__ void mla_scatter_token(const MlaParams& p, int t) {
  const int lane = threadIdx.x & 63;
  if (t >= p.T) return;
  const int n_live = mla_live_rows(p);
  if (n_live <= 0 || t < p.qsl[0] || t >= p.qsl[n_live]) return;
  const int i = find_seq_wave(p.qsl, n_live, t);
  const int q0 = p.qsl[i], q_len = p.qsl[i + 1] - q0;
  const int pos = p.context_lens[i] - q_len + (t - q0);
  if (pos < 0) return;
  const int page_idx = pos / p.page_size;
  if (page_idx >= p.M) return;
  const int page = p.block_tables[(int64_t)i * p.M + page_idx];
  if (page < 0 || page >= p.P) return;
  E* row = (E*)((char*)p.pages + (int64_t)page * p.page_stride + (int64_t)(pos % p.page_size) * p.token_stride);
  const E* kv = (const E*)p.new_kv + (int64_t)t * p.lkv;
  const E* pe = (const E*)p.new_pe + (int64_t)t * p.rope;
  for (int e = lane; e < p.row_elems; e += 64) {
    E v = 0;
    if (e < p.lkv) v = kv[e];
    else if (e >= p.rope_off && e < p.rope_off + p.rope) v = pe[e - p.rope_off];
    row[e] = v;
  }
}

template <typename E>
__global__ __launch_bounds__(256) void mla_scatter_kernel(MlaParams p) {
  mla_scatter_token<E>(p, blockIdx.x * 4 + (threadIdx.x >> 6));
}

// ---- fp32 kernel: one wavefront per (query token, head) ----------------------------------------------------------
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

constexpr int kGenMaxLkv = 512, kGenMaxRope = 256;

template <int QT, int KVT>
__global__ __launch_bounds__(64) void mla_generic_kernel(MlaParams p) {
  __shared__ float q_s[kGenMaxLkv + kGenMaxRope];
  const int t = blockIdx.x, hq = blockIdx.y, lane = threadIdx.x;
  const int n_live = mla_live_rows(p);
  if (n_live <= 0 || t < p.qsl[0] || t >= p.qsl[n_live]) return;
  const int i = find_seq_wave(p.qsl, n_live, t);
  const MlaSeq sp = mla_seq(p, i);
  if (!sp.live) return;
  const int lkv = p.lkv, rope = p.rope;
  const int pos = sp.ctx - sp.q_len + (t - sp.q0);
  const int k_hi = min(pos + 1, sp.ctx);
  const int k_lo = (p.window > 0 && pos - p.window + 1 > 0) ? pos - p.window + 1 : 0;

  for (int d = lane; d < lkv; d += 64) q_s[d] = load_elem<QT>(p.q_nope, ((int64_t)t * p.Hq + hq) * lkv + d);
  for (int d = lane; d < rope; d += 64) q_s[lkv + d] = load_elem<QT>(p.q_pe, ((int64_t)t * p.Hq + hq) * rope + d);
  __syncthreads();

  const char* pages = (const char*)p.pages;
  const int32_t* bt = p.block_tables + (int64_t)i * p.M;
  float m = -INFINITY, l = 0.f;
  float acc[kGenMaxLkv / 64];
#pragma unroll
  for (int k = 0; k < kGenMaxLkv / 64; ++k) acc[k] = 0.f;

  for (int base = k_lo; base < k_hi; base += 64) {
    const int j = base + lane;
    float s = -INFINITY;
    int64_t row = 0;
    if (j < k_hi) {
      const int page = min(max(bt[j / p.page_size], 0), p.P - 1);
      row = (int64_t)page * p.page_stride + (int64_t)(j % p.page_size) * p.token_stride;
      const void* kp = pages + row;
      // eight partial sums: a single chain of 576 float additions drifts past the 1e-5 the fp32 path is held to
      float part[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      int d = 0;
      for (; d + 8 <= lkv; d += 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) part[u] = fmaf(q_s[d + u], load_elem<KVT>(kp, d + u), part[u]);
      }
      for (; d < lkv; ++d) part[d & 7] = fmaf(q_s[d], load_elem<KVT>(kp, d), part[d & 7]);
      for (d = 0; d + 8 <= rope; d += 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) part[u] = fmaf(q_s[lkv + d + u], load_elem<KVT>(kp, p.rope_off + d + u), part[u]);
      }
      for (; d < rope; ++d) part[d & 7] = fmaf(q_s[lkv + d], load_elem<KVT>(kp, p.rope_off + d), part[d & 7]);
      const float dot = ((part[0] + part[1]) + (part[2] + part[3])) + ((part[4] + part[5]) + (part[6] + part[7]));
      s = dot * p.scale;
      if (p.softcap > 0.f) s = p.softcap * tanhf(s / p.softcap);
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: lane 0 of every block holds a visible key
    const float pj = (j < k_hi) ? __expf(s - m_new) : 0.f;
    const float alpha = __expf(m - m_new);
    l = l * alpha + wave_sum(pj);
    m = m_new;
#pragma unroll
    for (int k = 0; k < kGenMaxLkv / 64; ++k) acc[k] *= alpha;
    const int n_keys = min(64, k_hi - base);
    for (int jj = 0; jj < n_keys; ++jj) {
      const float w = __shfl(pj, jj);
      const char* vrow = pages + (int64_t)__shfl((unsigned long long)row, jj);
#pragma unroll
      for (int k = 0; k < kGenMaxLkv / 64; ++k) {
        const int d = lane + 64 * k;
        if (d < lkv) acc[k] = fmaf(w, load_elem<KVT>(vrow, d), acc[k]);
      }
    }
  }
  if (p.sinks && l > 0.f) l += expf(p.sinks[hq] - m);
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int k = 0; k < kGenMaxLkv / 64; ++k) {
    const int d = lane + 64 * k;
    if (d < lkv) {
      const int64_t o = ((int64_t)t * p.Hq + hq) * lkv + d;
      const float r = acc[k] * inv;
      store_out<QT>(p.out, o, r);
    }
  }
}

// The row tile at slot `slot` of the matrix-core kernel's grid: its sequence and the keys it must visit (0: no tile).
// `qsl` is query_start_loc, or a copy of its first n_live + 1 entries that is quicker to search.
__device__ __forceinline__ int mla_slot_span(const MlaParams& p, int slot, const int32_t* qsl, int* seq) {
  *seq = 0;
  const int n_live = mla_live_rows(p);
  if (n_live <= 0) return 0;
  int lo_i = 0, hi_i = n_live;  // the last sequence starting at or before `slot`
  while (hi_i - lo_i > 1) {
    const int mid = (lo_i + hi_i) >> 1;
    if ((int)(((int64_t)qsl[mid] * p.Hq) / kMlaRows) + mid <= slot) lo_i = mid; else hi_i = mid;
  }
  const MlaSeq sp = mla_seq(p, lo_i);
  const int tile_in_seq = slot - ((int)(((int64_t)sp.q0 * p.Hq) / kMlaRows) + lo_i);
  if (!sp.live || tile_in_seq < 0 || tile_in_seq * kMlaRows >= sp.q_len * p.Hq) return 0;
  const MlaTile mt = mla_tile(p, sp, tile_in_seq * kMlaRows, 0);
  *seq = lo_i;
  return max(mt.kv_hi - mt.kv_lo, 0);
}
// What the plan holds for such a tile: (sequence, key chunks | keys / 64 of a chunk << 8), chunks = 0 where there is none.
__device__ __forceinline__ int2 mla_plan_entry(const MlaParams& p, int seq, int span, int L) {
  int2 unit = {0, 0};
  if (span > 0) {
    int chunk, n_chunks;
    mla_cut(p, span, L, &chunk, &n_chunks);
    unit.x = seq;
    unit.y = n_chunks | ((min(chunk, span) >> 6) << 8);
  }
  return unit;
}

// ---- plan: which sequence and how many key chunks each row-tile slot of the MFMA kernel's grid holds -------------
// Sequence i starts at slot floor(qsl[i] * Hq / 128) + i (its row tiles follow), so the slots of a batch are found
// without a scan; slots between sequences, past the live ones, or of rows before position 0 hold no tile.
// In the fused call the blocks behind the plan's write the new rows into the pages (four tokens a block): one
// launch less before the attention kernel, which waits for both anyway.
__global__ __launch_bounds__(256) void mla_plan_kernel(MlaParams p, int n_slots, int plan_blocks) {
  if ((int)blockIdx.x >= plan_blocks) {
    const int t = ((int)blockIdx.x - plan_blocks) * 4 + (threadIdx.x >> 6);
    if (p.kv_dtype == RPA_F32) mla_scatter_token<uint32_t>(p, t);
    else mla_scatter_token<uint16_t>(p, t);
    return;
  }
  const int slot = blockIdx.x * 256 + threadIdx.x;
  if (slot >= n_slots) return;
  int seq;
  const int span = mla_slot_span(p, slot, p.qsl, &seq);
  p.plan[slot] = mla_plan_entry(p, seq, span, 0);
}

// Small batches (up to kMlaSortSlots slots): plan and unit list in one launch of one block -- thread t looks up slots
// 4t .. 4t+3, keeps them in registers, and the list is built longest first in eight classes of chunk length with one
// scan over eight counters instead of one scan per class.  Blocks behind the first write the new rows, as above.
constexpr int kMlaSortSlots = 4096;
constexpr int kMlaLenClasses = 8;
constexpr int kMlaRankSlots = 512;  // lists up to this many slots are sorted exactly
__global__ __launch_bounds__(1024) void mla_plan_sorted_kernel(MlaParams p, int n_slots) {
  constexpr int PER = kMlaSortSlots / 1024, NC = kMlaLenClasses;
  if (blockIdx.x > 0) {
    const int t = ((int)blockIdx.x - 1) * 16 + (threadIdx.x >> 6);
    if (p.kv_dtype == RPA_F32) mla_scatter_token<uint32_t>(p, t);
    else mla_scatter_token<uint16_t>(p, t);
    return;
  }
  __shared__ int wave_max_s[16];
  __shared__ int wave_cnt[16][NC];
  __shared__ int32_t qsl_s[kMlaSortSlots + 1];  // the sequence starts, searched four times per thread: from LDS, not through
                                                // a dozen dependent global loads (n_live <= S <= n_slots <= kMlaSortSlots)
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  for (int k = tid; k <= min(mla_live_rows(p), kMlaSortSlots); k += 1024) qsl_s[k] = p.qsl[k];
  __syncthreads();
  // A batch of few row tiles (a quarter of the CUs or fewer: a small decode batch) is cut by length, not by count: every
  // tile into chunks of about L keys, L such that the whole batch makes at most one unit per CU -- sum(ceil(span / L))
  // <= W / L + R <= CUs for L = W / (CUs - R), W the keys of all R tiles.  A single wave of near-equal units over the chip then takes
  // what one chunk takes, where even cuts of every tile leave units as different as the sequences are long.
  __shared__ long long wave_w[16];
  __shared__ int wave_r[16];
  int seq_k[PER], span_k[PER];
  long long w_keys = 0;
  int tiles = 0;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int slot = tid * PER + k;
    seq_k[k] = 0;
    span_k[k] = slot < n_slots ? mla_slot_span(p, slot, qsl_s, &seq_k[k]) : 0;
    w_keys += span_k[k];
    tiles += span_k[k] > 0;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    w_keys += __shfl_xor(w_keys, o);
    tiles += __shfl_xor(tiles, o);
  }
  if (lane == 0) {
    wave_w[wv] = w_keys;
    wave_r[wv] = tiles;
  }
  __syncthreads();
  w_keys = 0;
  tiles = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    w_keys += wave_w[w];
    tiles += wave_r[w];
  }
  int L = 0;
  if (p.auto_chunk && p.max_chunks > 1 && tiles > 0 && 4 * tiles <= p.cus) {
    const long long even = (w_keys + (p.cus - tiles) - 1) / (p.cus - tiles);
    L = (int)min(max((even + 63) & ~63ll, 128ll), (long long)1 << 30);
  }
  int y[PER];
  int max_len = 0;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int slot = tid * PER + k;
    const int2 unit = mla_plan_entry(p, seq_k[k], span_k[k], L);
    if (slot < n_slots) p.plan[slot] = unit;
    y[k] = unit.y;
    if (y[k] & 0xff) max_len = max(max_len, y[k] >> 8);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) max_len = max(max_len, __shfl_xor(max_len, o));
  if (lane == 0) wave_max_s[wv] = max_len;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < 16; ++w) max_len = max(max_len, wave_max_s[w]);
  // A list of up to kMlaRankSlots slots (the decode batches: a unit is a large share of a CU's work there, and the order
  // inside a length class, which is slot order, costs 5 % of such a call) is sorted exactly: every slot's (chunk length,
  // slot, chunks) goes to LDS as one key, thread t counts the units of all slots that come before slot t -- longer
  // chunks, or as long and a lower slot -- and writes slot t's units there.
  if (n_slots <= kMlaRankSlots) {
    __shared__ uint32_t key_s[kMlaRankSlots];
    __shared__ int seq_s[kMlaRankSlots];
    const unsigned len_div = max_len < 32768 ? 1u : (unsigned)(max_len / 32767 + 1);  // chunk lengths / 64 into 15 bits
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int slot = tid * PER + k;
      if (slot < n_slots) {
        key_s[slot] = (y[k] & 0xff) ? ((((unsigned)(y[k] >> 8) / len_div) << 17) | ((unsigned)(kMlaRankSlots - 1 - slot) << 8) | (unsigned)(y[k] & 0xff)) : 0u;
        seq_s[slot] = seq_k[k];
      }
    }
    __syncthreads();
    if (tid < 64) {  // the first wave adds up the units while the others place them
      int t = 0;
      for (int s2 = lane; s2 < n_slots; s2 += 64) t += (int)(key_s[s2] & 0xff);
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) t += __shfl_xor(t, o);
      if (lane == 0) {
        p.n_units[0] = t;
        p.n_units[1] = 1;
        p.n_units[2] = L;
      }
    }
    // The count is shared by as many threads per slot as the block has to spare (2 at 512 slots, 16 at 64 and fewer):
    // thread t serves slot t % s_pad and the (t / s_pad)-th share of the keys; a wave's lanes walk the same keys.
    __shared__ int part_s[1024];
    int s_pad = 64;
    while (s_pad < n_slots) s_pad <<= 1;
    const int ways = 1024 / s_pad, share = (n_slots + ways - 1) / ways;
    const int my_slot = tid & (s_pad - 1), my_part = tid / s_pad;
    const uint32_t mine = my_slot < n_slots ? key_s[my_slot] : 0u;
    {
      int at = 0;
      const int hi = min(n_slots, (my_part + 1) * share);
      if (mine & 0xff) {
#pragma unroll 4
        for (int s2 = my_part * share; s2 < hi; ++s2) {
          const uint32_t o = key_s[s2];
          at += (o > mine) ? (int)(o & 0xff) : 0;  // (length, -slot) differs between slots, so the low bits never decide
        }
      }
      part_s[tid] = at;
    }
    __syncthreads();
    if (my_part == 0 && (mine & 0xff)) {
      int at = 0;
      for (int w = 0; w < ways; ++w) at += part_s[w * s_pad + my_slot];
      const int v = (int)(mine & 0xff);
      for (int ch = 0; ch < v; ++ch) p.units[at + ch] = make_int2(my_slot, ch | (seq_s[my_slot] << 5));
    }
    return;
  }
  // units of this thread's slots per class, then an inclusive scan over the threads for all classes at once
  int cls[PER], cnt[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) cnt[c] = 0;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    cls[k] = min(NC - 1, ((y[k] >> 8) * NC) / (max_len + 1));
#pragma unroll
    for (int c = 0; c < NC; ++c) cnt[c] += (cls[k] == c) ? (y[k] & 0xff) : 0;
  }
  int incl[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    incl[c] = cnt[c];
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl[c], o);
      if (lane >= o) incl[c] += up;
    }
    if (lane == 63) wave_cnt[wv][c] = incl[c];
  }
  __syncthreads();
  // first list position of each class's units of this thread: the longer classes in full, then the class's units of
  // the waves and lanes before
  int first[NC];
  int longer = 0, total = 0;
#pragma unroll
  for (int c = NC - 1; c >= 0; --c) {
    int before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int v = wave_cnt[w][c];
      before += (w < wv) ? v : 0;
      all += v;
    }
    first[c] = longer + before + incl[c] - cnt[c];
    longer += all;
  }
  total = longer;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int v = y[k] & 0xff;
    if (v == 0) continue;
    int at = 0;
#pragma unroll
    for (int c = 0; c < NC; ++c)
      if (cls[k] == c) {
        at = first[c];
        first[c] += v;
      }
    for (int ch = 0; ch < v; ++ch) p.units[at + ch] = make_int2(tid * PER + k, ch | (seq_k[k] << 5));
  }
  if (tid == 0) {
    p.n_units[0] = total;
    p.n_units[1] = 1;
    p.n_units[2] = L;
  }
}



// The units (row tile, key chunk) of the batch in one dense list.  The MFMA kernel's grid is sized from the static
// bounds and most of its slots are empty; left in place, the empty ones form a regular pattern (a batch of single tokens
// with 128 heads fills every other slot) that the hardware's round-robin placement of consecutive blocks turns into
// idle shader engines: measured, each engine was busy 43 % of such a kernel's duration.
// A batch of up to kMlaSortSlots slots (decode and small mixed batches, where a unit is a sizeable share of a CU's work
// and the lengths differ many-fold) is listed longest first by mla_plan_sorted_kernel: workgroups are handed out in
// list order, so the long units start first and the short ones fill in behind them.  Larger batches are listed here,
// in slot order: one block, a scan over the plan's chunk counts, 1024 slots a pass.  n_units[1] says which.
__global__ __launch_bounds__(1024) void mla_compact_kernel(MlaParams p, int n_slots) {
  __shared__ int wave_tot[16];
  __shared__ int running_s;
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  if (tid == 0) running_s = 0;
  __syncthreads();
  for (int base = 0; base < n_slots; base += 1024) {
    const int slot = base + tid;
    const int2 entry = slot < n_slots ? p.plan[slot] : make_int2(0, 0);
    const int v = entry.y & 0xff;
    int incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_up(incl, o);
      if (lane >= o) incl += up;
    }
    if (lane == 63) wave_tot[wv] = incl;
    __syncthreads();
    int before = running_s;
    for (int w = 0; w < wv; ++w) before += wave_tot[w];
    const int first = before + incl - v;
    for (int c = 0; c < v; ++c) p.units[first + c] = make_int2(slot, c | (entry.x << 5));
    __syncthreads();
    if (tid == 1023) running_s = before + incl;
    __syncthreads();
  }
  if (tid == 0) {
    p.n_units[0] = running_s;
    p.n_units[1] = 0;
    p.n_units[2] = 0;
  }
}

// ---- MFMA kernel ----------------------------------------------------------------------------------------------------
// One LDS DMA of 1 KiB: every lane fetches 16 bytes from base + voff; lane L's bytes land at LDS byte address
// lds_addr + 16 L.
__device__ __forceinline__ void mla_dma16(uint32_t lds_addr, uint32_t voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
}
// ... with the non-temporal hint: for rows no other workgroup will ask for (see `once` in the kernel)
__device__ __forceinline__ void mla_dma16_nt(uint32_t lds_addr, uint32_t voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
}
template <int N>
__device__ __forceinline__ void mla_wait_loads_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// XOR key (on the low three bits of the 16-byte chunk index) of LDS row r.  Rows are 1152 bytes, so rows of equal
// parity start in the same bank group and rows of different parity half the banks apart.  Chosen by measurement
// (SQ_LDS_BANK_CONFLICT over the kernel, 32-key tiles read row-wise with ds_read_b128 and transposed with
// ds_read_b64_tr_b16): this key and `r & 7` count no conflict cycle at all; no key: three conflict cycles per
// useful one (8.4 ms instead of 5.7 ms on a 4 096-token prefill); keys that map two rows of equal parity among
// rows 0-7 to the same chunk pair, or that ignore the parity: 0.5 to 1 conflict cycle per useful one.
__device__ __forceinline__ int mla_key(int r) { return ((r >> 1) & 3) << 1; }

constexpr int kMlaWaves = 8;  // waves of an MFMA-kernel workgroup
constexpr int kXcds = 8;      // accelerator dies a grid's blocks are dealt to in turn

template <bool CAP>
__global__ __launch_bounds__(64 * kMlaWaves, 2) void mla_attn_kernel(MlaParams p) {
  constexpr int TT = 32, NW = kMlaWaves, RB = 1;
  constexpr int LKV = 512, ROPE = 64, DK = LKV + ROPE;
  constexpr int RKL = DK * 2;            // bytes of a key row in LDS
  constexpr int CPR = RKL / 16;          // 16-byte chunks per row
  constexpr int TILE = TT * RKL;         // bytes of a tile
  constexpr int NINS = TILE / 1024;      // DMA instructions per tile, dealt round-robin to the waves
  constexpr int NDMA = (NINS + NW - 1) / NW;  // most per wave
  static_assert(NINS % NW == NW / 2, "the first half of the waves issue NDMA instructions a tile, the others one fewer");
  constexpr int NSLOT = 3;               // tiles of the LDS ring: NSLOT - 1 are in flight ahead of the one in use
  constexpr int NS = TT / 16;            // 16-key sub-tiles per tile
  constexpr int DPL = LKV / 16;          // 16-dim row tiles of O^T
  constexpr int NKK = DK / 32;           // k-steps of the score product
  constexpr int NKN = LKV / 32;          // of which over the latent part
  constexpr int NKO = NS * NKK;          // K operands of a tile
  constexpr int KPD = 4, PD = 4;         // operand reads in flight ahead of the score / PV matrix instructions
  constexpr float kMaxSlack = 8.f;       // how far a score may exceed the softmax reference before it is raised
  static_assert(NW * RB * 16 == kMlaRows, "merge kernel assumes this row-tile height");

  constexpr int OFFW = NDMA * 256;       // bytes of a wave's table of load offsets (one dword per lane and instruction)
  __shared__ __attribute__((aligned(1024))) unsigned char lds_all[NSLOT * TILE + NW * OFFW];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, g4 = lane >> 4;
  const int Hq = p.Hq;

  // ---- block -> (sequence, row tile, key chunk) -------------------------------------------------------------
  // The grid is sized from the static bounds, so most of its blocks have nothing to do, and a workgroup holds a
  // whole compute unit: the plan kernel has looked every slot up beforehand, and a block learns with one load
  // whether it has work.
  // Block -> unit of the dense list.  Consecutive blocks go to the eight XCDs in turn.  A list in slot order (large
  // batches) is dealt in contiguous eighths, unit = (block % 8) * n8 + block / 8, so that the row tiles of a long
  // prompt, which read the same keys, share one XCD's L2; a list sorted longest first is dealt block by block.
  // The unit of a sorted list is asked for together with the list's length (the list has an entry for every block of
  // the grid, so the load is in bounds whatever it returns), and it names its sequence: two dependent loads fewer
  // before the first tile can be requested.
  int2 sc = p.units[blockIdx.x];
  const int total = p.n_units[0];
  const int n8 = (total + kXcds - 1) / kXcds;
  const bool sorted = p.n_units[1] != 0;
  const int u = sorted ? (int)blockIdx.x : (int)((blockIdx.x % kXcds) * n8 + blockIdx.x / kXcds);
  if ((!sorted && (int)(blockIdx.x / kXcds) >= n8) || u >= total) return;
  if (!sorted) sc = p.units[u];
  const int slot = sc.x, chunk = sc.y & 31, i = sc.y >> 5;
  const MlaSeq sp = mla_seq(p, i);
  const int tile_in_seq = slot - ((int)(((int64_t)sp.q0 * Hq) / kMlaRows) + i);
  const int rows_total = sp.q_len * Hq;
  const int R0 = tile_in_seq * kMlaRows;

  const MlaTile mt = mla_tile(p, sp, R0, p.n_units[2]);
  const int base_pos = sp.ctx - sp.q_len;
  const int vis_lo = mt.vis_lo;
  // the first tile must hold vis_lo, so that rows of it that nobody may see can borrow a visible row's address
  const int kv_lo = max(mt.kv_lo + chunk * mt.chunk, vis_lo & ~(TT - 1));
  const int kv_hi = min(mt.kv_hi, mt.kv_lo + (chunk + 1) * mt.chunk);
  const int n_tiles = (kv_hi - kv_lo + TT - 1) / TT;
  const bool single = mt.n_chunks == 1;
  // A unit of few keys carries its probabilities as two 16-bit numbers each (the rounded value and what the rounding
  // took off) through two PV products: with few keys whose values cancel, the 2^-9 relative error of a single bf16
  // weight reaches the output almost whole (seen: 1.4e-2 on an output of 3.55 with 32 visible keys); with many it
  // averages out.  Two tiles' worth of keys cost nothing measurable.
  const bool precise = kv_hi - kv_lo <= 2 * TT;

  // ---- tile loads --------------------------------------------------------------------------------------------
  // The tile is 36 KiB of LDS in row order (72 chunks a row); DMA instruction u = wave + 4 j fills its bytes
  // [1024 u, 1024 u + 1024): lane L holds chunk c = 64 u + L = (row c / 72, LDS chunk c % 72) and fetches the global
  // chunk that the swizzle maps there.  The block table is read through the constant address space: it does not change
  // while the kernel runs, and only so may the compiler keep these loads scalar after the assembly statements.
  typedef const __attribute__((address_space(4))) int32_t* ConstI32;
  ConstI32 bt = (ConstI32)(uintptr_t)(p.block_tables + (int64_t)i * p.M);
  const char* pages = (const char*)p.pages;
  const int pg = p.page_size;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds_all;
  // (row, global chunk) of DMA instruction j for this lane.  The offsets are the same for every tile whose rows are all
  // visible: they wait in LDS, one dword per lane and instruction, and an issue reads them back (five reads against
  // sixty integer instructions; registers to hold them the loop has none, and the lane number passes through an empty
  // assembly statement at every issue, or the compiler would hoist reads and arithmetic out of the loop and spill them).
  int dma_lane = lane;
  auto dma_row = [&](int j) -> int { return (64 * (wave + NW * j) + dma_lane) / CPR; };
  auto dma_chunk = [&](int j, int r) -> int { return ((64 * (wave + NW * j) + dma_lane) - r * CPR) ^ mla_key(r); };
  const bool dma_full = wave < NINS % NW;  // this wave issues NDMA instructions per tile (else NDMA - 1)
  int cur_idx = kv_lo / pg;
  int cur_off = kv_lo - cur_idx * pg;
  int cur_tb = kv_lo;
  int cur_slot = 0;
  auto load_page = [&](int idx) -> int { return __builtin_amdgcn_readfirstlane(bt[min(idx, p.M - 1)]); };
  int cur_page_raw = load_page(cur_idx);
  // A sequence with a single row tile (a decode batch: one token's heads) has its latent rows read by this workgroup
  // alone: they are streamed with the non-temporal hint, which reads HBM measurably faster.  The row tiles of a prompt
  // share their rows through the L2 and load them the ordinary way.
  const bool once = rows_total <= kMlaRows;
  {
    uint32_t* off_w = (uint32_t*)(lds_all + NSLOT * TILE + wave * OFFW) + lane;
#pragma unroll
    for (int j = 0; j < NDMA; ++j) {
      const int r = dma_row(j);
      off_w[j * 64] = (uint32_t)r * (uint32_t)p.token_stride + (uint32_t)(dma_chunk(j, r) << 4);
    }
  }
  auto issue = [&]() __attribute__((always_inline)) {
    const int cur_page = min(max(cur_page_raw, 0), p.P - 1);
    const char* base = pages + (int64_t)cur_page * p.page_stride + (int64_t)cur_off * p.token_stride;
    const bool edge = (cur_tb + TT > sp.ctx) || (cur_tb < vis_lo);
    const uint32_t dst = lds_base + (uint32_t)cur_slot * TILE + (uint32_t)wave * 1024u;
    const uint32_t ts = (uint32_t)p.token_stride;
    dma_lane = lane;
    asm volatile("" : "+v"(dma_lane));
    if (!edge) {
      const uint32_t* off_r = (const uint32_t*)(lds_all + NSLOT * TILE + wave * OFFW) + dma_lane;
      uint32_t voff[NDMA];
#pragma unroll
      for (int j = 0; j < NDMA; ++j) voff[j] = off_r[j * 64];
#pragma unroll
      for (int j = 0; j < NDMA; ++j) {
        if (j == NDMA - 1 && !dma_full) break;
        if (once) mla_dma16_nt(dst + j * NW * 1024, voff[j], base);
        else mla_dma16(dst + j * NW * 1024, voff[j], base);
      }
    } else {
#pragma unroll
      for (int j = 0; j < NDMA; ++j) {  // keys nobody may see: any visible row's bytes
        if (j == NDMA - 1 && !dma_full) break;
        const int r = dma_row(j);
        const int rv = min(max(cur_tb + r, vis_lo), sp.ctx - 1) - cur_tb;
        if (once) mla_dma16_nt(dst + j * NW * 1024, (uint32_t)rv * ts + (uint32_t)(dma_chunk(j, r) << 4), base);
        else mla_dma16(dst + j * NW * 1024, (uint32_t)rv * ts + (uint32_t)(dma_chunk(j, r) << 4), base);
      }
    }
    cur_tb += TT;
    cur_off += TT;
    if (cur_off >= pg) {
      cur_off -= pg;
      ++cur_idx;
    }
    cur_slot = (cur_slot == NSLOT - 1) ? 0 : cur_slot + 1;
    cur_page_raw = load_page(cur_idx);
  };

  const float cap_out = p.softcap * 1.4426950408889634f;
  const float cap_in = CAP ? p.scale / p.softcap : 0.f;
  const float sc_mul = CAP ? cap_out : p.scale_log2;

  float m_run[RB], l_run[RB];
  f32x4 o_acc[RB][DPL];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    m_run[rb] = -INFINITY;
    l_run[rb] = 0.f;
#pragma unroll
    for (int rt = 0; rt < DPL; ++rt) o_acc[rb][rt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  // per-lane LDS offsets of the operand reads inside a tile
  int k_base[NS][2];  // row-wise read of key st*16 + n, k-step parity
#pragma unroll
  for (int st = 0; st < NS; ++st)
#pragma unroll
    for (int par = 0; par < 2; ++par) k_base[st][par] = (st * 16 + n) * RKL + (((4 * par + g4) ^ mla_key(st * 16 + n)) << 4);
  // ds_read_b64_tr_b16: inside a 16-lane group, lane l supplies the address of 4 consecutive bf16 (key 4g4 + l/4,
  // dims d0 + 4(l%4)..) and receives the transposed column: for dim d0 + (l&15) the values of keys 4g4..4g4+3
  const int tr_key = 4 * g4 + (n >> 2);  // key (within a 16-key sub-tile) this lane addresses in a transposing read
  const int tr_byte = (n & 3) * 8;       // byte offset of its 4 dims inside the 32-byte row-tile span
  int v_base[NS][4];  // transposing read of sub-tile st, row tile rt & 3
#pragma unroll
  for (int st = 0; st < NS; ++st)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int tk = st * 16 + tr_key;
      v_base[st][q] = tk * RKL + (((2 * q + (tr_byte >> 4)) ^ mla_key(tk)) << 4) + (tr_byte & 15);
    }

  constexpr int AHEAD = NSLOT - 1;  // tiles issued ahead of the one in use
  static_assert(AHEAD >= 1 && AHEAD <= 3, "the waits below are written out for up to three tiles ahead");
#pragma unroll
  for (int a = 0; a < AHEAD; ++a)
    if (a < n_tiles) issue();

  // ---- per row-block lane state ----------------------------------------------------------------------------
  int row_lo[RB], row_hi[RB];
  bool row_ok[RB];
  int out_tok[RB], out_head[RB];
  bf16x8 qf[RB][NKK];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = R0 + (wave * RB + rb) * 16 + n;
    row_ok[rb] = row < rows_total;
    const int r_tok = row_ok[rb] ? row / Hq : (rows_total - 1) / Hq;  // padded rows shadow the last row
    const int r_head = row_ok[rb] ? row - r_tok * Hq : 0;
    const int pos = base_pos + r_tok;
    row_hi[rb] = min(pos + 1, sp.ctx);
    row_lo[rb] = (p.window > 0) ? max(pos - p.window + 1, 0) : 0;
    out_tok[rb] = sp.q0 + r_tok;
    out_head[rb] = r_head;
    const int64_t qrow = (int64_t)out_tok[rb] * Hq + r_head;
    const char* qn = (const char*)p.q_nope + qrow * (LKV * 2);
    const char* qp = (const char*)p.q_pe + qrow * (ROPE * 2);
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row_ok[rb]) v = kk < NKN ? *(const u32x4*)(qn + (kk * 32 + 8 * g4) * 2) : *(const u32x4*)(qp + ((kk - NKN) * 32 + 8 * g4) * 2);
      qf[rb][kk] = __builtin_bit_cast(bf16x8, v);
    }
  }
  // (The queries are loaded behind the first tiles' DMAs, so that the two latencies overlap.)  Use the query
  // registers once here, so that the compiler waits for these loads now and not at their first use inside the loop,
  // where its wait would also cover every tile in flight.
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      u32x4 v = __builtin_bit_cast(u32x4, qf[rb][kk]);
      asm volatile("" : "+v"(v));
      qf[rb][kk] = __builtin_bit_cast(bf16x8, v);
    }
  // a wave whose row blocks all lie past the sequence's rows only helps with the loads
  const bool wave_active = (R0 + wave * RB * 16) < rows_total;

  int rd_slot = 0;
  for (int tile = 0; tile < n_tiles; ++tile) {
    // tile `tile` must have landed; the tiles issued after it (at most AHEAD - 1) may still be in flight.  Behind the
    // barrier every wave is done with tile - 1, whose slot takes tile + AHEAD.
    const int later = min(AHEAD - 1, n_tiles - 1 - tile);
    if (later <= 0) mla_wait_loads_and_barrier<0>();
    else if (later == 1) {
      if (dma_full) mla_wait_loads_and_barrier<NDMA>(); else mla_wait_loads_and_barrier<NDMA - 1>();
    } else {
      if (dma_full) mla_wait_loads_and_barrier<2 * NDMA>(); else mla_wait_loads_and_barrier<2 * (NDMA - 1)>();
    }
    if (tile + AHEAD < n_tiles) issue();
    const unsigned char* lds_t = lds_all + rd_slot * TILE;
    rd_slot = (rd_slot == NSLOT - 1) ? 0 : rd_slot + 1;
    if (!wave_active) continue;
    const int tb = kv_lo + tile * TT;

    // ---- S^T = K . Q^T for both row blocks (K operands shared) ---------------------------------------------
    f32x4 s_acc[RB][NS];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int st = 0; st < NS; ++st) s_acc[rb][st] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // Operand i = (sub-tile i % NS, k-step i / NS): the two sub-tiles' accumulation chains alternate.  Chunk 4 kk + g4 under the key: only its low three bits move, so
    // a k-step's address is one of two per-lane bases (kk even / odd) plus a constant.  The operands are read KPD
    // steps ahead of the matrix instructions that use them: an LDS read under load lasts several times the 16 clocks
    // of one instruction, and read just in time the wave would wait at every step.
    {
      auto read_k = [&](int i) __attribute__((always_inline)) -> u32x4 {
        const int st = i % NS, kk = i / NS;
        return *(const u32x4*)(lds_t + k_base[st][kk & 1] + (kk >> 1) * 128);
      };
      u32x4 kp[KPD];
#pragma unroll
      for (int i = 0; i < KPD; ++i) kp[i] = read_k(i);
#pragma unroll
      for (int i = 0; i < NKO; ++i) {
        const u32x4 a = kp[i % KPD];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
          s_acc[rb][i % NS] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), qf[rb][i / NS], s_acc[rb][i % NS], 0, 0, 0);
        if (i + KPD < NKO) kp[i % KPD] = read_k(i + KPD);
      }
      // the order the scheduler must keep: KPD reads first, then a matrix instruction and the next read in turn
      __builtin_amdgcn_sched_group_barrier(0x100, KPD, 0);
#pragma unroll
      for (int i = 0; i + KPD < NKO; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, RB, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, RB * KPD, 0);
    }

    // ---- online softmax per row block ------------------------------------------------------------------------
    // The reference every probability of a row is taken against need not be the exact running maximum: any common
    // value works as long as exp2 stays in range.  It is raised -- the lanes of a row agree on the new maximum and
    // everything accumulated so far is scaled down -- only when some key of the tile exceeds it by more than kMaxSlack
    // (log2 units).  After the first tiles of a sequence that is rare, which matters here: the 256 accumulators of a
    // wave live in the accumulation registers, which the vector ALU reaches only through moves.
    uint32_t pfrag[RB][NS][2];
    uint32_t pfrag_lo[RB][NS][2];  // what rounding to 16 bits took off the probabilities, rounded again (precise units)
    {
      float lmx[RB];
      bool grow = false;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        lmx[rb] = -INFINITY;
#pragma unroll
        for (int st = 0; st < NS; ++st)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            float sv = s_acc[rb][st][j];
            if constexpr (CAP) sv = fast_tanh(sv * cap_in);
            const int tok = tb + st * 16 + 4 * g4 + j;
            sv = (tok >= row_lo[rb] && tok < row_hi[rb]) ? sv : -INFINITY;
            s_acc[rb][st][j] = sv;
            lmx[rb] = fmaxf(lmx[rb], sv);
          }
        lmx[rb] *= sc_mul;  // sc_mul > 0: scaling commutes with the maximum
        grow |= lmx[rb] > m_run[rb] + kMaxSlack;
      }
      if (__any(grow)) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          const float m_new = fmaxf(m_run[rb], xor32_max(xor16_max(lmx[rb])));
          const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
          float alpha = __builtin_amdgcn_exp2f(m_run[rb] - m_use);
          m_run[rb] = m_new;
          // opaque multiplications: the compiler does not pad the distance this chip wants between a transcendental
          // instruction and a reader of its result, so the padding is put here by hand
          asm volatile("s_nop 1" : "+v"(alpha));
          asm("v_mul_f32 %0, %1, %0" : "+v"(l_run[rb]) : "v"(alpha));
          if (tile > 0) {  // in a chunk's first tile nothing has been accumulated yet
#pragma unroll
            for (int rt = 0; rt < DPL; ++rt) o_acc[rb][rt] *= alpha;
          }
        }
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const float m_use = (m_run[rb] == -INFINITY) ? 0.f : m_run[rb];
        float psum = 0.f;
#pragma unroll
        for (int st = 0; st < NS; ++st) {
          float pr[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            pr[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[rb][st][j], sc_mul, -m_use));
            psum += pr[j];
          }
          pfrag[rb][st][0] = pack_bf16(pr[0], pr[1]);
          pfrag[rb][st][1] = pack_bf16(pr[2], pr[3]);
          if (precise) {
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
              const uint32_t w = pfrag[rb][st][h2];
              pfrag_lo[rb][st][h2] = pack_bf16(pr[2 * h2] - __uint_as_float(w << 16), pr[2 * h2 + 1] - __uint_as_float(w & 0xffff0000u));
            }
          }
        }
        l_run[rb] += psum;
      }
    }

    // ---- O^T += V^T . P^T: the values are the first LKV elements of the same rows -----------------------------
    // Row tile rt spans chunks 2 rt, 2 rt + 1: under the key one of four per-lane bases (rt & 3) plus a constant.
    // Read PD row tiles ahead, as above.
    {
      auto read_v = [&](int rt) __attribute__((always_inline)) -> u32x4 {
        const unsigned char* p0 = lds_t + v_base[0][rt & 3] + (rt >> 2) * 128;
        const unsigned char* p1 = lds_t + v_base[1][rt & 3] + (rt >> 2) * 128;
        const u32x2 a_lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p0));
        const u32x2 a_hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p1));
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
      __builtin_amdgcn_sched_group_barrier(0x100, 2 * PD, 0);
#pragma unroll
      for (int rt = 0; rt + PD < DPL; ++rt) {
        __builtin_amdgcn_sched_group_barrier(0x008, RB, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, RB * PD, 0);
      if (precise) {  // the same product over the low halves of the probabilities
#pragma unroll
        for (int rt = 0; rt < DPL; ++rt) {
          const u32x4 a4 = read_v(rt);
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            const u32x4 b4 = {pfrag_lo[rb][0][0], pfrag_lo[rb][0][1], pfrag_lo[rb][1][0], pfrag_lo[rb][1][1]};
            o_acc[rb][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a4), __builtin_bit_cast(bf16x8, b4),
                                                                    o_acc[rb][rt], 0, 0, 0);
          }
        }
      }
    }
  }

  // ---- epilogue ---------------------------------------------------------------------------------------------------
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    float l_tot = l_run[rb] + __shfl_xor(l_run[rb], 16);
    l_tot += __shfl_xor(l_tot, 32);
    if (!row_ok[rb]) continue;
    if (single) {
      float l_fin = l_tot;
      if (p.sinks != nullptr && l_tot > 0.f)
        l_fin += __builtin_amdgcn_exp2f(__builtin_fmaf(p.sinks[out_head[rb]], 1.4426950408889634f, -m_run[rb]));
      const float inv = l_fin > 0.f ? 1.f / l_fin : 0.f;
      uint16_t* orow = (uint16_t*)p.out + ((int64_t)out_tok[rb] * Hq + out_head[rb]) * LKV + 4 * g4;
#pragma unroll
      for (int rt = 0; rt < DPL; ++rt) {  // accumulator column j of row tile rt is dim 16rt + 4g4 + j
        const u32x2 w = {pack_bf16(o_acc[rb][rt][0] * inv, o_acc[rb][rt][1] * inv),
                         pack_bf16(o_acc[rb][rt][2] * inv, o_acc[rb][rt][3] * inv)};
        *(u32x2*)(orow + 16 * rt) = w;
      }
    } else {
      const int64_t pslot = ((int64_t)chunk * p.T + out_tok[rb]) * Hq + out_head[rb];
      float* prow = p.part_o + pslot * LKV + 4 * g4;
#pragma unroll
      for (int rt = 0; rt < DPL; ++rt) *(f32x4*)(prow + 16 * rt) = o_acc[rb][rt];
      if (g4 == 0) {
        p.part_ml[pslot * 2 + 0] = m_run[rb];
        p.part_ml[pslot * 2 + 1] = l_tot;
      }
    }
  }
}

// ---- merge: combines the key chunks of a row, and zero-fills the rows of padded tokens -----------------------------
template <int QT>
__global__ __launch_bounds__(256) void mla_merge_kernel(MlaParams p) {
  constexpr int NK = kGenMaxLkv / 64;
  const int lane = threadIdx.x & 63;
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= p.T * p.Hq) return;
  const int t = pair / p.Hq, hq = pair - t * p.Hq;
  const int n_live = mla_live_rows(p);
  const int lkv = p.lkv;
  bool zero = false;
  int n_pieces = 0;
  if (n_live <= 0 || t < p.qsl[0] || t >= p.qsl[n_live]) {
    zero = true;
  } else {
    const int i = find_seq_wave(p.qsl, n_live, t);
    const MlaSeq sp = mla_seq(p, i);
    if (!sp.live) zero = true;
    else if (p.mfma && p.max_chunks > 1) {
      const int row = (t - sp.q0) * p.Hq + hq;
      n_pieces = mla_tile(p, sp, (row / kMlaRows) * kMlaRows, p.n_units[2]).n_chunks;
    }
  }
  const bool merge = n_pieces > 1;
  if (!zero && !merge) return;
  float acc[NK];
#pragma unroll
  for (int k = 0; k < NK; ++k) acc[k] = 0.f;
  float inv = 0.f;
  if (merge) {
    const int64_t slot0 = (int64_t)t * p.Hq + hq;
    const int64_t stride = (int64_t)p.T * p.Hq;
    float m = -INFINITY;
    for (int c = lane; c < n_pieces; c += 64) m = fmaxf(m, p.part_ml[(slot0 + c * stride) * 2]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    const float m_use = (m == -INFINITY) ? 0.f : m;
    float l = 0.f;
    for (int c = 0; c < n_pieces; ++c) {  // n_pieces <= kMlaMaxChunks
      const float2 ml = *(const float2*)(p.part_ml + (slot0 + c * stride) * 2);
      const float w = __builtin_amdgcn_exp2f(ml.x - m_use);
      l += w * ml.y;
      const float* row = p.part_o + (slot0 + c * stride) * lkv;
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        const int d = lane + 64 * k;
        if (d < lkv) acc[k] = fmaf(w, row[d], acc[k]);
      }
    }
    if (p.sinks != nullptr && l > 0.f) l += __builtin_amdgcn_exp2f(__builtin_fmaf(p.sinks[hq], 1.4426950408889634f, -m_use));
    inv = l > 0.f ? 1.f / l : 0.f;
  }
#pragma unroll
  for (int k = 0; k < NK; ++k) {
    const int d = lane + 64 * k;
    if (d < lkv) {
      const int64_t o = ((int64_t)t * p.Hq + hq) * lkv + d;
      const float r = acc[k] * inv;
      store_out<QT>(p.out, o, r);
    }
  }
}

// The same for two neighbouring heads of a token per wave on the matrix-core path (latent 512, an even head count):
// their partial rows are neighbours in memory, and what bounds a row's merge is its chain of dependent loads (sequence
// look-up, lengths, (max, sum) pairs, partial rows), which here serves two rows.
__global__ __launch_bounds__(256, 4) void mla_merge_pair_kernel(MlaParams p) {
  constexpr int LKV = 512, HPW = 2, NK = LKV / 64, NKT = NK * HPW;
  const int lane = threadIdx.x & 63;
  const int groups = p.Hq / HPW;
  const int pair = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (pair >= p.T * groups) return;
  const int t = pair / groups, hq0 = (pair - t * groups) * HPW;
  const int n_live = mla_live_rows(p);
  bool zero = false;
  int n_p[HPW] = {0, 0};
  if (n_live <= 0 || t < p.qsl[0] || t >= p.qsl[n_live]) {
    zero = true;
  } else {
    const int i = find_seq_wave(p.qsl, n_live, t);
    const MlaSeq sp = mla_seq(p, i);
    if (!sp.live) zero = true;
    else if (p.max_chunks > 1) {
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) {  // the two heads can lie in different row tiles
        const int row = (t - sp.q0) * p.Hq + hq0 + hh;
        const int n = mla_tile(p, sp, (row / kMlaRows) * kMlaRows, p.n_units[2]).n_chunks;
        n_p[hh] = n > 1 ? n : 0;  // a row in one piece was written by the kernel that computed it
      }
    }
  }
  const int n_max = max(n_p[0], n_p[1]);
  if (!zero && n_max == 0) return;
  float acc[NKT];
#pragma unroll
  for (int k = 0; k < NKT; ++k) acc[k] = 0.f;
  float inv[HPW] = {0.f, 0.f};
  if (n_max > 0) {
    const int64_t slot0 = (int64_t)t * p.Hq + hq0;
    const int64_t stride = (int64_t)p.T * p.Hq;
    float m_use[HPW], l[HPW], w_c[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {  // n_pieces <= kMlaMaxChunks: lane c holds piece c
      float2 ml = {-INFINITY, 0.f};
      if (lane < n_p[hh]) ml = *(const float2*)(p.part_ml + (slot0 + hh + lane * stride) * 2);
      float m = ml.x;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
      m_use[hh] = (m == -INFINITY) ? 0.f : m;
      w_c[hh] = lane < n_p[hh] ? __builtin_amdgcn_exp2f(ml.x - m_use[hh]) : 0.f;
      float lt = w_c[hh] * ml.y;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) lt += __shfl_xor(lt, o);
      l[hh] = lt;
    }
    for (int c = 0; c < n_max; c += 2) {  // two pieces (32 floats per lane) in flight
      float v[2][NKT];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const float* row = p.part_o + (slot0 + (int64_t)(c + u) * stride) * LKV;
#pragma unroll
        for (int k = 0; k < NKT; ++k) v[u][k] = (c + u < n_p[k / NK]) ? row[lane + 64 * k] : 0.f;  // never a piece nobody wrote
      }
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const float w0 = __shfl(w_c[0], c + u), w1 = __shfl(w_c[1], c + u);  // zero past a head's pieces
#pragma unroll
        for (int k = 0; k < NKT; ++k) acc[k] = fmaf(k < NK ? w0 : w1, v[u][k], acc[k]);
      }
    }
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      float lt = l[hh];
      if (p.sinks != nullptr && lt > 0.f) lt += __builtin_amdgcn_exp2f(__builtin_fmaf(p.sinks[hq0 + hh], 1.4426950408889634f, -m_use[hh]));
      inv[hh] = lt > 0.f ? 1.f / lt : 0.f;
    }
  }
#pragma unroll
  for (int k = 0; k < NKT; ++k) {
    if (!zero && n_p[k / NK] == 0) continue;
    const int64_t o = ((int64_t)t * p.Hq + hq0) * LKV + lane + 64 * k;
    ((uint16_t*)p.out)[o] = float_to_bf16_bits(acc[k] * inv[k / NK]);
  }
}

template <int QT>
int launch_generic_q(hipStream_t stream, const MlaParams& p) {
  dim3 grid(p.T, p.Hq), block(64);
  switch (p.kv_dtype) {
    case RPA_F32: hipLaunchKernelGGL((mla_generic_kernel<QT, RPA_F32>), grid, block, 0, stream, p); break;
    case RPA_BF16: hipLaunchKernelGGL((mla_generic_kernel<QT, RPA_BF16>), grid, block, 0, stream, p); break;
    case RPA_F16: hipLaunchKernelGGL((mla_generic_kernel<QT, RPA_F16>), grid, block, 0, stream, p); break;
    case RPA_FP8_E4M3: hipLaunchKernelGGL((mla_generic_kernel<QT, RPA_FP8_E4M3>), grid, block, 0, stream, p); break;  // codes as cast, no scales
    default: return (int)hipErrorInvalidValue;
  }
  return (int)hipGetLastError();
}

}  // namespace

int launch_mla_scatter(hipStream_t stream, const MlaParams& p) {
  const int blocks = (p.T + 3) / 4;
  switch (elem_bytes(p.kv_dtype)) {  // the write copies bits, whatever they encode
    case 4: hipLaunchKernelGGL((mla_scatter_kernel<uint32_t>), dim3(blocks), dim3(256), 0, stream, p); break;
    case 2: hipLaunchKernelGGL((mla_scatter_kernel<uint16_t>), dim3(blocks), dim3(256), 0, stream, p); break;
    default: hipLaunchKernelGGL((mla_scatter_kernel<uint8_t>), dim3(blocks), dim3(256), 0, stream, p); break;
  }
  return (int)hipGetLastError();
}

int launch_mla_generic(hipStream_t stream, const MlaParams& p) {
  if (p.lkv > kGenMaxLkv || p.rope > kGenMaxRope) return (int)hipErrorInvalidValue;
  return p.q_dtype == RPA_F32 ? launch_generic_q<RPA_F32>(stream, p)
         : p.q_dtype == RPA_F16 ? launch_generic_q<RPA_F16>(stream, p) : launch_generic_q<RPA_BF16>(stream, p);
}

// bf16 queries and pages of the one shape every model with this cache uses (latent 512, rope 64, the rope key right
// behind the latent part), pages a multiple of the 32-key tile, and page rows a 32-bit byte offset can address
bool mla_mfma_supported(const MlaParams& p) {
  return p.q_dtype == RPA_BF16 && p.kv_dtype == RPA_BF16 && p.lkv == 512 && p.rope == 64 && p.rope_off == 512 &&
         p.page_size % 32 == 0 && (p.token_stride & 15) == 0 && (int64_t)32 * p.token_stride < ((int64_t)1 << 31);
}

int64_t mla_plan_slots(int T, int S, int Hq) { return ((int64_t)T * Hq) / kMlaRows + S; }  // upper bound on row tiles of the batch

static size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }
size_t mla_plan_bytes(int T, int S, int Hq, int max_chunks) {
  const size_t slots = (size_t)mla_plan_slots(T, S, Hq);
  // the unit list has an entry for every block of the attention kernel's grid, which is rounded up to a multiple of 8
  return up256(slots * 8) + 256 + up256((slots * (size_t)max_chunks + kXcds) * 8);
}

int launch_mla_mfma(hipStream_t stream, const MlaParams& p) {
  const int64_t slots = mla_plan_slots(p.T, p.S, p.Hq);
  const int64_t blocks = (slots * p.max_chunks + kXcds - 1) / kXcds * kXcds;  // most units the batch can have
  if (blocks > 0x7fffffff) return (int)hipErrorInvalidValue;
  if (slots <= kMlaSortSlots) {  // plan, sorted unit list and the page write in one launch
    const int write_blocks = p.new_kv ? (p.T + 15) / 16 : 0;
    hipLaunchKernelGGL(mla_plan_sorted_kernel, dim3((unsigned)(1 + write_blocks)), dim3(1024), 0, stream, p, (int)slots);
  } else {
    const int plan_blocks = (int)((slots + 255) / 256);
    const int write_blocks = p.new_kv ? (p.T + 3) / 4 : 0;  // the page write rides along (see mla_plan_kernel)
    hipLaunchKernelGGL(mla_plan_kernel, dim3((unsigned)(plan_blocks + write_blocks)), dim3(256), 0, stream, p, (int)slots, plan_blocks);
    hipLaunchKernelGGL(mla_compact_kernel, dim3(1), dim3(1024), 0, stream, p, (int)slots);
  }
  if (p.softcap > 0.f) hipLaunchKernelGGL((mla_attn_kernel<true>), dim3((unsigned)blocks), dim3(64 * kMlaWaves), 0, stream, p);
  else hipLaunchKernelGGL((mla_attn_kernel<false>), dim3((unsigned)blocks), dim3(64 * kMlaWaves), 0, stream, p);
  return (int)hipGetLastError();
}

int launch_mla_merge(hipStream_t stream, const MlaParams& p) {
  if (p.lkv > kGenMaxLkv) return (int)hipErrorInvalidValue;
  if (p.mfma && p.q_dtype == RPA_BF16 && p.lkv == 512 && p.Hq % 2 == 0) {
    const int pairs = (int)(((int64_t)p.T * (p.Hq / 2) + 3) / 4);
    hipLaunchKernelGGL(mla_merge_pair_kernel, dim3(pairs), dim3(256), 0, stream, p);
    return (int)hipGetLastError();
  }
  const int blocks = (int)(((int64_t)p.T * p.Hq + 3) / 4);
  if (p.q_dtype == RPA_F32) hipLaunchKernelGGL((mla_merge_kernel<RPA_F32>), dim3(blocks), dim3(256), 0, stream, p);
  else if (p.q_dtype == RPA_F16) hipLaunchKernelGGL((mla_merge_kernel<RPA_F16>), dim3(blocks), dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((mla_merge_kernel<RPA_BF16>), dim3(blocks), dim3(256), 0, stream, p);
  return (int)hipGetLastError();
}

}  // namespace rpa
