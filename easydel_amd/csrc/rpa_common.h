// Shared device-side definitions for the gfx950 ragged-paged-attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/rpa_hip.h"

namespace rpa {

constexpr int kWave = 64;
constexpr int kRowBlock = 16;      // MFMA M/N extent: rows (token, group-head pairs) per wave
constexpr int kMaxSplitsCap = 256;   // hard upper bound on split-K partials per sequence
constexpr int kPlanHeader = 16;      // ints before the prefix array in the decode plan
constexpr int kMaxDecodeWgs = 4096;  // persistent decode workgroups per KV-head group
constexpr int kMaxSortedSeqs = 1024; // batches of up to this many sequences get their large-row sequences ordered longest first
constexpr int kPrefillRows = 128;    // query rows (token x group head) one prefill workgroup owns (the 32x32-tile kernel: 256; AttnParams::pre_rows)
constexpr int kMaxPrefillChunks = 8; // key chunks one prefill row tile may be split into
constexpr int kMinPrefillChunk = 2048; // fewest keys of such a chunk
constexpr int kMaxDevices = 64;      // devices of one process the per-device caches hold

// Everything a kernel needs, passed by value.
struct AttnParams {
  const void* q;
  const void* k_pages;     // K of KV head h of a token: k_pages + page*page_stride + token*token_stride + h*head_stride
  const void* v_pages;     // V likewise.  Interleaved pages: v_pages = k_pages + one row, head_stride = two rows;
                           // separate K and V pools: two allocations, head_stride = one row
  const float* kv_scales;  // [P][C] or null
  const float* sinks;      // [Hq] attention-sink logits (natural-log units, not scaled, not soft-capped) or null
  const void* new_k;       // [T][Hkv][D] rows the decode plan kernel's launch also writes into the pages (fused v3
  const void* new_v;       // call on the MFMA path), or null: the pages are read as they are
  const int32_t* context_lens;
  const int32_t* block_tables;
  const int32_t* qsl;
  const int32_t* num_seqs;  // live rows, or null: every one of the S rows is live
  void* out;
  float* part_o;   // [max_splits][Tdec][Hq][D]   Tdec = t_dec_max: decode-class query tokens, compacted
  float* part_ml;  // [max_splits][Tdec][Hq][2]   (running max in log2 units, running sum)
  float* pre_o;    // prefill split-K partials [pre_max_chunks][T][Hq][D]
  float* pre_ml;   // [pre_max_chunks][T][Hq][2]
  int32_t* plan;   // decode plan: [0] = W (flattened keys), [1] = Q (keys per workgroup), [2] = 1 if any sequence needs
                   // the large-row kernel, [3] = 1 if the merge kernel has work, [4] = keys per split-K chunk of the
                   // large-row kernel, then at kPlanHeader:
                   // P[S+1] exclusive prefix of per-sequence key spans, R[S+1] exclusive prefix of
                   // decode-class query tokens (row of a token in the partial buffers), first_seq[kMaxDecodeWgs],
                   // then the large-row sequences longest first: [5] = their number L (-1: the batch has too many
                   // sequences, not ordered), order[kMaxSortedSeqs] (sequence of rank r), tile_start[kMaxSortedSeqs + 1]
                   // (exclusive prefix of their row-tile counts in that order)
  int T, S, M, P, page_size, Hq, Hkv, group, D, C;
  int Dq;                // elements of a q / out row.  D is the head size the kernels compute with: Dq itself, or -- on the
                         // MFMA path over padded head storage -- the stored row width (128 / 256), whose padding holds zeros
  int64_t token_stride;  // bytes between consecutive tokens of a page = C*D*elem
  int64_t page_stride;   // bytes between pages
  int64_t head_stride;   // bytes between KV heads inside a token
  int kv_pad_bytes;      // bytes of zero padding behind a head's Dq elements in the pages (padded head storage), else 0
  int q_dtype, kv_dtype;
  float scale;       // softmax scale
  float scale_log2;  // softmax scale * log2(e)
  int window;        // <= 0: none
  float softcap;     // <= 0: none
  int max_splits;    // >= 2: most partial slots one sequence may use
  int dec_rows;      // most query rows per KV head (q_len * group) of a sequence the decode kernel serves: 16 or 32
  int t_dec_max;     // static bound on decode-class query tokens = rows of one partial slot
  int n_wg;          // persistent decode workgroups per KV-head group
  int decode_wgs;    // override for n_wg, 0 = as many as are resident at once
  int pre_chunk;     // keys per prefill split-K chunk (multiple of 64) when pre_auto is 0
  int pre_max_chunks;  // chunks the prefill partial buffers hold; 1 = never split
  int pre_auto;        // 1: the plan kernel sets the chunk length from the batch's lengths; 0: pre_chunk as given
  int pre_slots;       // workgroups of the prefill kernel the chip holds at once
  int pre_rows;        // query rows (token x group head) one workgroup of the call's prefill kernel owns: 128 or 256
  int pre_x32;         // 1: the 32x32-tile prefill kernel serves the call (pre_rows is its row-tile height)
  int decode_sync;   // decode workgroups re-align their waves with a barrier every this many tiles (power of two), 0 = never
  int decode_pace;   // 0: the decode kernel never pauses a wave (see PACE there); default 1
  int decode_dma;    // 1: bf16 decode tiles go global -> LDS directly where that kernel applies; 0: always through registers
  int decode_which;  // launches of the decode stage: bit 0 plan kernel, bit 1 decode kernel
  int prefill_dma;   // 1: bf16 prefill tiles go global -> LDS directly where that kernel applies; 0: always through registers
  int mfma_path;     // 1: bf16 queries served by the MFMA kernels; 0: fp32 VALU kernel serves every row
  // 8-bit pages whose large-row sequences may be served from bf16 copies of their pages (null: never).  Written by the
  // decision kernel ahead of the plan: [0] = 1 if this batch is served that way, [1] = copied pages in use,
  // [2 + i] = the copied page of block-table column 0 of sequence i, were it copied (the visible columns follow in
  // block-table order; under a sliding window the first ones are not copied and this is below zero).
  const int32_t* wide;
  void* wide_pages;    // the copies: [wide_cap][page_size][2 Hkv][D] bf16, bare codes, K of head h at row 2h, V at 2h + 1
  int wide_cap;        // pages the copies hold
  int wide_rows;       // pre_rows of a batch served from the copies
  int wide_slots;      // pre_slots likewise
  int src_P;           // pages of the 8-bit pool, for the kernel that reads the copies (its P is wide_cap)
  int wide_min_rows;   // fewest query rows per KV head and copied page, on the batch's average, for the copies to be made ...
  int wide_min_rows_full;  // ... and the lower bar of a batch that gives the kernel that reads them wide_min_wgs
  int wide_min_wgs;        // workgroups (row tiles of wide_rows x KV heads) or more
  int wide_min_window;     // under a sliding window: the shortest window, and wide_min_wgs workgroups, for the copies to be made
};

// Row-tile height and resident workgroups of the large-row kernel that serves this batch.
__device__ __forceinline__ bool wide_mode(const AttnParams& p) { return p.wide != nullptr && p.wide[0] != 0; }
__device__ __forceinline__ int pre_rows_of(const AttnParams& p) { return wide_mode(p) ? p.wide_rows : p.pre_rows; }
__device__ __forceinline__ int pre_slots_of(const AttnParams& p) { return wide_mode(p) ? p.wide_slots : p.pre_slots; }

__device__ __forceinline__ int live_rows(const AttnParams& p);

// Per-sequence facts.  Every kernel derives them from device metadata with this one function, so the
// producers (attention kernels) and the consumer (merge) always agree on who wrote what.
struct SeqPlan {
  int q0, q_len, ctx;
  int lo, hi;       // key range any row of the sequence may see, lo rounded down to 64 tokens
  bool live;        // has queries and keys
  bool small_rows;  // q_len * group <= dec_rows (16 or 32): served by the split-K decode kernel
};

__device__ __forceinline__ SeqPlan seq_plan(const AttnParams& p, int i) {
  SeqPlan s;
  const int n_live = live_rows(p);
  s.q0 = p.qsl[i];
  s.q_len = p.qsl[i + 1] - s.q0;
  s.ctx = p.context_lens[i];
  if (s.ctx > p.M * p.page_size) s.ctx = p.M * p.page_size;  // never index past the block-table row
  s.live = (i < n_live) && (s.q_len > 0) && (s.ctx > 0);
  s.hi = s.ctx;
  s.lo = 0;
  if (p.window > 0) {
    int first = s.ctx - s.q_len - p.window + 1;  // lowest key visible to the first query row
    s.lo = first > 0 ? (first & ~63) : 0;
  }
  s.small_rows = (s.q_len * p.group <= p.dec_rows);
  return s;
}

// never more than the S rows the metadata arrays hold, whatever the device value says
__device__ __forceinline__ int live_rows(const AttnParams& p) { return p.num_seqs ? min(p.num_seqs[0], p.S) : p.S; }

// Attention sinks: the softmax of query head hq runs over the keys and one more logit, sinks[hq], whose
// probability is then dropped -- a key with that score and a zero value row.  Only the denominator changes:
// given l = sum over keys of exp2(score - m_log2), for any reference m_log2 common to the row (log2 units),
// this returns l + exp2(sinks[hq]*log2(e) - m_log2).  Rows that see no key (l == 0) keep their zero output.
__device__ __forceinline__ float with_sink(const AttnParams& p, int hq, float m_log2, float l) {
  if (p.sinks == nullptr || !(l > 0.f)) return l;
  return l + __builtin_amdgcn_exp2f(__builtin_fmaf(p.sinks[hq], 1.4426950408889634f, -m_log2));
}

// Key range [kv_lo, kv_hi) a prefill row tile (rows [R0, R0 + pre_rows_of(p)) of a sequence) must visit, kv_lo
// rounded down to 64, and the split-K chunks the prefill kernel cuts it into: the range over the chunk length the
// plan kernel chose (plan[4]), rounded to the nearest count the partial buffers hold, all chunks of one length (a
// multiple of 64; the last one holds what is left), so that the workgroups of a sequence finish together.
struct PrefillTile {
  int kv_lo, kv_hi, vis_lo, n_chunks, chunk_len;
};
__device__ __forceinline__ PrefillTile prefill_tile(const AttnParams& p, const SeqPlan& sp, int R0) {
  PrefillTile t;
  const int rows_total = sp.q_len * p.group;
  const int last_row = min(R0 + pre_rows_of(p), rows_total) - 1;
  const int base_pos = sp.ctx - sp.q_len;
  t.kv_hi = min(sp.ctx, base_pos + last_row / p.group + 1);
  t.vis_lo = (p.window > 0) ? max(base_pos + R0 / p.group - p.window + 1, 0) : 0;
  t.kv_lo = t.vis_lo & ~63;
  const int span = t.kv_hi - t.kv_lo;
  const int target = p.plan[4];  // >= 64
  t.n_chunks = span <= 0 ? 0 : min(max((int)(((int64_t)span + target / 2) / target), 1), p.pre_max_chunks);
  t.chunk_len = target;
  if (t.n_chunks > 1) {
    t.chunk_len = ((span + t.n_chunks - 1) / t.n_chunks + 63) & ~63;
    t.n_chunks = (span + t.chunk_len - 1) / t.chunk_len;  // rounding up to 64 may have emptied the last one
  }
  return t;
}

// Partial slots the decode kernel filled for sequence i (0 or 1: the output row is already final).
// P is the exclusive prefix of key spans in the decode plan, Q the span handled per workgroup.
__device__ __forceinline__ int decode_pieces(const int32_t* __restrict__ plan, int i) {
  const int Q = plan[1];
  const int p0 = plan[kPlanHeader + i], p1 = plan[kPlanHeader + i + 1];
  if (p1 <= p0) return 0;
  return (p1 - 1) / Q - p0 / Q + 1;
}

// Largest i in [0, n) with qsl[i] <= t (qsl non-decreasing); callers guarantee qsl[0] <= t < qsl[n].
__device__ __forceinline__ int find_seq(const int32_t* qsl, int n, int t) {
  int lo = 0, hi = n;  // invariant: qsl[lo] <= t < qsl[hi]
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (qsl[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}

// The same search by a whole wavefront whose 64 lanes (all active) ask for the same t: every round reads 64
// entries spread evenly over what is left of the range with one load and keeps the sixty-fourth that holds the
// answer, so up to 4096 sequences cost two dependent loads where the scalar search costs twelve.
__device__ __forceinline__ int find_seq_wave(const int32_t* qsl, int n, int t) {
  const int lane = threadIdx.x & 63;
  int lo = 0, hi = n;  // invariant: qsl[lo] <= t < qsl[hi]
  while (hi - lo > 1) {
    const int stride = (hi - lo + 63) >> 6;
    const int idx = lo + lane * stride;
    const bool le = idx < hi && qsl[idx] <= t;  // true for a prefix of the lanes (lane 0 by the invariant)
    const int last = __popcll(__ballot(le)) - 1;
    lo += last * stride;
    hi = min(lo + stride, hi);
  }
  return lo;
}

// New K/V rows of query token t into their page slot (the write half of the fused v3 operation): the token's
// sequence i and position ctx_i - q_len_i + (t - q0_i) give the page and slot; K of head h goes to k_pages' row of
// head h, V to v_pages'.  Called with the same t by nthreads threads (whole wavefronts) numbered tid = 0 .. nthreads-1,
// which share the copy; bit-exact copy of whole rows.
__device__ __forceinline__ void scatter_token(const char* __restrict__ key, const char* __restrict__ value,
                                              char* k_pages, char* v_pages, const int32_t* __restrict__ context_lens,
                                              const int32_t* __restrict__ block_tables, const int32_t* __restrict__ qsl,
                                              int n_live, int M, int P, int page_size, int Hkv, int head_bytes,
                                              int64_t head_stride, int64_t token_stride, int64_t page_stride, int t,
                                              int tid, int nthreads, int pad_bytes = 0) {
  if (n_live <= 0 || t < qsl[0] || t >= qsl[n_live]) return;
  const int i = find_seq_wave(qsl, n_live, t);
  const int q0 = qsl[i], q_len = qsl[i + 1] - q0;
  const int pos = context_lens[i] - q_len + (t - q0);
  if (pos < 0) return;
  const int page_idx = pos / page_size;
  if (page_idx >= M) return;
  const int page = block_tables[(int64_t)i * M + page_idx];
  if (page < 0 || page >= P) return;
  const int64_t row = (int64_t)page * page_stride + (int64_t)(pos % page_size) * token_stride;
  const char* ksrc = key + (int64_t)t * Hkv * head_bytes;
  const char* vsrc = value + (int64_t)t * Hkv * head_bytes;
  char* kdst = k_pages + row;
  char* vdst = v_pages + row;
  if ((head_bytes & 15) == 0 && ((((uintptr_t)kdst) | ((uintptr_t)vdst) | ((uintptr_t)ksrc) | ((uintptr_t)vsrc) | (uintptr_t)head_stride) & 15) == 0) {
    const int vec_per_head = head_bytes >> 4;
    const int n = 2 * Hkv * vec_per_head;
    for (int k = tid; k < n; k += nthreads) {
      const int ch = k / vec_per_head, w = k - ch * vec_per_head;  // (head, K or V), vector within the row
      const char* src = ((ch & 1) ? vsrc : ksrc) + (int64_t)(ch >> 1) * head_bytes;
      char* dst = ((ch & 1) ? vdst : kdst) + (int64_t)(ch >> 1) * head_stride;
      ((uint4*)dst)[w] = ((const uint4*)src)[w];
    }
  } else {
    const int n = 2 * Hkv * head_bytes;
    for (int k = tid; k < n; k += nthreads) {
      const int ch = k / head_bytes, w = k - ch * head_bytes;
      const char* src = ((ch & 1) ? vsrc : ksrc) + (int64_t)(ch >> 1) * head_bytes;
      char* dst = ((ch & 1) ? vdst : kdst) + (int64_t)(ch >> 1) * head_stride;
      dst[w] = src[w];
    }
  }
  // padded head storage: the bytes between a head's head_bytes and its stored row width are written as zeros
  if (pad_bytes > 0) {
    const int n = 2 * Hkv * pad_bytes;
    for (int k = tid; k < n; k += nthreads) {
      const int ch = k / pad_bytes, w = k - ch * pad_bytes;
      (((ch & 1) ? vdst : kdst) + (int64_t)(ch >> 1) * head_stride + head_bytes)[w] = 0;
    }
  }
}

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {  // round to nearest even, NaN kept quiet
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ float fp8_e4m3_to_float(uint8_t c) {
  auto v = __builtin_amdgcn_cvt_pk_f32_fp8((int)c, false);
  return v[0];
}

template <int DT> struct ElemBytes;
template <> struct ElemBytes<RPA_F32> { static constexpr int v = 4; };
template <> struct ElemBytes<RPA_BF16> { static constexpr int v = 2; };
template <> struct ElemBytes<RPA_FP8_E4M3> { static constexpr int v = 1; };
template <> struct ElemBytes<RPA_INT8> { static constexpr int v = 1; };
template <> struct ElemBytes<RPA_F16> { static constexpr int v = 2; };

inline int elem_bytes(int dt) { return dt == RPA_F32 ? 4 : (dt == RPA_BF16 || dt == RPA_F16) ? 2 : 1; }
__device__ __forceinline__ int elem_bytes_dev(int dt) { return dt == RPA_F32 ? 4 : (dt == RPA_BF16 || dt == RPA_F16) ? 2 : 1; }

template <int DT>
__device__ __forceinline__ float load_elem(const void* base, int64_t idx) {
  if constexpr (DT == RPA_F32) return ((const float*)base)[idx];
  else if constexpr (DT == RPA_BF16) return bf16_bits_to_float(((const uint16_t*)base)[idx]);
  else if constexpr (DT == RPA_FP8_E4M3) return fp8_e4m3_to_float(((const uint8_t*)base)[idx]);
  else if constexpr (DT == RPA_F16) return (float)((const _Float16*)base)[idx];
  else return (float)((const int8_t*)base)[idx];
}

// One result element in the q / out element type (round to nearest even).
template <int QT>
__device__ __forceinline__ void store_out(void* base, int64_t idx, float r) {
  if constexpr (QT == RPA_F32) ((float*)base)[idx] = r;
  else if constexpr (QT == RPA_F16) ((_Float16*)base)[idx] = (_Float16)r;
  else ((uint16_t*)base)[idx] = float_to_bf16_bits(r);
}

// Launchers (one per translation unit); all return a hipError_t as int.
int launch_attn_generic(hipStream_t stream, const AttnParams& p);
int launch_attn_decode(hipStream_t stream, const AttnParams& p, int which = 3);  // bit 0: plan kernel, bit 1: decode kernel
int launch_attn_prefill(hipStream_t stream, const AttnParams& p);
int launch_attn_prefill_dma(hipStream_t stream, const AttnParams& p);  // bf16 pages, tiles loaded straight into LDS
int launch_attn_merge(hipStream_t stream, const AttnParams& p);
bool decode_supported(const AttnParams& p);
int decode_row_limit(int T, int S, int D, int kv_dtype);
bool prefill_supported(const AttnParams& p);
bool prefill_dma_supported(const AttnParams& p);
int launch_attn_prefill_dma8(hipStream_t stream, const AttnParams& p);  // 8-bit pages: codes loaded straight into LDS, widened there
int launch_attn_prefill_x32(hipStream_t stream, const AttnParams& p);   // 16-bit pages, 32x32x16 tiles, one workgroup per CU
int prefill_x32_rows(const AttnParams& p);  // its row-tile height at the call's shape, 0 where it does not apply
bool prefill_dma8_supported(const AttnParams& p);
int launch_widen_decide(hipStream_t stream, const AttnParams& p);  // 8-bit pages: whether this batch's large rows are served from bf16 copies ...
int launch_widen_pages(hipStream_t stream, const AttnParams& p);   // ... and the copies

}  // namespace rpa
