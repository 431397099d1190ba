// Multi-latent attention (MLA) over latent ragged pages: parameters and launchers.
//
// One row per token and no head axis: row = [latent (lkv) | padding | rope key (rope) | padding], every query
// head reads the same row.  score = scale * (q_nope . latent + q_pe . rope key); the values are the latent rows.
#pragma once
#include "rpa_common.h"

namespace rpa {

constexpr int kMlaRows = 128;       // query rows (token x head) one workgroup of the MFMA kernel owns
constexpr int kMlaMaxChunks = 16;   // key chunks a row tile may be split into

struct MlaParams {
  const void* q_nope;  // [T][Hq][lkv]
  const void* q_pe;    // [T][Hq][rope]
  const void* new_kv;  // [T][lkv]  rows to write before attending, in the pages' dtype, or null
  const void* new_pe;  // [T][rope]
  void* pages;         // [P][page_size][row_elems]
  const float* sinks;  // [Hq] or null
  const int32_t* context_lens;
  const int32_t* block_tables;
  const int32_t* qsl;
  const int32_t* num_seqs;
  void* out;       // [T][Hq][lkv], query dtype
  float* part_o;   // [max_chunks][T][Hq][lkv]
  float* part_ml;  // [max_chunks][T][Hq][2]  (running max in log2 units, running sum)
  int2* plan;      // [row-tile slots] (sequence, key chunks | keys / 64 of a chunk << 8) of the row tile at a slot;
                   // chunks = 0: no such tile
  int32_t* n_units;  // [0] number of (row tile, key chunk) units of the batch = workgroups with work;
                     // [1] 1 if the list is sorted longest first, 0 if it is in slot order;
                     // [2] chunk length the plan kernel chose for this batch (keys, a multiple of 64), 0: the cut
                     //     follows rule_chunks / min_chunk
  int2* units;     // [n_units[0]] (slot, chunk | sequence << 5): what a workgroup needs to start, in one load
  int T, S, M, P, page_size, Hq, lkv, rope, rope_off, row_elems;
  int64_t token_stride, page_stride;  // bytes
  int q_dtype, kv_dtype;
  float scale, scale_log2;
  int window;
  float softcap;
  int max_chunks;  // chunks the partial buffers hold; 1 = never split
  int rule_chunks; // chunks a row tile is cut into when the cut follows the shapes (<= max_chunks)
  int min_chunk;   // fewest keys per chunk then (multiple of 64)
  int auto_chunk;  // 1: the plan kernel may choose a chunk length from the batch's own lengths (n_units[2])
  int cus;         // compute units of the device
  int mfma;        // 1: every row served by the MFMA kernel; 0: by the fp32 kernel
};

struct MlaSeq {
  int q0, q_len, ctx;
  bool live;
};

__device__ __forceinline__ int mla_live_rows(const MlaParams& p) { return p.num_seqs ? min(p.num_seqs[0], p.S) : p.S; }

__device__ __forceinline__ MlaSeq mla_seq(const MlaParams& p, int i) {
  MlaSeq s;
  s.q0 = p.qsl[i];
  s.q_len = p.qsl[i + 1] - s.q0;
  s.ctx = min(p.context_lens[i], p.M * p.page_size);  // never index past the block-table row
  s.live = i < mla_live_rows(p) && s.q_len > 0 && s.ctx > 0;
  return s;
}

// How a row tile's `span` keys are cut: n_chunks chunks of `chunk` keys (a multiple of 64).  With a chunk length L
// chosen by the plan kernel (small batches): as many even chunks as L asks for and the partial buffers hold; else as
// even as rule_chunks allows and never shorter than min_chunk.
__device__ __forceinline__ void mla_cut(const MlaParams& p, int span, int L, int* chunk, int* n_chunks) {
  *chunk = p.min_chunk;
  *n_chunks = 0;
  if (span <= 0) return;
  if (L > 0) {
    const int n = min(p.max_chunks, (span + L - 1) / L);
    *chunk = (((span + n - 1) / n) + 63) & ~63;
  } else {
    const int even = (((span + p.rule_chunks - 1) / p.rule_chunks) + 63) & ~63;
    *chunk = max(p.min_chunk, even);
  }
  *n_chunks = (span + *chunk - 1) / *chunk;
}

// Key range [kv_lo, kv_hi) the row tile [R0, R0 + kMlaRows) of a sequence must visit (kv_lo rounded down to 64), the
// lowest key any of its rows sees, and how the range is cut (mla_cut; L = n_units[2] of the batch's plan).  The plan,
// the attention kernel and the merge kernel all derive the cut from this one function.
struct MlaTile {
  int kv_lo, kv_hi, vis_lo, chunk, n_chunks;
};
__device__ __forceinline__ MlaTile mla_tile(const MlaParams& p, const MlaSeq& sp, int R0, int L) {
  MlaTile t;
  const int rows_total = sp.q_len * p.Hq;
  const int last_row = min(R0 + kMlaRows, rows_total) - 1;
  const int base_pos = sp.ctx - sp.q_len;
  t.kv_hi = min(sp.ctx, base_pos + last_row / p.Hq + 1);
  t.vis_lo = (p.window > 0) ? max(base_pos + R0 / p.Hq - p.window + 1, 0) : 0;
  t.kv_lo = t.vis_lo & ~63;
  mla_cut(p, t.kv_hi - t.kv_lo, L, &t.chunk, &t.n_chunks);
  return t;
}

int launch_mla_scatter(hipStream_t stream, const MlaParams& p);
int launch_mla_generic(hipStream_t stream, const MlaParams& p);
int launch_mla_mfma(hipStream_t stream, const MlaParams& p);
int64_t mla_plan_slots(int T, int S, int Hq);  // row-tile slots of a batch (upper bound) = entries of MlaParams::plan
size_t mla_plan_bytes(int T, int S, int Hq, int max_chunks);  // plan + unit count + unit list
int launch_mla_merge(hipStream_t stream, const MlaParams& p);
bool mla_mfma_supported(const MlaParams& p);

}  // namespace rpa
