// 8-bit pages served to the 32x32-tile prefill kernel through bf16 copies.
//
// The 8-bit large-row kernel widens every tile of codes in LDS, on the vector ALU, once per workgroup that visits it:
// at 2 048 query tokens a page is widened by dozens of workgroups, and the widening shares the issue port with the
// matrix instructions.  Where a batch's large-row sequences have enough query rows per cached page, it is cheaper to
// widen each of their pages once, into a scratch pool of bf16 pages, and run the 16-bit kernel on the copies:
//
// K and V rows are copied as bare codes (both code sets are exact in bf16) and the scales stay where they are: the
// kernel multiplies the scores of a page by the page's K scale in float32 and its probabilities by the page's V scale
// (a tile of 64 keys lies in one page).  A key or value scaled and rounded to bf16 would carry an error of 2^-9 of every
// term into the sums: measured on a row of six keys with cancelling values, 2.1e-2 on an output of 2.8.
//
// Two kernels: the decision (one workgroup, ahead of the plan kernel, which cuts row tiles at the height of whichever
// kernel serves the batch) and the copy (behind the plan kernel's launch, which may write the step's new rows into the
// pages).  The decision is all or nothing per batch: the plan and merge kernels work with one row-tile height, and a
// batch split between the two large-row kernels, one launched behind the other, leaves the chip half empty twice
// (measured slower than either kernel alone on chunks of mixed lengths).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rpa_common.h"
#include "rpa_mfma.h"

namespace rpa {

// (AttnParams::wide_min_rows: the fewest query rows per KV head (tokens x group) per copied page, on the batch's average,
// from which the copies pay -- a page costs 3 bytes per element to copy, and saves about a quarter of the matrix time
// of every row tile that reads it.  Measured at 5 query heads per KV head: chunks of 384 tokens and more win in batches
// of one to sixteen chunks, chunks of 256 tokens only where the batch gives the 32x32-tile kernel, whose row tiles are
// twice as tall as the 8-bit kernel's and one to a CU, two workgroups per CU: wide_min_rows_full, wide_min_wgs.)

// wide[0] = 1 and wide[2 + i] = where block-table column 0 of sequence i would lie among the copied pages (its first
// copied page less its first visible column: below zero under a sliding window, whose earlier pages are not copied) if
// the large-row sequences' visible pages fit wide_cap and their rows are worth it; else wide[0] = 0.  One workgroup of
// 256 threads.
__global__ __launch_bounds__(256) void widen_decide_kernel(AttnParams p, int32_t* wide) {
  __shared__ int s_scan[256];
  __shared__ int s_carry;
  __shared__ unsigned long long s_work;
  __shared__ int s_tiles;
  const int tid = threadIdx.x;
  if (tid == 0) {
    s_carry = 0;
    s_work = 0ull;
    s_tiles = 0;
  }
  __syncthreads();
  const int n_live = live_rows(p);
  unsigned long long work = 0;
  int tiles = 0;
  bool fits = true;
  for (int i0 = 0; i0 < p.S; i0 += 256) {  // (uniform trip count)
    const int i = i0 + tid;
    int need = 0, col_lo = 0;
    if (i < n_live) {
      const SeqPlan sp = seq_plan(p, i);
      if (sp.live && !sp.small_rows) {
        col_lo = sp.lo / p.page_size;  // (sp.lo: the first key any row of the sequence sees, rounded down to 64)
        need = (sp.ctx + p.page_size - 1) / p.page_size - col_lo;
        const int readers = p.window > 0 ? min(sp.q_len, p.window + p.page_size) : sp.q_len;  // tokens that see a page, at most
        work += (unsigned long long)need * (unsigned)(readers * p.group);
        tiles += (sp.q_len * p.group + p.wide_rows - 1) / p.wide_rows;
      }
    }
    s_scan[tid] = need;
    __syncthreads();
    for (int o = 1; o < 256; o <<= 1) {  // inclusive scan
      const int v = tid >= o ? s_scan[tid - o] : 0;
      __syncthreads();
      s_scan[tid] += v;
      __syncthreads();
    }
    const int carry = s_carry;
    const long long first = (long long)carry + s_scan[tid] - need;
    if (i < p.S) wide[2 + i] = first + need <= p.wide_cap ? (int)first - col_lo : 0;
    if (first + need > p.wide_cap) fits = false;
    __syncthreads();
    if (tid == 255) s_carry = (int)min((long long)carry + s_scan[255], (long long)0x3fffffff);
    __syncthreads();
  }
  if (work) atomicAdd(&s_work, work);
  if (tiles) atomicAdd(&s_tiles, tiles);
  const int all_fit = __syncthreads_and(fits ? 1 : 0);
  if (tid == 0) {
    const int total = s_carry;
    const bool rows_high = s_work >= (unsigned long long)p.wide_min_rows * (unsigned)total;
    const bool rows_low = s_work >= (unsigned long long)p.wide_min_rows_full * (unsigned)total;
    const bool full = (long long)s_tiles * p.Hkv >= p.wide_min_wgs;
    // (under a window a row tile's key range is short, and the 32x32-tile kernel's start and end weigh more: measured, the
    //  copies win at a window of 4 096 on a full chip, and lose by 4-6 % at a window of 1 024 or on 320 workgroups)
    const bool pays = total > 0 && (p.window > 0 ? rows_high && full && p.window >= p.wide_min_window : rows_high || (rows_low && full));
    wide[0] = (all_fit && pays) ? 1 : 0;
    wide[1] = total;
  }
}

// Visible pages j = first visible + blockIdx.x, + gridDim.x, ... of sequence blockIdx.y: 16 codes per thread and turn.
template <int KVT>
__global__ __launch_bounds__(256) void widen_pages_kernel(AttnParams p) {
  if (!wide_mode(p)) return;
  const int i = blockIdx.y;
  if (i >= live_rows(p)) return;
  const SeqPlan sp = seq_plan(p, i);
  if (!sp.live || sp.small_rows) return;
  const int n_pages = (sp.ctx + p.page_size - 1) / p.page_size;
  const int first = p.wide[2 + i];
  const int CH = p.D / 16;              // 16-code pieces of a head's row
  const int per_tok = 2 * p.Hkv * CH;   // pieces of a token: K and V of every head
  const int64_t dst_tok = (int64_t)2 * p.Hkv * p.D * 2, dst_page = dst_tok * p.page_size;
  for (int j = sp.lo / p.page_size + blockIdx.x; j < n_pages; j += gridDim.x) {
    if (first + j < 0 || first + j >= p.wide_cap) return;  // (the decision kernel has made sure of this)
    const int page = min(max(p.block_tables[(int64_t)i * p.M + j], 0), p.P - 1);
    const int n_tok = min(p.page_size, sp.ctx - j * p.page_size);  // rows past the context are never read
    char* dst = (char*)p.wide_pages + (int64_t)(first + j) * dst_page;
    for (int u = threadIdx.x; u < n_tok * per_tok; u += 256) {
      const int tok = u / per_tok, rem = u - tok * per_tok;
      const int c = rem / CH, ch = rem - c * CH, h = c >> 1;
      const char* src = (const char*)((c & 1) ? p.v_pages : p.k_pages) + (int64_t)page * p.page_stride +
                        (int64_t)tok * p.token_stride + (int64_t)h * p.head_stride + ch * 16;
      const u32x4 w = *(const u32x4*)src;
      const u32x4 lo = codes8_to_bf16x8<KVT>(w[0], w[1]), hi = codes8_to_bf16x8<KVT>(w[2], w[3]);
      u32x4* d = (u32x4*)(dst + (int64_t)tok * dst_tok + (int64_t)c * p.D * 2 + ch * 32);
      d[0] = lo;
      d[1] = hi;
    }
  }
}

int launch_widen_decide(hipStream_t stream, const AttnParams& p) {
  hipLaunchKernelGGL(widen_decide_kernel, dim3(1), dim3(256), 0, stream, p, const_cast<int32_t*>(p.wide));
  return (int)hipGetLastError();
}

int launch_widen_pages(hipStream_t stream, const AttnParams& p) {
  if (p.D % 16 != 0) return (int)hipErrorInvalidValue;
  const dim3 grid(64, (unsigned)p.S);
  if (p.kv_dtype == RPA_FP8_E4M3) hipLaunchKernelGGL(widen_pages_kernel<RPA_FP8_E4M3>, grid, dim3(256), 0, stream, p);
  else if (p.kv_dtype == RPA_INT8) hipLaunchKernelGGL(widen_pages_kernel<RPA_INT8>, grid, dim3(256), 0, stream, p);
  else return (int)hipErrorInvalidValue;
  return (int)hipGetLastError();
}

}  // namespace rpa
