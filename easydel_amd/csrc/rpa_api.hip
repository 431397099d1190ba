// extern "C" surface of librpa_hip.so: argument checking, kernel selection, launches.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "../../include/rpa_hip_probe.h"
#include "rpa_common.h"
#include "rpa_mla.h"

namespace rpa {
int launch_scatter_slices(hipStream_t, const void*, const int32_t*, const int32_t*, void*, int, int, int64_t, int,
                          int64_t, int);
int launch_scatter_ragged(hipStream_t, const void*, const void*, void*, const int32_t*, const int32_t*,
                          const int32_t*, const int32_t*, int, int, int, int, int, int, int, int, int, int);
#ifdef RPA_PROBES
int launch_calibration_copy(hipStream_t, void*, const void*, size_t);
size_t launch_read_probe(hipStream_t, const void*, size_t, int, int, uint32_t*);
size_t launch_read_probe_paged(hipStream_t, const void*, size_t, int, int, int, int, uint32_t*);
double launch_mfma_probe(hipStream_t, int, int, int, int, int, unsigned long long*, float*);
long long launch_issue_probe(hipStream_t, int, int, int, int, unsigned long long*, float*, const void*);
#endif
int launch_scatter_ragged_quant(hipStream_t, const void*, const void*, void*, float*, const int32_t*, const int32_t*,
                                const int32_t*, const int32_t*, int, int, int, int, int, int, int, int, int, int, int);
}  // namespace rpa

namespace {

thread_local char g_err[512] = "";

// Test and measurement knobs (rpa_set_tunable, declared in rpa_hip_probe.h).  A build without -DRPA_PROBES knows the
// tuning knobs only: the two that change what a call computes with ("stages", which can make it skip a launch, and
// "force_generic") and the measurement kernels exist in the test / benchmark build alone.  They belong to the thread that sets
// them: a call sees the values of its own thread only, read once when it starts, so a thread that never calls
// rpa_set_tunable always runs with the defaults below, whatever a profiling or test thread of the same process does.
struct Tunables {
  int max_splits = 0;      // 0 = sized from the shapes
  int prefill_chunks = 0;  // 0 = chunk length chosen on the device per batch; n = at most n chunks of a fixed length
  int decode_sync = 8;     // workgroup barrier every this many decode tiles (power of two, 0 = never)
  int decode_wgs = 0;      // 0 = as many persistent workgroups as are resident at once
  int force_generic = 0;
  int prefill_dma = 1;
  int prefill_x32 = 1;     // 1: the 32x32-tile prefill kernel serves the shapes it is built for
  int prefill_wide = 1;    // 8-bit pages reach that kernel through bf16 copies where the workspace has room and the batch's rows pay for
                           // them: 0 never, 1 at the default bars (kWideMinRows rows per copied page, kWideMinRowsFull in a batch
                           // of two workgroups per CU), n > 1 at a bar of n rows
  int decode_pace = 1;
  int decode_dma = -1;     // -1: where it measured faster (head size 256; int8 pages); 0: never; 1: wherever it applies; 2: same, one tile ahead; 3: same, K with V
  int mla_chunks = 0;      // 0 = sized from the shapes
  int mla_min_chunk = 0;   // 0 = default
  int stages = 15;         // bit 0: decode plan, 1: decode kernel, 2: prefill / large-row kernel, 3: merge
};
thread_local Tunables g_tun;

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(int err, const char* what) {
  if (err == 0) return 0;
  return fail(err, "%s: %s", what, hipGetErrorString((hipError_t)err));
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// Split-K partial storage per split: outputs [T][Hq][D] f32, then (max, sum) [T][Hq][2] f32.
size_t part_o_bytes(int T, int Hq, int D) { return align256((size_t)T * Hq * D * 4); }
size_t part_ml_bytes(int T, int Hq) { return align256((size_t)T * Hq * 2 * 4); }

// Partial slots per sequence the workspace is sized for: enough to spread one maximal sequence over
// 256-token pieces, capped so the partial buffers stay within ~1 GiB, never fewer than 2.  (Too few slots force
// long spans on every workgroup, so that one long sequence in a batch of short ones leaves most of the chip idle:
// with a 256 MiB cap a 100k-token sequence among 255 short ones ran on 40 % of the workgroups.)
int static_splits(int T, int M, int page_size, int Hq, int D) {
  const int forced = g_tun.max_splits;
  if (forced > 0) return forced < 2 ? 2 : forced;
  long want = ((long)M * page_size + 255) / 256 + 1;
  const size_t per = part_o_bytes(T, Hq, D) + part_ml_bytes(T, Hq);
  long cap = (long)(((size_t)1 << 30) / per);
  if (cap > rpa::kMaxSplitsCap) cap = rpa::kMaxSplitsCap;
  if (want > cap) want = cap;
  if (want < 2) want = 2;
  return (int)want;
}

// Prefill split-K: keys per chunk and number of chunks the partial buffers hold, from the static bounds.
// A row tile's key range is cut into at most kMaxPrefillChunks chunks of at least 8192 keys; the partial
// buffers ([chunks][T][Hq][D+2] floats) are kept under ~1 GiB by allowing fewer, longer chunks.
// Compute units of the current device (256 on MI355X); 0 if the query fails.
int device_cus() {
  static std::atomic<int> cached[rpa::kMaxDevices];  // per device; 0 = not looked up yet (a racing first call stores the same value)
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= rpa::kMaxDevices) return 0;
  const int v = cached[dev].load(std::memory_order_relaxed);
  if (v > 0) return v;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cus = 0;
  cached[dev].store(cus, std::memory_order_relaxed);
  return cus;
}

// How many chunks a prefill row tile's key range may be cut into (each a workgroup of its own, merged afterwards),
// and, when the caller fixed that number, the keys of one chunk.  Cutting pays when a batch holds few row tiles (a
// couple of long prompts): it fills the chip and evens out the workgroups' lengths.  It costs a float32 partial per
// chunk and row, written and read back by the merge, so a batch whose bounds already allow many times more row tiles
// than workgroups fit on the chip is not cut at all.  Otherwise this only sizes the partial buffers: the plan kernel
// picks the chunk length from the lengths of the batch it finds on the device.
void prefill_split(int T, int S, int M, int page_size, int Hq, int Hkv, int D, int* chunk_keys, int* max_chunks) {
  // (the row-tile bound below is taken with the smaller of the two row-tile heights: it only sizes buffers)
  const long span = (long)M * page_size;
  int chunks = g_tun.prefill_chunks > 0 ? g_tun.prefill_chunks : rpa::kMaxPrefillChunks;
  if (chunks > rpa::kMaxPrefillChunks) chunks = rpa::kMaxPrefillChunks;
  if (g_tun.prefill_chunks <= 0 && Hkv > 0) {
    const long row_tiles = ((long)T * (Hq / Hkv) / rpa::kPrefillRows + S) * Hkv;  // the prefill grid's bound without cutting
    const int cus = device_cus();
    if (cus > 0 && row_tiles >= 8L * cus) chunks = 1;  // eight units per CU even out by themselves
  }
  const size_t per = part_o_bytes(T, Hq, D) + part_ml_bytes(T, Hq);
  while (chunks > 1 && (size_t)chunks * per > ((size_t)1 << 30)) --chunks;
  long keys = (span + chunks - 1) / chunks;
  const long min_keys = g_tun.prefill_chunks > 0 ? 8192 : rpa::kMinPrefillChunk;
  if (keys < min_keys) keys = min_keys;
  keys = (keys + 63) & ~63L;
  chunks = (int)((span + keys - 1) / keys);
  if (chunks < 1) chunks = 1;
  *chunk_keys = (int)keys;
  *max_chunks = chunks;
}

size_t plan_bytes(int S) { return align256(((size_t)rpa::kPlanHeader + 2 * ((size_t)S + 1) + rpa::kMaxDecodeWgs + 2 * rpa::kMaxSortedSeqs + 1) * 4); }

// Static bound on query tokens the decode kernel can own: sequences with at most dec_rows rows per KV head.
int decode_token_bound(int T, int S, int Hq, int Hkv, int dec_rows) {
  const int group = Hq / Hkv;
  if (group > dec_rows) return 1;
  const long bound = (long)S * (dec_rows / group);
  return (int)(bound < T ? bound : T);
}

// MLA: how many key chunks a row tile may be cut into, and the shortest chunk.  Cutting fills the chip when the batch
// holds few row tiles and evens out sequences of different lengths; every chunk of a row costs a float32 partial
// row (lkv + 2 floats) written and read back, which with many heads per token is comparable to the keys themselves,
// hence the longer minimum there.  The partial buffers stay under ~1 GiB.
void mla_split(int T, int S, int Hq, int lkv, int* max_chunks, int* rule_chunks, int* min_chunk) {
  // Row tiles a batch of this shape typically holds (a bound it is not: a call may put all its tokens into one row).
  // About 400 units of work, 1.5 per CU, measured best on decode batches of 32 ... 1 024 sequences at 16 and at 128
  // heads: fewer leave CUs idle or the lengths uneven, more pay for their partial rows and their start.
  const long tiles = std::max((long)S, (long)T * Hq / rpa::kMlaRows);
  long rule = g_tun.mla_chunks > 0 ? g_tun.mla_chunks : (400 + tiles / 2) / tiles;
  if (rule > rpa::kMlaMaxChunks) rule = rpa::kMlaMaxChunks;
  if (rule < 1) rule = 1;
  // The partial buffers hold more chunks than that where they are cheap (up to 256 MiB in all), for the batches the
  // plan kernel cuts by length: a call of few tokens whose sequence rows are mostly empty (its row tiles number at
  // least T * Hq / 128, and a quarter of the CUs at most for that cut).  A set knob is taken literally.
  const size_t per = part_o_bytes(T, Hq, lkv) + part_ml_bytes(T, Hq);
  long chunks = rule;
  if (g_tun.mla_chunks <= 0 && (long)T * Hq / rpa::kMlaRows <= std::max(device_cus(), 4) / 4)
    chunks = std::max(rule, std::min((long)rpa::kMlaMaxChunks, (long)(((size_t)256 << 20) / std::max(per, (size_t)1))));
  while (chunks > 1 && (size_t)chunks * per > ((size_t)1 << 30)) --chunks;
  *max_chunks = (int)chunks;
  *rule_chunks = (int)std::min(rule, chunks);
  *min_chunk = g_tun.mla_min_chunk > 0 ? g_tun.mla_min_chunk : (Hq >= 64 ? 1024 : 512);
}

}  // namespace

extern "C" {

const char* rpa_version(void) { return "0.1.0"; }

const char* rpa_last_error(void) { return g_err; }

int rpa_set_tunable(const char* name, int value) {
  if (!name) return -1;
  auto swap = [](int& slot, int v) { const int old = slot; slot = v; return old; };
  if (!strcmp(name, "max_splits")) {
    if (value < 0) value = 0;
    if (value > rpa::kMaxSplitsCap) value = rpa::kMaxSplitsCap;
    return swap(g_tun.max_splits, value);
  }
  if (!strcmp(name, "prefill_chunks")) return swap(g_tun.prefill_chunks, value < 0 ? 0 : value);
  if (!strcmp(name, "decode_sync")) {
    int pow2 = 0;
    if (value > 0) for (pow2 = 1; pow2 * 2 <= value && pow2 < 1024; pow2 *= 2) {}
    return swap(g_tun.decode_sync, pow2);
  }
  if (!strcmp(name, "decode_wgs")) return swap(g_tun.decode_wgs, value < 0 ? 0 : value);
#ifdef RPA_PROBES
  if (!strcmp(name, "force_generic")) return swap(g_tun.force_generic, value != 0);
  if (!strcmp(name, "stages")) return swap(g_tun.stages, value & 15);
#endif
  if (!strcmp(name, "prefill_dma")) return swap(g_tun.prefill_dma, value != 0);
  if (!strcmp(name, "prefill_x32")) return swap(g_tun.prefill_x32, value != 0);
  if (!strcmp(name, "prefill_wide")) return swap(g_tun.prefill_wide, value < 0 ? 0 : value);
  if (!strcmp(name, "decode_pace")) return swap(g_tun.decode_pace, value != 0);
  if (!strcmp(name, "decode_dma")) return swap(g_tun.decode_dma, value < 0 ? -1 : value > 3 ? 3 : value);
  if (!strcmp(name, "mla_min_chunk")) return swap(g_tun.mla_min_chunk, value <= 0 ? 0 : ((value + 63) & ~63));
  if (!strcmp(name, "mla_chunks")) return swap(g_tun.mla_chunks, value < 0 ? 0 : (value > rpa::kMlaMaxChunks ? rpa::kMlaMaxChunks : value));
  return -1;
}

#ifdef RPA_PROBES
int rpa_calibration_copy(rpa_stream_t stream, void* dst, const void* src, size_t bytes) {
  if (!dst || !src || (bytes & 15) || ((uintptr_t)dst & 15) || ((uintptr_t)src & 15))
    return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_calibration_copy: pointers and size must be 16-byte aligned");
  if (bytes == 0) return RPA_OK;
  return hip_fail(rpa::launch_calibration_copy((hipStream_t)stream, dst, src, bytes), "rpa_calibration_copy launch");
}

size_t rpa_read_probe(rpa_stream_t stream, const void* src, size_t bytes, int workgroups, int kib_in_flight_per_wave,
                      void* sink) {
  if (!src || !sink || ((uintptr_t)src & 15) || ((uintptr_t)sink & 3)) {
    fail(RPA_ERR_INVALID_ARGUMENT, "rpa_read_probe: src must be 16-byte aligned and sink a 4-byte device word");
    return 0;
  }
  const size_t read = rpa::launch_read_probe((hipStream_t)stream, src, bytes, workgroups, kib_in_flight_per_wave, (uint32_t*)sink);
  if (read == 0)
    fail(RPA_ERR_INVALID_ARGUMENT, "rpa_read_probe: workgroups > 0, 2 / 4 / 8 / 16 / 32 KiB in flight per wave, and at least one round of loads per wave");
  return read;
}

size_t rpa_read_probe_paged(rpa_stream_t stream, const void* src, size_t bytes, int workgroups, int kib_in_flight_per_wave,
                            int chunk_kib, int split, void* sink) {
  if (!src || !sink || ((uintptr_t)src & 15) || ((uintptr_t)sink & 3)) {
    fail(RPA_ERR_INVALID_ARGUMENT, "rpa_read_probe_paged: src must be 16-byte aligned and sink a 4-byte device word");
    return 0;
  }
  const size_t read = rpa::launch_read_probe_paged((hipStream_t)stream, src, bytes, workgroups, kib_in_flight_per_wave, chunk_kib,
                                                   split, (uint32_t*)sink);
  if (read == 0)
    fail(RPA_ERR_INVALID_ARGUMENT, "rpa_read_probe_paged: workgroups > 0, chunk_kib a multiple of 8, 2 / 4 / 8 / 16 / 32 KiB in flight per wave "
                                   "and a multiple of chunk_kib / 8, split 0..2, and at least one group of chunks per workgroup");
  return read;
}

double rpa_mfma_probe(rpa_stream_t stream, int shape, int source, int mfmas_per_operand, int waves_per_simd, int iters,
                      void* clocks, void* sink) {
  if (!clocks || !sink || ((uintptr_t)clocks & 7) || ((uintptr_t)sink & 3)) {
    fail(RPA_ERR_INVALID_ARGUMENT, "rpa_mfma_probe: clocks must be two 8-byte device words, sink a 4-byte device word");
    return 0.0;
  }
  const double flops = rpa::launch_mfma_probe((hipStream_t)stream, shape, source, mfmas_per_operand, waves_per_simd, iters,
                                              (unsigned long long*)clocks, (float*)sink);
  if (flops == 0.0)
    fail(RPA_ERR_INVALID_ARGUMENT, "rpa_mfma_probe: shape 0 / 1, source 0..2, 1 / 2 / 4 MFMAs per operand, 1 or 2 waves per SIMD, iters > 0");
  return flops;
}

long long rpa_issue_probe(rpa_stream_t stream, int kind, int extra, int fill, int iters, void* clocks, void* sink, const void* src) {
  if (!clocks || !sink || !src || ((uintptr_t)clocks & 7) || ((uintptr_t)sink & 3) || ((uintptr_t)src & 15)) {
    fail(RPA_ERR_INVALID_ARGUMENT, "rpa_issue_probe: clocks must be two 8-byte device words, sink a 4-byte device word, src 1 MiB of 16-byte aligned device memory");
    return 0;
  }
  const long long n = rpa::launch_issue_probe((hipStream_t)stream, kind, extra, fill, iters, (unsigned long long*)clocks, (float*)sink, src);
  if (n == 0) fail(RPA_ERR_INVALID_ARGUMENT, "rpa_issue_probe: kind 0..9, extra 0 / 1 / 2 / 4, fill 0 or 6, iters > 0");
  return n;
}
#endif  // RPA_PROBES

int rpa_page_scatter_slices(rpa_stream_t stream, const void* new_kv, const int32_t* slice_indices,
                            const int32_t* num_slices, void* kv_pages, int T, int N, int64_t num_positions,
                            int page_size, int64_t row_bytes, int page_shard_index) {
  if (T < 0 || N < 0 || num_positions < 0 || page_size <= 0 || row_bytes <= 0 || page_shard_index < 0)
    return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_page_scatter_slices: bad size (T=%d N=%d positions=%lld page_size=%d row_bytes=%lld shard=%d)",
                T, N, (long long)num_positions, page_size, (long long)row_bytes, page_shard_index);
  if (T == 0 || N == 0 || num_positions == 0) return RPA_OK;  // nothing to move (the reference returns the cache unchanged)
  if (!new_kv || !slice_indices || !num_slices || !kv_pages)
    return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_page_scatter_slices: null pointer");
  return hip_fail(rpa::launch_scatter_slices((hipStream_t)stream, new_kv, slice_indices, num_slices, kv_pages, T, N,
                                             num_positions, page_size, row_bytes, page_shard_index),
                  "rpa_page_scatter_slices launch");
}

// Stored row width of a combined head: Dp >= D elements (the reference pads head sizes that are not 64 or a multiple of
// 128 up to the next multiple of 128, easydel/caching/ragged_page/cache.py:640-647); rows must keep 4-byte alignment.
static int check_row_width(const char* who, int D, int Dp, int elem) {
  if (Dp < D) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: stored head width Dp=%d < head_dim D=%d", who, Dp, D);
  if (((int64_t)Dp * elem) % 4 != 0 || ((int64_t)D * elem) % 4 != 0)
    return fail(RPA_ERR_UNSUPPORTED, "%s: head rows of D=%d / Dp=%d elements of %d bytes are not 4-byte multiples", who, D, Dp, elem);
  return RPA_OK;
}

int rpa_page_scatter_ragged(rpa_stream_t stream, const void* key, const void* value, void* kv_pages,
                            const int32_t* context_lens, const int32_t* block_tables,
                            const int32_t* query_start_loc, const int32_t* num_seqs, int T, int S, int M, int P,
                            int page_size, int Hkv, int D, int Dp, int C, int elem_bytes) {
  if (T < 0 || S <= 0 || M <= 0 || P <= 0 || page_size <= 0 || Hkv <= 0 || D <= 0 || C < 2 * Hkv ||
      (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4))
    return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_page_scatter_ragged: bad size (T=%d S=%d M=%d P=%d page_size=%d Hkv=%d D=%d C=%d elem=%d)",
                T, S, M, P, page_size, Hkv, D, C, elem_bytes);
  if (const int rc = check_row_width("rpa_page_scatter_ragged", D, Dp, elem_bytes)) return rc;
  if (T == 0) return RPA_OK;
  if (!key || !value || !kv_pages || !context_lens || !block_tables || !query_start_loc || !num_seqs)
    return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_page_scatter_ragged: null pointer");
  return hip_fail(rpa::launch_scatter_ragged((hipStream_t)stream, key, value, kv_pages, context_lens, block_tables,
                                             query_start_loc, num_seqs, T, S, M, P, page_size, Hkv, D, C, Dp, elem_bytes),
                  "rpa_page_scatter_ragged launch");
}

int rpa_page_scatter_ragged_quantised(rpa_stream_t stream, const void* key, const void* value, void* kv_pages,
                                      float* kv_scales, const int32_t* context_lens, const int32_t* block_tables,
                                      const int32_t* query_start_loc, const int32_t* num_seqs, int T, int S, int M, int P,
                                      int page_size, int Hkv, int D, int Dp, int C, int src_dtype, int kv_dtype) {
  if (T < 0 || S <= 0 || M <= 0 || P <= 0 || page_size <= 0 || Hkv <= 0 || D <= 0 || C < 2 * Hkv)
    return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_page_scatter_ragged_quantised: bad size (T=%d S=%d M=%d P=%d page_size=%d Hkv=%d D=%d C=%d)",
                T, S, M, P, page_size, Hkv, D, C);
  if (D % 4 != 0 || Dp % 4 != 0) return fail(RPA_ERR_UNSUPPORTED, "rpa_page_scatter_ragged_quantised: head_dim %d / stored width %d is not a multiple of 4", D, Dp);
  if (Dp < D) return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_page_scatter_ragged_quantised: stored head width Dp=%d < head_dim D=%d", Dp, D);
  if (src_dtype != RPA_F32 && src_dtype != RPA_BF16)
    return fail(RPA_ERR_UNSUPPORTED, "rpa_page_scatter_ragged_quantised: source dtype %d (want f32 or bf16)", src_dtype);
  if (kv_dtype != RPA_FP8_E4M3 && kv_dtype != RPA_INT8)
    return fail(RPA_ERR_UNSUPPORTED, "rpa_page_scatter_ragged_quantised: page dtype %d (want fp8-e4m3 or int8)", kv_dtype);
  if (T == 0) return RPA_OK;
  if (!key || !value || !kv_pages || !kv_scales || !context_lens || !block_tables || !query_start_loc || !num_seqs)
    return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_page_scatter_ragged_quantised: null pointer");
  if ((((uintptr_t)key) | ((uintptr_t)value)) & 15 || ((uintptr_t)kv_pages & 3))
    return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_page_scatter_ragged_quantised: key/value must be 16-byte and kv_pages 4-byte aligned");
  return hip_fail(rpa::launch_scatter_ragged_quant((hipStream_t)stream, key, value, kv_pages, kv_scales, context_lens,
                                                   block_tables, query_start_loc, num_seqs, T, S, M, P, page_size, Hkv, D, C, Dp,
                                                   src_dtype, kv_dtype),
                  "rpa_page_scatter_ragged_quantised launch");
}

// bf16 copies of 8-bit pages for the 32x32-tile prefill kernel (rpa_widen.hip): the pages the workspace is asked to
// hold, from the static bounds -- a large-row sequence has more than dec_rows query rows per KV head, so there are at
// most T group / (dec_rows + 1) of them, each with at most M pages -- capped at 4 GiB; 0 where the shapes rule the
// copies out (other head sizes, pages that are not a multiple of 64 tokens, too few rows to pay for a copy).
constexpr int64_t kWideMaxBytes = (int64_t)4 << 30;
// the decision kernel's default bars, in query rows per KV head and copied page on the batch's average: any batch, and a
// batch of two workgroups of the 32x32-tile kernel per CU or more
constexpr int kWideMinRows = 1792, kWideMinRowsFull = 1024;
static int wide_min_rows(int tunable) { return tunable > 1 ? tunable : kWideMinRowsFull; }  // the lower of the two
static int64_t wide_page_bytes(int page_size, int Hkv, int D) { return (int64_t)page_size * 2 * Hkv * D * 2; }
static int64_t wide_header_bytes(int S) { return (((int64_t)(2 + S) * 4) + 255) & ~(int64_t)255; }
static int64_t wide_pages_wanted(int T, int S, int M, int page_size, int Hq, int Hkv, int D, int kv_dtype, int dec_rows, int min_rows) {
  if (kv_dtype != RPA_FP8_E4M3 && kv_dtype != RPA_INT8) return 0;
  if ((D != 128 && D != 256) || page_size % 64 != 0 || S > 65535) return 0;
  const int64_t rows = (int64_t)T * (Hq / Hkv);
  // No batch of fewer rows (T x group) in all is served from copies: the upper bar is an average, so some sequence
  // reaches it; the lower bar counts only with two workgroups of 128 or 256 rows per CU, many times as many rows.
  if (rows < min_rows) return 0;
  const int64_t seqs = std::min<int64_t>(S, rows / (dec_rows + 1));
  return std::min<int64_t>(seqs * M, kWideMaxBytes / wide_page_bytes(page_size, Hkv, D));
}

size_t rpa_attention_workspace_bytes(int T, int S, int M, int page_size, int Hq, int Hkv, int D, int q_dtype,
                                     int kv_dtype) {
  (void)q_dtype;
  if (T <= 0 || S <= 0 || M <= 0 || page_size <= 0 || Hq <= 0 || D <= 0) return 256;
  if (Hkv <= 0 || Hq % Hkv != 0) return 256;
  const int td = decode_token_bound(T, S, Hq, Hkv, rpa::decode_row_limit(T, S, D, kv_dtype));
  const int splits = static_splits(td, M, page_size, Hq, D);
  int pre_keys, pre_chunks;
  prefill_split(T, S, M, page_size, Hq, Hkv, D, &pre_keys, &pre_chunks);
  const size_t pre = pre_chunks > 1 ? (size_t)pre_chunks * (part_o_bytes(T, Hq, D) + part_ml_bytes(T, Hq)) : 0;
  size_t wide = 0;
  if (g_tun.prefill_wide && g_tun.prefill_dma && g_tun.prefill_x32) {
    const int64_t pages = wide_pages_wanted(T, S, M, page_size, Hq, Hkv, D, kv_dtype, rpa::decode_row_limit(T, S, D, kv_dtype),
                                            g_tun.prefill_wide > 1 ? g_tun.prefill_wide : kWideMinRows);
    if (pages > 0) wide = (size_t)(wide_header_bytes(S) + pages * wide_page_bytes(page_size, Hkv, D) + 256);
  }
  return (size_t)splits * (part_o_bytes(td, Hq, D) + part_ml_bytes(td, Hq)) + pre + plan_bytes(S) + 256 + wide;
}

// Shared body of the attention entry points.  k_pages / v_pages and the strides describe where K and V of
// (page, token, KV head) lie (sizes are validated here, so the callers' stride arithmetic may see nonsense and
// must not act on it); Dp is the stored row width of a head (>= D), C the row length of kv_scales; num_seqs may be null
// (every row live) if the caller allows.  The workspace is laid out here from the bytes the caller hands over: the
// partial slots and key chunks shrink to what fits (never below two slots, else RPA_ERR_WORKSPACE), so the launch
// never writes past workspace_bytes whatever sizing call preceded it.
static int attention_impl(const char* who, rpa_stream_t stream, const void* q, const void* k_pages, const void* v_pages,
                          int64_t token_stride, int64_t head_stride, const float* kv_scales,
                          const int32_t* context_lens, const int32_t* block_tables, const int32_t* query_start_loc,
                          const int32_t* num_seqs, bool num_seqs_optional, void* out, void* workspace,
                          size_t workspace_bytes, int T, int S, int M, int P, int page_size, int Hq, int Hkv, int D, int Dp,
                          int C, int q_dtype, int kv_dtype, float softmax_scale, int sliding_window, float logits_soft_cap,
                          const float* softmax_aux, const void* new_key = nullptr, const void* new_value = nullptr) {
  if (T < 0 || S <= 0 || M <= 0 || P <= 0 || page_size <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: bad size (T=%d S=%d M=%d P=%d page_size=%d Hq=%d Hkv=%d D=%d)", who,
                T, S, M, P, page_size, Hq, Hkv, D);
  if (Hq % Hkv != 0) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: Hq=%d is not a multiple of Hkv=%d", who, Hq, Hkv);
  if (q_dtype != RPA_F32 && q_dtype != RPA_BF16 && q_dtype != RPA_F16)
    return fail(RPA_ERR_UNSUPPORTED, "%s: q_dtype %d (want f32, bf16 or f16)", who, q_dtype);
  if (kv_dtype < RPA_F32 || kv_dtype > RPA_F16) return fail(RPA_ERR_UNSUPPORTED, "%s: kv_dtype %d", who, kv_dtype);
  if (D > 256 || D % 4 != 0) return fail(RPA_ERR_UNSUPPORTED, "%s: head_dim %d (want a multiple of 4, <= 256)", who, D);
  if (const int rc = check_row_width(who, D, Dp, rpa::elem_bytes(kv_dtype))) return rc;
  if (kv_scales && kv_dtype != RPA_FP8_E4M3 && kv_dtype != RPA_INT8)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: kv_scales with pages that are not 8-bit (kv_dtype %d)", who, kv_dtype);
  if (kv_scales && ((uintptr_t)kv_scales & 7))
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: kv_scales must be 8-byte aligned", who);
  // Pages of bare codes exist for fp8 only (the reference's cast-only cache, ragged_page_attention.py:570-580); int8
  // codes mean nothing without their scales.
  if (!kv_scales && kv_dtype == RPA_INT8)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: int8 KV pages need kv_scales (only fp8 pages may be unscaled)", who);
  // The decode plan counts the keys of a batch in 32-bit integers (spans of the flattened key stream); pages shared
  // between sequences let that sum exceed the pool, so the bound is on what the block tables can address.
  if ((int64_t)S * M * page_size >= ((int64_t)1 << 31))
    return fail(RPA_ERR_UNSUPPORTED, "%s: S * M * page_size = %lld tokens addressable by the block tables, the limit is 2^31 - 1 per call",
                who, (long long)((int64_t)S * M * page_size));
  if (!std::isfinite(softmax_scale)) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: softmax_scale is not finite", who);
  if (softmax_aux && ((uintptr_t)softmax_aux & 3))
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: softmax_aux must be 4-byte aligned", who);
  if (T == 0) return RPA_OK;
  if (!q || !k_pages || !v_pages || !context_lens || !block_tables || !query_start_loc || (!num_seqs && !num_seqs_optional) || !out)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if ((((uintptr_t)q) | ((uintptr_t)out) | ((uintptr_t)k_pages) | ((uintptr_t)v_pages)) & 15)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: q, out and the page pools must be 16-byte aligned", who);

  const Tunables tun = g_tun;  // this thread's knobs, read once per call
  rpa::AttnParams p;
  memset(&p, 0, sizeof(p));
  p.q = q; p.k_pages = k_pages; p.v_pages = v_pages; p.kv_scales = kv_scales; p.sinks = softmax_aux;
  p.context_lens = context_lens; p.block_tables = block_tables; p.qsl = query_start_loc; p.num_seqs = num_seqs;
  p.out = out;
  p.T = T; p.S = S; p.M = M; p.P = P; p.page_size = page_size; p.Hq = Hq; p.Hkv = Hkv; p.group = Hq / Hkv; p.C = C;
  p.D = D; p.Dq = D;
  p.kv_pad_bytes = (Dp - D) * rpa::elem_bytes(kv_dtype);
  p.token_stride = token_stride;
  p.head_stride = head_stride;
  p.page_stride = p.token_stride * page_size;
  p.q_dtype = q_dtype; p.kv_dtype = kv_dtype;
  p.scale = softmax_scale;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  p.window = sliding_window > 0 ? sliding_window : 0;
  p.softcap = logits_soft_cap > 0.f ? logits_soft_cap : 0.f;
  p.decode_wgs = tun.decode_wgs;
  p.decode_sync = tun.decode_sync;
  p.prefill_dma = tun.prefill_dma;
  p.pre_rows = rpa::kPrefillRows;
  p.pre_x32 = 0;
  p.decode_pace = tun.decode_pace;
  p.decode_dma = tun.decode_dma < 0 ? ((p.D == 256 || p.kv_dtype == RPA_INT8) ? 1 : 0) : tun.decode_dma;
  p.max_splits = 2;
  p.pre_chunk = 1 << 30;
  p.pre_max_chunks = 1;
  // Padded head storage (Dp = 128 or 256 > D): the MFMA kernels compute with the stored width -- q rows are padded with
  // zeros in registers, the pages' padding holds zeros (the write puts them there), output dims past D are not stored.
  if (Dp > D && (Dp == 128 || Dp == 256)) p.D = Dp;
  p.dec_rows = rpa::decode_row_limit(T, S, p.D, kv_dtype);
  p.mfma_path = (!tun.force_generic && rpa::decode_supported(p)) ? 1 : 0;
  if (!p.mfma_path) p.D = D;

  hipStream_t s = (hipStream_t)stream;
  const int stages = tun.stages;
  if (new_key) {  // fused write + attention: the new rows go into the pages before any kernel reads them
    if (p.mfma_path && (stages & 1)) {
      p.new_k = new_key;  // copied by extra blocks of the decode plan kernel's launch
      p.new_v = new_value;
    } else {
      const int err = rpa::launch_scatter_ragged(s, new_key, new_value, const_cast<void*>(k_pages), context_lens, block_tables,
                                                 query_start_loc, num_seqs, T, S, M, P, page_size, Hkv, D, C, Dp, rpa::elem_bytes(kv_dtype));
      if (err) return hip_fail(err, "page scatter launch");
    }
  }
  if (p.mfma_path) {
    const int Dc = p.D;  // head size the partial rows are laid out with
    const int td = decode_token_bound(T, S, Hq, Hkv, p.dec_rows);
    p.t_dec_max = td;
    const size_t po = part_o_bytes(td, Hq, Dc), pml = part_ml_bytes(td, Hq), pb = plan_bytes(S);
    int splits = static_splits(td, M, page_size, Hq, Dc);
    int pre_keys, pre_chunks;
    prefill_split(T, S, M, page_size, Hq, Hkv, Dc, &pre_keys, &pre_chunks);
    const size_t pre_po = part_o_bytes(T, Hq, Dc), pre_pml = part_ml_bytes(T, Hq);
    size_t pre = pre_chunks > 1 ? (size_t)pre_chunks * (pre_po + pre_pml) : 0;
    size_t usable = workspace_bytes > 256 + pb ? workspace_bytes - 256 - pb : 0;
    if (!workspace || usable < 2 * (po + pml))
      return fail(RPA_ERR_WORKSPACE, "%s: workspace %zu bytes < %zu needed for two partial slots", who,
                  workspace_bytes, 2 * (po + pml) + pb + 256);
    if (usable < pre + 2 * (po + pml)) {  // a small workspace: prefill rows are split into fewer chunks, or not at all
      pre_chunks = (int)((usable - 2 * (po + pml)) / (pre_po + pre_pml));
      if (pre_chunks < 2) pre_chunks = 1;
      pre = pre_chunks > 1 ? (size_t)pre_chunks * (pre_po + pre_pml) : 0;
    }
    usable -= pre;
    if ((size_t)splits * (po + pml) > usable) splits = (int)(usable / (po + pml));
    p.max_splits = splits;
    p.pre_chunk = pre_keys;
    p.pre_max_chunks = pre_chunks;
    p.pre_auto = tun.prefill_chunks <= 0 ? 1 : 0;
    p.pre_slots = device_cus() * (Dc <= 128 ? 2 : 1);  // resident workgroups of the large-row kernels
    if (tun.prefill_dma && tun.prefill_x32 && rpa::prefill_x32_rows(p) > 0) {  // one workgroup per CU
      p.pre_x32 = 1;
      p.pre_rows = rpa::prefill_x32_rows(p);
      p.pre_slots = device_cus();
    }
    char* base = (char*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    p.plan = (int32_t*)base;
    p.part_o = (float*)(base + pb);
    p.part_ml = (float*)(base + pb + (size_t)splits * po);
    char* pre_base = base + pb + (size_t)splits * (po + pml);
    p.pre_o = (float*)pre_base;
    p.pre_ml = (float*)(pre_base + (size_t)pre_chunks * pre_po);
    // 8-bit pages: what the workspace holds beyond the partial rows takes bf16 copies of the large-row sequences' pages,
    // and the 32x32-tile kernel reads those where the decision kernel finds that they fit and pay (rpa_widen.hip).
    rpa::AttnParams pw;
    bool wide = false;
    if (tun.prefill_wide && tun.prefill_dma && tun.prefill_x32 && (p.D == 256 || (p.D == 128 && !(p.softcap > 0.f))) &&
        p.kv_pad_bytes == 0 && rpa::prefill_dma8_supported(p)) {
      p.wide_min_rows = tun.prefill_wide > 1 ? tun.prefill_wide : kWideMinRows;
      p.wide_min_rows_full = wide_min_rows(tun.prefill_wide);
      p.wide_min_wgs = tun.prefill_wide > 1 ? 0 : 2 * device_cus();
      p.wide_min_window = tun.prefill_wide > 1 ? 0 : 2048;
      const int64_t want = wide_pages_wanted(T, S, M, page_size, Hq, Hkv, p.D, kv_dtype, p.dec_rows, p.wide_min_rows);
      char* after = pre_base + pre;
      char* hdr = (char*)(((uintptr_t)after + 255) & ~(uintptr_t)255);
      char* pages0 = hdr + wide_header_bytes(S);
      char* end = (char*)workspace + workspace_bytes;
      const int64_t room = end > pages0 ? (int64_t)(end - pages0) / wide_page_bytes(page_size, Hkv, p.D) : 0;
      const int64_t cap = std::min(want, room);
      if (cap >= 1) {
        p.wide = (const int32_t*)hdr;
        p.wide_pages = pages0;
        p.wide_cap = (int)cap;
        p.wide_rows = p.D == 128 ? 256 : 128;  // the 32x32-tile kernel's row tiles at this head size
        p.wide_slots = device_cus();
        p.src_P = P;
        pw = p;
        pw.k_pages = pages0;
        pw.v_pages = pages0 + (size_t)p.D * 2;
        pw.head_stride = (int64_t)2 * p.D * 2;
        pw.token_stride = (int64_t)2 * Hkv * p.D * 2;
        pw.page_stride = pw.token_stride * page_size;
        pw.kv_dtype = RPA_BF16;
        pw.P = (int)cap;
        pw.pre_x32 = 1;
        pw.pre_rows = p.wide_rows;
        pw.pre_slots = p.wide_slots;
        wide = rpa::prefill_x32_rows(pw) == p.wide_rows;
        if (!wide) p.wide = nullptr;
      }
    }
    int err = 0;
    if (wide) err = rpa::launch_widen_decide(s, p);
    if (err) return hip_fail(err, "page-copy decision kernel launch");
    if (stages & 3) err = rpa::launch_attn_decode(s, p, stages & 3);
    if (err) return hip_fail(err, "decode kernel launch");
    // Rows too large for the decode kernel: MFMA prefill kernel where it applies, fp32 kernel otherwise.  No launch where
    // the call's bounds rule such rows out (all its tokens together make no more rows per KV head than the decode kernel takes).
    const bool large_rows_possible = (int64_t)T * p.group > p.dec_rows;
    if ((stages & 4) && large_rows_possible) err = rpa::prefill_supported(p) ? rpa::launch_attn_prefill(s, p) : rpa::launch_attn_generic(s, p);
    if (err) return hip_fail(err, "prefill kernel launch");
    if (wide && (stages & 4)) {  // (either this pair or the launch above finds work: the decision is the batch's)
      err = rpa::launch_widen_pages(s, p);
      if (err) return hip_fail(err, "page-copy kernel launch");
      err = rpa::launch_attn_prefill_x32(s, pw);
      if (err) return hip_fail(err, "prefill kernel launch (copied pages)");
    }
  } else {
    int err = (stages & 4) ? rpa::launch_attn_generic(s, p) : 0;
    if (err) return hip_fail(err, "fp32 kernel launch");
  }
  if (!(stages & 8)) return RPA_OK;
  return hip_fail(rpa::launch_attn_merge(s, p), "merge kernel launch");
}

int rpa_ragged_paged_attention(rpa_stream_t stream, const void* q, const void* kv_pages, const float* kv_scales,
                               const int32_t* context_lens, const int32_t* block_tables,
                               const int32_t* query_start_loc, const int32_t* num_seqs, void* out, void* workspace,
                               size_t workspace_bytes, int T, int S, int M, int P, int page_size, int Hq, int Hkv,
                               int D, int Dp, int C, int q_dtype, int kv_dtype, float softmax_scale, int sliding_window,
                               float logits_soft_cap, const float* softmax_aux) {
  if (Hkv > 0 && C < 2 * Hkv)
    return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_ragged_paged_attention: C=%d combined heads < 2*Hkv=%d", C, 2 * Hkv);
  // interleaved pages: K of head h in combined head 2h, V in 2h+1, one stored row of Dp elements each
  const int64_t row = (int64_t)Dp * rpa::elem_bytes(kv_dtype);
  const void* v_pages = kv_pages ? (const char*)kv_pages + row : nullptr;
  return attention_impl("rpa_ragged_paged_attention", stream, q, kv_pages, v_pages, (int64_t)C * row, 2 * row, kv_scales,
                        context_lens, block_tables, query_start_loc, num_seqs, false, out, workspace, workspace_bytes, T, S,
                        M, P, page_size, Hq, Hkv, D, Dp, C, q_dtype, kv_dtype, softmax_scale, sliding_window, logits_soft_cap,
                        softmax_aux);
}

int rpa_unified_attention(rpa_stream_t stream, const void* q, const void* key_cache, const void* value_cache,
                          const float* kv_scales, const int32_t* context_lens, const int32_t* block_tables,
                          const int32_t* query_start_loc, const int32_t* num_seqs, void* out, void* workspace,
                          size_t workspace_bytes, int T, int S, int M, int P, int page_size, int Hq, int Hkv, int D,
                          int q_dtype, int kv_dtype, float softmax_scale, int sliding_window, float logits_soft_cap,
                          const float* softmax_aux) {
  // separate pools [P][page_size][Hkv][D]: heads one row apart, tokens Hkv rows apart
  const int64_t row = (int64_t)D * rpa::elem_bytes(kv_dtype);
  return attention_impl("rpa_unified_attention", stream, q, key_cache, value_cache, (int64_t)Hkv * row, row, kv_scales,
                        context_lens, block_tables, query_start_loc, num_seqs, true, out, workspace, workspace_bytes, T, S, M,
                        P, page_size, Hq, Hkv, D, D, 2 * Hkv, q_dtype, kv_dtype, softmax_scale, sliding_window, logits_soft_cap,
                        softmax_aux);
}

int rpa_ragged_paged_attention_v3(rpa_stream_t stream, const void* q, const void* key, const void* value,
                                  void* kv_pages, const int32_t* context_lens, const int32_t* block_tables,
                                  const int32_t* query_start_loc, const int32_t* distribution, void* out,
                                  void* workspace, size_t workspace_bytes, int T, int S, int M, int P, int page_size,
                                  int Hq, int Hkv, int D, int Dp, int C, int q_dtype, int kv_dtype, float softmax_scale,
                                  int sliding_window, float logits_soft_cap, const float* softmax_aux) {
  const char* who = "rpa_ragged_paged_attention_v3";
  if (!distribution) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: null distribution", who);
  if (Hkv > 0 && C < 2 * Hkv) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: C=%d combined heads < 2*Hkv=%d", who, C, 2 * Hkv);
  if (T > 0 && (!key || !value)) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: null key / value", who);
  const int32_t* n_live = distribution + 2;
  const int64_t row = (int64_t)Dp * rpa::elem_bytes(kv_dtype);
  const void* v_pages = kv_pages ? (const char*)kv_pages + row : nullptr;
  // 8-bit pages here are unscaled: key / value hold the cast codes, which are copied and later read as the values
  return attention_impl(who, stream, q, kv_pages, v_pages, (int64_t)C * row, 2 * row, nullptr, context_lens, block_tables,
                        query_start_loc, n_live, false, out, workspace, workspace_bytes, T, S, M, P, page_size, Hq, Hkv, D, Dp,
                        C, q_dtype, kv_dtype, softmax_scale, sliding_window, logits_soft_cap, softmax_aux, key, value);
}

// ---- the entry point that allocates nothing ----------------------------------------------------------------
// Its workspace (decode plan, split-K partial slots, key-chunk partials) is this file-scope device array: every GPU
// the library runs on holds its own copy, at its own address, until the process ends.  In host code the array's name
// is only a handle for hipGetSymbolAddress: the address is looked up once per device (with that device current) and
// kept in scratch_ptr; kernels, like the ones behind the other entry points, get the pointer as an argument.
static __device__ __align__(256) unsigned char scratch[RPA_STATIC_WORKSPACE_BYTES];

static int static_workspace(void** ptr) {
  static std::mutex mu;
  static void* scratch_ptr[rpa::kMaxDevices];  // per device; null = not looked up yet
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return hip_fail((int)err, "hipGetDevice");
  if (dev < 0 || dev >= rpa::kMaxDevices) return fail(RPA_ERR_UNSUPPORTED, "device %d: the static workspace is kept for devices 0..%d", dev, rpa::kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(mu);
  if (!scratch_ptr[dev]) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess || !p) return hip_fail(err != hipSuccess ? (int)err : (int)hipErrorInvalidSymbol, "hipGetSymbolAddress(scratch)");
    scratch_ptr[dev] = p;
  }
  *ptr = scratch_ptr[dev];
  return RPA_OK;
}

int rpa_ragged_paged_attention_v3_static(rpa_stream_t stream, const void* q, const void* key, const void* value,
                                         void* kv_pages, const int32_t* context_lens, const int32_t* block_tables,
                                         const int32_t* query_start_loc, const int32_t* distribution, void* out, int T,
                                         int S, int M, int P, int page_size, int Hq, int Hkv, int D, int Dp, int C,
                                         int q_dtype, int kv_dtype, float softmax_scale, int sliding_window,
                                         float logits_soft_cap, const float* softmax_aux) {
  const char* who = "rpa_ragged_paged_attention_v3_static";
  // The smallest layout the attention accepts: plan + two partial slots of the decode-class tokens.  Checked here, from
  // the shapes alone, so that a batch too large for the array is refused by name instead of as a generic workspace error.
  if (T > 0 && S > 0 && M > 0 && page_size > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0 && D > 0 && Dp >= D) {
    const int Dc = Dp;  // partial rows are at most the stored width
    const int td = decode_token_bound(T, S, Hq, Hkv, rpa::decode_row_limit(T, S, Dc, kv_dtype));
    const size_t need = 2 * (part_o_bytes(td, Hq, Dc) + part_ml_bytes(td, Hq)) + plan_bytes(S) + 256;
    if (need > (size_t)RPA_STATIC_WORKSPACE_BYTES)
      return fail(RPA_ERR_WORKSPACE, "%s: these shapes need at least %zu bytes of workspace, the built-in array holds %u; "
                  "use rpa_ragged_paged_attention_v3 with a caller-owned workspace", who, need, (unsigned)RPA_STATIC_WORKSPACE_BYTES);
  }
  void* ws = nullptr;
  if (T > 0) {
    if (const int rc = static_workspace(&ws)) return rc;
  }
  return rpa_ragged_paged_attention_v3(stream, q, key, value, kv_pages, context_lens, block_tables, query_start_loc, distribution,
                                       out, ws, RPA_STATIC_WORKSPACE_BYTES, T, S, M, P, page_size, Hq, Hkv, D, Dp, C, q_dtype,
                                       kv_dtype, softmax_scale, sliding_window, logits_soft_cap, softmax_aux);
}

int rpa_ragged_paged_attention_v3_quantised(rpa_stream_t stream, const void* q, const void* key, const void* value,
                                            void* kv_pages, float* kv_scales, const int32_t* context_lens,
                                            const int32_t* block_tables, const int32_t* query_start_loc,
                                            const int32_t* distribution, void* out, void* workspace,
                                            size_t workspace_bytes, int T, int S, int M, int P, int page_size, int Hq,
                                            int Hkv, int D, int Dp, int C, int q_dtype, int kv_src_dtype, int kv_dtype,
                                            float softmax_scale, int sliding_window, float logits_soft_cap,
                                            const float* softmax_aux) {
  if (!distribution) return fail(RPA_ERR_INVALID_ARGUMENT, "rpa_ragged_paged_attention_v3_quantised: null distribution");
  const int32_t* n_live = distribution + 2;
  int err = rpa_page_scatter_ragged_quantised(stream, key, value, kv_pages, kv_scales, context_lens, block_tables,
                                              query_start_loc, n_live, T, S, M, P, page_size, Hkv, D, Dp, C, kv_src_dtype, kv_dtype);
  if (err) return err;
  return rpa_ragged_paged_attention(stream, q, kv_pages, kv_scales, context_lens, block_tables, query_start_loc, n_live,
                                    out, workspace, workspace_bytes, T, S, M, P, page_size, Hq, Hkv, D, Dp, C, q_dtype,
                                    kv_dtype, softmax_scale, sliding_window, logits_soft_cap, softmax_aux);
}

size_t rpa_mla_workspace_bytes(int T, int S, int M, int page_size, int Hq, int kv_lora_rank, int q_dtype, int kv_dtype) {
  (void)M; (void)page_size; (void)q_dtype; (void)kv_dtype;
  if (T <= 0 || S <= 0 || Hq <= 0 || kv_lora_rank <= 0) return 256;
  int chunks, rule_chunks, min_chunk;
  mla_split(T, S, Hq, kv_lora_rank, &chunks, &rule_chunks, &min_chunk);
  return (chunks > 1 ? (size_t)chunks * (part_o_bytes(T, Hq, kv_lora_rank) + part_ml_bytes(T, Hq)) : 0) +
         rpa::mla_plan_bytes(T, S, Hq, chunks) + 512;
}

static int mla_fill(const char* who, rpa::MlaParams& p, const void* keys_values, const void* keys_pe, void* kv_pages,
                    const int32_t* context_lens, const int32_t* block_tables, const int32_t* query_start_loc,
                    const int32_t* num_seqs, int T, int S, int M, int P, int page_size, int lkv, int rope, int row_elems,
                    int kv_dtype) {
  if (T < 0 || S <= 0 || M <= 0 || P <= 0 || page_size <= 0 || lkv <= 0 || rope < 0 || row_elems <= 0)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: bad size (T=%d S=%d M=%d P=%d page_size=%d kv_lora_rank=%d rope=%d row_elems=%d)",
                who, T, S, M, P, page_size, lkv, rope, row_elems);
  if (lkv > 512 || rope > 256 || lkv % 8 != 0 || rope % 8 != 0)
    return fail(RPA_ERR_UNSUPPORTED, "%s: kv_lora_rank %d / qk_rope_head_dim %d (want multiples of 8, <= 512 / <= 256)", who, lkv, rope);
  const int rope_off = (lkv + 127) / 128 * 128;
  if (row_elems < rope_off + rope)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: row_elems=%d < %d (latent part padded to 128, then the rope key)", who, row_elems, rope_off + rope);
  if (kv_dtype != RPA_F32 && kv_dtype != RPA_BF16 && kv_dtype != RPA_F16 && kv_dtype != RPA_FP8_E4M3)
    return fail(RPA_ERR_UNSUPPORTED, "%s: kv_dtype %d (want f32, bf16, f16 or fp8-e4m3 codes without scales)", who, kv_dtype);
  memset(&p, 0, sizeof(p));
  p.new_kv = keys_values; p.new_pe = keys_pe; p.pages = kv_pages;
  p.context_lens = context_lens; p.block_tables = block_tables; p.qsl = query_start_loc; p.num_seqs = num_seqs;
  p.T = T; p.S = S; p.M = M; p.P = P; p.page_size = page_size; p.lkv = lkv; p.rope = rope; p.rope_off = rope_off;
  p.row_elems = row_elems;
  p.token_stride = (int64_t)row_elems * rpa::elem_bytes(kv_dtype);
  p.page_stride = p.token_stride * page_size;
  p.kv_dtype = kv_dtype;
  p.max_chunks = 1;
  p.rule_chunks = 1;
  p.min_chunk = 512;
  return RPA_OK;
}

int rpa_mla_page_scatter(rpa_stream_t stream, const void* keys_values, const void* keys_pe, void* kv_pages,
                         const int32_t* context_lens, const int32_t* block_tables, const int32_t* query_start_loc,
                         const int32_t* num_seqs, int T, int S, int M, int P, int page_size, int kv_lora_rank,
                         int qk_rope_head_dim, int row_elems, int elem_bytes) {
  const char* who = "rpa_mla_page_scatter";
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4) return fail(RPA_ERR_UNSUPPORTED, "%s: elem_bytes %d (want 1, 2 or 4)", who, elem_bytes);
  rpa::MlaParams p;
  const int rc = mla_fill(who, p, keys_values, keys_pe, kv_pages, context_lens, block_tables, query_start_loc, num_seqs, T, S,
                          M, P, page_size, kv_lora_rank, qk_rope_head_dim, row_elems, elem_bytes == 4 ? RPA_F32 : elem_bytes == 2 ? RPA_BF16 : RPA_FP8_E4M3);
  if (rc) return rc;
  if (T == 0) return RPA_OK;
  if (!keys_values || (!keys_pe && qk_rope_head_dim > 0) || !kv_pages || !context_lens || !block_tables || !query_start_loc || !num_seqs)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  return hip_fail(rpa::launch_mla_scatter((hipStream_t)stream, p), "rpa_mla_page_scatter launch");
}

int rpa_mla_ragged_paged_attention(rpa_stream_t stream, const void* queries_nope, const void* queries_pe,
                                   const void* keys_values, const void* keys_pe, void* kv_pages,
                                   const int32_t* context_lens, const int32_t* block_tables,
                                   const int32_t* query_start_loc, const int32_t* distribution, void* out,
                                   void* workspace, size_t workspace_bytes, int T, int S, int M, int P, int page_size,
                                   int Hq, int kv_lora_rank, int qk_rope_head_dim, int row_elems, int q_dtype,
                                   int kv_dtype, float softmax_scale, int sliding_window, float logits_soft_cap,
                                   const float* softmax_aux) {
  const char* who = "rpa_mla_ragged_paged_attention";
  if (Hq <= 0) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: bad size (Hq=%d)", who, Hq);
  if (q_dtype != RPA_F32 && q_dtype != RPA_BF16 && q_dtype != RPA_F16) return fail(RPA_ERR_UNSUPPORTED, "%s: q_dtype %d (want f32, bf16 or f16)", who, q_dtype);
  if (!distribution) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: null distribution", who);
  if (!std::isfinite(softmax_scale)) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: softmax_scale is not finite", who);
  if (softmax_aux && ((uintptr_t)softmax_aux & 3)) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: softmax_aux must be 4-byte aligned", who);
  rpa::MlaParams p;
  const int rc = mla_fill(who, p, keys_values, keys_pe, kv_pages, context_lens, block_tables, query_start_loc, distribution + 2,
                          T, S, M, P, page_size, kv_lora_rank, qk_rope_head_dim, row_elems, kv_dtype);
  if (rc) return rc;
  if (T == 0) return RPA_OK;
  if (!queries_nope || (!queries_pe && qk_rope_head_dim > 0) || !kv_pages || !context_lens || !block_tables || !query_start_loc || !out)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if (keys_values && !keys_pe && qk_rope_head_dim > 0) return fail(RPA_ERR_INVALID_ARGUMENT, "%s: keys_values without keys_pe", who);
  if ((((uintptr_t)queries_nope) | ((uintptr_t)queries_pe) | ((uintptr_t)out) | ((uintptr_t)kv_pages)) & 15)
    return fail(RPA_ERR_INVALID_ARGUMENT, "%s: queries, out and the page pool must be 16-byte aligned", who);
  p.q_nope = queries_nope; p.q_pe = queries_pe; p.out = out; p.sinks = softmax_aux;
  p.Hq = Hq; p.q_dtype = q_dtype;
  p.scale = softmax_scale;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  p.window = sliding_window > 0 ? sliding_window : 0;
  p.softcap = logits_soft_cap > 0.f ? logits_soft_cap : 0.f;
  p.mfma = (!g_tun.force_generic && rpa::mla_mfma_supported(p)) ? 1 : 0;
  hipStream_t s = (hipStream_t)stream;
  if (keys_values && !p.mfma) {  // on the matrix-core path the write rides along with the plan kernel's launch
    const int err = rpa::launch_mla_scatter(s, p);
    if (err) return hip_fail(err, "MLA page write launch");
  }
  if (p.mfma) {
    int chunks, rule_chunks, min_chunk;
    mla_split(T, S, Hq, kv_lora_rank, &chunks, &rule_chunks, &min_chunk);
    const size_t po = part_o_bytes(T, Hq, kv_lora_rank), pml = part_ml_bytes(T, Hq);
    char* base = (char*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
    // the plan is sized for the chunks the shapes ask for; a small workspace then gets fewer, longer chunks
    const size_t plan_bytes_mla = rpa::mla_plan_bytes(T, S, Hq, chunks);
    if (!workspace || workspace_bytes < plan_bytes_mla + 256)
      return fail(RPA_ERR_WORKSPACE, "%s: workspace %zu bytes < %zu needed for the plan", who, workspace_bytes, plan_bytes_mla + 256);
    const size_t usable = workspace_bytes - 256 - plan_bytes_mla;
    if ((size_t)chunks * (po + pml) > usable) chunks = (int)(usable / (po + pml));
    if (chunks < 2) chunks = 1;  // a single chunk writes its rows directly and needs no partial buffers
    p.max_chunks = chunks;
    p.rule_chunks = std::min(rule_chunks, chunks);
    p.min_chunk = min_chunk;
    p.auto_chunk = g_tun.mla_chunks <= 0 && g_tun.mla_min_chunk <= 0;  // set knobs are taken literally
    p.cus = device_cus();
    const size_t slots = (size_t)rpa::mla_plan_slots(T, S, Hq);
    p.plan = (int2*)base;
    p.n_units = (int32_t*)(base + align256(slots * 8));
    p.units = (int2*)(base + align256(slots * 8) + 256);
    p.part_o = (float*)(base + plan_bytes_mla);
    p.part_ml = (float*)(base + plan_bytes_mla + (size_t)chunks * po);
    const int err = rpa::launch_mla_mfma(s, p);
    if (err) return hip_fail(err, "MLA kernel launch");
  } else {
    const int err = rpa::launch_mla_generic(s, p);
    if (err) return hip_fail(err, "MLA fp32 kernel launch");
  }
  return hip_fail(rpa::launch_mla_merge(s, p), "MLA merge kernel launch");
}

}  // extern "C"
