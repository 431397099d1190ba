/*
 * rpa_hip.h -- C ABI of the MI355X (gfx950) ragged-paged-attention library.
 *
 * One shared library, librpa_hip.so, exports the entry points below.  Every pointer marked
 * "device" is a HIP device pointer; metadata arrays are int32.  No entry point synchronises
 * the device, allocates device memory, or reads device data back to the host: work is
 * enqueued on `stream` with launch grids sized from the static bounds (T, S, M) and blocks
 * that exit early on padded rows, so the calls are legal inside a compiled serving step.
 *
 * Return value: 0 on success; a positive value is a hipError_t from a failed launch; a
 * negative value is one of the RPA_ERR_* codes.  rpa_last_error() returns a thread-local,
 * human-readable description of the most recent failure on the calling thread.
 *
 * The entry points keep no state between calls and may be called from any number of threads at
 * once (device properties are cached per device; the knobs of rpa_hip_probe.h, for tests and
 * measurement, belong to the thread that sets them).  HIP's current device must be the one the
 * pointers live on.
 *
 * KV page layout (all entry points): kv_pages[P][page_size][C][Dp] elements, where combined
 * head 2h holds K of KV head h and 2h+1 holds V (reference: easydel/caching/ragged_page/
 * cache.py:719-726 for the v2 shape, :711-718 for the v3 shape, :954-973 for the K-even /
 * V-odd interleave).  The reference's v3 storage [P][page][groups][packing][Dp] has the same
 * bytes as [P][page][C = groups*packing][Dp]; for head_dim 64 it stores K_h|V_h in one
 * 128-wide row, which is again the same bytes as C = 2*Hkv rows of Dp = 64.  C >= 2*Hkv.
 * Dp >= D is the stored width of a head row: the reference pads head sizes that are neither 64
 * nor a multiple of 128 up to the next multiple of 128 (cache.py:640-647: 80 / 96 / 112 -> 128,
 * 192 -> 256); Dp = D without padding.  The write entry points store zeros in the padding and
 * the attention over bf16 / 8-bit pages relies on finite values there (a pool that starts as
 * zeros, as the reference's does, and is written through these entry points qualifies).
 */
#ifndef RPA_HIP_H_
#define RPA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element formats of q / out (F32, BF16, F16) and of KV pages (all five). */
typedef enum rpa_dtype {
  RPA_F32 = 0,
  RPA_BF16 = 1,
  RPA_FP8_E4M3 = 2, /* OCP e4m3fn codes; value = code * kv_scales[page][combined head], or the code's own value
                       when no scales are passed (the reference's cast-only 8-bit cache, cache.py:143-158) */
  RPA_INT8 = 3,     /* signed 8-bit codes, scaled likewise */
  RPA_F16 = 4       /* IEEE half: half queries over half pages run on the matrix-core kernels, other mixes on the float32 kernel */
} rpa_dtype;

#define RPA_OK 0
#define RPA_ERR_INVALID_ARGUMENT (-1) /* null pointer, non-positive size, inconsistent heads */
#define RPA_ERR_UNSUPPORTED (-2)      /* dtype / head_dim combination no kernel covers */
#define RPA_ERR_WORKSPACE (-3)        /* workspace smaller than rpa_attention_workspace_bytes() */

typedef void* rpa_stream_t; /* a hipStream_t; NULL is the default stream */

/* Library version, "major.minor.patch". */
const char* rpa_version(void);

/* Description of the last failure seen by the calling thread ("" if none). */
const char* rpa_last_error(void);

/*
 * Page scatter, slice form.  Replaces kv_cache_update_jax
 * (easydel/caching/ragged_page/utils.py:302-387, with the shard localisation of :66-123),
 * which RaggedPagesCacheView.concatenate_to_cache calls for v2 caches (cache.py:853-930).
 *
 *   new_kv        device, [T][row_bytes]      token rows (K/V interleaved on the combined head axis)
 *   slice_indices device, int32 [3][N]        row 0 = destination flat cache position (global page
 *                                              space), row 1 = source token, row 2 = length
 *   num_slices    device, int32 [1]           number of valid columns
 *   kv_pages      device, [num_positions][row_bytes], updated in place
 *   page_shard_index                          which contiguous block of num_positions/page_size
 *                                              pages this buffer holds (0 when unsharded)
 * Bit-exact copy of whole token rows.  Columns >= num_slices[0], non-local slices, packed
 * tokens beyond T, sources outside [0,T) and destinations outside the buffer are dropped,
 * exactly as the reference's mode="drop" scatter does.
 */
int rpa_page_scatter_slices(rpa_stream_t stream, const void* new_kv, const int32_t* slice_indices,
                            const int32_t* num_slices, void* kv_pages, int T, int N,
                            int64_t num_positions, int page_size, int64_t row_bytes,
                            int page_shard_index);

/*
 * Page scatter, ragged form: the write half of the fused v3 operation
 * (ejkernel.modules.ragged_page_attention_v3 as called at
 * easydel/operations/kernels/ragged_page_attention.py:732-746).  Sequence i < num_seqs[0]
 * writes key/value[qsl[i] .. qsl[i+1]) to token positions [ctx_i - q_len_i, ctx_i) of the pages
 * block_tables[i][*]; K of head h goes to combined head 2h, V to 2h+1.
 *
 *   key, value    device, [T][Hkv][D] in the cache element type (elem_bytes each)
 *   kv_pages      device, [P][page_size][C][Dp], updated in place (elements D..Dp-1 of a written row become zero)
 *   block_tables  device, int32 [S][M] (the flattened [S*M] form is the same bytes)
 *   num_seqs      device, int32 [1]: number of live rows (pass distribution + 2 for v3 metadata)
 * Bit-exact.  Positions < 0 and padded tokens (t >= qsl[num_seqs]) are skipped.
 */
int rpa_page_scatter_ragged(rpa_stream_t stream, const void* key, const void* value, void* kv_pages,
                            const int32_t* context_lens, const int32_t* block_tables,
                            const int32_t* query_start_loc, const int32_t* num_seqs, int T, int S, int M,
                            int P, int page_size, int Hkv, int D, int Dp, int C, int elem_bytes);

/*
 * Page scatter, ragged form, into scaled 8-bit pages (RPA_FP8_E4M3 or RPA_INT8).  No counterpart in the
 * reference, whose ragged pages carry no scales (its 8-bit page dtypes store unscaled casts,
 * easydel/caching/ragged_page/cache.py:143-158): this is the write side of the page format the attention entry
 * points read with kv_scales.  key/value are in src_dtype (RPA_F32 or RPA_BF16), placed as by
 * rpa_page_scatter_ragged.  Per (sequence, page it writes to, combined head), in float32:
 *   old   = 0 if the sequence's new tokens start the page, else kv_scales[page][head]
 *   new   = max(old, amax|new values| / qmax), and 1 if that is 0        (qmax = 448 for fp8, 127 for int8)
 *   tokens already in the page are re-coded, code <- quant((decode(code) * old) / new), if new > old
 *   new tokens are coded quant(x / new); kv_scales[page][head] = new
 * with quant = clamp to the code range, round to nearest even.  Deterministic and bit-exact against that rule.
 * A page may be written by one sequence per call (pages shared between sequences are full pages).
 */
int rpa_page_scatter_ragged_quantised(rpa_stream_t stream, const void* key, const void* value, void* kv_pages,
                                      float* kv_scales, const int32_t* context_lens, const int32_t* block_tables,
                                      const int32_t* query_start_loc, const int32_t* num_seqs, int T, int S, int M, int P,
                                      int page_size, int Hkv, int D, int Dp, int C, int src_dtype, int kv_dtype);

/*
 * Bytes of scratch rpa_ragged_paged_attention needs for these static bounds (split-K
 * partial outputs and their running max / sum).  The caller owns the buffer (under XLA it
 * is an extra result of the custom call), 256-byte aligned.  D is the stored head width Dp when
 * the pages are padded.  The figure is what lets every sequence and row tile be split as finely
 * as the kernels would like; an attention call accepts any workspace that holds two partial
 * slots (it reports RPA_ERR_WORKSPACE below that), lays the buffer out from the bytes it is
 * given and splits less when they are fewer, so the two calls cannot disagree.  For 8-bit
 * pages of head size 128 or 256 the figure also holds room for bf16 copies of the pages of prompt
 * chunks (two bytes per element of at most T * group / (rows per decode sequence + 1)
 * sequences of M pages, at most 4 GiB): with them a long chunk runs on the faster 16-bit
 * prefill kernel; a workspace without that room gives the same results from the 8-bit kernel.
 */
size_t rpa_attention_workspace_bytes(int T, int S, int M, int page_size, int Hq, int Hkv, int D,
                                     int q_dtype, int kv_dtype);

/*
 * Ragged paged attention (read-only over the pages).  Replaces
 * ejkernel.modules.ragged_page_attention_v2 as called at
 * easydel/operations/kernels/ragged_page_attention.py:281-313, and the attention half of
 * ragged_page_attention_v3 (:684-695, :732-746).
 *
 *   q             device, [T][Hq][D]          q_dtype in {RPA_F32, RPA_BF16, RPA_F16}
 *   kv_pages      device, [P][page_size][C][Dp] kv_dtype
 *   kv_scales     device, float [P][C] or NULL; 8-bit pages only.  NULL with fp8 pages: the codes are the values
 *                 (scale 1), which is how the reference stores an fp8 cache (a bare cast, ragged_page_attention.py:570-580).
 *                 int8 pages always need their scales (RPA_ERR_INVALID_ARGUMENT without).
 *   context_lens  device, int32 [S]           tokens in the cache per sequence, new ones included
 *   block_tables  device, int32 [S][M]
 *   query_start_loc device, int32 [S+1]
 *   num_seqs      device, int32 [1]           live rows
 *   out           device, [T][Hq][D] q_dtype; rows of padded tokens are written as zeros
 *   workspace     device, workspace_bytes >= rpa_attention_workspace_bytes(...)
 *   softmax_scale                            multiplies q.k before the soft cap
 *   sliding_window                           <= 0: none; W: key j visible iff pos-W < j <= pos
 *   logits_soft_cap                          <= 0: none; cap: s = cap*tanh(s/cap)
 *   softmax_aux   device, float [Hq] or NULL: attention sinks, the reference's softmax_aux
 *                 (ragged_page_attention.py:469-471, :590-592: one float32 logit per query head).  The softmax of
 *                 head hq runs over the visible keys and the extra logit softmax_aux[hq] (taken as is: no
 *                 softmax_scale, no soft cap), whose probability is then dropped, so the weights of a row sum to
 *                 less than one: out = sum_j exp(s_j) v_j / (sum_j exp(s_j) + exp(softmax_aux[hq])).  This is the
 *                 GPT-OSS definition the reference's model file feeds (modules/gpt_oss/modeling_gpt_oss.py:436-442).
 * Query row r of sequence i sits at position ctx_i - q_len_i + r and attends causally.
 * Limits: S * M * page_size < 2^31 (what the block tables of one call can address; RPA_ERR_UNSUPPORTED beyond).
 * Padded head storage (Dp > D): the Dp - D padding elements of every stored row must be zero, or at least finite --
 * the matrix-core kernels multiply them by zero query elements, and 0 x NaN / Inf would reach the scores.  Pages written
 * through this library have zero padding (a pool must start zeroed, as the reference's does); a pool filled by another
 * writer must keep that promise.
 */
int rpa_ragged_paged_attention(rpa_stream_t stream, const void* q, const void* kv_pages,
                               const float* kv_scales, const int32_t* context_lens,
                               const int32_t* block_tables, const int32_t* query_start_loc,
                               const int32_t* num_seqs, void* out, void* workspace, size_t workspace_bytes,
                               int T, int S, int M, int P, int page_size, int Hq, int Hkv, int D, int Dp, int C,
                               int q_dtype, int kv_dtype, float softmax_scale, int sliding_window,
                               float logits_soft_cap, const float* softmax_aux);

/*
 * The same attention over separate K and V pools: key_cache and value_cache are each
 * [P][page_size][Hkv][D] (reference: easydel/caching/unified_attention/cache.py:216-218, :492-500).
 * Replaces ejkernel.modules.unified_attention as called at
 * easydel/operations/kernels/unified_attention.py:363-388 (and :319-331 for the shard-local form).
 * The pools are filled by rpa_page_scatter_slices, once for K and once for V, with
 * row_bytes = Hkv*D*elem (the reference's UnifiedAttentionCacheView.concatenate_to_cache, cache.py:523-610).
 *
 *   num_seqs   device, int32 [1], or NULL: the reference passes no row count to this kernel, every one of the
 *              S rows is live and padded rows are those with an empty query span
 *   kv_scales  device, float [P][2*Hkv] (K of head h at column 2h, V at 2h+1) or NULL; required for 8-bit pools
 * Everything else as for rpa_ragged_paged_attention; the workspace size is the same function of the bounds.
 */
int rpa_unified_attention(rpa_stream_t stream, const void* q, const void* key_cache, const void* value_cache,
                          const float* kv_scales, const int32_t* context_lens, const int32_t* block_tables,
                          const int32_t* query_start_loc, const int32_t* num_seqs, void* out, void* workspace,
                          size_t workspace_bytes, int T, int S, int M, int P, int page_size, int Hq, int Hkv, int D,
                          int q_dtype, int kv_dtype, float softmax_scale, int sliding_window, float logits_soft_cap,
                          const float* softmax_aux);

/*
 * Fused v3 form: rpa_page_scatter_ragged followed by rpa_ragged_paged_attention on the
 * same stream, pages updated in place (the reference returns (out, kv_pages) and the
 * caller stores the pages back, ragged_page_attention.py:747).  key/value must already be
 * in the cache element type (the reference casts them first, :570-580), whatever that type is:
 * for an 8-bit cache they hold the cast codes, which are copied bit for bit and read back as
 * their own values (scaled 8-bit pages have rpa_ragged_paged_attention_v3_quantised).
 */
int rpa_ragged_paged_attention_v3(rpa_stream_t stream, const void* q, const void* key, const void* value,
                                  void* kv_pages, const int32_t* context_lens, const int32_t* block_tables,
                                  const int32_t* query_start_loc, const int32_t* distribution, void* out,
                                  void* workspace, size_t workspace_bytes, int T, int S, int M, int P,
                                  int page_size, int Hq, int Hkv, int D, int Dp, int C, int q_dtype, int kv_dtype,
                                  float softmax_scale, int sliding_window, float logits_soft_cap,
                                  const float* softmax_aux);

/*
 * rpa_ragged_paged_attention_v3 for callers that cannot allocate or hand over scratch memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same operands and
 * results; the split-K partials and the decode plan live in a 64 MiB device array inside the library
 * (RPA_STATIC_WORKSPACE_BYTES, one copy per GPU, held until the process ends) instead of a caller's workspace, and the
 * call allocates nothing.  Shapes whose smallest layout (two partial slots + plan) exceeds the array are rejected with
 * RPA_ERR_WORKSPACE; shapes that fit but would like more run with fewer partial slots / key chunks than a caller-sized
 * workspace would allow.
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race --
 * serialise them.  Nothing in the array has to survive or be cleared between calls (each call writes what it reads).
 * The first call on a device looks up the array's address and the device's CU count, and the first call that reaches a
 * kernel variant its occupancy; these are not stream operations and may be refused while a stream is being captured.
 * Before capturing this entry point, make one ordinary call with the same shapes and dtypes on that device.
 */
#define RPA_STATIC_WORKSPACE_BYTES (64u << 20)
int rpa_ragged_paged_attention_v3_static(rpa_stream_t stream, const void* q, const void* key, const void* value,
                                         void* kv_pages, const int32_t* context_lens, const int32_t* block_tables,
                                         const int32_t* query_start_loc, const int32_t* distribution, void* out, int T,
                                         int S, int M, int P, int page_size, int Hq, int Hkv, int D, int Dp, int C,
                                         int q_dtype, int kv_dtype, float softmax_scale, int sliding_window,
                                         float logits_soft_cap, const float* softmax_aux);

/*
 * Fused v3 form over scaled 8-bit pages: rpa_page_scatter_ragged_quantised followed by
 * rpa_ragged_paged_attention on the same stream; pages and scales updated in place.  key/value in kv_src_dtype.
 */
int rpa_ragged_paged_attention_v3_quantised(rpa_stream_t stream, const void* q, const void* key, const void* value,
                                            void* kv_pages, float* kv_scales, const int32_t* context_lens,
                                            const int32_t* block_tables, const int32_t* query_start_loc,
                                            const int32_t* distribution, void* out, void* workspace,
                                            size_t workspace_bytes, int T, int S, int M, int P, int page_size, int Hq,
                                            int Hkv, int D, int Dp, int C, int q_dtype, int kv_src_dtype, int kv_dtype,
                                            float softmax_scale, int sliding_window, float logits_soft_cap,
                                  const float* softmax_aux);

/*
 * Multi-latent attention (MLA) over latent ragged pages.  Replaces
 * ejkernel.modules.multi_latent_ragged_page_attention (and its _v2 twin, same operands) as called at
 * easydel/operations/kernels/multi_latent_ragged_page_attention.py:495-511, 611-624 (v1) and :1019-1030, 1090-1101 (v2).
 * Fused like the v3 operation: the new rows are written into the pages, then every query attends.
 *
 *   queries_nope  device, [T][Hq][kv_lora_rank], q_dtype: queries already multiplied by the key half of the
 *                 up-projection (the caller's "weight absorption", layers/attention/_unified.py:1292-1298)
 *   queries_pe    device, [T][Hq][qk_rope_head_dim], q_dtype
 *   keys_values   device, [T][kv_lora_rank], already in the pages' element type, or NULL: the pages are read as they
 *                 are (then keys_pe is ignored)
 *   keys_pe       device, [T][qk_rope_head_dim], pages' element type
 *   kv_pages      device, [P][page_size][row_elems] (the reference's
 *                 [P][page_size / packing][packing][kv_dim_padded], caching/mla_ragged_page/cache.py:270-287, is the
 *                 same bytes): per token the latent row at [0, kv_lora_rank), the rope key at
 *                 [align128(kv_lora_rank), + qk_rope_head_dim), padding zeroed by the write.  row_elems is at least
 *                 align128(kv_lora_rank) + qk_rope_head_dim; the reference uses align128 of both parts (640 for 512 + 64)
 *   distribution  device, int32 [3]; only [2], the number of live rows, is read (the reference passes [0, 0, total],
 *                 multi_latent_ragged_page_attention.py:376-378)
 *   out           device, [T][Hq][kv_lora_rank], q_dtype: softmax-weighted sums of latent rows (the caller applies the
 *                 value half of the up-projection, _unified.py:1366-1371)
 *   workspace     device scratch of at least rpa_mla_workspace_bytes(...) bytes
 *   softmax_scale as passed by the caller: (qk_nope_head_dim + qk_rope_head_dim) ** -0.5 (_unified.py:1310)
 * q_dtype RPA_F32, RPA_BF16 or RPA_F16; kv_dtype RPA_F32, RPA_BF16, RPA_F16 or RPA_FP8_E4M3 (the latent cache holds
 * no scale arrays, caching/mla_ragged_page/cache.py:197-204, 344: fp8 pages are the plain cast of the rows and are
 * read back as the codes' own values); kv_lora_rank <= 512, qk_rope_head_dim <= 256, both multiples of 8.  bf16
 * queries over bf16 pages with kv_lora_rank 512, rope 64 and page_size % 32 == 0 run on the matrix cores; every
 * other combination on the fp32 kernel.  Window, soft cap, softmax_aux, padding and error behaviour as for
 * rpa_ragged_paged_attention.
 */
int rpa_mla_ragged_paged_attention(rpa_stream_t stream, const void* queries_nope, const void* queries_pe,
                                   const void* keys_values, const void* keys_pe, void* kv_pages,
                                   const int32_t* context_lens, const int32_t* block_tables,
                                   const int32_t* query_start_loc, const int32_t* distribution, void* out,
                                   void* workspace, size_t workspace_bytes, int T, int S, int M, int P, int page_size,
                                   int Hq, int kv_lora_rank, int qk_rope_head_dim, int row_elems, int q_dtype,
                                   int kv_dtype, float softmax_scale, int sliding_window, float logits_soft_cap,
                                   const float* softmax_aux);

/* Workspace the call above needs, from the static bounds alone (and the compute-unit count of the current device;
 * a call handed fewer bytes cuts its rows into fewer, longer key chunks, down to none). */
size_t rpa_mla_workspace_bytes(int T, int S, int M, int page_size, int Hq, int kv_lora_rank, int q_dtype, int kv_dtype);

/*
 * The write half of the MLA operation on its own (same operands and placement as above; num_seqs: device int32 [1]).
 * elem_bytes 1, 2 or 4.
 */
int rpa_mla_page_scatter(rpa_stream_t stream, const void* keys_values, const void* keys_pe, void* kv_pages,
                         const int32_t* context_lens, const int32_t* block_tables, const int32_t* query_start_loc,
                         const int32_t* num_seqs, int T, int S, int M, int P, int page_size, int kv_lora_rank,
                         int qk_rope_head_dim, int row_elems, int elem_bytes);

#ifdef __cplusplus
}
#endif
#endif /* RPA_HIP_H_ */
