/*
 * rpa_hip_probe.h -- test and measurement aids of librpa_hip.so, kept apart from the operator entry points of
 * rpa_hip.h.  Nothing here has a counterpart in the reference and a serving runtime needs none of it.  The measurement
 * kernels, and the two knobs of rpa_set_tunable that change what a call computes with ("stages", "force_generic"), exist
 * only in a library built with -DRPA_PROBES (easydel_amd/build.py builds that one for tests and benchmarks; its
 * --product switch leaves them out: rpa_set_tunable then answers -1 for those names and the probes are not exported).
 */
#ifndef RPA_HIP_PROBE_H_
#define RPA_HIP_PROBE_H_

#include "rpa_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Measurement aid with no counterpart in the reference: copies `bytes` (a multiple of 16, both
 * pointers 16-byte aligned) with a plain vector copy kernel.  Profiling a known-size copy next to
 * the attention kernels gives the factor that turns raw HBM traffic counters into bytes.
 */
int rpa_calibration_copy(rpa_stream_t stream, void* dst, const void* src, size_t bytes);

/*
 * Measurement aid with no counterpart in the reference: a read-only kernel that says what the memory system gives
 * a streaming reader.  `workgroups` workgroups of eight wavefronts (one per CU: each holds 96 KiB of LDS) read `src`
 * once, every wavefront its own contiguous share with 16-byte loads, `kib_in_flight_per_wave` (2, 4, 8, 16 or 32) KiB
 * of them in flight.  Returns the bytes the launch reads (the share of each wavefront is rounded down to whole rounds
 * of loads), 0 on bad arguments; time the launch with events on `stream`.  `sink` is one device word, never written in
 * practice.  The decode kernel's bandwidth is judged against this probe's at the same number of workgroups.
 */
size_t rpa_read_probe(rpa_stream_t stream, const void* src, size_t bytes, int workgroups, int kib_in_flight_per_wave,
                      void* sink);

/*
 * The same reader over pages (no counterpart in the reference either): `src` is cut into chunks of `chunk_kib` KiB (a
 * multiple of 8; their number is rounded down to a power of two), every workgroup visits an equal share of them in a
 * scattered order, `kib_in_flight_per_wave` (2, 4, 8, 16 or 32, a multiple of chunk_kib / 8) KiB per wavefront in flight,
 * i.e. kib_in_flight_per_wave / (chunk_kib / 8) chunks per workgroup.  `split` says how the eight wavefronts share a chunk:
 * 0 contiguous eighths; 1 and 2 the way the decode kernels split a page -- the chunk is rows of 4 KiB (a token's keys and
 * values of eight heads) and wavefront w reads bytes [512 w, 512 w + 512) of every row, two rows per instruction -- with
 * non-temporal (1) or ordinary (2) loads.  It is the access pattern of the decode kernel over a page pool without its
 * arithmetic: what separates 1 from 2 is what the non-temporal hint is worth to that kernel.  Returns the bytes the
 * launch reads, 0 on bad arguments.
 */
size_t rpa_read_probe_paged(rpa_stream_t stream, const void* src, size_t bytes, int workgroups, int kib_in_flight_per_wave,
                            int chunk_kib, int split, void* sink);

/*
 * Measurement aid with no counterpart in the reference: what a stream of bf16 MFMAs sustains on this chip when its A
 * operands come out of LDS, i.e. the ceiling of the prefill kernels' inner loops.  One workgroup of four wavefronts per
 * CU (waves_per_simd = 1) or two (= 2) issue, per wavefront, 32 * mfmas_per_operand * iters MFMAs of `shape` (0:
 * 16x16x32, 1: 32x32x16); `source` says where the A operands come from: 0 registers, 1 ds_read_b128 in the pattern the
 * prefill kernels read K tiles with, 2 pairs of ds_read_b64_tr_b16 in their V pattern; every operand feeds
 * mfmas_per_operand (1, 2 or 4) MFMAs with distinct B operands and accumulators, as a wavefront that owns so many row
 * blocks would; operands are read four ahead.  Returns the floating-point operations of the launch (0 on bad
 * arguments); time the launch with events on `stream`.  `clocks` is two 8-byte device words the caller zeroes: the
 * launch adds shader-clock cycles to the first and ticks of the 100 MHz wall clock to the second, summed over the
 * workgroups, so 100 * clocks[0] / clocks[1] is the clock in MHz the kernel ran at.  `sink` is one device word, never
 * written in practice.
 */
double rpa_mfma_probe(rpa_stream_t stream, int shape, int source, int mfmas_per_operand, int waves_per_simd, int iters,
                      void* clocks, void* sink);

/*
 * Measurement aid with no counterpart in the reference: what one more instruction costs a lone wavefront per SIMD that
 * streams 32x32x16 bf16 MFMAs (how the 32x32 prefill kernel runs).  One workgroup of four wavefronts per CU; every
 * wavefront issues 16 * iters MFMAs, each followed by `fill` (0 or 6) independent v_fma_f32 and `extra` (0, 1, 2 or 4)
 * instructions of `kind`: 0 v_fma_f32, 1 v_exp_f32, 2 v_rcp_f32, 3 v_cvt_pk_bf16_f32, 4 v_max3_f32 (a dependent chain),
 * 5 s_add_u32 (a dependent chain), 6 s_nop, 7 ds_read_b128, 8 ds_read_b64_tr_b16, 9 global_load_lds_dwordx4 (1 KiB per
 * instruction, m0 written each time).  An MFMA holds the matrix pipe for 32 cycles and the issue port for 8: with
 * fill = 6 the slot is full, and the cycles per MFMA above that say what an instruction of `kind` costs.  Returns the
 * MFMAs per wavefront (0 on bad arguments).  `clocks` and `sink` as for rpa_mfma_probe: clocks[0] / (workgroups *
 * MFMAs per wavefront) is the cycles per MFMA.  `src`: 1 MiB of initialised device memory, 16-byte aligned (read by
 * kind 9 only).
 */
long long rpa_issue_probe(rpa_stream_t stream, int kind, int extra, int fill, int iters, void* clocks, void* sink, const void* src);

/*
 * Knobs for tests and measurement.  They belong to the calling thread: a value set here is seen only by entry points
 * the same thread calls afterwards (each call reads them once, when it starts), so threads that never call this function
 * always run with the defaults.  Returns the previous value, -1 for an unknown name.
 *   "max_splits"     partial-output slots per sequence the decode kernel may use (2..256, 0 = sized
 *                    from the shapes); set it before sizing the workspace
 *   "decode_wgs"     persistent decode workgroups per KV-head group (0 = as many as are resident at once)
 *   "decode_sync"    decode workgroups re-align their waves every this many tiles (power of two, default 8, 0 = never)
 *   "decode_pace"    1 (default): in the bf16 eight-wave decode kernel a wave that finds four or more of its workgroup's
 *                    tiles in flight pauses once (512 clocks) before issuing its own; 0: never
 *   "decode_dma"     which decode batches (bf16 / float16 pages, fp8 / int8 pages at head size 128; pages of a multiple
 *                    of 64 tokens, four or more KV heads) run on the LDS-direct decode kernel, two tiles in flight per
 *                    wave: -1 (default) 16-bit pages of head size 256 and int8 pages, where it measured faster; 0 none; 1 all; 2 all,
 *                    with one tile in flight; 3 all, the K rows of a tile requested together with its V rows (later than
 *                    they could be, but the two halves of each token's bytes then reach the memory side by side)
 *   "prefill_chunks" 0 (default): the key chunks of a prefill row tile are sized on the device from the lengths in the
 *                    batch (up to 8 per row tile); 1..8: a row tile is cut into at most this many chunks of a length
 *                    fixed from the block-table bound (1 = never split); set it before sizing the workspace
 *   "prefill_dma"    1 (default): prefill tiles are loaded global -> LDS by the load unit where those kernels apply
 *                    (page_size % 32 == 0); 0: every prefill tile is staged through registers (bf16 / 8-bit pages only)
 *   "prefill_x32"    1 (default): pages of a multiple of 64 tokens take the prefill kernel built on 32x32x16 tiles, one
 *                    workgroup per CU, at head size 128 (bf16 / float16 pages, no soft cap: 256-row workgroups) and at
 *                    head size 256 (bf16 pages, with or without soft cap: 128-row workgroups); 0: never
 *   "prefill_wide"   1 (default): scaled or bare 8-bit pages of head size 128 or 256 (pages of a multiple of 64 tokens, a soft cap at
 *                    head size 256 only; under a sliding window only from 2 048 tokens of window and two workgroups
 *                    per CU on) reach that kernel through bf16 copies of the large-row sequences' pages, made once per
 *                    call in what the workspace holds beyond the partial rows, where a decision kernel finds that the
 *                    pages fit and that the batch has 1 792 query rows per KV head and copied page or more on average, or
 *                    1 024 and two workgroups of that kernel per CU (256 rows x KV heads); n > 1: a single bar of n
 *                    rows (tests, measurements); 0: never (set it before sizing the workspace: the sizing call then
 *                    asks for no room for copies)
 *   "mla_chunks"     most key chunks one row tile of the multi-latent kernel is split into (1..16, 0 = sized from
 *                    the shapes, and batches of few row tiles cut by a chunk length chosen on the device from their
 *                    own lengths); set it before sizing the workspace
 *   "mla_min_chunk"  fewest keys of such a chunk (rounded up to 64; 0 = default: 1024 at 64 heads and more, else 512)
 *   "force_generic"  non-zero: route every call through the fp32 VALU kernel
 *   "stages"         bit mask of the attention call's launches, for profiling one kernel in isolation:
 *                    1 = decode plan kernel, 2 = decode kernel, 4 = prefill / large-row kernel,
 *                    8 = merge (default 15)
 */
int rpa_set_tunable(const char* name, int value);

#ifdef __cplusplus
}
#endif
#endif /* RPA_HIP_PROBE_H_ */
