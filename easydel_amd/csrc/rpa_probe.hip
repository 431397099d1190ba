// Measurement aids of the library (declared in include/rpa_hip_probe.h; built only with -DRPA_PROBES): a known-size
// copy, read-only probes of the memory system, and a probe of the matrix cores fed from LDS.  None of them is an
// operator; nothing in the operator entry points depends on this file.
#include "rpa_common.h"

namespace rpa {

// Plain grid-stride copy of 16-byte vectors: the known-size kernel that calibrates HBM traffic counters.
__global__ __launch_bounds__(256) void calibration_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x; k < n16; k += stride) dst[k] = src[k];
}

int launch_calibration_copy(hipStream_t stream, void* dst, const void* src, size_t bytes) {
  hipLaunchKernelGGL(calibration_copy_kernel, dim3(4096), dim3(256), 0, stream, (const uint4*)src, (uint4*)dst, bytes >> 4);
  return (int)hipGetLastError();
}

// Read-only probe of the memory system: `workgroups` workgroups of eight waves (96 KiB of LDS each, so one per CU), every
// wave streaming its own contiguous share of the buffer with 16-byte loads, DEPTH instructions (KiB) in flight.
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
template <int DEPTH>
__global__ __launch_bounds__(512) void read_probe_kernel(const probe_u32x4* __restrict__ src, size_t kib_per_wave, uint32_t* __restrict__ sink) {
  __shared__ char occupy[98304];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const probe_u32x4* p = src + ((size_t)blockIdx.x * 8 + wave) * kib_per_wave * 64 + lane;
  probe_u32x4 acc = {0u, 0u, 0u, 0u};
  for (size_t c = 0; c + DEPTH <= kib_per_wave; c += DEPTH) {
    probe_u32x4 v[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) v[d] = __builtin_nontemporal_load(p + (c + d) * 64);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) acc ^= v[d];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[0] = occupy[lane];  // keeps the loads and the LDS alive
}

// Returns the bytes the launch reads (0: bad arguments): bytes / (8 workgroups) rounded down to whole rounds of loads.
size_t launch_read_probe(hipStream_t stream, const void* src, size_t bytes, int workgroups, int kib_in_flight_per_wave,
                         uint32_t* sink) {
  if (workgroups <= 0) return 0;
  size_t per = bytes / ((size_t)workgroups * 8) / 1024;
  per -= per % (size_t)(kib_in_flight_per_wave > 0 ? kib_in_flight_per_wave : 1);
  if (per == 0) return 0;
#define RPA_PROBE(D) hipLaunchKernelGGL(read_probe_kernel<D>, dim3(workgroups), dim3(512), 0, stream, (const probe_u32x4*)src, per, sink)
  switch (kib_in_flight_per_wave) {
    case 2: RPA_PROBE(2); break;
    case 4: RPA_PROBE(4); break;
    case 8: RPA_PROBE(8); break;
    case 16: RPA_PROBE(16); break;
    case 32: RPA_PROBE(32); break;
    default: return 0;
  }
#undef RPA_PROBE
  return hipGetLastError() == hipSuccess ? per * 1024 * 8 * (size_t)workgroups : 0;
}

// The same reader over pages: the buffer is cut into chunks of `chunk_kib` KiB, a workgroup visits its chunks in a
// scattered order (a multiplicative permutation of the chunk numbers, as a block table of a long-lived pool would hand
// them out), DEPTH KiB per wave in flight, i.e. DEPTH / (chunk_kib / 8) chunks per workgroup.  SPLIT says how the eight
// waves share a chunk: 0 contiguous eighths; 1 and 2 the decode kernel's own split -- the chunk is rows of 4 KiB (a
// token's keys and values of eight heads) and wave w reads bytes [512 w, 512 w + 512) of every row, two rows per
// instruction -- with non-temporal (1) or ordinary (2) loads.
template <int DEPTH, int SPLIT>
__global__ __launch_bounds__(512) void read_probe_paged_kernel(const probe_u32x4* __restrict__ src, uint32_t chunk_mask, uint32_t chunks_per_wg,
                                                               uint32_t kib_per_wave_chunk, uint32_t* __restrict__ sink) {
  __shared__ char occupy[98304];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t per = kib_per_wave_chunk;          // KiB of a chunk one wave reads (DEPTH is a multiple of it)
  const uint32_t group = DEPTH / per;               // chunks in flight per workgroup
  probe_u32x4 acc = {0u, 0u, 0u, 0u};
  for (uint32_t c = 0; c + group <= chunks_per_wg; c += group) {
    probe_u32x4 v[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const uint32_t step = c + (uint32_t)d / per;                                               // which of the workgroup's chunks
      const uint32_t chunk = ((blockIdx.x * chunks_per_wg + step) * 0x9E3779B1u) & chunk_mask;  // where it lies
      if constexpr (SPLIT == 0) {
        const probe_u32x4* p = src + ((size_t)chunk * 8 + wave) * per * 64 + lane;
        v[d] = __builtin_nontemporal_load(p + ((uint32_t)d % per) * 64);
      } else {
        const uint32_t row = 2 * ((uint32_t)d % per) + (lane >> 5);  // of the chunk's 2 per rows
        const probe_u32x4* p = src + (size_t)chunk * 8 * per * 64 + (size_t)row * 256 + wave * 32 + (lane & 31);
        if constexpr (SPLIT == 1) v[d] = __builtin_nontemporal_load(p);
        else v[d] = *p;
      }
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) acc ^= v[d];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) sink[0] = occupy[lane];  // keeps the loads and the LDS alive
}

// Returns the bytes the launch reads (0: bad arguments).  The number of chunks in the buffer is rounded down to a power of
// two (the permutation needs one), each workgroup takes an equal share of them in whole groups.
size_t launch_read_probe_paged(hipStream_t stream, const void* src, size_t bytes, int workgroups, int kib_in_flight_per_wave,
                               int chunk_kib, int split, uint32_t* sink) {
  if (workgroups <= 0 || chunk_kib < 8 || (chunk_kib & 7) || kib_in_flight_per_wave <= 0 || split < 0 || split > 2) return 0;
  const uint32_t per = (uint32_t)chunk_kib / 8;
  if ((uint32_t)kib_in_flight_per_wave % per) return 0;
  size_t n_chunks = bytes / ((size_t)chunk_kib * 1024);
  if (n_chunks == 0) return 0;
  size_t pow2 = 1;
  while (pow2 * 2 <= n_chunks && pow2 < ((size_t)1 << 31)) pow2 *= 2;
  const uint32_t group = (uint32_t)kib_in_flight_per_wave / per;
  uint32_t per_wg = (uint32_t)(pow2 / (size_t)workgroups);
  per_wg -= per_wg % group;
  if (per_wg == 0) return 0;
#define RPA_PROBE_S(D, S)                                                                                                \
  hipLaunchKernelGGL((read_probe_paged_kernel<D, S>), dim3(workgroups), dim3(512), 0, stream, (const probe_u32x4*)src, \
                     (uint32_t)(pow2 - 1), per_wg, per, sink)
#define RPA_PROBE(D)                \
  if (split == 0) RPA_PROBE_S(D, 0); \
  else if (split == 1) RPA_PROBE_S(D, 1); \
  else RPA_PROBE_S(D, 2)
  switch (kib_in_flight_per_wave) {
    case 2: RPA_PROBE(2); break;
    case 4: RPA_PROBE(4); break;
    case 8: RPA_PROBE(8); break;
    case 16: RPA_PROBE(16); break;
    case 32: RPA_PROBE(32); break;
    default: return 0;
  }
#undef RPA_PROBE
#undef RPA_PROBE_S
  return hipGetLastError() == hipSuccess ? (size_t)per_wg * (size_t)chunk_kib * 1024 * (size_t)workgroups : 0;
}

// ---- matrix-core feed probe -------------------------------------------------------------------------------------
// A stream of bf16 MFMAs whose A operands are constants in registers (SRC 0), or are read from a bf16 tile in LDS the
// way the prefill kernels read K (SRC 1: ds_read_b128, rows of 256 bytes, 16-byte chunks XOR-swizzled by row) or V
// (SRC 2: pairs of ds_read_b64_tr_b16).  Every operand feeds REUSE MFMAs (distinct B operands and accumulators, as a
// wave that owns REUSE row blocks would), operands are read four ahead of their MFMAs, and the order written is the
// order issued (sched_barrier after every operand).  SHAPE 0 = 16x16x32, 1 = 32x32x16.
typedef __bf16 mp_bf16x8 __attribute__((ext_vector_type(8)));
typedef short mp_s16x4 __attribute__((ext_vector_type(4)));
typedef float mp_f32x4 __attribute__((ext_vector_type(4)));
typedef float mp_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t mp_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t mp_u32x2 __attribute__((ext_vector_type(2)));

template <int SHAPE> struct MpAcc;
template <> struct MpAcc<0> { typedef mp_f32x4 T; static constexpr int N = 4; };
template <> struct MpAcc<1> { typedef mp_f32x16 T; static constexpr int N = 16; };

template <int SHAPE>
__device__ __forceinline__ typename MpAcc<SHAPE>::T mp_mfma(mp_u32x4 a, mp_u32x4 b, typename MpAcc<SHAPE>::T c) {
  if constexpr (SHAPE == 0)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mp_bf16x8, a), __builtin_bit_cast(mp_bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(mp_bf16x8, a), __builtin_bit_cast(mp_bf16x8, b), c, 0, 0, 0);
}

// Operand i (0..7) of a tile of 32 keys x 128 dims (8 KiB).  K pattern: SHAPE 0 reads key 16 (i / 4) + lane % 16, chunk
// 4 (i % 4) + lane / 16; SHAPE 1 reads key lane % 32, chunk 2 i + lane / 32.  V pattern: two transposing reads.
template <int SHAPE, int SRC>
__device__ __forceinline__ mp_u32x4 mp_read(const unsigned char* tile, int i, int lane) {
  if constexpr (SRC == 1) {
    int row, chunk;
    if constexpr (SHAPE == 0) { row = (i >> 2) * 16 + (lane & 15); chunk = 4 * (i & 3) + (lane >> 4); }
    else { row = lane & 31; chunk = 2 * i + (lane >> 5); }
    return *(const mp_u32x4*)(tile + row * 256 + ((chunk ^ (row & 15)) << 4));
  } else {
    const int n = lane & 15;
    int key0, key1, dim, swz0, swz1;
    if constexpr (SHAPE == 0) {  // dims 16 i .. + 15, keys 4 (lane / 16) + n / 4 and 16 more
      key0 = 4 * (lane >> 4) + (n >> 2); key1 = key0 + 16; dim = 16 * i + 4 * (n & 3);
      swz0 = (key0 & 7) << 1; swz1 = (key1 & 7) << 1;
    } else {                     // dims 32 (i / 2) + lane % 32, keys 16 (i % 2) + 4 (lane / 32) + n / 4 and 8 more
      key0 = 16 * (i & 1) + 4 * (lane >> 5) + (n >> 2); key1 = key0 + 8; dim = 32 * (i >> 1) + 16 * ((lane >> 4) & 1) + 4 * (n & 3);
      swz0 = (key0 & 3) << 2; swz1 = (key1 & 3) << 2;
    }
    const int off = dim * 2;
    const unsigned char* p0 = tile + key0 * 256 + (((off >> 4) ^ swz0) << 4) + (off & 15);
    const unsigned char* p1 = tile + key1 * 256 + (((off >> 4) ^ swz1) << 4) + (off & 15);
    const mp_u32x2 lo = __builtin_bit_cast(mp_u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) mp_s16x4*)p0));
    const mp_u32x2 hi = __builtin_bit_cast(mp_u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) mp_s16x4*)p1));
    return (mp_u32x4){lo[0], lo[1], hi[0], hi[1]};
  }
}

extern __shared__ unsigned char mp_lds[];

template <int SHAPE, int SRC, int REUSE>
__global__ __launch_bounds__(256) void mfma_probe_kernel(int iters, unsigned long long* clocks, float* sink) {
  typedef typename MpAcc<SHAPE>::T acc_t;
  constexpr int PD = 4, TILES = 4;
  constexpr int NACC = SHAPE ? 4 : 8;  // accumulators in rotation: enough that no MFMA waits for the one before it
  static_assert(NACC % REUSE == 0, "an operand's MFMAs use distinct accumulators");
  const int lane = threadIdx.x & 63;
  for (int k = threadIdx.x; k < TILES * 8192 / 4; k += blockDim.x) {  // plausible bf16 values: the clock depends on the data
    uint32_t x = (uint32_t)k * 2654435761u + blockIdx.x;
    x ^= x >> 13;
    ((uint32_t*)mp_lds)[k] = (x & 0x007f007fu) | 0x3f003f00u | ((x & 0x100) << 7) | ((x & 0x200) << 22);
  }
  __syncthreads();
  mp_u32x4 b[REUSE];
  acc_t acc[NACC];
#pragma unroll
  for (int r = 0; r < REUSE; ++r) b[r] = (mp_u32x4){0x3f803f00u + lane + r, 0x3f003f80u ^ ((uint32_t)lane << 16), 0xbf803f80u, 0x3f80bf00u + r};
#pragma unroll
  for (int a = 0; a < NACC; ++a)
#pragma unroll
    for (int j = 0; j < MpAcc<SHAPE>::N; ++j) acc[a][j] = 0.f;
  const unsigned long long t0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  mp_u32x4 ops[PD];
#pragma unroll
  for (int i = 0; i < PD; ++i) {
    if constexpr (SRC != 0) ops[i] = mp_read<SHAPE, SRC>(mp_lds, i, lane);
    else ops[i] = (mp_u32x4){0x3f803f80u + i, 0x3f003f00u + lane, 0xbf80bf80u, 0x3f803f00u};
  }
  for (int it = 0; it < iters; ++it) {
    for (int t = 0; t < TILES; t += 2) {  // 16 operands per trip
      const unsigned char* tile = mp_lds + t * 8192;
      asm volatile("" ::: "memory");  // the reads stay inside the loop
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const mp_u32x4 a = ops[i % PD];
#pragma unroll
        for (int r = 0; r < REUSE; ++r) {
          const int ai = (i * REUSE + r) % NACC;
          acc[ai] = mp_mfma<SHAPE>(a, b[r], acc[ai]);
        }
        if constexpr (SRC != 0) {
          const int nx = i + PD;
          const unsigned char* tl = tile + (nx / 8) * 8192;
          if (tl >= mp_lds + TILES * 8192) tl -= TILES * 8192;
          ops[i % PD] = mp_read<SHAPE, SRC>(tl, nx % 8, lane);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  const unsigned long long t1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int a = 0; a < NACC; ++a)
#pragma unroll
    for (int j = 0; j < MpAcc<SHAPE>::N; ++j) s += acc[a][j];
#pragma unroll
  for (int i = 0; i < PD; ++i) s += __uint_as_float(ops[i][0] & 1u);
  if (s == 12345.678f) sink[0] = s;
  if (threadIdx.x == 0) {
    atomicAdd(clocks, t1 - t0);
    atomicAdd(clocks + 1, w1 - w0);
  }
}

// Returns the floating-point operations of the launch (0: bad arguments).  clocks[0] += shader-clock cycles, clocks[1] +=
// ticks of the 100 MHz wall clock, each summed over the workgroups: their quotient times 100 is the clock in MHz.
double launch_mfma_probe(hipStream_t stream, int shape, int source, int reuse, int waves_per_simd, int iters,
                         unsigned long long* clocks, float* sink) {
  if (iters <= 0 || waves_per_simd < 1 || waves_per_simd > 2) return 0.0;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 0.0;
  const int lds = waves_per_simd == 1 ? 96 * 1024 : 64 * 1024;  // one or two workgroups of four waves per CU
  const int blocks = cus * waves_per_simd;
#define RPA_MP(SH, SR, RE)                                                                                                   \
  if (shape == SH && source == SR && reuse == RE) {                                                                          \
    auto k = mfma_probe_kernel<SH, SR, RE>;                                                                                  \
    if (hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) return 0.0;      \
    hipLaunchKernelGGL(k, dim3(blocks), dim3(256), lds, stream, iters, clocks, sink);                                        \
    if (hipGetLastError() != hipSuccess) return 0.0;                                                                         \
    return (double)blocks * 4.0 * iters * 32.0 * RE * (SH ? 32768.0 : 16384.0);                                              \
  }
#define RPA_MP3(SH, SR) RPA_MP(SH, SR, 1) RPA_MP(SH, SR, 2) RPA_MP(SH, SR, 4)
  RPA_MP3(0, 0) RPA_MP3(0, 1) RPA_MP3(0, 2) RPA_MP3(1, 0) RPA_MP3(1, 1) RPA_MP3(1, 2)
#undef RPA_MP3
#undef RPA_MP
  return 0.0;
}

// Issue cost of one instruction kind beside a stream of 32x32x16 bf16 MFMAs on a lone wave per SIMD (how the 32x32 prefill
// kernel runs): every MFMA is followed by FILL independent v_fma_f32 and NX instructions of kind KIND.  An MFMA holds the
// matrix pipe for 32 cycles and the issue port for 8; what a slot's other instructions take beyond the remaining 24
// shows as cycles per MFMA above 32.
// KIND: 0 v_fma_f32, 1 v_exp_f32, 2 v_rcp_f32, 3 v_cvt_pk_bf16_f32, 4 v_max3_f32 (a dependent chain), 5 s_add_u32 (a
// dependent chain), 6 s_nop 0, 7 ds_read_b128, 8 ds_read_b64_tr_b16, 9 global_load_lds_dwordx4 (1 KiB, m0 written each time).
template <int KIND, int NX, int FILL>
__global__ __launch_bounds__(256) void issue_probe_kernel(int iters, unsigned long long* clocks, float* sink, const char* src) {
  __shared__ mp_u32x4 lds[2048];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < 2048; i += 256) lds[i] = (mp_u32x4){(uint32_t)i, 1u, 2u, 3u};
  __syncthreads();
  typedef MpAcc<1>::T acc_t;
  acc_t acc[2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[a][j] = 0.f;
  const mp_u32x4 A = {0x3f803f00u + lane, 0x3f003f80u, 0xbf803f80u, 0x3f80bf00u}, B = {0x3f803f80u, 0x3f003f00u + lane, 0xbf80bf80u, 0x3f803f00u};
  float x[8], y[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    x[i] = lane * 0.001f + i;
    y[i] = 0.5f + lane * 0.01f;
  }
  uint32_t sc = blockIdx.x, pk = 0;
  float mx = 0.f;
  mp_u32x4 rd[8];
  mp_u32x2 rt[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    rd[i] = (mp_u32x4){0u, 0u, 0u, 0u};
    rt[i] = (mp_u32x2){0u, 0u};
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) mp_u32x4*)lds;
  const uint32_t la = lds0 + (uint32_t)lane * 16;
  const uint32_t lb = lds0 + (uint32_t)((lane >> 4) * 512 + (lane & 15) * 8);
  const uint32_t ldst = __builtin_amdgcn_readfirstlane(lds0 + (uint32_t)(1024 + wave * 64) * 16);  // the wave's 1 KiB landing area
  const uint32_t voff = (uint32_t)lane * 16;
  const uint64_t g = (uint64_t)(src + (size_t)((blockIdx.x * 4 + wave) & 255) * 4096);  // 1 KiB of a 1 MiB buffer per wave
  const char* gbase = (const char*)(((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(g >> 32)) << 32) |
                                    (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)g));
  const unsigned long long t0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      acc[i % 2] = mp_mfma<1>(A, B, acc[i % 2]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int f = 0; f < FILL; ++f) {
        const int q = (i * FILL + f) % 8;
        x[q] = __builtin_fmaf(x[q], 1.0001f, 0.5f);
        asm volatile("" : "+v"(x[q]));
      }
#pragma unroll
      for (int f = 0; f < NX; ++f) {
        const int q = (i * NX + f) % 8;
        if constexpr (KIND == 0) asm volatile("v_fma_f32 %0, %0, %1, 0.5" : "+v"(y[q]) : "v"(x[7 - q]));
        else if constexpr (KIND == 1) asm volatile("v_exp_f32 %0, %0" : "+v"(y[q]));
        else if constexpr (KIND == 2) asm volatile("v_rcp_f32 %0, %0" : "+v"(y[q]));
        else if constexpr (KIND == 3) asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(pk) : "v"(y[q]), "v"(y[(q + 1) % 8]));
        else if constexpr (KIND == 4) asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(mx) : "v"(y[q]), "v"(y[(q + 1) % 8]));
        else if constexpr (KIND == 5) asm volatile("s_add_u32 %0, %0, 7" : "+s"(sc) : : "scc");
        else if constexpr (KIND == 6) asm volatile("s_nop 0");
        else if constexpr (KIND == 7) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(rd[q]) : "v"(la), "n"(1024 * (q % 8)));
        else if constexpr (KIND == 8) asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(rt[q]) : "v"(lb), "n"(2048 * (q % 8)));
        else asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(ldst), "v"(voff), "s"(gbase) : "memory");
      }
      if constexpr ((KIND == 7 || KIND == 8) && NX > 0) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(NX >= 4 ? 4 : NX) : "memory");
      if constexpr (KIND == 9 && NX > 0) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  const unsigned long long t1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  float r = (float)sc + __uint_as_float(pk) + mx;
#pragma unroll
  for (int i = 0; i < 8; ++i) r += x[i] + y[i] + __uint_as_float(rd[i][0] & 1u) + __uint_as_float(rt[i][0] & 1u);
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int j = 0; j < 16; ++j) r += acc[a][j];
  if (r == 12345.678f) sink[0] = r + __uint_as_float(lds[1024 + lane][0]);
  if (threadIdx.x == 0) {
    atomicAdd(clocks, t1 - t0);
    atomicAdd(clocks + 1, w1 - w0);
  }
}

// Returns the MFMAs every wave issues (0: bad arguments).  clocks as for launch_mfma_probe; src: 1 MiB of device memory.
long long launch_issue_probe(hipStream_t stream, int kind, int extra, int fill, int iters, unsigned long long* clocks, float* sink,
                             const void* src) {
  if (iters <= 0) return 0;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 0;
#define RPA_IP(K, X, F)                                                                                              \
  if (kind == K && extra == X && fill == F) {                                                                        \
    hipLaunchKernelGGL((issue_probe_kernel<K, X, F>), dim3(cus), dim3(256), 0, stream, iters, clocks, sink, (const char*)src); \
    return hipGetLastError() == hipSuccess ? 16ll * iters : 0;                                                       \
  }
#define RPA_IP4(K) RPA_IP(K, 0, 0) RPA_IP(K, 1, 0) RPA_IP(K, 2, 0) RPA_IP(K, 4, 0) RPA_IP(K, 0, 6) RPA_IP(K, 1, 6) RPA_IP(K, 2, 6) RPA_IP(K, 4, 6)
  RPA_IP4(0) RPA_IP4(1) RPA_IP4(2) RPA_IP4(3) RPA_IP4(4) RPA_IP4(5) RPA_IP4(6) RPA_IP4(7) RPA_IP4(8) RPA_IP4(9)
#undef RPA_IP4
#undef RPA_IP
  return 0;
}

}  // namespace rpa
