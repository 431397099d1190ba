// MFMA building blocks shared by the decode and prefill kernels (gfx950, wave64).
//
// Operand layouts of the two instructions used, for lane l with i = l & 15, g = l >> 4:
//   v_mfma_f32_16x16x32_bf16 : A[row i][k = 8g..8g+7], B[k = 8g..8g+7][col i], C[row 4g+j][col i] (j = 0..3)
//   v_mfma_f32_16x16x16_bf16 : A[row i][k = 4g..4g+3], B[k = 4g..4g+3][col i], C[row 4g+j][col i]
// The contraction index k may be permuted freely as long as A and B use the same permutation.
#pragma once
#include "rpa_common.h"

namespace rpa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Two floats -> packed bf16 pair (lo = a, hi = b), round to nearest even.
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  f32x2 v = {a, b};
  bf16x2 r = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(uint32_t, r);
}

// The 16-bit float type of a kernel's MFMA operands: bfloat16 (bf16 queries over bf16, fp8 or int8 pages), or IEEE half
// (float16 queries over float16 pages).  Same instruction shapes, operand layouts and accumulators either way; the
// operands travel as raw dwords.
template <int ET>
struct Half16;
template <>
struct Half16<RPA_BF16> {
  static constexpr uint32_t kOnes = 0x3F803F80u;  // (1, 1)
  static __device__ __forceinline__ uint32_t pack(float a, float b) { return pack_bf16(a, b); }
  static __device__ __forceinline__ f32x4 mfma32(u32x4 a, u32x4 b, f32x4 c) {  // 16x16x32
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(u32x2 a, u32x2 b, f32x4 c) {  // 16x16x16
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
  }
};
template <>
struct Half16<RPA_F16> {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
  typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
  static constexpr uint32_t kOnes = 0x3C003C00u;
  static __device__ __forceinline__ uint32_t pack(float a, float b) {  // round to nearest even
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const f32x2 v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
  }
  static __device__ __forceinline__ f32x4 mfma32(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(u32x2 a, u32x2 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
  }
};
// ... as chosen by the page dtype of a kernel instance.
template <int KVT>
using HalfOf = Half16<KVT == RPA_F16 ? RPA_F16 : RPA_BF16>;

// Four 8-bit codes in one dword -> four floats.
template <int KVT>
__device__ __forceinline__ void decode4(uint32_t w, float* f) {
  if constexpr (KVT == RPA_FP8_E4M3) {
    auto lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    auto hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    f[0] = lo[0]; f[1] = lo[1]; f[2] = hi[0]; f[3] = hi[1];
  } else {
    f[0] = (float)(int8_t)(w & 0xff);
    f[1] = (float)(int8_t)((w >> 8) & 0xff);
    f[2] = (float)(int8_t)((w >> 16) & 0xff);
    f[3] = (float)(int8_t)(w >> 24);
  }
}

// Eight 8-bit codes (two dwords) -> one bf16 MFMA operand of eight elements (exact: both code sets fit bf16).
template <int KVT>
__device__ __forceinline__ u32x4 codes8_to_bf16x8(uint32_t w0, uint32_t w1) {
  float f[8];
  decode4<KVT>(w0, f);
  decode4<KVT>(w1, f + 4);
  const u32x4 r = {pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7])};
  return r;
}

// XOR swizzle of 16-byte chunks inside an LDS row of ROW_BYTES so that 16 consecutive token rows
// read at the same logical chunk land on distinct bank groups.
template <int ROW_BYTES>
__device__ __forceinline__ int swz_key(int tok) {
  constexpr int NCH = ROW_BYTES / 16;
  if constexpr (NCH >= 16) return tok & 15;
  else if constexpr (NCH == 8) return ((tok >> 1) ^ ((tok & 1) << 2)) & 7;
  else if constexpr (NCH == 4) return (tok >> 2) & 3;
  else return 0;
}

// Maximum over the lanes l, l^16 (xor16_max) or l, l^32 (xor32_max), through the gfx950 row-swap instructions:
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its second,
// v_permlane32_swap the upper half of the first with the lower half of the second.  Fed two copies of v, the
// results are (own-or-partner, partner-or-own) in every lane.  Pure VALU: no LDS round trip as with ds_bpermute.
// Swizzle of the V half of a tile, which is read with transposing loads: 16 lanes fetch 32 contiguous bytes of
// each of 4 consecutive token rows.  With swz_key those four rows share two 32-byte bank groups (a 2-way
// conflict on every read); XOR-ing the chunk index with twice the row number spreads them over four.
template <int ROW_BYTES>
__device__ __forceinline__ int swz_key_v(int tok) {
  constexpr int NCH = ROW_BYTES / 16;
  if constexpr (NCH >= 16) return (tok & 7) << 1;
  else if constexpr (NCH == 8) return (tok & 3) << 1;
  else return 0;
}

__device__ __forceinline__ float xor16_max(float v) {
  const uint32_t u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor32_max(float v) {
  const uint32_t u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// One LDS DMA of 1 KiB (global_load_lds_dwordx4): every lane fetches 16 bytes from base + voff; lane L's bytes land at
// LDS byte address lds_addr + 16 L.  (An instruction offset would move the LDS address as well, so none is used.)
// Issued through inline assembly: the compiler neither tracks these loads nor orders its own waits around them, the
// kernels that use them state their waits themselves (wait_loads).
__device__ __forceinline__ void dma16(uint32_t lds_addr, uint32_t voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

// N such DMAs of one wave into consecutive 1 KiB blocks of LDS starting at lds_addr: m0 is set once and the instruction
// offsets u * 1024 select the block.  The offset is added to the global address as well, so the caller's lane offset
// voff[u] must already have u * 1024 taken out of it.
template <int N>
__device__ __forceinline__ void dma16_group(uint32_t lds_addr, const uint32_t (&voff)[N], const void* base) {
  static_assert(N == 1 || N == 2 || N == 4, "one, two or four instructions per group");
  if constexpr (N == 4)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %5\n\tglobal_load_lds_dwordx4 %2, %5 offset:1024\n\t"
                 "global_load_lds_dwordx4 %3, %5 offset:2048\n\tglobal_load_lds_dwordx4 %4, %5 offset:3072"
                 ::"s"(lds_addr), "v"(voff[0]), "v"(voff[1]), "v"(voff[2]), "v"(voff[3]), "s"(base) : "memory");
  else if constexpr (N == 2)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %3\n\tglobal_load_lds_dwordx4 %2, %3 offset:1024"
                 ::"s"(lds_addr), "v"(voff[0]), "v"(voff[1]), "s"(base) : "memory");
  else
    dma16(lds_addr, voff[0], base);
}

// Instruction u of such a group on its own (u < 4): m0 is set again, the instruction offset u * 1024 selects the block.
__device__ __forceinline__ void dma16_at(uint32_t lds_addr, int u, uint32_t voff, const void* base) {
  if (u == 0) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
  else if (u == 1) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:1024" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
  else if (u == 2) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:2048" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
  else asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:3072" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

// ... and with m0 left as the instruction before of the same group set it (u > 0).  Only for instruction streams in
// which nothing between the group's instructions writes m0: the compiler does so for indexed register moves, lane reads
// by a vector index and LDS DMA of its own, none of which the pinned steps that use this contain.
__device__ __forceinline__ void dma16_at_same_m0(int u, uint32_t voff, const void* base) {
  if (u == 1) asm volatile("global_load_lds_dwordx4 %0, %1 offset:1024" ::"v"(voff), "s"(base) : "memory");
  else if (u == 2) asm volatile("global_load_lds_dwordx4 %0, %1 offset:2048" ::"v"(voff), "s"(base) : "memory");
  else asm volatile("global_load_lds_dwordx4 %0, %1 offset:3072" ::"v"(voff), "s"(base) : "memory");
}

// ... with the non-temporal hint, for data no wave will ask for again (the pages a decode kernel streams): kept out
// of the caches' longer-lived lines, such a stream reads HBM measurably faster.
__device__ __forceinline__ void dma16_nt(uint32_t lds_addr, uint32_t voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

// One LDS DMA of 256 bytes (global_load_lds_dword): every lane fetches 4 bytes from base + voff; lane L's bytes land
// at LDS byte address lds_addr + 4 L.
__device__ __forceinline__ void dma4(uint32_t lds_addr, uint32_t voff, const void* base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(lds_addr), "v"(voff), "s"(base) : "memory");
}

// Waits until at most N of this wave's vector-memory loads are in flight (they complete in issue order).
template <int N>
__device__ __forceinline__ void wait_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// ... and then joins the workgroup barrier.
template <int N>
__device__ __forceinline__ void wait_loads_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// tanh through the hardware exp2: tanh(x) = 1 - 2 / (exp(2x) + 1).  Good to ~1e-6 relative, far inside
// the bf16 tolerance of the MFMA kernels (the fp32 kernel uses tanhf).
__device__ __forceinline__ float fast_tanh(float x) {
  const float e = __builtin_amdgcn_exp2f(x * 2.8853900817779268f);  // exp(2x)
  return 1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f);
}


// Online-softmax step of one 16-row block over NS 16-key sub-tiles held as S^T accumulators (lane = query row
// n, 4 keys 4*g4 + j per sub-tile).  Applies the soft cap if CAP, masks keys outside [row_lo, row_hi) if MASK,
// updates the running max / sum, and leaves the probabilities as packed 16-bit B operands (bf16, or half if ET says so).  The maximum is taken
// over the raw scores and scaled once (sc_mul > 0, so scaling commutes with max); each probability is then one
// fused multiply-add and one exp2.  Returns the factor the output accumulators must be multiplied by.
template <bool MASK, bool CAP, int NS, int ET = RPA_BF16>
__device__ __forceinline__ float softmax_step(f32x4 (&s_acc)[NS], float sc_mul, float cap_in, int tb, int g4,
                                              int row_lo, int row_hi, float& m_run, float& l_run,
                                              uint32_t (&pfrag)[NS][2]) {
  float mx = -INFINITY;
#pragma unroll
  for (int st = 0; st < NS; ++st) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float s = s_acc[st][j];
      if constexpr (CAP) s = fast_tanh(s * cap_in);
      if constexpr (MASK) {
        const int tok = tb + st * 16 + 4 * g4 + j;
        s = (tok >= row_lo && tok < row_hi) ? s : -INFINITY;
      }
      s_acc[st][j] = s;
      mx = fmaxf(mx, s);
    }
  }
  mx = xor32_max(xor16_max(mx)) * sc_mul;
  const float m_new = fmaxf(m_run, mx);
  const float m_use = (MASK && m_new == -INFINITY) ? 0.f : m_new;
  const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
  m_run = m_new;
  float psum = 0.f;
#pragma unroll
  for (int st = 0; st < NS; ++st) {
    float pr[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      pr[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[st][j], sc_mul, -m_use));
      psum += pr[j];
    }
    pfrag[st][0] = Half16<ET>::pack(pr[0], pr[1]);
    pfrag[st][1] = Half16<ET>::pack(pr[2], pr[3]);
  }
  l_run = l_run * alpha + psum;
  return alpha;
}

}  // namespace rpa
