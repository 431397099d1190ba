// Stand-alone host of the C ABI: no Python, no PyTorch in the process.  Loads librpa_hip.so with dlopen, allocates
// with hipMalloc, runs the small float32 mixed batch of tests/golden/attention_c1_fp32.npz (handed over as a flat
// binary written by the pytest that starts this program) through rpa_ragged_paged_attention and compares with the
// expected output at 1e-5; then the fused write + attention call on a copy of the pool whose new rows were blanked
// (the call must put them back bit for bit and give the same output); then the same batch rounded to bf16 through
// the matrix-core kernels (against the float32 fixture, so only at the bf16 tolerance plus the rounding of the
// inputs).  Exit status 0 and a last line "abi_host OK" on success.
//
//   abi_host <path to librpa_hip.so> <input.bin>
// input.bin: int32 {magic 0x52504131, T, S, M, P, page_size, Hq, Hkv, D}, float32 softmax_scale, then float32
// q[T][Hq][D], float32 pages[P][page_size][2*Hkv][D], int32 context_lens[S], block_tables[S][M], query_start_loc[S+1],
// num_seqs[1], float32 expected[T][Hq][D].
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../include/rpa_hip.h"

#define HIP_OK(x)                                                                          \
  do {                                                                                     \
    hipError_t e_ = (x);                                                                   \
    if (e_ != hipSuccess) {                                                                \
      std::fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                  \
      return 2;                                                                            \
    }                                                                                      \
  } while (0)

static uint16_t to_bf16(float f) {  // round to nearest even
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
static float from_bf16(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

template <typename T>
static bool read_vec(FILE* f, std::vector<T>& v, size_t n) {
  v.resize(n);
  return std::fread(v.data(), sizeof(T), n, f) == n;
}

int main(int argc, char** argv) {
  if (argc != 3) {
    std::fprintf(stderr, "usage: %s <librpa_hip.so> <input.bin>\n", argv[0]);
    return 2;
  }
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!lib) {
    std::fprintf(stderr, "dlopen: %s\n", dlerror());
    return 2;
  }
  auto ws_bytes = (decltype(&rpa_attention_workspace_bytes))dlsym(lib, "rpa_attention_workspace_bytes");
  auto attention = (decltype(&rpa_ragged_paged_attention))dlsym(lib, "rpa_ragged_paged_attention");
  auto attention_v3 = (decltype(&rpa_ragged_paged_attention_v3))dlsym(lib, "rpa_ragged_paged_attention_v3");
  auto last_error = (decltype(&rpa_last_error))dlsym(lib, "rpa_last_error");
  auto version = (decltype(&rpa_version))dlsym(lib, "rpa_version");
  if (!ws_bytes || !attention || !attention_v3 || !last_error || !version) {
    std::fprintf(stderr, "missing symbol: %s\n", dlerror());
    return 2;
  }
  FILE* f = std::fopen(argv[2], "rb");
  if (!f) {
    std::perror(argv[2]);
    return 2;
  }
  int32_t hdr[9];
  float scale;
  if (std::fread(hdr, 4, 9, f) != 9 || hdr[0] != 0x52504131 || std::fread(&scale, 4, 1, f) != 1) {
    std::fprintf(stderr, "bad header\n");
    return 2;
  }
  const int T = hdr[1], S = hdr[2], M = hdr[3], P = hdr[4], pg = hdr[5], Hq = hdr[6], Hkv = hdr[7], D = hdr[8];
  const int C = 2 * Hkv;
  const size_t nq = (size_t)T * Hq * D, npool = (size_t)P * pg * C * D;
  std::vector<float> q, pool, expected;
  std::vector<int32_t> ctx, bt, qsl, nseq;
  if (!read_vec(f, q, nq) || !read_vec(f, pool, npool) || !read_vec(f, ctx, S) || !read_vec(f, bt, (size_t)S * M) ||
      !read_vec(f, qsl, S + 1) || !read_vec(f, nseq, 1) || !read_vec(f, expected, nq)) {
    std::fprintf(stderr, "short input file\n");
    return 2;
  }
  std::fclose(f);
  std::printf("librpa_hip %s: T=%d S=%d M=%d P=%d page=%d Hq=%d Hkv=%d D=%d\n", version(), T, S, M, P, pg, Hq, Hkv, D);

  int32_t *d_ctx, *d_bt, *d_qsl, *d_nseq, *d_dist;
  HIP_OK(hipMalloc(&d_ctx, S * 4));
  HIP_OK(hipMalloc(&d_bt, (size_t)S * M * 4));
  HIP_OK(hipMalloc(&d_qsl, (S + 1) * 4));
  HIP_OK(hipMalloc(&d_nseq, 4));
  HIP_OK(hipMalloc(&d_dist, 12));
  HIP_OK(hipMemcpy(d_ctx, ctx.data(), S * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_bt, bt.data(), (size_t)S * M * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_qsl, qsl.data(), (S + 1) * 4, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_nseq, nseq.data(), 4, hipMemcpyHostToDevice));
  const int32_t dist[3] = {0, 0, nseq[0]};
  HIP_OK(hipMemcpy(d_dist, dist, 12, hipMemcpyHostToDevice));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  // new K/V rows of every query token, taken out of the pool (token t of sequence i sits at position ctx_i - q_len_i + r)
  std::vector<float> new_k((size_t)T * Hkv * D), new_v((size_t)T * Hkv * D), blanked = pool;
  for (int i = 0; i < nseq[0]; ++i) {
    const int q_len = qsl[i + 1] - qsl[i];
    for (int r = 0; r < q_len; ++r) {
      const int pos = ctx[i] - q_len + r, t = qsl[i] + r;
      if (pos < 0) continue;
      const size_t row = ((size_t)bt[(size_t)i * M + pos / pg] * pg + pos % pg) * C * D;
      for (int h = 0; h < Hkv; ++h)
        for (int d = 0; d < D; ++d) {
          new_k[((size_t)t * Hkv + h) * D + d] = pool[row + (size_t)(2 * h) * D + d];
          new_v[((size_t)t * Hkv + h) * D + d] = pool[row + (size_t)(2 * h + 1) * D + d];
          blanked[row + (size_t)(2 * h) * D + d] = 1e30f;
          blanked[row + (size_t)(2 * h + 1) * D + d] = -1e30f;
        }
    }
  }

  int failures = 0;
  for (int pass = 0; pass < 2; ++pass) {  // 0: float32 (the fp32 kernel), 1: bf16 (the matrix-core kernels)
    const int dt = pass == 0 ? RPA_F32 : RPA_BF16;
    const size_t eb = pass == 0 ? 4 : 2;
    std::vector<uint16_t> q16, pool16, blank16, k16, v16;
    const void *hq = q.data(), *hpool = pool.data(), *hblank = blanked.data(), *hk = new_k.data(), *hv = new_v.data();
    if (pass == 1) {
      auto conv = [](const std::vector<float>& a, std::vector<uint16_t>& b) {
        b.resize(a.size());
        for (size_t k = 0; k < a.size(); ++k) b[k] = to_bf16(a[k]);
      };
      conv(q, q16); conv(pool, pool16); conv(blanked, blank16); conv(new_k, k16); conv(new_v, v16);
      hq = q16.data(); hpool = pool16.data(); hblank = blank16.data(); hk = k16.data(); hv = v16.data();
    }
    void *d_q, *d_pool, *d_out, *d_ws, *d_k, *d_v;
    const size_t wsb = ws_bytes(T, S, M, pg, Hq, Hkv, D, dt, dt);
    HIP_OK(hipMalloc(&d_q, nq * eb));
    HIP_OK(hipMalloc(&d_pool, npool * eb));
    HIP_OK(hipMalloc(&d_out, nq * eb));
    HIP_OK(hipMalloc(&d_ws, wsb));
    HIP_OK(hipMalloc(&d_k, new_k.size() * eb));
    HIP_OK(hipMalloc(&d_v, new_v.size() * eb));
    HIP_OK(hipMemcpy(d_q, hq, nq * eb, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_k, hk, new_k.size() * eb, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_v, hv, new_v.size() * eb, hipMemcpyHostToDevice));
    const float tol = pass == 0 ? 1e-5f : 3e-2f;  // bf16: 2e-2 of the kernel plus the rounding of the inputs
    std::vector<unsigned char> first_out(nq * eb);
    for (int fused = 0; fused < 2; ++fused) {
      HIP_OK(hipMemcpy(d_pool, fused ? hblank : hpool, npool * eb, hipMemcpyHostToDevice));
      HIP_OK(hipMemset(d_out, 0xff, nq * eb));
      int rc;
      if (!fused)
        rc = attention(stream, d_q, d_pool, nullptr, d_ctx, d_bt, d_qsl, d_nseq, d_out, d_ws, wsb, T, S, M, P, pg, Hq, Hkv, D, D, C,
                       dt, dt, scale, 0, 0.f, nullptr);
      else
        rc = attention_v3(stream, d_q, d_k, d_v, d_pool, d_ctx, d_bt, d_qsl, d_dist, d_out, d_ws, wsb, T, S, M, P, pg, Hq, Hkv, D,
                          D, C, dt, dt, scale, 0, 0.f, nullptr);
      if (rc != 0) {
        std::fprintf(stderr, "call failed (%d): %s\n", rc, last_error());
        return 1;
      }
      HIP_OK(hipStreamSynchronize(stream));
      std::vector<unsigned char> raw(nq * eb);
      HIP_OK(hipMemcpy(raw.data(), d_out, nq * eb, hipMemcpyDeviceToHost));
      double worst = 0;
      for (size_t k = 0; k < nq; ++k) {
        const float g = pass == 0 ? ((const float*)raw.data())[k] : from_bf16(((const uint16_t*)raw.data())[k]);
        const double e = std::fabs((double)g - (double)expected[k]);
        if (!(e <= worst)) worst = e;  // NaN counts as a failure
      }
      const bool ok = worst <= tol;
      std::printf("%s %s: max-abs %.3e (tolerance %.0e) %s\n", pass == 0 ? "float32" : "bf16", fused ? "fused write + attention" : "attention",
                  worst, (double)tol, ok ? "ok" : "FAILED");
      failures += !ok;
      if (!fused) first_out = raw;
      else {
        if (raw != first_out) {
          std::printf("  fused call's output differs from the read-only call's: FAILED\n");
          ++failures;
        }
        std::vector<unsigned char> back(npool * eb);
        HIP_OK(hipMemcpy(back.data(), d_pool, npool * eb, hipMemcpyDeviceToHost));
        if (std::memcmp(back.data(), hpool, npool * eb) != 0) {
          std::printf("  pages after the fused write differ from the original pool: FAILED\n");
          ++failures;
        }
      }
    }
    for (void* ptr : {d_q, d_pool, d_out, d_ws, d_k, d_v}) (void)hipFree(ptr);
  }
  if (failures) {
    std::printf("abi_host: %d check(s) failed\n", failures);
    return 1;
  }
  std::printf("abi_host OK\n");
  return 0;
}
