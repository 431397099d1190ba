/*
 * rpa_oracle_c.c -- C restatement of the ragged-paged-attention path.  TEST INFRASTRUCTURE ONLY.
 *
 * Same algorithm as oracle/rpa_oracle.py (which documents the reference lines each convention
 * comes from: easydel/operations/kernels/ragged_page_attention.py:281-313 and :732-746 for the
 * operation, easydel/caching/ragged_page/cache.py:954-973 for the K-even / V-odd interleave,
 * easydel/inference/esurge/core/single_type_cache_manager.py:497 for the window), written as
 * plain loops in fp32 with OpenMP over (sequence, KV head).  It exists so that bench.py's
 * cpu_baseline leg can time the path on all host cores; tests/test_oracle_c.py pins it against
 * the float64 numpy oracle.  Nothing under easydel_amd/ links or loads it.
 *
 * Build: see oracle/Makefile (gcc -O3 -fopenmp -shared).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { RPA_F32 = 0, RPA_BF16 = 1, RPA_FP8_E4M3 = 2, RPA_INT8 = 3 };

static float e4m3_table[256];
static int e4m3_ready = 0;

static void init_tables(void) {
  if (e4m3_ready) return;
  for (int c = 0; c < 256; ++c) {
    int s = c >> 7, e = (c >> 3) & 15, m = c & 7;
    float v;
    if (e == 15 && m == 7) v = NAN;
    else if (e == 0) v = ldexpf(m / 8.0f, -6);
    else v = ldexpf(1.0f + m / 8.0f, e - 7);
    e4m3_table[c] = s ? -v : v;
  }
  e4m3_ready = 1;
}

static inline float bf16_to_f32(uint16_t b) {
  uint32_t u = ((uint32_t)b) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static int elem_bytes(int dt) { return dt == RPA_F32 ? 4 : dt == RPA_BF16 ? 2 : 1; }

/* Decode n elements of storage type dt into floats. */
static void decode_row(const void* src, int dt, int n, float* dst) {
  switch (dt) {
    case RPA_F32: memcpy(dst, src, (size_t)n * 4); break;
    case RPA_BF16: { const uint16_t* s = (const uint16_t*)src; for (int i = 0; i < n; ++i) dst[i] = bf16_to_f32(s[i]); break; }
    case RPA_FP8_E4M3: { const uint8_t* s = (const uint8_t*)src; for (int i = 0; i < n; ++i) dst[i] = e4m3_table[s[i]]; break; }
    default: { const int8_t* s = (const int8_t*)src; for (int i = 0; i < n; ++i) dst[i] = (float)s[i]; break; }
  }
}

int rpa_oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/*
 * out[T][Hq][D] float.  Rows of padded tokens and of sequences without queries or keys are zero.
 * Returns 0, or -1 on allocation failure.
 */
int rpa_oracle_attention(const void* q, int q_dtype, const void* kv_pages, int kv_dtype, const float* kv_scales,
                         const int32_t* context_lens, const int32_t* block_tables, const int32_t* qsl, int num_seqs,
                         float* out, int T, int S, int M, int P, int page_size, int Hq, int Hkv, int D, int C,
                         float scale, int window, float softcap, int num_threads) {
  (void)S; (void)P;
  init_tables();
  const int G = Hq / Hkv;
  const int eb = elem_bytes(kv_dtype), qb = elem_bytes(q_dtype);
  const size_t token_stride = (size_t)C * D * eb, page_stride = token_stride * page_size;
  memset(out, 0, (size_t)T * Hq * D * sizeof(float));
  int failed = 0;
  const int RB = 16; /* query tokens per block, bounds the score buffer */
#ifdef _OPENMP
  if (num_threads > 0) omp_set_num_threads(num_threads);
#endif
#pragma omp parallel
  {
    float* krow = (float*)malloc((size_t)D * 4);
    float* qblk = (float*)malloc((size_t)RB * G * D * 4);
    float* acc = (float*)malloc((size_t)RB * G * D * 4);
    float* sc = NULL;
    size_t sc_cap = 0;
#pragma omp for schedule(dynamic, 1) collapse(2)
    for (int i = 0; i < num_seqs; ++i) {
      for (int h = 0; h < Hkv; ++h) {
        const int q0 = qsl[i], q_len = qsl[i + 1] - q0, ctx = context_lens[i];
        if (q_len <= 0 || ctx <= 0 || !krow || !qblk || !acc) continue;
        const int32_t* bt = block_tables + (size_t)i * M;
        for (int r0 = 0; r0 < q_len; r0 += RB) {
          const int nr = (q_len - r0 < RB) ? q_len - r0 : RB;
          const int rows = nr * G;
          /* keys any row of the block can see */
          const int pos_first = ctx - q_len + r0, pos_last = ctx - q_len + r0 + nr - 1;
          int hi = pos_last + 1; if (hi > ctx) hi = ctx;
          int lo = 0; if (window > 0 && pos_first - window + 1 > 0) lo = pos_first - window + 1;
          if (hi <= lo) continue;
          const size_t need = (size_t)rows * (hi - lo);
          if (need > sc_cap) { free(sc); sc = (float*)malloc(need * 4); sc_cap = sc ? need : 0; }
          if (!sc) { failed = 1; continue; }
          for (int r = 0; r < nr; ++r)
            for (int g = 0; g < G; ++g)
              decode_row((const char*)q + ((size_t)(q0 + r0 + r) * Hq + (size_t)h * G + g) * D * qb, q_dtype, D,
                         qblk + (size_t)(r * G + g) * D);
          /* scores */
          for (int j = lo; j < hi; ++j) {
            const int page = bt[j / page_size];
            const char* tok = (const char*)kv_pages + (size_t)page * page_stride + (size_t)(j % page_size) * token_stride;
            decode_row(tok + (size_t)(2 * h) * D * eb, kv_dtype, D, krow);
            const float ks = kv_scales ? kv_scales[(size_t)page * C + 2 * h] : 1.0f;
            for (int row = 0; row < rows; ++row) {
              const float* qr = qblk + (size_t)row * D;
              float dot = 0.f;
              for (int d = 0; d < D; ++d) dot += qr[d] * krow[d];
              float s = dot * ks * scale;
              if (softcap > 0.f) s = softcap * tanhf(s / softcap);
              const int pos = ctx - q_len + r0 + row / G;
              const int visible = (j <= pos) && (window <= 0 || j > pos - window);
              sc[(size_t)row * (hi - lo) + (j - lo)] = visible ? s : -INFINITY;
            }
          }
          /* softmax per row */
          for (int row = 0; row < rows; ++row) {
            float* s = sc + (size_t)row * (hi - lo);
            float m = -INFINITY;
            for (int j = 0; j < hi - lo; ++j) if (s[j] > m) m = s[j];
            if (!(m > -INFINITY)) m = 0.f;
            float l = 0.f;
            for (int j = 0; j < hi - lo; ++j) { s[j] = expf(s[j] - m); l += s[j]; }
            const float inv = l > 0.f ? 1.f / l : 0.f;
            for (int j = 0; j < hi - lo; ++j) s[j] *= inv;
          }
          /* P.V */
          memset(acc, 0, (size_t)rows * D * 4);
          for (int j = lo; j < hi; ++j) {
            const int page = bt[j / page_size];
            const char* tok = (const char*)kv_pages + (size_t)page * page_stride + (size_t)(j % page_size) * token_stride;
            decode_row(tok + (size_t)(2 * h + 1) * D * eb, kv_dtype, D, krow);
            const float vs = kv_scales ? kv_scales[(size_t)page * C + 2 * h + 1] : 1.0f;
            for (int row = 0; row < rows; ++row) {
              const float w = sc[(size_t)row * (hi - lo) + (j - lo)] * vs;
              if (w == 0.f) continue;
              float* a = acc + (size_t)row * D;
              for (int d = 0; d < D; ++d) a[d] += w * krow[d];
            }
          }
          for (int r = 0; r < nr; ++r)
            for (int g = 0; g < G; ++g)
              memcpy(out + ((size_t)(q0 + r0 + r) * Hq + (size_t)h * G + g) * D, acc + (size_t)(r * G + g) * D, (size_t)D * 4);
        }
      }
    }
    free(krow); free(qblk); free(acc); free(sc);
  }
  return failed ? -1 : 0;
}

/* The ragged (v3) write: token rows of sequence i go to positions [ctx_i - q_len_i, ctx_i) of its pages. */
void rpa_oracle_scatter_ragged(const void* key, const void* value, void* kv_pages, const int32_t* context_lens,
                               const int32_t* block_tables, const int32_t* qsl, int num_seqs, int M, int page_size,
                               int Hkv, int D, int C, int elem) {
  const size_t hb = (size_t)D * elem, token_stride = (size_t)C * hb, page_stride = token_stride * page_size;
  for (int i = 0; i < num_seqs; ++i) {
    const int q0 = qsl[i], q_len = qsl[i + 1] - q0, ctx = context_lens[i];
    for (int r = 0; r < q_len; ++r) {
      const int pos = ctx - q_len + r;
      if (pos < 0) continue;
      const int page = block_tables[(size_t)i * M + pos / page_size];
      char* row = (char*)kv_pages + (size_t)page * page_stride + (size_t)(pos % page_size) * token_stride;
      for (int h = 0; h < Hkv; ++h) {
        memcpy(row + (size_t)(2 * h) * hb, (const char*)key + ((size_t)(q0 + r) * Hkv + h) * hb, hb);
        memcpy(row + (size_t)(2 * h + 1) * hb, (const char*)value + ((size_t)(q0 + r) * Hkv + h) * hb, hb);
      }
    }
  }
}
