/*
 * CPU oracle, C restatement of the GlowQ W4A16 hot path.  TEST INFRASTRUCTURE ONLY: linked by
 * tests, the smoke check and the benchmark's cpu_baseline leg; never by the product library.
 *
 * Follows (paths relative to the reference checkout):
 *   oracle_unpack_u4        src/cuda_w4a16/csrc/gemv_w4a16.cu:16-32   nibble (k & 7) of word (k >> 3)
 *   oracle_dequant_f16      src/cuda_w4a16/csrc/gemm_w4a16.cu:19-50   fp16((code - z) * s), one rounding
 *   oracle_gemv_f32acc      src/cuda_w4a16/csrc/gemv_w4a16.cu:34-142  sum_k (code - z) * s * x, fp32
 *                           accumulate, weight never rounded to fp16, fp16 output
 *   oracle_gemm_deq_f32acc  src/cuda_w4a16/csrc/gemm_w4a16.cu:76-135  dequant to fp16 then matmul
 *   oracle_shared_proj      src/step3_eval_dataset.py:484    r = fp16(x R^T)
 *   oracle_add_correction   src/step3_eval_dataset.py:506-511 z += alpha * fp16(r L^T), fp16 add
 *
 * Pinned by tests/test_oracle_c.py: bit-exact dequant against the golden vectors under
 * tests/golden, and agreement with the numpy oracle (float64 accumulate) on seeded inputs.
 * Build: make -C oracle   (gcc -O2 -fopenmp -shared -fPIC).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- IEEE binary16 <-> binary32, exact / round-to-nearest-even ------------------------ */
static inline float h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static inline uint16_t f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7FFFFFFFu;
  if (absx >= 0x7F800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7C00u | ((absx > 0x7F800000u) ? 0x200u : 0u));
  }
  if (absx >= 0x477FF000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7C00u);
  }
  if (absx < 0x33000001u) { /* < 2^-25 (or exactly 2^-25: ties to even = 0) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t m = (absx & 0x7FFFFFu) | 0x800000u;
  uint32_t shift, half;
  if (e < -14) { /* subnormal result */
    shift = (uint32_t)(13 + (-14 - e));
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) ++q;
    return (uint16_t)(sign | q);
  }
  uint32_t q = ((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3FFu);
  uint32_t rem = m & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q; /* carry may bump the exponent: fine */
  return (uint16_t)(sign | q);
}

uint16_t oracle_f2h(float f) { return f2h(f); }
float oracle_h2f(uint16_t h) { return h2f(h); }

static inline uint32_t unpack_u4(const int32_t* row, int64_t idx) {
  return ((uint32_t)row[idx >> 3] >> (4 * (idx & 7))) & 0xFu;
}

void oracle_unpack_u4(const int32_t* packed, int64_t rows, int64_t ld_i32, int64_t total, uint8_t* out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t k = 0; k < total; ++k) out[r * total + k] = (uint8_t)unpack_u4(packed + r * ld_i32, k);
}

void oracle_dequant_f16(const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros, uint16_t* out,
                        int64_t N, int64_t K, int group_size, int64_t ldw_i32, int64_t lds, int64_t ldz_i32) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t k = 0; k < K; ++k) {
      int64_t g = k / group_size;
      float c = (float)unpack_u4(qweight + n * ldw_i32, k);
      float z = (float)unpack_u4(qzeros + n * ldz_i32, g);
      float s = h2f(scales[n * lds + g]);
      out[n * K + k] = f2h((c - z) * s);
    }
  }
}

/* y[m,n] = fp16( sum_k (code - z) * s * x[m,k] ), fp32 accumulate, sequential in k. */
void oracle_gemv_f32acc(const uint16_t* x, const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros,
                        uint16_t* y, int64_t M, int64_t K, int64_t N, int group_size, int64_t ldw_i32,
                        int64_t lds, int64_t ldz_i32) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t m = 0; m < M; ++m) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        int64_t g = k / group_size;
        float c = (float)unpack_u4(qweight + n * ldw_i32, k);
        float z = (float)unpack_u4(qzeros + n * ldz_i32, g);
        float s = h2f(scales[n * lds + g]);
        acc += (c - z) * s * h2f(x[m * K + k]);
      }
      y[m * N + n] = f2h(acc);
    }
  }
}

/* Same sum in double with no output rounding: the yardstick for error measurements. */
void oracle_linear_f64(const uint16_t* x, const int32_t* qweight, const uint16_t* scales, const int32_t* qzeros,
                       double* y, int64_t M, int64_t K, int64_t N, int group_size, int64_t ldw_i32, int64_t lds,
                       int64_t ldz_i32) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t m = 0; m < M; ++m) {
      double acc = 0.0;
      for (int64_t g0 = 0; g0 < K; g0 += group_size) {
        int64_t g = g0 / group_size;
        double z = (double)unpack_u4(qzeros + n * ldz_i32, g);
        double s = (double)h2f(scales[n * lds + g]);
        double part = 0.0;
        int64_t kend = g0 + group_size < K ? g0 + group_size : K;
        for (int64_t k = g0; k < kend; ++k)
          part += ((double)unpack_u4(qweight + n * ldw_i32, k) - z) * (double)h2f(x[m * K + k]);
        acc += part * s;
      }
      y[m * N + n] = acc;
    }
  }
}

/* dequantise each row to fp16 first (one rounding), then dot with fp32 accumulate. */
void oracle_gemm_deq_f32acc(const uint16_t* x, const int32_t* qweight, const uint16_t* scales,
                            const int32_t* qzeros, uint16_t* y, int64_t M, int64_t K, int64_t N, int group_size,
                            int64_t ldw_i32, int64_t lds, int64_t ldz_i32) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t m = 0; m < M; ++m) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        int64_t g = k / group_size;
        float c = (float)unpack_u4(qweight + n * ldw_i32, k);
        float z = (float)unpack_u4(qzeros + n * ldz_i32, g);
        float s = h2f(scales[n * lds + g]);
        float w = h2f(f2h((c - z) * s));
        acc += w * h2f(x[m * K + k]);
      }
      y[m * N + n] = f2h(acc);
    }
  }
}

/* r[m,j] = fp16( sum_k x[m,k] * R[j,k] ) */
void oracle_shared_proj(const uint16_t* x, const uint16_t* R, uint16_t* r, int64_t M, int64_t K, int64_t rank) {
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < rank; ++j) {
    for (int64_t m = 0; m < M; ++m) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) acc += h2f(x[m * K + k]) * h2f(R[j * K + k]);
      r[m * rank + j] = f2h(acc);
    }
  }
}

/* z[m,n] = fp16( z[m,n] + alpha * fp16( sum_j r[m,j] * L[n,j] ) ) */
void oracle_add_correction(uint16_t* z, const uint16_t* r, const uint16_t* L, float alpha, int64_t M, int64_t N,
                           int64_t rank) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t m = 0; m < M; ++m) {
      float acc = 0.0f;
      for (int64_t j = 0; j < rank; ++j) acc += h2f(r[m * rank + j]) * h2f(L[n * rank + j]);
      float svd = h2f(f2h(acc));
      z[m * N + n] = f2h(h2f(z[m * N + n]) + alpha * svd);
    }
  }
}
