/* CPU restatement (plain C, OpenMP over output rows) of the MLX affine-quantised
 * operators on the hot path.  TEST INFRASTRUCTURE ONLY: linked by tests/, by
 * __graft_entry__.smoke() and by the cpu_baseline leg of bench.py; never by the
 * shipped package.
 *
 * Follows the operator documentation carried by the reference:
 *   packing / quantise      .typings/mlx/core/__init__.pyi:4166-4188
 *   dequantise  w = s*q + b .typings/mlx/core/__init__.pyi:2444-2450
 *   quantized_matmul(x, w, scales, biases, transpose=True)
 *                           .typings/mlx/core/__init__.pyi:4198-4234
 * The arithmetic itself lives in mlx 0.32.0 (uv.lock:1376-1378), which is not
 * vendored; accumulation is float32 like a SIMD CPU kernel would do.
 * Pins: checked against the numpy restatement (oracle/affine.py), against dense
 * float64 matmul of the dequantised matrix, and on hand-packed words.
 */
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline float bf2f(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint16_t f2bf(float f) { /* round to nearest even */
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

int ref_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void ref_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}

void ref_unpack_codes(const uint32_t* w, uint8_t* out, int64_t n_words, int bits) {
  const int per = 32 / bits;
  const uint32_t mask = (1u << bits) - 1u;
  for (int64_t i = 0; i < n_words; ++i)
    for (int j = 0; j < per; ++j) out[i * per + j] = (uint8_t)((w[i] >> (bits * j)) & mask);
}

/* two_roundings: bf16(bf16(s*q) + b); else bf16(fma(s, q, b)) */
void ref_dequantize(const uint32_t* w, const uint16_t* scales, const uint16_t* biases,
                    uint16_t* out, int64_t rows, int K, int bits, int two_roundings) {
  const int per = 32 / bits, wpr = K / per, G = K / 64;
  const uint32_t mask = (1u << bits) - 1u;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r)
    for (int c = 0; c < wpr; ++c) {
      const uint32_t v = w[r * wpr + c];
      const int g = (c * per) / 64;
      const float s = bf2f(scales[r * G + g]), b = bf2f(biases[r * G + g]);
      for (int j = 0; j < per; ++j) {
        const float q = (float)((v >> (bits * j)) & mask);
        float o;
        if (two_roundings)
          o = bf2f(f2bf(s * q)) + b;
        else
          o = (float)((double)s * (double)q + (double)b);
        out[r * (int64_t)K + c * per + j] = f2bf(o);
      }
    }
}

/* y[M,N] = x[M,K] @ dq(w)[N,K]^T ; x,y bf16 bits ; float32 accumulation per row.
 * Per group: acc += s * sum(x*q) + b * sum(x)  (the factored form of sum x*(s*q+b)). */
void ref_qmm_t(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
               const uint16_t* biases, uint16_t* y, int M, int N, int K, int bits) {
  const int per = 32 / bits, wpr = K / per, G = K / 64, wpg = 64 / per;
  const uint32_t mask = (1u << bits) - 1u;
#pragma omp parallel
  {
    float xf[64];
#pragma omp for schedule(static)
    for (int n = 0; n < N; ++n) {
      for (int m = 0; m < M; ++m) {
        float acc = 0.f;
        for (int g = 0; g < G; ++g) {
          const float s = bf2f(scales[(int64_t)n * G + g]), b = bf2f(biases[(int64_t)n * G + g]);
          float xs = 0.f, xq = 0.f;
          for (int k = 0; k < 64; ++k) {
            xf[k] = bf2f(x[(int64_t)m * K + g * 64 + k]);
            xs += xf[k];
          }
          const uint32_t* wp = w + (int64_t)n * wpr + g * wpg;
          for (int c = 0; c < wpg; ++c) {
            const uint32_t v = wp[c];
            for (int j = 0; j < per; ++j)
              xq += xf[c * per + j] * (float)((v >> (bits * j)) & mask);
          }
          acc += s * xq + b * xs;
        }
        y[(int64_t)m * N + n] = f2bf(acc);
      }
    }
  }
}
