/*
 * CPU restatement (plain C + OpenMP) of the two device computations on the
 * dflash-mlx target-verify hot path.  TEST INFRASTRUCTURE: only the test-suite,
 * the smoke entry and the benchmark's cpu_baseline leg load this library; the
 * shipped package never calls it.
 *
 *   oracle_qmm_m16      y = x . (s*q + b)^T          verify_qmm.py:66-116 (math),
 *                                                     :154-156, 226-230, 314 (K-split)
 *   oracle_tape_replay  S <- g_t*S + k_t (x) d_t      kernels.py:244-293 (kernel form),
 *                                                     :328-358 (array-op form)
 *
 * bf16 values travel as uint16 bit patterns.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = ((uint32_t)h) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static inline float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

/*
 * x       [16, K]    bf16 bits
 * w       [N, K/8]   uint32, element k of row n in word k>>3 at bit 4*(k&7)
 * scales, biases [N, K/gs] bf16 bits
 * y_f32   [16, N]    fp32 result BEFORE the final rounding (caller may round)
 * y_bf16  [16, N]    bf16 bits of the rounded result (nullable)
 * flavour 0: exact affine weights, double accumulation
 *         1: reference-kernel arithmetic: w~ = bf16(float(q)*s + b), fp32
 *            accumulation per K-slice, fp32 sum of k_parts partials
 */
int oracle_qmm_m16(const uint16_t* x, const uint32_t* w, const uint16_t* scales,
                   const uint16_t* biases, float* y_f32, uint16_t* y_bf16, int M, int K, int N,
                   int gs, int flavour, int k_parts) {
  if (K % 8 || K % gs || k_parts < 1 || K % k_parts) return -1;
  const int G = K / gs;
  float* xf = (float*)malloc(sizeof(float) * (size_t)M * K);
  if (!xf) return -2;
  for (size_t i = 0; i < (size_t)M * K; ++i) xf[i] = bf16_to_f32(x[i]);
  const int ks = K / k_parts;
#pragma omp parallel
  {
    float* wrow = (float*)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(static)
    for (int n = 0; n < N; ++n) {
      const uint32_t* wr = w + (size_t)n * (K / 8);
      for (int k = 0; k < K; ++k) {
        const uint32_t q = (wr[k >> 3] >> (4 * (k & 7))) & 0xFu;
        const float s = bf16_to_f32(scales[(size_t)n * G + k / gs]);
        const float b = bf16_to_f32(biases[(size_t)n * G + k / gs]);
        if (flavour == 1) {
          wrow[k] = round_bf16((float)q * s + b);
        } else {
          wrow[k] = (float)((double)q * (double)s + (double)b); /* exact: <= 20 significant bits */
        }
      }
      for (int m = 0; m < M; ++m) {
        const float* xr = xf + (size_t)m * K;
        float out;
        if (flavour == 1) {
          float total = 0.f;
          for (int p = 0; p < k_parts; ++p) {
            float acc = 0.f;
            for (int k = p * ks; k < (p + 1) * ks; ++k) acc += xr[k] * wrow[k];
            total += acc;
          }
          out = total;
        } else {
          double acc = 0.0;
          for (int k = 0; k < K; ++k) acc += (double)xr[k] * (double)wrow[k];
          out = (float)acc;
        }
        y_f32[(size_t)m * N + n] = out;
        if (y_bf16) y_bf16[(size_t)m * N + n] = f32_to_bf16(out);
      }
    }
    free(wrow);
  }
  free(xf);
  return 0;
}

/*
 * slots independent (layer*batch) problems, each:
 *   tape  [T, Hv, Dv] bf16 bits (tape_f32 == 0) or fp32 (tape_f32 == 1)
 *   k     [T, Hk, Dk] bf16 bits
 *   g     [T, Hv] fp32 (g_per_dk == 0) or [T, Hv, Dk] fp32 (g_per_dk == 1)
 *   state [Hv, Dv, Dk] fp32, Dk contiguous
 *   steps[slot] in [0, T]: number of leading tape steps applied
 *   mask  [T] bytes per slot, nullable; a zero byte skips the step
 * Step form (kernels.py:273-284): s = s*g; s = s + k*delta  (fp32; the
 * reference's per-step round-trip through the state dtype is the identity for
 * an fp32 state).
 */
int oracle_tape_replay(const void* tape, const uint16_t* k, const float* g, const float* state_in,
                       float* state_out, const int32_t* steps, const uint8_t* mask, int slots,
                       int T, int Hk, int Hv, int Dk, int Dv, int tape_f32, int g_per_dk) {
  if (Hv % Hk) return -1;
  const int rf = Hv / Hk;
#pragma omp parallel for collapse(2) schedule(static)
  for (int sl = 0; sl < slots; ++sl) {
    for (int hv = 0; hv < Hv; ++hv) {
      const int hk = hv / rf;
      const size_t sbase = ((size_t)sl * Hv + hv) * (size_t)Dv * Dk;
      float* so = state_out + sbase;
      memcpy(so, state_in + sbase, sizeof(float) * (size_t)Dv * Dk);
      int a = steps ? steps[sl] : T;
      if (a > T) a = T;
      for (int t = 0; t < a; ++t) {
        if (mask && !mask[(size_t)sl * T + t]) continue;
        const uint16_t* kt = k + (((size_t)sl * T + t) * Hk + hk) * Dk;
        const size_t toff = (((size_t)sl * T + t) * Hv + hv) * Dv;
        const float* gv = g_per_dk ? g + (((size_t)sl * T + t) * Hv + hv) * Dk : NULL;
        const float gs_ = g_per_dk ? 0.f : g[((size_t)sl * T + t) * Hv + hv];
        for (int dv = 0; dv < Dv; ++dv) {
          const float d = tape_f32 ? ((const float*)tape)[toff + dv]
                                   : bf16_to_f32(((const uint16_t*)tape)[toff + dv]);
          float* row = so + (size_t)dv * Dk;
          for (int dk = 0; dk < Dk; ++dk) {
            float s = row[dk] * (g_per_dk ? gv[dk] : gs_);
            s = s + bf16_to_f32(kt[dk]) * d;
            row[dk] = s;
          }
        }
      }
    }
  }
  return 0;
}

int oracle_num_threads(void) {
  int n = 1;
#ifdef _OPENMP
#pragma omp parallel
  {
#pragma omp single
    n = __builtin_omp_get_num_threads();
  }
#endif
  return n;
}
