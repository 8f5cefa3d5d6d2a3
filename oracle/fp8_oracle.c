/*
 * CPU oracle of the W8A8 FP8 linear path in plain C.  TEST INFRASTRUCTURE ONLY: tests, the smoke
 * check and the CPU-baseline leg of the bench load it; the product library never does.
 *
 * Same arithmetic as oracle/fp8_oracle.py (which is pinned against closed forms and torch's CPU
 * conversions in tests/test_oracle.py); tests/test_oracle.py also checks this file against the
 * numpy version bit for bit.  Parallelised with OpenMP so it can serve as the CPU baseline.
 *
 * Reference lines followed (paths relative to the SGLang checkout):
 *   group quant   python/sglang/test/test_block_fp8.py:23-48
 *   block matmul  python/sglang/test/test_block_fp8.py:273-325
 *   scaled_mm     sgl-kernel/tests/test_fp8_gemm.py:6-14
 *   W8A16 twin    sgl-kernel/csrc/cpu/gemm_fp8.cpp:46-100 (weight block -> bf16 with its scale), :256-298, :356-424
 */
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if (f != f) return 0x7fc0;
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

/* OCP e4m3fn encode, round to nearest even, no saturation (>= 464 and NaN -> 0x7F | sign). */
static inline uint8_t f32_to_e4m3fn(float x) {
  uint32_t u = f32_bits(x);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80);
  uint32_t a = u & 0x7fffffffu;
  if (a >= 0x7f800000u) return sign | 0x7f;
  if (a >= 0x3c800000u) { /* |x| >= 2^-6: normal */
    uint32_t r = a + 0x7ffffu + ((a >> 20) & 1u);
    int32_t code = (int32_t)(r >> 20) - (120 << 3);
    if (code > 0x7f) code = 0x7f;
    return sign | (uint8_t)code;
  }
  /* subnormal: multiples of 2^-9, ties to even */
  return sign | (uint8_t)lrintf(bits_f32(a) * 512.0f);
}

static float g_lut[256];
static int g_lut_ready = 0;
static void build_lut(void) {
  for (int v = 0; v < 256; ++v) {
    int s = v >> 7, e = (v >> 3) & 15, m = v & 7;
    float r;
    if (e == 0) r = ldexpf((float)m, -9);
    else if (e == 15 && m == 7) r = NAN;
    else r = ldexpf(1.0f + m / 8.0f, e - 7);
    g_lut[v] = s ? -r : r;
  }
  g_lut_ready = 1;
}

int oracle_num_threads(void) {
  int n = 1;
#ifdef _OPENMP
#pragma omp parallel
  {
#pragma omp master
    n = omp_get_num_threads();
  }
#endif
  return n;
}

/* x bf16 bits [M,K] -> q [M,K], s [M,K/group] row-major.  eps is applied as given (callers pass the
 * bf16-rounded value, as the torch-native path clamps in the input dtype). */
void oracle_group_quant_bf16(const uint16_t* x, uint8_t* q, float* s, int64_t M, int64_t K, int group, float eps,
                             int ue8m0) {
  const int64_t G = K / group;
#pragma omp parallel for schedule(static)
  for (int64_t gi = 0; gi < M * G; ++gi) {
    const uint16_t* xp = x + gi * group;
    float amax = 0.f;
    for (int i = 0; i < group; ++i) amax = fmaxf(amax, fabsf(bf16_to_f32(xp[i])));
    amax = fmaxf(amax, eps);
    float sc = amax / 448.0f;
    if (ue8m0) {
      uint32_t b = f32_bits(fmaxf(sc, 1e-10f));
      uint32_t e = (b >> 23) + ((b & 0x7fffffu) != 0);
      sc = bits_f32(e << 23);
    }
    s[gi] = sc;
    for (int i = 0; i < group; ++i) {
      float y = bf16_to_f32(xp[i]) / sc;
      y = y < -448.0f ? -448.0f : y;
      y = y > 448.0f ? 448.0f : y;
      q[gi * group + i] = f32_to_e4m3fn(y);
    }
  }
}

/* C[m,n] = sum_kb (A[m,kb] . B[n,kb]) * As[m,kb] * Bs[n/128,kb]; float accumulation per 128-block,
 * then bf16.  A [M,K], B [N,K] e4m3fn bytes; As [M,K/128], Bs [ceil(N/128),K/128] row-major. */
void oracle_block_gemm(const uint8_t* A, const uint8_t* B, const float* As, const float* Bs, uint16_t* C, int64_t M,
                       int64_t N, int64_t K) {
  if (!g_lut_ready) build_lut();
  const int64_t KB = (K + 127) / 128;
  float* Af = (float*)malloc((size_t)M * K * sizeof(float));
  for (int64_t i = 0; i < M * K; ++i) Af[i] = g_lut[A[i]];
#pragma omp parallel
  {
    float* brow = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(dynamic, 8)
    for (int64_t n = 0; n < N; ++n) {
      for (int64_t k = 0; k < K; ++k) brow[k] = g_lut[B[n * K + k]];
      const float* bs = Bs + (n / 128) * KB;
      for (int64_t m = 0; m < M; ++m) {
        const float* a = Af + m * K;
        float acc = 0.f;
        for (int64_t kb = 0; kb < KB; ++kb) {
          const int64_t k0 = kb * 128, k1 = (k0 + 128 < K) ? k0 + 128 : K;
          float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0}; /* fixed 8-way partial sums: vectorisable, deterministic */
          int64_t k = k0;
          for (; k + 8 <= k1; k += 8)
            for (int j = 0; j < 8; ++j) lane[j] += a[k + j] * brow[k + j];
          float part = ((lane[0] + lane[4]) + (lane[2] + lane[6])) + ((lane[1] + lane[5]) + (lane[3] + lane[7]));
          for (; k < k1; ++k) part += a[k] * brow[k];
          acc += part * (As[m * KB + kb] * bs[kb]);
        }
        C[m * N + n] = f32_to_bf16(acc);
      }
    }
    free(brow);
  }
  free(Af);
}

/* C = bf16((A . B^T) * sa[m] * sb[n] + bias[n]) with float accumulation; bias may be NULL. */
void oracle_scaled_mm(const uint8_t* A, const uint8_t* B, const float* sa, const float* sb, const float* bias,
                      uint16_t* C, int64_t M, int64_t N, int64_t K) {
  if (!g_lut_ready) build_lut();
  float* Af = (float*)malloc((size_t)M * K * sizeof(float));
  for (int64_t i = 0; i < M * K; ++i) Af[i] = g_lut[A[i]];
#pragma omp parallel
  {
    float* brow = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(dynamic, 8)
    for (int64_t n = 0; n < N; ++n) {
      for (int64_t k = 0; k < K; ++k) brow[k] = g_lut[B[n * K + k]];
      for (int64_t m = 0; m < M; ++m) {
        const float* a = Af + m * K;
        float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int64_t k = 0;
        for (; k + 8 <= K; k += 8)
          for (int j = 0; j < 8; ++j) lane[j] += a[k + j] * brow[k + j];
        float acc = ((lane[0] + lane[4]) + (lane[2] + lane[6])) + ((lane[1] + lane[5]) + (lane[3] + lane[7]));
        for (; k < K; ++k) acc += a[k] * brow[k];
        acc = acc * sb[n] * sa[m];
        if (bias) acc += bias[n];
        C[m * N + n] = f32_to_bf16(acc);
      }
    }
    free(brow);
  }
  free(Af);
}

/* The ALGORITHM of the reference's CPU kernel fp8_scaled_mm_cpu for more than four rows (W8A16, not the W8A8 path of
 * the rest of this file; a timing baseline and a sanity check, never a bit oracle): the bf16 activations are used as
 * they are, every weight element becomes bf16(float(bf16(w8)) * Bs[n/128, k/128]) (gemm_fp8.cpp:46-100: e4m3 -> bf16 is
 * exact, the product with the block scale is rounded to bf16), the dot products accumulate in float over the whole K,
 * the result (+ float bias) is rounded to bf16.  A bf16 bits [M,K]; B e4m3fn bytes [N,K]; Bs [ceil(N/128), K/128]. */
void oracle_w8a16_block_gemm(const uint16_t* A, const uint8_t* B, const float* Bs, const float* bias, uint16_t* C, int64_t M,
                             int64_t N, int64_t K) {
  if (!g_lut_ready) build_lut();
  const int64_t KB = (K + 127) / 128;
  float* Af = (float*)malloc((size_t)M * K * sizeof(float));
  for (int64_t i = 0; i < M * K; ++i) Af[i] = bf16_to_f32(A[i]);
#pragma omp parallel
  {
    float* brow = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(dynamic, 8)
    for (int64_t n = 0; n < N; ++n) {
      const float* bs = Bs + (n / 128) * KB;
      for (int64_t k = 0; k < K; ++k) brow[k] = bf16_to_f32(f32_to_bf16(g_lut[B[n * K + k]] * bs[k / 128]));
      for (int64_t m = 0; m < M; ++m) {
        const float* a = Af + m * K;
        float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int64_t k = 0;
        for (; k + 8 <= K; k += 8)
          for (int j = 0; j < 8; ++j) lane[j] += a[k + j] * brow[k + j];
        float acc = ((lane[0] + lane[4]) + (lane[2] + lane[6])) + ((lane[1] + lane[5]) + (lane[3] + lane[7]));
        for (; k < K; ++k) acc += a[k] * brow[k];
        if (bias) acc += bias[n];
        C[m * N + n] = f32_to_bf16(acc);
      }
    }
    free(brow);
  }
  free(Af);
}
