/*
 * kron_oracle.c -- CPU restatement of FastKron's sliced-multiply algorithm.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls this file;
 * it is the checker that the GPU results are compared against (tests, the smoke check and the
 * CPU-baseline leg of the benchmark).
 *
 * What is restated, and from where (paths relative to the FastKron reference tree):
 *   ko_sliced_multiply_{f32,f64}  tests/testBase.h:230-319   serial slicedMatmul: factor order
 *                                 last -> first (:241-244), output width (:247), slice/q of an
 *                                 output column (:248,:261), input column (:273-275 MKM,
 *                                 :304-306 KMM), factor element for opF N/T (:264-268 MKM,
 *                                 :295-299 KMM), intermediates and batch strides (:271,:279,:310),
 *                                 alpha*r + beta*y on the last step only (:281,:313).
 *   ko_gekmm_sizes                src/handle/handle.cpp:305-342,375-388  (temp = M * widest step output,
 *                                 N == 1: M * max(K, L))
 *   ko_gekmm_sizes_forward        src/handle/handle.cpp:390-408 with src/kmm/kmmalgo.cpp:96-112
 *   ko_flop                       src/kmm/kmmalgo.h:174-184
 *   ko_kron_bruteforce            not in the reference: the defining sum
 *                                 Z[m,l] = sum_k X[m,k] * prod_i F_i[k_i, l_i] (digit 1 slowest), which is
 *                                 what tests/python/test_torch.py:15-38 builds with torch.kron + matmul.
 *
 * How it is pinned (none of it by re-typing its own formula): tests/test_oracle.py checks
 * ko_sliced_multiply against numpy.kron + matmul, against ko_kron_bruteforce, against the closed
 * forms (N=1 is a GEMM, identity factors, all-ones inputs), and the size functions against the values
 * the reference library itself returned for the five benchmark configurations.
 *
 * Arithmetic: products are accumulated in double and rounded to the element type once per step,
 * like the reference's per-step stores; ko_sliced_multiply_fast_* accumulates in the element type
 * with the loops arranged for the vectoriser and is the variant the benchmark times as a CPU baseline.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define KO_MKM 0
#define KO_KMM 1
#define KO_OP_N 1
#define KO_OP_T 2

/* ------------------------------------------------------------------------------------------ */

uint64_t ko_flop(uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs) {
  uint64_t ops = 0, kk = 1;
  for (uint32_t i = 0; i < N; i++) kk *= Ps[i];
  for (int i = (int)N - 1; i >= 0; i--) {
    kk = (kk / Ps[i]) * Qs[i];
    ops += kk * Ps[i];
  }
  return 2ull * M * ops;
}

/* widths[j] = columns of the matrix produced by the step that multiplies factor j (j = N-1 first). */
static void step_widths(uint32_t N, const uint32_t* Ps, const uint32_t* Qs, uint64_t* widths) {
  uint64_t w = 1;
  for (uint32_t i = 0; i < N; i++) w *= Ps[i];
  for (int i = (int)N - 1; i >= 0; i--) {
    w = (w / Ps[i]) * Qs[i];
    widths[i] = w;
  }
}

int ko_gekmm_sizes(uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs,
                   size_t* yElems, size_t* tmpElems) {
  if (!yElems || !tmpElems || N == 0) return 4;
  uint64_t K = 1, L = 1;
  for (uint32_t i = 0; i < N; i++) { K *= Ps[i]; L *= Qs[i]; }
  *yElems = (size_t)M * L;
  if (N == 1) { *tmpElems = (size_t)M * (K > L ? K : L); return 0; }
  uint64_t* w = (uint64_t*)calloc(N, sizeof(uint64_t));
  if (!w) return 4;
  step_widths(N, Ps, Qs, w);
  uint64_t mx = 0;
  for (uint32_t i = 0; i < N; i++) if (w[i] > mx) mx = w[i];
  free(w);
  *tmpElems = (size_t)M * mx;
  return 0;
}

int ko_gekmm_sizes_forward(uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs,
                           size_t* yElems, size_t* intermediateElems) {
  if (!yElems || !intermediateElems || N == 0) return 4;
  uint64_t* w = (uint64_t*)calloc(N, sizeof(uint64_t));
  if (!w) return 4;
  step_widths(N, Ps, Qs, w);
  *yElems = (size_t)M * w[0];
  for (uint32_t i = 1; i < N; i++) intermediateElems[i - 1] = (size_t)M * w[i];
  free(w);
  return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* Defining sum, double in / double out, tiny shapes only.  X is M x K (MKM) or K x M (KMM),
 * F_i is P_i x Q_i (MKM) or Q_i x P_i (KMM), all row-major, no transposes, no epilogue. */
void ko_kron_bruteforce(int mmtype, uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs,
                        const double* X, const double* const* Fs, double* Z) {
  uint64_t K = 1, L = 1;
  for (uint32_t i = 0; i < N; i++) { K *= Ps[i]; L *= Qs[i]; }
  for (uint32_t m = 0; m < M; m++) {
    for (uint64_t l = 0; l < L; l++) {
      double acc = 0.0;
      for (uint64_t k = 0; k < K; k++) {
        double w = 1.0;
        uint64_t kr = k, lr = l;
        for (int i = (int)N - 1; i >= 0; i--) {      /* digit N is the fastest one */
          uint32_t ki = (uint32_t)(kr % Ps[i]), li = (uint32_t)(lr % Qs[i]);
          kr /= Ps[i]; lr /= Qs[i];
          w *= (mmtype == KO_MKM) ? Fs[i][(size_t)ki * Qs[i] + li] : Fs[i][(size_t)li * Ps[i] + ki];
        }
        double x = (mmtype == KO_MKM) ? X[(size_t)m * K + k] : X[(size_t)k * M + m];
        acc += x * w;
      }
      if (mmtype == KO_MKM) Z[(size_t)m * L + l] = acc; else Z[(size_t)l * M + m] = acc;
    }
  }
}

/* ------------------------------------------------------------------------------------------ */
/* Step-wise sliced multiply.  One step with factor F (P x Q) on an M x Kin input:
 *   out[m, j] = sum_p in[m, (j*P) % Kin + p] * F[p, (j / (Kin/P)) % Q],   j in [0, (Kin/P)*Q)
 * Buffers of the steps: `inter[i-1]` receives the output of the step multiplying factor i
 * (i = N-1 .. 1); the step multiplying factor 0 writes Z with the epilogue.  When `inter` is NULL
 * two scratch buffers are allocated internally.  */
#define KO_DEFINE_SLICED(NAME, T)                                                                     \
int NAME(int mmtype, uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs,                  \
         const T* X, int opX, uint64_t strideX,                                                       \
         const T* const* Fs, int opFs, const uint64_t* strideF,                                       \
         T* Z, uint64_t strideZ, double alpha, double beta,                                           \
         const T* Y, uint64_t strideY, uint32_t batchCount,                                           \
         T* const* inter, const uint64_t* strideInter) {                                              \
  if (N == 0 || !X || !Z || !Fs) return 4;                                                            \
  uint64_t K = 1;                                                                                     \
  for (uint32_t i = 0; i < N; i++) K *= Ps[i];                                                        \
  uint64_t* widths = (uint64_t*)malloc(sizeof(uint64_t) * N);                                         \
  step_widths(N, Ps, Qs, widths);                                                                     \
  uint64_t maxw = K;                                                                                  \
  for (uint32_t i = 0; i < N; i++) if (widths[i] > maxw) maxw = widths[i];                            \
  T* scratch[2] = {NULL, NULL};                                                                       \
  if (!inter && N > 1) {                                                                              \
    scratch[0] = (T*)malloc(sizeof(T) * (size_t)M * maxw);                                            \
    scratch[1] = (T*)malloc(sizeof(T) * (size_t)M * maxw);                                            \
  }                                                                                                   \
  for (uint32_t b = 0; b < batchCount; b++) {                                                         \
    const T* in = X + (size_t)b * strideX;                                                            \
    uint64_t Kin = K;                                                                                 \
    int inIsX = 1, flip = 0;                                                                          \
    for (int i = (int)N - 1; i >= 0; i--) {                                                           \
      const uint32_t P = Ps[i], Q = Qs[i];                                                            \
      const uint64_t S = Kin / P, Kout = S * Q;                                                       \
      const T* F = Fs[i] + (size_t)b * (strideF ? strideF[i] : 0);                                    \
      const int last = (i == 0);                                                                      \
      T* out;                                                                                         \
      if (last) out = Z + (size_t)b * strideZ;                                                        \
      else if (inter) out = inter[i - 1] + (size_t)b * (strideInter ? strideInter[i - 1] : (uint64_t)M * Kout); \
      else { out = scratch[flip]; flip ^= 1; }                                                        \
      const T* Yb = (Y && last) ? Y + (size_t)b * strideY : NULL;                                     \
      const int xT = (inIsX && opX == KO_OP_T);                                                       \
      _Pragma("omp parallel for collapse(2) schedule(static)")                                        \
      for (uint32_t m = 0; m < M; m++) {                                                              \
        for (uint64_t j = 0; j < Kout; j++) {                                                         \
          const uint32_t q = (uint32_t)((j / S) % Q);                                                 \
          const uint64_t c0 = (j * P) % Kin;                                                          \
          double r = 0.0;                                                                             \
          for (uint32_t p = 0; p < P; p++) {                                                          \
            double f;                                                                                 \
            if (mmtype == KO_MKM) f = (opFs == KO_OP_T) ? F[(size_t)q * P + p] : F[(size_t)p * Q + q]; \
            else                  f = (opFs == KO_OP_T) ? F[(size_t)p * Q + q] : F[(size_t)q * P + p]; \
            /* element (m, c0+p) of the M x Kin operand; MKM stores it row-major, KMM stores its   */ \
            /* transpose (Kin x M); opX == T on the very first step swaps the two storages.        */ \
            const int rowMajorMK = (mmtype == KO_MKM) ? !xT : xT;                                     \
            double x = rowMajorMK ? in[(size_t)m * Kin + c0 + p] : in[(size_t)(c0 + p) * M + m];      \
            r += x * f;                                                                               \
          }                                                                                           \
          const size_t o = (mmtype == KO_MKM) ? (size_t)m * Kout + j : (size_t)j * M + m;             \
          if (last) out[o] = (T)(alpha * r + (Yb ? beta * (double)Yb[o] : 0.0));                      \
          else      out[o] = (T)r;                                                                    \
        }                                                                                             \
      }                                                                                               \
      in = out; Kin = Kout; inIsX = 0;                                                                \
    }                                                                                                 \
  }                                                                                                   \
  free(scratch[0]); free(scratch[1]); free(widths);                                                   \
  return 0;                                                                                           \
}

KO_DEFINE_SLICED(ko_sliced_multiply_f32, float)
KO_DEFINE_SLICED(ko_sliced_multiply_f64, double)

/* ------------------------------------------------------------------------------------------ */
/* Same algorithm, MKM / opX = opF = N / contiguous rows only, arranged for speed: one OpenMP task
 * per row, the row ping-pongs between two thread-private buffers; per step a block of KO_SB slices
 * is first transposed to p-major so that the multiply is Q*P contiguous axpy loops over slices,
 * which the compiler vectorises.  Accumulation is in the element type.  This is the variant timed
 * as "cpu_baseline" by the benchmark. */
#define KO_SB 512
#define KO_DEFINE_FAST(NAME, T)                                                                       \
int NAME(uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs,                              \
         const T* X, const T* const* Fs, T* Z, T alpha, T beta, const T* Y) {                         \
  if (N == 0 || !X || !Z || !Fs) return 4;                                                            \
  uint64_t K = 1, L = 1;                                                                              \
  uint32_t maxP = 1;                                                                                  \
  for (uint32_t i = 0; i < N; i++) { K *= Ps[i]; L *= Qs[i]; if (Ps[i] > maxP) maxP = Ps[i]; }        \
  uint64_t* widths = (uint64_t*)malloc(sizeof(uint64_t) * N);                                         \
  step_widths(N, Ps, Qs, widths);                                                                     \
  uint64_t maxw = K;                                                                                  \
  for (uint32_t i = 0; i < N; i++) if (widths[i] > maxw) maxw = widths[i];                            \
  _Pragma("omp parallel")                                                                             \
  {                                                                                                   \
    T* buf0 = (T*)aligned_alloc(64, ((sizeof(T) * maxw + 63) / 64) * 64);                             \
    T* buf1 = (T*)aligned_alloc(64, ((sizeof(T) * maxw + 63) / 64) * 64);                             \
    T* tr   = (T*)aligned_alloc(64, ((sizeof(T) * (size_t)maxP * KO_SB + 63) / 64) * 64);             \
    _Pragma("omp for schedule(static)")                                                               \
    for (uint32_t m = 0; m < M; m++) {                                                                \
      const T* in = X + (size_t)m * K;                                                                \
      uint64_t Kin = K;                                                                               \
      int flip = 0;                                                                                   \
      for (int i = (int)N - 1; i >= 0; i--) {                                                         \
        const uint32_t P = Ps[i], Q = Qs[i];                                                          \
        const uint64_t S = Kin / P;                                                                   \
        const T* F = Fs[i];                                                                           \
        T* out = (i == 0) ? Z + (size_t)m * L : (flip ? buf1 : buf0);                                 \
        flip ^= 1;                                                                                    \
        for (uint64_t s0 = 0; s0 < S; s0 += KO_SB) {                                                  \
          const uint32_t sb = (uint32_t)((S - s0 < KO_SB) ? (S - s0) : KO_SB);                        \
          for (uint32_t s = 0; s < sb; s++)                                                           \
            for (uint32_t p = 0; p < P; p++) tr[(size_t)p * KO_SB + s] = in[(s0 + s) * P + p];        \
          for (uint32_t q = 0; q < Q; q++) {                                                          \
            T* restrict o = out + (size_t)q * S + s0;                                                 \
            const T f0 = F[q];                                                                        \
            for (uint32_t s = 0; s < sb; s++) o[s] = tr[s] * f0;                                      \
            for (uint32_t p = 1; p < P; p++) {                                                        \
              const T f = F[(size_t)p * Q + q];                                                       \
              const T* restrict t = tr + (size_t)p * KO_SB;                                           \
              for (uint32_t s = 0; s < sb; s++) o[s] += t[s] * f;                                     \
            }                                                                                         \
          }                                                                                           \
        }                                                                                             \
        if (i == 0) {                                                                                 \
          const T* y = Y ? Y + (size_t)m * L : NULL;                                                  \
          for (uint64_t l = 0; l < L; l++) out[l] = alpha * out[l] + (y ? beta * y[l] : (T)0);        \
        }                                                                                             \
        in = out; Kin = S * Q;                                                                        \
      }                                                                                               \
    }                                                                                                 \
    free(buf0); free(buf1); free(tr);                                                                 \
  }                                                                                                   \
  free(widths);                                                                                       \
  return 0;                                                                                           \
}

KO_DEFINE_FAST(ko_sliced_multiply_fast_f32, float)
KO_DEFINE_FAST(ko_sliced_multiply_fast_f64, double)
