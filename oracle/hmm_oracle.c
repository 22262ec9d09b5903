/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the batched HMM forward
 * algorithm that the reference expresses as ParPy user code.  Nothing in the
 * product path may link or call this file; it is the checker for tests/, the
 * smoke test and the cpu_baseline leg of bench.py.
 *
 * Two models are restated:
 *
 *  hmm_ref_forward_*  : the 16-duration-layer k-mer model of the reference's
 *      test kernel, /root/reference/test/test_forward.py:83-160 (same
 *      arithmetic, split over helpers, in benchmarks/forward.py:94-187 and as
 *      CUDA in benchmarks/7mer/hmm.cu:61-114,201-235).  Pinned by the golden
 *      files test/data/{3mer,5mer}-expected.txt.
 *
 *  hmm_syn_forward_*  : the single-layer de Bruijn model of the synthetic
 *      benchmark configurations (4^k states, four shift predecessors plus a
 *      stay transition).  Pinned by closed forms (zero emissions with
 *      row-stochastic transitions give LL = 0; T = 1 gives a plain
 *      log-sum-exp) and by brute-force path enumeration for tiny k.
 *
 * The _f32 variants keep the operation order of the reference kernel in
 * single precision (expf/logf, fmaxf's NaN-dropping rule for the all -inf
 * case, test_forward.py:135-143); the _f64 variants do the same in double.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define DEFINE_HMM(T, SUF, EXP, LOG, FMAX)                                        \
/* test_forward.py:107-145: one state of one time step, reference model */       \
static inline T ref_state_##SUF(const T *src, int64_t s, int64_t S, int64_t K,   \
                                const T *trans1, const T *trans2, T gamma,       \
                                T syn248, const T *emis_row) {                    \
  int64_t q = (s / 4) % (S / 64);                                                 \
  int64_t pr[4] = {q, S / 64 + q, 2 * S / 64 + q, 3 * S / 64 + q};               \
  T t2 = trans2[s / K];                                                           \
  T p[5];                                                                         \
  for (int j = 0; j < 4; j++)                                                     \
    p[j] = trans1[(pr[j] % K) * 4 + s % 4] + t2 + src[pr[j]];                     \
  int64_t layer = s / K;                                                          \
  if (layer == 15) p[4] = gamma + src[s];                                         \
  else if (layer == 14) p[4] = syn248 + src[(layer + 1) * K + s % K];            \
  else p[4] = (T)0 + src[(layer + 1) * K + s % K];                                \
  T m = FMAX(p[0], p[1]); m = FMAX(m, p[2]); m = FMAX(m, p[3]); m = FMAX(m, p[4]);\
  T l = m + LOG(EXP(p[0] - m) + EXP(p[1] - m) + EXP(p[2] - m) + EXP(p[3] - m) +   \
                EXP(p[4] - m));                                                   \
  l = FMAX(l, (T)-INFINITY);                                                      \
  return l + emis_row[s % K];                                                     \
}                                                                                 \
/* test_forward.py:149-160: final log-sum-exp over the state vector */            \
static inline T final_lse_##SUF(const T *a, int64_t S) {                          \
  T m = (T)-INFINITY;                                                             \
  for (int64_t s = 0; s < S; s++) m = FMAX(m, a[s]);                              \
  T sum = 0;                                                                      \
  for (int64_t s = 0; s < S; s++) sum += EXP(a[s] - m);                           \
  return m + LOG(sum);                                                            \
}                                                                                 \
/* Reference model.  trans1 [K,4], trans2 [16], emis [101,K] (obs-major),        \
 * init [S], data int8 [n,maxlen], lens [n]; out [n].  alpha_out (optional)      \
 * receives the final state vector of every sequence, [n,S]. */                   \
void hmm_ref_forward_##SUF(int64_t S, const T *trans1, const T *trans2,          \
                           const T *emis, const T *init, T gamma, T syn248,      \
                           const int8_t *data, const int64_t *lens, int64_t n,   \
                           int64_t maxlen, T *out, T *alpha_out) {                \
  int64_t K = S / 16;                                                             \
  _Pragma("omp parallel for schedule(dynamic, 1)")                                \
  for (int64_t i = 0; i < n; i++) {                                               \
    T *a = (T *)malloc(sizeof(T) * S), *b = (T *)malloc(sizeof(T) * S);           \
    const int8_t *o = data + i * maxlen;                                          \
    for (int64_t s = 0; s < S; s++) a[s] = init[s] + emis[(int64_t)o[0] * K + s % K]; \
    for (int64_t t = 1; t < lens[i]; t++) {                                       \
      const T *row = emis + (int64_t)o[t] * K;                                    \
      for (int64_t s = 0; s < S; s++)                                             \
        b[s] = ref_state_##SUF(a, s, S, K, trans1, trans2, gamma, syn248, row);   \
      T *tmp = a; a = b; b = tmp;                                                 \
    }                                                                             \
    out[i] = final_lse_##SUF(a, S);                                               \
    if (alpha_out) memcpy(alpha_out + i * S, a, sizeof(T) * S);                   \
    free(a); free(b);                                                             \
  }                                                                               \
}                                                                                 \
/* Synthetic single-layer model.  trans1 [S,4] indexed [pred, s%4], stay [S],    \
 * emis [101,S] obs-major, init [S].  pred_j(s) = j*S/4 + s/4. */                 \
void hmm_syn_forward_##SUF(int64_t S, const T *trans1, const T *stay,            \
                           const T *emis, const T *init, const int8_t *data,     \
                           const int64_t *lens, int64_t n, int64_t maxlen,       \
                           int64_t max_steps, T *out, T *alpha_out) {             \
  _Pragma("omp parallel for schedule(dynamic, 1)")                                \
  for (int64_t i = 0; i < n; i++) {                                               \
    T *a = (T *)malloc(sizeof(T) * S), *b = (T *)malloc(sizeof(T) * S);           \
    const int8_t *o = data + i * maxlen;                                          \
    int64_t len = lens[i];                                                        \
    if (max_steps > 0 && len > max_steps) len = max_steps;                        \
    for (int64_t s = 0; s < S; s++) a[s] = init[s] + emis[(int64_t)o[0] * S + s]; \
    for (int64_t t = 1; t < len; t++) {                                           \
      const T *row = emis + (int64_t)o[t] * S;                                    \
      for (int64_t s = 0; s < S; s++) {                                           \
        T p[5];                                                                   \
        for (int j = 0; j < 4; j++) {                                             \
          int64_t pr = j * (S / 4) + s / 4;                                       \
          p[j] = trans1[pr * 4 + s % 4] + a[pr];                                  \
        }                                                                         \
        p[4] = stay[s] + a[s];                                                    \
        T m = FMAX(p[0], p[1]); m = FMAX(m, p[2]); m = FMAX(m, p[3]);             \
        m = FMAX(m, p[4]);                                                        \
        T l = m + LOG(EXP(p[0] - m) + EXP(p[1] - m) + EXP(p[2] - m) +             \
                      EXP(p[3] - m) + EXP(p[4] - m));                             \
        l = FMAX(l, (T)-INFINITY);                                                \
        b[s] = l + row[s];                                                        \
      }                                                                           \
      T *tmp = a; a = b; b = tmp;                                                 \
    }                                                                             \
    out[i] = final_lse_##SUF(a, S);                                               \
    if (alpha_out) memcpy(alpha_out + i * S, a, sizeof(T) * S);                   \
    free(a); free(b);                                                             \
  }                                                                               \
}

DEFINE_HMM(float, f32, expf, logf, fmaxf)
DEFINE_HMM(double, f64, exp, log, fmax)
