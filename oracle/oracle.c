/*
 * CPU oracle for the FlashAttention / mm_t / row-softmax path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this file; it exists so that the GPU kernels can be checked against a
 * scalar restatement of what the reference C backend emits for the same
 * components.  Callers are the test-suite, the smoke check and the
 * cpu_baseline leg of the benchmark.
 *
 * Every routine keeps the reference's evaluation order and its scalar
 * semantics (IEEE f32 throughout, exp spelled powf(2.71828175f, x), running
 * max/sum snapshots, per-tile normalisation) so that, compiled with the
 * reference's own flags (cc -O3, no fast-math), results agree bit for bit
 * with the reference-emitted C where such C exists.
 *
 * Pinning (see tests/test_oracle.py):
 *   oracle_attention_tiled   bit-exact vs the compiled reference emission
 *                            ilang-python/annotated-flashattn.c (oracle/_ref),
 *                            committed golden outputs, fp64 closed form
 *   oracle_mm_t              fp64 closed form A @ B.T, brute force
 *   oracle_row_softmax       fp64 closed form, rows sum to 1
 *   oracle_attention_naive   fp64 closed form, agreement with the tiled form
 */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>

/* Unary pow default base: the f32 literal the C backend prints for e
 * (compiler/src/lower/exec_plan_to_module.rs:630-633,
 *  compiler/src/backends/c/expr.rs:350-366). */
#define I_E 2.71828175f

/*
 * Blockwise online-softmax attention, the loop nest of
 * ilang-python/annotated-flashattn.c:52-310 with
 *   - leading batch*head loop (schedule prefix "bh", outermost, independent),
 *   - optional scalar multiply of the score tile before the max
 *     (component  i("bhij*.~bhij | ... ") chained after mm_t),
 *   - tile sizes ti (query rows) / tj (keys) taken from the split factors
 *     (16/16 in the reference demo).
 * q [bh,nq,d], k [bh,nk,d], v [bh,nk,dv], o [bh,nq,dv]; all row-major f32.
 * Scratch mirrors the reference's buffers: S/P tiles, m, m_old, l, l_old.
 */
int oracle_attention_tiled(const float* q, const float* k, const float* v, float* o,
                           size_t bh, size_t nq, size_t nk, size_t d, size_t dv,
                           int has_scale, float scale, size_t ti, size_t tj)
{
  float* s1 = (float*)malloc(ti * tj * sizeof(float)); /* S_ij          (:327-333) */
  float* s3 = (float*)malloc(ti * tj * sizeof(float)); /* S_ij - m      (:340-346) */
  float* s4 = (float*)malloc(ti * tj * sizeof(float)); /* P_ij          (:348-354) */
  float* s6 = (float*)malloc(ti * tj * sizeof(float)); /* P_ij / l      (:361-367) */
  float* m = (float*)malloc(nq * sizeof(float));       /* s2 running max   */
  float* m_old = (float*)malloc(nq * sizeof(float));   /* s8 snapshot      */
  float* l = (float*)malloc(nq * sizeof(float));       /* s5 running sum   */
  float* l_old = (float*)malloc(nq * sizeof(float));   /* s9 snapshot      */
  if (!s1 || !s3 || !s4 || !s6 || !m || !m_old || !l || !l_old) return -1;

  for (size_t b = 0; b < bh; ++b) {
    const float* Q = q + b * nq * d;
    const float* K = k + b * nk * d;
    const float* V = v + b * nk * dv;
    float* O = o + b * nq * dv;
    for (size_t jt = 0; jt < (nk + tj - 1) / tj; ++jt) {
      for (size_t it = 0; it < (nq + ti - 1) / ti; ++it) {
        /* S tile = Q_i K_j^T, scalar product temp then accumulate (:57-89) */
        for (size_t a = 0; a < ti; ++a) {
          if (it * ti + a >= nq) continue;
          for (size_t c = 0; c < tj; ++c) {
            if (jt * tj + c >= nk) continue;
            float acc = 0.0f;
            for (size_t x = 0; x < d; ++x) {
              float prod = Q[(it * ti + a) * d + x] * K[(jt * tj + c) * d + x];
              acc = acc + prod;
            }
            s1[a * tj + c] = has_scale ? acc * scale : acc;
          }
        }
        /* running max with snapshot (:92-127) */
        for (size_t a = 0; a < ti; ++a) {
          size_t r = it * ti + a;
          if (r >= nq) continue;
          if (jt == 0) m[r] = -INFINITY;
          m_old[r] = m[r];
          for (size_t c = 0; c < tj; ++c) {
            if (jt * tj + c >= nk) continue;
            m[r] = fmaxf(m[r], s1[a * tj + c]);
          }
        }
        /* shift (:130-147) and exp (:150-164) */
        for (size_t a = 0; a < ti; ++a) {
          if (it * ti + a >= nq) continue;
          for (size_t c = 0; c < tj; ++c) {
            if (jt * tj + c >= nk) continue;
            s3[a * tj + c] = s1[a * tj + c] - m[it * ti + a];
          }
        }
        for (size_t a = 0; a < ti; ++a) {
          if (it * ti + a >= nq) continue;
          for (size_t c = 0; c < tj; ++c) {
            if (jt * tj + c >= nk) continue;
            s4[a * tj + c] = powf(I_E, s3[a * tj + c]);
          }
        }
        /* running sum: snapshot, exp-shift correction, accumulate (:167-217) */
        for (size_t a = 0; a < ti; ++a) {
          size_t r = it * ti + a;
          if (r >= nq) continue;
          if (jt == 0) l[r] = 0.0f;
          l_old[r] = l[r];
          l[r] = l[r] * powf(I_E, m_old[r] - m[r]);
          for (size_t c = 0; c < tj; ++c) {
            if (jt * tj + c >= nk) continue;
            l[r] = l[r] + s4[a * tj + c];
          }
        }
        /* per-tile normalisation (:220-237) */
        for (size_t a = 0; a < ti; ++a) {
          if (it * ti + a >= nq) continue;
          for (size_t c = 0; c < tj; ++c) {
            if (jt * tj + c >= nk) continue;
            s6[a * tj + c] = s4[a * tj + c] / l[it * ti + a];
          }
        }
        /* O corrections then O += P V (:240-305).  As in the reference, the
         * two Scale loops run before the guarded init, so on the first key
         * tile they touch whatever the output buffer held; the init that
         * follows overwrites it. */
        for (size_t a = 0; a < ti; ++a) {
          size_t r = it * ti + a;
          if (r >= nq) continue;
          for (size_t x = 0; x < dv; ++x)
            O[r * dv + x] = O[r * dv + x] * powf(I_E, m_old[r] - m[r]);
          for (size_t x = 0; x < dv; ++x)
            O[r * dv + x] = O[r * dv + x] * (l_old[r] / l[r]);
          for (size_t x = 0; x < dv; ++x) {
            if (jt == 0) O[r * dv + x] = 0.0f;
            for (size_t c = 0; c < tj; ++c) {
              if (jt * tj + c >= nk) continue;
              float prod = s6[a * tj + c] * V[(jt * tj + c) * dv + x];
              O[r * dv + x] = O[r * dv + x] + prod;
            }
          }
        }
      }
    }
  }
  free(l_old); free(l); free(m_old); free(m);
  free(s6); free(s4); free(s3); free(s1);
  return 0;
}

/*
 * mm_t:  i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | ... | jii'j'k0")
 * (README.md:16).  The fused nest is the S-tile nest of
 * annotated-flashattn.c:57-89 with a full-size output: per output element a
 * zero init, then for k ascending  tmp = a*b; c = c + tmp  in f32.  The tile
 * loops only reorder independent output elements, so the plain (i,j) order
 * gives identical bits.
 * a [bh,m,kk], b [bh,n,kk], c [bh,m,n].
 */
int oracle_mm_t(const float* a, const float* b, float* c,
                size_t bh, size_t m, size_t n, size_t kk)
{
  for (size_t z = 0; z < bh; ++z) {
    const float* A = a + z * m * kk;
    const float* B = b + z * n * kk;
    float* C = c + z * m * n;
    for (size_t i = 0; i < m; ++i) {
      for (size_t j = 0; j < n; ++j) {
        float acc = 0.0f;
        for (size_t x = 0; x < kk; ++x) {
          float prod = A[i * kk + x] * B[j * kk + x];
          acc = acc + prod;
        }
        C[i * n + j] = acc;
      }
    }
  }
  return 0;
}

/*
 * Row softmax,  row_max_shift >> exp >> row_normalize  in a reference-valid
 * (non-online) schedule: three kernels
 *   (I & i(">ij~i")) >> i("ij-i~ij"),  i("^ij~ij"),  (I & i("+ij~i")) >> i("ij/i~ij")
 * (ilang-python/flash-attn.py:60-62).  Reductions start from the identity
 * (-inf / 0, exec_plan_to_module.rs:592-603) and fold j ascending:
 * m = fmaxf(m, x), l = l + p; exp is powf(2.71828175f, x).
 * x, y [rows, cols].  `tmp` holds the shifted / exponentiated row.
 */
int oracle_row_softmax(const float* x, float* y, size_t rows, size_t cols)
{
  for (size_t i = 0; i < rows; ++i) {
    const float* X = x + i * cols;
    float* Y = y + i * cols;
    float m = -INFINITY;
    for (size_t j = 0; j < cols; ++j) m = fmaxf(m, X[j]);
    for (size_t j = 0; j < cols; ++j) Y[j] = X[j] - m;
    for (size_t j = 0; j < cols; ++j) Y[j] = powf(I_E, Y[j]);
    float l = 0.0f;
    for (size_t j = 0; j < cols; ++j) l = l + Y[j];
    for (size_t j = 0; j < cols; ++j) Y[j] = Y[j] / l;
  }
  return 0;
}

/*
 * Naive attention (five kernels, full intermediates), the schedule of
 * ilang-python/flash-attn.py:57-65 and ilang-python/test.py:75-82:
 * S = Q K^T (optionally scaled), row softmax, O = P V with keys folded in
 * ascending order through a scalar product temp.
 */
int oracle_attention_naive(const float* q, const float* k, const float* v, float* o,
                           size_t bh, size_t nq, size_t nk, size_t d, size_t dv,
                           int has_scale, float scale)
{
  float* s = (float*)malloc(nq * nk * sizeof(float));
  float* p = (float*)malloc(nq * nk * sizeof(float));
  if (!s || !p) return -1;
  for (size_t b = 0; b < bh; ++b) {
    oracle_mm_t(q + b * nq * d, k + b * nk * d, s, 1, nq, nk, d);
    if (has_scale)
      for (size_t x = 0; x < nq * nk; ++x) s[x] = s[x] * scale;
    oracle_row_softmax(s, p, nq, nk);
    const float* V = v + b * nk * dv;
    float* O = o + b * nq * dv;
    for (size_t i = 0; i < nq; ++i) {
      for (size_t x = 0; x < dv; ++x) {
        float acc = 0.0f;
        for (size_t j = 0; j < nk; ++j) {
          float prod = p[i * nk + j] * V[j * dv + x];
          acc = acc + prod;
        }
        O[i * dv + x] = acc;
      }
    }
  }
  free(p); free(s);
  return 0;
}
