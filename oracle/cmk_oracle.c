/*
 * CPU restatement of the reference's algorithms for bmm, mbmm, min_bmm and
 * topk_bmm.  TEST INFRASTRUCTURE ONLY: it is the checker that tests, the
 * smoke run and the CPU-baseline leg of the benchmark compare against; no
 * product path may call it.
 *
 * Every output element is accumulated the way one reference thread does it:
 * a single fp32 accumulator, k ascending, one fused multiply-add per step
 * (reference kernels/bmm_helpers.cu:20-26 `madd`, :140-164 thread_matmul_v3,
 * with --use_fast_math contracting to FMA, bmm.py:29).
 *
 * Pinned by tests/test_oracle.py: exact-integer fixtures computed with int64
 * arithmetic, float64 closed forms, brute-force loops on tiny shapes, and the
 * 0/1 principle for the sorting network.  The (a-b)^2 and |a-b| accumulate
 * functions (:28-35, :46-52) are run by none of the reference's notebooks; they
 * are pinned by exact int64 distances, a brute-force loop in the reference's
 * order of operations, torch.cdist in float64 and the zero-distance case.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
  int L, M, N, K;
  int transA, transB;
  long long lda, ldb, strideA, strideB;
} orc_desc;

static inline float a_at(const float* A, const orc_desc* d, int b, int m, int k) {
  const float* p = A + (long long)b * d->strideA;
  return d->transA ? p[(long long)k * d->lda + m] : p[(long long)m * d->lda + k];
}
static inline float b_at(const float* B, const orc_desc* d, int b, int k, int n) {
  const float* p = B + (long long)b * d->strideB;
  return d->transB ? p[(long long)n * d->ldb + k] : p[(long long)k * d->ldb + n];
}

/* accumulate functions, reference kernels/bmm_helpers.cu:20-52 */
static inline float accumulate(int distance, float a, float b, float c) {
  if (distance == 0) return fmaf(a, b, c);          /* madd        :20-26 */
  if (distance == 1) { float d = a - b; return fmaf(d, d, c); } /* squared_l2 :28-35 */
  return c + fabsf(a - b);                          /* l1          :46-52 */
}

static float dot(const float* A, const float* B, const orc_desc* d, int b, int m, int n,
                 int distance) {
  float c = 0.f; /* init_cCache, reference kernels/bmm_helpers.cu:166-176 */
  for (int k = 0; k < d->K; ++k) c = accumulate(distance, a_at(A, d, b, m, k), b_at(B, d, b, k, n), c);
  return c;
}

/* C[b][m][n], reference kernels/bmm.cu:184-274 */
void orc_bmm(const float* A, const float* B, float* C, const orc_desc* d) {
  for (int b = 0; b < d->L; ++b)
    for (int m = 0; m < d->M; ++m)
      for (int n = 0; n < d->N; ++n)
        C[((long long)b * d->M + m) * d->N + n] = dot(A, B, d, b, m, n, 0);
}

/*
 * Masked product, reference kernels/mbmm.cu:208-374: a tile with
 * block_mask == 0 is left at the host's zero fill (:251-255); a thread with
 * thread_mask == 0 never accumulates, so its 8x8 micro-tile stays 0 (:360-363);
 * every accumulator is multiplied by the element mask byte (:127-128; the guard
 * at :370 is always true).
 */
void orc_mbmm(const float* A, const float* B, float* C, const uint8_t* block_mask,
              const uint8_t* thread_mask, const uint8_t* element_mask, int share_mask,
              const orc_desc* d) {
  const int bM = (d->M + 127) / 128, bN = (d->N + 127) / 128;
  const int tM = (d->M + 7) / 8, tN = (d->N + 7) / 8;
  for (int b = 0; b < d->L; ++b) {
    const long long mb = share_mask ? 0 : b;
    for (int m = 0; m < d->M; ++m)
      for (int n = 0; n < d->N; ++n) {
        float c = 0.f;
        const uint8_t bm = block_mask[(mb * bM + m / 128) * bN + n / 128];
        const uint8_t tm = thread_mask[(mb * tM + m / 8) * tN + n / 8];
        if (bm != 0) {
          if (tm != 0) c = dot(A, B, d, b, m, n, 0);
          c *= (float)element_mask[(mb * d->M + m) * d->N + n];
        }
        C[((long long)b * d->M + m) * d->N + n] = c;
      }
  }
}

/*
 * min / argmin along dim (1: over m -> [L][N], 2: over n -> [L][M]), reference
 * kernels/minbmm.cu:13-153: strict '<' keeps the first (lowest) index inside a
 * thread and a block; across blocks the reference's index write is racy
 * (:76-79) - the restatement takes the lowest index there too.
 */
void orc_min_bmm(const float* A, const float* B, float* values, long long* indices,
                 const orc_desc* d, int dim, int distance) {
  const int kept = dim == 1 ? d->N : d->M;
  const int red = dim == 1 ? d->M : d->N;
  for (int b = 0; b < d->L; ++b)
    for (int y = 0; y < kept; ++y) {
      float best = INFINITY; /* values.fill_(inf), reference minbmm.py:122 */
      long long bi = 0;
      for (int x = 0; x < red; ++x) {
        const float c = dim == 1 ? dot(A, B, d, b, x, y, distance) : dot(A, B, d, b, y, x, distance);
        if (c < best) { best = c; bi = x; }
      }
      values[(long long)b * kept + y] = best;
      indices[(long long)b * kept + y] = bi;
    }
}

/* ---- the sorting network, reference kernels/topkbmm.cu:63-183 ------------- */

/* One compare-exchange stage over 128 slots: slot i looks at slot i^stride and
 * takes the partner's entry when (value < other) == direction(i)
 * (warp_comparator :63-74, block_comparator :76-96). */
static void stage(float* v, long long* ix, int stride, const int* direction) {
  float nv[128];
  long long ni[128];
  for (int i = 0; i < 128; ++i) {
    const int j = i ^ stride;
    const int cond = (v[i] < v[j]) == direction[i];
    nv[i] = cond ? v[j] : v[i];
    ni[i] = cond ? ix[j] : ix[i];
  }
  memcpy(v, nv, sizeof(nv));
  memcpy(ix, ni, sizeof(ni));
}
static inline int bit(int x, int b) { return (x >> b) & 1; }

/* Ascending bitonic sort of 128 entries, reference kernels/topkbmm.cu:98-139:
 * for each size 2^s (s = 1..6) the direction of slot i in the stage with
 * stride 2^t is bit(i, s) ^ bit(i, t); the final merge (size 128) uses
 * bit(i, t) alone. */
void orc_bitonic_sort_128(float* v, long long* ix) {
  int dir[128];
  for (int s = 1; s <= 6; ++s)
    for (int t = s - 1; t >= 0; --t) {
      for (int i = 0; i < 128; ++i) dir[i] = bit(i, s) ^ bit(i, t);
      stage(v, ix, 1 << t, dir);
    }
  for (int t = 6; t >= 0; --t) {
    for (int i = 0; i < 128; ++i) dir[i] = bit(i, t);
    stage(v, ix, 1 << t, dir);
  }
}

/* Merge of an ascending list `v` into the running descending top-128 `g`,
 * reference kernels/topkbmm.cu:141-183: slot-wise keep the larger (the
 * reference swaps with an add/sub trick, :161-168; a plain swap is used here),
 * which leaves a bitonic sequence holding the 128 largest of both lists, then
 * seven descending merge stages with direction !bit(i, t). */
void orc_bitonic_merge_desc(float* v, long long* ix, float* g, long long* gi) {
  int dir[128];
  for (int i = 0; i < 128; ++i)
    if (!(v[i] > g[i])) { v[i] = g[i]; ix[i] = gi[i]; }
  for (int t = 6; t >= 0; --t) {
    for (int i = 0; i < 128; ++i) dir[i] = !bit(i, t);
    stage(v, ix, 1 << t, dir);
  }
  memcpy(g, v, 128 * sizeof(float));
  memcpy(gi, ix, 128 * sizeof(long long));
}

/*
 * Top-k along dim (1: over m -> [L][N][k], 2: over n -> [L][M][k]), reference
 * kernels/topkbmm.cu:193-303: the reduced axis is cut into tiles of 128;
 * out-of-range slots hold (-inf, -1) (:221-224); each tile is sorted ascending
 * and merged into the row's running descending list, which starts at -inf
 * (reference topkbmm.py:127); the first k entries are returned (:150-151).
 * Index of never-filled slots: -1 here (uninitialised in the reference).
 */
void orc_topk_bmm(const float* A, const float* B, float* values, long long* indices,
                  const orc_desc* d, int dim, int k, int distance) {
  const int kept = dim == 1 ? d->N : d->M;
  const int red = dim == 1 ? d->M : d->N;
  for (int b = 0; b < d->L; ++b)
    for (int y = 0; y < kept; ++y) {
      float g[128];
      long long gi[128];
      for (int i = 0; i < 128; ++i) { g[i] = -INFINITY; gi[i] = -1; }
      for (int x0 = 0; x0 < red; x0 += 128) {
        float v[128];
        long long ix[128];
        for (int i = 0; i < 128; ++i) {
          const int x = x0 + i;
          if (x < red) {
            v[i] = dim == 1 ? dot(A, B, d, b, x, y, distance) : dot(A, B, d, b, y, x, distance);
            ix[i] = x;
          } else {
            v[i] = -INFINITY;
            ix[i] = -1;
          }
        }
        orc_bitonic_sort_128(v, ix);
        orc_bitonic_merge_desc(v, ix, g, gi);
      }
      for (int i = 0; i < k; ++i) {
        values[((long long)b * kept + y) * k + i] = g[i];
        indices[((long long)b * kept + y) * k + i] = gi[i];
      }
    }
}

/* Top-k of a 1-D array with the same network, reference
 * kernels/bitonic_sort.cu:122-216. */
void orc_topk_1d(const float* arr, long long n, float* values, long long* indices, int k) {
  float g[128];
  long long gi[128];
  for (int i = 0; i < 128; ++i) { g[i] = -INFINITY; gi[i] = -1; }
  for (long long x0 = 0; x0 < n; x0 += 128) {
    float v[128];
    long long ix[128];
    for (int i = 0; i < 128; ++i) {
      const long long x = x0 + i;
      v[i] = x < n ? arr[x] : -INFINITY;
      ix[i] = x < n ? x : -1;
    }
    orc_bitonic_sort_128(v, ix);
    orc_bitonic_merge_desc(v, ix, g, gi);
  }
  for (int i = 0; i < k; ++i) { values[i] = g[i]; indices[i] = gi[i]; }
}
