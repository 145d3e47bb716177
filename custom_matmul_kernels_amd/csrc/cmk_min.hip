// min_bmm: fused min / argmin of A@B along one axis; the product never
// reaches HBM.
//
// X = the reduced axis, Y = the kept axis.  With X inside the lane, the
// running (min, argmin) of an output element lives in one lane for the whole
// walk over X; the finish is one exchange between the two half-waves and one
// LDS step between the two waves that share a Y range.  When the kept axis
// has too few 128-wide strips to fill the chip, the reduced axis is also cut
// into `splits` ranges; their partial results go to a workspace and a small
// second kernel folds them in order, so ties always resolve to the lowest
// index and the result does not depend on scheduling.
//
// Plays the role of min_bmm_* with min_dim_1 / min_dim_2 and the float
// atomicMin (reference kernels/minbmm.cu:1-153, 347-440).
//
// The squared-l2 distance has a second route through the matrix pipe.  Its
// result must equal, bit for bit, the sequential fmaf(x-y, x-y, c) sum E(x, y)
// of the vector route, so the matrix pipe only *screens*: it computes
// t(x, y) = |x|^2 - 2 x.y, which differs from E(x, y) - |y|^2 by at most
// e(x, y) = beta * (|x|^2 + |y|^2) with beta = (4K + 32) * 2^-24 * 1.02 (rounding
// of the K products and additions of either sum, of the norms and of the final
// fused multiply-add; see l2_beta()).  Per kept row y the kernel keeps the two
// smallest t with their indices and a lower bound h of every other t.  If
// h > t1 + W with W = 2 * beta * (max|x|^2 + |y|^2), no x outside those two can
// reach or tie the minimum of E, and E is evaluated exactly for the one or two
// candidates.  Otherwise the row is recomputed exactly: a few such rows one at
// a time (min_l2_rows_kernel), many of them (ties among duplicated points,
// non-finite input) by the vector route over the whole problem.
#include <math.h>

#include <atomic>

#include "cmk_core.hpp"
#include "cmk_launch.hpp"

namespace cmk {

struct MinArgs {
  Operand X, Y;                 // batch 0 views
  long long strideX, strideY;   // batch strides
  float* values;                // [L][Yext]
  long long* indices;           // [L][Yext]
  float* part_val;              // [splits][L][Yext]  (splits > 1)
  int* part_idx;
  int L, K;
  int ystrips, xtiles, splits, tiles_per_split;
  int ygroup;                   // y strips that run side by side with all their splits
  int total;                    // work-groups with real work slots (before XCD padding)
  // screening route of the squared-l2 distance (DIST == kL2M)
  const float* nx;              // [L][XP] squared norms of the X rows, +inf beyond the last row
  int XP;                       // xtiles * 128
  float *pc1, *pc2, *ph;        // [splits][L][Yext]: smallest, second smallest t, bound of the rest
  int *pi1, *pi2;               // their indices
  // exact pass behind a screening pass: runs only when *gate > gate_limit
  const int* gate;
  int gate_limit;
};

constexpr int kL2M = 3;   // squared l2 screened on the matrix pipe (this file only)

// The two smallest screening values of a set of x with their indices, and a
// lower bound of all the others'.
struct Cand {
  float c1; int i1;
  float c2; int i2;
  float h;
};

__device__ __forceinline__ bool cand_less(float v, int i, float w, int j) {
  return v < w || (v == w && i < j);
}

// Union of two disjoint sets.  No value is ever NaN: they are only assigned
// through '<', fminf and med3.
__device__ __forceinline__ Cand cand_merge(const Cand& a, const Cand& b) {
  const bool af = cand_less(a.c1, a.i1, b.c1, b.i1);
  const Cand& p = af ? a : b;   // the set whose head wins
  const Cand& q = af ? b : a;
  Cand r;
  r.c1 = p.c1; r.i1 = p.i1;
  const bool ps = cand_less(p.c2, p.i2, q.c1, q.i1);
  r.c2 = ps ? p.c2 : q.c1;
  r.i2 = ps ? p.i2 : q.i1;
  const float dropped = ps ? q.c1 : p.c2;   // q.c2 >= q.c1 is dropped in either case
  r.h = fminf(fminf(a.h, b.h), fminf(dropped, q.c2));
  return r;
}

template <int XK, int YK, int DIST>
__global__ __launch_bounds__(kThreads, 2) void min_kernel(MinArgs a) {
  using C = Core<XK, YK, 2, 2, 2, 2, 32, kReadsPaired, true>;
  __shared__ __attribute__((aligned(16))) float lds[C::ldsFloats];

  // Work-groups that are resident on one XCD at the same time form a block of
  // `ygroup` y strips x `splits` ranges of X: the strips of Y they re-read for
  // every tile stay in that XCD's L2, and each X tile is fetched once for the
  // `ygroup` work-groups that walk the same range.
  // Every id is a real work slot (a padded last group would push whole XCDs into
  // a second round): the last group simply has fewer strips.
  const int logical = xcd_logical_id(blockIdx.x, a.total);
  if (logical < 0) return;
  const int gsz = a.ygroup * a.splits;
  const int group = logical / gsz;
  const int ybase = group * a.ygroup;
  const int yg = min(a.ygroup, a.L * a.ystrips - ybase);   // strips of this group
  const int within = logical - group * gsz;
  const int split = within / yg;
  const int yflat = ybase + within % yg;
  const int b = yflat / a.ystrips;
  const int ystrip = yflat - b * a.ystrips;
  const int y0 = ystrip * C::TY;
  const int xt_begin = split * a.tiles_per_split;
  const int xt_end = min(a.xtiles, xt_begin + a.tiles_per_split);
  if (a.gate != nullptr && *a.gate <= a.gate_limit) return;

  constexpr bool SCREEN = DIST == kL2M;
  constexpr int TILE_DIST = SCREEN ? kInner : DIST;   // what the tile engine accumulates

  Operand X = a.X, Y = a.Y;
  X.p = uniform_ptr(X.p + (long long)b * a.strideX);
  Y.p = uniform_ptr(Y.p + (long long)b * a.strideY);

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  const int wx = wave % 2, wy = wave / 2;

  float best[2] = {INFINITY, INFINITY};
  float best2[2] = {INFINITY, INFINITY};   // SCREEN: second smallest value this lane has seen
  int bidx[2] = {xt_begin * C::TX, xt_begin * C::TX};
  const float* nxb = SCREEN ? a.nx + (long long)b * a.XP + 4 * half : nullptr;

  C core;
  core.begin(X, Y, xt_begin * C::TX, y0, a.K, xt_end - xt_begin, lds);
  for (int xt = xt_begin; xt < xt_end; ++xt) {
    f32x16 acc[2][2];
    if constexpr (TILE_DIST != kInner) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    }
    core.template tile<TILE_DIST, TILE_DIST == kInner>(X, Y, lds, acc);
    // Fold this tile into the running minimum.  Inside the tile a lane tracks the
    // position of its minimum as a small code (block * 16 + register: a literal
    // per compare, no index registers); indices ascend with the code, so a strict
    // '<' keeps the first occurrence.  The code becomes an index once per tile.
    const int xb = xt * C::TX + wx * 64;
    // (every search starts from +inf, not from the first product: a NaN there
    // would lose every later comparison and hide the rest of the tile)
    float tbest[2] = {INFINITY, INFINITY};
    int tcode[2] = {0, 0};
    if constexpr (SCREEN) {
      // t = |x|^2 - 2 x.y.  Rows beyond the last have |x|^2 = +inf and lose every
      // compare (their products are finite, or NaN).  med3 of (smallest, new,
      // second) is the new second smallest; with a NaN it returns the smallest
      // of the others, which only lowers the bound.
      float tsec[2] = {INFINITY, INFINITY};
#pragma unroll
      for (int bx = 0; bx < 2; ++bx)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          const f32x4 n4 = *reinterpret_cast<const f32x4*>(nxb + xb + bx * 32 + 8 * rg);
          const float nr[4] = {n4.x, n4.y, n4.z, n4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int r = 4 * rg + e;
#pragma unroll
            for (int by = 0; by < 2; ++by) {
              const float v = __builtin_fmaf(-2.f, acc[bx][by][r], nr[e]);
              tsec[by] = __builtin_amdgcn_fmed3f(tbest[by], v, tsec[by]);
              if (v < tbest[by]) { tbest[by] = v; tcode[by] = bx * 16 + r; }
            }
          }
        }
#pragma unroll
      for (int by = 0; by < 2; ++by)
        best2[by] = fminf(fmaxf(best[by], tbest[by]), fminf(best2[by], tsec[by]));
    } else if (xb + 64 <= X.rows) {
#pragma unroll
      for (int bx = 0; bx < 2; ++bx)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
#pragma unroll
          for (int by = 0; by < 2; ++by) {
            const float v = acc[bx][by][r];
            if (v < tbest[by]) { tbest[by] = v; tcode[by] = bx * 16 + r; }
          }
        }
    } else {
#pragma unroll
      for (int bx = 0; bx < 2; ++bx)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int x = xb + bx * 32 + acc_row(r, half);
#pragma unroll
          for (int by = 0; by < 2; ++by) {
            const float v = acc[bx][by][r];
            if (x < X.rows && v < tbest[by]) { tbest[by] = v; tcode[by] = bx * 16 + r; }
          }
        }
    }
#pragma unroll
    for (int by = 0; by < 2; ++by) {
      const int x = xb + (tcode[by] >> 4) * 32 + acc_row(tcode[by] & 15, half);
      if (tbest[by] < best[by]) { best[by] = tbest[by]; bidx[by] = x; }
    }
  }
  __syncthreads();  // the operand buffers are reused below

  if constexpr (SCREEN) {
    // the same two exchanges as below, on candidate sets
    Cand c[2];
#pragma unroll
    for (int by = 0; by < 2; ++by) {
      const float ov = __shfl_xor(best[by], 32);
      const int oi = __shfl_xor(bidx[by], 32);
      const float o2 = __shfl_xor(best2[by], 32);
      const bool mine = cand_less(best[by], bidx[by], ov, oi);
      c[by].c1 = mine ? best[by] : ov;
      c[by].i1 = mine ? bidx[by] : oi;
      c[by].c2 = mine ? ov : best[by];
      c[by].i2 = mine ? oi : bidx[by];
      c[by].h = fminf(best2[by], o2);
    }
    float* red = lds;   // [2 wy][2 by][5 words][32]
    if (wx == 1 && half == 0) {
#pragma unroll
      for (int by = 0; by < 2; ++by) {
        float* w = red + (wy * 2 + by) * 160 + l32;
        w[0] = c[by].c1;
        w[32] = __int_as_float(c[by].i1);
        w[64] = c[by].c2;
        w[96] = __int_as_float(c[by].i2);
        w[128] = c[by].h;
      }
    }
    __syncthreads();
    if (wx == 0 && half == 0) {
      const int Yext = Y.rows;
#pragma unroll
      for (int by = 0; by < 2; ++by) {
        const float* w = red + (wy * 2 + by) * 160 + l32;
        Cand o;
        o.c1 = w[0];
        o.i1 = __float_as_int(w[32]);
        o.c2 = w[64];
        o.i2 = __float_as_int(w[96]);
        o.h = w[128];
        const Cand m = cand_merge(c[by], o);
        const int y = y0 + wy * 64 + by * 32 + l32;
        if (y < Yext) {
          const long long at = ((long long)split * a.L + b) * Yext + y;
          a.pc1[at] = m.c1;
          a.pi1[at] = m.i1;
          a.pc2[at] = m.c2;
          a.pi2[at] = m.i2;
          a.ph[at] = m.h;
        }
      }
    }
    return;
  }

  // the two half-waves hold different x for the same y
#pragma unroll
  for (int by = 0; by < 2; ++by) {
    const float ov = __shfl_xor(best[by], 32);
    const int oi = __shfl_xor(bidx[by], 32);
    if (ov < best[by] || (ov == best[by] && oi < bidx[by])) { best[by] = ov; bidx[by] = oi; }
  }
  // the two waves with the same wy hold different x for the same y
  float* red_v = lds;                                   // [2 wy][2 by][32]
  int* red_i = reinterpret_cast<int*>(lds + 128);
  if (wx == 1 && half == 0) {
#pragma unroll
    for (int by = 0; by < 2; ++by) {
      red_v[(wy * 2 + by) * 32 + l32] = best[by];
      red_i[(wy * 2 + by) * 32 + l32] = bidx[by];
    }
  }
  __syncthreads();
  if (wx == 0 && half == 0) {
    const int Yext = Y.rows;
#pragma unroll
    for (int by = 0; by < 2; ++by) {
      const float ov = red_v[(wy * 2 + by) * 32 + l32];
      const int oi = red_i[(wy * 2 + by) * 32 + l32];
      float v = best[by];
      int i = bidx[by];
      if (ov < v || (ov == v && oi < i)) { v = ov; i = oi; }
      const int y = y0 + wy * 64 + by * 32 + l32;
      if (y < Yext) {
        if (a.splits == 1) {
          a.values[(long long)b * Yext + y] = v;
          a.indices[(long long)b * Yext + y] = i;
        } else {
          const long long o = ((long long)split * a.L + b) * Yext + y;
          a.part_val[o] = v;
          a.part_idx[o] = i;
        }
      }
    }
  }
}

// Folds the per-split partial results in ascending split (= ascending index)
// order.  The partials of up to sixteen splits are requested together, so that
// the kernel waits for memory once (the usual plans have at most sixteen splits);
// 64 threads per work-group spread a small problem over more CUs.
constexpr int kFoldThreads = 64;
constexpr int kFoldBatch = 16;
__global__ __launch_bounds__(kFoldThreads) void min_fold_kernel(const float* part_val, const int* part_idx,
                                                                float* values, long long* indices,
                                                                long long rows, int splits,
                                                                const int* gate, int gate_limit) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows) return;
  if (gate != nullptr && *gate <= gate_limit) return;
  float v = INFINITY;
  int idx = part_idx[i];
  for (int s0 = 0; s0 < splits; s0 += kFoldBatch) {
    float pv[kFoldBatch];
    int pi[kFoldBatch];
#pragma unroll
    for (int j = 0; j < kFoldBatch; ++j) {
      const int s = s0 + j < splits ? s0 + j : splits - 1;   // clamped: repeats fold to nothing
      pv[j] = part_val[(long long)s * rows + i];
      pi[j] = part_idx[(long long)s * rows + i];
    }
#pragma unroll
    for (int j = 0; j < kFoldBatch; ++j)
      if (pv[j] < v) { v = pv[j]; idx = pi[j]; }
  }
  values[i] = v;
  indices[i] = idx;
}


// ---------------------------------------------------------------------------
// Squared l2 through the matrix pipe: the kernels around the screening pass.
// ---------------------------------------------------------------------------

// Rows that the screening cannot decide are recomputed one at a time up to this
// many; beyond it the vector route recomputes the whole problem.
constexpr int kRowLimit = 512;
constexpr int kRowMaxParts = 64;     // work-groups that share one such row, at most
constexpr int kRowGrid = 2048;
constexpr int kRowBuckets = 16;      // atomic minima per row, so that work-groups do not queue on one address

// Rounding budget per unit of |x|^2 + |y|^2 (see the head of this file).  With
// u = 2^-24: the exact route's K subtractions, squares and additions err by at
// most 2(K+2)u of |x|^2+|y|^2 (its value is at most twice that sum); the matrix
// pipe's K products and additions by (K+2)u', where u' = 2u allows for an
// accumulator that truncates; the norms and the final fused multiply-add by 3u.
static float l2_beta(int K) { return (float)((4.0 * K + 32.0) * 5.9604644775390625e-8 * 1.02); }

__device__ __forceinline__ const float* row_base(const Operand& o, int kind, int row) {
  return kind == KC ? o.p + (long long)row * o.ld : o.p + row;
}
__device__ __forceinline__ long long k_step(const Operand& o, int kind) { return kind == KC ? 1 : o.ld; }

// The exact distance of the vector route: d = x - y, c = fmaf(d, d, c), k ascending.
__device__ __forceinline__ float l2_exact(const float* x, long long xs, const float* y, long long ys, int K) {
  // thirty-two elements of either operand are requested before the first is
  // used: the chain of K dependent fmaf is short, the K loads are what takes time
  float c = 0.f;
  int k = 0;
  for (; k + 32 <= K; k += 32) {
    float xv[32], yv[32];
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      xv[j] = x[(k + j) * xs];
      yv[j] = y[(k + j) * ys];
    }
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const float d = xv[j] - yv[j];
      c = __builtin_fmaf(d, d, c);
    }
  }
  for (; k < K; ++k) {
    const float d = x[k * xs] - y[k * ys];
    c = __builtin_fmaf(d, d, c);
  }
  return c;
}

// The same for two k-contiguous rows that 16-byte loads may fetch (K a multiple
// of 4): a quarter of the load instructions, each lane still reads its own rows.
__device__ __forceinline__ float l2_exact_vec(const float* x, const float* y, int K) {
  typedef const f32x4 __attribute__((address_space(1))) * g16p;
  float c = 0.f;
  int k = 0;
  for (; k + 32 <= K; k += 32) {
    f32x4 xv[8], yv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      xv[j] = *(g16p)(x + k + 4 * j);
      yv[j] = *(g16p)(y + k + 4 * j);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float d = xv[j].x - yv[j].x;
      c = __builtin_fmaf(d, d, c);
      d = xv[j].y - yv[j].y;
      c = __builtin_fmaf(d, d, c);
      d = xv[j].z - yv[j].z;
      c = __builtin_fmaf(d, d, c);
      d = xv[j].w - yv[j].w;
      c = __builtin_fmaf(d, d, c);
    }
  }
  for (; k < K; ++k) {
    const float d = x[k] - y[k];
    c = __builtin_fmaf(d, d, c);
  }
  return c;
}

// The same with y in LDS (unit stride) and sixty-four elements of x in flight.
__device__ __forceinline__ float l2_exact_lds(const float* x, long long xs, const float* y, int K) {
  float c = 0.f;
  int k = 0;
  for (; k + 64 <= K; k += 64) {
    float xv[64];
#pragma unroll
    for (int j = 0; j < 64; ++j) xv[j] = x[(k + j) * xs];
#pragma unroll
    for (int j = 0; j < 64; ++j) {
      const float d = xv[j] - y[k + j];
      c = __builtin_fmaf(d, d, c);
    }
  }
  for (; k < K; ++k) {
    const float d = x[k * xs] - y[k];
    c = __builtin_fmaf(d, d, c);
  }
  return c;
}

struct L2Args {
  Operand X, Y;
  long long strideX, strideY;
  int xk, yk;
  int L, K, Yext, XP, xtiles, yblocks, splits;
  float beta;
  float* nx;        // [L][XP]
  float* ny;        // [L][Yext]
  float* xmax;      // [L][xtiles] largest |x|^2 of each 128 rows
  float* xt;        // [L][Xext][K] k-contiguous copy of a row-contiguous X, else null
  int Xext;
  int* ctrl;        // [0] undecided rows
  int* list;        // [kRowLimit] undecided rows
  unsigned long long* rowbest;   // [kRowLimit][kRowBuckets] (value bits << 32 | index)
  const float *pc1, *pc2, *ph;
  const int *pi1, *pi2;
  float* values;
  long long* indices;
};

// Squared norms, summed in double and rounded once.  A work-group takes 128
// rows of one batch of X or of Y: sixteen lanes share a k-contiguous row,
// a row-contiguous operand has one lane per row.  Non-finite norms become +inf,
// which sends every row that meets them to the exact route.
__global__ __launch_bounds__(256) void l2_norms_kernel(L2Args n) {
  __shared__ float red[4];
  const int tid = threadIdx.x;
  int id = blockIdx.x;
  if (id == 0 && tid == 0) n.ctrl[0] = 0;
  const bool isx = id < n.L * n.xtiles;
  if (!isx) id -= n.L * n.xtiles;
  const int per = isx ? n.xtiles : n.yblocks;
  const int b = id / per;
  const int r0 = (id - b * per) * 128;
  Operand o = isx ? n.X : n.Y;
  o.p += (long long)b * (isx ? n.strideX : n.strideY);
  const int kind = isx ? n.xk : n.yk;
  float* out = isx ? n.nx + (long long)b * n.XP : n.ny + (long long)b * n.Yext;
  const int out_rows = isx ? n.XP : n.Yext;
  float big = 0.f;
  __shared__ double halves[128];
  if (kind == KC) {
    // eight rows per lane group at a time, so that eight loads are in flight
    const int sub = tid & 15;
    const float* p[8];
    double s[8];
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
      const int row = min(r0 + pass * 16 + (tid >> 4), o.rows - 1);
      p[pass] = o.p + (long long)row * o.ld;
      s[pass] = 0.0;
    }
    // (loads are gathered into an array first: written as load-and-add, each load
    // is waited for before the next is issued)
    int k = sub;
    for (; k + 48 < n.K; k += 64) {
      float v[4][8];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int pass = 0; pass < 8; ++pass) v[j][pass] = p[pass][k + 16 * j];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int pass = 0; pass < 8; ++pass) s[pass] += (double)v[j][pass] * (double)v[j][pass];
    }
    for (; k < n.K; k += 16) {
      float v[8];
#pragma unroll
      for (int pass = 0; pass < 8; ++pass) v[pass] = p[pass][k];
#pragma unroll
      for (int pass = 0; pass < 8; ++pass) s[pass] += (double)v[pass] * (double)v[pass];
    }
#pragma unroll
    for (int pass = 0; pass < 8; ++pass) {
      const int row = r0 + pass * 16 + (tid >> 4);
      double t = s[pass];
      t += __shfl_xor(t, 1);
      t += __shfl_xor(t, 2);
      t += __shfl_xor(t, 4);
      t += __shfl_xor(t, 8);
      float f = (float)t;
      if (!(f < INFINITY)) f = INFINITY;
      if (row >= o.rows) f = INFINITY;
      else big = fmaxf(big, f);
      if (sub == 0 && row < out_rows) out[row] = f;
    }
  } else {
    // one row per lane; the two halves of the work-group take alternate k
    const int rl = tid & 127;
    const int row = r0 + rl;
    const float* p = o.p + min(row, o.rows - 1);
    double s = 0.0;
    int k = tid >> 7;
    for (; k + 62 < n.K; k += 64) {
      float v[32];
#pragma unroll
      for (int j = 0; j < 32; ++j) v[j] = p[(long long)(k + 2 * j) * o.ld];
#pragma unroll
      for (int j = 0; j < 32; ++j) s += (double)v[j] * (double)v[j];
    }
    for (; k < n.K; k += 2) {
      const double v = p[(long long)k * o.ld];
      s += v * v;
    }
    if (tid >= 128) halves[rl] = s;
    __syncthreads();
    if (tid < 128) {
      float f = (float)(s + halves[rl]);
      if (!(f < INFINITY)) f = INFINITY;
      if (row >= o.rows) f = INFINITY;
      else big = fmaxf(big, f);
      if (row < out_rows) out[row] = f;
    }
  }
  if (isx) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) big = fmaxf(big, __shfl_xor(big, m));
    if ((tid & 63) == 0) red[tid >> 6] = big;
    __syncthreads();
    if (tid == 0) n.xmax[blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  }
}

// k-contiguous copy of a row-contiguous X, in 64 x 64 tiles through LDS: the
// settle step reads whole rows of X, which this layout would spread over K cache
// lines each.
__global__ __launch_bounds__(256) void l2_transpose_kernel(L2Args n) {
  __shared__ float tile[64][65];
  const int kt = (n.K + 63) / 64, rt = (n.Xext + 63) / 64;
  int id = blockIdx.x;
  const int b = id / (kt * rt);
  id -= b * kt * rt;
  const int r0 = (id / kt) * 64, k0 = (id % kt) * 64;
  const float* src = n.X.p + (long long)b * n.strideX;
  float* dst = n.xt + (long long)b * n.Xext * n.K;
  const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
  float v[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int k = k0 + q + 4 * j, row = r0 + lane;
    v[j] = (k < n.K && row < n.Xext) ? src[(long long)k * n.X.ld + row] : 0.f;
  }
#pragma unroll
  for (int j = 0; j < 16; ++j) tile[lane][q + 4 * j] = v[j];
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int row = r0 + q + 4 * j, k = k0 + lane;
    if (row < n.Xext && k < n.K) dst[(long long)row * n.K + k] = tile[q + 4 * j][lane];
  }
}

constexpr unsigned long long kRowInit = 0x7f80000000000000ull;   // (+inf, index 0)

// One thread per kept row: folds the candidate sets of the splits, decides
// whether the screening settles the row, and if so evaluates the exact distance
// of its one or two candidates.  Undecided rows are queued.
__global__ __launch_bounds__(kFoldThreads) void min_l2_fold_kernel(L2Args f) {
  const int yb = (f.Yext + kFoldThreads - 1) / kFoldThreads;
  const int b = blockIdx.x / yb;
  const int y = (blockIdx.x - b * yb) * kFoldThreads + threadIdx.x;
  // largest |x|^2 of the batch: the wave reads the per-tile maxima side by side
  static_assert(kFoldThreads == 64, "one wave per work-group");
  float xm = 0.f;
  for (int t = threadIdx.x; t < f.xtiles; t += kFoldThreads) xm = fmaxf(xm, f.xmax[b * f.xtiles + t]);
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) xm = fmaxf(xm, __shfl_xor(xm, m));
  if (y >= f.Yext) return;
  const long long rows = (long long)f.L * f.Yext;
  const long long i = (long long)b * f.Yext + y;
  Cand c{f.pc1[i], f.pi1[i], f.pc2[i], f.pi2[i], f.ph[i]};
  for (int s = 1; s < f.splits; ++s) {
    const long long at = (long long)s * rows + i;
    const Cand o{f.pc1[at], f.pi1[at], f.pc2[at], f.pi2[at], f.ph[at]};
    c = cand_merge(c, o);
  }
  const float scale = xm + f.ny[i];
  const float W = 2.f * f.beta * scale;
  // (all three compares are false for NaN; a tiny scale would let underflow
  // matter, which the rounding budget does not cover)
  const bool settled = scale >= 1e-25f && W < INFINITY && c.h > c.c1 + W;
  if (!settled) {
    const int slot = atomicAdd(f.ctrl, 1);
    if (slot < kRowLimit) {
      f.list[slot] = (int)i;
      for (int q = 0; q < kRowBuckets; ++q) f.rowbest[slot * kRowBuckets + q] = kRowInit;
    }
    return;
  }
  const float* yp = row_base(f.Y, f.yk, y) + (long long)b * f.strideY;
  const long long ys = k_step(f.Y, f.yk);
  const long long xs = f.xt ? 1 : k_step(f.X, f.xk);
  auto xrow = [&](int x) {
    return f.xt ? f.xt + ((long long)b * f.Xext + x) * f.K : row_base(f.X, f.xk, x) + (long long)b * f.strideX;
  };
  // (the same for every thread of the launch)
  const bool vec = (f.K & 3) == 0 && ys == 1 && f.Y.vec && (f.xt != nullptr || (xs == 1 && f.X.vec));
  float v = vec ? l2_exact_vec(xrow(c.i1), yp, f.K) : l2_exact(xrow(c.i1), xs, yp, ys, f.K);
  int idx = c.i1;
  if (c.c2 <= c.c1 + W) {
    const float v2 = vec ? l2_exact_vec(xrow(c.i2), yp, f.K) : l2_exact(xrow(c.i2), xs, yp, ys, f.K);
    if (v2 < v || (v2 == v && c.i2 < idx)) { v = v2; idx = c.i2; }
  }
  if (!(v < INFINITY)) {
    // an exact distance overflowed or is NaN, the rounding budget does not hold
    const int slot = atomicAdd(f.ctrl, 1);
    if (slot < kRowLimit) {
      f.list[slot] = (int)i;
      for (int q = 0; q < kRowBuckets; ++q) f.rowbest[slot * kRowBuckets + q] = kRowInit;
    }
    return;
  }
  f.values[i] = v;
  f.indices[i] = idx;
}

// Exact recomputation of the queued rows, `parts` work-groups per row, each
// over a range of x; a 64-bit atomic minimum of (value bits, index) merges them
// (distances are non-negative, so their bit patterns order like the values, and
// equal values fall to the lowest index); min_l2_rows_finish_kernel writes the rows.
__global__ __launch_bounds__(256) void min_l2_rows_kernel(L2Args f, int Xext, int parts) {
  __shared__ unsigned long long red[4];
  constexpr int kYCache = 2048;
  __shared__ float yrow[kYCache];
  const int count = f.ctrl[0];
  if (count > kRowLimit) return;
  const int tid = threadIdx.x;
  const int xper = (Xext + parts - 1) / parts;
  for (int item = blockIdx.x; item < count * parts; item += gridDim.x) {
    const int slot = item / parts;
    const int part = item - slot * parts;
    const int i = f.list[slot];
    const int b = i / f.Yext;
    const int y = i - b * f.Yext;
    const int x0 = part * xper;
    const int x1 = min(Xext, x0 + xper);
    const float* yp = row_base(f.Y, f.yk, y) + (long long)b * f.strideY;
    const long long ys = k_step(f.Y, f.yk);
    const long long xs = k_step(f.X, f.xk);
    const bool cached = f.K <= kYCache;
    if (cached)
      for (int k = tid; k < f.K; k += 256) yrow[k] = yp[k * ys];
    __syncthreads();
    unsigned long long mine = kRowInit;
    for (int x = x0 + tid; x < x1; x += 256) {
      const float* xp = row_base(f.X, f.xk, x) + (long long)b * f.strideX;
      const float v = cached ? l2_exact_lds(xp, xs, yrow, f.K) : l2_exact(xp, xs, yp, ys, f.K);
      if (v < INFINITY) {
        const unsigned long long pk = ((unsigned long long)__float_as_uint(v) << 32) | (unsigned)x;
        mine = pk < mine ? pk : mine;
      }
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
      const unsigned long long o = __shfl_xor(mine, m);
      mine = o < mine ? o : mine;
    }
    if ((tid & 63) == 0) red[tid >> 6] = mine;
    __syncthreads();
    if (tid == 0) {
      unsigned long long m = red[0];
      for (int w = 1; w < 4; ++w) m = red[w] < m ? red[w] : m;
      if (m != kRowInit) atomicMin(&f.rowbest[slot * kRowBuckets + part % kRowBuckets], m);
    }
    __syncthreads();
  }
}

// The same for contractions of up to kTiledMaxK: a work-group keeps 32 rows of X
// in LDS and walks all queued rows against them, eight at a time (one per group
// of 32 lanes), so that X is read once whatever the number of queued rows.
constexpr int kTiledX = 32;
constexpr int kTiledMaxK = 400;
__global__ __launch_bounds__(256) void min_l2_rows_tiled_kernel(L2Args f) {
  constexpr int RG = 256 / kTiledX;
  __shared__ float xs[kTiledX * (kTiledMaxK + 1)];
  __shared__ float ysh[RG * kTiledMaxK];
  const int count = f.ctrl[0];
  if (count > kRowLimit || count == 0) return;
  const int tid = threadIdx.x;
  const int K = f.K, KP = K + 1;
  const int per_batch = (f.Xext + kTiledX - 1) / kTiledX;
  const int b = blockIdx.x / per_batch;
  const int x0 = (blockIdx.x - b * per_batch) * kTiledX;
  // X tile: [x][k], pitch K + 1.  Loads are gathered sixteen at a time before
  // they are used, so that they are in flight together.
  {
    const float* xb = f.X.p + (long long)b * f.strideX;
    if (f.xk == KC) {
      const int kl = tid & 63, xq = tid >> 6;
      for (int k0 = 0; k0 < K; k0 += 128) {
        float v[2][8];
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int k = k0 + 64 * m + kl, x = x0 + xq + 4 * j;
            v[m][j] = (k < K && x < f.Xext) ? xb[(long long)x * f.X.ld + k] : 0.f;
          }
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int k = k0 + 64 * m + kl;
            if (k < K) xs[(xq + 4 * j) * KP + k] = v[m][j];
          }
      }
    } else {
      const int x = tid & (kTiledX - 1), kq = tid / kTiledX;
      for (int k0 = 0; k0 < K; k0 += 128) {
        float v[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int k = k0 + kq + 8 * j;
          v[j] = (k < K && x0 + x < f.Xext) ? xb[(long long)k * f.X.ld + x0 + x] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int k = k0 + kq + 8 * j;
          if (k < K) xs[x * KP + k] = v[j];
        }
      }
    }
  }
  const int xl = tid & (kTiledX - 1), rg = tid / kTiledX;
  const long long ys = k_step(f.Y, f.yk);
  for (int s0 = 0; s0 < count; s0 += RG) {
    __syncthreads();   // the X tile is written; the previous round's y rows are no longer read
    {
      // y rows of this round: row r is loaded by the 32 lanes that will use it
      const int r = tid / kTiledX, kl = tid & (kTiledX - 1);
      const float* yp = nullptr;
      if (s0 + r < count) {
        const int i = f.list[s0 + r];
        const int rb = i / f.Yext;
        yp = row_base(f.Y, f.yk, i - rb * f.Yext) + (long long)rb * f.strideY;
      }
      static_assert(kTiledMaxK <= 16 * kTiledX, "one batch of sixteen loads covers a row");
      float v[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int k = kl + kTiledX * j;
        v[j] = (yp && k < K) ? yp[k * ys] : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int k = kl + kTiledX * j;
        if (k < K) ysh[r * K + k] = v[j];
      }
    }
    __syncthreads();
    const int slot = s0 + rg;
    unsigned long long mine = kRowInit;
    if (slot < count && f.list[slot] / f.Yext == b && x0 + xl < f.Xext) {
      const float* xr = xs + xl * KP;
      const float* yr = ysh + rg * K;
      float c = 0.f;
#pragma unroll 8
      for (int k = 0; k < K; ++k) {
        const float d = xr[k] - yr[k];
        c = __builtin_fmaf(d, d, c);
      }
      if (c < INFINITY) mine = ((unsigned long long)__float_as_uint(c) << 32) | (unsigned)(x0 + xl);
    }
#pragma unroll
    for (int m = kTiledX / 2; m >= 1; m >>= 1) {
      const unsigned long long o = __shfl_xor(mine, m);
      mine = o < mine ? o : mine;
    }
    if (xl == 0 && mine != kRowInit)
      atomicMin(&f.rowbest[slot * kRowBuckets + blockIdx.x % kRowBuckets], mine);
  }
}

// Writes the recomputed rows.
__global__ __launch_bounds__(256) void min_l2_rows_finish_kernel(L2Args f) {
  const int count = f.ctrl[0];
  if (count > kRowLimit) return;
  for (int slot = threadIdx.x; slot < count; slot += 256) {
    unsigned long long r = kRowInit;
    for (int q = 0; q < kRowBuckets; ++q) {
      const unsigned long long o = f.rowbest[slot * kRowBuckets + q];
      r = o < r ? o : r;
    }
    const int i = f.list[slot];
    f.values[i] = __uint_as_float((unsigned)(r >> 32));
    f.indices[i] = (long long)(unsigned)(r & 0xffffffffu);
  }
}

// How the work is cut.  Splitting the reduced axis gives more work-groups than
// the kept axis alone has strips; every candidate split count is priced as
// (rounds the machine needs for all work-groups, two per CU) x (slabs one
// work-group multiplies + what a work-group costs besides: filling the pipeline
// and the reduction across lanes and waves, measured at 2.2 us against 3.4 us per
// slab) + the fold launch when there is a split (about one slab), in quarter
// slabs, and the cheapest is taken.  When X is too large to stay in an XCD's L2
// at least four splits are used, so that fewer distinct Y strips are live per XCD.
static void plan_min(int L, int Xext, int Yext, int K, int* ystrips, int* xtiles, int* splits,
                     int* tiles_per_split, int* ygroup) {
  *ystrips = ceil_div(Yext, 128);
  *xtiles = ceil_div(Xext, 128);
  const long long strips = (long long)L * *ystrips;
  const long long slots = 2ll * compute_units();
  const long long slabs = K > 0 ? ceil_div(K, 32) : 1;
  const bool big_x = (long long)Xext * K * 4 > (2ll << 20) && *xtiles >= 32;
  const int most = *xtiles < 64 ? *xtiles : 64;
  long long best_cost = -1;
  int best_tps = *xtiles > 0 ? *xtiles : 1;
  for (int want = big_x ? 4 : 1; want <= most; ++want) {
    const int tps = ceil_div(*xtiles, want);
    const int s = ceil_div(*xtiles, tps);
    const long long total = strips * s;
    const long long rounds = (total + slots - 1) / slots;
    const long long cost = rounds * (4 * tps * slabs + 3) + (s > 1 ? 4 : 0);
    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_tps = tps; }
  }
  *tiles_per_split = best_tps;
  *splits = *xtiles > 0 ? ceil_div(*xtiles, best_tps) : 1;
  *ygroup = 64 / *splits > 0 ? 64 / *splits : 1;
}

size_t min_workspace_bytes(int L, int Xext, int Yext, int K) {
  int ys, xt, sp, tps, yg;
  plan_min(L, Xext, Yext, K, &ys, &xt, &sp, &tps, &yg);
  if (sp <= 1) return 0;
  return (size_t)sp * L * Yext * 8;
}

// Where the pieces of the screening route's workspace start (256-byte aligned).
struct L2Layout {
  size_t nx, ny, xmax, ctrl, list, rowbest, xt, parts, total;
};
static L2Layout l2_layout(int L, int Xext, int Yext, int K, int xtiles, int splits) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  L2Layout w{};
  size_t o = 0;
  w.nx = o;      o += up((size_t)L * xtiles * 128 * 4);
  w.ny = o;      o += up((size_t)L * Yext * 4);
  w.xmax = o;    o += up((size_t)L * xtiles * 4);
  w.ctrl = o;    o += up(4);
  w.list = o;    o += up((size_t)kRowLimit * 4);
  w.rowbest = o; o += up((size_t)kRowLimit * kRowBuckets * 8);
  w.xt = o;      o += up((size_t)L * Xext * K * 4);          // used when X is row-contiguous
  w.parts = o;   o += up((size_t)splits * L * Yext * 20);   // the exact route's partials reuse this piece
  w.total = o;
  return w;
}

// 0 when the screening route does not apply to the shape.
size_t min_l2_workspace_bytes(int L, int Xext, int Yext, int K) {
  if (L <= 0 || Xext <= 0 || Yext <= 0 || K <= 0) return 0;
  if ((long long)L * Yext > 0x7fffffffLL) return 0;
  int ys, xt, sp, tps, yg;
  plan_min(L, Xext, Yext, K, &ys, &xt, &sp, &tps, &yg);
  if ((long long)L * (xt + ys) > 0x7fffffffLL) return 0;
  if ((long long)L * ceil_div(Xext, 64) * ceil_div(K, 64) > 0x7fffffffLL) return 0;
  return l2_layout(L, Xext, Yext, K, xt, sp).total;
}

}  // namespace cmk

using namespace cmk;

// Validates, plans and enqueues one min_bmm; `workspace` is whatever device
// memory holds the per-split partial results (the caller's buffer, or the
// library's static scratch array).
static int min_bmm_enqueue(const float* A, const float* B, float* values, long long* indices,
                           const cmk_gemm_desc* d, int dim, int distance, void* workspace,
                           size_t workspace_bytes, void* stream) {
  if (int e = check_desc(d)) return e;
  if (dim != 1 && dim != 2) return fail(CMK_ERR_INVALID_ARG, "cmk_min_bmm_f32: dim must be 1 or 2");
  if (distance < CMK_DIST_INNER || distance > CMK_DIST_L1)
    return fail(CMK_ERR_INVALID_ARG, "cmk_min_bmm_f32: unknown distance %d", distance);
  const int Xext = dim == 2 ? d->N : d->M;
  const int Yext = dim == 2 ? d->M : d->N;
  if (Xext == 0) return fail(CMK_ERR_INVALID_ARG, "cmk_min_bmm_f32: reduction over an empty axis");
  if (d->L == 0 || Yext == 0) return CMK_OK;
  if (!values || !indices || (d->K > 0 && (!A || !B)))
    return fail(CMK_ERR_INVALID_ARG, "cmk_min_bmm_f32: null pointer");

  MinArgs a{};
  // operand kinds: A "n" is k-contiguous, A "t" is m-contiguous; B "n" is
  // n-contiguous, B "t" is k-contiguous
  const Operand opA{A, d->lda, d->M, vec_ok(A, d->lda, d->strideA)};
  const Operand opB{B, d->ldb, d->N, vec_ok(B, d->ldb, d->strideB)};
  const int kindA = d->transA ? RC : KC;
  const int kindB = d->transB ? KC : RC;
  int xk, yk;
  if (dim == 2) { a.X = opB; a.Y = opA; a.strideX = d->strideB; a.strideY = d->strideA; xk = kindB; yk = kindA; }
  else          { a.X = opA; a.Y = opB; a.strideX = d->strideA; a.strideY = d->strideB; xk = kindA; yk = kindB; }
  a.values = values;
  a.indices = indices;
  a.L = d->L;
  a.K = d->K;
  plan_min(d->L, Xext, Yext, d->K, &a.ystrips, &a.xtiles, &a.splits, &a.tiles_per_split, &a.ygroup);
  const long long total = (long long)d->L * a.ystrips * a.splits;
  if (int e = check_grid(total)) return e;
  a.total = (int)total;
  const dim3 grid((unsigned)(((total + 7) / 8) * 8)), block(kThreads);
  hipStream_t st = (hipStream_t)stream;
  const long long rows = (long long)d->L * Yext;
  const dim3 fold_grid((unsigned)((rows + kFoldThreads - 1) / kFoldThreads)), fold_block(kFoldThreads);
#define CMK_MIN_LAUNCH(DIST)                                                                        \
  do {                                                                                           \
    if (xk == KC && yk == KC) hipLaunchKernelGGL((min_kernel<KC, KC, DIST>), grid, block, 0, st, a);      \
    else if (xk == KC && yk == RC) hipLaunchKernelGGL((min_kernel<KC, RC, DIST>), grid, block, 0, st, a); \
    else if (xk == RC && yk == KC) hipLaunchKernelGGL((min_kernel<RC, KC, DIST>), grid, block, 0, st, a); \
    else hipLaunchKernelGGL((min_kernel<RC, RC, DIST>), grid, block, 0, st, a);                           \
  } while (0)
  static_assert(CMK_DIST_INNER == kInner && CMK_DIST_L2 == kL2 && CMK_DIST_L1 == kL1, "distance codes");

  // Squared l2 with the larger workspace: screen on the matrix pipe, settle
  // exactly (see the head of this file).
  const size_t l2_need = distance == CMK_DIST_L2 ? min_l2_workspace_bytes(d->L, Xext, Yext, d->K) : 0;
  if (l2_need > 0 && workspace && workspace_bytes >= l2_need &&
      (reinterpret_cast<uintptr_t>(workspace) & 255) == 0) {
    const L2Layout w = l2_layout(d->L, Xext, Yext, d->K, a.xtiles, a.splits);
    char* base = static_cast<char*>(workspace);
    const size_t n = (size_t)a.splits * d->L * Yext;
    L2Args f{};
    f.X = a.X; f.Y = a.Y; f.strideX = a.strideX; f.strideY = a.strideY; f.xk = xk; f.yk = yk;
    f.L = d->L; f.K = d->K; f.Yext = Yext; f.XP = a.xtiles * 128; f.xtiles = a.xtiles;
    f.yblocks = ceil_div(Yext, 128); f.splits = a.splits;
    f.beta = l2_beta(d->K);
    f.nx = reinterpret_cast<float*>(base + w.nx);
    f.ny = reinterpret_cast<float*>(base + w.ny);
    f.xmax = reinterpret_cast<float*>(base + w.xmax);
    f.ctrl = reinterpret_cast<int*>(base + w.ctrl);
    f.list = reinterpret_cast<int*>(base + w.list);
    f.rowbest = reinterpret_cast<unsigned long long*>(base + w.rowbest);
    f.xt = xk == RC ? reinterpret_cast<float*>(base + w.xt) : nullptr;
    f.Xext = Xext;
    float* parts = reinterpret_cast<float*>(base + w.parts);
    a.pc1 = parts;
    a.pi1 = reinterpret_cast<int*>(parts + n);
    a.pc2 = parts + 2 * n;
    a.pi2 = reinterpret_cast<int*>(parts + 3 * n);
    a.ph = parts + 4 * n;
    f.pc1 = a.pc1; f.pi1 = a.pi1; f.pc2 = a.pc2; f.pi2 = a.pi2; f.ph = a.ph;
    f.values = values; f.indices = indices;
    a.nx = f.nx;
    a.XP = f.XP;
    hipLaunchKernelGGL(l2_norms_kernel, dim3((unsigned)(d->L * (a.xtiles + f.yblocks))), dim3(256), 0, st, f);
    if (f.xt)
      hipLaunchKernelGGL(l2_transpose_kernel,
                         dim3((unsigned)(d->L * ceil_div(Xext, 64) * ceil_div(d->K, 64))), dim3(256), 0, st, f);
    CMK_MIN_LAUNCH(kL2M);
    hipLaunchKernelGGL(min_l2_fold_kernel, dim3((unsigned)(d->L * ceil_div(Yext, kFoldThreads))), fold_block,
                       0, st, f);
    const long long tiled_grid = (long long)d->L * ceil_div(Xext, kTiledX);
    if (d->K <= kTiledMaxK && tiled_grid <= 0x7fffffffLL) {
      hipLaunchKernelGGL(min_l2_rows_tiled_kernel, dim3((unsigned)tiled_grid), dim3(256), 0, st, f);
    } else {
      const int row_parts = ceil_div(Xext, 256) < kRowMaxParts ? ceil_div(Xext, 256) : kRowMaxParts;
      hipLaunchKernelGGL(min_l2_rows_kernel, dim3(kRowGrid), dim3(256), 0, st, f, Xext, row_parts);
    }
    hipLaunchKernelGGL(min_l2_rows_finish_kernel, dim3(1), dim3(256), 0, st, f);
    // the vector route over everything, alive only when too many rows are undecided
    a.gate = f.ctrl;
    a.gate_limit = kRowLimit;
    a.part_val = parts;
    a.part_idx = reinterpret_cast<int*>(parts + n);
    CMK_MIN_LAUNCH(kL2);
    if (a.splits > 1)
      hipLaunchKernelGGL(min_fold_kernel, fold_grid, fold_block, 0, st, a.part_val, a.part_idx, values,
                         indices, rows, a.splits, a.gate, a.gate_limit);
    return hip_status(hipGetLastError(), "cmk_min_bmm_f32 (screened l2) launch");
  }

  if (a.splits > 1) {
    const size_t need = (size_t)a.splits * d->L * Yext * 8;
    if (!workspace || workspace_bytes < need)
      return fail(CMK_ERR_WORKSPACE, "cmk_min_bmm_f32: workspace of %zu bytes required, %zu given",
                  need, workspace_bytes);
    a.part_val = static_cast<float*>(workspace);
    a.part_idx = reinterpret_cast<int*>(a.part_val + (size_t)a.splits * d->L * Yext);
  }
  if (distance == CMK_DIST_INNER) CMK_MIN_LAUNCH(kInner);
  else if (distance == CMK_DIST_L2) CMK_MIN_LAUNCH(kL2);
  else CMK_MIN_LAUNCH(kL1);
  if (int e = hip_status(hipGetLastError(), "cmk_min_bmm_f32 launch")) return e;
  if (a.splits > 1) {
    hipLaunchKernelGGL(min_fold_kernel, fold_grid, fold_block, 0, st, a.part_val, a.part_idx, values, indices,
                       rows, a.splits, (const int*)nullptr, 0);
    if (int e = hip_status(hipGetLastError(), "cmk_min_bmm_f32 fold launch")) return e;
  }
#undef CMK_MIN_LAUNCH
  return CMK_OK;
}

extern "C" int cmk_min_bmm_f32(const float* A, const float* B, float* values, long long* indices,
                               const cmk_gemm_desc* d, int dim, int distance, void* workspace,
                               size_t workspace_bytes, void* stream) {
  return min_bmm_enqueue(A, B, values, indices, d, dim, distance, workspace, workspace_bytes, stream);
}

// Scratch of the allocation-free entry point: one array per GPU, created with
// the code object and kept until the process ends.  In host code this name is
// only a handle for hipGetSymbolAddress; kernels and copies get the device
// address that call returns.
static __device__ __align__(256) unsigned char scratch[CMK_STATIC_SCRATCH_BYTES];

namespace cmk {
constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device, looked up once per device.
static int static_scratch(void** out) {
  int dev = -1;
  if (int e = hip_status(hipGetDevice(&dev), "cmk_min_bmm_f32_static: hipGetDevice")) return e;
  if (dev < 0 || dev >= kMaxDevices)
    return fail(CMK_ERR_UNSUPPORTED, "cmk_min_bmm_f32_static: device ordinal %d beyond %d", dev, kMaxDevices - 1);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (int e = hip_status(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)),
                           "cmk_min_bmm_f32_static: hipGetSymbolAddress"))
      return e;
    if (!p) return fail(CMK_ERR_UNSUPPORTED, "cmk_min_bmm_f32_static: no address for the scratch array");
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return CMK_OK;
}
}  // namespace cmk

extern "C" int cmk_min_bmm_f32_static(const float* A, const float* B, float* values, long long* indices,
                                      const cmk_gemm_desc* d, int dim, int distance, void* stream) {
  if (int e = check_desc(d)) return e;
  if (dim != 1 && dim != 2) return fail(CMK_ERR_INVALID_ARG, "cmk_min_bmm_f32_static: dim must be 1 or 2");
  const size_t need = cmk_workspace_bytes(CMK_OP_MIN_BMM, d->L, d->M, d->N, d->K, dim);
  if (need > (size_t)CMK_STATIC_SCRATCH_BYTES)
    return fail(CMK_ERR_WORKSPACE,
                "cmk_min_bmm_f32_static: this problem needs %zu bytes of scratch, the static array holds %zu; "
                "use cmk_min_bmm_f32 with a workspace", need, (size_t)CMK_STATIC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (need > 0)
    if (int e = static_scratch(&ws)) return e;
  return min_bmm_enqueue(A, B, values, indices, d, dim, distance, ws, need, stream);
}
