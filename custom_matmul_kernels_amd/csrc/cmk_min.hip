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
};

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

  Operand X = a.X, Y = a.Y;
  X.p = uniform_ptr(X.p + (long long)b * a.strideX);
  Y.p = uniform_ptr(Y.p + (long long)b * a.strideY);

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  const int wx = wave % 2, wy = wave / 2;

  float best[2] = {INFINITY, INFINITY};
  int bidx[2] = {xt_begin * C::TX, xt_begin * C::TX};

  C core;
  core.begin(X, Y, xt_begin * C::TX, y0, a.K, xt_end - xt_begin, lds);
  for (int xt = xt_begin; xt < xt_end; ++xt) {
    f32x16 acc[2][2];
    if constexpr (DIST != kInner) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    }
    core.template tile<DIST, DIST == kInner>(X, Y, lds, acc);
    // Fold this tile into the running minimum.  Inside the tile a lane tracks the
    // position of its minimum as a small code (block * 16 + register: a literal
    // per compare, no index registers); indices ascend with the code, so a strict
    // '<' keeps the first occurrence.  The code becomes an index once per tile.
    const int xb = xt * C::TX + wx * 64;
    // (every search starts from +inf, not from the first product: a NaN there
    // would lose every later comparison and hide the rest of the tile)
    float tbest[2] = {INFINITY, INFINITY};
    int tcode[2] = {0, 0};
    if (xb + 64 <= X.rows) {
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
                                                                long long rows, int splits) {
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows) return;
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
  if (a.splits > 1) {
    const size_t need = (size_t)a.splits * d->L * Yext * 8;
    if (!workspace || workspace_bytes < need)
      return fail(CMK_ERR_WORKSPACE, "cmk_min_bmm_f32: workspace of %zu bytes required, %zu given",
                  need, workspace_bytes);
    a.part_val = static_cast<float*>(workspace);
    a.part_idx = reinterpret_cast<int*>(a.part_val + (size_t)a.splits * d->L * Yext);
  }
  const long long total = (long long)d->L * a.ystrips * a.splits;
  if (int e = check_grid(total)) return e;
  a.total = (int)total;
  const dim3 grid((unsigned)(((total + 7) / 8) * 8)), block(kThreads);
  hipStream_t st = (hipStream_t)stream;
#define CMK_MIN_LAUNCH(DIST)                                                                        \
  do {                                                                                           \
    if (xk == KC && yk == KC) hipLaunchKernelGGL((min_kernel<KC, KC, DIST>), grid, block, 0, st, a);      \
    else if (xk == KC && yk == RC) hipLaunchKernelGGL((min_kernel<KC, RC, DIST>), grid, block, 0, st, a); \
    else if (xk == RC && yk == KC) hipLaunchKernelGGL((min_kernel<RC, KC, DIST>), grid, block, 0, st, a); \
    else hipLaunchKernelGGL((min_kernel<RC, RC, DIST>), grid, block, 0, st, a);                           \
  } while (0)
  static_assert(CMK_DIST_INNER == kInner && CMK_DIST_L2 == kL2 && CMK_DIST_L1 == kL1, "distance codes");
  if (distance == CMK_DIST_INNER) CMK_MIN_LAUNCH(kInner);
  else if (distance == CMK_DIST_L2) CMK_MIN_LAUNCH(kL2);
  else CMK_MIN_LAUNCH(kL1);
#undef CMK_MIN_LAUNCH
  if (int e = hip_status(hipGetLastError(), "cmk_min_bmm_f32 launch")) return e;
  if (a.splits > 1) {
    const long long rows = (long long)d->L * Yext;
    hipLaunchKernelGGL(min_fold_kernel, dim3((unsigned)((rows + kFoldThreads - 1) / kFoldThreads)),
                       dim3(kFoldThreads), 0, st,
                       a.part_val, a.part_idx, values, indices, rows, a.splits);
    if (int e = hip_status(hipGetLastError(), "cmk_min_bmm_f32 fold launch")) return e;
  }
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
