// topk_bmm: fused per-row top-128 (largest, sorted descending) of A@B along
// one axis; the product never reaches HBM.
//
// X = the reduced axis (inside a lane), Y = the kept axis.  A work-group of
// sixteen waves owns a strip of 64 complete output rows and walks the reduced
// axis in chunks of 1024 candidates (4 tiles of 256) whose accumulators all
// stay in registers.  After each chunk the accumulators go through LDS, sixteen
// rows at a time, so that one wave sees one row's 1024 candidates (16 per lane)
// together with the row's running list (2 per lane); select128() keeps the best
// 128 in the running list in LDS.  After the last chunk each wave orders its
// rows' lists with the bitonic network and stores them.  When the kept axis has
// too few strips to fill the chip, the reduced axis is cut into `splits` ranges
// whose unordered lists go to a workspace and are merged by a second kernel.
//
// Plays the role of topk_bmm_* with topk_dim_1 / topk_dim_2, bitonic_sort_128,
// bitonic_sort_256 and the row mutex (reference kernels/topkbmm.cu:13-303,
// 499-594), and of the standalone bitonic_sort kernel
// (reference kernels/bitonic_sort.cu:182-216).
#include "cmk_topk_kernel.hpp"

namespace cmk {

// One wave per output row: folds `parts` unordered 128-entry lists into one,
// orders it and stores the first k entries.
__global__ __launch_bounds__(kThreads) void topk_merge_kernel(const entry_t* part, float* values,
                                                              long long* indices, long long rows,
                                                              int parts, int k) {
  __shared__ entry_t list[4][kTop];
  __shared__ entry_t cands[4][kCand];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const long long row = (long long)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  list[wave][lane] = 0ull;
  list[wave][lane + 64] = 0ull;
  uint32_t seed = 0u;
  for (int p0 = 0; p0 < parts; p0 += 8) {
    uint32_t key[18];  // fp32 bit patterns
    int idx[18];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int p = p0 + (j >> 1);
      const entry_t e = p < parts ? part[((long long)p * rows + row) * kTop + lane + 64 * (j & 1)] : 0ull;
      key[j] = key2raw(entry_key(e));
      idx[j] = entry_idx(e);
    }
    const entry_t r0 = list[wave][lane], r1 = list[wave][lane + 64];
    key[16] = key2raw(entry_key(r0));
    idx[16] = entry_idx(r0);
    key[17] = key2raw(entry_key(r1));
    idx[17] = entry_idx(r1);
    select128<18>(key, [&](int j) { return idx[j]; }, seed, cands[wave], list[wave]);
  }
  const entry_t* const lists[1] = {list[wave]};
  uint32_t* const scratch[1] = {reinterpret_cast<uint32_t*>(cands[wave])};
  float* const cv[1] = {values + row * k};
  long long* const ci[1] = {indices + row * k};
  sort_and_store<1>(lists, scratch, cv, ci, k);
}

// One wave per part of a 1-D array: keeps the best 128 of its range.
__global__ __launch_bounds__(kThreads) void topk1d_partial_kernel(const float* arr, long long n,
                                                                  long long span, int parts,
                                                                  entry_t* part) {
  __shared__ entry_t list[4][kTop];
  __shared__ entry_t cands[4][kCand];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int p = blockIdx.x * 4 + wave;
  if (p >= parts) return;
  list[wave][lane] = 0ull;
  list[wave][lane + 64] = 0ull;
  uint32_t seed = 0u;
  const long long begin = (long long)p * span;
  const long long end = begin + span < n ? begin + span : n;
  for (long long c0 = begin; c0 < end; c0 += 1024) {
    uint32_t key[18];  // fp32 bit patterns
    int idx[18];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const long long x = c0 + lane + 64 * j;
      const bool ok = x < end;
      key[j] = ok ? __float_as_uint(arr[x]) : kNoCandidate;
      idx[j] = (int)x;
    }
    const entry_t r0 = list[wave][lane], r1 = list[wave][lane + 64];
    key[16] = key2raw(entry_key(r0));
    idx[16] = entry_idx(r0);
    key[17] = key2raw(entry_key(r1));
    idx[17] = entry_idx(r1);
    select128<18>(key, [&](int j) { return idx[j]; }, seed, cands[wave], list[wave]);
  }
  const long long o = (long long)p * kTop;
  part[o + lane] = list[wave][lane];
  part[o + lane + 64] = list[wave][lane + 64];
}

static void plan_topk(int L, int Xext, int Yext, int K, int* ystrips, int* xtiles, int* splits,
                      int* tiles_per_split) {
  *ystrips = ceil_div(Yext, kStripRows);
  *xtiles = ceil_div(Xext, kTileX);
  const long long strips = (long long)L * *ystrips;
  const int chunks = ceil_div(*xtiles, kChunkTiles);
  // Every candidate split count is priced as (rounds the machine needs, one
  // work-group per CU) x (chunks per work-group x (slabs of a chunk + its
  // selection, worth about 3.5 slabs) + ordering and start-up), plus the merge
  // launch when the reduced axis is split; the cheapest wins.
  const long long slots = compute_units();
  const long long slabs = K > 0 ? ceil_div(K, 32) : 1;
  const int most = chunks < 64 ? chunks : 64;
  long long best_cost = -1;
  int best_cps = chunks > 0 ? chunks : 1;
  for (int want = 1; want <= most; ++want) {
    const int cps = ceil_div(chunks, want);
    const int s = ceil_div(chunks, cps);
    const long long rounds = (strips * s + slots - 1) / slots;
    const long long cost = rounds * (cps * (2 * slabs + 7) + 4) + (s > 1 ? 3 : 0);   // in half slabs
    if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_cps = cps; }
  }
  *tiles_per_split = best_cps * kChunkTiles;
  *splits = *xtiles > 0 ? ceil_div(*xtiles, *tiles_per_split) : 1;
}

size_t topk_workspace_bytes(int L, int Xext, int Yext, int K) {
  int ys, xt, sp, tps;
  plan_topk(L, Xext, Yext, K, &ys, &xt, &sp, &tps);
  if (sp <= 1) return 0;
  return (size_t)sp * L * Yext * kTop * 8;
}

static void plan_topk1d(long long n, long long* span, int* parts) {
  long long s = (n + 1023) / 1024;   // chunks in total
  long long per = (s + 1023) / 1024; // chunks per part, at most 1024 parts
  if (per < 1) per = 1;
  *span = per * 1024;
  *parts = (int)((n + *span - 1) / *span);
  if (*parts < 1) *parts = 1;
}

size_t topk1d_workspace_bytes(long long n) {
  long long span;
  int parts;
  plan_topk1d(n, &span, &parts);
  return (size_t)parts * kTop * 8;
}

}  // namespace cmk

using namespace cmk;

extern "C" int cmk_topk_bmm_f32(const float* A, const float* B, float* values, long long* indices,
                                const cmk_gemm_desc* d, int dim, int k, int distance,
                                void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_desc(d)) return e;
  if (dim != 1 && dim != 2) return fail(CMK_ERR_INVALID_ARG, "cmk_topk_bmm_f32: dim must be 1 or 2");
  if (k <= 0 || k > kTop) return fail(CMK_ERR_INVALID_ARG, "cmk_topk_bmm_f32: k must be in 1..128");
  if (distance < CMK_DIST_INNER || distance > CMK_DIST_L1)
    return fail(CMK_ERR_INVALID_ARG, "cmk_topk_bmm_f32: unknown distance %d", distance);
  const int Xext = dim == 2 ? d->N : d->M;
  const int Yext = dim == 2 ? d->M : d->N;
  if (d->L == 0 || Yext == 0) return CMK_OK;
  if (!values || !indices || (d->K > 0 && Xext > 0 && (!A || !B)))
    return fail(CMK_ERR_INVALID_ARG, "cmk_topk_bmm_f32: null pointer");

  TopkArgs a{};
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
  a.k = k;
  plan_topk(d->L, Xext, Yext, d->K, &a.ystrips, &a.xtiles, &a.splits, &a.tiles_per_split);
  if (a.xtiles == 0) { a.xtiles = 0; a.splits = 1; a.tiles_per_split = kChunkTiles; }
  if (a.splits > 1) {
    const size_t need = (size_t)a.splits * d->L * Yext * kTop * 8;
    if (!workspace || workspace_bytes < need)
      return fail(CMK_ERR_WORKSPACE, "cmk_topk_bmm_f32: workspace of %zu bytes required, %zu given",
                  need, workspace_bytes);
    a.part = static_cast<entry_t*>(workspace);
  }
  const long long total = (long long)d->L * a.ystrips * a.splits;
  if (int e = check_grid(total)) return e;
  // one sixteen-wave work-group per CU is resident at a time; a grid of two per CU evens out the tail
  const long long padded = ((total + 7) / 8) * 8;
  const long long machine = 2ll * compute_units();
  const dim3 grid((unsigned)(padded < machine ? padded : machine)), block(kTopkThreads);
  hipStream_t st = (hipStream_t)stream;
  // an empty reduced axis takes the multi-chunk instance, whose lists start out
  // empty: every slot of the result is then -inf / -1
  const bool multi = a.splits > 1 || a.xtiles > kChunkTiles || a.xtiles == 0;
  if (distance == CMK_DIST_INNER) launch_topk_kernel<kInner>(xk, yk, multi, grid, block, st, a);
  else launch_topk_dist(distance, xk, yk, multi, grid, block, st, a);
  if (int e = hip_status(hipGetLastError(), "cmk_topk_bmm_f32 launch")) return e;
  if (a.splits > 1) {
    const long long rows = (long long)d->L * Yext;
    if (int e = check_grid((rows + 3) / 4)) return e;
    hipLaunchKernelGGL(topk_merge_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(kThreads), 0, st,
                       a.part, values, indices, rows, a.splits, k);
    if (int e = hip_status(hipGetLastError(), "cmk_topk_bmm_f32 merge launch")) return e;
  }
  return CMK_OK;
}

extern "C" int cmk_topk_1d_f32(const float* arr, long long n, float* values, long long* indices,
                               int k, void* workspace, size_t workspace_bytes, void* stream) {
  if (n < 0 || n > 0x7fffffffLL) return fail(CMK_ERR_INVALID_ARG, "cmk_topk_1d_f32: bad length");
  if (k <= 0 || k > kTop) return fail(CMK_ERR_INVALID_ARG, "cmk_topk_1d_f32: k must be in 1..128");
  if (!values || !indices || (n > 0 && !arr))
    return fail(CMK_ERR_INVALID_ARG, "cmk_topk_1d_f32: null pointer");
  long long span;
  int parts;
  plan_topk1d(n, &span, &parts);
  const size_t need = (size_t)parts * kTop * 8;
  if (!workspace || workspace_bytes < need)
    return fail(CMK_ERR_WORKSPACE, "cmk_topk_1d_f32: workspace of %zu bytes required, %zu given",
                need, workspace_bytes);
  entry_t* part = static_cast<entry_t*>(workspace);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(topk1d_partial_kernel, dim3((unsigned)((parts + 3) / 4)), dim3(kThreads), 0, st,
                     arr, n, span, parts, part);
  if (int e = hip_status(hipGetLastError(), "cmk_topk_1d_f32 launch")) return e;
  hipLaunchKernelGGL(topk_merge_kernel, dim3(1), dim3(kThreads), 0, st, part, values, indices,
                     (long long)1, parts, k);
  return hip_status(hipGetLastError(), "cmk_topk_1d_f32 merge launch");
}
