// The top-k kernel template, shared by the translation units that instantiate
// it (the inner product in cmk_topk.hip, the vector-unit distances in
// cmk_topk_dist.hip, so that they compile side by side).
#pragma once
#include "cmk_core.hpp"
#include "cmk_launch.hpp"
#include "cmk_select.hpp"

namespace cmk {

constexpr int kTileX = 256;                    // candidates per tile
constexpr int kChunkTiles = 4;                 // tiles per chunk: 1024 candidates
constexpr int kStagePitch = kTileX * kChunkTiles + 8;

struct TopkArgs {
  Operand X, Y;
  long long strideX, strideY;
  float* values;        // [L][Yext][k]
  long long* indices;   // [L][Yext][k]
  entry_t* part;        // [splits][L*Yext][128] unordered lists (splits > 1)
  int L, K, k;
  int ystrips, xtiles, splits, tiles_per_split;
};

constexpr int kTopkThreads = 1024;
constexpr int kStripRows = 64;    // output rows per work-group
constexpr int kPassRows = 16;     // rows staged through LDS per selection pass

// MULTI = false: the whole reduced axis is one chunk (at most 1024 candidates);
// the lists are then only written after the product is finished and may share
// LDS with the operand buffers.  MULTI = true: the lists carry state from chunk
// to chunk and sit behind the operand buffers.
template <int XK, int YK, bool MULTI, int DIST>
__global__ __launch_bounds__(kTopkThreads, 1) void topk_kernel(TopkArgs a) {
  // Sixteen waves, four per SIMD: selection and ordering are long chains of
  // dependent vector, scalar and LDS instructions, of which one wave issues one
  // every 5 to 10 cycles; four waves keep the SIMD's issue slots far better
  // filled than two (measured: 1.4x).  The phases of a work-group cannot
  // overlap on this part (vector instructions of one wave do not issue while
  // another wave of the SIMD streams MFMAs): all waves multiply, then all select.
  // wave % 8 picks 32 of a tile's 256 candidates, wave / 8 one of the two 32-row
  // halves of the strip; a wave's 64 accumulator registers cover 4 tiles =
  // 1024 candidates x 32 rows.
  // With a single chunk the operand buffers may fill LDS (the lists are written
  // after the product), which allows tiles of 512 candidates, two 32x32 blocks
  // per wave: half as many fragment reads of the strip's rows and half as many
  // barriers per MFMA.
  constexpr int kBX = MULTI ? 1 : 2;
  constexpr int kTX = kTileX * kBX;             // candidates per tile in this kernel
  constexpr int kCT = kChunkTiles / kBX;        // tiles per chunk in this kernel
  using C = Core<XK, YK, 8, 2, kBX, 1, 32, kReadsSingle, false, true, false>;
  static_assert(C::TX == kTX && C::TY == kStripRows && C::NT == kTopkThreads, "tile shape");
  // LDS: operand buffers, reused as the staging area; the lists follow the
  // staging area (MULTI: the operand buffers, which they must outlive)
  constexpr int stageFloats = kPassRows * kStagePitch;
  constexpr int listFloats = kStripRows * kTop * 2;
  constexpr int listAt = MULTI ? (C::ldsFloats > stageFloats ? C::ldsFloats : stageFloats) : stageFloats;
  // MULTI: behind the lists, the smallest key of every row's list once it is full
  constexpr int thrAt = listAt + listFloats;
  constexpr int endFloats = thrAt + (MULTI ? kStripRows : 0);
  constexpr int selFloats = endFloats > C::ldsFloats ? endFloats : C::ldsFloats;
  static_assert(selFloats * 4 <= 160 * 1024, "LDS capacity");
  __shared__ __attribute__((aligned(16))) float lds[selFloats];
  // running top-128 of every row of the strip
  entry_t(*list)[kTop] = reinterpret_cast<entry_t(*)[kTop]>(lds + listAt);
  uint32_t* const row_thr = reinterpret_cast<uint32_t*>(lds + thrAt);


  // the previous row's threshold seeds the next search; it carries over from
  // strip to strip, since neighbouring strips are statistically alike
  uint32_t seed = 0u;

  // A work-group walks strips blockIdx.x, blockIdx.x + gridDim.x, ... (the
  // grid is sized to the machine, not to the problem).
  const int per_split = a.L * a.ystrips;
  const int total = per_split * a.splits;
  const int padded = ((total + 7) >> 3) << 3;
#pragma unroll 1
  for (int hw = blockIdx.x; hw < padded; hw += gridDim.x) {
  const int logical = xcd_logical_id(hw, total);
  if (logical < 0) continue;
  __syncthreads();  // the previous strip's lists have been stored
  const int split = logical / per_split;
  const int rem = logical - split * per_split;
  const int b = rem / a.ystrips;
  const int ystrip = rem - b * a.ystrips;
  const int y0 = ystrip * kStripRows;
  const int xt_begin = split * a.tiles_per_split;
  const int xt_end = min(a.xtiles, xt_begin + a.tiles_per_split);

  Operand X = a.X, Y = a.Y;
  X.p = uniform_ptr(X.p + (long long)b * a.strideX);
  Y.p = uniform_ptr(Y.p + (long long)b * a.strideY);
  const int x_limit = min(X.rows, xt_end * kTileX);
  const int Yext = Y.rows;

  if constexpr (MULTI) {
    // running lists start empty
    for (int e = threadIdx.x; e < kStripRows * kTop; e += kTopkThreads) (&list[0][0])[e] = 0ull;
    __syncthreads();
  }
  C core;

  for (int xt0 = xt_begin; xt0 < xt_end; xt0 += kChunkTiles) {
    const int nt = (min(kChunkTiles, xt_end - xt0) + kBX - 1) / kBX;
    __syncthreads();  // previous chunk's staging reads are finished
    core.begin(X, Y, xt0 * kTileX, y0, a.K, nt, lds);
    f32x16 acc[kCT][kBX][1];
    // k-slabs outside, tiles inside: a slab of the strip's own rows is fetched
    // once and meets the chunk's tiles one after the other
    // The first k-slab starts the accumulators from a literal zero (matrix path):
    // no clearing.  Tiles a short last chunk does not have are cleared instead.
    static_for<0, kCT>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      if (i < nt) {
        if constexpr (DIST != kInner) {
#pragma unroll
          for (int bx = 0; bx < kBX; ++bx)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][bx][0][r] = 0.f;
        }
        core.template slab<DIST, DIST == kInner>(X, Y, lds, acc[i]);
      } else {
#pragma unroll
        for (int bx = 0; bx < kBX; ++bx)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][bx][0][r] = 0.f;
      }
    });
    for (int s = 1; s < core.S; ++s) {
#pragma unroll
      for (int i = 0; i < kCT; ++i)
        if (i < nt) core.template slab<DIST>(X, Y, lds, acc[i]);
    }
    __syncthreads();  // all fragment reads are done; the buffers become the staging area

    // Everything derived from the lane id is derived here, after the product and
    // again for every chunk: kept across the product (or across strips) it would
    // only occupy, or spill, registers there, and a reload from scratch costs
    // more than the two or three instructions that recompute it.
    int tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int half = lane >> 5;
    const int wx = wave & 7;   // which 32 candidates of a tile
    const int wy = wave >> 3;  // which half of the strip's rows
    // a staged row, once in registers, lends its space to the candidate list
    entry_t* cand = reinterpret_cast<entry_t*>(lds + wave * kStagePitch);

    // selection, sixteen rows of the strip per pass
    const int xc0 = xt0 * kTileX;
#pragma unroll 1
    for (int g = 0; g < kStripRows / kPassRows; ++g) {
      if (g) __syncthreads();  // previous pass has been read
      // rows 16g .. 16g+15 live in the waves with wy == g / 2, lanes l32 / 16 == g % 2
      if (wy == (g >> 1) && (l32 >> 4) == (g & 1)) {
        float* row = lds + (l32 & 15) * kStagePitch + wx * 32 * kBX + 4 * half;
#pragma unroll
        for (int i = 0; i < kCT; ++i)
#pragma unroll
          for (int bx = 0; bx < kBX; ++bx)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              f32x4 v = {acc[i][bx][0][4 * q], acc[i][bx][0][4 * q + 1], acc[i][bx][0][4 * q + 2],
                         acc[i][bx][0][4 * q + 3]};
              *reinterpret_cast<f32x4*>(row + i * kTX + bx * 32 + 8 * q) = v;
            }
      }
      __syncthreads();
#pragma unroll 1
      for (int rr = 0; rr < 1; ++rr) {
        const int pr = wave;                   // row of the pass, owned by this wave
        const int r = kPassRows * g + pr;      // row of the strip
        if (y0 + r >= Yext) continue;
        const float* src = lds + pr * kStagePitch;
        const int xl = xc0 + lane;
        uint32_t k16[16];  // fp32 bit patterns
        if (xc0 + 1024 <= x_limit) {
#pragma unroll
          for (int j = 0; j < 16; ++j) k16[j] = __float_as_uint(src[lane + 64 * j]);
        } else {
#pragma unroll
          for (int j = 0; j < 16; ++j)
            k16[j] = xl + 64 * j < x_limit ? __float_as_uint(src[lane + 64 * j]) : kNoCandidate;
        }
        if (!MULTI || xt0 == xt_begin) {
          // first chunk: the running list is empty
          select128<16>(k16, [&](int j) { return xl + 64 * j; }, seed, cand, list[r]);
          if constexpr (MULTI) row_thr[r] = seed;
        } else {
          // a full list takes the few candidates that beat its smallest entry by
          // the short route; otherwise list and chunk are selected from together
          uint32_t thr = row_thr[r];
          if (thr == 0u || !insert128(k16, [&](int j) { return xl + 64 * j; }, thr, cand, list[r])) {
            uint32_t key[18];
#pragma unroll
            for (int j = 0; j < 16; ++j) key[j] = k16[j];
            const entry_t e0 = list[r][lane], e1 = list[r][lane + 64];
            key[16] = key2raw(entry_key(e0));
            key[17] = key2raw(entry_key(e1));
            const int ri0 = entry_idx(e0), ri1 = entry_idx(e1);
            select128<18>(key, [&](int j) { return j < 16 ? xl + 64 * j : (j == 16 ? ri0 : ri1); },
                          seed, cand, list[r]);
            thr = seed;
          }
          row_thr[r] = thr;
        }
      }
    }
  }

  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63;
  const int wave = tid >> 6;
  uint32_t* sort_scratch = reinterpret_cast<uint32_t*>(lds + wave * kStagePitch);
  // each wave finishes the four rows it owns, two at a time
#pragma unroll 1
  for (int g = 0; g < 4; g += 2) {
    const int ra = kPassRows * g + wave, rb = ra + kPassRows;
    if (a.splits == 1) {
      float* vals[2];
      long long* inds[2];
#pragma unroll
      for (int rr = 0; rr < 2; ++rr) {
        const int y = y0 + (rr ? rb : ra);
        const long long orow = (long long)b * Yext + y;
        vals[rr] = y < Yext ? a.values + orow * a.k : nullptr;
        inds[rr] = y < Yext ? a.indices + orow * a.k : nullptr;
      }
      sort_and_store_pair((lds_entry_ptr)list[ra], (lds_entry_ptr)list[rb], (lds_u32_ptr)sort_scratch,
                          vals[0], vals[1], inds[0], inds[1], a.k);
    } else {
#pragma unroll
      for (int rr = 0; rr < 2; ++rr) {
        const int r = rr ? rb : ra;
        const int y = y0 + r;
        if (y >= Yext) continue;
        const long long o = ((long long)split * a.L * Yext + (long long)b * Yext + y) * kTop;
        a.part[o + lane] = list[r][lane];
        a.part[o + lane + 64] = list[r][lane + 64];
      }
    }
  }
  }  // strips
}


// Launches topk_kernel<., ., ., DIST> for the operand kinds and chunking given.
template <int DIST>
inline void launch_topk_kernel(int xk, int yk, bool multi, dim3 grid, dim3 block, hipStream_t st,
                               const TopkArgs& a) {
#define CMK_TOPK_LAUNCH(XKIND, YKIND)                                                              \
  do {                                                                                             \
    if (multi) hipLaunchKernelGGL((topk_kernel<XKIND, YKIND, true, DIST>), grid, block, 0, st, a);  \
    else hipLaunchKernelGGL((topk_kernel<XKIND, YKIND, false, DIST>), grid, block, 0, st, a);       \
  } while (0)
  if (xk == KC && yk == KC) CMK_TOPK_LAUNCH(KC, KC);
  else if (xk == KC && yk == RC) CMK_TOPK_LAUNCH(KC, RC);
  else if (xk == RC && yk == KC) CMK_TOPK_LAUNCH(RC, KC);
  else CMK_TOPK_LAUNCH(RC, RC);
#undef CMK_TOPK_LAUNCH
}
// defined in cmk_topk_dist.hip
void launch_topk_dist(int distance, int xk, int yk, bool multi, dim3 grid, dim3 block, hipStream_t st,
                      const TopkArgs& a);

}  // namespace cmk
