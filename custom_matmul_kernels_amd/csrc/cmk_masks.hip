// Derivation of mbmm's block and thread masks from an element mask.
//
// thread_mask[b][i][j] = number of non-zero element-mask bytes in the 8x8
// micro-tile (i, j) (0..64), block_mask[b][I][J] = 1 when the 128x128 tile
// (I, J) holds any (the rule of reference colab/test_mbmm.ipynb:1295-1313,
// extended with zero padding to extents that are not multiples of 8 / 128).
//
// Byte work bound by HBM reads.  A thread owns two neighbouring micro-tiles: it
// loads their 16 bytes of each of the 8 rows (8 independent 16-byte loads in
// flight) and counts in registers, so no lanes exchange data.  LPR lanes sit
// side by side along a row (LPR x 16 contiguous bytes per row), the 64 / LPR
// lane groups of a wave take consecutive micro-rows, and a work-group of four
// waves covers 128 rows x LPR*16 columns, i.e. LPR / 8 block tiles.
#include "cmk_launch.hpp"

namespace cmk {

constexpr int kMaskThreads = 256;

struct MaskArgs {
  const uint8_t* element_mask;
  uint8_t* block_mask;
  uint8_t* thread_mask;
  int Lm, M, N;
  int tiles_m, tiles_n, spans_n, m8, n8;
  int aligned;  // rows of the element mask start on 16-byte boundaries
  int pairs;    // rows of the thread mask start on 2-byte boundaries
};

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// number of non-zero bytes of a 32-bit word
__device__ __forceinline__ unsigned nonzero_bytes(unsigned x) {
  const unsigned hi = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;
  return __builtin_popcount(hi);
}

template <int LPR>
__global__ __launch_bounds__(kMaskThreads) void derive_masks_kernel(MaskArgs a) {
  constexpr int kSpan = LPR * 16;             // columns per work-group
  constexpr int kBlocks = LPR / 8;            // block tiles per work-group
  constexpr int kRowsPerPass = 4 * (64 / LPR);  // micro-rows the four waves cover at once
  constexpr int kPasses = 16 / kRowsPerPass;
  static_assert(kPasses >= 1, "a pass must not exceed the 128-row tile");
  __shared__ int kept_blocks[kBlocks];

  const int per_batch = a.tiles_m * a.spans_n;
  const int b = blockIdx.x / per_batch;
  const int t = blockIdx.x - b * per_batch;
  const int tile_m = t / a.spans_n;
  const int span = t - tile_m * a.spans_n;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = span * kSpan + (lane % LPR) * 16;
  const uint8_t* eb = a.element_mask + (long long)b * a.M * a.N;
  const bool fast_cols = a.aligned && col + 16 <= a.N;

  if (threadIdx.x < kBlocks) kept_blocks[threadIdx.x] = 0;
  __syncthreads();

  unsigned kept = 0;
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int micro_row = tile_m * 16 + p * kRowsPerPass + wave * (64 / LPR) + lane / LPR;
    const int row0 = micro_row * 8;
    unsigned lo = 0, hi = 0;
    if (fast_cols && row0 + 8 <= a.M) {
      typedef const u32x4 __attribute__((address_space(1))) * g16p;
      u32x4 v[8];
      // read once: non-temporal loads (measured: 6.1 instead of 5.75 TB/s on a 4 GiB mask)
#pragma unroll
      for (int r = 0; r < 8; ++r) v[r] = __builtin_nontemporal_load((g16p)(eb + (long long)(row0 + r) * a.N + col));
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        lo += nonzero_bytes(v[r][0]) + nonzero_bytes(v[r][1]);
        hi += nonzero_bytes(v[r][2]) + nonzero_bytes(v[r][3]);
      }
    } else {
      for (int r = 0; r < 8; ++r) {
        if (row0 + r >= a.M) break;
        const uint8_t* rp = eb + (long long)(row0 + r) * a.N;
        for (int j = 0; j < 16; ++j)
          if (col + j < a.N && rp[col + j]) (j < 8 ? lo : hi) += 1;
      }
    }
    kept |= lo | hi;
    const int gj = col >> 3;
    if (micro_row < a.m8) {
      uint8_t* tp = a.thread_mask + ((long long)b * a.m8 + micro_row) * a.n8 + gj;
      if (a.pairs && gj + 1 < a.n8) {
        // two counts as one 16-bit store: lanes along a row write contiguously
        typedef unsigned short __attribute__((address_space(1))) * g2p;
        *(g2p)tp = static_cast<unsigned short>(lo | (hi << 8));
      } else {
        if (gj < a.n8) tp[0] = static_cast<uint8_t>(lo);
        if (gj + 1 < a.n8) tp[1] = static_cast<uint8_t>(hi);
      }
    }
  }
  // lanes 8j .. 8j+7 of a row belong to block tile j of the span
  if (kept) kept_blocks[(lane % LPR) >> 3] = 1;  // every writer stores the same value
  __syncthreads();
  if (threadIdx.x < kBlocks) {
    const int tile_n = span * kBlocks + threadIdx.x;
    if (tile_n < a.tiles_n)
      a.block_mask[((long long)b * a.tiles_m + tile_m) * a.tiles_n + tile_n] = kept_blocks[threadIdx.x] ? 1 : 0;
  }
}

}  // namespace cmk

using namespace cmk;

extern "C" int cmk_derive_masks_u8(const uint8_t* element_mask, uint8_t* block_mask,
                                   uint8_t* thread_mask, int Lm, int M, int N, void* stream) {
  if (Lm < 0 || M < 0 || N < 0)
    return fail(CMK_ERR_INVALID_ARG, "cmk_derive_masks_u8: negative extent (Lm=%d M=%d N=%d)", Lm, M, N);
  if (Lm == 0 || M == 0 || N == 0) return CMK_OK;
  if (!element_mask || !block_mask || !thread_mask)
    return fail(CMK_ERR_INVALID_ARG, "cmk_derive_masks_u8: null pointer");
  MaskArgs a{};
  a.element_mask = element_mask;
  a.block_mask = block_mask;
  a.thread_mask = thread_mask;
  a.Lm = Lm; a.M = M; a.N = N;
  a.tiles_m = ceil_div(M, 128);
  a.tiles_n = ceil_div(N, 128);
  a.m8 = ceil_div(M, 8);
  a.n8 = ceil_div(N, 8);
  a.aligned = ((reinterpret_cast<uintptr_t>(element_mask) & 15) == 0 && (N & 15) == 0) ? 1 : 0;
  a.pairs = ((reinterpret_cast<uintptr_t>(thread_mask) & 1) == 0 && (a.n8 & 1) == 0) ? 1 : 0;
  // widest span that the row length fills: 1024, 512 or 256 columns per work-group
  const int lpr = N > 512 ? 64 : (N > 256 ? 32 : 16);
  a.spans_n = ceil_div(N, lpr * 16);
  const long long groups = (long long)Lm * a.tiles_m * a.spans_n;
  if (int e = check_grid(groups)) return e;
  const dim3 grid((unsigned)groups), block(kMaskThreads);
  hipStream_t st = (hipStream_t)stream;
  if (lpr == 64) hipLaunchKernelGGL(derive_masks_kernel<64>, grid, block, 0, st, a);
  else if (lpr == 32) hipLaunchKernelGGL(derive_masks_kernel<32>, grid, block, 0, st, a);
  else hipLaunchKernelGGL(derive_masks_kernel<16>, grid, block, 0, st, a);
  return hip_status(hipGetLastError(), "cmk_derive_masks_u8 launch");
}
