// bmm / mbmm: dense and masked batched product with a store epilogue.
//
// X = the m side (rows of C, inside a lane), Y = the n side (columns of C,
// across lanes): a store of one accumulator register writes two 128-byte row
// segments of C.  One work-group = one 128x128 tile of C, which is also the
// granularity of the block mask (reference kernels/mbmm.cu:247-255).
#include "cmk_core.hpp"
#include "cmk_launch.hpp"

namespace cmk {

struct BmmArgs {
  const float* A;
  const float* B;
  float* C;
  const uint8_t* block_mask;
  const uint8_t* thread_mask;
  const uint8_t* element_mask;
  long long lda, ldb, strideA, strideB;
  int L, M, N, K;
  int tiles_m, tiles_n;
  int run;           // consecutive tiles along m per work-group
  int mask_batched;  // 1: masks have a leading batch axis, 0: shared by all batches
  int vecA, vecB;
  // contraction cut into `ksplits` ranges of `klen` (a multiple of the slab depth):
  // the launch then has L * ksplits "batches", batch b * ksplits + j holds the
  // partial product of range j of batch b, and C is the workspace of partials
  int ksplits, klen;
};

constexpr int kMaskRows = 128;    // element-mask tile staged in LDS: rows ...
constexpr int kMaskPitch = 144;   // ... of 128 bytes, 16-byte aligned, skewed over the banks

// B = 32x32 blocks per wave and axis: 2 gives the 128x128 tile, 1 a 64x64 tile
// for products with too few 128x128 tiles to occupy the chip (dense only).
template <int XK, int YK, bool MASKED, int B = 2>
__global__ __launch_bounds__(kThreads, 2) void bmm_kernel(BmmArgs a) {
  // In the masked product a lane's two accumulators of one row are neighbouring
  // columns (Y_PAIRS): C leaves as 8-byte stores, the two element-mask bytes come
  // with one LDS read and share a thread-mask byte (3 % faster on the masked
  // shapes; the dense product measured 3 % slower with it and keeps its columns
  // 32 apart).
  constexpr bool PAIRS = B == 2 && MASKED;
  using C = Core<XK, YK, 2, 2, B, B, 32, kReadsPaired, false, false, true, PAIRS>;
  // column of block `by` of this lane within the wave's columns
  auto col_of = [](int by, int l32) { return PAIRS ? 2 * l32 + by : by * 32 + l32; };
  static_assert(B == 2 || !MASKED, "the masks are laid out for 128x128 tiles");
  __shared__ __attribute__((aligned(16))) float lds[C::ldsFloats];

  // A work-group owns `run` consecutive tiles along m of one 128-wide column
  // strip; the slab pipeline runs across them, so the stores of one tile
  // overlap the loads of the next.  Masked products use run == 1 because
  // skipped tiles break the sequence.
  const int mgroups = (a.tiles_m + a.run - 1) / a.run;
  const int per_batch = mgroups * a.tiles_n;
  const int logical = xcd_logical_id(blockIdx.x, a.L * per_batch);
  if (logical < 0) return;
  const int b = logical / per_batch;
  const int t = logical - b * per_batch;
  // column strips of one row group are neighbours, so that concurrently
  // running work-groups share their panels of A in L2
  const int mg = t / a.tiles_n;
  const int tile_n = t - mg * a.tiles_n;
  const int tile_m0 = mg * a.run;
  const int ntiles = min(a.run, a.tiles_m - tile_m0);
  const int n0 = tile_n * C::TY;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int l32 = lane & 31;
  const int half = lane >> 5;
  float* Cb = a.C + (long long)b * a.M * a.N;

  long long mb = 0;  // batch index into the masks
  if constexpr (MASKED) {
    mb = a.mask_batched ? b : 0;
    // The work-group's first dependent step.  The byte is the same for all lanes:
    // it comes through the scalar cache as the aligned word around it (a third of
    // the latency of a vector byte load), unless that word reaches past the array.
    const long long bi = (mb * a.tiles_m + tile_m0) * a.tiles_n + tile_n;
    const long long bytes = (long long)(a.mask_batched ? a.L : 1) * a.tiles_m * a.tiles_n;
    const uintptr_t at = reinterpret_cast<uintptr_t>(a.block_mask) + bi;
    uint8_t bm;
    if ((reinterpret_cast<uintptr_t>(a.block_mask) & 3) == 0 && (bi | 3) < bytes) {
      typedef const uint32_t __attribute__((address_space(4))) * c32p;
      const uint32_t word = *(c32p)(at & ~static_cast<uintptr_t>(3));
      bm = static_cast<uint8_t>(word >> (8 * (at & 3)));
    } else {
      bm = a.block_mask[bi];
    }
    if (bm == 0) {
      // skipped tile: nothing is loaded or multiplied, zeros are written
      const int m0 = tile_m0 * C::TX;
      for (int e = threadIdx.x; e < 128 * 32; e += kThreads) {
        const int r = m0 + (e >> 5);
        const int c = n0 + (e & 31) * 4;
        if (r < a.M) {
          float* dst = Cb + (long long)r * a.N + c;
          if ((a.N & 3) == 0 && c + 3 < a.N) {
            // non-temporal: the zeros must not displace what kept tiles read (measured:
            // 133 instead of 165 us at the benchmark shape)
            __builtin_nontemporal_store(f32x4{0.f, 0.f, 0.f, 0.f}, reinterpret_cast<f32x4*>(dst));
          } else {
            for (int j = 0; j < 4; ++j)
              if (c + j < a.N) dst[j] = 0.f;
          }
        }
      }
      return;
    }
  }

  Operand X{uniform_ptr(a.A + (long long)b * a.strideA), a.lda, a.M, a.vecA};
  Operand Y{uniform_ptr(a.B + (long long)b * a.strideB), a.ldb, a.N, a.vecB};
  int K = a.K;
  if constexpr (!MASKED) {
    if (a.ksplits > 1) {
      const int bb = b / a.ksplits;
      const int k0 = (b - bb * a.ksplits) * a.klen;
      K = min(a.klen, a.K - k0);
      X.p = uniform_ptr(a.A + (long long)bb * a.strideA + (XK == KC ? (long long)k0 : (long long)k0 * a.lda));
      Y.p = uniform_ptr(a.B + (long long)bb * a.strideB + (YK == KC ? (long long)k0 : (long long)k0 * a.ldb));
    }
  }

  C core;
  core.begin(X, Y, tile_m0 * C::TX, n0, K, ntiles, lds);
  for (int ti = 0; ti < ntiles; ++ti) {
    // the dense product starts its accumulators from a literal zero; for the
    // masked one that form measured slower (191 vs 165 us at the benchmark shape)
    f32x16 acc[B][B];
    if constexpr (MASKED) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    }
    // A kept tile whose masks can be fetched with 16-byte loads gets them staged
    // in LDS: 128 rows of 128 element-mask bytes, then the tile's 16x16
    // thread-mask bytes.  They are requested before the product starts, so that
    // they arrive while it runs, and go to LDS once the operand buffers are free.
    bool staged = false;
    f32x4 mask_regs[4];
    uint8_t tmask_reg = 0;
    if constexpr (MASKED) {
      const int m0 = (tile_m0 + ti) * C::TX;
      staged = m0 + 128 <= a.M && n0 + 128 <= a.N && (a.N & 15) == 0 &&
               (reinterpret_cast<uintptr_t>(a.element_mask) & 15) == 0;
      if (staged) {
        typedef const f32x4 __attribute__((address_space(1))) * g16p;
        typedef const uint8_t __attribute__((address_space(1))) * g1p;
        const uint8_t* eb = a.element_mask + (mb * a.M + m0) * a.N + n0;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const int idx = threadIdx.x + kThreads * p;
          const int row = idx >> 3, c16 = (idx & 7) * 16;
          mask_regs[p] = *(g16p)(eb + (long long)row * a.N + c16);
        }
        const int tn8 = (a.N + 7) >> 3;
        const int tm8 = (a.M + 7) >> 3;
        tmask_reg = *(g1p)(a.thread_mask + (mb * tm8 + (m0 >> 3) + (threadIdx.x >> 4)) * tn8 + (n0 >> 3) +
                           (threadIdx.x & 15));
      }
    }
    core.template tile<kInner, !MASKED>(X, Y, lds, acc);

    if constexpr (MASKED) {
      if (staged) {
        core.wait_loads();
        __syncthreads();  // nobody reads operand fragments any more
        uint8_t* ml = reinterpret_cast<uint8_t*>(lds);
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const int idx = threadIdx.x + kThreads * p;
          const int row = idx >> 3, c16 = (idx & 7) * 16;
          *reinterpret_cast<f32x4*>(ml + row * kMaskPitch + c16) = mask_regs[p];
        }
        ml[kMaskRows * kMaskPitch + threadIdx.x] = tmask_reg;
        __syncthreads();
      }
    }

    // store: one accumulator register covers two 128-byte row segments of C.
    // C is written once and not read again here: non-temporal stores keep it from
    // displacing the operands in L2 (measured: 4 % on the dense product)
    const int wv = __builtin_amdgcn_readfirstlane(wave);
    const int mw = (tile_m0 + ti) * C::TX + (wv % 2) * 32 * B;
    const int nw = n0 + (wv / 2) * 32 * B;
    if (mw + 32 * B <= a.M && nw + 32 * B <= a.N && (long long)a.N * 68 * 4 < (1ll << 31)) {
      // interior: row addresses are scalar, the lane part is one 32-bit offset
      typedef float __attribute__((address_space(1))) * gfp;
      typedef const uint8_t __attribute__((address_space(1))) * gbp;
      typedef f32x2 __attribute__((address_space(1))) * gf2p;
      char* base = reinterpret_cast<char*>(uniform_ptr(Cb + (long long)mw * a.N + nw));
      const unsigned voff = static_cast<unsigned>((4 * half * a.N + col_of(0, l32)) * 4);
      constexpr int kByStep = PAIRS ? 4 : 128;   // bytes from block by = 0 to by = 1
      // both accumulators of a row in one store: rows of C must stay 8-byte aligned
      const bool pair_store = PAIRS && (a.N & 1) == 0 && (reinterpret_cast<uintptr_t>(Cb) & 7) == 0;
      auto put = [&](char* rp, float v0, float v1) {
        if (pair_store) {
          __builtin_nontemporal_store(f32x2{v0, v1}, (gf2p)(rp + voff));
        } else {
          __builtin_nontemporal_store(v0, (gfp)(rp + voff));
          __builtin_nontemporal_store(v1, (gfp)(rp + voff + kByStep));
        }
      };
      if constexpr (!MASKED) {
#pragma unroll
        for (int bx = 0; bx < B; ++bx)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            char* rp = base + (long long)(bx * 32 + 8 * (r >> 2) + (r & 3)) * a.N * 4;
            if constexpr (B == 2) {
              put(rp, acc[bx][0][r], acc[bx][1][r]);
            } else {
              __builtin_nontemporal_store(acc[bx][0][r], (gfp)(rp + voff));
            }
          }
      } else if (staged) {
        // masks come from LDS: byte reads there cost no vector-memory instructions
        const uint8_t* ml = reinterpret_cast<const uint8_t*>(lds);
        const int mwl = (wv % 2) * 64, nwl = (wv / 2) * 64;
        // (the lane's two columns 2 * l32 and 2 * l32 + 1 share a micro-tile and are
        // two neighbouring element-mask bytes)
        const uint8_t* tl = ml + kMaskRows * kMaskPitch + (mwl >> 3) * 16 + (nwl >> 3) + (l32 >> 2);
        const uint8_t* el = ml + (mwl + 4 * half) * kMaskPitch + nwl + 2 * l32;
#pragma unroll
        for (int bx = 0; bx < 2; ++bx)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint8_t tmk = tl[(bx * 4 + q) * 16];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int r = 4 * q + e;
              const int rowc = bx * 32 + 8 * q + e;
              char* rp = base + (long long)rowc * a.N * 4;
              const unsigned em2 = *reinterpret_cast<const uint16_t*>(el + rowc * kMaskPitch);
              put(rp, tmk ? acc[bx][0][r] * (float)(em2 & 0xffu) : 0.f, tmk ? acc[bx][1][r] * (float)(em2 >> 8) : 0.f);
            }
          }
      } else {
        const int tn8 = (a.N + 7) >> 3;
        const int tm8 = (a.M + 7) >> 3;
        const uint8_t* eb = uniform_ptr(a.element_mask + (mb * a.M + mw) * a.N + nw);
        const uint8_t* tb = uniform_ptr(a.thread_mask + (mb * tm8 + (mw >> 3)) * tn8 + (nw >> 3));
        const unsigned eoff = static_cast<unsigned>(4 * half * a.N + 2 * l32);
        const unsigned toff = static_cast<unsigned>(l32 >> 2);
#pragma unroll
        for (int bx = 0; bx < 2; ++bx)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint8_t tmk = *(gbp)(tb + (long long)(bx * 4 + q) * tn8 + toff);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int r = 4 * q + e;
              const long long rowc = bx * 32 + 8 * q + e;
              char* rp = base + rowc * a.N * 4;
              const uint8_t* ep = eb + rowc * a.N;
              const uint8_t em0 = *(gbp)(ep + eoff), em1 = *(gbp)(ep + eoff + 1);
              put(rp, tmk ? acc[bx][0][r] * (float)em0 : 0.f, tmk ? acc[bx][1][r] * (float)em1 : 0.f);
            }
          }
      }
    } else {
#pragma unroll
      for (int bx = 0; bx < B; ++bx) {
#pragma unroll
        for (int by = 0; by < B; ++by) {
          const int n = nw + col_of(by, l32);
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = mw + bx * 32 + acc_row(r, half);
            if (m < a.M && n < a.N) {
              float v = acc[bx][by][r];
              if constexpr (MASKED) {
                const int tn8 = (a.N + 7) >> 3;
                const int tm8 = (a.M + 7) >> 3;
                const uint8_t tm = a.thread_mask[(mb * tm8 + (m >> 3)) * tn8 + (n >> 3)];
                const uint8_t em = a.element_mask[(mb * a.M + m) * a.N + n];
                v = tm ? v * (float)em : 0.f;
              }
              Cb[(long long)m * a.N + n] = v;
            }
          }
        }
      }
    }
  }
}

template <bool MASKED, int B = 2>
static hipError_t launch_bmm(const BmmArgs& a, int transA, int transB, hipStream_t st) {
  const int total = a.L * ((a.tiles_m + a.run - 1) / a.run) * a.tiles_n;
  const dim3 grid(((total + 7) / 8) * 8), block(kThreads);
  // A "n" is k-contiguous (KC), A "t" is m-contiguous (RC);
  // B "n" is n-contiguous (RC), B "t" is k-contiguous (KC).
  if (!transA && !transB) hipLaunchKernelGGL((bmm_kernel<KC, RC, MASKED, B>), grid, block, 0, st, a);
  else if (!transA && transB) hipLaunchKernelGGL((bmm_kernel<KC, KC, MASKED, B>), grid, block, 0, st, a);
  else if (transA && !transB) hipLaunchKernelGGL((bmm_kernel<RC, RC, MASKED, B>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((bmm_kernel<RC, KC, MASKED, B>), grid, block, 0, st, a);
  return hipGetLastError();
}

static BmmArgs make_args(const float* A, const float* B, float* C, const cmk_gemm_desc* d, int tile = 128) {
  BmmArgs a{};
  a.A = A; a.B = B; a.C = C;
  a.lda = d->lda; a.ldb = d->ldb; a.strideA = d->strideA; a.strideB = d->strideB;
  a.L = d->L; a.M = d->M; a.N = d->N; a.K = d->K;
  a.tiles_m = (d->M + tile - 1) / tile;
  a.tiles_n = (d->N + tile - 1) / tile;
  a.run = 1;
  a.vecA = vec_ok(A, d->lda, d->strideA);
  a.vecB = vec_ok(B, d->ldb, d->strideB);
  return a;
}

// Long contractions with few tiles: how many ranges the contraction is cut into
// so that the chip has work (each range at least four slabs), and their length.
static int plan_bmm_ksplits(int L, int M, int N, int K, int* klen) {
  const long long tiles = (long long)L * ((M + 63) / 64) * ((N + 63) / 64);
  const int slabs = (K + 31) / 32;
  *klen = K;
  if (tiles == 0 || slabs < 8) return 1;
  // Up to half a chip of tiles: one 64x64 work-group per CU (more ranges measured
  // slower: the sum reads every partial once more; fewer leave CUs idle).  Up to
  // a whole chip: four ranges, so that every SIMD has waves to switch between,
  // once the contraction is long enough to pay for the second kernel (measured:
  // from about 48 slabs).
  const long long cus = compute_units();
  long long want;
  if (tiles * 2 > cus) want = (tiles <= cus && slabs >= 48) ? 4 : 1;
  else want = (cus + tiles - 1) / tiles;
  if (want > slabs / 4) want = slabs / 4;
  if (want > 64) want = 64;
  if (want < 2) return 1;
  const int per = (slabs + (int)want - 1) / (int)want;
  *klen = per * 32;
  return (slabs + per - 1) / per;
}

size_t bmm_workspace_bytes(int L, int M, int N, int K) {
  int klen;
  const int s = plan_bmm_ksplits(L, M, N, K, &klen);
  return s > 1 ? (size_t)s * L * M * N * sizeof(float) : 0;
}

// C[b][e] = sum over j, in ascending j, of part[b * s + j][e]; `mn` elements per
// matrix.  V = 4 when everything can move as 16-byte vectors.
template <int V>
__global__ __launch_bounds__(256) void bmm_sum_kernel(const float* __restrict__ part, float* __restrict__ C,
                                                      long long mn, long long total, int s) {
  typedef float vec_t __attribute__((ext_vector_type(V)));
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i * V < total; i += stride) {
    const long long o = i * V;
    const long long b = o / mn, e = o - b * mn;
    const float* p = part + (b * s) * mn + e;
    vec_t acc = *reinterpret_cast<const vec_t*>(p);
    for (int j = 1; j < s; ++j) acc += *reinterpret_cast<const vec_t*>(p + j * mn);
    *reinterpret_cast<vec_t*>(C + o) = acc;
  }
}

}  // namespace cmk

using namespace cmk;

extern "C" int cmk_bmm_ws_f32(const float* A, const float* B, float* C, const cmk_gemm_desc* d,
                              void* workspace, size_t workspace_bytes, void* stream) {
  if (int e = check_desc(d)) return e;
  if (d->L == 0 || d->M == 0 || d->N == 0) return CMK_OK;
  int klen;
  const int s = plan_bmm_ksplits(d->L, d->M, d->N, d->K, &klen);
  if (s <= 1) return cmk_bmm_f32(A, B, C, d, stream);
  if (!C || !A || !B) return fail(CMK_ERR_INVALID_ARG, "cmk_bmm_ws_f32: null pointer");
  const size_t need = (size_t)s * d->L * d->M * d->N * sizeof(float);
  if (!workspace || workspace_bytes < need)
    return fail(CMK_ERR_WORKSPACE, "cmk_bmm_ws_f32: workspace of %zu bytes required, %zu given", need,
                workspace_bytes);
  BmmArgs a = make_args(A, B, static_cast<float*>(workspace), d, 64);
  a.ksplits = s;
  a.klen = klen;
  a.L = d->L * s;
  if (int e = check_grid((long long)a.L * a.tiles_m * a.tiles_n)) return e;
  hipStream_t st = (hipStream_t)stream;
  if (int e = hip_status(launch_bmm<false, 1>(a, d->transA, d->transB, st), "cmk_bmm_ws_f32 launch")) return e;
  const long long mn = (long long)d->M * d->N, total = mn * d->L;
  const bool vec = (mn & 3) == 0 && ((reinterpret_cast<uintptr_t>(workspace) | reinterpret_cast<uintptr_t>(C)) & 15) == 0;
  const long long items = vec ? total / 4 : total;
  long long blocks = (items + 255) / 256;
  if (blocks > 8ll * compute_units()) blocks = 8ll * compute_units();
  if (vec) hipLaunchKernelGGL(bmm_sum_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, st,
                              static_cast<const float*>(workspace), C, mn, total, s);
  else hipLaunchKernelGGL(bmm_sum_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, st,
                          static_cast<const float*>(workspace), C, mn, total, s);
  return hip_status(hipGetLastError(), "cmk_bmm_ws_f32 sum launch");
}

extern "C" int cmk_bmm_f32(const float* A, const float* B, float* C, const cmk_gemm_desc* d,
                           void* stream) {
  if (int e = check_desc(d)) return e;
  if (d->L == 0 || d->M == 0 || d->N == 0) return CMK_OK;
  if (!C || (d->K > 0 && (!A || !B))) return fail(CMK_ERR_INVALID_ARG, "cmk_bmm_f32: null pointer");
  if (int e = check_grid((long long)d->L * ((d->M + 127) / 128) * ((d->N + 127) / 128))) return e;
  BmmArgs a = make_args(A, B, C, d);
  const long long tiles = (long long)d->L * a.tiles_m * a.tiles_n;
  if (tiles < 3 * compute_units()) {
    // too few 128x128 tiles for two even rounds of the chip (measured: up to ~600
    // tiles the smaller tile wins, at 1024 the larger): 64x64 tiles, four times as many
    a = make_args(A, B, C, d, 64);
    return hip_status(launch_bmm<false, 1>(a, d->transA, d->transB, (hipStream_t)stream),
                      "cmk_bmm_f32 launch");
  }
  // longer runs amortise the pipeline fill; keep at least ~4 work-groups per CU
  a.run = tiles >= 8192 ? 4 : (tiles >= 4096 ? 2 : 1);
  return hip_status(launch_bmm<false>(a, d->transA, d->transB, (hipStream_t)stream),
                    "cmk_bmm_f32 launch");
}

extern "C" int cmk_mbmm_f32(const float* A, const float* B, float* C, const uint8_t* block_mask,
                            const uint8_t* thread_mask, const uint8_t* element_mask,
                            int share_mask, const cmk_gemm_desc* d, void* stream) {
  if (int e = check_desc(d)) return e;
  if (d->L == 0 || d->M == 0 || d->N == 0) return CMK_OK;
  if (!C || (d->K > 0 && (!A || !B)) || !block_mask || !thread_mask || !element_mask)
    return fail(CMK_ERR_INVALID_ARG, "cmk_mbmm_f32: null pointer");
  if (int e = check_grid((long long)d->L * ((d->M + 127) / 128) * ((d->N + 127) / 128))) return e;
  BmmArgs a = make_args(A, B, C, d);
  a.block_mask = block_mask;
  a.thread_mask = thread_mask;
  a.element_mask = element_mask;
  a.mask_batched = share_mask ? 0 : 1;
  return hip_status(launch_bmm<true>(a, d->transA, d->transB, (hipStream_t)stream), "cmk_mbmm_f32 launch");
}
