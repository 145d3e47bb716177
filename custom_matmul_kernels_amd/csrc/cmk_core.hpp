// Shared fp32-MFMA tiled GEMM core for gfx950 (CDNA4, wave64).
//
// One 256-thread work-group (4 waves) computes a TX x TY macro tile of the
// product of two operands that both have a contraction axis k:
//   X : TX "rows"  -> MFMA source A, the axis that ends up INSIDE a lane
//   Y : TY "rows"  -> MFMA source B, the axis that ends up ACROSS lanes
// Which matrix of the user's problem plays X and which plays Y is chosen by
// each kernel so that its epilogue is cheap: a reduction wants the reduced
// axis in X (running state stays in one lane), a row-major store wants the
// contiguous axis in Y (a store instruction writes 128-byte row segments).
//
// The contraction is walked in slabs of KS (32 unless a kernel asks otherwise).  A slab of each operand is
// fetched from global memory into registers, written to one of two LDS
// buffers, and consumed from the other with v_mfma_f32_32x32x2_f32.  Inside a
// slab, k is consumed in groups of 8: lanes 0-31 feed k = 8g+0..3 and lanes
// 32-63 feed k = 8g+4..7 of both operands, so one 128-bit LDS read per 32x32
// block supplies four MFMA steps.  (A sum over k does not care about the
// order, as long as both operands use the same one.)
//
// An operand tile can sit in memory, and in LDS, in one of two ways:
//   KC : element(row, k) at row*ld + k   (k contiguous)  -> LDS [row][KS+4]
//   RC : element(row, k) at k*ld + row   (rows contiguous) -> LDS [k][T+8]
// Both are written with 128-bit stores straight from 128-bit global loads;
// no transposition is needed on the way in.
//
// Plays the role of load_ab_*, buffer2smem_* and thread_matmul_* of the
// reference (kernels/bmm_helpers.cu:114-164, 240-622).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cmk {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Operands live in global memory; loading through pointers that say so gives
// global_load instructions (a generic pointer would give flat loads, which
// also count against the LDS wait counter).
typedef const f32x4 __attribute__((address_space(1))) * global_f32x4_ptr;
typedef const float __attribute__((address_space(1))) * global_f32_ptr;

constexpr int kThreads = 256;
constexpr int KC = 0;   // k-contiguous operand
constexpr int RC = 1;   // row-contiguous operand

struct Operand {
  const float* p;  // base of this batch's matrix
  long long ld;    // KC: distance between rows; RC: distance between k
  int rows;        // extent of the non-contracted axis
  int vec;         // non-zero when 16-byte loads are legal (base and ld aligned)
};

// Marks a pointer that is the same for every lane of the wave as such, so that
// address arithmetic on it stays on the scalar unit.
template <class P>
__device__ __forceinline__ P* uniform_ptr(P* p) {
  const unsigned long long v = reinterpret_cast<unsigned long long>(p);
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v >> 32));
  return reinterpret_cast<P*>((static_cast<unsigned long long>(hi) << 32) | lo);
}

// LDS footprint of one slab (KS deep) of a T-row operand tile.
template <int KIND, int T, int KS>
struct TileLayout;
template <int T, int KS>
struct TileLayout<KC, T, KS> {
  static constexpr int pitch = KS + 4;
  static constexpr int floats = T * pitch;
};
template <int T, int KS>
struct TileLayout<RC, T, KS> {
  static constexpr int pitch = T + 8;
  static constexpr int floats = KS * pitch;
};

// ---- global -> registers ---------------------------------------------------
// Each of the NT threads fetches NV = T*KS/(4*NT) groups of four consecutive floats.  For
// both kinds the element a thread fetches in pass p sits at
//     tile + (t / TPR + p * RPP) * ld + (t % TPR) * 4
// (KC: row-major rows x k, RC: k-major k x rows), so the per-lane part
// `lane_off` is fixed for a whole kernel and everything else is scalar.
template <int KIND, int T, int KS, int NT>
struct LoadMap {
  static constexpr int NV = T * KS / (NT * 4);             // float4 per thread
  static constexpr int TPR = KIND == KC ? KS / 4 : T / 4;  // threads per contiguous run
  static constexpr int RPP = NT / TPR;                     // runs per pass
  static_assert(NV >= 1 && NV * NT * 4 == T * KS, "tile does not divide among the threads");
};

template <int KIND, int T, int KS, int NT>
__device__ __forceinline__ void lane_offsets_bytes(const Operand& o,
                                                   unsigned (&off)[T * KS / (NT * 4)]) {
  using M = LoadMap<KIND, T, KS, NT>;
  const int t = threadIdx.x;
#pragma unroll
  for (int p = 0; p < M::NV; ++p)
    off[p] = static_cast<unsigned>(((long long)(t / M::TPR + p * M::RPP) * o.ld + (t % M::TPR) * 4) * 4);
}

// r0, k0, K are wave-uniform.  A tile that lies completely inside the matrix
// takes the branch-free path.
template <int KIND, int T, int KS, int NT>
__device__ __forceinline__ void gload(const Operand& o,
                                      const unsigned (&lane_off)[T * KS / (NT * 4)], int r0, int k0,
                                      int K, f32x4 (&v)[T * KS / (NT * 4)]) {
  using M = LoadMap<KIND, T, KS, NT>;
  constexpr int NV = M::NV, TPR = M::TPR, RPP = M::RPP;
  const int t = threadIdx.x;
  const bool interior = o.vec && (k0 + KS <= K) && (r0 + T <= o.rows) &&
                        ((long long)(T + KS) * o.ld < (1ll << 29));
  if (interior) {
    const long long first = KIND == KC ? (long long)r0 * o.ld + k0 : (long long)k0 * o.ld + r0;
    const char* tile = reinterpret_cast<const char*>(o.p + first);
#pragma unroll
    for (int p = 0; p < NV; ++p) v[p] = *(global_f32x4_ptr)(tile + lane_off[p]);
  } else if (K > 0 && o.rows > 0) {
    // edge tile: every element is fetched from a clamped (always valid)
    // address and zeroed when it lies outside the matrix; no divergent branches
    if constexpr (KIND == KC) {
      const int kk = k0 + (t % TPR) * 4;
      const int rr = r0 + t / TPR;
#pragma unroll
      for (int p = 0; p < NV; ++p) {
        const int row = rr + RPP * p;
        const float* src = o.p + (long long)row * o.ld + kk;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[p][j] = *(global_f32_ptr)((row < o.rows && kk + j < K) ? src + j : o.p);
      }
#pragma unroll
      for (int p = 0; p < NV; ++p) {
        const int row = rr + RPP * p;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[p][j] = (row < o.rows && kk + j < K) ? v[p][j] : 0.f;
      }
    } else {
      const int rr = r0 + (t % TPR) * 4;
      const int kb = k0 + t / TPR;
#pragma unroll
      for (int p = 0; p < NV; ++p) {
        const int kk = kb + p * RPP;
        const float* src = o.p + (long long)kk * o.ld + rr;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[p][j] = *(global_f32_ptr)((kk < K && rr + j < o.rows) ? src + j : o.p);
      }
#pragma unroll
      for (int p = 0; p < NV; ++p) {
        const int kk = kb + p * RPP;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[p][j] = (kk < K && rr + j < o.rows) ? v[p][j] : 0.f;
      }
    }
  } else {
#pragma unroll
    for (int p = 0; p < NV; ++p) v[p] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
}

// ---- registers -> LDS --------------------------------------------------------
template <int KIND, int T, int KS, int NT>
__device__ __forceinline__ void lstore(float* lds, const f32x4 (&v)[T * KS / (NT * 4)]) {
  using M = LoadMap<KIND, T, KS, NT>;
  const int t = threadIdx.x;
  constexpr int pitch = TileLayout<KIND, T, KS>::pitch;
#pragma unroll
  for (int p = 0; p < M::NV; ++p)
    *reinterpret_cast<f32x4*>(&lds[(t / M::TPR + p * M::RPP) * pitch + (t % M::TPR) * 4]) = v[p];
}

// ---- LDS -> MFMA fragment ----------------------------------------------------
// Four k values (8*kg + 4*half + 0..3) of tile row `row` for this lane.
template <int KIND, int T, int KS>
__device__ __forceinline__ f32x4 frag(const float* lds, int row, int kg, int half) {
  constexpr int pitch = TileLayout<KIND, T, KS>::pitch;
  if constexpr (KIND == KC) {
    return *reinterpret_cast<const f32x4*>(&lds[row * pitch + kg * 8 + half * 4]);
  } else {
    const float* q = &lds[(kg * 8 + half * 4) * pitch + row];
    f32x4 r;
    r.x = q[0];
    r.y = q[pitch];
    r.z = q[2 * pitch];
    r.w = q[3 * pitch];
    return r;
  }
}

// Work-group level tile engine.  WX x WY waves (4 or 8 of them), each wave owns
// BX x BY blocks of 32x32; KS is the contraction depth of one LDS slab.
//
// The engine walks a flat sequence of slabs: `ntiles` consecutive X tiles
// (starting at element `xbase`) against one Y strip, S = ceil(K/KS) slabs per
// tile.  While slab i is multiplied, slab i+1 is written to the other LDS
// buffer (in the middle of the slab) and slab i+2 is on its way from global
// memory.  The one barrier per slab sits inside the last k-group; right after
// it the first fragments of slab i+1 are read, so the matrix pipe keeps running
// across slab and tile boundaries.  Inside a k-group all LDS and global traffic
// is issued directly behind the group's first MFMA step, where it costs no
// matrix-pipe time.
template <int XK, int YK, int WX, int WY, int BX, int BY, int KS_ = 32>
struct Core {
  static_assert(WX * WY == 4 || WX * WY == 8, "four or eight waves per work-group");
  static constexpr int NT = WX * WY * 64;      // threads per work-group
  static constexpr int KS = KS_;
  static constexpr int NG = KS / 8;            // k-groups per slab
  static constexpr int WRITE_AT = NG / 2 - 1;  // k-group after which the next slab goes to LDS
  static constexpr int TX = WX * BX * 32;
  static constexpr int TY = WY * BY * 32;
  static_assert(NG >= 2 && NG % 2 == 0, "slab depth");
  static constexpr int xFloats = TileLayout<XK, TX, KS>::floats;
  static constexpr int yFloats = TileLayout<YK, TY, KS>::floats;
  static constexpr int bufFloats = xFloats + yFloats;
  static constexpr int ldsFloats = 2 * bufFloats;

  f32x4 xv[TX * KS / (NT * 4)];  // slab in flight from global memory
  f32x4 yv[TY * KS / (NT * 4)];
  f32x4 xf[2][BX];           // fragments; [0] holds k-group 0 of the current slab at slab entry
  f32x4 yf[2][BY];
  int it, iters, S;          // flat slab counter (wave-uniform)
  int lt, ls;                // (tile, slab) of the next slab to fetch (wave-uniform)
  int xbase, y0, K;
  int xr, yr, half;
  unsigned xoff[TX * KS / (NT * 4)];  // this lane's byte offsets inside an operand tile
  unsigned yoff[TY * KS / (NT * 4)];

  __device__ __forceinline__ void load(const Operand& X, const Operand& Y) {
    // the slab coordinates are the same for every lane; saying so keeps the
    // address arithmetic on the scalar unit
    const int x0 = __builtin_amdgcn_readfirstlane(xbase + lt * TX);
    const int k0 = __builtin_amdgcn_readfirstlane(ls * KS);
    gload<XK, TX, KS, NT>(X, xoff, x0, k0, K, xv);
    gload<YK, TY, KS, NT>(Y, yoff, y0, k0, K, yv);
    if (++ls == S) { ls = 0; ++lt; }
  }
  __device__ __forceinline__ void store(float* buf) {
    lstore<XK, TX, KS, NT>(buf, xv);
    lstore<YK, TY, KS, NT>(buf + xFloats, yv);
  }
  __device__ __forceinline__ void read_frags(const float* buf, int kg, f32x4 (&fx)[BX],
                                             f32x4 (&fy)[BY]) {
#pragma unroll
    for (int b = 0; b < BX; ++b) fx[b] = frag<XK, TX, KS>(buf, xr + 32 * b, kg, half);
#pragma unroll
    for (int b = 0; b < BY; ++b) fy[b] = frag<YK, TY, KS>(buf + xFloats, yr + 32 * b, kg, half);
  }

  // Fills the pipeline: slab 0 in LDS with its first fragments in registers,
  // slab 1 in flight.  Ends with every wave past a barrier.
  __device__ __forceinline__ void begin(const Operand& X, const Operand& Y, int xbase_, int y0_,
                                        int K_, int ntiles, float* lds) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    half = lane >> 5;
    xr = (wave % WX) * BX * 32 + (lane & 31);
    yr = (wave / WX) * BY * 32 + (lane & 31);
    xbase = __builtin_amdgcn_readfirstlane(xbase_);
    y0 = __builtin_amdgcn_readfirstlane(y0_);
    K = __builtin_amdgcn_readfirstlane(K_);
    S = max(1, (K + KS - 1) / KS);
    iters = __builtin_amdgcn_readfirstlane(ntiles) * S;
    lane_offsets_bytes<XK, TX, KS, NT>(X, xoff);
    lane_offsets_bytes<YK, TY, KS, NT>(Y, yoff);
    it = 0;
    lt = 0;
    ls = 0;
    load(X, Y);
    store(lds);
    __syncthreads();
    read_frags(lds, 0, xf[0], yf[0]);
    if (iters > 1) load(X, Y);
  }

  // acc += the current tile's product: S slabs of the flat sequence.
  __device__ __forceinline__ void tile(const Operand& X, const Operand& Y, float* lds,
                                       f32x16 (&acc)[BX][BY]) {
    for (int s = 0; s < S; ++s) {
      const float* cur = lds + (it & 1) * bufFloats;
      float* nxt = lds + ((it + 1) & 1) * bufFloats;
      const bool has1 = it + 1 < iters;
      const bool has2 = it + 2 < iters;
#pragma unroll
      for (int kg = 0; kg < NG; ++kg) {
        // first k-step of the group; everything that is not an MFMA is issued
        // right behind it, in the shadow of the matrix pipe
#pragma unroll
        for (int bx = 0; bx < BX; ++bx)
#pragma unroll
          for (int by = 0; by < BY; ++by)
            acc[bx][by] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                xf[kg & 1][bx][0], yf[kg & 1][by][0], acc[bx][by], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (kg + 1 < NG) {
          read_frags(cur, kg + 1, xf[(kg + 1) & 1], yf[(kg + 1) & 1]);
        } else if (has1) {
          __syncthreads();
          read_frags(nxt, 0, xf[0], yf[0]);
        }
        if (kg == WRITE_AT) {
          if (has1) store(nxt);
          if (has2) load(X, Y);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 1; j < 4; ++j)
#pragma unroll
          for (int bx = 0; bx < BX; ++bx)
#pragma unroll
            for (int by = 0; by < BY; ++by)
              acc[bx][by] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                  xf[kg & 1][bx][j], yf[kg & 1][by][j], acc[bx][by], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      ++it;
    }
  }
};

// Element (bx, by, r) of a wave's accumulators sits at
//   x = wave_x*BX*32 + bx*32 + acc_row(r, half),   y = wave_y*BY*32 + by*32 + lane%32.
__device__ __forceinline__ int acc_row(int r, int half) {
  return 8 * (r >> 2) + 4 * half + (r & 3);
}

// Work-group ids are dealt round-robin to the 8 XCDs (each with a private
// L2).  This maps the hardware id to a logical id such that every XCD walks a
// contiguous range of logical ids; `per` = ceil(total / 8) and the grid is
// launched with 8*per work-groups.  Returns -1 for the padding ids.
__device__ __forceinline__ int xcd_logical_id(int hw_id, int total) {
  const int per = (total + 7) >> 3;
  const int logical = (hw_id & 7) * per + (hw_id >> 3);
  return logical < total ? logical : -1;
}

}  // namespace cmk
