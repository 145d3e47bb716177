// Shared fp32-MFMA tiled GEMM core for gfx950 (CDNA4, wave64).
//
// One work-group (4, 8 or 16 waves) computes a TX x TY macro tile of the product
// of two operands that both have a contraction axis k:
//   X : TX "rows"  -> MFMA source A, the axis that ends up INSIDE a lane
//   Y : TY "rows"  -> MFMA source B, the axis that ends up ACROSS lanes
// Which matrix of the user's problem plays X and which plays Y is chosen by
// each kernel so that its epilogue is cheap: a reduction wants the reduced
// axis in X (running state stays in one lane), a row-major store wants the
// contiguous axis in Y (a store instruction writes 128-byte row segments).
//
// The contraction is walked in slabs of KS (32 unless a kernel asks
// otherwise).  A slab of each operand travels from global memory straight into
// one of two LDS buffers (global_load_lds_dwordx4: no registers, no LDS store
// instructions) and is consumed from there with v_mfma_f32_32x32x2_f32.
// Inside a slab, k is consumed in groups of 8: lanes 0-31 feed k = 8g+0..3 and
// lanes 32-63 feed k = 8g+4..7 of both operands, so one 128-bit LDS read per
// 32x32 block supplies four MFMA steps.  (A sum over k does not care about the
// order, as long as both operands use the same one.)
//
// An operand tile can sit in memory in one of two ways, and keeps that order
// in LDS:
//   KC : element(row, k) at row*ld + k   (k contiguous).  LDS holds rows of KS
//        floats; the 16-byte chunk c of row r is stored at chunk c ^ (r & 7),
//        so that the 128-bit fragment reads of 32 consecutive rows spread over
//        all banks.
//   RC : element(row, k) at k*ld + row   (rows contiguous).  LDS holds KS rows
//        of T floats; fragment reads are four 32-bit reads down a column.
// A direct load deposits lane i's 16 bytes at (instruction base + 16*i), so
// the layout above is produced by choosing which global chunk each lane asks
// for.  Tiles that touch the edge of a matrix (or are not 16-byte aligned) go
// through registers instead: clamped scalar loads, zero fill, LDS stores.
//
// Plays the role of load_ab_*, buffer2smem_* and thread_matmul_* of the
// reference (kernels/bmm_helpers.cu:114-164, 240-622).
#pragma once
#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>

namespace cmk {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// Operands live in global memory; loading through pointers that say so gives
// global_load instructions (a generic pointer would give flat loads, which
// also count against the LDS wait counter).
typedef const float __attribute__((address_space(1))) * global_f32_ptr;
typedef const void __attribute__((address_space(1))) * global_void_ptr;
typedef void __attribute__((address_space(3))) * lds_void_ptr;
typedef const float __attribute__((address_space(3))) * lds_f32_ptr;
typedef const f32x4 __attribute__((address_space(3))) * lds_f32x4_ptr;

constexpr int kThreads = 256;
// what one (x, y, k) triple contributes to an accumulator
constexpr int kInner = 0;   // x*y, on the matrix pipe
constexpr int kL2 = 1;      // (x-y)^2, vector unit
constexpr int kL1 = 2;      // |x-y|,   vector unit
constexpr int KC = 0;   // k-contiguous operand
constexpr int RC = 1;   // row-contiguous operand

// f(integral_constant<int, I>) for I = 0 .. N-1, unrolled at compile time.
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

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

// Position (in floats) of element (row, k) of a T x KS operand tile in LDS.
template <int KIND, int T, int KS>
__device__ __forceinline__ int lds_pos(int row, int k) {
  if constexpr (KIND == KC)
    return row * KS + ((((k >> 2) ^ row) & 7) | ((k >> 2) & ~7)) * 4 + (k & 3);
  else
    return k * T + row;
}

// How the 1 KB pieces that one direct-load instruction moves are dealt to the
// waves: piece q = p * NW + wave covers, for KC, 256/KS consecutive rows of
// the tile and, for RC, 256 consecutive floats of the [KS][T] tile.
template <int KIND, int T, int KS, int NT>
struct LoadMap {
  static constexpr int NW = NT / 64;
  static constexpr int NI = T * KS / 256;     // pieces per tile
  static constexpr int NV = (NI + NW - 1) / NW;  // pieces (instructions) per wave
  static constexpr bool kEven = NV * NW == NI;   // otherwise only pieces q < NI exist
  static_assert(NI >= 1, "tile smaller than one piece");
  static_assert(KIND == RC || KS >= 32, "the chunk swizzle needs at least 8 chunks per row");
  static_assert(KIND == KC || 256 % T == 0 || T % 256 == 0, "row-contiguous tile width");
};

// Byte offset, relative to the tile's first element in global memory, of the 16
// bytes this lane fetches with its p-th direct load.
template <int KIND, int T, int KS, int NT>
__device__ __forceinline__ void lane_offsets_bytes(const Operand& o, int tid,
                                                   unsigned (&off)[LoadMap<KIND, T, KS, NT>::NV]) {
  using M = LoadMap<KIND, T, KS, NT>;
  const int lane = tid & 63;
  const int wave = tid >> 6;
#pragma unroll
  for (int p = 0; p < M::NV; ++p) {
    const int q = p * M::NW + wave;
    long long e;
    if constexpr (KIND == KC) {
      constexpr int CPR = KS / 4;  // chunks per row
      const int row = q * (256 / KS) + lane / CPR;
      const int slot = lane % CPR;
      const int chunk = ((slot ^ row) & 7) | (slot & ~7);
      e = (long long)row * o.ld + chunk * 4;
    } else {
      const int f = q * 256 + lane * 4;  // float position inside the [KS][T] tile
      e = (long long)(f / T) * o.ld + f % T;
    }
    off[p] = static_cast<unsigned>(e * 4);
  }
}

// One operand's slab -> LDS for a tile that crosses an edge of the matrix or
// whose operand rules out direct loads: every element is fetched from a clamped
// (always valid) address, zeroed when it lies outside the matrix, and stored
// from registers.  A real function on purpose: it runs for edge tiles only, and
// inlined at every request site it made up most of a kernel's code, which the
// interior path then had to jump across (instruction-cache misses).
template <int KIND, int T, int KS, int NT>
__device__ __noinline__ void fetch_edge(const float* p, long long ld, int rows, int K, int r0,
                                        int k0, float* dst, int tid) {
  // NT threads x 4 floats per pass, walking the tile in its memory order
  constexpr int RUN = KIND == KC ? KS : T;        // contiguous floats per line
  constexpr int TPR = RUN / 4;                    // threads per line
  constexpr int LPP = NT / TPR;                   // lines per pass
  constexpr int LINES = KIND == KC ? T : KS;
  constexpr int PASSES = (LINES + LPP - 1) / LPP;
  constexpr bool kAllLines = PASSES * LPP == LINES;  // otherwise some threads have no line
  const int t = tid;
  const int c4 = (t % TPR) * 4;
  f32x4 v[PASSES];
  const bool any = K > 0 && rows > 0;
#pragma unroll
  for (int q = 0; q < PASSES; ++q) {
    const int line = t / TPR + q * LPP;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int rj = KIND == KC ? r0 + line : r0 + c4 + j;
      const int kj = KIND == KC ? k0 + c4 + j : k0 + line;
      const bool ok = any && rj < rows && kj < K && (kAllLines || line < LINES);
      const long long e = KIND == KC ? (long long)rj * ld + kj : (long long)kj * ld + rj;
      v[q][j] = any ? *(global_f32_ptr)(ok ? p + e : p) : 0.f;
    }
  }
#pragma unroll
  for (int q = 0; q < PASSES; ++q) {
    const int line = t / TPR + q * LPP;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int rj = KIND == KC ? r0 + line : r0 + c4 + j;
      const int kj = KIND == KC ? k0 + c4 + j : k0 + line;
      v[q][j] = (rj < rows && kj < K) ? v[q][j] : 0.f;
    }
    const int pos = KIND == KC ? lds_pos<KC, T, KS>(line, c4) : lds_pos<RC, T, KS>(c4, line);
    if (kAllLines || line < LINES) *reinterpret_cast<f32x4*>(dst + pos) = v[q];
  }
}

// The same for an operand whose edge tiles can still use direct loads: 16-byte
// aligned, and the extent that a 16-byte chunk runs along (k for KC, rows for RC)
// a multiple of 4, so that a chunk lies wholly inside or wholly outside the
// matrix.  Chunks beyond K are written as zeros; chunks beyond the last row are
// fetched from the last rows instead (their products belong to output elements
// that no epilogue uses, and stay finite when the operand is).
// Inlined where registers allow (fetch_edge_direct_call below is the same as a
// real function): a call waits for the loads before it returns - the calling
// convention drains the memory counters at function boundaries - so that an edge
// tile pays the full memory latency once per slab.
template <int KIND, int T, int KS, int NT>
__device__ __forceinline__ void fetch_edge_direct(const float* p, long long ld, int rows, int K, int r0,
                                               int k0, float* dst, int tid) {
  using M = LoadMap<KIND, T, KS, NT>;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
#pragma unroll
  for (int pp = 0; pp < M::NV; ++pp) {
    const int q = pp * M::NW + wave;
    if (!M::kEven && q >= M::NI) continue;
    int k;
    long long e;
    if constexpr (KIND == KC) {
      constexpr int CPR = KS / 4;
      const int row = q * (256 / KS) + lane / CPR;
      const int slot = lane % CPR;
      const int chunk = ((slot ^ row) & 7) | (slot & ~7);
      k = k0 + chunk * 4;
      const int rr = min(r0 + row, rows - 1);
      e = (long long)rr * ld + k;
    } else {
      const int f = q * 256 + lane * 4;
      k = k0 + f / T;
      const int rr = min(r0 + f % T, rows - 4);
      e = (long long)k * ld + rr;
    }
    float* piece = dst + q * 256;
    if (k < K) {
      __builtin_amdgcn_global_load_lds((global_void_ptr)(p + e), (lds_void_ptr)piece, 16, 0, 0);
    } else {
      *reinterpret_cast<f32x4*>(piece + lane * 4) = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  }
}

template <int KIND, int T, int KS, int NT>
__device__ __noinline__ void fetch_edge_direct_call(const float* p, long long ld, int rows, int K, int r0,
                                                    int k0, float* dst, int tid) {
  fetch_edge_direct<KIND, T, KS, NT>(p, ld, rows, K, r0, k0, dst, tid);
}

// Work-group level tile engine.  WX x WY waves (4, 8 or 16 of them), each wave owns
// BX x BY blocks of 32x32; KS is the contraction depth of one LDS slab.
//
// The engine walks a flat sequence of slabs: `ntiles` consecutive X tiles
// (starting at element `xbase`) against one Y strip, S = ceil(K/KS) slabs per
// tile.  While slab i is multiplied, slab i+1 is landing in the other LDS
// buffer.  The one barrier per slab sits inside the last k-group; right after
// it the loads of slab i+2 are issued into the buffer that just became free
// and the first fragments of slab i+1 are read, so the matrix pipe keeps
// running across slab and tile boundaries.  Inside a k-group all LDS traffic is
// issued directly behind the group's first MFMA step, where it costs no
// matrix-pipe time.
// RC_READS picks how the four 32-bit column reads of a row-contiguous
// operand's fragment are issued (vector adds cost matrix-pipe time, LDS reads
// do not; which form wins was measured per tile shape):
constexpr int kReadsPaired = 1;   // two-address reads (k, k+1) with immediate offsets, one bank each
constexpr int kReadsSingle = 2;   // four single reads with immediate offsets

// ADDR_REGS keeps every fragment address in a register of its own for the whole
// sequence (no vector arithmetic in the slab loop); without it the compiler is
// free to re-derive them, which a kernel short of registers prefers.
//
// Y_PAIRS (BY == 2) deals the Y rows of a wave to its two blocks alternately -
// block b of lane l takes row 2 * (l % 32) + b of the wave's 64 instead of
// (l % 32) + 32 * b - so that a lane's two accumulators of one X row are
// neighbours along Y: an epilogue that stores along Y writes them as one
// 8-byte store.  Only the fragment addresses change.
template <int XK, int YK, int WX, int WY, int BX, int BY, int KS_ = 32, int RC_READS = kReadsPaired,
          bool STAGGER = false, bool Y_ONCE = false, bool ADDR_REGS = true, bool Y_PAIRS = false>
struct Core {
  static_assert(!Y_PAIRS || BY == 2, "Y_PAIRS pairs the two Y blocks of a wave");
  static_assert(WX * WY == 4 || WX * WY == 8 || WX * WY == 16, "4, 8 or 16 waves per work-group");
  static constexpr int NT = WX * WY * 64;      // threads per work-group
  static constexpr int KS = KS_;
  static constexpr int NG = KS / 8;            // k-groups per slab
  static constexpr int TX = WX * BX * 32;
  static constexpr int TY = WY * BY * 32;
  static_assert(NG >= 2 && NG % 2 == 0, "slab depth");
  static constexpr int xFloats = TX * KS;
  static constexpr int yFloats = TY * KS;
  static constexpr int bufFloats = xFloats + yFloats;
  static constexpr int ldsFloats = 2 * bufFloats;
  using MX = LoadMap<XK, TX, KS, NT>;
  using MY = LoadMap<YK, TY, KS, NT>;

  f32x4 xf[2][BX];           // fragments; [0] holds k-group 0 of the current slab at slab entry
  f32x4 yf[2][BY];
  int it, iters, S;          // flat slab counter (wave-uniform)
  int lt, ls;                // (tile, slab) of the next slab to fetch (wave-uniform)
  int ct, cs, nt;            // Y_ONCE: (tile, slab) being multiplied, tiles in the sequence
  // element offset of the next slab to fetch within each operand, advanced by
  // additions from slab to slab (all wave-uniform)
  long long xrun, yrun, xstep_in, xstep_out, ystep;
  int xbase, y0, K;
  int xr, yr, half, tid;
  // Interior test of a slab in three scalar subtractions: last first-row (and
  // last first-k) at which a whole tile still lies inside the matrix; -2 * tile
  // size for an operand that rules out direct loads (unaligned, or offsets beyond
  // 32 bits).
  int xlast, ylast, klast;
  // LDS byte addresses of this lane's fragments in buffer 0, kept in registers
  // for the whole sequence so that a fragment read is (register + immediate):
  // a row-contiguous operand needs one per block (k advances by immediates), a
  // k-contiguous one needs one per block and k-group (the chunk swizzle is an
  // exclusive-or, not a sum)
  static constexpr int NAX = XK == KC ? NG : 1;
  static constexpr int NAY = YK == KC ? NG : 1;
  unsigned xad[BX][NAX], yad[BY][NAY];
  unsigned xoff[MX::NV];     // this lane's byte offsets for the direct loads
  unsigned yoff[MY::NV];
  float* pend_buf;           // where the Y slab that is still to be requested goes (wave-uniform)
  float* ybase;              // Y_ONCE: the two Y buffers, behind the two X buffers
  int pend_k0;
  long long pend_y;          // and its element offset
  float* pend_xbuf;          // buffer whose X half is still to be requested (wave-uniform)
  bool late;                 // this wave requests its slabs two k-groups after its SIMD partner
  int wave_s;                // ADDR_REGS: the wave's index, kept in a scalar register

  // One operand's slab -> LDS.  Interior tiles: NV direct loads per wave.  Edge
  // tiles: fetch_edge().
  template <int KIND, int T, class M>
  __device__ __forceinline__ void fetch(const Operand& o, unsigned (&off)[M::NV], int r0,
                                        int k0, long long first, float* dst, int rlast) {
    // both differences are non-negative exactly for an interior slab; one sign
    // test on plain 32-bit scalars
    const bool interior = ((klast - k0) | (rlast - r0)) >= 0;
    // Keeps each offset a plain 32-bit register where the loads use it (the load
    // is then scalar base + lane offset).  Pinned in place and ahead of the
    // branch: no copies, and both paths leave the same registers behind.
    if constexpr (ADDR_REGS) {
#pragma unroll
      for (int p = 0; p < M::NV; ++p) asm volatile("" : "+v"(off[p]));
    }
    if (interior) {
      // the tile's address is the same in every lane; pinned to scalar registers
      // so that each load is (scalar base + 32-bit lane offset) with no vector add
      unsigned long long tile_bits = reinterpret_cast<unsigned long long>(o.p + first);
      asm volatile("" : "+s"(tile_bits));
      const char* tile = reinterpret_cast<const char*>(tile_bits);
      const int wave = ADDR_REGS ? wave_s : __builtin_amdgcn_readfirstlane(tid >> 6);
#pragma unroll
      for (int p = 0; p < M::NV; ++p)
        if (M::kEven || p * M::NW + wave < M::NI) {
          if constexpr (!ADDR_REGS) asm volatile("" : "+v"(off[p]));  // short of registers: pinned where used
          const unsigned o32 = off[p];
          __builtin_amdgcn_global_load_lds((global_void_ptr)(tile + o32),
                                           (lds_void_ptr)(dst + (p * M::NW + wave) * 256), 16, 0, 0);
        }
    } else if (rlast >= -T && (KIND == KC ? (K & 3) == 0 : (o.rows & 3) == 0)) {
      // (rlast >= -T: direct loads are legal for this operand and it has at least 4 rows / 1 row)
      // (a kernel that runs without address registers is short of registers altogether)
      if constexpr (ADDR_REGS) fetch_edge_direct<KIND, T, KS, NT>(o.p, o.ld, o.rows, K, r0, k0, dst, tid);
      else fetch_edge_direct_call<KIND, T, KS, NT>(o.p, o.ld, o.rows, K, r0, k0, dst, tid);
    } else {
      fetch_edge<KIND, T, KS, NT>(o.p, o.ld, o.rows, K, r0, k0, dst, tid);
    }
  }

  // Starts the transfer of the next slab of the sequence into `buf`: the X
  // operand now, the Y operand one k-group later (issue_y), so that the waves'
  // loads do not all queue up at the memory pipeline in the same few cycles.
  __device__ __forceinline__ void issue_x(const Operand& X, float* buf) {
    // the slab coordinates are the same for every lane; saying so keeps the
    // address arithmetic on the scalar unit
    const int x0 = __builtin_amdgcn_readfirstlane(xbase + lt * TX);
    pend_k0 = __builtin_amdgcn_readfirstlane(ls * KS);
    fetch<XK, TX, MX>(X, xoff, x0, pend_k0, xrun, buf, xlast);
    if constexpr (Y_ONCE) {
      // tiles run inside slabs: the Y slab is fetched with the first tile only
      pend_buf = lt == 0 ? ybase + (ls & 1) * yFloats : nullptr;
      pend_y = yrun;
      xrun += xstep_in;
      if (++lt == nt) { lt = 0; ++ls; xrun += xstep_out; yrun += ystep; }
    } else {
      pend_buf = buf + xFloats;
      pend_y = yrun;
      xrun += xstep_in;
      yrun += ystep;
      if (++ls == S) { ls = 0; ++lt; xrun += xstep_out; yrun -= S * ystep; }
    }
  }
  __device__ __forceinline__ void issue_y(const Operand& Y) {
    if (pend_buf) fetch<YK, TY, MY>(Y, yoff, y0, pend_k0, pend_y, pend_buf, ylast);
    pend_buf = nullptr;
  }
  __device__ __forceinline__ void issue_pending_x(const Operand& X) {
    if (pend_xbuf) issue_x(X, pend_xbuf);
    pend_xbuf = nullptr;
  }

  // Four k values (8*kg + 4*half + 0..3) of one block row of this lane, from the
  // buffer `off` floats behind buffer 0.  With a compile-time `off` the whole
  // displacement is an immediate of the read.
  template <int KIND, int T, int NA>
  __device__ __forceinline__ f32x4 frag(const unsigned (&ad)[NA], int off, int kg) const {
    if constexpr (KIND == KC) {
      return *(lds_f32x4_ptr)static_cast<uintptr_t>(ad[kg] + 4u * off);
    } else {
      f32x4 r;
      const unsigned at = ad[0] + 4u * (off + kg * 8 * T);
      if constexpr (RC_READS == kReadsSingle) {
        // volatile keeps the reads single: 16-bit immediate offsets from one
        // address register
        const volatile float __attribute__((address_space(3)))* q =
            (const volatile float __attribute__((address_space(3)))*)static_cast<uintptr_t>(at);
        r.x = q[0];
        r.y = q[T];
        r.z = q[2 * T];
        r.w = q[3 * T];
        return r;
      }
      lds_f32_ptr q = (lds_f32_ptr)static_cast<uintptr_t>(at);
      r.x = q[0];
      r.y = q[T];
      r.z = q[2 * T];
      r.w = q[3 * T];
      return r;
    }
  }
  // Fragments of k-group kg from the X buffer at float offset xo and the Y buffer at yo.
  __device__ __forceinline__ void read_frags(int xo, int yo, int kg,
                                             f32x4 (&fx)[BX], f32x4 (&fy)[BY]) const {
#pragma unroll
    for (int b = 0; b < BX; ++b) fx[b] = frag<XK, TX, NAX>(xad[b], xo, kg);
#pragma unroll
    for (int b = 0; b < BY; ++b) fy[b] = frag<YK, TY, NAY>(yad[b], yo, kg);
  }

  // Waits until this wave's direct loads have landed in LDS.
  __device__ __forceinline__ void wait_loads() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), leave expcnt / lgkmcnt alone
  }

  // Fills the pipeline: slab 0 in LDS with its first fragments in registers,
  // slab 1 in flight.  Ends with every wave past a barrier.
  __device__ __forceinline__ void begin(const Operand& X, const Operand& Y, int xbase_, int y0_,
                                        int K_, int ntiles, float* lds) {
    // The thread id is made opaque per sequence: values derived from it are
    // then computed where they are used instead of being hoisted out of a
    // kernel's outer loops, where they would only occupy (or spill) registers.
    tid = threadIdx.x;
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63;
    const int wave = tid >> 6;
    half = lane >> 5;
    wave_s = __builtin_amdgcn_readfirstlane(wave);
    xr = (wave % WX) * BX * 32 + (lane & 31);
    yr = (wave / WX) * BY * 32 + (lane & 31);
    {
      // Opaque to the compiler, so that the addresses stay in their registers
      // instead of being re-derived (vector adds cost matrix-pipe time) and so
      // that reads of neighbouring blocks are not fused into two-address reads
      // whose 8-bit offsets would need an add per pair.
      const unsigned base = static_cast<unsigned>(reinterpret_cast<uintptr_t>((lds_f32_ptr)lds));
#pragma unroll
      for (int b = 0; b < BX; ++b)
#pragma unroll
        for (int g = 0; g < NAX; ++g) {
          const int row = xr + 32 * b;
          xad[b][g] = base + 4u * (XK == KC ? lds_pos<KC, TX, KS>(row, g * 8 + half * 4) : half * 4 * TX + row);
          if (ADDR_REGS) asm volatile("" : "+v"(xad[b][g]));
        }
#pragma unroll
      for (int b = 0; b < BY; ++b)
#pragma unroll
        for (int g = 0; g < NAY; ++g) {
          const int row = Y_PAIRS ? (wave / WX) * BY * 32 + 2 * (lane & 31) + b : yr + 32 * b;
          yad[b][g] = base + 4u * (YK == KC ? lds_pos<KC, TY, KS>(row, g * 8 + half * 4) : half * 4 * TY + row);
          if (ADDR_REGS) asm volatile("" : "+v"(yad[b][g]));
        }
    }
    xbase = __builtin_amdgcn_readfirstlane(xbase_);
    y0 = __builtin_amdgcn_readfirstlane(y0_);
    K = __builtin_amdgcn_readfirstlane(K_);
    S = max(1, (K + KS - 1) / KS);
    // (first row of the last tile that lies wholly inside; negative when there is none;
    // below -tile size: no direct loads for this operand at all)
    xlast = (X.vec != 0 && X.rows > 0 && (long long)(TX + KS) * X.ld < (1ll << 29)) ? X.rows - TX : -2 * TX;
    ylast = (Y.vec != 0 && Y.rows > 0 && (long long)(TY + KS) * Y.ld < (1ll << 29)) ? Y.rows - TY : -2 * TY;
    klast = K - KS;
    nt = __builtin_amdgcn_readfirstlane(ntiles);
    iters = nt * S;
    ct = 0;
    cs = 0;
    {
      // steps of the running offsets: to the next slab of the inner loop, and
      // the correction when the inner loop wraps
      const long long xs_tile = XK == KC ? (long long)TX * X.ld : TX;
      const long long xs_slab = XK == KC ? KS : (long long)KS * X.ld;
      xrun = XK == KC ? (long long)xbase * X.ld : xbase;
      yrun = YK == KC ? (long long)y0 * Y.ld : y0;
      ystep = YK == KC ? KS : (long long)KS * Y.ld;
      if (Y_ONCE) { xstep_in = xs_tile; xstep_out = xs_slab - nt * xs_tile; }
      else        { xstep_in = xs_slab; xstep_out = xs_tile - S * xs_slab; }
    }
    ybase = lds + 2 * xFloats;
    lane_offsets_bytes<XK, TX, KS, NT>(X, tid, xoff);
    lane_offsets_bytes<YK, TY, KS, NT>(Y, tid, yoff);
    it = 0;
    lt = 0;
    ls = 0;
    pend_xbuf = nullptr;
    // STAGGER: the upper half of the waves does its address arithmetic and load
    // requests two k-groups after the lower half, which spreads the requests
    // over the slab (measured: a gain for the 4-wave min kernel, none for the
    // top-k kernel)
    late = STAGGER && __builtin_amdgcn_readfirstlane(wave) >= WX * WY / 2;
    issue_x(X, lds);
    issue_y(Y);
    wait_loads();
    __syncthreads();
    if (iters > 1) issue_x(X, xbuf(lds, 1));
    read_frags(xoff_of(0), yoff_of(0, 0), 0, xf[0], yf[0]);
  }

  // LDS buffers of flat slab `i`, whose k-slab index is `s`.  Without Y_ONCE an
  // X and a Y slab sit side by side, twice; with it, two X buffers are followed
  // by two Y buffers that alternate with the k-slab.
  __device__ __forceinline__ int xoff_of(int i) const {
    return (i & 1) * (Y_ONCE ? xFloats : bufFloats);
  }
  __device__ __forceinline__ int yoff_of(int i, int s) const {
    return Y_ONCE ? 2 * xFloats + (s & 1) * yFloats : xoff_of(i) + xFloats;
  }
  __device__ __forceinline__ float* xbuf(float* lds, int i) const { return lds + xoff_of(i); }
  __device__ __forceinline__ float* ybuf(float* lds, int i, int s) const { return lds + yoff_of(i, s); }

  // acc += the current tile's product: S slabs of the flat sequence.
  // With FRESH the accumulators need no clearing: the tile's first matrix
  // instructions take a literal zero as their addend, which saves the 16 * BX * BY
  // vector moves that would otherwise stall the matrix pipe.
  template <int DIST = kInner, bool FRESH = false>
  __device__ __forceinline__ void tile(const Operand& X, const Operand& Y, float* lds,
                                       f32x16 (&acc)[BX][BY]) {
    static_assert(!Y_ONCE, "with Y_ONCE the kernel walks slabs itself: tiles inside k-slabs");
    static_assert(!FRESH || DIST == kInner, "only the matrix path can start from a literal zero");
    if constexpr (DIST != kInner) {
      for (int s = 0; s < S; ++s) slab<DIST>(X, Y, lds, acc);
    } else if ((S & 1) == 0) {
      // an even slab count keeps the flat slab counter even at every tile
      // start: the buffer of each slab is then known at compile time
      slab<DIST, FRESH, 0>(X, Y, lds, acc);
      slab<DIST, false, 1>(X, Y, lds, acc);
      for (int s = 2; s < S; s += 2) {
        slab<DIST, false, 0>(X, Y, lds, acc);
        slab<DIST, false, 1>(X, Y, lds, acc);
      }
    } else {
      slab<DIST, FRESH>(X, Y, lds, acc);
      for (int s = 1; s < S; ++s) slab<DIST>(X, Y, lds, acc);
    }
  }

  // The distances other than the inner product have no matrix-pipe form.  They
  // run on the vector unit over the same LDS slabs and into the same accumulator
  // layout as the MFMA path (register r of a lane: X row acc_row(r, half) of the
  // block, Y row lane % 32), so the kernels' epilogues do not change.  Per
  // accumulator the k values are taken in ascending order with the reference's
  // operations (kernels/bmm_helpers.cu:28-35, 46-52): d = x - y, then
  // fmaf(d, d, c) or c + fabsf(d).  Zero-filled padding along k adds nothing.
  template <int DIST>
  __device__ __forceinline__ void dist_group(const float* xb, const float* yb, int kg,
                                             f32x16 (&acc)[BX][BY]) {
    const int l32 = tid & 31;
    const int xw = ((tid >> 6) % WX) * BX * 32 + 4 * half;   // first X row of this half-wave
    static_assert(!Y_PAIRS, "the vector-unit distances deal Y rows block by block");
    const int yl = ((tid >> 6) / WX) * BY * 32 + l32;        // this lane's first Y row
    float y[BY][8];
#pragma unroll
    for (int by = 0; by < BY; ++by) {
      if constexpr (YK == KC) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const f32x4 v = *reinterpret_cast<const f32x4*>(&yb[lds_pos<KC, TY, KS>(yl + 32 * by, kg * 8 + 4 * h)]);
          y[by][4 * h] = v.x; y[by][4 * h + 1] = v.y; y[by][4 * h + 2] = v.z; y[by][4 * h + 3] = v.w;
        }
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) y[by][k] = yb[(kg * 8 + k) * TY + yl + 32 * by];
      }
    }
    auto add = [](float xv, float yv, float cv) {
      const float d = xv - yv;
      return DIST == kL2 ? __builtin_fmaf(d, d, cv) : cv + __builtin_fabsf(d);
    };
#pragma unroll
    for (int bx = 0; bx < BX; ++bx)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int row0 = xw + 32 * bx + 8 * rg;   // rows row0 .. row0+3 are registers 4rg .. 4rg+3
        if constexpr (XK == KC) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float x[8];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
              const f32x4 v = *reinterpret_cast<const f32x4*>(&xb[lds_pos<KC, TX, KS>(row0 + e, kg * 8 + 4 * h)]);
              x[4 * h] = v.x; x[4 * h + 1] = v.y; x[4 * h + 2] = v.z; x[4 * h + 3] = v.w;
            }
#pragma unroll
            for (int by = 0; by < BY; ++by)
#pragma unroll
              for (int k = 0; k < 8; ++k) acc[bx][by][4 * rg + e] = add(x[k], y[by][k], acc[bx][by][4 * rg + e]);
          }
        } else {
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(&xb[(kg * 8 + k) * TX + row0]);
            const float x[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int by = 0; by < BY; ++by)
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[bx][by][4 * rg + e] = add(x[e], y[by][k], acc[bx][by][4 * rg + e]);
          }
        }
      }
  }

  // acc += one slab of the flat sequence.
  // PAR >= 0 states the parity of the flat slab counter, i.e. which X buffer
  // (and, without Y_ONCE, which Y buffer) the slab lives in, at compile time:
  // fragment reads then need no address arithmetic at all.
  // With Y_ONCE the Y buffer alternates with the k-slab instead: YPAR / YNPAR
  // state the k-slab parity of this slab and of the next one in the sequence.
  template <int DIST = kInner, bool FRESH = false, int PAR = -1, int YPAR = -1, int YNPAR = -1>
  __device__ __forceinline__ void slab(const Operand& X, const Operand& Y, float* lds,
                                       f32x16 (&acc)[BX][BY]) {
    if constexpr (DIST != kInner) {
      float* cur = xbuf(lds, it);
      const float* ycur = ybuf(lds, it, cs);
      const bool has1 = it + 1 < iters;
      const bool has2 = it + 2 < iters;
      issue_y(Y);
#pragma unroll 1   // a k-group is 2 * 64 * BX * BY * 8 vector instructions: keep the code in the instruction cache
      for (int kg = 0; kg < NG; ++kg) dist_group<DIST>(cur, ycur, kg, acc);
      if (has1) {
        wait_loads();     // this wave's part of slab it+1 is in LDS
        __syncthreads();  // everyone's is, and nobody reads `cur` any more
        pend_xbuf = has2 ? cur : nullptr;
        issue_pending_x(X);
      }
      ++it;
      if (Y_ONCE && ++ct == nt) { ct = 0; ++cs; }
    } else {
      const int ns = (Y_ONCE && ct + 1 == nt) ? cs + 1 : cs;   // k-slab of the next flat slab
      const int curx = xoff_of(PAR < 0 ? it : PAR);
      const int nxtx = xoff_of(PAR < 0 ? it + 1 : PAR + 1);
      const int cury = (Y_ONCE && YPAR >= 0) ? yoff_of(0, YPAR) : yoff_of(PAR < 0 ? it : PAR, cs);
      const int nxty = (Y_ONCE && YNPAR >= 0) ? yoff_of(0, YNPAR) : yoff_of(PAR < 0 ? it + 1 : PAR + 1, ns);
      float* cur = lds + curx;
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
                xf[kg & 1][bx][0], yf[kg & 1][by][0], (FRESH && kg == 0) ? f32x16{} : acc[bx][by], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (kg == 0 && !late) issue_y(Y);
        if (kg == 1 && late) issue_pending_x(X);
        if (kg == 2 && late) issue_y(Y);
        if (kg + 1 < NG) {
          read_frags(curx, cury, kg + 1, xf[(kg + 1) & 1], yf[(kg + 1) & 1]);
        } else if (has1) {
          wait_loads();     // this wave's part of slab it+1 is in LDS
          __syncthreads();  // everyone's is, and nobody reads `cur` any more
          pend_xbuf = has2 ? cur : nullptr;
          if (!late) issue_pending_x(X);
          read_frags(nxtx, nxty, 0, xf[0], yf[0]);
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
      if (Y_ONCE && ++ct == nt) { ct = 0; ++cs; }
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
