// Wave-level exact top-128 selection and a wave64 bitonic sorter.
//
// A wave holds NR*64 candidates of one output row, NR per lane, as 32-bit
// order-preserving keys plus 32-bit indices.  select128() finds the 128 largest
// in three moves:
//   1. Bracket the key of the 128th largest, [lo, hi), by counting candidates
//      >= t with wave ballots.  The bracket starts around the previous row's
//      answer (rows of one strip are statistically alike) and is bisected until
//      it holds at most 128 candidates.
//   2. One pass over the registers sends every candidate >= hi to the output
//      list and every candidate inside the bracket to a band list (both in LDS,
//      as 64-bit (key, ~index) entries).
//   3. The band, now two entries per lane, is bisected to the exact threshold
//      and its winners are appended to the output list.
// The output list is unordered; bitonic128_desc() orders it once, at the very
// end, so that values descend and equal values come out by ascending index.
//
// Replaces the reference's per-tile sort / lock / merge against a global
// running list (kernels/topkbmm.cu:13-47, 98-183; network also in
// kernels/bitonic_sort.cu:122-180): here a row is owned by one wave, nothing
// is locked and nothing is read back from HBM.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cmk {

// Monotone map float -> uint32: a < b  <=>  key(a) < key(b) (with -0 < +0 and
// NaNs at the extremes).  Key 0 is reserved for "no candidate".
__device__ __forceinline__ uint32_t f2key(float f) {
  const uint32_t u = __float_as_uint(f);
  return u ^ (static_cast<uint32_t>(static_cast<int32_t>(u) >> 31) | 0x80000000u);
}
__device__ __forceinline__ float key2f(uint32_t k) {
  if (k == 0) return -__builtin_inff();
  const uint32_t u = (k & 0x80000000u) ? (k ^ 0x80000000u) : ~k;
  return __uint_as_float(u);
}

constexpr int kTop = 128;
typedef unsigned long long entry_t;  // (key << 32) | ~index; 0 = empty slot (key 0, index -1)

__device__ __forceinline__ entry_t pack_entry(uint32_t key, int idx) {
  return (static_cast<entry_t>(key) << 32) | static_cast<uint32_t>(~idx);
}
__device__ __forceinline__ uint32_t entry_key(entry_t e) { return static_cast<uint32_t>(e >> 32); }
__device__ __forceinline__ int entry_idx(entry_t e) {
  return static_cast<int>(~static_cast<uint32_t>(e));
}

// Lanes below this one that are set in `mask`.
__device__ __forceinline__ int prefix_in(unsigned long long mask) {
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0));
}

// Middle of the bracket [lo, hi) where hi == 0 stands for 2^32 (hi - lo wraps
// to the right width except when lo == 0 as well).
__device__ __forceinline__ uint32_t bracket_mid(uint32_t lo, uint32_t hi) {
  return (lo == 0 && hi == 0) ? 0x80000000u : lo + ((hi - lo) >> 1);
}

// Selects, for each of R rows at once, the 128 largest keys among key[r][0..NR)
// of all 64 lanes and writes them as entries to out[r][0..128) (LDS owned by
// this wave).  The R rows are independent; working on them side by side lets
// the counting chains of one row hide the latency of the other.  band[r] is 128
// entries of wave-private LDS scratch.  seed[r] carries the threshold key from
// one call to the next (0 = none); idx_of(r, j) is the index of candidate
// key[r][j] of this lane.  Ties at the threshold: earliest (register,
// lane) position first.  Fewer than 128 real candidates leave empty entries.
template <int NR, int R, class IdxOf>
__device__ __forceinline__ void select128(const uint32_t (&key)[R][NR], IdxOf&& idx_of,
                                          uint32_t (&seed)[R], entry_t* const (&band)[R],
                                          entry_t* const (&out)[R]) {
  const int lane = threadIdx.x & 63;
  // bracket: count(>= lo) >= 128 > count(>= hi); hi == 0 stands for 2^32
  uint32_t lo[R], hi[R];
  int c_lo[R], c_hi[R];
#pragma unroll
  for (int r = 0; r < R; ++r) { lo[r] = 0; hi[r] = 0; c_lo[r] = NR * 64; c_hi[r] = 0; }

  auto count_ge = [&](int r, uint32_t t) {
    int c = 0;
#pragma unroll
    for (int j = 0; j < NR; ++j) c += __popcll(__ballot(key[r][j] >= t));
    return c;
  };
  auto narrow = [&](int r, uint32_t t, int c) {
    if (c >= kTop) { lo[r] = t; c_lo[r] = c; } else { hi[r] = t; c_hi[r] = c; }
  };

  constexpr uint32_t D = 1u << 20;  // +-12% of a float's magnitude
  {
    uint32_t t[R];
    int c[R];
#pragma unroll
    for (int r = 0; r < R; ++r) t[r] = seed[r] > D ? seed[r] - D : 1u;
#pragma unroll
    for (int r = 0; r < R; ++r) c[r] = seed[r] ? count_ge(r, t[r]) : 0;
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (seed[r]) narrow(r, t[r], c[r]);
    bool second[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      second[r] = seed[r] && hi[r] == 0 && seed[r] < 0xFFFFFFFFu - D;
      t[r] = seed[r] + D;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) c[r] = second[r] ? count_ge(r, t[r]) : 0;
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (second[r]) narrow(r, t[r], c[r]);
  }
  for (;;) {
    bool act[R], any = false;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      act[r] = c_lo[r] - c_hi[r] > kTop && hi[r] - lo[r] != 1u;
      any = any || act[r];
    }
    if (!any) break;
    uint32_t t[R];
    int c[R];
#pragma unroll
    for (int r = 0; r < R; ++r) t[r] = bracket_mid(lo[r], hi[r]);
#pragma unroll
    for (int r = 0; r < R; ++r) c[r] = act[r] ? count_ge(r, t[r]) : 0;
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (act[r]) narrow(r, t[r], c[r]);
  }

  // one pass: candidates >= hi go to out[0, c_hi), candidates in [lo, hi) to the band
  int base_band[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    int base_out = 0;
    base_band[r] = 0;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const uint32_t k = key[r][j];
      const bool ge_lo = k >= lo[r];
      const bool ge_hi = hi[r] != 0 && k >= hi[r];
      const unsigned long long m_lo = __ballot(ge_lo);
      const unsigned long long m_hi = __ballot(ge_hi);
      const unsigned long long m_band = m_lo & ~m_hi;
      const entry_t e = pack_entry(k, k ? idx_of(r, j) : -1);
      if (ge_hi) {
        out[r][base_out + prefix_in(m_hi)] = e;
      } else if (ge_lo) {
        const int pos = base_band[r] + prefix_in(m_band);
        if (pos < kTop) band[r][pos] = e;
      }
      base_out += __popcll(m_hi);
      base_band[r] += __popcll(m_band);
    }
  }

  // the band: two entries per lane and row, `need` of them are wanted
  int need[R], cb_lo[R];
  entry_t b0[R], b1[R];
  uint32_t k0[R], k1[R];
  bool v0[R], v1[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    need[r] = kTop - c_hi[r];
    const int nband = base_band[r] < kTop ? base_band[r] : kTop;
    v0[r] = lane < nband;
    v1[r] = lane + 64 < nband;
    b0[r] = v0[r] ? band[r][lane] : 0ull;
    b1[r] = v1[r] ? band[r][lane + 64] : 0ull;
    k0[r] = entry_key(b0[r]);
    k1[r] = entry_key(b1[r]);
    cb_lo[r] = base_band[r];  // everything in the band is >= lo
  }
  // exact threshold inside the band: largest t with count(band >= t) >= need
  for (;;) {
    bool act[R], any = false;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      act[r] = cb_lo[r] != need[r] && hi[r] - lo[r] != 1u;
      any = any || act[r];
    }
    if (!any) break;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32_t mid = bracket_mid(lo[r], hi[r]);
      const int c = __popcll(__ballot(v0[r] && k0[r] >= mid)) + __popcll(__ballot(v1[r] && k1[r] >= mid));
      if (act[r]) {
        if (c >= need[r]) { lo[r] = mid; cb_lo[r] = c; } else { hi[r] = mid; }
      }
    }
  }
  // winners: every band entry >= lo when that is exactly `need` of them,
  // otherwise (ties at lo) those above lo and then the first ones equal to lo
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const bool exact = cb_lo[r] == need[r];
    const bool g0 = v0[r] && (exact ? k0[r] >= lo[r] : k0[r] > lo[r]);
    const bool g1 = v1[r] && (exact ? k1[r] >= lo[r] : k1[r] > lo[r]);
    const unsigned long long mg0 = __ballot(g0), mg1 = __ballot(g1);
    const int ng0 = __popcll(mg0), ng = ng0 + __popcll(mg1);
    if (g0) out[r][c_hi[r] + prefix_in(mg0)] = b0[r];
    if (g1) out[r][c_hi[r] + ng0 + prefix_in(mg1)] = b1[r];
    if (!exact) {
      const bool q0 = v0[r] && k0[r] == lo[r], q1 = v1[r] && k1[r] == lo[r];
      const unsigned long long mq0 = __ballot(q0), mq1 = __ballot(q1);
      const int p0 = c_hi[r] + ng + prefix_in(mq0);
      const int p1 = c_hi[r] + ng + __popcll(mq0) + prefix_in(mq1);
      if (q0 && p0 < kTop) out[r][p0] = b0[r];
      if (q1 && p1 < kTop) out[r][p1] = b1[r];
    }
    seed[r] = lo[r];
  }
}

// Value of `v` in lane (lane ^ STRIDE).
template <int STRIDE>
__device__ __forceinline__ uint32_t lane_xor(uint32_t v) {
  if constexpr (STRIDE == 1) {
    return __builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
  } else if constexpr (STRIDE == 2) {
    return __builtin_amdgcn_mov_dpp(v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
  } else if constexpr (STRIDE < 32) {
    return __builtin_amdgcn_ds_swizzle(v, (STRIDE << 10) | 0x1F);  // lane ^= STRIDE inside 32
  } else {
    return __builtin_amdgcn_ds_bpermute(((threadIdx.x & 63) ^ 32) << 2, v);
  }
}

// Lanes (as a 64-bit mask) that keep the larger entry in the compare-exchange
// with stride STRIDE while sorting blocks of SIZE; ELEM 0 sits at position
// lane, ELEM 1 at position lane + 64.  Descending blocks keep the larger entry
// in the lower position.
template <int SIZE, int STRIDE, int ELEM>
constexpr unsigned long long keep_max_mask() {
  unsigned long long m = 0;
  for (int lane = 0; lane < 64; ++lane) {
    const bool lower = (lane & STRIDE) == 0;
    const int pos = lane + 64 * ELEM;
    const bool desc = SIZE == 128 ? true : ((pos & SIZE) == 0);
    if (lower == desc) m |= 1ull << lane;
  }
  return m;
}

template <int SIZE, int STRIDE, int R>
__device__ __forceinline__ void bitonic_stage(entry_t (&e0)[R], entry_t (&e1)[R]) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if constexpr (STRIDE == 64) {
      const entry_t hi = e0[r] > e1[r] ? e0[r] : e1[r];
      const entry_t lo = e0[r] > e1[r] ? e1[r] : e0[r];
      e0[r] = hi;
      e1[r] = lo;
    } else {
      const entry_t o0 =
          (static_cast<entry_t>(lane_xor<STRIDE>(static_cast<uint32_t>(e0[r] >> 32))) << 32) |
          lane_xor<STRIDE>(static_cast<uint32_t>(e0[r]));
      const entry_t o1 =
          (static_cast<entry_t>(lane_xor<STRIDE>(static_cast<uint32_t>(e1[r] >> 32))) << 32) |
          lane_xor<STRIDE>(static_cast<uint32_t>(e1[r]));
      // take the partner's entry where (partner larger) == (this lane keeps the larger)
      constexpr unsigned long long km0 = keep_max_mask<SIZE, STRIDE, 0>();
      constexpr unsigned long long km1 = keep_max_mask<SIZE, STRIDE, 1>();
      const bool t0 = __builtin_amdgcn_inverse_ballot_w64(__ballot(o0 > e0[r]) ^ ~km0);
      const bool t1 = __builtin_amdgcn_inverse_ballot_w64(__ballot(o1 > e1[r]) ^ ~km1);
      e0[r] = t0 ? o0 : e0[r];
      e1[r] = t1 ? o1 : e1[r];
    }
  }
}

template <int SIZE, int STRIDE, int R>
__device__ __forceinline__ void bitonic_merge(entry_t (&e0)[R], entry_t (&e1)[R]) {
  bitonic_stage<SIZE, STRIDE, R>(e0, e1);
  if constexpr (STRIDE > 1) bitonic_merge<SIZE, STRIDE / 2, R>(e0, e1);
}

// Sorts, for R rows at once, 128 entries held two per lane (e0 at position
// lane, e1 at position lane + 64) into descending order of position.  Must be
// called by whole waves.  The network is the one of the reference
// (bitonic_sort_128, kernels/topkbmm.cu:98-139) with the final merge turned to
// descending order.
template <int R>
__device__ __forceinline__ void bitonic128_desc(entry_t (&e0)[R], entry_t (&e1)[R]) {
  bitonic_merge<2, 1, R>(e0, e1);
  bitonic_merge<4, 2, R>(e0, e1);
  bitonic_merge<8, 4, R>(e0, e1);
  bitonic_merge<16, 8, R>(e0, e1);
  bitonic_merge<32, 16, R>(e0, e1);
  bitonic_merge<64, 32, R>(e0, e1);
  bitonic_merge<128, 64, R>(e0, e1);
}

// Sorts R 128-entry lists and writes the first k entries of each as fp32
// values and int64 indices; a null values[r] skips the store of that row.
template <int R>
__device__ __forceinline__ void sort_and_store(const entry_t* const (&list)[R],
                                               float* const (&values)[R],
                                               long long* const (&indices)[R], int k) {
  const int lane = threadIdx.x & 63;
  entry_t e0[R], e1[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    e0[r] = list[r][lane];
    e1[r] = list[r][lane + 64];
  }
  bitonic128_desc<R>(e0, e1);
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (!values[r]) continue;
    if (lane < k) {
      values[r][lane] = key2f(entry_key(e0[r]));
      indices[r][lane] = entry_idx(e0[r]);
    }
    if (lane + 64 < k) {
      values[r][lane + 64] = key2f(entry_key(e1[r]));
      indices[r][lane + 64] = entry_idx(e1[r]);
    }
  }
}

}  // namespace cmk
