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

// Number of candidates of the wave with key >= t.
template <int NR>
__device__ __forceinline__ int count_ge(const uint32_t (&key)[NR], uint32_t t) {
  int c = 0;
#pragma unroll
  for (int j = 0; j < NR; ++j) c += __popcll(__ballot(key[j] >= t));
  return c;
}

// Lanes below this one that are set in `mask`.
__device__ __forceinline__ int prefix_in(unsigned long long mask) {
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0));
}

// Selects the 128 largest keys among key[0..NR) of all 64 lanes and writes them
// as entries to out[0..128) (LDS owned by this wave).  `band` is 128 entries of
// wave-private LDS scratch.  `seed` carries the threshold key from one call to
// the next (0 = none).  Ties at the threshold: earliest (register, lane)
// position first.  Fewer than 128 real candidates leave empty (0) entries.
template <int NR>
__device__ __forceinline__ void select128(const uint32_t (&key)[NR], const int (&idx)[NR],
                                          uint32_t& seed, entry_t* band, entry_t* out) {
  const int lane = threadIdx.x & 63;
  // bracket: count(>= lo) >= 128 > count(>= hi); hi == 0 stands for 2^32
  uint32_t lo = 0, hi = 0;
  int c_lo = NR * 64, c_hi = 0;
  if (seed) {
    constexpr uint32_t D = 1u << 20;  // +-12% of a float's magnitude
    const uint32_t t0 = seed > D ? seed - D : 1u;
    const int c0 = count_ge<NR>(key, t0);
    if (c0 >= kTop) { lo = t0; c_lo = c0; } else { hi = t0; c_hi = c0; }
    if (hi == 0 && seed < 0xFFFFFFFFu - D) {
      const uint32_t t1 = seed + D;
      const int c1 = count_ge<NR>(key, t1);
      if (c1 >= kTop) { lo = t1; c_lo = c1; } else { hi = t1; c_hi = c1; }
    }
  }
  while (c_lo - c_hi > kTop && hi - lo != 1u) {
    // hi - lo wraps to the right width when hi stands for 2^32, except for lo == 0
    const uint32_t mid = (lo == 0 && hi == 0) ? 0x80000000u : lo + ((hi - lo) >> 1);
    const int c = count_ge<NR>(key, mid);
    if (c >= kTop) { lo = mid; c_lo = c; } else { hi = mid; c_hi = c; }
  }
  // one pass: candidates >= hi go to out[0, c_hi), candidates in [lo, hi) to the band
  int base_out = 0, base_band = 0;
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const bool ge_lo = key[j] >= lo;
    const bool ge_hi = hi != 0 && key[j] >= hi;
    const unsigned long long m_lo = __ballot(ge_lo);
    const unsigned long long m_hi = __ballot(ge_hi);
    const unsigned long long m_band = m_lo & ~m_hi;
    const entry_t e = pack_entry(key[j], key[j] ? idx[j] : -1);
    if (ge_hi) {
      out[base_out + prefix_in(m_hi)] = e;
    } else if (ge_lo) {
      const int pos = base_band + prefix_in(m_band);
      if (pos < kTop) band[pos] = e;
    }
    base_out += __popcll(m_hi);
    base_band += __popcll(m_band);
  }
  // the band: two entries per lane, `need` of them are wanted
  const int need = kTop - c_hi;
  const int nband = base_band < kTop ? base_band : kTop;
  const entry_t b0 = lane < nband ? band[lane] : 0ull;
  const entry_t b1 = lane + 64 < nband ? band[lane + 64] : 0ull;
  const uint32_t k0 = lane < nband ? entry_key(b0) : 0u;
  const uint32_t k1 = lane + 64 < nband ? entry_key(b1) : 0u;
  const bool v0 = lane < nband, v1 = lane + 64 < nband;
  // exact threshold inside the band: largest t with count(band >= t) >= need
  int cb_lo = base_band;  // everything in the band is >= lo
  while (cb_lo != need && hi - lo != 1u) {
    const uint32_t mid = (lo == 0 && hi == 0) ? 0x80000000u : lo + ((hi - lo) >> 1);
    const int c = __popcll(__ballot(v0 && k0 >= mid)) + __popcll(__ballot(v1 && k1 >= mid));
    if (c >= need) { lo = mid; cb_lo = c; } else { hi = mid; }
  }
  // winners: every band entry >= lo when that is exactly `need` of them,
  // otherwise (ties at lo) those above lo and then the first ones equal to lo
  const bool g0 = v0 && (cb_lo == need ? k0 >= lo : k0 > lo);
  const bool g1 = v1 && (cb_lo == need ? k1 >= lo : k1 > lo);
  const unsigned long long mg0 = __ballot(g0), mg1 = __ballot(g1);
  const int ng0 = __popcll(mg0), ng = ng0 + __popcll(mg1);
  if (g0) out[c_hi + prefix_in(mg0)] = b0;
  if (g1) out[c_hi + ng0 + prefix_in(mg1)] = b1;
  if (cb_lo != need) {
    const bool q0 = v0 && k0 == lo, q1 = v1 && k1 == lo;
    const unsigned long long mq0 = __ballot(q0), mq1 = __ballot(q1);
    const int p0 = c_hi + ng + prefix_in(mq0);
    const int p1 = c_hi + ng + __popcll(mq0) + prefix_in(mq1);
    if (q0 && p0 < kTop) out[p0] = b0;
    if (q1 && p1 < kTop) out[p1] = b1;
  }
  seed = lo;
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

template <int SIZE, int STRIDE>
__device__ __forceinline__ void bitonic_stage(entry_t& e0, entry_t& e1) {
  const int lane = threadIdx.x & 63;
  if constexpr (STRIDE == 64) {
    const entry_t hi = e0 > e1 ? e0 : e1;
    const entry_t lo = e0 > e1 ? e1 : e0;
    e0 = hi;
    e1 = lo;
  } else {
    // descending blocks keep the larger entry in the lower position
    const bool lower = (lane & STRIDE) == 0;
    const bool desc0 = SIZE == 128 ? true : ((lane & SIZE) == 0);
    const bool desc1 = SIZE == 128 ? true : (SIZE == 64 ? false : desc0);
    const entry_t o0 =
        (static_cast<entry_t>(lane_xor<STRIDE>(static_cast<uint32_t>(e0 >> 32))) << 32) |
        lane_xor<STRIDE>(static_cast<uint32_t>(e0));
    const entry_t o1 =
        (static_cast<entry_t>(lane_xor<STRIDE>(static_cast<uint32_t>(e1 >> 32))) << 32) |
        lane_xor<STRIDE>(static_cast<uint32_t>(e1));
    e0 = ((o0 > e0) == (lower == desc0)) ? o0 : e0;
    e1 = ((o1 > e1) == (lower == desc1)) ? o1 : e1;
  }
}

template <int SIZE, int STRIDE>
__device__ __forceinline__ void bitonic_merge(entry_t& e0, entry_t& e1) {
  bitonic_stage<SIZE, STRIDE>(e0, e1);
  if constexpr (STRIDE > 1) bitonic_merge<SIZE, STRIDE / 2>(e0, e1);
}

// Sorts 128 entries held two per lane (e0 at position lane, e1 at position
// lane + 64) into descending order of position.  The network is the one of
// the reference (bitonic_sort_128, kernels/topkbmm.cu:98-139) with the final
// merge turned to descending order.
__device__ __forceinline__ void bitonic128_desc(entry_t& e0, entry_t& e1) {
  bitonic_merge<2, 1>(e0, e1);
  bitonic_merge<4, 2>(e0, e1);
  bitonic_merge<8, 4>(e0, e1);
  bitonic_merge<16, 8>(e0, e1);
  bitonic_merge<32, 16>(e0, e1);
  bitonic_merge<64, 32>(e0, e1);
  bitonic_merge<128, 64>(e0, e1);
}

// Sorts the 128-entry list and writes its first k entries as fp32 values and
// int64 indices.
__device__ __forceinline__ void sort_and_store(const entry_t* list, float* values,
                                               long long* indices, int k) {
  const int lane = threadIdx.x & 63;
  entry_t e0 = list[lane];
  entry_t e1 = list[lane + 64];
  bitonic128_desc(e0, e1);
  if (lane < k) {
    values[lane] = key2f(entry_key(e0));
    indices[lane] = entry_idx(e0);
  }
  if (lane + 64 < k) {
    values[lane + 64] = key2f(entry_key(e1));
    indices[lane + 64] = entry_idx(e1);
  }
}

}  // namespace cmk
