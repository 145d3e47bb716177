// Wave-level exact top-128 selection and a wave64 bitonic sorter.
//
// A wave holds NR*64 candidates of one output row, NR per lane, as 32-bit
// order-preserving keys plus 32-bit indices.  select128() finds the 128 largest
// in three moves:
//   1. Bracket the key of the 128th largest, [lo, hi), by counting candidates
//      >= t with wave ballots.  The bracket starts around the previous row's
//      answer (rows of one strip are statistically alike) and is bisected until
//      at most 256 candidates lie at or above lo.
//   2. One pass over the registers compacts those candidates into a list in
//      LDS, as 64-bit (key, ~index) entries.
//   3. The list, now four entries per lane, is bisected to the exact threshold
//      and the 128 winners are written to the output list.
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

constexpr int kCand = 256;  // capacity of the candidate list select128() works in

// Selects the 128 largest keys among key[0..NR) of all 64 lanes and writes them
// as entries to out[0..128) (LDS owned by this wave).  `cand` is kCand entries of
// wave-private LDS scratch.  `seed` carries the threshold key from one call to
// the next (0 = none); idx_of(j) is the index of candidate key[j] of this lane.
// Ties at the threshold: earliest (register, lane) position first.  Fewer than
// 128 real candidates leave empty entries.
template <int NR, class IdxOf>
__device__ __forceinline__ void select128(const uint32_t (&key)[NR], IdxOf&& idx_of,
                                          uint32_t& seed, entry_t* cand, entry_t* out) {
  const int lane = threadIdx.x & 63;
  auto count_ge = [&](uint32_t t) {
    int c = 0;
#pragma unroll
    for (int j = 0; j < NR; ++j) c += __popcll(__ballot(key[j] >= t));
    return c;
  };
  // bracket: count(>= lo) >= 128 > count(>= hi); hi == 0 stands for 2^32
  uint32_t lo = 0, hi = 0;
  int c_lo = NR * 64, c_hi = 0;
  if (seed) {
    constexpr uint32_t D = 1u << 20;  // +-12% of a float's magnitude
    const uint32_t t0 = seed > D ? seed - D : 1u;
    const int c0 = count_ge(t0);
    if (c0 >= kTop) { lo = t0; c_lo = c0; } else { hi = t0; c_hi = c0; }
    if (hi == 0 && seed < 0xFFFFFFFFu - D) {
      const uint32_t t1 = seed + D;
      const int c1 = count_ge(t1);
      if (c1 >= kTop) { lo = t1; c_lo = c1; } else { hi = t1; c_hi = c1; }
    }
  }
  while (c_lo > kCand && hi - lo != 1u) {
    const uint32_t mid = bracket_mid(lo, hi);
    const int c = count_ge(mid);
    if (c >= kTop) { lo = mid; c_lo = c; } else { hi = mid; c_hi = c; }
  }

  if (c_lo <= kCand) {
    // one pass: every candidate >= lo goes to the candidate list, in (register,
    // lane) order; there are at least 128 and at most 256 of them
    int base = 0;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const bool ge = key[j] >= lo;
      const unsigned long long m = __ballot(ge);
      const int pos = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(m >> 32),
                                                __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(m), base));
      if (ge) cand[pos] = pack_entry(key[j], idx_of(j));
      base += __popcll(m);
    }
    // four entries per lane; bisect to the exact threshold: the largest t with
    // count(>= t) >= 128, stopping early when the count is exactly 128
    entry_t e[4];
    uint32_t k[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const bool valid = lane + 64 * m < c_lo;
      e[m] = valid ? cand[lane + 64 * m] : 0ull;
      k[m] = entry_key(e[m]);
      if (k[m] == 0u) e[m] = 0ull;  // "no candidate" carries index -1
    }
    int n_lo = c_lo;
    while (n_lo != kTop && hi - lo != 1u) {
      const uint32_t mid = bracket_mid(lo, hi);
      int c = 0;
#pragma unroll
      for (int m = 0; m < 4; ++m) c += __popcll(__ballot(lane + 64 * m < c_lo && k[m] >= mid));
      if (c >= kTop) { lo = mid; n_lo = c; } else { hi = mid; }
    }
    // winners: all entries >= lo if that is exactly 128, otherwise (ties at lo)
    // those above lo and then the first ones equal to lo
    const bool exact = n_lo == kTop;
    int pos_gt = 0;
    unsigned long long mg[4];
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const bool valid = lane + 64 * m < c_lo;
      const bool g = valid && (exact ? k[m] >= lo : k[m] > lo);
      mg[m] = __ballot(g);
      if (g) out[pos_gt + prefix_in(mg[m])] = e[m];
      pos_gt += __popcll(mg[m]);
    }
    if (!exact) {
      int pos_eq = pos_gt;
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        const bool q = lane + 64 * m < c_lo && k[m] == lo;
        const unsigned long long mq = __ballot(q);
        const int p = pos_eq + prefix_in(mq);
        if (q && p < kTop) out[p] = e[m];
        pos_eq += __popcll(mq);
      }
    }
  } else {
    // more than 256 candidates share the key lo (hi == lo + 1): take every
    // candidate above lo, then the first ones equal to lo
    int base = 0;
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const bool g = key[j] > lo;
      const unsigned long long m = __ballot(g);
      if (g) out[base + prefix_in(m)] = pack_entry(key[j], idx_of(j));
      base += __popcll(m);
    }
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const bool q = key[j] == lo;
      const unsigned long long m = __ballot(q);
      const int p = base + prefix_in(m);
      if (q && p < kTop) out[p] = lo ? pack_entry(lo, idx_of(j)) : 0ull;
      base += __popcll(m);
    }
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
