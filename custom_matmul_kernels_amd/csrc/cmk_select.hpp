// Wave-level exact top-128 selection and a wave64 bitonic sorter.
//
// A wave holds NR*64 candidates of one output row, NR per lane, as fp32 bit
// patterns; their order is that of 32-bit order-preserving keys.  select128()
// finds the 128 largest in three moves:
//   1. Bracket the key of the 128th largest, [lo, hi), by counting candidates
//      >= t with wave ballots.  The bracket starts just below the previous
//      row's answer (rows of one strip are statistically alike), which is
//      nearly always right at once; otherwise it is bisected until at most 256
//      candidates lie at or above lo.
//   2. The ballots of the last count compact those candidates into a list in
//      LDS, as 64-bit (raw, ~index) entries.
//   3. The list, now four entries per lane and turned into keys, is narrowed
//      four-fold per round to the exact threshold and the 128 winners are
//      written to the output list as (key, ~index) entries.
// The output list is unordered; bitonic128_desc() orders it once, at the very
// end, so that values descend and equal values come out by ascending index.
// insert128() is the short route for a later chunk of a long axis, when the
// list is full and few candidates beat its smallest entry.
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
__device__ __forceinline__ uint32_t raw2key(uint32_t u) {
  return u ^ (static_cast<uint32_t>(static_cast<int32_t>(u) >> 31) | 0x80000000u);
}
__device__ __forceinline__ uint32_t f2key(float f) { return raw2key(__float_as_uint(f)); }
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

// Candidates travel as raw fp32 bit patterns ("raw") until they reach the
// candidate list; comparing raws against a threshold key needs no key per
// candidate:  key(raw) >= t  <=>  (int)raw >= (int)(t ^ 0x80000000)  for t in the
// upper half of the key space, and  raw <= ~t  (unsigned) below it.  raw
// 0xFFFFFFFF has key 0 and stands for "no candidate".
constexpr uint32_t kNoCandidate = 0xFFFFFFFFu;
__device__ __forceinline__ uint32_t key2raw(uint32_t k) {
  return (k & 0x80000000u) ? (k ^ 0x80000000u) : ~k;
}

// m[j] = lanes whose raw[j] has a key >= t; returns how many there are.
template <int NR>
__device__ __forceinline__ int masks_ge(const uint32_t (&raw)[NR], uint32_t t,
                                        unsigned long long (&m)[NR]) {
  int c = 0;
  t = __builtin_amdgcn_readfirstlane(t);  // the same in every lane: the ballots stay scalar
  if (t & 0x80000000u) {
    const int b = static_cast<int>(t ^ 0x80000000u);
#pragma unroll
    for (int j = 0; j < NR; ++j) m[j] = __ballot(static_cast<int>(raw[j]) >= b);
  } else {
    const uint32_t b = ~t;
#pragma unroll
    for (int j = 0; j < NR; ++j) m[j] = __ballot(raw[j] <= b);
  }
#pragma unroll
  for (int j = 0; j < NR; ++j) c += __popcll(m[j]);
  return c;
}

// Selects the 128 candidates with the largest keys among raw[0..NR) of all 64
// lanes and writes them as entries to out[0..128) (LDS owned by this wave).
// `cand` is kCand entries of wave-private LDS scratch.  `seed` carries the
// threshold key from one call to the next (0 = none); idx_of(j) is the index of
// candidate raw[j] of this lane.  Fewer than 128 real candidates leave empty
// entries.
//
// Ties at the threshold go to the lowest indices, by this invariant: candidates
// are always taken in the order reg_order(0), reg_order(1), ... (lanes ascending
// within a register), callers hand over candidates whose indices ascend in that
// order among equal keys, and the output keeps equal keys in the order they were
// taken.  With NR == 18 registers 16 and 17 are a running list (the output of an
// earlier call, over lower indices) and are taken first.
template <int NR>
__device__ __forceinline__ constexpr int reg_order(int pos) {
  return NR == 18 ? (pos < 2 ? 16 + pos : pos - 2) : pos;
}

template <int NR, class IdxOf>
__device__ __forceinline__ void select128(const uint32_t (&raw)[NR], IdxOf&& idx_of,
                                          uint32_t& seed, entry_t* cand, entry_t* out) {
  const int lane = threadIdx.x & 63;
  constexpr uint32_t D = 1u << 21;  // a quarter of a binade: 12 to 25% of a float's magnitude
  // bracket: count(>= lo) >= 128 > count(>= hi); hi == 0 stands for 2^32.
  // m[] always holds the masks of the last threshold counted.
  unsigned long long m[NR];
  uint32_t lo = 0, hi = 0, counted = 0xFFFFFFFFu;
  int c_lo = NR * 64;
  seed = __builtin_amdgcn_readfirstlane(seed);
  if (seed) {
    // walk down from the seed, in growing steps, until at least 128 candidates
    // lie at or above; the first step nearly always does it
    uint32_t t = seed, step = D;
    while (t > step) {
      t -= step;
      const int c = masks_ge(raw, t, m);
      counted = t;
      if (c >= kTop) { lo = t; c_lo = c; break; }
      hi = t;
      if (step < (1u << 29)) step <<= 2;
    }
  }
  while (c_lo > kCand && hi - lo != 1u) {
    const uint32_t mid = bracket_mid(lo, hi);
    const int c = masks_ge(raw, mid, m);
    counted = mid;
    if (c >= kTop) { lo = mid; c_lo = c; } else { hi = mid; }
  }

  if (c_lo <= kCand) {
    if (counted != lo) masks_ge(raw, lo, m);
    // every candidate with a key >= lo goes to the candidate list, registers in
    // reg_order and lanes ascending, as (raw, ~index); there are at least 128 and
    // at most 256
    int base[NR];
    base[reg_order<NR>(0)] = 0;
#pragma unroll
    for (int p = 1; p < NR; ++p)
      base[reg_order<NR>(p)] = base[reg_order<NR>(p - 1)] + __popcll(m[reg_order<NR>(p - 1)]);
#pragma unroll
    for (int j = 0; j < NR; ++j) {
      const int pos = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(m[j] >> 32),
                                                __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(m[j]), base[j]));
      if (__builtin_amdgcn_inverse_ballot_w64(m[j])) cand[pos] = pack_entry(raw[j], idx_of(j));
    }
    // four entries per lane, now with keys
    entry_t e[4];
    uint32_t k[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const bool valid = lane + 64 * q < c_lo;
      const entry_t r = cand[lane + 64 * q];
      k[q] = valid ? raw2key(entry_key(r)) : 0u;
      e[q] = k[q] ? (static_cast<entry_t>(k[q]) << 32) | static_cast<uint32_t>(r) : 0ull;
    }
    auto count4 = [&](uint32_t t) {
      int c = 0;
#pragma unroll
      for (int q = 0; q < 4; ++q) c += __popcll(__ballot(k[q] >= t));
      return c;
    };
    int n_lo = c_lo;
    // the upper end of the bracket, if still open, is found by walking up from
    // the seed in the same way
    if (hi == 0 && seed) {
      uint32_t t = seed > lo ? seed : lo, step = D;
      while (t < 0xFFFFFFFFu - step) {
        t += step;
        const int c = count4(t);
        if (c < kTop) { hi = t; break; }
        lo = t;
        n_lo = c;
        if (step < (1u << 29)) step <<= 2;
      }
    }
    // narrow the bracket four-fold per round to the exact threshold: the largest
    // t with count(>= t) >= 128; stop early when a count is exactly 128
    while (n_lo != kTop && hi - lo != 1u) {
      const uint32_t w = hi - lo;
      uint32_t q = w ? w >> 2 : 0x40000000u;
      if (q == 0) q = 1;
      uint32_t t1 = lo + q, t2 = t1 + q, t3 = t2 + q;
      if (t2 < t1) t2 = 0xFFFFFFFFu;
      if (t3 < t2) t3 = 0xFFFFFFFFu;
      int c1 = 0, c2 = 0, c3 = 0;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        c1 += __popcll(__ballot(k[r] >= t1));
        c2 += __popcll(__ballot(k[r] >= t2));
        c3 += __popcll(__ballot(k[r] >= t3));
      }
      if (c3 >= kTop) { lo = t3; n_lo = c3; }
      else if (c2 >= kTop) { lo = t2; n_lo = c2; hi = t3; }
      else if (c1 >= kTop) { lo = t1; n_lo = c1; hi = t2; }
      else { hi = t1; }
    }
    // winners: all entries >= lo if that is exactly 128, otherwise (ties at lo)
    // those above lo and then the first ones equal to lo
    const bool exact = n_lo == kTop;
    unsigned long long mg[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) mg[q] = __ballot(exact ? k[q] >= lo : k[q] > lo);
    int pos_gt = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      if (__builtin_amdgcn_inverse_ballot_w64(mg[q])) out[pos_gt + prefix_in(mg[q])] = e[q];
      pos_gt += __popcll(mg[q]);
    }
    if (!exact) {
      int pos_eq = pos_gt;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const bool tie = k[q] == lo;
        const unsigned long long mq = __ballot(tie);
        const int p = pos_eq + prefix_in(mq);
        if (tie && p < kTop) out[p] = e[q];
        pos_eq += __popcll(mq);
      }
    }
  } else {
    // more than 256 candidates share the key lo (hi == lo + 1): take every
    // candidate above lo, then the first ones equal to lo.  `out` may be the list
    // that registers 16 and 17 were read from; it is only written after every
    // lane holds its candidates in registers, which the ballots below imply.
    int base = 0;
#pragma unroll
    for (int p = 0; p < NR; ++p) {
      const int j = reg_order<NR>(p);
      const uint32_t key = raw2key(raw[j]);
      const bool g = key > lo;
      const unsigned long long mm = __ballot(g);
      if (g) out[base + prefix_in(mm)] = pack_entry(key, idx_of(j));
      base += __popcll(mm);
    }
#pragma unroll
    for (int p = 0; p < NR; ++p) {
      const int j = reg_order<NR>(p);
      const bool tie = raw2key(raw[j]) == lo;
      const unsigned long long mm = __ballot(tie);
      const int q = base + prefix_in(mm);
      if (tie && q < kTop) out[q] = lo ? pack_entry(lo, idx_of(j)) : 0ull;
      base += __popcll(mm);
    }
  }
  seed = lo;
}

// Folds the candidates raw[0..16) of all lanes into a FULL running list of 128
// entries whose smallest key is `thr` (> 0), by a shorter route than
// select128<18>: only candidates with a key above thr can enter (an equal key
// loses the tie to the list, whose indices are lower), late chunks of a long
// axis bring few of those, and the new threshold lies just above the old one.
// The newcomers are compacted into `cand` (at most one per lane), the threshold
// is searched upwards from thr over three entries per lane, and the list is
// rewritten as its survivors followed by the surviving newcomers, both in their
// old order, which keeps equal keys in ascending index order.  Returns false,
// having changed nothing, when more than 64 candidates beat thr.
template <class IdxOf>
__device__ __forceinline__ bool insert128(const uint32_t (&raw)[16], IdxOf&& idx_of, uint32_t& thr,
                                          entry_t* cand, entry_t* list) {
  const int lane = threadIdx.x & 63;
  thr = __builtin_amdgcn_readfirstlane(thr);
  if (thr == 0xFFFFFFFFu) return true;  // nothing ranks above the list's smallest entry
  unsigned long long m[16];
  const int c = masks_ge(raw, thr + 1u, m);
  if (c == 0) return true;
  if (c > 64) return false;
  int base = 0;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    if (m[j]) {
      const int pos = __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(m[j] >> 32),
                                                __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(m[j]), base));
      if (__builtin_amdgcn_inverse_ballot_w64(m[j])) cand[pos] = pack_entry(raw[j], idx_of(j));
      base += __popcll(m[j]);
    }
  }
  entry_t e[3];
  uint32_t k[3];
  e[0] = list[lane];
  e[1] = list[lane + 64];
  k[0] = entry_key(e[0]);
  k[1] = entry_key(e[1]);
  {
    const entry_t r = cand[lane];
    k[2] = lane < c ? raw2key(entry_key(r)) : 0u;
    e[2] = k[2] ? (static_cast<entry_t>(k[2]) << 32) | static_cast<uint32_t>(r) : 0ull;
  }
  auto count3 = [&](uint32_t t) {
    int n = 0;
#pragma unroll
    for (int q = 0; q < 3; ++q) n += __popcll(__ballot(k[q] >= t));
    return n;
  };
  // bracket [lo, hi): count(>= lo) >= 128 > count(>= hi); hi == 0 stands for 2^32
  uint32_t lo = thr, hi = 0;
  int n_lo = kTop + c;
  {
    uint32_t t = lo, step = 1u << 13;
    while (t < 0xFFFFFFFFu - step) {
      t += step;
      const int n = count3(t);
      if (n < kTop) { hi = t; break; }
      lo = t;
      n_lo = n;
      if (n == kTop) break;
      if (step < (1u << 29)) step <<= 2;
    }
  }
  while (n_lo != kTop && hi - lo != 1u) {
    const uint32_t w = hi - lo;  // 2^32 - lo when hi == 0
    uint32_t q = w >> 2;
    if (q == 0) q = 1;
    uint32_t t1 = lo + q, t2 = t1 + q, t3 = t2 + q;
    if (t2 < t1) t2 = 0xFFFFFFFFu;
    if (t3 < t2) t3 = 0xFFFFFFFFu;
    int c1 = 0, c2 = 0, c3 = 0;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      c1 += __popcll(__ballot(k[r] >= t1));
      c2 += __popcll(__ballot(k[r] >= t2));
      c3 += __popcll(__ballot(k[r] >= t3));
    }
    if (c3 >= kTop) { lo = t3; n_lo = c3; }
    else if (c2 >= kTop) { lo = t2; n_lo = c2; hi = t3; }
    else if (c1 >= kTop) { lo = t1; n_lo = c1; hi = t2; }
    else { hi = t1; }
  }
  // survivors: every entry >= lo if those are exactly 128, otherwise those above
  // lo and then the first ones equal to lo.  Every lane holds its entries in
  // registers by now (the ballots above needed them), so the list can be
  // rewritten in place.
  const bool exact = n_lo == kTop;
  int pos = 0;
#pragma unroll
  for (int q = 0; q < 3; ++q) {
    const bool g = exact ? k[q] >= lo : k[q] > lo;
    const unsigned long long mq = __ballot(g);
    if (g) list[pos + prefix_in(mq)] = e[q];
    pos += __popcll(mq);
  }
  if (!exact) {
#pragma unroll
    for (int q = 0; q < 3; ++q) {
      const bool tie = k[q] == lo;
      const unsigned long long mq = __ballot(tie);
      const int p = pos + prefix_in(mq);
      if (tie && p < kTop) list[p] = e[q];
      pos += __popcll(mq);
    }
  }
  thr = lo;
  return true;
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

// The same network on bare keys.
template <int SIZE, int STRIDE, int R>
__device__ __forceinline__ void key_stage(uint32_t (&k0)[R], uint32_t (&k1)[R]) {
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if constexpr (STRIDE == 64) {
      const uint32_t hi = max(k0[r], k1[r]);
      const uint32_t lo = min(k0[r], k1[r]);
      k0[r] = hi;
      k1[r] = lo;
    } else {
      const uint32_t o0 = lane_xor<STRIDE>(k0[r]);
      const uint32_t o1 = lane_xor<STRIDE>(k1[r]);
      constexpr unsigned long long km0 = keep_max_mask<SIZE, STRIDE, 0>();
      constexpr unsigned long long km1 = keep_max_mask<SIZE, STRIDE, 1>();
      const bool t0 = __builtin_amdgcn_inverse_ballot_w64(__ballot(o0 > k0[r]) ^ ~km0);
      const bool t1 = __builtin_amdgcn_inverse_ballot_w64(__ballot(o1 > k1[r]) ^ ~km1);
      k0[r] = t0 ? o0 : k0[r];
      k1[r] = t1 ? o1 : k1[r];
    }
  }
}
template <int SIZE, int STRIDE, int R>
__device__ __forceinline__ void key_merge(uint32_t (&k0)[R], uint32_t (&k1)[R]) {
  key_stage<SIZE, STRIDE, R>(k0, k1);
  if constexpr (STRIDE > 1) key_merge<SIZE, STRIDE / 2, R>(k0, k1);
}

// Orders R 128-entry lists and writes the first k entries of each as fp32
// values and int64 indices; a null values[r] skips the store of that row.  The
// lists are left as they are; scratch[r] is 128 words of LDS owned by this wave.
//
// The network moves 32-bit words, half the work of moving entries: the upper 25
// bits of the key with the entry's slot in the list below them.  The entries
// are then fetched by slot, now in order except where neighbours agree in those
// 25 bits; one in-lane and one cross-lane compare-exchange of whole entries
// repair runs of two.  A final check of all neighbours sends the rare list
// with a longer run through the full network on entries.  Equal values come
// out by ascending index.
// results are stored through pointers that name global memory (a generic
// pointer would give flat stores)
typedef float __attribute__((address_space(1))) * global_f32_out;
typedef long long __attribute__((address_space(1))) * global_i64_out;

template <int R>
__device__ __forceinline__ void sort_and_store(const entry_t* const* list, uint32_t* const* scratch,
                                               float* const* values, long long* const* indices,
                                               int k) {
  const int lane = threadIdx.x & 63;
  uint32_t w0[R], w1[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    w0[r] = (entry_key(list[r][lane]) & ~0x7Fu) | lane;
    w1[r] = (entry_key(list[r][lane + 64]) & ~0x7Fu) | (lane + 64);
  }
  key_merge<2, 1, R>(w0, w1);
  key_merge<4, 2, R>(w0, w1);
  key_merge<8, 4, R>(w0, w1);
  key_merge<16, 8, R>(w0, w1);
  key_merge<32, 16, R>(w0, w1);
  key_merge<64, 32, R>(w0, w1);
  key_merge<128, 64, R>(w0, w1);
  // re-deal: lane l takes positions 2l and 2l+1, and fetches their entries
  entry_t a[R], b[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    scratch[r][lane] = w0[r];
    scratch[r][lane + 64] = w1[r];
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t sa = scratch[r][2 * lane], sb = scratch[r][2 * lane + 1];
    a[r] = list[r][sa & 0x7Fu];
    b[r] = list[r][sb & 0x7Fu];
  }
  const int up = ((lane + 1) & 63) << 2, down = ((lane + 63) & 63) << 2;
  auto from = [&](int sel, entry_t v) {
    return (static_cast<entry_t>(__builtin_amdgcn_ds_bpermute(sel, static_cast<uint32_t>(v >> 32))) << 32) |
           static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(sel, static_cast<uint32_t>(v)));
  };
  bool bad = false;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    // positions (2l, 2l+1)
    entry_t hi = a[r] > b[r] ? a[r] : b[r];
    entry_t lo = a[r] > b[r] ? b[r] : a[r];
    a[r] = hi;
    b[r] = lo;
    // positions (2l+1, 2l+2): b of this lane against a of the next
    const entry_t na = from(up, a[r]);    // a of lane + 1
    const entry_t pb = from(down, b[r]);  // b of lane - 1
    const entry_t b2 = (lane < 63 && na > b[r]) ? na : b[r];
    const entry_t a2 = (lane > 0 && a[r] > pb) ? pb : a[r];
    a[r] = a2;
    b[r] = b2;
    // all neighbours in order?
    const entry_t na2 = from(up, a[r]);
    bad |= b[r] > a[r] || (lane < 63 && na2 > b[r]);
  }
  if (__ballot(bad) != 0ull) {
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
      global_f32_out gv = (global_f32_out)values[r];
      global_i64_out gi = (global_i64_out)indices[r];
      if (lane < k) {
        gv[lane] = key2f(entry_key(e0[r]));
        gi[lane] = entry_idx(e0[r]);
      }
      if (lane + 64 < k) {
        gv[lane + 64] = key2f(entry_key(e1[r]));
        gi[lane + 64] = entry_idx(e1[r]);
      }
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (!values[r]) continue;
    global_f32_out gv = (global_f32_out)values[r];
    global_i64_out gi = (global_i64_out)indices[r];
    if (2 * lane < k) {
      gv[2 * lane] = key2f(entry_key(a[r]));
      gi[2 * lane] = entry_idx(a[r]);
    }
    if (2 * lane + 1 < k) {
      gv[2 * lane + 1] = key2f(entry_key(b[r]));
      gi[2 * lane + 1] = entry_idx(b[r]);
    }
  }
}

// sort_and_store<2> as a real function: its many mask constants and fragments
// then live in the callee's registers only, instead of crowding the caller's
// scalar registers for the whole kernel.  LDS pointers travel as such.
typedef const entry_t __attribute__((address_space(3))) * lds_entry_ptr;
typedef uint32_t __attribute__((address_space(3))) * lds_u32_ptr;
__device__ __attribute__((noinline)) inline void sort_and_store_pair(lds_entry_ptr l0, lds_entry_ptr l1,
                                                                     lds_u32_ptr scratch, float* v0,
                                                                     float* v1, long long* i0,
                                                                     long long* i1, int k) {
  const entry_t* const lists[2] = {(const entry_t*)l0, (const entry_t*)l1};
  uint32_t* const sc[2] = {(uint32_t*)scratch, (uint32_t*)scratch + kTop};
  float* const cv[2] = {v0, v1};
  long long* const ci[2] = {i0, i1};
  sort_and_store<2>(lists, sc, cv, ci, k);
}

}  // namespace cmk
