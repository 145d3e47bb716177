// Wave-level exact top-128 selection and a wave64 bitonic sorter.
//
// A wave holds NR*64 candidates of one output row, NR per lane, as 32-bit
// order-preserving keys plus 32-bit indices.  select128() finds the key of the
// 128th largest candidate by bisecting the key space one bit at a time (each
// step counts candidates with wave ballots), then compacts the winners into a
// 128-entry list in LDS.  The list is unordered; bitonic128_desc() orders it
// once, at the very end, as 64-bit (key, ~index) words so that equal values
// come out by ascending index.
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

// Selects the 128 largest keys among key[0..NR) of all 64 lanes (ties at the
// threshold: earliest (register, lane) position first) and writes them with
// their indices to out_key / out_idx (128 entries each, any memory the wave
// may write).  Fewer than 128 real candidates leave (0, -1) entries.
template <int NR>
__device__ __forceinline__ void select128(const uint32_t (&key)[NR], const int (&idx)[NR],
                                          uint32_t* out_key, int* out_idx) {
  const int lane = threadIdx.x & 63;
  uint32_t t = 0;
  for (int bit = 31; bit >= 0; --bit) {
    const uint32_t t2 = t | (1u << bit);
    int cnt = 0;
#pragma unroll
    for (int j = 0; j < NR; ++j) cnt += __popcll(__ballot(key[j] >= t2));
    if (cnt >= kTop) t = t2;
  }
  int ngt = 0;
#pragma unroll
  for (int j = 0; j < NR; ++j) ngt += __popcll(__ballot(key[j] > t));
  const unsigned long long below = (1ull << lane) - 1ull;
  int base_gt = 0, base_eq = ngt;
#pragma unroll
  for (int j = 0; j < NR; ++j) {
    const bool gt = key[j] > t;
    const bool eq = key[j] == t;
    const unsigned long long mgt = __ballot(gt);
    const unsigned long long meq = __ballot(eq);
    if (gt) {
      const int pos = base_gt + __popcll(mgt & below);
      out_key[pos] = key[j];
      out_idx[pos] = idx[j];
    } else if (eq) {
      const int pos = base_eq + __popcll(meq & below);
      if (pos < kTop) {
        out_key[pos] = t;
        out_idx[pos] = t ? idx[j] : -1;
      }
    }
    base_gt += __popcll(mgt);
    base_eq += __popcll(meq);
  }
}

__device__ __forceinline__ unsigned long long pack_entry(uint32_t key, int idx) {
  return (static_cast<unsigned long long>(key) << 32) | static_cast<uint32_t>(~idx);
}
__device__ __forceinline__ uint32_t entry_key(unsigned long long e) {
  return static_cast<uint32_t>(e >> 32);
}
__device__ __forceinline__ int entry_idx(unsigned long long e) {
  return static_cast<int>(~static_cast<uint32_t>(e));
}

// Sorts 128 packed entries held two per lane (e0 at position lane, e1 at
// position lane + 64) into descending order of position.
__device__ __forceinline__ void bitonic128_desc(unsigned long long& e0, unsigned long long& e1) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int size = 2; size <= 128; size <<= 1) {
#pragma unroll
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      if (stride == 64) {
        const unsigned long long hi = e0 > e1 ? e0 : e1;
        const unsigned long long lo = e0 > e1 ? e1 : e0;
        e0 = hi;
        e1 = lo;
      } else {
        const bool lower = (lane & stride) == 0;
        const bool desc0 = size == 128 ? true : ((lane & size) == 0);
        const bool desc1 = size == 128 ? true : (((lane + 64) & size) == 0);
        const unsigned long long o0 = __shfl_xor(e0, stride);
        const unsigned long long o1 = __shfl_xor(e1, stride);
        const bool max0 = lower == desc0;
        const bool max1 = lower == desc1;
        e0 = max0 ? (e0 > o0 ? e0 : o0) : (e0 < o0 ? e0 : o0);
        e1 = max1 ? (e1 > o1 ? e1 : o1) : (e1 < o1 ? e1 : o1);
      }
    }
  }
}

// Sorts the 128-entry list (list_key, list_idx) and writes its first k entries
// as fp32 values and int64 indices.
__device__ __forceinline__ void sort_and_store(const uint32_t* list_key, const int* list_idx,
                                               float* values, long long* indices, int k) {
  const int lane = threadIdx.x & 63;
  unsigned long long e0 = pack_entry(list_key[lane], list_idx[lane]);
  unsigned long long e1 = pack_entry(list_key[lane + 64], list_idx[lane + 64]);
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
