// Per-workgroup exclusive prefix sums over the rows of a small grid_thw table, kept in LDS.
#pragma once
#include "common.h"

namespace wx {

constexpr int kMaxGrids = 4096;

__device__ __forceinline__ void load_thw(const void* grid_thw, int grid_type, int64_t g, int64_t& t, int64_t& h,
                                         int64_t& w) {
  t = load_index(grid_thw, grid_type, 3 * g);
  h = load_index(grid_thw, grid_type, 3 * g + 1);
  w = load_index(grid_thw, grid_type, 3 * g + 2);
}

// In-place exclusive scan of s[0..n) by wavefront 0 (64 entries per step with a running carry);
// s[n] receives the total.  Call from all threads of the block; ends with a barrier.
__device__ __forceinline__ void lds_exclusive_scan(int32_t* s, int n) {
  __syncthreads();
  if (threadIdx.x < kWave) {
    const int lane = lane_id();
    int32_t carry = 0;
    for (int base = 0; base < n; base += kWave) {
      const int i = base + lane;
      const int32_t v = i < n ? s[i] : 0;
      int32_t incl = v;
#pragma unroll
      for (int d = 1; d < kWave; d <<= 1) {
        const int32_t up = __shfl_up(incl, d);
        if (lane >= d) incl += up;
      }
      if (i < n) s[i] = carry + incl - v;
      carry += __shfl(incl, kWave - 1);
    }
    if (lane == 0) s[n] = carry;
  }
  __syncthreads();
}

// Largest g in [0, n) with prefix[g] <= x, given prefix[] non-decreasing and prefix[0] == 0.  Rows with a
// zero count share their prefix with the next row; the search lands on the last of them, which is the
// row that actually owns x.
__device__ __forceinline__ int find_owner(const int32_t* prefix, int n, int32_t x) {
  int lo = 0, hi = n - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (prefix[mid] <= x) lo = mid; else hi = mid - 1;
  }
  return lo;
}

}  // namespace wx
