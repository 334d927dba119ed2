// Modality-routed token partition, row scatter (permute) and row gather (unpermute) for gfx950.
//
// The partition is a stable counting sort over at most 256 expert bins.  The key stream is cut into
// segments, one per wavefront.  Inside a segment a wavefront walks 64 keys at a time and ranks equal
// keys with ballots (rank = popcount of the equal-key mask below the lane), so order within a bin is
// source order -- the contract of a stable sort -- without any sorting network or atomics.
//   pass 1  partition_count    per-segment histogram  -> hist[segment][256]
//   pass 2  partition_scatter  per-block prefix over hist (bins, then earlier segments), then ranks
// The row movers are pure HBM streams: one wavefront per token row, 16-byte lanes, several rows in flight.
#include <mutex>

#include "common.h"
#include "tiled_layout.h"

namespace wx {
namespace {

constexpr int kBins = 256;
constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * kWave;

__host__ __device__ inline int64_t segment_len(int64_t n) {
  // 512 keys per wavefront until that would need more than 1024 segments
  int64_t seg = 512;
  if (n > seg * 1024) seg = ((n + 1023) / 1024 + 63) / 64 * 64;
  return seg;
}

__device__ __forceinline__ int load_key(const void* ids, int itype, int64_t i, int num_experts, bool& bad) {
  int64_t v = load_index(ids, itype, i);
  if (v < 0) { bad = true; v = 0; }
  if (v >= num_experts) { bad = true; v = num_experts - 1; }
  return static_cast<int>(v);
}

// Calls f(key, mask) once per distinct key among the active lanes; mask = lanes holding that key.
template <typename F>
__device__ __forceinline__ void for_each_key_group(int key, bool active, F f) {
  uint64_t todo = __ballot(active);
  while (todo) {
    const int leader = __ffsll(static_cast<long long>(todo)) - 1;
    const int k = __builtin_amdgcn_readlane(key, leader);
    const uint64_t mask = __ballot(active && key == k);
    f(k, mask);
    todo &= ~mask;
  }
}

__global__ __launch_bounds__(kBlock) void partition_count(const void* __restrict__ ids, int itype, int64_t n,
                                                          int num_experts, int64_t seg_len,
                                                          int32_t* __restrict__ hist, int32_t* status) {
  __shared__ int32_t s_hist[kWavesPerBlock][kBins];
  const int w = threadIdx.x / kWave, lane = lane_id();
  for (int i = lane; i < kBins; i += kWave) s_hist[w][i] = 0;
  const int64_t seg = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + w;
  const int64_t begin = seg * seg_len;
  const int64_t end = begin + seg_len < n ? begin + seg_len : n;
  bool bad = false;
  for (int64_t base = begin; base < end; base += kWave) {
    const int64_t i = base + lane;
    const bool active = i < end;
    const int key = active ? load_key(ids, itype, i, num_experts, bad) : 0;
    for_each_key_group(key, active, [&](int k, uint64_t mask) {
      if (lane == 0) s_hist[w][k] += __popcll(mask);
    });
  }
  if (begin < n) {
    for (int i = lane; i < kBins; i += kWave) hist[seg * kBins + i] = s_hist[w][i];
  }
  if (status != nullptr && __ballot(bad) != 0 && lane == 0) *status = 1;
}

__global__ __launch_bounds__(kBlock) void partition_scatter(
    const void* __restrict__ ids, int itype, int64_t num_tokens, int num_topk, int num_experts,
    int64_t num_out, int64_t seg_len, int64_t num_seg, const int32_t* __restrict__ hist,
    int32_t* __restrict__ row_id_map, int32_t* __restrict__ sorted_row_id,
    int32_t* __restrict__ expert_offsets) {
  __shared__ int32_t s_run[kWavesPerBlock][kBins];  // next free sorted position per (wave, bin)
  __shared__ int32_t s_wave_total[kWavesPerBlock];
  const int tid = threadIdx.x, w = tid / kWave, lane = lane_id();
  const int64_t n = num_tokens * num_topk;
  const int64_t first_seg = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock;

  // bin `tid`: rows of this bin in all segments (total) and in segments before this block (before)
  // (eight independent loads per trip: with one load per trip the loop costs a memory latency per segment)
  int32_t total = 0, before = 0;
  int64_t s = 0;
  for (; s + 8 <= num_seg; s += 8) {
    int32_t v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = hist[(s + u) * kBins + tid];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      total += v[u];
      if (s + u < first_seg) before += v[u];
    }
  }
  for (; s < num_seg; ++s) {
    const int32_t v = hist[s * kBins + tid];
    total += v;
    if (s < first_seg) before += v;
  }
  // exclusive prefix of `total` over the 256 bins: wave scan, then wave totals through LDS
  int32_t incl = total;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int32_t up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  if (lane == kWave - 1) s_wave_total[w] = incl;
  __syncthreads();
  int32_t bin_base = incl - total;
  for (int i = 0; i < w; ++i) bin_base += s_wave_total[i];
  if (blockIdx.x == 0 && expert_offsets != nullptr) {
    if (tid < num_experts) expert_offsets[tid] = bin_base;
    if (tid == 0) expert_offsets[num_experts] = static_cast<int32_t>(n);
  }
  int32_t run = bin_base + before;
#pragma unroll
  for (int i = 0; i < kWavesPerBlock; ++i) {
    s_run[i][tid] = run;
    if (first_seg + i < num_seg) run += hist[(first_seg + i) * kBins + tid];
  }
  __syncthreads();

  const int64_t seg = first_seg + w;
  const int64_t begin = seg * seg_len;
  const int64_t end = begin + seg_len < n ? begin + seg_len : n;
  const uint64_t below = (1ull << lane) - 1ull;
  bool bad = false;
  for (int64_t base = begin; base < end; base += kWave) {
    const int64_t i = base + lane;
    const bool active = i < end;
    const int key = active ? load_key(ids, itype, i, num_experts, bad) : 0;
    int32_t pos = 0;
    for_each_key_group(key, active, [&](int k, uint64_t mask) {
      const int32_t start = s_run[w][k];  // same address for the whole wave: LDS broadcast
      if (active && key == k) pos = start + __popcll(mask & below);
      __builtin_amdgcn_wave_barrier();
      if (lane == 0) s_run[w][k] = start + __popcll(mask);
      __builtin_amdgcn_wave_barrier();
    });
    if (active) {
      const int64_t t = i / num_topk, k = i - t * num_topk;
      row_id_map[k * num_tokens + t] = pos < num_out ? pos : -1;
      if (sorted_row_id != nullptr) sorted_row_id[pos] = static_cast<int32_t>(i);
    }
  }
}

// ---- the whole partition in one workgroup ---------------------------------------------------------------
// Up to kSmallKeys keys (a denoise step of the model is 2048): one launch of one 1024-thread workgroup does what
// the two launches above do -- per-wavefront histograms in LDS, the prefix over bins and wavefronts, then the same
// ballot ranking: 5 us instead of 12 at 2048 keys.  Beyond a few thousand keys one CU walking them all loses to the
// two launches over many CUs (36 us against 15 at 29184 keys).
constexpr int kSmallWaves = 16;
constexpr int64_t kSmallKeys = 4096;

__global__ __launch_bounds__(kSmallWaves* kWave) void partition_small_kernel(
    const void* __restrict__ ids, int itype, int64_t num_tokens, int num_topk, int num_experts, int64_t num_out,
    int32_t* __restrict__ row_id_map, int32_t* __restrict__ sorted_row_id, int32_t* __restrict__ expert_offsets,
    int32_t* status) {
  __shared__ int32_t s_run[kSmallWaves][kBins];  // counts, then the next free sorted position per (wave, bin)
  __shared__ int32_t s_wave_total[kBins / kWave];
  const int tid = threadIdx.x, w = tid / kWave, lane = lane_id();
  const int64_t n = num_tokens * num_topk;
  for (int i = lane; i < kBins; i += kWave) s_run[w][i] = 0;
  // keys of wavefront w: a contiguous run, a multiple of 64 long
  const int64_t chunk = ((n + kSmallWaves - 1) / kSmallWaves + kWave - 1) / kWave * kWave;
  const int64_t begin = w * chunk < n ? w * chunk : n;
  const int64_t end = begin + chunk < n ? begin + chunk : n;
  bool bad = false;
  __builtin_amdgcn_wave_barrier();
  for (int64_t base = begin; base < end; base += kWave) {
    const int64_t i = base + lane;
    const bool active = i < end;
    const int key = active ? load_key(ids, itype, i, num_experts, bad) : 0;
    for_each_key_group(key, active, [&](int k, uint64_t mask) {
      if (lane == 0) s_run[w][k] += __popcll(mask);
    });
  }
  if (status != nullptr && __ballot(bad) != 0 && lane == 0) *status = 1;
  __syncthreads();
  // bin `tid` (tid < 256): exclusive prefix over the bins of the totals, then running starts per wavefront
  int32_t total = 0, incl = 0;
  if (tid < kBins) {
    for (int i = 0; i < kSmallWaves; ++i) total += s_run[i][tid];
    incl = total;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int32_t up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    if (lane == kWave - 1) s_wave_total[w] = incl;
  }
  __syncthreads();
  if (tid < kBins) {
    int32_t run = incl - total;
    for (int i = 0; i < w; ++i) run += s_wave_total[i];
    if (expert_offsets != nullptr) {
      if (tid < num_experts) expert_offsets[tid] = run;
      if (tid == 0) expert_offsets[num_experts] = static_cast<int32_t>(n);
    }
    for (int i = 0; i < kSmallWaves; ++i) {
      const int32_t c = s_run[i][tid];
      s_run[i][tid] = run;
      run += c;
    }
  }
  __syncthreads();
  const uint64_t below = (1ull << lane) - 1ull;
  for (int64_t base = begin; base < end; base += kWave) {
    const int64_t i = base + lane;
    const bool active = i < end;
    const int key = active ? load_key(ids, itype, i, num_experts, bad) : 0;
    int32_t pos = 0;
    for_each_key_group(key, active, [&](int k, uint64_t mask) {
      const int32_t start = s_run[w][k];  // same address for the whole wave: LDS broadcast
      if (active && key == k) pos = start + __popcll(mask & below);
      __builtin_amdgcn_wave_barrier();
      if (lane == 0) s_run[w][k] = start + __popcll(mask);
      __builtin_amdgcn_wave_barrier();
    });
    if (active) {
      const int64_t t = i / num_topk, k = i - t * num_topk;
      row_id_map[k * num_tokens + t] = pos < num_out ? pos : -1;
      if (sorted_row_id != nullptr) sorted_row_id[pos] = static_cast<int32_t>(i);
    }
  }
}

// ---- row movers ---------------------------------------------------------------------------------
constexpr int kMoverWaves = 4;

__device__ __forceinline__ u32x4 ld16(const u32x4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st16(u32x4* p, const u32x4& v) { __builtin_nontemporal_store(v, p); }

// out[row_id_map[k*T + t]] = x[t] for every k; one wavefront per source row.
__global__ __launch_bounds__(kMoverWaves* kWave) void permute_rows_kernel(
    const u32x4* __restrict__ x, u32x4* __restrict__ out, const int32_t* __restrict__ row_id_map,
    int64_t num_tokens, int num_topk, int64_t vec_per_row) {
  const int lane = lane_id();
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kMoverWaves + threadIdx.x / kWave;
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kMoverWaves;
  for (int64_t t = wave; t < num_tokens; t += n_waves) {
    const u32x4* src = x + t * vec_per_row;
    if (num_topk == 1) {
      const int32_t dst_row = row_id_map[t];
      if (dst_row < 0) continue;
      u32x4* dst = out + static_cast<int64_t>(dst_row) * vec_per_row;
      int64_t v = lane;
      for (; v + 3 * kWave < vec_per_row; v += 4 * kWave) {
        const u32x4 a = ld16(src + v), b = ld16(src + v + kWave), c = ld16(src + v + 2 * kWave),
                    d = ld16(src + v + 3 * kWave);
        st16(dst + v, a); st16(dst + v + kWave, b); st16(dst + v + 2 * kWave, c); st16(dst + v + 3 * kWave, d);
      }
      for (; v < vec_per_row; v += kWave) st16(dst + v, ld16(src + v));
    } else {
      for (int64_t v = lane; v < vec_per_row; v += kWave) {
        const u32x4 a = ld16(src + v);
        for (int k = 0; k < num_topk; ++k) {
          const int32_t dst_row = row_id_map[k * num_tokens + t];
          if (dst_row >= 0) st16(out + static_cast<int64_t>(dst_row) * vec_per_row + v, a);
        }
      }
    }
  }
}

// Row scatter into the K-tiled, expert-padded layout the MFMA kernels read (bf16): row p of the sorted space lands
// at row p (expert 0) or p + pad (expert 1, which starts at the next multiple of 256 rows), cut into 64-byte
// column-block segments.  One wavefront per source row; lane q handles 16-byte chunks q, q + 64, ...
__global__ __launch_bounds__(kMoverWaves* kWave) void permute_rows_tiled_kernel(
    const u32x4* __restrict__ x, unsigned char* __restrict__ out, const int32_t* __restrict__ row_id_map,
    const int32_t* __restrict__ expert_offsets, int64_t num_tokens, int64_t chunks_per_row, int64_t row_blocks) {
  const int lane = lane_id();
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kMoverWaves + threadIdx.x / kWave;
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kMoverWaves;
  const int32_t first1 = expert_offsets[1];                                    // first sorted row of expert 1
  const int32_t pad = static_cast<int32_t>(round_up_256(first1 - expert_offsets[0])) - (first1 - expert_offsets[0]);
  for (int64_t t = wave; t < num_tokens; t += n_waves) {
    int32_t dst_row = row_id_map[t];
    if (dst_row < 0) continue;
    if (dst_row >= first1) dst_row += pad;
    const u32x4* src = x + t * chunks_per_row;
    const int64_t rb = dst_row >> 4;
    const int r = dst_row & 15, swz = (r >> 2) & 3;
    unsigned char* dst = out + (rb << 10) + (r << 6);
    int64_t q = lane;
    for (; q + 3 * kWave < chunks_per_row; q += 4 * kWave) {
      u32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = ld16(src + q + u * kWave);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t qq = q + u * kWave;
        st16(reinterpret_cast<u32x4*>(dst + (((qq >> 2) * row_blocks) << 10) + (((qq & 3) ^ swz) << 4)), v[u]);
      }
    }
    for (; q < chunks_per_row; q += kWave)
      st16(reinterpret_cast<u32x4*>(dst + (((q >> 2) * row_blocks) << 10) + (((q & 3) ^ swz) << 4)), ld16(src + q));
  }
}

// Same result, driven from the destination side: a wavefront owns one 16-row block of the tiled matrix and a
// range of column blocks; lane -> (row lane/4, slot lane%4) reads 16 bytes of its source row and the 64 lanes
// write one whole contiguous KiB block.  Needs the inverse map (sorted position -> source token).
#ifndef WX_GATHER_SPLIT
#define WX_GATHER_SPLIT 4
#endif
constexpr int kGatherSplit = WX_GATHER_SPLIT;  // wavefronts per 16-row block, each takes a quarter of the column blocks
__global__ __launch_bounds__(kMoverWaves* kWave) void permute_rows_tiled_gather_kernel(
    const u32x4* __restrict__ x, unsigned char* __restrict__ out, const int32_t* __restrict__ sorted_row_id,
    const int32_t* __restrict__ expert_offsets, int64_t num_tokens, int64_t col_blocks, int64_t row_blocks) {
  const int lane = lane_id();
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kMoverWaves + threadIdx.x / kWave;
  const int64_t rb = wave / kGatherSplit;
  const int part = static_cast<int>(wave % kGatherSplit);
  if (rb >= row_blocks) return;
  const int32_t o0 = expert_offsets[0], o1 = expert_offsets[1], o2 = expert_offsets[2];
  const int64_t pad0 = round_up_256(o1 - o0);
  // padded row -> sorted position (or none for the padding rows of either expert)
  const int r = lane >> 2, slot = lane & 3, chunk = slot ^ ((r >> 2) & 3);
  const int64_t prow = rb * kBlkRows + r;
  int64_t pos = -1;
  if (prow < pad0) { if (prow < o1 - o0) pos = o0 + prow; }
  else if (prow - pad0 < o2 - o1) pos = o1 + (prow - pad0);
  const int64_t src_tok = (pos >= 0 && pos < num_tokens) ? sorted_row_id[pos] : -1;
  const int64_t chunks_per_row = col_blocks * 4;
  const u32x4* src = x + (src_tok < 0 ? 0 : src_tok) * chunks_per_row + chunk;
  const int64_t kb_per = (col_blocks + kGatherSplit - 1) / kGatherSplit;
  const int64_t kb0 = part * kb_per, kb1 = kb0 + kb_per < col_blocks ? kb0 + kb_per : col_blocks;
  unsigned char* dst = out + (rb << 10) + lane * 16;
  const u32x4 zero = {0, 0, 0, 0};
  int64_t kb = kb0;
  for (; kb + 3 < kb1; kb += 4) {
    u32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = src_tok < 0 ? zero : ld16(src + (kb + u) * 4);
#pragma unroll
    for (int u = 0; u < 4; ++u) st16(reinterpret_cast<u32x4*>(dst + (((kb + u) * row_blocks) << 10)), v[u]);
  }
  for (; kb < kb1; ++kb)
    st16(reinterpret_cast<u32x4*>(dst + ((kb * row_blocks) << 10)), src_tok < 0 ? zero : ld16(src + kb * 4));
}

// The same gather with 128-byte reads: a lane takes chunk (lane & 7) of the 128 bytes that span a PAIR of column
// blocks, for rows (lane >> 3) and (lane >> 3) + 8 of the row block, so a load instruction touches 8 rows x one whole
// cache line instead of 16 rows x half a line, and a store instruction writes two 512-byte runs (the upper or lower
// 8 rows of the two blocks).  Needs an even number of column blocks.
// `split`: wavefronts per 16-row block (each takes that share of the column-block pairs); the host raises it for small
// token counts so that the launch still has a few wavefronts per SIMD to cover the latency of its dependent loads.
__global__ __launch_bounds__(kMoverWaves* kWave) void permute_rows_tiled_gather128_kernel(
    const u32x4* __restrict__ x, unsigned char* __restrict__ out, const int32_t* __restrict__ sorted_row_id,
    const int32_t* __restrict__ expert_offsets, int64_t num_tokens, int64_t col_blocks, int64_t row_blocks, int split) {
  const int lane = lane_id();
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kMoverWaves + threadIdx.x / kWave;
  const int64_t rb = wave / split;
  const int part = static_cast<int>(wave % split);
  if (rb >= row_blocks) return;
  const int32_t o0 = expert_offsets[0], o1 = expert_offsets[1], o2 = expert_offsets[2];
  const int64_t pad0 = round_up_256(o1 - o0);
  const int r8 = lane >> 3, c8 = lane & 7;
  const int64_t chunks_per_row = col_blocks * 4;
  const u32x4* src[2];
  bool live[2];
  int dst_off[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int r = 8 * h + r8;
    const int64_t prow = rb * kBlkRows + r;
    int64_t pos = -1;
    if (prow < pad0) { if (prow < o1 - o0) pos = o0 + prow; }
    else if (prow - pad0 < o2 - o1) pos = o1 + (prow - pad0);
    const int64_t tok = (pos >= 0 && pos < num_tokens) ? sorted_row_id[pos] : -1;
    live[h] = tok >= 0;
    src[h] = x + (tok < 0 ? 0 : tok) * chunks_per_row + c8;
    // inside its block the chunk (c8 & 3) of row r sits in slot (c8 & 3) ^ ((r >> 2) & 3)
    dst_off[h] = r * 64 + (((c8 & 3) ^ ((r >> 2) & 3)) << 4);
  }
  const int64_t pairs = col_blocks / 2;
  const int64_t per = (pairs + split - 1) / split;
  const int64_t p0 = part * per, p1 = p0 + per < pairs ? p0 + per : pairs;
  unsigned char* base = out + (rb << 10) + (((c8 >> 2) * row_blocks) << 10);  // block kb or kb + 1 of the pair
  const u32x4 zero = {0, 0, 0, 0};
  int64_t pr = p0;
  for (; pr + 1 < p1; pr += 2) {
    u32x4 v[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) v[u][h] = live[h] ? ld16(src[h] + (pr + u) * 8) : zero;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h)
        st16(reinterpret_cast<u32x4*>(base + (((pr + u) * 2 * row_blocks) << 10) + dst_off[h]), v[u][h]);
  }
  for (; pr < p1; ++pr)
#pragma unroll
    for (int h = 0; h < 2; ++h)
      st16(reinterpret_cast<u32x4*>(base + ((pr * 2 * row_blocks) << 10) + dst_off[h]), live[h] ? ld16(src[h] + pr * 8) : zero);
}

// out[t] = y[row_id_map[t]] (zeros when the map entry is -1); one wavefront per destination row.
__global__ __launch_bounds__(kMoverWaves* kWave) void gather_rows_kernel(
    const u32x4* __restrict__ y, u32x4* __restrict__ out, const int32_t* __restrict__ row_id_map,
    int64_t num_tokens, int64_t vec_per_row) {
  const int lane = lane_id();
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kMoverWaves + threadIdx.x / kWave;
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kMoverWaves;
  for (int64_t t = wave; t < num_tokens; t += n_waves) {
    const int32_t src_row = row_id_map[t];
    u32x4* dst = out + t * vec_per_row;
    if (src_row < 0) {
      for (int64_t v = lane; v < vec_per_row; v += kWave) st16(dst + v, u32x4{0, 0, 0, 0});
      continue;
    }
    const u32x4* src = y + static_cast<int64_t>(src_row) * vec_per_row;
    int64_t v = lane;
    for (; v + 3 * kWave < vec_per_row; v += 4 * kWave) {
      const u32x4 a = ld16(src + v), b = ld16(src + v + kWave), c = ld16(src + v + 2 * kWave),
                  d = ld16(src + v + 3 * kWave);
      st16(dst + v, a); st16(dst + v + kWave, b); st16(dst + v + 2 * kWave, c); st16(dst + v + 3 * kWave, d);
    }
    for (; v < vec_per_row; v += kWave) st16(dst + v, ld16(src + v));
  }
}

// out[t] = sum_k prob[t,k] * y[row_id_map[k*T+t]] for topK > 1.  The reference kernel multiplies and
// accumulates in the storage type (csrc/permute.cu:69-154 with TCompute == T for 16-bit types), one
// rounding per operation in k order; Elem<DT>::round reproduces that.
template <int DT>
__global__ __launch_bounds__(kMoverWaves* kWave) void combine_rows_kernel(
    const u32x4* __restrict__ y, u32x4* __restrict__ out, const int32_t* __restrict__ row_id_map,
    const float* __restrict__ probs, int64_t num_tokens, int num_topk, int64_t vec_per_row) {
  constexpr int E = elems_per_16<DT>();
  const int lane = lane_id();
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kMoverWaves + threadIdx.x / kWave;
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kMoverWaves;
  for (int64_t t = wave; t < num_tokens; t += n_waves) {
    for (int64_t v = lane; v < vec_per_row; v += kWave) {
      float acc[E];
#pragma unroll
      for (int e = 0; e < E; ++e) acc[e] = 0.f;
      for (int k = 0; k < num_topk; ++k) {
        const int32_t r = row_id_map[k * num_tokens + t];
        if (r < 0) continue;  // a dropped copy adds nothing (for k == 0 the sum starts at zero)
        float f[E];
        unpack16<DT>(ld16(y + static_cast<int64_t>(r) * vec_per_row + v), f);
        const float p = probs != nullptr ? Elem<DT>::round(probs[t * num_topk + k]) : 1.f;
#pragma unroll
        for (int e = 0; e < E; ++e) {
          const float term = probs != nullptr ? Elem<DT>::round(f[e] * p) : f[e];
          acc[e] = k == 0 ? term : Elem<DT>::round(acc[e] + term);
        }
      }
      st16(out + t * vec_per_row + v, pack16<DT>(acc));
    }
  }
}

// Backward of the weighted combine; one wavefront per token.
template <int DT>
__global__ __launch_bounds__(kMoverWaves* kWave) void combine_rows_bwd_kernel(
    const u32x4* __restrict__ grad_out, const u32x4* __restrict__ y_fwd, u32x4* __restrict__ act_grad,
    float* __restrict__ prob_grad, const int32_t* __restrict__ row_id_map, const float* __restrict__ probs,
    int64_t num_tokens, int num_topk, int64_t vec_per_row) {
  constexpr int E = elems_per_16<DT>();
  const int lane = lane_id();
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kMoverWaves + threadIdx.x / kWave;
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kMoverWaves;
  const bool weighted = num_topk > 1 && probs != nullptr;
  for (int64_t t = wave; t < num_tokens; t += n_waves) {
    for (int k = 0; k < num_topk; ++k) {
      const int32_t r = row_id_map[k * num_tokens + t];
      float dot = 0.f;
      if (r >= 0) {
        const float p = weighted ? Elem<DT>::round(probs[t * num_topk + k]) : 1.f;
        for (int64_t v = lane; v < vec_per_row; v += kWave) {
          const u32x4 g16 = ld16(grad_out + t * vec_per_row + v);
          if (!weighted) {
            st16(act_grad + static_cast<int64_t>(r) * vec_per_row + v, g16);
            continue;
          }
          float g[E], yv[E], o[E];
          unpack16<DT>(g16, g);
          unpack16<DT>(ld16(y_fwd + static_cast<int64_t>(r) * vec_per_row + v), yv);
#pragma unroll
          for (int e = 0; e < E; ++e) {
            o[e] = Elem<DT>::round(g[e] * p);
            dot += Elem<DT>::round(g[e] * yv[e]);
          }
          st16(act_grad + static_cast<int64_t>(r) * vec_per_row + v, pack16<DT>(o));
        }
      }
      if (weighted && prob_grad != nullptr) {
#pragma unroll
        for (int d = kWave / 2; d > 0; d >>= 1) dot += __shfl_xor(dot, d);
        if (lane == 0) prob_grad[t * num_topk + k] = dot;
      }
    }
  }
}

int elem_bytes(int dtype) {
  switch (dtype) {
    case WX_F32: return 4;
    case WX_F16:
    case WX_BF16: return 2;
    default: return 0;
  }
}

int mover_grid(int64_t rows) {
  // enough resident wavefronts to cover HBM latency: 8 blocks of 4 waves per CU, capped by the row count
  const int64_t want = static_cast<int64_t>(device_cu_count()) * 8;
  const int64_t need = (rows + kMoverWaves - 1) / kMoverWaves;
  return static_cast<int>(need < want ? (need < 1 ? 1 : need) : want);
}

int check_rows(const char* who, const void* a, const void* b, const void* map, int64_t num_tokens, int num_topk,
               int64_t num_cols, int dtype) {
  const int eb = elem_bytes(dtype);
  if (eb == 0) return fail(WX_ERR_UNSUPPORTED, "%s: dtype %d is not fp32/fp16/bf16", who, dtype);
  if (num_tokens < 0 || num_cols <= 0 || num_topk < 1) return fail(WX_ERR_INVALID_ARGUMENT, "%s: bad sizes", who);
  if (num_topk > 128) return fail(WX_ERR_UNSUPPORTED, "%s: num_topK cannot exceed 128.", who);
  if ((num_cols * eb) % 16 != 0)
    return fail(WX_ERR_UNSUPPORTED, "%s: row size %lld bytes is not a multiple of 16", who,
                static_cast<long long>(num_cols * eb));
  if (num_tokens > 0 && (a == nullptr || b == nullptr || map == nullptr))
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", who);
  if (num_tokens * num_topk > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "%s: more than 2^31-1 rows", who);
  return WX_OK;
}

}  // namespace
}  // namespace wx

using namespace wx;

extern "C" size_t wx_partition_workspace_bytes(int64_t n) {
  if (n <= 0) return 256;
  const int64_t seg = segment_len(n);
  const int64_t num_seg = (n + seg - 1) / seg;
  const int64_t padded = (num_seg + kWavesPerBlock - 1) / kWavesPerBlock * kWavesPerBlock;
  return static_cast<size_t>(padded) * kBins * sizeof(int32_t);
}

namespace {

// Argument checks and the two launches shared by the partition entry points; `hist` holds
// wx_partition_workspace_bytes(n) bytes.  Every histogram word the second launch reads is written by the first, so
// the buffer needs no clearing between calls.
int partition_launch(const char* who, const void* ids, int id_type, int64_t num_tokens, int num_topk, int num_experts,
                     int64_t num_out_tokens, int32_t* row_id_map, int32_t* sorted_row_id, int32_t* expert_offsets,
                     int32_t* status, int32_t* hist, size_t hist_bytes, hipStream_t s) {
  if (num_tokens < 0 || num_topk < 1) return fail(WX_ERR_INVALID_ARGUMENT, "%s: bad sizes", who);
  if (num_topk > 128) return fail(WX_ERR_UNSUPPORTED, "%s: num_topK cannot exceed 128.", who);
  if (num_experts < 1 || num_experts > kBins)
    return fail(WX_ERR_UNSUPPORTED, "%s: num_experts %d outside [1, %d]", who, num_experts, kBins);
  if (id_type != WX_I32 && id_type != WX_I64 && id_type != WX_U8)
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: bad id_type %d", who, id_type);
  const int64_t n = num_tokens * num_topk;
  if (n > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "%s: more than 2^31-1 expanded tokens", who);
  if (n > 0 && (ids == nullptr || row_id_map == nullptr || hist == nullptr))
    return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  if (hist_bytes < wx_partition_workspace_bytes(n))
    return fail(WX_ERR_WORKSPACE, "%s: workspace %zu < %zu bytes", who, hist_bytes, wx_partition_workspace_bytes(n));
  const int64_t num_out_small = num_out_tokens > 0 ? num_out_tokens : n;
  if (n <= kSmallKeys) {  // one workgroup, one launch, no histogram buffer
    hipLaunchKernelGGL(partition_small_kernel, dim3(1), dim3(kSmallWaves * kWave), 0, s, ids, id_type, num_tokens,
                       num_topk, num_experts, num_out_small, row_id_map, sorted_row_id, expert_offsets, status);
    return check_launch("partition_small_kernel");
  }
  const int64_t seg = segment_len(n > 0 ? n : 1);
  const int64_t num_seg = n > 0 ? (n + seg - 1) / seg : 0;
  // at least one block even for n == 0 so expert_offsets are written
  const int blocks = static_cast<int>(num_seg > 0 ? (num_seg + kWavesPerBlock - 1) / kWavesPerBlock : 1);
  const int64_t num_out = num_out_tokens > 0 ? num_out_tokens : n;
  if (n > 0) {
    hipLaunchKernelGGL(partition_count, dim3(blocks), dim3(kBlock), 0, s, ids, id_type, n, num_experts, seg, hist,
                       status);
    if (int rc = check_launch("partition_count")) return rc;
  }
  hipLaunchKernelGGL(partition_scatter, dim3(blocks), dim3(kBlock), 0, s, ids, id_type, num_tokens, num_topk,
                     num_experts, num_out, seg, num_seg, hist, row_id_map, sorted_row_id, expert_offsets);
  return check_launch("partition_scatter");
}

}  // namespace

extern "C" int wx_partition_build(const void* ids, int id_type, int64_t num_tokens, int num_topk, int num_experts,
                                  int64_t num_out_tokens, int32_t* row_id_map, int32_t* sorted_row_id,
                                  int32_t* expert_offsets, int32_t* status, void* workspace,
                                  size_t workspace_bytes, wx_stream_t stream) {
  return partition_launch("wx_partition_build", ids, id_type, num_tokens, num_topk, num_experts, num_out_tokens,
                          row_id_map, sorted_row_id, expert_offsets, status, static_cast<int32_t*>(workspace),
                          workspace_bytes, as_stream(stream));
}

// ---- the partition without a workspace argument ----------------------------------------------------------------
// The per-segment histograms live in a device array that is part of the library's code object: each GPU the library
// runs on holds its own 1 MiB copy from the moment the code object is loaded there until the process ends.
// segment_len() never cuts the key stream into more than 1024 segments, so the array covers every size the
// partition takes.  In host code the array's name is only a handle for hipGetSymbolAddress: the address kernels and
// copies use is looked up once per device, with that device current, and kept.
constexpr int kStaticSegments = 1024;
static __device__ __align__(256) int32_t scratch[kStaticSegments * wx::kBins];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
int32_t* g_scratch_ptr[kMaxDevices] = {};

// `capturing`: the call that asks is being recorded into a HIP graph.  The address lookup is a runtime call that does
// not belong inside a capture (it can fail there, or end the capture), so a first use on a device from inside one is
// refused with a message that says what to do instead.
int static_scratch(int32_t** out, bool capturing) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(WX_ERR_LAUNCH, "wx_partition_build_noalloc: no current device (or its index is %d or above)", kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    if (capturing)
      return fail(WX_ERR_INVALID_ARGUMENT,
                  "wx_partition_build_noalloc: first use on device %d comes from inside a stream capture; call "
                  "wx_partition_noalloc_init() (or make one call) on this device before capturing", dev);
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(WX_ERR_LAUNCH, "wx_partition_build_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<int32_t*>(p);
  }
  *out = g_scratch_ptr[dev];
  return WX_OK;
}

}  // namespace

extern "C" int wx_partition_build_noalloc(const void* ids, int id_type, int64_t num_tokens, int num_topk,
                                          int num_experts, int64_t num_out_tokens, int32_t* row_id_map,
                                          int32_t* sorted_row_id, int32_t* expert_offsets, int32_t* status,
                                          wx_stream_t stream) {
  constexpr size_t kScratchBytes = sizeof(int32_t) * kStaticSegments * kBins;
  // sizes the partition refuses anyway (negative, topK > 128, more than 2^31-1 expanded tokens) get their message
  // from partition_launch; anything else must fit the array
  const bool sane = num_tokens >= 0 && num_topk >= 1 && num_topk <= 128 && num_tokens <= INT32_MAX / num_topk;
  if (!sane)
    return partition_launch("wx_partition_build_noalloc", ids, id_type, num_tokens, num_topk, num_experts,
                            num_out_tokens, row_id_map, sorted_row_id, expert_offsets, status, nullptr, 0,
                            as_stream(stream));
  if (wx_partition_workspace_bytes(num_tokens * num_topk) > kScratchBytes)
    return fail(WX_ERR_WORKSPACE, "wx_partition_build_noalloc: %lld expanded tokens need %zu bytes of histograms, the built-in scratch has %zu",
                static_cast<long long>(num_tokens * num_topk), wx_partition_workspace_bytes(num_tokens * num_topk), kScratchBytes);
  int32_t* hist = nullptr;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(as_stream(stream), &cap) != hipSuccess) {
    (void)hipGetLastError();
    cap = hipStreamCaptureStatusNone;
  }
  if (int rc = static_scratch(&hist, cap != hipStreamCaptureStatusNone)) return rc;
  return partition_launch("wx_partition_build_noalloc", ids, id_type, num_tokens, num_topk, num_experts,
                          num_out_tokens, row_id_map, sorted_row_id, expert_offsets, status, hist, kScratchBytes,
                          as_stream(stream));
}

extern "C" int wx_partition_noalloc_init(void) {
  int32_t* hist = nullptr;
  return static_scratch(&hist, false);
}

extern "C" int wx_permute_rows(const void* x, void* out, const int32_t* row_id_map, int64_t num_tokens,
                               int num_topk, int64_t num_cols, int dtype, wx_stream_t stream) {
  if (int rc = check_rows("wx_permute_rows", x, out, row_id_map, num_tokens, num_topk, num_cols, dtype)) return rc;
  if (num_tokens == 0) return WX_OK;
  const int64_t vec = num_cols * elem_bytes(dtype) / 16;
  hipLaunchKernelGGL(permute_rows_kernel, dim3(mover_grid(num_tokens)), dim3(kMoverWaves * kWave), 0,
                     as_stream(stream), static_cast<const u32x4*>(x), static_cast<u32x4*>(out), row_id_map,
                     num_tokens, num_topk, vec);
  return check_launch("permute_rows_kernel");
}

extern "C" int wx_permute_rows_tiled(const void* x, void* out_tiled, const int32_t* row_id_map,
                                     const int32_t* sorted_row_id, const int32_t* expert_offsets,
                                     int64_t num_tokens, int64_t num_cols, wx_stream_t stream) {
  const int32_t* any_map = row_id_map != nullptr ? row_id_map : sorted_row_id;
  if (int rc = check_rows("wx_permute_rows_tiled", x, out_tiled, any_map, num_tokens, 1, num_cols, WX_BF16)) return rc;
  if (num_cols % kBlkCols != 0)
    return fail(WX_ERR_UNSUPPORTED, "wx_permute_rows_tiled: num_cols (%lld) must be a multiple of 32",
                static_cast<long long>(num_cols));
  if (num_tokens == 0) return WX_OK;
  if (expert_offsets == nullptr) return fail(WX_ERR_INVALID_ARGUMENT, "wx_permute_rows_tiled: null expert_offsets");
  const int64_t row_blocks = padded_sorted_rows(num_tokens) / kBlkRows;
  if (sorted_row_id != nullptr) {
    const dim3 block(kMoverWaves * kWave);
#ifndef WX_GATHER128
#define WX_GATHER128 1
#endif
    if (WX_GATHER128 && (num_cols / kBlkCols) % 2 == 0) {
      // kGatherSplit wavefronts per row block suit tens of thousands of tokens; a few thousand tokens would leave
      // most SIMDs with one wavefront or none, each walking a chain of dependent loads: split the row blocks
      // further, up to eight wavefronts per CU's worth or one pair of column blocks per two wavefronts' iteration
      const int64_t pairs = num_cols / kBlkCols / 2;
      int split = kGatherSplit;
      while (row_blocks * split < 8ll * device_cu_count() && 2 * split <= pairs / 2) split *= 2;
      const int64_t gather_waves = row_blocks * split;
      hipLaunchKernelGGL(permute_rows_tiled_gather128_kernel, dim3(static_cast<unsigned>((gather_waves + kMoverWaves - 1) / kMoverWaves)),
                         block, 0, as_stream(stream), static_cast<const u32x4*>(x),
                         static_cast<unsigned char*>(out_tiled), sorted_row_id, expert_offsets, num_tokens,
                         num_cols / kBlkCols, row_blocks, split);
      return check_launch("permute_rows_tiled_gather128_kernel");
    }
    const int64_t waves = row_blocks * kGatherSplit;
    const dim3 grid(static_cast<unsigned>((waves + kMoverWaves - 1) / kMoverWaves));
    hipLaunchKernelGGL(permute_rows_tiled_gather_kernel, grid, block, 0, as_stream(stream), static_cast<const u32x4*>(x),
                       static_cast<unsigned char*>(out_tiled), sorted_row_id, expert_offsets, num_tokens,
                       num_cols / kBlkCols, row_blocks);
    return check_launch("permute_rows_tiled_gather_kernel");
  }
  hipLaunchKernelGGL(permute_rows_tiled_kernel, dim3(mover_grid(num_tokens)), dim3(kMoverWaves * kWave), 0,
                     as_stream(stream), static_cast<const u32x4*>(x), static_cast<unsigned char*>(out_tiled),
                     row_id_map, expert_offsets, num_tokens, num_cols / 8, padded_sorted_rows(num_tokens) / kBlkRows);
  return check_launch("permute_rows_tiled_kernel");
}

extern "C" int wx_unpermute_rows(const void* y, void* out, const int32_t* row_id_map, const float* probs,
                                 int64_t num_tokens, int num_topk, int64_t num_cols, int dtype,
                                 wx_stream_t stream) {
  if (int rc = check_rows("wx_unpermute_rows", y, out, row_id_map, num_tokens, num_topk, num_cols, dtype)) return rc;
  if (num_tokens == 0) return WX_OK;
  const int64_t vec = num_cols * elem_bytes(dtype) / 16;
  const dim3 grid(mover_grid(num_tokens)), block(kMoverWaves * kWave);
  hipStream_t s = as_stream(stream);
  const u32x4* yy = static_cast<const u32x4*>(y);
  u32x4* oo = static_cast<u32x4*>(out);
  if (num_topk == 1) {
    hipLaunchKernelGGL(gather_rows_kernel, grid, block, 0, s, yy, oo, row_id_map, num_tokens, vec);
  } else if (dtype == WX_F32) {
    hipLaunchKernelGGL(combine_rows_kernel<WX_F32>, grid, block, 0, s, yy, oo, row_id_map, probs, num_tokens,
                       num_topk, vec);
  } else if (dtype == WX_F16) {
    hipLaunchKernelGGL(combine_rows_kernel<WX_F16>, grid, block, 0, s, yy, oo, row_id_map, probs, num_tokens,
                       num_topk, vec);
  } else {
    hipLaunchKernelGGL(combine_rows_kernel<WX_BF16>, grid, block, 0, s, yy, oo, row_id_map, probs, num_tokens,
                       num_topk, vec);
  }
  return check_launch("wx_unpermute_rows");
}

extern "C" int wx_unpermute_rows_bwd(const void* grad_out, const void* y_fwd, void* act_grad, float* prob_grad,
                                     const int32_t* row_id_map, const float* probs, int64_t num_tokens,
                                     int num_topk, int64_t num_cols, int dtype, wx_stream_t stream) {
  if (int rc = check_rows("wx_unpermute_rows_bwd", grad_out, act_grad, row_id_map, num_tokens, num_topk, num_cols,
                          dtype))
    return rc;
  if (num_topk > 1 && (probs == nullptr || y_fwd == nullptr || prob_grad == nullptr))
    return fail(WX_ERR_INVALID_ARGUMENT, "wx_unpermute_rows_bwd: probs, y_fwd and prob_grad are required for topK > 1");
  if (num_tokens == 0) return WX_OK;
  const int64_t vec = num_cols * elem_bytes(dtype) / 16;
  const dim3 grid(mover_grid(num_tokens)), block(kMoverWaves * kWave);
  hipStream_t s = as_stream(stream);
  const u32x4* g = static_cast<const u32x4*>(grad_out);
  const u32x4* yf = static_cast<const u32x4*>(y_fwd);
  u32x4* ag = static_cast<u32x4*>(act_grad);
  if (dtype == WX_F32) {
    hipLaunchKernelGGL(combine_rows_bwd_kernel<WX_F32>, grid, block, 0, s, g, yf, ag, prob_grad, row_id_map, probs,
                       num_tokens, num_topk, vec);
  } else if (dtype == WX_F16) {
    hipLaunchKernelGGL(combine_rows_bwd_kernel<WX_F16>, grid, block, 0, s, g, yf, ag, prob_grad, row_id_map, probs,
                       num_tokens, num_topk, vec);
  } else {
    hipLaunchKernelGGL(combine_rows_bwd_kernel<WX_BF16>, grid, block, 0, s, g, yf, ag, prob_grad, row_id_map, probs,
                       num_tokens, num_topk, vec);
  }
  return check_launch("wx_unpermute_rows_bwd");
}
