// 3D M-RoPE position ids (integer, exact) for gfx950.  Semantics: act.py:929-1149 of the reference.
//
// One workgroup per batch row.
//   kernel 1  rope_index_count   compacts the unmasked tokens of a row and counts its vision items
//                                (<vision_start> followed by an image / video token)
//   kernel 2  rope_index_fill    derives the row's grid cursors from the counts of earlier rows (the
//                                reference walks one cursor across the whole batch), then
//                                  (a) wavefront 0 walks the row's vision items in order -- "next image
//                                      token at or after st" is a ballot search over 64 flags at a time --
//                                      and records one descriptor per item in LDS,
//                                  (b) all threads evaluate their tokens against the descriptors
//                                      (binary search, then closed form t/h/w), reduce the row maximum.
//                                Items are processed in batches of kMaxSeg, so there is no cap on the
//                                number of images per row.
// The text-only branch (no grids) is a masked prefix sum, one workgroup per row.
#include "common.h"

namespace wx {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kMaxSeg = 128;
// The compacted row -- cidx (4 B) and flag (1 B) per token -- lives in LDS up to this many tokens (with the item
// table that stays under the 160 KiB a workgroup can have); longer rows keep it in the caller's workspace.
constexpr int kMaxSeqLds = 30720;
constexpr size_t kRowBytesAlign = 256;
__host__ __device__ inline size_t row_bytes(int64_t seq) {
  return (static_cast<size_t>(seq) * 5 + 16 + kRowBytesAlign - 1) / kRowBytesAlign * kRowBytesAlign;
}
constexpr uint8_t kImg = 1, kVid = 2, kStart = 4;

struct Segment {
  int32_t st;       // compacted index where the text run before the item starts
  int32_t ed;       // compacted index of the item's first vision token
  int32_t gt, gh, gw;
  int32_t is_video;
  float spg;        // seconds per temporal grid step
  int64_t st_idx;   // position of the first token of the text run
};

struct RowLayout {
  int32_t* cidx;  // [S] compacted index of each original position (valid where mask != 0)
  uint8_t* flag;  // [L] token class bits per compacted token
};

__device__ __forceinline__ int32_t block_exclusive_scan(int32_t v, int32_t* s_wave, int32_t& total) {
  const int lane = lane_id(), w = threadIdx.x / kWave;
  int32_t incl = v;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int32_t up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  __syncthreads();  // s_wave may still be read from a previous call
  if (lane == kWave - 1) s_wave[w] = incl;
  __syncthreads();
  int32_t base = 0;
  total = 0;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) {
    if (i < w) base += s_wave[i];
    total += s_wave[i];
  }
  return base + incl - v;
}

__device__ __forceinline__ int64_t block_max(int64_t v, int64_t* s_wave) {
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) {
    const int64_t o = __shfl_xor(v, d);
    v = o > v ? o : v;
  }
  __syncthreads();
  if (lane_id() == 0) s_wave[threadIdx.x / kWave] = v;
  __syncthreads();
  int64_t m = s_wave[0];
#pragma unroll
  for (int i = 1; i < kWaves; ++i) m = s_wave[i] > m ? s_wave[i] : m;
  return m;
}

// Compacts the row: fills cidx / flag, returns the number of unmasked tokens L.
__device__ int32_t compact_row(const int64_t* __restrict__ ids, const int64_t* __restrict__ mask, int64_t seq,
                               int64_t image_id, int64_t video_id, int64_t start_id, RowLayout lay,
                               int32_t* s_wave) {
  const int per = static_cast<int>((seq + kThreads - 1) / kThreads);
  const int64_t lo = static_cast<int64_t>(threadIdx.x) * per;
  const int64_t hi = lo + per < seq ? lo + per : seq;
  int32_t cnt = 0;
  for (int64_t i = lo; i < hi; ++i) cnt += (mask == nullptr || mask[i] == 1) ? 1 : 0;  // act.py:991
  int32_t total;
  int32_t run = block_exclusive_scan(cnt, s_wave, total);
  for (int64_t i = lo; i < hi; ++i) {
    if (mask == nullptr || mask[i] == 1) {
      const int64_t tok = ids[i];
      lay.cidx[i] = run;
      lay.flag[run] = (tok == image_id ? kImg : 0) | (tok == video_id ? kVid : 0) | (tok == start_id ? kStart : 0);
      ++run;
    } else {
      lay.cidx[i] = -1;
    }
  }
  __syncthreads();
  return total;
}

__device__ __forceinline__ RowLayout carve(unsigned char* smem, int64_t seq) {
  RowLayout lay;
  lay.cidx = reinterpret_cast<int32_t*>(smem);
  lay.flag = reinterpret_cast<uint8_t*>(smem + seq * sizeof(int32_t));
  return lay;
}

// counts[b] = (#image items, #video items) of row b (act.py:995-1000)
// ROW_IN_GLOBAL: the compacted row is kept in `row_ws` (row_bytes(seq) per row) instead of LDS.
template <bool ROW_IN_GLOBAL>
__global__ __launch_bounds__(kThreads) void rope_index_count(const int64_t* __restrict__ input_ids,
                                                             const int64_t* __restrict__ attention_mask,
                                                             int64_t seq, int64_t image_id, int64_t video_id,
                                                             int64_t start_id, int32_t* __restrict__ counts,
                                                             int32_t* status, unsigned char* row_ws) {
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int32_t s_wave[kWaves];
  const int64_t b = blockIdx.x;
  RowLayout lay = carve(ROW_IN_GLOBAL ? row_ws + b * row_bytes(seq) : smem, seq);
  const int64_t* mask = attention_mask ? attention_mask + b * seq : nullptr;
  const int32_t L = compact_row(input_ids + b * seq, mask, seq, image_id, video_id, start_id, lay, s_wave);
  int32_t n_img = 0, n_vid = 0;
  bool bad = false;
  for (int32_t j = threadIdx.x; j < L; j += kThreads) {
    if (lay.flag[j] & kStart) {
      if (j + 1 >= L) { bad = true; continue; }  // the reference indexes past the end here and raises
      n_img += (lay.flag[j + 1] & kImg) ? 1 : 0;
      n_vid += (lay.flag[j + 1] & kVid) ? 1 : 0;
    }
  }
  int32_t t_img, t_vid;
  block_exclusive_scan(n_img, s_wave, t_img);
  block_exclusive_scan(n_vid, s_wave, t_vid);
  if (threadIdx.x == 0) {
    counts[2 * b] = t_img;
    counts[2 * b + 1] = t_vid;
  }
  if (status != nullptr && (bad || (L == 0 && threadIdx.x == 0))) *status = 1;
}

// First compacted index >= st whose flag has `bit`, or -1.  Executed by a whole wavefront.
__device__ __forceinline__ int32_t wave_find(const uint8_t* flag, int32_t L, int32_t st, uint8_t bit) {
  const int lane = lane_id();
  for (int32_t base = st; base < L; base += kWave) {
    const int32_t j = base + lane;
    const uint64_t m = __ballot(j < L && (flag[j] & bit));
    if (m) return base + __ffsll(static_cast<long long>(m)) - 1;
  }
  return -1;
}

__device__ __forceinline__ int64_t temporal_id(int32_t t, const Segment& sg, float tps) {
  if (!sg.is_video) return 0;  // images: second_per_grid_t = 0 (act.py:1028)
  // act.py:1070-1076: (int64 t -> fp32) * second_per_grid (fp32) * tokens_per_second (fp32), truncated
  const float f = __fmul_rn(__fmul_rn(static_cast<float>(t), sg.spg), tps);
  return static_cast<int64_t>(f);
}

template <bool ROW_IN_GLOBAL>
__global__ __launch_bounds__(kThreads) void rope_index_fill(
    const int64_t* __restrict__ input_ids, const int64_t* __restrict__ attention_mask,
    const int64_t* __restrict__ image_grid, int64_t n_image, const int64_t* __restrict__ video_grid,
    int64_t n_video, const float* __restrict__ sec_per_grid, int64_t seq, int merge, int64_t image_id,
    int64_t video_id, int64_t start_id, float tps, const int32_t* __restrict__ counts,
    int64_t* __restrict__ position_ids, int64_t* __restrict__ deltas, int64_t batch, int32_t* status,
    unsigned char* row_ws) {
  extern __shared__ __align__(16) unsigned char smem[];
  __shared__ int32_t s_wave[kWaves];
  __shared__ int64_t s_wave64[kWaves];
  __shared__ Segment s_seg[kMaxSeg + 1];
  __shared__ int32_t s_nseg, s_done, s_next_st, s_bad;
  __shared__ int64_t s_next_idx;

  const int64_t b = blockIdx.x;
  const int tid = threadIdx.x, lane = lane_id();
  RowLayout lay = carve(ROW_IN_GLOBAL ? row_ws + b * row_bytes(seq) : smem, seq);
  const int64_t* ids = input_ids + b * seq;
  const int64_t* mask = attention_mask ? attention_mask + b * seq : nullptr;
  const int32_t L = compact_row(ids, mask, seq, image_id, video_id, start_id, lay, s_wave);

  // grid cursors: items consumed by earlier rows (act.py:986 keeps one cursor for the whole batch)
  int32_t pi = 0, pv = 0;
  for (int64_t r = tid; r < b; r += kThreads) {
    pi += counts[2 * r];
    pv += counts[2 * r + 1];
  }
  int32_t img_cursor, vid_cursor;
  block_exclusive_scan(pi, s_wave, img_cursor);
  block_exclusive_scan(pv, s_wave, vid_cursor);
  int32_t rem_img = counts[2 * b], rem_vid = counts[2 * b + 1];

  if (tid == 0) {
    s_next_st = 0;
    s_next_idx = 0;
    s_bad = (L == 0) ? 1 : 0;
    s_done = 0;
  }
  __syncthreads();

  int64_t row_max = INT64_MIN;
  int32_t covered = 0;  // tokens [0, covered) have been written
  while (true) {
    // ---- (a) wavefront 0 walks up to kMaxSeg items -------------------------------------------------
    if (tid < kWave) {
      int32_t st = s_next_st;
      int64_t st_idx = s_next_idx;
      int32_t n = 0;
      bool bad = false, done = false;
      while (n < kMaxSeg) {
        if (rem_img + rem_vid == 0) { done = true; break; }
        // act.py:1010-1018.  list.index raises when nothing is found at or after st.
        int32_t ed_img = L + 1, ed_vid = L + 1;
        if (rem_img > 0) {
          ed_img = wave_find(lay.flag, L, st, kImg);
          if (ed_img < 0) { bad = true; break; }
        }
        if (rem_vid > 0) {
          ed_vid = wave_find(lay.flag, L, st, kVid);
          if (ed_vid < 0) { bad = true; break; }
        }
        Segment sg;
        int64_t g0, g1, g2;
        if (ed_img < ed_vid) {  // act.py:1021-1031
          if (img_cursor >= n_image) { bad = true; break; }
          g0 = image_grid[3 * img_cursor]; g1 = image_grid[3 * img_cursor + 1]; g2 = image_grid[3 * img_cursor + 2];
          sg.is_video = 0; sg.spg = 0.f; sg.ed = ed_img;
          ++img_cursor; --rem_img;
        } else {                // act.py:1032-1045
          if (vid_cursor >= n_video) { bad = true; break; }
          g0 = video_grid[3 * vid_cursor]; g1 = video_grid[3 * vid_cursor + 1]; g2 = video_grid[3 * vid_cursor + 2];
          sg.is_video = 1; sg.spg = sec_per_grid ? sec_per_grid[vid_cursor] : 1.0f; sg.ed = ed_vid;
          ++vid_cursor; --rem_vid;
        }
        sg.gt = static_cast<int32_t>(g0);
        sg.gh = static_cast<int32_t>(g1 / merge);  // act.py:1048-1052
        sg.gw = static_cast<int32_t>(g2 / merge);
        sg.st = st;
        sg.st_idx = st_idx;
        const int64_t n_vis = static_cast<int64_t>(sg.gt) * sg.gh * sg.gw;
        if (n_vis <= 0) { bad = true; break; }
        const int64_t base = (sg.ed - st) + st_idx;  // act.py:1094: text_len + st_idx
        int64_t vmax = sg.gh - 1 > sg.gw - 1 ? sg.gh - 1 : sg.gw - 1;
        const int64_t t_last = temporal_id(sg.gt - 1, sg, tps);
        vmax = t_last > vmax ? t_last : vmax;
        if (lane == 0) s_seg[n] = sg;
        ++n;
        st_idx = base + vmax + 1;                       // act.py:1056-1060 for the next run
        const int64_t nst = sg.ed + n_vis;              // act.py:1096
        if (nst > L) { bad = true; st = L; done = true; break; }  // positions would outnumber tokens
        st = static_cast<int32_t>(nst);
      }
      if (bad) done = true;
      if (done) {
        // act.py:1099-1108: the trailing text run, as a pseudo item with no vision tokens
        Segment tail{};
        tail.st = st; tail.ed = L; tail.gt = 0; tail.gh = 1; tail.gw = 1; tail.st_idx = st_idx;
        if (lane == 0) s_seg[n] = tail;
        ++n;
        st = L;
      }
      if (lane == 0) {
        s_nseg = n;
        s_done = done ? 1 : 0;
        s_next_st = st;
        s_next_idx = st_idx;
        if (bad) s_bad = 1;
      }
    }
    __syncthreads();
    const int32_t nseg = s_nseg;
    const int32_t upto = s_next_st;  // compacted tokens [covered, upto) belong to s_seg[0..nseg)

    // ---- (b) evaluate ----------------------------------------------------------------------------
    for (int64_t i = tid; i < seq; i += kThreads) {
      const int32_t j = lay.cidx[i];
      if (j < covered || j >= upto) continue;
      int lo = 0, hi = nseg - 1;  // last segment with st <= j
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (s_seg[mid].st <= j) lo = mid; else hi = mid - 1;
      }
      const Segment& sg = s_seg[lo];
      int64_t pt, ph, pw;
      if (j < sg.ed) {
        pt = ph = pw = sg.st_idx + (j - sg.st);
      } else {
        const int32_t q = j - sg.ed;
        const int32_t frame = sg.gh * sg.gw;
        const int32_t t = q / frame, r = q - t * frame;
        const int32_t h = r / sg.gw, w = r - h * sg.gw;
        const int64_t base = (sg.ed - sg.st) + sg.st_idx;
        pt = base + temporal_id(t, sg, tps);
        ph = base + h;
        pw = base + w;
      }
      position_ids[(0 * batch + b) * seq + i] = pt;
      position_ids[(1 * batch + b) * seq + i] = ph;
      position_ids[(2 * batch + b) * seq + i] = pw;
      int64_t m = pt > ph ? pt : ph;
      m = pw > m ? pw : m;
      row_max = m > row_max ? m : row_max;
    }
    covered = upto;
    const bool finished = s_done != 0;
    __syncthreads();
    if (finished) break;
  }

  // masked positions keep the initial value 1 (act.py:978-984)
  for (int64_t i = tid; i < seq; i += kThreads) {
    if (lay.cidx[i] < 0 || lay.cidx[i] >= covered) {
      position_ids[(0 * batch + b) * seq + i] = 1;
      position_ids[(1 * batch + b) * seq + i] = 1;
      position_ids[(2 * batch + b) * seq + i] = 1;
    }
  }
  const int64_t m = block_max(row_max, s_wave64);
  if (tid == 0) {
    deltas[b] = (L > 0 ? m + 1 : 1) - seq;  // act.py:1115-1117
    if (status != nullptr && s_bad) *status = 1;
  }
}

// act.py:1123-1149: no vision grids at all.
__global__ __launch_bounds__(kThreads) void rope_index_text_only(const int64_t* __restrict__ attention_mask,
                                                                 int64_t seq, int64_t batch,
                                                                 int64_t* __restrict__ position_ids,
                                                                 int64_t* __restrict__ deltas) {
  __shared__ int32_t s_wave[kWaves];
  __shared__ int64_t s_wave64[kWaves];
  const int64_t b = blockIdx.x;
  const int tid = threadIdx.x;
  int64_t row_max = INT64_MIN;
  if (attention_mask == nullptr) {
    for (int64_t i = tid; i < seq; i += kThreads)
      for (int a = 0; a < 3; ++a) position_ids[(a * batch + b) * seq + i] = i;
    if (tid == 0) deltas[b] = 0;
    return;
  }
  const int64_t* mask = attention_mask + b * seq;
  const int per = static_cast<int>((seq + kThreads - 1) / kThreads);
  const int64_t lo = static_cast<int64_t>(tid) * per;
  const int64_t hi = lo + per < seq ? lo + per : seq;
  int64_t sum = 0;  // attention_mask.long().cumsum(-1): any integer values, not only 0/1
  for (int64_t i = lo; i < hi; ++i) sum += mask[i];
  // 64-bit block scan through two 32-bit scans is unnecessary: masks are 0/1 in practice, but keep exact
  int32_t total;
  const int32_t base32 = block_exclusive_scan(static_cast<int32_t>(sum), s_wave, total);
  int64_t run = base32;
  for (int64_t i = lo; i < hi; ++i) {
    run += mask[i];
    const int64_t p = mask[i] == 0 ? 1 : run - 1;
    for (int a = 0; a < 3; ++a) position_ids[(a * batch + b) * seq + i] = p;
    row_max = p > row_max ? p : row_max;
  }
  const int64_t m = block_max(row_max, s_wave64);
  if (tid == 0) deltas[b] = m + 1 - seq;
}

}  // namespace
}  // namespace wx

using namespace wx;

extern "C" size_t wx_rope_index_workspace_bytes(int64_t batch, int64_t seq) {
  const size_t counts = static_cast<size_t>((batch > 0 ? batch : 1) * 2 * sizeof(int32_t) + 255) / 256 * 256;
  const size_t rows = seq > kMaxSeqLds ? static_cast<size_t>(batch > 0 ? batch : 1) * row_bytes(seq) : 0;
  return counts + rows;
}

extern "C" int wx_rope_index(const int64_t* input_ids, const int64_t* attention_mask, const int64_t* image_grid_thw,
                             int64_t n_image, const int64_t* video_grid_thw, int64_t n_video,
                             const float* second_per_grid_ts, int64_t batch, int64_t seq, int spatial_merge_size,
                             int64_t image_token_id, int64_t video_token_id, int64_t vision_start_token_id,
                             float tokens_per_second, int64_t* position_ids, int64_t* deltas, int32_t* status,
                             void* workspace, size_t workspace_bytes, wx_stream_t stream) {
  if (batch < 0 || seq < 0 || n_image < 0 || n_video < 0)
    return fail(WX_ERR_INVALID_ARGUMENT, "wx_rope_index: negative size");
  if (batch == 0 || seq == 0) return WX_OK;
  if (!position_ids || !deltas) return fail(WX_ERR_INVALID_ARGUMENT, "wx_rope_index: null output");
  if (batch > INT32_MAX) return fail(WX_ERR_UNSUPPORTED, "wx_rope_index: batch too large");
  hipStream_t s = as_stream(stream);
  const bool text_only = image_grid_thw == nullptr && video_grid_thw == nullptr;
  if (text_only) {
    hipLaunchKernelGGL(rope_index_text_only, dim3(static_cast<unsigned>(batch)), dim3(kThreads), 0, s, attention_mask,
                       seq, batch, position_ids, deltas);
    return check_launch("rope_index_text_only");
  }
  if (!input_ids) return fail(WX_ERR_INVALID_ARGUMENT, "wx_rope_index: null input_ids");
  if (spatial_merge_size <= 0) return fail(WX_ERR_INVALID_ARGUMENT, "wx_rope_index: spatial_merge_size must be positive");
  if (seq > INT32_MAX / 8) return fail(WX_ERR_UNSUPPORTED, "wx_rope_index: seq %lld too long", static_cast<long long>(seq));
  if (!workspace || workspace_bytes < wx_rope_index_workspace_bytes(batch, seq))
    return fail(WX_ERR_WORKSPACE, "wx_rope_index: workspace too small");
  int32_t* counts = static_cast<int32_t*>(workspace);
  const dim3 grid(static_cast<unsigned>(batch)), block(kThreads);
  if (seq > kMaxSeqLds) {
    unsigned char* rows = static_cast<unsigned char*>(workspace) + wx_rope_index_workspace_bytes(batch, 0);
    hipLaunchKernelGGL(rope_index_count<true>, grid, block, 0, s, input_ids, attention_mask, seq, image_token_id,
                       video_token_id, vision_start_token_id, counts, status, rows);
    if (int rc = check_launch("rope_index_count")) return rc;
    hipLaunchKernelGGL(rope_index_fill<true>, grid, block, 0, s, input_ids, attention_mask, image_grid_thw, n_image,
                       video_grid_thw, n_video, second_per_grid_ts, seq, spatial_merge_size, image_token_id,
                       video_token_id, vision_start_token_id, tokens_per_second, counts, position_ids, deltas, batch,
                       status, rows);
    return check_launch("rope_index_fill");
  }
  const size_t lds = static_cast<size_t>(seq) * 5 + 16;
  if (lds > 48 * 1024) {  // above the default cap on dynamic LDS the kernels have to be told
    const int want = static_cast<int>(row_bytes(kMaxSeqLds));
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(rope_index_count<false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, want) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(rope_index_fill<false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, want) != hipSuccess) {
      (void)hipGetLastError();
      return fail(WX_ERR_LAUNCH, "wx_rope_index: cannot raise the dynamic LDS limit");
    }
  }
  hipLaunchKernelGGL(rope_index_count<false>, grid, block, lds, s, input_ids, attention_mask, seq, image_token_id,
                     video_token_id, vision_start_token_id, counts, status, nullptr);
  if (int rc = check_launch("rope_index_count")) return rc;
  hipLaunchKernelGGL(rope_index_fill<false>, grid, block, lds, s, input_ids, attention_mask, image_grid_thw, n_image,
                     video_grid_thw, n_video, second_per_grid_ts, seq, spatial_merge_size, image_token_id,
                     video_token_id, vision_start_token_id, tokens_per_second, counts, position_ids, deltas, batch,
                     status, nullptr);
  return check_launch("rope_index_fill");
}
