// Vision-tower index builders for gfx950: rotary (h, w) ids + frequency table, and the window
// attention permutation.  Semantics: vl.py:473-500 and vl.py:502-547 of the reference.
//
// Both are closed forms of the output index, so each is ONE launch with one thread per output element
// (no per-window counting, no serial prefix, no host round trip): every workgroup rebuilds the tiny
// per-image prefix table in LDS and threads binary-search it.
#include "common.h"
#include "grid_prefix.h"

namespace wx {
namespace {

constexpr int kThreads = 256;

// ---- rot_pos -------------------------------------------------------------------------------------
// Patch n of an image with grid (t, h, w), merge m: frames repeat every h*w patches; inside a frame
// patches are ordered by m x m merge block (row-major over blocks), then row-major inside the block.
__device__ __forceinline__ void patch_hw(int32_t local, int32_t h, int32_t w, int m, int32_t& hp, int32_t& wp) {
  const int32_t spatial = local % (h * w);
  const int32_t blk = spatial / (m * m), within = spatial - blk * (m * m);
  const int32_t blocks_w = w / m;
  hp = (blk / blocks_w) * m + within / m;
  wp = (blk % blocks_w) * m + within % m;
}

template <int VEC>
__global__ __launch_bounds__(kThreads) void rot_pos_kernel(const float* __restrict__ inv_freq, int n_freq,
                                                           const void* __restrict__ grid_thw, int grid_type,
                                                           int n_grid, int merge, int64_t total,
                                                           float* __restrict__ table,
                                                           int64_t* __restrict__ pos_ids) {
  __shared__ int32_t s_prefix[kMaxGrids + 1];
  for (int g = threadIdx.x; g < n_grid; g += kThreads) {
    int64_t t, h, w;
    load_thw(grid_thw, grid_type, g, t, h, w);
    s_prefix[g] = static_cast<int32_t>(t * h * w);
  }
  lds_exclusive_scan(s_prefix, n_grid);
  const int per_row = 2 * n_freq / VEC;  // output vectors per patch
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t n = idx / per_row;
  if (n >= total || n >= s_prefix[n_grid]) return;
  const int c = static_cast<int>(idx - n * per_row);
  const int g = find_owner(s_prefix, n_grid, static_cast<int32_t>(n));
  int64_t t, h, w;
  load_thw(grid_thw, grid_type, g, t, h, w);
  int32_t hp, wp;
  patch_hw(static_cast<int32_t>(n) - s_prefix[g], static_cast<int32_t>(h), static_cast<int32_t>(w), merge, hp, wp);
  if (pos_ids != nullptr && c == 0) {
    pos_ids[2 * n] = hp;
    pos_ids[2 * n + 1] = wp;
  }
  if (table == nullptr) return;
  float out[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    const int col = c * VEC + e;  // [0, n_freq): h half, [n_freq, 2 n_freq): w half
    const bool is_h = col < n_freq;
    // one fp32 product, as outer(arange, inv_freq)[id] in the reference (vl.py:114-119, 496-499)
    out[e] = __fmul_rn(static_cast<float>(is_h ? hp : wp), inv_freq[is_h ? col : col - n_freq]);
  }
  float* dst = table + n * 2 * n_freq + c * VEC;
  if constexpr (VEC == 4) {
    *reinterpret_cast<float4*>(dst) = make_float4(out[0], out[1], out[2], out[3]);
  } else {
    dst[0] = out[0];
  }
}

// ---- window_index --------------------------------------------------------------------------------
struct WinGeom {
  int32_t gh, gw;    // merged grid
  int32_t nwh, nww;  // windows per axis (ceil)
};
__device__ __forceinline__ WinGeom geom(int64_t h, int64_t w, int merge, int ws) {
  WinGeom g;
  g.gh = static_cast<int32_t>(h / merge);
  g.gw = static_cast<int32_t>(w / merge);
  g.nwh = (g.gh + ws - 1) / ws;
  g.nww = (g.gw + ws - 1) / ws;
  return g;
}

// One thread per output slot.  Slots [0, total_tokens) are window_index entries; slots
// [total_tokens, total_tokens + total_windows] are cu_window_seqlens entries.
__global__ __launch_bounds__(kThreads) void window_index_kernel(const void* __restrict__ grid_thw, int grid_type,
                                                                int n_grid, int merge, int ws, int unit,
                                                                int64_t total_tokens, int64_t total_windows,
                                                                int32_t* __restrict__ window_index,
                                                                int32_t* __restrict__ cu_seqlens) {
  __shared__ int32_t s_tok[kMaxGrids + 1];  // merged tokens before each image
  __shared__ int32_t s_win[kMaxGrids + 1];  // windows before each image
  for (int g = threadIdx.x; g < n_grid; g += kThreads) {
    int64_t t, h, w;
    load_thw(grid_thw, grid_type, g, t, h, w);
    const WinGeom gm = geom(h, w, merge, ws);
    s_tok[g] = static_cast<int32_t>(t) * gm.gh * gm.gw;
    s_win[g] = static_cast<int32_t>(t) * gm.nwh * gm.nww;
  }
  lds_exclusive_scan(s_tok, n_grid);
  lds_exclusive_scan(s_win, n_grid);
  const int64_t slot = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (slot < total_tokens) {
    if (slot >= s_tok[n_grid]) return;
    const int g = find_owner(s_tok, n_grid, static_cast<int32_t>(slot));
    int64_t t, h, w;
    load_thw(grid_thw, grid_type, g, t, h, w);
    const WinGeom gm = geom(h, w, merge, ws);
    const int32_t frame = gm.gh * gm.gw;
    const int32_t local = static_cast<int32_t>(slot) - s_tok[g];
    const int32_t f = local / frame;
    int32_t r = local - f * frame;
    // window row: full rows of windows hold ws*gw cells each, the last one holds the remainder
    int32_t wh = r / (ws * gm.gw);
    if (wh > gm.nwh - 1) wh = gm.nwh - 1;
    r -= wh * ws * gm.gw;
    const int32_t vh = wh < gm.nwh - 1 ? ws : gm.gh - (gm.nwh - 1) * ws;  // valid rows in this window row
    int32_t ww = r / (vh * ws);
    if (ww > gm.nww - 1) ww = gm.nww - 1;
    r -= ww * vh * ws;
    const int32_t vw = ww < gm.nww - 1 ? ws : gm.gw - (gm.nww - 1) * ws;
    const int32_t cr = r / vw, cc = r - cr * vw;
    window_index[slot] = s_tok[g] + f * frame + (wh * ws + cr) * gm.gw + ww * ws + cc;
  } else if (slot <= total_tokens + total_windows) {
    const int64_t wi = slot - total_tokens;
    if (wi >= s_win[n_grid]) {
      if (wi == s_win[n_grid] && wi == total_windows) cu_seqlens[wi] = s_tok[n_grid] * unit;
      return;
    }
    const int g = find_owner(s_win, n_grid, static_cast<int32_t>(wi));
    int64_t t, h, w;
    load_thw(grid_thw, grid_type, g, t, h, w);
    const WinGeom gm = geom(h, w, merge, ws);
    const int32_t per_frame = gm.nwh * gm.nww;
    const int32_t local = static_cast<int32_t>(wi) - s_win[g];
    const int32_t f = local / per_frame, r = local - f * per_frame;
    const int32_t wh = r / gm.nww, ww = r - wh * gm.nww;
    const int32_t vh = wh < gm.nwh - 1 ? ws : gm.gh - (gm.nwh - 1) * ws;
    // cells before this window: earlier images, earlier frames, earlier window rows, earlier windows
    const int32_t before = s_tok[g] + f * gm.gh * gm.gw + wh * ws * gm.gw + ww * vh * ws;
    cu_seqlens[wi] = before * unit;
  }
}

int check_grid(const char* who, const void* grid_thw, int grid_type, int64_t n_grid) {
  if (grid_type != WX_I32 && grid_type != WX_I64) return fail(WX_ERR_INVALID_ARGUMENT, "%s: grid_thw must be int32 or int64", who);
  if (n_grid < 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: negative n_grid", who);
  if (n_grid > kMaxGrids) return fail(WX_ERR_UNSUPPORTED, "%s: more than %d grids", who, kMaxGrids);
  if (n_grid > 0 && grid_thw == nullptr) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null grid_thw", who);
  return WX_OK;
}

}  // namespace
}  // namespace wx

using namespace wx;

extern "C" int wx_rot_pos_emb(const float* inv_freq, int n_freq, const void* grid_thw, int grid_type, int64_t n_grid,
                              int spatial_merge_size, int64_t total_patches, float* table, int64_t* pos_ids,
                              wx_stream_t stream) {
  if (int rc = check_grid("wx_rot_pos_emb", grid_thw, grid_type, n_grid)) return rc;
  if (spatial_merge_size <= 0) return fail(WX_ERR_INVALID_ARGUMENT, "wx_rot_pos_emb: spatial_merge_size must be positive");
  if (n_freq <= 0 || total_patches < 0) return fail(WX_ERR_INVALID_ARGUMENT, "wx_rot_pos_emb: bad sizes");
  if (total_patches > INT32_MAX / 2) return fail(WX_ERR_UNSUPPORTED, "wx_rot_pos_emb: too many patches");
  if (total_patches == 0 || n_grid == 0) return WX_OK;
  if (table != nullptr && inv_freq == nullptr) return fail(WX_ERR_INVALID_ARGUMENT, "wx_rot_pos_emb: null inv_freq");
  if (table == nullptr && pos_ids == nullptr) return WX_OK;
  hipStream_t s = as_stream(stream);
  const bool vec4 = (n_freq % 4 == 0) && (reinterpret_cast<uintptr_t>(table) % 16 == 0);
  const int per_row = vec4 ? 2 * n_freq / 4 : 2 * n_freq;
  const int64_t threads = total_patches * per_row;
  const dim3 grid(static_cast<unsigned>((threads + kThreads - 1) / kThreads)), block(kThreads);
  if (vec4) {
    hipLaunchKernelGGL(rot_pos_kernel<4>, grid, block, 0, s, inv_freq, n_freq, grid_thw, grid_type,
                       static_cast<int>(n_grid), spatial_merge_size, total_patches, table, pos_ids);
  } else {
    hipLaunchKernelGGL(rot_pos_kernel<1>, grid, block, 0, s, inv_freq, n_freq, grid_thw, grid_type,
                       static_cast<int>(n_grid), spatial_merge_size, total_patches, table, pos_ids);
  }
  return check_launch("rot_pos_kernel");
}

extern "C" int wx_window_index(const void* grid_thw, int grid_type, int64_t n_grid, int spatial_merge_size,
                               int vit_merger_window_size, int spatial_merge_unit, int64_t total_tokens,
                               int64_t total_windows, int32_t* window_index, int32_t* cu_window_seqlens,
                               wx_stream_t stream) {
  if (int rc = check_grid("wx_window_index", grid_thw, grid_type, n_grid)) return rc;
  if (spatial_merge_size <= 0 || vit_merger_window_size <= 0)
    return fail(WX_ERR_INVALID_ARGUMENT, "wx_window_index: merge and window size must be positive");
  if (total_tokens < 0 || total_windows < 0) return fail(WX_ERR_INVALID_ARGUMENT, "wx_window_index: negative totals");
  if (total_tokens > INT32_MAX / 2 / (spatial_merge_unit > 0 ? spatial_merge_unit : 1))
    return fail(WX_ERR_UNSUPPORTED, "wx_window_index: too many tokens for int32 offsets");
  if (cu_window_seqlens == nullptr || (total_tokens > 0 && window_index == nullptr))
    return fail(WX_ERR_INVALID_ARGUMENT, "wx_window_index: null output");
  const int64_t slots = total_tokens + total_windows + 1;
  const dim3 grid(static_cast<unsigned>((slots + kThreads - 1) / kThreads)), block(kThreads);
  hipLaunchKernelGGL(window_index_kernel, grid, block, 0, as_stream(stream), grid_thw, grid_type,
                     static_cast<int>(n_grid), spatial_merge_size, vit_merger_window_size, spatial_merge_unit,
                     total_tokens, total_windows, window_index, cu_window_seqlens);
  return check_launch("window_index_kernel");
}
