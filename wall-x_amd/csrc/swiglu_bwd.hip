// Elementwise backward of the SwiGLU inside an expert FFN, h = silu(g) * u (act.py:79-82), for the block's training
// path.  One pass reads gate, up (the two projections, kept by the forward or recomputed) and dh (the gradient
// arriving from the down projection) and writes the three tensors the remaining GEMMs need:
//   hmid  = bf16(bf16(silu(g)) * u)           what the forward fed to the down projection (its eager rounding)
//   dgate = dh * u * s * (1 + g * (1 - s))    with s = sigmoid(g)
//   dup   = dh * silu(g)
// fp32 math, one rounding per output.  HBM-bound: 6 x 2 bytes per element; a thread handles 8 elements (16 bytes).
#include "common.h"
#include "tiled_layout.h"

namespace wx {
namespace {

__device__ __forceinline__ void swiglu_bwd_8(const u32x4& gv, const u32x4& uv, const u32x4& dv, u32x4& hv, u32x4& dgv,
                                             u32x4& duv) {
  float g[8], u[8], d[8], h[8], dg[8], du[8];
  unpack16<WX_BF16>(gv, g);
  unpack16<WX_BF16>(uv, u);
  unpack16<WX_BF16>(dv, d);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float s = 1.0f / (1.0f + __expf(-g[e]));
    const float silu = g[e] * s;
    h[e] = round_bf16(silu) * u[e];
    dg[e] = d[e] * u[e] * s * (1.0f + g[e] * (1.0f - s));
    du[e] = d[e] * silu;
  }
  hv = pack16<WX_BF16>(h);
  dgv = pack16<WX_BF16>(dg);
  duv = pack16<WX_BF16>(du);
}

// The same with gate and up read from the K-tiled buffers the forward's gate/up launch kept (16 x 32 blocks ordered
// [column block][row block], tiled_layout.h); dh and the three outputs are row-major [rows, cols].  A wavefront
// instruction covers 8 rows x 64 columns: 128-byte runs of the row-major tensors, half blocks (512 bytes) of the
// tiled ones.
__global__ __launch_bounds__(256) void swiglu_bwd_tiled_kernel(const unsigned char* __restrict__ gate_t,
                                                               const unsigned char* __restrict__ up_t,
                                                               int64_t tiled_row_blocks, const u32x4* __restrict__ dh,
                                                               u32x4* __restrict__ hmid, u32x4* __restrict__ dgate,
                                                               u32x4* __restrict__ dup, int64_t rows, int64_t cols) {
  const int lane = lane_id();
  const int64_t col_pairs = cols / 64, row_blocks = (rows + kBlkRows - 1) / kBlkRows;
  const int64_t units = row_blocks * col_pairs * 2;  // (row block, pair of column blocks, upper / lower 8 rows)
  const int64_t wave0 = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) / kWave;
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * blockDim.x / kWave;
  for (int64_t unit = wave0; unit < units; unit += n_waves) {
    const int q = static_cast<int>(unit & 1);
    const int64_t kp = (unit >> 1) % col_pairs, rb = (unit >> 1) / col_pairs;
    const int r = q * 8 + (lane >> 3), c8 = lane & 7;
    const int64_t row = rb * kBlkRows + r;
    if (row >= rows) continue;
    const int64_t kb = kp * 2 + (c8 >> 2);
    const int slot = (c8 & 3) ^ ((r >> 2) & 3);
    const int64_t t_off = ((kb * tiled_row_blocks + rb) << 10) + (r << 6) + (slot << 4);
    const int64_t rm = (row * cols + kp * 64 + c8 * 8) / 8;  // 16-byte chunk index in the row-major tensors
    u32x4 hv, dgv, duv;
    swiglu_bwd_8(*reinterpret_cast<const u32x4*>(gate_t + t_off), *reinterpret_cast<const u32x4*>(up_t + t_off),
                 __builtin_nontemporal_load(dh + rm), hv, dgv, duv);
    if (hmid != nullptr) __builtin_nontemporal_store(hv, hmid + rm);
    __builtin_nontemporal_store(dgv, dgate + rm);
    __builtin_nontemporal_store(duv, dup + rm);
  }
}

__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const u32x4* __restrict__ gate, const u32x4* __restrict__ up,
                                                         const u32x4* __restrict__ dh, u32x4* __restrict__ hmid,
                                                         u32x4* __restrict__ dgate, u32x4* __restrict__ dup,
                                                         int64_t chunks) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; c < chunks; c += stride) {
    u32x4 hv, dgv, duv;
    swiglu_bwd_8(__builtin_nontemporal_load(gate + c), __builtin_nontemporal_load(up + c),
                 __builtin_nontemporal_load(dh + c), hv, dgv, duv);
    __builtin_nontemporal_store(hv, hmid + c);
    __builtin_nontemporal_store(dgv, dgate + c);
    __builtin_nontemporal_store(duv, dup + c);
  }
}

}  // namespace
}  // namespace wx

using namespace wx;

extern "C" int wx_swiglu_bwd(const void* gate, const void* up, const void* dh, void* hmid, void* dgate, void* dup,
                             int64_t num_elems, wx_stream_t stream) {
  const char* who = "wx_swiglu_bwd";
  if (num_elems < 0) return fail(WX_ERR_INVALID_ARGUMENT, "%s: negative size", who);
  if (num_elems % 8 != 0) return fail(WX_ERR_UNSUPPORTED, "%s: num_elems must be a multiple of 8", who);
  if (num_elems == 0) return WX_OK;
  if (!gate || !up || !dh || !hmid || !dgate || !dup) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  const void* all[6] = {gate, up, dh, hmid, dgate, dup};
  for (const void* ptr : all)
    if (reinterpret_cast<uintptr_t>(ptr) & 15) return fail(WX_ERR_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", who);
  const int64_t chunks = num_elems / 8;
  const int64_t want = (chunks + 255) / 256;
  const int64_t cap = static_cast<int64_t>(device_cu_count()) * 16;
  hipLaunchKernelGGL(swiglu_bwd_kernel, dim3(static_cast<unsigned>(want < cap ? want : cap)), dim3(256), 0,
                     as_stream(stream), static_cast<const u32x4*>(gate), static_cast<const u32x4*>(up),
                     static_cast<const u32x4*>(dh), static_cast<u32x4*>(hmid), static_cast<u32x4*>(dgate),
                     static_cast<u32x4*>(dup), chunks);
  return check_launch("swiglu_bwd_kernel");
}

extern "C" int wx_swiglu_bwd_tiled(const void* gate_tiled, const void* up_tiled, int64_t tiled_rows, const void* dh,
                                   void* hmid, void* dgate, void* dup, int64_t rows, int64_t cols, wx_stream_t stream) {
  const char* who = "wx_swiglu_bwd_tiled";
  if (rows < 0 || cols < 0 || tiled_rows < rows) return fail(WX_ERR_INVALID_ARGUMENT, "%s: bad sizes", who);
  if (cols % 64 != 0 || tiled_rows % kBlkRows != 0)
    return fail(WX_ERR_UNSUPPORTED, "%s: cols must be a multiple of 64 and tiled_rows of 16", who);
  if (rows == 0 || cols == 0) return WX_OK;
  if (!gate_tiled || !up_tiled || !dh || !dgate || !dup) return fail(WX_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
  const void* all[6] = {gate_tiled, up_tiled, dh, hmid, dgate, dup};  // hmid may be null: that output is not wanted
  for (const void* ptr : all)
    if (reinterpret_cast<uintptr_t>(ptr) & 15) return fail(WX_ERR_INVALID_ARGUMENT, "%s: buffers must be 16-byte aligned", who);
  const int64_t units = (rows + kBlkRows - 1) / kBlkRows * (cols / 64) * 2;
  const int64_t want = (units + 3) / 4;
  const int64_t cap = static_cast<int64_t>(device_cu_count()) * 16;
  hipLaunchKernelGGL(swiglu_bwd_tiled_kernel, dim3(static_cast<unsigned>(want < cap ? want : cap)), dim3(256), 0,
                     as_stream(stream), static_cast<const unsigned char*>(gate_tiled),
                     static_cast<const unsigned char*>(up_tiled), tiled_rows / kBlkRows, static_cast<const u32x4*>(dh),
                     static_cast<u32x4*>(hmid), static_cast<u32x4*>(dgate), static_cast<u32x4*>(dup), rows, cols);
  return check_launch("swiglu_bwd_tiled_kernel");
}
