// Elementwise backward of the SwiGLU inside an expert FFN, h = silu(g) * u (act.py:79-82), for the block's training
// path.  One pass reads gate, up (the recomputed projections) and dh (the gradient arriving from the down
// projection) and writes the three tensors the remaining GEMMs need:
//   hmid  = bf16(bf16(silu(g)) * u)           what the forward fed to the down projection (its eager rounding)
//   dgate = dh * u * s * (1 + g * (1 - s))    with s = sigmoid(g)
//   dup   = dh * silu(g)
// fp32 math, one rounding per output.  HBM-bound: 6 x 2 bytes per element; a thread handles 8 elements (16 bytes).
#include "common.h"

namespace wx {
namespace {

__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const u32x4* __restrict__ gate, const u32x4* __restrict__ up,
                                                         const u32x4* __restrict__ dh, u32x4* __restrict__ hmid,
                                                         u32x4* __restrict__ dgate, u32x4* __restrict__ dup,
                                                         int64_t chunks) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; c < chunks; c += stride) {
    float g[8], u[8], d[8], h[8], dg[8], du[8];
    unpack16<WX_BF16>(__builtin_nontemporal_load(gate + c), g);
    unpack16<WX_BF16>(__builtin_nontemporal_load(up + c), u);
    unpack16<WX_BF16>(__builtin_nontemporal_load(dh + c), d);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float s = 1.0f / (1.0f + __expf(-g[e]));
      const float silu = g[e] * s;
      h[e] = round_bf16(silu) * u[e];
      dg[e] = d[e] * u[e] * s * (1.0f + g[e] * (1.0f - s));
      du[e] = d[e] * silu;
    }
    __builtin_nontemporal_store(pack16<WX_BF16>(h), hmid + c);
    __builtin_nontemporal_store(pack16<WX_BF16>(dg), dgate + c);
    __builtin_nontemporal_store(pack16<WX_BF16>(du), dup + c);
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
