// bf16 / fp16 matrix transpose: a utility for callers that want a transposed copy (the dual GEMM itself reads every
// operand layout in place).
//
// 64 x 64 element tiles through LDS: 16-byte global reads along the source rows, 2-byte LDS writes into the
// transposed position, 16-byte reads of the transposed rows, 16-byte global stores.
#include "common.h"

namespace wx {
namespace {

constexpr int kT = 64;          // tile edge in elements
constexpr int kPitch = kT + 8;  // LDS row pitch in elements: keeps 16-byte alignment and spreads the banks

__global__ __launch_bounds__(256) void transpose16_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                          int64_t rows, int64_t cols) {
  __shared__ __attribute__((aligned(16))) uint16_t tile[kT * kPitch];  // tile[c][r]
  const int64_t tiles_c = (cols + kT - 1) / kT;
  const int64_t r0 = (blockIdx.x / tiles_c) * kT, c0 = (blockIdx.x % tiles_c) * kT;
  const int lr = threadIdx.x >> 3, lc = (threadIdx.x & 7) * 8;  // 32 rows x 8 chunks per pass
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int r = lr + 32 * pass;
    if (r0 + r < rows && c0 + lc < cols) {  // cols is a multiple of 8: a chunk is inside or outside as a whole
      const u32x4 v = *reinterpret_cast<const u32x4*>(src + (r0 + r) * cols + c0 + lc);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        tile[(lc + e) * kPitch + r] = static_cast<uint16_t>(e & 1 ? w[e >> 1] >> 16 : w[e >> 1] & 0xffffu);
    }
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int c = lr + 32 * pass;  // row of the transposed tile
    if (c0 + c < cols && r0 + lc < rows) {  // rows is a multiple of 8
      const u32x4 v = *reinterpret_cast<const u32x4*>(&tile[c * kPitch + lc]);
      *reinterpret_cast<u32x4*>(dst + (c0 + c) * rows + r0 + lc) = v;
    }
  }
}

}  // namespace
}  // namespace wx

using namespace wx;

extern "C" int wx_transpose_2d(const void* src, void* dst, int64_t rows, int64_t cols, int elem_bytes,
                               wx_stream_t stream) {
  if (rows < 0 || cols < 0) return fail(WX_ERR_INVALID_ARGUMENT, "wx_transpose_2d: negative size");
  if (elem_bytes != 2) return fail(WX_ERR_UNSUPPORTED, "wx_transpose_2d: only 2-byte elements");
  if (rows % 8 != 0 || cols % 8 != 0)
    return fail(WX_ERR_UNSUPPORTED, "wx_transpose_2d: rows (%lld) and cols (%lld) must be multiples of 8",
                static_cast<long long>(rows), static_cast<long long>(cols));
  if (rows == 0 || cols == 0) return WX_OK;
  if (!src || !dst) return fail(WX_ERR_INVALID_ARGUMENT, "wx_transpose_2d: null pointer");
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15)
    return fail(WX_ERR_INVALID_ARGUMENT, "wx_transpose_2d: buffers must be 16-byte aligned");
  const int64_t tiles = ((rows + kT - 1) / kT) * ((cols + kT - 1) / kT);
  if (tiles > 0x7fffffffll) return fail(WX_ERR_UNSUPPORTED, "wx_transpose_2d: matrix too large");
  hipLaunchKernelGGL(transpose16_kernel, dim3(static_cast<unsigned>(tiles)), dim3(256), 0, as_stream(stream),
                     static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), rows, cols);
  return check_launch("transpose16_kernel");
}
