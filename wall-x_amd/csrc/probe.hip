// Measurement probe: how fast one CU's MFMA pipes run bf16 32x32x16 instructions back to back on GIVEN operand
// values, with no LDS or memory traffic in the loop.  The rate depends on the values (switching activity moves
// the sustained clock), so benchmarks time this on the same kind of data as the GEMM they are judging: it is the
// ceiling an MFMA-bound kernel can reach on that data, below the nominal peak.
//
// Benchmark-only: built into its own library (libwallx_probe.so) next to the product library, never linked into it
// and not part of its C ABI.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace wx {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kProbeAcc = 8;       // independent accumulator blocks per wave (128 registers)
constexpr int kProbeFrags = 8;     // operand fragments per wave, 16 bytes per lane each
constexpr int kProbeMfmaPerIter = 32;

__global__ __launch_bounds__(256, 1) void mfma_rate_kernel(const u32x4* __restrict__ operands, int iters,
                                                            float* __restrict__ sink) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  bf16x8 f[kProbeFrags];
#pragma unroll
  for (int i = 0; i < kProbeFrags; ++i)
    f[i] = __builtin_bit_cast(bf16x8, operands[(wave * kProbeFrags + i) * 64 + lane]);
  f32x16 acc[kProbeAcc];
#pragma unroll
  for (int i = 0; i < kProbeAcc; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < kProbeMfmaPerIter; ++u)
      acc[u % kProbeAcc] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[u % kProbeFrags], f[(u + 3) % kProbeFrags],
                                                                   acc[u % kProbeAcc], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < kProbeAcc; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  if (s == 123.456f) sink[0] = s;  // keeps the loop alive; practically never true
#endif
}

}  // namespace
}  // namespace wx

using namespace wx;

extern "C" size_t wxprobe_mfma_operand_bytes(void) { return static_cast<size_t>(4) * kProbeFrags * 64 * 16; }

// Runs `iters` x 32 MFMAs per wave on every CU, operands (wxprobe_mfma_operand_bytes() bytes of bf16 values, device
// memory, 16-byte aligned) held in registers.  *flops_per_launch (host pointer, may be NULL) receives the flops one
// launch performs; sink is one float of device memory that is practically never written.  Returns 0, -1 for bad
// arguments, -4 when the launch failed.
extern "C" int wxprobe_mfma_rate(const void* operands, int iters, float* sink, double* flops_per_launch, void* stream) {
  if (!operands || !sink || (reinterpret_cast<uintptr_t>(operands) & 15) || iters < 1 || iters > (1 << 24)) return -1;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return -4;
  if (flops_per_launch)
    *flops_per_launch = 2.0 * 32 * 32 * 16 * kProbeMfmaPerIter * static_cast<double>(iters) * 4 * cus;
  hipLaunchKernelGGL(mfma_rate_kernel, dim3(cus), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     static_cast<const u32x4*>(operands), iters, sink);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}
