// Shared host/device helpers for libwallx_mi355 (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "wallx_mi355.h"

namespace wx {

// Records a formatted message for wx_last_error_string() on this thread and returns `code`.
int fail(int code, const char* fmt, ...);
// hipGetLastError() after a launch; WX_OK or WX_ERR_LAUNCH with the HIP error text recorded.
int check_launch(const char* what);

// Bits of wx_last_gemm_path() for the calling thread: cleared at the start of a dual GEMM call, set as it launches.
void gemm_path_reset();
void gemm_path_note(int bit);

inline hipStream_t as_stream(wx_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

constexpr int kWave = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte lane access

__device__ __forceinline__ int lane_id() { return static_cast<int>(threadIdx.x) & (kWave - 1); }

// ---- 16-bit float <-> fp32, round-to-nearest-even (NaN kept quiet) -------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// gfx950 converts fp32 -> bf16 in hardware (round to nearest even, NaN kept quiet): one instruction, no branches
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

__device__ __forceinline__ float round_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(b)));
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

template <int DT>
struct Elem;  // storage-type traits keyed by wx_dtype
template <>
struct Elem<WX_F32> {
  static constexpr int kBytes = 4;
  __device__ static float round(float f) { return f; }
};
template <>
struct Elem<WX_F16> {
  static constexpr int kBytes = 2;
  __device__ static float load(uint32_t bits) { return f16_bits_to_f32(bits); }
  __device__ static uint32_t store(float f) { return f32_to_f16_bits(f); }
  __device__ static float round(float f) { return f16_bits_to_f32(f32_to_f16_bits(f)); }
};
template <>
struct Elem<WX_BF16> {
  static constexpr int kBytes = 2;
  __device__ static float load(uint32_t bits) { return bf16_bits_to_f32(bits); }
  __device__ static uint32_t store(float f) { return f32_to_bf16_bits(f); }
  __device__ static float round(float f) { return round_bf16(f); }
};

// 16 bytes = 4 fp32 or 8 half-width values, unpacked to / packed from fp32.
template <int DT>
__device__ __forceinline__ void unpack16(const u32x4& v, float* f) {
  if constexpr (DT == WX_F32) {
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
    f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
  } else {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = Elem<DT>::load(w[i] & 0xffffu);
      f[2 * i + 1] = Elem<DT>::load(w[i] >> 16);
    }
  }
}
template <int DT>
__device__ __forceinline__ u32x4 pack16(const float* f) {
  u32x4 v;
  if constexpr (DT == WX_F32) {
    v.x = __float_as_uint(f[0]); v.y = __float_as_uint(f[1]);
    v.z = __float_as_uint(f[2]); v.w = __float_as_uint(f[3]);
  } else {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = Elem<DT>::store(f[2 * i]) | (Elem<DT>::store(f[2 * i + 1]) << 16);
    v.x = w[0]; v.y = w[1]; v.z = w[2]; v.w = w[3];
  }
  return v;
}
template <int DT>
constexpr int elems_per_16() { return DT == WX_F32 ? 4 : 8; }

__device__ __forceinline__ int64_t load_index(const void* p, int itype, int64_t i) {
  switch (itype) {
    case WX_I64: return static_cast<const int64_t*>(p)[i];
    case WX_U8: return static_cast<const uint8_t*>(p)[i];
    default: return static_cast<const int32_t*>(p)[i];
  }
}

// Number of compute units of the current device (cached per thread); 256 on MI355X.
int device_cu_count();

}  // namespace wx
