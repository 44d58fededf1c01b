// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/steptron_moe.h"

namespace stm {

constexpr int kWave = 64;  // CDNA wavefront width

// ----- element types (raw storage; arithmetic is always done in fp32) ---------
struct bf16_t {
  uint16_t bits;
};
struct f16_t {
  _Float16 v;
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float(uint32_t(x.bits) << 16); }
__device__ __forceinline__ float to_float(f16_t x) { return float(x.v); }

// round-to-nearest-even, NaN kept quiet
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return uint16_t(u >> 16);
}

template <typename T>
__device__ __forceinline__ T from_float(float f);
template <>
__device__ __forceinline__ float from_float<float>(float f) {
  return f;
}
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  return bf16_t{f32_to_bf16_bits(f)};
}
template <>
__device__ __forceinline__ f16_t from_float<f16_t>(float f) {
  return f16_t{_Float16(f)};
}

// ----- wave-level helpers ----------------------------------------------------------
__device__ __forceinline__ int lane_id() { return __lane_id(); }

__device__ __forceinline__ uint64_t lanemask_lt() {
  const int l = lane_id();
  return l == 0 ? 0ull : (~0ull >> (64 - l));
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

template <typename T>
__device__ __forceinline__ T wave_max(T v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    T o = __shfl_xor(v, off, kWave);
    v = o > v ? o : v;
  }
  return v;
}

// ----- host-side helpers -------------------------------------------------------------
inline hipStream_t as_stream(stm_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? STM_OK : STM_ERR_LAUNCH;
}

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace stm
