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
  // the hardware conversion of gfx950 (v_cvt_pk_bf16_f32): round to nearest even, quiet NaNs
  return bf16_t{__builtin_bit_cast(uint16_t, static_cast<__bf16>(f))};
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

// ---- wave-wide reductions of 32-bit values on the DPP path (row shifts inside the 16-lane rows,
// then two row broadcasts; the total arrives in lane 63 and is handed to every lane through a
// scalar register).  An order of magnitude less latency than six dependent LDS-crossbar
// shuffles, which is what the routing kernels are made of.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_move(int keep, int src) {
  return __builtin_amdgcn_update_dpp(keep, src, CTRL, ROW_MASK, 0xf, false);
}

template <typename T, typename Op>
__device__ __forceinline__ T wave_reduce_dpp(T v, T identity, Op op) {
  static_assert(sizeof(T) == 4, "32-bit values");
  const int id = __builtin_bit_cast(int, identity);
#define STM_DPP_STEP(CTRL, MASK) v = op(v, __builtin_bit_cast(T, dpp_move<CTRL, MASK>(id, __builtin_bit_cast(int, v))))
  STM_DPP_STEP(0x111, 0xf);  // row_shr:1
  STM_DPP_STEP(0x112, 0xf);  // row_shr:2
  STM_DPP_STEP(0x114, 0xf);  // row_shr:4
  STM_DPP_STEP(0x118, 0xf);  // row_shr:8   -> lane 15 of every row holds the row's total
  STM_DPP_STEP(0x142, 0xa);  // row_bcast:15 into rows 1 and 3
  STM_DPP_STEP(0x143, 0xc);  // row_bcast:31 into rows 2 and 3 -> lane 63 holds the total
#undef STM_DPP_STEP
  return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
  if constexpr (sizeof(T) == 4) {
    return wave_reduce_dpp(v, T(0), [](T a, T b) { return a + b; });
  } else {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
  }
}

// (callers pass values for which the smallest representable number is a neutral element)
__device__ __forceinline__ float wave_max(float v) {
  return wave_reduce_dpp(v, -__builtin_inff(), [](float a, float b) { return fmaxf(a, b); });
}
__device__ __forceinline__ int32_t wave_max(int32_t v) {
  return wave_reduce_dpp(v, int32_t(0x80000000), [](int32_t a, int32_t b) { return a > b ? a : b; });
}

// (value, index) arg-max over the wave: larger value wins, equal values -> smaller index.
__device__ __forceinline__ void wave_argmax(float& v, int& idx) {
  const int neutral_v = __builtin_bit_cast(int, -__builtin_inff());
#define STM_DPP_STEP(CTRL, MASK)                                                                   \
  {                                                                                                \
    const float ov = __builtin_bit_cast(float, dpp_move<CTRL, MASK>(neutral_v, __builtin_bit_cast(int, v))); \
    const int oi = dpp_move<CTRL, MASK>(0x7fffffff, idx);                                          \
    if (ov > v || (ov == v && oi < idx)) {                                                         \
      v = ov;                                                                                      \
      idx = oi;                                                                                    \
    }                                                                                              \
  }
  STM_DPP_STEP(0x111, 0xf)
  STM_DPP_STEP(0x112, 0xf)
  STM_DPP_STEP(0x114, 0xf)
  STM_DPP_STEP(0x118, 0xf)
  STM_DPP_STEP(0x142, 0xa)
  STM_DPP_STEP(0x143, 0xc)
#undef STM_DPP_STEP
  v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
  idx = __builtin_amdgcn_readlane(idx, 63);
}

// In-place exclusive scan of a[0..n) in LDS by the whole workgroup; returns the total.
// n <= 4 * blockDim.x.
__device__ inline int32_t block_exclusive_scan(int32_t* a, int n, int32_t* wave_sums) {
  const int tid = threadIdx.x;
  const int lane = tid % kWave;
  const int wave = tid / kWave;
  const int n_waves = blockDim.x / kWave;
  int32_t v[4];
  int32_t mine = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = tid * 4 + j;
    v[j] = i < n ? a[i] : 0;
    mine += v[j];
  }
  int32_t incl = mine;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int32_t o = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += o;
  }
  if (lane == kWave - 1) wave_sums[wave] = incl;
  __syncthreads();
  int32_t before = 0, total = 0;
  for (int w = 0; w < n_waves; ++w) {
    const int32_t s = wave_sums[w];
    if (w < wave) before += s;
    total += s;
  }
  int32_t run = before + incl - mine;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = tid * 4 + j;
    if (i < n) a[i] = run;
    run += v[j];
  }
  __syncthreads();
  return total;
}

// ----- host-side helpers -------------------------------------------------------------
inline hipStream_t as_stream(stm_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? STM_OK : STM_ERR_LAUNCH;
}

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Stable sort of the valid slots of a position map by the row they name (routing.hip); used
// by the combine backward when several slots name one row.
size_t sort_by_row_workspace_bytes(int64_t n_slots, int64_t n_rows);
int sort_slots_by_row(const void* pos, int pos_is_i64, int64_t n_slots, int64_t n_rows, int32_t* sorted_row,
                      int32_t* sorted_slot, int32_t* n_valid_out, void* workspace, size_t workspace_bytes,
                      hipStream_t stream);

}  // namespace stm
