// The SwiGLU of the expert FFN on one element: h = min(silu(gate), limit) * clamp(up, +-limit)
// (no clamps without a limit) and its derivatives.  Shared by the stand-alone kernels and the
// grouped-GEMM epilogues so that both compute the same fp32 values
// (reference steptronoss/model/common/feed_forward.py:20-26).
#pragma once
#include "common.hpp"

namespace stm {

// 1 / (1 + e^-x) with the hardware exponential and reciprocal (each within one fp32 ulp; an
// IEEE-rounded division would cost ten instructions per element of an epilogue that is bound by
// instruction issue, for a digit that the 16-bit rounding of the result discards).
__device__ __forceinline__ float swiglu_sigmoid(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }

// kLimit = false compiles the clamps away; callers branch once (or are instantiated) per case
// instead of once per element.
template <bool kLimit>
__device__ __forceinline__ float swiglu_value_t(float gate, float up, float lim) {
  float a = gate * swiglu_sigmoid(gate);
  float b = up;
  if constexpr (kLimit) {
    a = a > lim ? lim : a;
    b = up < -lim ? -lim : (up > lim ? lim : up);
  }
  return a * b;
}

// d gate and d up for an incoming gradient d of h; `value` receives h itself (the same
// arithmetic as swiglu_value_t).
template <bool kLimit>
__device__ __forceinline__ void swiglu_grads_t(float gate, float up, float d, float lim, float& d_gate, float& d_up,
                                               float& value) {
  const float s = swiglu_sigmoid(gate);
  float a = gate * s;
  float da = s * (1.f + gate * (1.f - s));
  float b = up;
  float db = 1.f;
  if constexpr (kLimit) {
    const bool a_clipped = a > lim;  // the clamp passes the gradient on (.., limit]
    a = a_clipped ? lim : a;
    da = a_clipped ? 0.f : da;
    const bool b_low = up < -lim, b_high = up > lim;
    b = b_low ? -lim : (b_high ? lim : up);
    db = (b_low || b_high) ? 0.f : 1.f;
  }
  d_gate = d * b * da;
  d_up = d * a * db;
  value = a * b;
}

}  // namespace stm
