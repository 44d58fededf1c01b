// The SwiGLU of the expert FFN on one element: h = min(silu(gate), limit) * clamp(up, +-limit)
// (no clamps without a limit) and its derivatives.  Shared by the stand-alone kernels and the
// grouped-GEMM epilogues so that both give the same bits
// (reference steptronoss/model/common/feed_forward.py:20-26).
#pragma once
#include "common.hpp"

namespace stm {

__device__ __forceinline__ float swiglu_sigmoid(float x) { return 1.f / (1.f + __expf(-x)); }

// Without a limit the clamps compare against infinity and change nothing: one branch-free
// code path serves both cases.
__device__ __forceinline__ float swiglu_bound(bool has_limit, float limit) {
  return has_limit ? limit : __builtin_inff();
}

__device__ __forceinline__ float swiglu_value(float gate, float up, bool has_limit, float limit) {
  const float lim = swiglu_bound(has_limit, limit);
  float a = gate * swiglu_sigmoid(gate);
  a = a > lim ? lim : a;
  const float b = up < -lim ? -lim : (up > lim ? lim : up);
  return a * b;
}

// d gate and d up for an incoming gradient d of h; `value` receives h itself (the same
// arithmetic as swiglu_value).
__device__ __forceinline__ void swiglu_grads(float gate, float up, float d, bool has_limit, float limit, float& d_gate,
                                             float& d_up, float& value) {
  const float lim = swiglu_bound(has_limit, limit);
  const float s = swiglu_sigmoid(gate);
  float a = gate * s;
  float da = s * (1.f + gate * (1.f - s));
  const bool a_clipped = a > lim;  // the clamp passes the gradient on (.., limit]
  a = a_clipped ? lim : a;
  da = a_clipped ? 0.f : da;
  const bool b_low = up < -lim, b_high = up > lim;
  const float b = b_low ? -lim : (b_high ? lim : up);
  const float db = (b_low || b_high) ? 0.f : 1.f;
  d_gate = d * b * da;
  d_up = d * a * db;
  value = a * b;
}

__device__ __forceinline__ void swiglu_grads(float gate, float up, float d, bool has_limit, float limit, float& d_gate,
                                             float& d_up) {
  float value;
  swiglu_grads(gate, up, d, has_limit, limit, d_gate, d_up, value);
}

}  // namespace stm
