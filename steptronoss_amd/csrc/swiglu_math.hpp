// The SwiGLU of the expert FFN on one element: h = min(silu(gate), limit) * clamp(up, +-limit)
// (no clamps without a limit) and its derivatives.  Shared by the stand-alone kernels and the
// grouped-GEMM epilogues so that both give the same bits
// (reference steptronoss/model/common/feed_forward.py:20-26).
#pragma once
#include "common.hpp"

namespace stm {

__device__ __forceinline__ float swiglu_sigmoid(float x) { return 1.f / (1.f + __expf(-x)); }

__device__ __forceinline__ float swiglu_value(float gate, float up, bool has_limit, float limit) {
  float a = gate * swiglu_sigmoid(gate);
  float b = up;
  if (has_limit) {
    a = fminf(a, limit);
    b = fminf(fmaxf(b, -limit), limit);
  }
  return a * b;
}

// d gate and d up for an incoming gradient d of h.
__device__ __forceinline__ void swiglu_grads(float gate, float up, float d, bool has_limit, float limit, float& d_gate,
                                             float& d_up) {
  const float s = swiglu_sigmoid(gate);
  float a = gate * s;
  float da = s * (1.f + gate * (1.f - s));
  float b = up;
  float db = 1.f;
  if (has_limit) {
    if (a > limit) da = 0.f;  // the clamp passes the gradient on (.., limit]
    a = fminf(a, limit);
    if (b < -limit || b > limit) db = 0.f;
    b = fminf(fmaxf(b, -limit), limit);
  }
  d_gate = d * b * da;
  d_up = d * a * db;
}

}  // namespace stm
