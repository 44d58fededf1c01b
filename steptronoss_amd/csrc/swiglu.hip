// SwiGLU between the two expert GEMMs: h = silu(gate) * up with gate = gu[:, :F], up = gu[:, F:],
// optional clamp (gate side from above after the SiLU, up side to [-limit, limit]); and its
// backward.  Element-wise, 128-bit accesses, fp32 math, one rounding per output.
#include "swiglu_math.hpp"

namespace stm {
namespace {

template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) Pack {
  T v[VEC];
};

// LIMIT is a template argument so that the code without a limit carries no clamps; the GEMM
// epilogues instantiate the same per-element functions.
template <typename T, int VEC, bool LIMIT>
__global__ __launch_bounds__(256) void swiglu_fwd_kernel(const T* __restrict__ gu, T* __restrict__ h, int64_t rows,
                                                         int64_t f, const int32_t* __restrict__ rows_dev, float limit) {
  using P = Pack<T, VEC>;
  const int64_t per_row = f / VEC;
  const int64_t live = rows_dev ? (rows_dev[0] < rows ? rows_dev[0] : rows) : rows;
  const int64_t total = live * per_row;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += int64_t(gridDim.x) * blockDim.x) {
    const int64_t r = i / per_row, c = (i % per_row) * VEC;
    const P g = *reinterpret_cast<const P*>(gu + r * 2 * f + c);
    const P u = *reinterpret_cast<const P*>(gu + r * 2 * f + f + c);
    P o;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      o.v[j] = from_float<T>(swiglu_value_t<LIMIT>(to_float(g.v[j]), to_float(u.v[j]), limit));
    }
    *reinterpret_cast<P*>(h + r * f + c) = o;
  }
}

template <typename T, int VEC, bool LIMIT>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ gu, const T* __restrict__ dh,
                                                         T* __restrict__ dgu, int64_t rows, int64_t f,
                                                         const int32_t* __restrict__ rows_dev, float limit) {
  using P = Pack<T, VEC>;
  const int64_t per_row = f / VEC;
  const int64_t live = rows_dev ? (rows_dev[0] < rows ? rows_dev[0] : rows) : rows;
  const int64_t total = live * per_row;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += int64_t(gridDim.x) * blockDim.x) {
    const int64_t r = i / per_row, c = (i % per_row) * VEC;
    const P g = *reinterpret_cast<const P*>(gu + r * 2 * f + c);
    const P u = *reinterpret_cast<const P*>(gu + r * 2 * f + f + c);
    const P d = *reinterpret_cast<const P*>(dh + r * f + c);
    P og, ou;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float dg, du, value;
      swiglu_grads_t<LIMIT>(to_float(g.v[j]), to_float(u.v[j]), to_float(d.v[j]), limit, dg, du, value);
      og.v[j] = from_float<T>(dg);
      ou.v[j] = from_float<T>(du);
    }
    *reinterpret_cast<P*>(dgu + r * 2 * f + c) = og;
    *reinterpret_cast<P*>(dgu + r * 2 * f + f + c) = ou;
  }
}

inline unsigned grid_for(int64_t work_items) {
  const int64_t blocks = (work_items + 255) / 256;
  return unsigned(blocks < 1 ? 1 : (blocks > 65536 ? 65536 : blocks));
}

template <typename T, bool LIMIT>
int fwd_limit(const void* gu, void* h, int64_t rows, int64_t f, const int32_t* rows_dev, float limit, hipStream_t s) {
  constexpr int W = 16 / int(sizeof(T));
  const bool vec = f % W == 0 && aligned_to(gu, 16) && aligned_to(h, 16);
  if (vec)
    swiglu_fwd_kernel<T, W, LIMIT><<<grid_for(rows * (f / W)), 256, 0, s>>>(static_cast<const T*>(gu),
                                                                            static_cast<T*>(h), rows, f, rows_dev, limit);
  else
    swiglu_fwd_kernel<T, 1, LIMIT><<<grid_for(rows * f), 256, 0, s>>>(static_cast<const T*>(gu), static_cast<T*>(h),
                                                                      rows, f, rows_dev, limit);
  return launch_status();
}

template <typename T>
int fwd_typed(const void* gu, void* h, int64_t rows, int64_t f, const int32_t* rows_dev, int has_limit, float limit,
              hipStream_t s) {
  return has_limit ? fwd_limit<T, true>(gu, h, rows, f, rows_dev, limit, s)
                   : fwd_limit<T, false>(gu, h, rows, f, rows_dev, limit, s);
}

template <typename T, bool LIMIT>
int bwd_limit(const void* gu, const void* dh, void* dgu, int64_t rows, int64_t f, const int32_t* rows_dev, float limit,
              hipStream_t s) {
  constexpr int W = 16 / int(sizeof(T));
  const bool vec = f % W == 0 && aligned_to(gu, 16) && aligned_to(dh, 16) && aligned_to(dgu, 16);
  if (vec)
    swiglu_bwd_kernel<T, W, LIMIT><<<grid_for(rows * (f / W)), 256, 0, s>>>(
        static_cast<const T*>(gu), static_cast<const T*>(dh), static_cast<T*>(dgu), rows, f, rows_dev, limit);
  else
    swiglu_bwd_kernel<T, 1, LIMIT><<<grid_for(rows * f), 256, 0, s>>>(
        static_cast<const T*>(gu), static_cast<const T*>(dh), static_cast<T*>(dgu), rows, f, rows_dev, limit);
  return launch_status();
}

template <typename T>
int bwd_typed(const void* gu, const void* dh, void* dgu, int64_t rows, int64_t f, const int32_t* rows_dev,
              int has_limit, float limit, hipStream_t s) {
  return has_limit ? bwd_limit<T, true>(gu, dh, dgu, rows, f, rows_dev, limit, s)
                   : bwd_limit<T, false>(gu, dh, dgu, rows, f, rows_dev, limit, s);
}

}  // namespace
}  // namespace stm

extern "C" {

int stm_swiglu_fwd(const void* gate_up, void* out, int64_t rows, int64_t ffn, const int32_t* live_rows_or_null,
                   int has_limit, float limit, int dtype, stm_stream_t stream) {
  using namespace stm;
  if (rows < 0 || ffn < 0) return STM_ERR_ARG;
  if (rows == 0 || ffn == 0) return STM_OK;
  if (!gate_up || !out) return STM_ERR_ARG;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case STM_F32: return fwd_typed<float>(gate_up, out, rows, ffn, live_rows_or_null, has_limit, limit, s);
    case STM_F16: return fwd_typed<f16_t>(gate_up, out, rows, ffn, live_rows_or_null, has_limit, limit, s);
    case STM_BF16: return fwd_typed<bf16_t>(gate_up, out, rows, ffn, live_rows_or_null, has_limit, limit, s);
    default: return STM_ERR_UNSUPPORTED;
  }
}

int stm_swiglu_bwd(const void* gate_up, const void* grad_out, void* grad_gate_up, int64_t rows, int64_t ffn,
                   const int32_t* live_rows_or_null, int has_limit, float limit, int dtype, stm_stream_t stream) {
  using namespace stm;
  if (rows < 0 || ffn < 0) return STM_ERR_ARG;
  if (rows == 0 || ffn == 0) return STM_OK;
  if (!gate_up || !grad_out || !grad_gate_up) return STM_ERR_ARG;
  hipStream_t s = as_stream(stream);
  switch (dtype) {
    case STM_F32: return bwd_typed<float>(gate_up, grad_out, grad_gate_up, rows, ffn, live_rows_or_null, has_limit, limit, s);
    case STM_F16: return bwd_typed<f16_t>(gate_up, grad_out, grad_gate_up, rows, ffn, live_rows_or_null, has_limit, limit, s);
    case STM_BF16: return bwd_typed<bf16_t>(gate_up, grad_out, grad_gate_up, rows, ffn, live_rows_or_null, has_limit, limit, s);
    default: return STM_ERR_UNSUPPORTED;
  }
}

}  // extern "C"
