// Top-k router: scores (softmax or sigmoid), stable top-k selection, weight normalisation and the
// load-balance statistics, plus its backward (gfx950).
//
// One wavefront owns one token at a time; lane l holds experts l, l+64, l+128, ... of the row,
// so the row is read with one coalesced load per 64 experts.  Selection is K rounds of a
// wave-wide arg-max over (score descending, expert id ascending) -- the order a stable
// descending sort produces -- so equal scores always go to the lower expert id.
// Column sums of the scores and the per-expert counts are kept per lane across a workgroup's
// tokens, combined through LDS and written as per-workgroup partials that one finishing
// workgroup adds in a fixed order: no atomics, bit-reproducible.
#include "common.hpp"

namespace stm {
namespace {

constexpr int kMaxPerLane = 16;  // experts per lane  => E <= 1024
constexpr int kRouterWaves = 16;  // 1024 threads: fewer, larger workgroups = fewer partial rows for the finish kernel
constexpr int kMaxGroupsRouted = 64;
constexpr int kMaxTopK = 64;

struct RouterArgs {
  const void* logits;
  int logits_dtype;
  const float* bias;  // added to the scores for selection only; may be null
  int64_t n_tokens;
  int n_experts, top_k;
  int use_sigmoid, norm_weights;
  int n_group, topk_group;
  float eps;
};

__device__ __forceinline__ float load_logit(const void* p, int dtype, int64_t i) {
  switch (dtype) {
    case STM_F32: return static_cast<const float*>(p)[i];
    case STM_F16: return to_float(static_cast<const f16_t*>(p)[i]);
    default: return to_float(static_cast<const bf16_t*>(p)[i]);
  }
}

__device__ __forceinline__ void store_logit(void* p, int dtype, int64_t i, float v) {
  switch (dtype) {
    case STM_F32: static_cast<float*>(p)[i] = v; break;
    case STM_F16: static_cast<f16_t*>(p)[i] = from_float<f16_t>(v); break;
    default: static_cast<bf16_t*>(p)[i] = from_float<bf16_t>(v); break;
  }
}

// scores of one token into p[] (lane-strided), returns nothing; V = experts per lane.
template <int V>
__device__ __forceinline__ void token_scores(const RouterArgs& a, int64_t t, int lane, float (&p)[V]) {
  const int E = a.n_experts;
  float x[V];
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const int e = j * kWave + lane;
    x[j] = e < E ? load_logit(a.logits, a.logits_dtype, t * E + e) : -INFINITY;
  }
  if (a.use_sigmoid) {
#pragma unroll
    for (int j = 0; j < V; ++j) p[j] = (j * kWave + lane) < E ? 1.f / (1.f + expf(-x[j])) : 0.f;
  } else {
    float m = x[0];
#pragma unroll
    for (int j = 1; j < V; ++j) m = fmaxf(m, x[j]);
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      p[j] = (j * kWave + lane) < E ? expf(x[j] - m) : 0.f;
      s += p[j];
    }
    s = wave_sum(s);
#pragma unroll
    for (int j = 0; j < V; ++j) p[j] = p[j] / s;
  }
}

template <int V>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_fwd_kernel(RouterArgs a, int64_t* __restrict__ ids,
                                                                         float* __restrict__ weights,
                                                                         float* __restrict__ col_partial,
                                                                         int32_t* __restrict__ cnt_partial) {
  __shared__ float lds_col[kRouterWaves][V * kWave];
  __shared__ int32_t lds_cnt[kRouterWaves][V * kWave];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int E = a.n_experts, K = a.top_k;
  float col[V];
  int32_t cnt[V];
#pragma unroll
  for (int j = 0; j < V; ++j) {
    col[j] = 0.f;
    cnt[j] = 0;
  }
  const int per_group = a.n_group > 1 ? E / a.n_group : E;

  for (int64_t t = int64_t(blockIdx.x) * kRouterWaves + wave; t < a.n_tokens; t += int64_t(gridDim.x) * kRouterWaves) {
    float p[V], c[V];
    token_scores<V>(a, t, lane, p);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const int e = j * kWave + lane;
      c[j] = e < E ? (a.bias ? p[j] + a.bias[e] : p[j]) : -INFINITY;
    }
    // ---- group-limited routing: keep the topk_group groups with the largest top-2 sums
    if (a.n_group > 1) {
      uint64_t keep = 0;
      float my_gscore = -INFINITY;  // lane g keeps the score of group g (n_group <= 64)
      for (int g = 0; g < a.n_group; ++g) {
        float best = -INFINITY;
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const int e = j * kWave + lane;
          if (e < E && e / per_group == g) best = fmaxf(best, c[j]);
        }
        const float top1 = wave_max(best);
        int n_top = 0;
        float second = -INFINITY;
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const int e = j * kWave + lane;
          if (e < E && e / per_group == g) {
            if (c[j] == top1)
              ++n_top;
            else
              second = fmaxf(second, c[j]);
          }
        }
        n_top = wave_sum(n_top);
        second = wave_max(second);
        const float gscore = per_group >= 2 ? top1 + (n_top >= 2 ? top1 : second) : top1;
        if (lane == g) my_gscore = gscore;
      }
      for (int r = 0; r < a.topk_group; ++r) {  // largest score first, equal scores: lower group
        const bool free_group = lane < a.n_group && !((keep >> lane) & 1);
        float best = free_group ? my_gscore : -INFINITY;
        int pick = free_group ? lane : INT32_MAX;
        wave_argmax(best, pick);
        if (pick != INT32_MAX) keep |= 1ull << pick;
      }
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const int e = j * kWave + lane;
        if (e < E && !((keep >> (e / per_group)) & 1)) c[j] = -INFINITY;
      }
    }
    // ---- K rounds of arg-max; `taken` marks this lane's experts already chosen
    uint32_t taken = 0;
    float tp_sum = 0.f;
    float my_tp = 0.f;  // lane r keeps the score of the r-th pick (K <= 64)
    int my_id = 0;
    for (int r = 0; r < K; ++r) {
      float bv = -INFINITY;
      int bi = INT32_MAX;
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const int e = j * kWave + lane;
        if (e < E && !((taken >> j) & 1) && (c[j] > bv || (c[j] == bv && e < bi))) {
          bv = c[j];
          bi = e;
        }
      }
      // a lane with nothing left still offers (-inf, its smallest free id) so that rows whose
      // remaining scores are all -inf keep the ascending-id order of a stable sort
      if (bi == INT32_MAX) {
#pragma unroll
        for (int j = V - 1; j >= 0; --j) {
          const int e = j * kWave + lane;
          if (e < E && !((taken >> j) & 1)) bi = e;
        }
      }
      wave_argmax(bv, bi);
      const int owner = bi % kWave, slot = bi / kWave;
      float pv = 0.f;
#pragma unroll
      for (int j = 0; j < V; ++j)
        if (j == slot) pv = p[j];
      pv = __shfl(pv, owner, kWave);
      if (lane == owner) {
        taken |= 1u << slot;
#pragma unroll
        for (int j = 0; j < V; ++j)
          if (j == slot) ++cnt[j];
      }
      tp_sum += pv;
      if (lane == r) {
        my_tp = pv;
        my_id = bi;
      }
    }
    // ---- weights and score normalisation
    float row_sum = 0.f;
    if (a.use_sigmoid) {
#pragma unroll
      for (int j = 0; j < V; ++j) row_sum += p[j];
      row_sum = wave_sum(row_sum) + a.eps;
    }
    const bool renorm = a.use_sigmoid || a.norm_weights;
    if (lane < K) {
      ids[t * K + lane] = my_id;
      weights[t * K + lane] = renorm ? my_tp / (tp_sum + a.eps) : my_tp;
    }
#pragma unroll
    for (int j = 0; j < V; ++j) col[j] += a.use_sigmoid ? p[j] / row_sum : p[j];
  }
  // ---- per-workgroup partials of the column sums and counts
#pragma unroll
  for (int j = 0; j < V; ++j) {
    lds_col[wave][j * kWave + lane] = col[j];
    lds_cnt[wave][j * kWave + lane] = cnt[j];
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += kRouterWaves * kWave) {
    float s = 0.f;
    int32_t n = 0;
#pragma unroll
    for (int w = 0; w < kRouterWaves; ++w) {
      s += lds_col[w][e];
      n += lds_cnt[w][e];
    }
    col_partial[int64_t(blockIdx.x) * E + e] = s;
    cnt_partial[int64_t(blockIdx.x) * E + e] = n;
  }
}

// me[e] = sum_t score[t,e] / T, hist[e] = count, aux = E * sum_e me[e] * hist[e].
__global__ __launch_bounds__(1024) void router_finish_kernel(const float* __restrict__ col_partial,
                                                             const int32_t* __restrict__ cnt_partial, int n_blocks,
                                                             int n_experts, int64_t n_tokens, float* __restrict__ me,
                                                             int32_t* __restrict__ hist, float* __restrict__ aux) {
  __shared__ float wave_part[1024 / kWave];
  __shared__ float s_part[1024];
  __shared__ int32_t n_part[1024];
  // The block's threads form `slices` rows of `width` experts; a row sums every slices-th
  // partial of its experts, row 0 then adds the rows up in a fixed order.
  int width = kWave;
  while (width < n_experts && width < 1024) width <<= 1;
  const int slices = 1024 / width;
  const int col = threadIdx.x % width, slice = threadIdx.x / width;
  float mine = 0.f;
  for (int e0 = 0; e0 < n_experts; e0 += width) {
    const int e = e0 + col;
    float s = 0.f;
    int32_t n = 0;
    if (e < n_experts) {
#pragma unroll 8
      for (int b = slice; b < n_blocks; b += slices) {
        s += col_partial[int64_t(b) * n_experts + e];
        n += cnt_partial[int64_t(b) * n_experts + e];
      }
    }
    s_part[threadIdx.x] = s;
    n_part[threadIdx.x] = n;
    __syncthreads();
    if (slice == 0 && e < n_experts) {
      for (int r = 1; r < slices; ++r) {
        s += s_part[r * width + col];
        n += n_part[r * width + col];
      }
      const float m = n_tokens > 0 ? s / float(n_tokens) : 0.f;
      me[e] = m;
      hist[e] = n;
      mine += m * float(n);
    }
    __syncthreads();
  }
  mine = wave_sum(mine);
  if (threadIdx.x % kWave == 0) wave_part[threadIdx.x / kWave] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.f;
    for (int w = 0; w < 1024 / kWave; ++w) s += wave_part[w];
    aux[0] = s * float(n_experts);
  }
}

// d logits from d weights and d aux.
template <int V>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_bwd_kernel(RouterArgs a, const int64_t* __restrict__ ids,
                                                                         const float* __restrict__ grad_w,
                                                                         const float* __restrict__ grad_aux,
                                                                         const int32_t* __restrict__ hist,
                                                                         void* __restrict__ grad_logits) {
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int E = a.n_experts, K = a.top_k;
  const float gaux = grad_aux ? grad_aux[0] : 0.f;
  float dcol[V];  // d aux / d (normalised score) of this lane's experts
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const int e = j * kWave + lane;
    dcol[j] = (e < E && a.n_tokens > 0) ? gaux * float(E) * float(hist[e]) / float(a.n_tokens) : 0.f;
  }
  for (int64_t t = int64_t(blockIdx.x) * kRouterWaves + wave; t < a.n_tokens; t += int64_t(gridDim.x) * kRouterWaves) {
    float p[V], dp[V];
    token_scores<V>(a, t, lane, p);
    // lane r < K holds the r-th pick
    int my_id = -1;
    float my_gw = 0.f, my_tp = 0.f;
    if (lane < K) {
      my_id = int(ids[t * K + lane]);
      my_gw = grad_w[t * K + lane];
    }
    // fetch the picked scores from their owner lanes
    for (int r = 0; r < K; ++r) {
      const int e = __shfl(my_id, r, kWave);
      float pv = 0.f;
#pragma unroll
      for (int j = 0; j < V; ++j)
        if (j == e / kWave) pv = p[j];
      pv = __shfl(pv, e % kWave, kWave);
      if (lane == r) my_tp = pv;
    }
    const bool renorm = a.use_sigmoid || a.norm_weights;
    float dtp = my_gw;  // d L / d (picked raw score), lane r
    if (renorm) {
      const float s = wave_sum(lane < K ? my_tp : 0.f) + a.eps;
      const float dot = wave_sum(lane < K ? my_gw * (my_tp / s) : 0.f);
      dtp = (my_gw - dot) / s;
    }
    // d L / d raw score
    if (a.use_sigmoid) {
      float row_sum = 0.f;
#pragma unroll
      for (int j = 0; j < V; ++j) row_sum += p[j];
      row_sum = wave_sum(row_sum) + a.eps;
      float dot = 0.f;
#pragma unroll
      for (int j = 0; j < V; ++j) dot += dcol[j] * (p[j] / row_sum);
      dot = wave_sum(dot);
#pragma unroll
      for (int j = 0; j < V; ++j) dp[j] = (dcol[j] - dot) / row_sum;
    } else {
#pragma unroll
      for (int j = 0; j < V; ++j) dp[j] = dcol[j];
    }
    for (int r = 0; r < K; ++r) {
      const int e = __shfl(my_id, r, kWave);
      const float g = __shfl(dtp, r, kWave);
      if (lane == e % kWave) {
#pragma unroll
        for (int j = 0; j < V; ++j)
          if (j == e / kWave) dp[j] += g;
      }
    }
    // through the activation
    if (a.use_sigmoid) {
#pragma unroll
      for (int j = 0; j < V; ++j) dp[j] = dp[j] * p[j] * (1.f - p[j]);
    } else {
      float dot = 0.f;
#pragma unroll
      for (int j = 0; j < V; ++j) dot += dp[j] * p[j];
      dot = wave_sum(dot);
#pragma unroll
      for (int j = 0; j < V; ++j) dp[j] = p[j] * (dp[j] - dot);
    }
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const int e = j * kWave + lane;
      if (e < E) store_logit(grad_logits, a.logits_dtype, t * E + e, dp[j]);
    }
  }
}

// Aux-loss-free load balancing: bias[e] += sign(mean(tokens) - tokens[e]) * rate, then the token
// counters start over.  One block; the mean is the exact integer total, rounded once, over E.
__global__ __launch_bounds__(1024) void router_bias_update_kernel(int32_t* __restrict__ tokens,
                                                                  float* __restrict__ bias, int n_experts, float rate,
                                                                  bool zero_tokens) {
  __shared__ long long wave_part[1024 / kWave];
  __shared__ float mean_s;
  long long mine = 0;
  for (int e = threadIdx.x; e < n_experts; e += 1024) mine += tokens[e];
  mine = wave_sum(mine);
  if (threadIdx.x % kWave == 0) wave_part[threadIdx.x / kWave] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    long long total = 0;
    for (int w = 0; w < 1024 / kWave; ++w) total += wave_part[w];
    mean_s = float(total) / float(n_experts);
  }
  __syncthreads();
  const float mean = mean_s;
  for (int e = threadIdx.x; e < n_experts; e += 1024) {
    const float offset = mean - float(tokens[e]);
    const float sign = offset > 0.f ? 1.f : (offset < 0.f ? -1.f : 0.f);
    bias[e] += sign * rate;
    if (zero_tokens) tokens[e] = 0;
  }
}

inline int router_blocks(int64_t n_tokens) {
  const int64_t want = (n_tokens + kRouterWaves - 1) / kRouterWaves;
  return int(want < 1 ? 1 : (want > 512 ? 512 : want));
}

inline int check_router_args(const RouterArgs& a) {
  if (a.n_tokens < 0 || a.n_experts < 0 || a.top_k < 0) return STM_ERR_ARG;
  if (a.top_k > a.n_experts) return STM_ERR_ARG;
  if (a.n_experts > kMaxPerLane * kWave || a.top_k > kMaxTopK) return STM_ERR_UNSUPPORTED;
  if (a.logits_dtype < STM_F32 || a.logits_dtype > STM_BF16) return STM_ERR_UNSUPPORTED;
  if (a.n_group > 1) {
    if (a.n_group > kMaxGroupsRouted || a.n_experts % a.n_group != 0) return STM_ERR_UNSUPPORTED;
    if (a.topk_group < 1 || a.topk_group > a.n_group) return STM_ERR_ARG;
  }
  return STM_OK;
}

#define STM_ROUTER_DISPATCH(V_NEEDED, CALL) \
  if ((V_NEEDED) <= 1) { constexpr int V = 1; CALL; } \
  else if ((V_NEEDED) <= 2) { constexpr int V = 2; CALL; } \
  else if ((V_NEEDED) <= 4) { constexpr int V = 4; CALL; } \
  else if ((V_NEEDED) <= 8) { constexpr int V = 8; CALL; } \
  else { constexpr int V = 16; CALL; }

}  // namespace
}  // namespace stm

extern "C" {

size_t stm_router_workspace_bytes(int64_t n_tokens, int n_experts) {
  if (n_tokens < 0 || n_experts < 0) return 0;
  return stm::round_up(size_t(stm::router_blocks(n_tokens)) * size_t(n_experts) * 8 + 256, 256);
}

int stm_router_fwd(const void* logits, int logits_dtype, const float* bias_or_null, int64_t n_tokens, int n_experts,
                   int top_k, int use_sigmoid, int norm_weights, float eps, int n_group, int topk_group,
                   int64_t* ids_out, float* weights_out, float* aux_out, int32_t* hist_out, float* me_out,
                   void* workspace, size_t workspace_bytes, stm_stream_t stream) {
  using namespace stm;
  RouterArgs a{logits, logits_dtype, bias_or_null, n_tokens, n_experts, top_k, use_sigmoid, norm_weights,
               n_group,  topk_group,  eps};
  const int st = check_router_args(a);
  if (st != STM_OK) return st;
  if (!aux_out || (n_experts > 0 && (!hist_out || !me_out))) return STM_ERR_ARG;
  if (n_tokens > 0 && n_experts > 0 && (!logits || (top_k > 0 && (!ids_out || !weights_out)))) return STM_ERR_ARG;
  if (workspace_bytes < stm_router_workspace_bytes(n_tokens, n_experts) || !workspace) return STM_ERR_WORKSPACE;
  hipStream_t s = as_stream(stream);
  const int blocks = router_blocks(n_tokens);
  float* col_partial = static_cast<float*>(workspace);
  int32_t* cnt_partial = reinterpret_cast<int32_t*>(col_partial + size_t(blocks) * n_experts);
  const int need = (n_experts + kWave - 1) / kWave;
  STM_ROUTER_DISPATCH(need, (router_fwd_kernel<V><<<blocks, kRouterWaves * kWave, 0, s>>>(a, ids_out, weights_out,
                                                                                           col_partial, cnt_partial)));
  router_finish_kernel<<<1, 1024, 0, s>>>(col_partial, cnt_partial, blocks, n_experts, n_tokens, me_out, hist_out,
                                          aux_out);
  return launch_status();
}

int stm_router_bwd(const void* logits, int logits_dtype, int64_t n_tokens, int n_experts, int top_k, int use_sigmoid,
                   int norm_weights, float eps, const int64_t* ids, const float* grad_weights,
                   const float* grad_aux_or_null, const int32_t* hist, void* grad_logits, stm_stream_t stream) {
  using namespace stm;
  RouterArgs a{logits, logits_dtype, nullptr, n_tokens, n_experts, top_k, use_sigmoid, norm_weights, 1, 1, eps};
  const int st = check_router_args(a);
  if (st != STM_OK) return st;
  if (n_tokens == 0 || n_experts == 0) return STM_OK;
  if (!logits || !grad_logits || !hist || (top_k > 0 && (!ids || !grad_weights))) return STM_ERR_ARG;
  hipStream_t s = as_stream(stream);
  const int blocks = router_blocks(n_tokens);
  const int need = (n_experts + kWave - 1) / kWave;
  STM_ROUTER_DISPATCH(need, (router_bwd_kernel<V><<<blocks, kRouterWaves * kWave, 0, s>>>(
                                a, ids, grad_weights, grad_aux_or_null, hist, grad_logits)));
  return launch_status();
}

int stm_router_bias_update(int32_t* tokens_per_expert, float* bias, int n_experts, float rate, int zero_tokens,
                           stm_stream_t stream) {
  using namespace stm;
  if (n_experts < 0) return STM_ERR_ARG;
  if (n_experts == 0) return STM_OK;
  if (!tokens_per_expert || !bias) return STM_ERR_ARG;
  router_bias_update_kernel<<<1, 1024, 0, as_stream(stream)>>>(tokens_per_expert, bias, n_experts, rate,
                                                               zero_tokens != 0);
  return launch_status();
}

}  // extern "C"
