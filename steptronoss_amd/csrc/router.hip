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
  int force_balance;  // round-robin ids instead of the selection (the reference's debug switch)
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

// One token: scores from the logits of row t_in, selection, weights of row t_out; the column
// sums and pick counts of this lane's experts are added to col / cnt.
template <int V>
__device__ __forceinline__ void route_one(const RouterArgs& a, int64_t t_in, int64_t t_out, int lane,
                                          int64_t* __restrict__ ids, float* __restrict__ weights, float (&col)[V],
                                          int32_t (&cnt)[V]) {
  const int E = a.n_experts, K = a.top_k;
  const int per_group = a.n_group > 1 ? E / a.n_group : E;
  float p[V], c[V];
  token_scores<V>(a, t_in, lane, p);
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
    // the largest remaining score, then its lowest expert id: ids grow with (j, lane), so the
    // first j with a lane holding that score, and there the first such lane
    float bv = -INFINITY;
#pragma unroll
    for (int j = 0; j < V; ++j)
      if (!((taken >> j) & 1)) bv = fmaxf(bv, c[j]);
    const float top = wave_max(bv);
    int slot = -1, owner = 0;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      const uint64_t holders = __ballot(j * kWave + lane < E && !((taken >> j) & 1) && c[j] == top);
      if (slot < 0 && holders != 0) {
        slot = j;
        owner = __builtin_ctzll(holders);
      }
    }
    if (a.force_balance) {  // reference moe_block.py:253-254: slot (t, r) goes to expert (t*K + r) % E
      const int forced = __builtin_amdgcn_readfirstlane(int((t_out * K + r) % E));
      slot = forced / kWave;
      owner = forced % kWave;
    }
    if (slot < 0) {  // nothing compares equal (NaN scores): the lowest id not taken yet
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const uint64_t free_lanes = __ballot(j * kWave + lane < E && !((taken >> j) & 1));
        if (slot < 0 && free_lanes != 0) {
          slot = j;
          owner = __builtin_ctzll(free_lanes);
        }
      }
      if (slot < 0) slot = 0;  // (K > E is rejected by the caller)
    }
    const int bi = slot * kWave + owner;
    float pv = 0.f;
#pragma unroll
    for (int j = 0; j < V; ++j)
      if (j == slot) pv = p[j];
    pv = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, pv), owner));
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
    ids[t_out * K + lane] = my_id;
    weights[t_out * K + lane] = renorm ? my_tp / (tp_sum + a.eps) : my_tp;
  }
#pragma unroll
  for (int j = 0; j < V; ++j) col[j] += a.use_sigmoid ? p[j] / row_sum : p[j];
}

// Column sums and counts of a workgroup's tokens -> its row of the partials.
template <int V>
__device__ __forceinline__ void write_partials(const float (&col)[V], const int32_t (&cnt)[V], float* lds_col,
                                               int32_t* lds_cnt, int n_experts, float* __restrict__ col_partial,
                                               int32_t* __restrict__ cnt_partial) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
#pragma unroll
  for (int j = 0; j < V; ++j) {
    lds_col[wave * (V * kWave) + j * kWave + lane] = col[j];
    lds_cnt[wave * (V * kWave) + j * kWave + lane] = cnt[j];
  }
  __syncthreads();
  for (int e = threadIdx.x; e < n_experts; e += kRouterWaves * kWave) {
    float sum = 0.f;
    int32_t n = 0;
#pragma unroll
    for (int w = 0; w < kRouterWaves; ++w) {
      sum += lds_col[w * (V * kWave) + e];
      n += lds_cnt[w * (V * kWave) + e];
    }
    col_partial[int64_t(blockIdx.x) * n_experts + e] = sum;
    cnt_partial[int64_t(blockIdx.x) * n_experts + e] = n;
  }
}

template <int V>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_fwd_kernel(RouterArgs a, int64_t* __restrict__ ids,
                                                                         float* __restrict__ weights,
                                                                         float* __restrict__ col_partial,
                                                                         int32_t* __restrict__ cnt_partial) {
  __shared__ float lds_col[kRouterWaves * V * kWave];
  __shared__ int32_t lds_cnt[kRouterWaves * V * kWave];
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  float col[V];
  int32_t cnt[V];
#pragma unroll
  for (int j = 0; j < V; ++j) {
    col[j] = 0.f;
    cnt[j] = 0;
  }
  for (int64_t t = int64_t(blockIdx.x) * kRouterWaves + wave; t < a.n_tokens; t += int64_t(gridDim.x) * kRouterWaves)
    route_one<V>(a, t, t, lane, ids, weights, col, cnt);
  write_partials<V>(col, cnt, lds_col, lds_cnt, a.n_experts, col_partial, cnt_partial);
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

// d logits of one token (row t_out of ids / grad_w / grad_logits) from the logits of row t_in.
template <int V>
__device__ __forceinline__ void route_one_bwd(const RouterArgs& a, int64_t t_in, int64_t t_out, int lane,
                                              const int64_t* __restrict__ ids, const float* __restrict__ grad_w,
                                              const float (&dcol)[V], void* __restrict__ grad_logits, int grad_dtype) {
  const int E = a.n_experts, K = a.top_k;
  float p[V], dp[V];
  token_scores<V>(a, t_in, lane, p);
  // lane r < K holds the r-th pick
  int my_id = -1;
  float my_gw = 0.f, my_tp = 0.f;
  if (lane < K) {
    my_id = int(ids[t_out * K + lane]);
    my_gw = grad_w[t_out * K + lane];
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
    if (e < E) store_logit(grad_logits, grad_dtype, t_out * E + e, dp[j]);
  }
}

// d aux / d (normalised score) of this lane's experts
template <int V>
__device__ __forceinline__ void aux_column_grads(const RouterArgs& a, const float* grad_aux, const int32_t* hist, int lane,
                                                 float (&dcol)[V]) {
  const float gaux = grad_aux ? grad_aux[0] : 0.f;
#pragma unroll
  for (int j = 0; j < V; ++j) {
    const int e = j * kWave + lane;
    dcol[j] = (e < a.n_experts && a.n_tokens > 0) ? gaux * float(a.n_experts) * float(hist[e]) / float(a.n_tokens) : 0.f;
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
  float dcol[V];
  aux_column_grads<V>(a, grad_aux, hist, lane, dcol);
  for (int64_t t = int64_t(blockIdx.x) * kRouterWaves + wave; t < a.n_tokens; t += int64_t(gridDim.x) * kRouterWaves)
    route_one_bwd<V>(a, t, t, lane, ids, grad_w, dcol, grad_logits, a.logits_dtype);
}

// ---------------------------------------------------------------- gate GEMM in front of the router
// logits = x * Wg^T (x [T, H], Wg [E, H], 16-bit elements, fp32 accumulation) computed per chunk of
// 64 tokens (32 when the logits of 64 would not fit) into LDS and routed from there: the logits
// never reach HBM.  A workgroup's 16 waves split a chunk's [tokens, E] tile into blocks of 64
// experts and, as there are fewer than 16 of those, into ranges of the contraction as well; the
// partial tiles are added in a fixed order that depends on E and the hidden size alone, so the
// forward pass and the recomputation in the backward pass see the same logits bit for bit,
// whatever the launch geometry.
struct GateArgs {
  const void* x;
  const void* w;
  int hidden;
  int fp32_logits;  // 0: the logits are rounded to the element type first (a 16-bit gate output)
};

constexpr int kGateExpertBlocks = 2;           // 32-expert blocks of one wave's tile
constexpr int kGateLdsBudget = 144 * 1024;     // stage + the forward kernel's partial rows
constexpr int kGatePrefetch = 2;               // contraction steps in flight ahead of the matrix unit

template <int V>
struct GateShape {
  static constexpr int kPartialBytes = kRouterWaves * V * kWave * 8;
};

// 32-token blocks of a chunk: two where the chunk's logits fit in LDS beside the partial rows
inline int gate_token_blocks(int n_experts) {
  const int lanes_per_row = (n_experts + kWave - 1) / kWave;
  const int v = lanes_per_row <= 1 ? 1 : lanes_per_row <= 2 ? 2 : lanes_per_row <= 4 ? 4 : lanes_per_row <= 8 ? 8 : 16;
  return 64 * n_experts * 4 + kRouterWaves * v * kWave * 8 <= kGateLdsBudget ? 2 : 1;
}

// how a chunk's work is split; a function of the expert count alone
struct GateSplit {
  int n_eb;    // expert blocks of 32 * kGateExpertBlocks
  int parts;   // ranges of the contraction
  int n_buf;   // partial tiles held in LDS at once
};

template <int V, int MT>
__host__ __device__ inline GateSplit gate_split(int E) {
  GateSplit sp;
  sp.n_eb = (E + 32 * kGateExpertBlocks - 1) / (32 * kGateExpertBlocks);
  sp.parts = kRouterWaves / sp.n_eb;
  const int tile_bytes = MT * 32 * E * 4;
  int fit = (kGateLdsBudget - GateShape<V>::kPartialBytes) / tile_bytes;
  sp.n_buf = fit < 1 ? 1 : (fit > sp.parts ? sp.parts : fit);
  return sp;
}

typedef float gate_f32x16_t __attribute__((ext_vector_type(16)));
typedef __bf16 gate_bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 gate_f16x8_t __attribute__((ext_vector_type(8)));

__device__ __forceinline__ gate_f32x16_t gate_mfma(bf16_t, uint4 a, uint4 b, gate_f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(gate_bf16x8_t, a), __builtin_bit_cast(gate_bf16x8_t, b), c,
                                                 0, 0, 0);
}
__device__ __forceinline__ gate_f32x16_t gate_mfma(f16_t, uint4 a, uint4 b, gate_f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(gate_f16x8_t, a), __builtin_bit_cast(gate_f16x8_t, b), c, 0,
                                                0, 0);
}

// stage[tt * E + e] = logits of token t0 + tt (tt < 32 * MT) for every expert e; all threads take part.
template <typename T, int V, int MT>
__device__ __forceinline__ void gate_tile(const GateArgs& g, int64_t t0, int64_t n_tokens, int E, float* stage) {
  constexpr int NT = kGateExpertBlocks, D = kGatePrefetch;
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // (uniform: step offsets stay scalar)
  const GateSplit sp = gate_split<V, MT>(E);
  const int eb = wave % sp.n_eb, part = wave / sp.n_eb;
  const int tile_floats = MT * 32 * E;
  const int row = lane % 32, half = lane / 32;
  gate_f32x16_t acc[MT][NT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[m][n][r] = 0.f;
  if (part < sp.parts) {
    // The contraction runs in batches of 64 elements, four matrix steps each.  A lane holds row
    // lane % 32 and reads 64 contiguous bytes of that row's 128-byte line per batch (the lanes
    // lane and lane + 32 share the line); x and the weights use the same positions along the
    // contraction in every step, which is all a dot product asks for.
    const int batches = g.hidden / 64;
    const int per = (batches + sp.parts - 1) / sp.parts;
    const int b0 = part * per;
    const int steps = (b0 + per < batches ? per : batches - b0) * 4;
    const uint32_t row_bytes = uint32_t(g.hidden) * uint32_t(sizeof(T));
    const int64_t rows_left = n_tokens - t0;
    const uint32_t live_rows = uint32_t(rows_left < MT * 32 ? rows_left : MT * 32);
    // (buffer loads: a row past the end of x or of the weights reads as zero)
    const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(static_cast<const T*>(g.x) + t0 * g.hidden), 0, int(live_rows * row_bytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T*>(static_cast<const T*>(g.w)), 0, int(uint32_t(E) * row_bytes), 0x00020000);
    uint32_t va[MT], vb[NT];
#pragma unroll
    for (int m = 0; m < MT; ++m) va[m] = uint32_t(m * 32 + row) * row_bytes + uint32_t(b0 * 128 + half * 64);
#pragma unroll
    for (int n = 0; n < NT; ++n) vb[n] = uint32_t((eb * NT + n) * 32 + row) * row_bytes + uint32_t(b0 * 128 + half * 64);
    auto offset_of = [](int step) { return uint32_t((step >> 2) * 128 + (step & 3) * 16); };
    auto fetch = [](__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff) {
      return __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0));
    };
    uint4 fa[D][MT], fb[D][NT];
    if (steps > 0) {
      // (earlier stores drained here: with loads alone in flight the waits inside the loop can
      // count them instead of draining everything)
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
#pragma unroll
      for (int d = 0; d < D; ++d) {
        const uint32_t off = offset_of(d < steps ? d : steps - 1);
#pragma unroll
        for (int m = 0; m < MT; ++m) fa[d][m] = fetch(rsrc_x, va[m], off);
#pragma unroll
        for (int n = 0; n < NT; ++n) fb[d][n] = fetch(rsrc_w, vb[n], off);
      }
      for (int s0 = 0; s0 < steps; s0 += D) {  // steps is a multiple of 4, D divides 4
#pragma unroll
        for (int d = 0; d < D; ++d) {
#pragma unroll
          for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[m][n] = gate_mfma(T{}, fa[d][m], fb[d][n], acc[m][n]);
          const int nxt = s0 + d + D;  // (the last steps fetch the last step again: never used)
          const uint32_t off = offset_of(nxt < steps ? nxt : steps - 1);
#pragma unroll
          for (int m = 0; m < MT; ++m) fa[d][m] = fetch(rsrc_x, va[m], off);
#pragma unroll
          for (int n = 0; n < NT; ++n) fb[d][n] = fetch(rsrc_w, vb[n], off);
        }
      }
    }
  }
  // Partial tiles: part p adds into buffer p % n_buf in round p / n_buf, then the buffers are
  // summed in order.  Register 4*blk + q of lane l: token 8*blk + (l/32)*4 + q, expert l%32.
  const int rounds = (sp.parts + sp.n_buf - 1) / sp.n_buf;
  const int my_round = part < sp.parts ? part / sp.n_buf : -1;
  for (int r = 0; r < rounds; ++r) {
    if (r == my_round) {
      // (the index is made opaque so that the 16 * MT * NT addresses are formed here, one at a
      // time, instead of being kept in registers across the chunk loop)
      int first = (part % sp.n_buf) * tile_floats + half * 4 * E + eb * NT * 32 + row;
      asm volatile("" : "+v"(first));
#pragma unroll
      for (int n = 0; n < NT; ++n) {
        if ((eb * NT + n) * 32 + row < E) {
#pragma unroll
          for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int blk = 0; blk < 4; ++blk)
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                float* at = stage + first + n * 32 + (m * 32 + 8 * blk + q) * E;
                *at = r == 0 ? acc[m][n][blk * 4 + q] : *at + acc[m][n][blk * 4 + q];
              }
        }
      }
    }
    __syncthreads();
  }
  for (int i = threadIdx.x; i < tile_floats; i += kRouterWaves * kWave) {
    float v = stage[i];
    for (int q = 1; q < sp.n_buf; ++q) v += stage[q * tile_floats + i];
    stage[i] = g.fp32_logits ? v : to_float(from_float<T>(v));
  }
  __syncthreads();
}

template <int V, typename T, int MT>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_gate_fwd_kernel(RouterArgs a, GateArgs g,
                                                                              int64_t* __restrict__ ids,
                                                                              float* __restrict__ weights,
                                                                              float* __restrict__ col_partial,
                                                                              int32_t* __restrict__ cnt_partial) {
  extern __shared__ __align__(16) unsigned char gate_smem[];
  constexpr int kTokens = MT * 32;
  float* lds_col = reinterpret_cast<float*>(gate_smem);
  int32_t* lds_cnt = reinterpret_cast<int32_t*>(lds_col + kRouterWaves * V * kWave);
  float* stage = reinterpret_cast<float*>(gate_smem + GateShape<V>::kPartialBytes);
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  float col[V];
  int32_t cnt[V];
#pragma unroll
  for (int j = 0; j < V; ++j) {
    col[j] = 0.f;
    cnt[j] = 0;
  }
  RouterArgs staged = a;  // the router reads this chunk's logits from LDS, as fp32
  staged.logits = stage;
  staged.logits_dtype = STM_F32;
  for (int64_t t0 = int64_t(blockIdx.x) * kTokens; t0 < a.n_tokens; t0 += int64_t(gridDim.x) * kTokens) {
    gate_tile<T, V, MT>(g, t0, a.n_tokens, a.n_experts, stage);
    for (int tt = wave; tt < kTokens; tt += kRouterWaves)
      if (t0 + tt < a.n_tokens) route_one<V>(staged, tt, t0 + tt, lane, ids, weights, col, cnt);
    __syncthreads();  // the next chunk overwrites the stage
  }
  write_partials<V>(col, cnt, lds_col, lds_cnt, a.n_experts, col_partial, cnt_partial);
}

template <int V, typename T, int MT>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_gate_bwd_kernel(RouterArgs a, GateArgs g,
                                                                              const int64_t* __restrict__ ids,
                                                                              const float* __restrict__ grad_w,
                                                                              const float* __restrict__ grad_aux,
                                                                              const int32_t* __restrict__ hist,
                                                                              void* __restrict__ grad_logits,
                                                                              int grad_dtype) {
  extern __shared__ __align__(16) unsigned char gate_smem[];
  constexpr int kTokens = MT * 32;
  float* stage = reinterpret_cast<float*>(gate_smem);
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  float dcol[V];
  aux_column_grads<V>(a, grad_aux, hist, lane, dcol);
  RouterArgs staged = a;
  staged.logits = stage;
  staged.logits_dtype = STM_F32;
  for (int64_t t0 = int64_t(blockIdx.x) * kTokens; t0 < a.n_tokens; t0 += int64_t(gridDim.x) * kTokens) {
    gate_tile<T, V, MT>(g, t0, a.n_tokens, a.n_experts, stage);
    for (int tt = wave; tt < kTokens; tt += kRouterWaves)
      if (t0 + tt < a.n_tokens) route_one_bwd<V>(staged, tt, t0 + tt, lane, ids, grad_w, dcol, grad_logits, grad_dtype);
    __syncthreads();
  }
}

// workgroups of a launch: one per chunk, at most 512 (never more than router_blocks(), which sizes
// the workspace of partial rows)
inline int gate_blocks(int64_t n_tokens, int n_experts) {
  const int chunk = 32 * gate_token_blocks(n_experts);
  const int64_t want = (n_tokens + chunk - 1) / chunk;
  return int(want < 1 ? 1 : (want > 512 ? 512 : want));
}

template <int V, int MT>
inline size_t gate_stage_bytes(int E) {
  return size_t(gate_split<V, MT>(E).n_buf) * MT * 32 * E * 4;
}

// shapes the fused gate takes: 16-bit elements, hidden a multiple of 64, at most 512 experts
inline int check_gate_args(const void* x, const void* w, int dtype, int hidden, int n_experts) {
  if (dtype != STM_BF16 && dtype != STM_F16) return STM_ERR_UNSUPPORTED;
  if (hidden <= 0 || hidden % 64 != 0 || n_experts > 32 * kRouterWaves) return STM_ERR_UNSUPPORTED;
  if (!aligned_to(x, 16) || !aligned_to(w, 16)) return STM_ERR_UNSUPPORTED;
  return STM_OK;
}

template <typename K>
int allow_large_lds(K kernel, size_t bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                             int(bytes)) == hipSuccess
             ? STM_OK
             : STM_ERR_LAUNCH;
}

template <int V, typename T, int MT>
int launch_gate_fwd_as(const RouterArgs& a, const GateArgs& g, int blocks, int64_t* ids, float* weights,
                       float* col_partial, int32_t* cnt_partial, hipStream_t s) {
  const size_t lds = gate_stage_bytes<V, MT>(a.n_experts) + GateShape<V>::kPartialBytes;
  if (allow_large_lds(router_gate_fwd_kernel<V, T, MT>, lds) != STM_OK) return STM_ERR_LAUNCH;
  router_gate_fwd_kernel<V, T, MT><<<blocks, kRouterWaves * kWave, lds, s>>>(a, g, ids, weights, col_partial, cnt_partial);
  return STM_OK;
}

template <int V, typename T, int MT>
int launch_gate_bwd_as(const RouterArgs& a, const GateArgs& g, int blocks, const int64_t* ids, const float* grad_w,
                       const float* grad_aux, const int32_t* hist, void* grad_logits, int grad_dtype, hipStream_t s) {
  const size_t lds = gate_stage_bytes<V, MT>(a.n_experts);
  if (allow_large_lds(router_gate_bwd_kernel<V, T, MT>, lds) != STM_OK) return STM_ERR_LAUNCH;
  router_gate_bwd_kernel<V, T, MT><<<blocks, kRouterWaves * kWave, lds, s>>>(a, g, ids, grad_w, grad_aux, hist, grad_logits,
                                                                             grad_dtype);
  return STM_OK;
}

// (only rows of 257 to 512 experts come in both chunk sizes)
template <int V, typename T>
int launch_gate_fwd(const RouterArgs& a, const GateArgs& g, int blocks, int64_t* ids, float* weights, float* col_partial,
                    int32_t* cnt_partial, hipStream_t s) {
  if constexpr (V <= 4) return launch_gate_fwd_as<V, T, 2>(a, g, blocks, ids, weights, col_partial, cnt_partial, s);
  if constexpr (V == 8)
    if (gate_token_blocks(a.n_experts) == 2)
      return launch_gate_fwd_as<V, T, 2>(a, g, blocks, ids, weights, col_partial, cnt_partial, s);
  return launch_gate_fwd_as<V, T, 1>(a, g, blocks, ids, weights, col_partial, cnt_partial, s);
}

template <int V, typename T>
int launch_gate_bwd(const RouterArgs& a, const GateArgs& g, int blocks, const int64_t* ids, const float* grad_w,
                    const float* grad_aux, const int32_t* hist, void* grad_logits, int grad_dtype, hipStream_t s) {
  if constexpr (V <= 4) return launch_gate_bwd_as<V, T, 2>(a, g, blocks, ids, grad_w, grad_aux, hist, grad_logits, grad_dtype, s);
  if constexpr (V == 8)
    if (gate_token_blocks(a.n_experts) == 2)
      return launch_gate_bwd_as<V, T, 2>(a, g, blocks, ids, grad_w, grad_aux, hist, grad_logits, grad_dtype, s);
  return launch_gate_bwd_as<V, T, 1>(a, g, blocks, ids, grad_w, grad_aux, hist, grad_logits, grad_dtype, s);
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
                   int force_balance, int64_t* ids_out, float* weights_out, float* aux_out, int32_t* hist_out,
                   float* me_out, void* workspace, size_t workspace_bytes, stm_stream_t stream) {
  using namespace stm;
  RouterArgs a{logits, logits_dtype, bias_or_null, n_tokens, n_experts, top_k, use_sigmoid, norm_weights,
               n_group,  topk_group,  eps, force_balance != 0};
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

int stm_router_gate_fwd(const void* x, const void* gate_w, int dtype, int hidden, int fp32_logits,
                        const float* bias_or_null, int64_t n_tokens, int n_experts, int top_k, int use_sigmoid,
                        int norm_weights, float eps, int n_group, int topk_group, int force_balance, int64_t* ids_out,
                        float* weights_out, float* aux_out, int32_t* hist_out, float* me_out, void* workspace,
                        size_t workspace_bytes, stm_stream_t stream) {
  using namespace stm;
  RouterArgs a{nullptr, STM_F32, bias_or_null, n_tokens, n_experts, top_k, use_sigmoid, norm_weights,
               n_group, topk_group,   eps, force_balance != 0};
  int st = check_router_args(a);
  if (st != STM_OK) return st;
  if (n_tokens > 0 && n_experts > 0 && (!x || !gate_w)) return STM_ERR_ARG;
  st = check_gate_args(x, gate_w, dtype, hidden, n_experts);
  if (st != STM_OK) return st;
  if (!aux_out || (n_experts > 0 && (!hist_out || !me_out))) return STM_ERR_ARG;
  if (n_tokens > 0 && top_k > 0 && (!ids_out || !weights_out)) return STM_ERR_ARG;
  if (workspace_bytes < stm_router_workspace_bytes(n_tokens, n_experts) || !workspace) return STM_ERR_WORKSPACE;
  hipStream_t s = as_stream(stream);
  const int need = (n_experts + kWave - 1) / kWave;
  const int blocks = gate_blocks(n_tokens, n_experts);
  float* col_partial = static_cast<float*>(workspace);
  int32_t* cnt_partial = reinterpret_cast<int32_t*>(col_partial + size_t(blocks) * n_experts);
  GateArgs g{x, gate_w, hidden, fp32_logits};
  if (dtype == STM_BF16) {
    STM_ROUTER_DISPATCH(need, (st = launch_gate_fwd<V, bf16_t>(a, g, blocks, ids_out, weights_out, col_partial, cnt_partial, s)));
  } else {
    STM_ROUTER_DISPATCH(need, (st = launch_gate_fwd<V, f16_t>(a, g, blocks, ids_out, weights_out, col_partial, cnt_partial, s)));
  }
  if (st != STM_OK) return st;
  router_finish_kernel<<<1, 1024, 0, s>>>(col_partial, cnt_partial, blocks, n_experts, n_tokens, me_out, hist_out,
                                          aux_out);
  return launch_status();
}

int stm_router_gate_bwd(const void* x, const void* gate_w, int dtype, int hidden, int fp32_logits, int64_t n_tokens,
                        int n_experts, int top_k, int use_sigmoid, int norm_weights, float eps, const int64_t* ids,
                        const float* grad_weights, const float* grad_aux_or_null, const int32_t* hist,
                        void* grad_logits, int grad_dtype, stm_stream_t stream) {
  using namespace stm;
  RouterArgs a{nullptr, STM_F32, nullptr, n_tokens, n_experts, top_k, use_sigmoid, norm_weights, 1, 1, eps};
  int st = check_router_args(a);
  if (st != STM_OK) return st;
  if (grad_dtype < STM_F32 || grad_dtype > STM_BF16) return STM_ERR_UNSUPPORTED;
  if (n_tokens == 0 || n_experts == 0) return STM_OK;
  if (!x || !gate_w || !grad_logits || !hist || (top_k > 0 && (!ids || !grad_weights))) return STM_ERR_ARG;
  st = check_gate_args(x, gate_w, dtype, hidden, n_experts);
  if (st != STM_OK) return st;
  hipStream_t s = as_stream(stream);
  GateArgs g{x, gate_w, hidden, fp32_logits};
  const int need = (n_experts + kWave - 1) / kWave;
  const int blocks = gate_blocks(n_tokens, n_experts);
  if (dtype == STM_BF16) {
    STM_ROUTER_DISPATCH(need, (st = launch_gate_bwd<V, bf16_t>(a, g, blocks, ids, grad_weights, grad_aux_or_null, hist, grad_logits, grad_dtype, s)));
  } else {
    STM_ROUTER_DISPATCH(need, (st = launch_gate_bwd<V, f16_t>(a, g, blocks, ids, grad_weights, grad_aux_or_null, hist, grad_logits, grad_dtype, s)));
  }
  if (st != STM_OK) return st;
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
