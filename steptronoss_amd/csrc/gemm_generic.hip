// Grouped GEMM over ragged per-expert row ranges: tile table, the any-shape fallback kernel
// and the C entry points (which prefer the MFMA kernels of gemm_mfma.hip when those apply).
//
//   rows form  : C[r, :] = A[r, :] * op(B[g])     for rows r of group g      (fwd, dgrad)
//   wgrad form : Out[g]  = X[rows of g]^T * Y[rows of g]                      (wgrad)
//
// The fallback is a plain LDS-tiled fp32-FMA kernel driven by element strides, so one body
// covers every layout, every dtype and shapes with no alignment at all (k = 8, n = 6 ...).
#include "gemm_common.hpp"

namespace stm {

int launch_mfma_rows(int dtype, const void* a, const void* b, void* c, const int32_t* offsets, int n_groups,
                     int64_t m_cap, int n, int k, int b_is_nk, void* ws, size_t ws_bytes, hipStream_t s);
int launch_mfma_wgrad(int dtype, const void* x, const void* y, void* out, const int32_t* offsets, int n_groups,
                      int64_t m_cap, int p_dim, int q_dim, int accumulate, hipStream_t s,
                      const int32_t* src_rows = nullptr, int gather_operand = 0, int64_t src_buffer_rows = 0);

namespace {

constexpr int kMaxGroups = 4096;

__global__ __launch_bounds__(1024) void tile_table_kernel(const int32_t* __restrict__ offsets, int n_groups, int bm,
                                                          int64_t m_cap, int32_t* __restrict__ header,
                                                          MTile* __restrict__ tiles) {
  __shared__ int32_t first[kMaxGroups];
  __shared__ int32_t wave_sums[1024 / kWave];
  for (int g = threadIdx.x; g < n_groups; g += 1024) {
    int64_t lo = offsets[g], hi = offsets[g + 1];
    hi = hi > m_cap ? m_cap : hi;
    const int64_t m = hi > lo ? hi - lo : 0;
    first[g] = int32_t((m + bm - 1) / bm);
  }
  __syncthreads();
  const int32_t total = block_exclusive_scan(first, n_groups, wave_sums);
  if (threadIdx.x == 0) header[0] = total;
  for (int g = threadIdx.x; g < n_groups; g += 1024) {
    int64_t lo = offsets[g], hi = offsets[g + 1];
    hi = hi > m_cap ? m_cap : hi;
    const int32_t m = hi > lo ? int32_t(hi - lo) : 0;
    const int32_t base = first[g];
    for (int32_t i = 0; i * bm < m; ++i) {
      const int32_t left = m - i * bm;
      tiles[base + i] = MTile{g, int32_t(lo) + i * bm, left < bm ? left : bm, 0};
    }
  }
}

// ------------------------------------------------------------------------ fallback kernel
constexpr int kGT = 64;  // tile edge
constexpr int kGK = 16;  // contraction step

struct GenericArgs {
  const void* a;
  const void* b;
  void* c;
  const int32_t* offsets;
  const int32_t* header;  // rows form: number of M-tiles
  const MTile* tiles;
  int64_t sa_i, sa_k;  // A(i, kk) = a[i * sa_i + kk * sa_k]
  int64_t sb_k, sb_j;  // B(kk, j) = b[kk * sb_k + j * sb_j]
  int64_t b_group, c_group;  // per-group strides (elements)
  int64_t ldc;
  int n_i, n_j, n_k;  // wgrad: n_i = P, n_j = Q; rows: n_j = N, n_k = K
  int wgrad;
};

template <typename T>
__global__ __launch_bounds__(256) void generic_gemm_kernel(GenericArgs p) {
  __shared__ float As[kGK][kGT + 1];
  __shared__ float Bs[kGK][kGT + 1];
  const T* a = static_cast<const T*>(p.a);
  const T* b = static_cast<const T*>(p.b);
  T* c = static_cast<T*>(p.c);
  int n_i, n_k;
  int i0 = 0, j0;
  if (p.wgrad) {
    j0 = blockIdx.x * kGT;
    const int g = blockIdx.z;
    const int64_t lo = p.offsets[g], hi = p.offsets[g + 1];
    n_k = hi > lo ? int(hi - lo) : 0;
    n_i = p.n_i;
    i0 = blockIdx.y * kGT;
    a += lo * p.sa_k;
    b += lo * p.sb_k;
    c += int64_t(g) * p.c_group;
  } else {
    if (int(blockIdx.x) >= p.header[0]) return;
    const MTile t = p.tiles[blockIdx.x];
    j0 = blockIdx.y * kGT;
    n_i = t.rows;
    n_k = p.n_k;
    a += int64_t(t.row0) * p.sa_i;
    b += int64_t(t.group) * p.b_group;
    c += int64_t(t.row0) * p.ldc;
  }
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < n_k; k0 += kGK) {
    for (int e = threadIdx.x; e < kGK * kGT; e += 256) {
      const int kk = e / kGT, ij = e % kGT;
      const int k = k0 + kk;
      const int i = i0 + ij, j = j0 + ij;
      As[kk][ij] = (k < n_k && i < n_i) ? to_float(a[int64_t(i) * p.sa_i + int64_t(k) * p.sa_k]) : 0.f;
      Bs[kk][ij] = (k < n_k && j < p.n_j) ? to_float(b[int64_t(k) * p.sb_k + int64_t(j) * p.sb_j]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kGK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) av[r] = As[kk][ty * 4 + r];
#pragma unroll
      for (int r = 0; r < 4; ++r) bv[r] = Bs[kk][tx * 4 + r];
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int s = 0; s < 4; ++s) acc[r][s] += av[r] * bv[s];
    }
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int i = i0 + ty * 4 + r;
    if (i >= n_i) continue;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int j = j0 + tx * 4 + s;
      if (j < p.n_j) c[int64_t(i) * p.ldc + j] = from_float<T>(acc[r][s]);
    }
  }
}

template <typename T>
void launch_generic(const GenericArgs& p, dim3 grid, hipStream_t s) {
  generic_gemm_kernel<T><<<grid, 256, 0, s>>>(p);
}

int dispatch_generic(int dtype, const GenericArgs& p, dim3 grid, hipStream_t s) {
  switch (dtype) {
    case STM_F32: launch_generic<float>(p, grid, s); break;
    case STM_F16: launch_generic<f16_t>(p, grid, s); break;
    case STM_BF16: launch_generic<bf16_t>(p, grid, s); break;
    default: return STM_ERR_UNSUPPORTED;
  }
  return launch_status();
}

}  // namespace

int build_tile_table(const int32_t* offsets, int n_groups, int bm, int64_t m_cap, void* table, hipStream_t stream) {
  if (n_groups > kMaxGroups) return STM_ERR_UNSUPPORTED;
  int32_t* header = static_cast<int32_t*>(table);
  MTile* tiles = reinterpret_cast<MTile*>(static_cast<char*>(table) + 16);
  tile_table_kernel<<<1, 1024, 0, stream>>>(offsets, n_groups, bm, m_cap, header, tiles);
  return launch_status();
}

}  // namespace stm

extern "C" {

size_t stm_gemm_workspace_bytes(int64_t m_cap, int n_groups) {
  if (m_cap < 0 || n_groups < 0) return 0;
  // sized for the smallest tile height any kernel uses (64 rows)
  return stm::round_up(stm::tile_table_bytes(m_cap, n_groups, 64), 256);
}

int stm_grouped_gemm(const void* a, const void* b, void* c, const int32_t* offsets, int n_groups, int64_t m_cap, int n,
                     int k, int b_is_nk, int dtype, void* workspace, size_t workspace_bytes, stm_stream_t stream) {
  using namespace stm;
  if (n_groups < 0 || m_cap < 0 || n < 0 || k < 0) return STM_ERR_ARG;
  if (dtype < STM_F32 || dtype > STM_BF16 || n_groups > kMaxGroups) return STM_ERR_UNSUPPORTED;
  if (m_cap == 0 || n == 0 || n_groups == 0) return STM_OK;
  if (!a || !b || !c || !offsets || !workspace) return STM_ERR_ARG;
  if (workspace_bytes < stm_gemm_workspace_bytes(m_cap, n_groups)) return STM_ERR_WORKSPACE;
  hipStream_t s = as_stream(stream);
  const int fast = launch_mfma_rows(dtype, a, b, c, offsets, n_groups, m_cap, n, k, b_is_nk, workspace,
                                    workspace_bytes, s);
  if (fast != STM_ERR_UNSUPPORTED) return fast;
  int st = build_tile_table(offsets, n_groups, kGT, m_cap, workspace, s);
  if (st != STM_OK) return st;
  GenericArgs p{};
  p.a = a;
  p.b = b;
  p.c = c;
  p.offsets = offsets;
  p.header = static_cast<const int32_t*>(workspace);
  p.tiles = reinterpret_cast<const MTile*>(static_cast<const char*>(workspace) + 16);
  p.sa_i = k;
  p.sa_k = 1;
  p.sb_k = b_is_nk ? 1 : n;
  p.sb_j = b_is_nk ? k : 1;
  p.b_group = int64_t(n) * k;
  p.ldc = n;
  p.n_j = n;
  p.n_k = k;
  p.wgrad = 0;
  dim3 grid(unsigned(max_m_tiles(m_cap, n_groups, kGT)), unsigned((n + kGT - 1) / kGT), 1);
  return dispatch_generic(dtype, p, grid, s);
}

namespace {
// Common checks and argument block of the two fused entries.
int fused_args(const void* a, const void* b, void* c, void* c2, const int32_t* offsets, int n_groups, int64_t m_cap,
               int ffn, int k, int has_limit, float limit, int dtype, void* workspace, size_t workspace_bytes,
               stm::GemmArgs& p) {
  using namespace stm;
  if (n_groups < 0 || m_cap < 0 || ffn < 0 || k < 0) return STM_ERR_ARG;
  if ((dtype != STM_BF16 && dtype != STM_F16) || n_groups > kMaxGroups) return STM_ERR_UNSUPPORTED;
  if (m_cap < 4096 || ffn == 0 || k == 0 || n_groups == 0) return STM_ERR_UNSUPPORTED;  // the unfused path handles it
  if (!a || !b || !c || !c2 || !offsets || !workspace) return STM_ERR_ARG;
  if (workspace_bytes < stm_gemm_workspace_bytes(m_cap, n_groups)) return STM_ERR_WORKSPACE;
  if (!aligned_to(a, 16) || !aligned_to(b, 16) || !aligned_to(c, 16) || !aligned_to(c2, 16)) return STM_ERR_UNSUPPORTED;
  p = GemmArgs{};
  p.a = a;
  p.b = b;
  p.c = c;
  p.c2 = c2;
  p.offsets = offsets;
  p.header = static_cast<const int32_t*>(workspace);
  p.tiles = reinterpret_cast<const MTile*>(static_cast<const char*>(workspace) + 16);
  p.n_groups = n_groups;
  p.ffn = ffn;
  p.has_limit = has_limit;
  p.limit = limit;
  return STM_OK;
}
}  // namespace

int stm_grouped_gemm_swiglu(const void* a, const void* w1, void* gate_up, void* h, const float* row_scale,
                            const int32_t* offsets, int n_groups, int64_t m_cap, int ffn, int k, int has_limit,
                            float limit, int dtype, void* workspace, size_t workspace_bytes, stm_stream_t stream) {
  using namespace stm;
  GemmArgs p;
  const int st = fused_args(a, w1, gate_up, h, offsets, n_groups, m_cap, ffn, k, has_limit, limit, dtype, workspace,
                            workspace_bytes, p);
  if (st != STM_OK) return st;
  p.lda = k;
  p.ldb = k;
  p.ldc = 2 * int64_t(ffn);
  p.ldc2 = ffn;
  p.b_group = 2 * int64_t(ffn) * k;
  p.n_j = 2 * ffn;
  p.n_k = k;
  p.row_scale = row_scale;
  return launch_dma_swiglu_fwd(dtype, p, offsets, n_groups, m_cap, workspace, as_stream(stream));
}

int stm_grouped_gemm_dswiglu_row_dot_parts(int ffn) { return ffn > 0 ? 2 * ((ffn + 255) / 256) : 0; }

int stm_grouped_gemm_dswiglu(const void* grad_y, const void* w2, const void* gate_up, void* grad_gate_up,
                             const float* row_scale, float* row_dot, const int32_t* offsets, int n_groups,
                             int64_t m_cap, int ffn, int k, int has_limit, float limit, int dtype, void* workspace,
                             size_t workspace_bytes, stm_stream_t stream) {
  using namespace stm;
  GemmArgs p;
  const int st = fused_args(grad_y, w2, grad_gate_up, const_cast<void*>(gate_up), offsets, n_groups, m_cap, ffn, k,
                            has_limit, limit, dtype, workspace, workspace_bytes, p);
  if (st != STM_OK) return st;
  p.lda = k;
  p.ldb = ffn;  // w2[g] is [k, ffn]: contraction rows, K-major for this product
  p.ldc = 2 * int64_t(ffn);
  p.ldc2 = 2 * int64_t(ffn);
  p.b_group = int64_t(ffn) * k;
  p.n_j = ffn;
  p.n_k = k;
  p.row_scale = row_scale;
  p.row_dot = row_dot;
  return launch_dma_swiglu_bwd(dtype, p, offsets, n_groups, m_cap, workspace, as_stream(stream));
}

int stm_grouped_gemm_wgrad_accum(const void* x, const void* y, float* accum, const int32_t* offsets, int n_groups,
                                 int64_t m_cap, int p_dim, int q_dim, int dtype, stm_stream_t stream) {
  using namespace stm;
  if (n_groups < 0 || m_cap < 0 || p_dim < 0 || q_dim < 0) return STM_ERR_ARG;
  if ((dtype != STM_BF16 && dtype != STM_F16) || n_groups > kMaxGroups) return STM_ERR_UNSUPPORTED;
  if (n_groups == 0 || p_dim == 0 || q_dim == 0) return STM_OK;
  if (!accum || !offsets || (m_cap > 0 && (!x || !y))) return STM_ERR_ARG;
  return launch_mfma_wgrad(dtype, x, y, accum, offsets, n_groups, m_cap, p_dim, q_dim, 1, as_stream(stream));
}

int stm_grouped_gemm_wgrad(const void* x, const void* y, void* out, const int32_t* offsets, int n_groups,
                           int64_t m_cap, int p_dim, int q_dim, int dtype, stm_stream_t stream) {
  using namespace stm;
  if (n_groups < 0 || m_cap < 0 || p_dim < 0 || q_dim < 0) return STM_ERR_ARG;
  if (dtype < STM_F32 || dtype > STM_BF16 || n_groups > kMaxGroups) return STM_ERR_UNSUPPORTED;
  if (n_groups == 0 || p_dim == 0 || q_dim == 0) return STM_OK;
  if (!out || !offsets || (m_cap > 0 && (!x || !y))) return STM_ERR_ARG;
  hipStream_t s = as_stream(stream);
  const int fast = launch_mfma_wgrad(dtype, x, y, out, offsets, n_groups, m_cap, p_dim, q_dim, 0, s);
  if (fast != STM_ERR_UNSUPPORTED) return fast;
  GenericArgs p{};
  p.a = x;
  p.b = y;
  p.c = out;
  p.offsets = offsets;
  p.sa_i = 1;
  p.sa_k = p_dim;
  p.sb_k = q_dim;
  p.sb_j = 1;
  p.c_group = int64_t(p_dim) * q_dim;
  p.ldc = q_dim;
  p.n_i = p_dim;
  p.n_j = q_dim;
  p.wgrad = 1;
  dim3 grid(unsigned((q_dim + kGT - 1) / kGT), unsigned((p_dim + kGT - 1) / kGT), unsigned(n_groups));
  return dispatch_generic(dtype, p, grid, s);
}

namespace {
// The gathered operand of a fused entry: rows of `src` [src_rows_n, k] named by row_sources [m_cap].
int gathered_source(stm::GemmArgs& p, const int32_t* row_sources, int64_t src_rows_n, int k, int64_t m_cap) {
  if (!row_sources || src_rows_n < 0) return STM_ERR_ARG;
  const int64_t bytes = src_rows_n * int64_t(k) * 2;
  if (bytes <= 0 || bytes >= (int64_t(1) << 31)) return STM_ERR_UNSUPPORTED;
  p.src_rows = row_sources;
  p.src_n_rows = m_cap;
  p.src_bytes = uint32_t(bytes);
  p.gather_operand = 1;
  return STM_OK;
}
}  // namespace

int stm_row_sources_padding(void) { return 512; }

int stm_grouped_gemm_swiglu_gathered(const void* src, int64_t src_rows_n, const int32_t* row_sources, const void* w1,
                                     void* gate_up, void* h, const float* row_scale, const int32_t* offsets,
                                     int n_groups, int64_t m_cap, int ffn, int k, int has_limit, float limit, int dtype,
                                     void* workspace, size_t workspace_bytes, stm_stream_t stream) {
  using namespace stm;
  GemmArgs p;
  int st = fused_args(src, w1, gate_up, h, offsets, n_groups, m_cap, ffn, k, has_limit, limit, dtype, workspace,
                      workspace_bytes, p);
  if (st != STM_OK) return st;
  st = gathered_source(p, row_sources, src_rows_n, k, m_cap);
  if (st != STM_OK) return st;
  p.lda = k;
  p.ldb = k;
  p.ldc = 2 * int64_t(ffn);
  p.ldc2 = ffn;
  p.b_group = 2 * int64_t(ffn) * k;
  p.n_j = 2 * ffn;
  p.n_k = k;
  p.row_scale = row_scale;
  return launch_dma_swiglu_fwd(dtype, p, offsets, n_groups, m_cap, workspace, as_stream(stream));
}

int stm_grouped_gemm_dswiglu_gathered(const void* src, int64_t src_rows_n, const int32_t* row_sources, const void* w2,
                                      const void* gate_up, void* grad_gate_up, const float* row_scale, float* row_dot,
                                      const int32_t* offsets, int n_groups, int64_t m_cap, int ffn, int k,
                                      int has_limit, float limit, int dtype, void* workspace, size_t workspace_bytes,
                                      stm_stream_t stream) {
  using namespace stm;
  GemmArgs p;
  int st = fused_args(src, w2, grad_gate_up, const_cast<void*>(gate_up), offsets, n_groups, m_cap, ffn, k, has_limit,
                      limit, dtype, workspace, workspace_bytes, p);
  if (st != STM_OK) return st;
  st = gathered_source(p, row_sources, src_rows_n, k, m_cap);
  if (st != STM_OK) return st;
  p.lda = k;
  p.ldb = ffn;
  p.ldc = 2 * int64_t(ffn);
  p.ldc2 = 2 * int64_t(ffn);
  p.b_group = int64_t(ffn) * k;
  p.n_j = ffn;
  p.n_k = k;
  p.row_scale = row_scale;
  p.row_dot = row_dot;
  return launch_dma_swiglu_bwd(dtype, p, offsets, n_groups, m_cap, workspace, as_stream(stream));
}

int stm_grouped_gemm_wgrad_gathered(const void* x, const void* y, void* out, const int32_t* offsets, int n_groups,
                                    int64_t m_cap, int p_dim, int q_dim, int dtype, const int32_t* row_sources,
                                    int gathered_operand, int64_t src_rows_n, stm_stream_t stream) {
  using namespace stm;
  if (n_groups < 0 || m_cap < 0 || p_dim < 0 || q_dim < 0 || src_rows_n < 0) return STM_ERR_ARG;
  if (gathered_operand != 1 && gathered_operand != 2) return STM_ERR_ARG;
  if ((dtype != STM_BF16 && dtype != STM_F16) || n_groups > kMaxGroups) return STM_ERR_UNSUPPORTED;
  if (n_groups == 0 || p_dim == 0 || q_dim == 0 || m_cap == 0) return STM_ERR_UNSUPPORTED;
  if (!out || !offsets || !x || !y || !row_sources) return STM_ERR_ARG;
  return launch_mfma_wgrad(dtype, x, y, out, offsets, n_groups, m_cap, p_dim, q_dim, 0, as_stream(stream), row_sources,
                           gathered_operand, src_rows_n);
}

}  // extern "C"
