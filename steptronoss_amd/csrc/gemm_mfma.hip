// bf16 / fp16 grouped GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x16_{bf16,f16}).
//
// One workgroup computes a BM x BN tile of one expert's output, stepping BK = 64 through the
// contraction.  Tiles are fetched from HBM with 128-bit loads in whatever direction memory is
// contiguous, staged in LDS (two stages), and handed to the matrix cores either with
// ds_read_b128 (operand stored contraction-contiguous, "KC") or with the CDNA4 transposing
// ds_read_b64_tr_b16 (operand stored contraction-major, "KM").  That covers all three products
// of the expert FFN without ever materialising a transposed copy of a weight or activation:
//
//   fwd   C = A  * W^T   A:[M,K] KC   W[g]:[N,K] KC          (trans_b = True)
//   dgrad C = dY * W     dY:[M,K] KC  W[g]:[K,N] KM          (contraction runs over W's rows)
//   wgrad O = X^T * Y    X:[M,P] KM   Y:[M,Q] KM             (contraction runs over the rows)
//
// The MFMA is issued with the operands swapped (D^T = B^T A^T), so every lane ends up owning
// four consecutive output columns and stores them as one 64-bit word.
#include "gemm_common.hpp"

namespace stm {

int launch_dma_rows(int dtype, const GemmArgs& base, const int32_t* offsets, int n_groups, int64_t m_cap, int b_is_nk,
                    void* ws, hipStream_t s);
int launch_dma_wgrad(int dtype, const GemmArgs& base, int n_groups, int64_t m_cap, int accumulate, hipStream_t s);

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4_t* lds_s16x4_ptr;

template <typename T>
struct Mfma;
template <>
struct Mfma<bf16_t> {
  static __device__ __forceinline__ f32x16_t run(uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
  }
};
template <>
struct Mfma<f16_t> {
  static __device__ __forceinline__ f32x16_t run(uint4 a, uint4 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c,
                                                  0, 0, 0);
  }
};

constexpr int kBK = 64;     // contraction elements per stage
constexpr int kPadKC = 8;   // elements of padding per KC row  (16 B: conflict-free ds_read_b128)
constexpr int kPadKM = 32;  // elements of padding per KM row  (64 B: conflict-free transposing reads)

// Geometry of one staged operand tile of R rows/columns of the output.
template <int R, bool KM>
struct TileShape {
  static constexpr int kRows = KM ? kBK : R;               // rows as stored
  static constexpr int kCols = KM ? R : kBK;               // contiguous elements per stored row
  static constexpr int kLd = kCols + (KM ? kPadKM : kPadKC);  // LDS leading dimension (elements)
  static constexpr int kElems = kRows * kLd;
};

template <typename T, int R, bool KM, int THREADS>
struct TileIO {
  using S = TileShape<R, KM>;
  static constexpr int kVecPerRow = S::kCols / 8;
  static constexpr int kVecs = S::kRows * kVecPerRow / THREADS;
  static_assert(S::kRows * kVecPerRow % THREADS == 0, "tile must split evenly over the workgroup");

  // origin: first element of the tile in memory; zero-fills outside [valid_rows, valid_cols).
  static __device__ __forceinline__ void load(uint4 (&regs)[kVecs], const T* origin, int64_t ld, int valid_rows,
                                              int valid_cols) {
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
      const int v = threadIdx.x + i * THREADS;
      const int r = v / kVecPerRow;
      const int c = (v % kVecPerRow) * 8;
      uint4 val = make_uint4(0, 0, 0, 0);
      if (r < valid_rows && c < valid_cols) val = *reinterpret_cast<const uint4*>(origin + int64_t(r) * ld + c);
      regs[i] = val;
    }
  }
  static __device__ __forceinline__ void store(const uint4 (&regs)[kVecs], T* lds) {
#pragma unroll
    for (int i = 0; i < kVecs; ++i) {
      const int v = threadIdx.x + i * THREADS;
      const int r = v / kVecPerRow;
      const int c = (v % kVecPerRow) * 8;
      *reinterpret_cast<uint4*>(lds + r * S::kLd + c) = regs[i];
    }
  }
};

// 8 contraction values (k = kk*16 + (lane/32)*8 .. +8) of output row/column  r0 + lane%32.
template <typename T, int R, bool KM>
__device__ __forceinline__ uint4 read_fragment(const T* lds, int r0, int kk) {
  using S = TileShape<R, KM>;
  const int lane = threadIdx.x % kWave;
  if constexpr (!KM) {
    return *reinterpret_cast<const uint4*>(lds + (r0 + lane % 32) * S::kLd + kk * 16 + (lane / 32) * 8);
  } else {
    // transposing read: in each 16-lane group, lanes 4r..4r+3 name stored row r (4 elements
    // each) and lane i receives column i of those four rows.
    const int i = lane % 16;
    const int col = r0 + ((lane / 16) & 1) * 16 + 4 * (i % 4);
    const int row = kk * 16 + (lane / 32) * 8 + i / 4;
    const T* p0 = lds + row * S::kLd + col;
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p0));
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p0 + 4 * S::kLd));
    uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
    return make_uint4(a.x, a.y, b.x, b.y);
  }
}

using MfmaArgs = GemmArgs;

template <typename T>
struct alignas(sizeof(T) * 4) Pack4 {
  T v[4];
};

template <int BM_, int BN_, int WM_, int WN_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
  static constexpr int kThreads = WM * WN * kWave;
  static constexpr int TM = BM / WM / 32;  // 32x32 MFMA tiles per wave along M
  static constexpr int TN = BN / WN / 32;
};

template <typename T, typename C, bool A_KM, bool B_KM>
constexpr size_t smem_bytes() {
  return 2 * size_t(TileShape<C::BM, A_KM>::kElems + TileShape<C::BN, B_KM>::kElems) * sizeof(T);
}

template <typename T, typename C, bool A_KM, bool B_KM, bool WGRAD>
__global__ __launch_bounds__(C::kThreads) void mfma_gemm_kernel(MfmaArgs p) {
  using SA = TileShape<C::BM, A_KM>;
  using SB = TileShape<C::BN, B_KM>;
  using IOA = TileIO<T, C::BM, A_KM, C::kThreads>;
  using IOB = TileIO<T, C::BN, B_KM, C::kThreads>;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T* smem = reinterpret_cast<T*>(smem_raw);
  T* lds_a[2] = {smem, smem + SA::kElems};
  T* lds_b[2] = {smem + 2 * SA::kElems, smem + 2 * SA::kElems + SB::kElems};

  // ---- which tile is this workgroup's?
  const int64_t n_tiles = WGRAD ? int64_t(p.n_groups) * p.tiles_i * p.tiles_j : int64_t(p.header[0]) * p.tiles_j;
  const int64_t id = xcd_contiguous_id(blockIdx.x, n_tiles);
  if (id < 0) return;
  const T* a = static_cast<const T*>(p.a);
  const T* b = static_cast<const T*>(p.b);
  T* c = static_cast<T*>(p.c);
  int valid_i, valid_j, n_k, i0 = 0;
  const int jt = int(id % p.tiles_j);
  const int j0 = jt * C::BN;
  valid_j = p.n_j - j0;
  if constexpr (WGRAD) {
    const int64_t rest = id / p.tiles_j;
    const int it = int(rest % p.tiles_i);
    const int64_t g = rest / p.tiles_i;
    if (g >= p.n_groups) return;  // padding workgroups of the XCD-aligned grid
    const int64_t lo = p.offsets[g], hi = p.offsets[g + 1];
    n_k = hi > lo ? int(hi - lo) : 0;
    i0 = it * C::BM;
    valid_i = p.n_i - i0;
    a += lo * p.lda + i0;  // KM: rows are contraction steps
    b += lo * p.ldb + j0;
    c += g * p.c_group + int64_t(i0) * p.ldc + j0;
  } else {
    const int64_t mt = id / p.tiles_j;
    if (mt >= p.header[0]) return;
    const MTile t = p.tiles[mt];
    n_k = p.n_k;
    valid_i = t.rows;
    a += int64_t(t.row0) * p.lda;
    b += int64_t(t.group) * p.b_group + (B_KM ? int64_t(j0) : int64_t(j0) * p.ldb);
    c += int64_t(t.row0) * p.ldc + j0;
  }

  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int wave_i = (wave / C::WN) * (C::TM * 32);
  const int wave_j = (wave % C::WN) * (C::TN * 32);

  f32x16_t acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  uint4 ra[IOA::kVecs], rb[IOB::kVecs];
  auto fetch = [&](int k0) {
    const int left = n_k - k0;
    if constexpr (A_KM)
      IOA::load(ra, a + int64_t(k0) * p.lda, p.lda, left, valid_i);
    else
      IOA::load(ra, a + k0, p.lda, valid_i, left);
    if constexpr (B_KM)
      IOB::load(rb, b + int64_t(k0) * p.ldb, p.ldb, left, valid_j);
    else
      IOB::load(rb, b + k0, p.ldb, valid_j, left);
  };

  const int n_steps = (n_k + kBK - 1) / kBK;
  if (n_steps > 0) {
    fetch(0);
    IOA::store(ra, lds_a[0]);
    IOB::store(rb, lds_b[0]);
  }
  __syncthreads();
  for (int step = 0; step < n_steps; ++step) {
    const int cur = step & 1;
    const bool more = step + 1 < n_steps;
    if (more) fetch((step + 1) * kBK);
    const T* sa = lds_a[cur];
    const T* sb = lds_b[cur];
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      uint4 fa[C::TM], fb[C::TN];
#pragma unroll
      for (int i = 0; i < C::TM; ++i) fa[i] = read_fragment<T, C::BM, A_KM>(sa, wave_i + i * 32, kk);
#pragma unroll
      for (int j = 0; j < C::TN; ++j) fb[j] = read_fragment<T, C::BN, B_KM>(sb, wave_j + j * 32, kk);
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j) acc[i][j] = Mfma<T>::run(fb[j], fa[i], acc[i][j]);
    }
    if (more) {
      IOA::store(ra, lds_a[cur ^ 1]);
      IOB::store(rb, lds_b[cur ^ 1]);
    }
    __syncthreads();
  }

  // ---- epilogue: lane owns row (lane % 32) and, per group of four registers, four
  // consecutive columns starting at (r/4)*8 + (lane/32)*4.
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    const int row = wave_i + i * 32 + lane % 32;
    if (row >= valid_i) continue;
    T* crow = c + int64_t(row) * p.ldc;
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = wave_j + j * 32 + q * 8 + (lane / 32) * 4;
        if (col >= valid_j) continue;  // N is a multiple of 8, so a group of four is all in or all out
        Pack4<T> out;
#pragma unroll
        for (int e = 0; e < 4; ++e) out.v[e] = from_float<T>(acc[i][j][q * 4 + e]);
        *reinterpret_cast<Pack4<T>*>(crow + col) = out;
      }
    }
  }
}

template <typename T, typename C, bool A_KM, bool B_KM, bool WGRAD>
int launch(const MfmaArgs& p, int64_t n_blocks, hipStream_t s) {
  auto kernel = mfma_gemm_kernel<T, C, A_KM, B_KM, WGRAD>;
  constexpr size_t smem = smem_bytes<T, C, A_KM, B_KM>();
  static bool configured = false;  // raising the dynamic-LDS limit is a per-function, process-wide setting
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            int(smem)) != hipSuccess)
      return STM_ERR_LAUNCH;
    configured = true;
  }
  MfmaArgs q = p;
  q.blocks_padded = pad_to_xcd(n_blocks);
  kernel<<<unsigned(q.blocks_padded), C::kThreads, smem, s>>>(q);
  return launch_status();
}

using Big = Cfg<256, 256, 2, 2>;
using Mid = Cfg<128, 128, 2, 2>;

template <typename T>
int rows_typed(const MfmaArgs& base, const int32_t* offsets, int n_groups, int64_t m_cap, int b_is_nk, void* ws,
               hipStream_t s) {
  MfmaArgs p = base;
  const bool big = m_cap >= 8192 && p.n_j >= 512;
  const int bm = big ? Big::BM : Mid::BM;
  const int bn = big ? Big::BN : Mid::BN;
  int st = build_tile_table(offsets, n_groups, bm, m_cap, ws, s);
  if (st != STM_OK) return st;
  p.tiles_j = (p.n_j + bn - 1) / bn;
  const int64_t blocks = max_m_tiles(m_cap, n_groups, bm) * p.tiles_j;
  if (big) {
    return b_is_nk ? launch<T, Big, false, false, false>(p, blocks, s) : launch<T, Big, false, true, false>(p, blocks, s);
  }
  return b_is_nk ? launch<T, Mid, false, false, false>(p, blocks, s) : launch<T, Mid, false, true, false>(p, blocks, s);
}

template <typename T>
int wgrad_typed(const MfmaArgs& base, int n_groups, hipStream_t s) {
  MfmaArgs p = base;
  const bool big = p.n_i >= 512 && p.n_j >= 512;
  const int bm = big ? Big::BM : Mid::BM;
  const int bn = big ? Big::BN : Mid::BN;
  p.tiles_i = (p.n_i + bm - 1) / bm;
  p.tiles_j = (p.n_j + bn - 1) / bn;
  const int64_t blocks = int64_t(n_groups) * p.tiles_i * p.tiles_j;
  return big ? launch<T, Big, true, true, true>(p, blocks, s) : launch<T, Mid, true, true, true>(p, blocks, s);
}

}  // namespace

int launch_mfma_rows(int dtype, const void* a, const void* b, void* c, const int32_t* offsets, int n_groups,
                     int64_t m_cap, int n, int k, int b_is_nk, void* ws, size_t ws_bytes, hipStream_t s) {
  if (dtype != STM_BF16 && dtype != STM_F16) return STM_ERR_UNSUPPORTED;
  if (n % 8 != 0 || k % 8 != 0 || k == 0) return STM_ERR_UNSUPPORTED;
  if (!aligned_to(a, 16) || !aligned_to(b, 16) || !aligned_to(c, 16)) return STM_ERR_UNSUPPORTED;
  if (ws_bytes < tile_table_bytes(m_cap, n_groups, Mid::BM)) return STM_ERR_WORKSPACE;
  MfmaArgs p{};
  p.a = a;
  p.b = b;
  p.c = c;
  p.offsets = offsets;
  p.header = static_cast<const int32_t*>(ws);
  p.tiles = reinterpret_cast<const MTile*>(static_cast<const char*>(ws) + 16);
  p.lda = k;
  p.ldb = b_is_nk ? k : n;
  p.ldc = n;
  p.b_group = int64_t(n) * k;
  p.n_j = n;
  p.n_k = k;
  p.n_groups = n_groups;
  if (m_cap >= 4096 && n >= 256) {  // enough work for 256x256 tiles: the buffer_load->LDS kernels
    const int st = launch_dma_rows(dtype, p, offsets, n_groups, m_cap, b_is_nk, ws, s);
    if (st != STM_ERR_UNSUPPORTED) return st;
  }
  return dtype == STM_BF16 ? rows_typed<bf16_t>(p, offsets, n_groups, m_cap, b_is_nk, ws, s)
                           : rows_typed<f16_t>(p, offsets, n_groups, m_cap, b_is_nk, ws, s);
}

// accumulate != 0: `out` is an fp32 buffer the product is added to (only the 256 x 256 kernels do that).
int launch_mfma_wgrad(int dtype, const void* x, const void* y, void* out, const int32_t* offsets, int n_groups,
                      int64_t m_cap, int p_dim, int q_dim, int accumulate, hipStream_t s, const int32_t* src_rows,
                      int gather_operand, int64_t src_buffer_rows) {
  (void)m_cap;
  if (dtype != STM_BF16 && dtype != STM_F16) return STM_ERR_UNSUPPORTED;
  if (p_dim % 8 != 0 || q_dim % 8 != 0) return STM_ERR_UNSUPPORTED;
  if (!aligned_to(x, 16) || !aligned_to(y, 16) || !aligned_to(out, 16)) return STM_ERR_UNSUPPORTED;
  MfmaArgs p{};
  p.a = x;
  p.b = y;
  p.c = out;
  p.offsets = offsets;
  p.lda = p_dim;
  p.ldb = q_dim;
  p.ldc = q_dim;
  p.c_group = int64_t(p_dim) * q_dim;
  p.n_i = p_dim;
  p.n_j = q_dim;
  p.n_groups = n_groups;
  if (src_rows) {  // a gathered operand: the persistent kernel or nothing
    const int64_t bytes = src_buffer_rows * (gather_operand == 2 ? q_dim : p_dim) * 2;
    if (p_dim < 256 || q_dim < 256 || bytes <= 0 || bytes >= (int64_t(1) << 31)) return STM_ERR_UNSUPPORTED;
    p.src_rows = src_rows;
    p.src_n_rows = m_cap;
    p.src_bytes = uint32_t(bytes);
    p.gather_operand = gather_operand;
    return launch_dma_wgrad(dtype, p, n_groups, m_cap, accumulate, s);
  }
  if (p_dim >= 256 && q_dim >= 256) {
    const int st = launch_dma_wgrad(dtype, p, n_groups, m_cap, accumulate, s);
    if (st != STM_ERR_UNSUPPORTED) return st;
  }
  if (accumulate) return STM_ERR_UNSUPPORTED;
  return dtype == STM_BF16 ? wgrad_typed<bf16_t>(p, n_groups, s) : wgrad_typed<f16_t>(p, n_groups, s);
}

}  // namespace stm
