// bf16 / fp16 grouped GEMM, main kernels: buffer_load ... lds (HBM -> LDS without a register
// stop), four LDS stages of 32 contraction elements, XOR-swizzled LDS rows, 32x32x16 MFMA.
//
// Compared with the register-staged kernels of gemm_mfma.hip this keeps three stages of
// loads in flight per workgroup (the latency of a load is covered by three compute steps
// instead of one) and spends no VGPRs on staging.  The loads are raw buffer loads: anything
// past the end of the operand's valid region (rows past a ragged group, rows past the tile
// of a short M-tile) comes back as zero from the bounds check, so ragged edges need no
// branches.  The same three products are covered as in gemm_mfma.hip:
//
//   fwd   C = A  * W^T   A:[M,K] KC   W[g]:[N,K] KC
//   dgrad C = dY * W     dY:[M,K] KC  W[g]:[K,N] KM
//   wgrad O = X^T * Y    X:[M,P] KM   Y:[M,Q] KM
//
// KC = rows of the operand are contraction-contiguous (read with ds_read_b128),
// KM = rows of the operand are contraction steps   (read with ds_read_b64_tr_b16).
//
// LDS layout of one stage (BK = 32):
//   KC tile: row r (64 B) at r*64, its four 16-byte chunks stored at chunk ^ ((r >> 2) & 3);
//            16 consecutive rows read the same logical chunk from 16 distinct bank groups.
//   KM tile: contraction row k (R*2 B) at k*R*2, its 64-byte chunks stored at chunk ^ (k & 3);
//            the four rows a transposing read touches land in the four quarters of the banks.
// A wave-wide buffer_load ... lds writes 1024 consecutive LDS bytes (lane l at +16*l), so the
// swizzle is applied on the global-address side.
#include "gemm_common.hpp"

namespace stm {

using DmaGemmArgs = GemmArgs;

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
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

constexpr int kBK = 32;
constexpr int kStages = 4;
constexpr int kThreads = 256;

template <typename T>
struct alignas(sizeof(T) * 4) Pack4 {
  T v[4];
};

// Raw buffer descriptor over [base, base + bytes): reads past the end return zero.
__device__ __forceinline__ i32x4_t make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t p = reinterpret_cast<uint64_t>(base);
  i32x4_t r;
  r[0] = int(uint32_t(p));
  r[1] = int(uint32_t(p >> 32) & 0xffffu);  // stride 0
  r[2] = int(bytes);
  r[3] = 0x00020000;
  return r;
}

// One wave-wide 16-byte-per-lane load straight into LDS at lds_addr + 16*lane.
__device__ __forceinline__ void dma16(i32x4_t rsrc, uint32_t lds_addr, uint32_t voffset, uint32_t soffset) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen lds"
      :
      : "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset)
      : "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// Per-thread plan of one operand's loads for a stage: R/64 wave-loads per wave.
template <int R, bool KM>
struct OperandPlan {
  static constexpr int kLoadsPerWave = R / 64;     // (R*64 B per stage) / 1024 B / 4 waves
  static constexpr int kStageBytes = R * kBK * 2;  // 16-bit elements
  uint32_t voff[kLoadsPerWave];                    // byte offset of this lane's 16 bytes at step 0
  uint32_t lds_off[kLoadsPerWave];                 // wave-uniform LDS offset of the wave-load
  uint32_t step_bytes;                             // soffset increment per contraction step

  __device__ __forceinline__ void init(int64_t ld_elems) {
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
#pragma unroll
    for (int j = 0; j < kLoadsPerWave; ++j) {
      const int wl = wave * kLoadsPerWave + j;
      lds_off[j] = uint32_t(wl) * 1024u;
      if constexpr (!KM) {
        const int row = wl * 16 + lane / 4;
        const int logical = (lane % 4) ^ (lane / 16);  // == phys ^ ((row >> 2) & 3)
        voff[j] = uint32_t(row) * uint32_t(ld_elems * 2) + uint32_t(logical) * 16u;
      } else {
        constexpr int kChunks16 = R / 8;  // 16-byte chunks per stored row
        constexpr int kRowsPerLoad = 64 / kChunks16;
        const int row = wl * kRowsPerLoad + lane / kChunks16;
        const int c16 = lane % kChunks16;
        const int logical64 = (c16 / 4) ^ (row & 3);
        const int col = logical64 * 32 + (c16 % 4) * 8;
        voff[j] = uint32_t(row) * uint32_t(ld_elems * 2) + uint32_t(col) * 2u;
      }
    }
    step_bytes = KM ? uint32_t(kBK * ld_elems * 2) : uint32_t(kBK * 2);
  }

  __device__ __forceinline__ void issue(i32x4_t rsrc, uint32_t lds_stage_addr, int step) const {
    const uint32_t soff = __builtin_amdgcn_readfirstlane(uint32_t(step) * step_bytes);
#pragma unroll
    for (int j = 0; j < kLoadsPerWave; ++j)
      dma16(rsrc, __builtin_amdgcn_readfirstlane(lds_stage_addr + lds_off[j]), voff[j], soff);
  }
};

// 8 contraction values (k = kk*16 + (lane/32)*8 .. +8) of output row/column r0 + lane%32.
template <int R, bool KM>
__device__ __forceinline__ uint4 read_fragment(const unsigned char* tile, int r0, int kk) {
  const int lane = threadIdx.x % kWave;
  if constexpr (!KM) {
    const int r = r0 + lane % 32;
    const int chunk = (kk * 2 + lane / 32) ^ ((r >> 2) & 3);
    return *reinterpret_cast<const uint4*>(tile + r * 64 + chunk * 16);
  } else {
    const int i = lane % 16;
    const int col = r0 + ((lane / 16) & 1) * 16 + 4 * (i % 4);
    const int row = kk * 16 + (lane / 32) * 8 + i / 4;  // second read: row + 4 (same row & 3)
    const int chunk = (col / 32) ^ (row & 3);
    const unsigned char* p0 = tile + row * (R * 2) + chunk * 64 + (col % 32) * 2;
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p0));
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p0 + 4 * R * 2));
    const uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
    return make_uint4(a.x, a.y, b.x, b.y);
  }
}

template <typename T, int BM, int BN, bool A_KM, bool B_KM, bool WGRAD>
__global__ __launch_bounds__(kThreads) void dma_gemm_kernel(DmaGemmArgs p) {
  constexpr int TM = BM / 64, TN = BN / 64;  // 32x32 MFMA tiles per wave (waves are laid out 2 x 2)
  using PlanA = OperandPlan<BM, A_KM>;
  using PlanB = OperandPlan<BN, B_KM>;
  constexpr uint32_t kStageBytes = PlanA::kStageBytes + PlanB::kStageBytes;
  constexpr int kLoadsPerStep = PlanA::kLoadsPerWave + PlanB::kLoadsPerWave;
  extern __shared__ __align__(1024) unsigned char smem[];

  // ---- which tile is this workgroup's?
  const int64_t id = xcd_contiguous_id(blockIdx.x, p.blocks_padded);
  const T* a = static_cast<const T*>(p.a);
  const T* b = static_cast<const T*>(p.b);
  T* c = static_cast<T*>(p.c);
  int valid_i, valid_j, n_k;
  uint32_t a_bytes, b_bytes;
  const int jt = int(id % p.tiles_j);
  const int j0 = jt * BN;
  valid_j = p.n_j - j0;
  if constexpr (WGRAD) {
    const int64_t rest = id / p.tiles_j;
    const int it = int(rest % p.tiles_i);
    const int64_t g = rest / p.tiles_i;
    if (g >= p.n_groups) return;
    const int64_t lo = p.offsets[g], hi = p.offsets[g + 1];
    n_k = hi > lo ? int(hi - lo) : 0;
    const int i0 = it * BM;
    valid_i = p.n_i - i0;
    a += lo * p.lda + i0;
    b += lo * p.ldb + j0;
    c += g * p.c_group + int64_t(i0) * p.ldc + j0;
    // contraction rows past the end of the group are past the end of the buffer: zeros
    a_bytes = uint32_t(int64_t(n_k) * p.lda * 2 - int64_t(i0) * 2);
    b_bytes = uint32_t(int64_t(n_k) * p.ldb * 2 - int64_t(j0) * 2);
  } else {
    const int64_t mt = id / p.tiles_j;
    if (mt >= p.header[0]) return;
    const MTile t = p.tiles[mt];
    n_k = p.n_k;
    valid_i = t.rows;
    a += int64_t(t.row0) * p.lda;
    c += int64_t(t.row0) * p.ldc + j0;
    a_bytes = uint32_t(int64_t(t.rows) * p.lda * 2);
    if constexpr (B_KM) {
      b += int64_t(t.group) * p.b_group + j0;
      b_bytes = uint32_t(int64_t(p.n_k) * p.ldb * 2 - int64_t(j0) * 2);
    } else {
      b += int64_t(t.group) * p.b_group + int64_t(j0) * p.ldb;
      b_bytes = uint32_t(int64_t(valid_j < BN ? valid_j : BN) * p.ldb * 2);
    }
  }
  i32x4_t rsrc_a = make_rsrc(a, a_bytes);
  i32x4_t rsrc_b = make_rsrc(b, b_bytes);
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    rsrc_a[w] = __builtin_amdgcn_readfirstlane(rsrc_a[w]);
    rsrc_b[w] = __builtin_amdgcn_readfirstlane(rsrc_b[w]);
  }

  PlanA plan_a;
  PlanB plan_b;
  plan_a.init(p.lda);
  plan_b.init(p.ldb);
  const uint32_t lds_base =
      uint32_t(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char*)smem));  // LDS offset

  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int wave_i = (wave / 2) * (BM / 2);
  const int wave_j = (wave % 2) * (BN / 2);

  f32x16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int n_steps = (n_k + kBK - 1) / kBK;
  auto issue = [&](int step) {
    const uint32_t stage = lds_base + uint32_t(step % kStages) * kStageBytes;
    plan_a.issue(rsrc_a, stage, step);
    plan_b.issue(rsrc_b, stage + PlanA::kStageBytes, step);
  };
#pragma unroll
  for (int s = 0; s < kStages - 1; ++s)
    if (s < n_steps) issue(s);

  for (int step = 0; step < n_steps; ++step) {
    // loads of stages step+1, step+2 may stay in flight; everything older must have landed
    const int later = n_steps - 1 - step;
    if (later >= 2)
      wait_vmcnt<2 * kLoadsPerStep>();
    else if (later == 1)
      wait_vmcnt<kLoadsPerStep>();
    else
      wait_vmcnt<0>();
    __syncthreads();  // every wave's part of this stage is in LDS; stage (step-1) is free again
    if (step + kStages - 1 < n_steps) issue(step + kStages - 1);
    const unsigned char* ta = smem + (step % kStages) * kStageBytes;
    const unsigned char* tb = ta + PlanA::kStageBytes;
#pragma unroll
    for (int kk = 0; kk < kBK / 16; ++kk) {
      uint4 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = read_fragment<BM, A_KM>(ta, wave_i + i * 32, kk);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = read_fragment<BN, B_KM>(tb, wave_j + j * 32, kk);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<T>::run(fb[j], fa[i], acc[i][j]);
    }
  }

  // ---- epilogue: lane owns row (lane % 32) and, per group of four registers, four
  // consecutive columns starting at (r/4)*8 + (lane/32)*4.
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int row = wave_i + i * 32 + lane % 32;
    if (row >= valid_i) continue;
    T* crow = c + int64_t(row) * p.ldc;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = wave_j + j * 32 + q * 8 + (lane / 32) * 4;
        if (col >= valid_j) continue;
        Pack4<T> out;
#pragma unroll
        for (int e = 0; e < 4; ++e) out.v[e] = from_float<T>(acc[i][j][q * 4 + e]);
        *reinterpret_cast<Pack4<T>*>(crow + col) = out;
      }
    }
  }
}

template <typename T, int BM, int BN, bool A_KM, bool B_KM, bool WGRAD>
int launch(const DmaGemmArgs& p, int64_t n_blocks, hipStream_t s) {
  auto kernel = dma_gemm_kernel<T, BM, BN, A_KM, B_KM, WGRAD>;
  constexpr size_t smem = size_t(kStages) * (BM + BN) * kBK * 2;
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            int(smem)) != hipSuccess)
      return STM_ERR_LAUNCH;
    configured = true;
  }
  DmaGemmArgs q = p;
  q.blocks_padded = pad_to_xcd(n_blocks);
  kernel<<<unsigned(q.blocks_padded), kThreads, smem, s>>>(q);
  return launch_status();
}

}  // namespace

constexpr int kDmaBM = 256, kDmaBN = 256;

// rows form; returns STM_ERR_UNSUPPORTED when the shape does not fit these kernels.
int launch_dma_rows(int dtype, const DmaGemmArgs& base, const int32_t* offsets, int n_groups, int64_t m_cap,
                    int b_is_nk, void* ws, hipStream_t s) {
  DmaGemmArgs p = base;
  if (p.n_k % kBK != 0 || p.n_j % 8 != 0) return STM_ERR_UNSUPPORTED;
  if (int64_t(p.n_k) * p.ldb * 2 >= (int64_t(1) << 32) || int64_t(kDmaBM) * p.lda * 2 >= (int64_t(1) << 32))
    return STM_ERR_UNSUPPORTED;
  const int st = build_tile_table(offsets, n_groups, kDmaBM, m_cap, ws, s);
  if (st != STM_OK) return st;
  p.tiles_j = (p.n_j + kDmaBN - 1) / kDmaBN;
  const int64_t blocks = max_m_tiles(m_cap, n_groups, kDmaBM) * p.tiles_j;
  if (dtype == STM_BF16)
    return b_is_nk ? launch<bf16_t, kDmaBM, kDmaBN, false, false, false>(p, blocks, s)
                   : launch<bf16_t, kDmaBM, kDmaBN, false, true, false>(p, blocks, s);
  return b_is_nk ? launch<f16_t, kDmaBM, kDmaBN, false, false, false>(p, blocks, s)
                 : launch<f16_t, kDmaBM, kDmaBN, false, true, false>(p, blocks, s);
}

int launch_dma_wgrad(int dtype, const DmaGemmArgs& base, int n_groups, int64_t m_cap, hipStream_t s) {
  DmaGemmArgs p = base;
  if (p.n_i % 8 != 0 || p.n_j % 8 != 0) return STM_ERR_UNSUPPORTED;
  if (m_cap * p.lda * 2 >= (int64_t(1) << 32) || m_cap * p.ldb * 2 >= (int64_t(1) << 32)) return STM_ERR_UNSUPPORTED;
  p.tiles_i = (p.n_i + kDmaBM - 1) / kDmaBM;
  p.tiles_j = (p.n_j + kDmaBN - 1) / kDmaBN;
  const int64_t blocks = int64_t(n_groups) * p.tiles_i * p.tiles_j;
  if (dtype == STM_BF16) return launch<bf16_t, kDmaBM, kDmaBN, true, true, true>(p, blocks, s);
  return launch<f16_t, kDmaBM, kDmaBN, true, true, true>(p, blocks, s);
}

}  // namespace stm
