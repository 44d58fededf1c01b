// fp8 (OCP e4m3, max 448) path of the expert GEMMs: a quantiser with one fp32 scale per row per
// 128 contraction elements, and a grouped GEMM C[m,n] = sum_kb sa[m,kb] * sb[n,kb] * (qa . qb)
// over such operands (32x32x16 fp8 MFMA, fp32 block accumulators folded into the fp32 result
// once per 128-block).  This path has no counterpart in the reference; it serves the fp8
// configuration of the benchmark (forward and dgrad: dgrad is the same product on the
// transposed, separately quantised weights).
#include "gemm_common.hpp"

namespace stm {
namespace {

constexpr int kQBlock = 128;  // contraction elements per scale
constexpr float kE4m3Max = 448.f;

// Nearest e4m3 value, ties to even, saturating; returns the code.
__device__ __forceinline__ uint32_t e4m3_code(float v) {
  const uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
  float a = fminf(fabsf(v), kE4m3Max);
  uint32_t code;
  if (a < 0.015625f) {  // below the smallest normal 2^-6: multiples of 2^-9
    code = uint32_t(rintf(a * 512.f));  // 8 = the smallest normal
  } else {
    uint32_t bits = __float_as_uint(a);
    bits += 0x7ffffu + ((bits >> 20) & 1u);  // round the 23-bit mantissa to 3 bits, ties to even
    code = (((bits >> 23) - 120u) << 3) | ((bits >> 20) & 7u);
  }
  return sign | code;
}

// The scale of a block whose largest magnitude is amax: amax / 448, or (POW2) the smallest power
// of two that is not below it, which the block-scaled MFMA takes as an exponent byte.
template <bool POW2>
__device__ __forceinline__ float block_scale(float amax) {
  if (!(amax > 0.f)) return 1.f;
  const float s = amax / kE4m3Max;
  if constexpr (!POW2) return s;
  uint32_t b = __float_as_uint(s);
  b = (b & 0x7fffffu) ? (b & 0x7f800000u) + 0x00800000u : (b & 0x7f800000u);
  return __uint_as_float(b < 0x00800000u ? 0x00800000u : b);  // at least the smallest normal
}

// 16 lanes per (row, block), eight elements per lane (one 16-byte load of 16-bit inputs, one
// 8-byte store of codes); a wavefront takes four blocks.  cols is a multiple of 8 here.
template <typename T>
struct alignas(sizeof(T) * 8) In8 {
  T v[8];
};

// POW2: power-of-two scales, stored block-major (scales[b * rows + r]) for the GEMM that reads
// them by row; otherwise scales[r * n_blocks + b].
template <typename T, bool POW2>
__global__ __launch_bounds__(256) void quantize_vec_kernel(const T* __restrict__ x, uint8_t* __restrict__ codes,
                                                           float* __restrict__ scales, int64_t rows, int64_t cols,
                                                           int64_t n_blocks) {
  const int sub = threadIdx.x % 16;
  const int64_t unit = (int64_t(blockIdx.x) * 256 + threadIdx.x) / 16;
  const bool live = unit < rows * n_blocks;
  const int64_t r = live ? unit / n_blocks : 0, b = live ? unit % n_blocks : 0;
  const int64_t c0 = b * kQBlock + sub * 8;
  float v[8];
  const bool in = live && c0 < cols;
  if (in) {
    In8<T> raw;
    if constexpr (sizeof(In8<T>) == 16) {  // streamed: every input byte is read once
      typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
      raw = __builtin_bit_cast(In8<T>, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + r * cols + c0)));
    } else {
      raw = *reinterpret_cast<const In8<T>*>(x + r * cols + c0);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = to_float(raw.v[e]);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = 0.f;
  }
  float amax = 0.f;
#pragma unroll
  for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[e]));
  // the largest magnitude of the 16 lanes of this block: four rotations inside the 16-lane row
  // (row_ror 8, 4, 2, 1 on the data-parallel path; every lane ends up with the maximum)
#define STM_ROW_ROR_MAX(CTRL) \
  amax = fmaxf(amax, __builtin_bit_cast(float, dpp_move<CTRL, 0xf>(0, __builtin_bit_cast(int, amax))))
  STM_ROW_ROR_MAX(0x128);
  STM_ROW_ROR_MAX(0x124);
  STM_ROW_ROR_MAX(0x122);
  STM_ROW_ROR_MAX(0x121);
#undef STM_ROW_ROR_MAX
  const float scale = block_scale<POW2>(amax);
  if (live && sub == 0) scales[POW2 ? b * rows + r : r * n_blocks + b] = scale;
  if (in) {
    float q[8];
    if constexpr (POW2) {
      // 1 / 2^e as a bit pattern: the product is the exact quotient
      const float inv = __uint_as_float(0x7f000000u - __float_as_uint(scale));
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = v[e] * inv;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = v[e] / scale;
    }
    // the hardware conversion (OCP e4m3 on gfx950: nearest even, subnormals kept); |q| <= 448
    int lo = 0, hi = 0;
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], lo, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], lo, true);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], hi, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], hi, true);
    *reinterpret_cast<uint2*>(codes + r * cols + c0) = make_uint2(uint32_t(lo), uint32_t(hi));
  }
}

// Any width / alignment: one wavefront per (row, block), two elements per lane.
template <typename T, bool POW2>
__global__ __launch_bounds__(256) void quantize_kernel(const T* __restrict__ x, uint8_t* __restrict__ codes,
                                                       float* __restrict__ scales, int64_t rows, int64_t cols,
                                                       int64_t n_blocks) {
  const int lane = threadIdx.x % kWave;
  const int64_t unit = int64_t(blockIdx.x) * (256 / kWave) + threadIdx.x / kWave;
  if (unit >= rows * n_blocks) return;
  const int64_t r = unit / n_blocks, b = unit % n_blocks;
  const int64_t c0 = b * kQBlock + lane * 2;
  float v0 = c0 < cols ? to_float(x[r * cols + c0]) : 0.f;
  float v1 = c0 + 1 < cols ? to_float(x[r * cols + c0 + 1]) : 0.f;
  const float amax = wave_max(fmaxf(fabsf(v0), fabsf(v1)));
  const float scale = block_scale<POW2>(amax);
  if (lane == 0) scales[POW2 ? b * rows + r : r * n_blocks + b] = scale;
  if (c0 < cols) codes[r * cols + c0] = uint8_t(e4m3_code(v0 / scale));
  if (c0 + 1 < cols) codes[r * cols + c0 + 1] = uint8_t(e4m3_code(v1 / scale));
}

template <typename T, bool POW2>
int quantize_typed(const void* x, uint8_t* codes, float* scales, int64_t rows, int64_t cols, hipStream_t s) {
  const int64_t n_blocks = (cols + kQBlock - 1) / kQBlock;
  const int64_t units = rows * n_blocks;
  const T* in = static_cast<const T*>(x);
  if (cols % 8 == 0 && aligned_to(x, sizeof(T) * 8) && aligned_to(codes, 8))
    quantize_vec_kernel<T, POW2><<<unsigned((units + 15) / 16), 256, 0, s>>>(in, codes, scales, rows, cols, n_blocks);
  else
    quantize_kernel<T, POW2><<<unsigned((units + 3) / 4), 256, 0, s>>>(in, codes, scales, rows, cols, n_blocks);
  return launch_status();
}

template <bool POW2>
int quantize_any(const void* x, int dtype, int64_t rows, int64_t cols, uint8_t* codes_out, float* scales_out,
                 hipStream_t s) {
  if (rows < 0 || cols < 0) return STM_ERR_ARG;
  if (dtype < STM_F32 || dtype > STM_BF16) return STM_ERR_UNSUPPORTED;
  if (rows == 0 || cols == 0) return STM_OK;
  if (!x || !codes_out || !scales_out) return STM_ERR_ARG;
  const int64_t units = rows * ((cols + kQBlock - 1) / kQBlock);
  if (units > 0x7fffffffll * 4) return STM_ERR_UNSUPPORTED;
  switch (dtype) {
    case STM_F32: return quantize_typed<float, POW2>(x, codes_out, scales_out, rows, cols, s);
    case STM_F16: return quantize_typed<f16_t, POW2>(x, codes_out, scales_out, rows, cols, s);
    default: return quantize_typed<bf16_t, POW2>(x, codes_out, scales_out, rows, cols, s);
  }
}

typedef float f32x16_t __attribute__((ext_vector_type(16)));

struct Fp8Args {
  const uint8_t* a;   // [M, K] codes
  const float* sa;    // [M, K/128]
  const uint8_t* b;   // [G, N, K] codes
  const float* sb;    // [G, N, K/128]
  void* c;            // [M, N]
  const int32_t* header;
  const MTile* tiles;
  int n, k;
};

constexpr int kFT = 128;          // tile edge
constexpr int kRowStride = 136;   // bytes per LDS row of 128 codes: 34 dwords, 8-byte reads of 32 rows conflict-free

// 128 x 128 tile, 4 waves (2 x 2) of 64 x 64; per 128-block of the contraction: both operand
// blocks through LDS, 32 MFMAs per wave into block accumulators, then acc += blk * sa * sb.
template <typename T>
__global__ __launch_bounds__(256) void fp8_gemm_kernel(Fp8Args p) {
  __shared__ __align__(16) unsigned char lds_a[kFT * kRowStride];
  __shared__ __align__(16) unsigned char lds_b[kFT * kRowStride];
  __shared__ __align__(16) float s_a[kFT];
  __shared__ __align__(16) float s_b[kFT];
  const int n_m_tiles = p.header[0];
  if (int(blockIdx.x) >= n_m_tiles) return;
  const MTile mt = p.tiles[blockIdx.x];
  const int j0 = blockIdx.y * kFT;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int wi = (wave / 2) * 64, wj = (wave % 2) * 64;
  const int nkb = p.k / kQBlock;
  const uint8_t* a = p.a + int64_t(mt.row0) * p.k;
  const uint8_t* b = p.b + (int64_t(mt.group) * p.n + j0) * p.k;
  const float* sa = p.sa + int64_t(mt.row0) * nkb;
  const float* sb = p.sb + (int64_t(mt.group) * p.n + j0) * nkb;
  const int valid_j = p.n - j0 < kFT ? p.n - j0 : kFT;

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  for (int kb = 0; kb < nkb; ++kb) {
    __syncthreads();  // the previous block's readers are done
    // 128 rows x 128 bytes per operand = 1024 16-byte pieces: 4 per thread
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int piece = it * 256 + threadIdx.x;
      const int row = piece / 8, c16 = piece % 8;
      uint4 va = make_uint4(0, 0, 0, 0), vb = make_uint4(0, 0, 0, 0);
      if (row < mt.rows) va = *reinterpret_cast<const uint4*>(a + int64_t(row) * p.k + kb * kQBlock + c16 * 16);
      if (row < valid_j) vb = *reinterpret_cast<const uint4*>(b + int64_t(row) * p.k + kb * kQBlock + c16 * 16);
      uint2* da = reinterpret_cast<uint2*>(lds_a + row * kRowStride + c16 * 16);
      uint2* db = reinterpret_cast<uint2*>(lds_b + row * kRowStride + c16 * 16);
      da[0] = make_uint2(va.x, va.y);
      da[1] = make_uint2(va.z, va.w);
      db[0] = make_uint2(vb.x, vb.y);
      db[1] = make_uint2(vb.z, vb.w);
    }
    if (threadIdx.x < kFT) {
      s_a[threadIdx.x] = int(threadIdx.x) < mt.rows ? sa[int64_t(threadIdx.x) * nkb + kb] : 0.f;
    } else {
      const int c = threadIdx.x - kFT;
      s_b[c] = c < valid_j ? sb[int64_t(c) * nkb + kb] : 0.f;
    }
    __syncthreads();
    f32x16_t blk[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) blk[i][j][r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < kQBlock / 16; ++kk) {
      long fa[2], fb[2];
      const int koff = kk * 16 + (lane / 32) * 8;
#pragma unroll
      for (int i = 0; i < 2; ++i)
        fa[i] = *reinterpret_cast<const long*>(lds_a + (wi + i * 32 + lane % 32) * kRowStride + koff);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        fb[j] = *reinterpret_cast<const long*>(lds_b + (wj + j * 32 + lane % 32) * kRowStride + koff);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)  // operands swapped: a lane owns 4 consecutive output columns per register group
          blk[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(fb[j], fa[i], blk[i][j], 0, 0, 0);
    }
    // lane: row lane%32 of a sub-tile; register r: column (r/4)*8 + (lane/32)*4 + r%4
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const float ra = s_a[wi + i * 32 + lane % 32];
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 cb = *reinterpret_cast<const float4*>(&s_b[wj + j * 32 + q * 8 + (lane / 32) * 4]);
          acc[i][j][q * 4 + 0] += blk[i][j][q * 4 + 0] * (ra * cb.x);
          acc[i][j][q * 4 + 1] += blk[i][j][q * 4 + 1] * (ra * cb.y);
          acc[i][j][q * 4 + 2] += blk[i][j][q * 4 + 2] * (ra * cb.z);
          acc[i][j][q * 4 + 3] += blk[i][j][q * 4 + 3] * (ra * cb.w);
        }
    }
  }
  T* c = static_cast<T*>(p.c) + int64_t(mt.row0) * p.n + j0;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = wi + i * 32 + lane % 32;
    if (row >= mt.rows) continue;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = wj + j * 32 + q * 8 + (lane / 32) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (col + e < valid_j) c[int64_t(row) * p.n + col + e] = from_float<T>(acc[i][j][q * 4 + e]);
      }
  }
}

}  // namespace
}  // namespace stm

extern "C" {

int stm_quantize_e4m3_1x128(const void* x, int dtype, int64_t rows, int64_t cols, uint8_t* codes_out, float* scales_out,
                            stm_stream_t stream) {
  return stm::quantize_any<false>(x, dtype, rows, cols, codes_out, scales_out, stm::as_stream(stream));
}

int stm_quantize_e4m3_1x128_pow2(const void* x, int dtype, int64_t rows, int64_t cols, uint8_t* codes_out,
                                 float* scales_by_block_out, stm_stream_t stream) {
  return stm::quantize_any<true>(x, dtype, rows, cols, codes_out, scales_by_block_out, stm::as_stream(stream));
}

int stm_grouped_gemm_fp8(const uint8_t* a_codes, const float* a_scales, const uint8_t* b_codes, const float* b_scales,
                         void* c, const int32_t* offsets, int n_groups, int64_t m_cap, int n, int k, int out_dtype,
                         void* workspace, size_t workspace_bytes, stm_stream_t stream) {
  using namespace stm;
  if (n_groups < 0 || m_cap < 0 || n < 0 || k < 0) return STM_ERR_ARG;
  if (out_dtype < STM_F32 || out_dtype > STM_BF16 || k % kQBlock != 0) return STM_ERR_UNSUPPORTED;
  if (m_cap == 0 || n == 0 || n_groups == 0) return STM_OK;
  if (!a_codes || !a_scales || !b_codes || !b_scales || !c || !offsets || !workspace) return STM_ERR_ARG;
  if (!aligned_to(a_codes, 16) || !aligned_to(b_codes, 16)) return STM_ERR_UNSUPPORTED;
  if (workspace_bytes < stm_gemm_workspace_bytes(m_cap, n_groups)) return STM_ERR_WORKSPACE;
  hipStream_t s = as_stream(stream);
  const int st = build_tile_table(offsets, n_groups, kFT, m_cap, workspace, s);
  if (st != STM_OK) return st;
  Fp8Args p{a_codes, a_scales, b_codes, b_scales, c, static_cast<const int32_t*>(workspace),
            reinterpret_cast<const MTile*>(static_cast<const char*>(workspace) + 16), n, k};
  dim3 grid(unsigned(max_m_tiles(m_cap, n_groups, kFT)), unsigned((n + kFT - 1) / kFT), 1);
  switch (out_dtype) {
    case STM_F32: fp8_gemm_kernel<float><<<grid, 256, 0, s>>>(p); break;
    case STM_F16: fp8_gemm_kernel<f16_t><<<grid, 256, 0, s>>>(p); break;
    default: fp8_gemm_kernel<bf16_t><<<grid, 256, 0, s>>>(p); break;
  }
  return launch_status();
}

int stm_grouped_gemm_fp8_pow2(const uint8_t* a_codes, const float* a_scales_by_block, const uint8_t* b_codes,
                              const float* b_scales_by_block, void* c, const int32_t* offsets, int n_groups,
                              int64_t m_cap, int n, int k, int out_dtype, void* workspace, size_t workspace_bytes,
                              stm_stream_t stream) {
  using namespace stm;
  if (n_groups < 0 || m_cap < 0 || n < 0 || k < 0) return STM_ERR_ARG;
  if (k % kQBlock != 0 || n_groups > 4096) return STM_ERR_UNSUPPORTED;
  if (m_cap == 0 || n == 0 || n_groups == 0 || k == 0) return STM_ERR_UNSUPPORTED;  // the plain entry handles it
  if (!a_codes || !a_scales_by_block || !b_codes || !b_scales_by_block || !c || !offsets || !workspace)
    return STM_ERR_ARG;
  if (!aligned_to(a_codes, 16) || !aligned_to(b_codes, 16) || !aligned_to(c, 16)) return STM_ERR_UNSUPPORTED;
  if (workspace_bytes < stm_gemm_workspace_bytes(m_cap, n_groups)) return STM_ERR_WORKSPACE;
  GemmArgs p{};
  p.a = a_codes;
  p.b = b_codes;
  p.c = c;
  p.offsets = offsets;
  p.header = static_cast<const int32_t*>(workspace);
  p.tiles = reinterpret_cast<const MTile*>(static_cast<const char*>(workspace) + 16);
  p.n_groups = n_groups;
  p.lda = k / 2;  // 16-bit units of two codes
  p.ldb = k / 2;
  p.ldc = n;
  p.b_group = int64_t(n) * (k / 2);
  p.n_j = n;
  p.n_k = k / 2;
  p.a_scales = a_scales_by_block;
  p.b_scales = b_scales_by_block;
  p.a_scale_rows = m_cap;
  p.b_scale_rows = int64_t(n_groups) * n;
  return launch_dma_fp8(out_dtype, p, offsets, n_groups, m_cap, workspace, as_stream(stream));
}

}  // extern "C"
