// Per-expert histogram and stable counting-sort positions for MoE routing (gfx950).
//
// The flat slot array (token-major, k-minor) is cut into segments of kSegment slots;
// one wavefront owns one segment.  Inside a wavefront the rank of a slot among earlier
// slots with the same expert comes from a bitwise ballot match (no atomics): after
// intersecting the ballots of every id bit, each lane holds the mask of lanes with its
// id; popcount(mask & lanes_below) is its rank in this step, popcount(mask) is what the
// first lane of the mask adds to the wave's private LDS counter row.
//
//   count kernel : counts[segment][expert]
//   scan kernel  : histogram, expert base offsets, counts[][] -> first position of every
//                  (segment, expert) pair                      (one workgroup)
//   index kernel : replays the ranking, starting every counter from the scanned table
//
// Everything is integer arithmetic, so results are bit-reproducible.
#include "common.hpp"

namespace stm {
namespace {

constexpr int kSegment = 256;       // slots ranked by one wavefront
constexpr int kWavesPerBlock = 4;   // 256 threads
constexpr int kMaxExperts = 4096;   // LDS: kWavesPerBlock * E * 4 bytes <= 64 KiB
constexpr int kScanThreads = 1024;

template <bool I64>
__device__ __forceinline__ int load_id(const void* ids, int64_t i) {
  if constexpr (I64) {
    const int64_t v = static_cast<const int64_t*>(ids)[i];
    return v < 0 ? (v < INT32_MIN ? INT32_MIN : int(v)) : (v > INT32_MAX ? INT32_MAX : int(v));
  } else {
    return static_cast<const int32_t*>(ids)[i];
  }
}

// Mask of the lanes whose (valid) key equals this lane's key.
__device__ __forceinline__ uint64_t match_lanes(int key, bool valid, int key_bits) {
  uint64_t m = __ballot(valid);
  for (int b = 0; b < key_bits; ++b) {
    const bool bit = (key >> b) & 1;
    const uint64_t set = __ballot(bit);
    m &= bit ? set : ~set;
  }
  return valid ? m : 0ull;
}

__device__ __forceinline__ int bits_for(int n_experts) {
  int b = 0;
  while ((1 << b) < n_experts) ++b;
  return b;
}

template <bool I64>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void count_kernel(const void* __restrict__ ids, int64_t n_slots,
                                                                      int n_experts, int32_t* __restrict__ counts,
                                                                      int32_t* __restrict__ status) {
  extern __shared__ int32_t lds[];
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int64_t seg = int64_t(blockIdx.x) * kWavesPerBlock + wave;
  const int64_t first = seg * kSegment;
  if (first >= n_slots) return;
  int32_t* row = lds + wave * n_experts;
  for (int e = lane; e < n_experts; e += kWave) row[e] = 0;
  const int key_bits = bits_for(n_experts);
  const uint64_t below = lanemask_lt();
#pragma unroll
  for (int it = 0; it < kSegment / kWave; ++it) {
    const int64_t i = first + it * kWave + lane;
    const int id = i < n_slots ? load_id<I64>(ids, i) : -1;
    if (id >= n_experts) status[STM_ST_ID_OUT_OF_RANGE] = 1;
    const bool valid = id >= 0 && id < n_experts;
    const uint64_t same = match_lanes(id, valid, key_bits);
    if (valid && (same & below) == 0) row[id] += __popcll(same);
  }
  int32_t* out = counts + seg * n_experts;
  for (int e = lane; e < n_experts; e += kWave) out[e] = row[e];
}

template <bool I64>
__global__ __launch_bounds__(kWavesPerBlock* kWave) void index_kernel(const void* __restrict__ ids, int64_t n_slots,
                                                                      int n_experts,
                                                                      const int32_t* __restrict__ first_pos,
                                                                      int32_t* __restrict__ pos) {
  extern __shared__ int32_t lds[];
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x % kWave;
  const int64_t seg = int64_t(blockIdx.x) * kWavesPerBlock + wave;
  const int64_t first = seg * kSegment;
  if (first >= n_slots) return;
  int32_t* row = lds + wave * n_experts;
  const int32_t* start = first_pos + seg * n_experts;
  for (int e = lane; e < n_experts; e += kWave) row[e] = start[e];
  const int key_bits = bits_for(n_experts);
  const uint64_t below = lanemask_lt();
#pragma unroll
  for (int it = 0; it < kSegment / kWave; ++it) {
    const int64_t i = first + it * kWave + lane;
    const int id = i < n_slots ? load_id<I64>(ids, i) : -1;
    const bool valid = id >= 0 && id < n_experts;
    const uint64_t same = match_lanes(id, valid, key_bits);
    int p = id < 0 ? id : -1;  // unused slots keep their marker; out-of-range ids become unused
    if (valid) {
      const int running = row[id];
      p = running + __popcll(same & below);
      if ((same & below) == 0) row[id] = running + __popcll(same);
    }
    if (i < n_slots) pos[i] = p;
  }
}

// One workgroup.  counts[S][E] (per-segment counts) -> per-(segment, expert) first
// positions, plus histogram / offsets.  `given` (optional) supplies the histogram the
// base offsets are taken from.
template <bool GIVEN_I64>
__global__ __launch_bounds__(kScanThreads) void scan_kernel(int32_t* __restrict__ counts, int64_t n_segments,
                                                            int n_experts, const void* __restrict__ given,
                                                            int32_t* __restrict__ hist_out,
                                                            int32_t* __restrict__ offsets_out, bool write_table,
                                                            int32_t* __restrict__ status) {
  __shared__ int32_t partial[kMaxExperts];  // [G][E] with G*E <= max(E, 1024)
  __shared__ int32_t base[kMaxExperts];
  __shared__ int32_t wave_sums[kScanThreads / kWave];
  __shared__ int32_t flags[2];
  const int tid = threadIdx.x;
  int lanes_e = 1;
  while (lanes_e < n_experts && lanes_e < kScanThreads) lanes_e <<= 1;
  const int groups = kScanThreads / lanes_e;  // slices of the segment axis
  const int g = tid / lanes_e;
  const int el = tid % lanes_e;
  const int64_t chunk = (n_segments + groups - 1) / groups;
  const int64_t s_begin = g * chunk;
  const int64_t s_end = s_begin + chunk < n_segments ? s_begin + chunk : n_segments;
  if (tid < 2) flags[tid] = 0;

  for (int e = el; e < n_experts; e += lanes_e) {
    int32_t sum = 0;
    for (int64_t s = s_begin; s < s_end; ++s) sum += counts[s * n_experts + e];
    partial[g * n_experts + e] = sum;
  }
  __syncthreads();
  // per expert: totals over the slices, slices -> exclusive prefixes
  int32_t sum_actual = 0;
  for (int e = tid; e < n_experts; e += kScanThreads) {
    int32_t run = 0;
    for (int gg = 0; gg < groups; ++gg) {
      const int32_t c = partial[gg * n_experts + e];
      partial[gg * n_experts + e] = run;
      run += c;
    }
    if (hist_out) hist_out[e] = run;
    sum_actual += run;
    int32_t b = run;
    if (given) {
      if constexpr (GIVEN_I64) {
        const int64_t v = static_cast<const int64_t*>(given)[e];
        if (v < 0) flags[0] = 1;
        b = int32_t(v);
      } else {
        b = static_cast<const int32_t*>(given)[e];
        if (b < 0) flags[0] = 1;
      }
    }
    base[e] = b;
  }
  __syncthreads();
  // number of valid slots (sum of the actual counts) via a throw-away scan
  __shared__ int32_t per_thread[kScanThreads];
  per_thread[tid] = sum_actual;
  __syncthreads();
  int32_t n_valid = 0;
  if (tid < kWave) {
    int32_t acc = 0;
    for (int i = tid; i < kScanThreads; i += kWave) acc += per_thread[i];
    n_valid = wave_sum(acc);
  }
  const int32_t given_total = block_exclusive_scan(base, n_experts, wave_sums);
  if (tid == 0) {
    status[STM_ST_N_VALID] = n_valid;
    if (given && given_total != n_valid) status[STM_ST_HIST_MISMATCH] = 1;
    if (flags[0]) status[STM_ST_HIST_NEGATIVE] = 1;
  }
  if (offsets_out) {
    for (int e = tid; e < n_experts; e += kScanThreads) offsets_out[e] = base[e];
    if (tid == 0) offsets_out[n_experts] = given_total;
  }
  if (!write_table) return;
  for (int e = el; e < n_experts; e += lanes_e) {
    int32_t run = base[e] + partial[g * n_experts + e];
    for (int64_t s = s_begin; s < s_end; ++s) {
      const int32_t c = counts[s * n_experts + e];
      counts[s * n_experts + e] = run;
      run += c;
    }
  }
}

template <bool I64>
__global__ __launch_bounds__(kScanThreads) void group_offsets_kernel(const void* __restrict__ sizes, int n_groups,
                                                                     int32_t* __restrict__ offsets) {
  __shared__ int32_t a[kMaxExperts];
  __shared__ int32_t wave_sums[kScanThreads / kWave];
  for (int i = threadIdx.x; i < n_groups; i += kScanThreads) {
    int64_t v = I64 ? static_cast<const int64_t*>(sizes)[i] : int64_t(static_cast<const int32_t*>(sizes)[i]);
    a[i] = v < 0 ? 0 : int32_t(v);
  }
  __syncthreads();
  const int32_t total = block_exclusive_scan(a, n_groups, wave_sums);
  for (int i = threadIdx.x; i < n_groups; i += kScanThreads) offsets[i] = a[i];
  if (threadIdx.x == 0) offsets[n_groups] = total;
}

__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
  const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

inline int64_t n_segments_of(int64_t n_slots) { return (n_slots + kSegment - 1) / kSegment; }

int run_sort(const void* ids, int ids_are_i64, int64_t n_slots, int n_experts, const void* hist_in, int hist_is_i64,
             int32_t* hist_out, int32_t* offsets_out, int32_t* pos_out, int32_t* status, void* workspace,
             size_t workspace_bytes, hipStream_t stream) {
  if (n_slots < 0 || n_experts < 0 || !status) return STM_ERR_ARG;
  if (n_slots > 0 && !ids) return STM_ERR_ARG;
  if (n_experts > kMaxExperts || n_slots > (int64_t(1) << 31) - 1) return STM_ERR_UNSUPPORTED;
  if (workspace_bytes < stm_route_workspace_bytes(n_slots, n_experts)) return STM_ERR_WORKSPACE;
  if (n_experts == 0) {
    // nothing to count; positions of an expert-less routing are all "unused"
    if (offsets_out) fill_i32_kernel<<<1, 64, 0, stream>>>(offsets_out, 1, 0);
    if (pos_out && n_slots)
      fill_i32_kernel<<<unsigned((n_slots + 255) / 256), 256, 0, stream>>>(pos_out, n_slots, -1);
    return launch_status();
  }
  int32_t* counts = static_cast<int32_t*>(workspace);
  const int64_t segs = n_segments_of(n_slots);
  const unsigned blocks = unsigned((segs + kWavesPerBlock - 1) / kWavesPerBlock);
  const size_t lds = size_t(kWavesPerBlock) * n_experts * sizeof(int32_t);
  if (blocks) {
    if (ids_are_i64)
      count_kernel<true><<<blocks, kWavesPerBlock * kWave, lds, stream>>>(ids, n_slots, n_experts, counts, status);
    else
      count_kernel<false><<<blocks, kWavesPerBlock * kWave, lds, stream>>>(ids, n_slots, n_experts, counts, status);
  }
  const bool table = pos_out != nullptr;
  if (hist_is_i64)
    scan_kernel<true><<<1, kScanThreads, 0, stream>>>(counts, segs, n_experts, hist_in, hist_out, offsets_out, table,
                                                      status);
  else
    scan_kernel<false><<<1, kScanThreads, 0, stream>>>(counts, segs, n_experts, hist_in, hist_out, offsets_out, table,
                                                       status);
  if (pos_out && blocks) {
    if (ids_are_i64)
      index_kernel<true><<<blocks, kWavesPerBlock * kWave, lds, stream>>>(ids, n_slots, n_experts, counts, pos_out);
    else
      index_kernel<false><<<blocks, kWavesPerBlock * kWave, lds, stream>>>(ids, n_slots, n_experts, counts, pos_out);
  }
  return launch_status();
}

}  // namespace
}  // namespace stm

extern "C" {

size_t stm_route_workspace_bytes(int64_t n_slots, int n_experts) {
  if (n_slots < 0 || n_experts < 0) return 0;
  const size_t cells = size_t(stm::n_segments_of(n_slots)) * size_t(n_experts);
  return stm::round_up(cells * sizeof(int32_t) + 256, 256);
}

int stm_histogram(const void* ids, int ids_are_i64, int64_t n_slots, int n_experts, int32_t* hist_out, int32_t* status,
                  void* workspace, size_t workspace_bytes, stm_stream_t stream) {
  if (n_experts > 0 && !hist_out) return STM_ERR_ARG;
  return stm::run_sort(ids, ids_are_i64, n_slots, n_experts, nullptr, 0, hist_out, nullptr, nullptr, status, workspace,
                       workspace_bytes, stm::as_stream(stream));
}

int stm_index_compute(const void* ids, int ids_are_i64, int64_t n_slots, int n_experts, const void* hist_in,
                      int hist_is_i64, int32_t* pos_out, int32_t* status, void* workspace, size_t workspace_bytes,
                      stm_stream_t stream) {
  if (n_slots > 0 && !pos_out) return STM_ERR_ARG;
  if (n_experts > 0 && !hist_in) return STM_ERR_ARG;
  if (n_slots == 0) return STM_OK;
  return stm::run_sort(ids, ids_are_i64, n_slots, n_experts, hist_in, hist_is_i64, nullptr, nullptr, pos_out, status,
                       workspace, workspace_bytes, stm::as_stream(stream));
}

int stm_route_plan(const void* ids, int ids_are_i64, int64_t n_slots, int n_experts, int32_t* hist_out,
                   int32_t* offsets_out, int32_t* pos_out, int32_t* status, void* workspace, size_t workspace_bytes,
                   stm_stream_t stream) {
  if (!offsets_out || (n_slots > 0 && !pos_out)) return STM_ERR_ARG;
  return stm::run_sort(ids, ids_are_i64, n_slots, n_experts, nullptr, 0, hist_out, offsets_out, pos_out, status,
                       workspace, workspace_bytes, stm::as_stream(stream));
}

int stm_group_offsets(const void* sizes, int sizes_are_i64, int n_groups, int32_t* offsets_out, stm_stream_t stream) {
  if (n_groups < 0 || !offsets_out || (n_groups > 0 && !sizes)) return STM_ERR_ARG;
  if (n_groups > stm::kMaxExperts) return STM_ERR_UNSUPPORTED;
  hipStream_t s = stm::as_stream(stream);
  if (sizes_are_i64)
    stm::group_offsets_kernel<true><<<1, stm::kScanThreads, 0, s>>>(sizes, n_groups, offsets_out);
  else
    stm::group_offsets_kernel<false><<<1, stm::kScanThreads, 0, s>>>(sizes, n_groups, offsets_out);
  return stm::launch_status();
}

}  // extern "C"
