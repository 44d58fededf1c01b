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
#include <atomic>

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

  constexpr int kAhead = 8;  // segment counters fetched together: the loops below are latency-bound
  for (int e = el; e < n_experts; e += lanes_e) {
    int32_t sum = 0;
    for (int64_t s0 = s_begin; s0 < s_end; s0 += kAhead) {
      int32_t c[kAhead];
#pragma unroll
      for (int j = 0; j < kAhead; ++j) c[j] = s0 + j < s_end ? counts[(s0 + j) * n_experts + e] : 0;
#pragma unroll
      for (int j = 0; j < kAhead; ++j) sum += c[j];
    }
    partial[g * n_experts + e] = sum;
  }
  __syncthreads();
  // per expert: totals over the slices, slices -> exclusive prefixes
  int32_t sum_actual = 0, max_actual = 0;
  for (int e = tid; e < n_experts; e += kScanThreads) {
    int32_t run = 0;
    for (int gg = 0; gg < groups; ++gg) {
      const int32_t c = partial[gg * n_experts + e];
      partial[gg * n_experts + e] = run;
      run += c;
    }
    if (hist_out) hist_out[e] = run;
    sum_actual += run;
    max_actual = run > max_actual ? run : max_actual;
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
  __shared__ int32_t per_thread_max[kScanThreads];
  per_thread[tid] = sum_actual;
  per_thread_max[tid] = max_actual;
  __syncthreads();
  int32_t n_valid = 0, largest = 0;
  if (tid < kWave) {
    int32_t acc = 0, most = 0;
    for (int i = tid; i < kScanThreads; i += kWave) {
      acc += per_thread[i];
      most = per_thread_max[i] > most ? per_thread_max[i] : most;
    }
    n_valid = wave_sum(acc);
    largest = wave_max(most);
  }
  const int32_t given_total = block_exclusive_scan(base, n_experts, wave_sums);
  if (tid == 0) {
    status[STM_ST_N_VALID] = n_valid;
    status[STM_ST_MAX_COUNT] = largest;
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
    for (int64_t s0 = s_begin; s0 < s_end; s0 += kAhead) {
      int32_t c[kAhead];
#pragma unroll
      for (int j = 0; j < kAhead; ++j) c[j] = s0 + j < s_end ? counts[(s0 + j) * n_experts + e] : 0;
#pragma unroll
      for (int j = 0; j < kAhead; ++j) {
        if (s0 + j < s_end) counts[(s0 + j) * n_experts + e] = run;
        run += c[j];
      }
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

// ---------------------------------------------------------------- slots sorted by row
// Helpers of the two-pass (12 bits each) least-significant-digit radix sort below.
__global__ void copy_i32_kernel(int32_t* dst, const int32_t* src, int64_t n) {
  const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

template <bool I64>
__global__ void row_digit_kernel(const void* __restrict__ keys, int64_t n, int64_t n_rows, int shift,
                                 int32_t* __restrict__ digit) {
  const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int64_t k = I64 ? static_cast<const int64_t*>(keys)[i] : int64_t(static_cast<const int32_t*>(keys)[i]);
  digit[i] = (k < 0 || k >= n_rows) ? -1 : int32_t((k >> shift) & (kMaxExperts - 1));
}

template <bool I64>
__global__ void scatter_pairs_kernel(const int32_t* __restrict__ dest, const void* __restrict__ keys,
                                     const int32_t* __restrict__ vals_or_null, int64_t n,
                                     int32_t* __restrict__ keys_out, int32_t* __restrict__ vals_out) {
  const int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int32_t d = dest[i];
  if (d < 0) return;
  keys_out[d] = I64 ? int32_t(static_cast<const int64_t*>(keys)[i]) : static_cast<const int32_t*>(keys)[i];
  vals_out[d] = vals_or_null ? vals_or_null[i] : int32_t(i);
}

}  // namespace

namespace {
inline size_t slots_bytes(int64_t n_slots) { return round_up(size_t(n_slots) * sizeof(int32_t), 256); }
inline int digits_of(int64_t n_rows) { return int(n_rows < kMaxExperts ? n_rows : kMaxExperts); }
}  // namespace

size_t sort_by_row_workspace_bytes(int64_t n_slots, int64_t n_rows) {
  // digit, dest, keys1, vals1, then the counter rows of the counting sort, then status words
  return 4 * slots_bytes(n_slots) + stm_route_workspace_bytes(n_slots, digits_of(n_rows)) + 256;
}

// The valid slots of a position map (0 <= pos < n_rows), stably sorted by the row they name:
// sorted_row[j] ascending (padded with INT32_MAX up to n_slots), sorted_slot[j] the flat slot;
// n_valid_out (optional, device) receives the number of valid slots.
// Every pass is the stable counting sort of the routing kernels on one 12-bit digit.
int sort_slots_by_row(const void* pos, int pos_is_i64, int64_t n_slots, int64_t n_rows, int32_t* sorted_row,
                      int32_t* sorted_slot, int32_t* n_valid_out, void* workspace, size_t workspace_bytes,
                      hipStream_t stream) {
  if (n_slots < 0 || n_rows < 0) return STM_ERR_ARG;
  if (n_rows > (int64_t(1) << 24) || n_slots > (int64_t(1) << 31) - 1) return STM_ERR_UNSUPPORTED;
  if (n_slots == 0 || n_rows == 0) {
    if (n_valid_out) fill_i32_kernel<<<1, 64, 0, stream>>>(n_valid_out, 1, 0);
    if (n_slots && sorted_row)
      fill_i32_kernel<<<unsigned((n_slots + 255) / 256), 256, 0, stream>>>(sorted_row, n_slots, 0x7fffffff);
    return launch_status();
  }
  if (!pos || !sorted_row || !sorted_slot || !workspace) return STM_ERR_ARG;
  if (workspace_bytes < sort_by_row_workspace_bytes(n_slots, n_rows)) return STM_ERR_WORKSPACE;
  unsigned char* w = static_cast<unsigned char*>(workspace);
  int32_t* digit = reinterpret_cast<int32_t*>(w);
  int32_t* dest = reinterpret_cast<int32_t*>(w + slots_bytes(n_slots));
  int32_t* keys1 = reinterpret_cast<int32_t*>(w + 2 * slots_bytes(n_slots));
  int32_t* vals1 = reinterpret_cast<int32_t*>(w + 3 * slots_bytes(n_slots));
  void* counters = w + 4 * slots_bytes(n_slots);
  const size_t counters_bytes = stm_route_workspace_bytes(n_slots, digits_of(n_rows));
  int32_t* status = reinterpret_cast<int32_t*>(w + 4 * slots_bytes(n_slots) + counters_bytes);
  const unsigned grid = unsigned((n_slots + 255) / 256);
  const bool two_passes = n_rows > kMaxExperts;
  fill_i32_kernel<<<1, 64, 0, stream>>>(status, STM_STATUS_WORDS, 0);
  fill_i32_kernel<<<grid, 256, 0, stream>>>(sorted_row, n_slots, 0x7fffffff);
  int32_t* keys_a = two_passes ? keys1 : sorted_row;
  int32_t* vals_a = two_passes ? vals1 : sorted_slot;
  if (two_passes) fill_i32_kernel<<<grid, 256, 0, stream>>>(keys1, n_slots, -1);
  // pass on the low digit
  if (pos_is_i64)
    row_digit_kernel<true><<<grid, 256, 0, stream>>>(pos, n_slots, n_rows, 0, digit);
  else
    row_digit_kernel<false><<<grid, 256, 0, stream>>>(pos, n_slots, n_rows, 0, digit);
  int st = run_sort(digit, 0, n_slots, digits_of(n_rows), nullptr, 0, nullptr, nullptr, dest, status, counters,
                    counters_bytes, stream);
  if (st != STM_OK) return st;
  if (n_valid_out) copy_i32_kernel<<<1, 64, 0, stream>>>(n_valid_out, status + STM_ST_N_VALID, 1);
  if (pos_is_i64)
    scatter_pairs_kernel<true><<<grid, 256, 0, stream>>>(dest, pos, nullptr, n_slots, keys_a, vals_a);
  else
    scatter_pairs_kernel<false><<<grid, 256, 0, stream>>>(dest, pos, nullptr, n_slots, keys_a, vals_a);
  if (two_passes) {  // pass on the high digit (the tail of keys1 is -1: dropped)
    const int high_digits = int(((n_rows - 1) >> 12) + 1);
    row_digit_kernel<false><<<grid, 256, 0, stream>>>(keys1, n_slots, n_rows, 12, digit);
    st = run_sort(digit, 0, n_slots, high_digits, nullptr, 0, nullptr, nullptr, dest, status, counters, counters_bytes,
                  stream);
    if (st != STM_OK) return st;
    scatter_pairs_kernel<false><<<grid, 256, 0, stream>>>(dest, keys1, vals1, n_slots, sorted_row, sorted_slot);
  }
  return launch_status();
}

}  // namespace stm

namespace stm {
namespace {

// Counter rows of stm_route_plan_static: device memory owned by the library, one copy per GPU,
// held until the process ends.  Host code never uses the array's name as an address: the
// device address is looked up once per device and kept.
constexpr size_t kStaticScratchBytes = size_t(2) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::atomic<void*> scratch_address[kMaxDevices];

// Device address of `scratch` on the current device (nullptr on failure).
void* static_scratch() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void* p = scratch_address[dev].load(std::memory_order_acquire);
  if (p) return p;
  void* looked_up = nullptr;
  if (hipGetSymbolAddress(&looked_up, HIP_SYMBOL(scratch)) != hipSuccess || !looked_up) {
    (void)hipGetLastError();
    return nullptr;
  }
  scratch_address[dev].store(looked_up, std::memory_order_release);
  return looked_up;
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

size_t stm_route_plan_static_capacity_bytes(void) { return stm::kStaticScratchBytes; }

int stm_route_plan_static(const void* ids, int ids_are_i64, int64_t n_slots, int n_experts, int32_t* hist_out,
                          int32_t* offsets_out, int32_t* pos_out, int32_t* status, stm_stream_t stream) {
  if (!offsets_out || (n_slots > 0 && !pos_out)) return STM_ERR_ARG;
  if (n_slots < 0 || n_experts < 0) return STM_ERR_ARG;
  const size_t need = stm_route_workspace_bytes(n_slots, n_experts);
  if (need > stm::kStaticScratchBytes) return STM_ERR_CAPACITY;
  void* ws = stm::static_scratch();
  if (!ws) return STM_ERR_LAUNCH;
  // every counter cell the scan reads is first written by the count kernel of the same call, so
  // what an earlier (larger) call left in the array is never seen
  return stm::run_sort(ids, ids_are_i64, n_slots, n_experts, nullptr, 0, hist_out, offsets_out, pos_out, status, ws,
                       stm::kStaticScratchBytes, stm::as_stream(stream));
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
