// A host that is not Python and knows nothing of torch: it owns its device memory through the HIP
// runtime, calls the C ABI of libsteptron_moe_gfx950.so through include/steptron_moe.h only, and
// checks what comes back against loops on the host.  Built as a small shared library (one
// function) so that a test can call it in-process.
//
//   route plan  -> histogram, offsets and positions of a stable counting sort (integers, exact)
//   permute     -> rows copied to their positions (exact)
//   grouped GEMM-> fp32, every group against a triple loop (1e-5 relative)
//   gathered weight gradient (bf16) -> the product read through the row -> token table against
//                  the same product on copied rows (bit for bit) and a host loop (1e-2 relative)
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <vector>

#include "../../include/steptron_moe.h"

namespace {

#define CHECK_HIP(call)                                                              \
  do {                                                                               \
    hipError_t e_ = (call);                                                          \
    if (e_ != hipSuccess) {                                                          \
      snprintf(msg, cap, "%s failed: %s", #call, hipGetErrorString(e_));             \
      return 1;                                                                      \
    }                                                                                \
  } while (0)
#define CHECK_STM(call)                                                              \
  do {                                                                               \
    int s_ = (call);                                                                 \
    if (s_ != STM_OK) {                                                              \
      snprintf(msg, cap, "%s returned %d (%s)", #call, s_, stm_status_string(s_));   \
      return 2;                                                                      \
    }                                                                                \
  } while (0)

uint16_t to_bf16(float f) {  // round to nearest even
  uint32_t u;
  memcpy(&u, &f, 4);
  return uint16_t((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
float from_bf16(uint16_t h) {
  const uint32_t u = uint32_t(h) << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

template <typename T>
struct DeviceBuffer {
  T* p = nullptr;
  ~DeviceBuffer() {
    if (p) (void)hipFree(p);
  }
  hipError_t alloc(size_t n) { return hipMalloc(reinterpret_cast<void**>(&p), (n ? n : 1) * sizeof(T)); }
};

}  // namespace

extern "C" int stm_host_check(char* msg, int cap) {
  const int T = 300, K = 3, E = 7, H = 40, N_OUT = 24;
  const int64_t n_slots = int64_t(T) * K;
  // ids: a fixed pseudo-random pattern with some unused (-1) slots
  std::vector<int32_t> ids(n_slots);
  uint32_t state = 12345u;
  for (auto& v : ids) {
    state = state * 1664525u + 1013904223u;
    const uint32_t r = state >> 8;
    v = (r % 10u == 0u) ? -1 : int32_t(r % uint32_t(E));
  }
  // host truth: histogram, offsets, stable positions
  std::vector<int32_t> hist(E, 0), offsets(E + 1, 0), pos(n_slots, -1), next(E, 0);
  for (int32_t e : ids)
    if (e >= 0) ++hist[e];
  for (int e = 0; e < E; ++e) offsets[e + 1] = offsets[e] + hist[e];
  for (int e = 0; e < E; ++e) next[e] = offsets[e];
  for (int64_t s = 0; s < n_slots; ++s) pos[s] = ids[s] >= 0 ? next[ids[s]]++ : ids[s];
  const int n_rows = offsets[E];

  DeviceBuffer<int32_t> d_ids, d_hist, d_offsets, d_pos, d_status;
  DeviceBuffer<unsigned char> d_ws;
  CHECK_HIP(d_ids.alloc(n_slots));
  CHECK_HIP(d_hist.alloc(E));
  CHECK_HIP(d_offsets.alloc(E + 1));
  CHECK_HIP(d_pos.alloc(n_slots));
  CHECK_HIP(d_status.alloc(STM_STATUS_WORDS));
  const size_t ws_bytes = stm_route_workspace_bytes(n_slots, E);
  CHECK_HIP(d_ws.alloc(ws_bytes));
  CHECK_HIP(hipMemcpy(d_ids.p, ids.data(), n_slots * sizeof(int32_t), hipMemcpyHostToDevice));
  CHECK_HIP(hipMemset(d_status.p, 0, STM_STATUS_WORDS * sizeof(int32_t)));
  CHECK_STM(stm_route_plan(d_ids.p, 0, n_slots, E, d_hist.p, d_offsets.p, d_pos.p, d_status.p, d_ws.p, ws_bytes, nullptr));
  CHECK_HIP(hipDeviceSynchronize());
  std::vector<int32_t> got_hist(E), got_offsets(E + 1), got_pos(n_slots);
  CHECK_HIP(hipMemcpy(got_hist.data(), d_hist.p, E * sizeof(int32_t), hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(got_offsets.data(), d_offsets.p, (E + 1) * sizeof(int32_t), hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(got_pos.data(), d_pos.p, n_slots * sizeof(int32_t), hipMemcpyDeviceToHost));
  if (got_hist != hist || got_offsets != offsets || got_pos != pos) {
    snprintf(msg, cap, "route plan differs from the host's stable counting sort");
    return 3;
  }

  // permute: fp32 rows to their positions
  std::vector<float> x(size_t(T) * H);
  for (size_t i = 0; i < x.size(); ++i) x[i] = float(int(i % 97) - 48) * 0.125f;
  DeviceBuffer<float> d_x, d_rows;
  CHECK_HIP(d_x.alloc(x.size()));
  CHECK_HIP(d_rows.alloc(size_t(n_rows) * H));
  CHECK_HIP(hipMemcpy(d_x.p, x.data(), x.size() * sizeof(float), hipMemcpyHostToDevice));
  CHECK_STM(stm_permute_fwd(d_x.p, d_pos.p, 0, d_rows.p, T, K, int64_t(H) * sizeof(float), n_rows, nullptr, nullptr));
  CHECK_HIP(hipDeviceSynchronize());
  std::vector<float> rows(size_t(n_rows) * H);
  CHECK_HIP(hipMemcpy(rows.data(), d_rows.p, rows.size() * sizeof(float), hipMemcpyDeviceToHost));
  for (int64_t s = 0; s < n_slots; ++s) {
    if (pos[s] < 0) continue;
    for (int h = 0; h < H; ++h)
      if (rows[size_t(pos[s]) * H + h] != x[size_t(s / K) * H + h]) {
        snprintf(msg, cap, "permuted row %d differs from token %d", pos[s], int(s / K));
        return 4;
      }
  }

  // grouped GEMM, fp32, weights [E, N_OUT, H] (trans_b form)
  std::vector<float> w(size_t(E) * N_OUT * H);
  for (size_t i = 0; i < w.size(); ++i) w[i] = float(int(i % 53) - 26) * 0.0625f;
  DeviceBuffer<float> d_w, d_c;
  DeviceBuffer<unsigned char> d_gws;
  const size_t gws_bytes = stm_gemm_workspace_bytes(n_rows, E);
  CHECK_HIP(d_w.alloc(w.size()));
  CHECK_HIP(d_c.alloc(size_t(n_rows) * N_OUT));
  CHECK_HIP(d_gws.alloc(gws_bytes));
  CHECK_HIP(hipMemcpy(d_w.p, w.data(), w.size() * sizeof(float), hipMemcpyHostToDevice));
  CHECK_STM(stm_grouped_gemm(d_rows.p, d_w.p, d_c.p, d_offsets.p, E, n_rows, N_OUT, H, 1, STM_F32, d_gws.p, gws_bytes,
                             nullptr));
  CHECK_HIP(hipDeviceSynchronize());
  std::vector<float> c(size_t(n_rows) * N_OUT);
  CHECK_HIP(hipMemcpy(c.data(), d_c.p, c.size() * sizeof(float), hipMemcpyDeviceToHost));
  for (int e = 0; e < E; ++e)
    for (int r = offsets[e]; r < offsets[e + 1]; ++r)
      for (int n = 0; n < N_OUT; ++n) {
        double ref = 0.0;
        for (int h = 0; h < H; ++h) ref += double(rows[size_t(r) * H + h]) * double(w[(size_t(e) * N_OUT + n) * H + h]);
        if (fabs(double(c[size_t(r) * N_OUT + n]) - ref) > 1e-5 * (fabs(ref) + 1.0)) {
          snprintf(msg, cap, "grouped GEMM: row %d col %d is %g, expected %g", r, n, double(c[size_t(r) * N_OUT + n]), ref);
          return 5;
        }
      }
  // weight gradient with a gathered operand, bf16: out[g] = d[rows of g]^T @ tokens[token_of_row[rows of g]]
  {
    const int T2 = 512, K2 = 2, E2 = 4, P = 256, Q = 256;
    const int64_t slots2 = int64_t(T2) * K2;
    std::vector<int32_t> ids2(slots2);
    for (auto& v : ids2) {
      state = state * 1664525u + 1013904223u;
      v = int32_t((state >> 9) % uint32_t(E2));
    }
    std::vector<int32_t> off2(E2 + 1, 0), pos2(slots2), nxt(E2, 0);
    for (int32_t e : ids2) ++off2[e + 1];
    for (int e = 0; e < E2; ++e) off2[e + 1] += off2[e];
    for (int e = 0; e < E2; ++e) nxt[e] = off2[e];
    for (int64_t i = 0; i < slots2; ++i) pos2[i] = nxt[ids2[i]]++;
    std::vector<uint16_t> tok(size_t(T2) * Q), d(size_t(slots2) * P);
    for (size_t i = 0; i < tok.size(); ++i) tok[i] = to_bf16(float(int((i * 7u) % 31u) - 15) * 0.0625f);
    for (size_t i = 0; i < d.size(); ++i) d[i] = to_bf16(float(int((i * 5u) % 23u) - 11) * 0.125f);
    DeviceBuffer<int32_t> d_ids2, d_hist2, d_off2, d_pos2, d_st2, d_table;
    DeviceBuffer<unsigned char> d_ws2;
    DeviceBuffer<uint16_t> d_tok, d_d, d_copy, d_out_g, d_out_c;
    const size_t ws2 = stm_route_workspace_bytes(slots2, E2);
    CHECK_HIP(d_ids2.alloc(slots2));
    CHECK_HIP(d_hist2.alloc(E2));
    CHECK_HIP(d_off2.alloc(E2 + 1));
    CHECK_HIP(d_pos2.alloc(slots2));
    CHECK_HIP(d_st2.alloc(STM_STATUS_WORDS));
    CHECK_HIP(d_ws2.alloc(ws2));
    CHECK_HIP(d_table.alloc(size_t(slots2) + size_t(stm_row_sources_padding())));
    CHECK_HIP(d_tok.alloc(tok.size()));
    CHECK_HIP(d_d.alloc(d.size()));
    CHECK_HIP(d_copy.alloc(size_t(slots2) * Q));
    CHECK_HIP(d_out_g.alloc(size_t(E2) * P * Q));
    CHECK_HIP(d_out_c.alloc(size_t(E2) * P * Q));
    CHECK_HIP(hipMemcpy(d_ids2.p, ids2.data(), slots2 * sizeof(int32_t), hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_tok.p, tok.data(), tok.size() * 2, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_d.p, d.data(), d.size() * 2, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemset(d_st2.p, 0, STM_STATUS_WORDS * sizeof(int32_t)));
    CHECK_STM(stm_route_plan(d_ids2.p, 0, slots2, E2, d_hist2.p, d_off2.p, d_pos2.p, d_st2.p, d_ws2.p, ws2, nullptr));
    CHECK_STM(stm_slot_tokens_to_rows(d_pos2.p, slots2, K2, d_table.p, slots2, nullptr));
    CHECK_STM(stm_grouped_gemm_wgrad_gathered(d_d.p, d_tok.p, d_out_g.p, d_off2.p, E2, slots2, P, Q, STM_BF16, d_table.p, 2,
                                              T2, nullptr));
    CHECK_STM(stm_permute_fwd(d_tok.p, d_pos2.p, 0, d_copy.p, T2, K2, int64_t(Q) * 2, slots2, nullptr, nullptr));
    CHECK_STM(stm_grouped_gemm_wgrad(d_d.p, d_copy.p, d_out_c.p, d_off2.p, E2, slots2, P, Q, STM_BF16, nullptr));
    CHECK_HIP(hipDeviceSynchronize());
    std::vector<int32_t> st2(STM_STATUS_WORDS);
    CHECK_HIP(hipMemcpy(st2.data(), d_st2.p, st2.size() * sizeof(int32_t), hipMemcpyDeviceToHost));
    int largest = 0;
    for (int e = 0; e < E2; ++e) largest = off2[e + 1] - off2[e] > largest ? off2[e + 1] - off2[e] : largest;
    if (st2[STM_ST_N_VALID] != int32_t(slots2) || st2[STM_ST_MAX_COUNT] != largest) {
      snprintf(msg, cap, "status words: %d valid, largest %d; expected %d, %d", st2[STM_ST_N_VALID], st2[STM_ST_MAX_COUNT],
               int(slots2), largest);
      return 6;
    }
    std::vector<uint16_t> out_g(size_t(E2) * P * Q), out_c(out_g.size());
    CHECK_HIP(hipMemcpy(out_g.data(), d_out_g.p, out_g.size() * 2, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(out_c.data(), d_out_c.p, out_c.size() * 2, hipMemcpyDeviceToHost));
    if (out_g != out_c) {
      snprintf(msg, cap, "gathered weight gradient differs from the one on copied rows");
      return 7;
    }
    std::vector<int32_t> token_of(slots2);
    for (int64_t i = 0; i < slots2; ++i) token_of[pos2[i]] = int32_t(i / K2);
    for (int e = 0; e < E2; ++e)
      for (int pi = 0; pi < P; pi += 37)
        for (int qi = 0; qi < Q; qi += 41) {
          double ref = 0.0;
          for (int r = off2[e]; r < off2[e + 1]; ++r)
            ref += double(from_bf16(d[size_t(r) * P + pi])) * double(from_bf16(tok[size_t(token_of[r]) * Q + qi]));
          const double got = from_bf16(out_g[(size_t(e) * P + pi) * Q + qi]);
          if (fabs(got - ref) > 1e-2 * (fabs(ref) + 1.0)) {
            snprintf(msg, cap, "gathered weight gradient: expert %d [%d, %d] is %g, expected %g", e, pi, qi, got, ref);
            return 8;
          }
        }
  }
  snprintf(msg, cap, "ok: %d slots, %d rows, %d experts (abi %d)", int(n_slots), n_rows, E, stm_abi_version());
  return 0;
}
