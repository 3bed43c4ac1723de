/* A plain C99 client of the C ABI (include/lancet_hip.h): no Python, no torch, only the HIP runtime for
 * device memory.  It runs raf.op.moe_encode and raf.op.moe_decode on a case small enough to work out by
 * hand (the rule of src/op/dialect/cuda/kernels/tutel_moe_dispatch.cu:164-212: locations count tokens of
 * the same expert in token order, a token is dropped when its location reaches the capacity) and checks
 * every output value.  Exit status 0 = all values as expected. */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "lancet_hip.h"

#define CHECK_HIP(x)                                                              \
  do {                                                                            \
    hipError_t e_ = (x);                                                          \
    if (e_ != hipSuccess) {                                                       \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                     \
      return 2;                                                                   \
    }                                                                             \
  } while (0)
#define CHECK_LANCET(x)                                                           \
  do {                                                                            \
    int s_ = (x);                                                                 \
    if (s_ != LANCET_OK) {                                                        \
      fprintf(stderr, "%s: status %d (%s)\n", #x, s_, lancet_status_string(s_));  \
      return 3;                                                                   \
    }                                                                             \
  } while (0)

enum { S = 4, M = 2, E = 2 };

int main(void) {
  const float gate[S * E] = {0.9f, 0.1f, 0.2f, 0.8f, 0.6f, 0.4f, 0.7f, 0.3f};
  const float data[S * M] = {1.f, 10.f, 2.f, 20.f, 3.f, 30.f, 4.f, 40.f};
  const int64_t C = lancet_moe_capacity(S, E, 1.0f);
  if (lancet_abi_version() != LANCET_ABI_VERSION || C != 2) {
    fprintf(stderr, "abi %d, capacity %lld\n", lancet_abi_version(), (long long)C);
    return 1;
  }
  const size_t ws_bytes = lancet_moe_encode_workspace_bytes(S, E, 1);
  float *d_gate, *d_data, *d_gates_s, *d_disp, *d_out;
  int32_t *d_il, *d_used;
  uint64_t* d_elems;
  void* d_ws;
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));
  CHECK_HIP(hipMalloc((void**)&d_gate, sizeof(gate)));
  CHECK_HIP(hipMalloc((void**)&d_data, sizeof(data)));
  CHECK_HIP(hipMalloc((void**)&d_gates_s, S * sizeof(float)));
  CHECK_HIP(hipMalloc((void**)&d_il, 2 * S * sizeof(int32_t)));
  CHECK_HIP(hipMalloc((void**)&d_used, E * sizeof(int32_t)));
  CHECK_HIP(hipMalloc((void**)&d_elems, E * sizeof(uint64_t)));
  CHECK_HIP(hipMalloc((void**)&d_disp, E * 2 * M * sizeof(float)));
  CHECK_HIP(hipMalloc((void**)&d_out, S * M * sizeof(float)));
  CHECK_HIP(hipMalloc(&d_ws, ws_bytes));
  CHECK_HIP(hipMemcpy(d_gate, gate, sizeof(gate), hipMemcpyHostToDevice));
  CHECK_HIP(hipMemcpy(d_data, data, sizeof(data), hipMemcpyHostToDevice));
  CHECK_HIP(hipMemset(d_disp, 0xff, E * 2 * M * sizeof(float))); /* stale contents must not survive */
  CHECK_LANCET(lancet_scan_workspace_init(d_ws, ws_bytes, stream)); /* once per workspace */

  CHECK_LANCET(lancet_moe_encode(d_data, d_gate, NULL, NULL, S, M, E, C, 1, LANCET_F32, LANCET_F32, 0u, d_gates_s, d_il, d_used,
                                 d_elems, d_disp, d_ws, ws_bytes, stream));
  CHECK_LANCET(lancet_moe_decode(d_disp, d_gates_s, d_il, S, M, E, C, 1, LANCET_F32, LANCET_F32, d_out, stream));
  CHECK_HIP(hipStreamSynchronize(stream));

  float gates_s[S], disp[E * 2 * M], out[S * M];
  int32_t il[2 * S], used[E];
  uint64_t elems[E];
  CHECK_HIP(hipMemcpy(gates_s, d_gates_s, sizeof(gates_s), hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(il, d_il, sizeof(il), hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(used, d_used, sizeof(used), hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(elems, d_elems, sizeof(elems), hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(disp, d_disp, sizeof(disp), hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(out, d_out, sizeof(out), hipMemcpyDeviceToHost));

  /* tokens 0, 2, 3 choose expert 0 (capacity 2: token 3 is dropped and keeps its location), token 1 expert 1 */
  const float want_gates[S] = {0.9f, 0.8f, 0.6f, 0.7f};
  const int32_t want_il[2 * S] = {0, 1, 0, -1, 0, 0, 1, 2};
  const int32_t want_used[E] = {2, 1};
  const uint64_t want_elems[E] = {2 * M, 1 * M};
  const float want_disp[E * 2 * M] = {1.f, 10.f, 3.f, 30.f, 2.f, 20.f, 0.f, 0.f};
  float want_out[S * M];
  int s, k, bad = 0;
  for (s = 0; s < S; ++s)
    for (k = 0; k < M; ++k) want_out[s * M + k] = want_il[s] < 0 ? 0.f : want_gates[s] * data[s * M + k];
  bad += memcmp(gates_s, want_gates, sizeof(gates_s)) != 0;
  bad += memcmp(il, want_il, sizeof(il)) != 0;
  bad += memcmp(used, want_used, sizeof(used)) != 0;
  bad += memcmp(elems, want_elems, sizeof(elems)) != 0;
  bad += memcmp(disp, want_disp, sizeof(disp)) != 0;
  bad += memcmp(out, want_out, sizeof(out)) != 0;

  /* a rejected call launches nothing and says why */
  if (lancet_moe_encode(d_data, d_gate, NULL, NULL, S, M, E, C, 3, LANCET_F32, LANCET_F32, 0u, d_gates_s, d_il, d_used, d_elems,
                        d_disp, d_ws, ws_bytes, stream) != LANCET_ERR_TOPK)
    ++bad;
  if (lancet_moe_decode(d_disp, d_gates_s, d_il, S, M, E, C, 1, 99, LANCET_F32, d_out, stream) != LANCET_ERR_DTYPE) ++bad;

  hipFree(d_gate), hipFree(d_data), hipFree(d_gates_s), hipFree(d_il), hipFree(d_used);
  hipFree(d_elems), hipFree(d_disp), hipFree(d_out), hipFree(d_ws);
  hipStreamDestroy(stream);
  if (bad) {
    fprintf(stderr, "lancet_client: %d mismatching outputs\n", bad);
    return 1;
  }
  printf("lancet_client: encode + decode through the C ABI match the hand-computed case\n");
  return 0;
}
