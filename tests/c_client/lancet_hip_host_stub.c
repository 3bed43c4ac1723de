/* Host-only stand-in for liblancet_hip, for the sanitizer build of the C++ op layer (TEST INFRASTRUCTURE).
 *
 * The op layer (raf_hip/) only passes pointers and sizes on; what can go wrong there is host logic: a shape
 * taken from the wrong argument, an output declared too small, a workspace request that does not match the
 * call.  This file implements every C-ABI entry point the op layer uses so that it runs on HOST memory: each
 * "launch" reads every byte the real kernels read and writes every byte they write, with the extents the header
 * documents.  Built with -fsanitize=address,undefined together with raf_hip/ and op_layer_san.cc, a buffer the
 * op layer sized or passed wrongly is a heap-buffer-overflow report.  (The reference builds its host code
 * under the sanitizers the same way, cmake/modules/Sanitizer.cmake:13-40.)  No GPU, no HIP. */
#include <stdlib.h>
#include <string.h>

#include "../../include/lancet_hip.h"

static volatile unsigned char g_sink;

static void touch_read(const void* p, size_t n) {
  const unsigned char* b = (const unsigned char*)p;
  unsigned char s = 0;
  for (size_t i = 0; i < n; ++i) s ^= b[i];
  g_sink = s;
}
static void touch_write(void* p, size_t n) { memset(p, 0x5a, n); }
static size_t eb(int dtype) { return dtype == LANCET_F32 ? 4 : (dtype == LANCET_BF16 || dtype == LANCET_F16 ? 2 : 0); }
static size_t tiles(int64_t S) { return S > 0 ? (size_t)((S + 255) / 256) : 1; }

int lancet_abi_version(void) { return LANCET_ABI_VERSION; }
const char* lancet_status_string(int status) { return status == 0 ? "ok" : "error (host stub)"; }
int64_t lancet_moe_capacity(int64_t S, int64_t E, float cf) {
  if (E <= 0 || S < 0) return -1;
  return (int64_t)(int)(cf * (float)((S + E - 1) / E));
}

size_t lancet_moe_encode_workspace_bytes(int64_t S, int64_t E, int top_k) { return 32 + tiles(S) * (size_t)top_k * (size_t)E * 8; }
size_t lancet_moe_encode_bpr_workspace_bytes(int64_t S0, int64_t E, int P) {
  return 32 + tiles(S0 / P) * 2 * (size_t)E * 8 + ((size_t)S0 + 3 * (size_t)E) * 8;
}
size_t lancet_moe_merge_masks_workspace_bytes(int P, int64_t E) { return (size_t)P * (size_t)E * 4; }
size_t lancet_moe_redispatch_workspace_bytes(int P, int64_t E) { return (size_t)P * (size_t)E * 4; }
size_t lancet_moe_decode_dx_workspace_bytes(int64_t E, int64_t C) { return (size_t)E * (size_t)C * 4; }

int lancet_scan_workspace_init(void* ws, size_t nbytes, lancet_stream_t st) {
  (void)st;
  if (!ws || nbytes < 32) return LANCET_ERR_WORKSPACE;
  touch_write(ws, nbytes);
  return 0;
}

/* as the library decides it: top-1 on at most 32 tiles, or on request (the stub's OpEnvs then also run the set-up) */
int lancet_scan_call_is_stateful(int64_t S, int64_t E, int top_k, unsigned flags, int bpr) {
  (void)E;
  if (flags & LANCET_SCAN_LOOKBACK) return 1;
  return !bpr && top_k == 1 && tiles(S) <= 32;
}

int lancet_scan_workspace_error(void* ws, lancet_stream_t st, int* error_out) {
  (void)st;
  if (!ws || !error_out) return LANCET_ERR_NULL;
  touch_read(ws, 32);
  *error_out = 0;
  return 0;
}

int lancet_moe_encode(const void* data, const void* gate, const void* noise, const int32_t* used_in, int64_t S, int64_t M,
                      int64_t E, int64_t C, int top_k, int dtype, int gate_dtype, unsigned flags, void* gates_s,
                      int32_t* il, int32_t* used_out, uint64_t* elems, void* dispatched, void* ws, size_t ws_bytes,
                      lancet_stream_t st) {
  (void)flags, (void)st;
  if (!eb(dtype) || !eb(gate_dtype)) return LANCET_ERR_DTYPE;
  if (ws_bytes < lancet_moe_encode_workspace_bytes(S, E, top_k)) return LANCET_ERR_WORKSPACE;
  touch_read(data, (size_t)S * M * eb(dtype));
  touch_read(gate, (size_t)S * E * eb(gate_dtype));
  if (noise) touch_read(noise, (size_t)S * E * eb(gate_dtype));
  if (used_in) touch_read(used_in, (size_t)E * 4);
  touch_write(gates_s, (size_t)top_k * S * eb(gate_dtype));
  touch_write(il, (size_t)2 * top_k * S * 4);
  touch_write(used_out, (size_t)E * 4);
  touch_write(elems, (size_t)E * 8);
  touch_write(dispatched, (size_t)E * C * M * eb(dtype));
  touch_write(ws, lancet_moe_encode_workspace_bytes(S, E, top_k));
  return 0;
}

int lancet_moe_encode_bpr(const void* data, const void* gate, int64_t S0, int64_t M, int64_t E, int64_t C, int P, int pid,
                          int dtype, int gate_dtype, unsigned flags, void* gates_s, int32_t* il, int32_t* used_out,
                          uint64_t* elems, void* dispatched, void* ws, size_t ws_bytes, lancet_stream_t st) {
  (void)flags, (void)st;
  if (!eb(dtype) || !eb(gate_dtype)) return LANCET_ERR_DTYPE;
  if (P < 1 || pid < 0 || pid >= P) return LANCET_ERR_PARTITION;
  if (ws_bytes < lancet_moe_encode_bpr_workspace_bytes(S0, E, P)) return LANCET_ERR_WORKSPACE;
  const int64_t S = S0 / P;
  touch_read(data, (size_t)S0 * M * eb(dtype));
  touch_read(gate, (size_t)S0 * E * eb(gate_dtype));
  touch_write(gates_s, (size_t)S * eb(gate_dtype));
  touch_write(il, (size_t)2 * S * 4);
  touch_write(used_out, (size_t)E * 4);
  touch_write(elems, (size_t)E * 8);
  touch_write(dispatched, (size_t)E * C * M * eb(dtype));
  touch_write(ws, lancet_moe_encode_bpr_workspace_bytes(S0, E, P));
  return 0;
}

int lancet_moe_decode(const void* expert_out, const void* gates_s, const int32_t* il, int64_t S, int64_t M, int64_t E,
                      int64_t C, int top_k, int dtype, int gate_dtype, void* out, lancet_stream_t st) {
  (void)st;
  if (!eb(dtype) || !eb(gate_dtype)) return LANCET_ERR_DTYPE;
  touch_read(expert_out, (size_t)E * C * M * eb(dtype));
  touch_read(gates_s, (size_t)top_k * S * eb(gate_dtype));
  touch_read(il, (size_t)2 * top_k * S * 4);
  touch_write(out, (size_t)S * M * eb(dtype));
  return 0;
}

int lancet_moe_merge_masks(const int32_t* const* ils, int P, int64_t S, int64_t E, int32_t* out, void* ws, size_t ws_bytes,
                           lancet_stream_t st) {
  (void)st;
  if (ws_bytes < lancet_moe_merge_masks_workspace_bytes(P, E)) return LANCET_ERR_WORKSPACE;
  for (int p = 0; p < P; ++p) touch_read(ils[p], (size_t)2 * S * 4);
  touch_write(out, (size_t)2 * P * S * 4);
  touch_write(ws, lancet_moe_merge_masks_workspace_bytes(P, E));
  return 0;
}

int lancet_moe_redispatch(const void* const* data, const int32_t* const* ils, int P, int64_t S, int64_t M, int64_t C,
                          int64_t E, int dtype, void* out, void* ws, size_t ws_bytes, lancet_stream_t st) {
  (void)st;
  if (!eb(dtype)) return LANCET_ERR_DTYPE;
  if (ws_bytes < lancet_moe_redispatch_workspace_bytes(P, E)) return LANCET_ERR_WORKSPACE;
  for (int p = 0; p < P; ++p) {
    touch_read(data[p], (size_t)E * C * M * eb(dtype));
    touch_read(ils[p], (size_t)2 * S * 4);
  }
  touch_write(out, (size_t)E * C * M * eb(dtype));
  touch_write(ws, lancet_moe_redispatch_workspace_bytes(P, E));
  return 0;
}

int lancet_moe_redispatch_expert_input(const void* const* data, const uint64_t* const* recv_cnts, int P, int le, int LE,
                                       int64_t C, int64_t M, int64_t G, int scale, int dtype, void* out, lancet_stream_t st) {
  (void)st, (void)le, (void)scale;
  if (!eb(dtype)) return LANCET_ERR_DTYPE;
  for (int p = 0; p < P; ++p) {
    touch_read(data[p], (size_t)C * G * M * eb(dtype));
    touch_read(recv_cnts[p], (size_t)G * LE * 8);
  }
  touch_write(out, (size_t)C * G * M * eb(dtype));
  return 0;
}

int lancet_moe_encode_dx(const void* dy, const int32_t* il, int64_t S, int64_t M, int64_t E, int64_t C, int top_k, int dtype,
                         void* dx, lancet_stream_t st) {
  (void)st;
  if (!eb(dtype)) return LANCET_ERR_DTYPE;
  touch_read(dy, (size_t)E * C * M * eb(dtype));
  touch_read(il, (size_t)2 * top_k * S * 4);
  touch_write(dx, (size_t)S * M * eb(dtype));
  return 0;
}

int lancet_moe_encode_dg(const void* dy, const int32_t* il, int64_t S, int64_t E, int top_k, int gate_dtype, void* grad,
                         lancet_stream_t st) {
  (void)st;
  if (!eb(gate_dtype)) return LANCET_ERR_DTYPE;
  touch_read(dy, (size_t)top_k * S * eb(gate_dtype));
  touch_read(il, (size_t)2 * top_k * S * 4);
  touch_write(grad, (size_t)S * E * eb(gate_dtype));
  return 0;
}

int lancet_moe_decode_dx(const void* dy, const void* gates_s, const int32_t* il, int64_t S, int64_t M, int64_t E, int64_t C,
                         int top_k, int dtype, int gate_dtype, void* grad, void* ws, size_t ws_bytes, lancet_stream_t st) {
  (void)st;
  if (!eb(dtype) || !eb(gate_dtype)) return LANCET_ERR_DTYPE;
  if (ws_bytes < lancet_moe_decode_dx_workspace_bytes(E, C)) return LANCET_ERR_WORKSPACE;
  touch_read(dy, (size_t)S * M * eb(dtype));
  touch_read(gates_s, (size_t)top_k * S * eb(gate_dtype));
  touch_read(il, (size_t)2 * top_k * S * 4);
  touch_write(grad, (size_t)E * C * M * eb(dtype));
  touch_write(ws, lancet_moe_decode_dx_workspace_bytes(E, C));
  return 0;
}

int lancet_moe_decode_dg(const void* dy, const void* expert_out, const int32_t* il, int64_t S, int64_t M, int64_t E,
                         int64_t C, int top_k, int dtype, int gate_dtype, void* grad, lancet_stream_t st) {
  (void)st;
  if (!eb(dtype) || !eb(gate_dtype)) return LANCET_ERR_DTYPE;
  touch_read(dy, (size_t)S * M * eb(dtype));
  touch_read(expert_out, (size_t)E * C * M * eb(dtype));
  touch_read(il, (size_t)2 * top_k * S * 4);
  touch_write(grad, (size_t)top_k * S * eb(gate_dtype));
  return 0;
}

/* ---- LANS: a plan remembers the sizes; a step reads g and reads and writes p, m, v ---- */
struct lancet_lans_plan {
  int T;
  int64_t* numels;
};

int lancet_lans_plan_create(const int64_t* numels, int T, lancet_lans_plan_t* plan) {
  if (!numels || !plan || T < 1) return LANCET_ERR_NULL;
  struct lancet_lans_plan* p = (struct lancet_lans_plan*)malloc(sizeof(*p));
  p->T = T;
  p->numels = (int64_t*)malloc(sizeof(int64_t) * (size_t)T);
  memcpy(p->numels, numels, sizeof(int64_t) * (size_t)T);
  *plan = p;
  return 0;
}
int lancet_lans_plan_destroy(lancet_lans_plan_t plan) {
  if (!plan) return LANCET_ERR_PLAN;
  free(plan->numels);
  free(plan);
  return 0;
}
int lancet_lans_plan_set_schedule(lancet_lans_plan_t plan, int schedule) {
  (void)schedule;
  return plan ? 0 : LANCET_ERR_PLAN;
}
int lancet_lans_plan_error(lancet_lans_plan_t plan, lancet_stream_t st, int* error_out) {
  (void)st;
  if (!plan || !error_out) return LANCET_ERR_PLAN;
  *error_out = 0;
  return 0;
}
int lancet_lans_step(lancet_lans_plan_t plan, const float* const* g, float* const* p, float* const* m, float* const* v,
                     int step_host, const float* step_dev, const lancet_lans_hyper* hyper, const float* grad_norms,
                     lancet_stream_t st) {
  (void)st, (void)step_host;
  if (!plan || !hyper) return LANCET_ERR_PLAN;
  if (step_dev) touch_read(step_dev, 4);
  if (grad_norms) touch_read(grad_norms, (size_t)plan->T * 4);
  for (int i = 0; i < plan->T; ++i) {
    const size_t n = (size_t)plan->numels[i] * 4;
    touch_read(g[i], n);
    touch_read(p[i], n), touch_read(m[i], n), touch_read(v[i], n);
    touch_write(p[i], n), touch_write(m[i], n), touch_write(v[i], n);
  }
  return 0;
}

int lancet_lans_step_mixed(lancet_lans_plan_t plan, const void* const* g, int g_dtype, float* const* p, float* const* m,
                           float* const* v, void* const* p_lowp, int lowp_dtype, int step_host, const float* step_dev,
                           const lancet_lans_hyper* hyper, const float* grad_norms, lancet_stream_t st) {
  (void)st, (void)step_host;
  if (!plan || !hyper) return LANCET_ERR_PLAN;
  if (!eb(g_dtype) || (p_lowp && eb(lowp_dtype) != 2)) return LANCET_ERR_DTYPE;
  if (step_dev) touch_read(step_dev, 4);
  if (grad_norms) touch_read(grad_norms, (size_t)plan->T * 4);
  for (int i = 0; i < plan->T; ++i) {
    const size_t n = (size_t)plan->numels[i];
    touch_read(g[i], n * eb(g_dtype));
    touch_read(p[i], n * 4), touch_read(m[i], n * 4), touch_read(v[i], n * 4);
    touch_write(p[i], n * 4), touch_write(m[i], n * 4), touch_write(v[i], n * 4);
    if (p_lowp) touch_write(p_lowp[i], n * 2);
  }
  return 0;
}

int lancet_moe_encode_dgate(const void* dy, const void* gate, const int32_t* il, int64_t S, int64_t E, int top_k,
                            int gate_dtype, unsigned flags, void* grad, lancet_stream_t st) {
  (void)st;
  if (!eb(gate_dtype)) return LANCET_ERR_DTYPE;
  touch_read(dy, (size_t)top_k * S * eb(gate_dtype));
  touch_read(il, (size_t)top_k * S * 4);                      /* the index row only */
  if (top_k == 2 || (flags & LANCET_GATE_IS_LOGITS)) touch_read(gate, (size_t)S * E * eb(gate_dtype));
  touch_write(grad, (size_t)S * E * eb(gate_dtype));
  return 0;
}

int lancet_moe_route(const void* gate, const void* noise, const int32_t* used_in, int64_t S, int64_t M, int64_t E, int64_t C,
                     int top_k, int gate_dtype, unsigned flags, void* gates_s, int32_t* il, int32_t* used_out,
                     uint64_t* elems, void* ws, size_t ws_bytes, lancet_stream_t st) {
  (void)flags, (void)st, (void)M, (void)C;
  if (!eb(gate_dtype)) return LANCET_ERR_DTYPE;
  if (ws_bytes < lancet_moe_encode_workspace_bytes(S, E, top_k)) return LANCET_ERR_WORKSPACE;
  touch_read(gate, (size_t)S * E * eb(gate_dtype));
  if (noise) touch_read(noise, (size_t)S * E * eb(gate_dtype));
  if (used_in) touch_read(used_in, (size_t)E * 4);
  touch_write(gates_s, (size_t)top_k * S * eb(gate_dtype));
  touch_write(il, (size_t)2 * top_k * S * 4);
  touch_write(used_out, (size_t)E * 4);
  touch_write(elems, (size_t)E * 8);
  touch_write(ws, lancet_moe_encode_workspace_bytes(S, E, top_k));
  return 0;
}

int lancet_moe_scatter_tokens(const void* data, const int32_t* il, const int32_t* used_in, const int32_t* used_out,
                              int64_t S_total, int64_t token_first, int64_t n_tokens, int64_t M, int64_t E, int64_t C,
                              int top_k, int dtype, unsigned flags, void* dispatched, lancet_stream_t st) {
  (void)st;
  if (!eb(dtype)) return LANCET_ERR_DTYPE;
  if (token_first < 0 || n_tokens < 0 || token_first + n_tokens > S_total) return LANCET_ERR_SHAPE;
  touch_read(data, (size_t)n_tokens * M * eb(dtype));
  for (int j = 0; j < 2 * top_k; ++j) touch_read(il + (size_t)j * S_total + token_first, (size_t)n_tokens * 4);
  if (!(flags & LANCET_NO_TAIL_ZERO)) {
    if (used_in) touch_read(used_in, (size_t)E * 4);
    touch_read(used_out, (size_t)E * 4);
  }
  touch_write(dispatched, (size_t)E * C * M * eb(dtype));      /* any row of the buffer may be this call's */
  return 0;
}

int lancet_moe_decode_tokens(const void* expert_out, const void* gates_s, const int32_t* il, int64_t S_total,
                             int64_t token_first, int64_t n_tokens, int64_t M, int64_t E, int64_t C, int top_k, int dtype,
                             int gate_dtype, void* out, lancet_stream_t st) {
  (void)st;
  if (!eb(dtype) || !eb(gate_dtype)) return LANCET_ERR_DTYPE;
  if (token_first < 0 || n_tokens < 0 || token_first + n_tokens > S_total) return LANCET_ERR_SHAPE;
  touch_read(expert_out, (size_t)E * C * M * eb(dtype));
  for (int j = 0; j < top_k; ++j)
    touch_read((const char*)gates_s + ((size_t)j * S_total + token_first) * eb(gate_dtype), (size_t)n_tokens * eb(gate_dtype));
  for (int j = 0; j < 2 * top_k; ++j) touch_read(il + (size_t)j * S_total + token_first, (size_t)n_tokens * 4);
  touch_write(out, (size_t)n_tokens * M * eb(dtype));
  return 0;
}

size_t lancet_moe_partition_ranges_workspace_bytes(int top_k, int P, int64_t E) { return (size_t)top_k * (size_t)P * (size_t)E * 4; }
int lancet_moe_partition_ranges(const int32_t* il, int64_t S_total, int top_k, int P, int64_t E, int64_t M, uint64_t* starts,
                                uint64_t* counts, void* ws, size_t ws_bytes, lancet_stream_t st) {
  (void)st, (void)M;
  if (ws_bytes < lancet_moe_partition_ranges_workspace_bytes(top_k, P, E)) return LANCET_ERR_WORKSPACE;
  touch_read(il, (size_t)top_k * S_total * 4);
  touch_write(starts, (size_t)top_k * P * E * 8);
  touch_write(counts, (size_t)top_k * P * E * 8);
  touch_write(ws, lancet_moe_partition_ranges_workspace_bytes(top_k, P, E));
  return 0;
}
