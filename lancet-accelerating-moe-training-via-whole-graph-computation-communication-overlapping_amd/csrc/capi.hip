// C ABI of the MoE dispatch path: argument validation, then kernel launches on the caller's
// stream.  Nothing here allocates, synchronises or keeps state between calls.
#include "../../include/lancet_hip_debug.h"
#include "common.hpp"
#include "launchers.hpp"
#include "scan.hpp"

using namespace lancet;

namespace {

inline hipStream_t S_(lancet_stream_t s) { return static_cast<hipStream_t>(s); }
inline int rc(hipError_t e) { return static_cast<int>(e); }

inline int elem_bytes(int dtype) {
  switch (dtype) {
    case LANCET_F32: return 4;
    case LANCET_BF16:
    case LANCET_F16: return 2;
    default: return 0;
  }
}

inline bool misaligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; }

// S, M, C, E and the products the kernels index with must fit what the kernels assume.
int check_dims(int64_t S, int64_t M, int64_t E, int64_t C) {
  if (S < 0 || M < 0 || C < 0 || E < 1) return LANCET_ERR_SHAPE;
  if (E > LANCET_MAX_EXPERTS) return LANCET_ERR_SHAPE;
  if (S > 0x3fffffff || M > 0x3fffffff || C > 0x3fffffff) return LANCET_ERR_SHAPE;
  if (E * C > 0x7fffffff) return LANCET_ERR_SHAPE;
  return LANCET_OK;
}

int fill_table(PtrTable& t, const void* const* ptrs, int P, size_t align) {
  for (int p = 0; p < P; ++p) {
    if (!ptrs[p]) return LANCET_ERR_NULL;
    if (misaligned(ptrs[p], align)) return LANCET_ERR_ALIGN;
    t.p[p] = ptrs[p];
  }
  for (int p = P; p < kMaxPartitions; ++p) t.p[p] = nullptr;
  return LANCET_OK;
}

}  // namespace

extern "C" int lancet_abi_version(void) { return LANCET_ABI_VERSION; }

extern "C" const char* lancet_status_string(int status) {
  switch (status) {
    case LANCET_OK: return "ok";
    case LANCET_ERR_NULL: return "required pointer is NULL";
    case LANCET_ERR_SHAPE: return "bad or unsupported size";
    case LANCET_ERR_DTYPE: return "unknown dtype";
    case LANCET_ERR_WORKSPACE: return "workspace missing or too small";
    case LANCET_ERR_ALIGN: return "pointer not aligned to its element type";
    case LANCET_ERR_TOPK: return "top_k must be 1 or 2 (2 needs at least two experts)";
    case LANCET_ERR_PARTITION: return "bad n_partitions / partition_id";
    case LANCET_ERR_PLAN: return "invalid LANS plan";
    case LANCET_ERR_STALLED: return "an earlier LANS step of this plan gave up a wait (call lancet_lans_plan_error)";
    case LANCET_ERR_SCRATCH: return "sizes exceed the static scratch of the allocation-free entry point";
    default: return status > 0 ? hipGetErrorString(static_cast<hipError_t>(status)) : "unknown status";
  }
}

extern "C" int64_t lancet_moe_capacity(int64_t S, int64_t E, float capacity_factor) {
  if (E <= 0 || S < 0) return -1;
  // float * integer in float, truncated: src/op/dialect/cuda/moe.cc:109.  A product that no int holds (or a NaN
  // factor) has no capacity: -1, which every entry point that takes a capacity rejects.
  const float c = capacity_factor * static_cast<float>(S / E + (S % E != 0));
  if (!(c > -2147483648.f && c < 2147483648.f)) return -1;
  return static_cast<int64_t>(static_cast<int>(c));
}

extern "C" int lancet_debug_scan_workspace_spin_limit(void* workspace, unsigned limit, lancet_stream_t stream) {
  if (!workspace) return LANCET_ERR_NULL;
  if (misaligned(workspace, 8)) return LANCET_ERR_ALIGN;
  return rc(run_scan_ws_set_spin(workspace, limit, S_(stream)));
}

extern "C" int lancet_debug_scan_workspace_epoch(void* workspace, unsigned epoch, lancet_stream_t stream) {
  if (!workspace) return LANCET_ERR_NULL;
  if (misaligned(workspace, 8)) return LANCET_ERR_ALIGN;
  if (epoch < 1u || epoch > 0x3fffffffu) return LANCET_ERR_SHAPE;
  return rc(run_scan_ws_set_epoch(workspace, epoch, S_(stream)));
}

extern "C" int lancet_scan_workspace_init(void* workspace, size_t workspace_bytes, lancet_stream_t stream) {
  if (!workspace) return LANCET_ERR_NULL;
  if (misaligned(workspace, 8)) return LANCET_ERR_ALIGN;
  if (workspace_bytes < scan_workspace_bytes(0, 1, 1)) return LANCET_ERR_WORKSPACE;
  return rc(run_scan_ws_init(workspace, workspace_bytes, S_(stream)));
}

extern "C" int lancet_scan_call_is_stateful(int64_t S, int64_t E, int top_k, unsigned flags, int batch_prioritized) {
  if (S < 0 || E < 1 || (top_k != 1 && top_k != 2)) return 0;
  const int nsets = batch_prioritized ? 2 : top_k;
  return scan_form(scan_num_tiles(S), static_cast<int64_t>(nsets) * E, nsets, (flags & LANCET_SCAN_LOOKBACK) != 0) == kScanLookback;
}

extern "C" int lancet_scan_workspace_error(void* workspace, lancet_stream_t stream, int* error_out) {
  if (!workspace || !error_out) return LANCET_ERR_NULL;
  return rc(run_scan_ws_take_error(workspace, error_out, S_(stream)));
}

// ---- plain streaming kernels (measurement aid) -------------------------------------------
namespace {
template <int KIND>
__global__ __launch_bounds__(256) void stream_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src) {
  const size_t i = blockIdx.x * static_cast<size_t>(256) + threadIdx.x;
  if (KIND == 0) {
    const u32x4 x = ld_stream(src + i);
    if ((x.x ^ x.y ^ x.z ^ x.w) == 0x5eedf00du && dst) st_stream(dst, x);  // keeps the load alive; practically never taken
  } else if (KIND == 1) {
    const u32x4 z = {0u, 0u, 0u, 0u};
    st_stream(dst + i, z);
  } else {
    st_stream(dst + i, ld_stream(src + i));
  }
}
typedef float f32x4 __attribute__((ext_vector_type(4)));
// the access pattern of an optimizer step and nothing else: four arrays read, three of them written, one
// float4 per thread and array, workgroups in address order
__global__ __launch_bounds__(256) void stream_4r3w_kernel(const f32x4* __restrict__ g, f32x4* __restrict__ p,
                                                          f32x4* __restrict__ m, f32x4* __restrict__ v) {
  const size_t i = blockIdx.x * static_cast<size_t>(256) + threadIdx.x;
  const f32x4 xg = __builtin_nontemporal_load(g + i);
  f32x4 xp = __builtin_nontemporal_load(p + i), xm = __builtin_nontemporal_load(m + i), xv = __builtin_nontemporal_load(v + i);
  xm = xm * 0.9f + xg * 0.1f;
  xv = xv * 0.999f + xg * xg * 0.001f;
  xp = xp - xm * 1e-3f;
  __builtin_nontemporal_store(xm, m + i);
  __builtin_nontemporal_store(xv, v + i);
  __builtin_nontemporal_store(xp, p + i);
}
}  // namespace

extern "C" int lancet_debug_stream_4r3w(const float* g, float* p, float* m, float* v, size_t n, lancet_stream_t stream) {
  if (!g || !p || !m || !v) return LANCET_ERR_NULL;
  if (n % 1024 != 0 || n / 1024 > 0x7fffffffu) return LANCET_ERR_SHAPE;
  if (misaligned(g, 16) || misaligned(p, 16) || misaligned(m, 16) || misaligned(v, 16)) return LANCET_ERR_ALIGN;
  if (n == 0) return LANCET_OK;
  stream_4r3w_kernel<<<static_cast<unsigned>(n / 1024), 256, 0, S_(stream)>>>(
      reinterpret_cast<const f32x4*>(g), reinterpret_cast<f32x4*>(p), reinterpret_cast<f32x4*>(m),
      reinterpret_cast<f32x4*>(v));
  return rc(hipGetLastError());
}

extern "C" int lancet_debug_stream(int kind, void* dst, const void* src, size_t bytes, lancet_stream_t stream) {
  if (kind < 0 || kind > 2) return LANCET_ERR_SHAPE;
  if (bytes % 4096 != 0 || bytes / 4096 > 0x7fffffffu) return LANCET_ERR_SHAPE;
  if ((kind != 1 && !src) || (kind != 0 && !dst)) return LANCET_ERR_NULL;
  if (misaligned(dst, 16) || misaligned(src, 16)) return LANCET_ERR_ALIGN;
  if (bytes == 0) return LANCET_OK;
  const unsigned blocks = static_cast<unsigned>(bytes / 4096);
  u32x4* d = static_cast<u32x4*>(dst);
  const u32x4* s = static_cast<const u32x4*>(src);
  if (kind == 0) stream_kernel<0><<<blocks, 256, 0, S_(stream)>>>(d, s);
  else if (kind == 1) stream_kernel<1><<<blocks, 256, 0, S_(stream)>>>(d, s);
  else stream_kernel<2><<<blocks, 256, 0, S_(stream)>>>(d, s);
  return rc(hipGetLastError());
}

// Measurement aid: the scatter and the gather-combine fed with ONE routing word per slot (dest[j*S + s] = e * C + location,
// -1 = none) instead of the four of indices_locations and the capacity arrays.
extern "C" int lancet_debug_scatter_dest(const void* data, const int32_t* dest, const int32_t* used_in, const int32_t* used_out,
                                         int64_t S, int64_t M, int64_t E, int64_t C, int top_k, int dtype, void* dispatched,
                                         lancet_stream_t stream) {
  if (!data || !dest || !used_out || !dispatched) return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, M, E, C)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if ((M * eb) % 16 != 0 || misaligned(data, 16) || misaligned(dispatched, 16) || misaligned(dest, 4)) return LANCET_ERR_ALIGN;
  return rc(run_scatter_rows(data, dispatched, nullptr, nullptr, nullptr, nullptr, used_in, used_out, static_cast<int>(S),
                             static_cast<int>(M), static_cast<int>(E), static_cast<int>(C), top_k, eb, S_(stream), -1, dest));
}

extern "C" int lancet_debug_decode_dest(const void* expert_out, const void* gates_s, const int32_t* dest, int64_t S, int64_t M,
                                        int64_t E, int64_t C, int top_k, int dtype, int gate_dtype, void* out,
                                        lancet_stream_t stream) {
  if (!expert_out || !gates_s || !dest || !out) return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype), gb = elem_bytes(gate_dtype);
  if (!eb || !gb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, M, E, C)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if ((M * eb) % 16 != 0 || misaligned(expert_out, 16) || misaligned(out, 16) || misaligned(dest, 4)) return LANCET_ERR_ALIGN;
  return rc(run_decode_rows(expert_out, gates_s, gate_dtype, nullptr, nullptr, out, static_cast<int>(S), static_cast<int>(M),
                            static_cast<int>(E), static_cast<int>(C), top_k, dtype, S_(stream), -1, dest));
}

// ---- routing front end ---------------------------------------------------------------
extern "C" int lancet_gate_topk(const void* gate, const void* gate2_noise, int64_t S, int64_t E, int top_k,
                                int gate_dtype, unsigned flags, int32_t* idx, void* val, lancet_stream_t stream) {
  if (!gate || !idx || !val) return LANCET_ERR_NULL;
  const int gb = elem_bytes(gate_dtype);
  if (!gb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, 0, E, 0)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if (top_k == 2 && E < 2) return LANCET_ERR_TOPK;
  if (gate2_noise && top_k != 2) return LANCET_ERR_TOPK;  // the noise only exists for the second choice
  if (misaligned(gate, gb) || misaligned(gate2_noise, gb) || misaligned(idx, 4) || misaligned(val, gb))
    return LANCET_ERR_ALIGN;
  return rc(run_gate_topk(gate, gate2_noise, static_cast<int>(S), static_cast<int>(E), top_k,
                          (flags & LANCET_GATE_IS_LOGITS) != 0, gate_dtype, idx, val, S_(stream)));
}

// ---- launcher level ------------------------------------------------------------------
extern "C" size_t lancet_gen_location_workspace_bytes(int64_t S, int64_t E) {
  if (S < 0 || E < 1) return 0;
  return scan_workspace_bytes(S, E, 1);
}

extern "C" int lancet_launch_gen_location(int32_t* indices, const int32_t* in_capused, int32_t* locations,
                                          int32_t* out_capused, uint64_t* out_elements_per_expert,
                                          int64_t C, int64_t S, int64_t E, int64_t M, void* workspace,
                                          size_t workspace_bytes, lancet_stream_t stream) {
  if (!indices || !locations || !out_capused || !out_elements_per_expert) return LANCET_ERR_NULL;
  if (int r = check_dims(S, M, E, C)) return r;
  if (!workspace || workspace_bytes < lancet_gen_location_workspace_bytes(S, E)) return LANCET_ERR_WORKSPACE;
  if (misaligned(indices, 4) || misaligned(locations, 4) || misaligned(out_capused, 4) ||
      misaligned(out_elements_per_expert, 8) || misaligned(workspace, 8) || misaligned(in_capused, 4))
    return LANCET_ERR_ALIGN;
  return rc(run_route_scan(nullptr, nullptr, indices, in_capused, static_cast<int>(S), static_cast<int>(E),
                           static_cast<int>(C), static_cast<int>(M), 1, false, LANCET_F32, nullptr, indices, locations,
                           out_capused, out_elements_per_expert, workspace, S_(stream)));
}

extern "C" int lancet_launch_encode_forward(const int32_t* indices, const int32_t* locations,
                                            const int32_t* capused, const void* data, void* dispatched,
                                            int64_t S, int64_t M, int64_t C, int64_t E, int dtype,
                                            lancet_stream_t stream) {
  if (!indices || !locations || !dispatched || (!data && S > 0)) return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, M, E, C)) return r;
  if (misaligned(data, eb) || misaligned(dispatched, eb) || misaligned(indices, 4) || misaligned(locations, 4))
    return LANCET_ERR_ALIGN;
  // rows filled by an arbitrary (indices, locations) pair need not form a prefix, so the
  // buffer is cleared first, as the reference launcher does
  hipError_t e = run_zero_bytes(dispatched, static_cast<size_t>(E) * C * M * eb, S_(stream));
  if (e != hipSuccess) return rc(e);
  return rc(run_scatter_rows(data, dispatched, indices, locations, capused, nullptr, nullptr, nullptr,
                             static_cast<int>(S), static_cast<int>(M), static_cast<int>(E),
                             static_cast<int>(C), 1, eb, S_(stream)));
}

// ---- raf.op.moe_encode ---------------------------------------------------------------
extern "C" size_t lancet_moe_encode_workspace_bytes(int64_t S, int64_t E, int top_k) {
  if (S < 0 || E < 1 || (top_k != 1 && top_k != 2)) return 0;
  return scan_workspace_bytes(S, E, top_k);
}

extern "C" int lancet_moe_route(const void* gate, const void* gate2_noise, const int32_t* used_in, int64_t S,
                                int64_t M, int64_t E, int64_t C, int top_k, int gate_dtype, unsigned flags, void* gates_s,
                                int32_t* indices_locations, int32_t* used_out, uint64_t* elements_per_expert,
                                void* workspace, size_t workspace_bytes, lancet_stream_t stream) {
  if (((!gate || !gates_s || !indices_locations) && S > 0) || !used_out || !elements_per_expert)
    return LANCET_ERR_NULL;
  const int gb = elem_bytes(gate_dtype);
  if (!gb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, M, E, C)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if (top_k == 2 && E < 2) return LANCET_ERR_TOPK;
  if (gate2_noise && top_k != 2) return LANCET_ERR_TOPK;
  if (!workspace || workspace_bytes < lancet_moe_encode_workspace_bytes(S, E, top_k)) return LANCET_ERR_WORKSPACE;
  if (misaligned(gate, gb) || misaligned(gate2_noise, gb) || misaligned(gates_s, gb) || misaligned(indices_locations, 4) || misaligned(used_in, 4) ||
      misaligned(used_out, 4) || misaligned(elements_per_expert, 8) || misaligned(workspace, 8))
    return LANCET_ERR_ALIGN;
  const int s = static_cast<int>(S);
  return rc(run_route_scan(gate, gate2_noise, nullptr, used_in, s, static_cast<int>(E), static_cast<int>(C),
                           static_cast<int>(M), top_k, (flags & LANCET_GATE_IS_LOGITS) != 0, gate_dtype, gates_s,
                           indices_locations, indices_locations + static_cast<size_t>(top_k) * s, used_out,
                           elements_per_expert, workspace, S_(stream), (flags & LANCET_SCAN_LOOKBACK) != 0));
}

extern "C" int lancet_moe_scatter(const void* data, const int32_t* indices_locations, const int32_t* used_in,
                                  const int32_t* used_out, int64_t S, int64_t M, int64_t E, int64_t C, int top_k,
                                  int dtype, unsigned flags, void* dispatched, lancet_stream_t stream) {
  if ((!data && S > 0 && M > 0) || (!indices_locations && S > 0) || !used_out || (!dispatched && C > 0 && M > 0))
    return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, M, E, C)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if (misaligned(data, eb) || misaligned(dispatched, eb) || misaligned(indices_locations, 4) ||
      misaligned(used_in, 4) || misaligned(used_out, 4))
    return LANCET_ERR_ALIGN;
  const int s = static_cast<int>(S);
  const bool tail = !(flags & LANCET_NO_TAIL_ZERO);
  // rows of this call start at row 0 of every expert, or behind the rows earlier calls used
  const bool at_used = (flags & LANCET_ROWS_AT_USED) != 0 && used_in != nullptr;
  return rc(run_scatter_rows(data, dispatched, indices_locations, indices_locations + static_cast<size_t>(top_k) * s,
                             nullptr, at_used ? used_in : nullptr, (tail && !at_used) ? used_in : nullptr,
                             tail ? used_out : nullptr, s, static_cast<int>(M),
                             static_cast<int>(E), static_cast<int>(C), top_k, eb, S_(stream)));
}

extern "C" int lancet_moe_encode(const void* data, const void* gate, const void* gate2_noise,
                                 const int32_t* used_in, int64_t S, int64_t M, int64_t E, int64_t C, int top_k,
                                 int dtype, int gate_dtype, unsigned flags,
                                 void* gates_s, int32_t* indices_locations, int32_t* used_out,
                                 uint64_t* elements_per_expert, void* dispatched, void* workspace,
                                 size_t workspace_bytes, lancet_stream_t stream) {
  // validate everything before the first launch
  if ((!data && S > 0 && M > 0) || (!dispatched && C > 0 && M > 0)) return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (misaligned(data, eb) || misaligned(dispatched, eb)) return LANCET_ERR_ALIGN;
  if (int r = lancet_moe_route(gate, gate2_noise, used_in, S, M, E, C, top_k, gate_dtype, flags, gates_s, indices_locations, used_out,
                               elements_per_expert, workspace, workspace_bytes, stream))
    return r;
  return lancet_moe_scatter(data, indices_locations, used_in, used_out, S, M, E, C, top_k, dtype, flags, dispatched,
                            stream);
}

// ---- token ranges of a whole-batch mask ------------------------------------------------
namespace {
int check_range(int64_t S_total, int64_t token_first, int64_t n_tokens) {
  if (S_total < 0 || S_total > 0x3fffffff || token_first < 0 || n_tokens < 0 || token_first > S_total ||
      n_tokens > S_total - token_first)
    return LANCET_ERR_SHAPE;
  return LANCET_OK;
}
}  // namespace

extern "C" int lancet_moe_scatter_tokens(const void* data, const int32_t* indices_locations, const int32_t* used_in,
                                         const int32_t* used_out, int64_t S_total, int64_t token_first, int64_t n_tokens, int64_t M, int64_t E,
                                         int64_t C, int top_k, int dtype, unsigned flags, void* dispatched,
                                         lancet_stream_t stream) {
  const bool tail = !(flags & LANCET_NO_TAIL_ZERO);
  if ((!data && n_tokens > 0 && M > 0) || (!indices_locations && n_tokens > 0) || (tail && !used_out) ||
      (!dispatched && C > 0 && M > 0))
    return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S_total, M, E, C)) return r;
  if (int r = check_range(S_total, token_first, n_tokens)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if (misaligned(data, eb) || misaligned(dispatched, eb) || misaligned(indices_locations, 4) ||
      misaligned(used_in, 4) || misaligned(used_out, 4))
    return LANCET_ERR_ALIGN;
  const size_t st = static_cast<size_t>(S_total);
  return rc(run_scatter_rows(data, dispatched, indices_locations + token_first,
                             indices_locations + static_cast<size_t>(top_k) * st + token_first, nullptr, nullptr,
                             tail ? used_in : nullptr, tail ? used_out : nullptr, static_cast<int>(n_tokens), static_cast<int>(M),
                             static_cast<int>(E), static_cast<int>(C), top_k, eb, S_(stream), static_cast<int>(S_total)));
}

extern "C" int lancet_moe_decode_tokens(const void* expert_out, const void* gates_s, const int32_t* indices_locations,
                                        int64_t S_total, int64_t token_first, int64_t n_tokens, int64_t M, int64_t E,
                                        int64_t C, int top_k, int dtype, int gate_dtype, void* out, lancet_stream_t stream) {
  if ((!expert_out && C > 0 && M > 0) || ((!gates_s || !indices_locations) && n_tokens > 0) ||
      (!out && n_tokens > 0 && M > 0))
    return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S_total, M, E, C)) return r;
  if (int r = check_range(S_total, token_first, n_tokens)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  const int gb = elem_bytes(gate_dtype);
  if (!gb) return LANCET_ERR_DTYPE;
  if (misaligned(expert_out, eb) || misaligned(out, eb) || misaligned(gates_s, gb) || misaligned(indices_locations, 4))
    return LANCET_ERR_ALIGN;
  const size_t st = static_cast<size_t>(S_total);
  return rc(run_decode_rows(expert_out, static_cast<const char*>(gates_s) + static_cast<size_t>(token_first) * gb, gate_dtype,
                            indices_locations + token_first,
                            indices_locations + static_cast<size_t>(top_k) * st + token_first, out,
                            static_cast<int>(n_tokens), static_cast<int>(M), static_cast<int>(E), static_cast<int>(C),
                            top_k, dtype, S_(stream), static_cast<int>(S_total)));
}

// ---- raf.op.moe_encode_batch_prioritized ----------------------------------------------
extern "C" size_t lancet_moe_encode_bpr_workspace_bytes(int64_t S0, int64_t E, int n_partitions) {
  if (S0 < 0 || E < 1 || n_partitions < 1) return 0;
  return bpr_workspace_bytes(S0, S0 / n_partitions, E);
}

extern "C" int lancet_moe_encode_bpr(const void* data, const void* gate, int64_t S0, int64_t M, int64_t E,
                                     int64_t C, int n_partitions, int partition_id, int dtype, int gate_dtype, unsigned flags,
                                     void* gates_s, int32_t* indices_locations, int32_t* used_out,
                                     uint64_t* elements_per_expert, void* dispatched, void* workspace,
                                     size_t workspace_bytes, lancet_stream_t stream) {
  if ((!data && S0 > 0 && M > 0) || ((!gate || !gates_s || !indices_locations) && S0 > 0) || !used_out ||
      !elements_per_expert || (!dispatched && C > 0 && M > 0))
    return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype), gb = elem_bytes(gate_dtype);
  if (!eb || !gb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S0, M, E, C)) return r;
  // src/op/declare/moe.cc:74-75
  if (n_partitions < 1 || partition_id < 0 || partition_id >= n_partitions) return LANCET_ERR_PARTITION;
  if (!workspace || workspace_bytes < lancet_moe_encode_bpr_workspace_bytes(S0, E, n_partitions))
    return LANCET_ERR_WORKSPACE;
  if (misaligned(data, eb) || misaligned(dispatched, eb) || misaligned(gate, gb) || misaligned(gates_s, gb) ||
      misaligned(indices_locations, 4) || misaligned(used_out, 4) || misaligned(elements_per_expert, 8) ||
      misaligned(workspace, 8))
    return LANCET_ERR_ALIGN;
  const int s0 = static_cast<int>(S0);
  const int s = s0 / n_partitions;
  int32_t* idx = indices_locations;
  int32_t* loc = indices_locations + s;
  hipError_t e = run_bpr_route(gate, s0, static_cast<int>(E), static_cast<int>(C), static_cast<int>(M),
                               n_partitions, partition_id, (flags & LANCET_GATE_IS_LOGITS) != 0, gate_dtype, gates_s, idx,
                               loc, used_out, elements_per_expert, workspace, S_(stream), (flags & LANCET_SCAN_LOOKBACK) != 0);
  if (e != hipSuccess) return rc(e);
  const char* part = static_cast<const char*>(data) + static_cast<size_t>(partition_id) * s * M * eb;
  return rc(run_scatter_rows(part, dispatched, idx, loc, nullptr, nullptr, nullptr,
                             (flags & LANCET_NO_TAIL_ZERO) ? nullptr : used_out, s, static_cast<int>(M),
                             static_cast<int>(E), static_cast<int>(C), 1, eb, S_(stream)));
}

// ---- raf.op.moe_decode ---------------------------------------------------------------
extern "C" int lancet_moe_decode(const void* expert_out, const void* gates_s, const int32_t* indices_locations,
                                 int64_t S, int64_t M, int64_t E, int64_t C, int top_k, int dtype, int gate_dtype, void* out,
                                 lancet_stream_t stream) {
  if ((!expert_out && C > 0 && M > 0) || ((!gates_s || !indices_locations) && S > 0) || (!out && S > 0 && M > 0))
    return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, M, E, C)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  const int gb = elem_bytes(gate_dtype);
  if (!gb) return LANCET_ERR_DTYPE;
  if (misaligned(expert_out, eb) || misaligned(out, eb) || misaligned(gates_s, gb) || misaligned(indices_locations, 4))
    return LANCET_ERR_ALIGN;
  const int s = static_cast<int>(S);
  return rc(run_decode_rows(expert_out, gates_s, gate_dtype, indices_locations, indices_locations + static_cast<size_t>(top_k) * s,
                            out, s, static_cast<int>(M), static_cast<int>(E), static_cast<int>(C), top_k, dtype,
                            S_(stream)));
}

extern "C" int lancet_moe_redispatch_expert_input(const void* const* data, const uint64_t* const* recv_cnts, int P,
                                                  int local_expert_id, int n_local_experts, int64_t C, int64_t M,
                                                  int64_t G, int recv_cnts_scale, int dtype, void* out,
                                                  lancet_stream_t stream) {
  if (!data || !recv_cnts || (!out && C > 0 && M > 0 && G > 0)) return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (P < 1 || P > LANCET_MAX_PARTITIONS) return LANCET_ERR_PARTITION;
  if (C < 0 || M < 0 || G < 1 || n_local_experts < 1 || local_expert_id < 0 || local_expert_id >= n_local_experts ||
      recv_cnts_scale < 1 || C > 0x3fffffff || M > 0x3fffffff || G > 0x3fffffff || C * G > 0x7fffffff)
    return LANCET_ERR_SHAPE;
  if (misaligned(out, eb)) return LANCET_ERR_ALIGN;
  PtrTable bufs;
  if (int r = fill_table(bufs, data, P, eb)) return r;
  for (int p = 0; p < P; ++p) {
    if (!recv_cnts[p]) return LANCET_ERR_NULL;
    if (misaligned(recv_cnts[p], 8)) return LANCET_ERR_ALIGN;
  }
  return rc(run_redispatch_expert_input(bufs, reinterpret_cast<const void* const*>(recv_cnts), P, local_expert_id,
                                        n_local_experts, static_cast<int>(C), static_cast<int>(M), static_cast<int>(G),
                                        static_cast<uint64_t>(recv_cnts_scale), out, eb, S_(stream)));
}

// ---- sparse <-> packed copies ---------------------------------------------------------------
namespace {
int sparse_copy(const void* src, void* dst, const uint64_t* counts, const uint64_t* starts, int64_t n_counts, int stride, int offset, int axis,
                int64_t dim0, int64_t dim1, int64_t dim2, int64_t cont_elems, int scale, int shrink, int dtype,
                unsigned flags, bool to_cont, lancet_stream_t stream) {
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (axis != 0 && axis != 1) return LANCET_ERR_SHAPE;
  if (dim0 < 0 || dim1 < 0 || dim2 < 0 || cont_elems < 0 || scale < 1 || shrink < 1 || stride < 1 || offset < 0)
    return LANCET_ERR_SHAPE;
  if (dim0 > 0x7fffffff || dim1 > 0x7fffffff || dim2 > 0x7fffffff) return LANCET_ERR_SHAPE;
  const int64_t nblocks = axis == 0 ? dim0 : dim1;
  const int64_t other = axis == 0 ? dim1 : dim0;
  if (other > 0 && dim2 > 0x7fffffff / other) return LANCET_ERR_SHAPE;  // one block's elements fit in 31 bits
  if (nblocks > 65535) return LANCET_ERR_SHAPE;                         // grid y
  if (nblocks == 0 || other * dim2 == 0) return LANCET_OK;
  if (!src || !dst || !counts) return LANCET_ERR_NULL;
  if ((nblocks - 1) * stride + offset >= n_counts) return LANCET_ERR_SHAPE;
  if (misaligned(src, eb) || misaligned(dst, eb) || misaligned(counts, 8) || misaligned(starts, 8)) return LANCET_ERR_ALIGN;
  return rc(run_sparse_copy_3d(src, dst, counts, starts, stride, offset, axis, static_cast<int>(dim0), static_cast<int>(dim1),
                               static_cast<int>(dim2), static_cast<uint64_t>(cont_elems), static_cast<uint64_t>(scale),
                               static_cast<uint64_t>(shrink), to_cont, (flags & LANCET_ZERO_TAIL) != 0, eb, S_(stream)));
}
}  // namespace

extern "C" int lancet_memcpy_sparse_to_cont_3d(const void* src, void* dst, const uint64_t* nelements_per_dim,
                                               int64_t n_counts, int nelements_stride, int nelements_offset, int axis,
                                               int64_t dim0, int64_t dim1, int64_t dim2, int64_t dst_elems,
                                               int scale_element_size_by, int shrink_element_size_by, int dtype,
                                               lancet_stream_t stream) {
  return sparse_copy(src, dst, nelements_per_dim, nullptr, n_counts, nelements_stride, nelements_offset, axis, dim0, dim1, dim2,
                     dst_elems, scale_element_size_by, shrink_element_size_by, dtype, 0u, true, stream);
}

extern "C" int lancet_memcpy_cont_to_sparse_3d(const void* src, void* dst, const uint64_t* nelements_per_dim,
                                               int64_t n_counts, int nelements_stride, int nelements_offset, int axis,
                                               int64_t dim0, int64_t dim1, int64_t dim2, int64_t src_elems,
                                               int scale_element_size_by, int shrink_element_size_by, int dtype,
                                               unsigned flags, lancet_stream_t stream) {
  return sparse_copy(src, dst, nelements_per_dim, nullptr, n_counts, nelements_stride, nelements_offset, axis, dim0, dim1, dim2,
                     src_elems, scale_element_size_by, shrink_element_size_by, dtype, flags, false, stream);
}

extern "C" int lancet_memcpy_sparse_ranges_to_cont_3d(const void* src, void* dst, const uint64_t* nelements_per_dim,
                                                      const uint64_t* starts_per_dim, int64_t n_counts,
                                                      int nelements_stride, int nelements_offset, int axis, int64_t dim0,
                                                      int64_t dim1, int64_t dim2, int64_t dst_elems, int dtype,
                                                      lancet_stream_t stream) {
  if (!starts_per_dim && dim0 > 0 && dim1 > 0 && dim2 > 0) return LANCET_ERR_NULL;
  return sparse_copy(src, dst, nelements_per_dim, starts_per_dim, n_counts, nelements_stride, nelements_offset, axis, dim0,
                     dim1, dim2, dst_elems, 1, 1, dtype, 0u, true, stream);
}

extern "C" int lancet_memcpy_cont_to_sparse_ranges_3d(const void* src, void* dst, const uint64_t* nelements_per_dim,
                                                      const uint64_t* starts_per_dim, int64_t n_counts,
                                                      int nelements_stride, int nelements_offset, int axis, int64_t dim0,
                                                      int64_t dim1, int64_t dim2, int64_t src_elems, int dtype,
                                                      lancet_stream_t stream) {
  if (!starts_per_dim && dim0 > 0 && dim1 > 0 && dim2 > 0) return LANCET_ERR_NULL;
  return sparse_copy(src, dst, nelements_per_dim, starts_per_dim, n_counts, nelements_stride, nelements_offset, axis, dim0,
                     dim1, dim2, src_elems, 1, 1, dtype, 0u, false, stream);
}

// ---- row ranges of token partitions inside a whole-batch routing --------------------------------
namespace {
__global__ __launch_bounds__(256) void partition_ranges_kernel(const uint32_t* __restrict__ counts, int Q, int E, int64_t M,
                                                               uint64_t* __restrict__ starts, uint64_t* __restrict__ cnts) {
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= E) return;
  uint64_t run = 0;
  for (int q = 0; q < Q; ++q) {  // capacity order: slot-major, then partition
    const uint64_t k = counts[static_cast<size_t>(q) * E + e];
    starts[static_cast<size_t>(q) * E + e] = run * static_cast<uint64_t>(M);
    cnts[static_cast<size_t>(q) * E + e] = k * static_cast<uint64_t>(M);
    run += k;
  }
}
}  // namespace

extern "C" size_t lancet_moe_partition_ranges_workspace_bytes(int top_k, int n_partitions, int64_t E) {
  if (top_k < 1 || top_k > 2 || n_partitions < 1 || E < 1) return 0;
  return static_cast<size_t>(top_k) * n_partitions * E * sizeof(uint32_t);
}

extern "C" int lancet_moe_partition_ranges(const int32_t* indices_locations, int64_t S_total, int top_k, int n_partitions,
                                           int64_t E, int64_t M, uint64_t* starts, uint64_t* counts, void* workspace,
                                           size_t workspace_bytes, lancet_stream_t stream) {
  if ((!indices_locations && S_total > 0) || !starts || !counts) return LANCET_ERR_NULL;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if (int r = check_dims(S_total, M, E, 0)) return r;
  if (n_partitions < 1 || top_k * n_partitions > LANCET_MAX_PARTITIONS || S_total % n_partitions != 0)
    return LANCET_ERR_PARTITION;
  if (!workspace || workspace_bytes < lancet_moe_partition_ranges_workspace_bytes(top_k, n_partitions, E))
    return LANCET_ERR_WORKSPACE;
  if (misaligned(indices_locations, 4) || misaligned(starts, 8) || misaligned(counts, 8) || misaligned(workspace, 4))
    return LANCET_ERR_ALIGN;
  const int Q = top_k * n_partitions;
  const int64_t Sp = S_total / n_partitions;
  PtrTable t;
  for (int q = 0; q < kMaxPartitions; ++q) t.p[q] = nullptr;
  for (int j = 0; j < top_k; ++j)
    for (int p = 0; p < n_partitions; ++p) t.p[j * n_partitions + p] = indices_locations + j * S_total + p * Sp;
  uint32_t* hist = static_cast<uint32_t*>(workspace);
  hipError_t e = run_count_experts(t, Q, static_cast<int>(Sp), static_cast<int>(E), hist, S_(stream));
  if (e != hipSuccess) return rc(e);
  partition_ranges_kernel<<<static_cast<unsigned>((E + 255) / 256), 256, 0, S_(stream)>>>(hist, Q, static_cast<int>(E), M,
                                                                                         starts, counts);
  return rc(hipGetLastError());
}

// ---- backward ops -------------------------------------------------------------------
extern "C" int lancet_moe_encode_dx(const void* dy, const int32_t* indices_locations, int64_t S, int64_t M,
                                    int64_t E, int64_t C, int top_k, int dtype, void* dx, lancet_stream_t stream) {
  if ((!dy && C > 0 && M > 0) || (!indices_locations && S > 0) || (!dx && S > 0 && M > 0)) return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, M, E, C)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if (misaligned(dy, eb) || misaligned(dx, eb) || misaligned(indices_locations, 4)) return LANCET_ERR_ALIGN;
  const int s = static_cast<int>(S);
  return rc(run_decode_rows(dy, nullptr, LANCET_F32, indices_locations, indices_locations + static_cast<size_t>(top_k) * s, dx, s,
                            static_cast<int>(M), static_cast<int>(E), static_cast<int>(C), top_k, dtype, S_(stream)));
}

extern "C" int lancet_moe_encode_dg(const void* dy_gates_s, const int32_t* indices_locations, int64_t S, int64_t E,
                                    int top_k, int gate_dtype, void* grad_gates, lancet_stream_t stream) {
  if (S > 0 && (!dy_gates_s || !indices_locations || !grad_gates)) return LANCET_ERR_NULL;
  const int gb = elem_bytes(gate_dtype);
  if (!gb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, 0, E, 0)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if (misaligned(dy_gates_s, gb) || misaligned(indices_locations, 4) || misaligned(grad_gates, gb)) return LANCET_ERR_ALIGN;
  // top-1: the kernel of lancet_moe_encode_dgate in its plainest form (same result; it writes the block of a
  // workgroup's tokens in memory order, which streams several times faster on wide gates)
  if (top_k == 1 && S * E <= 0x7fffffff)
    return rc(run_encode_dgate(dy_gates_s, nullptr, indices_locations, static_cast<int>(S), static_cast<int>(E), 1, false,
                               gate_dtype, grad_gates, S_(stream)));
  return rc(run_encode_dg(dy_gates_s, indices_locations, static_cast<int>(S), static_cast<int>(E), top_k, gate_dtype, grad_gates,
                          S_(stream)));
}

extern "C" int lancet_moe_encode_dgate(const void* dy_gates_s, const void* gate, const int32_t* indices_locations,
                                       int64_t S, int64_t E, int top_k, int gate_dtype, unsigned flags, void* grad_gate,
                                       lancet_stream_t stream) {
  const bool is_logits = (flags & LANCET_GATE_IS_LOGITS) != 0;
  const bool needs_gate = top_k == 2 || is_logits;
  if (S > 0 && (!dy_gates_s || !indices_locations || !grad_gate || (needs_gate && !gate))) return LANCET_ERR_NULL;
  const int gb = elem_bytes(gate_dtype);
  if (!gb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, 0, E, 0)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if (top_k == 2 && E < 2) return LANCET_ERR_TOPK;
  if (S * E > 0x7fffffff) return LANCET_ERR_SHAPE;  // a tile's elements are indexed with 32 bits above its base
  if (misaligned(dy_gates_s, gb) || misaligned(gate, gb) || misaligned(indices_locations, 4) || misaligned(grad_gate, gb))
    return LANCET_ERR_ALIGN;
  return rc(run_encode_dgate(dy_gates_s, gate, indices_locations, static_cast<int>(S), static_cast<int>(E), top_k,
                             is_logits, gate_dtype, grad_gate, S_(stream)));
}

extern "C" size_t lancet_moe_decode_dx_workspace_bytes(int64_t E, int64_t C) {
  if (E < 1 || C < 0) return 0;
  return static_cast<size_t>(E) * static_cast<size_t>(C) * sizeof(int32_t);
}

extern "C" int lancet_moe_decode_dx(const void* dy, const void* gates_s, const int32_t* indices_locations, int64_t S,
                                    int64_t M, int64_t E, int64_t C, int top_k, int dtype, int gate_dtype, void* grad_expert_out,
                                    void* workspace, size_t workspace_bytes, lancet_stream_t stream) {
  if (((!dy && M > 0) || !gates_s || !indices_locations) && S > 0) return LANCET_ERR_NULL;
  if (!grad_expert_out && C > 0 && M > 0) return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, M, E, C)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  if (C > 0 && (!workspace || workspace_bytes < lancet_moe_decode_dx_workspace_bytes(E, C))) return LANCET_ERR_WORKSPACE;
  const int gb = elem_bytes(gate_dtype);
  if (!gb) return LANCET_ERR_DTYPE;
  if (misaligned(dy, eb) || misaligned(grad_expert_out, eb) || misaligned(gates_s, gb) ||
      misaligned(indices_locations, 4) || misaligned(workspace, 4))
    return LANCET_ERR_ALIGN;
  const int s = static_cast<int>(S);
  return rc(run_decode_dx(dy, gates_s, gate_dtype, indices_locations, indices_locations + static_cast<size_t>(top_k) * s,
                          grad_expert_out, static_cast<int32_t*>(workspace), s, static_cast<int>(M),
                          static_cast<int>(E), static_cast<int>(C), top_k, dtype, S_(stream)));
}

extern "C" int lancet_moe_decode_dg(const void* dy, const void* expert_out, const int32_t* indices_locations, int64_t S,
                                    int64_t M, int64_t E, int64_t C, int top_k, int dtype, int gate_dtype, void* grad_gates_s,
                                    lancet_stream_t stream) {
  if (S > 0 && (!indices_locations || !grad_gates_s || ((!dy || !expert_out) && M > 0))) return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (int r = check_dims(S, M, E, C)) return r;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  const int gb = elem_bytes(gate_dtype);
  if (!gb) return LANCET_ERR_DTYPE;
  if (misaligned(dy, eb) || misaligned(expert_out, eb) || misaligned(grad_gates_s, gb) || misaligned(indices_locations, 4))
    return LANCET_ERR_ALIGN;
  const int s = static_cast<int>(S);
  return rc(run_decode_dg(dy, expert_out, indices_locations, indices_locations + static_cast<size_t>(top_k) * s,
                          grad_gates_s, gate_dtype, s, static_cast<int>(M), static_cast<int>(E), static_cast<int>(C), top_k, dtype,
                          S_(stream)));
}

extern "C" int lancet_moe_top2_normalize_gates(const void* raw_gates, const int32_t* merged_indices, int64_t S,
                                               int gate_dtype, void* gates_out, lancet_stream_t stream) {
  if (S < 0 || S > 0x3fffffff) return LANCET_ERR_SHAPE;
  if (S == 0) return LANCET_OK;
  if (!raw_gates || !merged_indices || !gates_out) return LANCET_ERR_NULL;
  const int gb = elem_bytes(gate_dtype);
  if (!gb) return LANCET_ERR_DTYPE;
  if (misaligned(raw_gates, gb) || misaligned(merged_indices, 4) || misaligned(gates_out, gb)) return LANCET_ERR_ALIGN;
  return rc(run_top2_normalize(raw_gates, merged_indices, static_cast<int>(S), gate_dtype, gates_out, S_(stream)));
}

// ---- raf.op.moe_merge_masks / raf.op.moe_redispatch -------------------------------------

extern "C" size_t lancet_moe_merge_masks_workspace_bytes(int P, int64_t E) {
  if (P < 1 || E < 1) return 0;
  return static_cast<size_t>(P) * E * sizeof(uint32_t);
}

extern "C" int lancet_moe_merge_masks(const int32_t* const* indices_locations, int P, int64_t S, int64_t E,
                                      int32_t* out, void* workspace, size_t workspace_bytes,
                                      lancet_stream_t stream) {
  if (!indices_locations || (!out && S > 0)) return LANCET_ERR_NULL;
  if (P < 1 || P > LANCET_MAX_PARTITIONS) return LANCET_ERR_PARTITION;
  if (int r = check_dims(S, 0, E, 0)) return r;
  if (static_cast<int64_t>(P) * S > 0x3fffffff) return LANCET_ERR_SHAPE;
  if (!workspace || workspace_bytes < lancet_moe_merge_masks_workspace_bytes(P, E)) return LANCET_ERR_WORKSPACE;
  if (misaligned(out, 4) || misaligned(workspace, 4)) return LANCET_ERR_ALIGN;
  PtrTable t;
  if (int r = fill_table(t, reinterpret_cast<const void* const*>(indices_locations), P, 4)) return r;
  uint32_t* counts = static_cast<uint32_t*>(workspace);
  hipError_t e = run_count_experts(t, P, static_cast<int>(S), static_cast<int>(E), counts, S_(stream));
  if (e != hipSuccess) return rc(e);
  return rc(run_merge_masks(t, P, static_cast<int>(S), static_cast<int>(E), counts, out, S_(stream)));
}

extern "C" size_t lancet_moe_redispatch_workspace_bytes(int P, int64_t E) {
  return lancet_moe_merge_masks_workspace_bytes(P, E);
}

extern "C" int lancet_moe_redispatch(const void* const* data, const int32_t* const* indices_locations, int P,
                                     int64_t S, int64_t M, int64_t C, int64_t E, int dtype, void* out,
                                     void* workspace, size_t workspace_bytes, lancet_stream_t stream) {
  if (!data || !indices_locations || (!out && C > 0 && M > 0)) return LANCET_ERR_NULL;
  const int eb = elem_bytes(dtype);
  if (!eb) return LANCET_ERR_DTYPE;
  if (P < 1 || P > LANCET_MAX_PARTITIONS) return LANCET_ERR_PARTITION;
  if (int r = check_dims(S, M, E, C)) return r;
  if (!workspace || workspace_bytes < lancet_moe_redispatch_workspace_bytes(P, E)) return LANCET_ERR_WORKSPACE;
  if (misaligned(out, eb) || misaligned(workspace, 4)) return LANCET_ERR_ALIGN;
  PtrTable masks, bufs;
  if (int r = fill_table(masks, reinterpret_cast<const void* const*>(indices_locations), P, 4)) return r;
  if (int r = fill_table(bufs, data, P, eb)) return r;
  uint32_t* counts = static_cast<uint32_t*>(workspace);
  hipError_t e = run_count_experts(masks, P, static_cast<int>(S), static_cast<int>(E), counts, S_(stream));
  if (e != hipSuccess) return rc(e);
  return rc(run_redispatch_rows(bufs, P, static_cast<int>(M), static_cast<int>(C), static_cast<int>(E), counts, out,
                                eb, S_(stream)));
}
