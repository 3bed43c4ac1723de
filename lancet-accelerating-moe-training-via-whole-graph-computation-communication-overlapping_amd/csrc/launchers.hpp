// Host-side launch functions of the kernels; the C ABI (capi.hip) validates arguments and
// calls these.  All sizes have been checked by the caller: S, M, E, C fit in int32,
// E <= LANCET_MAX_EXPERTS, pointers are non-null where required.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace lancet {

constexpr int kMaxPartitions = 64;

// ---- routing (moe_route.hip) ------------------------------------------------------
int64_t scan_num_tiles(int64_t S);
size_t scan_workspace_bytes(int64_t S, int64_t E, int nsets);
size_t bpr_workspace_bytes(int64_t S0, int64_t S, int64_t E);
// one-time set-up of a scan workspace; its bound for waits; its sticky error word, read and cleared
hipError_t run_scan_ws_init(void* ws, size_t nbytes, hipStream_t st);
hipError_t run_scan_ws_set_spin(void* ws, uint32_t limit, hipStream_t st);
hipError_t run_scan_ws_set_epoch(void* ws, uint32_t epoch, hipStream_t st);
hipError_t run_scan_ws_take_error(void* ws, int* error_out, hipStream_t st);

hipError_t run_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t st);
// noise (top-2 only, may be null): [S,E] values added to the row for the second choice
// gate_dtype (LANCET_F32 / _BF16 / _F16): storage type of gate, noise, val / gates_s
hipError_t run_gate_topk(const void* gate, const void* noise, int S, int E, int K, bool is_logits, int gate_dtype,
                         int32_t* idx, void* val, hipStream_t st);
// gate-driven (idx_in == nullptr) or index-driven (gate == nullptr, K == 1) routing + scan.
// idx_out/loc_out are [K*S] each.
hipError_t run_route_scan(const void* gate, const void* noise, const int32_t* idx_in, const int32_t* used_in, int S,
                          int E, int C, int M, int K, bool is_logits, int gate_dtype, void* gates_s,
                          int32_t* idx_out, int32_t* loc_out, int32_t* used_out,
                          uint64_t* elems_out, void* ws, hipStream_t st, bool force_lookback = false);
// between count and place on long batches: sums of the table's rows in segments of R tiles (scan.hpp)
hipError_t run_scan_segsum(void* ws, int ntiles, int NC, int R, hipStream_t st);
hipError_t run_bpr_route(const void* gate, int S0, int E, int C, int M, int n_partitions,
                         int partition_id, bool is_logits, int gate_dtype, void* gates_s, int32_t* idx_out,
                         int32_t* loc_out, int32_t* used_out, uint64_t* elems_out, void* ws,
                         hipStream_t st, bool force_lookback = false);
hipError_t run_top2_normalize(const void* raw, const int32_t* idx, int S, int gate_dtype, void* out, hipStream_t st);

// ---- row movers (moe_rows.hip) ------------------------------------------------------
// Scatter of token rows into [E,C,M].  avail_used (may be null): only rows with
// loc < C - avail_used[idx] are written (the reference's capused test).  row_base (may be null):
// location l of expert e goes to row row_base[e] + l instead of row l.  When rows_hi is
// non-null the launch also zero-fills rows [rows_hi[e] - rows_lo[e], C) of every expert
// (rows_lo may be null = zeros); otherwise the caller has cleared the buffer.  slot_stride: distance
// between the K slots of one token in idx / loc (and gates, for decode); negative = S.  A call that
// moves a token range of a larger mask passes pointers to the range's first token and the mask's
// token count here.  dest (may be null; rows of whole 16-byte granules only): [K*S] destination rows e * C + location,
// -1 for none, ONE routing word per slot; idx, loc, avail_used and row_base are then not read.
hipError_t run_scatter_rows(const void* data, void* out, const int32_t* idx, const int32_t* loc,
                            const int32_t* avail_used, const int32_t* row_base, const int32_t* rows_lo,
                            const int32_t* rows_hi,
                            int S, int M, int E, int C, int K, int elem_bytes, hipStream_t st, int slot_stride = -1,
                            const int32_t* dest = nullptr);
hipError_t run_zero_bytes(void* p, size_t nbytes, hipStream_t st);
hipError_t run_decode_rows(const void* expert_out, const void* gates, int gate_dtype, const int32_t* idx,
                           const int32_t* loc, void* out, int S, int M, int E, int C, int K,
                           int dtype, hipStream_t st, int slot_stride = -1, const int32_t* dest = nullptr);

// backward (gates == nullptr in run_decode_rows gives moe_encode_dx)
hipError_t run_encode_dg(const void* dy, const int32_t* idx, int S, int E, int K, int gate_dtype, void* grad_gates, hipStream_t st);
// moe_gate_grad.hip: gradient of gates_s [K*S] back to the [S,E] gate through the top-2 normalisation and, with
// is_logits, the fused softmax; gate may be null for K == 1 on probabilities
hipError_t run_encode_dgate(const void* dy, const void* gate, const int32_t* idx, int S, int E, int K, bool is_logits,
                            int gate_dtype, void* out, hipStream_t st);
hipError_t run_decode_dx(const void* dy, const void* gates, int gate_dtype, const int32_t* idx, const int32_t* loc, void* out,
                         int32_t* src_map, int S, int M, int E, int C, int K, int dtype, hipStream_t st);
hipError_t run_decode_dg(const void* dy, const void* expert_out, const int32_t* idx, const int32_t* loc, void* out,
                         int gate_dtype, int S, int M, int E, int C, int K, int dtype, hipStream_t st);

struct PtrTable {
  const void* p[kMaxPartitions];
};
// counts[P][E] (zeroed by the call) = number of tokens of partition p whose index is e
hipError_t run_count_experts(const PtrTable& indlocs, int P, int S, int E, uint32_t* counts, hipStream_t st);
hipError_t run_merge_masks(const PtrTable& indlocs, int P, int S, int E, const uint32_t* counts,
                           int32_t* out, hipStream_t st);
hipError_t run_redispatch_rows(const PtrTable& bufs, int P, int M, int C, int E, const uint32_t* counts,
                               void* out, int elem_bytes, hipStream_t st);

// merge of P partitions of one local expert's all-to-all output, layout [C, G, M]; cnt_ptrs are P device
// arrays of uint64 [G*LE]
hipError_t run_redispatch_expert_input(const PtrTable& bufs, const void* const* cnt_ptrs, int P, int le, int LE, int C,
                                       int M, int G, uint64_t scale, void* out, int elem_bytes, hipStream_t st);

// ---- sparse <-> packed copies (sparse_copy.hip) -----------------------------------------
// counts[b*stride + offset] elements of block b along `axis` (0 or 1) of a [dim0, dim1, dim2] buffer;
// cont_cap = elements the packed stream holds.  to_cont: buffer -> stream.  starts (may be null = zeros): first
// element of block b that takes part, read like the counts.
hipError_t run_sparse_copy_3d(const void* src, void* dst, const uint64_t* counts, const uint64_t* starts, int stride, int offset, int axis,
                              int dim0, int dim1, int dim2, uint64_t cont_cap, uint64_t scale, uint64_t shrink,
                              bool to_cont, bool zero_tail, int elem_bytes, hipStream_t st);

}  // namespace lancet
