/*
 * lancet_hip.h - C ABI of the MI355X (gfx950) implementation of one GPU's share of
 * the MoE token-dispatch path and the fused LANS step.
 *
 * Every entry point replaces one piece of the reference's native launcher surface
 * (src/op/dialect/cuda/kernels/kernel_util.cuh:25-79) or of the OpEnv that drives it
 * (src/op/dialect/cuda/moe.cc, src/op/dialect/cuda/lans.cc); the citation on each
 * declaration names the piece.  Conventions:
 *
 *   - plain pointers and sizes only; all data pointers are DEVICE pointers unless a
 *     parameter is documented as a host array;
 *   - every call takes the HIP stream to launch on (a hipStream_t passed as void*;
 *     NULL = the default stream), is asynchronous with respect to the host and
 *     allocates nothing (the two lans_plan calls excepted, which own small tables);
 *   - outputs and workspaces are caller-owned; *_workspace_bytes() sizes the
 *     workspace.  Plain workspaces need no initialisation and are not preserved.  The
 *     workspaces of the position scan (lancet_launch_gen_location, lancet_moe_encode,
 *     lancet_moe_route, lancet_moe_encode_bpr) carry a few words of state from call to
 *     call: set each up ONCE with lancet_scan_workspace_init after allocating it, let
 *     nothing else write to it, and use it for one call at a time;
 *   - the return value is a status: 0 = ok, < 0 = rejected argument (nothing was
 *     launched), > 0 = a hipError_t from the runtime.  Nothing aborts the process
 *     (the reference CHECK/LOG(FATAL)s, src/common/cuda_utils.h:18-22).
 *
 * Token rows are `dtype` (LANCET_F32 / LANCET_BF16 / LANCET_F16).  Gate arrays (gate and
 * gate2_noise [S,E], gates_s [top_k*S], their gradients) are `gate_dtype`, one of the same three
 * codes: the reference's kernels take the gate in the data type (`__dtype* gates1_s`,
 * tutel_moe_dispatch.cu:110-116,126-157) and mixed-precision graphs feed a half gate
 * (python/raf/amp/type_hints.py:97,105).  All arithmetic on gate values is fp32, with one rounding
 * to gate_dtype where a value is stored; 16-bit gates tie often, and selection keeps its rule (first
 * maximum wins).  LANS parameters and moments are fp32 (gradients may be 16-bit: lancet_lans_step_mixed);
 * indices/locations/used capacity are int32 and elements_per_expert is uint64, as in
 * src/op/declare/moe.cc:48-58.
 */
#ifndef LANCET_HIP_H_
#define LANCET_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LANCET_ABI_VERSION 8

/* element type of token rows (dtype) and of gate arrays (gate_dtype) */
#define LANCET_F32 0
#define LANCET_BF16 1
#define LANCET_F16 2

/* status codes (negative = argument rejected, nothing launched) */
#define LANCET_OK 0
#define LANCET_ERR_NULL (-1)      /* a required pointer is NULL */
#define LANCET_ERR_SHAPE (-2)     /* a size is negative, zero where not allowed, or above a limit */
#define LANCET_ERR_DTYPE (-3)     /* unknown dtype code */
#define LANCET_ERR_WORKSPACE (-4) /* workspace missing or too small */
#define LANCET_ERR_ALIGN (-5)     /* a pointer is not aligned to its element type */
#define LANCET_ERR_TOPK (-6)      /* top_k not 1 or 2, or top_k = 2 with fewer than 2 experts */
#define LANCET_ERR_PARTITION (-7) /* bad n_partitions / partition_id */
#define LANCET_ERR_PLAN (-8)      /* invalid LANS plan handle, or a plan of another device than the current one */
#define LANCET_ERR_SCRATCH (-9)   /* lancet_moe_encode_noalloc: the sizes need more than LANCET_NOALLOC_SCRATCH_BYTES */
#define LANCET_ERR_STALLED (-10)  /* lancet_lans_step: an earlier step of the plan gave up a wait; call lancet_lans_plan_error */

/* limits */
#define LANCET_MAX_EXPERTS 512
#define LANCET_MAX_PARTITIONS 64

/* flags of lancet_moe_encode / lancet_moe_encode_bpr / lancet_gate_topk */
#define LANCET_GATE_IS_LOGITS 1u /* `gate` holds logits: select on them, gates_s = softmax prob */
/* lancet_moe_encode / lancet_moe_encode_bpr / lancet_moe_scatter: leave the rows past the used
 * capacity unwritten instead of zero-filling them.  For partition buffers that only feed
 * moe_redispatch (which reads the used rows and zero-fills the merged tail itself); it is what the
 * reference's own cost for this pattern, a full memset per partition buffer
 * (tutel_moe_dispatch.cu:466), is spent on. */
#define LANCET_NO_TAIL_ZERO 2u
#define LANCET_ZERO_TAIL 4u /* lancet_memcpy_cont_to_sparse_3d: clear what the copy leaves untouched */
/* lancet_moe_encode / lancet_moe_scatter: write the rows of expert e from row used_in[e] on instead of
 * row 0, i.e. behind the rows that the calls chained before this one (through used_capacity) wrote into
 * the same buffer; the zero-fill, if any, then covers rows [used_out[e], C).  Chained partition encodes
 * that share one buffer this way leave it as moe_redispatch would build it from separate buffers
 * (reference: redispatch_kernel, tutel_moe_dispatch.cu:365-408), without that second pass over the rows.
 * indices_locations are unchanged (locations stay relative to the call, as moe_merge_masks expects). */
#define LANCET_ROWS_AT_USED 8u
/* lancet_moe_encode / lancet_moe_route / lancet_moe_encode_bpr: run the position scan as ONE kernel with a
 * decoupled look-back between its tiles, whatever the size.  By default only top-1 calls of at most 8192 tokens
 * do; everything else is faster as two or three kernels in which no workgroup waits for another.  For callers
 * that want the fewest launches, and for tests of the look-back's bounded waits. */
#define LANCET_SCAN_LOOKBACK 16u

typedef void* lancet_stream_t;

int lancet_abi_version(void);
const char* lancet_status_string(int status);

/* Capacity C = int(float(cf) * ((S + E - 1) / E)); -1 for E <= 0, S < 0 or a product that no int holds.
 * Replaces: src/op/dialect/cuda/moe.cc:107-109, src/op/declare/moe.cc:46, src/op/ty/moe.cc:50. */
int64_t lancet_moe_capacity(int64_t S, int64_t E, float capacity_factor);

/* ---- routing front end -------------------------------------------------------------
 * idx[j*S + s], val[j*S + s] for j < top_k: first-max expert of row s of gate[S,E] (slot 2:
 * with slot 1's expert masked), and gate[s, idx] or its softmax probability.
 * Replaces: the three TVM-compiled micro-kernels argmax / one_hot / multiply+sum that
 * MoeEncode runs first (src/op/dialect/cuda/moe.cc:177-250, executed :366-371) and, with
 * LANCET_GATE_IS_LOGITS, the softmax in front of the op (models/benchmark/pytorch/utils.py:565-573).
 * gate2_noise (top_k = 2 only, may be NULL): [S,E] values added to `gate` for the second choice alone,
 * the first choice masked out - the Gumbel noise of docker/resources/sharded_moe.py:275-278, drawn by
 * the caller; val is always read from `gate` itself. */
int lancet_gate_topk(const void* gate, const void* gate2_noise, int64_t S, int64_t E, int top_k,
                     int gate_dtype, unsigned flags, int32_t* idx, void* val, lancet_stream_t stream);

/* ---- launcher level ----------------------------------------------------------------
 * Replaces launch_gen_location (kernel_util.cuh:60; tutel_moe_dispatch.cu:164-212,548-553).
 * indices[S] is mutated (dropped tokens -> -1); locations[S] receives the rank of every token
 * among the tokens of its expert. */
size_t lancet_gen_location_workspace_bytes(int64_t S, int64_t E);
int lancet_launch_gen_location(int32_t* indices, const int32_t* in_capused, int32_t* locations,
                               int32_t* out_capused, uint64_t* out_elements_per_expert,
                               int64_t C, int64_t S, int64_t E, int64_t M,
                               void* workspace, size_t workspace_bytes, lancet_stream_t stream);

/* Replaces both launch_encode_forward overloads (kernel_util.cuh:37-40;
 * tutel_moe_dispatch.cu:61-81,461-484): capused == NULL is the "_wo_usedcap" overload.
 * Every byte of dispatched[E,C,M] is written exactly once (rows that receive no token are
 * zero-filled by the same launch; there is no memset + atomicAdd). */
int lancet_launch_encode_forward(const int32_t* indices, const int32_t* locations,
                                 const int32_t* capused, const void* data, void* dispatched,
                                 int64_t S, int64_t M, int64_t C, int64_t E, int dtype,
                                 lancet_stream_t stream);

/* ---- raf.op.moe_encode -------------------------------------------------------------
 * Replaces MoeEncode::Execute (src/op/dialect/cuda/moe.cc:346-396); outputs are the 5-tuple of
 * src/op/declare/moe.cc:48-58.  top_k = 2 is an extension with GShard semantics
 * (docker/resources/sharded_moe.py:253-324, no noise): outputs are slot-major
 * (gates_s[2S], indices_locations[2, 2S]) in the layout moe_merge_masks produces for the two
 * chained top-1 encodes it is equivalent to, and gates_s holds the normalised combine weights.
 * used_in may be NULL (= zeros); gate2_noise as in lancet_gate_topk, NULL = none.  With a 16-bit
 * gate_dtype and top_k = 2 the two raw gate values are rounded to gate_dtype, as a gates_s array of that
 * type holds them, before the combine weights are formed from them in fp32. */
size_t lancet_moe_encode_workspace_bytes(int64_t S, int64_t E, int top_k);
int lancet_moe_encode(const void* data, const void* gate, const void* gate2_noise, const int32_t* used_in,
                      int64_t S, int64_t M, int64_t E, int64_t C, int top_k, int dtype, int gate_dtype,
                      unsigned flags, void* gates_s, int32_t* indices_locations,
                      int32_t* used_out, uint64_t* elements_per_expert, void* dispatched,
                      void* workspace, size_t workspace_bytes, lancet_stream_t stream);

/* lancet_moe_encode without the workspace argument, for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  (No counterpart in the
 * reference, whose executor allocates a workspace before every Execute, src/impl/vm/vm.cc:1260-1266.)
 * The scan's workspace (ticket, error word, descriptor table) lives in a static device array of
 * LANCET_NOALLOC_SCRATCH_BYTES that each GPU holds until the process ends; sizes whose
 * lancet_moe_encode_workspace_bytes(S, E, top_k) exceeds it are rejected with LANCET_ERR_SCRATCH
 * (it covers S * top_k * E <= 67 million, e.g. S = 65536, E = 512, top_k = 2).  The call allocates
 * nothing and launches the same kernels as lancet_moe_encode, with identical results.  All calls on one
 * GPU share the array: calls that overlap on one GPU race, so issue them on one stream or order them
 * yourself.  The first call on a device looks the array's address up, sets the workspace up (one small
 * launch on `stream`, no allocation) and waits for `stream`; make that call once before recording a graph. */
#define LANCET_NOALLOC_SCRATCH_BYTES ((2u << 20) + 4096u)
int lancet_moe_encode_noalloc(const void* data, const void* gate, const void* gate2_noise,
                              const int32_t* used_in, int64_t S, int64_t M, int64_t E, int64_t C, int top_k,
                              int dtype, int gate_dtype, unsigned flags, void* gates_s, int32_t* indices_locations,
                              int32_t* used_out, uint64_t* elements_per_expert, void* dispatched,
                              lancet_stream_t stream);

/* The two phases of lancet_moe_encode as separate calls, for callers that overlap the routing of
 * one token partition with the row movement of another (Lancet's forward pipelining,
 * src/pass/dist_optimization/partition_exprs.cc:1709-1795):
 *   lancet_moe_route   = selection + position scan (everything of MoeEncode::Execute up to and
 *                        including launch_gen_location, moe.cc:366-380); outputs as above
 *                        except the buffer;
 *   lancet_moe_scatter = launch_encode_forward (moe.cc:381-395) on routing produced by
 *                        lancet_moe_route; zero-fills the rows past used_out - used_in. */
int lancet_moe_route(const void* gate, const void* gate2_noise, const int32_t* used_in, int64_t S, int64_t M,
                     int64_t E, int64_t C, int top_k, int gate_dtype, unsigned flags, void* gates_s,
                     int32_t* indices_locations, int32_t* used_out, uint64_t* elements_per_expert,
                     void* workspace, size_t workspace_bytes, lancet_stream_t stream);
int lancet_moe_scatter(const void* data, const int32_t* indices_locations, const int32_t* used_in,
                       const int32_t* used_out, int64_t S, int64_t M, int64_t E, int64_t C, int top_k,
                       int dtype, unsigned flags, void* dispatched, lancet_stream_t stream);

/* ---- raf.op.moe_encode_batch_prioritized --------------------------------------------
 * Replaces MoeEncodeBatchPrioritized::Execute (moe.cc:543-684), the TVM argsort it calls
 * (:701-719) and launch_gen_location_bpr (kernel_util.cuh:65; tutel_moe_dispatch.cu:259-363).
 * data[S0,M], gate[S0,E] are the whole batch; S = S0 / n_partitions tokens of partition
 * partition_id are encoded.  The per-expert keep set is the C best tokens by
 * (gate value descending, token index ascending), found with a radix select, not a sort.
 * The workspace holds, behind the scan's table, 16 bytes per token of the batch (first choice and priority; the
 * order keys of each tile of 256 tokens grouped by expert) and 8 bytes per (expert, tile of the batch). */
size_t lancet_moe_encode_bpr_workspace_bytes(int64_t S0, int64_t E, int n_partitions);
int lancet_moe_encode_bpr(const void* data, const void* gate, int64_t S0, int64_t M, int64_t E,
                          int64_t C, int n_partitions, int partition_id, int dtype, int gate_dtype, unsigned flags,
                          void* gates_s, int32_t* indices_locations, int32_t* used_out,
                          uint64_t* elements_per_expert, void* dispatched,
                          void* workspace, size_t workspace_bytes, lancet_stream_t stream);

/* ---- raf.op.moe_decode -------------------------------------------------------------
 * Replaces MoeDecode::Execute / launch_decode_forward (moe.cc:1262-1291; kernel_util.cuh:45;
 * tutel_moe_dispatch.cu:46-55,110-116,511-521).  top_k = 2 sums the two slots of the
 * slot-major layout in fp32 and rounds once. */
int lancet_moe_decode(const void* expert_out, const void* gates_s,
                      const int32_t* indices_locations, int64_t S, int64_t M, int64_t E,
                      int64_t C, int top_k, int dtype, int gate_dtype, void* out, lancet_stream_t stream);

/* ---- token ranges of a whole-batch mask -------------------------------------------------
 * The partition pass cuts the token batch so that the exchange of one partition overlaps the work on
 * another (src/pass/dist_optimization/partition_exprs.cc:1709-1795) and chains the partitions' encodes
 * through used_capacity; the chained encodes, merged by moe_merge_masks, are by construction the routing
 * of the whole batch (tests/python/op/cuda/test_cuda_moe.py:384-471).  Routing only needs the [S, E] gate,
 * so a caller that has the gate of the whole batch routes once (lancet_moe_route, S = S_total) and then
 * moves rows partition by partition with these two calls: tokens [token_first, token_first + n_tokens)
 * of the whole-batch indices_locations [2, top_k * S_total] (and gates_s [top_k * S_total]).  data and
 * out hold the rows of those tokens only ([n_tokens, M]); dispatched / expert_out is the whole [E, C, M]
 * buffer, rows at their final places, so no moe_merge_masks / moe_redispatch pass is needed and each
 * token row is read once also for top_k = 2.  lancet_moe_scatter_tokens zero-fills the rows
 * past used_out - used_in (used_in, used_out as given to and returned by the routing call; used_in NULL =
 * zeros) unless LANCET_NO_TAIL_ZERO is set: one call of the sequence should do it; both may be NULL with
 * that flag.  The partitions' scatters together give bit for bit the buffer of one
 * lancet_moe_encode over the batch. */
int lancet_moe_scatter_tokens(const void* data, const int32_t* indices_locations, const int32_t* used_in,
                              const int32_t* used_out, int64_t S_total, int64_t token_first, int64_t n_tokens, int64_t M, int64_t E,
                              int64_t C, int top_k, int dtype, unsigned flags, void* dispatched,
                              lancet_stream_t stream);
int lancet_moe_decode_tokens(const void* expert_out, const void* gates_s, const int32_t* indices_locations,
                             int64_t S_total, int64_t token_first, int64_t n_tokens, int64_t M, int64_t E,
                             int64_t C, int top_k, int dtype, int gate_dtype, void* out, lancet_stream_t stream);

/* ---- raf.op.moe_redispatch_expert_input ------------------------------------------------
 * Replaces MoeRedispatchExpertInput::Execute / launch_redispatch_expert_input (moe.cc:945-1073;
 * kernel_util.cuh:55; tutel_moe_dispatch.cu:436-456,586-598): merge, for one local expert, of the
 * all-to-all outputs of P token partitions.  data: HOST array of P device pointers to [C, G, M]
 * buffers (capacity row, source GPU, model dim); recv_cnts: HOST array of P device pointers to
 * uint64 [G * n_local_experts] received element counts (the elements_per_expert side channel of the
 * all-to-allv).  Rows of out[C, G, M] past the merged stream are zero. */
int lancet_moe_redispatch_expert_input(const void* const* data, const uint64_t* const* recv_cnts, int P,
                                       int local_expert_id, int n_local_experts, int64_t C, int64_t M,
                                       int64_t G, int recv_cnts_scale, int dtype, void* out,
                                       lancet_stream_t stream);

/* ---- sparse <-> packed copies ------------------------------------------------------------
 * Replace launch_memcpy_sparse_to_cont_3d / launch_memcpy_cont_to_sparse_3d (kernel_util.cuh:69-79;
 * sparse_memcpy.cu:11-96).  Block b along `axis` (0 or 1) of the [dim0, dim1, dim2] buffer holds
 * n_b = nelements_per_dim[b*stride + offset] * scale / shrink valid elements (in the block's own
 * row-major order: [dim1, dim2] for axis 0, [dim0, dim2] for axis 1); the packed side is their
 * concatenation.  n_counts = length of nelements_per_dim, dst_elems / src_elems = length of the packed
 * array (both bound what the kernels touch; the reference takes neither).  Counts that exceed a block
 * or the packed array are clipped.  cont_to_sparse leaves the rest of each block untouched, as the
 * reference does, unless flags has LANCET_ZERO_TAIL. */
int lancet_memcpy_sparse_to_cont_3d(const void* src, void* dst, const uint64_t* nelements_per_dim,
                                    int64_t n_counts, int nelements_stride, int nelements_offset, int axis,
                                    int64_t dim0, int64_t dim1, int64_t dim2, int64_t dst_elems,
                                    int scale_element_size_by, int shrink_element_size_by, int dtype,
                                    lancet_stream_t stream);
int lancet_memcpy_cont_to_sparse_3d(const void* src, void* dst, const uint64_t* nelements_per_dim,
                                    int64_t n_counts, int nelements_stride, int nelements_offset, int axis,
                                    int64_t dim0, int64_t dim1, int64_t dim2, int64_t src_elems,
                                    int scale_element_size_by, int shrink_element_size_by, int dtype,
                                    unsigned flags, lancet_stream_t stream);

/* The same copies on row ranges (no counterpart in the reference): block b's valid elements are
 * [starts_per_dim[b*stride + offset], + nelements_per_dim[b*stride + offset]) instead of the block's first ones.
 * For a buffer that several token partitions share (lancet_moe_scatter_tokens): what one partition owns is, per
 * expert, a run of rows behind those of the partitions before it, and these copies pack that run for the
 * partition's exchange and unpack what comes back.  Nothing outside the ranges is touched. */
int lancet_memcpy_sparse_ranges_to_cont_3d(const void* src, void* dst, const uint64_t* nelements_per_dim,
                                           const uint64_t* starts_per_dim, int64_t n_counts, int nelements_stride,
                                           int nelements_offset, int axis, int64_t dim0, int64_t dim1, int64_t dim2,
                                           int64_t dst_elems, int dtype, lancet_stream_t stream);
int lancet_memcpy_cont_to_sparse_ranges_3d(const void* src, void* dst, const uint64_t* nelements_per_dim,
                                           const uint64_t* starts_per_dim, int64_t n_counts, int nelements_stride,
                                           int nelements_offset, int axis, int64_t dim0, int64_t dim1, int64_t dim2,
                                           int64_t src_elems, int dtype, lancet_stream_t stream);
/* Row ranges of n_partitions equal token partitions inside a whole-batch routing (indices_locations
 * [2, top_k * S_total] of lancet_moe_route over all tokens): starts and counts are [top_k * n_partitions, E]
 * uint64 in ELEMENTS (rows x M), rows ordered slot-major, then partition, which is the order in which the rows
 * follow each other inside every expert (the capacity order moe_merge_masks uses, moe.cc:772-802).
 * counts[j*P + p][e] = M x kept tokens of partition p whose slot j went to expert e; starts = the sum of the counts
 * before it.  counts rows are what elements_per_expert would be for the partition's own encode. */
size_t lancet_moe_partition_ranges_workspace_bytes(int top_k, int n_partitions, int64_t E);
int lancet_moe_partition_ranges(const int32_t* indices_locations, int64_t S_total, int top_k, int n_partitions,
                                int64_t E, int64_t M, uint64_t* starts, uint64_t* counts, void* workspace,
                                size_t workspace_bytes, lancet_stream_t stream);

/* ---- backward ops (raf.op.moe_encode_dx / _dg, raf.op.moe_decode_dx / _dg) ------------------
 * Gradients wired by src/op/grad/moe.cc:30-93.  Gate-side gradients are gate_dtype like gates_s; top_k = 2
 * takes the slot-major layout of the forward ops.
 *
 * moe_encode_dx: dx[s,:] = sum over slots of dy[idx, loc, :] (0 for dropped slots).  Replaces
 * MoeEncodeDx / launch_encode_backward_data (moe.cc:1075-1153; kernel_util.cuh:41;
 * tutel_moe_dispatch.cu:88-94,486-497). */
int lancet_moe_encode_dx(const void* dy, const int32_t* indices_locations, int64_t S, int64_t M,
                         int64_t E, int64_t C, int top_k, int dtype, void* dx, lancet_stream_t stream);
/* moe_encode_dg: grad_gates[S,E] = 0 except grad_gates[s, idx] = dy_gates_s of that slot.  Replaces
 * MoeEncodeDg / launch_encode_backward_gate (moe.cc:1155-1225; kernel_util.cuh:43;
 * tutel_moe_dispatch.cu:96-105,499-506). */
int lancet_moe_encode_dg(const void* dy_gates_s, const int32_t* indices_locations, int64_t S,
                         int64_t E, int top_k, int gate_dtype, void* grad_gates, lancet_stream_t stream);
/* Gate gradient of moe_encode as a whole, for the forms of the op that do more to a gate value than select it:
 * grad_gate[S,E] = d loss / d gate given dy_gates_s = d loss / d gates_s (the op's OUTPUT, [top_k*S]), through
 *   - top_k = 2: the normalisation g_k / max(g_1 + g_2, eps) of the two kept values (docker/resources/sharded_moe.py:
 *     304-312): d g_1 = (dy_1 - dy_2) * g_2 / (g_1 + g_2)^2, d g_2 = (dy_2 - dy_1) * g_1 / (g_1 + g_2)^2; below eps the
 *     clamped denominator is a constant (d g_k = dy_k / eps); a dropped slot has g = 0 and gets no gradient, which
 *     leaves the other slot's weight at the constant 1;
 *   - LANCET_GATE_IS_LOGITS in flags: the softmax the op fused (sharded_moe.py:260): d x[e] = p[e] * (d p[e] - sum_j
 *     p[i_j] * d p[i_j]), p recomputed from `gate` (the logits) in fp32.
 * gate and indices_locations are the forward's input and output; second-choice noise (gate2_noise) only moved the
 * selection and needs no gradient.  With top_k = 1 and no flag the result is moe_encode_dg's (gate may then be NULL).
 * Extends MoeEncodeGrad (src/op/grad/moe.cc:30-58), which differentiates the op end to end for the one form the
 * reference has (top-1 on probabilities), to the top-2 / fused-softmax forms of lancet_moe_encode.  One pass: reads
 * and writes S*E gate elements. */
int lancet_moe_encode_dgate(const void* dy_gates_s, const void* gate, const int32_t* indices_locations, int64_t S,
                            int64_t E, int top_k, int gate_dtype, unsigned flags, void* grad_gate,
                            lancet_stream_t stream);
/* moe_decode_dx: grad_expert_out[idx, loc, :] = gates_s * dy[s, :], zero elsewhere.  Replaces
 * MoeDecodeDx / launch_decode_backward_data (moe.cc:1313-1395; kernel_util.cuh:47;
 * tutel_moe_dispatch.cu:118-124,523-533).  Workspace: an [E*C] int32 row -> token map. */
size_t lancet_moe_decode_dx_workspace_bytes(int64_t E, int64_t C);
int lancet_moe_decode_dx(const void* dy, const void* gates_s, const int32_t* indices_locations,
                         int64_t S, int64_t M, int64_t E, int64_t C, int top_k, int dtype, int gate_dtype,
                         void* grad_expert_out, void* workspace, size_t workspace_bytes,
                         lancet_stream_t stream);
/* moe_decode_dg: grad_gates_s[slot-token] = <expert_out[idx, loc, :], dy[s, :]>, 0 for dropped slots.
 * Replaces MoeDecodeDg / launch_decode_backward_gate (moe.cc:1397-1481; kernel_util.cuh:49;
 * tutel_moe_dispatch.cu:126-157,535-546). */
int lancet_moe_decode_dg(const void* dy, const void* expert_out, const int32_t* indices_locations,
                         int64_t S, int64_t M, int64_t E, int64_t C, int top_k, int dtype, int gate_dtype,
                         void* grad_gates_s, lancet_stream_t stream);

/* Combine weights of the top-2 extension from raw per-slot gate values and merged indices
 * (docker/resources/sharded_moe.py:304-312); in place when gates_out == raw_gates. */
int lancet_moe_top2_normalize_gates(const void* raw_gates, const int32_t* merged_indices,
                                    int64_t S, int gate_dtype, void* gates_out, lancet_stream_t stream);

/* ---- raf.op.moe_merge_masks --------------------------------------------------------
 * Replaces MoeMergeMasks::Execute / launch_merge_masks (moe.cc:772-802; kernel_util.cuh:62;
 * tutel_moe_dispatch.cu:214-255,555-563).  indices_locations is a HOST array of P device
 * pointers to [2,S] int32 tensors; out is [2, P*S]. */
size_t lancet_moe_merge_masks_workspace_bytes(int P, int64_t E);
int lancet_moe_merge_masks(const int32_t* const* indices_locations, int P, int64_t S, int64_t E,
                           int32_t* out, void* workspace, size_t workspace_bytes,
                           lancet_stream_t stream);

/* ---- raf.op.moe_redispatch ---------------------------------------------------------
 * Replaces MoeRedispatch::Execute / launch_redispatch (moe.cc:881-920; kernel_util.cuh:52;
 * tutel_moe_dispatch.cu:365-408,572-584).  data / indices_locations are HOST arrays of P
 * device pointers ([E,C,M] buffers and [2,S] masks).  Rows of out[E,C,M] past the merged
 * count are zero (the reference leaves them uninitialised). */
size_t lancet_moe_redispatch_workspace_bytes(int P, int64_t E);
int lancet_moe_redispatch(const void* const* data, const int32_t* const* indices_locations,
                          int P, int64_t S, int64_t M, int64_t C, int64_t E, int dtype,
                          void* out, void* workspace, size_t workspace_bytes,
                          lancet_stream_t stream);

/* ---- raf.op.lans -------------------------------------------------------------------
 * Replaces LansImpl (src/op/dialect/cuda/lans.cc:26-180) and multi_tensor_lans_cuda
 * (kernel_util.cuh:25-33; multi_tensor_lans.cu:401-450).  A plan captures the tensor sizes of
 * one parameter set (what the LansImpl constructor captures) and owns the chunk tables,
 * per-chunk partial sums and norm vectors; it is created once and reused every step (T >= 1; a tensor may be empty).
 * g/p/m/v are HOST arrays of T device pointers to fp32 tensors (the four quarters of the
 * reference's tensor_list).  p, m, v are updated in place; g is not modified.
 * step: pass step_host >= 1, or a device pointer step_dev to the fp32 step scalar the
 * reference passes (read on the device; no host synchronisation).
 * grad_norms: NULL, or a device array of T floats holding ||g_i||_2 in the order of the lists, for a caller
 * that already has them (per-tensor norms from gradient clipping): the step then skips its own pass over g
 * for them (the first l2norm sweep of multi_tensor_lans.cu:412-418).
 * A plan's steps share its partial sums and control words: issue them on one stream, or order
 * them yourself; two steps of one plan that overlap on the device race.  Plans are independent
 * of each other. */
typedef struct lancet_lans_plan* lancet_lans_plan_t;

typedef struct lancet_lans_hyper {
  float learning_rate;
  float beta1;
  float beta2;
  float eps;
  int bias_correction;
  float weight_decay;
  int grad_averaging;
  int mode;           /* 0 = L2 into the gradient, 1 = decoupled weight decay */
  int normalize_grad;
} lancet_lans_hyper;

int lancet_lans_plan_create(const int64_t* numels, int T, lancet_lans_plan_t* plan);
int lancet_lans_plan_destroy(lancet_lans_plan_t plan);
int lancet_lans_step(lancet_lans_plan_t plan, const float* const* g, float* const* p,
                     float* const* m, float* const* v, int step_host, const float* step_dev,
                     const lancet_lans_hyper* hyper, const float* grad_norms, lancet_stream_t stream);
/* The step of a mixed-precision trainer: fp32 master parameters and moments, a 16-bit model.  The reference's
 * traced optimizer casts every gradient to fp32 in front of the op and every new parameter back to the model type
 * behind it (python/raf/optim/lans.py:256-257, 285-288): two more passes over the state, 6 + 6 bytes per parameter on
 * top of the step's 28.  Here the step itself reads the gradients in g_dtype (LANCET_F32 / _BF16 / _F16; widened in
 * registers, which is exact, so every value of the step is what the cast would have given) and, when p_lowp is not
 * NULL, writes next to each new fp32 parameter its copy in lowp_dtype (LANCET_BF16 / _F16, round to nearest even:
 * the cast's result, bit for bit).  g and p_lowp are HOST arrays of T device pointers like the others; with
 * g_dtype = LANCET_F32 and p_lowp = NULL this is lancet_lans_step.  16-bit gradients and both 16-bit types in and
 * out: 2 + 24 + 2 = 28 bytes per parameter. */
int lancet_lans_step_mixed(lancet_lans_plan_t plan, const void* const* g, int g_dtype, float* const* p,
                           float* const* m, float* const* v, void* const* p_lowp, int lowp_dtype, int step_host,
                           const float* step_dev, const lancet_lans_hyper* hyper, const float* grad_norms,
                           lancet_stream_t stream);
/* A step may be recorded into a HIP graph (either schedule): with step_dev the step number is read on the
 * device, and everything else that changes from step to step lives in the plan's device memory, so each
 * replay is a new step.  The pointer tables are uploaded (one host-to-device copy) by the first call that
 * sees a new set of pointers: make that call once before recording. */
/* Schedules of the step.
 * LANCET_LANS_RESIDENT (what a new plan has when at least one tensor fits it): one persistent kernel that
 * reads and writes every array once (28 B/param).  Each workgroup runs a three-stage pipeline over chunks of
 * 8192 parameters (sum of g^2 / moments and the two updates / parameter write) and keeps a chunk on chip
 * between the stages; it publishes the sums of its chunks and forms the norms it needs from the published
 * sums of all the tensor's chunks.  The kernel takes the tensors that are whole multiples of 8192
 * parameters and have at most lancet_lans_plan_resident_capacity() chunks; the other tensors of the plan
 * take the three sweeps in the same step, and so does every tensor of a step in which an array of a tensor
 * the kernel would take is not 16-byte aligned.
 * Contract of this schedule: its workgroups wait for one another (for chunks of the same tensor only), so
 * at least half of them must be running on the device at the same time.  The grid is sized to what an
 * otherwise idle device runs at once; other kernels on the device delay the step until enough of its
 * workgroups have started, and only something that keeps the device occupied without end (e.g. another
 * kernel that itself waits for this step) can stall it.  Every wait is bounded: a wait that gives up leaves
 * the parameters of the tensors concerned unwritten (their m and v may already hold the new moments), sets
 * the plan's sticky error, and the NEXT lancet_lans_step on the plan returns LANCET_ERR_STALLED without
 * launching anything, until lancet_lans_plan_error has been called.  Steps that were already queued behind the
 * one that stalled (a loop that never synchronises, a replayed graph) see the error word on the device when they
 * begin and skip themselves as a whole, either schedule: no array is touched again before the error is read.
 * LANCET_LANS_SWEEPS: three whole-state sweeps with two per-tensor reductions between them (48 B/param of
 * traffic).  No workgroup waits for another: the schedule for a device that is shared with kernels of
 * unbounded duration.  set_schedule(LANCET_LANS_RESIDENT) on a plan with no tensor that fits returns
 * LANCET_ERR_SHAPE and the plan keeps the sweeps.
 * Each schedule is deterministic; the two agree to fp32 rounding of the per-chunk sums. */
#define LANCET_LANS_SWEEPS 0
#define LANCET_LANS_RESIDENT 1
int lancet_lans_plan_set_schedule(lancet_lans_plan_t plan, int schedule);
/* *schedule = the schedule the plan's next step runs. */
int lancet_lans_plan_schedule(lancet_lans_plan_t plan, int* schedule);
/* workgroups: chunks (of 8192 parameters) of the largest tensor the resident kernel takes on this device
 * (larger tensors of the plan go through the sweeps; 512 = 4M parameters on a device that runs 512 of the
 * kernel's workgroups at once); max_tensor_chunks: chunks of the plan's largest tensor.  Either may be
 * NULL. */
int lancet_lans_plan_resident_capacity(lancet_lans_plan_t plan, int* workgroups, int* max_tensor_chunks);
/* Reads (synchronising `stream`) and clears the plan's sticky error: 1 when a bounded wait of the resident
 * schedule gave up in any step since the last call. */
int lancet_lans_plan_error(lancet_lans_plan_t plan, lancet_stream_t stream, int* error_out);

/* Copies the four per-tensor norm vectors of the last step (||g||, ||p||, ||u_m||, ||u_g||;
 * the reference's grad_norm_tensor_ ... q_norm_tensor_ workspaces, lans.cc:77-82) into
 * norms4xT, a device buffer of 4*T floats, asynchronously on `stream`. */
int lancet_lans_plan_norms(lancet_lans_plan_t plan, float* norms4xT, lancet_stream_t stream);

/* ---- workspaces of the position scan ---------------------------------------------------
 * (No counterpart in the reference, whose scan kernel keeps no state: tutel_moe_dispatch.cu:164-212.)
 * lancet_scan_workspace_init sets a workspace of workspace_bytes bytes (8-byte aligned, at least what the
 * *_workspace_bytes() of the calls it will serve ask for) up, asynchronously on `stream`: once after
 * allocation; every call that uses the workspace leaves it ready for the next, so that no call spends a
 * launch on clearing it.  A call that is handed a workspace that is not set up launches nothing harmful:
 * it sets every indices/locations entry and every used_out entry to -1 and the error word.
 * The scan has several forms and a call picks one by its size.  Top-1 calls of at most 32 tiles of 256 tokens
 * (8192 tokens), and calls with LANCET_SCAN_LOOKBACK, run as one kernel with a look-back between tiles, to which
 * everything said here about state and waits applies.  All others run as two kernels (three on long batches: tiles
 * x counters above 32768) in which no workgroup waits for another: they use the workspace as plain scratch (no
 * state, no wait that could give up, and memory that was never set up works as well).
 * Every wait inside the scan is bounded.  A wait that gives up sets the workspace's sticky error word, and
 * every token whose position was built on it gets indices = locations = -1 (gates_s 0 for top_k = 2), as if
 * dropped, so that no consumer moves a row on a wrong position; when the totals themselves were built on it,
 * used_out = -1 for every expert (elements_per_expert 0; all tokens marked for top_k = 2).  What is not marked
 * is right.  The workspace stays usable.
 * lancet_scan_workspace_error reads (synchronising `stream`) and clears the error word: *error_out = 1
 * when any call on this workspace gave up a wait, or found it not set up, since the last read. */
int lancet_scan_workspace_init(void* workspace, size_t workspace_bytes, lancet_stream_t stream);
int lancet_scan_workspace_error(void* workspace, lancet_stream_t stream, int* error_out);
/* 1 when a call of these sizes and flags (batch_prioritized != 0: lancet_moe_encode_bpr, S = S0 / n_partitions; else
 * lancet_moe_encode / lancet_moe_route) runs the scan in its look-back form, the only form that reads state from
 * the workspace: such a call needs the first lancet_moe_encode_workspace_bytes(S, E, top_k or 2) bytes of its
 * workspace set up and can give up a wait; 0: it uses the whole workspace as plain scratch, which needs neither
 * set-up nor a look at the error word.  For executors that hand an operator fresh workspace memory before every
 * call (src/impl/vm/vm.cc:1260-1266) and would otherwise pay a set-up launch each time. */
int lancet_scan_call_is_stateful(int64_t S, int64_t E, int top_k, unsigned flags, int batch_prioritized);

#ifdef __cplusplus
}
#endif
#endif /* LANCET_HIP_H_ */
