/*
 * lancet_hip_debug.h - test and measurement hooks of liblancet_hip.so.  Not part of the operator surface:
 * nothing here replaces a piece of the reference, and a product build may leave these symbols out.
 */
#ifndef LANCET_HIP_DEBUG_H_
#define LANCET_HIP_DEBUG_H_

#include "lancet_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Host-only view of what a LANS plan builds for `numels` when the resident kernel takes tensors of up to
 * resident_limit chunks and runs `round` workgroups (no device needed): for every chunk slot, in the order the
 * kernel hands them out, the position of its tensor in the caller's list, or -1 for a padding slot (a tensor
 * that does not fit into what is left of a round of `round` slots starts the next round);
 * *n_resident_chunks = slots the resident kernel hands out (the rest go through the sweeps).  Returns the
 * number of slots; fills at most `capacity` entries (either output may be NULL). */
int64_t lancet_lans_debug_chunk_table(const int64_t* numels, int T, int resident_limit, int round,
                                      int32_t* chunk_tensor_out, int64_t capacity, int64_t* n_resident_chunks);

/* Test hook of one plan: spin_limit = times a workgroup of the resident schedule reads again the chunk sums it
 * misses before it gives up (0 restores the default); flags bit 0: no workgroup publishes its chunk sums, so
 * that every wait for them runs into the limit.  Lets a host test exercise the bounded waits and the error
 * path while every kernel still exits normally. */
int lancet_lans_plan_debug(lancet_lans_plan_t plan, unsigned spin_limit, unsigned flags);

/* *slots = chunk slots the resident kernel handed out in the plan's last lancet_lans_step, 0 when that step
 * went through the sweeps alone (schedule, no tensor that fits, or a resident tensor whose arrays were not
 * 16-byte aligned).  Lets a test tell which kernels it has exercised. */
int lancet_lans_plan_debug_last_resident(lancet_lans_plan_t plan, int* slots);

/* Test hook: number of polls a workgroup of the position scan waits for a predecessor's word before it gives
 * up (0 restores the default), kept in the workspace itself and read by every later call that uses it; set
 * asynchronously on `stream`.  Lets a host test exercise the bounded wait while every kernel still exits
 * normally. */
int lancet_debug_scan_workspace_spin_limit(void* workspace, unsigned limit, lancet_stream_t stream);
/* Test hook: sets the launch epoch of a scan workspace that is set up and idle (1 .. 2^30 - 1), asynchronously on
 * `stream`.  The epoch tags the scan's descriptor words and moves on by one per call; the call that runs with the
 * last value clears the descriptor table before the epoch starts again at 1.  Lets a test reach that call. */
int lancet_debug_scan_workspace_epoch(void* workspace, unsigned epoch, lancet_stream_t stream);
/* Measurement aid (no counterpart in the reference): one plain streaming kernel over `bytes` bytes (a multiple
 * of 4096), one 16-byte non-temporal access per thread, workgroups in address order: the launch shape that
 * streams fastest on this device.  kind 0 reads src, 1 fills dst with zeros, 2 copies src to dst.  bench.py
 * times these beside the row movers so that their fractions of the peak can be read against what the
 * memory system delivers to the simplest possible kernel. */
int lancet_debug_stream(int kind, void* dst, const void* src, size_t bytes, lancet_stream_t stream);
/* Measurement aid (no counterpart in the reference): the memory access pattern of an optimizer step and
 * nothing else.  Reads g, p, m, v (n floats each, n a multiple of 1024, 16-byte aligned) and writes p, m, v,
 * 28 bytes per element, with a few multiply-adds in between, one float4 per thread and array.  bench.py times
 * it beside the LANS step: what the memory system delivers to a kernel that needs no norms. */
int lancet_debug_stream_4r3w(const float* g, float* p, float* m, float* v, size_t n, lancet_stream_t stream);
/* Measurement aid (no counterpart in the reference): lancet_moe_scatter and lancet_moe_decode fed with ONE routing
 * word per slot instead of the four of indices_locations and the capacity arrays: dest[j*S + s] = e * C + location of
 * slot j of token s, -1 when the slot moves no row.  Rows of whole 16-byte granules only.  Results are those of the
 * operator calls.  Built to test whether the routing words a wave reads in front of its row cost the row movers
 * their distance to a plain copy; measured slower than the four-word form (339 against 333 us, 258 against 256 at
 * S = 65536, M = 4096 bf16, E = 32, top-2), so the operators keep indices_locations as their only format. */
int lancet_debug_scatter_dest(const void* data, const int32_t* dest, const int32_t* used_in, const int32_t* used_out,
                              int64_t S, int64_t M, int64_t E, int64_t C, int top_k, int dtype, void* dispatched,
                              lancet_stream_t stream);
int lancet_debug_decode_dest(const void* expert_out, const void* gates_s, const int32_t* dest, int64_t S, int64_t M,
                             int64_t E, int64_t C, int top_k, int dtype, int gate_dtype, void* out, lancet_stream_t stream);
#ifdef __cplusplus
}
#endif
#endif /* LANCET_HIP_DEBUG_H_ */
