// lancet_moe_encode_noalloc: moe_encode for callers that cannot allocate device memory (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The position scan needs
// scratch memory beyond the inputs and outputs (the table of the tiles' counts; ticket, error word and
// descriptors in its look-back form); lancet_moe_encode takes it as a caller-owned workspace, this entry point keeps
// it in a file-scope device array of LANCET_NOALLOC_SCRATCH_BYTES instead.  Every GPU the library runs
// on holds its own copy of the array, at its own address, until the process ends.
//
// The array's name is only a host-side stand-in for the symbol: the device address is looked up once
// per device with hipGetSymbolAddress (with that device current) and kept; every launch gets that
// pointer, never the name.  Nothing here calls hipMalloc, hipFree or an allocating library routine.
// All calls on one GPU share the array, which keeps the last call's contents: it is a scan workspace, set
// up (lancet_scan_workspace_init, a fill kernel on the caller's stream) by the first call on a device and
// left ready for the next call by every call; calls that overlap on one GPU (two streams, two host
// threads) race.
#include "../../include/lancet_hip.h"
#include "common.hpp"
#include "launchers.hpp"
#include <atomic>
#include <mutex>

static __device__ __align__(256) unsigned char scratch[LANCET_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_lookup_mutex;
std::atomic<void*> g_scratch_ptr[kMaxDevices];  // device address of `scratch` on device i, or null

// Device address of this device's copy of the array; looked up, and the workspace in it set up on `stream`,
// on the first call on a device.
int scratch_for_current_device(void** out, lancet_stream_t stream) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return static_cast<int>(e);
  if (device < 0 || device >= kMaxDevices) return LANCET_ERR_SHAPE;
  void* p = g_scratch_ptr[device].load(std::memory_order_acquire);
  if (!p) {
    std::lock_guard<std::mutex> lock(g_lookup_mutex);
    p = g_scratch_ptr[device].load(std::memory_order_relaxed);
    if (!p) {
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess) return static_cast<int>(e);
      if (!p) return static_cast<int>(hipErrorInvalidSymbol);
      if (int r = lancet_scan_workspace_init(p, LANCET_NOALLOC_SCRATCH_BYTES, stream)) return r;
      // later calls may come on other streams: the set-up is complete before any of them can start
      e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
      if (e != hipSuccess) return static_cast<int>(e);
      g_scratch_ptr[device].store(p, std::memory_order_release);
    }
  }
  *out = p;
  return LANCET_OK;
}

}  // namespace

extern "C" int lancet_moe_encode_noalloc(const void* data, const void* gate, const void* gate2_noise,
                                         const int32_t* used_in, int64_t S, int64_t M, int64_t E, int64_t C,
                                         int top_k, int dtype, int gate_dtype, unsigned flags, void* gates_s,
                                         int32_t* indices_locations, int32_t* used_out,
                                         uint64_t* elements_per_expert, void* dispatched, lancet_stream_t stream) {
  if (S < 0 || E < 1 || E > LANCET_MAX_EXPERTS) return LANCET_ERR_SHAPE;
  if (top_k != 1 && top_k != 2) return LANCET_ERR_TOPK;
  const size_t need = lancet_moe_encode_workspace_bytes(S, E, top_k);
  if (need > LANCET_NOALLOC_SCRATCH_BYTES) return LANCET_ERR_SCRATCH;
  void* ws = nullptr;
  if (int r = scratch_for_current_device(&ws, stream)) return r;
  // the same kernels as lancet_moe_encode
  return lancet_moe_encode(data, gate, gate2_noise, used_in, S, M, E, C, top_k, dtype, gate_dtype, flags, gates_s,
                           indices_locations, used_out, elements_per_expert, dispatched, ws,
                           LANCET_NOALLOC_SCRATCH_BYTES, stream);
}
