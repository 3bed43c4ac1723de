// Shared device helpers for the gfx950 kernels (wave64 throughout).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lancet {

constexpr int kWave = 64;
constexpr int kTile = 256;                 // tokens per scan tile == threads per workgroup
constexpr int kWavesPerTile = kTile / kWave;

// ---- wave64 primitives ------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// number of set bits of `mask` strictly below the calling lane
__device__ __forceinline__ uint32_t popc_below(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// ---- device-scope loads/stores for data other workgroups publish ----------------------
__device__ __forceinline__ uint32_t ld_agent(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_acquire_agent(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_release_agent(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- pointers known to be device global memory ------------------------------------------
// A pointer read from a table in memory, or picked at run time among several, is a generic (flat)
// pointer to the compiler: flat loads and stores need a 64-bit address in vector registers each.
// Typed as global memory they take a scalar base plus a 32-bit offset.
#define LANCET_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ LANCET_GLOBAL T* as_global(T* p) {
  return (LANCET_GLOBAL T*)p;
}

// ---- 16-byte streaming row moves ---------------------------------------------------
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ u32x4 ld_stream(const u32x4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st_stream(u32x4* p, u32x4 v) { __builtin_nontemporal_store(v, p); }

// ---- storage-type conversion (fp32 math, one rounding) ------------------------------
__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint32_t f32_to_bf16(float f) {  // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;  // NaN
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float f16_to_f32(uint32_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h)));
}
__device__ __forceinline__ uint32_t f32_to_f16(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

// ---- gate values in their storage type ------------------------------------------------------
// Gate arrays (gate [S,E], gates_s [k*S], their gradients) are fp32, bf16 or fp16 (the LANCET_F32 / _BF16 / _F16
// codes 0 / 1 / 2); all arithmetic on them is fp32, with one rounding to the storage type on a store.
__device__ __forceinline__ float ld_gate(const void* p, size_t i, int gd) {
  if (gd == 0) return static_cast<const float*>(p)[i];
  const uint32_t h = static_cast<const uint16_t*>(p)[i];
  return gd == 1 ? bf16_to_f32(h) : f16_to_f32(h);
}
__device__ __forceinline__ void st_gate(void* p, size_t i, float v, int gd) {
  if (gd == 0) static_cast<float*>(p)[i] = v;
  else static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(gd == 1 ? f32_to_bf16(v) : f32_to_f16(v));
}
// the value a gate array of type gd holds after v is stored in it
__device__ __forceinline__ float round_gate(float v, int gd) {
  if (gd == 0) return v;
  return gd == 1 ? bf16_to_f32(f32_to_bf16(v)) : f16_to_f32(f32_to_f16(v));
}

}  // namespace lancet
