// Fused multi-tensor LANS step.  The reference makes six sweeps over the optimizer state
// (src/op/dialect/cuda/kernels/multi_tensor_lans.cu:401-450: l2norm(g), l2norm(p), stage 1,
// l2norm(u_m), l2norm(u_g), stage 2, 68 B/param of traffic).  Here the step has three phases
//   phase 1  reads g               -> per-chunk sums of g^2
//   phase 2  reads g, p, m, v      -> writes m, v; per-chunk sums of p^2, u_m^2 and u_g^2
//   phase 3  reads g, p, m, v      -> recomputes u_m, u_g (never stored) and writes p
// and two schedules:
//   * sweeps (default): three plain launches + two tiny per-tensor reductions.  Real HBM traffic
//     is 48 B/param (g read three times, p, m, v twice) and each sweep streams at the rate a plain
//     copy reaches on this chip.
//   * resident (opt-in): a sweep over g alone for ||g|| (4 B/param), then ONE persistent kernel in
//     which a workgroup takes a chunk through phases 2 and 3 and keeps it on chip in between (u_m and
//     u_g in registers, p in LDS), so every array is read once and written once: 32 B/param with the
//     sweep.  Before phase 3 the workgroups of a tensor exchange three chunk partials (p^2, u_m^2,
//     u_g^2) as self-validating 64-bit words (step epoch in the high half, fp32 sum in the low half,
//     one agent-scope atomic store each); the workgroup that arrives last at a per-tensor counter
//     sums them in a fixed order and publishes the norms the same way.  Nothing else crosses
//     workgroups, so no fences are needed.  Chunks are handed out in order by a ticket; a workgroup
//     only ever waits for chunks of its own tensor, so the kernel drains as long as the chunks of one
//     tensor all fit on the chip at once (the limit is the register file: about 4M parameters per
//     tensor on 256 CUs).  The plan orders its tensors so that those within the limit come first;
//     the kernel takes them, and larger tensors go through the sweeps in the same step.  Waits are
//     bounded.
// Work is cut into fixed-size chunks described by device-resident tables built once per
// parameter set, instead of kernel arguments re-packed for every launch
// (multi_tensor_apply.cuh:39-92).  Chunk partials are combined in a fixed order in double
// precision, so each schedule is deterministic (the two differ in the last bits: a chunk's own sum is
// accumulated in a different order).
#include "launchers.hpp"
#include "common.hpp"
#include "../../include/lancet_hip.h"
#include <algorithm>
#include <new>
#include <vector>

namespace lancet {

constexpr int kLansThreads = 256;
constexpr int kLansChunk = 8192;  // elements per task: 8 float4 per thread and array
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct LansTables {
  const float* const* g;  // [T] device pointers
  float* const* p;
  float* const* m;
  float* const* v;
  const int64_t* numel;        // [T]
  const int32_t* chunk_tensor; // [nchunks]
  const int32_t* tensor_first; // [T+1] first chunk of each tensor
  float* partial;              // [3][nchunks * kSweepSplit]  (sweeps: one sum per slice)
  uint64_t* part_word;         // [4][nchunks]      (resident schedule: epoch | fp32 sum of squares)
  uint64_t* norm_word;         // [4][T]            (resident schedule: epoch | fp32 norm)
  uint32_t* ticket;            // [1] next task; [1] error flag; [T] arrivals; [1] step epoch (resident schedule)
  float* norms;                // [4][T]: g, p, u_m, u_g
  float* consts;               // [2]: bias_correction1, bias_correction2
  const int32_t* order;        // [T] position in the caller's lists of the plan's i-th tensor
  int T;
  int nchunks;
  int nres;                    // chunks [0, nres) belong to tensors the resident schedule can hold
};

struct LansScalars {
  float lr, beta1, beta2, beta3, eps, wd;
  int mode, normalize_grad, bias_correction;
  int step_host;
  const float* step_dev;
  uint32_t epoch;              // filled in on the device (the word behind the arrival counters)
  uint32_t spin_limit;
};

__device__ __forceinline__ float block_sum(float v, float* s_red) {
  v = wave_sum(v);
  const int w = threadIdx.x / kWave;
  if (lane_id() == 0) s_red[w] = v;
  __syncthreads();
  float r = 0.f;
  if (threadIdx.x == 0) {
#pragma unroll
    for (int k = 0; k < kLansThreads / kWave; ++k) r += s_red[k];
  }
  __syncthreads();
  return r;  // valid on thread 0
}

struct ChunkView {
  int tensor;
  int64_t begin;  // first element of the chunk inside the tensor
  int n;          // elements in the chunk
};

__device__ __forceinline__ ChunkView chunk_view(const LansTables& t, int chunk) {
  ChunkView c;
  c.tensor = t.chunk_tensor[chunk];
  c.begin = static_cast<int64_t>(chunk - t.tensor_first[c.tensor]) * kLansChunk;
  const int64_t left = t.numel[c.tensor] - c.begin;
  c.n = static_cast<int>(left < kLansChunk ? left : kLansChunk);
  return c;
}

template <typename A, typename B, typename C, typename D>
__device__ __forceinline__ bool vec_ok(A a, B b, C c, D d) {
  return (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c | (uintptr_t)d) & 15u) == 0;
}

// A value every lane holds alike, moved to a scalar register: it then costs no vector register
// for as long as it lives.
__device__ __forceinline__ float uniform(float x) {
  return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(x)));
}

// ---- elementwise math, in the reference's operation order (multi_tensor_lans.cu:283-307) ----
struct LansElem {
  float gnorm_eps;  // ||g|| + eps
  bool normalize;   // normalize_grad && ||g|| != 0
  float beta1, beta2, beta3, one_minus_beta2, bc1, bc2, eps, wd;
  int mode;

  __device__ __forceinline__ float scaled_grad(float g, float p) const {
#pragma clang fp contract(off)
    float sg = g;
    if (normalize) sg = sg / gnorm_eps;
    if (mode == 0) sg = sg + wd * p;
    return sg;
  }
  __device__ __forceinline__ void moments(float sg, float& m, float& v) const {
#pragma clang fp contract(off)
    m = m * beta1 + beta3 * sg;
    v = v * beta2 + one_minus_beta2 * sg * sg;
  }
  __device__ __forceinline__ void updates(float sg, float p, float m, float v, float& um, float& ug) const {
#pragma clang fp contract(off)
    const float denom = sqrtf(v / bc2) + eps;
    um = (m / bc1) / denom;
    ug = sg / denom;
    if (mode != 0) {
      const float sp = wd * p;
      um = um + sp;
      ug = ug + sp;
    }
  }
};

__device__ __forceinline__ LansElem make_elem(const LansScalars& sc, float gn, float bc1, float bc2) {
  LansElem e;
  e.gnorm_eps = uniform(gn + sc.eps);
  e.normalize = sc.normalize_grad && uniform(gn) != 0.f;
  e.beta1 = sc.beta1;
  e.beta2 = sc.beta2;
  e.beta3 = sc.beta3;
  e.one_minus_beta2 = uniform(1.f - sc.beta2);
  e.bc1 = uniform(bc1);
  e.bc2 = uniform(bc2);
  e.eps = sc.eps;
  e.wd = sc.wd;
  e.mode = sc.mode;
  return e;
}

// bias corrections 1 - beta^step (src/op/dialect/cuda/lans.cc:108-113), from a host step or
// from the fp32 step scalar in device memory (no host synchronisation, unlike lans.cc:102-107)
__device__ __forceinline__ void bias_corrections(const LansScalars& sc, float& bc1, float& bc2) {
  int step = sc.step_host;
  if (sc.step_dev) step = static_cast<int>(*sc.step_dev);
  bc1 = 1.f;
  bc2 = 1.f;
  if (sc.bias_correction) {
    bc1 = static_cast<float>(1.0 - pow(static_cast<double>(sc.beta1), step));
    bc2 = static_cast<float>(1.0 - pow(static_cast<double>(sc.beta2), step));
  }
}

// Streaming accesses: every array is touched once per sweep and is far larger than the caches; non-temporal
// loads and stores stream measurably faster here than plain ones.
__device__ __forceinline__ f32x4 ldn(const LANCET_GLOBAL f32x4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void stn(LANCET_GLOBAL f32x4* p, f32x4 x) { __builtin_nontemporal_store(x, p); }

// ---- the three phases on one chunk, executed by one workgroup ------------------------------
// phase 1: sum of squares of g (L2NormFunctor, multi_tensor_lans.cu:95-167); valid on thread 0.
// (The sum of squares of p is not needed before phase 3 and is taken in phase 2, which reads p anyway.)
__device__ __forceinline__ float chunk_norm_g(const LansTables& t, const ChunkView& c, float* s_red) {
  const LANCET_GLOBAL float* g = as_global(t.g[c.tensor] + c.begin);
  float ag = 0.f;
  int scalar_from = 0;
  if (vec_ok(g, g, g, g)) {
    const int nv = c.n / 4;
    const LANCET_GLOBAL f32x4* g4 = (const LANCET_GLOBAL f32x4*)g;
#pragma unroll 8
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 x = ldn(g4 + i);
      ag += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
    }
    scalar_from = nv * 4;
  }
  for (int i = scalar_from + threadIdx.x; i < c.n; i += kLansThreads) ag += g[i] * g[i];
  return block_sum(ag, s_red);
}

// phase 2: moments + sums of squares of p and of the two updates (LANSStage1Functor :207-322 and the
// l2norm sweeps around it, :428-441); sums valid on thread 0
__device__ __forceinline__ void chunk_moments(const LansTables& t, const ChunkView& c, const LansElem& el,
                                              float* s_red, float& sum_p, float& sum_um, float& sum_ug) {
  const LANCET_GLOBAL float* g = as_global(t.g[c.tensor] + c.begin);
  const LANCET_GLOBAL float* p = as_global(t.p[c.tensor] + c.begin);
  LANCET_GLOBAL float* m = as_global(t.m[c.tensor] + c.begin);
  LANCET_GLOBAL float* v = as_global(t.v[c.tensor] + c.begin);
  float ap = 0.f, am = 0.f, ag = 0.f;
  int scalar_from = 0;
  if (vec_ok(g, p, m, v)) {
    const int nv = c.n / 4;
    const LANCET_GLOBAL f32x4* g4 = (const LANCET_GLOBAL f32x4*)g;
    const LANCET_GLOBAL f32x4* p4 = (const LANCET_GLOBAL f32x4*)p;
    LANCET_GLOBAL f32x4* m4 = (LANCET_GLOBAL f32x4*)m;
    LANCET_GLOBAL f32x4* v4 = (LANCET_GLOBAL f32x4*)v;
#pragma unroll 2
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 xg = ldn(g4 + i), xp = ldn(p4 + i);
      f32x4 xm = ldn(m4 + i), xv = ldn(v4 + i);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float sg = el.scaled_grad(xg[k], xp[k]);
        float mm = xm[k], vv = xv[k], um, ug;
        el.moments(sg, mm, vv);
        el.updates(sg, xp[k], mm, vv, um, ug);
        xm[k] = mm;
        xv[k] = vv;
        ap += xp[k] * xp[k];
        am += um * um;
        ag += ug * ug;
      }
      stn(m4 + i, xm);
      stn(v4 + i, xv);
    }
    scalar_from = nv * 4;
  }
  for (int i = scalar_from + threadIdx.x; i < c.n; i += kLansThreads) {
    const float sg = el.scaled_grad(g[i], p[i]);
    float mm = m[i], vv = v[i], um, ug;
    el.moments(sg, mm, vv);
    el.updates(sg, p[i], mm, vv, um, ug);
    m[i] = mm;
    v[i] = vv;
    ap += p[i] * p[i];
    am += um * um;
    ag += ug * ug;
  }
  sum_p = block_sum(ap, s_red);
  sum_um = block_sum(am, s_red);
  sum_ug = block_sum(ag, s_red);
}

// phase 3: trust ratios and parameter update (LANSStage2Functor :326-399)
__device__ __forceinline__ void chunk_update(const LansTables& t, const ChunkView& c, const LansElem& el,
                                             const LansScalars& sc, float pn, float umn, float ugn) {
  float ratio_m = (umn != 0.f && pn != 0.f) ? sc.lr * (pn / umn) : sc.lr;
  float ratio_g = (ugn != 0.f && pn != 0.f) ? sc.lr * (pn / ugn) : sc.lr;
  ratio_m *= sc.beta1;
  ratio_g *= sc.beta3;
  const LANCET_GLOBAL float* g = as_global(t.g[c.tensor] + c.begin);
  LANCET_GLOBAL float* p = as_global(t.p[c.tensor] + c.begin);
  const LANCET_GLOBAL float* m = as_global(t.m[c.tensor] + c.begin);
  const LANCET_GLOBAL float* v = as_global(t.v[c.tensor] + c.begin);
  int scalar_from = 0;
  if (vec_ok(g, p, m, v)) {
    const int nv = c.n / 4;
    const LANCET_GLOBAL f32x4* g4 = (const LANCET_GLOBAL f32x4*)g;
    LANCET_GLOBAL f32x4* p4 = (LANCET_GLOBAL f32x4*)p;
    const LANCET_GLOBAL f32x4* m4 = (const LANCET_GLOBAL f32x4*)m;
    const LANCET_GLOBAL f32x4* v4 = (const LANCET_GLOBAL f32x4*)v;
#pragma unroll 2
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 xg = ldn(g4 + i), xm = ldn(m4 + i), xv = ldn(v4 + i);
      f32x4 xp = ldn(p4 + i);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
#pragma clang fp contract(off)
        const float sg = el.scaled_grad(xg[k], xp[k]);
        float um, ug;
        el.updates(sg, xp[k], xm[k], xv[k], um, ug);
        xp[k] = xp[k] - (ratio_m * um) - (ratio_g * ug);
      }
      stn(p4 + i, xp);
    }
    scalar_from = nv * 4;
  }
  for (int i = scalar_from + threadIdx.x; i < c.n; i += kLansThreads) {
#pragma clang fp contract(off)
    const float sg = el.scaled_grad(g[i], p[i]);
    float um, ug;
    el.updates(sg, p[i], m[i], v[i], um, ug);
    p[i] = p[i] - (ratio_m * um) - (ratio_g * ug);
  }
}

// sqrt of the sum of a tensor's chunk partials: one wave, lane-strided double sums, xor tree
// (fixed order, so every caller gets the same bits).  get(c) returns the partial of chunk c.
template <typename Get>
__device__ __forceinline__ float wave_norm(int lo, int hi, Get get) {
  double acc = 0.0;
  for (int c = lo + lane_id(); c < hi; c += kWave) acc += static_cast<double>(get(c));
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
  return static_cast<float>(sqrt(acc));
}

// =======================================================================================
// schedule "sweeps": three launches + two per-tensor reductions
// =======================================================================================
__global__ void lans_prepare_kernel(LansTables t, LansScalars sc) {
  if (threadIdx.x == 0 && blockIdx.x == 0) bias_corrections(sc, t.consts[0], t.consts[1]);
}

// The sweeps hand every chunk to kSweepSplit workgroups (a slice of kLansChunk / kSweepSplit elements each:
// one float4 per thread and array).  Short workgroups in address order stream a few percent faster than
// workgroups that loop over a whole chunk; the chunk stays the unit of the tables and of the resident kernel.
#ifndef LANCET_SWEEP_SPLIT
#define LANCET_SWEEP_SPLIT 8
#endif
constexpr int kSweepSplit = LANCET_SWEEP_SPLIT;
constexpr int kSweepSlice = kLansChunk / kSweepSplit;

// slice blockIdx.x % kSweepSplit of chunk chunk_base + blockIdx.x / kSweepSplit (n may be 0: past the tensor's end)
__device__ __forceinline__ ChunkView slice_view(const LansTables& t, int chunk_base, int& slot) {
  const int chunk = chunk_base + static_cast<int>(blockIdx.x / kSweepSplit);
  const int sub = static_cast<int>(blockIdx.x % kSweepSplit);
  slot = chunk * kSweepSplit + sub;
  ChunkView c = chunk_view(t, chunk);
  const int first = sub * kSweepSlice;
  c.begin += first;
  c.n = c.n > first ? (c.n - first < kSweepSlice ? c.n - first : kSweepSlice) : 0;
  return c;
}

// The sweep over g covers chunks [chunk_base, chunk_base + gridDim.x), the other two
// [chunk_base, chunk_base + gridDim.x / kSweepSplit): all of them, or the ones the resident
// kernel takes (first sweep only), or the ones it leaves (tensors too large for it).
__global__ __launch_bounds__(kLansThreads) void lans_norm_g_kernel(LansTables t, int chunk_base) {
  __shared__ float s_red[kLansThreads / kWave];
  const int chunk = chunk_base + blockIdx.x;  // a whole chunk per workgroup: this sweep only reads, and splitting it costs more in reductions than it gains
  const float sg = chunk_norm_g(t, chunk_view(t, chunk), s_red);
  if (threadIdx.x == 0) t.partial[chunk] = sg;
}

// per-tensor sqrt(sum of chunk partials) (cleanup, multi_tensor_lans.cu:169-185)
// split: partial sums per chunk (1 after the sweep over g, kSweepSplit after the moments sweep)
__global__ __launch_bounds__(kLansThreads) void lans_reduce_kernel(LansTables t, int first_norm, int tensor_base,
                                                                   int tensor_end, int count, int split) {
  const int tensor = tensor_base + blockIdx.x * (kLansThreads / kWave) + threadIdx.x / kWave;
  if (tensor >= tensor_end) return;
  const int lo = t.tensor_first[tensor], hi = t.tensor_first[tensor + 1];
  for (int k = 0; k < count; ++k) {
    const float* part = t.partial + static_cast<size_t>(k) * t.nchunks * split;
    const float n = wave_norm(lo * split, hi * split, [&](int c) { return part[c]; });
    if (lane_id() == 0) t.norms[(first_norm + k) * t.T + tensor] = n;
  }
}

__global__ __launch_bounds__(kLansThreads) void lans_moments_kernel(LansTables t, LansScalars sc, int chunk_base) {
  __shared__ float s_red[kLansThreads / kWave];
  int slot;
  const ChunkView c = slice_view(t, chunk_base, slot);
  const LansElem el = make_elem(sc, t.norms[c.tensor], t.consts[0], t.consts[1]);
  float sp, sm, sg;
  chunk_moments(t, c, el, s_red, sp, sm, sg);
  if (threadIdx.x == 0) {
    const size_t row = static_cast<size_t>(t.nchunks) * kSweepSplit;
    t.partial[slot] = sp;
    t.partial[row + slot] = sm;
    t.partial[2 * row + slot] = sg;
  }
}

__global__ __launch_bounds__(kLansThreads) void lans_update_kernel(LansTables t, LansScalars sc, int chunk_base) {
  int slot;
  const ChunkView c = slice_view(t, chunk_base, slot);
  const LansElem el = make_elem(sc, t.norms[c.tensor], t.consts[0], t.consts[1]);
  chunk_update(t, c, el, sc, t.norms[1 * t.T + c.tensor], t.norms[2 * t.T + c.tensor], t.norms[3 * t.T + c.tensor]);
}

// norms live in the plan's tensor order; callers get them in the order of their lists
__global__ void lans_gather_norms_kernel(LansTables t, float* dst) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= t.T) return;
#pragma unroll
  for (int k = 0; k < 4; ++k) dst[k * t.T + t.order[i]] = t.norms[k * t.T + i];
}

// =======================================================================================
// words published between workgroups: step epoch in the high half, fp32 value in the low half
// =======================================================================================
__device__ __forceinline__ uint64_t ld_word(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_word(uint64_t* p, uint32_t epoch, float v) {
  __hip_atomic_store(p, (static_cast<uint64_t>(epoch) << 32) | __float_as_uint(v), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// =======================================================================================
// schedule "resident": a sweep over g, then one persistent kernel in which a workgroup keeps its
// chunk on chip between moments and update, so every array is read once and written once, g twice
// =======================================================================================
constexpr int kVecPerThread = kLansChunk / 4 / kLansThreads;  // float4 per thread and array

__device__ __forceinline__ f32x4 ld4(const LANCET_GLOBAL float* a, int e) { return ldn((const LANCET_GLOBAL f32x4*)(a + e)); }
__device__ __forceinline__ void st4(LANCET_GLOBAL float* a, int e, f32x4 x) { stn((LANCET_GLOBAL f32x4*)(a + e), x); }

constexpr int kMaxResidentChunks = 512;  // chunks of one tensor the resident schedule can gather

struct ResidentShared {
  f32x4 p[kVecPerThread][kLansThreads];  // the chunk's parameters, one private slot per thread and float4
  float part[3][kMaxResidentChunks];     // gathered chunk partials of the tensor
  float red[kLansThreads / kWave];
  float norm[4];
  int chunk;
  int last;
};

__device__ __forceinline__ uint64_t wait_word(const LansTables& t, const LansScalars& sc, const uint64_t* src) {
  uint64_t x = ld_word(src);
  uint32_t spins = 0;
  while (static_cast<uint32_t>(x >> 32) != sc.epoch) {
    if (++spins > sc.spin_limit) {  // bounded: flag the plan, carry on
      st_agent(t.ticket + 1, 1u);
      break;
    }
    __builtin_amdgcn_s_sleep(2);
    x = ld_word(src);
  }
  return x;
}

// Norms first .. first+N-1 of the tensor from the partials its workgroups publish (this one has
// published its own, a[], just before).  The workgroup that arrives last (a per-tensor counter, cleared
// by the host before the step) gathers the partials into LDS, sums them in the fixed order of
// wave_norm and publishes the norms as self-validating words; every other workgroup waits for those
// words only.  Waits are bounded.
template <int N>
__device__ __forceinline__ void resident_norms(const LansTables& t, const LansScalars& sc, int first, int tensor,
                                               const float (&a)[N], ResidentShared& sh) {
  const int lo = t.tensor_first[tensor];
  const int nc = t.tensor_first[tensor + 1] - lo;
  const int w = threadIdx.x / kWave;
  if (nc == 1) {
    if (threadIdx.x == 0) {
#pragma unroll
      for (int k = 0; k < N; ++k) sh.part[k][0] = a[k];
    }
    __syncthreads();
  } else {
    if (threadIdx.x == 0) {
      uint32_t* arrive = t.ticket + 2 + tensor;
      const uint32_t old = __hip_atomic_fetch_add(arrive, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      sh.last = old == static_cast<uint32_t>(nc - 1);
    }
    __syncthreads();
    if (!sh.last) {
      if (w < N && lane_id() == 0) {
        const uint64_t x = wait_word(t, sc, t.norm_word + static_cast<size_t>(first + w) * t.T + tensor);
        sh.norm[first + w] = __uint_as_float(static_cast<uint32_t>(x));
      }
      __syncthreads();
      return;
    }
    for (int idx = threadIdx.x; idx < N * nc; idx += kLansThreads) {
      const int which = idx / nc;
      const uint64_t x = wait_word(t, sc, t.part_word + static_cast<size_t>(first + which) * t.nchunks + lo + (idx - which * nc));
      sh.part[which][idx - which * nc] = __uint_as_float(static_cast<uint32_t>(x));
    }
    __syncthreads();
  }
  if (w < N) {
    const float n = wave_norm(0, nc, [&](int c) { return sh.part[w][c]; });
    if (lane_id() == 0) {
      sh.norm[first + w] = n;
      if (nc > 1) st_word(t.norm_word + static_cast<size_t>(first + w) * t.T + tensor, sc.epoch, n);
    }
  }
  __syncthreads();
}

// One whole chunk of 16-byte aligned arrays, every access an unconditional float4.  ||g|| of the tensor is
// already in t.norms (a sweep over g alone ran first), so one pass loads everything, writes m and v and
// leaves u_m, u_g in registers and p in LDS; Sum p^2 joins the two update sums at the single wait, after
// which p is written: every array is read once and written once, g twice.
__device__ __forceinline__ void resident_chunk(const LansTables& t, const LansScalars& sc, const ChunkView& c,
                                                       int chunk, float bc1, float bc2, ResidentShared& sh) {
  const LANCET_GLOBAL float* g = as_global(t.g[c.tensor] + c.begin);
  LANCET_GLOBAL float* p = as_global(t.p[c.tensor] + c.begin);
  LANCET_GLOBAL float* m = as_global(t.m[c.tensor] + c.begin);
  LANCET_GLOBAL float* v = as_global(t.v[c.tensor] + c.begin);
  f32x4 xg[kVecPerThread], xu[kVecPerThread];  // u_g and u_m of the thread's eight float4
  // a wave owns 2048 consecutive elements: float4 k of lane l is element 4 * (64 k + l) of them, so one
  // load instruction of a wave covers 1 KB of consecutive memory
  const int e0 = (threadIdx.x / kWave) * (kLansChunk / kWavesPerTile) + 4 * lane_id();
  const LansElem el = make_elem(sc, t.norms[c.tensor], bc1, bc2);
  float a0 = 0.f, a1 = 0.f, a2 = 0.f;
#pragma unroll
  for (int k = 0; k < kVecPerThread; ++k) {
    const int e = e0 + k * (4 * kWave);
    const f32x4 g4 = ld4(g, e), xp = ld4(p, e);
    f32x4 xm = ld4(m, e), xv = ld4(v, e);
    sh.p[k][threadIdx.x] = xp;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float sg = el.scaled_grad(g4[j], xp[j]);
      float mm = xm[j], vv = xv[j], u0, u1;
      el.moments(sg, mm, vv);
      el.updates(sg, xp[j], mm, vv, u0, u1);
      // the two updates are final here: nothing of their computation may be left for after the wait (the
      // compiler otherwise carries a third value per element, wd * p, across it and spills)
      asm volatile("" : "+v"(u0), "+v"(u1));
      xm[j] = mm;
      xv[j] = vv;
      xu[k][j] = u0;
      xg[k][j] = u1;
      a0 += xp[j] * xp[j];
      a1 += u0 * u0;
      a2 += u1 * u1;
    }
    st4(m, e, xm);
    st4(v, e, xv);
  }
  a0 = block_sum(a0, sh.red);
  a1 = block_sum(a1, sh.red);
  a2 = block_sum(a2, sh.red);
  if (threadIdx.x == 0) {
    st_word(t.part_word + 1 * static_cast<size_t>(t.nchunks) + chunk, sc.epoch, a0);
    st_word(t.part_word + 2 * static_cast<size_t>(t.nchunks) + chunk, sc.epoch, a1);
    st_word(t.part_word + 3 * static_cast<size_t>(t.nchunks) + chunk, sc.epoch, a2);
  }
  {
    const float a[3] = {a0, a1, a2};
    resident_norms<3>(t, sc, 1, c.tensor, a, sh);
  }
  if (threadIdx.x == 0 && chunk == t.tensor_first[c.tensor]) {
#pragma unroll
    for (int k = 1; k < 4; ++k) t.norms[k * t.T + c.tensor] = sh.norm[k];
  }
  const float pn = uniform(sh.norm[1]), umn = uniform(sh.norm[2]), ugn = uniform(sh.norm[3]);
  float ratio_m = (umn != 0.f && pn != 0.f) ? sc.lr * (pn / umn) : sc.lr;
  float ratio_g = (ugn != 0.f && pn != 0.f) ? sc.lr * (pn / ugn) : sc.lr;
  ratio_m = uniform(ratio_m * sc.beta1);
  ratio_g = uniform(ratio_g * sc.beta3);
#pragma unroll
  for (int k = 0; k < kVecPerThread; ++k) {
    const int e = e0 + k * (4 * kWave);
    f32x4 xp = sh.p[k][threadIdx.x];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma clang fp contract(off)
      xp[j] = xp[j] - (ratio_m * xu[k][j]) - (ratio_g * xg[k][j]);
    }
    st4(p, e, xp);
  }
}

// A partial or unaligned chunk through the same protocol with the streaming chunk functions of the
// sweeps (nothing held in registers; m and v written before the wait are read back after it by the thread
// that wrote them).  At most one chunk per tensor takes this path when arrays are aligned.
__device__ __forceinline__ void resident_chunk_streamed(const LansTables& t, const LansScalars& sc, const ChunkView& c,
                                                        int chunk, float bc1, float bc2, ResidentShared& sh) {
  float a0, a1, a2;
  const LansElem el = make_elem(sc, t.norms[c.tensor], bc1, bc2);
  chunk_moments(t, c, el, sh.red, a0, a1, a2);
  if (threadIdx.x == 0) {
    st_word(t.part_word + 1 * static_cast<size_t>(t.nchunks) + chunk, sc.epoch, a0);
    st_word(t.part_word + 2 * static_cast<size_t>(t.nchunks) + chunk, sc.epoch, a1);
    st_word(t.part_word + 3 * static_cast<size_t>(t.nchunks) + chunk, sc.epoch, a2);
  }
  const float a[3] = {a0, a1, a2};
  resident_norms<3>(t, sc, 1, c.tensor, a, sh);
  if (threadIdx.x == 0 && chunk == t.tensor_first[c.tensor]) {
#pragma unroll
    for (int k = 1; k < 4; ++k) t.norms[k * t.T + c.tensor] = sh.norm[k];
  }
  chunk_update(t, c, el, sc, sh.norm[1], sh.norm[2], sh.norm[3]);
}

// Compiled for four waves per SIMD (128 registers per lane), i.e. four workgroups per CU, which is also
// what the 36 KB of LDS per workgroup allows: 1024 chunks on 256 CUs, two of the largest supported
// tensors at once, so that memory stays busy while the workgroups of one tensor wait.
constexpr int kResidentWavesPerSimd = 4;

// Start of a resident step: clears the ticket, the error flag and the arrival counters and moves the
// step epoch on.  The epoch lives on the device so that a step recorded in a graph tags every replay
// differently; when it wraps (2^32 steps) every word of earlier steps is forgotten.
__global__ __launch_bounds__(kLansThreads) void lans_begin_kernel(LansTables t, size_t nwords) {
  const size_t i = blockIdx.x * static_cast<size_t>(kLansThreads) + threadIdx.x;
  if (i < 2 + static_cast<size_t>(t.T)) t.ticket[i] = 0u;
  if (blockIdx.x == 0) {
    uint32_t* ep = t.ticket + 2 + t.T;
    const uint32_t e = *ep + 1u;
    if (e == 0u)
      for (size_t k = threadIdx.x; k < nwords; k += kLansThreads) t.part_word[k] = 0;  // norm words follow
    __syncthreads();
    if (threadIdx.x == 0) *ep = e == 0u ? 1u : e;
  }
}

__global__ __launch_bounds__(kLansThreads, kResidentWavesPerSimd) void lans_resident_kernel(LansTables t, LansScalars sc) {
  __shared__ ResidentShared sh;
  sc.epoch = __builtin_amdgcn_readfirstlane(t.ticket[2 + t.T]);
  float bc1, bc2;
  bias_corrections(sc, bc1, bc2);
  while (true) {
    __syncthreads();  // shared words of the previous chunk are no longer read
    if (threadIdx.x == 0) sh.chunk = static_cast<int>(atomicAdd(t.ticket, 1u));
    __syncthreads();
    // one value for the whole workgroup, and known to be: pointers and sizes derived from it stay scalar
    const int chunk = __builtin_amdgcn_readfirstlane(sh.chunk);
    if (chunk >= t.nres) break;  // every workgroup reaches this: chunks are finite
    const ChunkView c = chunk_view(t, chunk);
    const bool full = c.n == kLansChunk &&
                      vec_ok(t.g[c.tensor], t.p[c.tensor], t.m[c.tensor], t.v[c.tensor]);
    if (full) resident_chunk(t, sc, c, chunk, bc1, bc2, sh);
    else resident_chunk_streamed(t, sc, c, chunk, bc1, bc2, sh);
  }
}

}  // namespace lancet

// ---------------------------------------------------------------------------------------
// plan object and C entry points
// ---------------------------------------------------------------------------------------
using namespace lancet;

struct lancet_lans_plan {
  uint32_t magic;
  int device;
  int T;
  int nchunks;
  std::vector<int64_t> numels;
  std::vector<const void*> shadow;  // last uploaded 4T pointers
  void* dev_block;                  // one allocation holding every table
  void** h_ptrs;                    // pinned staging for the pointer tables
  hipEvent_t upload_done;
  bool upload_pending;
  LansTables tables;
  int schedule;           // LANCET_LANS_SWEEPS or LANCET_LANS_RESIDENT
  int resident_grid;      // workgroups of the resident schedule the device runs at once
  int max_tensor_chunks;  // chunks of the largest tensor
  int resident_limit;     // chunks of the largest tensor the resident schedule holds on this device
  int n_res_tensors;      // tensors within that limit: the first ones in the plan's own order
  int n_res_chunks;
  std::vector<int32_t> order;  // plan position -> position in the caller's lists
  size_t words_offset; // part_word + norm_word inside dev_block
  size_t words_bytes;
};

static constexpr uint32_t kPlanMagic = 0x4c414e53u;  // "LANS"

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

static void chunk_tables(const int64_t* numels, int T, std::vector<int32_t>& ctensor, std::vector<int32_t>& first) {
  first.assign(T + 1, 0);
  ctensor.clear();
  int c = 0;
  for (int i = 0; i < T; ++i) {
    first[i] = c;
    const int k = static_cast<int>((numels[i] + kLansChunk - 1) / kLansChunk);
    for (int j = 0; j < k; ++j) ctensor.push_back(i);
    c += k;
  }
  first[T] = c;
}

// The plan's own tensor order: tensors of at most `limit` chunks first (the resident schedule takes
// those), the larger ones after them (they go through the sweeps), list order kept inside each group.
static int tensor_order(const int64_t* numels, int T, int limit, std::vector<int32_t>& order) {
  order.clear();
  for (int pass = 0; pass < 2; ++pass)
    for (int i = 0; i < T; ++i) {
      const bool fits = (numels[i] + kLansChunk - 1) / kLansChunk <= limit;
      if (fits == (pass == 0)) order.push_back(i);
    }
  int n_fit = 0;
  for (int i = 0; i < T; ++i) n_fit += (numels[i] + kLansChunk - 1) / kLansChunk <= limit;
  return n_fit;
}

// Host-only view of what a plan builds for `numels` when the resident schedule holds tensors of up to
// `resident_limit` chunks (no device needed): for every chunk, in ticket order, the position of its
// tensor in the caller's list; *n_resident_chunks = chunks the resident kernel hands out.
extern "C" int64_t lancet_lans_debug_chunk_table(const int64_t* numels, int T, int resident_limit,
                                                 int32_t* chunk_tensor_out, int64_t capacity,
                                                 int64_t* n_resident_chunks) {
  if (!numels || T <= 0) return -1;
  std::vector<int32_t> order, ctensor, first;
  const int n_fit = tensor_order(numels, T, resident_limit, order);
  std::vector<int64_t> perm(T);
  for (int i = 0; i < T; ++i) perm[i] = numels[order[i]];
  chunk_tables(perm.data(), T, ctensor, first);
  for (int64_t i = 0; i < capacity && i < static_cast<int64_t>(ctensor.size()); ++i)
    if (chunk_tensor_out) chunk_tensor_out[i] = order[ctensor[i]];
  if (n_resident_chunks) *n_resident_chunks = first[n_fit];
  return static_cast<int64_t>(ctensor.size());
}

extern "C" int lancet_lans_plan_create(const int64_t* numels, int T, lancet_lans_plan_t* out) {
  if (!numels || !out) return LANCET_ERR_NULL;
  if (T <= 0) return LANCET_ERR_SHAPE;
  int64_t nchunks64 = 0;
  for (int i = 0; i < T; ++i) {
    if (numels[i] < 0) return LANCET_ERR_SHAPE;
    nchunks64 += (numels[i] + kLansChunk - 1) / kLansChunk;
  }
  if (nchunks64 * kSweepSplit > 0x7fffffff) return LANCET_ERR_SHAPE;  // slices index the partial sums and the grids
  lancet_lans_plan* pl = new (std::nothrow) lancet_lans_plan();
  if (!pl) return static_cast<int>(hipErrorOutOfMemory);
  pl->magic = kPlanMagic;
  pl->T = T;
  pl->nchunks = static_cast<int>(nchunks64);
  pl->numels.assign(numels, numels + T);
  pl->shadow.assign(4 * static_cast<size_t>(T), nullptr);
  pl->dev_block = nullptr;
  pl->h_ptrs = nullptr;
  pl->upload_done = nullptr;
  pl->upload_pending = false;
  hipError_t err = hipGetDevice(&pl->device);
  // device block layout
  const size_t n = static_cast<size_t>(pl->nchunks);
  size_t off = 0;
  const size_t o_ptrs = off;      off = align_up(off + 4 * T * sizeof(void*), 256);
  const size_t o_numel = off;     off = align_up(off + T * sizeof(int64_t), 256);
  const size_t o_ctensor = off;   off = align_up(off + (n ? n : 1) * sizeof(int32_t), 256);
  const size_t o_first = off;     off = align_up(off + (T + 1) * sizeof(int32_t), 256);
  const size_t o_partial = off;   off = align_up(off + 3 * (n ? n : 1) * kSweepSplit * sizeof(float), 256);
  const size_t o_norms = off;     off = align_up(off + 4 * T * sizeof(float), 256);
  const size_t o_consts = off;    off = align_up(off + 2 * sizeof(float), 256);
  const size_t o_words = off;     off = align_up(off + 4 * ((n ? n : 1) + T) * sizeof(uint64_t), 256);
  const size_t o_ticket = off;    off = align_up(off + (3 + static_cast<size_t>(T)) * sizeof(uint32_t), 256);
  const size_t o_order = off;     off = align_up(off + T * sizeof(int32_t), 256);
  pl->schedule = LANCET_LANS_SWEEPS;
  pl->words_offset = o_words;
  pl->words_bytes = 4 * ((n ? n : 1) + T) * sizeof(uint64_t);
  int cus = 256;
  if (err == hipSuccess) err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, pl->device);
  pl->resident_grid = 0;
  pl->max_tensor_chunks = 0;
  for (int i = 0; i < T; ++i)
    pl->max_tensor_chunks = std::max<int>(pl->max_tensor_chunks, static_cast<int>((numels[i] + kLansChunk - 1) / kLansChunk));
  if (err == hipSuccess) {
    int per_cu = 0;
    err = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, lans_resident_kernel, kLansThreads, 0);
    pl->resident_grid = per_cu * cus;
  }
  pl->resident_limit = std::min(pl->resident_grid, kMaxResidentChunks);
  pl->n_res_tensors = tensor_order(numels, T, pl->resident_limit, pl->order);
  if (err == hipSuccess) err = hipMalloc(&pl->dev_block, off);
  if (err == hipSuccess) err = hipHostMalloc(reinterpret_cast<void**>(&pl->h_ptrs), 4 * T * sizeof(void*), hipHostMallocDefault);
  if (err == hipSuccess) err = hipEventCreateWithFlags(&pl->upload_done, hipEventDisableTiming);
  if (err == hipSuccess) {
    std::vector<int32_t> ctensor, first;
    std::vector<int64_t> perm(T);
    for (int i = 0; i < T; ++i) perm[i] = numels[pl->order[i]];
    chunk_tables(perm.data(), T, ctensor, first);
    pl->n_res_chunks = first[pl->n_res_tensors];
    char* base = static_cast<char*>(pl->dev_block);
    err = hipMemcpy(base + o_numel, perm.data(), T * sizeof(int64_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(base + o_order, pl->order.data(), T * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess && n) err = hipMemcpy(base + o_ctensor, ctensor.data(), n * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(base + o_first, first.data(), (T + 1) * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemset(base + o_norms, 0, 4 * T * sizeof(float));
    if (err == hipSuccess) err = hipMemset(base + o_words, 0, pl->words_bytes);
    if (err == hipSuccess) err = hipMemset(base + o_ticket, 0, (3 + static_cast<size_t>(T)) * sizeof(uint32_t));
    LansTables& t = pl->tables;
    t.part_word = reinterpret_cast<uint64_t*>(base + o_words);
    t.norm_word = t.part_word + 4 * (n ? n : 1);
    t.ticket = reinterpret_cast<uint32_t*>(base + o_ticket);
    void** dptrs = reinterpret_cast<void**>(base + o_ptrs);
    t.g = reinterpret_cast<const float* const*>(dptrs);
    t.p = reinterpret_cast<float* const*>(dptrs + T);
    t.m = reinterpret_cast<float* const*>(dptrs + 2 * T);
    t.v = reinterpret_cast<float* const*>(dptrs + 3 * T);
    t.numel = reinterpret_cast<const int64_t*>(base + o_numel);
    t.chunk_tensor = reinterpret_cast<const int32_t*>(base + o_ctensor);
    t.tensor_first = reinterpret_cast<const int32_t*>(base + o_first);
    t.partial = reinterpret_cast<float*>(base + o_partial);
    t.norms = reinterpret_cast<float*>(base + o_norms);
    t.consts = reinterpret_cast<float*>(base + o_consts);
    t.order = reinterpret_cast<const int32_t*>(base + o_order);
    t.T = T;
    t.nchunks = pl->nchunks;
    t.nres = pl->n_res_chunks;
  }
  if (err != hipSuccess) {
    lancet_lans_plan_destroy(pl);
    return static_cast<int>(err);
  }
  *out = pl;
  return LANCET_OK;
}

extern "C" int lancet_lans_plan_destroy(lancet_lans_plan_t pl) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (pl->upload_done) {
    if (pl->upload_pending) (void)hipEventSynchronize(pl->upload_done);
    (void)hipEventDestroy(pl->upload_done);
  }
  if (pl->h_ptrs) (void)hipHostFree(pl->h_ptrs);
  if (pl->dev_block) (void)hipFree(pl->dev_block);
  pl->magic = 0;
  delete pl;
  return LANCET_OK;
}

extern "C" int lancet_lans_plan_norms(lancet_lans_plan_t pl, float* norms, lancet_stream_t stream) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (!norms) return LANCET_ERR_NULL;
  lans_gather_norms_kernel<<<(pl->T + 255) / 256, 256, 0, static_cast<hipStream_t>(stream)>>>(pl->tables, norms);
  return static_cast<int>(hipGetLastError());
}

extern "C" int lancet_lans_step(lancet_lans_plan_t pl, const float* const* g, float* const* p,
                                float* const* m, float* const* v, int step_host,
                                const float* step_dev, const lancet_lans_hyper* h,
                                lancet_stream_t stream) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (!g || !p || !m || !v || !h) return LANCET_ERR_NULL;
  if (!step_dev && step_host < 1) return LANCET_ERR_SHAPE;
  if (h->mode != 0 && h->mode != 1) return LANCET_ERR_SHAPE;
  int current = -1;
  if (hipGetDevice(&current) != hipSuccess || current != pl->device) return LANCET_ERR_PLAN;  // tables live on pl->device
  const int T = pl->T;
  hipStream_t st = static_cast<hipStream_t>(stream);
  bool changed = false;
  for (int i = 0; i < T; ++i) {
    if (pl->numels[i] > 0 && (!g[i] || !p[i] || !m[i] || !v[i])) return LANCET_ERR_NULL;
    if ((reinterpret_cast<uintptr_t>(g[i]) | reinterpret_cast<uintptr_t>(p[i]) |
         reinterpret_cast<uintptr_t>(m[i]) | reinterpret_cast<uintptr_t>(v[i])) & 3u)
      return LANCET_ERR_ALIGN;
    changed = changed || pl->shadow[i] != g[i] || pl->shadow[T + i] != p[i] ||
              pl->shadow[2 * T + i] != m[i] || pl->shadow[3 * T + i] != v[i];
  }
  hipError_t err = hipSuccess;
  if (changed) {
    // the pinned staging buffer may still be the source of the previous upload
    if (pl->upload_pending) {
      err = hipEventSynchronize(pl->upload_done);
      if (err != hipSuccess) return static_cast<int>(err);
    }
    for (int i = 0; i < T; ++i) {
      pl->shadow[i] = const_cast<float*>(g[i]);
      pl->shadow[T + i] = p[i];
      pl->shadow[2 * T + i] = m[i];
      pl->shadow[3 * T + i] = v[i];
      const int u = pl->order[i];  // the plan's i-th tensor is the caller's u-th
      pl->h_ptrs[i] = const_cast<float*>(g[u]);
      pl->h_ptrs[T + i] = p[u];
      pl->h_ptrs[2 * T + i] = m[u];
      pl->h_ptrs[3 * T + i] = v[u];
    }
    err = hipMemcpyAsync(pl->dev_block, pl->h_ptrs,
                         4 * static_cast<size_t>(T) * sizeof(void*), hipMemcpyHostToDevice, st);
    if (err == hipSuccess) err = hipEventRecord(pl->upload_done, st);
    if (err != hipSuccess) return static_cast<int>(err);
    pl->upload_pending = true;
  }
  if (pl->nchunks == 0) return LANCET_OK;
  LansScalars sc;
  sc.lr = h->learning_rate;
  sc.beta1 = h->beta1;
  sc.beta2 = h->beta2;
  sc.beta3 = h->grad_averaging ? 1.f - h->beta1 : 1.f;
  sc.eps = h->eps;
  sc.wd = h->weight_decay;
  sc.mode = h->mode;
  sc.normalize_grad = h->normalize_grad;
  sc.bias_correction = h->bias_correction;
  sc.step_host = step_host;
  sc.step_dev = step_dev;
  const LansTables& t = pl->tables;
  sc.spin_limit = current_spin_limit();
  // chunks [0, chunk_base) and tensors [0, tensor_base) go through the resident kernel, the rest
  // (everything, under the sweeps schedule) through the three sweeps
  int chunk_base = 0, tensor_base = 0;
  sc.epoch = 0;
  if (pl->schedule == LANCET_LANS_RESIDENT && pl->n_res_chunks > 0) {
    const unsigned begin_blocks = static_cast<unsigned>((2 + static_cast<size_t>(T) + kLansThreads - 1) / kLansThreads);
    lans_begin_kernel<<<begin_blocks, kLansThreads, 0, st>>>(t, pl->words_bytes / sizeof(uint64_t));
    const int grid = std::min(pl->resident_grid, pl->n_res_chunks);
    const int per_block = kLansThreads / kWave;
    lans_norm_g_kernel<<<pl->n_res_chunks, kLansThreads, 0, st>>>(t, 0);
    lans_reduce_kernel<<<(pl->n_res_tensors + per_block - 1) / per_block, kLansThreads, 0, st>>>(t, 0, 0, pl->n_res_tensors, 1, 1);
    lans_resident_kernel<<<grid, kLansThreads, 0, st>>>(t, sc);
    chunk_base = pl->n_res_chunks;
    tensor_base = pl->n_res_tensors;
  }
  const int nsweep = t.nchunks - chunk_base;
  if (nsweep > 0) {
    const int per_block = kLansThreads / kWave;
    const int rblocks = (T - tensor_base + per_block - 1) / per_block;
    lans_prepare_kernel<<<1, 64, 0, st>>>(t, sc);
    lans_norm_g_kernel<<<nsweep, kLansThreads, 0, st>>>(t, chunk_base);
    lans_reduce_kernel<<<rblocks, kLansThreads, 0, st>>>(t, 0, tensor_base, T, 1, 1);
    lans_moments_kernel<<<nsweep * kSweepSplit, kLansThreads, 0, st>>>(t, sc, chunk_base);
    lans_reduce_kernel<<<rblocks, kLansThreads, 0, st>>>(t, 1, tensor_base, T, 3, kSweepSplit);
    lans_update_kernel<<<nsweep * kSweepSplit, kLansThreads, 0, st>>>(t, sc, chunk_base);
  }
  return static_cast<int>(hipGetLastError());
}

extern "C" int lancet_lans_plan_set_schedule(lancet_lans_plan_t pl, int schedule) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (schedule != LANCET_LANS_SWEEPS && schedule != LANCET_LANS_RESIDENT) return LANCET_ERR_SHAPE;
  // a tensor's chunks must all be held by running workgroups at once; tensors too large for that go
  // through the sweeps inside the same step, and a plan made only of such tensors has no use for the kernel
  if (schedule == LANCET_LANS_RESIDENT && pl->n_res_chunks == 0 && pl->nchunks > 0) return LANCET_ERR_SHAPE;
  pl->schedule = schedule;
  return LANCET_OK;
}

extern "C" int lancet_lans_plan_resident_capacity(lancet_lans_plan_t pl, int* workgroups, int* max_tensor_chunks) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (workgroups) *workgroups = pl->resident_limit;
  if (max_tensor_chunks) *max_tensor_chunks = pl->max_tensor_chunks;
  return LANCET_OK;
}

extern "C" int lancet_lans_plan_error(lancet_lans_plan_t pl, lancet_stream_t stream, int* error_out) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (!error_out) return LANCET_ERR_NULL;
  uint32_t word = 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipError_t e = hipMemcpyAsync(&word, pl->tables.ticket + 1, sizeof(word), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  *error_out = static_cast<int>(word);
  return static_cast<int>(e);
}
