// Fused multi-tensor LANS step.  The reference makes six sweeps over the optimizer state
// (src/op/dialect/cuda/kernels/multi_tensor_lans.cu:401-450: l2norm(g), l2norm(p), stage 1,
// l2norm(u_m), l2norm(u_g), stage 2, 68 B/param of traffic).  Here the step has three phases
//   phase N  reads g               -> per-chunk sums of g^2
//   phase M  reads g, p, m, v      -> writes m, v; per-chunk sums of p^2, u_m^2 and u_g^2
//   phase U  reads g, p, m, v      -> recomputes u_m, u_g (never stored) and writes p
// and two schedules:
//   * sweeps: three plain launches + two tiny per-tensor reductions.  Real HBM traffic
//     is 48 B/param (g read three times, p, m, v twice).  No workgroup waits for another.
//   * resident (what a new plan runs): ONE persistent kernel in which every array is read once and written
//     once (28 B/param).  A workgroup runs a three-stage software pipeline over the chunks it draws from a
//     ticket: stage N loads g of a chunk into registers and publishes its sum of squares; stage M, one
//     iteration later, loads p, m, v of that chunk, writes m and v and keeps u_m, u_g in registers and p
//     in LDS; stage U, another iteration later, writes p.  Between the stages of one chunk the workgroup
//     works on its other two chunks, so the per-tensor norms a stage needs (||g|| for M; ||p||, ||u_m||,
//     ||u_g|| for U) have normally been published long before it asks for them.  Workgroups exchange
//     chunk partials as self-validating 64-bit words (step epoch in the high half, fp32 sum in the low
//     half, one agent-scope atomic store each); the workgroup that arrives last at a per-tensor counter
//     sums them in a fixed order and publishes the norms the same way.  Nothing else crosses
//     workgroups, so no fences are needed.  The plan packs tensors into rounds of as many chunks as the
//     device runs workgroups (padding a round rather than splitting a tensor over two), so that all
//     chunks of a tensor are drawn in the same pipeline iteration.  A workgroup waits only for chunks of
//     tensors it holds, chunks are drawn in order, and a workgroup holds at most two chunks that have not
//     passed stage M: the kernel drains as long as half as many workgroups as the largest tensor has
//     chunks are running.  Larger tensors go through the sweeps in the same step.  Waits are bounded; a
//     wait that gives up poisons what it would have fed, so that no parameter is written from an unknown
//     norm, and raises a sticky error the next step reports.
// Work is cut into fixed-size chunks described by device-resident tables built once per
// parameter set, instead of kernel arguments re-packed for every launch
// (multi_tensor_apply.cuh:39-92).  Chunk partials are combined in a fixed order in double
// precision, so each schedule is deterministic (the two differ in the last bits: a chunk's own sum is
// accumulated in a different order).
#include "launchers.hpp"
#include "common.hpp"
#include "../../include/lancet_hip_debug.h"
#include <algorithm>
#include <new>
#include <vector>

namespace lancet {

constexpr int kLansThreads = 256;
#ifndef LANCET_LANS_CHUNK
#define LANCET_LANS_CHUNK 8192
#endif
constexpr int kLansChunk = LANCET_LANS_CHUNK;  // elements per task: kLansChunk / 1024 float4 per thread and array
typedef float f32x4 __attribute__((ext_vector_type(4)));

// control words of a plan (uint32): [0] next ticket of the resident kernel, [1] error (sticky: only
// lancet_lans_plan_error clears it), [2] step epoch, [3] skip: the step that is running found the error word set
// when it began and leaves every array alone (a step queued behind one that stalled must not build on its
// half-applied state: moments written, parameters not)
constexpr int kCtlTicket = 0, kCtlError = 1, kCtlEpoch = 2, kCtlSkip = 3, kCtlWords = 4;

struct LansTables {
  const void* const* g;   // [T] device pointers; elements of the step's gradient type (fp32, bf16 or fp16)
  float* const* p;
  float* const* m;
  float* const* v;
  void* const* plow;      // [T] device pointers or unused: 16-bit copies of the new parameters, written with p
  const int64_t* numel;        // [T]
  const int32_t* chunk_tensor; // [nchunks] tensor of a chunk slot, -1 = padding slot of a round
  const int32_t* tensor_first; // [T] first chunk slot of each tensor (its chunks are consecutive)
  const int32_t* tensor_chunks;// [T] chunks of each tensor
  float* partial;              // [3][nchunks * kSweepSplit]  (sweeps: one sum per slice)
  uint64_t* part_word;         // [4][nchunks]      (resident schedule: tag | fp32 sum of squares)
  uint64_t* norm_word;         // [4][T]            (resident schedule: tag | fp32 norm)
  uint32_t* ctl;               // control words, see kCtl*
  uint32_t* host_status;       // device view of a pinned host word: set with the error word, read by the next step
  float* norms;                // [4][T]: g, p, u_m, u_g
  float* consts;               // [2]: bias_correction1, bias_correction2
  const int32_t* order;        // [T] position in the caller's lists of the plan's i-th tensor
  const float* grad_norms;     // [T] ||g|| per tensor in the caller's order, or null: computed by the step
  int T;
  int nchunks;                 // chunk slots, padding included
  int nres;                    // slots [0, nres) are handed out by the resident kernel
  uint32_t debug_flags;        // bit 0: nothing is published (exercises the bounded waits); bit 1 is the host's
};

struct LansScalars {
  float lr, beta1, beta2, beta3, eps, wd;
  int mode, normalize_grad, bias_correction;
  int step_host;
  const float* step_dev;
  uint32_t epoch;              // filled in on the device
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
  int tensor;     // -1: a padding slot
  int64_t begin;  // first element of the chunk inside the tensor
  int n;          // elements in the chunk
};

__device__ __forceinline__ ChunkView chunk_view(const LansTables& t, int chunk) {
  ChunkView c;
  c.tensor = t.chunk_tensor[chunk];
  c.begin = 0;
  c.n = 0;
  if (c.tensor >= 0) {
    c.begin = static_cast<int64_t>(chunk - t.tensor_first[c.tensor]) * kLansChunk;
    const int64_t left = t.numel[c.tensor] - c.begin;
    c.n = static_cast<int>(left < kLansChunk ? left : kLansChunk);
  }
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
// Divisions by a value the whole tensor shares (||g|| + eps, the two bias corrections) are multiplications
// by its correctly rounded reciprocal, and the two quotients over the same per-element denominator share one
// correctly rounded reciprocal: one division and one square root per element instead of five and one.  Each
// such product is within 1.5 ulp of the quotient the reference forms (0.5 ulp), far inside the 1e-6 the
// parameters are held to; a step is bound by memory only as long as the arithmetic stays this small.
struct LansElem {
  float inv_gnorm_eps;  // 1 / (||g|| + eps)
  bool normalize;       // normalize_grad && ||g|| != 0
  float beta1, beta2, beta3, one_minus_beta2, inv_bc1, inv_bc2, eps, wd;
  int mode;

  __device__ __forceinline__ float scaled_grad(float g, float p) const {
#pragma clang fp contract(off)
    float sg = g;
    if (normalize) sg = sg * inv_gnorm_eps;
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
    const float denom = sqrtf(v * inv_bc2) + eps;
    const float r = 1.f / denom;
    um = (m * inv_bc1) * r;
    ug = sg * r;
    if (mode != 0) {
      const float sp = wd * p;
      um = um + sp;
      ug = ug + sp;
    }
  }
};

__device__ __forceinline__ LansElem make_elem(const LansScalars& sc, float gn, float bc1, float bc2) {
  LansElem e;
  e.inv_gnorm_eps = uniform(1.f / (gn + sc.eps));
  e.normalize = sc.normalize_grad && uniform(gn) != 0.f;
  e.beta1 = sc.beta1;
  e.beta2 = sc.beta2;
  e.beta3 = sc.beta3;
  e.one_minus_beta2 = uniform(1.f - sc.beta2);
  e.inv_bc1 = uniform(1.f / bc1);
  e.inv_bc2 = uniform(1.f / bc2);
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

// ---- gradients and parameter copies of a 16-bit model ---------------------------------------------------------
// A mixed-precision trainer keeps fp32 master parameters and moments and a 16-bit model: the reference casts every
// gradient to fp32 in front of the op and every new parameter back behind it (python/raf/optim/lans.py:256-257,
// 285-288), two more sweeps over the state.  Here the step reads the gradients in the type they have (GT: the
// conversion to fp32 is exact, so every later value is what the cast would have given) and writes the 16-bit copy
// of a new parameter (PL; round to nearest even, what the cast does) with the fp32 one.  Four consecutive
// elements are one access: 16 bytes of fp32, 8 bytes of a 16-bit type.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
constexpr int kNoLowp = -1;  // PL: no 16-bit copy

template <int GT>
struct Grad {  // GT = LANCET_F32
  typedef float S;   // storage type of an element
  typedef f32x4 R;   // four consecutive elements as they are kept in registers
  static constexpr uintptr_t kAlign4 = 15u;  // alignment mask of a 4-element access
  static __device__ __forceinline__ float ld1(const LANCET_GLOBAL S* p) { return *p; }
  static __device__ __forceinline__ R ldr4(const LANCET_GLOBAL S* p) { return ldn((const LANCET_GLOBAL f32x4*)p); }
  static __device__ __forceinline__ f32x4 wide(const R& x) { return x; }
  static __device__ __forceinline__ f32x4 ld4(const LANCET_GLOBAL S* p) { return ldr4(p); }
};
template <int GT>
__device__ __forceinline__ float half_to_f32(uint32_t h) {
  return GT == LANCET_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
}
template <int GT>
struct GradHalf {
  typedef uint16_t S;
  typedef u32x2 R;   // kept packed: half the registers of the fp32 form, widened where a value is used
  static constexpr uintptr_t kAlign4 = 7u;
  static __device__ __forceinline__ float ld1(const LANCET_GLOBAL S* p) { return half_to_f32<GT>(*p); }
  static __device__ __forceinline__ R ldr4(const LANCET_GLOBAL S* p) {
    return __builtin_nontemporal_load((const LANCET_GLOBAL u32x2*)p);
  }
  static __device__ __forceinline__ f32x4 wide(const R& x) {
    return f32x4{half_to_f32<GT>(x.x & 0xffffu), half_to_f32<GT>(x.x >> 16), half_to_f32<GT>(x.y & 0xffffu),
                 half_to_f32<GT>(x.y >> 16)};
  }
  static __device__ __forceinline__ f32x4 ld4(const LANCET_GLOBAL S* p) { return wide(ldr4(p)); }
};
template <>
struct Grad<LANCET_BF16> : GradHalf<LANCET_BF16> {};
template <>
struct Grad<LANCET_F16> : GradHalf<LANCET_F16> {};

template <int PL>
__device__ __forceinline__ uint32_t f32_to_half(float f) {
  return PL == LANCET_BF16 ? f32_to_bf16(f) : f32_to_f16(f);
}
// the 16-bit copy of four consecutive new parameters (nothing for PL = kNoLowp)
template <int PL>
__device__ __forceinline__ void st_lowp4(LANCET_GLOBAL uint16_t* p, f32x4 x) {
  if (PL == kNoLowp) return;
  u32x2 y;
  y.x = (f32_to_half<PL>(x.x) & 0xffffu) | (f32_to_half<PL>(x.y) << 16);
  y.y = (f32_to_half<PL>(x.z) & 0xffffu) | (f32_to_half<PL>(x.w) << 16);
  __builtin_nontemporal_store(y, (LANCET_GLOBAL u32x2*)p);
}
template <int PL>
__device__ __forceinline__ void st_lowp1(LANCET_GLOBAL uint16_t* p, float x) {
  if (PL != kNoLowp) *p = static_cast<uint16_t>(f32_to_half<PL>(x));
}

// ---- the three phases on one chunk, executed by one workgroup ------------------------------
// phase 1: sum of squares of g (L2NormFunctor, multi_tensor_lans.cu:95-167); valid on thread 0.
// (The sum of squares of p is not needed before phase 3 and is taken in phase 2, which reads p anyway.)
template <int GT>
__device__ __forceinline__ float chunk_norm_g(const LansTables& t, const ChunkView& c, float* s_red) {
  typedef Grad<GT> G;
  const LANCET_GLOBAL typename G::S* g = as_global(static_cast<const typename G::S*>(t.g[c.tensor]) + c.begin);
  float ag = 0.f;
  int scalar_from = 0;
  if (((uintptr_t)g & G::kAlign4) == 0) {
    const int nv = c.n / 4;
#pragma unroll 8
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 x = G::ld4(g + 4 * i);
      ag += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
    }
    scalar_from = nv * 4;
  }
  for (int i = scalar_from + threadIdx.x; i < c.n; i += kLansThreads) {
    const float x = G::ld1(g + i);
    ag += x * x;
  }
  return block_sum(ag, s_red);
}

// phase 2: moments + sums of squares of p and of the two updates (LANSStage1Functor :207-322 and the
// l2norm sweeps around it, :428-441); sums valid on thread 0
template <int GT>
__device__ __forceinline__ void chunk_moments(const LansTables& t, const ChunkView& c, const LansElem& el,
                                              float* s_red, float& sum_p, float& sum_um, float& sum_ug) {
  typedef Grad<GT> G;
  const LANCET_GLOBAL typename G::S* g = as_global(static_cast<const typename G::S*>(t.g[c.tensor]) + c.begin);
  const LANCET_GLOBAL float* p = as_global(t.p[c.tensor] + c.begin);
  LANCET_GLOBAL float* m = as_global(t.m[c.tensor] + c.begin);
  LANCET_GLOBAL float* v = as_global(t.v[c.tensor] + c.begin);
  float ap = 0.f, am = 0.f, ag = 0.f;
  int scalar_from = 0;
  if (vec_ok(p, p, m, v) && ((uintptr_t)g & G::kAlign4) == 0) {
    const int nv = c.n / 4;
    const LANCET_GLOBAL f32x4* p4 = (const LANCET_GLOBAL f32x4*)p;
    LANCET_GLOBAL f32x4* m4 = (LANCET_GLOBAL f32x4*)m;
    LANCET_GLOBAL f32x4* v4 = (LANCET_GLOBAL f32x4*)v;
#pragma unroll 2
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 xg = G::ld4(g + 4 * i), xp = ldn(p4 + i);
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
    const float sg = el.scaled_grad(G::ld1(g + i), p[i]);
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
template <int GT, int PL>
__device__ __forceinline__ void chunk_update(const LansTables& t, const ChunkView& c, const LansElem& el,
                                             const LansScalars& sc, float pn, float umn, float ugn) {
  typedef Grad<GT> G;
  float ratio_m = (umn != 0.f && pn != 0.f) ? sc.lr * (pn / umn) : sc.lr;
  float ratio_g = (ugn != 0.f && pn != 0.f) ? sc.lr * (pn / ugn) : sc.lr;
  ratio_m *= sc.beta1;
  ratio_g *= sc.beta3;
  const LANCET_GLOBAL typename G::S* g = as_global(static_cast<const typename G::S*>(t.g[c.tensor]) + c.begin);
  LANCET_GLOBAL uint16_t* pl = PL == kNoLowp ? nullptr : as_global(static_cast<uint16_t*>(t.plow[c.tensor]) + c.begin);
  LANCET_GLOBAL float* p = as_global(t.p[c.tensor] + c.begin);
  const LANCET_GLOBAL float* m = as_global(t.m[c.tensor] + c.begin);
  const LANCET_GLOBAL float* v = as_global(t.v[c.tensor] + c.begin);
  int scalar_from = 0;
  if (vec_ok(p, p, m, v) && ((uintptr_t)g & G::kAlign4) == 0 && (PL == kNoLowp || ((uintptr_t)pl & 7u) == 0)) {
    const int nv = c.n / 4;
    LANCET_GLOBAL f32x4* p4 = (LANCET_GLOBAL f32x4*)p;
    const LANCET_GLOBAL f32x4* m4 = (const LANCET_GLOBAL f32x4*)m;
    const LANCET_GLOBAL f32x4* v4 = (const LANCET_GLOBAL f32x4*)v;
#pragma unroll 2
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 xg = G::ld4(g + 4 * i), xm = ldn(m4 + i), xv = ldn(v4 + i);
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
      st_lowp4<PL>(pl + 4 * i, xp);
    }
    scalar_from = nv * 4;
  }
  for (int i = scalar_from + threadIdx.x; i < c.n; i += kLansThreads) {
#pragma clang fp contract(off)
    const float sg = el.scaled_grad(G::ld1(g + i), p[i]);
    float um, ug;
    el.updates(sg, p[i], m[i], v[i], um, ug);
    const float np = p[i] - (ratio_m * um) - (ratio_g * ug);
    p[i] = np;
    st_lowp1<PL>(pl + i, np);
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
// A step begins by looking at the plan's sticky error word: if an earlier step gave up a wait, its tensors hold
// new moments and old parameters, and a step queued behind it (enqueued before the host could see the failure, or
// replayed from a graph) must not advance them again.  Such a step is skipped as a whole: every kernel of it reads
// the skip word first and leaves when it is set, until lancet_lans_plan_error has cleared the error.
__device__ __forceinline__ bool step_is_skipped(const LansTables& t) {
  return __builtin_amdgcn_readfirstlane(static_cast<int>(ld_agent(t.ctl + kCtlSkip))) != 0;
}

__global__ void lans_prepare_kernel(LansTables t, LansScalars sc) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    t.ctl[kCtlSkip] = ld_agent(t.ctl + kCtlError) != 0u ? 1u : 0u;
    bias_corrections(sc, t.consts[0], t.consts[1]);
  }
}

// The sweeps hand every chunk to kSweepSplit workgroups (a slice of kLansChunk / kSweepSplit elements each:
// one float4 per thread and array).  Short workgroups in address order stream a few percent faster than
// workgroups that loop over a whole chunk; the chunk stays the unit of the tables and of the resident kernel.
#ifndef LANCET_SWEEP_SPLIT
#define LANCET_SWEEP_SPLIT (LANCET_LANS_CHUNK / 1024)
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
template <int GT>
__global__ __launch_bounds__(kLansThreads) void lans_norm_g_kernel(LansTables t, int chunk_base) {
  __shared__ float s_red[kLansThreads / kWave];
  if (step_is_skipped(t)) return;
  const int chunk = chunk_base + blockIdx.x;  // a whole chunk per workgroup: this sweep only reads, and splitting it costs more in reductions than it gains
  const ChunkView c = chunk_view(t, chunk);
  if (c.tensor < 0) return;  // padding slot (uniform over the workgroup)
  const float sg = chunk_norm_g<GT>(t, c, s_red);
  if (threadIdx.x == 0) t.partial[chunk] = sg;
}

// per-tensor sqrt(sum of chunk partials) (cleanup, multi_tensor_lans.cu:169-185)
// split: partial sums per chunk (1 after the sweep over g, kSweepSplit after the moments sweep)
__global__ __launch_bounds__(kLansThreads) void lans_reduce_kernel(LansTables t, int first_norm, int tensor_base,
                                                                   int tensor_end, int count, int split) {
  if (step_is_skipped(t)) return;  // the norms of the last step that ran stay
  const int tensor = tensor_base + blockIdx.x * (kLansThreads / kWave) + threadIdx.x / kWave;
  if (tensor >= tensor_end) return;
  const int lo = t.tensor_first[tensor], hi = lo + t.tensor_chunks[tensor];
  for (int k = 0; k < count; ++k) {
    const float* part = t.partial + static_cast<size_t>(k) * t.nchunks * split;
    const float n = wave_norm(lo * split, hi * split, [&](int c) { return part[c]; });
    if (lane_id() == 0) t.norms[(first_norm + k) * t.T + tensor] = n;
  }
}

template <int GT>
__global__ __launch_bounds__(kLansThreads) void lans_moments_kernel(LansTables t, LansScalars sc, int chunk_base) {
  __shared__ float s_red[kLansThreads / kWave];
  if (step_is_skipped(t)) return;
  int slot;
  const ChunkView c = slice_view(t, chunk_base, slot);
  if (c.tensor < 0) return;  // padding slot (uniform over the workgroup)
  const LansElem el = make_elem(sc, t.norms[c.tensor], t.consts[0], t.consts[1]);
  float sp, sm, sg;
  chunk_moments<GT>(t, c, el, s_red, sp, sm, sg);
  if (threadIdx.x == 0) {
    const size_t row = static_cast<size_t>(t.nchunks) * kSweepSplit;
    t.partial[slot] = sp;
    t.partial[row + slot] = sm;
    t.partial[2 * row + slot] = sg;
  }
}

template <int GT, int PL>
__global__ __launch_bounds__(kLansThreads) void lans_update_kernel(LansTables t, LansScalars sc, int chunk_base) {
  if (step_is_skipped(t)) return;
  int slot;
  const ChunkView c = slice_view(t, chunk_base, slot);
  if (c.tensor < 0) return;
  const LansElem el = make_elem(sc, t.norms[c.tensor], t.consts[0], t.consts[1]);
  chunk_update<GT, PL>(t, c, el, sc, t.norms[1 * t.T + c.tensor], t.norms[2 * t.T + c.tensor], t.norms[3 * t.T + c.tensor]);
}

// ||g|| per tensor supplied by the caller (in the order of its lists) instead of the sweep over g
__global__ void lans_take_grad_norms_kernel(LansTables t) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (step_is_skipped(t)) return;
  if (i < t.T) t.norms[i] = t.grad_norms[t.order[i]];
}

// norms live in the plan's tensor order; callers get them in the order of their lists
__global__ void lans_gather_norms_kernel(LansTables t, float* dst) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= t.T) return;
#pragma unroll
  for (int k = 0; k < 4; ++k) dst[k * t.T + t.order[i]] = t.norms[k * t.T + i];
}

// =======================================================================================
// words published between workgroups: a tag in the high half (bit 31: poisoned, bits 0..30: the
// step epoch), an fp32 value in the low half
// =======================================================================================
constexpr uint32_t kPoison = 0x80000000u;

__device__ __forceinline__ uint64_t ld_word(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_word(uint64_t* p, uint32_t tag, float v) {
  __hip_atomic_store(p, (static_cast<uint64_t>(tag) << 32) | __float_as_uint(v), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// sticky: the device word for lancet_lans_plan_error, the pinned host word for the next lancet_lans_step
__device__ __forceinline__ void flag_error(const LansTables& t) {
  st_agent(t.ctl + kCtlError, 1u);
  __hip_atomic_store(t.host_status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ __forceinline__ bool word_is_current(uint64_t x, uint32_t epoch) {
  return (static_cast<uint32_t>(x >> 32) & ~kPoison) == epoch;
}
__device__ __forceinline__ bool word_is_poisoned(uint64_t x) { return (static_cast<uint32_t>(x >> 32) & kPoison) != 0; }

// =======================================================================================
// schedule "resident": one persistent kernel, a three-stage software pipeline per workgroup
// =======================================================================================
constexpr int kVecPerThread = kLansChunk / 4 / kLansThreads;  // float4 per thread and array
constexpr int kPrefetch = 3;  // float4 of each array stage M keeps in flight ahead of the one it works on
#define LIKELY(x) __builtin_expect(!!(x), 1)
#define UNLIKELY(x) __builtin_expect(!!(x), 0)

// The thread's place in its workgroup, formed anew wherever it is needed: the wave's index is handed down in a
// scalar register and the lane's number costs two instructions.  A value kept in a vector register from the
// start of the kernel gets spilled in this code, and a reload that follows stores waits for all of them.
__device__ __forceinline__ int fresh_lane() {
  int l;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
  return l;
}
__device__ __forceinline__ int fresh_tid(int wave) { return wave * kWave + fresh_lane(); }
__device__ __forceinline__ bool is_first(int wave) { return (fresh_lane() | wave) == 0; }  // thread 0, in one vector compare

// Workgroup barrier that orders LDS accesses only.  __syncthreads() also waits for every global load and
// store the wave has in flight, which would drain the streams of this kernel several times per chunk; all
// that crosses the waves of a workgroup here is in LDS (global words other workgroups read are atomics).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

constexpr int kMaxResidentChunks = 4 * 1024 * 1024 / kLansChunk;      // chunks of the largest tensor the kernel takes (4M parameters)
constexpr int kGatherPerThread = kMaxResidentChunks / kLansThreads;  // partials of one norm a thread reads
static_assert(kLansThreads / kWave == 4, "one wave per norm");

struct PipeShared {
  f32x4 p[2][kVecPerThread][kLansThreads];  // parameters of the two chunks between stages M and U, one private slot per thread and float4
  float part[4][kMaxResidentChunks];        // chunk partials: [0] of s2's tensor (g^2), [1..3] of s0's (p^2, u_m^2, u_g^2)
  float red[3][kLansThreads / kWave];
  float norm[4];   // [1..3]: the norms stage U of this pass needs
  float g_next;    // ||g|| of s2's tensor: for stage M of the next pass
  int g_next_bad;  // ... is unknown
  int u_bad;       // a norm of s0's tensor is unknown
  int retry;             // a sum read ahead was not there yet
  int give_up;           // ... and never came (sticky for the rest of the kernel)
  int chunk;
};

// a chunk a workgroup holds between stages; every field is uniform over the workgroup
struct Slot {
  int chunk;   // -1: empty (the ticket ran out)
  int tensor;  // -1: padding slot, nothing to do
  int dead;    // stage M was skipped (||g|| unknown): the parameters stay as they are
  int lo, nc;  // first chunk slot and number of chunks of the tensor
  int64_t begin;
  __device__ __forceinline__ bool real() const { return chunk >= 0 && tensor >= 0; }
};

// The resident kernel only takes whole chunks of 16-byte aligned arrays (the plan leaves tensors that are not a
// multiple of the chunk to the sweeps; a step whose pointers are not aligned runs as sweeps altogether): every
// access is an unconditional, non-temporal float4.
// A table entry (tensor pointers, chunk tables) read as constant memory: nothing writes the tables while a
// kernel runs, and said this way the read goes through the scalar unit and its result stays in scalar
// registers.  A plain read behind the kernel's own stores has to assume they changed the table, takes the
// vector unit, and every pointer it yields costs two vector registers for as long as it lives.
template <typename T>
__device__ __forceinline__ T ld_table(const T* p) {
  return *(const __attribute__((address_space(4))) T*)(p);
}

// float4 k of a thread: the wave's quarter of the chunk starts lane_offset() elements into it, float4 k lies
// k * 256 elements further on (one load instruction of a wave covers 1 KB of consecutive memory).  The
// address is a uniform 64-bit base plus an unsigned 32-bit offset per lane, the form that takes its base
// from scalar registers and one vector register for the offset.
__device__ __forceinline__ uint32_t lane_offset(int wave) {
  return static_cast<uint32_t>(wave * (kLansChunk / kWavesPerTile) + 4 * fresh_lane());
}
__device__ __forceinline__ f32x4 ld_chunk4(const LANCET_GLOBAL float* a, int k, int wave) {
  return __builtin_nontemporal_load((const LANCET_GLOBAL f32x4*)(a + k * (4 * kWave) + lane_offset(wave)));
}
__device__ __forceinline__ void st_chunk4(LANCET_GLOBAL float* a, int k, f32x4 x, int wave) {
  __builtin_nontemporal_store(x, (LANCET_GLOBAL f32x4*)(a + k * (4 * kWave) + lane_offset(wave)));
}
// the same four elements of a gradient chunk in its own type, as fp32, and of the 16-bit parameter copy
template <int GT>
__device__ __forceinline__ typename Grad<GT>::R ld_grad4(const LANCET_GLOBAL typename Grad<GT>::S* a, int k, int wave) {
  return Grad<GT>::ldr4(a + k * (4 * kWave) + lane_offset(wave));
}
template <int PL>
__device__ __forceinline__ void st_lowp_chunk4(LANCET_GLOBAL uint16_t* a, int k, f32x4 x, int wave) {
  st_lowp4<PL>(a + k * (4 * kWave) + lane_offset(wave), x);
}

// Thread 0: publishes the N chunk sums a[] of slot s as words first .. first+N-1 (fire and forget).
template <int N>
__device__ __forceinline__ void publish(const LansTables& t, const LansScalars& sc, int first, const Slot& s,
                                        const float (&a)[N], bool poison) {
  if (t.debug_flags & 1u) return;  // test hook: nothing is ever published, every wait runs into its bound
  const uint32_t tag = sc.epoch | (poison ? kPoison : 0u);
#pragma unroll
  for (int k = 0; k < N; ++k) st_word(t.part_word + static_cast<size_t>(first + k) * t.nchunks + s.chunk, tag, a[k]);
}

// the partials of one norm of slot s's tensor as this thread reads them (issued, not yet looked at)
__device__ __forceinline__ void gather_issue(const LansTables& t, int kind, const Slot& s, uint64_t (&word)[kGatherPerThread], int wave) {
  const uint64_t* src = t.part_word + static_cast<size_t>(kind) * t.nchunks + s.lo;
#pragma unroll
  for (int i = 0; i < kGatherPerThread; ++i) {
    const int c = fresh_tid(wave) + i * kLansThreads;
    word[i] = c < s.nc ? ld_word(src + c) : 0;
  }
}
// ... looked at: values into LDS.  Bit first_bit + i of `missing` is set for a word that is not of this step
// yet; `poisoned` for one that is and carries the poison mark.
__device__ __forceinline__ void gather_take(const LansScalars& sc, const Slot& s, const uint64_t (&word)[kGatherPerThread],
                                            float* part, int first_bit, uint32_t& missing, bool& poisoned, int wave) {
#pragma unroll
  for (int i = 0; i < kGatherPerThread; ++i) {
    const int c = fresh_tid(wave) + i * kLansThreads;
    if (c < s.nc) {
      part[c] = __uint_as_float(static_cast<uint32_t>(word[i]));
      const bool there = word_is_current(word[i], sc.epoch);
      if (!there) missing |= 1u << (first_bit + i);
      poisoned = poisoned || (there && word_is_poisoned(word[i]));
    }
  }
}

// Moments and the two updates (LANSStage1Functor, multi_tensor_lans.cu:207-322, and the l2norm sweeps
// around it, :428-441) of a chunk whose g sits in registers.  m and v are written; u_m, u_g stay in
// registers and p in LDS for stage U.  The loads of float4 k+1 are issued before the stores of float4 k:
// memory operations of a wave complete in order, so a load behind a store would wait for it.
template <int PAR, int GT>
__device__ __forceinline__ void moments_chunk(const LansTables& t, const Slot& s, const LansElem& el,
                                              const typename Grad<GT>::R (&g)[kVecPerThread], f32x4 (&um)[kVecPerThread],
                                              f32x4 (&ug)[kVecPerThread], PipeShared& sh, float (&a)[3], uint32_t ticket, int wave) {
  const LANCET_GLOBAL float* p = as_global(ld_table(t.p + s.tensor) + s.begin);
  LANCET_GLOBAL float* m = as_global(ld_table(t.m + s.tensor) + s.begin);
  LANCET_GLOBAL float* v = as_global(ld_table(t.v + s.tensor) + s.begin);
  float a0 = 0.f, a1 = 0.f, a2 = 0.f;
  // kPrefetch float4 of each array are in flight ahead of the one being worked on
  f32x4 np[kPrefetch], nm[kPrefetch], nv[kPrefetch];
#pragma unroll
  for (int d = 0; d < kPrefetch; ++d) {
    np[d] = ld_chunk4(p, d, wave);
    nm[d] = ld_chunk4(m, d, wave);
    nv[d] = ld_chunk4(v, d, wave);
  }
  // the ticket drawn at the start of the pass is looked at here, behind the first loads and in front of every
  // store of the stage: looked at behind the stores it would cost their completion
  if (is_first(wave)) sh.chunk = static_cast<int>(ticket);
#pragma unroll
  for (int k = 0; k < kVecPerThread; ++k) {
    const f32x4 xp = np[k % kPrefetch];
    f32x4 xm = nm[k % kPrefetch], xv = nv[k % kPrefetch];
    if (k + kPrefetch < kVecPerThread) {
      np[k % kPrefetch] = ld_chunk4(p, k + kPrefetch, wave);
      nm[k % kPrefetch] = ld_chunk4(m, k + kPrefetch, wave);
      nv[k % kPrefetch] = ld_chunk4(v, k + kPrefetch, wave);
    }
    sh.p[PAR][k][fresh_tid(wave)] = xp;
    const f32x4 xg = Grad<GT>::wide(g[k]);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float sg = el.scaled_grad(xg[j], xp[j]);
      float mm = xm[j], vv = xv[j], u0, u1;
      el.moments(sg, mm, vv);
      el.updates(sg, xp[j], mm, vv, u0, u1);
      // the two updates are final here: nothing of their computation may be left for stage U (the
      // compiler otherwise carries a third value per element, wd * p, across the stages and spills)
      asm volatile("" : "+v"(u0), "+v"(u1));
      xm[j] = mm;
      xv[j] = vv;
      um[k][j] = u0;
      ug[k][j] = u1;
      a0 += xp[j] * xp[j];
      a1 += u0 * u0;
      a2 += u1 * u1;
    }
    st_chunk4(m, k, xm, wave);
    st_chunk4(v, k, xv, wave);
    // the sums are up to date here: left to itself the compiler keeps every p of the chunk in registers and
    // adds the squares up at the end of the stage
    asm volatile("" : "+v"(a0), "+v"(a1), "+v"(a2));
  }
  a[0] = a0;
  a[1] = a1;
  a[2] = a2;
}

// The slow path of a pass's gather: some of the sums this workgroup needs are not published yet.  Every
// thread reads the words it misses again (bit kind * kGatherPerThread + i of `missing`: word i of its share of
// that kind; lo_g / lo_u: first chunk slot of the tensor whose g sums / whose other sums are gathered) until
// they are all there, or until the bound.  A function of its own on purpose: it runs rarely, is full of
// loops, and inlined it misleads the register allocation of the straight-line code around it.
__device__ __noinline__ void regather(const uint64_t* part_word, int nchunks, uint32_t* ctl, uint32_t* host_status,
                                      uint32_t epoch, uint32_t spin_limit, int lo_g, int lo_u, uint32_t missing,
                                      PipeShared* shp, int wave) {
  PipeShared& sh = *shp;
#pragma unroll 1
  for (uint32_t spins = 1;; ++spins) {
    lds_barrier();  // everyone has seen the flag
    if (is_first(wave)) {
      sh.retry = 0;
      if (sh.give_up != 0 || spins > spin_limit || ((spins & 15u) == 0u && ld_agent(ctl + kCtlError) != 0u)) {
        st_agent(ctl + kCtlError, 1u);
        __hip_atomic_store(host_status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        sh.give_up = 1;
      }
    }
    lds_barrier();
    if (__builtin_amdgcn_readfirstlane(sh.give_up) != 0) {
      if (missing >> kGatherPerThread) sh.u_bad = 1;
      if (missing & ((1u << kGatherPerThread) - 1u)) sh.g_next_bad = 1;
      lds_barrier();
      return;
    }
    __builtin_amdgcn_s_sleep(16);
#pragma unroll 1
    for (uint32_t left = missing; left != 0u; left &= left - 1u) {
      const int bit = __builtin_ctz(left);
      const int kind = bit / kGatherPerThread;
      const int c = fresh_tid(wave) + (bit % kGatherPerThread) * kLansThreads;
      const uint64_t x = ld_word(part_word + static_cast<size_t>(kind) * nchunks + (kind == 0 ? lo_g : lo_u) + c);
      if (word_is_current(x, epoch)) {
        missing &= ~(1u << bit);
        sh.part[kind][c] = __uint_as_float(static_cast<uint32_t>(x));
        if (word_is_poisoned(x)) {
          if (kind == 0) sh.g_next_bad = 1; else sh.u_bad = 1;
        }
      }
    }
    if (missing != 0u) sh.retry = 1;
    lds_barrier();
    if (__builtin_amdgcn_readfirstlane(sh.retry) == 0) return;
  }
}

// wave_norm over nc <= kMaxResidentChunks sums in LDS: the same additions in the same order (a sum that is not
// there counts as +0, which changes no bit of a sum of squares), with all of a lane's reads issued at once.
__device__ __forceinline__ float wave_norm_lds(const float* part, int nc) {
  float x[kMaxResidentChunks / kWave];
#pragma unroll
  for (int i = 0; i < kMaxResidentChunks / kWave; ++i) {
    const int c = fresh_lane() + i * kWave;
    x[i] = c < nc ? part[c] : 0.f;
  }
  double acc = 0.0;
#pragma unroll
  for (int i = 0; i < kMaxResidentChunks / kWave; ++i) acc += static_cast<double>(x[i]);
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
  return static_cast<float>(sqrt(acc));
}

// Gives register arrays a value on the paths that do not fill them.  Without it the value they held before
// would count as still needed there, and with it the registers, all through the stage in front.
__device__ __forceinline__ void forget(f32x4 (&a)[kVecPerThread], f32x4 (&b)[kVecPerThread]) {
#pragma unroll
  for (int k = 0; k < kVecPerThread; ++k) a[k] = b[k] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// One pass of the pipeline: stage M on s1 (its g in `g`; its updates go to um_new / ug_new, its parameters to
// sh.p[PAR]), stage N on a newly drawn slot, whose g goes into `g`, which stage M has just used up, stage U
// on s0 (updates in um_old / ug_old, parameters in sh.p[PAR ^ 1]); then the slots move up.  Consecutive
// passes alternate between the two g arrays and between the two parities.
//
// Norms.  Every workgroup publishes the sums of its chunks (one word for stage N, three for stage M) and
// every workgroup forms the norms it needs itself, from the published sums of all the tensor's chunks, in
// the fixed order of wave_norm: they all get the same bits, nobody waits for a workgroup in charge, and the
// workgroup that is behind the others has no more to do than they.  A tensor has at most
// kMaxResidentChunks chunks: kGatherPerThread words per thread and norm.
//
// Memory operations of a wave complete in order, and under load a round trip takes microseconds: a value
// that comes from memory is free when it is asked for before a stage's loads and looked at after them, and
// costs a drain of the wave's stores when it is looked at behind them.  So the ticket is drawn at the start
// of the pass and looked at behind the first loads of stage M, and the sums of other workgroups are read in
// front of the loads of stage N and looked at behind them: those of s0's tensor, whose stage M was a pass
// ago, for the stage U that follows, and those of s2's, whose stage N was a pass ago, for stage M of the
// next pass (the norm is carried there in LDS; a register carried over would be looked at behind stage U's
// stores).  Only a sum that is still missing then is polled for.  Returns false when the workgroup holds
// nothing any more.
template <int PAR, int GT, int PL>
__device__ __forceinline__ bool pipeline_pass(const LansTables& t, const LansScalars& sc, float bc1, float bc2,
                                              Slot& s0, Slot& s1, Slot& s2,
                                              typename Grad<GT>::R (&g)[kVecPerThread],
                                              f32x4 (&um_new)[kVecPerThread], f32x4 (&ug_new)[kVecPerThread],
                                              const f32x4 (&um_old)[kVecPerThread], const f32x4 (&ug_old)[kVecPerThread],
                                              PipeShared& sh, int wave) {
  const bool own_norms = t.grad_norms == nullptr;
  // ---- start of the pass ---------------------------------------------------------------------------------
  lds_barrier();
  float g_norm = 0.f;
  bool bad = false;
  if (LIKELY(s1.real())) {
    if (own_norms) {
      g_norm = sh.g_next;  // formed at the end of the pass before
      bad = __builtin_amdgcn_readfirstlane(sh.g_next_bad) != 0;
    } else {
      g_norm = t.norms[s1.tensor];  // copied from the caller's array before this kernel
    }
  }
  uint32_t ticket = 0u;  // thread 0: for this pass's stage N
  if (is_first(wave)) ticket = atomicAdd(t.ctl + kCtlTicket, 1u);
  // ---- stage M on s1 ---------------------------------------------------------------------------------------
  if (LIKELY(s1.real())) {
    float a[3] = {0.f, 0.f, 0.f};
    if (LIKELY(!bad)) {
      const LansElem el = make_elem(sc, g_norm, bc1, bc2);
      moments_chunk<PAR, GT>(t, s1, el, g, um_new, ug_new, sh, a, ticket, wave);
    } else {
      if (is_first(wave)) sh.chunk = static_cast<int>(ticket);
      s1.dead = 1;  // ||g|| is unknown: the chunk is left as it is, and so will its tensor's parameters be
      forget(um_new, ug_new);
    }
#pragma unroll
    for (int k = 0; k < 3; ++k) a[k] = wave_sum(a[k]);
    if (fresh_lane() == 0) {
#pragma unroll
      for (int k = 0; k < 3; ++k) sh.red[k][wave] = a[k];
    }
    lds_barrier();
    if (is_first(wave)) {
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        float r = 0.f;
#pragma unroll
        for (int w = 0; w < kLansThreads / kWave; ++w) r += sh.red[k][w];
        a[k] = r;
      }
      publish<3>(t, sc, 1, s1, a, bad);
    }
  } else {
    if (is_first(wave)) sh.chunk = static_cast<int>(ticket);
    forget(um_new, ug_new);
  }
  // ---- stage N on a new slot -------------------------------------------------------------------------------
  uint64_t words_g[kGatherPerThread], words_u[3][kGatherPerThread];
  const bool need_u = s0.real();
  const bool need_g = s2.real() && own_norms;
  if (is_first(wave)) {
    sh.u_bad = 0;
    sh.g_next_bad = 0;
    sh.retry = 0;
  }
  lds_barrier();
  Slot s3;
  {
    // one value for the whole workgroup, and known to be: pointers and sizes derived from it stay scalar
    const int chunk = __builtin_amdgcn_readfirstlane(sh.chunk);
    s3.chunk = (chunk >= 0 && chunk < t.nres) ? chunk : -1;
    s3.tensor = -1;
    s3.dead = 0;
    if (s3.chunk >= 0) {
      s3.tensor = ld_table(t.chunk_tensor + s3.chunk);
      if (s3.tensor >= 0) {
        s3.lo = ld_table(t.tensor_first + s3.tensor);
        s3.nc = ld_table(t.tensor_chunks + s3.tensor);
        s3.begin = static_cast<int64_t>(s3.chunk - s3.lo) * kLansChunk;
      }
    }
  }
  // g of the chunk into registers (L2NormFunctor, multi_tensor_lans.cu:95-167) and, right behind those loads,
  // the sums other workgroups have published: read as late as possible, and still back before anything waits
  // for them alone
  if (LIKELY(s3.real())) {
    typedef typename Grad<GT>::S GS;
    const LANCET_GLOBAL GS* src = as_global(static_cast<const GS*>(ld_table(t.g + s3.tensor)) + s3.begin);
#pragma unroll
    for (int k = 0; k < kVecPerThread; ++k) g[k] = ld_grad4<GT>(src, k, wave);
  }
  if (LIKELY(need_u)) {
#pragma unroll
    for (int k = 0; k < 3; ++k) gather_issue(t, 1 + k, s0, words_u[k], wave);
  }
  if (LIKELY(need_g)) gather_issue(t, 0, s2, words_g, wave);
  if (LIKELY(s3.real())) {
    float a = 0.f;
#pragma unroll
    for (int k = 0; k < kVecPerThread; ++k) {
      const f32x4 x = Grad<GT>::wide(g[k]);
      a += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
    }
    a = wave_sum(a);
    if (fresh_lane() == 0) sh.red[0][wave] = a;
  }
  // ---- the norms ---------------------------------------------------------------------------------------------
  // bit kind * kGatherPerThread + i: word i of this thread's share of that norm's sums is still missing
  uint32_t missing = 0u;
  {
    bool poisoned_u = false, poisoned_g = false;
    if (LIKELY(need_u)) {
#pragma unroll
      for (int k = 1; k < 4; ++k) gather_take(sc, s0, words_u[k - 1], sh.part[k], k * kGatherPerThread, missing, poisoned_u, wave);
    }
    if (LIKELY(need_g)) gather_take(sc, s2, words_g, sh.part[0], 0, missing, poisoned_g, wave);
    if (UNLIKELY(poisoned_u)) sh.u_bad = 1;
    if (UNLIKELY(poisoned_g)) sh.g_next_bad = 1;
    if (UNLIKELY(missing != 0u)) sh.retry = 1;
  }
  lds_barrier();
  if (is_first(wave) && s3.real() && own_norms) {
    float r = 0.f;
#pragma unroll
    for (int w = 0; w < kLansThreads / kWave; ++w) r += sh.red[0][w];
    const float sums[1] = {r};
    publish<1>(t, sc, 0, s3, sums, false);
  }
  // A workgroup that is ahead of one it depends on gets here before that one has published.  Its threads
  // read the words they miss again (only those: hundreds of workgroups wait like this at any time, and what
  // they read while they wait competes with the one they wait for) until they are all there.  Bounded; and
  // once any wait of the plan has given up the others stop at their next look, so that a stalled step ends
  // after about one bound, not one per chunk.
  if (UNLIKELY(__builtin_amdgcn_readfirstlane(sh.retry) != 0)) {
    regather(t.part_word, t.nchunks, t.ctl, t.host_status, sc.epoch, sc.spin_limit, s2.lo, s0.lo, missing, &sh, wave);
  }
  {
    const int w = wave;  // wave w sums norm w: the same fixed order in every workgroup
    if (w == 0) {
      if (need_g) {
        const float n = wave_norm_lds(sh.part[0], s2.nc);
        if (fresh_lane() == 0) {
          sh.g_next = n;
          if (s2.chunk == s2.lo) t.norms[s2.tensor] = n;  // for lancet_lans_plan_norms
        }
      }
    } else if (need_u) {
      const float n = wave_norm_lds(sh.part[w], s0.nc);
      if (fresh_lane() == 0) {
        sh.norm[w] = n;
        if (s0.chunk == s0.lo) t.norms[w * t.T + s0.tensor] = n;
      }
    }
  }
  lds_barrier();
  // ---- stage U on s0 ---------------------------------------------------------------------------------------
  // Trust ratios and the parameter update (LANSStage2Functor, multi_tensor_lans.cu:326-399) from the updates
  // in registers and the parameters in LDS.  Nothing is written unless all three norms are known.
  if (LIKELY(need_u && !s0.dead && __builtin_amdgcn_readfirstlane(sh.u_bad) == 0)) {
    const float pn = uniform(sh.norm[1]), umn = uniform(sh.norm[2]), ugn = uniform(sh.norm[3]);
    float ratio_m = (umn != 0.f && pn != 0.f) ? sc.lr * (pn / umn) : sc.lr;
    float ratio_g = (ugn != 0.f && pn != 0.f) ? sc.lr * (pn / ugn) : sc.lr;
    ratio_m = uniform(ratio_m * sc.beta1);
    ratio_g = uniform(ratio_g * sc.beta3);
    LANCET_GLOBAL float* p = as_global(ld_table(t.p + s0.tensor) + s0.begin);
    LANCET_GLOBAL uint16_t* pl = nullptr;
    if (PL != kNoLowp) pl = as_global(static_cast<uint16_t*>(ld_table(t.plow + s0.tensor)) + s0.begin);
#pragma unroll
    for (int k = 0; k < kVecPerThread; ++k) {
      f32x4 xp = sh.p[PAR ^ 1][k][fresh_tid(wave)];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma clang fp contract(off)
        xp[j] = xp[j] - (ratio_m * um_old[k][j]) - (ratio_g * ug_old[k][j]);
      }
      st_chunk4(p, k, xp, wave);
      st_lowp_chunk4<PL>(pl, k, xp, wave);
    }
  }
  // ---- the slots move up ------------------------------------------------------------------------------------
  s0 = s1;
  s1 = s2;
  s2 = s3;
  return s0.chunk >= 0 || s1.chunk >= 0 || s2.chunk >= 0;
}

// Workgroups per CU = waves per SIMD: with two, a wave has 256 registers for g of two chunks, u_m and u_g of
// two more (one of them being filled from the first g) and the sums read ahead, and a workgroup 64 KB of
// LDS for parameters.
constexpr int kResidentWavesPerSimd = 2;

// Start of a resident step: clears the ticket, moves the step epoch on and forms the two bias corrections
// (pow in double: kept out of the resident kernel, whose registers are all spoken for).  The epoch lives on the device so
// that a step recorded in a graph tags every replay differently; when it wraps (2^31 steps) every word of
// earlier steps is forgotten.  The error word is left alone.
__global__ __launch_bounds__(kLansThreads) void lans_begin_kernel(LansTables t, LansScalars sc, size_t nwords) {
  uint32_t* ep = t.ctl + kCtlEpoch;
  const uint32_t e = (*ep + 1u) & ~kPoison;
  if (e == 0u)
    for (size_t k = threadIdx.x; k < nwords; k += kLansThreads) t.part_word[k] = 0;
  __syncthreads();
  if (threadIdx.x == 0) {
    *ep = e == 0u ? 1u : e;
    t.ctl[kCtlTicket] = 0u;
    t.ctl[kCtlSkip] = ld_agent(t.ctl + kCtlError) != 0u ? 1u : 0u;  // step_is_skipped
    bias_corrections(sc, t.consts[0], t.consts[1]);
  }
}

template <int GT, int PL>
__global__ __launch_bounds__(kLansThreads, kResidentWavesPerSimd) void lans_resident_kernel(LansTables t, LansScalars sc) {
  __shared__ PipeShared sh;
  if (step_is_skipped(t)) return;
  const int wave = static_cast<int>(static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(threadIdx.x)) / kWave);
  sc.epoch = __builtin_amdgcn_readfirstlane(t.ctl[kCtlEpoch]);
  const float bc1 = uniform(t.consts[0]), bc2 = uniform(t.consts[1]);  // lans_begin_kernel
  // s0: between stages M and U; s1, s2: between stages N and M, s1 the older.  Register arrays rotate with
  // the slots: g of s1 / s2 alternates between ga and gb, the updates between parity 0 and 1.
  typename Grad<GT>::R ga[kVecPerThread], gb[kVecPerThread];
  f32x4 um0[kVecPerThread], ug0[kVecPerThread], um1[kVecPerThread], ug1[kVecPerThread];
  Slot s0, s1, s2;
  s0.chunk = s1.chunk = s2.chunk = -1;
  s0.tensor = s1.tensor = s2.tensor = -1;
  s0.dead = s1.dead = s2.dead = 0;
  if (threadIdx.x == 0) {
    sh.g_next = 0.f;
    sh.g_next_bad = 0;
    sh.give_up = 0;
  }
  // the first two passes find empty slots (their stages M and U have nothing to do) and fill the pipeline;
  // every pass draws a ticket, tickets run out, and every wait is bounded: all workgroups leave
  for (;;) {
    if (!pipeline_pass<0, GT, PL>(t, sc, bc1, bc2, s0, s1, s2, ga, um0, ug0, um1, ug1, sh, wave)) break;
    if (!pipeline_pass<1, GT, PL>(t, sc, bc1, bc2, s0, s1, s2, gb, um1, ug1, um0, ug0, sh, wave)) break;
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
  int nchunks;                      // chunk slots, padding included
  std::vector<int64_t> numels;
  std::vector<const void*> shadow;  // last uploaded 5T pointers (g, p, m, v, 16-bit parameter copies or null)
  void* dev_block;                  // one allocation holding every table
  void** h_ptrs;                    // pinned staging for the pointer tables
  uint32_t* h_status;               // pinned word the resident kernel sets with its error word
  hipEvent_t upload_done;
  bool upload_pending;
  LansTables tables;
  int schedule;           // LANCET_LANS_SWEEPS or LANCET_LANS_RESIDENT
  int resident_grid;      // workgroups of the resident schedule the device runs at once
  int max_tensor_chunks;  // chunks of the largest tensor
  int resident_limit;     // chunks of the largest tensor the resident schedule takes on this device
  int n_res_tensors;      // tensors within that limit: the first ones in the plan's own order
  int n_res_chunks;       // chunk slots the resident kernel hands out (padding included)
  std::vector<int32_t> order;  // plan position -> position in the caller's lists
  std::vector<char> is_resident;  // by position in the caller's lists: the resident kernel takes this tensor
  size_t words_bytes;
  uint32_t spin_limit;
  int last_resident_slots;  // chunk slots the resident kernel of the last step handed out (0: it did not run)
};

static constexpr uint32_t kPlanMagic = 0x4c414e53u;  // "LANS"
static constexpr uint32_t kDefaultSpinLimit = 1u << 20;  // about a second of polling; a healthy wait is microseconds

// GT / PL as compile-time constants inside `...` for the run-time codes gt (LANCET_F32 / _BF16 / _F16) and pl (the
// same 16-bit codes, or kNoLowp)
#define LANS_TYPE_SWITCH(gt, pl, ...)                                                                      \
  switch ((gt) * 4 + ((pl) == kNoLowp ? 0 : (pl))) {                                                       \
    case LANCET_F32 * 4 + 0: { constexpr int GT = LANCET_F32, PL = kNoLowp; (void)PL; __VA_ARGS__; } break;          \
    case LANCET_F32 * 4 + LANCET_BF16: { constexpr int GT = LANCET_F32, PL = LANCET_BF16; (void)PL; __VA_ARGS__; } break;   \
    case LANCET_F32 * 4 + LANCET_F16: { constexpr int GT = LANCET_F32, PL = LANCET_F16; (void)PL; __VA_ARGS__; } break;     \
    case LANCET_BF16 * 4 + 0: { constexpr int GT = LANCET_BF16, PL = kNoLowp; (void)PL; __VA_ARGS__; } break;        \
    case LANCET_BF16 * 4 + LANCET_BF16: { constexpr int GT = LANCET_BF16, PL = LANCET_BF16; (void)PL; __VA_ARGS__; } break; \
    case LANCET_BF16 * 4 + LANCET_F16: { constexpr int GT = LANCET_BF16, PL = LANCET_F16; (void)PL; __VA_ARGS__; } break;   \
    case LANCET_F16 * 4 + 0: { constexpr int GT = LANCET_F16, PL = kNoLowp; (void)PL; __VA_ARGS__; } break;          \
    case LANCET_F16 * 4 + LANCET_BF16: { constexpr int GT = LANCET_F16, PL = LANCET_BF16; (void)PL; __VA_ARGS__; } break;   \
    default: { constexpr int GT = LANCET_F16, PL = LANCET_F16; (void)PL; __VA_ARGS__; } break;                       \
  }

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
static inline int chunks_of(int64_t numel) { return static_cast<int>((numel + kLansChunk - 1) / kLansChunk); }

// The plan's own tensor order and chunk slots.  Tensors of at most `limit` whole chunks come first, largest first
// (list order among equals), packed into rounds of `round` slots: a tensor that does not fit into what is
// left of a round starts the next one and the rest of the round is padding (chunk_tensor -1), so that all
// chunks of a tensor are drawn in the same pass of the resident kernel's workgroups.  The other tensors (larger,
// or not a multiple of the chunk) follow in list order, without padding: they go through the sweeps.  first[i] / ctensor are in plan order.
struct ChunkLayout {
  std::vector<int32_t> order, ctensor, first, count;
  int n_fit = 0;       // tensors the resident kernel takes
  int n_res_slots = 0; // slots it hands out
};

static ChunkLayout chunk_layout(const int64_t* numels, int T, int limit, int round) {
  ChunkLayout L;
  std::vector<int32_t> fit, big;
  // the resident kernel takes whole chunks only
  for (int i = 0; i < T; ++i)
    ((chunks_of(numels[i]) <= limit && numels[i] % kLansChunk == 0) ? fit : big).push_back(i);
  std::stable_sort(fit.begin(), fit.end(), [&](int a, int b) { return chunks_of(numels[a]) > chunks_of(numels[b]); });
  L.n_fit = static_cast<int>(fit.size());
  L.order = fit;
  L.order.insert(L.order.end(), big.begin(), big.end());
  L.first.assign(T, 0);
  L.count.assign(T, 0);
  if (round < 1) round = 1;
  for (int i = 0; i < T; ++i) {
    const int k = chunks_of(numels[L.order[i]]);
    if (i < L.n_fit && k <= round) {
      const int used = static_cast<int>(L.ctensor.size()) % round;
      if (used + k > round) L.ctensor.insert(L.ctensor.end(), round - used, -1);
    }
    if (i == L.n_fit) L.n_res_slots = static_cast<int>(L.ctensor.size());
    L.first[i] = static_cast<int32_t>(L.ctensor.size());
    L.count[i] = k;
    L.ctensor.insert(L.ctensor.end(), k, i);
  }
  if (L.n_fit == T) L.n_res_slots = static_cast<int>(L.ctensor.size());
  return L;
}

// Host-only view of what a plan builds for `numels` when the resident kernel takes tensors of up to
// `resident_limit` chunks and runs `round` workgroups (no device needed): for every chunk slot, in ticket
// order, the position of its tensor in the caller's list (-1: padding); *n_resident_chunks = slots the
// resident kernel hands out.
extern "C" int64_t lancet_lans_debug_chunk_table(const int64_t* numels, int T, int resident_limit, int round,
                                                 int32_t* chunk_tensor_out, int64_t capacity,
                                                 int64_t* n_resident_chunks) {
  if (!numels || T <= 0) return -1;
  for (int i = 0; i < T; ++i)
    if (numels[i] < 0) return -1;
  const ChunkLayout L = chunk_layout(numels, T, resident_limit, round);
  for (int64_t i = 0; i < capacity && i < static_cast<int64_t>(L.ctensor.size()); ++i)
    if (chunk_tensor_out) chunk_tensor_out[i] = L.ctensor[i] < 0 ? -1 : L.order[L.ctensor[i]];
  if (n_resident_chunks) *n_resident_chunks = L.n_res_slots;
  return static_cast<int64_t>(L.ctensor.size());
}

extern "C" int lancet_lans_plan_create(const int64_t* numels, int T, lancet_lans_plan_t* out) {
  if (!numels || !out) return LANCET_ERR_NULL;
  if (T <= 0) return LANCET_ERR_SHAPE;
  int64_t nchunks64 = 0;
  for (int i = 0; i < T; ++i) {
    if (numels[i] < 0) return LANCET_ERR_SHAPE;
    nchunks64 += chunks_of(numels[i]);
  }
  // slices index the partial sums and the grids; padding at most doubles the slots
  if (2 * nchunks64 * kSweepSplit > 0x7fffffff) return LANCET_ERR_SHAPE;
  lancet_lans_plan* pl = new (std::nothrow) lancet_lans_plan();
  if (!pl) return static_cast<int>(hipErrorOutOfMemory);
  pl->magic = kPlanMagic;
  pl->T = T;
  pl->numels.assign(numels, numels + T);
  pl->shadow.assign(5 * static_cast<size_t>(T), nullptr);
  pl->dev_block = nullptr;
  pl->h_ptrs = nullptr;
  pl->h_status = nullptr;
  pl->upload_done = nullptr;
  pl->upload_pending = false;
  pl->spin_limit = kDefaultSpinLimit;
  pl->schedule = LANCET_LANS_SWEEPS;  // until the layout below says that the resident kernel has something to take
  pl->last_resident_slots = 0;
  hipError_t err = hipGetDevice(&pl->device);
  int cus = 256;
  if (err == hipSuccess) err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, pl->device);
  pl->resident_grid = 0;
  pl->max_tensor_chunks = 0;
  for (int i = 0; i < T; ++i) pl->max_tensor_chunks = std::max(pl->max_tensor_chunks, chunks_of(numels[i]));
  if (err == hipSuccess) {
    // every variant of the kernel has the same launch bounds and LDS but its own register count: the grid is what
    // the variant with the fewest workgroups per CU runs at once, so that whichever variant a step launches, all of
    // its workgroups are on the chip together (the waits between them rely on that)
    int per_cu = 1 << 30;
    for (int gt : {LANCET_F32, LANCET_BF16, LANCET_F16})
      for (int plt : {static_cast<int>(kNoLowp), static_cast<int>(LANCET_BF16), static_cast<int>(LANCET_F16)}) {
        int n = 0;
        LANS_TYPE_SWITCH(gt, plt, if (err == hipSuccess) err = hipOccupancyMaxActiveBlocksPerMultiprocessor(
                                      &n, lans_resident_kernel<GT, PL>, kLansThreads, 0))
        per_cu = std::min(per_cu, n);
      }
    if (err != hipSuccess) per_cu = 0;
    pl->resident_grid = per_cu * cus;
  }
  // a tensor's chunks fit one round, so the kernel drains with half of its workgroups on the chip
  // a tensor's chunks fit one round: they are all drawn in one pass
  pl->resident_limit = std::min(pl->resident_grid, kMaxResidentChunks);
  const ChunkLayout L = chunk_layout(numels, T, pl->resident_limit, pl->resident_grid);
  pl->order = L.order;
  pl->n_res_tensors = L.n_fit;
  pl->n_res_chunks = L.n_res_slots;
  pl->nchunks = static_cast<int>(L.ctensor.size());
  if (pl->n_res_chunks > 0) pl->schedule = LANCET_LANS_RESIDENT;
  pl->is_resident.assign(T, 0);
  for (int k = 0; k < pl->n_res_tensors; ++k) pl->is_resident[pl->order[k]] = 1;
  // device block layout
  const size_t n = static_cast<size_t>(pl->nchunks);
  const size_t n1 = n ? n : 1;
  size_t off = 0;
  const size_t o_ptrs = off;      off = align_up(off + 5 * T * sizeof(void*), 256);
  const size_t o_numel = off;     off = align_up(off + T * sizeof(int64_t), 256);
  const size_t o_ctensor = off;   off = align_up(off + n1 * sizeof(int32_t), 256);
  const size_t o_first = off;     off = align_up(off + T * sizeof(int32_t), 256);
  const size_t o_count = off;     off = align_up(off + T * sizeof(int32_t), 256);
  const size_t o_partial = off;   off = align_up(off + 3 * n1 * kSweepSplit * sizeof(float), 256);
  const size_t o_norms = off;     off = align_up(off + 4 * T * sizeof(float), 256);
  const size_t o_consts = off;    off = align_up(off + 2 * sizeof(float), 256);
  const size_t o_words = off;     off = align_up(off + 4 * (n1 + T) * sizeof(uint64_t), 256);
  const size_t n_ctl = kCtlWords;
  const size_t o_ctl = off;       off = align_up(off + n_ctl * sizeof(uint32_t), 256);
  const size_t o_order = off;     off = align_up(off + T * sizeof(int32_t), 256);
  pl->words_bytes = 4 * (n1 + T) * sizeof(uint64_t);
  if (err == hipSuccess) err = hipMalloc(&pl->dev_block, off);
  if (err == hipSuccess) err = hipHostMalloc(reinterpret_cast<void**>(&pl->h_ptrs), 5 * T * sizeof(void*), hipHostMallocDefault);
  if (err == hipSuccess) err = hipHostMalloc(reinterpret_cast<void**>(&pl->h_status), 64, hipHostMallocDefault);
  if (err == hipSuccess) err = hipEventCreateWithFlags(&pl->upload_done, hipEventDisableTiming);
  if (err == hipSuccess) {
    *pl->h_status = 0u;
    std::vector<int64_t> perm(T);
    for (int i = 0; i < T; ++i) perm[i] = numels[pl->order[i]];
    char* base = static_cast<char*>(pl->dev_block);
    err = hipMemcpy(base + o_numel, perm.data(), T * sizeof(int64_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(base + o_order, pl->order.data(), T * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess && n) err = hipMemcpy(base + o_ctensor, L.ctensor.data(), n * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(base + o_first, L.first.data(), T * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(base + o_count, L.count.data(), T * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemset(base + o_norms, 0, 4 * T * sizeof(float));
    if (err == hipSuccess) err = hipMemset(base + o_words, 0, pl->words_bytes);
    if (err == hipSuccess) err = hipMemset(base + o_ctl, 0, n_ctl * sizeof(uint32_t));
    LansTables& t = pl->tables;
    t.part_word = reinterpret_cast<uint64_t*>(base + o_words);
    t.norm_word = t.part_word + 4 * n1;
    t.ctl = reinterpret_cast<uint32_t*>(base + o_ctl);
    t.host_status = nullptr;
    if (err == hipSuccess) err = hipHostGetDevicePointer(reinterpret_cast<void**>(&t.host_status), pl->h_status, 0);
    void** dptrs = reinterpret_cast<void**>(base + o_ptrs);
    t.g = reinterpret_cast<const void* const*>(dptrs);
    t.p = reinterpret_cast<float* const*>(dptrs + T);
    t.m = reinterpret_cast<float* const*>(dptrs + 2 * T);
    t.v = reinterpret_cast<float* const*>(dptrs + 3 * T);
    t.plow = reinterpret_cast<void* const*>(dptrs + 4 * T);
    t.numel = reinterpret_cast<const int64_t*>(base + o_numel);
    t.chunk_tensor = reinterpret_cast<const int32_t*>(base + o_ctensor);
    t.tensor_first = reinterpret_cast<const int32_t*>(base + o_first);
    t.tensor_chunks = reinterpret_cast<const int32_t*>(base + o_count);
    t.partial = reinterpret_cast<float*>(base + o_partial);
    t.norms = reinterpret_cast<float*>(base + o_norms);
    t.consts = reinterpret_cast<float*>(base + o_consts);
    t.order = reinterpret_cast<const int32_t*>(base + o_order);
    t.grad_norms = nullptr;
    t.T = T;
    t.nchunks = pl->nchunks;
    t.nres = pl->n_res_chunks;
    t.debug_flags = 0u;
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
  if (pl->h_status) (void)hipHostFree(pl->h_status);
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

namespace {

int lans_step_impl(lancet_lans_plan_t pl, const void* const* g, int g_dtype, float* const* p, float* const* m,
                   float* const* v, void* const* p_lowp, int lowp_dtype, int step_host, const float* step_dev,
                   const lancet_lans_hyper* h, const float* grad_norms, lancet_stream_t stream) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (!g || !p || !m || !v || !h) return LANCET_ERR_NULL;
  if (g_dtype != LANCET_F32 && g_dtype != LANCET_BF16 && g_dtype != LANCET_F16) return LANCET_ERR_DTYPE;
  if (p_lowp && lowp_dtype != LANCET_BF16 && lowp_dtype != LANCET_F16) return LANCET_ERR_DTYPE;
  const int plt = p_lowp ? lowp_dtype : kNoLowp;
  if (!step_dev && step_host < 1) return LANCET_ERR_SHAPE;
  if (h->mode != 0 && h->mode != 1) return LANCET_ERR_SHAPE;
  int current = -1;
  if (hipGetDevice(&current) != hipSuccess || current != pl->device) return LANCET_ERR_PLAN;  // tables live on pl->device
  // an earlier step of this plan gave up a wait: nothing more is launched until lancet_lans_plan_error
  // has been called (the word is written by the device; reading it needs no synchronisation).  Steps that were
  // queued before the word arrived skip themselves on the device (step_is_skipped).
  if (!(pl->tables.debug_flags & 2u) && __atomic_load_n(pl->h_status, __ATOMIC_RELAXED) != 0u) return LANCET_ERR_STALLED;
  if (reinterpret_cast<uintptr_t>(grad_norms) & 3u) return LANCET_ERR_ALIGN;
  const int T = pl->T;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uintptr_t g_elem = g_dtype == LANCET_F32 ? 3u : 1u;   // alignment masks: one element, four elements
  const uintptr_t g_vec = g_dtype == LANCET_F32 ? 15u : 7u;
  bool changed = false;
  bool aligned16 = true;  // the resident kernel moves four elements per access: a step in which one of its tensors is not aligned to that runs as sweeps
  for (int i = 0; i < T; ++i) {
    void* const lo = p_lowp ? p_lowp[i] : nullptr;
    if (pl->numels[i] > 0 && (!g[i] || !p[i] || !m[i] || !v[i] || (p_lowp && !lo))) return LANCET_ERR_NULL;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(p[i]) | reinterpret_cast<uintptr_t>(m[i]) | reinterpret_cast<uintptr_t>(v[i]);
    const uintptr_t gbits = reinterpret_cast<uintptr_t>(g[i]), lbits = reinterpret_cast<uintptr_t>(lo);
    if ((bits & 3u) || (gbits & g_elem) || (lbits & 1u)) return LANCET_ERR_ALIGN;
    aligned16 = aligned16 && (!pl->is_resident[i] || ((bits & 15u) == 0 && (gbits & g_vec) == 0 && (lbits & 7u) == 0));
    changed = changed || pl->shadow[i] != g[i] || pl->shadow[T + i] != p[i] ||
              pl->shadow[2 * T + i] != m[i] || pl->shadow[3 * T + i] != v[i] || pl->shadow[4 * T + i] != lo;
  }
  hipError_t err = hipSuccess;
  if (changed) {
    // the pinned staging buffer may still be the source of the previous upload
    if (pl->upload_pending) {
      err = hipEventSynchronize(pl->upload_done);
      if (err != hipSuccess) return static_cast<int>(err);
    }
    for (int i = 0; i < T; ++i) {
      pl->shadow[i] = g[i];
      pl->shadow[T + i] = p[i];
      pl->shadow[2 * T + i] = m[i];
      pl->shadow[3 * T + i] = v[i];
      pl->shadow[4 * T + i] = p_lowp ? p_lowp[i] : nullptr;
      const int u = pl->order[i];  // the plan's i-th tensor is the caller's u-th
      pl->h_ptrs[i] = const_cast<void*>(g[u]);
      pl->h_ptrs[T + i] = p[u];
      pl->h_ptrs[2 * T + i] = m[u];
      pl->h_ptrs[3 * T + i] = v[u];
      pl->h_ptrs[4 * T + i] = p_lowp ? p_lowp[u] : nullptr;
    }
    err = hipMemcpyAsync(pl->dev_block, pl->h_ptrs,
                         5 * static_cast<size_t>(T) * sizeof(void*), hipMemcpyHostToDevice, st);
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
  LansTables t = pl->tables;
  t.grad_norms = grad_norms;
  sc.spin_limit = pl->spin_limit;
  sc.epoch = 0;
  // slots [0, chunk_base) and tensors [0, tensor_base) go through the resident kernel, the rest
  // (everything, under the sweeps schedule) through the three sweeps
  int chunk_base = 0, tensor_base = 0;
  pl->last_resident_slots = 0;
  const bool resident = pl->schedule == LANCET_LANS_RESIDENT && pl->n_res_chunks > 0 && aligned16;
  // the first kernel of a step forms the bias corrections and decides whether the step runs at all
  if (resident) lans_begin_kernel<<<1, kLansThreads, 0, st>>>(t, sc, pl->words_bytes / sizeof(uint64_t));
  else lans_prepare_kernel<<<1, 64, 0, st>>>(t, sc);
  if (grad_norms) lans_take_grad_norms_kernel<<<(T + 255) / 256, 256, 0, st>>>(t);
  if (resident) {
    const int grid = std::min(pl->resident_grid, pl->n_res_chunks);
    LANS_TYPE_SWITCH(g_dtype, plt, (lans_resident_kernel<GT, PL><<<grid, kLansThreads, 0, st>>>(t, sc)))
    chunk_base = pl->n_res_chunks;
    tensor_base = pl->n_res_tensors;
    pl->last_resident_slots = chunk_base;
  }
  const int nsweep = t.nchunks - chunk_base;
  if (nsweep > 0) {
    const int per_block = kLansThreads / kWave;
    const int rblocks = (T - tensor_base + per_block - 1) / per_block;
    if (!grad_norms) {
      LANS_TYPE_SWITCH(g_dtype, kNoLowp, (lans_norm_g_kernel<GT><<<nsweep, kLansThreads, 0, st>>>(t, chunk_base)))
      lans_reduce_kernel<<<rblocks, kLansThreads, 0, st>>>(t, 0, tensor_base, T, 1, 1);
    }
    LANS_TYPE_SWITCH(g_dtype, kNoLowp, (lans_moments_kernel<GT><<<nsweep * kSweepSplit, kLansThreads, 0, st>>>(t, sc, chunk_base)))
    lans_reduce_kernel<<<rblocks, kLansThreads, 0, st>>>(t, 1, tensor_base, T, 3, kSweepSplit);
    LANS_TYPE_SWITCH(g_dtype, plt, (lans_update_kernel<GT, PL><<<nsweep * kSweepSplit, kLansThreads, 0, st>>>(t, sc, chunk_base)))
  }
  return static_cast<int>(hipGetLastError());
}

}  // namespace

extern "C" int lancet_lans_step(lancet_lans_plan_t pl, const float* const* g, float* const* p,
                                float* const* m, float* const* v, int step_host,
                                const float* step_dev, const lancet_lans_hyper* h,
                                const float* grad_norms, lancet_stream_t stream) {
  return lans_step_impl(pl, reinterpret_cast<const void* const*>(g), LANCET_F32, p, m, v, nullptr, LANCET_F32, step_host,
                        step_dev, h, grad_norms, stream);
}

extern "C" int lancet_lans_step_mixed(lancet_lans_plan_t pl, const void* const* g, int g_dtype, float* const* p,
                                      float* const* m, float* const* v, void* const* p_lowp, int lowp_dtype,
                                      int step_host, const float* step_dev, const lancet_lans_hyper* h,
                                      const float* grad_norms, lancet_stream_t stream) {
  return lans_step_impl(pl, g, g_dtype, p, m, v, p_lowp, lowp_dtype, step_host, step_dev, h, grad_norms, stream);
}

extern "C" int lancet_lans_plan_set_schedule(lancet_lans_plan_t pl, int schedule) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (schedule != LANCET_LANS_SWEEPS && schedule != LANCET_LANS_RESIDENT) return LANCET_ERR_SHAPE;
  // tensors too large for the resident kernel go through the sweeps inside the same step; a plan made only
  // of such tensors has no use for the kernel
  if (schedule == LANCET_LANS_RESIDENT && pl->n_res_chunks == 0 && pl->nchunks > 0) return LANCET_ERR_SHAPE;
  pl->schedule = schedule;
  return LANCET_OK;
}

extern "C" int lancet_lans_plan_schedule(lancet_lans_plan_t pl, int* schedule) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (!schedule) return LANCET_ERR_NULL;
  *schedule = pl->schedule;
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
  hipError_t e = hipMemcpyAsync(&word, pl->tables.ctl + kCtlError, sizeof(word), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  // the reader, and only the reader, clears the error (the steps on `stream` have finished)
  if (e == hipSuccess && (word != 0u || __atomic_load_n(pl->h_status, __ATOMIC_RELAXED) != 0u)) {
    word = 1u;
    e = hipMemsetAsync(pl->tables.ctl + kCtlError, 0, sizeof(uint32_t), st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    __atomic_store_n(pl->h_status, 0u, __ATOMIC_RELAXED);
  }
  *error_out = static_cast<int>(word);
  return static_cast<int>(e);
}

extern "C" int lancet_lans_plan_debug_last_resident(lancet_lans_plan_t pl, int* slots) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (!slots) return LANCET_ERR_NULL;
  *slots = pl->last_resident_slots;
  return LANCET_OK;
}

extern "C" int lancet_lans_plan_debug(lancet_lans_plan_t pl, unsigned spin_limit, unsigned flags) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  pl->spin_limit = spin_limit ? spin_limit : kDefaultSpinLimit;
  pl->tables.debug_flags = flags;  // bit 1 (host only): lancet_lans_step does not look at the pinned status word
  return LANCET_OK;
}
