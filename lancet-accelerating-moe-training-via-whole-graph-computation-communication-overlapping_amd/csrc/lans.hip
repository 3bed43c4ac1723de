// Fused multi-tensor LANS step.  The reference makes six sweeps over the optimizer state
// (src/op/dialect/cuda/kernels/multi_tensor_lans.cu:401-450: l2norm(g), l2norm(p), stage 1,
// l2norm(u_m), l2norm(u_g), stage 2, 68 B/param of traffic).  Here the step has three phases
//   phase 1  reads g, p            -> per-chunk sums of g^2 and p^2
//   phase 2  reads g, p, m, v      -> writes m, v; per-chunk sums of u_m^2 and u_g^2
//   phase 3  reads g, p, m, v      -> recomputes u_m, u_g (never stored) and writes p
// and two schedules that give the same bits:
//   * sweeps (default): three plain launches + two tiny per-tensor reductions.  Real HBM traffic
//     is 52 B/param (g, p read three times, m, v twice) and each sweep streams at the rate a plain
//     copy reaches on this chip.
//   * pipelined (opt-in): ONE persistent kernel.  Workgroups pull (phase, chunk) tasks from a
//     queue built once per parameter set, ordered so that phase 2 of a bundle of tensors (about
//     4M parameters, 64 MB of state) runs while phase 1 of the next bundle and phase 3 of the
//     previous one run, with the aim of re-reading a tensor while it is still in the 256 MB
//     Infinity Cache.  A task that needs a per-tensor norm waits for the chunk partials of that
//     tensor, which are self-validating 64-bit words (step epoch in the high half, fp32 sum in
//     the low half) published with one agent-scope atomic store each: no counters, nothing to
//     clear between steps.  Tasks only ever wait for tasks that are earlier in the queue (already
//     taken by a running workgroup) and phase-1 tasks never wait, so the queue always drains;
//     waits are bounded.  m and v cross workgroups (and XCDs, whose L2s are private) between
//     phase 2 and phase 3, which costs one release fence per phase-2 task and one acquire per
//     phase-3 task; on MI355X the release (an L2 write-back) makes this schedule about 3x slower
//     than the sweeps, which is why it is not the default.
// Work is cut into fixed-size chunks described by device-resident tables built once per
// parameter set, instead of kernel arguments re-packed for every launch
// (multi_tensor_apply.cuh:39-92).  Chunk partials are combined in a fixed order in double
// precision, so results are deterministic and identical between the two schedules.
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
  float* partial;              // [2][nchunks]      (sweeps schedule)
  uint64_t* part_word;         // [4][nchunks]      (pipelined schedule: epoch | fp32 bits)
  uint64_t* norm_word;         // [4][T]            (pipelined schedule: published norms)
  const uint32_t* tasks;       // [3*nchunks]       (pipelined schedule: phase << 30 | chunk)
  uint32_t* ticket;            // [1] next task; [1] error flag
  float* norms;                // [4][T]: g, p, u_m, u_g
  float* consts;               // [2]: bias_correction1, bias_correction2
  int T;
  int nchunks;
};

struct LansScalars {
  float lr, beta1, beta2, beta3, eps, wd;
  int mode, normalize_grad, bias_correction;
  int step_host;
  const float* step_dev;
  uint32_t epoch;
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

__device__ __forceinline__ bool vec_ok(const void* a, const void* b, const void* c, const void* d) {
  return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
           reinterpret_cast<uintptr_t>(c) | reinterpret_cast<uintptr_t>(d)) & 15u) == 0;
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
  e.gnorm_eps = gn + sc.eps;
  e.normalize = sc.normalize_grad && gn != 0.f;
  e.beta1 = sc.beta1;
  e.beta2 = sc.beta2;
  e.beta3 = sc.beta3;
  e.one_minus_beta2 = 1.f - sc.beta2;
  e.bc1 = bc1;
  e.bc2 = bc2;
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

// ---- the three phases on one chunk, executed by one workgroup ------------------------------
// phase 1: sums of squares of g and p (L2NormFunctor, multi_tensor_lans.cu:95-167); valid on thread 0
__device__ __forceinline__ void chunk_norm_gp(const LansTables& t, const ChunkView& c, float* s_red,
                                              float& sum_g, float& sum_p) {
  const float* g = t.g[c.tensor] + c.begin;
  const float* p = t.p[c.tensor] + c.begin;
  float ag = 0.f, ap = 0.f;
  int scalar_from = 0;
  if (vec_ok(g, p, g, p)) {
    const int nv = c.n / 4;
    const f32x4* g4 = reinterpret_cast<const f32x4*>(g);
    const f32x4* p4 = reinterpret_cast<const f32x4*>(p);
#pragma unroll 4
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 x = g4[i], y = p4[i];
      ag += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
      ap += y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w;
    }
    scalar_from = nv * 4;
  }
  for (int i = scalar_from + threadIdx.x; i < c.n; i += kLansThreads) {
    ag += g[i] * g[i];
    ap += p[i] * p[i];
  }
  sum_g = block_sum(ag, s_red);
  sum_p = block_sum(ap, s_red);
}

// phase 2: moments + sums of squares of the two updates (LANSStage1Functor :207-322 and the two
// l2norm sweeps after it, :434-441); sums valid on thread 0
__device__ __forceinline__ void chunk_moments(const LansTables& t, const ChunkView& c, const LansElem& el,
                                              float* s_red, float& sum_um, float& sum_ug) {
  const float* g = t.g[c.tensor] + c.begin;
  const float* p = t.p[c.tensor] + c.begin;
  float* m = t.m[c.tensor] + c.begin;
  float* v = t.v[c.tensor] + c.begin;
  float am = 0.f, ag = 0.f;
  int scalar_from = 0;
  if (vec_ok(g, p, m, v)) {
    const int nv = c.n / 4;
    const f32x4* g4 = reinterpret_cast<const f32x4*>(g);
    const f32x4* p4 = reinterpret_cast<const f32x4*>(p);
    f32x4* m4 = reinterpret_cast<f32x4*>(m);
    f32x4* v4 = reinterpret_cast<f32x4*>(v);
#pragma unroll 2
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 xg = g4[i], xp = p4[i];
      f32x4 xm = m4[i], xv = v4[i];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float sg = el.scaled_grad(xg[k], xp[k]);
        float mm = xm[k], vv = xv[k], um, ug;
        el.moments(sg, mm, vv);
        el.updates(sg, xp[k], mm, vv, um, ug);
        xm[k] = mm;
        xv[k] = vv;
        am += um * um;
        ag += ug * ug;
      }
      m4[i] = xm;
      v4[i] = xv;
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
    am += um * um;
    ag += ug * ug;
  }
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
  const float* g = t.g[c.tensor] + c.begin;
  float* p = t.p[c.tensor] + c.begin;
  const float* m = t.m[c.tensor] + c.begin;
  const float* v = t.v[c.tensor] + c.begin;
  int scalar_from = 0;
  if (vec_ok(g, p, m, v)) {
    const int nv = c.n / 4;
    const f32x4* g4 = reinterpret_cast<const f32x4*>(g);
    f32x4* p4 = reinterpret_cast<f32x4*>(p);
    const f32x4* m4 = reinterpret_cast<const f32x4*>(m);
    const f32x4* v4 = reinterpret_cast<const f32x4*>(v);
#pragma unroll 2
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 xg = g4[i], xm = m4[i], xv = v4[i];
      f32x4 xp = p4[i];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
#pragma clang fp contract(off)
        const float sg = el.scaled_grad(xg[k], xp[k]);
        float um, ug;
        el.updates(sg, xp[k], xm[k], xv[k], um, ug);
        xp[k] = xp[k] - (ratio_m * um) - (ratio_g * ug);
      }
      p4[i] = xp;
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

__global__ __launch_bounds__(kLansThreads) void lans_norm_gp_kernel(LansTables t) {
  __shared__ float s_red[kLansThreads / kWave];
  const ChunkView c = chunk_view(t, blockIdx.x);
  float sg, sp;
  chunk_norm_gp(t, c, s_red, sg, sp);
  if (threadIdx.x == 0) {
    t.partial[blockIdx.x] = sg;
    t.partial[t.nchunks + blockIdx.x] = sp;
  }
}

// per-tensor sqrt(sum of chunk partials) (cleanup, multi_tensor_lans.cu:169-185)
__global__ __launch_bounds__(kLansThreads) void lans_reduce_kernel(LansTables t, int first_norm) {
  const int tensor = blockIdx.x * (kLansThreads / kWave) + threadIdx.x / kWave;
  if (tensor >= t.T) return;
  const int lo = t.tensor_first[tensor], hi = t.tensor_first[tensor + 1];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const float* part = t.partial + static_cast<size_t>(k) * t.nchunks;
    const float n = wave_norm(lo, hi, [&](int c) { return part[c]; });
    if (lane_id() == 0) t.norms[(first_norm + k) * t.T + tensor] = n;
  }
}

__global__ __launch_bounds__(kLansThreads) void lans_moments_kernel(LansTables t, LansScalars sc) {
  __shared__ float s_red[kLansThreads / kWave];
  const ChunkView c = chunk_view(t, blockIdx.x);
  const LansElem el = make_elem(sc, t.norms[c.tensor], t.consts[0], t.consts[1]);
  float sm, sg;
  chunk_moments(t, c, el, s_red, sm, sg);
  if (threadIdx.x == 0) {
    t.partial[blockIdx.x] = sm;
    t.partial[t.nchunks + blockIdx.x] = sg;
  }
}

__global__ __launch_bounds__(kLansThreads) void lans_update_kernel(LansTables t, LansScalars sc) {
  const ChunkView c = chunk_view(t, blockIdx.x);
  const LansElem el = make_elem(sc, t.norms[c.tensor], t.consts[0], t.consts[1]);
  chunk_update(t, c, el, sc, t.norms[1 * t.T + c.tensor], t.norms[2 * t.T + c.tensor], t.norms[3 * t.T + c.tensor]);
}

// =======================================================================================
// schedule "pipelined": one persistent kernel over a task queue
// =======================================================================================
__device__ __forceinline__ uint64_t ld_word(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_word(uint64_t* p, uint32_t epoch, float v) {
  __hip_atomic_store(p, (static_cast<uint64_t>(epoch) << 32) | __float_as_uint(v), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// Norm `which` (0 g, 1 p, 2 u_m, 3 u_g) of a tensor, called by the first wave of the workgroup.
// Uses the published norm word when some workgroup has already summed the partials of this step,
// else waits for the partials (bounded) and sums them itself, then publishes.
__device__ __forceinline__ float pipeline_norm(const LansTables& t, const LansScalars& sc, int which, int tensor) {
  uint64_t* nw = t.norm_word + static_cast<size_t>(which) * t.T + tensor;
  const uint64_t w = ld_word(nw);
  // one value for the whole wave, whatever each lane's load returned
  const uint32_t w_hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(w >> 32));
  const uint32_t w_lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(w));
  if (w_hi == sc.epoch) return __uint_as_float(w_lo);
  const uint64_t* part = t.part_word + static_cast<size_t>(which) * t.nchunks;
  const int lo = t.tensor_first[tensor], hi = t.tensor_first[tensor + 1];
  const float n = wave_norm(lo, hi, [&](int c) {
    uint64_t x = ld_word(part + c);
    uint32_t spins = 0;
    while (static_cast<uint32_t>(x >> 32) != sc.epoch) {
      if (++spins > sc.spin_limit) {  // bounded wait: flag the plan, carry on
        st_agent(t.ticket + 1, 1u);
        break;
      }
      __builtin_amdgcn_s_sleep(8);
      x = ld_word(part + c);
    }
    return __uint_as_float(static_cast<uint32_t>(x));
  });
  if (lane_id() == 0) {
    st_word(nw, sc.epoch, n);
    t.norms[which * t.T + tensor] = n;
  }
  return n;
}

__global__ __launch_bounds__(kLansThreads) void lans_pipeline_kernel(LansTables t, LansScalars sc) {
  __shared__ float s_red[kLansThreads / kWave];
  __shared__ uint32_t s_task;
  __shared__ float s_norm[4];
  float bc1, bc2;
  bias_corrections(sc, bc1, bc2);
  const uint32_t ntasks = 3u * static_cast<uint32_t>(t.nchunks);
  while (true) {
    __syncthreads();  // s_task / s_norm of the previous task are no longer read
    if (threadIdx.x == 0) s_task = atomicAdd(t.ticket, 1u);
    __syncthreads();
    const uint32_t slot = s_task;
    if (slot >= ntasks) break;  // every workgroup reaches this: the queue is finite
    const uint32_t task = t.tasks[slot];
    const int phase = static_cast<int>(task >> 30);
    const int chunk = static_cast<int>(task & 0x3fffffffu);
    const ChunkView c = chunk_view(t, chunk);
    if (phase == 0) {
      float sg, sp;
      chunk_norm_gp(t, c, s_red, sg, sp);
      if (threadIdx.x == 0) {
        st_word(t.part_word + chunk, sc.epoch, sg);
        st_word(t.part_word + t.nchunks + chunk, sc.epoch, sp);
      }
    } else if (phase == 1) {
      if (threadIdx.x < kWave) {
        const float gn = pipeline_norm(t, sc, 0, c.tensor);
        if (threadIdx.x == 0) s_norm[0] = gn;
      }
      __syncthreads();
      const LansElem el = make_elem(sc, s_norm[0], bc1, bc2);
      float sm, sg;
      chunk_moments(t, c, el, s_red, sm, sg);
      // m and v of this chunk are read in phase 3 by another workgroup, possibly on another XCD
      // (private L2): make them visible device-wide before the words that announce them
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
      __syncthreads();
      if (threadIdx.x == 0) {
        st_word(t.part_word + 2 * static_cast<size_t>(t.nchunks) + chunk, sc.epoch, sm);
        st_word(t.part_word + 3 * static_cast<size_t>(t.nchunks) + chunk, sc.epoch, sg);
      }
    } else {
      if (threadIdx.x < kWave) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float n = pipeline_norm(t, sc, k, c.tensor);
          if (threadIdx.x == 0) s_norm[k] = n;
        }
      }
      __syncthreads();
      // pairs with the release above: drop stale cached copies of m and v
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      const LansElem el = make_elem(sc, s_norm[0], bc1, bc2);
      chunk_update(t, c, el, sc, s_norm[1], s_norm[2], s_norm[3]);
    }
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
  int schedule;        // LANCET_LANS_SWEEPS or LANCET_LANS_PIPELINED
  int grid;            // workgroups of the persistent kernel
  uint32_t epoch;      // step counter that tags the words of the pipelined schedule
  size_t words_offset; // part_word + norm_word inside dev_block
  size_t words_bytes;
};

// Tensors are taken in list order and bundled until a bundle holds this many elements; the
// pipelined schedule keeps about three bundles (x 16 B/element) in flight.
static constexpr int64_t kBundleElems = 4 << 20;

static constexpr uint32_t kPlanMagic = 0x4c414e53u;  // "LANS"

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Task queue of the pipelined schedule: stage s runs phase 3 of bundle s-2, phase 2 of bundle
// s-1 and phase 1 of bundle s, interleaved chunk by chunk.  Every task of phase k of a tensor
// therefore precedes every task of phase k+1 of the same tensor: the order a waiting task relies on.
static void build_task_queue(const int64_t* numels, int T, const std::vector<int32_t>& first,
                             std::vector<uint32_t>& tasks) {
  std::vector<std::pair<int, int>> bundles;  // [first chunk, last chunk)
  int64_t acc = 0;
  int start = 0;
  for (int i = 0; i < T; ++i) {
    acc += numels[i];
    if (acc >= kBundleElems || i == T - 1) {
      if (first[i + 1] > start) bundles.emplace_back(start, first[i + 1]);
      start = first[i + 1];
      acc = 0;
    }
  }
  tasks.clear();
  tasks.reserve(3 * static_cast<size_t>(first[T]));
  const int nb = static_cast<int>(bundles.size());
  for (int sidx = 0; sidx < nb + 2; ++sidx) {
    int lo[3], hi[3];
    for (int ph = 0; ph < 3; ++ph) {  // phase ph works on bundle sidx - ph
      const int b = sidx - ph;
      lo[ph] = (b >= 0 && b < nb) ? bundles[b].first : 0;
      hi[ph] = (b >= 0 && b < nb) ? bundles[b].second : 0;
    }
    const int longest = std::max(hi[0] - lo[0], std::max(hi[1] - lo[1], hi[2] - lo[2]));
    for (int k = 0; k < longest; ++k)
      for (int ph = 2; ph >= 0; --ph)
        if (lo[ph] + k < hi[ph]) tasks.push_back((static_cast<uint32_t>(ph) << 30) | static_cast<uint32_t>(lo[ph] + k));
  }
}

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

// Host-only view of the tables a plan would build (no device needed): the chunk -> tensor map and
// the task queue.  Returns the number of tasks; fills at most `capacity` entries of each array.
extern "C" int64_t lancet_lans_debug_task_queue(const int64_t* numels, int T, uint32_t* tasks_out,
                                                int32_t* chunk_tensor_out, int64_t capacity) {
  if (!numels || T <= 0) return -1;
  std::vector<int32_t> ctensor, first;
  chunk_tables(numels, T, ctensor, first);
  std::vector<uint32_t> tasks;
  build_task_queue(numels, T, first, tasks);
  for (int64_t i = 0; i < capacity && i < static_cast<int64_t>(tasks.size()); ++i)
    if (tasks_out) tasks_out[i] = tasks[i];
  for (int64_t i = 0; i < capacity && i < static_cast<int64_t>(ctensor.size()); ++i)
    if (chunk_tensor_out) chunk_tensor_out[i] = ctensor[i];
  return static_cast<int64_t>(tasks.size());
}

extern "C" int lancet_lans_plan_create(const int64_t* numels, int T, lancet_lans_plan_t* out) {
  if (!numels || !out) return LANCET_ERR_NULL;
  if (T <= 0) return LANCET_ERR_SHAPE;
  int64_t nchunks64 = 0;
  for (int i = 0; i < T; ++i) {
    if (numels[i] < 0) return LANCET_ERR_SHAPE;
    nchunks64 += (numels[i] + kLansChunk - 1) / kLansChunk;
  }
  if (nchunks64 > 0x7fffffff) return LANCET_ERR_SHAPE;
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
  const size_t o_partial = off;   off = align_up(off + 2 * (n ? n : 1) * sizeof(float), 256);
  const size_t o_norms = off;     off = align_up(off + 4 * T * sizeof(float), 256);
  const size_t o_consts = off;    off = align_up(off + 2 * sizeof(float), 256);
  const size_t o_words = off;     off = align_up(off + 4 * ((n ? n : 1) + T) * sizeof(uint64_t), 256);
  const size_t o_tasks = off;     off = align_up(off + 3 * (n ? n : 1) * sizeof(uint32_t), 256);
  const size_t o_ticket = off;    off = align_up(off + 2 * sizeof(uint32_t), 256);
  pl->schedule = LANCET_LANS_SWEEPS;
  pl->epoch = 0;
  pl->words_offset = o_words;
  pl->words_bytes = 4 * ((n ? n : 1) + T) * sizeof(uint64_t);
  int cus = 256;
  if (err == hipSuccess) err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, pl->device);
  pl->grid = static_cast<int>(std::min<size_t>(3 * n, static_cast<size_t>(cus) * 4));
  if (err == hipSuccess) err = hipMalloc(&pl->dev_block, off);
  if (err == hipSuccess) err = hipHostMalloc(reinterpret_cast<void**>(&pl->h_ptrs), 4 * T * sizeof(void*), hipHostMallocDefault);
  if (err == hipSuccess) err = hipEventCreateWithFlags(&pl->upload_done, hipEventDisableTiming);
  if (err == hipSuccess) {
    std::vector<int32_t> ctensor, first;
    chunk_tables(numels, T, ctensor, first);
    char* base = static_cast<char*>(pl->dev_block);
    err = hipMemcpy(base + o_numel, numels, T * sizeof(int64_t), hipMemcpyHostToDevice);
    if (err == hipSuccess && n) err = hipMemcpy(base + o_ctensor, ctensor.data(), n * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(base + o_first, first.data(), (T + 1) * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemset(base + o_norms, 0, 4 * T * sizeof(float));
    if (err == hipSuccess) err = hipMemset(base + o_words, 0, pl->words_bytes);
    std::vector<uint32_t> tasks;
    build_task_queue(numels, T, first, tasks);
    if (err == hipSuccess && !tasks.empty())
      err = hipMemcpy(base + o_tasks, tasks.data(), tasks.size() * sizeof(uint32_t), hipMemcpyHostToDevice);
    LansTables& t = pl->tables;
    t.part_word = reinterpret_cast<uint64_t*>(base + o_words);
    t.norm_word = t.part_word + 4 * (n ? n : 1);
    t.tasks = reinterpret_cast<const uint32_t*>(base + o_tasks);
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
    t.T = T;
    t.nchunks = pl->nchunks;
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
  return static_cast<int>(hipMemcpyAsync(norms, pl->tables.norms, 4 * static_cast<size_t>(pl->T) * sizeof(float),
                                         hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
}

extern "C" int lancet_lans_step(lancet_lans_plan_t pl, const float* const* g, float* const* p,
                                float* const* m, float* const* v, int step_host,
                                const float* step_dev, const lancet_lans_hyper* h,
                                lancet_stream_t stream) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (!g || !p || !m || !v || !h) return LANCET_ERR_NULL;
  if (!step_dev && step_host < 1) return LANCET_ERR_SHAPE;
  if (h->mode != 0 && h->mode != 1) return LANCET_ERR_SHAPE;
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
      pl->shadow[i] = pl->h_ptrs[i] = const_cast<float*>(g[i]);
      pl->shadow[T + i] = pl->h_ptrs[T + i] = p[i];
      pl->shadow[2 * T + i] = pl->h_ptrs[2 * T + i] = m[i];
      pl->shadow[3 * T + i] = pl->h_ptrs[3 * T + i] = v[i];
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
  if (pl->schedule == LANCET_LANS_PIPELINED) {
    if (++pl->epoch == 0) {  // tag wrapped: forget every word of earlier steps
      err = hipMemsetAsync(static_cast<char*>(pl->dev_block) + pl->words_offset, 0, pl->words_bytes, st);
      if (err != hipSuccess) return static_cast<int>(err);
      pl->epoch = 1;
    }
    sc.epoch = pl->epoch;
    err = run_fill_u32(t.ticket, 2, 0u, st);
    if (err != hipSuccess) return static_cast<int>(err);
    lans_pipeline_kernel<<<pl->grid, kLansThreads, 0, st>>>(t, sc);
    return static_cast<int>(hipGetLastError());
  }
  sc.epoch = 0;
  const int rblocks = (T + kLansThreads / kWave - 1) / (kLansThreads / kWave);
  lans_prepare_kernel<<<1, 64, 0, st>>>(t, sc);
  lans_norm_gp_kernel<<<t.nchunks, kLansThreads, 0, st>>>(t);
  lans_reduce_kernel<<<rblocks, kLansThreads, 0, st>>>(t, 0);
  lans_moments_kernel<<<t.nchunks, kLansThreads, 0, st>>>(t, sc);
  lans_reduce_kernel<<<rblocks, kLansThreads, 0, st>>>(t, 2);
  lans_update_kernel<<<t.nchunks, kLansThreads, 0, st>>>(t, sc);
  return static_cast<int>(hipGetLastError());
}

extern "C" int lancet_lans_plan_set_schedule(lancet_lans_plan_t pl, int schedule) {
  if (!pl || pl->magic != kPlanMagic) return LANCET_ERR_PLAN;
  if (schedule != LANCET_LANS_PIPELINED && schedule != LANCET_LANS_SWEEPS) return LANCET_ERR_SHAPE;
  pl->schedule = schedule;
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
