// Fused multi-tensor LANS step in three sweeps over the optimizer state (the reference makes
// six: src/op/dialect/cuda/kernels/multi_tensor_lans.cu:401-450):
//   sweep 1  reads g, p            -> per-chunk sums of g^2 and p^2
//   sweep 2  reads g, p, m, v      -> writes m, v; per-chunk sums of u_m^2 and u_g^2
//   sweep 3  reads g, p, m, v      -> recomputes u_m, u_g (never stored) and writes p
// with a tiny per-tensor reduction after sweeps 1 and 2.  Work is cut into fixed-size chunks
// described by device-resident tables built once per parameter set, instead of kernel
// arguments re-packed for every launch (multi_tensor_apply.cuh:39-92).  Per-chunk partial
// sums are combined in a fixed order in double precision, so results are deterministic.
#include "launchers.hpp"
#include "common.hpp"
#include "../../include/lancet_hip.h"
#include <new>
#include <vector>

namespace lancet {

constexpr int kLansThreads = 256;
constexpr int kLansChunk = 16384;  // elements per workgroup: 16 float4 per thread
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct LansTables {
  const float* const* g;  // [T] device pointers
  float* const* p;
  float* const* m;
  float* const* v;
  const int64_t* numel;        // [T]
  const int32_t* chunk_tensor; // [nchunks]
  const int32_t* tensor_first; // [T+1] first chunk of each tensor
  float* partial;              // [2][nchunks]
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

// bias corrections 1 - beta^step (src/op/dialect/cuda/lans.cc:108-113), from a host step or
// from the fp32 step scalar in device memory (no host synchronisation, unlike lans.cc:102-107)
__global__ void lans_prepare_kernel(LansTables t, LansScalars sc) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int step = sc.step_host;
    if (sc.step_dev) step = static_cast<int>(*sc.step_dev);
    float bc1 = 1.f, bc2 = 1.f;
    if (sc.bias_correction) {
      bc1 = static_cast<float>(1.0 - pow(static_cast<double>(sc.beta1), step));
      bc2 = static_cast<float>(1.0 - pow(static_cast<double>(sc.beta2), step));
    }
    t.consts[0] = bc1;
    t.consts[1] = bc2;
  }
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

__device__ __forceinline__ LansElem make_elem(const LansTables& t, const LansScalars& sc, int tensor) {
  LansElem e;
  const float gn = t.norms[tensor];
  e.gnorm_eps = gn + sc.eps;
  e.normalize = sc.normalize_grad && gn != 0.f;
  e.beta1 = sc.beta1;
  e.beta2 = sc.beta2;
  e.beta3 = sc.beta3;
  e.one_minus_beta2 = 1.f - sc.beta2;
  e.bc1 = t.consts[0];
  e.bc2 = t.consts[1];
  e.eps = sc.eps;
  e.wd = sc.wd;
  e.mode = sc.mode;
  return e;
}

// ---- sweep 1: sums of squares of g and p (L2NormFunctor, multi_tensor_lans.cu:95-167) -------
__global__ __launch_bounds__(kLansThreads) void lans_norm_gp_kernel(LansTables t) {
  __shared__ float s_red[kLansThreads / kWave];
  const ChunkView c = chunk_view(t, blockIdx.x);
  const float* g = t.g[c.tensor] + c.begin;
  const float* p = t.p[c.tensor] + c.begin;
  float ag = 0.f, ap = 0.f;
  if (vec_ok(g, p, g, p)) {
    const int nv = c.n / 4;
    const f32x4* g4 = reinterpret_cast<const f32x4*>(g);
    const f32x4* p4 = reinterpret_cast<const f32x4*>(p);
    for (int i = threadIdx.x; i < nv; i += kLansThreads) {
      const f32x4 x = g4[i], y = p4[i];
      ag += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
      ap += y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w;
    }
    for (int i = nv * 4 + threadIdx.x; i < c.n; i += kLansThreads) {
      ag += g[i] * g[i];
      ap += p[i] * p[i];
    }
  } else {
    for (int i = threadIdx.x; i < c.n; i += kLansThreads) {
      ag += g[i] * g[i];
      ap += p[i] * p[i];
    }
  }
  const float sg = block_sum(ag, s_red);
  const float sp = block_sum(ap, s_red);
  if (threadIdx.x == 0) {
    t.partial[blockIdx.x] = sg;
    t.partial[t.nchunks + blockIdx.x] = sp;
  }
}

// per-tensor sqrt(sum of chunk partials) in double, fixed order (cleanup, :169-185)
__global__ __launch_bounds__(kLansThreads) void lans_reduce_kernel(LansTables t, int first_norm) {
  const int tensor = blockIdx.x * (kLansThreads / kWave) + threadIdx.x / kWave;
  if (tensor >= t.T) return;
  const int lo = t.tensor_first[tensor], hi = t.tensor_first[tensor + 1];
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    double acc = 0.0;
    for (int c = lo + lane_id(); c < hi; c += kWave) acc += static_cast<double>(t.partial[k * t.nchunks + c]);
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
    if (lane_id() == 0) t.norms[(first_norm + k) * t.T + tensor] = static_cast<float>(sqrt(acc));
  }
}

// ---- sweep 2: moments + sums of squares of the two updates (LANSStage1Functor :207-322 and the
//      two l2norm sweeps after it, :434-441) -----------------------------------------------
__global__ __launch_bounds__(kLansThreads) void lans_moments_kernel(LansTables t, LansScalars sc) {
  __shared__ float s_red[kLansThreads / kWave];
  const ChunkView c = chunk_view(t, blockIdx.x);
  const LansElem el = make_elem(t, sc, c.tensor);
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
  const float sm = block_sum(am, s_red);
  const float sgs = block_sum(ag, s_red);
  if (threadIdx.x == 0) {
    t.partial[blockIdx.x] = sm;
    t.partial[t.nchunks + blockIdx.x] = sgs;
  }
}

// ---- sweep 3: trust ratios and parameter update (LANSStage2Functor :326-399) ---------------
__global__ __launch_bounds__(kLansThreads) void lans_update_kernel(LansTables t, LansScalars sc) {
  const ChunkView c = chunk_view(t, blockIdx.x);
  const LansElem el = make_elem(t, sc, c.tensor);
  const float pn = t.norms[1 * t.T + c.tensor];
  const float umn = t.norms[2 * t.T + c.tensor];
  const float ugn = t.norms[3 * t.T + c.tensor];
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
};

static constexpr uint32_t kPlanMagic = 0x4c414e53u;  // "LANS"

static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

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
  if (err == hipSuccess) err = hipMalloc(&pl->dev_block, off);
  if (err == hipSuccess) err = hipHostMalloc(reinterpret_cast<void**>(&pl->h_ptrs), 4 * T * sizeof(void*), hipHostMallocDefault);
  if (err == hipSuccess) err = hipEventCreateWithFlags(&pl->upload_done, hipEventDisableTiming);
  if (err == hipSuccess) {
    std::vector<int32_t> ctensor(n ? n : 1), first(T + 1);
    int c = 0;
    for (int i = 0; i < T; ++i) {
      first[i] = c;
      const int k = static_cast<int>((numels[i] + kLansChunk - 1) / kLansChunk);
      for (int j = 0; j < k; ++j) ctensor[c++] = i;
    }
    first[T] = c;
    char* base = static_cast<char*>(pl->dev_block);
    err = hipMemcpy(base + o_numel, numels, T * sizeof(int64_t), hipMemcpyHostToDevice);
    if (err == hipSuccess && n) err = hipMemcpy(base + o_ctensor, ctensor.data(), n * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemcpy(base + o_first, first.data(), (T + 1) * sizeof(int32_t), hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipMemset(base + o_norms, 0, 4 * T * sizeof(float));
    LansTables& t = pl->tables;
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
  const int rblocks = (T + kLansThreads / kWave - 1) / (kLansThreads / kWave);
  lans_prepare_kernel<<<1, 64, 0, st>>>(t, sc);
  lans_norm_gp_kernel<<<t.nchunks, kLansThreads, 0, st>>>(t);
  lans_reduce_kernel<<<rblocks, kLansThreads, 0, st>>>(t, 0);
  lans_moments_kernel<<<t.nchunks, kLansThreads, 0, st>>>(t, sc);
  lans_reduce_kernel<<<rblocks, kLansThreads, 0, st>>>(t, 2);
  lans_update_kernel<<<t.nchunks, kLansThreads, 0, st>>>(t, sc);
  return static_cast<int>(hipGetLastError());
}
