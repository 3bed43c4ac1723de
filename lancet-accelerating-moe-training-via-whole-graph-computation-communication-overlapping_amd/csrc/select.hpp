// Per-token selection (gate softmax + top-1 / top-2) shared by the routing kernels (moe_route.hip) and the
// batch-prioritised routing (moe_bpr.hip).
#pragma once
#include "scan.hpp"
#include "../../include/lancet_hip.h"

namespace lancet {

// ---------------------------------------------------------------------------------------
// Per-token selection on the array the op is given (first max wins; slot 2 = first max with
// slot 1's expert excluded).  With logits the returned values are softmax probabilities,
// exp(x - max) / sum_e exp(x - max), the sum taken in expert order.
// Replaces the argmax / one_hot / multiply+sum micro-kernels of
// src/op/dialect/cuda/moe.cc:177-250 (three passes over [S,E] plus an [S,E] workspace).
// ---------------------------------------------------------------------------------------
// Running first-max / second-max of a row, all in scalars (no arrays, no references: the state has
// to stay in registers).  Branch-free: a lane either takes a new first choice (the old one becomes
// the second), or a new second choice, or nothing.
struct TopState {
  float v1, v2;
  int i1, i2;
};

template <int K>
__device__ __forceinline__ TopState consider(TopState t, float x, int j) {
  const bool first = (t.i1 < 0) | (x > t.v1);
  if (K == 2) {
    const bool second = !first & ((t.i2 < 0) | (x > t.v2));
    t.v2 = first ? t.v1 : (second ? x : t.v2);
    t.i2 = first ? t.i1 : (second ? j : t.i2);
  }
  t.v1 = first ? x : t.v1;
  t.i1 = first ? j : t.i1;
  return t;
}

struct Routed {
  int e0, e1;
  float p0, p1;
};

// ---- a gate row in its storage type (GD = LANCET_F32 / LANCET_BF16 / LANCET_F16), read as fp32 ----------
template <int GD>
__device__ __forceinline__ float gate_at(const void* row, int j) {
  if (GD == LANCET_F32) return static_cast<const float*>(row)[j];
  const uint32_t h = static_cast<const uint16_t*>(row)[j];
  return GD == LANCET_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
}
template <int GD>
__device__ __forceinline__ float half_word(uint32_t h) {
  return GD == LANCET_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
}

// the values of granule g of a row, in order
template <int GD, typename F>
__device__ __forceinline__ void walk_granule(const u32x4 x, int g, F& f) {
  if (GD == LANCET_F32) {
    f(__uint_as_float(x.x), 4 * g);
    f(__uint_as_float(x.y), 4 * g + 1);
    f(__uint_as_float(x.z), 4 * g + 2);
    f(__uint_as_float(x.w), 4 * g + 3);
  } else {
    f(half_word<GD>(x.x & 0xffffu), 8 * g);
    f(half_word<GD>(x.x >> 16), 8 * g + 1);
    f(half_word<GD>(x.y & 0xffffu), 8 * g + 2);
    f(half_word<GD>(x.y >> 16), 8 * g + 3);
    f(half_word<GD>(x.z & 0xffffu), 8 * g + 4);
    f(half_word<GD>(x.z >> 16), 8 * g + 5);
    f(half_word<GD>(x.w & 0xffffu), 8 * g + 6);
    f(half_word<GD>(x.w >> 16), 8 * g + 7);
  }
}

// Calls f(x, j) for j = 0 .. E-1 in order and returns f (the functor carries its state by value, so that it
// stays in registers).  16-byte granules (4 fp32 or 8 half values) when the row allows.
template <int GD, typename F>
__device__ __forceinline__ F walk_row(const void* row, int E, F f) {
  constexpr int V = GD == LANCET_F32 ? 4 : 8;
  const bool vec = ((E & (V - 1)) == 0) && ((reinterpret_cast<uintptr_t>(row) & 15u) == 0);
  if (vec) {
    const u32x4* r = static_cast<const u32x4*>(row);
    const int n = E / V;
    // Rows longer than a line: eight granules (one 128-byte line) are loaded before any of them is used (5-10 %
    // on routing with hundreds of experts).  The last block of up to eight granules, which is all of a short row,
    // is walked load by load (measured faster for rows of one line and less).
    constexpr int kAhead = 8;
    for (int g0 = 0; g0 < n - kAhead; g0 += kAhead) {
      u32x4 xs[kAhead];
#pragma unroll
      for (int i = 0; i < kAhead; ++i) xs[i] = r[g0 + i];
#pragma unroll
      for (int i = 0; i < kAhead; ++i) walk_granule<GD>(xs[i], g0 + i, f);
    }
    for (int g = n > kAhead ? (n - 1) / kAhead * kAhead : 0; g < n; ++g) walk_granule<GD>(r[g], g, f);
  } else {
    for (int j = 0; j < E; ++j) f(gate_at<GD>(row, j), j);
  }
  return f;
}

template <int K>
struct SelectTop {
  TopState t;
  __device__ __forceinline__ void operator()(float x, int j) { t = consider<K>(t, x, j); }
};
// Selection and the softmax denominator in one walk: the sum is kept relative to the running maximum and
// rescaled when a larger value comes (the values the two-pass form adds, exp(x - max), each within an ulp or two;
// used where the row is staged through LDS and a second walk would move it through LDS again).
template <int K>
struct SelectSum {
  TopState t;
  float sum;
  __device__ __forceinline__ void operator()(float x, int j) {
    const bool first = (t.i1 < 0) | (x > t.v1);
    if (first) sum = (t.i1 < 0 ? 0.f : sum * __expf(t.v1 - x)) + 1.f;
    else sum += __expf(x - t.v1);
    t = consider<K>(t, x, j);
  }
};
// The terms of the denominator go through the hardware exponential (__expf); the two gate values themselves
// through expf.  Against an fp64 softmax the gates are as close as with expf in the sum (largest relative error
// 4e-7 at 32 experts, 1.6e-6 at 512, either way: what shows is the rounding of the fp32 sum), and routing with
// 64 experts or more takes 10-15 % less time.
struct SumExp {  // sequential sum in expert order
  float top, sum;
  __device__ __forceinline__ void operator()(float x, int) { sum += __expf(x - top); }
};

// noise (K = 2 only, may be null): values added to the row for the second choice alone, the first
// choice masked out (docker/resources/sharded_moe.py:275-278); gate values always come from the row.
// Row and noise are stored as GD; 16-bit values tie massively, and the first maximum wins as always.
template <int K, int GD>
__device__ __forceinline__ Routed route_token(const void* __restrict__ row, const void* __restrict__ noise, int E,
                                              bool is_logits) {
  SelectTop<K> sel = {{0.f, 0.f, -1, -1}};
  TopState t = walk_row<GD>(row, E, sel).t;
  if (K == 2 && noise) {
    // second choice again, on row + noise: first max over the experts other than the first choice
    float best = 0.f;
    t.i2 = -1;
    for (int j = 0; j < E; ++j) {
      const float x = gate_at<GD>(row, j);
      const float y = x + gate_at<GD>(noise, j);
      const bool take = (j != t.i1) & ((t.i2 < 0) | (y > best));
      best = take ? y : best;
      t.v2 = take ? x : t.v2;
      t.i2 = take ? j : t.i2;
    }
  }
  float sum = 1.f;
  if (is_logits) {
    SumExp se = {t.v1, 0.f};
    sum = walk_row<GD>(row, E, se).sum;
  }
  Routed r;
  r.e0 = t.i1;
  r.p0 = is_logits ? expf(t.v1 - t.v1) / sum : t.v1;
  r.e1 = K == 2 ? t.i2 : -1;
  r.p1 = K == 2 ? (is_logits ? expf(t.v2 - t.v1) / sum : t.v2) : 0.f;
  return r;
}

// ---- rows longer than a cache line: staged through LDS ------------------------------------------------------
// A lane that walks its own row touches each 128-byte line of it in eight loads, and every load of the wave
// touches 64 different lines; with rows of several lines and many waves on a CU the lines are evicted between a
// lane's visits and fetched again (1M tokens x 64 fp32 experts: 0.55 TB/s).  Such rows are therefore read the way
// they lie in memory, a wave's 64 rows 128 bytes at a time (eight lanes per row and line, every line whole in one
// load), passed through LDS and walked from there, each lane its own row as before: the values and their order
// are the same, so is the result.  It pays from about two workgroups per CU on (512 tiles: routing of 1M tokens x
// 64 experts 482 -> 98 us, 262144 x 256 274 -> 92); launches of fewer tiles keep the direct walk, whose lines survive
// in the cache (65536 x 256 top-2: 50 against 64 us).
constexpr int kStageMinTiles = 512;
constexpr int kStageChunk = 128;                   // bytes of a row staged at a time
constexpr int kStageRow = kStageChunk + 16;        // row pitch in LDS (the pad spreads the lanes' reads over the banks)
constexpr int kStageWave = kWave * kStageRow;      // bytes per wave
constexpr int kStageBytes = kWavesPerTile * kStageWave;

template <int GD>
__host__ __device__ inline bool rows_are_staged(const void* gate, const void* noise, int S, int E) {
  constexpr int gb = GD == LANCET_F32 ? 4 : 2;
  return noise == nullptr && (S + kTile - 1) / kTile >= kStageMinTiles && E * gb > kStageChunk && (E * gb) % 16 == 0 &&
         (reinterpret_cast<uintptr_t>(gate) & 15u) == 0;
}

// Calls f(x, j), j = 0 .. E-1 in order, for the lane's row of the wave's rows (rows = first of them, nrows <= 64
// valid ones, E * sizeof(value) a multiple of 16, 16-byte aligned).  All lanes of the wave, uniform control flow;
// stage = the wave's kStageWave bytes of LDS.
// the lane's eight granules of chunk c0 of the wave's rows (zeros beyond the rows and beyond the chunk)
__device__ __forceinline__ void stage_load(const char* rows, int nrows, int row_bytes, int c0, u32x4 (&x)[8]) {
  const int lane = lane_id();
  const int gpr = min(kStageChunk, row_bytes - c0) / 16;  // granules per row in this chunk: 8, less in the last
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int g = i * kWave + lane;
    const int r = gpr == 8 ? (g >> 3) : g / gpr;
    const int part = gpr == 8 ? (g & 7) : g - r * gpr;
    x[i] = u32x4{0u, 0u, 0u, 0u};
    if (r < nrows) x[i] = *reinterpret_cast<const u32x4*>(rows + static_cast<size_t>(r) * row_bytes + c0 + part * 16);
  }
}

template <int GD, typename F>
__device__ __forceinline__ F walk_rows_staged(const char* rows, int nrows, int E, char* stage, F f) {
  constexpr int gb = GD == LANCET_F32 ? 4 : 2;
  constexpr int V = 16 / gb;  // values per 16-byte granule
  const int row_bytes = E * gb;
  const int lane = lane_id();
  u32x4 x[8], nx[8];
  stage_load(rows, nrows, row_bytes, 0, x);
  for (int c0 = 0; c0 < row_bytes; c0 += kStageChunk) {
    const int gpr = min(kStageChunk, row_bytes - c0) / 16;
    // the next chunk's loads are in flight while this one is walked
    const bool more = c0 + kStageChunk < row_bytes;
    if (more) stage_load(rows, nrows, row_bytes, c0 + kStageChunk, nx);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int g = i * kWave + lane;
      const int r = gpr == 8 ? (g >> 3) : g / gpr;
      const int part = gpr == 8 ? (g & 7) : g - r * gpr;
      if (r < kWave) *reinterpret_cast<u32x4*>(stage + r * kStageRow + part * 16) = x[i];
    }
    // the wave's own LDS traffic is in order; the fences keep the compiler from moving the reads above the writes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int j0 = c0 / gb;
    for (int p = 0; p < gpr; ++p) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(stage + lane * kStageRow + p * 16);
      const int j = j0 + p * V;
      if (GD == LANCET_F32) {
        f(__uint_as_float(v.x), j);
        f(__uint_as_float(v.y), j + 1);
        f(__uint_as_float(v.z), j + 2);
        f(__uint_as_float(v.w), j + 3);
      } else {
        f(half_word<GD>(v.x & 0xffffu), j);
        f(half_word<GD>(v.x >> 16), j + 1);
        f(half_word<GD>(v.y & 0xffffu), j + 2);
        f(half_word<GD>(v.y >> 16), j + 3);
        f(half_word<GD>(v.z & 0xffffu), j + 4);
        f(half_word<GD>(v.z >> 16), j + 5);
        f(half_word<GD>(v.w & 0xffffu), j + 6);
        f(half_word<GD>(v.w >> 16), j + 7);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (more) {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = nx[i];
    }
  }
  return f;
}

// Selection for token s of a workgroup whose thread t holds token s = first + t (kTile consecutive tokens): what
// route_token gives, by the direct walk or through LDS.  All kTile threads, uniform control flow; lds = at least
// kStageBytes when rows_are_staged (it may be reused after the call).  Threads with s >= S get {-1, -1, 0, 0}.
template <int K, int GD>
__device__ __forceinline__ Routed route_tile_token(const void* gate, const void* noise, int s, int S, int E, bool is_logits,
                                                   void* lds) {
  constexpr size_t gb = GD == LANCET_F32 ? 4 : 2;
  Routed r = {-1, -1, 0.f, 0.f};
  if (!rows_are_staged<GD>(gate, noise, S, E)) {
    if (s < S) {
      const size_t off = static_cast<size_t>(s) * E * gb;
      r = route_token<K, GD>(static_cast<const char*>(gate) + off, noise ? static_cast<const char*>(noise) + off : nullptr, E,
                             is_logits);
    }
    return r;
  }
  const int first = s - lane_id();  // the wave's first token
  const int nrows = min(max(S - first, 0), kWave);
  const char* rows = static_cast<const char*>(gate) + static_cast<size_t>(first) * E * gb;
  char* stage = static_cast<char*>(lds) + (threadIdx.x / kWave) * kStageWave;
  TopState t;
  float sum = 1.f;
  if (is_logits) {
    SelectSum<K> sel = {{0.f, 0.f, -1, -1}, 0.f};
    sel = walk_rows_staged<GD>(rows, nrows, E, stage, sel);
    t = sel.t;
    sum = sel.sum;
  } else {
    SelectTop<K> sel = {{0.f, 0.f, -1, -1}};
    t = walk_rows_staged<GD>(rows, nrows, E, stage, sel).t;
  }
  if (s < S) {
    r.e0 = t.i1;
    r.p0 = is_logits ? expf(t.v1 - t.v1) / sum : t.v1;
    r.e1 = K == 2 ? t.i2 : -1;
    r.p1 = K == 2 ? (is_logits ? expf(t.v2 - t.v1) / sum : t.v2) : 0.f;
  }
  __syncthreads();  // the caller may use the LDS for something else now
  return r;
}

// GD as a compile-time constant inside `...` for the run-time code gd
#define LANCET_GATE_SWITCH(gd, ...)                                \
  switch (gd) {                                                    \
    case LANCET_BF16: { constexpr int GD = LANCET_BF16; __VA_ARGS__; } break; \
    case LANCET_F16: { constexpr int GD = LANCET_F16; __VA_ARGS__; } break;   \
    default: { constexpr int GD = LANCET_F32; __VA_ARGS__; } break;           \
  }

// LDS a selecting kernel needs for the rows it stages (0: it walks them directly)
inline size_t stage_lds_bytes(int gate_dtype, const void* gate, const void* noise, int S, int E) {
  bool staged = false;
  LANCET_GATE_SWITCH(gate_dtype, staged = rows_are_staged<GD>(gate, noise, S, E))
  return staged ? kStageBytes : 0;
}

}  // namespace lancet
