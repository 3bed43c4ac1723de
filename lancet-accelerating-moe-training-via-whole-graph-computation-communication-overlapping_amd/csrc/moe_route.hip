// Routing kernels: gate softmax + top-1/top-2 selection fused with the capacity-bounded
// position scan, the top-2 finalisation, and the batch-prioritised (radix select) variant.
#include "launchers.hpp"
#include "scan.hpp"
#include "../../include/lancet_hip.h"
#include <algorithm>

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

// Calls f(x, j) for j = 0 .. E-1 in order and returns f (the functor carries its state by value, so that it
// stays in registers).  16-byte granules (4 fp32 or 8 half values) when the row allows.
template <int GD, typename F>
__device__ __forceinline__ F walk_row(const void* row, int E, F f) {
  constexpr int V = GD == LANCET_F32 ? 4 : 8;
  const bool vec = ((E & (V - 1)) == 0) && ((reinterpret_cast<uintptr_t>(row) & 15u) == 0);
  if (vec) {
    const u32x4* r = static_cast<const u32x4*>(row);
    for (int g = 0; g < E / V; ++g) {
      const u32x4 x = r[g];
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
    if (first) sum = (t.i1 < 0 ? 0.f : sum * expf(t.v1 - x)) + 1.f;
    else sum += expf(x - t.v1);
    t = consider<K>(t, x, j);
  }
};
struct SumExp {  // sequential sum in expert order
  float top, sum;
  __device__ __forceinline__ void operator()(float x, int) { sum += expf(x - top); }
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

struct RouteArgs {
  const void* gate;       // [S,E] of gate_dtype (NULL when idx_in is given)
  const void* noise;      // [S,E] of gate_dtype or NULL: added for the second choice (K = 2)
  const int32_t* idx_in;  // launcher-level entry: expert per token already chosen (may alias idx_out)
  const int32_t* used_in; // [E] or NULL (= zeros)
  void* gates_s;          // [K*S] of gate_dtype (NULL when idx_in is given)
  int32_t* idx_out;       // [K*S]
  int32_t* loc_out;       // [K*S]
  int32_t* used_out;      // [E]
  uint64_t* elems_out;    // [E]
  ScanWs ws;
  int S, E, C, M;
  int ntiles;
  int is_logits;
  int gate_dtype;         // LANCET_F32 / _BF16 / _F16: storage type of gate, noise and gates_s
  int seg_rows;           // place kernel: tiles per segment of the segment sums, 0 = there are none
};

// K = 1: everything is final when the tile knows its prefix.
// K = 2: ranks of both slots are produced in one pass (2E counters); slot-2 locations need the
//        slot-1 totals of all tiles, so raw (expert, rank, value) are left in the output arrays
//        and finalize_top2_kernel completes them.
template <int K, int GD>
__global__ __launch_bounds__(kTile) void route_scan_kernel(RouteArgs a) {
  extern __shared__ uint32_t s_cnt[];
  const int tid = threadIdx.x;
  const TileStart me = tile_begin(a.ws, a.ntiles);
  const uint32_t tile = me.tile;
  const int s = static_cast<int>(tile) * kTile + tid;
  const bool valid = s < a.S;
  if (!me.ok) {
    // no workspace to scan with: every token of this workgroup's range is marked, and so are the totals
    if (valid) {
#pragma unroll
      for (int j = 0; j < K; ++j) {
        a.idx_out[static_cast<size_t>(j) * a.S + s] = -1;
        a.loc_out[static_cast<size_t>(j) * a.S + s] = -1;
        if (a.gates_s) st_gate(a.gates_s, static_cast<size_t>(j) * a.S + s, 0.f, GD);
      }
    }
    if (blockIdx.x == 0) {
      for (int c = tid; c < a.E; c += kTile) {
        a.used_out[c] = -1;
        a.elems_out[c] = 0;
      }
    }
    return;
  }

  int e[K];
  float p[K];
#pragma unroll
  for (int j = 0; j < K; ++j) {
    e[j] = -1;
    p[j] = 0.f;
  }
  if (a.idx_in) {
    if (valid) {
      const int x = a.idx_in[s];
      e[0] = (x >= 0 && x < a.E) ? x : -1;
    }
  } else {
    const Routed r = route_tile_token<K, GD>(a.gate, a.noise, s, a.S, a.E, a.is_logits != 0, s_cnt);
    if (valid) {
      e[0] = r.e0;
      p[0] = r.p0;
      if (K == 2) {
        e[K - 1] = r.e1;
        p[K - 1] = r.p1;
      }
    }
  }
  uint32_t rank[K];
  bool mem[K];
#pragma unroll
  for (int j = 0; j < K; ++j) mem[j] = e[j] >= 0;
  const bool poisoned = tile_scan<K>(e, mem, a.E, me, a.ws, s_cnt, rank);

  if (K == 1) {
    if (valid) {
      if (poisoned) {
        a.idx_out[s] = -1;
        a.loc_out[s] = -1;
      } else if (e[0] >= 0) {
        const int used = a.used_in ? a.used_in[e[0]] : 0;
        const int r = static_cast<int>(rank[0]);
        a.loc_out[s] = r;
        a.idx_out[s] = (r >= a.C - used) ? -1 : e[0];
      } else if (!a.idx_in) {
        a.idx_out[s] = -1;
        a.loc_out[s] = 0;
      }
      if (a.gates_s) st_gate(a.gates_s, s, p[0], GD);
    }
    if (static_cast<int>(tile) == a.ntiles - 1) {
      // the last tile's inclusive prefix is the total; poisoned, it is worth nothing
      const uint32_t* s_agg = s_cnt + kWavesPerTile * a.E;
      const uint32_t* s_base = s_agg + a.E;
      for (int c = tid; c < a.E; c += kTile) {
        const int64_t used = a.used_in ? a.used_in[c] : 0;
        const int64_t total = static_cast<int64_t>(s_base[c]) + s_agg[c];
        const int64_t uo = min(used + total, static_cast<int64_t>(a.C));
        a.used_out[c] = poisoned ? -1 : static_cast<int32_t>(uo);
        a.elems_out[c] = poisoned ? 0 : static_cast<uint64_t>((uo - used) * a.M);
      }
    }
  } else {
    // raw values for finalize_top2_kernel; a poisoned tile marks its tokens, which that kernel passes on
    if (valid) {
#pragma unroll
      for (int j = 0; j < K; ++j) {
        a.idx_out[static_cast<size_t>(j) * a.S + s] = poisoned ? -1 : e[j];
        a.loc_out[static_cast<size_t>(j) * a.S + s] = poisoned ? -1 : static_cast<int>(rank[j]);
        st_gate(a.gates_s, static_cast<size_t>(j) * a.S + s, p[j], GD);
      }
    }
  }
  tile_end(a.ws, me, a.ntiles, K * a.E);
}

// ---- the same routing as two or three kernels that wait for nothing (scan_form) ------------------------------
// route_count_kernel: selection, ranks inside the tile, the tile's counts -> table.  Leaves expert, rank inside the
// tile and raw gate value in idx_out / loc_out / gates_s (idx_out is not written when the experts are given).
template <int K, int GD>
__global__ __launch_bounds__(kTile) void route_count_kernel(RouteArgs a) {
  extern __shared__ uint32_t s_cnt[];
  const int tid = threadIdx.x;
  const uint32_t tile = blockIdx.x;
  const int s = static_cast<int>(tile) * kTile + tid;
  const bool valid = s < a.S;
  int e[K];
  float p[K];
#pragma unroll
  for (int j = 0; j < K; ++j) {
    e[j] = -1;
    p[j] = 0.f;
  }
  if (a.idx_in) {
    if (valid) {
      const int x = a.idx_in[s];
      e[0] = (x >= 0 && x < a.E) ? x : -1;
    }
  } else {
    const Routed r = route_tile_token<K, GD>(a.gate, a.noise, s, a.S, a.E, a.is_logits != 0, s_cnt);
    if (valid) {
      e[0] = r.e0;
      p[0] = r.p0;
      if (K == 2) {
        e[K - 1] = r.e1;
        p[K - 1] = r.p1;
      }
    }
  }
  uint32_t rank[K];
  bool mem[K];
#pragma unroll
  for (int j = 0; j < K; ++j) mem[j] = e[j] >= 0;
  TileStart me;
  me.tile = tile, me.epoch = 0u, me.spin = 0u, me.ok = true;
  tile_scan<K, false>(e, mem, a.E, me, a.ws, s_cnt, rank);
  store_tile_counts(a.ws, tile, K * a.E, s_cnt);
  if (valid) {
#pragma unroll
    for (int j = 0; j < K; ++j) {
      if (!a.idx_in) a.idx_out[static_cast<size_t>(j) * a.S + s] = e[j];
      if (!a.idx_in || e[j] >= 0) a.loc_out[static_cast<size_t>(j) * a.S + s] = static_cast<int>(rank[j]);
      if (a.gates_s) st_gate(a.gates_s, static_cast<size_t>(j) * a.S + s, p[j], GD);
    }
  }
}

// route_place_kernel: every tile adds up what the tiles before it counted (and what all tiles counted) and finishes
// its tokens: what route_scan_kernel does after its look-back and, for K = 2, what finalize_top2_kernel does.
template <int K>
__global__ __launch_bounds__(kTile) void route_place_kernel(RouteArgs a) {
  extern __shared__ uint32_t s_sum[];  // [2][K * E]: before this tile, all tiles
  const int NC = K * a.E;
  uint32_t* s_before = s_sum;
  uint32_t* s_total = s_sum + NC;
  const uint32_t tile = blockIdx.x;
  sum_tile_counts(a.ws, tile, a.ntiles, NC, a.seg_rows, s_before, s_total);
  const int s = static_cast<int>(tile) * kTile + threadIdx.x;
  if (s < a.S) {
    if (K == 1) {
      const int x = a.idx_in ? a.idx_in[s] : a.idx_out[s];
      const int e = (x >= 0 && x < a.E) ? x : -1;
      if (e >= 0) {
        const int used = a.used_in ? a.used_in[e] : 0;
        const int r = static_cast<int>(s_before[e]) + a.loc_out[s];
        a.loc_out[s] = r;
        a.idx_out[s] = (r >= a.C - used) ? -1 : e;
      } else if (!a.idx_in) {
        a.idx_out[s] = -1;
        a.loc_out[s] = 0;
      }
    } else {
      const int e1 = a.idx_out[s], e2 = a.idx_out[a.S + s];
      const bool in1 = e1 >= 0 && e1 < a.E, in2 = e2 >= 0 && e2 < a.E;  // always (two experts at least)
      const int r1 = (in1 ? static_cast<int>(s_before[e1]) : 0) + a.loc_out[s];
      const int r2 = (in2 ? static_cast<int>(s_before[a.E + e2]) : 0) + a.loc_out[a.S + s];
      const int u1 = (a.used_in && in1) ? a.used_in[e1] : 0;
      const int u2 = (a.used_in && in2) ? a.used_in[e2] : 0;
      const bool keep1 = in1 && r1 < a.C - u1;
      const int64_t after1 = min(static_cast<int64_t>(u2) + (in2 ? s_total[e2] : 0u), static_cast<int64_t>(a.C));
      const bool keep2 = in2 && r2 < a.C - after1;
      a.idx_out[s] = keep1 ? e1 : -1;
      a.loc_out[s] = keep1 ? r1 : -1;
      a.idx_out[a.S + s] = keep2 ? e2 : -1;
      a.loc_out[a.S + s] = keep2 ? r2 + static_cast<int>(after1 - u2) : -1;
      // the raw values as the first kernel stored them (rounded to the gate type), normalised in fp32, rounded once
      const float g1 = keep1 ? ld_gate(a.gates_s, s, a.gate_dtype) : 0.f;
      const float g2 = keep2 ? ld_gate(a.gates_s, static_cast<size_t>(a.S) + s, a.gate_dtype) : 0.f;
      const float den = fmaxf(g1 + g2, 1.1920929e-07f);
      st_gate(a.gates_s, s, g1 / den, a.gate_dtype);
      st_gate(a.gates_s, static_cast<size_t>(a.S) + s, g2 / den, a.gate_dtype);
    }
  }
  if (tile == 0) {
    for (int c = threadIdx.x; c < a.E; c += kTile) {
      const int64_t used = a.used_in ? a.used_in[c] : 0;
      const int64_t total = static_cast<int64_t>(s_total[c]) + (K == 2 ? s_total[a.E + c] : 0u);
      const int64_t uo = min(used + total, static_cast<int64_t>(a.C));
      a.used_out[c] = static_cast<int32_t>(uo);
      a.elems_out[c] = static_cast<uint64_t>((uo - used) * a.M);
    }
  }
}

// Between count and place on long batches: one workgroup per segment of R tiles adds up the segment's rows.
__global__ __launch_bounds__(kTile) void scan_segsum_kernel(ScanWs ws, int ntiles, int NC, int R) {
  extern __shared__ uint32_t s_sum[];  // [NC]
  tile_segsum(ws, blockIdx.x, ntiles, NC, R, s_sum);
}

// Completes top-2 routing once all tiles are done: slot 1 is an ordinary top-1 encode with
// used_in; slot 2 is a top-1 encode whose used capacity is slot 1's result; locations are in
// the merged layout (slot-2 rows follow slot-1 rows of the same expert); combine weights are
// taken after the drop and normalised (docker/resources/sharded_moe.py:282-312).
__global__ __launch_bounds__(kTile) void finalize_top2_kernel(RouteArgs a) {
  const int s = blockIdx.x * kTile + threadIdx.x;
  // a workspace that is not set up: route_scan_kernel has marked every output already
  if (ld_agent(a.ws.hdr + kWsMagic) != kWsMagicValue) return;
  // totals of both slots = the last tile's inclusive descriptors, [2][E]; if that tile was poisoned there are
  // no totals and every token is marked, else the tokens of poisoned tiles carry marks of their own
  const uint64_t* tot = a.ws.desc + static_cast<size_t>(a.ntiles - 1) * 2 * a.E;
  const bool poisoned = desc_is_poisoned(ld_desc(tot));
  if (s < a.S) {
    if (poisoned) {
      a.idx_out[s] = a.idx_out[a.S + s] = -1;
      a.loc_out[s] = a.loc_out[a.S + s] = -1;
      st_gate(a.gates_s, s, 0.f, a.gate_dtype);
      st_gate(a.gates_s, static_cast<size_t>(a.S) + s, 0.f, a.gate_dtype);
    } else {
      const int e1 = a.idx_out[s], e2 = a.idx_out[a.S + s];
      const int r1 = a.loc_out[s], r2 = a.loc_out[a.S + s];
      const bool in1 = e1 >= 0 && e1 < a.E, in2 = e2 >= 0 && e2 < a.E;  // always, unless the scan left marks behind
      const int u1 = (a.used_in && in1) ? a.used_in[e1] : 0;
      const int u2 = (a.used_in && in2) ? a.used_in[e2] : 0;
      const bool keep1 = in1 && r1 < a.C - u1;
      const int64_t after1 = min(static_cast<int64_t>(u2) + (in2 ? static_cast<uint32_t>(ld_desc(tot + e2)) & kDescCountMask : 0u),
                                 static_cast<int64_t>(a.C));
      const bool keep2 = in2 && r2 < a.C - after1;
      a.idx_out[s] = keep1 ? e1 : -1;
      a.loc_out[s] = keep1 ? r1 : -1;
      a.idx_out[a.S + s] = keep2 ? e2 : -1;
      a.loc_out[a.S + s] = keep2 ? r2 + static_cast<int>(after1 - u2) : -1;
      // the raw values as the scan stored them (rounded to the gate type), normalised in fp32, rounded once
      const float g1 = keep1 ? ld_gate(a.gates_s, s, a.gate_dtype) : 0.f;
      const float g2 = keep2 ? ld_gate(a.gates_s, static_cast<size_t>(a.S) + s, a.gate_dtype) : 0.f;
      const float den = fmaxf(g1 + g2, 1.1920929e-07f);
      st_gate(a.gates_s, s, g1 / den, a.gate_dtype);
      st_gate(a.gates_s, static_cast<size_t>(a.S) + s, g2 / den, a.gate_dtype);
    }
  }
  if (blockIdx.x == 0) {
    for (int c = threadIdx.x; c < a.E; c += kTile) {
      const int64_t used = a.used_in ? a.used_in[c] : 0;
      const int64_t total = static_cast<int64_t>(static_cast<uint32_t>(ld_desc(tot + c)) & kDescCountMask) +
                            (static_cast<uint32_t>(ld_desc(tot + a.E + c)) & kDescCountMask);
      const int64_t uo = min(used + total, static_cast<int64_t>(a.C));
      a.used_out[c] = poisoned ? -1 : static_cast<int32_t>(uo);
      a.elems_out[c] = poisoned ? 0 : static_cast<uint64_t>((uo - used) * a.M);
    }
  }
}

// Selection only (no scan).
template <int K, int GD>
__global__ __launch_bounds__(kTile) void gate_topk_kernel(const void* gate, const void* noise, int S, int E,
                                                          int is_logits, int32_t* idx, void* val) {
  extern __shared__ uint32_t s_stage[];
  const int s = blockIdx.x * kTile + threadIdx.x;
  const Routed r = route_tile_token<K, GD>(gate, noise, s, S, E, is_logits != 0, s_stage);
  if (s >= S) return;
  idx[s] = r.e0;
  st_gate(val, s, r.p0, GD);
  if (K == 2) {
    idx[static_cast<size_t>(S) + s] = r.e1;
    st_gate(val, static_cast<size_t>(S) + s, r.p1, GD);
  }
}

__global__ void top2_normalize_kernel(const void* raw, const int32_t* idx, int S, void* out, int gd) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= S) return;
  const float g1 = idx[s] >= 0 ? ld_gate(raw, s, gd) : 0.f;
  const float g2 = idx[S + s] >= 0 ? ld_gate(raw, static_cast<size_t>(S) + s, gd) : 0.f;
  const float den = fmaxf(g1 + g2, 1.1920929e-07f);
  st_gate(out, s, g1 / den, gd);
  st_gate(out, static_cast<size_t>(S) + s, g2 / den, gd);
}

__global__ void fill_u32_kernel(uint32_t* p, size_t n, uint32_t v) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x)
    p[i] = v;
}

// ---------------------------------------------------------------------------------------
// Batch-prioritised routing.
//   bpr_select_kernel : one workgroup per expert.  Finds, with a 4 x 8-bit radix select on the
//                       order-preserving integer image of the fp32 priority, the C-th largest
//                       priority among the expert's tokens (threshold), how many ties at the
//                       threshold may stay (quota, lowest token ids first) and how many ties
//                       lie before the partition (ties_before).
//   bpr_scan_kernel   : tile scan over the partition with two counter sets (tokens above the
//                       threshold / tokens at the threshold); a token stays iff it is above,
//                       or at the threshold with global tie rank < quota; its location is
//                       above_before + min(tie_rank, quota) - min(ties_before, quota).
// Equivalent to the reference's stable descending argsort + keep-first-C + compaction
// (src/op/dialect/cuda/moe.cc:638-683, tutel_moe_dispatch.cu:259-363) without sorting.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ uint32_t order_key(float x) {
  if (x == 0.f) x = 0.f;  // -0 and +0 compare equal in a float sort
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Everything the batch-prioritised routing keeps in the scan's workspace behind the descriptor table is a
// 64-bit word tagged "not a descriptor" (foreign_word), the value in the low half: tok[s] also carries the
// token's expert + 1 in the tag's low bits; par[0..2][e] = threshold, tie quota, ties before the partition,
// par[3][e] = tokens of the expert before the partition inside the tile of 256 tokens that holds its start.
// For the select kernel the prepare kernel also leaves every tile's keys grouped by expert, in token order
// (keys[tile][256]) and where each expert's group lies (groups[e][tile] = start | count << 16): an expert's
// workgroup then reads its own keys and one word per tile instead of the whole batch.
struct BprArgs {
  uint64_t* tok;         // [S0] expert and priority (gate value of the chosen expert) per token
  uint64_t* par;         // [4][E]
  uint64_t* keys;        // [ntiles0][256] order keys, grouped by expert inside a tile
  uint64_t* groups;      // [E][ntiles0]
  int ntiles0;           // tiles of the whole batch
  int S0, S, E, C, M;
  int part_lo;           // first token of the partition
  int ntiles;
  int seg_rows;          // place kernel: tiles per segment of the segment sums, 0 = there are none
  int gate_dtype;        // storage type of gates_s (and of the gate the priorities came from)
  void* gates_s;         // [S]
  int32_t* idx_out;      // [S]
  int32_t* loc_out;      // [S]
  int32_t* used_out;     // [E]
  uint64_t* elems_out;   // [E]
  ScanWs ws;
};

constexpr int kSelectThreads = 1024;

__device__ __forceinline__ int tok_expert(uint64_t w) { return static_cast<int>((w >> 32) & 0xffffu) - 1; }
__device__ __forceinline__ float tok_prio(uint64_t w) { return __uint_as_float(static_cast<uint32_t>(w)); }
__device__ __forceinline__ uint32_t par_value(const uint64_t* p) { return static_cast<uint32_t>(*p); }

// first choice and its gate value (or softmax probability) of every token of the batch
// (the priority is the gate value as gates_s will hold it: rounded to the gate type); the tile's keys grouped
// by expert
template <int GD>
__global__ __launch_bounds__(kTile) void bpr_prepare_kernel(const void* gate, int is_logits, BprArgs a) {
  extern __shared__ uint32_t s_cnt[];
  const int tid = threadIdx.x;
  const uint32_t tile = blockIdx.x;
  const int s = static_cast<int>(tile) * kTile + tid;
  int cls[1] = {-1};
  uint32_t key = 0;
  const Routed r = route_tile_token<1, GD>(gate, nullptr, s, a.S0, a.E, is_logits != 0, s_cnt);
  if (s < a.S0) {
    const float prio = round_gate(r.p0, GD);
    a.tok[s] = foreign_word(static_cast<uint32_t>(r.e0 + 1), __float_as_uint(prio));
    cls[0] = r.e0;
    key = order_key(prio);
  }
  const bool mem[1] = {cls[0] >= 0};
  uint32_t rank[1];
  TileStart me;
  me.tile = tile, me.epoch = 0u, me.spin = 0u, me.ok = true;
  tile_scan<1, false>(cls, mem, a.E, me, a.ws, s_cnt, rank);  // rank among the tile's tokens of the same expert
  __syncthreads();  // every wave has its ranks: rows of s_cnt can be reused
  // rows of s_cnt the scan without look-back leaves unused (zero): where each expert's group starts, and how many
  // of its tokens come before the partition
  const uint32_t* s_agg = s_cnt + kWavesPerTile * a.E;
  uint32_t* s_start = s_cnt + (kWavesPerTile + 1) * a.E;
  uint32_t* s_early = s_start + a.E;
  const bool holds_start = static_cast<int>(tile) == a.part_lo / kTile;
  if (tid < kWave) {
    // exclusive scan of the tile's counts over the experts: lane l owns `per` consecutive experts
    const int per = (a.E + kWave - 1) / kWave;
    uint32_t mine = 0;
    for (int i = 0; i < per; ++i) mine += (tid * per + i < a.E) ? s_agg[tid * per + i] : 0u;
    uint32_t inc = mine;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const uint32_t v = __shfl_up(inc, off, kWave);
      if (tid >= off) inc += v;
    }
    uint32_t run = inc - mine;
    for (int i = 0; i < per; ++i) {
      const int c = tid * per + i;
      if (c < a.E) {
        s_start[c] = run;
        run += s_agg[c];
      }
    }
  }
  if (holds_start && cls[0] >= 0 && s < a.part_lo) atomicAdd(&s_early[cls[0]], 1u);
  __syncthreads();
  if (cls[0] >= 0) a.keys[static_cast<size_t>(tile) * kTile + s_start[cls[0]] + rank[0]] = foreign_word(0u, key);
  for (int c = tid; c < a.E; c += kTile) {
    a.groups[static_cast<size_t>(c) * a.ntiles0 + tile] = foreign_word(0u, s_start[c] | (s_agg[c] << 16));
    if (holds_start) a.par[3 * a.E + c] = foreign_word(0u, s_early[c]);
  }
}

// One descending step of the radix select, by the first wave of the workgroup: the digit that holds the need-th
// largest key among the keys counted in hist[256], and what is still needed inside that digit.  Lane l owns the
// digits 255 - 4l .. 252 - 4l; a wave scan of the lanes' sums finds the lane, the lane finds the digit.  (A single
// thread walking the 256 counters is a chain of dependent LDS reads: it was most of this kernel's time.)
__device__ __forceinline__ void select_digit(const uint32_t* hist, uint32_t prefix, uint32_t* s_prefix, uint32_t* s_need) {
  const int lane = threadIdx.x;  // called with threadIdx.x < kWave
  const uint32_t need = *s_need;
  uint32_t h[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) h[j] = hist[255 - (4 * lane + j)];
  const uint32_t mine = h[0] + h[1] + h[2] + h[3];
  uint32_t inc = mine;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t v = __shfl_up(inc, off, kWave);
    if (lane >= off) inc += v;
  }
  uint32_t run = inc - mine;  // keys in digits above this lane's
  if (run < need && need <= inc) {
    int j = 0;
    for (; j < 3; ++j) {
      if (need <= run + h[j]) break;
      run += h[j];
    }
    *s_need = need - run;
    *s_prefix = (prefix << 8) | static_cast<uint32_t>(255 - (4 * lane + j));
  } else if (lane == kWave - 1 && inc < need) {
    // fewer keys than needed (does not happen with consistent counts): digit 0 takes what is left
    *s_need = need - (inc - h[3]);
    *s_prefix = prefix << 8;
  }
}

constexpr int kSelectKeys = 10240;  // keys of one expert kept in LDS (40 KB)
constexpr int kSelectTiles = 4096;  // tiles whose group positions fit in LDS (16 KB): batches up to 1M tokens

// exclusive scan over the kSelectThreads values of a workgroup; *total = their sum.  s_wave: 16 words of LDS.
__device__ __forceinline__ uint32_t select_block_scan(uint32_t v, uint32_t* s_wave, uint32_t* total) {
  const int lane = lane_id(), w = threadIdx.x / kWave;
  uint32_t inc = v;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t u = __shfl_up(inc, off, kWave);
    if (lane >= off) inc += u;
  }
  __syncthreads();  // s_wave may still be read from an earlier call
  if (lane == kWave - 1) s_wave[w] = inc;
  __syncthreads();
  uint32_t before = 0, all = 0;
#pragma unroll
  for (int k = 0; k < kSelectThreads / kWave; ++k) {
    const uint32_t t = s_wave[k];
    before += (k < w) ? t : 0u;
    all += t;
  }
  *total = all;
  return before + inc - v;
}

// the i-th key of the expert in token order: its tile by bisection over the tiles' positions (s_pos: position of
// the tile's first key in the low 22 bits, start of the expert's group inside the tile above them)
__device__ __forceinline__ uint32_t select_gather(const BprArgs& a, const uint32_t* s_pos, uint32_t i) {
  int lo = 0, hi = a.ntiles0 - 1;  // last tile whose position is <= i
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if ((s_pos[mid] & 0x3fffffu) <= i) lo = mid; else hi = mid - 1;
  }
  const uint32_t w = s_pos[lo];
  return static_cast<uint32_t>(a.keys[static_cast<size_t>(lo) * kTile + (w >> 22) + (i - (w & 0x3fffffu))]);
}

__global__ __launch_bounds__(kSelectThreads) void bpr_select_kernel(BprArgs a) {
  __shared__ uint32_t s_keys[kSelectKeys];
  __shared__ uint32_t s_pos[kSelectTiles];
  __shared__ uint32_t hist[256];
  __shared__ uint32_t s_wave[kSelectThreads / kWave];
  __shared__ uint32_t s_prefix, s_need, s_count;
  const int e = blockIdx.x;
  const int tid = threadIdx.x;
  // The expert's keys, in token order.  Up to kSelectTiles tiles, the prepare kernel's groups say where they are:
  // positions by a scan over the tiles, then the keys themselves into LDS (or, more than LDS holds, fetched again
  // in every pass).  Longer batches are read whole, once per pass.
  const bool grouped = a.ntiles0 <= kSelectTiles;
  uint32_t count = 0, nfront = 0;
  if (grouped) {
    uint32_t carry = 0;
    const int tstart = a.part_lo / kTile;  // the tile that holds the partition's first token
    for (int base = 0; base < a.ntiles0; base += kSelectThreads) {
      const int t = base + tid;
      const uint32_t g = t < a.ntiles0 ? static_cast<uint32_t>(a.groups[static_cast<size_t>(e) * a.ntiles0 + t]) : 0u;
      uint32_t total;
      const uint32_t pos = carry + select_block_scan(g >> 16, s_wave, &total);
      if (t < a.ntiles0) s_pos[t] = pos | ((g & 0xffffu) << 22);
      carry += total;
    }
    __syncthreads();
    count = carry;
    nfront = a.S0 > 0 ? (s_pos[tstart] & 0x3fffffu) + par_value(a.par + 3 * a.E + e) : 0u;
  } else {
    if (tid == 0) s_count = 0;
    __syncthreads();
    uint32_t local = 0;
    for (int s = tid; s < a.S0; s += kSelectThreads) local += (tok_expert(a.tok[s]) == e);
    if (local) atomicAdd(&s_count, local);
    __syncthreads();
    count = s_count;
  }
  if (a.C <= 0) {
    // nothing fits: no key is above the largest threshold and the tie quota is zero
    if (tid == 0) {
      a.par[e] = foreign_word(0u, 0xffffffffu);
      a.par[a.E + e] = foreign_word(0u, 0u);
      a.par[2 * a.E + e] = foreign_word(0u, 0u);
    }
    return;
  }
  if (count <= static_cast<uint32_t>(a.C)) {
    // everything fits: every key is above threshold 0 or ties with it under an unlimited quota
    if (tid == 0) {
      a.par[e] = foreign_word(0u, 0u);
      a.par[a.E + e] = foreign_word(0u, 0x7fffffffu);
      a.par[2 * a.E + e] = foreign_word(0u, 0u);
    }
    return;
  }
  const bool in_lds = grouped && count <= kSelectKeys;
  if (in_lds) {
    for (uint32_t i = tid; i < count; i += kSelectThreads) s_keys[i] = select_gather(a, s_pos, i);
  }
  if (tid == 0) {
    s_prefix = 0;
    s_need = static_cast<uint32_t>(a.C);
  }
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    const uint32_t prefix = s_prefix;
    if (grouped) {
      for (uint32_t i = tid; i < count; i += kSelectThreads) {
        const uint32_t k = in_lds ? s_keys[i] : select_gather(a, s_pos, i);
        if (pass == 0 || (k >> (shift + 8)) == prefix) atomicAdd(&hist[(k >> shift) & 0xffu], 1u);
      }
    } else {
      for (int s = tid; s < a.S0; s += kSelectThreads) {
        const uint64_t t = a.tok[s];
        if (tok_expert(t) != e) continue;
        const uint32_t k = order_key(tok_prio(t));
        if (pass == 0 || (k >> (shift + 8)) == prefix) atomicAdd(&hist[(k >> shift) & 0xffu], 1u);
      }
    }
    __syncthreads();
    if (tid < kWave) select_digit(hist, prefix, &s_prefix, &s_need);
    __syncthreads();
  }
  const uint32_t thr = s_prefix;
  // ties that precede the partition
  if (tid == 0) s_count = 0;
  __syncthreads();
  uint32_t local = 0;
  if (grouped) {
    for (uint32_t i = tid; i < nfront; i += kSelectThreads) local += ((in_lds ? s_keys[i] : select_gather(a, s_pos, i)) == thr);
  } else {
    for (int s = tid; s < a.part_lo; s += kSelectThreads) {
      const uint64_t t = a.tok[s];
      local += (tok_expert(t) == e && order_key(tok_prio(t)) == thr);
    }
  }
  if (local) atomicAdd(&s_count, local);
  __syncthreads();
  if (tid == 0) {
    a.par[e] = foreign_word(0u, thr);
    a.par[a.E + e] = foreign_word(0u, s_need);
    a.par[2 * a.E + e] = foreign_word(0u, s_count);
  }
}

__global__ __launch_bounds__(kTile) void bpr_scan_kernel(BprArgs a) {
  extern __shared__ uint32_t s_cnt[];
  const int tid = threadIdx.x;
  const TileStart me = tile_begin(a.ws, a.ntiles);
  const uint32_t tile = me.tile;
  const int sl = static_cast<int>(tile) * kTile + tid;  // token inside the partition
  const bool valid = sl < a.S;
  if (!me.ok) {
    if (valid) {
      a.idx_out[sl] = -1;
      a.loc_out[sl] = -1;
      st_gate(a.gates_s, sl, 0.f, a.gate_dtype);
    }
    if (blockIdx.x == 0) {
      for (int c = tid; c < a.E; c += kTile) {
        a.used_out[c] = -1;
        a.elems_out[c] = 0;
      }
    }
    return;
  }
  int cls[2] = {-1, -1};
  bool mem[2] = {false, false};
  float prio = 0.f;
  if (valid) {
    const uint64_t t = a.tok[a.part_lo + sl];
    const int e = tok_expert(t);
    prio = tok_prio(t);
    if (e >= 0 && e < a.E) {
      const uint32_t k = order_key(prio);
      const uint32_t thr = par_value(a.par + e);
      cls[0] = cls[1] = e;
      mem[0] = k > thr;   // above the threshold: always stays
      mem[1] = k == thr;  // at the threshold: stays while the quota lasts
    }
  }
  uint32_t rank[2];
  const bool poisoned = tile_scan<2>(cls, mem, a.E, me, a.ws, s_cnt, rank);
  if (valid) {
    int idx = -1, loc = -1;
    if (cls[0] >= 0 && !poisoned) {
      const int e = cls[0];
      const int64_t q = static_cast<int32_t>(par_value(a.par + a.E + e));
      const int64_t tb = static_cast<int32_t>(par_value(a.par + 2 * a.E + e));
      const int64_t tie_rank = tb + rank[1];
      if (mem[0] || (mem[1] && tie_rank < q)) {
        idx = e;
        loc = static_cast<int>(static_cast<int64_t>(rank[0]) + min(tie_rank, q) - min(tb, q));
      }
    }
    a.idx_out[sl] = idx;
    a.loc_out[sl] = loc;
    st_gate(a.gates_s, sl, prio, a.gate_dtype);
  }
  if (static_cast<int>(tile) == a.ntiles - 1) {
    const uint32_t* s_agg = s_cnt + kWavesPerTile * 2 * a.E;
    const uint32_t* s_base = s_agg + 2 * a.E;
    for (int c = tid; c < a.E; c += kTile) {
      const int64_t q = static_cast<int32_t>(par_value(a.par + a.E + c));
      const int64_t tb = static_cast<int32_t>(par_value(a.par + 2 * a.E + c));
      const int64_t above = static_cast<int64_t>(s_base[c]) + s_agg[c];
      const int64_t ties = static_cast<int64_t>(s_base[a.E + c]) + s_agg[a.E + c];
      const int64_t kept = above + min(tb + ties, q) - min(tb, q);
      const int64_t uo = min(kept, static_cast<int64_t>(a.C));
      a.used_out[c] = poisoned ? -1 : static_cast<int32_t>(uo);
      a.elems_out[c] = poisoned ? 0 : static_cast<uint64_t>(uo * a.M);
    }
  }
  tile_end(a.ws, me, a.ntiles, 2 * a.E);
}

// ---- the same scan as two or three kernels that wait for nothing (scan_form) ---------------------------------
// class and membership of a partition token in the two counter sets, from its word and the expert's threshold
struct BprClass {
  int e;        // expert, -1 = none
  bool above;   // above the threshold: always stays
  bool tie;     // at the threshold: stays while the quota lasts
  float prio;
};
__device__ __forceinline__ BprClass bpr_classify(const BprArgs& a, int sl) {
  BprClass c = {-1, false, false, 0.f};
  const uint64_t t = a.tok[a.part_lo + sl];
  const int e = tok_expert(t);
  c.prio = tok_prio(t);
  if (e >= 0 && e < a.E) {
    const uint32_t k = order_key(c.prio);
    const uint32_t thr = par_value(a.par + e);
    c.e = e;
    c.above = k > thr;
    c.tie = k == thr;
  }
  return c;
}

// bpr_count_kernel: ranks inside the tile in both counter sets (left in loc_out, 16 bits each: a tile has 256
// tokens), the tile's counts -> table.
__global__ __launch_bounds__(kTile) void bpr_count_kernel(BprArgs a) {
  extern __shared__ uint32_t s_cnt[];
  const uint32_t tile = blockIdx.x;
  const int sl = static_cast<int>(tile) * kTile + threadIdx.x;
  const bool valid = sl < a.S;
  int cls[2] = {-1, -1};
  bool mem[2] = {false, false};
  if (valid) {
    const BprClass c = bpr_classify(a, sl);
    cls[0] = cls[1] = c.e;
    mem[0] = c.above;
    mem[1] = c.tie;
  }
  uint32_t rank[2];
  TileStart me;
  me.tile = tile, me.epoch = 0u, me.spin = 0u, me.ok = true;
  tile_scan<2, false>(cls, mem, a.E, me, a.ws, s_cnt, rank);
  store_tile_counts(a.ws, tile, 2 * a.E, s_cnt);
  if (valid) a.loc_out[sl] = static_cast<int>(rank[0] | (rank[1] << 16));
}

// bpr_place_kernel: adds what the tiles before counted and finishes the tile's tokens (what bpr_scan_kernel does
// after its look-back).
__global__ __launch_bounds__(kTile) void bpr_place_kernel(BprArgs a) {
  extern __shared__ uint32_t s_sum[];  // [2][2E]: before this tile, all tiles
  const int NC = 2 * a.E;
  uint32_t* s_before = s_sum;
  uint32_t* s_total = s_sum + NC;
  const uint32_t tile = blockIdx.x;
  sum_tile_counts(a.ws, tile, a.ntiles, NC, a.seg_rows, s_before, s_total);
  const int sl = static_cast<int>(tile) * kTile + threadIdx.x;
  if (sl < a.S) {
    const BprClass c = bpr_classify(a, sl);
    int idx = -1, loc = -1;
    if (c.e >= 0) {
      const uint32_t packed = static_cast<uint32_t>(a.loc_out[sl]);
      const int64_t q = static_cast<int32_t>(par_value(a.par + a.E + c.e));
      const int64_t tb = static_cast<int32_t>(par_value(a.par + 2 * a.E + c.e));
      const int64_t above_before = static_cast<int64_t>(s_before[c.e]) + (packed & 0xffffu);
      const int64_t tie_rank = tb + s_before[a.E + c.e] + (packed >> 16);
      if (c.above || (c.tie && tie_rank < q)) {
        idx = c.e;
        loc = static_cast<int>(above_before + min(tie_rank, q) - min(tb, q));
      }
    }
    a.idx_out[sl] = idx;
    a.loc_out[sl] = loc;
    st_gate(a.gates_s, sl, c.prio, a.gate_dtype);
  }
  if (tile == 0) {
    for (int c = threadIdx.x; c < a.E; c += kTile) {
      const int64_t q = static_cast<int32_t>(par_value(a.par + a.E + c));
      const int64_t tb = static_cast<int32_t>(par_value(a.par + 2 * a.E + c));
      const int64_t kept = static_cast<int64_t>(s_total[c]) + min(tb + static_cast<int64_t>(s_total[a.E + c]), q) - min(tb, q);
      const int64_t uo = min(kept, static_cast<int64_t>(a.C));
      a.used_out[c] = static_cast<int32_t>(uo);
      a.elems_out[c] = static_cast<uint64_t>(uo * a.M);
    }
  }
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
int64_t scan_num_tiles(int64_t S) { return S > 0 ? (S + kTile - 1) / kTile : 1; }

// LDS a selecting kernel needs for the rows it stages (0: it walks them directly)
static size_t stage_lds_bytes(int gate_dtype, const void* gate, const void* noise, int S, int E) {
  bool staged = false;
  LANCET_GATE_SWITCH(gate_dtype, staged = rows_are_staged<GD>(gate, noise, S, E))
  return staged ? kStageBytes : 0;
}

size_t scan_workspace_bytes(int64_t S, int64_t E, int nsets) {
  // (two words per tile at least: the forms without look-back keep the tiles' counts, two to a word, and the
  // segments' sums in the room of the look-back's table)
  return scan_ws_bytes(scan_num_tiles(S), std::max<int64_t>(nsets * E, 2));
}

size_t bpr_workspace_bytes(int64_t S0, int64_t S, int64_t E) {
  // descriptor table of the partition's scan | tok[S0] | par[4][E] | keys[tiles of the batch][256] | groups[E][tiles]
  const size_t t0 = static_cast<size_t>(scan_num_tiles(S0));
  return scan_workspace_bytes(S, E, 2) +
         (static_cast<size_t>(S0) + 4 * static_cast<size_t>(E) + t0 * kTile + static_cast<size_t>(E) * t0) * 8;
}

hipError_t run_scan_ws_init(void* ws, size_t nbytes, hipStream_t st) {
  const size_t nwords = nbytes / sizeof(uint32_t);
  if (nwords < kScanHeaderWords) return hipErrorInvalidValue;
  const int blocks = static_cast<int>(std::min<size_t>((nwords + 255) / 256, 1024));
  scan_ws_init_kernel<<<blocks, 256, 0, st>>>(static_cast<uint32_t*>(ws), nwords);
  return hipGetLastError();
}

hipError_t run_scan_ws_set_spin(void* ws, uint32_t limit, hipStream_t st) {
  return run_fill_u32(static_cast<uint32_t*>(ws) + kWsSpin, 1, limit, st);
}

hipError_t run_scan_ws_set_epoch(void* ws, uint32_t epoch, hipStream_t st) {
  return run_fill_u32(static_cast<uint32_t*>(ws) + kWsEpoch, 1, epoch, st);
}

hipError_t run_scan_ws_take_error(void* ws, int* error_out, hipStream_t st) {
  uint32_t word = 0;
  uint32_t* err = static_cast<uint32_t*>(ws) + kWsError;
  hipError_t e = hipMemcpyAsync(&word, err, sizeof(word), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e == hipSuccess && word != 0u) {  // the reader, and only the reader, clears it
    e = run_fill_u32(err, 1, 0u, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
  }
  *error_out = word != 0u;
  return e;
}

hipError_t run_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t st) {
  if (n == 0) return hipSuccess;
  const int blocks = static_cast<int>(std::min<size_t>((n + 255) / 256, 1024));
  fill_u32_kernel<<<blocks, 256, 0, st>>>(p, n, v);
  return hipGetLastError();
}

hipError_t run_gate_topk(const void* gate, const void* noise, int S, int E, int K, bool is_logits, int gate_dtype,
                         int32_t* idx, void* val, hipStream_t st) {
  if (S == 0) return hipSuccess;
  const int blocks = (S + kTile - 1) / kTile;
  const size_t lds = stage_lds_bytes(gate_dtype, gate, K == 2 ? noise : nullptr, S, E);
  LANCET_GATE_SWITCH(gate_dtype,
    if (K == 1) gate_topk_kernel<1, GD><<<blocks, kTile, lds, st>>>(gate, nullptr, S, E, is_logits, idx, val);
    else gate_topk_kernel<2, GD><<<blocks, kTile, lds, st>>>(gate, noise, S, E, is_logits, idx, val))
  return hipGetLastError();
}

hipError_t run_route_scan(const void* gate, const void* noise, const int32_t* idx_in, const int32_t* used_in, int S,
                          int E, int C, int M, int K, bool is_logits, int gate_dtype, void* gates_s,
                          int32_t* idx_out, int32_t* loc_out, int32_t* used_out,
                          uint64_t* elems_out, void* ws, hipStream_t st, bool force_lookback) {
  RouteArgs a;
  a.gate = gate;
  a.noise = K == 2 ? noise : nullptr;
  a.idx_in = idx_in;
  a.used_in = used_in;
  a.gates_s = gates_s;
  a.idx_out = idx_out;
  a.loc_out = loc_out;
  a.used_out = used_out;
  a.elems_out = elems_out;
  a.S = S;
  a.E = E;
  a.C = C;
  a.M = M;
  a.ntiles = static_cast<int>(scan_num_tiles(S));
  a.is_logits = is_logits;
  a.gate_dtype = gate_dtype;
  a.ws = scan_ws_view(ws);
  a.seg_rows = 0;
  hipError_t err = hipSuccess;
  const size_t lds = std::max(scan_lds_bytes(K * E), idx_in ? size_t(0) : stage_lds_bytes(gate_dtype, gate, a.noise, S, E));
  const ScanForm form = scan_form(a.ntiles, static_cast<int64_t>(K) * E, K, force_lookback);
  if (form != kScanLookback) {
    // two or three kernels that wait for nothing instead of a look-back between tiles that all run at once
    const int NC = K * E;
    const size_t lds2 = 2 * static_cast<size_t>(NC) * sizeof(uint32_t);
    if (K == 1) {
      LANCET_GATE_SWITCH(gate_dtype, (route_count_kernel<1, GD><<<a.ntiles, kTile, lds, st>>>(a)))
    } else {
      LANCET_GATE_SWITCH(gate_dtype, (route_count_kernel<2, GD><<<a.ntiles, kTile, lds, st>>>(a)))
    }
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    if (form == kScanCountSegPlace) {
      a.seg_rows = seg_rows(a.ntiles);
      scan_segsum_kernel<<<(a.ntiles + a.seg_rows - 1) / a.seg_rows, kTile, NC * sizeof(uint32_t), st>>>(a.ws, a.ntiles, NC, a.seg_rows);
      err = hipGetLastError();
      if (err != hipSuccess) return err;
    }
    if (K == 1) route_place_kernel<1><<<a.ntiles, kTile, lds2, st>>>(a);
    else route_place_kernel<2><<<a.ntiles, kTile, lds2, st>>>(a);
    return hipGetLastError();
  }
  if (K == 1) {
    LANCET_GATE_SWITCH(gate_dtype, (route_scan_kernel<1, GD><<<a.ntiles, kTile, lds, st>>>(a)))
  } else {
    LANCET_GATE_SWITCH(gate_dtype, (route_scan_kernel<2, GD><<<a.ntiles, kTile, lds, st>>>(a)))
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    finalize_top2_kernel<<<a.ntiles, kTile, 0, st>>>(a);
  }
  return hipGetLastError();
}

hipError_t run_bpr_route(const void* gate, int S0, int E, int C, int M, int n_partitions,
                         int partition_id, bool is_logits, int gate_dtype, void* gates_s, int32_t* idx_out,
                         int32_t* loc_out, int32_t* used_out, uint64_t* elems_out, void* ws,
                         hipStream_t st, bool force_lookback) {
  const int S = S0 / n_partitions;
  BprArgs a;
  a.S0 = S0;
  a.S = S;
  a.E = E;
  a.C = C;
  a.M = M;
  a.part_lo = partition_id * S;
  a.ntiles = static_cast<int>(scan_num_tiles(S));
  a.ws = scan_ws_view(ws);
  a.tok = reinterpret_cast<uint64_t*>(static_cast<char*>(ws) + scan_workspace_bytes(S, E, 2));
  a.par = a.tok + S0;
  a.ntiles0 = static_cast<int>(scan_num_tiles(S0));
  a.keys = a.par + 4 * static_cast<size_t>(E);
  a.groups = a.keys + static_cast<size_t>(a.ntiles0) * kTile;
  a.gates_s = gates_s;
  a.gate_dtype = gate_dtype;
  a.idx_out = idx_out;
  a.loc_out = loc_out;
  a.used_out = used_out;
  a.elems_out = elems_out;
  hipError_t err = hipSuccess;
  // (an empty batch still runs one tile, which leaves empty groups for the select kernel)
  LANCET_GATE_SWITCH(gate_dtype, (bpr_prepare_kernel<GD><<<a.ntiles0, kTile, std::max(scan_lds_bytes(E), stage_lds_bytes(gate_dtype, gate, nullptr, S0, E)), st>>>(gate, is_logits, a)))
  err = hipGetLastError();
  if (err != hipSuccess) return err;
  bpr_select_kernel<<<E, kSelectThreads, 0, st>>>(a);
  err = hipGetLastError();
  if (err != hipSuccess) return err;
  a.seg_rows = 0;
  const ScanForm form = scan_form(a.ntiles, 2 * static_cast<int64_t>(E), 2, force_lookback);
  if (form != kScanLookback) {
    bpr_count_kernel<<<a.ntiles, kTile, scan_lds_bytes(2 * E), st>>>(a);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    if (form == kScanCountSegPlace) {
      a.seg_rows = seg_rows(a.ntiles);
      scan_segsum_kernel<<<(a.ntiles + a.seg_rows - 1) / a.seg_rows, kTile, 2 * E * sizeof(uint32_t), st>>>(a.ws, a.ntiles, 2 * E, a.seg_rows);
      err = hipGetLastError();
      if (err != hipSuccess) return err;
    }
    bpr_place_kernel<<<a.ntiles, kTile, 4 * static_cast<size_t>(E) * sizeof(uint32_t), st>>>(a);
    return hipGetLastError();
  }
  bpr_scan_kernel<<<a.ntiles, kTile, scan_lds_bytes(2 * E), st>>>(a);
  return hipGetLastError();
}

hipError_t run_top2_normalize(const void* raw, const int32_t* idx, int S, int gate_dtype, void* out, hipStream_t st) {
  if (S == 0) return hipSuccess;
  top2_normalize_kernel<<<(S + 255) / 256, 256, 0, st>>>(raw, idx, S, out, gate_dtype);
  return hipGetLastError();
}

}  // namespace lancet
