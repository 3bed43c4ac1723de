// Batch-prioritised routing (raf.op.moe_encode_batch_prioritized): radix select instead of an argsort, then
// a position scan with two counter sets.
#include "launchers.hpp"
#include "select.hpp"
#include <algorithm>

namespace lancet {

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
size_t bpr_workspace_bytes(int64_t S0, int64_t S, int64_t E) {
  // descriptor table of the partition's scan | tok[S0] | par[4][E] | keys[tiles of the batch][256] | groups[E][tiles]
  const size_t t0 = static_cast<size_t>(scan_num_tiles(S0));
  return scan_workspace_bytes(S, E, 2) +
         (static_cast<size_t>(S0) + 4 * static_cast<size_t>(E) + t0 * kTile + static_cast<size_t>(E) * t0) * 8;
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
      err = run_scan_segsum(ws, a.ntiles, 2 * E, a.seg_rows, st);
      if (err != hipSuccess) return err;
    }
    bpr_place_kernel<<<a.ntiles, kTile, 4 * static_cast<size_t>(E) * sizeof(uint32_t), st>>>(a);
    return hipGetLastError();
  }
  bpr_scan_kernel<<<a.ntiles, kTile, scan_lds_bytes(2 * E), st>>>(a);
  return hipGetLastError();
}

}  // namespace lancet
