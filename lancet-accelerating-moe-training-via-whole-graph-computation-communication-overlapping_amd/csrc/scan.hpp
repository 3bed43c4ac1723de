// Capacity-bounded position scan: for every token, the number of earlier tokens (in token
// order) that chose the same expert.  One pass over token tiles:
//   1. wave level  - match lanes with the same expert by ballots over the bits of the expert
//                    id; rank inside the wave = popcount of the peer mask below the lane;
//   2. tile level  - per-wave counts in LDS, exclusive scan over the waves of the tile;
//   3. across tiles - decoupled look-back over a [tiles][counters] descriptor table.  Every
//                    descriptor is ONE 64-bit word: the launch epoch (30 bits, plus a poison
//                    bit and a "not a descriptor" bit) in the high half; 2 status bits (1 = the tile's own count,
//                    2 = inclusive prefix over all tiles up to it) above a 30-bit count in the
//                    low half.  A word is self-validating: no fence separates "data" from
//                    "flag", and a word of an earlier launch is simply not there yet, so
//                    nothing clears the table between launches.  A tile publishes its counts,
//                    then reads the words of its predecessors, a window of rows at a time, all
//                    (row, counter) pairs in parallel, and stops per counter at the nearest row
//                    that already holds an inclusive prefix.
// Tiles are numbered by an atomic ticket, so a tile only ever waits for tiles that are
// already running, and it only waits for their own counts, never for their prefixes: the
// look-back is one round of parallel loads, not a serial chain.  Descriptor words are read
// and written with agent-scope atomics (the eight XCDs of the chip have private L2 caches).
//
// The workspace carries its state from launch to launch (ticket and epoch, one 64-bit word): it is set up once
// (scan_ws_init_kernel), every launch leaves it ready for the next (the tile with the last ticket, which knows
// that every tile has drawn ticket and epoch, resets the one and moves the other on), and a launch that finds no
// set-up workspace flags it, marks its outputs and touches nothing else.  Every wait is bounded; a tile whose
// wait gives up sets the workspace's sticky error word and poisons what it publishes, every tile that builds on
// a poisoned word is poisoned too, and poisoned tiles write -1 for their tokens: a consumer sees the failure
// in the outputs, without a synchronisation, and what carries no mark is right.
//
// Replaces the per-expert serial Blelloch scan of the reference
// (src/op/dialect/cuda/kernels/tutel_moe_dispatch.cu:164-212: grid = E blocks, each
// re-reading all S indices, 20 barriers per 1024 tokens).
#pragma once
#include "common.hpp"

namespace lancet {

// Header words of the workspace (uint32), followed by the descriptor table (uint64).
enum : uint32_t {
  kWsTicket = 0,  // next tile number, 0 between launches; with kWsEpoch ONE 64-bit word, so that a tile gets
  kWsEpoch = 1,   // both with one atomic add: the tag of the running launch's descriptor words (1 .. 2^30-1)
  kWsError = 2,   // sticky: a bounded wait gave up, or a launch found the workspace not set up
  kWsDone = 3,    // finished tiles; counted only in the launch whose epoch is the last before the wrap
  kWsSpin = 4,    // polls a tile waits for a predecessor's word before it gives up (0: the default)
  kWsMagic = 5,   // kWsMagicValue once the workspace is set up (with kWsSpin one 8-byte load)
  kWsExtent = 6,  // largest number of descriptor words a launch has used
  kWsFailed = 7,  // a tile of the running launch found the workspace unusable (bad ticket or epoch) and published
                  // nothing: read by the kernel that finishes a top-2 launch from the totals row, which would
                  // otherwise take the row an earlier launch left there; cleared by the launch sequence behind it
  kScanHeaderWords = 8
};
constexpr uint32_t kWsMagicValue = 0x4c53434eu;  // "LSCN"
constexpr uint32_t kDefaultScanSpin = 1u << 22;  // ~ seconds of polling; a healthy wait is microseconds

struct ScanWs {
  uint32_t* hdr;   // [kScanHeaderWords]
  uint64_t* desc;  // [T][NC] descriptor words
};

constexpr uint32_t kDescCountMask = 0x3fffffffu;
constexpr uint32_t kDescAggregate = 1u << 30;
constexpr uint32_t kDescInclusive = 2u << 30;
constexpr uint32_t kDescPoison = 0x80000000u;   // in the high (epoch) half
// Also in the high half: the word is no descriptor.  Callers that keep other data in a scan workspace (the
// batch-prioritised routing does) store it as 64-bit words with this bit set, so that whatever a later launch
// finds where it expects a descriptor is either a descriptor, tagged with its launch's epoch, or a word that
// no epoch matches: launches of any shapes and kinds can share one workspace.
constexpr uint32_t kDescForeign = 0x40000000u;
constexpr uint32_t kEpochMask = 0x3fffffffu;

__host__ __device__ inline uint64_t foreign_word(uint32_t tag_bits, uint32_t low) {
  return (static_cast<uint64_t>(kDescForeign | (tag_bits & kEpochMask)) << 32) | low;
}

__host__ __device__ inline size_t scan_ws_bytes(int64_t ntiles, int64_t ncounters) {
  return kScanHeaderWords * sizeof(uint32_t) + static_cast<size_t>(ntiles) * static_cast<size_t>(ncounters) * sizeof(uint64_t);
}

inline ScanWs scan_ws_view(void* base) {
  ScanWs ws;
  ws.hdr = static_cast<uint32_t*>(base);
  ws.desc = reinterpret_cast<uint64_t*>(ws.hdr + kScanHeaderWords);
  return ws;
}

__device__ __forceinline__ uint64_t ld_desc(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_desc(uint64_t* p, uint32_t tag, uint32_t low) {
  __hip_atomic_store(p, (static_cast<uint64_t>(tag) << 32) | low, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool desc_is_current(uint64_t x, uint32_t epoch) {
  return (static_cast<uint32_t>(x >> 32) & ~kDescPoison) == epoch;
}
__device__ __forceinline__ bool desc_is_poisoned(uint64_t x) { return (static_cast<uint32_t>(x >> 32) & kDescPoison) != 0; }

// What a tile learns when it starts.  ok == false: the workspace is not set up (or its state is damaged); the
// caller marks the outputs of tile `tile` (= its workgroup index then) and returns without tile_scan.
struct TileStart {
  uint32_t tile, epoch, spin;
  bool ok;
};

// Must be called from uniform control flow by all kTile threads, first thing in the kernel.  Two independent
// memory round trips (the ticket fetch and the 8-byte load of spin limit and magic), issued together.
__device__ __forceinline__ TileStart tile_begin(const ScanWs& ws, int ntiles) {
  __shared__ uint32_t s_start[4];
  if (threadIdx.x == 0) {
    const uint64_t state = __hip_atomic_fetch_add(reinterpret_cast<uint64_t*>(ws.hdr + kWsTicket), 1ull,
                                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t sm = __hip_atomic_load(reinterpret_cast<const uint64_t*>(ws.hdr + kWsSpin), __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t t = static_cast<uint32_t>(state), epoch = static_cast<uint32_t>(state >> 32);
    const uint32_t spin = static_cast<uint32_t>(sm), magic = static_cast<uint32_t>(sm >> 32);
    const bool ok = magic == kWsMagicValue && t < static_cast<uint32_t>(ntiles) && epoch != 0u && (epoch & ~kEpochMask) == 0u;
    if (!ok) {
      st_agent(ws.hdr + kWsError, 1u);
      st_agent(ws.hdr + kWsFailed, 1u);
    }
    s_start[0] = ok ? t : blockIdx.x;
    s_start[1] = epoch;
    s_start[2] = spin ? spin : kDefaultScanSpin;
    s_start[3] = ok;
  }
  __syncthreads();
  TileStart r;
  r.tile = s_start[0];
  r.epoch = s_start[1];
  r.spin = s_start[2];
  r.ok = s_start[3] != 0u;
  return r;
}

// Last thing a tile that passed tile_begin does (uniform control flow, all threads).  The tile with the last
// ticket knows that every tile of the launch has its ticket and, with it, the epoch: it leaves the workspace
// ready for the next launch (ticket 0, next epoch) without waiting for anybody.  Only in the launch whose
// epoch is the last before the wrap the tiles are counted as they finish, and the one that finishes last
// first clears the table (words of 2^30 launches ago would look current again), keeping the counts of the
// totals row under a tag that is nobody's epoch for the kernel that reads them after this one.
__device__ __forceinline__ void tile_end(const ScanWs& ws, const TileStart& me, int ntiles, int ncounters) {
  const uint32_t used = static_cast<uint32_t>(ntiles) * static_cast<uint32_t>(ncounters);
  if (me.epoch != kEpochMask) {
    if (me.tile == static_cast<uint32_t>(ntiles) - 1u && threadIdx.x == 0) {
      atomicMax(ws.hdr + kWsExtent, used);
      __hip_atomic_store(reinterpret_cast<uint64_t*>(ws.hdr + kWsTicket), static_cast<uint64_t>(me.epoch + 1u) << 32,
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return;
  }
  __shared__ uint32_t s_last;
  __syncthreads();
  if (threadIdx.x == 0) s_last = atomicAdd(ws.hdr + kWsDone, 1u) == static_cast<uint32_t>(ntiles) - 1u;
  __syncthreads();
  if (!s_last) return;
  const uint32_t extent = max(ld_agent(ws.hdr + kWsExtent), used);
  const uint32_t tot_lo = used - static_cast<uint32_t>(ncounters);
  for (uint32_t i = threadIdx.x; i < extent; i += kTile) {
    uint32_t tag = 0u, low = 0u;
    if (i >= tot_lo && i < used) {
      // the last tile published these before it counted itself done, but nothing orders the two for another
      // workgroup; the words validate themselves, so wait for them (bounded)
      uint64_t x = ld_desc(ws.desc + i);
      uint32_t spins = 0;
      while (!(desc_is_current(x, me.epoch) && (static_cast<uint32_t>(x) & kDescInclusive))) {
        if (++spins > me.spin) {
          st_agent(ws.hdr + kWsError, 1u);
          x = static_cast<uint64_t>(kDescPoison) << 32;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
        x = ld_desc(ws.desc + i);
      }
      tag = static_cast<uint32_t>(x >> 32) & kDescPoison;
      low = static_cast<uint32_t>(x);
    }
    st_desc(ws.desc + i, tag, low);
  }
  if (threadIdx.x == 0) {
    st_agent(ws.hdr + kWsExtent, extent);
    st_agent(ws.hdr + kWsDone, 0u);
    __hip_atomic_store(reinterpret_cast<uint64_t*>(ws.hdr + kWsTicket), 1ull << 32, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// LDS layout used by tile_scan: (kWavesPerTile + 3) rows of NC words:
//   rows 0..3 : per-wave counts, turned into exclusive prefixes over the waves of the tile
//   row  4    : tile aggregate
//   row  5    : exclusive prefix of the tile over all earlier tiles
//   row  6    : per counter, the nearest look-back row that held an inclusive prefix
constexpr int kScanLdsRows = kWavesPerTile + 3;
__host__ __device__ inline size_t scan_lds_bytes(int ncounters) {
  return static_cast<size_t>(kScanLdsRows) * ncounters * sizeof(uint32_t);
}

// Descriptor words in flight per thread and window.  Measured at 256 tiles x 64 counters (all tiles running at
// once, the deepest look-back): 4 loads 22.7 us, 8 loads 23.2, 16 loads 25.8, 32 loads 29.4 for the routing call;
// at 16 to 64 tiles 8 is the fastest by 0.5 us.
constexpr int kLookbackLoads = 8;

// cls[j] in [0, E) is the class whose running count the token asks for in counter set j
// (negative = none); mem[j] says whether the token itself counts in that set.
// On return rank[j] = number of earlier member tokens of class cls[j] in set j (0 when
// cls[j] < 0); s_cnt row 5 holds the tile's exclusive base and row 4 its aggregate.
// Returns true when the tile is poisoned (a wait gave up here or in a tile it builds on): its ranks mean
// nothing.  Must be called from uniform control flow by all kTile threads.
// LOOKBACK = false: the first two levels only.  rank[j] is then the rank inside the tile, row 4 of s_cnt the
// tile's counts, and neither `me` nor the descriptor table is touched: the caller stores the counts
// (store_tile_counts) and a second kernel adds what the earlier tiles counted (sum_tile_counts).
template <int NSETS, bool LOOKBACK = true>
__device__ __forceinline__ bool tile_scan(const int (&cls)[NSETS], const bool (&mem)[NSETS], int E,
                                          const TileStart& me, const ScanWs& ws, uint32_t* s_cnt,
                                          uint32_t (&rank)[NSETS]) {
  __shared__ int s_open;    // counters whose look-back has not reached an inclusive prefix yet
  __shared__ int s_poison;  // this tile's prefix cannot be trusted
  const int tid = threadIdx.x;
  const int w = tid / kWave;
  const int NC = NSETS * E;
  const uint32_t tile = me.tile;
  uint32_t* s_agg = s_cnt + kWavesPerTile * NC;
  uint32_t* s_base = s_agg + NC;
  uint32_t* s_stop = s_base + NC;

  for (int c = tid; c < kScanLdsRows * NC; c += kTile) s_cnt[c] = 0;
  if (tid == 0) s_poison = 0;
  __syncthreads();

  // 1. wave level
  const int nbits = (E > 1) ? (32 - __clz(E - 1)) : 0;
  uint32_t wrank[NSETS];
#pragma unroll
  for (int j = 0; j < NSETS; ++j) {
    const bool has = cls[j] >= 0;
    uint64_t peers = __ballot(has);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = has && ((cls[j] >> b) & 1);
      const uint64_t bal = __ballot(bit);
      peers &= bit ? bal : ~bal;
    }
    const uint64_t members = peers & __ballot(has && mem[j]);
    wrank[j] = popc_below(members);
    if (has && popc_below(peers) == 0) s_cnt[w * NC + j * E + cls[j]] = __popcll(members);
  }
  __syncthreads();

  // 2. tile level: exclusive scan over the waves, publish the tile's counts
  for (int c = tid; c < NC; c += kTile) {
    uint32_t run = 0;
#pragma unroll
    for (int k = 0; k < kWavesPerTile; ++k) {
      const uint32_t t = s_cnt[k * NC + c];
      s_cnt[k * NC + c] = run;
      run += t;
    }
    s_agg[c] = run;
    if (LOOKBACK)
      st_desc(ws.desc + static_cast<size_t>(tile) * NC + c, me.epoch, (tile == 0 ? kDescInclusive : kDescAggregate) | run);
  }

  // 3. decoupled look-back
  if (LOOKBACK && tile > 0) {
    if (tid == 0) s_open = NC;
    for (int c = tid; c < NC; c += kTile) s_stop[c] = 0xffffffffu;
    __syncthreads();
    int newest = static_cast<int>(tile) - 1;  // newest row not looked at yet
    const int win_rows = max(1, (kTile * kLookbackLoads) / NC);  // rows examined per window
    // pair k of this thread is (row newest - lrow[k], counter lcol[k]), the same in every window: the one
    // division by the run-time NC is done here and the pairs follow by addition
    int lrow[kLookbackLoads], lcol[kLookbackLoads];
    {
      const int dl = kTile / NC, dc = kTile - dl * NC;
      int l = tid / NC, c = tid - l * NC;
#pragma unroll
      for (int k = 0; k < kLookbackLoads; ++k) {
        lrow[k] = l;
        lcol[k] = c;
        l += dl;
        c += dc;
        if (c >= NC) {
          c -= NC;
          l += 1;
        }
      }
    }
    while (true) {
      const int nrows = min(win_rows, newest + 1);
      uint64_t word[kLookbackLoads];
      // issue all loads of the window, then wait for the ones that are not published yet
#pragma unroll
      for (int k = 0; k < kLookbackLoads; ++k) {
        word[k] = 0;
        if (lrow[k] < nrows) word[k] = ld_desc(ws.desc + static_cast<size_t>(newest - lrow[k]) * NC + lcol[k]);
      }
#pragma unroll
      for (int k = 0; k < kLookbackLoads; ++k) {
        if (lrow[k] < nrows && !desc_is_current(word[k], me.epoch)) {
          const uint64_t* ptr = ws.desc + static_cast<size_t>(newest - lrow[k]) * NC + lcol[k];
          uint32_t spins = 0;
          do {
            if (++spins > me.spin) {  // bounded wait: flag the workspace, poison the tile
              st_agent(ws.hdr + kWsError, 1u);
              word[k] = (static_cast<uint64_t>(me.epoch | kDescPoison) << 32) | kDescInclusive;
              break;
            }
            __builtin_amdgcn_s_sleep(1);
            word[k] = ld_desc(ptr);
          } while (!desc_is_current(word[k], me.epoch));
        }
        if (lrow[k] < nrows && (static_cast<uint32_t>(word[k]) & kDescInclusive))
          atomicMin(&s_stop[lcol[k]], static_cast<uint32_t>(static_cast<int>(tile) - 1 - (newest - lrow[k])));
      }
      __syncthreads();
      // add what counts: rows newer than the counter's stop row, and the stop row itself
#pragma unroll
      for (int k = 0; k < kLookbackLoads; ++k) {
        if (lrow[k] < nrows) {
          const int c = lcol[k];
          const uint32_t depth = static_cast<uint32_t>(static_cast<int>(tile) - 1 - (newest - lrow[k]));
          const uint32_t stop = s_stop[c];
          if (depth <= stop) {
            const uint32_t v = static_cast<uint32_t>(word[k]) & kDescCountMask;
            if (v) atomicAdd(&s_base[c], v);
            if (desc_is_poisoned(word[k])) s_poison = 1;
            if (depth == stop) atomicSub(&s_open, 1);
          }
        }
      }
      __syncthreads();
      if (s_open <= 0 || newest - nrows < 0) break;
      newest -= nrows;
      __syncthreads();
    }
    const uint32_t tag = me.epoch | (s_poison ? kDescPoison : 0u);
    for (int c = tid; c < NC; c += kTile)
      st_desc(ws.desc + static_cast<size_t>(tile) * NC + c, tag, kDescInclusive | ((s_base[c] + s_agg[c]) & kDescCountMask));
  }
  __syncthreads();

#pragma unroll
  for (int j = 0; j < NSETS; ++j) {
    const int c = j * E + (cls[j] >= 0 ? cls[j] : 0);
    rank[j] = (cls[j] >= 0) ? s_base[c] + s_cnt[w * NC + c] + wrank[j] : 0u;
  }
  return s_poison != 0;
}

// ---- two or three kernels instead of a look-back -----------------------------------------------------------
// When the tiles of a launch all run at once no inclusive prefix exists until the first tiles finish, and the
// look-back degenerates into a chain of memory round trips from tile to tile (8 of the 21 us of a 256-tile
// launch, 70 us at 1024 tiles, 430 us at 8192).  Except for one counter set on at most 32 tiles (one short
// kernel) the scan is therefore cut into kernels that wait for nothing: the first stores every tile's counts,
// the last lets every tile add up the counts of the tiles before it (and of all tiles: the totals) with plain
// loads, eight in flight per thread.  A tile's counts are stored two to a 64-bit word, the high half tagged "not
// a descriptor", so that the workspace keeps its property that no word of it can pass for a descriptor of a
// later look-back launch.
// Adding up ALL rows in every tile costs T * NC words per tile, quadratic in the tile count T: beyond
// T * NC = 32768 a kernel between the two adds the rows up in segments of R consecutive tiles (R about the
// square root of T), and a tile then reads the sums of the segments before its own and the rows of its own
// segment before itself: about 2 * sqrt(T) rows instead of T.  Three launches, still no waits and no state.
// Routing of S tokens x E experts (us; two kernels / three kernels / look-back): 65536 x 32 top-2 12.7 / 15.7 / 24;
// 131072 x 32 top-2 19 / 21 / 38; 262144 x 32 top-2 42 / 33 / 69; 1048576 x 16 top-1 88 / 39 / 208;
// 2097152 x 16 top-1 275 / 68 / 432.
enum ScanForm { kScanLookback = 0, kScanCountPlace = 1, kScanCountSegPlace = 2 };
constexpr int64_t kFlatPlaceMaxWork = 32768;  // tiles x counters up to which the extra launch costs more than it saves
__host__ inline ScanForm scan_form(int64_t ntiles, int64_t ncounters, int nsets, bool force_lookback = false) {
  if (force_lookback) return kScanLookback;
  // one counter set and few tiles: the look-back is a single short kernel
  if (nsets == 1 && ntiles <= 32) return kScanLookback;
  return ntiles * ncounters <= kFlatPlaceMaxWork ? kScanCountPlace : kScanCountSegPlace;
}
// rows per segment: the smallest power of two from 32 on whose square covers the tiles
__host__ __device__ inline int seg_rows(int64_t ntiles) {
  int r = 32;
  while (static_cast<int64_t>(r) * r < ntiles && r < (1 << 15)) r <<= 1;
  return r;
}

__host__ __device__ inline int count_pairs(int ncounters) { return (ncounters + 1) / 2; }

// after tile_scan<NSETS, false>: row 4 of s_cnt -> the tile's row of the table
__device__ __forceinline__ void store_tile_counts(const ScanWs& ws, uint32_t tile, int NC, const uint32_t* s_cnt) {
  const uint32_t* s_agg = s_cnt + kWavesPerTile * NC;
  const int PP = count_pairs(NC);
  for (int q = threadIdx.x; q < PP; q += kTile) {
    const uint32_t lo = s_agg[2 * q], hi = (2 * q + 1 < NC) ? s_agg[2 * q + 1] : 0u;
    ws.desc[static_cast<size_t>(tile) * PP + q] = foreign_word(hi, lo);
  }
}

// Adds up nrows rows of a table of counts (count_pairs(NC) words per row): s_total[c] += all of them (TOTAL),
// s_before[c] += the rows below `cut`.  The caller has zeroed (or pre-loaded) both arrays and synchronised; on
// return the sums are complete and visible.  Uniform control flow, all kTile threads; the table was written by an
// earlier kernel.
template <bool TOTAL>
__device__ __forceinline__ void sum_count_rows(const uint64_t* table, int nrows, int cut, int NC, uint32_t* s_before,
                                               uint32_t* s_total) {
  const int PP = count_pairs(NC);
  const int n = nrows * PP;
  const int dl = kTile / PP, dc = kTile - dl * PP;
  int row = static_cast<int>(threadIdx.x) / PP, q = static_cast<int>(threadIdx.x) - row * PP;
  if (PP > kTile && PP % kTile == 0 && PP / kTile <= 2) {
    // two pairs per thread and row (more than 256 pairs: several hundred experts)
    uint32_t tl[2] = {0, 0}, th[2] = {0, 0}, bl[2] = {0, 0}, bh[2] = {0, 0};
    constexpr int kRows = 4;  // rows in flight per thread
    for (int r = 0; r < nrows; r += kRows) {
      uint64_t w[kRows][2];
#pragma unroll
      for (int k = 0; k < kRows; ++k)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          w[k][j] = (r + k < nrows) ? table[static_cast<size_t>(r + k) * PP + threadIdx.x + j * kTile] : 0ull;
#pragma unroll
      for (int k = 0; k < kRows; ++k)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const uint32_t lo = static_cast<uint32_t>(w[k][j]), hi = static_cast<uint32_t>(w[k][j] >> 32) & kEpochMask;
          tl[j] += lo, th[j] += hi;
          if (r + k < cut) bl[j] += lo, bh[j] += hi;
        }
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int c = 2 * (static_cast<int>(threadIdx.x) + j * kTile);  // this thread alone owns the pair
      if (TOTAL) s_total[c] += tl[j];
      s_before[c] += bl[j];
      if (c + 1 < NC) {
        if (TOTAL) s_total[c + 1] += th[j];
        s_before[c + 1] += bh[j];
      }
    }
    __syncthreads();
    return;
  }
  if (dc == 0) {
    // the pairs of a row divide the workgroup: a thread meets the same pair in every row it reads, adds up in
    // registers and goes to LDS once
    uint32_t tl = 0, th = 0, bl = 0, bh = 0;
    constexpr int kBatch = 8;  // loads in flight per thread (one at a time would be a chain of round trips)
    int i = threadIdx.x;
    for (; i + (kBatch - 1) * kTile < n; i += kBatch * kTile) {
      uint64_t w[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) w[k] = table[i + k * kTile];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const uint32_t lo = static_cast<uint32_t>(w[k]), hi = static_cast<uint32_t>(w[k] >> 32) & kEpochMask;
        tl += lo, th += hi;
        if (row + k * dl < cut) bl += lo, bh += hi;
      }
      row += kBatch * dl;
    }
    for (; i < n; i += kTile) {
      const uint64_t w = table[i];
      const uint32_t lo = static_cast<uint32_t>(w), hi = static_cast<uint32_t>(w >> 32) & kEpochMask;
      tl += lo, th += hi;
      if (row < cut) bl += lo, bh += hi;
      row += dl;
    }
    if (TOTAL && tl) atomicAdd(&s_total[2 * q], tl);
    if (TOTAL && th) atomicAdd(&s_total[2 * q + 1], th);
    if (bl) atomicAdd(&s_before[2 * q], bl);
    if (bh) atomicAdd(&s_before[2 * q + 1], bh);
    __syncthreads();
    return;
  }
  for (int i = threadIdx.x; i < n; i += kTile) {
    const uint64_t w = table[i];
    const uint32_t lo = static_cast<uint32_t>(w), hi = static_cast<uint32_t>(w >> 32) & kEpochMask;
    if (lo) {
      if (TOTAL) atomicAdd(&s_total[2 * q], lo);
      if (row < cut) atomicAdd(&s_before[2 * q], lo);
    }
    if (hi) {
      if (TOTAL) atomicAdd(&s_total[2 * q + 1], hi);
      if (row < cut) atomicAdd(&s_before[2 * q + 1], hi);
    }
    row += dl, q += dc;
    if (q >= PP) q -= PP, row += 1;
  }
  __syncthreads();
}

// the table of segment sums lies behind the tiles' rows (the look-back form's table has room for both)
__device__ __forceinline__ uint64_t* seg_table(const ScanWs& ws, int ntiles, int NC) {
  return ws.desc + static_cast<size_t>(ntiles) * count_pairs(NC);
}

// s_before[c] = counts of tiles [0, tile), s_total[c] = counts of all ntiles tiles (LDS, NC words each).
// R = 0: every row is read; R > 0: the sums of segments of R tiles (tile_segsum) are there.
__device__ __forceinline__ void sum_tile_counts(const ScanWs& ws, uint32_t tile, int ntiles, int NC, int R,
                                                uint32_t* s_before, uint32_t* s_total) {
  for (int c = threadIdx.x; c < NC; c += kTile) s_before[c] = s_total[c] = 0u;
  __syncthreads();
  if (R <= 0) {
    sum_count_rows<true>(ws.desc, ntiles, static_cast<int>(tile), NC, s_before, s_total);
    return;
  }
  const int seg = static_cast<int>(tile) / R, nseg = (ntiles + R - 1) / R;
  sum_count_rows<true>(seg_table(ws, ntiles, NC), nseg, seg, NC, s_before, s_total);
  const int first = seg * R;
  sum_count_rows<false>(ws.desc + static_cast<size_t>(first) * count_pairs(NC), min(R, ntiles - first),
                        static_cast<int>(tile) - first, NC, s_before, s_total);
}

// the segment's sums (LDS s_sum[NC], all kTile threads) -> its row of the segment table
__device__ __forceinline__ void tile_segsum(const ScanWs& ws, int seg, int ntiles, int NC, int R, uint32_t* s_sum) {
  for (int c = threadIdx.x; c < NC; c += kTile) s_sum[c] = 0u;
  __syncthreads();
  const int first = seg * R;
  const int PP = count_pairs(NC);
  sum_count_rows<true>(ws.desc + static_cast<size_t>(first) * PP, min(R, ntiles - first), 0, NC, s_sum, s_sum);
  uint64_t* out = seg_table(ws, ntiles, NC) + static_cast<size_t>(seg) * PP;
  for (int q = threadIdx.x; q < PP; q += kTile) {
    const uint32_t lo = s_sum[2 * q], hi = (2 * q + 1 < NC) ? s_sum[2 * q + 1] : 0u;
    out[q] = foreign_word(hi, lo);
  }
}

}  // namespace lancet
