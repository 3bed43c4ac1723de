// Capacity-bounded position scan: for every token, the number of earlier tokens (in token
// order) that chose the same expert.  One pass over token tiles:
//   1. wave level  - match lanes with the same expert by ballots over the bits of the expert
//                    id; rank inside the wave = popcount of the peer mask below the lane;
//   2. tile level  - per-wave counts in LDS, exclusive scan over the waves of the tile;
//   3. across tiles - decoupled look-back over a [tiles][counters] descriptor table.  Every
//                    descriptor is ONE 32-bit word: 2 status bits (1 = the tile's own count,
//                    2 = inclusive prefix over all tiles up to it) above a 30-bit count, so a
//                    word is self-validating and no fence separates "data" from "flag".  A
//                    tile publishes its counts, then reads the words of its predecessors, a
//                    window of rows at a time, all (row, counter) pairs in parallel, and stops
//                    per counter at the nearest row that already holds an inclusive prefix.
// Tiles are numbered by an atomic ticket, so a tile only ever waits for tiles that are
// already running, and it only waits for their own counts, never for their prefixes: the
// look-back is one round of parallel loads, not a serial chain.  Descriptor words are read
// and written with agent-scope atomics (the eight XCDs of the chip have private L2 caches).
//
// Replaces the per-expert serial Blelloch scan of the reference
// (src/op/dialect/cuda/kernels/tutel_moe_dispatch.cu:164-212: grid = E blocks, each
// re-reading all S indices, 20 barriers per 1024 tokens).
#pragma once
#include "common.hpp"

namespace lancet {

// Views into the caller's workspace (all uint32 words).
struct ScanWs {
  uint32_t* ticket;  // [1]  next tile number
  uint32_t* error;   // [1]  set to 1 when a bounded wait gave up
  uint32_t* desc;    // [T][NC] descriptor words, zero before the launch
};

constexpr uint32_t kScanHeaderWords = 2;  // ticket, error
constexpr uint32_t kDescCountMask = 0x3fffffffu;
constexpr uint32_t kDescAggregate = 1u << 30;
constexpr uint32_t kDescInclusive = 2u << 30;

// words that must be zero when the kernel starts
__host__ __device__ inline size_t scan_ws_words(int64_t ntiles, int64_t ncounters) {
  return kScanHeaderWords + static_cast<size_t>(ntiles) * static_cast<size_t>(ncounters);
}

inline ScanWs scan_ws_view(void* base) {
  uint32_t* w = static_cast<uint32_t*>(base);
  ScanWs ws;
  ws.ticket = w;
  ws.error = w + 1;
  ws.desc = w + kScanHeaderWords;
  return ws;
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

constexpr int kLookbackLoads = 8;  // descriptor words in flight per thread and window

// cls[j] in [0, E) is the class whose running count the token asks for in counter set j
// (negative = none); mem[j] says whether the token itself counts in that set.
// On return rank[j] = number of earlier member tokens of class cls[j] in set j (0 when
// cls[j] < 0); s_cnt row 5 holds the tile's exclusive base and row 4 its aggregate.
// Must be called from uniform control flow by all kTile threads.
template <int NSETS>
__device__ __forceinline__ void tile_scan(const int (&cls)[NSETS], const bool (&mem)[NSETS], int E,
                                          uint32_t tile, const ScanWs& ws, uint32_t* s_cnt,
                                          uint32_t spin_limit, uint32_t (&rank)[NSETS]) {
  __shared__ int s_open;  // counters whose look-back has not reached an inclusive prefix yet
  const int tid = threadIdx.x;
  const int w = tid / kWave;
  const int NC = NSETS * E;
  uint32_t* s_agg = s_cnt + kWavesPerTile * NC;
  uint32_t* s_base = s_agg + NC;
  uint32_t* s_stop = s_base + NC;

  for (int c = tid; c < kScanLdsRows * NC; c += kTile) s_cnt[c] = 0;
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
    st_agent(ws.desc + static_cast<size_t>(tile) * NC + c, (tile == 0 ? kDescInclusive : kDescAggregate) | run);
  }

  // 3. decoupled look-back
  if (tile > 0) {
    if (tid == 0) s_open = NC;
    for (int c = tid; c < NC; c += kTile) s_stop[c] = 0xffffffffu;
    __syncthreads();
    const int win_rows = max(1, (kTile * kLookbackLoads) / NC);  // rows examined per window
    int newest = static_cast<int>(tile) - 1;                      // newest row of the window
    while (true) {
      const int nrows = min(win_rows, newest + 1);
      const int npairs = nrows * NC;
      uint32_t word[kLookbackLoads];
      // issue all loads of the window, then wait for the ones that are not published yet
#pragma unroll
      for (int k = 0; k < kLookbackLoads; ++k) {
        const int i = tid + k * kTile;
        word[k] = kDescAggregate;
        if (i < npairs) {
          const int l = i / NC;
          word[k] = ld_agent(ws.desc + static_cast<size_t>(newest - l) * NC + (i - l * NC));
        }
      }
#pragma unroll
      for (int k = 0; k < kLookbackLoads; ++k) {
        const int i = tid + k * kTile;
        if (i < npairs && word[k] == 0) {
          const int l = i / NC;
          const uint32_t* ptr = ws.desc + static_cast<size_t>(newest - l) * NC + (i - l * NC);
          uint32_t spins = 0;
          do {
            if (++spins > spin_limit) {  // bounded wait: flag the workspace, carry on
              st_agent(ws.error, 1u);
              word[k] = kDescAggregate;
              break;
            }
            __builtin_amdgcn_s_sleep(1);
            word[k] = ld_agent(ptr);
          } while (word[k] == 0);
        }
        if (i < npairs && (word[k] & kDescInclusive)) {
          const int l = i / NC;
          atomicMin(&s_stop[i - l * NC], static_cast<uint32_t>(static_cast<int>(tile) - 1 - (newest - l)));
        }
      }
      __syncthreads();
      // add what counts: rows newer than the counter's stop row, and the stop row itself
#pragma unroll
      for (int k = 0; k < kLookbackLoads; ++k) {
        const int i = tid + k * kTile;
        if (i < npairs) {
          const int l = i / NC;
          const int c = i - l * NC;
          const uint32_t depth = static_cast<uint32_t>(static_cast<int>(tile) - 1 - (newest - l));
          const uint32_t stop = s_stop[c];
          if (depth <= stop) {
            const uint32_t v = word[k] & kDescCountMask;
            if (v) atomicAdd(&s_base[c], v);
            if (depth == stop) atomicSub(&s_open, 1);
          }
        }
      }
      __syncthreads();
      if (s_open <= 0 || newest - nrows < 0) break;
      newest -= nrows;
      __syncthreads();
    }
    for (int c = tid; c < NC; c += kTile)
      st_agent(ws.desc + static_cast<size_t>(tile) * NC + c, kDescInclusive | ((s_base[c] + s_agg[c]) & kDescCountMask));
  }
  __syncthreads();

#pragma unroll
  for (int j = 0; j < NSETS; ++j) {
    const int c = j * E + (cls[j] >= 0 ? cls[j] : 0);
    rank[j] = (cls[j] >= 0) ? s_base[c] + s_cnt[w * NC + c] + wrank[j] : 0u;
  }
}

}  // namespace lancet
