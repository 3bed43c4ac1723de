// Capacity-bounded position scan: for every token, the number of earlier tokens (in token
// order) that chose the same expert.  One pass over token tiles:
//   1. wave level  - match lanes with the same expert by ballots over the bits of the expert
//                    id; rank inside the wave = popcount of the peer mask below the lane;
//   2. tile level  - per-wave counts in LDS, exclusive scan over the waves of the tile;
//   3. across tiles - decoupled look-back over a [tiles][counters] descriptor table: a tile
//                    publishes its aggregate, then sums the aggregates of its predecessors
//                    (in parallel over predecessors and counters) back to the nearest tile
//                    that has already published an inclusive prefix.
// Tiles are numbered by an atomic ticket, so a tile only ever waits for tiles that are
// already running.  All cross-workgroup traffic uses agent-scope atomics and fences: the
// eight XCDs of the chip have private L2 caches.
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
  uint32_t* status;  // [T]  0 = nothing, 1 = aggregate published, 2 = inclusive prefix published
  uint32_t* agg;     // [T][NC] per-tile counts
  uint32_t* incl;    // [T][NC] inclusive prefix over tiles
};

constexpr uint32_t kScanHeaderWords = 2;  // ticket, error (zeroed together with status)

__host__ __device__ inline size_t scan_ws_words(int64_t ntiles, int64_t ncounters) {
  return kScanHeaderWords + static_cast<size_t>(ntiles) * (1 + 2 * static_cast<size_t>(ncounters));
}

inline ScanWs scan_ws_view(void* base, int64_t ntiles, int64_t ncounters) {
  uint32_t* w = static_cast<uint32_t*>(base);
  ScanWs ws;
  ws.ticket = w;
  ws.error = w + 1;
  ws.status = w + kScanHeaderWords;
  ws.agg = ws.status + ntiles;
  ws.incl = ws.agg + ntiles * ncounters;
  return ws;
}

// LDS layout used by tile_scan: (kWavesPerTile + 2) rows of NC words:
//   rows 0..3 : per-wave counts, turned into exclusive prefixes over the waves of the tile
//   row  4    : tile aggregate
//   row  5    : exclusive prefix of the tile over all earlier tiles
__host__ __device__ inline size_t scan_lds_bytes(int ncounters) {
  return static_cast<size_t>(kWavesPerTile + 2) * ncounters * sizeof(uint32_t);
}

// cls[j] in [0, E) is the class whose running count the token asks for in counter set j
// (negative = none); mem[j] says whether the token itself counts in that set.
// On return rank[j] = number of earlier member tokens of class cls[j] in set j (0 when
// cls[j] < 0); s_cnt row 5 holds the tile's exclusive base and row 4 its aggregate.
// Must be called from uniform control flow by all kTile threads.
template <int NSETS>
__device__ __forceinline__ void tile_scan(const int (&cls)[NSETS], const bool (&mem)[NSETS], int E,
                                          uint32_t tile, const ScanWs& ws, uint32_t* s_cnt,
                                          uint32_t spin_limit, uint32_t (&rank)[NSETS]) {
  __shared__ int s_nearest;
  const int tid = threadIdx.x;
  const int w = tid / kWave;
  const int NC = NSETS * E;
  uint32_t* s_agg = s_cnt + kWavesPerTile * NC;
  uint32_t* s_base = s_agg + NC;

  for (int c = tid; c < (kWavesPerTile + 2) * NC; c += kTile) s_cnt[c] = 0;
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

  // 2. tile level: exclusive scan over the waves, publish the aggregate
  for (int c = tid; c < NC; c += kTile) {
    uint32_t run = 0;
#pragma unroll
    for (int k = 0; k < kWavesPerTile; ++k) {
      const uint32_t t = s_cnt[k * NC + c];
      s_cnt[k * NC + c] = run;
      run += t;
    }
    s_agg[c] = run;
    st_agent(ws.agg + static_cast<size_t>(tile) * NC + c, run);
    if (tile == 0) st_agent(ws.incl + c, run);
  }
  __threadfence();
  __syncthreads();
  if (tid == 0) st_release_agent(ws.status + tile, tile == 0 ? 2u : 1u);

  // 3. decoupled look-back
  if (tile > 0) {
    int newest = static_cast<int>(tile) - 1;  // newest predecessor not yet accounted for
    while (true) {
      const int nwin = min(kTile, newest + 1);
      if (tid == 0) s_nearest = nwin;
      __syncthreads();
      if (tid < nwin) {
        const uint32_t* st_ptr = ws.status + (newest - tid);
        uint32_t st = ld_acquire_agent(st_ptr);
        uint32_t spins = 0;
        while (st == 0) {
          if (++spins > spin_limit) {  // bounded wait: flag and carry on with what is there
            st_agent(ws.error, 1u);
            st = 1;
            break;
          }
          __builtin_amdgcn_s_sleep(2);
          st = ld_acquire_agent(st_ptr);
        }
        if (st == 2) atomicMin(&s_nearest, tid);
      }
      __syncthreads();
      __threadfence();
      const int nearest = s_nearest;
      const bool found = nearest < nwin;
      const int nrows = found ? nearest + 1 : nwin;
      for (int i = tid; i < nrows * NC; i += kTile) {
        const int l = i / NC;
        const int c = i - l * NC;
        const size_t off = static_cast<size_t>(newest - l) * NC + c;
        const uint32_t v = (found && l == nearest) ? ld_agent(ws.incl + off) : ld_agent(ws.agg + off);
        if (v) atomicAdd(&s_base[c], v);
      }
      __syncthreads();
      if (found || newest - nwin < 0) break;
      newest -= nwin;
    }
    for (int c = tid; c < NC; c += kTile)
      st_agent(ws.incl + static_cast<size_t>(tile) * NC + c, s_base[c] + s_agg[c]);
    __threadfence();
    __syncthreads();
    if (tid == 0) st_release_agent(ws.status + tile, 2u);
  }

#pragma unroll
  for (int j = 0; j < NSETS; ++j) {
    const int c = j * E + (cls[j] >= 0 ? cls[j] : 0);
    rank[j] = (cls[j] >= 0) ? s_base[c] + s_cnt[w * NC + c] + wrank[j] : 0u;
  }
}

}  // namespace lancet
