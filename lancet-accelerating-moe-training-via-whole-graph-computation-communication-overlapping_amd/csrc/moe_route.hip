// Routing kernels: gate softmax + top-1/top-2 selection (select.hpp) fused with the capacity-bounded
// position scan (scan.hpp) in its three forms, and the top-2 finalisation.
#include "launchers.hpp"
#include "select.hpp"
#include <algorithm>

namespace lancet {

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
  // no totals and every token is marked, else the tokens of poisoned tiles carry marks of their own.  A tile
  // that could not take part (its ticket or epoch was out of range: the workspace's state is damaged, e.g. by a
  // call that overlapped this one) has published nothing, and the row may be what an earlier launch left: no
  // totals either.
  const uint64_t* tot = a.ws.desc + static_cast<size_t>(a.ntiles - 1) * 2 * a.E;
  const bool poisoned = ld_agent(a.ws.hdr + kWsFailed) != 0u || desc_is_poisoned(ld_desc(tot));
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

// One-time set-up of a workspace of nwords 32-bit words (a later launch may use any part of it).
__global__ void scan_ws_init_kernel(uint32_t* ws, size_t nwords) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < nwords;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    uint32_t v = 0u;
    if (i == kWsEpoch) v = 1u;
    if (i == kWsMagic) v = kWsMagicValue;
    ws[i] = v;
  }
}

__global__ void fill_u32_kernel(uint32_t* p, size_t n, uint32_t v) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x)
    p[i] = v;
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
int64_t scan_num_tiles(int64_t S) { return S > 0 ? (S + kTile - 1) / kTile : 1; }


size_t scan_workspace_bytes(int64_t S, int64_t E, int nsets) {
  // (two words per tile at least: the forms without look-back keep the tiles' counts, two to a word, and the
  // segments' sums in the room of the look-back's table)
  return scan_ws_bytes(scan_num_tiles(S), std::max<int64_t>(nsets * E, 2));
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

hipError_t run_scan_segsum(void* ws, int ntiles, int NC, int R, hipStream_t st) {
  scan_segsum_kernel<<<(ntiles + R - 1) / R, kTile, NC * sizeof(uint32_t), st>>>(scan_ws_view(ws), ntiles, NC, R);
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
      err = run_scan_segsum(ws, a.ntiles, NC, a.seg_rows, st);
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
    err = hipGetLastError();
    if (err != hipSuccess) return err;
    return run_fill_u32(a.ws.hdr + kWsFailed, 1, 0u, st);  // read by the kernel before; the next launch starts clear
  }
  return hipGetLastError();
}


hipError_t run_top2_normalize(const void* raw, const int32_t* idx, int S, int gate_dtype, void* out, hipStream_t st) {
  if (S == 0) return hipSuccess;
  top2_normalize_kernel<<<(S + 255) / 256, 256, 0, st>>>(raw, idx, S, out, gate_dtype);
  return hipGetLastError();
}

}  // namespace lancet
