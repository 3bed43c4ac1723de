// Row movers: scatter of token rows into the [E,C,M] expert buffer, weighted gather-combine
// back, partition merge of masks and buffers.  All are pure HBM streaming: one wave per row,
// 16-byte accesses, streaming (non-temporal) loads and stores, every output byte written once.
#include "launchers.hpp"
#include "common.hpp"
#include "../../include/lancet_hip.h"
#include <algorithm>

namespace lancet {

constexpr int kRowsPerBlock = kTile / kWave;  // waves per workgroup; a wave moves a row or a share of one
constexpr int kTailRows = 16;                 // rows zero-filled by one tail workgroup

// Access granule: 16 bytes when the row size and the pointers allow, else one element.
template <typename V>
__device__ __forceinline__ V ldv(const V* p) { return __builtin_nontemporal_load(p); }
template <typename V>
__device__ __forceinline__ void stv(V* p, V v) { __builtin_nontemporal_store(v, p); }
template <typename V>
__device__ __forceinline__ void stv(LANCET_GLOBAL V* p, V v) { __builtin_nontemporal_store(v, p); }
template <typename V>
__device__ __forceinline__ V zero_v() { return V(0); }
template <>
__device__ __forceinline__ u32x4 zero_v<u32x4>() { return u32x4{0u, 0u, 0u, 0u}; }

// ---------------------------------------------------------------------------------------
// encode_forward: out[idx, loc, :] = data[s, :]; rows no token lands on are zero.
// Replaces cudaMemsetAsync + atomicAdd per element of
// src/op/dialect/cuda/kernels/tutel_moe_dispatch.cu:61-81,461-484.
// ---------------------------------------------------------------------------------------
template <typename V>
struct ScatterArgs {
  const V* data;
  V* out;
  const int32_t* idx;         // [K*S]
  const int32_t* loc;         // [K*S]
  const int32_t* dest;        // [K*S] or null: destination row e * C + location (-1: none) in ONE word per slot,
                              // instead of idx / loc / avail_used / row_base
  const int32_t* avail_used;  // [E] or null
  const int32_t* row_base;    // [E] or null: row of expert e that location 0 maps to
  const int32_t* rows_lo;     // [E] or null
  const int32_t* rows_hi;     // [E] or null (no tail fill)
  int S, E, C, K;
  int slot_stride;            // distance between the slots of one token in idx / loc (S, or the whole batch's
                              // token count when this call moves a token range of a larger mask)
  int row_vecs;               // granules per row
  int wpr_shift;              // 2^wpr_shift waves share one token row
  int token_blocks;
  int tail_chunks;            // tail workgroups per expert
};

template <typename V, int K, bool DEST = false>
__global__ __launch_bounds__(kTile) void scatter_rows_kernel(ScatterArgs<V> a) {
  const int w = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  if (static_cast<int>(blockIdx.x) < a.token_blocks) {
    // 2^wpr_shift waves share a token row, each moving every 2^wpr_shift-th run of 64 granules: short
    // waves in row order keep the chip-wide write stream close to address order, which the memory system
    // rewards (one granule per lane streams ~8 % faster than a wave walking a whole 8 KB row)
    const uint32_t gw = blockIdx.x * static_cast<uint32_t>(kRowsPerBlock) + w;  // below 2^32: the launcher sees to it
    const int s = static_cast<int>(gw >> a.wpr_shift);
    const int part = static_cast<int>(gw & ((1u << a.wpr_shift) - 1u));
    if (s >= a.S) return;
    // The row's granules do not depend on the routing, only their destinations do: the first loads of the row
    // go out before idx / loc are known, so that a wave waits for the longer of the two latencies and not for
    // their sum (a dropped token's row is then read for nothing).  338 -> 333 us at the headline shape.
    const V* src = a.data + static_cast<size_t>(s) * a.row_vecs;
    const int step = kWave << a.wpr_shift;
    int v = part * kWave + lane;
    const bool has0 = v < a.row_vecs, has1 = v + step < a.row_vecs;
    V x0 = zero_v<V>(), x1 = zero_v<V>();
    if (has0) x0 = ldv(src + v);
    if (has1) x1 = ldv(src + v + step);
    // destinations picked at run time: typed as global memory so the stores are not flat.  (The routing words of a
    // row are the same for every lane; loading them through the scalar cache, or forming the row addresses on the
    // scalar unit from vector-loaded words, was measured slower: 346 and 340 us against 333 at the headline shape.)
    LANCET_GLOBAL V* dst[K];
    int nd = 0;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      if (DEST) {
        const int d = a.dest[static_cast<size_t>(j) * a.slot_stride + s];
        dst[j] = as_global(a.out);
        if (d >= 0 && d < a.E * a.C) dst[nd++] = as_global(a.out + static_cast<size_t>(d) * a.row_vecs);
        continue;
      }
      const int e = a.idx[static_cast<size_t>(j) * a.slot_stride + s];
      int l = a.loc[static_cast<size_t>(j) * a.slot_stride + s];
      bool ok = e >= 0 && e < a.E && l >= 0 && l < a.C;
      if (ok && a.avail_used) ok = l < a.C - a.avail_used[e];
      dst[j] = as_global(a.out);
      if (ok && a.row_base) {
        l += a.row_base[e];
        ok = l < a.C;
      }
      if (ok) dst[nd++] = as_global(a.out + (static_cast<size_t>(e) * a.C + l) * a.row_vecs);
    }
    if (nd == 0) return;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      if (j < nd) {
        if (has0) stv(dst[j] + v, x0);
        if (has1) stv(dst[j] + v + step, x1);
      }
    }
    v += 2 * step;
    for (; v + step < a.row_vecs; v += 2 * step) {
      const V x0 = ldv(src + v), x1 = ldv(src + v + step);
#pragma unroll
      for (int j = 0; j < K; ++j) {
        if (j < nd) {
          stv(dst[j] + v, x0);
          stv(dst[j] + v + step, x1);
        }
      }
    }
    if (v < a.row_vecs) {
      const V x = ldv(src + v);
#pragma unroll
      for (int j = 0; j < K; ++j)
        if (j < nd) stv(dst[j] + v, x);
    }
  } else {
    // tail: zero rows [used, C) of expert e, kTailRows rows per workgroup
    const int tb = blockIdx.x - a.token_blocks;
    const int e = tb / a.tail_chunks;
    const int ch = tb - e * a.tail_chunks;
    const int used = a.rows_hi[e] - (a.rows_lo ? a.rows_lo[e] : 0);
    const int first = max(used, 0) + ch * kTailRows;
    const int last = min(first + kTailRows, a.C);
    const V z = zero_v<V>();
    for (int r = first + w; r < last; r += kRowsPerBlock) {
      V* row = a.out + (static_cast<size_t>(e) * a.C + r) * a.row_vecs;
      for (int v = lane; v < a.row_vecs; v += kWave) stv(row + v, z);
    }
  }
}

__global__ void zero_bytes_kernel(u32x4* p, size_t nvec, uint8_t* tail, size_t ntail) {
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  const u32x4 z = {0u, 0u, 0u, 0u};
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < nvec; i += stride)
    __builtin_nontemporal_store(z, p + i);
  if (blockIdx.x == 0 && threadIdx.x < ntail) tail[threadIdx.x] = 0;
}

// ---------------------------------------------------------------------------------------
// decode_forward: out[s,:] = sum_j gates[j*S+s] * expert_out[idx, loc, :], fp32 products and
// sum (no fused multiply-add, so that the result is one well-defined rounding sequence), one
// rounding to the storage type.  Replaces tutel_moe_dispatch.cu:46-55,110-116,511-521.
// ---------------------------------------------------------------------------------------
template <int DT>
struct Codec;
template <>
struct Codec<LANCET_F32> {
  typedef uint32_t S;  // scalar storage
  static constexpr int kPerVec = 4;
  static __device__ __forceinline__ float get(S x) { return __uint_as_float(x); }
  static __device__ __forceinline__ S put(float f) { return __float_as_uint(f); }
};
template <>
struct Codec<LANCET_BF16> {
  typedef uint16_t S;
  static constexpr int kPerVec = 8;
  static __device__ __forceinline__ float get(S x) { return bf16_to_f32(x); }
  static __device__ __forceinline__ S put(float f) { return static_cast<S>(f32_to_bf16(f)); }
};
template <>
struct Codec<LANCET_F16> {
  typedef uint16_t S;
  static constexpr int kPerVec = 8;
  static __device__ __forceinline__ float get(S x) { return f16_to_f32(x); }
  static __device__ __forceinline__ S put(float f) { return static_cast<S>(f32_to_f16(f)); }
};

// One IEEE multiply / add each, never contracted into a fused multiply-add (the operators of
// the HIP headers' __fmul_rn/__fadd_rn carry the translation unit's contraction setting).
__device__ __forceinline__ float mul_rn(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float add_rn(float a, float b) {
#pragma clang fp contract(off)
  return a + b;
}

template <int DT, int K>
__device__ __forceinline__ u32x4 combine_vec(const u32x4 (&x)[K], const float (&g)[K]) {
#pragma clang fp contract(off)
  typedef Codec<DT> Cd;
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (Cd::kPerVec == 4) {
      float acc = mul_rn(g[0], Cd::get(x[0][i]));
      if (K == 2) acc = add_rn(acc, mul_rn(g[1], Cd::get(x[1][i])));
      r[i] = Cd::put(acc);
    } else {
      float lo = mul_rn(g[0], Cd::get(static_cast<typename Cd::S>(x[0][i] & 0xffffu)));
      float hi = mul_rn(g[0], Cd::get(static_cast<typename Cd::S>(x[0][i] >> 16)));
      if (K == 2) {
        lo = add_rn(lo, mul_rn(g[1], Cd::get(static_cast<typename Cd::S>(x[1][i] & 0xffffu))));
        hi = add_rn(hi, mul_rn(g[1], Cd::get(static_cast<typename Cd::S>(x[1][i] >> 16))));
      }
      r[i] = static_cast<uint32_t>(Cd::put(lo)) | (static_cast<uint32_t>(Cd::put(hi)) << 16);
    }
  }
  return r;
}

struct DecodeArgs {
  const void* expert_out;
  const void* gates;     // [K*S] of gate_dtype; null = all ones (moe_encode_dx)
  int gate_dtype;
  const int32_t* idx;    // [K*S]
  const int32_t* loc;    // [K*S]
  const int32_t* dest;   // [K*S] or null: row e * C + location of the slot (-1: none) instead of idx / loc
  void* out;             // [S, M]
  int S, M, E, C;
  int slot_stride;       // distance between the slots of one token in gates / idx / loc
  int wpr_shift;         // 2^wpr_shift waves share one token row (each takes every 2^wpr_shift-th run of 64 granules)
};

template <int DT, int K, bool VEC, bool DEST = false>
__global__ __launch_bounds__(kTile) void decode_rows_kernel(DecodeArgs a) {
  typedef Codec<DT> Cd;
  const int w = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const uint32_t gw = blockIdx.x * static_cast<uint32_t>(kRowsPerBlock) + w;
  const int s = static_cast<int>(gw >> a.wpr_shift);
  const int part = static_cast<int>(gw & ((1u << a.wpr_shift) - 1u));
  if (s >= a.S) return;
  const int step = kWave << a.wpr_shift;
  float g[K];
  size_t row[K];
  bool ok[K];
  bool any = false;
#pragma unroll
  for (int j = 0; j < K; ++j) {
    if (DEST) {
      const int d = a.dest[static_cast<size_t>(j) * a.slot_stride + s];
      ok[j] = d >= 0 && d < a.E * a.C;
      row[j] = ok[j] ? static_cast<size_t>(d) : 0;
    } else {
      const int e = a.idx[static_cast<size_t>(j) * a.slot_stride + s];
      const int l = a.loc[static_cast<size_t>(j) * a.slot_stride + s];
      ok[j] = e >= 0 && e < a.E && l >= 0 && l < a.C;
      row[j] = ok[j] ? (static_cast<size_t>(e) * a.C + l) : 0;
    }
    g[j] = ok[j] ? (a.gates ? ld_gate(a.gates, static_cast<size_t>(j) * a.slot_stride + s, a.gate_dtype) : 1.f) : 0.f;
    any = any || ok[j];
  }
  if (VEC) {
    const int row_vecs = a.M / Cd::kPerVec;
    u32x4* dst = static_cast<u32x4*>(a.out) + static_cast<size_t>(s) * row_vecs;
    const u32x4* base = static_cast<const u32x4*>(a.expert_out);
    const u32x4 z = {0u, 0u, 0u, 0u};
    int v = part * kWave + lane;
    if (!any) {
      for (; v < row_vecs; v += step) st_stream(dst + v, z);
      return;
    }
    for (; v + step < row_vecs; v += 2 * step) {  // two granules in flight per slot
      u32x4 xa[K], xb[K];
#pragma unroll
      for (int j = 0; j < K; ++j) {
        xa[j] = ok[j] ? ld_stream(base + row[j] * row_vecs + v) : z;
        xb[j] = ok[j] ? ld_stream(base + row[j] * row_vecs + v + step) : z;
      }
      st_stream(dst + v, combine_vec<DT, K>(xa, g));
      st_stream(dst + v + step, combine_vec<DT, K>(xb, g));
    }
    if (v < row_vecs) {
      u32x4 xa[K];
#pragma unroll
      for (int j = 0; j < K; ++j) xa[j] = ok[j] ? ld_stream(base + row[j] * row_vecs + v) : z;
      st_stream(dst + v, combine_vec<DT, K>(xa, g));
    }
  } else {
    typedef typename Cd::S St;
    St* dst = static_cast<St*>(a.out) + static_cast<size_t>(s) * a.M;
    const St* base = static_cast<const St*>(a.expert_out);
    for (int i = part * kWave + lane; i < a.M; i += step) {
#pragma clang fp contract(off)
      float acc = ok[0] ? mul_rn(g[0], Cd::get(base[row[0] * a.M + i])) : 0.f;
      if (K == 2) acc = add_rn(acc, ok[1] ? mul_rn(g[1], Cd::get(base[row[1] * a.M + i])) : 0.f);
      dst[i] = Cd::put(acc);
    }
  }
}

// ---------------------------------------------------------------------------------------
// merge_masks / redispatch.  Both need kept[p][e] = number of tokens of partition p routed to
// expert e; one counting pass over the masks (the reference re-counts with a tree reduction in
// each of its E blocks, tutel_moe_dispatch.cu:238-253,377-392).
// ---------------------------------------------------------------------------------------
constexpr int kCountPerThread = 4;

__global__ __launch_bounds__(kTile) void count_experts_kernel(PtrTable t, int S, int E, uint32_t* counts) {
  extern __shared__ uint32_t hist[];
  const int p = blockIdx.y;
  const int32_t* idx = static_cast<const int32_t*>(t.p[p]);
  for (int c = threadIdx.x; c < E; c += kTile) hist[c] = 0;
  __syncthreads();
  const int base = blockIdx.x * kTile * kCountPerThread;
#pragma unroll
  for (int k = 0; k < kCountPerThread; ++k) {
    const int i = base + k * kTile + threadIdx.x;
    if (i < S) {
      const int e = idx[i];
      if (e >= 0 && e < E) atomicAdd(&hist[e], 1u);
    }
  }
  __syncthreads();
  for (int c = threadIdx.x; c < E; c += kTile)
    if (hist[c]) atomicAdd(counts + static_cast<size_t>(p) * E + c, hist[c]);
}

// out[0, p*S+i] = idx, out[1, p*S+i] = loc + sum_{q<p} kept[q][idx]; dropped -> (-1,-1)
// (tutel_moe_dispatch.cu:214-236).
__global__ __launch_bounds__(kTile) void merge_masks_kernel(PtrTable t, int P, int S, int E,
                                                            const uint32_t* counts, int32_t* out) {
  extern __shared__ uint32_t s_off[];
  const int p = blockIdx.y;
  for (int c = threadIdx.x; c < E; c += kTile) {
    uint32_t off = 0;
    for (int q = 0; q < p; ++q) off += counts[static_cast<size_t>(q) * E + c];
    s_off[c] = off;
  }
  __syncthreads();
  const int i = blockIdx.x * kTile + threadIdx.x;
  if (i >= S) return;
  const int32_t* il = static_cast<const int32_t*>(t.p[p]);
  const int e = il[i];
  const int l = il[S + i];
  const bool kept = e >= 0 && e < E;
  const size_t o = static_cast<size_t>(p) * S + i;
  out[o] = kept ? e : -1;
  out[static_cast<size_t>(P) * S + o] = kept ? l + static_cast<int>(s_off[e]) : -1;
}

// out[e, off_p[e] + r, :] = buf_p[e, r, :] for r < kept[p][e]; other rows zero
// (tutel_moe_dispatch.cu:365-408, which leaves them uninitialised).
template <typename V>
__global__ __launch_bounds__(kTile) void redispatch_rows_kernel(PtrTable bufs, int P, int E, int C,
                                                                int row_vecs, int wpr_shift,
                                                                const uint32_t* counts, V* out) {
  const int w = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const uint32_t gw = blockIdx.x * static_cast<uint32_t>(kRowsPerBlock) + w;
  const long r = gw >> wpr_shift;
  const int part = static_cast<int>(gw & ((1u << wpr_shift) - 1u));
  const int step = kWave << wpr_shift;
  if (r >= static_cast<long>(E) * C) return;
  const int e = static_cast<int>(r / C);
  const int c = static_cast<int>(r - static_cast<long>(e) * C);
  // which partition holds row c of expert e: lane q takes partition q's count (P <= 64), an inclusive scan
  // over the lanes gives every partition's row range, one ballot finds the owner
  const uint32_t k = lane < P ? counts[static_cast<size_t>(lane) * E + e] : 0u;
  uint32_t incl = k;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t t = __shfl_up(incl, o, kWave);
    if (lane >= o) incl += t;
  }
  const uint32_t excl = incl - k;
  const uint64_t owner = __ballot(lane < P && static_cast<uint32_t>(c) >= excl && static_cast<uint32_t>(c) < incl);
  V* dst = out + static_cast<size_t>(r) * row_vecs;
  if (owner) {
    const int q = __ffsll(static_cast<unsigned long long>(owner)) - 1;
    const int off = static_cast<int>(__shfl(excl, q, kWave));
    const V* src = static_cast<const V*>(bufs.p[q]) + (static_cast<size_t>(e) * C + (c - off)) * row_vecs;
    int v = part * kWave + lane;
    for (; v + step < row_vecs; v += 2 * step) {
      const V x0 = ldv(src + v), x1 = ldv(src + v + step);
      stv(dst + v, x0);
      stv(dst + v + step, x1);
    }
    if (v < row_vecs) stv(dst + v, ldv(src + v));
  } else {
    const V z = zero_v<V>();
    for (int v = part * kWave + lane; v < row_vecs; v += step) stv(dst + v, z);
  }
}

// ---------------------------------------------------------------------------------------
// redispatch_expert_input: merge of P partitions of one local expert's all-to-all output, layout
// [C, G, M] (capacity row, source GPU, model dim).  For source g the partitions' received element
// streams (recv_cnts_p[g*LE + le] * scale elements each, stored from row 0 of partition p) are
// concatenated: stream element x lands at out[x / M, g, x % M]
// (redispatch_expert_input_kernel_CGM, tutel_moe_dispatch.cu:436-456, 586-598).  Rows past the merged
// stream are zero-filled (the reference leaves them as they were).  One wave per output row (c, g);
// whole rows are moved in 16-byte granules when every count is a multiple of M.
// ---------------------------------------------------------------------------------------
struct CountTable {
  const uint64_t* p[kMaxPartitions];
};

// EL = element storage type; VEC = rows and pointers allow 16-byte granules (the row-aligned case then
// moves whole rows with them; streams that are not row aligned always take the element path).
template <typename EL, bool VEC>
__global__ __launch_bounds__(kTile) void redispatch_expert_input_kernel(PtrTable bufs, CountTable cnts, int P,
                                                                        int le, int LE, int C, int M, int G,
                                                                        uint64_t scale, EL* out) {
  const int w = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const long r = static_cast<long>(blockIdx.x) * kRowsPerBlock + w;  // output row index c*G + g
  if (r >= static_cast<long>(C) * G) return;
  const int c = static_cast<int>(r / G);
  const int g = static_cast<int>(r - static_cast<long>(c) * G);
  EL* dst = out + static_cast<size_t>(r) * M;
  const uint64_t x0 = static_cast<uint64_t>(c) * M;  // first stream element of this row
  uint64_t cum = 0, cum0 = 0;
  int p0 = -1;
  bool rows_only = true;
  for (int q = 0; q < P; ++q) {
    const uint64_t n = cnts.p[q][static_cast<size_t>(g) * LE + le] * scale;
    rows_only = rows_only && (n % M == 0);
    if (p0 < 0 && x0 < cum + n) {
      p0 = q;
      cum0 = cum;
    }
    cum += n;
  }
  const uint64_t total = cum;
  constexpr int kPer = 16 / sizeof(EL);
  if (x0 >= total) {  // past the merged stream
    if (VEC) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (int v = lane; v < M / kPer; v += kWave) st_stream(reinterpret_cast<u32x4*>(dst) + v, z);
    } else {
      for (int i = lane; i < M; i += kWave) dst[i] = EL(0);
    }
    return;
  }
  if (rows_only) {
    const uint64_t src_row = (x0 - cum0) / M;
    const bool readable = src_row < static_cast<uint64_t>(C);  // counts larger than the buffer read nothing
    const EL* src = static_cast<const EL*>(bufs.p[p0]) + (readable ? (src_row * G + g) * M : 0);
    if (VEC) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (int v = lane; v < M / kPer; v += kWave)
        st_stream(reinterpret_cast<u32x4*>(dst) + v, readable ? ld_stream(reinterpret_cast<const u32x4*>(src) + v) : z);
    } else {
      for (int i = lane; i < M; i += kWave) dst[i] = readable ? src[i] : EL(0);
    }
    return;
  }
  // element-granular streams: every element finds its partition
  for (int i = lane; i < M; i += kWave) {
    const uint64_t x = x0 + i;
    EL val = EL(0);
    if (x < total) {
      uint64_t run = 0;
      for (int q = 0; q < P; ++q) {
        const uint64_t n = cnts.p[q][static_cast<size_t>(g) * LE + le] * scale;
        if (x < run + n) {
          const uint64_t y = x - run;
          const uint64_t sr = y / M;
          if (sr < static_cast<uint64_t>(C)) val = static_cast<const EL*>(bufs.p[q])[(sr * G + g) * M + (y - sr * M)];
          break;
        }
        run += n;
      }
    }
    dst[i] = val;
  }
}

// ---------------------------------------------------------------------------------------
// backward kernels.  moe_encode_dx is decode_rows_kernel with unit gates
// (encode_backward_data_kernel, tutel_moe_dispatch.cu:88-94).
// ---------------------------------------------------------------------------------------
// grad_gates[s, e] = dy[j*S+s] where e is token s's expert in slot j, else 0: the memset + scatter of
// encode_backward_gate_kernel (tutel_moe_dispatch.cu:96-105, 499-506) as one pass that writes every
// element once.
template <int K>
__global__ __launch_bounds__(kTile) void encode_dg_kernel(const void* dy, const int32_t* idx, int S, int E,
                                                          void* grad_gates, int gd) {
  const size_t n = static_cast<size_t>(S) * E;
  for (size_t i = blockIdx.x * static_cast<size_t>(kTile) + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * kTile) {
    const int s = static_cast<int>(i / E);
    const int e = static_cast<int>(i - static_cast<size_t>(s) * E);
    float v = 0.f;
    if (idx[s] == e) v = ld_gate(dy, s, gd);
    if (K == 2 && idx[S + s] == e) v = ld_gate(dy, static_cast<size_t>(S) + s, gd);
    st_gate(grad_gates, i, v, gd);
  }
}

// src[e*C + l] = slot-token id (j*S + s) of the token that owns row (e, l); src is -1 elsewhere.
__global__ __launch_bounds__(kTile) void inverse_map_kernel(const int32_t* idx, const int32_t* loc, int n, int E,
                                                            int C, int32_t* src) {
  const int i = blockIdx.x * kTile + threadIdx.x;
  if (i >= n) return;
  const int e = idx[i], l = loc[i];
  if (e >= 0 && e < E && l >= 0 && l < C) src[static_cast<size_t>(e) * C + l] = i;
}

// grad_expert_out[e, l, :] = gates[i] * dy[s, :] for the slot-token i = src[e*C+l] (s = i mod S), zero
// for rows nobody owns: decode_backward_data_kernel (tutel_moe_dispatch.cu:118-124, 523-533) without
// the memset + atomicAdd; every output byte is written once.
template <int DT, bool VEC>
__global__ __launch_bounds__(kTile) void decode_dx_rows_kernel(const void* dy, const void* gates, int gd,
                                                               const int32_t* src, void* out, int S, int M,
                                                               long rows, int wpr_shift) {
  typedef Codec<DT> Cd;
  const int w = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const uint32_t gw = blockIdx.x * static_cast<uint32_t>(kRowsPerBlock) + w;
  const long r = gw >> wpr_shift;
  const int part = static_cast<int>(gw & ((1u << wpr_shift) - 1u));
  const int step = kWave << wpr_shift;
  if (r >= rows) return;
  const int i = src[r];
  const float g1[1] = {i >= 0 ? ld_gate(gates, i, gd) : 0.f};
  const size_t s = i >= 0 ? static_cast<size_t>(i % S) : 0;
  if (VEC) {
    const int row_vecs = M / Cd::kPerVec;
    u32x4* dst = static_cast<u32x4*>(out) + static_cast<size_t>(r) * row_vecs;
    const u32x4 z = {0u, 0u, 0u, 0u};
    int v = part * kWave + lane;
    if (i < 0) {
      for (; v < row_vecs; v += step) st_stream(dst + v, z);
      return;
    }
    const u32x4* sp = static_cast<const u32x4*>(dy) + s * row_vecs;
    for (; v + step < row_vecs; v += 2 * step) {
      const u32x4 xa[1] = {ld_stream(sp + v)};
      const u32x4 xb[1] = {ld_stream(sp + v + step)};
      st_stream(dst + v, combine_vec<DT, 1>(xa, g1));
      st_stream(dst + v + step, combine_vec<DT, 1>(xb, g1));
    }
    if (v < row_vecs) {
      const u32x4 xa[1] = {ld_stream(sp + v)};
      st_stream(dst + v, combine_vec<DT, 1>(xa, g1));
    }
  } else {
    typedef typename Cd::S St;
    St* dst = static_cast<St*>(out) + static_cast<size_t>(r) * M;
    const St* sp = static_cast<const St*>(dy) + s * M;
    for (int k = part * kWave + lane; k < M; k += step)
      dst[k] = i >= 0 ? Cd::put(mul_rn(g1[0], Cd::get(sp[k]))) : Cd::put(0.f);
  }
}

// grad_gates_s[i] = <expert_out[idx, loc, :], dy[s, :]> for slot-token i, 0 when the slot is dropped
// (decode_backward_gate_kernel, tutel_moe_dispatch.cu:126-157): one wave per slot-token, fp32 partial
// sums per lane, xor-tree over the wave.
template <int DT, bool VEC>
__global__ __launch_bounds__(kTile) void decode_dg_kernel(const void* dy, const void* expert_out,
                                                          const int32_t* idx, const int32_t* loc, void* out, int gd,
                                                          int S, int M, int E, int C, int n) {
  typedef Codec<DT> Cd;
  const int w = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const int i = blockIdx.x * kRowsPerBlock + w;
  if (i >= n) return;
  const int e = idx[i], l = loc[i];
  if (!(e >= 0 && e < E && l >= 0 && l < C)) {
    if (lane == 0) st_gate(out, i, 0.f, gd);
    return;
  }
  const size_t s = static_cast<size_t>(i % S);
  const size_t row = static_cast<size_t>(e) * C + l;
  float acc = 0.f;
  if (VEC) {
    const int row_vecs = M / Cd::kPerVec;
    const u32x4* a = static_cast<const u32x4*>(expert_out) + row * row_vecs;
    const u32x4* b = static_cast<const u32x4*>(dy) + s * row_vecs;
    for (int v = lane; v < row_vecs; v += kWave) {
      const u32x4 x = ld_stream(a + v), y = ld_stream(b + v);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (Cd::kPerVec == 4) {
          acc += Cd::get(x[k]) * Cd::get(y[k]);
        } else {
          acc += Cd::get(static_cast<typename Cd::S>(x[k] & 0xffffu)) * Cd::get(static_cast<typename Cd::S>(y[k] & 0xffffu));
          acc += Cd::get(static_cast<typename Cd::S>(x[k] >> 16)) * Cd::get(static_cast<typename Cd::S>(y[k] >> 16));
        }
      }
    }
  } else {
    typedef typename Cd::S St;
    const St* a = static_cast<const St*>(expert_out) + row * M;
    const St* b = static_cast<const St*>(dy) + s * M;
    for (int k = lane; k < M; k += kWave) acc += Cd::get(a[k]) * Cd::get(b[k]);
  }
  acc = wave_sum(acc);
  if (lane == 0) st_gate(out, i, acc, gd);
}

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// log2 of the number of waves that share one row of `units` granules: a power of two (the kernels split the wave
// index with a shift), per_lane granules per lane where the grid allows it, at most 16 waves.  Measured at 8 KB
// rows: the scatter is fastest with one granule per lane (8 waves a row), the gather-combine with two (4 waves).
static inline int split_waves(long units, long rows, int per_lane = 1) {
  const long span = static_cast<long>(kWave) * per_lane;
  const long want = std::max<long>((units + span - 1) / span, 1);
  int shift = 0;
  while (shift < 4 && (1L << shift) < want) ++shift;
  // the grid stays below 2^30 workgroups and the wave index below 2^32
  while (shift > 0 && ((rows << shift) + kRowsPerBlock - 1) / kRowsPerBlock > 0x3fffffffL) --shift;
  return shift;
}

template <typename V>
static hipError_t scatter_launch(const void* data, void* out, const int32_t* idx, const int32_t* loc,
                                 const int32_t* avail_used, const int32_t* row_base, const int32_t* rows_lo,
                                 const int32_t* rows_hi, int S, int E, int C, int K, int row_vecs,
                                 int slot_stride, hipStream_t st, const int32_t* dest = nullptr) {
  ScatterArgs<V> a;
  a.dest = dest;
  a.data = static_cast<const V*>(data);
  a.out = static_cast<V*>(out);
  a.idx = idx;
  a.loc = loc;
  a.avail_used = avail_used;
  a.row_base = row_base;
  a.rows_lo = rows_lo;
  a.rows_hi = rows_hi;
  a.S = S;
  a.E = E;
  a.C = C;
  a.K = K;
  a.slot_stride = slot_stride;
  a.row_vecs = row_vecs;
  a.wpr_shift = split_waves(row_vecs, S);
  a.token_blocks = static_cast<int>(((static_cast<long>(S) << a.wpr_shift) + kRowsPerBlock - 1) / kRowsPerBlock);
  a.tail_chunks = rows_hi ? (C + kTailRows - 1) / kTailRows : 0;
  const long blocks = static_cast<long>(a.token_blocks) + static_cast<long>(a.tail_chunks) * E;
  if (blocks == 0) return hipSuccess;
  if (dest) {
    if (K == 1) scatter_rows_kernel<V, 1, true><<<static_cast<unsigned>(blocks), kTile, 0, st>>>(a);
    else scatter_rows_kernel<V, 2, true><<<static_cast<unsigned>(blocks), kTile, 0, st>>>(a);
  } else if (K == 1) scatter_rows_kernel<V, 1><<<static_cast<unsigned>(blocks), kTile, 0, st>>>(a);
  else scatter_rows_kernel<V, 2><<<static_cast<unsigned>(blocks), kTile, 0, st>>>(a);
  return hipGetLastError();
}

hipError_t run_scatter_rows(const void* data, void* out, const int32_t* idx, const int32_t* loc,
                            const int32_t* avail_used, const int32_t* row_base, const int32_t* rows_lo,
                            const int32_t* rows_hi,
                            int S, int M, int E, int C, int K, int elem_bytes, hipStream_t st, int slot_stride,
                            const int32_t* dest) {
  const size_t row_bytes = static_cast<size_t>(M) * elem_bytes;
  if (row_bytes == 0) return hipSuccess;
  const int ss = slot_stride < 0 ? S : slot_stride;
  if (row_bytes % 16 == 0 && aligned16(data) && aligned16(out))
    return scatter_launch<u32x4>(data, out, idx, loc, avail_used, row_base, rows_lo, rows_hi, S, E, C, K,
                                 static_cast<int>(row_bytes / 16), ss, st, dest);
  if (dest) return hipErrorInvalidValue;  // the one-word form is for rows of 16-byte granules
  if (elem_bytes == 4)
    return scatter_launch<uint32_t>(data, out, idx, loc, avail_used, row_base, rows_lo, rows_hi, S, E, C, K, M, ss, st);
  return scatter_launch<uint16_t>(data, out, idx, loc, avail_used, row_base, rows_lo, rows_hi, S, E, C, K, M, ss, st);
}

hipError_t run_zero_bytes(void* p, size_t nbytes, hipStream_t st) {
  if (nbytes == 0) return hipSuccess;
  uint8_t* b = static_cast<uint8_t*>(p);
  // head bytes up to 16-byte alignment are cleared together with the tail by a second launch
  const size_t head = (16 - (reinterpret_cast<uintptr_t>(b) & 15u)) & 15u;
  const size_t h = std::min(head, nbytes);
  if (h) {
    zero_bytes_kernel<<<1, 64, 0, st>>>(nullptr, 0, b, h);
    b += h;
    nbytes -= h;
  }
  const size_t nvec = nbytes / 16;
  const size_t ntail = nbytes - nvec * 16;
  if (nvec || ntail) {
    // one granule per thread up to 2^22 workgroups (16 GiB), a loop beyond that
    const int blocks = static_cast<int>(std::min<size_t>((nvec + 255) / 256 + 1, size_t(1) << 22));
    zero_bytes_kernel<<<blocks, 256, 0, st>>>(reinterpret_cast<u32x4*>(b), nvec, b + nvec * 16, ntail);
  }
  return hipGetLastError();
}

template <int DT>
static hipError_t decode_launch(DecodeArgs a, int K, bool vec, hipStream_t st) {
  if (a.S == 0 || a.M == 0) return hipSuccess;
  a.wpr_shift = split_waves(vec ? a.M / Codec<DT>::kPerVec : a.M, a.S, 2);
  const unsigned blocks = static_cast<unsigned>(((static_cast<long>(a.S) << a.wpr_shift) + kRowsPerBlock - 1) / kRowsPerBlock);
  if (a.dest) {
    if (!vec) return hipErrorInvalidValue;
    if (K == 1) decode_rows_kernel<DT, 1, true, true><<<blocks, kTile, 0, st>>>(a);
    else decode_rows_kernel<DT, 2, true, true><<<blocks, kTile, 0, st>>>(a);
  } else if (K == 1) {
    if (vec) decode_rows_kernel<DT, 1, true><<<blocks, kTile, 0, st>>>(a);
    else decode_rows_kernel<DT, 1, false><<<blocks, kTile, 0, st>>>(a);
  } else {
    if (vec) decode_rows_kernel<DT, 2, true><<<blocks, kTile, 0, st>>>(a);
    else decode_rows_kernel<DT, 2, false><<<blocks, kTile, 0, st>>>(a);
  }
  return hipGetLastError();
}

hipError_t run_decode_rows(const void* expert_out, const void* gates, int gate_dtype, const int32_t* idx,
                           const int32_t* loc, void* out, int S, int M, int E, int C, int K,
                           int dtype, hipStream_t st, int slot_stride, const int32_t* dest) {
  DecodeArgs a;
  a.dest = dest;
  a.expert_out = expert_out;
  a.gates = gates;
  a.gate_dtype = gate_dtype;
  a.idx = idx;
  a.loc = loc;
  a.out = out;
  a.S = S;
  a.M = M;
  a.E = E;
  a.C = C;
  a.slot_stride = slot_stride < 0 ? S : slot_stride;
  const int per_vec = (dtype == LANCET_F32) ? 4 : 8;
  const bool vec = (M % per_vec == 0) && aligned16(expert_out) && aligned16(out);
  switch (dtype) {
    case LANCET_F32: return decode_launch<LANCET_F32>(a, K, vec, st);
    case LANCET_BF16: return decode_launch<LANCET_BF16>(a, K, vec, st);
    default: return decode_launch<LANCET_F16>(a, K, vec, st);
  }
}

hipError_t run_count_experts(const PtrTable& indlocs, int P, int S, int E, uint32_t* counts, hipStream_t st) {
  hipError_t err = run_fill_u32(counts, static_cast<size_t>(P) * E, 0u, st);
  if (err != hipSuccess || S == 0) return err;
  dim3 grid((S + kTile * kCountPerThread - 1) / (kTile * kCountPerThread), P);
  count_experts_kernel<<<grid, kTile, E * sizeof(uint32_t), st>>>(indlocs, S, E, counts);
  return hipGetLastError();
}

hipError_t run_merge_masks(const PtrTable& indlocs, int P, int S, int E, const uint32_t* counts,
                           int32_t* out, hipStream_t st) {
  if (S == 0) return hipSuccess;
  dim3 grid((S + kTile - 1) / kTile, P);
  merge_masks_kernel<<<grid, kTile, E * sizeof(uint32_t), st>>>(indlocs, P, S, E, counts, out);
  return hipGetLastError();
}

hipError_t run_redispatch_rows(const PtrTable& bufs, int P, int M, int C, int E, const uint32_t* counts,
                               void* out, int elem_bytes, hipStream_t st) {
  const size_t row_bytes = static_cast<size_t>(M) * elem_bytes;
  const long rows = static_cast<long>(E) * C;
  if (rows == 0 || row_bytes == 0) return hipSuccess;
  bool vec = row_bytes % 16 == 0 && aligned16(out);
  for (int p = 0; p < P; ++p) vec = vec && aligned16(bufs.p[p]);
  const int units = vec ? static_cast<int>(row_bytes / 16) : M;
  const int shift = split_waves(units, rows, 2);  // two granules per lane: 426 -> 408 us
  const unsigned blocks = static_cast<unsigned>(((rows << shift) + kRowsPerBlock - 1) / kRowsPerBlock);
  if (vec)
    redispatch_rows_kernel<u32x4><<<blocks, kTile, 0, st>>>(bufs, P, E, C, units, shift, counts, static_cast<u32x4*>(out));
  else if (elem_bytes == 4)
    redispatch_rows_kernel<uint32_t><<<blocks, kTile, 0, st>>>(bufs, P, E, C, units, shift, counts,
                                                               static_cast<uint32_t*>(out));
  else
    redispatch_rows_kernel<uint16_t><<<blocks, kTile, 0, st>>>(bufs, P, E, C, units, shift, counts,
                                                               static_cast<uint16_t*>(out));
  return hipGetLastError();
}

hipError_t run_encode_dg(const void* dy, const int32_t* idx, int S, int E, int K, int gate_dtype, void* grad_gates, hipStream_t st) {
  const size_t n = static_cast<size_t>(S) * E;
  if (n == 0) return hipSuccess;
  const int blocks = static_cast<int>(std::min<size_t>((n + kTile - 1) / kTile, 65536));
  if (K == 1) encode_dg_kernel<1><<<blocks, kTile, 0, st>>>(dy, idx, S, E, grad_gates, gate_dtype);
  else encode_dg_kernel<2><<<blocks, kTile, 0, st>>>(dy, idx, S, E, grad_gates, gate_dtype);
  return hipGetLastError();
}

template <int DT>
static hipError_t decode_dx_launch(const void* dy, const void* gates, int gd, const int32_t* src, void* out, int S, int M,
                                   long rows, bool vec, hipStream_t st) {
  const int shift = split_waves(vec ? M / Codec<DT>::kPerVec : M, rows, 2);  // two granules per lane: 442 -> 408 us
  const unsigned blocks = static_cast<unsigned>(((rows << shift) + kRowsPerBlock - 1) / kRowsPerBlock);
  if (vec) decode_dx_rows_kernel<DT, true><<<blocks, kTile, 0, st>>>(dy, gates, gd, src, out, S, M, rows, shift);
  else decode_dx_rows_kernel<DT, false><<<blocks, kTile, 0, st>>>(dy, gates, gd, src, out, S, M, rows, shift);
  return hipGetLastError();
}

hipError_t run_decode_dx(const void* dy, const void* gates, int gate_dtype, const int32_t* idx, const int32_t* loc, void* out,
                         int32_t* src_map, int S, int M, int E, int C, int K, int dtype, hipStream_t st) {
  const long rows = static_cast<long>(E) * C;
  if (rows == 0 || M == 0) return hipSuccess;
  hipError_t err = run_fill_u32(reinterpret_cast<uint32_t*>(src_map), static_cast<size_t>(rows), 0xffffffffu, st);
  if (err != hipSuccess) return err;
  const int n = K * S;
  if (n > 0) {
    inverse_map_kernel<<<(n + kTile - 1) / kTile, kTile, 0, st>>>(idx, loc, n, E, C, src_map);
    err = hipGetLastError();
    if (err != hipSuccess) return err;
  }
  const int per_vec = (dtype == LANCET_F32) ? 4 : 8;
  const bool vec = (M % per_vec == 0) && aligned16(dy) && aligned16(out);
  switch (dtype) {
    case LANCET_F32: return decode_dx_launch<LANCET_F32>(dy, gates, gate_dtype, src_map, out, S, M, rows, vec, st);
    case LANCET_BF16: return decode_dx_launch<LANCET_BF16>(dy, gates, gate_dtype, src_map, out, S, M, rows, vec, st);
    default: return decode_dx_launch<LANCET_F16>(dy, gates, gate_dtype, src_map, out, S, M, rows, vec, st);
  }
}

template <int DT>
static hipError_t decode_dg_launch(const void* dy, const void* expert_out, const int32_t* idx, const int32_t* loc,
                                   void* out, int gd, int S, int M, int E, int C, int n, bool vec, hipStream_t st) {
  const int blocks = (n + kRowsPerBlock - 1) / kRowsPerBlock;
  if (vec) decode_dg_kernel<DT, true><<<blocks, kTile, 0, st>>>(dy, expert_out, idx, loc, out, gd, S, M, E, C, n);
  else decode_dg_kernel<DT, false><<<blocks, kTile, 0, st>>>(dy, expert_out, idx, loc, out, gd, S, M, E, C, n);
  return hipGetLastError();
}

hipError_t run_decode_dg(const void* dy, const void* expert_out, const int32_t* idx, const int32_t* loc, void* out,
                         int gate_dtype, int S, int M, int E, int C, int K, int dtype, hipStream_t st) {
  const int n = K * S;
  if (n == 0) return hipSuccess;
  const int per_vec = (dtype == LANCET_F32) ? 4 : 8;
  const bool vec = (M % per_vec == 0) && aligned16(dy) && aligned16(expert_out);
  switch (dtype) {
    case LANCET_F32: return decode_dg_launch<LANCET_F32>(dy, expert_out, idx, loc, out, gate_dtype, S, M, E, C, n, vec, st);
    case LANCET_BF16: return decode_dg_launch<LANCET_BF16>(dy, expert_out, idx, loc, out, gate_dtype, S, M, E, C, n, vec, st);
    default: return decode_dg_launch<LANCET_F16>(dy, expert_out, idx, loc, out, gate_dtype, S, M, E, C, n, vec, st);
  }
}

hipError_t run_redispatch_expert_input(const PtrTable& bufs, const void* const* cnt_ptrs, int P, int le, int LE, int C,
                                       int M, int G, uint64_t scale, void* out, int elem_bytes, hipStream_t st) {
  const long rows = static_cast<long>(C) * G;
  if (rows == 0 || M == 0) return hipSuccess;
  CountTable ct;
  for (int q = 0; q < kMaxPartitions; ++q) ct.p[q] = q < P ? static_cast<const uint64_t*>(cnt_ptrs[q]) : nullptr;
  const unsigned blocks = static_cast<unsigned>((rows + kRowsPerBlock - 1) / kRowsPerBlock);
  const size_t row_bytes = static_cast<size_t>(M) * elem_bytes;
  bool vec = row_bytes % 16 == 0 && aligned16(out);
  for (int q = 0; q < P; ++q) vec = vec && aligned16(bufs.p[q]);
  if (elem_bytes == 4) {
    if (vec) redispatch_expert_input_kernel<uint32_t, true><<<blocks, kTile, 0, st>>>(bufs, ct, P, le, LE, C, M, G, scale, static_cast<uint32_t*>(out));
    else redispatch_expert_input_kernel<uint32_t, false><<<blocks, kTile, 0, st>>>(bufs, ct, P, le, LE, C, M, G, scale, static_cast<uint32_t*>(out));
  } else {
    if (vec) redispatch_expert_input_kernel<uint16_t, true><<<blocks, kTile, 0, st>>>(bufs, ct, P, le, LE, C, M, G, scale, static_cast<uint16_t*>(out));
    else redispatch_expert_input_kernel<uint16_t, false><<<blocks, kTile, 0, st>>>(bufs, ct, P, le, LE, C, M, G, scale, static_cast<uint16_t*>(out));
  }
  return hipGetLastError();
}

}  // namespace lancet
