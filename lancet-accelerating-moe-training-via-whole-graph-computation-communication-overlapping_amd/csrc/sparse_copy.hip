// Copies between a 3-D "sparse" buffer, in which block b along one axis holds only its first n_b
// elements, and the packed stream of those elements (memcpy_sparse_to_cont_3d /
// memcpy_cont_to_sparse_3d, src/op/dialect/cuda/kernels/sparse_memcpy.cu:11-96).  n_b comes from a
// device array of uint64 element counts read with a stride and an offset, which is how a caller
// picks one column of elements_per_expert viewed as [G, LE].
//
//   n_b   = counts[b*stride + offset] * scale / shrink
//   off_b = (sum_{j<b} counts[j*stride + offset]) * scale / shrink          (sum first, as the source does)
//   axis 0: stream[off_b + t] <-> buf[b, t / dim2, t % dim2]
//   axis 1: stream[off_b + t] <-> buf[t / dim2, b, t % dim2]
// With a second array `starts` (same indexing and scaling as the counts) block b's elements are
// [start_b, start_b + n_b) instead of [0, n_b): the rows one token partition owns inside a buffer that
// several partitions share.
//
// The grid is (chunks, blocks along the axis): unlike one workgroup per block, a few long blocks
// still fill the chip.  Elements move in 16-byte granules where offsets and rows allow it.
#include "common.hpp"
#include "launchers.hpp"

namespace lancet {

namespace {

__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const uint32_t lo = __shfl_xor(static_cast<uint32_t>(v), o, kWave);
    const uint32_t hi = __shfl_xor(static_cast<uint32_t>(v >> 32), o, kWave);
    v += (static_cast<uint64_t>(hi) << 32) | lo;
  }
  return v;
}

// position of stream element t of block b inside the 3-D buffer
template <int AXIS>
__device__ __forceinline__ size_t sparse_index(uint32_t b, uint32_t t, uint32_t dim1, uint32_t dim2) {
  if (AXIS == 0) return static_cast<size_t>(b) * dim1 * dim2 + t;
  const uint32_t r = t / dim2;
  return (static_cast<size_t>(r) * dim1 + b) * dim2 + (t - r * dim2);
}

// EL: element storage type.  TO_CONT: buffer -> stream, else stream -> buffer.  VEC: the dims and base
// pointers allow 16-byte granules (the block's own offset is checked at run time).  ZERO_TAIL (only
// stream -> buffer): elements [n_b, block_cap) of every block are cleared.
template <typename EL, int AXIS, bool TO_CONT, bool VEC, bool ZERO_TAIL>
__global__ __launch_bounds__(kTile) void sparse_copy_3d_kernel(const EL* __restrict__ src, EL* __restrict__ dst,
                                                               const uint64_t* __restrict__ counts,
                                                               const uint64_t* __restrict__ starts, int stride,
                                                               int offset, uint32_t dim1, uint32_t dim2,
                                                               uint32_t block_cap, uint64_t cont_cap, uint64_t scale,
                                                               uint64_t shrink) {
  __shared__ uint64_t s_part[kWavesPerTile];
  const uint32_t b = blockIdx.y;
  uint64_t acc = 0;
  for (uint32_t j = threadIdx.x; j < b; j += kTile) acc += counts[static_cast<size_t>(j) * stride + offset];
  acc = wave_sum_u64(acc);
  if (lane_id() == 0) s_part[threadIdx.x / kWave] = acc;
  __syncthreads();
  uint64_t before = 0;
#pragma unroll
  for (int w = 0; w < kWavesPerTile; ++w) before += s_part[w];
  const uint64_t off = before * scale / shrink;
  uint64_t n64 = counts[static_cast<size_t>(b) * stride + offset] * scale / shrink;
  uint64_t start64 = starts ? starts[static_cast<size_t>(b) * stride + offset] * scale / shrink : 0;
  // never leave the block or the stream
  if (start64 > block_cap) start64 = block_cap;
  if (n64 > block_cap - start64) n64 = block_cap - start64;
  const uint32_t start = static_cast<uint32_t>(start64);
  if (off >= cont_cap) n64 = 0;
  else if (n64 > cont_cap - off) n64 = cont_cap - off;
  const uint32_t n = static_cast<uint32_t>(n64);
  const uint32_t end = (!TO_CONT && ZERO_TAIL) ? block_cap - start : n;  // the fill covers [start + n, block_cap)

  constexpr uint32_t kPer = 16 / sizeof(EL);
  const uint32_t step = gridDim.x * kTile;
  const uint32_t first = blockIdx.x * kTile + threadIdx.x;
  if (VEC && off % kPer == 0 && start % kPer == 0) {
    const uint32_t n_vec = n / kPer;                  // whole granules inside the copied part
    const uint32_t end_vec = end / kPer;              // dims are multiples of kPer, so is block_cap
    for (uint32_t v = first; v < end_vec; v += step) {
      const uint32_t t = v * kPer;
      const size_t si = sparse_index<AXIS>(b, start + t, dim1, dim2);
      if (TO_CONT) {
        st_stream(reinterpret_cast<u32x4*>(dst + off + t), ld_stream(reinterpret_cast<const u32x4*>(src + si)));
      } else if (v < n_vec) {
        st_stream(reinterpret_cast<u32x4*>(dst + si), ld_stream(reinterpret_cast<const u32x4*>(src + off + t)));
      } else if (t >= n) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        st_stream(reinterpret_cast<u32x4*>(dst + si), z);
      } else {  // the granule that holds element n
        for (uint32_t i = 0; i < kPer; ++i) dst[si + i] = t + i < n ? src[off + t + i] : EL(0);
      }
    }
    // elements of the copied part after its last whole granule (buffer -> stream, or no zero fill)
    if (TO_CONT || !ZERO_TAIL) {
      const uint32_t t = n_vec * kPer + first;
      if (blockIdx.x == 0 && t < n) {
        const size_t si = sparse_index<AXIS>(b, start + t, dim1, dim2);
        if (TO_CONT) dst[off + t] = src[si];
        else dst[si] = src[off + t];
      }
    }
    return;
  }
  for (uint32_t t = first; t < end; t += step) {
    const size_t si = sparse_index<AXIS>(b, start + t, dim1, dim2);
    if (TO_CONT) dst[off + t] = src[si];
    else dst[si] = t < n ? src[off + t] : EL(0);
  }
}

template <typename EL, int AXIS, bool TO_CONT>
hipError_t launch(const void* src, void* dst, const uint64_t* counts, const uint64_t* starts, int stride, int offset, int nblocks, uint32_t dim1,
                  uint32_t dim2, uint32_t block_cap, uint64_t cont_cap, uint64_t scale, uint64_t shrink, bool vec,
                  bool zero_tail, hipStream_t st) {
  constexpr uint32_t kPer = 16 / sizeof(EL);
  const uint32_t per_wg = kTile * kPer * 4;  // about four granules per thread
  uint32_t chunks = (block_cap + per_wg - 1) / per_wg;
  if (chunks < 1) chunks = 1;
  if (chunks > 1024) chunks = 1024;
  const dim3 grid(chunks, static_cast<unsigned>(nblocks));
  const EL* s = static_cast<const EL*>(src);
  EL* d = static_cast<EL*>(dst);
#define LANCET_SPARSE_LAUNCH(V, Z) \
  sparse_copy_3d_kernel<EL, AXIS, TO_CONT, V, Z><<<grid, kTile, 0, st>>>(s, d, counts, starts, stride, offset, dim1, dim2, block_cap, cont_cap, scale, shrink)
  if (!TO_CONT && zero_tail) {
    if (vec) LANCET_SPARSE_LAUNCH(true, true);
    else LANCET_SPARSE_LAUNCH(false, true);
  } else {
    if (vec) LANCET_SPARSE_LAUNCH(true, false);
    else LANCET_SPARSE_LAUNCH(false, false);
  }
#undef LANCET_SPARSE_LAUNCH
  return hipGetLastError();
}

template <typename EL>
hipError_t launch_el(const void* src, void* dst, const uint64_t* counts, const uint64_t* starts, int stride, int offset, int axis, int dim0,
                     int dim1, int dim2, uint64_t cont_cap, uint64_t scale, uint64_t shrink, bool to_cont,
                     bool zero_tail, hipStream_t st) {
  constexpr uint32_t kPer = 16 / sizeof(EL);
  const int nblocks = axis == 0 ? dim0 : dim1;
  const uint32_t block_cap = static_cast<uint32_t>(axis == 0 ? static_cast<int64_t>(dim1) * dim2 : static_cast<int64_t>(dim0) * dim2);
  if (nblocks == 0 || block_cap == 0) return hipSuccess;
  // axis 0 moves flat runs of dim1*dim2 elements, axis 1 runs of dim2
  const uint32_t run = axis == 0 ? block_cap : static_cast<uint32_t>(dim2);
  const bool vec = run % kPer == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
  const uint32_t d1 = static_cast<uint32_t>(dim1), d2 = static_cast<uint32_t>(dim2);
  if (axis == 0) {
    return to_cont ? launch<EL, 0, true>(src, dst, counts, starts, stride, offset, nblocks, d1, d2, block_cap, cont_cap, scale, shrink, vec, zero_tail, st)
                   : launch<EL, 0, false>(src, dst, counts, starts, stride, offset, nblocks, d1, d2, block_cap, cont_cap, scale, shrink, vec, zero_tail, st);
  }
  return to_cont ? launch<EL, 1, true>(src, dst, counts, starts, stride, offset, nblocks, d1, d2, block_cap, cont_cap, scale, shrink, vec, zero_tail, st)
                 : launch<EL, 1, false>(src, dst, counts, starts, stride, offset, nblocks, d1, d2, block_cap, cont_cap, scale, shrink, vec, zero_tail, st);
}

}  // namespace

hipError_t run_sparse_copy_3d(const void* src, void* dst, const uint64_t* counts, const uint64_t* starts, int stride, int offset, int axis,
                              int dim0, int dim1, int dim2, uint64_t cont_cap, uint64_t scale, uint64_t shrink,
                              bool to_cont, bool zero_tail, int elem_bytes, hipStream_t st) {
  if (elem_bytes == 4)
    return launch_el<uint32_t>(src, dst, counts, starts, stride, offset, axis, dim0, dim1, dim2, cont_cap, scale, shrink, to_cont, zero_tail, st);
  return launch_el<uint16_t>(src, dst, counts, starts, stride, offset, axis, dim0, dim1, dim2, cont_cap, scale, shrink, to_cont, zero_tail, st);
}

}  // namespace lancet
