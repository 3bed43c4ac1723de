// Gate gradient of moe_encode as a whole: from the gradient of the op's OUTPUT gates_s back to the [S,E] array
// the op was given, through everything the op does to a gate value on the way:
//   top_k = 1, probabilities   nothing: grad[s, idx] = dy            (encode_backward_gate_kernel,
//                              src/op/dialect/cuda/kernels/tutel_moe_dispatch.cu:96-105; wired by
//                              src/op/grad/moe.cc:30-58)
//   top_k = 2                  the normalisation g_k / max(g_1 + g_2, eps) of the two kept values
//                              (docker/resources/sharded_moe.py:304-312; the clamp passes no gradient to the sum
//                              below eps)
//   LANCET_GATE_IS_LOGITS      the softmax the op fuses in front of the selection (sharded_moe.py:260):
//                              d x[e] = p[e] * (d p[e] - sum_j p[i_j] * d p[i_j])
// Probabilities of a 16-bit softmax are taken as computed (fp32), not as a 16-bit gates_s array would hold them:
// the difference is below that type's own rounding.  Dropped slots carry no gradient (their mask is zero,
// sharded_moe.py:296-297,306-307).  One launch: four lanes per token form the token's few scalars (row maximum,
// 1 / sum of exponentials, the two slot gradients), then the workgroup writes its 64 tokens' block of the
// result in memory order, every element once.
#include "launchers.hpp"
#include "select.hpp"
#include <algorithm>

namespace lancet {

struct GateGradArgs {
  const void* dy;        // [K*S] gradient of gates_s
  const void* gate;      // [S,E] the forward's gate input (may be null for top-1 on probabilities)
  const int32_t* idx;    // [K*S] expert per slot after the drop (row 0 of indices_locations)
  void* out;             // [S,E]
  int S, E;
  int is_logits;
  int vec;               // rows and pointers allow 16-byte granules
};

// A token's row is walked by kSub lanes, each taking every kSub-th 16-byte granule (or element), with the maximum
// and the sum of exponentials kept together and rescaled when a larger value comes; the lanes' pairs are then
// merged.  Few tokens per workgroup and few loads per lane: the launch is short (a 65536 x 32 gate is 8 MB) and
// only gets up to the memory system's speed when many waves are in flight.
constexpr int kSub = 4;                      // lanes per token
constexpr int kGradTokens = kTile / kSub;    // tokens per workgroup

// Maximum and sum of exponentials of a row WITHOUT the entries that carry a slot gradient: with those the sum would
// hide how far a selected probability is from 1 (1 - p = rest / sum loses every digit to rounding once the row is
// peaked; kept apart it is exact to a few ulp, and with it the gradient p (1 - p) dy of a saturated gate).
struct MaxSumRest {
  float top, sum;
  int skip1, skip2;
  __device__ __forceinline__ void operator()(float x, int j) {
    if (j == skip1 || j == skip2) return;
    if (x > top) {
      sum = sum * expf(top - x) + 1.f;   // top = -inf at first: exp(-inf) * 0 = 0
      top = x;
    } else {
      sum += expf(x - top);
    }
  }
};

// per-token scalars of a workgroup's tokens, in LDS
struct GateGradTile {
  int i1[kGradTokens], i2[kGradTokens];      // experts that receive a slot gradient (-1: none)
  // factor of the entry of expert i1 / i2 / of every other expert: the gradient with respect to that array entry
  // (probabilities), or what p[e] is multiplied with (logits: d_j (1 - p_j) - p_other d_other, and -sum_j p_j d_j)
  float c1[kGradTokens], c2[kGradTokens], rest[kGradTokens];
  float top[kGradTokens], inv[kGradTokens];  // logits: row maximum and 1 / sum_e exp(x - max)
};

template <int K, int GD>
__global__ __launch_bounds__(kTile) void encode_dgate_kernel(GateGradArgs a) {
  __shared__ GateGradTile sh;
  constexpr size_t gb = GD == LANCET_F32 ? 4 : 2;
  constexpr int V = 16 / gb;
  const int tid = threadIdx.x;
  const int first = blockIdx.x * kGradTokens;
  const int t = tid / kSub, sub = tid % kSub;
  const int s = min(first + t, a.S - 1);  // lanes past the batch repeat its last token (their result is not stored)
  // ---- kSub lanes per token ---------------------------------------------------------------------------------
  {
    const char* row = static_cast<const char*>(a.gate) + static_cast<size_t>(s) * a.E * gb;
    int e[2] = {-1, -1};
    float dy[2] = {0.f, 0.f}, raw[2] = {0.f, 0.f};
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const int x = a.idx[static_cast<size_t>(j) * a.S + s];
      if (x >= 0 && x < a.E) {
        e[j] = x;
        dy[j] = ld_gate(a.dy, static_cast<size_t>(j) * a.S + s, GD);
        if (K == 2 || a.is_logits) raw[j] = gate_at<GD>(row, x);  // top-1 on probabilities needs no gate
      }
    }
    float top = 0.f, inv = 1.f, rest = 0.f;  // rest: sum of exponentials of the entries without a slot gradient
    float g[2] = {raw[0], raw[1]};           // the two kept probabilities (0 for a dropped slot)
    if (a.is_logits) {
      MaxSumRest ms = {-INFINITY, 0.f, e[0], e[1]};
      if (a.vec) {
        const u32x4* r = reinterpret_cast<const u32x4*>(row);
        const int n = a.E / V;
        for (int g0 = sub; g0 < n; g0 += 2 * kSub) {  // two granules in flight per lane
          const u32x4 x0 = r[g0];
          const bool two = g0 + kSub < n;
          const u32x4 x1 = two ? r[g0 + kSub] : x0;
          walk_granule<GD>(x0, g0, ms);
          if (two) walk_granule<GD>(x1, g0 + kSub, ms);
        }
      } else {
        for (int j = sub; j < a.E; j += kSub) ms(gate_at<GD>(row, j), j);
      }
      // merge the kSub lanes' (max, sum) pairs: they are neighbours in the wave
#pragma unroll
      for (int o = 1; o < kSub; o <<= 1) {
        const float ot = __shfl_xor(ms.top, o, kWave), os = __shfl_xor(ms.sum, o, kWave);
        const float nt = fmaxf(ms.top, ot);
        // a lane that saw no value holds (-inf, 0): its term is 0 whatever the other maximum is
        ms.sum = (ms.sum > 0.f ? ms.sum * expf(ms.top - nt) : 0.f) + (os > 0.f ? os * expf(ot - nt) : 0.f);
        ms.top = nt;
      }
      top = ms.top;
      if (e[0] >= 0) top = fmaxf(top, raw[0]);
      if (e[1] >= 0) top = fmaxf(top, raw[1]);
      rest = ms.sum > 0.f ? ms.sum * expf(ms.top - top) : 0.f;
      g[0] = e[0] >= 0 ? expf(raw[0] - top) : 0.f;   // exponentials for now, probabilities below
      g[1] = e[1] >= 0 ? expf(raw[1] - top) : 0.f;
      inv = 1.f / (rest + g[0] + g[1]);              // a row has at least one entry, and the largest one adds 1
      rest *= inv;
      g[0] *= inv;
      g[1] *= inv;
    }
    float d[2] = {0.f, 0.f};
    if (K == 1) {
      d[0] = dy[0];
    } else {
      const float sum = g[0] + g[1];
      if (sum >= 1.1920929e-07f) {
        const float r = 1.f / (sum * sum);
        d[0] = (dy[0] - dy[1]) * g[1] * r;
        d[1] = (dy[1] - dy[0]) * g[0] * r;
      } else {  // the clamped denominator is a constant
        d[0] = dy[0] / 1.1920929e-07f;
        d[1] = dy[1] / 1.1920929e-07f;
      }
      if (e[0] < 0) d[0] = 0.f;
      if (e[1] < 0) d[1] = 0.f;
    }
    if (sub == 0) {
      sh.i1[t] = e[0];
      sh.i2[t] = e[1];
      sh.top[t] = top;
      sh.inv[t] = inv;
      if (a.is_logits) {  // 1 - p_1 = rest + p_2 and 1 - p_2 = rest + p_1: sums of positive terms
        sh.c1[t] = d[0] * (rest + g[1]) - g[1] * d[1];
        sh.c2[t] = d[1] * (rest + g[0]) - g[0] * d[0];
        sh.rest[t] = -(g[0] * d[0] + g[1] * d[1]);
      } else {
        sh.c1[t] = d[0];
        sh.c2[t] = d[1];
        sh.rest[t] = 0.f;
      }
    }
  }
  __syncthreads();
  // ---- the workgroup's block of the result, in memory order ---------------------------------------------------
  const int ntok = min(kGradTokens, a.S - first);
  const size_t base = static_cast<size_t>(first) * a.E;  // first element of the block
  auto value = [&](int tk, int ex, float x) -> float {
    float c = sh.rest[tk];
    if (ex == sh.i1[tk]) c = sh.c1[tk];
    if (K == 2 && ex == sh.i2[tk]) c = sh.c2[tk];
    if (!a.is_logits) return c;
    return expf(x - sh.top[tk]) * sh.inv[tk] * c;
  };
  if (a.vec) {
    const int gpr = a.E / V;  // granules per row
    const int n = ntok * gpr;
    const u32x4* src = reinterpret_cast<const u32x4*>(static_cast<const char*>(a.gate) + base * gb);
    u32x4* dst = reinterpret_cast<u32x4*>(static_cast<char*>(a.out) + base * gb);
    for (int q = tid; q < n; q += kTile) {
      const int tk = q / gpr;
      const int e0 = (q - tk * gpr) * V;
      u32x4 x = {0u, 0u, 0u, 0u};
      if (a.is_logits) x = src[q];
      u32x4 r;
      if (GD == LANCET_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] = __float_as_uint(value(tk, e0 + i, __uint_as_float(x[i])));
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float lo = value(tk, e0 + 2 * i, half_word<GD>(x[i] & 0xffffu));
          const float hi = value(tk, e0 + 2 * i + 1, half_word<GD>(x[i] >> 16));
          const uint32_t l = GD == LANCET_BF16 ? f32_to_bf16(lo) : f32_to_f16(lo);
          const uint32_t h = GD == LANCET_BF16 ? f32_to_bf16(hi) : f32_to_f16(hi);
          r[i] = (l & 0xffffu) | (h << 16);
        }
      }
      dst[q] = r;
    }
  } else {
    const int n = ntok * a.E;
    for (int q = tid; q < n; q += kTile) {
      const int tk = q / a.E;
      const int ex = q - tk * a.E;
      const float x = a.is_logits ? ld_gate(a.gate, base + q, GD) : 0.f;
      st_gate(a.out, base + q, value(tk, ex, x), GD);
    }
  }
}

hipError_t run_encode_dgate(const void* dy, const void* gate, const int32_t* idx, int S, int E, int K, bool is_logits,
                            int gate_dtype, void* out, hipStream_t st) {
  if (S == 0) return hipSuccess;
  GateGradArgs a;
  a.dy = dy;
  a.gate = gate;
  a.idx = idx;
  a.out = out;
  a.S = S;
  a.E = E;
  a.is_logits = is_logits;
  const int gb = gate_dtype == LANCET_F32 ? 4 : 2;
  a.vec = (static_cast<size_t>(E) * gb) % 16 == 0 && ((reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  const int blocks = (S + kGradTokens - 1) / kGradTokens;
  LANCET_GATE_SWITCH(gate_dtype,
    if (K == 1) encode_dgate_kernel<1, GD><<<blocks, kTile, 0, st>>>(a);
    else encode_dgate_kernel<2, GD><<<blocks, kTile, 0, st>>>(a))
  return hipGetLastError();
}

}  // namespace lancet
