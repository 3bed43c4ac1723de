/*
 * CPU restatement in plain C (OpenMP) of the reference's MoE dispatch ops and LANS step.
 *
 * TEST INFRASTRUCTURE ONLY: this is the checker and the timed CPU baseline, never a code
 * path of the product.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg load the library built from this file.
 *
 * The parallel structure follows the reference's kernels: the position scan runs one expert
 * per thread, each walking all tokens (gen_location_kernel has one block per expert,
 * src/op/dialect/cuda/kernels/tutel_moe_dispatch.cu:164-212); row moves run one token per
 * iteration (encode/decode kernels, :39-81); LANS runs the reference's sweeps per tensor
 * (multi_tensor_lans.cu:401-450).  It is cross-checked against the NumPy oracle
 * (oracle/moe_oracle.py, oracle/lans_oracle.py) in tests/test_oracle_c.py; what pins the NumPy
 * oracle is listed in its header.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void oracle_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ---- A0/A1/A2: selection on the array given; softmax value when the array holds logits
 * (src/op/dialect/cuda/moe.cc:177-250; docker/resources/sharded_moe.py:270-278) ---------- */
void oracle_select_topk(const float* gate, int64_t S, int E, int k, int is_logits, int32_t* idx,
                        float* val) {
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < S; ++s) {
    const float* row = gate + s * E;
    int i1 = 0, i2 = -1;
    for (int j = 1; j < E; ++j)
      if (row[j] > row[i1]) i1 = j;
    if (k == 2) {
      for (int j = 0; j < E; ++j) {
        if (j == i1) continue;
        if (i2 < 0 || row[j] > row[i2]) i2 = j;
      }
    }
    float sum = 1.0f;
    if (is_logits) {
      sum = 0.0f;
      for (int j = 0; j < E; ++j) sum += expf(row[j] - row[i1]);
    }
    idx[s] = i1;
    val[s] = is_logits ? expf(row[i1] - row[i1]) / sum : row[i1];
    if (k == 2) {
      idx[S + s] = i2;
      val[S + s] = is_logits ? expf(row[i2] - row[i1]) / sum : row[i2];
    }
  }
}

/* ---- A3: gen_location (tutel_moe_dispatch.cu:164-212): one expert per thread ------------- */
void oracle_gen_location(int32_t* idx, const int32_t* used_in, int32_t* loc, int32_t* used_out,
                         uint64_t* elems, int64_t S, int E, int C, int64_t M) {
#pragma omp parallel for schedule(dynamic, 1)
  for (int e = 0; e < E; ++e) {
    const int in = used_in ? used_in[e] : 0;
    int64_t cnt = 0;
    for (int64_t s = 0; s < S; ++s) {
      if (idx[s] != e) continue;
      loc[s] = (int32_t)cnt;                    /* :198 */
      if (cnt >= (int64_t)C - in) idx[s] = -1;  /* :199-201 */
      ++cnt;
    }
    int64_t out = in + cnt;                     /* :207-209 */
    if (out > C) out = C;
    used_out[e] = (int32_t)out;
    elems[e] = (uint64_t)((out - in) * M);      /* :210 */
  }
}

/* ---- A4: encode_forward (:61-81, :461-484): zero, then one row copy per kept token ------- */
void oracle_scatter_rows(const void* data, void* out, const int32_t* idx, const int32_t* loc,
                         int64_t S, int64_t M, int E, int C, int elem_bytes) {
  const size_t row = (size_t)M * elem_bytes;
  memset(out, 0, (size_t)E * C * row);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < S; ++s) {
    const int e = idx[s], l = loc[s];
    if (e >= 0 && e < E && l >= 0 && l < C)
      memcpy((char*)out + ((size_t)e * C + l) * row, (const char*)data + (size_t)s * row, row);
  }
}

/* ---- A.3 merge_masks for two partitions that share one [2, 2S] output (top-2 layout) ----- */
static void merge_two(const int32_t* i1, const int32_t* l1, const int32_t* i2, const int32_t* l2,
                      int64_t S, int E, int32_t* out_idx, int32_t* out_loc) {
  int64_t* kept1 = (int64_t*)calloc((size_t)E, sizeof(int64_t));
  for (int64_t s = 0; s < S; ++s)
    if (i1[s] >= 0) kept1[i1[s]]++;
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < S; ++s) {
    out_idx[s] = i1[s] >= 0 ? i1[s] : -1;
    out_loc[s] = i1[s] >= 0 ? l1[s] : -1;
    out_idx[S + s] = i2[s] >= 0 ? i2[s] : -1;
    out_loc[S + s] = i2[s] >= 0 ? l2[s] + (int32_t)kept1[i2[s]] : -1;
  }
  free(kept1);
}

static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

/* ---- A.1 / A.6: moe_encode, top-1 (reference op) or top-2 (two chained top-1 encodes, merged).
 * dtype: 0 = fp32 rows, 1 = bf16 rows.  Outputs as in src/op/declare/moe.cc:48-58, slot-major
 * for k = 2.  Returns 0, or -1 when scratch memory cannot be allocated. ------------------- */
int oracle_moe_encode(const void* data, const float* gate, const int32_t* used_in, int64_t S,
                      int64_t M, int E, int C, int k, int dtype, int is_logits, float* gates_s,
                      int32_t* indloc, int32_t* used_out, uint64_t* elems, void* dispatched) {
  const int eb = dtype == 0 ? 4 : 2;
  int32_t* idx = indloc;
  int32_t* loc = indloc + (size_t)k * S;
  oracle_select_topk(gate, S, E, k, is_logits, idx, gates_s);
  if (k == 1) {
    oracle_gen_location(idx, used_in, loc, used_out, elems, S, E, C, M);
    oracle_scatter_rows(data, dispatched, idx, loc, S, M, E, C, eb);
    return 0;
  }
  int32_t* used1 = (int32_t*)malloc((size_t)E * sizeof(int32_t));
  uint64_t* el = (uint64_t*)malloc((size_t)E * sizeof(uint64_t));
  int32_t* tmp = (int32_t*)malloc((size_t)4 * S * sizeof(int32_t));
  if (!used1 || !el || !tmp) {
    free(used1), free(el), free(tmp);
    return -1;
  }
  int32_t *i1 = tmp, *l1 = tmp + S, *i2 = tmp + 2 * S, *l2 = tmp + 3 * S;
  memcpy(i1, idx, (size_t)S * 4);
  memcpy(i2, idx + S, (size_t)S * 4);
  oracle_gen_location(i1, used_in, l1, used1, el, S, E, C, M);
  oracle_gen_location(i2, used1, l2, used_out, el, S, E, C, M);
  merge_two(i1, l1, i2, l2, S, E, idx, loc);
  for (int e = 0; e < E; ++e)
    elems[e] = (uint64_t)(((int64_t)used_out[e] - (used_in ? used_in[e] : 0)) * M);
  /* combine weights after the drop (sharded_moe.py:296-312) */
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < S; ++s) {
    const float g1 = idx[s] >= 0 ? gates_s[s] : 0.0f;
    const float g2 = idx[S + s] >= 0 ? gates_s[S + s] : 0.0f;
    float den = g1 + g2;
    if (den < 1.1920929e-07f) den = 1.1920929e-07f;
    gates_s[s] = g1 / den;
    gates_s[S + s] = g2 / den;
  }
  /* rows: both slots read the same token rows */
  const size_t row = (size_t)M * eb;
  memset(dispatched, 0, (size_t)E * C * row);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < S; ++s) {
    for (int j = 0; j < 2; ++j) {
      const int e = idx[(size_t)j * S + s], l = loc[(size_t)j * S + s];
      if (e >= 0 && e < E && l >= 0 && l < C)
        memcpy((char*)dispatched + ((size_t)e * C + l) * row, (const char*)data + (size_t)s * row, row);
    }
  }
  free(used1), free(el), free(tmp);
  return 0;
}

/* ---- A.5: moe_decode (tutel_moe_dispatch.cu:46-55,110-116), k slots summed in fp32 -------- */
void oracle_moe_decode(const void* expert_out, const float* gates_s, const int32_t* indloc, int64_t S,
                       int64_t M, int E, int C, int k, int dtype, void* out) {
  const int32_t* idx = indloc;
  const int32_t* loc = indloc + (size_t)k * S;
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < S; ++s) {
    for (int64_t i = 0; i < M; ++i) {
      float acc = 0.0f;
      for (int j = 0; j < k; ++j) {
        const int e = idx[(size_t)j * S + s], l = loc[(size_t)j * S + s];
        float term = 0.0f;
        if (e >= 0 && e < E && l >= 0 && l < C) {
          const size_t at = ((size_t)e * C + l) * M + i;
          const float x = dtype == 0 ? ((const float*)expert_out)[at]
                                     : bf16_to_f32(((const uint16_t*)expert_out)[at]);
          term = gates_s[(size_t)j * S + s] * x;
        }
        acc = j == 0 ? term : acc + term;
      }
      if (dtype == 0) ((float*)out)[s * M + i] = acc;
      else ((uint16_t*)out)[s * M + i] = f32_to_bf16(acc);
    }
  }
}

/* ---- L1-L4: LANS (multi_tensor_lans.cu:95-450; lans.cc:92-148) ---------------------------- */
static float l2norm(const float* x, int64_t n) {
  double acc = 0.0;
#pragma omp parallel for reduction(+ : acc) schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    const float sq = x[i] * x[i];
    acc += (double)sq;
  }
  return (float)sqrt(acc);
}

/* In place on p, m, v; g untouched; `scratch` holds 2*max(numel) floats (the reference's q
 * workspace and its reuse of g for u_m).  norms (optional) receives 4 floats per tensor. */
void oracle_lans_step(float* const* g, float* const* p, float* const* m, float* const* v,
                      const int64_t* numels, int T, int step, float lr, float beta1, float beta2,
                      float eps, int bias_correction, float wd, int grad_averaging, int mode,
                      int normalize_grad, float* scratch, float* norms) {
  float bc1 = 1.0f, bc2 = 1.0f;
  if (bias_correction) {
    bc1 = (float)(1.0 - pow((double)beta1, step));
    bc2 = (float)(1.0 - pow((double)beta2, step));
  }
  const float beta3 = grad_averaging ? 1.0f - beta1 : 1.0f;
  const float omb2 = 1.0f - beta2;
  for (int t = 0; t < T; ++t) {
    const int64_t n = numels[t];
    const float gn = l2norm(g[t], n), pn = l2norm(p[t], n);
    float* um = scratch;
    float* ug = scratch + n;
    const float* gt = g[t];
    float *pt = p[t], *mt = m[t], *vt = v[t];
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
      float sg = gt[i];
      if (normalize_grad && gn != 0.0f) sg = sg / (gn + eps);
      const float rp = wd == 0.0f ? 0.0f : pt[i];
      if (mode == 0) sg = sg + wd * rp;
      const float mm = mt[i] * beta1 + beta3 * sg;
      const float vv = vt[i] * beta2 + omb2 * sg * sg;
      const float denom = sqrtf(vv / bc2) + eps;
      float a = (mm / bc1) / denom, b = sg / denom;
      if (mode != 0) {
        const float sp = wd * rp;
        a = a + sp;
        b = b + sp;
      }
      mt[i] = mm;
      vt[i] = vv;
      um[i] = a;
      ug[i] = b;
    }
    const float umn = l2norm(um, n), ugn = l2norm(ug, n);
    float rm = (umn != 0.0f && pn != 0.0f) ? lr * (pn / umn) : lr;
    float rg = (ugn != 0.0f && pn != 0.0f) ? lr * (pn / ugn) : lr;
    rm *= beta1;
    rg *= beta3;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) pt[i] = pt[i] - (rm * um[i]) - (rg * ug[i]);
    if (norms) {
      norms[4 * t] = gn, norms[4 * t + 1] = pn, norms[4 * t + 2] = umn, norms[4 * t + 3] = ugn;
    }
  }
}
