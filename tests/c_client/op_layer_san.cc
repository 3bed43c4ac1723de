// Sanitizer run of the C++ op layer (raf_hip/) on host memory (TEST INFRASTRUCTURE): plays the executor for every
// operator of the hip dialect - push arguments, Declare, allocate exactly what Declare describes, Dispatch, bind
// exactly the workspace the OpEnv requested, Execute - against lancet_hip_host_stub.c, whose "launches" touch every
// byte the real kernels touch.  Built with -fsanitize=address,undefined: a wrong shape, dtype or size anywhere in the
// op layer is a sanitizer report and a non-zero exit.  Counterpart of the reference's sanitizer build of its host
// code (cmake/modules/Sanitizer.cmake:13-40).  Usage: ./op_layer_san  (prints one line per operator).
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

extern "C" {
const char* raf_hip_last_error();
void* raf_hip_call_create(const char* op_name);
void raf_hip_call_destroy(void* h);
int raf_hip_push_tensor(void* h, void* data, int device_id, int dtype_code, int bits, int ndim, const int64_t* shape);
int raf_hip_push_int(void* h, int64_t v);
int raf_hip_push_float(void* h, double v);
int raf_hip_push_bool(void* h, int v);
int raf_hip_begin_tuple(void* h);
int raf_hip_end_tuple(void* h);
int raf_hip_declare(void* h);
int raf_hip_num_outputs(void* h);
int raf_hip_output_info(void* h, int i, int* dtype_code, int* bits, int64_t* shape, void** data);
int raf_hip_set_output_data(void* h, int i, void* data);
int raf_hip_dispatch(void* h);
const char* raf_hip_env_name(void* h);
int raf_hip_num_workspaces(void* h);
int64_t raf_hip_workspace_bytes(void* h, int i);
int raf_hip_bind_workspace(void* h, int i, void* data);
int raf_hip_execute(void* h);
int raf_hip_check_device_status(void* h);
}

namespace {

enum { kInt = 0, kUInt = 1, kFloat = 2, kBFloat = 4 };  // DLPack codes

struct Arena {  // every buffer is its own heap block of exactly the bytes asked for, so that overruns are seen
  std::vector<void*> blocks;
  void* get(size_t n) {
    void* p = malloc(n ? n : 1);
    memset(p, 0, n);
    blocks.push_back(p);
    return p;
  }
  ~Arena() {
    for (void* p : blocks) free(p);
  }
};

int g_failures = 0;

#define MUST(call)                                                                   \
  do {                                                                               \
    if ((call) != 0) {                                                               \
      fprintf(stderr, "%s:%d: %s failed: %s\n", __FILE__, __LINE__, #call, raf_hip_last_error()); \
      ++g_failures;                                                                  \
      return;                                                                        \
    }                                                                                \
  } while (0)

void tensor(void* h, Arena& a, int code, int bits, std::vector<int64_t> shape) {
  size_t n = bits / 8;
  for (int64_t d : shape) n *= static_cast<size_t>(d);
  if (raf_hip_push_tensor(h, a.get(n), 0, code, bits, static_cast<int>(shape.size()), shape.data()) != 0) ++g_failures;
}

// Declare ... Execute, twice (the second Execute runs on a workspace that is already set up), then a re-bind
void run(void* h, Arena& a, const char* what) {
  MUST(raf_hip_declare(h));
  for (int i = 0; i < raf_hip_num_outputs(h); ++i) {
    int code, bits;
    int64_t shape[8];
    void* data = nullptr;
    const int nd = raf_hip_output_info(h, i, &code, &bits, shape, &data);
    if (data) continue;  // in-place output: aliases an input
    size_t n = bits / 8;
    for (int d = 0; d < nd; ++d) n *= static_cast<size_t>(shape[d]);
    MUST(raf_hip_set_output_data(h, i, a.get(n)));
  }
  MUST(raf_hip_dispatch(h));
  for (int rebind = 0; rebind < 2; ++rebind) {
    for (int i = 0; i < raf_hip_num_workspaces(h); ++i)
      MUST(raf_hip_bind_workspace(h, i, a.get(static_cast<size_t>(raf_hip_workspace_bytes(h, i)))));
    MUST(raf_hip_execute(h));
    MUST(raf_hip_execute(h));
    MUST(raf_hip_check_device_status(h));
  }
  printf("ok   %-40s %s\n", raf_hip_env_name(h), what);
}

void expect_rejected(void* h, const char* what) {
  if (raf_hip_declare(h) == 0 && raf_hip_dispatch(h) == 0) {
    fprintf(stderr, "%s: accepted, should have been rejected\n", what);
    ++g_failures;
  } else {
    printf("ok   rejected: %s (%s)\n", what, raf_hip_last_error());
  }
}

struct CallH {
  void* h;
  explicit CallH(const char* op) : h(raf_hip_call_create(op)) {}
  ~CallH() { raf_hip_call_destroy(h); }
};

void all_ops() {
  const int64_t S = 300, M = 40, E = 6;  // E does not divide S; rows of 40 elements
  for (int gate_bits : {32, 16}) {
    for (int k : {1, 2}) {
      Arena a;
      CallH c("raf.op.moe_encode");
      tensor(c.h, a, kBFloat, 16, {S, M});
      tensor(c.h, a, gate_bits == 32 ? kFloat : kBFloat, gate_bits, {S, E});
      tensor(c.h, a, kInt, 32, {E});
      raf_hip_push_float(c.h, 1.25);
      raf_hip_push_int(c.h, k);
      raf_hip_push_int(c.h, 1);  // gate_is_logits
      raf_hip_push_int(c.h, 1);  // zero_tail
      if (k == 2) tensor(c.h, a, gate_bits == 32 ? kFloat : kBFloat, gate_bits, {S, E});  // gate2_noise
      run(c.h, a, k == 2 ? "top-2 with noise" : "top-1");
    }
  }
  {
    Arena a;
    CallH c("raf.op.moe_encode_batch_prioritized");
    tensor(c.h, a, kFloat, 16, {S, M});
    tensor(c.h, a, kFloat, 16, {S, E});
    raf_hip_push_int(c.h, 3);
    raf_hip_push_int(c.h, 2);
    raf_hip_push_float(c.h, 3.0);
    run(c.h, a, "3 partitions, fp16 rows and gate");
  }
  const int64_t C = 70, P = 3;
  {
    Arena a;
    CallH c("raf.op.moe_merge_masks");
    raf_hip_begin_tuple(c.h);
    for (int p = 0; p < P; ++p) tensor(c.h, a, kInt, 32, {2, S});
    raf_hip_end_tuple(c.h);
    raf_hip_push_int(c.h, E);
    run(c.h, a, "3 masks");
  }
  {
    Arena a;
    CallH c("raf.op.moe_redispatch");
    raf_hip_begin_tuple(c.h);
    for (int p = 0; p < P; ++p) tensor(c.h, a, kFloat, 32, {E, C, M});
    raf_hip_end_tuple(c.h);
    raf_hip_begin_tuple(c.h);
    for (int p = 0; p < P; ++p) tensor(c.h, a, kInt, 32, {2, S});
    raf_hip_end_tuple(c.h);
    run(c.h, a, "3 buffers");
  }
  for (int k : {1, 2}) {
    Arena a;
    CallH c("raf.op.moe_decode");
    tensor(c.h, a, kBFloat, 16, {E, C, M});
    tensor(c.h, a, kBFloat, 16, {k * S});
    tensor(c.h, a, kInt, 32, {2, k * S});
    raf_hip_push_int(c.h, k);
    run(c.h, a, k == 2 ? "top-2, bf16 gate" : "top-1, bf16 gate");
  }
  {
    Arena a;
    const int64_t G = 4, LE = 2;
    CallH c("raf.op.moe_redispatch_expert_input");
    raf_hip_begin_tuple(c.h);
    for (int p = 0; p < P; ++p) tensor(c.h, a, kBFloat, 16, {C, G, M});
    raf_hip_end_tuple(c.h);
    raf_hip_begin_tuple(c.h);
    for (int p = 0; p < P; ++p) tensor(c.h, a, kUInt, 64, {G * LE});
    raf_hip_end_tuple(c.h);
    raf_hip_push_int(c.h, 1);
    raf_hip_push_int(c.h, LE);
    run(c.h, a, "3 partitions, 4 source ranks");
  }
  for (int k : {1, 2}) {
    {
      Arena a;
      CallH c("raf.op.moe_encode_dx");
      tensor(c.h, a, kFloat, 32, {E, C, M});
      tensor(c.h, a, kInt, 32, {2, k * S});
      raf_hip_push_int(c.h, k);
      run(c.h, a, "");
    }
    {
      Arena a;
      CallH c("raf.op.moe_encode_dg");
      tensor(c.h, a, kFloat, 16, {k * S});
      tensor(c.h, a, kInt, 32, {2, k * S});
      raf_hip_push_int(c.h, E);
      raf_hip_push_int(c.h, k);
      run(c.h, a, "fp16 gradient");
    }
    {
      Arena a;
      CallH c("raf.op.moe_decode_dx");
      tensor(c.h, a, kBFloat, 16, {S, M});
      tensor(c.h, a, kFloat, 32, {k * S});
      tensor(c.h, a, kInt, 32, {2, k * S});
      raf_hip_push_int(c.h, E);
      raf_hip_push_int(c.h, C);
      raf_hip_push_int(c.h, k);
      run(c.h, a, "");
    }
    for (int gd : {0, 1, 2}) {
      Arena a;
      CallH c("raf.op.moe_decode_dg");
      tensor(c.h, a, kBFloat, 16, {S, M});
      tensor(c.h, a, kBFloat, 16, {E, C, M});
      tensor(c.h, a, kInt, 32, {2, k * S});
      raf_hip_push_int(c.h, k);
      raf_hip_push_int(c.h, gd);
      run(c.h, a, "gate gradient in each gate dtype");
    }
  }
  {
    Arena a;
    CallH c("raf.op.lans");
    const std::vector<std::vector<int64_t>> shapes = {{17, 5}, {129}, {1}, {64, 3}};
    raf_hip_begin_tuple(c.h);
    for (int q = 0; q < 4; ++q)
      for (const auto& s : shapes) tensor(c.h, a, kFloat, 32, s);
    raf_hip_end_tuple(c.h);
    tensor(c.h, a, kFloat, 32, {});  // the step as a 0-dim tensor, as the reference passes it
    raf_hip_push_float(c.h, 1e-3), raf_hip_push_float(c.h, 0.9), raf_hip_push_float(c.h, 0.999), raf_hip_push_float(c.h, 1e-6);
    raf_hip_push_int(c.h, 1), raf_hip_push_float(c.h, 0.01), raf_hip_push_int(c.h, 1), raf_hip_push_int(c.h, 1);
    raf_hip_push_bool(c.h, 1);
    run(c.h, a, "4 tensors, step tensor");
  }
  for (int g_bits : {32, 16}) {  // a 16-bit model: 16-bit gradients in, 16-bit copies of the new parameters out
    Arena a;
    CallH c("raf.op.lans");
    const std::vector<std::vector<int64_t>> shapes = {{17, 5}, {129}, {8192}};
    raf_hip_begin_tuple(c.h);
    for (int q = 0; q < 4; ++q)
      for (const auto& s : shapes) tensor(c.h, a, q == 0 && g_bits == 16 ? kBFloat : kFloat, q == 0 ? g_bits : 32, s);
    raf_hip_end_tuple(c.h);
    raf_hip_push_int(c.h, 3);
    raf_hip_push_float(c.h, 1e-3), raf_hip_push_float(c.h, 0.9), raf_hip_push_float(c.h, 0.999), raf_hip_push_float(c.h, 1e-6);
    raf_hip_push_int(c.h, 1), raf_hip_push_float(c.h, 0.01), raf_hip_push_int(c.h, 1), raf_hip_push_int(c.h, 1);
    raf_hip_push_bool(c.h, 1);
    raf_hip_begin_tuple(c.h);
    for (const auto& s : shapes) tensor(c.h, a, kBFloat, 16, s);
    raf_hip_end_tuple(c.h);
    run(c.h, a, g_bits == 16 ? "bf16 gradients, bf16 parameter copies" : "fp32 gradients, bf16 parameter copies");
  }
  // the routed-once form of the partitioned dispatch: one routing of the whole batch, per-partition row movement
  for (int k : {1, 2}) {
    const int64_t P = 3, Sp = S / P, C = 140 * k;
    {
      Arena a;
      CallH c("raf.op.moe_route");
      tensor(c.h, a, kFloat, 32, {S, E});
      tensor(c.h, a, kInt, 32, {E});
      raf_hip_push_int(c.h, M);
      raf_hip_push_float(c.h, 1.25);
      raf_hip_push_int(c.h, k);
      raf_hip_push_int(c.h, 1);
      run(c.h, a, k == 1 ? "top-1 on few tiles: the stateful form, workspace set up" : "top-2: plain scratch");
    }
    {
      Arena a;
      CallH c("raf.op.moe_scatter_tokens");
      tensor(c.h, a, kBFloat, 16, {Sp, M});
      tensor(c.h, a, kInt, 32, {2, k * S});
      tensor(c.h, a, kInt, 32, {E});
      tensor(c.h, a, kInt, 32, {E});
      tensor(c.h, a, kBFloat, 16, {E, C, M});
      raf_hip_push_int(c.h, 2 * Sp);  // the last partition
      raf_hip_push_int(c.h, k);
      run(c.h, a, "in place on the shared buffer");
    }
    {
      Arena a;
      CallH c("raf.op.moe_decode_tokens");
      tensor(c.h, a, kBFloat, 16, {E, C, M});
      tensor(c.h, a, kFloat, 32, {k * S});
      tensor(c.h, a, kInt, 32, {2, k * S});
      raf_hip_push_int(c.h, 2 * Sp);
      raf_hip_push_int(c.h, Sp);
      raf_hip_push_int(c.h, k);
      run(c.h, a, "");
    }
    {
      Arena a;
      CallH c("raf.op.moe_partition_ranges");
      tensor(c.h, a, kInt, 32, {2, k * S});
      raf_hip_push_int(c.h, P), raf_hip_push_int(c.h, E), raf_hip_push_int(c.h, M), raf_hip_push_int(c.h, k);
      run(c.h, a, "");
    }
    for (int logits : {0, 1}) {
      Arena a;
      CallH c("raf.op.moe_encode_dgate");
      tensor(c.h, a, kBFloat, 16, {k * S});
      tensor(c.h, a, kBFloat, 16, {S, E});
      tensor(c.h, a, kInt, 32, {2, k * S});
      raf_hip_push_int(c.h, k);
      raf_hip_push_int(c.h, logits);
      run(c.h, a, "gate gradient through the normalisation / the softmax");
    }
  }
  {
    Arena a;
    CallH c("raf.op.moe_scatter_tokens");
    tensor(c.h, a, kFloat, 32, {100, 4});
    tensor(c.h, a, kInt, 32, {2, 300});
    tensor(c.h, a, kInt, 32, {6});
    tensor(c.h, a, kInt, 32, {6});
    tensor(c.h, a, kFloat, 32, {6, 50, 4});
    raf_hip_push_int(c.h, 250);
    expect_rejected(c.h, "token range past the routed batch");
  }
  // error paths: the message is built, the call object is destroyed with a half-built state
  {
    Arena a;
    CallH c("raf.op.moe_encode");
    tensor(c.h, a, kFloat, 32, {10, 4});
    tensor(c.h, a, kFloat, 32, {11, 2});
    tensor(c.h, a, kInt, 32, {2});
    expect_rejected(c.h, "data and gate disagree on the token count");
  }
  {
    Arena a;
    CallH c("raf.op.moe_encode");
    tensor(c.h, a, kFloat, 32, {10, 4});
    tensor(c.h, a, kInt, 32, {10, 2});  // an integer gate
    tensor(c.h, a, kInt, 32, {2});
    expect_rejected(c.h, "integer gate");
  }
  {
    Arena a;
    CallH c("raf.op.moe_decode_dg");
    tensor(c.h, a, kFloat, 32, {10, 4});
    tensor(c.h, a, kFloat, 32, {2, 5, 4});
    tensor(c.h, a, kInt, 32, {2, 10});
    raf_hip_push_int(c.h, 1);
    raf_hip_push_int(c.h, 7);
    expect_rejected(c.h, "unknown gate dtype code");
  }
  {
    CallH c("raf.op.not_an_op");
    expect_rejected(c.h, "unknown operator");
  }
}

}  // namespace

int main() {
  all_ops();
  if (g_failures) {
    fprintf(stderr, "%d failure(s)\n", g_failures);
    return 1;
  }
  printf("op layer: every operator ran under the sanitizers\n");
  return 0;
}
