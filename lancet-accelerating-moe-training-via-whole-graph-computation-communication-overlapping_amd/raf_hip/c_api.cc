// C bridge over the op layer, playing the part RAF's packed-function FFI plays for Python
// (RAF_REGISTER_GLOBAL): build a CallValues, run Declare, let the caller (the "executor")
// allocate outputs and workspaces, dispatch to an OpEnv, execute on a stream.  Exceptions of the
// op layer become a non-zero return code and a thread-local message.
#include <string.h>

#include <memory>
#include <string>
#include <vector>

#include "op.h"

using namespace raf;
using namespace raf::op;

namespace {

thread_local std::string g_last_error;

struct Call {
  CallValues cv;
  std::vector<std::vector<Value>*> tuple_stack;  // open tuples while arguments are pushed
  std::vector<std::unique_ptr<std::vector<Value>>> owned;
  std::vector<Tensor*> flat_out;                 // leaves of cv.out in order
  OpEnvPtr env;
  std::vector<void*> ws_storage;
};

void Push(Call* c, Value v) {
  if (!c->tuple_stack.empty()) c->tuple_stack.back()->push_back(std::move(v));
  else c->cv.args.push_back(std::move(v));
}

void Flatten(Value& v, std::vector<Tensor*>& out) {
  if (v.kind == Value::kTensor) out.push_back(&v.tensor);
  else if (v.kind == Value::kTuple)
    for (auto& f : v.fields) Flatten(f, out);
}

template <typename F>
int Guard(F&& f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    g_last_error = e.what();
    return 1;
  }
}

}  // namespace

extern "C" {

const char* raf_hip_last_error() { return g_last_error.c_str(); }

void* raf_hip_call_create(const char* op_name) {
  Call* c = new Call();
  c->cv.op_name = op_name;
  return c;
}
void raf_hip_call_destroy(void* h) { delete static_cast<Call*>(h); }

// dtype_code: DLPack codes (0 int, 1 uint, 2 float, 4 bfloat)
int raf_hip_push_tensor(void* h, void* data, int device_id, int dtype_code, int bits, int ndim, const int64_t* shape) {
  return Guard([&] {
    Tensor t;
    t.data = data;
    t.device_id = device_id;
    t.dtype.code = static_cast<DTypeCode>(dtype_code);
    t.dtype.bits = bits;
    t.shape.assign(shape, shape + ndim);
    Push(static_cast<Call*>(h), Value::MakeTensor(t));
  });
}
int raf_hip_push_int(void* h, int64_t v) { return Guard([&] { Push(static_cast<Call*>(h), Value::MakeInt(v)); }); }
int raf_hip_push_float(void* h, double v) { return Guard([&] { Push(static_cast<Call*>(h), Value::MakeFloat(v)); }); }
int raf_hip_push_bool(void* h, int v) { return Guard([&] { Push(static_cast<Call*>(h), Value::MakeBool(v != 0)); }); }
int raf_hip_begin_tuple(void* h) {
  return Guard([&] {
    Call* c = static_cast<Call*>(h);
    c->owned.emplace_back(new std::vector<Value>());
    c->tuple_stack.push_back(c->owned.back().get());
  });
}
int raf_hip_end_tuple(void* h) {
  return Guard([&] {
    Call* c = static_cast<Call*>(h);
    RAF_CHECK(!c->tuple_stack.empty(), "end_tuple without begin_tuple");
    std::vector<Value> fields = std::move(*c->tuple_stack.back());
    c->tuple_stack.pop_back();
    Push(c, Value::MakeTuple(std::move(fields)));
  });
}

// FRAFDeclare: fills the output description (shapes, dtypes) of the call
int raf_hip_declare(void* h) {
  return Guard([&] {
    Call* c = static_cast<Call*>(h);
    RunDeclare(c->cv);
    c->flat_out.clear();
    Flatten(c->cv.out, c->flat_out);
  });
}
int raf_hip_num_outputs(void* h) { return static_cast<int>(static_cast<Call*>(h)->flat_out.size()); }
int raf_hip_output_is_tuple(void* h) { return static_cast<Call*>(h)->cv.out.kind == Value::kTuple; }
// returns ndim; shape must hold 8 entries; data is the aliased input pointer for in-place outputs
int raf_hip_output_info(void* h, int i, int* dtype_code, int* bits, int64_t* shape, void** data) {
  Call* c = static_cast<Call*>(h);
  if (i < 0 || i >= static_cast<int>(c->flat_out.size())) return -1;
  const Tensor* t = c->flat_out[i];
  *dtype_code = static_cast<int>(t->dtype.code);
  *bits = t->dtype.bits;
  for (size_t d = 0; d < t->shape.size() && d < 8; ++d) shape[d] = t->shape[d];
  *data = t->data;
  return static_cast<int>(t->shape.size());
}
int raf_hip_set_output_data(void* h, int i, void* data) {
  return Guard([&] {
    Call* c = static_cast<Call*>(h);
    RAF_CHECK(i >= 0 && i < static_cast<int>(c->flat_out.size()), "output index out of range");
    c->flat_out[i]->data = data;
  });
}

// Dispatch(call): picks the dialect op by priority and constructs its OpEnv
int raf_hip_dispatch(void* h) {
  return Guard([&] {
    Call* c = static_cast<Call*>(h);
    c->env = Dispatch(c->cv);
    RAF_CHECK(c->env != nullptr, "dispatch returned no OpEnv");
  });
}
const char* raf_hip_env_name(void* h) {
  Call* c = static_cast<Call*>(h);
  static thread_local std::string name;
  name = c->env ? c->env->name() : "";
  return name.c_str();
}
int raf_hip_num_workspaces(void* h) {
  Call* c = static_cast<Call*>(h);
  return c->env ? static_cast<int>(c->env->GetRequests().size()) : 0;
}
int64_t raf_hip_workspace_bytes(void* h, int i) {
  Call* c = static_cast<Call*>(h);
  const auto& reqs = c->env->GetRequests();
  return (i >= 0 && i < static_cast<int>(reqs.size())) ? reqs[i].nbytes : -1;
}
int raf_hip_bind_workspace(void* h, int i, void* data) {
  return Guard([&] {
    Call* c = static_cast<Call*>(h);
    const auto& reqs = c->env->GetRequests();
    RAF_CHECK(i >= 0 && i < static_cast<int>(reqs.size()), "workspace index out of range");
    *reqs[i].dest = data;
    c->env->WorkspaceBound();
  });
}
int raf_hip_num_arg_indices(void* h) { return static_cast<int>(static_cast<Call*>(h)->env->arg_indices.size()); }
int raf_hip_arg_index(void* h, int i) { return static_cast<Call*>(h)->env->arg_indices[i]; }

void raf_hip_set_stream(int device_id, void* stream) { OpEnv::SetStreamForAllBackends(device_id, stream); }

int raf_hip_execute(void* h) {
  return Guard([&] {
    Call* c = static_cast<Call*>(h);
    RAF_CHECK(c->env != nullptr, "dispatch the call before executing it");
    c->env->Execute(c->cv);
  });
}

// the executor has synchronised (or is about to): failures the device recorded become an error here
int raf_hip_check_device_status(void* h) {
  return Guard([&] {
    Call* c = static_cast<Call*>(h);
    RAF_CHECK(c->env != nullptr, "dispatch the call before checking it");
    c->env->CheckDeviceStatus(OpEnv::GetStream(c->cv.device_id));
  });
}

// dialect preference scope + registry queries
int raf_hip_push_dialect_preference(const char* comma_separated) {
  return Guard([&] {
    std::vector<std::string> names;
    std::string cur;
    for (const char* p = comma_separated; *p; ++p) {
      if (*p == ',') {
        if (!cur.empty()) names.push_back(cur);
        cur.clear();
      } else {
        cur.push_back(*p);
      }
    }
    if (!cur.empty()) names.push_back(cur);
    DialectPreference(names).EnterWithScope();
  });
}
int raf_hip_pop_dialect_preference() {
  return Guard([&] { DialectPreference({}).ExitWithScope(); });
}
int raf_hip_num_registered_ops() { return static_cast<int>(ListRegisteredOps().size()); }
const char* raf_hip_registered_op(int i) {
  static thread_local std::string name;
  auto ops = ListRegisteredOps();
  name = (i >= 0 && i < static_cast<int>(ops.size())) ? ops[i] : "";
  return name.c_str();
}
const char* raf_hip_dispatch_list(const char* base_op) {
  static thread_local std::string s;
  s.clear();
  try {
    for (const auto& e : OpDialect::GetDispatchList(base_op, "hip"))
      s += e.dialect_op + ":" + std::to_string(e.plevel) + ";";
  } catch (const std::exception& e) {
    g_last_error = e.what();
  }
  return s.c_str();
}

}  // extern "C"
