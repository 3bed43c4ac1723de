// Op layer of the "hip" dialect: the vocabulary of RAF's operator/dialect layer
// (include/raf/op.h:55-135,326-332; include/raf/dialect.h:30-242; src/impl/op.cc:121-194;
// src/impl/dialect.cc:36-68) without TVM underneath, so that the six operators of the dispatch
// path register, dispatch and execute the way RAF's do: a base op ("raf.op.moe_encode") has a
// Declare function (output shapes/dtypes) and dialect ops ("raf.op.hip.moe_encode") with a
// priority level and an OpEnv maker; an executor declares, allocates outputs and workspaces,
// dispatches and calls Execute.
//
// Errors: the reference CHECK/LOG(FATAL)s; here every failed check throws raf::Error, which the
// C bridge (c_api.cc) turns into a status + message.
#pragma once
#include <stdint.h>

#include <functional>
#include <list>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace raf {

struct Error : public std::runtime_error {
  explicit Error(const std::string& what) : std::runtime_error(what) {}
};

#define RAF_CHECK(cond, msg)                                                        \
  do {                                                                              \
    if (!(cond)) throw ::raf::Error(std::string("Check failed: " #cond ": ") + msg); \
  } while (0)

// ---- values (the subset of raf::value the six ops use) ---------------------------------
enum class DTypeCode { kInt = 0, kUInt = 1, kFloat = 2, kBFloat = 4 };  // DLPack codes

struct DType {
  DTypeCode code = DTypeCode::kFloat;
  int bits = 32;
  bool operator==(const DType& o) const { return code == o.code && bits == o.bits; }
  int bytes() const { return bits / 8; }
};

// A tensor the executor owns: device pointer + shape (contiguous, row-major), like a DLTensor.
struct Tensor {
  void* data = nullptr;
  int device_id = 0;
  DType dtype;
  std::vector<int64_t> shape;
  int64_t numel() const {
    int64_t n = 1;
    for (auto d : shape) n *= d;
    return n;
  }
  int64_t nbytes() const { return numel() * dtype.bytes(); }
};

struct Value {
  enum Kind { kNone, kTensor, kInt, kFloat, kBool, kTuple } kind = kNone;
  Tensor tensor;
  int64_t i = 0;
  double f = 0.0;
  std::vector<Value> fields;

  static Value MakeTensor(const Tensor& t) {
    Value v;
    v.kind = kTensor;
    v.tensor = t;
    return v;
  }
  static Value MakeInt(int64_t x) {
    Value v;
    v.kind = kInt;
    v.i = x;
    return v;
  }
  static Value MakeFloat(double x) {
    Value v;
    v.kind = kFloat;
    v.f = x;
    return v;
  }
  static Value MakeBool(bool x) {
    Value v;
    v.kind = kBool;
    v.i = x;
    return v;
  }
  static Value MakeTuple(std::vector<Value> f) {
    Value v;
    v.kind = kTuple;
    v.fields = std::move(f);
    return v;
  }
  const Tensor& AsTensor() const {
    RAF_CHECK(kind == kTensor, "expected a tensor value");
    return tensor;
  }
  int64_t AsInt() const {
    RAF_CHECK(kind == kInt || kind == kBool, "expected an integer value");
    return i;
  }
  double AsFloat() const {
    RAF_CHECK(kind == kFloat || kind == kInt, "expected a float value");
    return kind == kFloat ? f : static_cast<double>(i);
  }
  const std::vector<Value>& AsTuple() const {
    RAF_CHECK(kind == kTuple, "expected a tuple value");
    return fields;
  }
};

// include/raf/op.h:36-53: callee + args + out + device.  `args` are positional, in the order of
// the op's schema (scripts/src_codegen/def_schema.py); trailing defaulted args may be omitted.
struct CallValues {
  std::string op_name;  // base op, e.g. "raf.op.moe_encode"
  std::vector<Value> args;
  Value out;            // filled by Declare (shapes) and then by the executor (pointers)
  int device_id = 0;
};

namespace op {

// ---- requests (src/requests.h): what an OpEnv asks the executor for -----------------------
struct WorkspaceRequest {
  void** dest;
  int device_id;
  int64_t nbytes;
};

// ---- OpEnv (include/raf/op.h:55-91) ---------------------------------------------------------
class OpEnv {
 public:
  virtual ~OpEnv() = default;
  virtual std::string name() const = 0;
  virtual void Execute(const CallValues& call) = 0;
  virtual void Execute(const std::vector<Value>& inputs, Value output) = 0;

  void RequestWorkspace(void** dest, int device_id, int64_t nbytes) {
    workspace_.push_back({dest, device_id, nbytes});
  }
  const std::vector<WorkspaceRequest>& GetRequests() const { return workspace_; }
  // Called by the executor after it has written a request's destination: the memory behind a workspace is
  // new (or has been used by others since the last Execute), whatever its address.
  virtual void WorkspaceBound() {}
  // Called by the executor where it waits for the device anyway (after a run, at a synchronisation point of
  // the schedule): throws if the device recorded a failure in work this OpEnv launched.  The reference aborts the
  // process on any failure (src/common/cuda_utils.h:18-22); here failures that only show on the device (a
  // bounded wait that gave up) mark the outputs at once and are reported here.  Synchronises `stream`.
  virtual void CheckDeviceStatus(void* stream) { (void)stream; }

  // Data input indices in the argument list (used by the VM executor).
  std::vector<int> arg_indices;

  // The stream kernels are launched on: the executor's current stream
  // (DeviceAPI::GetStream(), include/raf/device_api.h:107-114).
  static void SetStreamForAllBackends(int device_id, void* stream);
  static void* GetStream(int device_id);

 private:
  std::vector<WorkspaceRequest> workspace_;
};

using OpEnvPtr = std::shared_ptr<OpEnv>;
using FRAFDeclare = std::function<void(CallValues&)>;
using FMakeOpEnv = std::function<OpEnv*(const CallValues&)>;

// ---- registries (dmlc::Registry in the reference) ---------------------------------------------
class OpEnvMaker {
 public:
  OpEnvMaker& set_name(const std::string& n) {
    name = n;
    return *this;
  }
  OpEnvMaker& set_func(FMakeOpEnv f) {
    func_ = std::move(f);
    return *this;
  }
  OpEnv* operator()(const CallValues& call) const {
    RAF_CHECK(func_ != nullptr, "no maker registered for " + name);
    return func_(call);
  }
  static OpEnvMaker& RegisterOrGet(const std::string& op_name);
  static const OpEnvMaker* Get(const std::string& op_name);
  static OpEnvPtr Make(const std::string& op_name, const CallValues& call);
  std::string name;

 private:
  FMakeOpEnv func_ = nullptr;
};

class Dialect {
 public:
  Dialect& set_name(const std::string& n) {
    name = n;
    return *this;
  }
  Dialect& set_enable(const std::string& device_type) {
    enable_devices_.push_back(device_type);
    return *this;
  }
  bool is_enabled(const std::string& device_type) const;
  static Dialect& RegisterOrGet(const std::string& dialect_name);
  static const Dialect* Get(const std::string& dialect_name);
  static bool IsEnabled(const std::string& dialect, const std::string& device_type);
  static std::vector<std::string> GetEnabledDialects(const std::string& device_type);
  std::string name;

 private:
  std::vector<std::string> enable_devices_;
};

class OpDialect {
 public:
  struct DialectOpEntry {
    std::string dialect;
    std::string dialect_op;
    int plevel;
  };
  OpDialect& set_name(const std::string& n) {
    name = n;
    return *this;
  }
  // kept sorted by descending plevel (src/impl/dialect.cc add_dialect)
  OpDialect& add_dialect(const std::string& dialect, const std::string& dialect_op, int plevel);
  static OpDialect& RegisterOrGet(const std::string& base_op);
  static const OpDialect* Get(const std::string& base_op);
  // dialect ops of a base op enabled for the device type, highest priority first
  static std::vector<DialectOpEntry> GetDispatchList(const std::string& base_op, const std::string& device_type);
  std::string name;

 private:
  std::list<DialectOpEntry> entries_;
};

class OpDeclare {
 public:
  static void Register(const std::string& base_op, FRAFDeclare f);
  static const FRAFDeclare* Get(const std::string& base_op);
};

// Thread-local dialect preference stack (include/raf/dialect.h:30-60, src/impl/dialect.cc:36-68).
class DialectPreference {
 public:
  explicit DialectPreference(std::vector<std::string> dialects) : dialects_(std::move(dialects)) {}
  void EnterWithScope();
  void ExitWithScope();
  static const DialectPreference* Current();
  const std::vector<std::string>& dialects() const { return dialects_; }

 private:
  std::vector<std::string> dialects_;
};

// src/impl/op.cc:130-194: run Declare, then try the op's own maker, else the dialect ops by
// descending priority (restricted/ordered by the current DialectPreference); a maker that returns
// nullptr declines and the next one is tried.
void RunDeclare(CallValues& call);
OpEnvPtr Dispatch(const CallValues& call);
std::vector<std::string> ListRegisteredOps();

}  // namespace op
}  // namespace raf

// ---- registration macros (include/raf/op.h:326-332, include/raf/dialect.h:220-242) -------------
#define RAF_STR_CONCAT_(a, b) a##b
#define RAF_STR_CONCAT(a, b) RAF_STR_CONCAT_(a, b)
#define RAF_STRINGIZE_(S) #S
#define RAF_BASE_OP_NAME(NAME) RAF_STRINGIZE_(raf.op.NAME)
#define RAF_DIALECT_OP_NAME(DIALECT, NAME) RAF_STRINGIZE_(raf.op.DIALECT.NAME)

#define RAF_REGISTER_DIALECT(DIALECT_NAME)                                                 \
  static ::raf::op::Dialect& RAF_STR_CONCAT(__make_Dialect, __COUNTER__) __attribute__((unused)) = \
      ::raf::op::Dialect::RegisterOrGet(DIALECT_NAME).set_name(DIALECT_NAME)

#define RAF_REGISTER_DIALECT_OP(DIALECT, OP, PLEVEL)                                            \
  static ::raf::op::OpDialect& RAF_STR_CONCAT(__make_OpDialect, __COUNTER__) __attribute__((unused)) = \
      ::raf::op::OpDialect::RegisterOrGet(RAF_BASE_OP_NAME(OP))                                  \
          .set_name(RAF_BASE_OP_NAME(OP))                                                        \
          .add_dialect(#DIALECT, RAF_DIALECT_OP_NAME(DIALECT, OP), PLEVEL)

#define RAF_OP_ENV_MAKER(OP_NAME, FOP_ENV_MAKER)                                                  \
  static ::raf::op::OpEnvMaker& RAF_STR_CONCAT(__make_OpEnvMaker, __COUNTER__) __attribute__((unused)) = \
      ::raf::op::OpEnvMaker::RegisterOrGet(OP_NAME).set_name(OP_NAME).set_func(FOP_ENV_MAKER)

#define RAF_OP_DECLARE(OP_NAME, BODY)                                                      \
  static int RAF_STR_CONCAT(__make_OpDeclare, __COUNTER__) __attribute__((unused)) =          \
      (::raf::op::OpDeclare::Register(OP_NAME, BODY), 0)
