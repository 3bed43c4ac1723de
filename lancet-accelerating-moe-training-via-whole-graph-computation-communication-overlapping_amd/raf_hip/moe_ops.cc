// The MoE dispatch operators of the "hip" dialect: Declare functions (output shapes and dtypes)
// and one OpEnv per operator, registered under RAF's base-op names with RAF's argument schemas
// (scripts/src_codegen/def_schema.py:642-698).  Each OpEnv captures shapes and attributes in its
// constructor, requests its workspace from the executor and, in Execute, hands raw pointers to
// the C ABI (include/lancet_hip.h) on the executor's current stream.
//
// Counterparts in the reference: src/op/declare/moe.cc:26-213 (Declare) and
// src/op/dialect/cuda/moe.cc:330-412 (MoeEncode), :415-729 (MoeEncodeBatchPrioritized),
// :731-823 (MoeMergeMasks), :826-943 (MoeRedispatch), :1228-1311 (MoeDecode).
//
// Extensions are trailing, defaulted arguments only:
//   moe_encode(data, gate, used_capacity, capacity_factor=1.0, top_k=1, gate_is_logits=false, zero_tail=true)
//   moe_encode_batch_prioritized(..., capacity_factor=1.0, gate_is_logits=false, zero_tail=true)
//   moe_decode(data, gate, indices_locations, top_k=1)
#include <string>
#include <vector>

#include "lancet_hip.h"
#include "op.h"

namespace raf {
namespace op {
namespace hip {

namespace {

int DTypeToLancet(const DType& dt) {
  if (dt.code == DTypeCode::kFloat && dt.bits == 32) return LANCET_F32;
  if (dt.code == DTypeCode::kFloat && dt.bits == 16) return LANCET_F16;
  if (dt.code == DTypeCode::kBFloat && dt.bits == 16) return LANCET_BF16;
  throw Error("token rows must be float32, float16 or bfloat16");
}

// Gate arrays come in the type the graph has them in: fp32, or a half type under mixed precision
// (python/raf/amp/type_hints.py:97,105; the reference's kernels take `__dtype* gates1_s`).
int GateDTypeToLancet(const DType& dt) {
  if (dt.code == DTypeCode::kFloat && dt.bits == 32) return LANCET_F32;
  if (dt.code == DTypeCode::kFloat && dt.bits == 16) return LANCET_F16;
  if (dt.code == DTypeCode::kBFloat && dt.bits == 16) return LANCET_BF16;
  throw Error("gate values must be float32, float16 or bfloat16");
}
bool IsI32(const DType& dt) { return dt.code == DTypeCode::kInt && dt.bits == 32; }

void CheckStatus(int status, const char* what) {
  if (status != LANCET_OK)
    throw Error(std::string(what) + " failed: " + lancet_status_string(status) + " (status " +
                std::to_string(status) + ")");
}

// Only the look-back form of the scan carries state in its workspace from call to call (ticket, epoch, descriptors)
// and needs it set up once (lancet_scan_workspace_init); the forms most calls take use the workspace as plain
// scratch (lancet_scan_call_is_stateful).  The executor binds the memory after the OpEnv is built and may bind other
// memory later (an interpreter keeps one allocation per cached OpEnv, a VM allocates before every Execute,
// src/impl/vm/vm.cc:1260-1266, and other operators may have used that memory in between): a stateful OpEnv sets up
// whatever binding it has not set up yet, on the stream it executes on, and only the header and descriptor table
// the scan reads (init_bytes), not the scratch behind them; a stateless one sets up nothing, and has nothing to
// report at CheckDeviceStatus either (no waits, so no synchronisation there).
struct ScanWorkspaceState {
  bool stateful = false;  // the OpEnv's calls run the look-back form
  size_t init_bytes = 0;  // header + descriptor table
  void* ready = nullptr;  // the binding lancet_scan_workspace_init has run on
  void Configure(int64_t S, int64_t E, int nsets, unsigned flags, bool bpr) {
    stateful = lancet_scan_call_is_stateful(S, E, bpr ? 1 : nsets, flags, bpr ? 1 : 0) != 0;
    init_bytes = lancet_moe_encode_workspace_bytes(S, E, nsets);
  }
  void Ensure(void* ws, size_t nbytes, void* stream) {
    if (!stateful || ws == ready) return;
    CheckStatus(lancet_scan_workspace_init(ws, init_bytes < nbytes ? init_bytes : nbytes, stream), "lancet_scan_workspace_init");
    ready = ws;
  }
  // the workspace's sticky error word (read and cleared; synchronises the stream)
  void Check(void* ws, void* stream, const char* op) {
    if (!stateful || !ws || ws != ready) return;
    int err = 0;
    CheckStatus(lancet_scan_workspace_error(ws, stream, &err), "lancet_scan_workspace_error");
    if (err)
      throw Error(std::string(op) + ": the position scan gave up a wait for another workgroup; the tokens concerned "
                  "carry indices_locations = -1 (used_capacity = -1 if the totals were lost)");
  }
};

Tensor MakeOut(int device_id, DTypeCode code, int bits, std::vector<int64_t> shape) {
  Tensor t;
  t.device_id = device_id;
  t.dtype.code = code;
  t.dtype.bits = bits;
  t.shape = std::move(shape);
  return t;
}

int64_t OptInt(const CallValues& cv, size_t i, int64_t dflt) {
  return cv.args.size() > i && cv.args[i].kind != Value::kNone ? cv.args[i].AsInt() : dflt;
}
double OptFloat(const CallValues& cv, size_t i, double dflt) {
  return cv.args.size() > i && cv.args[i].kind != Value::kNone ? cv.args[i].AsFloat() : dflt;
}

// dtype of a gate gradient that no gate-typed input fixes, from an optional trailing integer argument
// (the LANCET_* code: 0 float32, the default; 1 bfloat16; 2 float16)
DType GateGradDType(const CallValues& cv, size_t i) {
  DType dt;
  switch (OptInt(cv, i, LANCET_F32)) {
    case LANCET_F32: dt.code = DTypeCode::kFloat, dt.bits = 32; break;
    case LANCET_BF16: dt.code = DTypeCode::kBFloat, dt.bits = 16; break;
    case LANCET_F16: dt.code = DTypeCode::kFloat, dt.bits = 16; break;
    default: throw Error("gate_dtype must be 0 (float32), 1 (bfloat16) or 2 (float16)");
  }
  return dt;
}

struct EncodeShape {
  int64_t S, M, E, C;
};

// dim checks of MoeEncodeDeclare / MoeEncodeInitBody (declare/moe.cc:32-46, cuda/moe.cc:95-121)
EncodeShape CheckEncodeInputs(const Tensor& data, const Tensor& gate, int64_t n_partitions, float cf) {
  RAF_CHECK(data.shape.size() == 2, "Input data should be 2-D.");
  RAF_CHECK(gate.shape.size() == 2, "Input gate should be 2-D.");
  RAF_CHECK(data.shape[0] == gate.shape[0], "Input data and gate should have matching shape in dim 0.");
  GateDTypeToLancet(gate.dtype);
  DTypeToLancet(data.dtype);
  EncodeShape s;
  s.S = data.shape[0] / n_partitions;
  s.M = data.shape[1];
  s.E = gate.shape[1];
  s.C = lancet_moe_capacity(s.S, s.E, cf);
  RAF_CHECK(s.C >= 0, "bad capacity");
  return s;
}

// the 5-tuple of declare/moe.cc:48-58; gates_s has the gate's dtype (what the reference's kernels write,
// tutel_moe_dispatch.cu:110-116; its declaration says fp32 whatever the gate is), the buffer the data dtype
Value EncodeOutputs(const Tensor& data, const Tensor& gate, const EncodeShape& s, int64_t k) {
  std::vector<Value> ret;
  ret.push_back(Value::MakeTensor(MakeOut(data.device_id, gate.dtype.code, gate.dtype.bits, {k * s.S})));
  ret.push_back(Value::MakeTensor(MakeOut(data.device_id, DTypeCode::kInt, 32, {2, k * s.S})));
  ret.push_back(Value::MakeTensor(MakeOut(data.device_id, DTypeCode::kInt, 32, {s.E})));
  ret.push_back(Value::MakeTensor(MakeOut(data.device_id, DTypeCode::kUInt, 64, {s.E})));
  Tensor buf = MakeOut(data.device_id, data.dtype.code, data.dtype.bits, {s.E, s.C, s.M});
  ret.push_back(Value::MakeTensor(buf));
  return Value::MakeTuple(std::move(ret));
}

}  // namespace

// =====================================================================================
// raf.op.moe_encode
// =====================================================================================
void MoeEncodeDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 3, "moe_encode(data, gate, used_capacity, capacity_factor=1.0)");
  const Tensor& data = call.args[0].AsTensor();
  const Tensor& gate = call.args[1].AsTensor();
  const Tensor& used = call.args[2].AsTensor();
  RAF_CHECK(used.shape.size() == 1, "Input used_capacity should be 1-D.");
  const int64_t k = OptInt(call, 4, 1);
  RAF_CHECK(k == 1 || k == 2, "top_k must be 1 or 2");
  const float cf = static_cast<float>(OptFloat(call, 3, 1.0)) * (k == 2 ? 2.0f : 1.0f);
  const EncodeShape s = CheckEncodeInputs(data, gate, 1, cf);
  RAF_CHECK(used.shape[0] == s.E && IsI32(used.dtype), "used_capacity must be int32 [E]");
  call.out = EncodeOutputs(data, gate, s, k);
  call.device_id = data.device_id;
}

class MoeEncode : public OpEnv {
 public:
  explicit MoeEncode(const CallValues& cv) {
    const Tensor& data = cv.args[0].AsTensor();
    top_k_ = static_cast<int>(OptInt(cv, 4, 1));
    const float cf = static_cast<float>(OptFloat(cv, 3, 1.0)) * (top_k_ == 2 ? 2.0f : 1.0f);
    shape_ = CheckEncodeInputs(data, cv.args[1].AsTensor(), 1, cf);
    flags_ = (OptInt(cv, 5, 0) ? LANCET_GATE_IS_LOGITS : 0u) | (OptInt(cv, 6, 1) ? 0u : LANCET_NO_TAIL_ZERO);
    // trailing extension (argument 8, after the optional noise tensor): the scan as one look-back kernel
    if (cv.args.size() > 8 && cv.args[8].kind != Value::kTensor && OptInt(cv, 8, 0)) flags_ |= LANCET_SCAN_LOOKBACK;
    dtype_ = DTypeToLancet(data.dtype);
    gate_dtype_ = GateDTypeToLancet(cv.args[1].AsTensor().dtype);
    device_id_ = data.device_id;
    RAF_CHECK(cv.out.kind == Value::kTuple && cv.out.fields.size() == 5, "Expected output to be a 5-Tuple");
    ws_bytes_ = lancet_moe_encode_workspace_bytes(shape_.S, shape_.E, top_k_);
    scan_ws_.Configure(shape_.S, shape_.E, top_k_, flags_, false);
    RequestWorkspace(&ws_, device_id_, static_cast<int64_t>(ws_bytes_));
    this->arg_indices = {0, 1, 2};  // data, gate, used_capacity
    // trailing extension: gate2_noise [S, E] for the second choice of top_k = 2
    has_noise_ = cv.args.size() > 7 && cv.args[7].kind == Value::kTensor;
    if (has_noise_) {
      const Tensor& noise = cv.args[7].AsTensor();
      RAF_CHECK(top_k_ == 2, "gate2_noise only exists for the second choice (top_k = 2)");
      RAF_CHECK(noise.shape == cv.args[1].AsTensor().shape && noise.dtype == cv.args[1].AsTensor().dtype,
                "gate2_noise must have the gate's shape and dtype");
      this->arg_indices.push_back(7);
    }
  }

  void Execute(const CallValues& cv) override {
    std::vector<Value> inputs = {cv.args[0], cv.args[1], cv.args[2]};
    if (has_noise_) inputs.push_back(cv.args[7]);
    Execute(inputs, cv.out);
  }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    const Tensor& data = inputs[0].AsTensor();
    const Tensor& gate = inputs[1].AsTensor();
    const Tensor& used = inputs[2].AsTensor();
    const void* noise = has_noise_ ? inputs[3].AsTensor().data : nullptr;
    const auto& out = output.AsTuple();
    RAF_CHECK(out.size() == 5, "Expected output to be a 5-Tuple");
    scan_ws_.Ensure(ws_, ws_bytes_, GetStream(device_id_));
    CheckStatus(lancet_moe_encode(data.data, gate.data, noise,
                                  static_cast<const int32_t*>(used.data), shape_.S, shape_.M, shape_.E, shape_.C,
                                  top_k_, dtype_, gate_dtype_, flags_, out[0].AsTensor().data,
                                  static_cast<int32_t*>(out[1].AsTensor().data),
                                  static_cast<int32_t*>(out[2].AsTensor().data),
                                  static_cast<uint64_t*>(out[3].AsTensor().data), out[4].AsTensor().data, ws_,
                                  ws_bytes_, GetStream(device_id_)),
                "lancet_moe_encode");
  }

  void WorkspaceBound() override { scan_ws_.ready = nullptr; }
  void CheckDeviceStatus(void* stream) override { scan_ws_.Check(ws_, stream, "moe_encode"); }
  std::string name() const override { return "raf.op.hip.moe_encode"; }
  static OpEnv* make(const CallValues& cv) { return new MoeEncode(cv); }

 private:
  EncodeShape shape_;
  int top_k_, dtype_, gate_dtype_, device_id_;
  unsigned flags_;
  bool has_noise_ = false;
  void* ws_ = nullptr;
  size_t ws_bytes_ = 0;
  ScanWorkspaceState scan_ws_;
};

// =====================================================================================
// raf.op.moe_encode_batch_prioritized
// =====================================================================================
void MoeEncodeBatchPrioritizedDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 2, "moe_encode_batch_prioritized(data, gate, n_partitions=1, partition_id=0, capacity_factor=1.0)");
  const Tensor& data = call.args[0].AsTensor();
  const int64_t n_part = OptInt(call, 2, 1), pid = OptInt(call, 3, 0);
  RAF_CHECK(n_part > 0, "n_partitions should be greater than 0.");
  RAF_CHECK(pid >= 0 && pid < n_part, "partition_id should be less than n_partitions.");
  const EncodeShape s = CheckEncodeInputs(data, call.args[1].AsTensor(), n_part,
                                          static_cast<float>(OptFloat(call, 4, 1.0)));
  call.out = EncodeOutputs(data, call.args[1].AsTensor(), s, 1);
  call.device_id = data.device_id;
}

class MoeEncodeBatchPrioritized : public OpEnv {
 public:
  explicit MoeEncodeBatchPrioritized(const CallValues& cv) {
    const Tensor& data = cv.args[0].AsTensor();
    n_partitions_ = static_cast<int>(OptInt(cv, 2, 1));
    partition_id_ = static_cast<int>(OptInt(cv, 3, 0));
    RAF_CHECK(n_partitions_ > 0 && partition_id_ >= 0 && partition_id_ < n_partitions_, "bad partition");
    shape_ = CheckEncodeInputs(data, cv.args[1].AsTensor(), n_partitions_, static_cast<float>(OptFloat(cv, 4, 1.0)));
    orig_S_ = data.shape[0];
    flags_ = (OptInt(cv, 5, 0) ? LANCET_GATE_IS_LOGITS : 0u) | (OptInt(cv, 6, 1) ? 0u : LANCET_NO_TAIL_ZERO);
    dtype_ = DTypeToLancet(data.dtype);
    gate_dtype_ = GateDTypeToLancet(cv.args[1].AsTensor().dtype);
    device_id_ = data.device_id;
    // sorted indices, dropping mask, indices and gate buffers of the reference (cuda/moe.cc:512-520)
    // are replaced by one workspace for the radix select and the scan
    ws_bytes_ = lancet_moe_encode_bpr_workspace_bytes(orig_S_, shape_.E, n_partitions_);
    scan_ws_.Configure(shape_.S, shape_.E, 2, flags_, true);
    RequestWorkspace(&ws_, device_id_, static_cast<int64_t>(ws_bytes_));
    this->arg_indices = {0, 1};
  }

  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1]}, cv.out); }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    const auto& out = output.AsTuple();
    RAF_CHECK(out.size() == 5, "Expected output to be a 5-Tuple");
    scan_ws_.Ensure(ws_, ws_bytes_, GetStream(device_id_));
    CheckStatus(lancet_moe_encode_bpr(inputs[0].AsTensor().data, inputs[1].AsTensor().data,
                                      orig_S_, shape_.M, shape_.E, shape_.C, n_partitions_, partition_id_, dtype_,
                                      gate_dtype_, flags_, out[0].AsTensor().data,
                                      static_cast<int32_t*>(out[1].AsTensor().data),
                                      static_cast<int32_t*>(out[2].AsTensor().data),
                                      static_cast<uint64_t*>(out[3].AsTensor().data), out[4].AsTensor().data, ws_,
                                      ws_bytes_, GetStream(device_id_)),
                "lancet_moe_encode_bpr");
  }

  void WorkspaceBound() override { scan_ws_.ready = nullptr; }
  void CheckDeviceStatus(void* stream) override { scan_ws_.Check(ws_, stream, "moe_encode_batch_prioritized"); }
  std::string name() const override { return "raf.op.hip.moe_encode_batch_prioritized"; }
  static OpEnv* make(const CallValues& cv) { return new MoeEncodeBatchPrioritized(cv); }

 private:
  EncodeShape shape_;
  int64_t orig_S_;
  int n_partitions_, partition_id_, dtype_, gate_dtype_, device_id_;
  unsigned flags_;
  void* ws_ = nullptr;
  size_t ws_bytes_ = 0;
  ScanWorkspaceState scan_ws_;
};

// =====================================================================================
// raf.op.moe_merge_masks
// =====================================================================================
void MoeMergeMasksDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() == 2, "moe_merge_masks(indices_locations, n_experts)");
  const auto& masks = call.args[0].AsTuple();
  RAF_CHECK(!masks.empty(), "indices_locations must not be empty");
  const Tensor& m0 = masks[0].AsTensor();
  RAF_CHECK(m0.shape.size() == 2, "Input indices_locations should be 2-D.");
  const int64_t P = static_cast<int64_t>(masks.size());
  call.out = Value::MakeTensor(MakeOut(m0.device_id, DTypeCode::kInt, 32, {2, m0.shape[1] * P}));
  call.device_id = m0.device_id;
}

class MoeMergeMasks : public OpEnv {
 public:
  explicit MoeMergeMasks(const CallValues& cv) {
    const auto& masks = cv.args[0].AsTuple();
    n_partitions_ = static_cast<int>(masks.size());
    RAF_CHECK(n_partitions_ >= 1 && n_partitions_ <= LANCET_MAX_PARTITIONS, "unsupported number of partitions");
    const Tensor& m0 = masks[0].AsTensor();
    RAF_CHECK(m0.shape.size() == 2 && m0.shape[0] == 2, "Expected input indices_locations to be [2, S].");
    dim_S_ = m0.shape[1];
    dim_E_ = cv.args[1].AsInt();
    device_id_ = m0.device_id;
    // the reference keeps a pinned host table and a device table of 2P pointers
    // (cuda/moe.cc:751-755); pointer tables travel as kernel arguments here
    ws_bytes_ = lancet_moe_merge_masks_workspace_bytes(n_partitions_, dim_E_);
    RequestWorkspace(&ws_, device_id_, static_cast<int64_t>(ws_bytes_));
    this->arg_indices = {0};
  }

  void Execute(const CallValues& cv) override { Execute({cv.args[0]}, cv.out); }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    const auto& masks = inputs[0].AsTuple();
    RAF_CHECK(static_cast<int>(masks.size()) == n_partitions_, "partition count changed");
    std::vector<const int32_t*> ptrs;
    for (const auto& m : masks) {
      const Tensor& t = m.AsTensor();
      RAF_CHECK(IsI32(t.dtype) && t.shape.size() == 2 && t.shape[1] == dim_S_, "indices_locations must be int32 [2, S]");
      ptrs.push_back(static_cast<const int32_t*>(t.data));
    }
    CheckStatus(lancet_moe_merge_masks(ptrs.data(), n_partitions_, dim_S_, dim_E_,
                                       static_cast<int32_t*>(output.AsTensor().data), ws_, ws_bytes_,
                                       GetStream(device_id_)),
                "lancet_moe_merge_masks");
  }

  std::string name() const override { return "raf.op.hip.moe_merge_masks"; }
  static OpEnv* make(const CallValues& cv) { return new MoeMergeMasks(cv); }

 private:
  int64_t dim_S_, dim_E_;
  int n_partitions_, device_id_;
  void* ws_ = nullptr;
  size_t ws_bytes_ = 0;
};

// =====================================================================================
// raf.op.moe_redispatch
// =====================================================================================
void MoeRedispatchDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() == 2, "moe_redispatch(data, indices_locations)");
  const auto& bufs = call.args[0].AsTuple();
  const auto& masks = call.args[1].AsTuple();
  RAF_CHECK(!bufs.empty() && bufs.size() == masks.size(), "data and indices_locations must have one entry per partition");
  const Tensor& d0 = bufs[0].AsTensor();
  RAF_CHECK(d0.shape.size() == 3 || d0.shape.size() == 4, "Input data should be 3 or 4-D.");
  RAF_CHECK(masks[0].AsTensor().shape.size() == 2, "Input indices_locations should be 2-D.");
  // data dtype, as the type relation says (src/op/ty/moe.cc:141); Declare hard-codes float32
  // (declare/moe.cc:136), which cannot hold for 16-bit buffers
  call.out = Value::MakeTensor(MakeOut(d0.device_id, d0.dtype.code, d0.dtype.bits, d0.shape));
  call.device_id = d0.device_id;
}

class MoeRedispatch : public OpEnv {
 public:
  explicit MoeRedispatch(const CallValues& cv) {
    const auto& bufs = cv.args[0].AsTuple();
    const auto& masks = cv.args[1].AsTuple();
    n_partitions_ = static_cast<int>(masks.size());
    RAF_CHECK(n_partitions_ >= 1 && n_partitions_ <= LANCET_MAX_PARTITIONS, "unsupported number of partitions");
    const Tensor& d0 = bufs[0].AsTensor();
    if (d0.shape.size() == 3) {  // [E, C, M]
      dim_E_ = d0.shape[0], dim_C_ = d0.shape[1], dim_M_ = d0.shape[2];
    } else {                     // [G, LE, C, M]
      RAF_CHECK(d0.shape.size() == 4, "Expected input data to be 3 or 4D.");
      dim_E_ = d0.shape[0] * d0.shape[1], dim_C_ = d0.shape[2], dim_M_ = d0.shape[3];
    }
    dim_S_ = masks[0].AsTensor().shape[1];
    dtype_ = DTypeToLancet(d0.dtype);
    device_id_ = d0.device_id;
    ws_bytes_ = lancet_moe_redispatch_workspace_bytes(n_partitions_, dim_E_);
    RequestWorkspace(&ws_, device_id_, static_cast<int64_t>(ws_bytes_));
    this->arg_indices = {0, 1};
  }

  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1]}, cv.out); }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    const auto& bufs = inputs[0].AsTuple();
    const auto& masks = inputs[1].AsTuple();
    RAF_CHECK(static_cast<int>(masks.size()) == n_partitions_ && bufs.size() == masks.size(), "partition count changed");
    std::vector<const void*> dptrs;
    std::vector<const int32_t*> mptrs;
    for (int i = 0; i < n_partitions_; ++i) {
      dptrs.push_back(bufs[i].AsTensor().data);
      mptrs.push_back(static_cast<const int32_t*>(masks[i].AsTensor().data));
    }
    CheckStatus(lancet_moe_redispatch(dptrs.data(), mptrs.data(), n_partitions_, dim_S_, dim_M_, dim_C_, dim_E_,
                                      dtype_, output.AsTensor().data, ws_, ws_bytes_, GetStream(device_id_)),
                "lancet_moe_redispatch");
  }

  std::string name() const override { return "raf.op.hip.moe_redispatch"; }
  static OpEnv* make(const CallValues& cv) { return new MoeRedispatch(cv); }

 private:
  int64_t dim_S_, dim_E_, dim_C_, dim_M_;
  int n_partitions_, dtype_, device_id_;
  void* ws_ = nullptr;
  size_t ws_bytes_ = 0;
};

// =====================================================================================
// raf.op.moe_decode
// =====================================================================================
void MoeDecodeDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 3, "moe_decode(data, gate, indices_locations)");
  const Tensor& data = call.args[0].AsTensor();
  const Tensor& gate = call.args[1].AsTensor();
  RAF_CHECK(data.shape.size() == 3, "Input data should be 3-D.");
  RAF_CHECK(gate.shape.size() == 1, "Input gate should be 1-D.");
  DTypeToLancet(data.dtype);
  const int64_t k = OptInt(call, 3, 1);
  RAF_CHECK(k == 1 || k == 2, "top_k must be 1 or 2");
  RAF_CHECK(gate.shape[0] % k == 0, "gate length must be a multiple of top_k");
  call.out = Value::MakeTensor(MakeOut(data.device_id, data.dtype.code, data.dtype.bits, {gate.shape[0] / k, data.shape[2]}));
  call.device_id = data.device_id;
}

class MoeDecode : public OpEnv {
 public:
  explicit MoeDecode(const CallValues& cv) {
    const Tensor& data = cv.args[0].AsTensor();
    const Tensor& gate = cv.args[1].AsTensor();
    RAF_CHECK(data.shape.size() == 3, "Expected input data to be 3D.");
    RAF_CHECK(gate.shape.size() == 1, "Expected input gate to be 1D.");
    gate_dtype_ = GateDTypeToLancet(gate.dtype);
    top_k_ = static_cast<int>(OptInt(cv, 3, 1));
    dim_S_ = gate.shape[0] / top_k_;
    dim_E_ = data.shape[0], dim_C_ = data.shape[1], dim_M_ = data.shape[2];
    dtype_ = DTypeToLancet(data.dtype);
    device_id_ = data.device_id;
    this->arg_indices = {0, 1, 2};
  }

  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1], cv.args[2]}, cv.out); }

  void Execute(const std::vector<Value>& inputs, Value output) override {
    const Tensor& il = inputs[2].AsTensor();
    RAF_CHECK(IsI32(il.dtype) && il.shape.size() == 2 && il.shape[1] == dim_S_ * top_k_, "indices_locations must be int32 [2, k*S]");
    CheckStatus(lancet_moe_decode(inputs[0].AsTensor().data, inputs[1].AsTensor().data,
                                  static_cast<const int32_t*>(il.data), dim_S_, dim_M_, dim_E_, dim_C_, top_k_,
                                  dtype_, gate_dtype_, output.AsTensor().data, GetStream(device_id_)),
                "lancet_moe_decode");
  }

  std::string name() const override { return "raf.op.hip.moe_decode"; }
  static OpEnv* make(const CallValues& cv) { return new MoeDecode(cv); }

 private:
  int64_t dim_S_, dim_E_, dim_C_, dim_M_;
  int top_k_, dtype_, gate_dtype_, device_id_;
};

// =====================================================================================
// raf.op.moe_redispatch_expert_input(data, recv_cnts, local_expert_id, n_local_experts, recv_cnts_scale=1)
// (src/op/declare/moe.cc:140-163; src/op/dialect/cuda/moe.cc:945-1073)
// =====================================================================================
namespace {
struct ExpertInputShape {
  int64_t C, G, M;
};
ExpertInputShape ExpertInputDims(const Tensor& d0, const Tensor& c0, int64_t LE) {
  RAF_CHECK(c0.shape.size() == 1, "Expected input recv_cnts to be 1D.");
  RAF_CHECK((c0.dtype.code == DTypeCode::kUInt || c0.dtype.code == DTypeCode::kInt) && c0.dtype.bits == 64,
            "recv_cnts must be 64-bit counts");
  ExpertInputShape s;
  if (d0.shape.size() == 4) {  // [C, 1, G, M]
    RAF_CHECK(d0.shape[1] == 1, "4D Input data should have dim 1 at axis 1.");
    s.C = d0.shape[0], s.G = d0.shape[2], s.M = d0.shape[3];
  } else if (d0.shape.size() == 3) {  // [C, G, M]
    s.C = d0.shape[0], s.G = d0.shape[1], s.M = d0.shape[2];
  } else {  // [C x G, M]
    RAF_CHECK(d0.shape.size() == 2, "Input data should be 2,3 or 4-D.");
    RAF_CHECK(LE > 0 && c0.shape[0] >= LE, "bad n_local_experts");
    s.G = c0.shape[0] / LE;
    s.C = d0.shape[0] / s.G, s.M = d0.shape[1];
  }
  RAF_CHECK(s.G > 0 && c0.shape[0] / s.G == LE, "Expected input recv_cnts to be 1D of size G x LE.");
  return s;
}
}  // namespace

void MoeRedispatchExpertInputDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 4, "moe_redispatch_expert_input(data, recv_cnts, local_expert_id, n_local_experts, recv_cnts_scale=1)");
  const auto& bufs = call.args[0].AsTuple();
  const auto& cnts = call.args[1].AsTuple();
  RAF_CHECK(!bufs.empty() && bufs.size() == cnts.size(), "data and recv_cnts must have one entry per partition");
  const Tensor& d0 = bufs[0].AsTensor();
  ExpertInputDims(d0, cnts[0].AsTensor(), call.args[3].AsInt());
  DTypeToLancet(d0.dtype);
  // data dtype (Declare hard-codes float32, declare/moe.cc:161, which cannot hold for 16-bit buffers)
  call.out = Value::MakeTensor(MakeOut(d0.device_id, d0.dtype.code, d0.dtype.bits, d0.shape));
  call.device_id = d0.device_id;
}

class MoeRedispatchExpertInput : public OpEnv {
 public:
  explicit MoeRedispatchExpertInput(const CallValues& cv) {
    const auto& bufs = cv.args[0].AsTuple();
    const auto& cnts = cv.args[1].AsTuple();
    n_partitions_ = static_cast<int>(cnts.size());
    RAF_CHECK(n_partitions_ >= 1 && n_partitions_ <= LANCET_MAX_PARTITIONS, "unsupported number of partitions");
    local_expert_id_ = static_cast<int>(cv.args[2].AsInt());
    dim_LE_ = static_cast<int>(cv.args[3].AsInt());
    recv_cnts_scale_ = static_cast<int>(OptInt(cv, 4, 1));
    const Tensor& d0 = bufs[0].AsTensor();
    shape_ = ExpertInputDims(d0, cnts[0].AsTensor(), dim_LE_);
    dtype_ = DTypeToLancet(d0.dtype);
    device_id_ = d0.device_id;
    this->arg_indices = {0, 1};
  }
  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1]}, cv.out); }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    const auto& bufs = inputs[0].AsTuple();
    const auto& cnts = inputs[1].AsTuple();
    RAF_CHECK(static_cast<int>(cnts.size()) == n_partitions_ && bufs.size() == cnts.size(), "partition count changed");
    std::vector<const void*> dptrs;
    std::vector<const uint64_t*> cptrs;
    for (int i = 0; i < n_partitions_; ++i) {
      dptrs.push_back(bufs[i].AsTensor().data);
      cptrs.push_back(static_cast<const uint64_t*>(cnts[i].AsTensor().data));
    }
    CheckStatus(lancet_moe_redispatch_expert_input(dptrs.data(), cptrs.data(), n_partitions_, local_expert_id_, dim_LE_,
                                                   shape_.C, shape_.M, shape_.G, recv_cnts_scale_, dtype_,
                                                   output.AsTensor().data, GetStream(device_id_)),
                "lancet_moe_redispatch_expert_input");
  }
  std::string name() const override { return "raf.op.hip.moe_redispatch_expert_input"; }
  static OpEnv* make(const CallValues& cv) { return new MoeRedispatchExpertInput(cv); }

 private:
  ExpertInputShape shape_;
  int n_partitions_, local_expert_id_, dim_LE_, recv_cnts_scale_, dtype_, device_id_;
};

// =====================================================================================
// backward ops: raf.op.moe_encode_dx / moe_encode_dg / moe_decode_dx / moe_decode_dg
// (src/op/declare/moe.cc:165-247; src/op/dialect/cuda/moe.cc:1075-1225, 1313-1481; gradients wired in
// src/op/grad/moe.cc:30-93).  Gate-side tensors are float32; an optional trailing top_k selects the
// slot-major two-slot layout.
// =====================================================================================
namespace {
int64_t MaskTokens(const Tensor& il, int64_t k) {
  RAF_CHECK(IsI32(il.dtype) && il.shape.size() == 2 && il.shape[0] == 2, "Input indices_locations should be int32 [2, k*S].");
  RAF_CHECK(k == 1 || k == 2, "top_k must be 1 or 2");
  RAF_CHECK(il.shape[1] % k == 0, "mask length must be a multiple of top_k");
  return il.shape[1] / k;
}
}  // namespace

void MoeEncodeDxDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 2, "moe_encode_dx(dy, indices_locations)");
  const Tensor& dy = call.args[0].AsTensor();
  RAF_CHECK(dy.shape.size() == 3, "Input dy should be 3-D.");
  DTypeToLancet(dy.dtype);
  const int64_t S = MaskTokens(call.args[1].AsTensor(), OptInt(call, 2, 1));
  call.out = Value::MakeTensor(MakeOut(dy.device_id, dy.dtype.code, dy.dtype.bits, {S, dy.shape[2]}));
  call.device_id = dy.device_id;
}

class MoeEncodeDx : public OpEnv {
 public:
  explicit MoeEncodeDx(const CallValues& cv) {
    const Tensor& dy = cv.args[0].AsTensor();
    RAF_CHECK(dy.shape.size() == 3, "Expected input dy to be 3D.");
    top_k_ = static_cast<int>(OptInt(cv, 2, 1));
    dim_S_ = MaskTokens(cv.args[1].AsTensor(), top_k_);
    dim_E_ = dy.shape[0], dim_C_ = dy.shape[1], dim_M_ = dy.shape[2];
    dtype_ = DTypeToLancet(dy.dtype);
    device_id_ = dy.device_id;
    this->arg_indices = {0, 1};
  }
  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1]}, cv.out); }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    CheckStatus(lancet_moe_encode_dx(inputs[0].AsTensor().data, static_cast<const int32_t*>(inputs[1].AsTensor().data),
                                     dim_S_, dim_M_, dim_E_, dim_C_, top_k_, dtype_, output.AsTensor().data,
                                     GetStream(device_id_)),
                "lancet_moe_encode_dx");
  }
  std::string name() const override { return "raf.op.hip.moe_encode_dx"; }
  static OpEnv* make(const CallValues& cv) { return new MoeEncodeDx(cv); }

 private:
  int64_t dim_S_, dim_E_, dim_C_, dim_M_;
  int top_k_, dtype_, device_id_;
};

void MoeEncodeDgDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 3, "moe_encode_dg(dy, indices_locations, n_experts)");
  const Tensor& dy = call.args[0].AsTensor();
  RAF_CHECK(dy.shape.size() == 1, "Input dy should be 1-D.");
  GateDTypeToLancet(dy.dtype);
  const int64_t S = MaskTokens(call.args[1].AsTensor(), OptInt(call, 3, 1));
  call.out = Value::MakeTensor(MakeOut(dy.device_id, dy.dtype.code, dy.dtype.bits, {S, call.args[2].AsInt()}));  // declare/moe.cc:194
  call.device_id = dy.device_id;
}

class MoeEncodeDg : public OpEnv {
 public:
  explicit MoeEncodeDg(const CallValues& cv) {
    const Tensor& dy = cv.args[0].AsTensor();
    RAF_CHECK(dy.shape.size() == 1, "Expected input dy to be 1D.");
    gate_dtype_ = GateDTypeToLancet(dy.dtype);
    top_k_ = static_cast<int>(OptInt(cv, 3, 1));
    dim_S_ = MaskTokens(cv.args[1].AsTensor(), top_k_);
    RAF_CHECK(dy.shape[0] == dim_S_ * top_k_, "dy and indices_locations disagree");
    dim_E_ = cv.args[2].AsInt();
    device_id_ = dy.device_id;
    this->arg_indices = {0, 1};
  }
  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1]}, cv.out); }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    CheckStatus(lancet_moe_encode_dg(inputs[0].AsTensor().data,
                                     static_cast<const int32_t*>(inputs[1].AsTensor().data), dim_S_, dim_E_, top_k_,
                                     gate_dtype_, output.AsTensor().data, GetStream(device_id_)),
                "lancet_moe_encode_dg");
  }
  std::string name() const override { return "raf.op.hip.moe_encode_dg"; }
  static OpEnv* make(const CallValues& cv) { return new MoeEncodeDg(cv); }

 private:
  int64_t dim_S_, dim_E_;
  int top_k_, gate_dtype_, device_id_;
};

void MoeDecodeDxDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 5, "moe_decode_dx(dy, gate, indices_locations, n_experts, capacity)");
  const Tensor& dy = call.args[0].AsTensor();
  RAF_CHECK(dy.shape.size() == 2, "Input dy should be 2-D.");
  DTypeToLancet(dy.dtype);
  call.out = Value::MakeTensor(MakeOut(dy.device_id, dy.dtype.code, dy.dtype.bits,
                                       {call.args[3].AsInt(), call.args[4].AsInt(), dy.shape[1]}));
  call.device_id = dy.device_id;
}

class MoeDecodeDx : public OpEnv {
 public:
  explicit MoeDecodeDx(const CallValues& cv) {
    const Tensor& dy = cv.args[0].AsTensor();
    const Tensor& gate = cv.args[1].AsTensor();
    RAF_CHECK(dy.shape.size() == 2, "Expected input dy to be 2D.");
    RAF_CHECK(gate.shape.size() == 1, "Expected input gate to be 1D.");
    gate_dtype_ = GateDTypeToLancet(gate.dtype);
    top_k_ = static_cast<int>(OptInt(cv, 5, 1));
    dim_S_ = MaskTokens(cv.args[2].AsTensor(), top_k_);
    RAF_CHECK(dy.shape[0] == dim_S_ && gate.shape[0] == dim_S_ * top_k_, "dy, gate and indices_locations disagree");
    dim_M_ = dy.shape[1];
    dim_E_ = cv.args[3].AsInt();
    dim_C_ = cv.args[4].AsInt();
    dtype_ = DTypeToLancet(dy.dtype);
    device_id_ = dy.device_id;
    ws_bytes_ = lancet_moe_decode_dx_workspace_bytes(dim_E_, dim_C_);
    RequestWorkspace(&ws_, device_id_, static_cast<int64_t>(ws_bytes_));
    this->arg_indices = {0, 1, 2};
  }
  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1], cv.args[2]}, cv.out); }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    CheckStatus(lancet_moe_decode_dx(inputs[0].AsTensor().data, inputs[1].AsTensor().data,
                                     static_cast<const int32_t*>(inputs[2].AsTensor().data), dim_S_, dim_M_, dim_E_,
                                     dim_C_, top_k_, dtype_, gate_dtype_, output.AsTensor().data, ws_, ws_bytes_,
                                     GetStream(device_id_)),
                "lancet_moe_decode_dx");
  }
  std::string name() const override { return "raf.op.hip.moe_decode_dx"; }
  static OpEnv* make(const CallValues& cv) { return new MoeDecodeDx(cv); }

 private:
  int64_t dim_S_, dim_E_, dim_C_, dim_M_;
  int top_k_, dtype_, gate_dtype_, device_id_;
  void* ws_ = nullptr;
  size_t ws_bytes_ = 0;
};

void MoeDecodeDgDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 3, "moe_decode_dg(dy, data, indices_locations)");
  const Tensor& dy = call.args[0].AsTensor();
  RAF_CHECK(dy.shape.size() == 2, "Input dy should be 2-D.");
  DTypeToLancet(dy.dtype);
  const int64_t k = OptInt(call, 3, 1);
  const int64_t S = MaskTokens(call.args[2].AsTensor(), k);
  // the gradient of gates_s has the gate's dtype: fp32 by default, or what the trailing gate_dtype argument
  // names (a mixed-precision graph passes the half type; the reference gives it dy's dtype, declare/moe.cc:239)
  const DType gd = GateGradDType(call, 4);
  call.out = Value::MakeTensor(MakeOut(dy.device_id, gd.code, gd.bits, {k * S}));
  call.device_id = dy.device_id;
}

class MoeDecodeDg : public OpEnv {
 public:
  explicit MoeDecodeDg(const CallValues& cv) {
    const Tensor& dy = cv.args[0].AsTensor();
    const Tensor& data = cv.args[1].AsTensor();
    RAF_CHECK(dy.shape.size() == 2, "Expected input dy to be 2D.");
    RAF_CHECK(data.shape.size() == 3, "Expected input data to be 3D.");
    RAF_CHECK(dy.dtype == data.dtype && dy.shape[1] == data.shape[2], "dy and data must agree in dtype and model dim");
    top_k_ = static_cast<int>(OptInt(cv, 3, 1));
    dim_S_ = MaskTokens(cv.args[2].AsTensor(), top_k_);
    RAF_CHECK(dy.shape[0] == dim_S_, "dy and indices_locations disagree");
    dim_E_ = data.shape[0], dim_C_ = data.shape[1], dim_M_ = data.shape[2];
    dtype_ = DTypeToLancet(dy.dtype);
    gate_dtype_ = GateDTypeToLancet(GateGradDType(cv, 4));
    device_id_ = dy.device_id;
    this->arg_indices = {0, 1, 2};
  }
  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1], cv.args[2]}, cv.out); }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    CheckStatus(lancet_moe_decode_dg(inputs[0].AsTensor().data, inputs[1].AsTensor().data,
                                     static_cast<const int32_t*>(inputs[2].AsTensor().data), dim_S_, dim_M_, dim_E_,
                                     dim_C_, top_k_, dtype_, gate_dtype_, output.AsTensor().data,
                                     GetStream(device_id_)),
                "lancet_moe_decode_dg");
  }
  std::string name() const override { return "raf.op.hip.moe_decode_dg"; }
  static OpEnv* make(const CallValues& cv) { return new MoeDecodeDg(cv); }

 private:
  int64_t dim_S_, dim_E_, dim_C_, dim_M_;
  int top_k_, dtype_, gate_dtype_, device_id_;
};

// =====================================================================================
// raf.op.moe_encode_dgate(dy, gate, indices_locations, top_k=1, gate_is_logits=false): gate gradient of moe_encode
// as a whole, for the forms of the op that transform the gate value (top-2 normalisation, fused softmax).  Extends
// MoeEncodeGrad (src/op/grad/moe.cc:30-58), whose moe_encode_dg covers the reference's one form.
// =====================================================================================
void MoeEncodeDgateDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 3, "moe_encode_dgate(dy, gate, indices_locations, top_k=1, gate_is_logits=false)");
  const Tensor& dy = call.args[0].AsTensor();
  const Tensor& gate = call.args[1].AsTensor();
  RAF_CHECK(dy.shape.size() == 1, "Input dy should be 1-D.");
  RAF_CHECK(gate.shape.size() == 2, "Input gate should be 2-D.");
  GateDTypeToLancet(gate.dtype);
  RAF_CHECK(dy.dtype == gate.dtype, "dy takes the gate's dtype");
  const int64_t k = OptInt(call, 3, 1);
  const int64_t S = MaskTokens(call.args[2].AsTensor(), k);
  RAF_CHECK(gate.shape[0] == S && dy.shape[0] == k * S, "dy, gate and indices_locations disagree");
  call.out = Value::MakeTensor(MakeOut(gate.device_id, gate.dtype.code, gate.dtype.bits, gate.shape));
  call.device_id = gate.device_id;
}

class MoeEncodeDgate : public OpEnv {
 public:
  explicit MoeEncodeDgate(const CallValues& cv) {
    const Tensor& gate = cv.args[1].AsTensor();
    RAF_CHECK(gate.shape.size() == 2, "Expected input gate to be 2D.");
    gate_dtype_ = GateDTypeToLancet(gate.dtype);
    top_k_ = static_cast<int>(OptInt(cv, 3, 1));
    flags_ = OptInt(cv, 4, 0) ? LANCET_GATE_IS_LOGITS : 0u;
    dim_S_ = MaskTokens(cv.args[2].AsTensor(), top_k_);
    dim_E_ = gate.shape[1];
    device_id_ = gate.device_id;
    this->arg_indices = {0, 1, 2};
  }
  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1], cv.args[2]}, cv.out); }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    CheckStatus(lancet_moe_encode_dgate(inputs[0].AsTensor().data, inputs[1].AsTensor().data,
                                        static_cast<const int32_t*>(inputs[2].AsTensor().data), dim_S_, dim_E_, top_k_,
                                        gate_dtype_, flags_, output.AsTensor().data, GetStream(device_id_)),
                "lancet_moe_encode_dgate");
  }
  std::string name() const override { return "raf.op.hip.moe_encode_dgate"; }
  static OpEnv* make(const CallValues& cv) { return new MoeEncodeDgate(cv); }

 private:
  int64_t dim_S_, dim_E_;
  int top_k_, gate_dtype_, device_id_;
  unsigned flags_;
};

// =====================================================================================
// The routed-once form of Lancet's partitioned dispatch.  The partition pass emits, per token partition p, a
// moe_encode chained to the one before it through used_capacity, then moe_merge_masks and moe_redispatch over all
// of them (src/pass/dist_optimization/partition_exprs.cc:1709-1874).  Routing only reads the [S, E] gate, and the
// merged masks of the chained encodes are by construction the routing of the whole batch
// (tests/python/op/cuda/test_cuda_moe.py:384-471), so a graph that has the whole gate can be rewritten to
//   moe_route(gate_all, used, M, cf, top_k)                         -> (gates_s, indices_locations, used, elems)
//   moe_scatter_tokens(data_p, indices_locations, used_in, used, buffer, token_first_p)   per partition, in place
//   moe_partition_ranges(indices_locations, P, E, M, top_k)         -> (starts, counts) for the partitions' exchanges
//   moe_decode_tokens(expert_out, gates_s, indices_locations, token_first_p, n_tokens)    per partition
// with no merge or redispatch pass: rows go straight to their final places in ONE [E, C, M] buffer.
// =====================================================================================
void MoeRouteDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 3, "moe_route(gate, used_capacity, M, capacity_factor=1.0, top_k=1, gate_is_logits=false)");
  const Tensor& gate = call.args[0].AsTensor();
  const Tensor& used = call.args[1].AsTensor();
  RAF_CHECK(gate.shape.size() == 2, "Input gate should be 2-D.");
  RAF_CHECK(used.shape.size() == 1 && used.shape[0] == gate.shape[1] && IsI32(used.dtype), "used_capacity must be int32 [E]");
  GateDTypeToLancet(gate.dtype);
  const int64_t k = OptInt(call, 4, 1);
  RAF_CHECK(k == 1 || k == 2, "top_k must be 1 or 2");
  const int64_t S = gate.shape[0], E = gate.shape[1];
  std::vector<Value> ret;
  ret.push_back(Value::MakeTensor(MakeOut(gate.device_id, gate.dtype.code, gate.dtype.bits, {k * S})));
  ret.push_back(Value::MakeTensor(MakeOut(gate.device_id, DTypeCode::kInt, 32, {2, k * S})));
  ret.push_back(Value::MakeTensor(MakeOut(gate.device_id, DTypeCode::kInt, 32, {E})));
  ret.push_back(Value::MakeTensor(MakeOut(gate.device_id, DTypeCode::kUInt, 64, {E})));
  call.out = Value::MakeTuple(std::move(ret));
  call.device_id = gate.device_id;
}

class MoeRoute : public OpEnv {
 public:
  explicit MoeRoute(const CallValues& cv) {
    const Tensor& gate = cv.args[0].AsTensor();
    RAF_CHECK(gate.shape.size() == 2, "Expected input gate to be 2D.");
    dim_S_ = gate.shape[0], dim_E_ = gate.shape[1];
    dim_M_ = cv.args[2].AsInt();
    top_k_ = static_cast<int>(OptInt(cv, 4, 1));
    const float cf = static_cast<float>(OptFloat(cv, 3, 1.0)) * (top_k_ == 2 ? 2.0f : 1.0f);
    dim_C_ = lancet_moe_capacity(dim_S_, dim_E_, cf);
    RAF_CHECK(dim_C_ >= 0 && dim_M_ >= 0, "bad capacity or model dim");
    flags_ = OptInt(cv, 5, 0) ? LANCET_GATE_IS_LOGITS : 0u;
    if (cv.args.size() > 7 && cv.args[7].kind != Value::kTensor && OptInt(cv, 7, 0)) flags_ |= LANCET_SCAN_LOOKBACK;
    gate_dtype_ = GateDTypeToLancet(gate.dtype);
    device_id_ = gate.device_id;
    ws_bytes_ = lancet_moe_encode_workspace_bytes(dim_S_, dim_E_, top_k_);
    scan_ws_.Configure(dim_S_, dim_E_, top_k_, flags_, false);
    RequestWorkspace(&ws_, device_id_, static_cast<int64_t>(ws_bytes_));
    this->arg_indices = {0, 1};
    has_noise_ = cv.args.size() > 6 && cv.args[6].kind == Value::kTensor;  // gate2_noise [S, E], top_k = 2
    if (has_noise_) {
      RAF_CHECK(top_k_ == 2, "gate2_noise only exists for the second choice (top_k = 2)");
      RAF_CHECK(cv.args[6].AsTensor().shape == gate.shape && cv.args[6].AsTensor().dtype == gate.dtype,
                "gate2_noise must have the gate's shape and dtype");
      this->arg_indices.push_back(6);
    }
  }
  void Execute(const CallValues& cv) override {
    std::vector<Value> inputs = {cv.args[0], cv.args[1]};
    if (has_noise_) inputs.push_back(cv.args[6]);
    Execute(inputs, cv.out);
  }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    const auto& out = output.AsTuple();
    RAF_CHECK(out.size() == 4, "Expected output to be a 4-Tuple");
    scan_ws_.Ensure(ws_, ws_bytes_, GetStream(device_id_));
    CheckStatus(lancet_moe_route(inputs[0].AsTensor().data, has_noise_ ? inputs[2].AsTensor().data : nullptr,
                                 static_cast<const int32_t*>(inputs[1].AsTensor().data), dim_S_, dim_M_, dim_E_, dim_C_,
                                 top_k_, gate_dtype_, flags_, out[0].AsTensor().data,
                                 static_cast<int32_t*>(out[1].AsTensor().data), static_cast<int32_t*>(out[2].AsTensor().data),
                                 static_cast<uint64_t*>(out[3].AsTensor().data), ws_, ws_bytes_, GetStream(device_id_)),
                "lancet_moe_route");
  }
  void WorkspaceBound() override { scan_ws_.ready = nullptr; }
  void CheckDeviceStatus(void* stream) override { scan_ws_.Check(ws_, stream, "moe_route"); }
  std::string name() const override { return "raf.op.hip.moe_route"; }
  static OpEnv* make(const CallValues& cv) { return new MoeRoute(cv); }

 private:
  int64_t dim_S_, dim_E_, dim_M_, dim_C_;
  int top_k_, gate_dtype_, device_id_;
  unsigned flags_;
  bool has_noise_ = false;
  void* ws_ = nullptr;
  size_t ws_bytes_ = 0;
  ScanWorkspaceState scan_ws_;
};

// moe_scatter_tokens(data [n, M], indices_locations [2, k*S_total], used_in [E], used_out [E], buffer [E, C, M],
//                    token_first, top_k=1, zero_tail=true): in place on `buffer`, which is also the output (the way
// lans aliases its tensor list, src/op/declare/optimizer.cc:46-62): every partition's call writes its own rows.
void MoeScatterTokensDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 6, "moe_scatter_tokens(data, indices_locations, used_in, used_out, buffer, token_first, top_k=1, zero_tail=true)");
  const Tensor& data = call.args[0].AsTensor();
  const Tensor& buf = call.args[4].AsTensor();
  RAF_CHECK(data.shape.size() == 2, "Input data should be 2-D.");
  RAF_CHECK(buf.shape.size() == 3 && buf.shape[2] == data.shape[1] && buf.dtype == data.dtype,
            "buffer must be [E, C, M] of the data's dtype");
  DTypeToLancet(data.dtype);
  const int64_t S_total = MaskTokens(call.args[1].AsTensor(), OptInt(call, 6, 1));
  const int64_t first = call.args[5].AsInt();
  RAF_CHECK(first >= 0 && first + data.shape[0] <= S_total, "token range outside the routed batch");
  call.out = call.args[4];  // in place
  call.device_id = data.device_id;
}

class MoeScatterTokens : public OpEnv {
 public:
  explicit MoeScatterTokens(const CallValues& cv) {
    const Tensor& data = cv.args[0].AsTensor();
    const Tensor& buf = cv.args[4].AsTensor();
    top_k_ = static_cast<int>(OptInt(cv, 6, 1));
    dim_S_total_ = MaskTokens(cv.args[1].AsTensor(), top_k_);
    n_tokens_ = data.shape[0], dim_M_ = data.shape[1];
    dim_E_ = buf.shape[0], dim_C_ = buf.shape[1];
    token_first_ = cv.args[5].AsInt();
    flags_ = OptInt(cv, 7, 1) ? 0u : LANCET_NO_TAIL_ZERO;
    for (int i : {2, 3})
      RAF_CHECK(IsI32(cv.args[i].AsTensor().dtype) && cv.args[i].AsTensor().numel() == dim_E_, "used capacities must be int32 [E]");
    dtype_ = DTypeToLancet(data.dtype);
    device_id_ = data.device_id;
    this->arg_indices = {0, 1, 2, 3, 4};
  }
  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1], cv.args[2], cv.args[3], cv.args[4]}, cv.out); }
  void Execute(const std::vector<Value>& inputs, Value /*output: the buffer itself*/) override {
    CheckStatus(lancet_moe_scatter_tokens(inputs[0].AsTensor().data, static_cast<const int32_t*>(inputs[1].AsTensor().data),
                                          static_cast<const int32_t*>(inputs[2].AsTensor().data),
                                          static_cast<const int32_t*>(inputs[3].AsTensor().data), dim_S_total_, token_first_,
                                          n_tokens_, dim_M_, dim_E_, dim_C_, top_k_, dtype_, flags_, inputs[4].AsTensor().data,
                                          GetStream(device_id_)),
                "lancet_moe_scatter_tokens");
  }
  std::string name() const override { return "raf.op.hip.moe_scatter_tokens"; }
  static OpEnv* make(const CallValues& cv) { return new MoeScatterTokens(cv); }

 private:
  int64_t dim_S_total_, n_tokens_, token_first_, dim_M_, dim_E_, dim_C_;
  int top_k_, dtype_, device_id_;
  unsigned flags_;
};

// moe_decode_tokens(data [E, C, M], gate [k*S_total], indices_locations [2, k*S_total], token_first, n_tokens, top_k=1)
void MoeDecodeTokensDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 5, "moe_decode_tokens(data, gate, indices_locations, token_first, n_tokens, top_k=1)");
  const Tensor& data = call.args[0].AsTensor();
  const Tensor& gate = call.args[1].AsTensor();
  RAF_CHECK(data.shape.size() == 3, "Input data should be 3-D.");
  RAF_CHECK(gate.shape.size() == 1, "Input gate should be 1-D.");
  DTypeToLancet(data.dtype);
  GateDTypeToLancet(gate.dtype);
  const int64_t k = OptInt(call, 5, 1);
  const int64_t S_total = MaskTokens(call.args[2].AsTensor(), k);
  RAF_CHECK(gate.shape[0] == k * S_total, "gate and indices_locations disagree on the token count");
  const int64_t first = call.args[3].AsInt(), n = call.args[4].AsInt();
  RAF_CHECK(first >= 0 && n >= 0 && first + n <= S_total, "token range outside the routed batch");
  call.out = Value::MakeTensor(MakeOut(data.device_id, data.dtype.code, data.dtype.bits, {n, data.shape[2]}));
  call.device_id = data.device_id;
}

class MoeDecodeTokens : public OpEnv {
 public:
  explicit MoeDecodeTokens(const CallValues& cv) {
    const Tensor& data = cv.args[0].AsTensor();
    top_k_ = static_cast<int>(OptInt(cv, 5, 1));
    dim_S_total_ = MaskTokens(cv.args[2].AsTensor(), top_k_);
    dim_E_ = data.shape[0], dim_C_ = data.shape[1], dim_M_ = data.shape[2];
    token_first_ = cv.args[3].AsInt(), n_tokens_ = cv.args[4].AsInt();
    dtype_ = DTypeToLancet(data.dtype);
    gate_dtype_ = GateDTypeToLancet(cv.args[1].AsTensor().dtype);
    device_id_ = data.device_id;
    this->arg_indices = {0, 1, 2};
  }
  void Execute(const CallValues& cv) override { Execute({cv.args[0], cv.args[1], cv.args[2]}, cv.out); }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    CheckStatus(lancet_moe_decode_tokens(inputs[0].AsTensor().data, inputs[1].AsTensor().data,
                                         static_cast<const int32_t*>(inputs[2].AsTensor().data), dim_S_total_, token_first_,
                                         n_tokens_, dim_M_, dim_E_, dim_C_, top_k_, dtype_, gate_dtype_,
                                         output.AsTensor().data, GetStream(device_id_)),
                "lancet_moe_decode_tokens");
  }
  std::string name() const override { return "raf.op.hip.moe_decode_tokens"; }
  static OpEnv* make(const CallValues& cv) { return new MoeDecodeTokens(cv); }

 private:
  int64_t dim_S_total_, n_tokens_, token_first_, dim_M_, dim_E_, dim_C_;
  int top_k_, dtype_, gate_dtype_, device_id_;
};

// moe_partition_ranges(indices_locations [2, k*S_total], n_partitions, n_experts, M, top_k=1) -> (starts, counts),
// uint64 [k*P, E] in elements: what the partitions' exchanges (sparse copies on row ranges, all-to-allv counts) take
void MoePartitionRangesDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() >= 4, "moe_partition_ranges(indices_locations, n_partitions, n_experts, M, top_k=1)");
  const Tensor& il = call.args[0].AsTensor();
  const int64_t k = OptInt(call, 4, 1);
  const int64_t S_total = MaskTokens(il, k);
  const int64_t P = call.args[1].AsInt(), E = call.args[2].AsInt();
  RAF_CHECK(P >= 1 && S_total % P == 0 && k * P <= LANCET_MAX_PARTITIONS, "the token count must divide into n_partitions");
  RAF_CHECK(E >= 1, "n_experts must be positive");
  std::vector<Value> ret;
  for (int i = 0; i < 2; ++i) ret.push_back(Value::MakeTensor(MakeOut(il.device_id, DTypeCode::kUInt, 64, {k * P, E})));
  call.out = Value::MakeTuple(std::move(ret));
  call.device_id = il.device_id;
}

class MoePartitionRanges : public OpEnv {
 public:
  explicit MoePartitionRanges(const CallValues& cv) {
    const Tensor& il = cv.args[0].AsTensor();
    top_k_ = static_cast<int>(OptInt(cv, 4, 1));
    dim_S_total_ = MaskTokens(il, top_k_);
    n_partitions_ = static_cast<int>(cv.args[1].AsInt());
    dim_E_ = cv.args[2].AsInt();
    dim_M_ = cv.args[3].AsInt();
    device_id_ = il.device_id;
    ws_bytes_ = lancet_moe_partition_ranges_workspace_bytes(top_k_, n_partitions_, dim_E_);
    RequestWorkspace(&ws_, device_id_, static_cast<int64_t>(ws_bytes_));
    this->arg_indices = {0};
  }
  void Execute(const CallValues& cv) override { Execute({cv.args[0]}, cv.out); }
  void Execute(const std::vector<Value>& inputs, Value output) override {
    const auto& out = output.AsTuple();
    RAF_CHECK(out.size() == 2, "Expected output to be a 2-Tuple");
    CheckStatus(lancet_moe_partition_ranges(static_cast<const int32_t*>(inputs[0].AsTensor().data), dim_S_total_, top_k_,
                                            n_partitions_, dim_E_, dim_M_, static_cast<uint64_t*>(out[0].AsTensor().data),
                                            static_cast<uint64_t*>(out[1].AsTensor().data), ws_, ws_bytes_,
                                            GetStream(device_id_)),
                "lancet_moe_partition_ranges");
  }
  std::string name() const override { return "raf.op.hip.moe_partition_ranges"; }
  static OpEnv* make(const CallValues& cv) { return new MoePartitionRanges(cv); }

 private:
  int64_t dim_S_total_, dim_E_, dim_M_;
  int top_k_, n_partitions_, device_id_;
  void* ws_ = nullptr;
  size_t ws_bytes_ = 0;
};

// ---- registration (cuda/cuda_utils.cc:17; cuda/moe.cc:411-412,728-729,822-823,942-943,1310-1311) ----
RAF_REGISTER_DIALECT("hip").set_enable("hip");

RAF_OP_DECLARE("raf.op.moe_encode", MoeEncodeDeclare);
RAF_OP_DECLARE("raf.op.moe_encode_batch_prioritized", MoeEncodeBatchPrioritizedDeclare);
RAF_OP_DECLARE("raf.op.moe_merge_masks", MoeMergeMasksDeclare);
RAF_OP_DECLARE("raf.op.moe_redispatch", MoeRedispatchDeclare);
RAF_OP_DECLARE("raf.op.moe_decode", MoeDecodeDeclare);

RAF_REGISTER_DIALECT_OP(hip, moe_encode, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_encode", MoeEncode::make);
RAF_REGISTER_DIALECT_OP(hip, moe_encode_batch_prioritized, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_encode_batch_prioritized", MoeEncodeBatchPrioritized::make);
RAF_REGISTER_DIALECT_OP(hip, moe_merge_masks, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_merge_masks", MoeMergeMasks::make);
RAF_REGISTER_DIALECT_OP(hip, moe_redispatch, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_redispatch", MoeRedispatch::make);
RAF_REGISTER_DIALECT_OP(hip, moe_decode, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_decode", MoeDecode::make);

RAF_OP_DECLARE("raf.op.moe_redispatch_expert_input", MoeRedispatchExpertInputDeclare);
RAF_REGISTER_DIALECT_OP(hip, moe_redispatch_expert_input, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_redispatch_expert_input", MoeRedispatchExpertInput::make);
RAF_OP_DECLARE("raf.op.moe_encode_dx", MoeEncodeDxDeclare);
RAF_OP_DECLARE("raf.op.moe_encode_dg", MoeEncodeDgDeclare);
RAF_OP_DECLARE("raf.op.moe_decode_dx", MoeDecodeDxDeclare);
RAF_OP_DECLARE("raf.op.moe_decode_dg", MoeDecodeDgDeclare);
RAF_REGISTER_DIALECT_OP(hip, moe_encode_dx, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_encode_dx", MoeEncodeDx::make);
RAF_REGISTER_DIALECT_OP(hip, moe_encode_dg, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_encode_dg", MoeEncodeDg::make);
RAF_REGISTER_DIALECT_OP(hip, moe_decode_dx, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_decode_dx", MoeDecodeDx::make);
RAF_REGISTER_DIALECT_OP(hip, moe_decode_dg, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_decode_dg", MoeDecodeDg::make);
// no base op of these names exists in the reference: they are what a graph rewrite for this dialect introduces
RAF_OP_DECLARE("raf.op.moe_encode_dgate", MoeEncodeDgateDeclare);
RAF_REGISTER_DIALECT_OP(hip, moe_encode_dgate, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_encode_dgate", MoeEncodeDgate::make);
RAF_OP_DECLARE("raf.op.moe_route", MoeRouteDeclare);
RAF_REGISTER_DIALECT_OP(hip, moe_route, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_route", MoeRoute::make);
RAF_OP_DECLARE("raf.op.moe_scatter_tokens", MoeScatterTokensDeclare);
RAF_REGISTER_DIALECT_OP(hip, moe_scatter_tokens, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_scatter_tokens", MoeScatterTokens::make);
RAF_OP_DECLARE("raf.op.moe_decode_tokens", MoeDecodeTokensDeclare);
RAF_REGISTER_DIALECT_OP(hip, moe_decode_tokens, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_decode_tokens", MoeDecodeTokens::make);
RAF_OP_DECLARE("raf.op.moe_partition_ranges", MoePartitionRangesDeclare);
RAF_REGISTER_DIALECT_OP(hip, moe_partition_ranges, 20);
RAF_OP_ENV_MAKER("raf.op.hip.moe_partition_ranges", MoePartitionRanges::make);

}  // namespace hip
}  // namespace op
}  // namespace raf
