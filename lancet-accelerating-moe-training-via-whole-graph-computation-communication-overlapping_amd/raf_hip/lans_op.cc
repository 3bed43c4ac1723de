// raf.op.lans in the "hip" dialect.  Counterparts in the reference: LansDecl
// (src/op/declare/optimizer.cc:46-62: the output tuple aliases the 4T input tensors, in place)
// and LansImpl (src/op/dialect/cuda/lans.cc:26-180).
//
// The constructor captures hyper-parameters and tensor sizes and creates the native plan (chunk
// tables, partial sums, norm vectors): this replaces the q workspace of sum(numel) floats, the
// per-chunk partials and the four norm vectors the reference requests (lans.cc:56-82); the update
// vectors are recomputed instead of stored, so there is no q buffer and none of its offset
// arithmetic (lans.cc:126-129).  The step scalar is read on the device (no host synchronisation,
// unlike lans.cc:102-107); a host integer is accepted as well.
//
// Trailing extension for a 16-bit model (argument 11, optional): a tuple of T bfloat16 / float16 tensors that
// receive the new parameters rounded to that type, and the gradient quarter of tensor_list may then be (or be
// anyway) bfloat16 / float16: the casts the reference's traced optimizer puts around the op
// (python/raf/optim/lans.py:256-257, 285-288) happen inside the step.
#include <string>
#include <vector>

#include "lancet_hip.h"
#include <cstdlib>
#include <cstring>

#include "op.h"

namespace raf {
namespace op {
namespace hip {

void LansDeclare(CallValues& call) {
  RAF_CHECK(call.args.size() == 11 || call.args.size() == 12,
            "lans(tensor_list, step, learning_rate, beta1, beta2, eps, bias_correction, weight_decay, "
            "grad_averaging, mode, normalize_grad, p_lowp=None)");
  const auto& list = call.args[0].AsTuple();
  RAF_CHECK(!list.empty() && list.size() % 4 == 0, "tensor_list must hold 4 lists of equal length");
  call.device_id = list[0].AsTensor().device_id;
  call.out = Value::MakeTuple(list);  // in place: outputs alias the inputs
}

class LansImpl : public OpEnv {
 public:
  explicit LansImpl(const CallValues& cv) {
    const auto& list = cv.args[0].AsTuple();
    RAF_CHECK(!list.empty() && list.size() % 4 == 0, "tensor_list must hold 4 lists of equal length");
    const Tensor& t0 = list[0].AsTensor();
    param_group_n_ = static_cast<int>(list.size() / 4);
    // parameters and moments are float32 (the reference's fp16 path is a LOG(FATAL), lans.cc:143-146); the
    // gradients may have the type of a 16-bit model
    g_dtype_ = HalfOrFloat(t0.dtype, "gradients must be float32, bfloat16 or float16");
    for (size_t i = 0; i < list.size(); ++i) {
      const DType& dt = list[i].AsTensor().dtype;
      if (static_cast<int>(i) < param_group_n_) RAF_CHECK(dt == t0.dtype, "every gradient must have one dtype");
      else RAF_CHECK(dt.code == DTypeCode::kFloat && dt.bits == 32, "parameters and moments must be float32");
    }
    has_lowp_ = cv.args.size() > 11 && cv.args[11].kind == Value::kTuple;
    if (has_lowp_) {
      const auto& low = cv.args[11].AsTuple();
      RAF_CHECK(static_cast<int>(low.size()) == param_group_n_, "p_lowp must hold one tensor per parameter");
      lowp_dtype_ = HalfOrFloat(low[0].AsTensor().dtype, "p_lowp must be bfloat16 or float16");
      RAF_CHECK(lowp_dtype_ != LANCET_F32, "p_lowp must be bfloat16 or float16");
      for (int i = 0; i < param_group_n_; ++i)
        RAF_CHECK(low[i].AsTensor().dtype == low[0].AsTensor().dtype && low[i].AsTensor().numel() == list[i].AsTensor().numel(),
                  "p_lowp must match the parameters in size and share one 16-bit dtype");
    }
    hyper_.learning_rate = static_cast<float>(cv.args[2].AsFloat());
    hyper_.beta1 = static_cast<float>(cv.args[3].AsFloat());
    hyper_.beta2 = static_cast<float>(cv.args[4].AsFloat());
    hyper_.eps = static_cast<float>(cv.args[5].AsFloat());
    hyper_.bias_correction = static_cast<int>(cv.args[6].AsInt());
    hyper_.weight_decay = static_cast<float>(cv.args[7].AsFloat());
    hyper_.grad_averaging = static_cast<int>(cv.args[8].AsInt());
    hyper_.mode = static_cast<int>(cv.args[9].AsInt());
    hyper_.normalize_grad = cv.args[10].AsInt() != 0;
    for (int i = 0; i < param_group_n_; ++i) numels_.push_back(list[i].AsTensor().numel());
    for (int q = 1; q < 4; ++q)
      for (int i = 0; i < param_group_n_; ++i)
        RAF_CHECK(list[q * param_group_n_ + i].AsTensor().numel() == numels_[i], "the four lists must have matching sizes");
    device_id_ = t0.device_id;
    int st = lancet_lans_plan_create(numels_.data(), param_group_n_, &plan_);
    if (st != LANCET_OK) throw Error(std::string("lancet_lans_plan_create failed: ") + lancet_status_string(st));
    // a new plan runs the one-kernel schedule for every tensor that fits it; LANCET_LANS_SCHEDULE=sweeps
    // asks for the three sweeps (a device shared with kernels of unbounded duration)
    const char* schedule = std::getenv("LANCET_LANS_SCHEDULE");
    if (schedule && std::strcmp(schedule, "sweeps") == 0) (void)lancet_lans_plan_set_schedule(plan_, LANCET_LANS_SWEEPS);
    this->arg_indices = {0, 1};  // tensor_list, step
    if (has_lowp_) this->arg_indices.push_back(11);
  }

  ~LansImpl() override {
    if (plan_) lancet_lans_plan_destroy(plan_);
  }

  void Execute(const CallValues& cv) override {
    std::vector<Value> inputs = {cv.args[0], cv.args[1]};
    if (has_lowp_) inputs.push_back(cv.args[11]);
    Execute(inputs, cv.out);
  }

  void Execute(const std::vector<Value>& inputs, Value /*output*/) override {
    const auto& list = inputs[0].AsTuple();
    RAF_CHECK(static_cast<int>(list.size()) == 4 * param_group_n_, "tensor_list length changed");
    std::vector<float*> ptrs;
    for (const auto& v : list) ptrs.push_back(static_cast<float*>(v.AsTensor().data));
    const int n = param_group_n_;
    std::vector<void*> low;
    if (has_lowp_) {
      RAF_CHECK(inputs.size() > 2 && static_cast<int>(inputs[2].AsTuple().size()) == n, "p_lowp length changed");
      for (const auto& v : inputs[2].AsTuple()) low.push_back(v.AsTensor().data);
    }
    int step_host = 0;
    const float* step_dev = nullptr;
    if (inputs[1].kind == Value::kTensor) {
      const Tensor& ts = inputs[1].AsTensor();
      RAF_CHECK(ts.numel() == 1 && ts.dtype.code == DTypeCode::kFloat && ts.dtype.bits == 32,
                "step must be a float32 scalar tensor");
      step_dev = static_cast<const float*>(ts.data);
    } else {
      step_host = static_cast<int>(inputs[1].AsInt());
    }
    int st;
    if (g_dtype_ == LANCET_F32 && !has_lowp_)
      st = lancet_lans_step(plan_, ptrs.data(), ptrs.data() + n, ptrs.data() + 2 * n, ptrs.data() + 3 * n,
                            step_host, step_dev, &hyper_, /*grad_norms=*/nullptr, GetStream(device_id_));
    else
      st = lancet_lans_step_mixed(plan_, reinterpret_cast<const void* const*>(ptrs.data()), g_dtype_, ptrs.data() + n,
                                  ptrs.data() + 2 * n, ptrs.data() + 3 * n, has_lowp_ ? low.data() : nullptr, lowp_dtype_,
                                  step_host, step_dev, &hyper_, /*grad_norms=*/nullptr, GetStream(device_id_));
    if (st != LANCET_OK)
      throw Error(std::string("lancet_lans_step failed: ") + lancet_status_string(st) + " (status " + std::to_string(st) + ")");
  }

  void CheckDeviceStatus(void* stream) override {
    int err = 0;
    int st = lancet_lans_plan_error(plan_, stream, &err);
    if (st != LANCET_OK) throw Error(std::string("lancet_lans_plan_error failed: ") + lancet_status_string(st));
    if (err) throw Error("lans: a step of the resident schedule gave up a wait; the parameters of that step were left unwritten");
  }

  std::string name() const override { return "raf.op.hip.lans"; }
  static OpEnv* make(const CallValues& cv) { return new LansImpl(cv); }

 private:
  static int HalfOrFloat(const DType& dt, const char* what) {
    if (dt.code == DTypeCode::kFloat && dt.bits == 32) return LANCET_F32;
    if (dt.code == DTypeCode::kFloat && dt.bits == 16) return LANCET_F16;
    if (dt.code == DTypeCode::kBFloat && dt.bits == 16) return LANCET_BF16;
    throw Error(what);
  }
  int g_dtype_ = LANCET_F32, lowp_dtype_ = LANCET_BF16;
  bool has_lowp_ = false;
  lancet_lans_hyper hyper_;
  std::vector<int64_t> numels_;
  int param_group_n_ = 0;
  int device_id_ = 0;
  lancet_lans_plan_t plan_ = nullptr;
};

RAF_OP_DECLARE("raf.op.lans", LansDeclare);
RAF_REGISTER_DIALECT_OP(hip, lans, 20);
RAF_OP_ENV_MAKER("raf.op.hip.lans", LansImpl::make);

}  // namespace hip
}  // namespace op
}  // namespace raf
