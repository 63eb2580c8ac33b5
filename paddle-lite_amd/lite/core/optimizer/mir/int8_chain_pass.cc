#include "lite/core/optimizer/mir/int8_chain_pass.h"

#include <map>

#include "lite/core/op_registry.h"

namespace paddle {
namespace lite {
namespace mir {
namespace {

struct VarState {
  bool on_device = false;
  bool int8 = false;
  std::string name;  // variable that currently holds the value
};

bool IsInt8Op(const OpInfo& op) { return op.HasAttr("enable_int8") && op.GetAttr<bool>("enable_int8"); }

ProgramStep IoCopy(const std::string& from, const std::string& to, bool to_device) {
  ProgramStep s;
  s.op = OpInfo("io_copy");
  s.op.SetInput("Input", {from});
  s.op.SetOutput("Out", {to});
  s.kernel = to_device ? "io_copy/host_to_device" : "io_copy/device_to_host";
  s.place = lite_api::Place(TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny));
  return s;
}

ProgramStep Calib(const std::string& from, const std::string& to, float scale, bool to_int8) {
  ProgramStep s;
  s.op = OpInfo("calib");
  s.op.SetInput("Input", {from});
  s.op.SetOutput("Out", {to});
  s.op.SetAttr<float>("scale", scale);
  s.kernel = to_int8 ? "calib/fp32_to_int8" : "calib/int8_to_fp32";
  s.place = lite_api::Place(TARGET(kHIP), PRECISION(kInt8), DATALAYOUT(kNCHW));
  return s;
}

}  // namespace

std::vector<ProgramStep> Int8ChainPass::Apply(const std::vector<OpInfo>& ops, const std::vector<std::string>& feeds, const std::vector<std::string>& fetches, Scope* scope) const {
  std::vector<ProgramStep> steps;
  std::map<std::string, VarState> vars;
  for (const std::string& f : feeds) {
    CHECK(scope->FindVar(f) != nullptr) << "feed " << f << " is not in the scope";
    vars[f] = VarState{false, false, f};
  }
  auto is_fetch = [&](const std::string& v) { return std::find(fetches.begin(), fetches.end(), v) != fetches.end(); };

  for (size_t i = 0; i < ops.size(); ++i) {
    OpInfo op = ops[i];
    const bool depthwise = op.Type() == "depthwise_conv2d";
    CHECK(op.Type() == "sparse_conv2d" || depthwise) << "this pass handles chains of sparse_conv2d and depthwise_conv2d, got " << op.Type();
    const bool int8 = IsInt8Op(op);
    CHECK(int8 || !depthwise) << "depthwise_conv2d has int8 kernels only on this target";
    const std::string in = op.Input("Input").front();
    const std::string out = op.Output("Output").front();
    CHECK(vars.count(in) != 0) << "input " << in << " of op " << i << " has no producer and is not fed";

    // output type: int8 only if the value is consumed, only by int8 ops, and
    // not wanted by the caller
    bool out_int8 = int8 && !is_fetch(out);
    bool consumed = false;
    float consumer_scale = 1.f;
    for (size_t j = i + 1; j < ops.size() && out_int8; ++j) {
      if (ops[j].Input("Input").front() != out) continue;
      if (!IsInt8Op(ops[j])) {
        out_int8 = false;
        break;
      }
      CHECK(ops[j].HasInputScale("Input0_scale", true)) << "int8 consumer without an input scale";
      if (!consumed) consumer_scale = ops[j].GetInputScale("Input0_scale", true)[0];
      consumed = true;
    }
    out_int8 = out_int8 && consumed;
    if (out_int8) op.SetOutputScale("Output0_scale", {consumer_scale}, true);

    // bring the input where and how the kernel declares it
    VarState cur = vars[in];
    if (!cur.on_device) {
      const std::string dev = cur.name + "/hip";
      steps.push_back(IoCopy(cur.name, dev, true));
      cur.on_device = true;
      cur.name = dev;
    }
    if (int8 && !cur.int8) {
      CHECK(op.HasInputScale("Input0_scale", true)) << "int8 op without an input scale";
      const std::string q = cur.name + "/int8";
      steps.push_back(Calib(cur.name, q, op.GetInputScale("Input0_scale", true)[0], true));
      cur.int8 = true;
      cur.name = q;
    } else if (!int8 && cur.int8) {
      LOG(FATAL) << "an fp32 op consumes the int8 output of op " << in << ": the output-type rule forbids it";
    }
    vars[in] = cur;  // later consumers of the same variable reuse the casts
    op.SetInput("Input", {cur.name});

    ProgramStep s;
    s.op = op;
    // aliases as the reference registers them (sparse_conv_compute.cc:393-430, conv_compute.cc:252-300)
    s.kernel = depthwise ? std::string("depthwise_conv2d/") + (out_int8 ? "int8_out" : "fp32_out")
                         : std::string("sparse_conv2d/") + (!int8 ? "def" : (out_int8 ? "int8_int8_out" : "int8_fp32_out"));
    s.place = lite_api::Place(TARGET(kHIP), int8 ? PRECISION(kInt8) : PRECISION(kFloat), DATALAYOUT(kNCHW));
    steps.push_back(s);
    vars[out] = VarState{true, out_int8, out};
  }
  for (const std::string& f : fetches) {
    CHECK(vars.count(f) != 0) << "fetch " << f << " is never produced";
    const VarState& v = vars[f];
    CHECK(!v.int8) << "a fetched variable is fp32 by the output-type rule";
    if (v.on_device) steps.push_back(IoCopy(v.name, f + "/host", false));
  }
  return steps;
}

HipProgram::HipProgram(const std::vector<ProgramStep>& steps, Scope* scope) {
  for (const ProgramStep& s : steps) {
    for (const auto& kv : s.op.outputs())
      for (const std::string& name : kv.second) scope->Var(name);
    auto op = LiteOpRegistry::Global().Create(s.op.Type());
    CHECK(op != nullptr) << "no op " << s.op.Type();
    CHECK(op->Attach(s.op, scope)) << "attach failed for " << s.op.Type();
    auto ks = op->CreateKernels({s.place}, s.kernel);
    CHECK(ks.size() == 1) << "expected one kernel for " << s.kernel << ", found " << ks.size();
    ops_.emplace_back(std::move(op));
    kernels_.emplace_back(std::move(ks[0]));
  }
}

void HipProgram::Run() {
  for (size_t i = 0; i < kernels_.size(); ++i) {
    CHECK(ops_[i]->CheckShape()) << "shape check failed at step " << i;
    CHECK(ops_[i]->InferShape()) << "shape inference failed at step " << i;
    kernels_[i]->Launch();
  }
  if (!kernels_.empty()) kernels_.back()->mutable_context_as<HIPContext>()->Sync();
}

}  // namespace mir
}  // namespace lite
}  // namespace paddle
