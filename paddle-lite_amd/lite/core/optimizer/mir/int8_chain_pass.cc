#include "lite/core/optimizer/mir/int8_chain_pass.h"

#include "lite/kernels/hip/pair_launch.h"
#include "pl_sparse_conv.h"

#include <algorithm>
#include <map>

#include "lite/core/op_registry.h"

namespace paddle {
namespace lite {
namespace mir {
namespace {

// Where the value of a variable can be read from: the host tensor (feeds),
// the fp32 tensor on the device, and int8 tensors on the device, one per
// quantisation scale that a consumer asked for.
struct VarState {
  std::string host;
  std::string dev_fp32;
  std::map<float, std::string> dev_int8;
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
  const Graph graph(ops, *scope);
  return Apply(graph, feeds, fetches, scope);
}

std::vector<ProgramStep> Int8ChainPass::Apply(const Graph& graph, const std::vector<std::string>& feeds, const std::vector<std::string>& fetches, Scope* scope) const {
  std::vector<ProgramStep> steps;
  std::map<std::string, VarState> vars;
  for (const std::string& f : feeds) {
    CHECK(scope->FindVar(f) != nullptr) << "feed " << f << " is not in the scope";
    vars[f].host = f;
  }
  auto is_fetch = [&](const std::string& v) { return std::find(fetches.begin(), fetches.end(), v) != fetches.end(); };

  const std::vector<OpInfo> ops = graph.TopologicalOps();
  for (size_t i = 0; i < ops.size(); ++i) {
    OpInfo op = ops[i];
    const bool depthwise = op.Type() == "depthwise_conv2d";
    CHECK(op.Type() == "sparse_conv2d" || depthwise) << "this pass handles graphs of sparse_conv2d and depthwise_conv2d, got " << op.Type();
    const bool int8 = IsInt8Op(op);
    CHECK(int8 || !depthwise) << "depthwise_conv2d has int8 kernels only on this target";
    const std::string in = op.Input("Input").front();
    const std::string out = op.Output("Output").front();
    CHECK(vars.count(in) != 0) << "input " << in << " of op " << i << " has no producer and is not fed";

    // Output type (static_kernel_pick_pass.cc:97-135): int8 only if the
    // value is consumed, by int8 ops only, and not wanted by the caller; the
    // output scale is then the consumers' input scale.  Consumers that
    // disagree on that scale cannot share one int8 tensor: the op then
    // produces fp32 and each consumer gets its own calib.
    bool out_int8 = int8 && !is_fetch(out);
    bool consumed = false;
    float consumer_scale = 1.f;
    for (const Graph::Node* consumer : graph.Consumers(out)) {
      if (!out_int8) break;
      const OpInfo& c = consumer->op;
      if (!c.HasInput("Input") || c.Input("Input").front() != out || !IsInt8Op(c)) {
        out_int8 = false;  // read as something else than an int8 activation
        break;
      }
      CHECK(c.HasInputScale("Input0_scale", true)) << "int8 consumer without an input scale";
      const float sc = c.GetInputScale("Input0_scale", true)[0];
      if (consumed && sc != consumer_scale) out_int8 = false;
      consumer_scale = sc;
      consumed = true;
    }
    out_int8 = out_int8 && consumed;
    if (out_int8) op.SetOutputScale("Output0_scale", {consumer_scale}, true);

    // bring the input where and how the kernel declares it; later consumers
    // of the same variable reuse the copies and casts made here
    VarState& cur = vars[in];
    std::string src;
    if (int8) {
      CHECK(op.HasInputScale("Input0_scale", true)) << "int8 op without an input scale";
      const float sc = op.GetInputScale("Input0_scale", true)[0];
      auto q = cur.dev_int8.find(sc);
      if (q == cur.dev_int8.end()) {
        CHECK(cur.dev_int8.empty() || !cur.dev_fp32.empty() || !cur.host.empty())
            << "variable " << in << " exists as int8 with another scale only: the output-type rule forbids it";
        if (cur.dev_fp32.empty()) {
          CHECK(!cur.host.empty()) << "variable " << in << " has no fp32 form to quantise";
          cur.dev_fp32 = cur.host + "/hip";
          steps.push_back(IoCopy(cur.host, cur.dev_fp32, true));
        }
        const std::string name = cur.dev_fp32 + (cur.dev_int8.empty() ? "/int8" : "/int8_" + std::to_string(cur.dev_int8.size()));
        steps.push_back(Calib(cur.dev_fp32, name, sc, true));
        q = cur.dev_int8.emplace(sc, name).first;
      }
      src = q->second;
    } else {
      if (cur.dev_fp32.empty()) {
        CHECK(!cur.host.empty()) << "an fp32 op consumes variable " << in << ", which exists as int8 only: the output-type rule forbids it";
        cur.dev_fp32 = cur.host + "/hip";
        steps.push_back(IoCopy(cur.host, cur.dev_fp32, true));
      }
      src = cur.dev_fp32;
    }
    op.SetInput("Input", {src});

    ProgramStep s;
    s.op = op;
    // aliases as the reference registers them (sparse_conv_compute.cc:393-430, conv_compute.cc:252-300)
    s.kernel = depthwise ? std::string("depthwise_conv2d/") + (out_int8 ? "int8_out" : "fp32_out")
                         : std::string("sparse_conv2d/") + (!int8 ? "def" : (out_int8 ? "int8_int8_out" : "int8_fp32_out"));
    s.place = lite_api::Place(TARGET(kHIP), int8 ? PRECISION(kInt8) : PRECISION(kFloat), DATALAYOUT(kNCHW));
    steps.push_back(s);
    VarState& produced = vars[out];
    if (out_int8) {
      produced.dev_int8[consumer_scale] = out;
    } else {
      produced.dev_fp32 = out;
    }
  }
  for (const std::string& f : fetches) {
    CHECK(vars.count(f) != 0) << "fetch " << f << " is never produced";
    const VarState& v = vars[f];
    if (!v.host.empty()) continue;  // a feed wanted back: already on the host
    CHECK(!v.dev_fp32.empty()) << "a fetched variable is fp32 by the output-type rule";
    steps.push_back(IoCopy(v.dev_fp32, f + "/host", false));
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
  // which steps hand their output to the next step alone
  only_reader_is_next_.assign(steps.size(), 0);
  for (size_t i = 0; i + 1 < steps.size(); ++i) {
    std::vector<std::string> outs;
    for (const auto& kv : steps[i].op.outputs()) outs.insert(outs.end(), kv.second.begin(), kv.second.end());
    if (outs.size() != 1) continue;
    size_t readers = 0;
    bool next_reads = false;
    for (size_t j = 0; j < steps.size(); ++j)
      for (const auto& kv : steps[j].op.inputs())
        for (const std::string& name : kv.second)
          if (name == outs[0]) {
            ++readers;
            if (j == i + 1) next_reads = true;
          }
    only_reader_is_next_[i] = readers == 1 && next_reads;
  }
}

void HipProgram::Enqueue(size_t first, size_t last) {
  CHECK(first <= last && last <= kernels_.size()) << "steps " << first << " .. " << last << " of " << kernels_.size();
  pairs_joined_ = 0;
  for (size_t i = first; i < last; ++i) {
    CHECK(ops_[i]->CheckShape()) << "shape check failed at step " << i;
    CHECK(ops_[i]->InferShape()) << "shape inference failed at step " << i;
    if (pair_launch_ && i + 1 < last && only_reader_is_next_[i]) {
      auto* a = dynamic_cast<kernels::hip::PairLaunch*>(kernels_[i].get());
      auto* b = dynamic_cast<kernels::hip::PairLaunch*>(kernels_[i + 1].get());
      if (a && b && a->pair_role() == kernels::hip::PairLaunch::kFirst && b->pair_role() == kernels::hip::PairLaunch::kSecond) {
        CHECK(ops_[i + 1]->CheckShape()) << "shape check failed at step " << i + 1;
        CHECK(ops_[i + 1]->InferShape()) << "shape inference failed at step " << i + 1;
        kernels::hip::PairEndpoint ea, eb;
        if (a->pair_endpoint(&ea) && b->pair_endpoint(&eb) && eb.x == ea.out && ea.stream == eb.stream &&
            pl_sparse_conv_dwconv3x3_pays(static_cast<pl_sparse_conv_handle*>(ea.handle), static_cast<pl_dwconv_handle*>(eb.handle), ea.batch, ea.h, ea.w)) {
          const int rc = pl_sparse_conv_dwconv3x3_run(static_cast<pl_sparse_conv_handle*>(ea.handle), static_cast<pl_dwconv_handle*>(eb.handle), ea.x, eb.out, ea.batch, ea.h, ea.w, ea.stream);
          if (rc != PL_OK) LOG(FATAL) << "pl_sparse_conv_dwconv3x3_run failed (" << rc << "): " << pl_last_error();
          ++pairs_joined_;
          ++i;  // the depthwise step ran with this one
          continue;
        }
      }
    }
    kernels_[i]->Launch();
  }
}

void HipProgram::Sync() {
  if (!kernels_.empty()) kernels_.back()->mutable_context_as<HIPContext>()->Sync();
}

void HipProgram::Run() {
  Enqueue(0, kernels_.size());
  Sync();
}

}  // namespace mir
}  // namespace lite
}  // namespace paddle
