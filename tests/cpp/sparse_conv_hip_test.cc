// Host-side test of the Lite surface for sparse_conv2d on TARGET(kHIP), in the
// shape of the reference's math tests (lite/tests/math/
// sparse_conv_{f32,int8}_compute_test.cc: fill, mask, pack, run, compare with
// the naive dense reference) but through the whole op path the reference never
// tests: detect pass -> SparseConvOp::Attach/InferShape -> registered kernel
// -> Launch.  Seeds are fixed.
//
//   sparse_conv_hip_test --cpu   registry, op, pass and error paths (no device)
//   sparse_conv_hip_test --gpu   the above plus execution on the device
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <unistd.h>
#include <string>
#include <vector>

#include "lite/core/op_registry.h"
#include "lite/core/optimizer/mir/graph.h"
#include "lite/core/optimizer/mir/int8_chain_pass.h"
#include "lite/core/optimizer/mir/sparse_conv_detect_pass.h"
#include "lite/kernels/hip/sparse_conv_compute.h"
#include "lite/model_parser/model_parser.h"
#include "lite/operators/conv_op.h"
#include "lite/operators/sparse_conv_op.h"
#include "pl_sparse_conv.h"
#include "sparse_conv_oracle.h"

using namespace paddle::lite;  // NOLINT

static int g_failures = 0;
#define EXPECT(cond)                                                   \
  do {                                                                 \
    if (!(cond)) {                                                     \
      std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
      ++g_failures;                                                    \
    }                                                                  \
  } while (0)

// true when f() raises a FatalError whose text contains `what`
template <typename F>
static bool ThrowsWith(const char* what, F f) {
  try {
    f();
  } catch (const FatalError& e) {
    return std::string(e.what()).find(what) != std::string::npos;
  }
  return false;
}

template <typename F>
static bool Throws(F f) {
  try {
    f();
  } catch (const FatalError&) {
    return true;
  }
  return false;
}

struct Problem {
  int batch, ic, oc, h, w;
  float sparsity;
  bool paired, int8, out_int8, bias;
  std::string act;  // "", relu, relu6, leaky_relu, hard_swish
  unsigned seed;
};

// Builds a scope holding a conv2d (Input, Filter, Bias) and its op description.
static OpInfo MakeConv(const Problem& p, Scope* scope, std::vector<float>* ws, float* in_scale, float* out_scale) {
  std::mt19937 gen(p.seed);
  std::uniform_real_distribution<float> uni(0.f, 1.f);
  std::normal_distribution<float> nrm(0.f, 1.f);
  Tensor* x = scope->NewTensor("x");
  Tensor* w = scope->NewTensor("conv_w");
  x->Resize({p.batch, p.ic, p.h, p.w});
  w->Resize({p.oc, p.ic, 1, 1});
  std::vector<char> keep(static_cast<size_t>(p.oc) * p.ic);
  for (int r = 0; r < p.oc; ++r)
    for (int c = 0; c < p.ic; ++c) {
      if (p.paired && (r & 1)) {
        keep[r * p.ic + c] = keep[(r - 1) * p.ic + c];
      } else {
        keep[r * p.ic + c] = uni(gen) >= p.sparsity;
      }
    }
  if (p.int8) {
    int8_t* xd = x->mutable_data<int8_t>(TargetType::kHost);
    for (int64_t i = 0; i < x->numel(); ++i) xd[i] = static_cast<int8_t>(static_cast<int>(uni(gen) * 255.f) - 127);
    int8_t* wd = w->mutable_data<int8_t>(TargetType::kHost);
    for (int64_t i = 0; i < w->numel(); ++i) {
      int v = static_cast<int>(uni(gen) * 127.f) + 1;
      if (uni(gen) < 0.5f) v = -v;
      wd[i] = keep[i] ? static_cast<int8_t>(v) : 0;
    }
  } else {
    float* xd = x->mutable_data<float>(TargetType::kHost);
    for (int64_t i = 0; i < x->numel(); ++i) xd[i] = uni(gen) * 2.f - 1.f;
    float* wd = w->mutable_data<float>(TargetType::kHost);
    for (int64_t i = 0; i < w->numel(); ++i) {
      float v = nrm(gen) * 0.1f;
      wd[i] = keep[i] ? (v == 0.f ? 0.1f : v) : 0.f;
    }
  }
  OpInfo conv("conv2d");
  conv.SetInput("Input", {"x"});
  conv.SetInput("Filter", {"conv_w"});
  if (p.bias) {
    Tensor* b = scope->NewTensor("conv_b");
    b->Resize({p.oc});
    float* bd = b->mutable_data<float>(TargetType::kHost);
    for (int i = 0; i < p.oc; ++i) bd[i] = nrm(gen) * 0.1f;
    conv.SetInput("Bias", {"conv_b"});
  }
  conv.SetOutput("Output", {"y"});
  scope->NewTensor("y");
  conv.SetAttr<std::vector<int>>("strides", {1, 1});
  conv.SetAttr<std::vector<int>>("paddings", {0, 0});
  conv.SetAttr<std::vector<int>>("dilations", {1, 1});
  conv.SetAttr<int>("groups", 1);
  if (!p.act.empty()) {
    conv.SetAttr<bool>("with_act", true);
    conv.SetAttr<std::string>("act_type", p.act);
    conv.SetAttr<float>("fuse_brelu_threshold", 6.f);
    conv.SetAttr<float>("leaky_relu_alpha", 0.1f);
    conv.SetAttr<float>("hard_swish_threshold", 6.f);
    conv.SetAttr<float>("hard_swish_scale", 6.f);
    conv.SetAttr<float>("hard_swish_offset", 3.f);
  }
  if (p.int8) {
    ws->resize(p.oc);
    for (float& s : *ws) s = 0.001f + 0.019f * uni(gen);
    *in_scale = 0.01f;
    *out_scale = p.out_int8 ? 0.05f : 1.f;
    conv.SetAttr<bool>("enable_int8", true);
    conv.SetInputScale("Input0_scale", {*in_scale}, true);
    conv.SetInputScale("Filter0_scale", *ws, true);
    conv.SetOutputScale("Output0_scale", {*out_scale}, true);
  }
  return conv;
}

static int ActCode(const std::string& a) { return a == "relu" ? 1 : a == "relu6" ? 2 : a == "leaky_relu" ? 4 : a == "hard_swish" ? 10 : 0; }

// Whole op path on one problem. With run_on_device false stops before Launch.
static void RunProblem(const Problem& p, bool run_on_device) {
  std::printf("case ic=%d oc=%d n=%d %dx%d sparsity=%.2f %s %s%s act=%s bias=%d\n", p.ic, p.oc, p.batch, p.h, p.w, p.sparsity, p.paired ? "semi" : "unstructured", p.int8 ? "int8" : "fp32",
              p.out_int8 ? "->int8" : "", p.act.c_str(), p.bias);
  std::fflush(stdout);
  Scope scope;
  std::vector<float> ws;
  float in_scale = 1.f, out_scale = 1.f;
  std::vector<OpInfo> ops{MakeConv(p, &scope, &ws, &in_scale, &out_scale)};
  // keep dense copies for the reference
  const int64_t wn = static_cast<int64_t>(p.oc) * p.ic;
  std::vector<int8_t> w8;
  std::vector<float> wf;
  if (p.int8) {
    w8.assign(scope.FindMutableTensor("conv_w")->data<int8_t>(), scope.FindMutableTensor("conv_w")->data<int8_t>() + wn);
  } else {
    wf.assign(scope.FindMutableTensor("conv_w")->data<float>(), scope.FindMutableTensor("conv_w")->data<float>() + wn);
  }

  mir::SparseConvDetectPass pass;
  pass.SetSparseThreshold(0.5f);
  EXPECT(mir::SparseConvDetectPass::BoundTo(TARGET(kHIP)));
  const int replaced = pass.Apply(&ops, &scope);
  EXPECT(replaced == 1);
  EXPECT(ops[0].Type() == "sparse_conv2d");
  EXPECT(scope.FindVar("conv_w") == nullptr);
  EXPECT(ops[0].GetAttr<int>("flag_semi") == (p.paired ? 1 : 0));
  Tensor* ocn = scope.FindMutableTensor("conv_w_oc_nonzeros");
  EXPECT(ocn != nullptr && ocn->dims()[0] == p.oc && ocn->persistable());

  auto op = LiteOpRegistry::Global().Create("sparse_conv2d");
  EXPECT(op != nullptr);
  EXPECT(op->Attach(ops[0], &scope));
  EXPECT(op->CheckShape());
  EXPECT(op->InferShape());
  Tensor* y = scope.FindMutableTensor("y");
  EXPECT(y->dims() == DDim({p.batch, p.oc, p.h, p.w}));
  {
    // what the op reports to the profiler (sparse_conv_op.h:41-63)
    paddle::lite::profile::OpCharacter ch;
    static_cast<operators::SparseConvOp*>(op.get())->GetOpRuntimeInfo(&ch);
    const std::string dims = std::to_string(p.batch) + "x";
    EXPECT(ch.input_shape == dims + std::to_string(p.ic) + "x" + std::to_string(p.h) + "x" + std::to_string(p.w));
    EXPECT(ch.output_shape == dims + std::to_string(p.oc) + "x" + std::to_string(p.h) + "x" + std::to_string(p.w));
    EXPECT(ch.filter_shape == std::to_string(p.oc) + "x" + std::to_string(p.ic) + "x1x1");
    // the reference's name table has "Silu" inserted at position 6 while its enum has not
    // (lite/api/paddle_place.cc:48-69 against paddle_place.h:122-148): kHardSwish = 10 prints as "Abs"
    const std::string act = p.act == "relu" ? "Relu" : p.act == "relu6" ? "Relu6" : p.act == "leaky_relu" ? "LeakyRelu" : p.act == "hard_swish" ? "Abs" : "unk";
    EXPECT(ch.remark == std::string("1x1p0s1g1d1") + (p.bias ? "Bias" : "") + act);
    EXPECT(ch.macs == 2.f * p.batch * p.oc * p.h * p.w * p.ic);
  }

  const PrecisionType prec = p.int8 ? PRECISION(kInt8) : PRECISION(kFloat);
  const std::string alias = !p.int8 ? "def" : (p.out_int8 ? "int8_int8_out" : "int8_fp32_out");
  if (!run_on_device) {
    auto all = KernelRegistry::Global().Create("sparse_conv2d", TARGET(kHIP), prec, DATALAYOUT(kNCHW));
    EXPECT(all.size() == (p.int8 ? 2u : 1u));
    return;
  }
  // the io_copy an optimiser would insert in front of a kHIP kernel
  OpInfo h2d("io_copy");
  h2d.SetInput("Input", {"x"});
  h2d.SetOutput("Out", {"x_dev"});
  auto copy_op = LiteOpRegistry::Global().Create("io_copy");
  EXPECT(copy_op->Attach(h2d, &scope) && copy_op->InferShape());
  auto copy_kernels = copy_op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny))}, "io_copy/host_to_device");
  EXPECT(copy_kernels.size() == 1);
  copy_kernels[0]->Launch();
  ops[0].SetInput("Input", {"x_dev"});
  EXPECT(op->Attach(ops[0], &scope) && op->InferShape());

  auto kernels = op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), prec, DATALAYOUT(kNCHW))}, "sparse_conv2d/" + alias);
  EXPECT(kernels.size() == 1);
  KernelBase* k = kernels[0].get();
  EXPECT(k->alias() == alias && k->target() == TARGET(kHIP));
  k->Launch();
  k->Launch();  // second epoch: no PrepareForRun
  k->mutable_context_as<HIPContext>()->Sync();
  {
    paddle::lite::profile::OpCharacter ch;
    if (!p.int8) static_cast<kernels::hip::SparseConvCompute<PRECISION(kFloat), PRECISION(kFloat)>*>(k)->SetProfileRuntimeKernelInfo(&ch);
    else if (p.out_int8) static_cast<kernels::hip::SparseConvCompute<PRECISION(kInt8), PRECISION(kInt8)>*>(k)->SetProfileRuntimeKernelInfo(&ch);
    else static_cast<kernels::hip::SparseConvCompute<PRECISION(kInt8), PRECISION(kFloat)>*>(k)->SetProfileRuntimeKernelInfo(&ch);
    // int8: the row walk for at most 256 positions in all, else the block kernel
    // (none of these shapes is one of the image kernel's)
    const bool few_positions = p.batch * p.h * p.w <= 256;
    EXPECT(ch.kernel_func_name == (p.int8 && !few_positions ? "pl_sparse_conv_run/block_mfma" : "pl_sparse_conv_run/row_walk"));
  }
  EXPECT(y->target() == TARGET(kHIP));
  Tensor y_host;
  y_host.CopyDataFrom(*y, TargetType::kHost);

  // reference: the oracle's dense per-image GEMM with the merged parameters
  // (the kernel class scales the activation once here)
  const int hw = p.h * p.w;
  plo_act act{ActCode(p.act), 6.f, 0.1f, 6.f, 3.f, 6.f};
  const float* bias = p.bias ? scope.FindMutableTensor("conv_b")->data<float>() : nullptr;
  std::vector<float> ms(p.oc), mb(p.oc);
  const int kind = !p.int8 ? 0 : (p.out_int8 ? 2 : 1);
  EXPECT(plo_merge_params(kind, p.oc, ws.data(), static_cast<int>(ws.size()), in_scale, out_scale, bias, ms.data(), bias ? mb.data() : nullptr, &act) == 0);
  if (kind == 2 && act.type == 4) act.leaky_alpha = 0.1f;  // slope left alone
  const Tensor* xt = scope.FindMutableTensor("x");
  if (!p.int8) {
    std::vector<float> want(static_cast<size_t>(p.batch) * p.oc * hw);
    plo_dense_conv1x1(0, wf.data(), xt->data<float>(), bias, nullptr, want.data(), p.batch, p.oc, p.ic, hw, &act, 1);
    double max_ratio = 0, max_diff = 0;
    for (size_t i = 0; i < want.size(); ++i) {
      const double d = std::fabs(want[i] - y_host.data<float>()[i]);
      const double r = d / (std::fabs(want[i]) + 1e-6);
      if (r > max_ratio) {
        max_ratio = r;
        max_diff = d;
      }
    }
    // the reference test's criterion (sparse_conv_f32_compute_test.cc:336-361)
    EXPECT(!(max_ratio > 1e-4 && max_diff > 5e-5));
  } else if (!p.out_int8) {
    std::vector<float> want(static_cast<size_t>(p.batch) * p.oc * hw);
    plo_dense_conv1x1(1, w8.data(), xt->data<int8_t>(), bias, ms.data(), want.data(), p.batch, p.oc, p.ic, hw, &act, 1);
    EXPECT(std::memcmp(want.data(), y_host.raw_data(), want.size() * 4) == 0);
  } else {
    std::vector<int8_t> want(static_cast<size_t>(p.batch) * p.oc * hw);
    plo_dense_conv1x1(2, w8.data(), xt->data<int8_t>(), bias ? mb.data() : nullptr, ms.data(), want.data(), p.batch, p.oc, p.ic, hw, &act, 1);
    EXPECT(std::memcmp(want.data(), y_host.raw_data(), want.size()) == 0);
  }
}

static void RegistryAndErrorPaths() {
  std::printf("registry and error paths\n");
  // the three registrations beside the ARM ones, same aliases
  auto fp32 = KernelRegistry::Global().Create("sparse_conv2d", TARGET(kHIP), PRECISION(kFloat), DATALAYOUT(kNCHW));
  auto int8 = KernelRegistry::Global().Create("sparse_conv2d", TARGET(kHIP), PRECISION(kInt8), DATALAYOUT(kNCHW));
  EXPECT(fp32.size() == 1 && fp32.front()->alias() == "def");
  EXPECT(int8.size() == 2);
  bool a = false, b = false;
  for (auto& k : int8) {
    a |= k->alias() == "int8_fp32_out";
    b |= k->alias() == "int8_int8_out";
  }
  EXPECT(a && b);
  EXPECT(KernelRegistry::Global().Create("sparse_conv2d", TARGET(kARM), PRECISION(kFloat), DATALAYOUT(kNCHW)).empty());
  const auto* types = ParamTypeRegistry::Global().Retrieve("sparse_conv2d/int8_int8_out", paddle::lite_api::Place(TARGET(kHIP), PRECISION(kInt8), DATALAYOUT(kNCHW)));
  EXPECT(types != nullptr && types->size() == 6);
  if (types) {
    for (auto& e : *types) {
      if (e.arg == "Input" || e.arg == "Output") EXPECT(e.type.target == TARGET(kHIP) && e.type.precision == PRECISION(kInt8));
      if (e.arg == "OcNonZeros" || e.arg == "Diffs") EXPECT(e.type.target == TARGET(kHost) && e.type.precision == PRECISION(kInt32));
    }
  }
  EXPECT(static_cast<int>(TARGET(kHIP)) == 19 && static_cast<int>(TARGET(kNNAdapter)) == 18);
  {
    EXPECT(Throws([&] { mir::SparseConvDetectPass::CheckedToolThreshold(1.5f); }));
    EXPECT(Throws([&] { mir::SparseConvDetectPass::CheckedToolThreshold(-0.1f); }));
    EXPECT(mir::SparseConvDetectPass::CheckedToolThreshold(1.0f) == 1.0f);
  }

  // unknown fused activation and bad paddings are fatal in the op
  Scope scope;
  std::vector<float> ws;
  float is, os;
  Problem p{1, 8, 4, 2, 2, 0.6f, false, false, false, true, "relu", 1};
  std::vector<OpInfo> ops{MakeConv(p, &scope, &ws, &is, &os)};
  mir::SparseConvDetectPass pass;
  pass.SetSparseThreshold(0.0f);
  EXPECT(pass.Apply(&ops, &scope) == 1);
  auto op = LiteOpRegistry::Global().Create("sparse_conv2d");
  OpInfo bad = ops[0];
  bad.SetAttr<std::string>("act_type", "sigmoid");
  EXPECT(Throws([&] { op->Attach(bad, &scope); }));
  bad = ops[0];
  bad.SetAttr<std::vector<int>>("paddings", {0, 0, 0});
  EXPECT(Throws([&] { op->Attach(bad, &scope); }));
  bad = ops[0];
  bad.SetAttr<std::vector<int>>("paddings", {0, 0, 0, 0});
  EXPECT(op->Attach(bad, &scope));
  // hard_sigmoid is accepted by the op (no kernel implements it)
  bad = ops[0];
  bad.SetAttr<std::string>("act_type", "hard_sigmoid");
  bad.SetAttr<float>("slope", 0.2f);
  bad.SetAttr<float>("offset", 0.5f);
  EXPECT(op->Attach(bad, &scope));

  // the pass leaves ineligible convs alone: 3x3, stride 2, groups, threshold
  auto untouched = [&](const char* what, std::function<void(OpInfo*, Scope*)> edit) {
    Scope s;
    std::vector<float> w2;
    Problem q{1, 8, 4, 4, 4, 0.7f, false, false, false, false, "", 2};
    std::vector<OpInfo> o{MakeConv(q, &s, &w2, &is, &os)};
    edit(&o[0], &s);
    mir::SparseConvDetectPass ps;
    ps.SetSparseThreshold(0.5f);
    const int n = ps.Apply(&o, &s);
    if (n != 0 || o[0].Type() != "conv2d") {
      std::printf("  FAILED: pass rewrote a conv it must skip (%s)\n", what);
      ++g_failures;
    }
  };
  untouched("stride 2", [](OpInfo* o, Scope*) { o->SetAttr<std::vector<int>>("strides", {2, 2}); });
  untouched("padding 1", [](OpInfo* o, Scope*) { o->SetAttr<std::vector<int>>("paddings", {1, 1}); });
  untouched("groups 2", [](OpInfo* o, Scope*) { o->SetAttr<int>("groups", 2); });
  untouched("3x3", [](OpInfo*, Scope* s) { s->FindMutableTensor("conv_w")->Resize({4, 8, 3, 3}); });
  untouched("dense weights", [](OpInfo*, Scope* s) {
    Tensor* w = s->FindMutableTensor("conv_w");
    float* d = w->mutable_data<float>(TargetType::kHost);
    for (int64_t i = 0; i < w->numel(); ++i) d[i] = 1.f;
  });
  // threshold 1.5 is how the predictor switches the pass off
  {
    Scope s;
    std::vector<float> w2;
    Problem q{1, 8, 4, 4, 4, 0.9f, false, false, false, false, "", 3};
    std::vector<OpInfo> o{MakeConv(q, &s, &w2, &is, &os)};
    mir::SparseConvDetectPass ps;
    ps.SetSparseThreshold(1.5f);
    EXPECT(ps.Apply(&o, &s) == 0);
  }
  // weight_scale of the wrong size is fatal in PrepareForRun, before any device work
  {
    Scope s;
    std::vector<float> w2;
    Problem q{1, 8, 4, 2, 2, 0.6f, false, true, false, false, "", 4};
    std::vector<OpInfo> o{MakeConv(q, &s, &w2, &is, &os)};
    o[0].SetInputScale("Filter0_scale", {0.1f, 0.2f}, true);
    mir::SparseConvDetectPass ps;
    ps.SetSparseThreshold(0.0f);
    EXPECT(ps.Apply(&o, &s) == 1);
    auto sp = LiteOpRegistry::Global().Create("sparse_conv2d");
    EXPECT(sp->Attach(o[0], &s) && sp->InferShape());
    auto ks = sp->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kInt8), DATALAYOUT(kNCHW))}, "sparse_conv2d/int8_fp32_out");
    EXPECT(ks.size() == 1);
    EXPECT(Throws([&] { ks[0]->Launch(); }));
  }
  // An op description that is not 1x1 / stride 1 / pad 0 / dilation 1 / group 1 (only a model file can
  // carry one: the pass never creates it) is refused by the kHIP kernel before any device work: its
  // output would be larger than the input the kernel reads.
  auto refused = [&](const char* what, std::function<void(OpInfo*)> edit) {
    Scope s;
    std::vector<float> w2;
    Problem q{1, 8, 4, 4, 4, 0.6f, false, false, false, false, "", 5};
    std::vector<OpInfo> o{MakeConv(q, &s, &w2, &is, &os)};
    mir::SparseConvDetectPass ps;
    ps.SetSparseThreshold(0.0f);
    EXPECT(ps.Apply(&o, &s) == 1);
    edit(&o[0]);
    auto sp = LiteOpRegistry::Global().Create("sparse_conv2d");
    EXPECT(sp->Attach(o[0], &s) && sp->InferShape());
    auto ks = sp->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kFloat), DATALAYOUT(kNCHW))}, "sparse_conv2d/def");
    EXPECT(ks.size() == 1);
    if (!ThrowsWith(what, [&] { ks[0]->Launch(); })) {
      std::printf("  FAILED: the kHIP kernel accepted an op with %s\n", what);
      ++g_failures;
    }
  };
  refused("paddings must be 0", [](OpInfo* o) { o->SetAttr<std::vector<int>>("paddings", {1, 1}); });
  refused("strides must be 1", [](OpInfo* o) { o->SetAttr<std::vector<int>>("strides", {2, 2}); });
  refused("dilations must be 1", [](OpInfo* o) { o->SetAttr<std::vector<int>>("dilations", {2, 2}); });
  refused("groups must be 1", [](OpInfo* o) { o->SetAttr<int>("groups", 2); });
}

// The precision changes either side of an int8 convolution: op attach /
// shape inference / registrations on the host, and on the device the chain
// fp32 -> io_copy -> calib(fp32_to_int8) -> calib(int8_to_fp32) -> io_copy
// against the oracle's fp32_to_int8 / int8_to_fp32.
static void CalibChain(bool run_on_device) {
  std::printf("calib chain\n");
  std::fflush(stdout);
  auto all = KernelRegistry::Global().Create("calib", TARGET(kHIP), PRECISION(kInt8), DATALAYOUT(kNCHW));
  EXPECT(all.size() == 2);
  bool a = false, b = false;
  for (auto& k : all) {
    a |= k->alias() == "fp32_to_int8";
    b |= k->alias() == "int8_to_fp32";
  }
  EXPECT(a && b);

  Scope scope;
  const int64_t n = 3 * 5 * 7 * 11 + 0;  // not a multiple of 16
  const float scale = 0.0371f;
  Tensor* x = scope.Var("cx")->GetMutable<Tensor>();
  x->Resize({3, 5, 7, 11});
  float* xd = x->mutable_data<float>(TargetType::kHost);
  std::mt19937 rng(5);
  std::normal_distribution<float> dist(0.f, 2.5f);
  for (int64_t i = 0; i < n; ++i) xd[i] = dist(rng);
  xd[0] = 0.5f * scale;
  xd[1] = -0.5f * scale;
  xd[2] = 500.f;
  xd[3] = -500.f;
  scope.Var("cx_dev");
  scope.Var("cq");
  scope.Var("cf");

  OpInfo q("calib");
  q.SetInput("Input", {"cx_dev"});
  q.SetOutput("Out", {"cq"});
  q.SetAttr<float>("scale", scale);
  OpInfo dq("calib");
  dq.SetInput("Input", {"cq"});
  dq.SetOutput("Out", {"cf"});
  dq.SetAttr<float>("scale", scale);
  OpInfo missing("calib");
  missing.SetInput("Input", {"nowhere"});
  missing.SetOutput("Out", {"cq"});
  EXPECT(Throws([&] { LiteOpRegistry::Global().Create("calib")->Attach(missing, &scope); }));
  if (!run_on_device) {
    // shape inference needs no device: attach on the host tensor
    q.SetInput("Input", {"cx"});
    auto op = LiteOpRegistry::Global().Create("calib");
    EXPECT(op != nullptr && op->Attach(q, &scope) && op->CheckShape() && op->InferShape());
    EXPECT(scope.FindMutableTensor("cq")->dims() == DDim({3, 5, 7, 11}));
    return;
  }
  OpInfo h2d("io_copy");
  h2d.SetInput("Input", {"cx"});
  h2d.SetOutput("Out", {"cx_dev"});
  auto copy_op = LiteOpRegistry::Global().Create("io_copy");
  EXPECT(copy_op->Attach(h2d, &scope) && copy_op->InferShape());
  auto copy_kernels = copy_op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny))}, "io_copy/host_to_device");
  EXPECT(copy_kernels.size() == 1);
  copy_kernels[0]->Launch();

  auto q_op = LiteOpRegistry::Global().Create("calib");
  EXPECT(q_op->Attach(q, &scope) && q_op->CheckShape() && q_op->InferShape());
  auto qk = q_op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kInt8), DATALAYOUT(kNCHW))}, "calib/fp32_to_int8");
  EXPECT(qk.size() == 1);
  qk[0]->Launch();
  auto dq_op = LiteOpRegistry::Global().Create("calib");
  EXPECT(dq_op->Attach(dq, &scope) && dq_op->InferShape());
  auto dqk = dq_op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kInt8), DATALAYOUT(kNCHW))}, "calib/int8_to_fp32");
  EXPECT(dqk.size() == 1);
  dqk[0]->Launch();
  dqk[0]->mutable_context_as<HIPContext>()->Sync();
  qk[0]->mutable_context_as<HIPContext>()->Sync();

  Tensor q_host, f_host;
  q_host.CopyDataFrom(*scope.FindMutableTensor("cq"), TargetType::kHost);
  f_host.CopyDataFrom(*scope.FindMutableTensor("cf"), TargetType::kHost);
  std::vector<int8_t> want_q(n);
  std::vector<float> want_f(n);
  plo_fp32_to_int8(xd, want_q.data(), scale, n);
  plo_int8_to_fp32(want_q.data(), want_f.data(), scale, n);
  EXPECT(std::memcmp(want_q.data(), q_host.raw_data(), n) == 0);
  EXPECT(std::memcmp(want_f.data(), f_host.raw_data(), n * 4) == 0);
  EXPECT(want_q[2] == 127 && want_q[3] == -127);
}

// The half-precision registration: fp32 sparse tensors from the pass, fp16
// activations on the device, checked against the oracle's binary16 walker.
static void HalfPrecision(bool run_on_device) {
  std::printf("half precision\n");
  std::fflush(stdout);
  auto regs = KernelRegistry::Global().Create("sparse_conv2d", TARGET(kHIP), PRECISION(kFP16), DATALAYOUT(kNCHW));
  EXPECT(regs.size() == 1 && regs.front()->alias() == "def");
  if (!run_on_device) return;
  Problem p{2, 70, 33, 6, 6, 0.7f, true, false, false, true, "hard_swish", 21};
  Scope scope;
  std::vector<float> ws;
  float is = 1.f, os = 1.f;
  std::vector<OpInfo> ops{MakeConv(p, &scope, &ws, &is, &os)};
  const int hw = p.h * p.w;
  const int64_t xn = static_cast<int64_t>(p.batch) * p.ic * hw;
  // fp16 copy of the input
  const float* xf = scope.FindMutableTensor("x")->data<float>();
  Tensor* xh = scope.NewTensor("xh");
  xh->Resize({p.batch, p.ic, p.h, p.w});
  uint16_t* xhd = xh->mutable_data<uint16_t>(TargetType::kHost);
  plo_fp32_to_fp16(xf, xhd, xn);
  mir::SparseConvDetectPass pass;
  pass.SetSparseThreshold(0.5f);
  EXPECT(pass.Apply(&ops, &scope) == 1);
  // oracle on the tensors the pass made
  const Tensor* nzw = scope.FindMutableTensor("conv_w_nonzeros_output");
  const Tensor* ocn = scope.FindMutableTensor("conv_w_oc_nonzeros");
  const Tensor* dif = scope.FindMutableTensor("conv_w_ic_diffs");
  EXPECT(nzw && ocn && dif);
  if (!(nzw && ocn && dif)) return;
  std::vector<uint16_t> w16(nzw->numel()), b16(p.oc), want(static_cast<size_t>(p.batch) * p.oc * hw);
  plo_fp32_to_fp16(nzw->data<float>(), w16.data(), nzw->numel());
  plo_fp32_to_fp16(scope.FindMutableTensor("conv_b")->data<float>(), b16.data(), p.oc);
  plo_act act{10, 6.f, 0.1f, 6.f, 3.f, 6.f};
  plo_sparse_conv_fp16(w16.data(), xhd, dif->data<int32_t>(), ocn->data<uint32_t>(), b16.data(), want.data(), p.batch, p.oc, p.ic, hw, ops[0].GetAttr<int>("first_ic"), ops[0].GetAttr<int>("flag_semi"), &act);

  OpInfo h2d("io_copy");
  h2d.SetInput("Input", {"xh"});
  h2d.SetOutput("Out", {"xh_dev"});
  auto copy_op = LiteOpRegistry::Global().Create("io_copy");
  EXPECT(copy_op->Attach(h2d, &scope) && copy_op->InferShape());
  auto ck = copy_op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny))}, "io_copy/host_to_device");
  EXPECT(ck.size() == 1);
  ck[0]->Launch();
  ops[0].SetInput("Input", {"xh_dev"});
  auto op = LiteOpRegistry::Global().Create("sparse_conv2d");
  EXPECT(op->Attach(ops[0], &scope) && op->CheckShape() && op->InferShape());
  auto ks = op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kFP16), DATALAYOUT(kNCHW))}, "sparse_conv2d/def");
  EXPECT(ks.size() == 1);
  ks[0]->Launch();
  ks[0]->mutable_context_as<HIPContext>()->Sync();
  Tensor y_host;
  y_host.CopyDataFrom(*scope.FindMutableTensor("y"), TargetType::kHost);
  const uint16_t* got = static_cast<const uint16_t*>(y_host.raw_data());
  size_t bad = 0;
  for (size_t i = 0; i < want.size(); ++i) bad += (got[i] != want[i]) && !(((got[i] | want[i]) & 0x7fffu) == 0);  // zeros of either sign agree
  EXPECT(bad == 0);
}

// Three quantised 1x1 convolutions in a row, fed and fetched as fp32 on the
// host: detect pass -> output-type rule / calib / io_copy insertion ->
// program run on the device, against the oracle's chain
// fp32_to_int8 -> int8 conv (int8 out) x2 -> int8 conv (fp32 out).
static void Int8Chain(bool run_on_device) {
  std::printf("int8 chain\n");
  std::fflush(stdout);
  const int batch = 2, hw_h = 8, hw_w = 6, hw = hw_h * hw_w;
  const int ch[4] = {40, 64, 33, 48};
  const float act_scale[3] = {0.02f, 0.05f, 0.04f};  // input scale of layer 1..3
  Scope scope;
  std::mt19937 gen(77);
  std::uniform_real_distribution<float> uni(0.f, 1.f);
  std::normal_distribution<float> nrm(0.f, 1.f);
  Tensor* a0 = scope.NewTensor("a0");
  a0->Resize({batch, ch[0], hw_h, hw_w});
  float* a0d = a0->mutable_data<float>(TargetType::kHost);
  for (int64_t i = 0; i < a0->numel(); ++i) a0d[i] = uni(gen) * 2.f - 1.f;
  std::vector<OpInfo> ops;
  std::vector<std::vector<int8_t>> w8(3);
  std::vector<std::vector<float>> ws(3), bias(3);
  for (int l = 0; l < 3; ++l) {
    const int ic = ch[l], oc = ch[l + 1];
    const std::string n = std::to_string(l + 1);
    Tensor* w = scope.NewTensor("w" + n);
    w->Resize({oc, ic, 1, 1});
    int8_t* wd = w->mutable_data<int8_t>(TargetType::kHost);
    for (int64_t i = 0; i < w->numel(); ++i) {
      int v = static_cast<int>(uni(gen) * 127.f) + 1;
      if (uni(gen) < 0.5f) v = -v;
      wd[i] = uni(gen) >= 0.7f ? static_cast<int8_t>(v) : 0;
    }
    w8[l].assign(wd, wd + w->numel());
    Tensor* b = scope.NewTensor("b" + n);
    b->Resize({oc});
    float* bd = b->mutable_data<float>(TargetType::kHost);
    bias[l].resize(oc);
    for (int i = 0; i < oc; ++i) bias[l][i] = bd[i] = nrm(gen) * 0.1f;
    ws[l].resize(oc);
    for (float& v : ws[l]) v = 0.001f + 0.004f * uni(gen);
    OpInfo conv("conv2d");
    conv.SetInput("Input", {"a" + std::to_string(l)});
    conv.SetInput("Filter", {"w" + n});
    conv.SetInput("Bias", {"b" + n});
    conv.SetOutput("Output", {"a" + n});
    scope.NewTensor("a" + n);
    conv.SetAttr<std::vector<int>>("strides", {1, 1});
    conv.SetAttr<std::vector<int>>("paddings", {0, 0});
    conv.SetAttr<std::vector<int>>("dilations", {1, 1});
    conv.SetAttr<int>("groups", 1);
    conv.SetAttr<bool>("with_act", true);
    conv.SetAttr<std::string>("act_type", "relu");
    conv.SetAttr<bool>("enable_int8", true);
    conv.SetInputScale("Input0_scale", {act_scale[l]}, true);
    conv.SetInputScale("Filter0_scale", ws[l], true);
    conv.SetOutputScale("Output0_scale", {1.f}, true);  // the pick rule overwrites it where the output stays int8
    ops.push_back(conv);
  }
  // the first layer's input tensor must have a shape for the detect pass
  mir::SparseConvDetectPass detect;
  detect.SetSparseThreshold(0.5f);
  // the pass needs the spatial size of every conv input: give the later
  // inputs their shapes (shape inference would have done so in a graph)
  for (int l = 1; l < 3; ++l) scope.FindMutableTensor("a" + std::to_string(l))->Resize({batch, ch[l], hw_h, hw_w});
  EXPECT(detect.Apply(&ops, &scope) == 3);

  mir::Int8ChainPass chain;
  std::vector<mir::ProgramStep> steps = chain.Apply(ops, {"a0"}, {"a3"}, &scope);
  EXPECT(steps.size() == 6);
  if (steps.size() == 6) {
    EXPECT(steps[0].kernel == "io_copy/host_to_device");
    EXPECT(steps[1].kernel == "calib/fp32_to_int8" && steps[1].op.GetAttr<float>("scale") == act_scale[0]);
    EXPECT(steps[2].kernel == "sparse_conv2d/int8_int8_out" && steps[2].op.GetOutputScale("Output0_scale", true)[0] == act_scale[1]);
    EXPECT(steps[3].kernel == "sparse_conv2d/int8_int8_out" && steps[3].op.GetOutputScale("Output0_scale", true)[0] == act_scale[2]);
    EXPECT(steps[4].kernel == "sparse_conv2d/int8_fp32_out");
    EXPECT(steps[5].kernel == "io_copy/device_to_host" && steps[5].op.Output("Out").front() == "a3/host");
    EXPECT(steps[2].op.Input("Input").front() == "a0/hip/int8");
  }
  // an fp32 consumer in the middle keeps its producer's output fp32
  {
    std::vector<OpInfo> mixed = ops;
    mixed[1].SetAttr<bool>("enable_int8", false);
    Scope dummy;
    dummy.NewTensor("a0");
    auto st = chain.Apply({mixed[0]}, {"a0"}, {"a1"}, &dummy);
    EXPECT(st.size() == 4 && st[2].kernel == "sparse_conv2d/int8_fp32_out");
  }
  EXPECT(Throws([&] { chain.Apply(ops, {"a0"}, {"nothing"}, &scope); }));
  if (!run_on_device) return;

  mir::HipProgram program(steps, &scope);
  program.Run();
  program.Run();  // second epoch
  const Tensor* got = scope.FindMutableTensor("a3/host");
  EXPECT(got != nullptr && got->dims() == DDim({batch, ch[3], hw_h, hw_w}));

  // oracle chain
  std::vector<int8_t> q(a0->numel());
  plo_fp32_to_int8(a0d, q.data(), act_scale[0], a0->numel());
  std::vector<float> want;
  for (int l = 0; l < 3; ++l) {
    const int ic = ch[l], oc = ch[l + 1];
    plo_act act{1, 6.f, 0.1f, 6.f, 3.f, 6.f};
    std::vector<float> ms(oc), mb(oc);
    const int kind = l < 2 ? 2 : 1;
    EXPECT(plo_merge_params(kind, oc, ws[l].data(), oc, act_scale[l], l < 2 ? act_scale[l + 1] : 1.f, bias[l].data(), ms.data(), mb.data(), &act) == 0);
    if (kind == 2) {
      std::vector<int8_t> next(static_cast<size_t>(batch) * oc * hw);
      plo_dense_conv1x1(2, w8[l].data(), q.data(), mb.data(), ms.data(), next.data(), batch, oc, ic, hw, &act, 1);
      q.swap(next);
    } else {
      want.resize(static_cast<size_t>(batch) * oc * hw);
      plo_dense_conv1x1(1, w8[l].data(), q.data(), bias[l].data(), ms.data(), want.data(), batch, oc, ic, hw, &act, 1);
    }
  }
  if (got) EXPECT(std::memcmp(want.data(), got->raw_data(), want.size() * 4) == 0);
}

// Runs a sparse_conv2d description against the tensors of `scope` on the
// device ("x" is copied over first) and returns the output on the host.
static Tensor RunSparseOnDevice(OpInfo info, Scope* scope, PrecisionType prec, const std::string& alias) {
  OpInfo h2d("io_copy");
  h2d.SetInput("Input", {"x"});
  h2d.SetOutput("Out", {"x_dev"});
  auto copy_op = LiteOpRegistry::Global().Create("io_copy");
  EXPECT(copy_op->Attach(h2d, scope) && copy_op->InferShape());
  auto copy_kernels = copy_op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny))}, "io_copy/host_to_device");
  copy_kernels[0]->Launch();
  info.SetInput("Input", {"x_dev"});
  scope->NewTensor(info.Output("Output").front());
  auto op = LiteOpRegistry::Global().Create("sparse_conv2d");
  EXPECT(op->Attach(info, scope) && op->CheckShape() && op->InferShape());
  auto kernels = op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), prec, DATALAYOUT(kNCHW))}, "sparse_conv2d/" + alias);
  EXPECT(kernels.size() == 1);
  kernels[0]->Launch();
  kernels[0]->mutable_context_as<HIPContext>()->Sync();
  Tensor y_host;
  y_host.CopyDataFrom(*scope->FindMutableTensor(info.Output("Output").front()), TargetType::kHost);
  return y_host;
}

// A graph with a branch: one int8 layer whose output feeds an int8 layer and
// an fp32 layer.  The output-type rule (static_kernel_pick_pass.cc:97-135)
// keeps the producer's output fp32 ("int8 out only if all consumers are
// int8"), the int8 consumer gets a calib, the fp32 consumer reads the fp32
// tensor; on the device both fetched outputs equal the oracle's.  Also: int8
// consumers that disagree on their input scale, a filter shared by two convs,
// and the graph bookkeeping of the detect pass.
static void BranchingGraph(bool run_on_device) {
  std::printf("branching graph\n");
  std::fflush(stdout);
  const int batch = 2, hh = 6, ww = 6, hw = hh * ww;
  const int c0 = 48, c1 = 64, c2 = 40, c3 = 24;
  const float s0 = 0.02f, s1 = 0.05f;
  Scope scope;
  std::mt19937 gen(99);
  std::uniform_real_distribution<float> uni(0.f, 1.f);
  std::normal_distribution<float> nrm(0.f, 1.f);
  Tensor* a0 = scope.NewTensor("a0");
  a0->Resize({batch, c0, hh, ww});
  float* a0d = a0->mutable_data<float>(TargetType::kHost);
  for (int64_t i = 0; i < a0->numel(); ++i) a0d[i] = uni(gen) * 2.f - 1.f;
  struct Layer {
    std::vector<int8_t> w8;
    std::vector<float> wf, ws, bias;
  };
  auto make = [&](const std::string& n, const std::string& in, const std::string& out, int ic, int oc, bool int8, float in_scale, Layer* L) {
    Tensor* w = scope.NewTensor("w" + n);
    w->Resize({oc, ic, 1, 1});
    if (int8) {
      int8_t* wd = w->mutable_data<int8_t>(TargetType::kHost);
      for (int64_t i = 0; i < w->numel(); ++i) {
        int v = static_cast<int>(uni(gen) * 127.f) + 1;
        if (uni(gen) < 0.5f) v = -v;
        wd[i] = uni(gen) >= 0.7f ? static_cast<int8_t>(v) : 0;
      }
      L->w8.assign(wd, wd + w->numel());
    } else {
      float* wd = w->mutable_data<float>(TargetType::kHost);
      for (int64_t i = 0; i < w->numel(); ++i) wd[i] = uni(gen) >= 0.7f ? nrm(gen) * 0.1f : 0.f;
      L->wf.assign(wd, wd + w->numel());
    }
    Tensor* b = scope.NewTensor("b" + n);
    b->Resize({oc});
    float* bd = b->mutable_data<float>(TargetType::kHost);
    L->bias.resize(oc);
    for (int i = 0; i < oc; ++i) L->bias[i] = bd[i] = nrm(gen) * 0.1f;
    L->ws.resize(oc);
    for (float& v : L->ws) v = 0.001f + 0.004f * uni(gen);
    OpInfo conv("conv2d");
    conv.SetInput("Input", {in});
    conv.SetInput("Filter", {"w" + n});
    conv.SetInput("Bias", {"b" + n});
    conv.SetOutput("Output", {out});
    scope.NewTensor(out);
    conv.SetAttr<std::vector<int>>("strides", {1, 1});
    conv.SetAttr<std::vector<int>>("paddings", {0, 0});
    conv.SetAttr<std::vector<int>>("dilations", {1, 1});
    conv.SetAttr<int>("groups", 1);
    conv.SetAttr<bool>("with_act", true);
    conv.SetAttr<std::string>("act_type", "relu");
    if (int8) {
      conv.SetAttr<bool>("enable_int8", true);
      conv.SetInputScale("Input0_scale", {in_scale}, true);
      conv.SetInputScale("Filter0_scale", L->ws, true);
      conv.SetOutputScale("Output0_scale", {1.f}, true);
    }
    return conv;
  };
  Layer A, B, Cc;
  std::vector<OpInfo> ops;
  ops.push_back(make("A", "a0", "a1", c0, c1, true, s0, &A));
  ops.push_back(make("B", "a1", "yb", c1, c2, true, s1, &B));
  ops.push_back(make("C", "a1", "yc", c1, c3, false, 1.f, &Cc));
  scope.FindMutableTensor("a1")->Resize({batch, c1, hh, ww});

  mir::Graph graph(ops, scope);
  const mir::Graph& cgraph = graph;
  EXPECT(graph.OpNodes().size() == 3 && cgraph.Consumers("a1").size() == 2 && cgraph.Producer("a1") == cgraph.OpNodes()[0]);
  EXPECT(graph.Var("wA") != nullptr);
  mir::SparseConvDetectPass detect;
  detect.SetSparseThreshold(0.5f);
  EXPECT(detect.Apply(&graph, &scope) == 3);
  // the conv nodes are gone, the sparse ops hold their links, the dense filters left graph and scope
  EXPECT(graph.OpNodes().size() == 3 && cgraph.Consumers("a1").size() == 2);
  for (const auto* n : cgraph.OpNodes()) EXPECT(n->op.Type() == "sparse_conv2d" && n->inlinks.size() == 5 && n->outlinks.size() == 1);
  EXPECT(graph.Var("wA") == nullptr && scope.FindVar("wA") == nullptr && graph.Var("wA_ic_diffs") != nullptr && graph.Var("wA_ic_diffs")->is_weight);
  EXPECT(cgraph.Producer("a1") != nullptr && cgraph.Producer("a1")->op.Type() == "sparse_conv2d" && cgraph.Producer("a0") == nullptr);

  mir::Int8ChainPass chain;
  std::vector<mir::ProgramStep> steps = chain.Apply(cgraph, {"a0"}, {"yb", "yc"}, &scope);
  // io_copy a0, calib a0, A (fp32 out), calib a1 for B, B, C, two fetches
  EXPECT(steps.size() == 8);
  if (steps.size() == 8) {
    EXPECT(steps[2].kernel == "sparse_conv2d/int8_fp32_out");
    EXPECT(steps[3].kernel == "calib/fp32_to_int8" && steps[3].op.GetAttr<float>("scale") == s1 && steps[3].op.Input("Input").front() == "a1");
    EXPECT(steps[4].kernel == "sparse_conv2d/int8_fp32_out" && steps[4].op.Input("Input").front() == "a1/int8");
    EXPECT(steps[5].kernel == "sparse_conv2d/def" && steps[5].op.Input("Input").front() == "a1");
    EXPECT(steps[6].kernel == "io_copy/device_to_host" && steps[7].kernel == "io_copy/device_to_host");
  }
  // the same with the fp32 consumer first in the list: the int8 consumer still gets its calib
  {
    std::vector<OpInfo> reordered = cgraph.TopologicalOps();
    std::swap(reordered[1], reordered[2]);
    auto st = chain.Apply(reordered, {"a0"}, {"yb", "yc"}, &scope);
    EXPECT(st.size() == 8 && st[3].kernel == "sparse_conv2d/def" && st[4].kernel == "calib/fp32_to_int8" && st[5].kernel == "sparse_conv2d/int8_fp32_out");
  }
  // two int8 consumers that agree on the scale share an int8 output; if they disagree the producer
  // keeps fp32 and each gets its own calib
  {
    std::vector<OpInfo> two = cgraph.TopologicalOps();
    two[2] = two[1];
    two[2].SetOutput("Output", {"yb2"});
    auto st = chain.Apply(two, {"a0"}, {"yb", "yb2"}, &scope);
    EXPECT(st.size() == 7 && st[2].kernel == "sparse_conv2d/int8_int8_out" && st[2].op.GetOutputScale("Output0_scale", true)[0] == s1 && st[3].op.Input("Input").front() == "a1" &&
           st[4].op.Input("Input").front() == "a1");
    two[2].SetInputScale("Input0_scale", {0.07f}, true);
    st = chain.Apply(two, {"a0"}, {"yb", "yb2"}, &scope);
    EXPECT(st.size() == 9 && st[2].kernel == "sparse_conv2d/int8_fp32_out" && st[3].kernel == "calib/fp32_to_int8" && st[5].kernel == "calib/fp32_to_int8" &&
           st[3].op.GetAttr<float>("scale") == s1 && st[5].op.GetAttr<float>("scale") == 0.07f && st[3].op.Output("Out").front() != st[5].op.Output("Out").front());
  }
  // a filter read by two convs stays in the graph and in the scope while one of them still reads it
  {
    Scope s2;
    std::vector<float> w2;
    float is, os;
    Problem q{1, 8, 4, 4, 4, 0.7f, false, false, false, false, "", 6};
    OpInfo c1op = MakeConv(q, &s2, &w2, &is, &os);
    OpInfo c2op = c1op;
    c2op.SetOutput("Output", {"y2"});
    s2.NewTensor("y2");
    c2op.SetAttr<std::vector<int>>("strides", {2, 2});  // not eligible: keeps reading the dense filter
    std::vector<OpInfo> shared{c1op, c2op};
    mir::SparseConvDetectPass ps;
    ps.SetSparseThreshold(0.5f);
    EXPECT(ps.Apply(&shared, &s2) == 1);
    EXPECT(shared[0].Type() == "sparse_conv2d" && shared[1].Type() == "conv2d" && s2.FindVar("conv_w") != nullptr);
  }
  // a variable written twice is refused
  {
    std::vector<OpInfo> twice = cgraph.TopologicalOps();
    twice[2].SetOutput("Output", {"yb"});
    EXPECT(Throws([&] { mir::Graph g(twice, scope); }));
  }
  if (!run_on_device) return;

  mir::HipProgram program(steps, &scope);
  program.Run();
  const Tensor* yb = scope.FindMutableTensor("yb/host");
  const Tensor* yc = scope.FindMutableTensor("yc/host");
  EXPECT(yb != nullptr && yb->dims() == DDim({batch, c2, hh, ww}) && yc != nullptr && yc->dims() == DDim({batch, c3, hh, ww}));
  // oracle: A int8 -> fp32, then B on the requantised tensor and C (fp32 weights) on the fp32 one
  std::vector<int8_t> q0(a0->numel());
  plo_fp32_to_int8(a0d, q0.data(), s0, a0->numel());
  plo_act act{1, 6.f, 0.1f, 6.f, 3.f, 6.f};
  std::vector<float> ms(c1), mb(c1), a1(static_cast<size_t>(batch) * c1 * hw);
  EXPECT(plo_merge_params(1, c1, A.ws.data(), c1, s0, 1.f, A.bias.data(), ms.data(), mb.data(), &act) == 0);
  plo_dense_conv1x1(1, A.w8.data(), q0.data(), A.bias.data(), ms.data(), a1.data(), batch, c1, c0, hw, &act, 1);
  std::vector<int8_t> q1(a1.size());
  plo_fp32_to_int8(a1.data(), q1.data(), s1, static_cast<int64_t>(a1.size()));
  std::vector<float> msb(c2), mbb(c2), want_b(static_cast<size_t>(batch) * c2 * hw), want_c(static_cast<size_t>(batch) * c3 * hw);
  plo_act act_b{1, 6.f, 0.1f, 6.f, 3.f, 6.f};
  EXPECT(plo_merge_params(1, c2, B.ws.data(), c2, s1, 1.f, B.bias.data(), msb.data(), mbb.data(), &act_b) == 0);
  plo_dense_conv1x1(1, B.w8.data(), q1.data(), B.bias.data(), msb.data(), want_b.data(), batch, c2, c1, hw, &act_b, 1);
  plo_dense_conv1x1(0, Cc.wf.data(), a1.data(), Cc.bias.data(), nullptr, want_c.data(), batch, c3, c1, hw, &act, 1);
  if (yb) EXPECT(std::memcmp(want_b.data(), yb->raw_data(), want_b.size() * 4) == 0);
  if (yc) {
    const float* g = yc->data<float>();
    double worst = 0;
    for (size_t i = 0; i < want_c.size(); ++i) worst = std::max(worst, std::fabs(static_cast<double>(g[i]) - want_c[i]) / std::max(1.0, std::fabs(static_cast<double>(want_c[i]))));
    EXPECT(worst < 1e-5);
  }
}

// The optimised-model file: what the detect pass produced is written as a
// "<name>.nb" file, read back into an empty scope, and the loaded
// sparse_conv2d gives the same output bytes as the one that was saved.
static void ModelFile(bool run_on_device) {
  std::printf("case model file round trip\n");
  std::fflush(stdout);
  const std::vector<Problem> problems = {
      {2, 64, 48, 7, 7, 0.8f, true, false, false, true, "relu6", 31},
      {2, 128, 64, 7, 7, 0.85f, false, true, false, true, "leaky_relu", 32},
      {2, 96, 32, 8, 8, 0.75f, true, true, true, true, "hard_swish", 33},
  };
  for (const Problem& p : problems) {
    Scope scope;
    std::vector<float> ws;
    float in_scale = 1.f, out_scale = 1.f;
    std::vector<OpInfo> ops{MakeConv(p, &scope, &ws, &in_scale, &out_scale)};
    mir::SparseConvDetectPass pass;
    pass.SetSparseThreshold(0.5f);
    EXPECT(pass.Apply(&ops, &scope) == 1);

    cpp::ProgramDesc prog;
    cpp::BlockDesc* block = prog.AddBlock();
    block->SetParentIdx(-1);
    prog.SetVersion(1);
    auto add_var = [&](const std::string& name, bool persistable) {
      cpp::VarDesc* v = block->AddVar();
      v->SetName(name);
      v->SetPersistable(persistable);
      const Tensor* t = scope.FindMutableTensor(name);
      v->SetShape(t->dims().Vectorize());
      v->SetDataType(t->precision() == PRECISION(kInt8) ? VarDataType::INT8 : t->precision() == PRECISION(kInt32) ? VarDataType::INT32 : VarDataType::FP32);
    };
    add_var("x", false);
    for (const char* arg : {"NonZeroWeights", "OcNonZeros", "Diffs", "Bias"}) add_var(ops[0].Input(arg).front(), true);
    *block->AddOp() = ops[0];

    const std::string base = "/tmp/pl_model_file_test_" + std::to_string(static_cast<long>(getpid())) + "_" + std::to_string(p.seed);
    SaveModelNaive(base, scope, prog);
    Scope loaded;
    cpp::ProgramDesc back;
    LoadModelNaiveFromFile(base + ".nb", &loaded, &back);
    std::remove((base + ".nb").c_str());
    EXPECT(back.BlocksSize() == 1 && back.GetBlock(0)->OpsSize() == 1);
    if (back.BlocksSize() != 1 || back.GetBlock(0)->OpsSize() != 1) continue;
    const OpInfo& op2 = back.GetBlock(0)->GetOp(0);
    EXPECT(op2.Type() == "sparse_conv2d");
    EXPECT(op2.GetAttr<int>("first_ic") == ops[0].GetAttr<int>("first_ic") && op2.GetAttr<int>("flag_semi") == ops[0].GetAttr<int>("flag_semi"));
    EXPECT(op2.GetAttr<std::string>("act_type") == p.act);
    if (p.int8) EXPECT(op2.GetInputScale("Filter0_scale", true) == ws);
    for (const char* arg : {"NonZeroWeights", "OcNonZeros", "Diffs", "Bias"}) {
      const std::string name = ops[0].Input(arg).front();
      const Tensor* a = scope.FindMutableTensor(name);
      const Tensor* b = loaded.FindMutableTensor(name);
      EXPECT(b != nullptr && b->persistable() && b->dims() == a->dims() && b->precision() == a->precision() && b->memory_size() == a->memory_size());
      if (b && b->memory_size() == a->memory_size()) EXPECT(std::memcmp(a->raw_data(), b->raw_data(), a->memory_size()) == 0);
    }
    EXPECT(loaded.FindVar("x") == nullptr);
    {
      // another resolution: the reloaded Diffs, rewritten for 5x3 inputs,
      // equal what the detect pass makes of the same weights at 5x3
      Problem q = p;
      q.h = 5, q.w = 3;
      Scope scope_q;
      std::vector<float> ws_q;
      float is_q, os_q;
      std::vector<OpInfo> ops_q{MakeConv(q, &scope_q, &ws_q, &is_q, &os_q)};
      EXPECT(pass.Apply(&ops_q, &scope_q) == 1);
      Scope again;
      cpp::ProgramDesc prog_q;
      SaveModelNaive(base, scope, prog);
      LoadModelNaiveFromFile(base + ".nb", &again, &prog_q);
      std::remove((base + ".nb").c_str());
      EXPECT(RebakeSparseConvDiffs(&prog_q, &again, q.h, q.w) == 1);
      const std::string dn = ops[0].Input("Diffs").front();
      const Tensor* want = scope_q.FindMutableTensor(dn);
      const Tensor* got = again.FindMutableTensor(dn);
      EXPECT(want->numel() == got->numel() && std::memcmp(want->raw_data(), got->raw_data(), want->memory_size()) == 0);
      EXPECT(prog_q.GetBlock(0)->GetVar(0).GetShape() == (std::vector<int64_t>{q.batch, q.ic, q.h, q.w}));
      // the saved model itself is unchanged, and a second rewrite starts from the recorded 5x3
      EXPECT(RebakeSparseConvDiffs(&prog_q, &again, p.h, p.w) == 1);
      EXPECT(std::memcmp(scope.FindMutableTensor(dn)->raw_data(), again.FindMutableTensor(dn)->raw_data(), got->memory_size()) == 0);
    }
    if (!run_on_device) continue;
    // the input is not part of the file
    const Tensor* x = scope.FindMutableTensor("x");
    loaded.NewTensor("x")->CopyDataFrom(*x, TargetType::kHost);
    const PrecisionType prec = p.int8 ? PRECISION(kInt8) : PRECISION(kFloat);
    const std::string alias = !p.int8 ? "def" : (p.out_int8 ? "int8_int8_out" : "int8_fp32_out");
    const Tensor y_saved = RunSparseOnDevice(ops[0], &scope, prec, alias);
    const Tensor y_loaded = RunSparseOnDevice(op2, &loaded, prec, alias);
    EXPECT(y_saved.memory_size() > 0 && y_saved.memory_size() == y_loaded.memory_size());
    if (y_saved.memory_size() == y_loaded.memory_size()) EXPECT(std::memcmp(y_saved.raw_data(), y_loaded.raw_data(), y_saved.memory_size()) == 0);
  }
}

// depthwise_conv2d (int8, 3x3) through the op and the registered kHIP
// kernels, against the oracle with the parameters merged as the reference's
// DepthwiseConv::PrepareForRun merges them.
static void Depthwise(bool run_on_device) {
  std::printf("case depthwise 3x3\n");
  std::fflush(stdout);
  struct Dw {
    int n, c, h, w, stride, pad;
    bool out_int8;
    std::string act;
    unsigned seed;
  };
  const std::vector<Dw> cases = {{2, 16, 14, 14, 1, 1, true, "relu", 41}, {2, 8, 15, 13, 2, 1, true, "relu6", 42}, {1, 5, 9, 6, 1, 0, false, "leaky_relu", 43}, {2, 32, 7, 7, 2, 1, false, "", 44}};
  for (const Dw& q : cases) {
    std::mt19937 gen(q.seed);
    std::uniform_real_distribution<float> uni(0.f, 1.f);
    Scope scope;
    Tensor* x = scope.NewTensor("x");
    x->Resize({q.n, q.c, q.h, q.w});
    int8_t* xd = x->mutable_data<int8_t>(TargetType::kHost);
    for (int64_t i = 0; i < x->numel(); ++i) xd[i] = static_cast<int8_t>(static_cast<int>(uni(gen) * 255.f) - 127);
    Tensor* f = scope.NewTensor("dw_w");
    f->Resize({q.c, 1, 3, 3});
    int8_t* fd = f->mutable_data<int8_t>(TargetType::kHost);
    for (int64_t i = 0; i < f->numel(); ++i) fd[i] = static_cast<int8_t>(static_cast<int>(uni(gen) * 255.f) - 127);
    Tensor* b = scope.NewTensor("dw_b");
    b->Resize({q.c});
    float* bd = b->mutable_data<float>(TargetType::kHost);
    for (int i = 0; i < q.c; ++i) bd[i] = uni(gen) - 0.5f;
    scope.NewTensor("y");
    std::vector<float> ws(q.c);
    for (float& v : ws) v = 0.002f + 0.018f * uni(gen);
    const float in_scale = 0.02f, out_scale = q.out_int8 ? 0.11f : 1.f;
    OpInfo info("depthwise_conv2d");
    info.SetInput("Input", {"x"});
    info.SetInput("Filter", {"dw_w"});
    info.SetInput("Bias", {"dw_b"});
    info.SetOutput("Output", {"y"});
    info.SetAttr<std::vector<int>>("strides", {q.stride, q.stride});
    info.SetAttr<std::vector<int>>("paddings", {q.pad, q.pad});
    info.SetAttr<std::vector<int>>("dilations", {1, 1});
    info.SetAttr<int>("groups", q.c);
    if (!q.act.empty()) {
      info.SetAttr<bool>("with_act", true);
      info.SetAttr<std::string>("act_type", q.act);
      info.SetAttr<float>("fuse_brelu_threshold", 6.f);
      info.SetAttr<float>("leaky_relu_alpha", 0.1f);
    }
    info.SetAttr<bool>("enable_int8", true);
    info.SetInputScale("Input0_scale", {in_scale}, true);
    info.SetInputScale("Filter0_scale", ws, true);
    info.SetOutputScale("Output0_scale", {out_scale}, true);

    auto op = LiteOpRegistry::Global().Create("depthwise_conv2d");
    EXPECT(op != nullptr);
    EXPECT(op->Attach(info, &scope) && op->CheckShape() && op->InferShape());
    const int oh = (q.h + 2 * q.pad - 3) / q.stride + 1, ow = (q.w + 2 * q.pad - 3) / q.stride + 1;
    Tensor* y = scope.FindMutableTensor("y");
    EXPECT(y->dims() == DDim({q.n, q.c, oh, ow}));
    if (!run_on_device) {
      EXPECT(KernelRegistry::Global().Create("depthwise_conv2d", TARGET(kHIP), PRECISION(kInt8), DATALAYOUT(kNCHW)).size() == 2u);
      continue;
    }
    OpInfo h2d("io_copy");
    h2d.SetInput("Input", {"x"});
    h2d.SetOutput("Out", {"x_dev"});
    auto copy_op = LiteOpRegistry::Global().Create("io_copy");
    EXPECT(copy_op->Attach(h2d, &scope) && copy_op->InferShape());
    auto copy_kernels = copy_op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kAny), DATALAYOUT(kAny))}, "io_copy/host_to_device");
    copy_kernels[0]->Launch();
    info.SetInput("Input", {"x_dev"});
    EXPECT(op->Attach(info, &scope) && op->InferShape());
    auto kernels = op->CreateKernels({paddle::lite_api::Place(TARGET(kHIP), PRECISION(kInt8), DATALAYOUT(kNCHW))}, std::string("depthwise_conv2d/") + (q.out_int8 ? "int8_out" : "fp32_out"));
    EXPECT(kernels.size() == 1);
    if (kernels.size() != 1) continue;
    kernels[0]->Launch();
    kernels[0]->Launch();
    kernels[0]->mutable_context_as<HIPContext>()->Sync();
    Tensor y_host;
    y_host.CopyDataFrom(*y, TargetType::kHost);
    // merged parameters (conv_depthwise.cc:158-200, :257-322)
    std::vector<float> ms(q.c), mb(q.c);
    for (int i = 0; i < q.c; ++i) {
      ms[i] = q.out_int8 ? ws[i] * in_scale / out_scale : ws[i] * in_scale;
      mb[i] = q.out_int8 ? bd[i] / out_scale : bd[i];
    }
    plo_act act{ActCode(q.act), q.out_int8 ? 6.f / out_scale : 6.f, 0.1f, 6.f, 3.f, 6.f};
    if (q.out_int8) {
      std::vector<int8_t> want(static_cast<size_t>(q.n) * q.c * oh * ow);
      EXPECT(plo_dwconv3x3_int8(xd, fd, ms.data(), mb.data(), &act, 2, q.n, q.c, q.h, q.w, q.stride, q.pad, want.data()) == 0);
      EXPECT(y_host.memory_size() == want.size() && std::memcmp(want.data(), y_host.raw_data(), want.size()) == 0);
    } else {
      std::vector<float> want(static_cast<size_t>(q.n) * q.c * oh * ow);
      EXPECT(plo_dwconv3x3_int8(xd, fd, ms.data(), mb.data(), &act, 1, q.n, q.c, q.h, q.w, q.stride, q.pad, want.data()) == 0);
      EXPECT(y_host.memory_size() == want.size() * 4 && std::memcmp(want.data(), y_host.raw_data(), want.size() * 4) == 0);
    }
  }
}

// Two MobileNet blocks (depthwise 3x3 then pointwise 1x1, twice; the second
// depthwise layer has stride 2): conv2d -> sparse_conv2d by the detect pass,
// the whole program saved as a model file and loaded into an empty scope,
// precision and target casts placed by the chain pass, run on the device from
// an fp32 feed to an fp32 fetch, and compared with the oracle's chain.
static void MobileNetBlocks(bool run_on_device) {
  std::printf("mobilenet blocks from a model file\n");
  std::fflush(stdout);
  const int batch = 2, size0 = 12;
  const int ch[3] = {24, 40, 56};            // channels: input, after block 1, after block 2
  const int dw_stride[2] = {1, 2};
  // input scale of: dw1, pw1, dw2, pw2
  const float in_scale[4] = {0.02f, 0.03f, 0.025f, 0.04f};
  Scope scope;
  std::mt19937 gen(99);
  std::uniform_real_distribution<float> uni(0.f, 1.f);
  Tensor* a0 = scope.NewTensor("t0");
  a0->Resize({batch, ch[0], size0, size0});
  float* a0d = a0->mutable_data<float>(TargetType::kHost);
  for (int64_t i = 0; i < a0->numel(); ++i) a0d[i] = uni(gen) * 2.f - 1.f;
  std::vector<float> feed(a0d, a0d + a0->numel());
  std::vector<OpInfo> ops;
  std::vector<std::vector<int8_t>> dw_w(2), pw_w(2);
  std::vector<std::vector<float>> dw_ws(2), pw_ws(2), dw_b(2), pw_b(2);
  int size = size0;
  cpp::ProgramDesc prog;
  cpp::BlockDesc* block = prog.AddBlock();
  block->SetParentIdx(-1);
  auto add_var = [&](const std::string& name, bool persistable, VarDataType dt, const std::vector<int64_t>& shape) {
    cpp::VarDesc* v = block->AddVar();
    v->SetName(name);
    v->SetPersistable(persistable);
    v->SetDataType(dt);
    v->SetShape(shape);
  };
  add_var("t0", false, VarDataType::FP32, {batch, ch[0], size0, size0});
  for (int l = 0; l < 2; ++l) {
    const int c = ch[l], oc = ch[l + 1];
    const std::string n = std::to_string(l + 1);
    const int out_size = (size + 2 - 3) / dw_stride[l] + 1;
    // depthwise
    Tensor* f = scope.NewTensor("dw_w" + n);
    f->Resize({c, 1, 3, 3});
    int8_t* fd = f->mutable_data<int8_t>(TargetType::kHost);
    for (int64_t i = 0; i < f->numel(); ++i) fd[i] = static_cast<int8_t>(static_cast<int>(uni(gen) * 255.f) - 127);
    dw_w[l].assign(fd, fd + f->numel());
    Tensor* b = scope.NewTensor("dw_b" + n);
    b->Resize({c});
    float* bd = b->mutable_data<float>(TargetType::kHost);
    dw_b[l].resize(c);
    for (int i = 0; i < c; ++i) dw_b[l][i] = bd[i] = uni(gen) - 0.5f;
    dw_ws[l].resize(c);
    for (float& v : dw_ws[l]) v = 0.0005f + 0.001f * uni(gen);
    OpInfo dw("depthwise_conv2d");
    dw.SetInput("Input", {"t" + std::to_string(2 * l)});
    dw.SetInput("Filter", {"dw_w" + n});
    dw.SetInput("Bias", {"dw_b" + n});
    dw.SetOutput("Output", {"t" + std::to_string(2 * l + 1)});
    dw.SetAttr<std::vector<int>>("strides", {dw_stride[l], dw_stride[l]});
    dw.SetAttr<std::vector<int>>("paddings", {1, 1});
    dw.SetAttr<std::vector<int>>("dilations", {1, 1});
    dw.SetAttr<int>("groups", c);
    dw.SetAttr<bool>("with_act", true);
    dw.SetAttr<std::string>("act_type", "relu");
    dw.SetAttr<bool>("enable_int8", true);
    dw.SetInputScale("Input0_scale", {in_scale[2 * l]}, true);
    dw.SetInputScale("Filter0_scale", dw_ws[l], true);
    dw.SetOutputScale("Output0_scale", {1.f}, true);
    ops.push_back(dw);
    add_var("dw_w" + n, true, VarDataType::INT8, {c, 1, 3, 3});
    add_var("dw_b" + n, true, VarDataType::FP32, {c});
    add_var("t" + std::to_string(2 * l + 1), false, VarDataType::FP32, {batch, c, out_size, out_size});
    // pointwise
    Tensor* w = scope.NewTensor("pw_w" + n);
    w->Resize({oc, c, 1, 1});
    int8_t* wd = w->mutable_data<int8_t>(TargetType::kHost);
    for (int64_t i = 0; i < w->numel(); ++i) {
      int v = static_cast<int>(uni(gen) * 127.f) + 1;
      if (uni(gen) < 0.5f) v = -v;
      wd[i] = uni(gen) >= 0.7f ? static_cast<int8_t>(v) : 0;
    }
    pw_w[l].assign(wd, wd + w->numel());
    Tensor* pb = scope.NewTensor("pw_b" + n);
    pb->Resize({oc});
    float* pbd = pb->mutable_data<float>(TargetType::kHost);
    pw_b[l].resize(oc);
    for (int i = 0; i < oc; ++i) pw_b[l][i] = pbd[i] = (uni(gen) - 0.5f) * 0.2f;
    pw_ws[l].resize(oc);
    for (float& v : pw_ws[l]) v = 0.001f + 0.004f * uni(gen);
    OpInfo conv("conv2d");
    conv.SetInput("Input", {"t" + std::to_string(2 * l + 1)});
    conv.SetInput("Filter", {"pw_w" + n});
    conv.SetInput("Bias", {"pw_b" + n});
    conv.SetOutput("Output", {"t" + std::to_string(2 * l + 2)});
    conv.SetAttr<std::vector<int>>("strides", {1, 1});
    conv.SetAttr<std::vector<int>>("paddings", {0, 0});
    conv.SetAttr<std::vector<int>>("dilations", {1, 1});
    conv.SetAttr<int>("groups", 1);
    conv.SetAttr<bool>("with_act", true);
    conv.SetAttr<std::string>("act_type", "relu");
    conv.SetAttr<bool>("enable_int8", true);
    conv.SetInputScale("Input0_scale", {in_scale[2 * l + 1]}, true);
    conv.SetInputScale("Filter0_scale", pw_ws[l], true);
    conv.SetOutputScale("Output0_scale", {1.f}, true);
    ops.push_back(conv);
    // the detect pass reads the spatial size of the conv input from its tensor
    scope.NewTensor("t" + std::to_string(2 * l + 1))->Resize({batch, c, out_size, out_size});
    scope.NewTensor("t" + std::to_string(2 * l + 2));
    add_var("pw_b" + n, true, VarDataType::FP32, {oc});
    add_var("t" + std::to_string(2 * l + 2), false, VarDataType::FP32, {batch, oc, out_size, out_size});
    size = out_size;
  }
  mir::SparseConvDetectPass detect;
  detect.SetSparseThreshold(0.5f);
  EXPECT(detect.Apply(&ops, &scope) == 2);  // the two pointwise layers; the depthwise ops are left alone
  EXPECT(ops[0].Type() == "depthwise_conv2d" && ops[1].Type() == "sparse_conv2d");
  for (int l = 0; l < 2; ++l) {
    const std::string n = std::to_string(l + 1);
    const OpInfo& sp = ops[2 * l + 1];
    const Tensor* nz = scope.FindMutableTensor(sp.Input("NonZeroWeights").front());
    const Tensor* dif = scope.FindMutableTensor(sp.Input("Diffs").front());
    add_var(sp.Input("NonZeroWeights").front(), true, VarDataType::INT8, nz->dims().Vectorize());
    add_var(sp.Input("OcNonZeros").front(), true, VarDataType::INT32, {ch[l + 1]});
    add_var(sp.Input("Diffs").front(), true, VarDataType::INT32, dif->dims().Vectorize());
  }
  for (const OpInfo& op : ops) *block->AddOp() = op;

  // through a model file into an empty scope
  const std::string base = "/tmp/pl_mobilenet_blocks_" + std::to_string(static_cast<long>(getpid()));
  SaveModelNaive(base, scope, prog);
  Scope loaded;
  cpp::ProgramDesc back;
  LoadModelNaiveFromFile(base + ".nb", &loaded, &back);
  std::remove((base + ".nb").c_str());
  EXPECT(back.BlocksSize() == 1 && back.GetBlock(0)->OpsSize() == 4);
  if (back.BlocksSize() != 1 || back.GetBlock(0)->OpsSize() != 4) return;
  EXPECT(loaded.FindVar("pw_w1") == nullptr && loaded.FindVar("dw_w1") != nullptr);  // dense pointwise filters are gone
  loaded.NewTensor("t0")->Assign<float>(feed.data(), DDim({batch, ch[0], size0, size0}));
  mir::Int8ChainPass chain;
  std::vector<mir::ProgramStep> steps = chain.Apply(back.GetBlock(0)->ops(), {"t0"}, {"t4"}, &loaded);
  EXPECT(steps.size() == 7);
  if (steps.size() == 7) {
    EXPECT(steps[1].kernel == "calib/fp32_to_int8" && steps[2].kernel == "depthwise_conv2d/int8_out" && steps[3].kernel == "sparse_conv2d/int8_int8_out");
    EXPECT(steps[4].kernel == "depthwise_conv2d/int8_out" && steps[5].kernel == "sparse_conv2d/int8_fp32_out" && steps[6].kernel == "io_copy/device_to_host");
    EXPECT(steps[2].op.GetOutputScale("Output0_scale", true)[0] == in_scale[1]);
  }
  if (!run_on_device) return;
  mir::HipProgram program(steps, &loaded);
  program.Run();
  program.Run();
  const Tensor* got = loaded.FindMutableTensor("t4/host");
  EXPECT(got != nullptr);
  if (!got) return;

  // oracle chain
  std::vector<int8_t> q(feed.size());
  plo_fp32_to_int8(feed.data(), q.data(), in_scale[0], static_cast<int64_t>(feed.size()));
  std::vector<float> want;
  size = size0;
  plo_act relu{1, 6.f, 0.1f, 6.f, 3.f, 6.f};
  for (int l = 0; l < 2; ++l) {
    const int c = ch[l], oc = ch[l + 1];
    const int out_size = (size + 2 - 3) / dw_stride[l] + 1;
    const float dw_out = in_scale[2 * l + 1];
    std::vector<float> ms(c), mb(c);
    for (int i = 0; i < c; ++i) {
      ms[i] = dw_ws[l][i] * in_scale[2 * l] / dw_out;
      mb[i] = dw_b[l][i] / dw_out;
    }
    std::vector<int8_t> t(static_cast<size_t>(batch) * c * out_size * out_size);
    EXPECT(plo_dwconv3x3_int8(q.data(), dw_w[l].data(), ms.data(), mb.data(), &relu, 2, batch, c, size, size, dw_stride[l], 1, t.data()) == 0);
    const int hw = out_size * out_size;
    std::vector<float> ps(oc), pb(oc);
    plo_act act = relu;
    const bool last = l == 1;
    EXPECT(plo_merge_params(last ? 1 : 2, oc, pw_ws[l].data(), oc, in_scale[2 * l + 1], last ? 1.f : in_scale[2 * l + 2], pw_b[l].data(), ps.data(), pb.data(), &act) == 0);
    if (!last) {
      std::vector<int8_t> next(static_cast<size_t>(batch) * oc * hw);
      plo_dense_conv1x1(2, pw_w[l].data(), t.data(), pb.data(), ps.data(), next.data(), batch, oc, c, hw, &act, 1);
      q.swap(next);
    } else {
      want.resize(static_cast<size_t>(batch) * oc * hw);
      plo_dense_conv1x1(1, pw_w[l].data(), t.data(), pw_b[l].data(), ps.data(), want.data(), batch, oc, c, hw, &act, 1);
    }
    size = out_size;
  }
  EXPECT(got->memory_size() == want.size() * 4 && std::memcmp(want.data(), got->raw_data(), want.size() * 4) == 0);
}

// Pair launches of mir::HipProgram: pointwise (128 -> 128, int8 out) -> depthwise (stride 2 and stride 1, int8 out)
// -> pointwise (fp32 out) on 14 x 14 maps.  With pair launches on, a pointwise step and the depthwise step that
// alone reads its output run as one launch where the library says it pays (stride 2: at any batch; stride 1: not
// at a batch of two, which leaves most of the chip idle); the fetched output must not change by a bit.  A depthwise output with a second reader is
// never joined.
static void PairLaunches(bool run_on_device) {
  std::printf("pair launches\n");
  std::fflush(stdout);
  for (int stride = 1; stride <= 2; ++stride) {
    for (int second_reader = 0; second_reader <= 1; ++second_reader) {
      const int batch = 2, size = 14, c = 128;
      const int out_size = (size + 2 - 3) / stride + 1;
      Scope scope;
      std::mt19937 gen(500 + stride);
      std::uniform_real_distribution<float> uni(0.f, 1.f);
      Tensor* a0 = scope.NewTensor("p0");
      a0->Resize({batch, c, size, size});
      float* a0d = a0->mutable_data<float>(TargetType::kHost);
      for (int64_t i = 0; i < a0->numel(); ++i) a0d[i] = uni(gen) * 2.f - 1.f;
      std::vector<OpInfo> ops;
      auto pointwise = [&](const std::string& n, const std::string& in, const std::string& out, int oc, float in_scale) {
        Tensor* w = scope.NewTensor("ppw_w" + n);
        w->Resize({oc, c, 1, 1});
        int8_t* wd = w->mutable_data<int8_t>(TargetType::kHost);
        for (int64_t i = 0; i < w->numel(); ++i) {
          int v = static_cast<int>(uni(gen) * 127.f) + 1;
          if (uni(gen) < 0.5f) v = -v;
          wd[i] = uni(gen) >= 0.8f ? static_cast<int8_t>(v) : 0;
        }
        Tensor* b = scope.NewTensor("ppw_b" + n);
        b->Resize({oc});
        float* bd = b->mutable_data<float>(TargetType::kHost);
        for (int i = 0; i < oc; ++i) bd[i] = (uni(gen) - 0.5f) * 0.2f;
        std::vector<float> ws(oc);
        for (float& v : ws) v = 0.001f + 0.004f * uni(gen);
        OpInfo conv("conv2d");
        conv.SetInput("Input", {in});
        conv.SetInput("Filter", {"ppw_w" + n});
        conv.SetInput("Bias", {"ppw_b" + n});
        conv.SetOutput("Output", {out});
        conv.SetAttr<std::vector<int>>("strides", {1, 1});
        conv.SetAttr<std::vector<int>>("paddings", {0, 0});
        conv.SetAttr<std::vector<int>>("dilations", {1, 1});
        conv.SetAttr<int>("groups", 1);
        conv.SetAttr<bool>("with_act", true);
        conv.SetAttr<std::string>("act_type", "relu");
        conv.SetAttr<bool>("enable_int8", true);
        conv.SetInputScale("Input0_scale", {in_scale}, true);
        conv.SetInputScale("Filter0_scale", ws, true);
        conv.SetOutputScale("Output0_scale", {1.f}, true);
        ops.push_back(conv);
      };
      pointwise("1", "p0", "p1", c, 0.02f);
      scope.NewTensor("p1")->Resize({batch, c, size, size});
      {
        Tensor* f = scope.NewTensor("pdw_w");
        f->Resize({c, 1, 3, 3});
        int8_t* fd = f->mutable_data<int8_t>(TargetType::kHost);
        for (int64_t i = 0; i < f->numel(); ++i) fd[i] = static_cast<int8_t>(static_cast<int>(uni(gen) * 255.f) - 127);
        Tensor* b = scope.NewTensor("pdw_b");
        b->Resize({c});
        float* bd = b->mutable_data<float>(TargetType::kHost);
        for (int i = 0; i < c; ++i) bd[i] = uni(gen) - 0.5f;
        std::vector<float> ws(c);
        for (float& v : ws) v = 0.0005f + 0.001f * uni(gen);
        OpInfo dw("depthwise_conv2d");
        dw.SetInput("Input", {"p1"});
        dw.SetInput("Filter", {"pdw_w"});
        dw.SetInput("Bias", {"pdw_b"});
        dw.SetOutput("Output", {"p2"});
        dw.SetAttr<std::vector<int>>("strides", {stride, stride});
        dw.SetAttr<std::vector<int>>("paddings", {1, 1});
        dw.SetAttr<std::vector<int>>("dilations", {1, 1});
        dw.SetAttr<int>("groups", c);
        dw.SetAttr<bool>("with_act", true);
        dw.SetAttr<std::string>("act_type", "relu");
        dw.SetAttr<bool>("enable_int8", true);
        dw.SetInputScale("Input0_scale", {0.03f}, true);
        dw.SetInputScale("Filter0_scale", ws, true);
        dw.SetOutputScale("Output0_scale", {1.f}, true);
        ops.push_back(dw);
      }
      scope.NewTensor("p2")->Resize({batch, c, out_size, out_size});
      pointwise("2", "p2", "p3", 256, 0.025f);
      scope.NewTensor("p3");
      // a second reader of the pointwise output p1: it must then be written, so the pair is not joined
      if (second_reader) {
        pointwise("3", "p1", "p4", 128, 0.03f);
        scope.NewTensor("p4");
      }
      mir::SparseConvDetectPass detect;
      detect.SetSparseThreshold(0.5f);
      EXPECT(detect.Apply(&ops, &scope) == (second_reader ? 3 : 2));
      mir::Int8ChainPass chain;
      std::vector<std::string> fetches = {"p3"};
      if (second_reader) fetches.push_back("p4");
      std::vector<mir::ProgramStep> steps = chain.Apply(ops, {"p0"}, fetches, &scope);
      EXPECT(steps.size() >= 6);
      if (!run_on_device || steps.size() < 6) continue;
      mir::HipProgram program(steps, &scope);
      program.Run();
      EXPECT(program.pairs_joined_last_enqueue() == 0);
      const Tensor* got = scope.FindMutableTensor("p3/host");
      EXPECT(got != nullptr);
      if (!got) continue;
      std::vector<char> two_launches(static_cast<const char*>(got->raw_data()), static_cast<const char*>(got->raw_data()) + got->memory_size());
      program.set_pair_launch(true);
      program.Run();
      // stride 2 pays at any batch, stride 1 only when the launch fills the chip
      const size_t expect_pairs = (stride == 2 && !second_reader) ? 1 : 0;
      EXPECT(program.pairs_joined_last_enqueue() == expect_pairs);
      EXPECT(got->memory_size() == two_launches.size() && std::memcmp(got->raw_data(), two_launches.data(), two_launches.size()) == 0);
      program.set_pair_launch(false);
      program.Run();
      EXPECT(program.pairs_joined_last_enqueue() == 0);
      EXPECT(std::memcmp(got->raw_data(), two_launches.data(), two_launches.size()) == 0);
    }
  }
}

int main(int argc, char** argv) {
  const bool gpu = argc > 1 && std::string(argv[1]) == "--gpu";
  RegistryAndErrorPaths();
  const std::vector<Problem> problems = {
      {2, 64, 48, 8, 8, 0.8f, false, false, false, true, "relu", 11},
      {2, 57, 31, 7, 7, 0.8f, true, false, false, true, "relu6", 12},
      {1, 109, 16, 4, 8, 0.7f, false, false, false, false, "hard_swish", 13},
      {3, 128, 64, 14, 14, 0.85f, false, true, false, true, "leaky_relu", 14},
      {2, 96, 40, 7, 7, 0.75f, true, true, false, true, "", 15},
      {2, 128, 64, 8, 8, 0.75f, true, true, true, true, "hard_swish", 16},
      {2, 70, 33, 5, 5, 0.8f, false, true, true, true, "relu6", 17},
      {1, 512, 32, 14, 14, 0.85f, false, true, true, false, "leaky_relu", 18},
  };
  paddle::lite::kernels::hip::SetSparseConvReferenceQuirks(false);
  if (gpu && pl_device_count() < 1) {
    std::printf("no gfx950 device\n");
    return 2;
  }
  for (const Problem& p : problems) RunProblem(p, gpu);
  CalibChain(gpu);
  Int8Chain(gpu);
  BranchingGraph(gpu);
  HalfPrecision(gpu);
  ModelFile(gpu);
  Depthwise(gpu);
  MobileNetBlocks(gpu);
  PairLaunches(gpu);
  std::printf("%s: %d failure(s)\n", gpu ? "gpu" : "cpu", g_failures);
  return g_failures ? 1 : 0;
}
