// Host cost of a launch through the C++ operator surface, and the same steps replayed as a HIP graph.
//
// Builds the convolutional body of MobileNetV1-1.0 at batch 64 as op descriptions (thirteen times
// depthwise 3x3 + relu, then a dense-described 1x1 conv2d with 90 % zeros + relu, all enable_int8), lets
// SparseConvDetectPass turn the 1x1 layers into sparse_conv2d and Int8ChainPass place calib / io_copy, and
// runs the steps with mir::HipProgram on a stream of its own.  Printed as one JSON line:
//   host_enqueue_us     per step: host time of CheckShape + InferShape + KernelBase::Launch, averaged over
//                       whole sequences (the stream is drained between sequences, so no step waits for a
//                       full queue)
//   eager_sequence_us   the 26 convolution steps enqueued one by one, device time between two events
//   graph_sequence_us   the same 26 steps captured once (kernel nodes only) and replayed
//   graph_matches_eager the fetched fp32 output after graph replays equals the eager one byte for byte
//   pairs_joined, pair_launch_sequence_us, pair_launch_matches_eager
//                       the eager sequence with HipProgram's pair launches switched on
// Parity of this path against the CPU oracle is the business of tests/cpp/sparse_conv_hip_test.cc; this
// program only measures.
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "lite/core/op_registry.h"
#include "lite/core/optimizer/mir/int8_chain_pass.h"
#include "lite/core/optimizer/mir/sparse_conv_detect_pass.h"
#include "lite/operators/conv_op.h"
#include "lite/operators/sparse_conv_op.h"

using namespace paddle::lite;  // NOLINT

#define HIP_OK(call)                                                                         \
  do {                                                                                       \
    hipError_t e_ = (call);                                                                  \
    if (e_ != hipSuccess) {                                                                  \
      std::fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      return 1;                                                                              \
    }                                                                                        \
  } while (0)

namespace {

const int kPointwise[13][3] = {{32, 64, 112},  {64, 128, 56},  {128, 128, 56}, {128, 256, 28}, {256, 256, 28},  {256, 512, 14},  {512, 512, 14},
                               {512, 512, 14}, {512, 512, 14}, {512, 512, 14}, {512, 512, 14}, {512, 1024, 7}, {1024, 1024, 7}};
const int kDepthwiseStride[13] = {1, 2, 1, 2, 1, 2, 1, 1, 1, 1, 1, 2, 1};

std::string Var(int i) { return "t" + std::to_string(i); }

double NowUs() { return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

}  // namespace

int main(int argc, char** argv) {
  int batch = 64, sequences = 40;
  for (int i = 1; i + 1 < argc; i += 2) {
    if (!std::strcmp(argv[i], "--batch")) batch = std::atoi(argv[i + 1]);
    if (!std::strcmp(argv[i], "--sequences")) sequences = std::atoi(argv[i + 1]);
  }
  if (batch < 1 || batch > 256 || sequences < 1 || sequences > 10000) {
    std::fprintf(stderr, "usage: lite_program_bench [--batch 1..256] [--sequences 1..10000]\n");
    return 2;
  }
  hipStream_t stream = nullptr;
  HIP_OK(hipSetDevice(0));
  HIP_OK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
  ContextScheduler::Global().SetDefaultHIPStream(stream);

  Scope scope;
  std::mt19937 gen(7);
  std::uniform_real_distribution<float> uni(0.f, 1.f);
  const float sparsity = 0.9f, dw_in_scale = 0.01f;
  std::vector<OpInfo> ops;
  int size = 112;  // spatial size of the body's input, 32 channels
  {
    Tensor* t0 = scope.NewTensor(Var(0));
    t0->Resize({batch, 32, size, size});
    float* d = t0->mutable_data<float>(TargetType::kHost);
    for (int64_t i = 0; i < t0->numel(); ++i) d[i] = (uni(gen) * 2.f - 1.f) * 127.f * dw_in_scale;
  }
  for (int l = 0; l < 13; ++l) {
    const int c = kPointwise[l][0], oc = kPointwise[l][1], out_size = kPointwise[l][2], stride = kDepthwiseStride[l];
    if ((size + 2 - 3) / stride + 1 != out_size) {
      std::fprintf(stderr, "layer table is inconsistent at %d\n", l);
      return 1;
    }
    const std::string n = std::to_string(l + 1);
    // depthwise 3x3: uniform filters, scales as in the Python workload of the same layer
    Tensor* f = scope.NewTensor("dw_w" + n);
    f->Resize({c, 1, 3, 3});
    int8_t* fd = f->mutable_data<int8_t>(TargetType::kHost);
    for (int64_t i = 0; i < f->numel(); ++i) fd[i] = static_cast<int8_t>(static_cast<int>(uni(gen) * 255.f) - 127);
    Tensor* b = scope.NewTensor("dw_b" + n);
    b->Resize({c});
    float* bd = b->mutable_data<float>(TargetType::kHost);
    for (int i = 0; i < c; ++i) bd[i] = (uni(gen) - 0.5f) * 0.2f;
    std::vector<float> dw_ws(c);
    double mean_ws = 0;
    for (float& v : dw_ws) {
      v = 0.001f + 0.019f * uni(gen);
      mean_ws += v / c;
    }
    // scale of the depthwise output = input scale of the pointwise layer: three sigma of the accumulator on 127
    const float pw_in_scale = static_cast<float>(3.0 * 3.0 * 73.3 * 40.0 * mean_ws * dw_in_scale / 127.0);
    OpInfo dw("depthwise_conv2d");
    dw.SetInput("Input", {Var(2 * l)});
    dw.SetInput("Filter", {"dw_w" + n});
    dw.SetInput("Bias", {"dw_b" + n});
    dw.SetOutput("Output", {Var(2 * l + 1)});
    dw.SetAttr<std::vector<int>>("strides", {stride, stride});
    dw.SetAttr<std::vector<int>>("paddings", {1, 1});
    dw.SetAttr<std::vector<int>>("dilations", {1, 1});
    dw.SetAttr<int>("groups", c);
    dw.SetAttr<bool>("with_act", true);
    dw.SetAttr<std::string>("act_type", "relu");
    dw.SetAttr<bool>("enable_int8", true);
    dw.SetInputScale("Input0_scale", {dw_in_scale}, true);
    dw.SetInputScale("Filter0_scale", dw_ws, true);
    dw.SetOutputScale("Output0_scale", {1.f}, true);
    ops.push_back(dw);
    // pointwise 1x1, described dense; 90 % of the weights are zero
    Tensor* w = scope.NewTensor("pw_w" + n);
    w->Resize({oc, c, 1, 1});
    int8_t* wd = w->mutable_data<int8_t>(TargetType::kHost);
    for (int64_t i = 0; i < w->numel(); ++i) {
      int v = static_cast<int>(uni(gen) * 127.f) + 1;
      if (uni(gen) < 0.5f) v = -v;
      wd[i] = uni(gen) >= sparsity ? static_cast<int8_t>(v) : 0;
    }
    Tensor* pb = scope.NewTensor("pw_b" + n);
    pb->Resize({oc});
    float* pbd = pb->mutable_data<float>(TargetType::kHost);
    for (int i = 0; i < oc; ++i) pbd[i] = (uni(gen) - 0.5f) * 0.2f;
    // weight scales such that three sigma of the accumulator lands on the next layer's 127
    const double sigma_acc = std::sqrt(c * (1.0 - sparsity)) * 64.0 * 40.0;
    std::vector<float> pw_ws(oc);
    for (float& v : pw_ws) v = static_cast<float>(127.0 * dw_in_scale / (3.0 * sigma_acc * pw_in_scale) * (0.8 + 0.4 * uni(gen)));
    OpInfo conv("conv2d");
    conv.SetInput("Input", {Var(2 * l + 1)});
    conv.SetInput("Filter", {"pw_w" + n});
    conv.SetInput("Bias", {"pw_b" + n});
    conv.SetOutput("Output", {Var(2 * l + 2)});
    conv.SetAttr<std::vector<int>>("strides", {1, 1});
    conv.SetAttr<std::vector<int>>("paddings", {0, 0});
    conv.SetAttr<std::vector<int>>("dilations", {1, 1});
    conv.SetAttr<int>("groups", 1);
    conv.SetAttr<bool>("with_act", true);
    conv.SetAttr<std::string>("act_type", "relu");
    conv.SetAttr<bool>("enable_int8", true);
    conv.SetInputScale("Input0_scale", {pw_in_scale}, true);
    conv.SetInputScale("Filter0_scale", pw_ws, true);
    conv.SetOutputScale("Output0_scale", {1.f}, true);
    ops.push_back(conv);
    // the detect pass reads the spatial size of the conv input from its tensor
    scope.NewTensor(Var(2 * l + 1))->Resize({batch, c, out_size, out_size});
    scope.NewTensor(Var(2 * l + 2));
    size = out_size;
  }
  try {
    mir::SparseConvDetectPass detect;
    detect.SetSparseThreshold(0.5f);
    const int converted = detect.Apply(&ops, &scope);
    if (converted != 13) {
      std::fprintf(stderr, "the detect pass converted %d of 13 pointwise layers\n", converted);
      return 1;
    }
    mir::Int8ChainPass chain;
    std::vector<mir::ProgramStep> steps = chain.Apply(ops, {Var(0)}, {Var(26)}, &scope);
    // io_copy to the device, calib to int8, 26 convolutions, io_copy of the fp32 result to the host
    if (steps.size() != 29) {
      std::fprintf(stderr, "expected 29 steps, found %zu\n", steps.size());
      return 1;
    }
    const size_t first = 2, last = 28;
    mir::HipProgram program(steps, &scope);
    program.Run();
    program.Run();
    const Tensor* fetched = scope.FindMutableTensor(Var(26) + "/host");
    if (!fetched) {
      std::fprintf(stderr, "no fetched tensor\n");
      return 1;
    }
    std::vector<char> eager_out(fetched->memory_size());
    std::memcpy(eager_out.data(), fetched->raw_data(), eager_out.size());

    // host time per step, whole sequences, stream drained between them
    std::vector<double> host_us(steps.size(), 0.0);
    for (int s = 0; s < sequences; ++s) {
      for (size_t i = first; i < last; ++i) {
        const double t0 = NowUs();
        program.Enqueue(i, i + 1);
        host_us[i] += NowUs() - t0;
      }
      program.Sync();
    }
    // eager sequence: device time of back-to-back sequences
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    for (int s = 0; s < 5; ++s) program.Enqueue(first, last);
    HIP_OK(hipEventRecord(e0, stream));
    const double h0 = NowUs();
    for (int s = 0; s < sequences; ++s) program.Enqueue(first, last);
    const double host_sequence_us = (NowUs() - h0) / sequences;
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipEventSynchronize(e1));
    float ms = 0.f;
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    const double eager_us = ms * 1e3 / sequences;

    // the same steps as a graph: kernel nodes only (the steps enqueue nothing but kernels)
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    HIP_OK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    program.Enqueue(first, last);
    HIP_OK(hipStreamEndCapture(stream, &graph));
    size_t nodes = 0;
    HIP_OK(hipGraphGetNodes(graph, nullptr, &nodes));
    HIP_OK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    bool graph_ok = true;
    for (int r = 0; r < 3; ++r) {
      // eager work and a wait between replays, then the replay, then the fetch step eagerly
      program.Enqueue(first, first + 3);
      program.Sync();
      HIP_OK(hipGraphLaunch(exec, stream));
      program.Enqueue(last, steps.size());
      program.Sync();
      graph_ok = graph_ok && fetched->memory_size() == eager_out.size() && std::memcmp(fetched->raw_data(), eager_out.data(), eager_out.size()) == 0;
    }
    for (int s = 0; s < 5; ++s) HIP_OK(hipGraphLaunch(exec, stream));
    HIP_OK(hipEventRecord(e0, stream));
    const double g0 = NowUs();
    for (int s = 0; s < sequences; ++s) HIP_OK(hipGraphLaunch(exec, stream));
    const double host_graph_us = (NowUs() - g0) / sequences;
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipEventSynchronize(e1));
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    const double graph_us = ms * 1e3 / sequences;

    // pair launches: a pointwise step and the depthwise step behind it as one launch where the library says it pays
    program.set_pair_launch(true);
    program.Run();
    const size_t pairs = program.pairs_joined_last_enqueue();
    const bool pairs_ok = fetched->memory_size() == eager_out.size() && std::memcmp(fetched->raw_data(), eager_out.data(), eager_out.size()) == 0;
    for (int s = 0; s < 5; ++s) program.Enqueue(first, last);
    HIP_OK(hipEventRecord(e0, stream));
    const double p0 = NowUs();
    for (int s = 0; s < sequences; ++s) program.Enqueue(first, last);
    const double pairs_host_us = (NowUs() - p0) / sequences;
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipEventSynchronize(e1));
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    const double pairs_us = ms * 1e3 / sequences;
    program.set_pair_launch(false);

    std::printf("{\"workload\": \"mobilenet_v1_body_int8 through mir::HipProgram\", \"batch\": %d, \"sequences\": %d, \"steps\": [", batch, sequences);
    double host_sum = 0;
    for (size_t i = first; i < last; ++i) {
      host_sum += host_us[i] / sequences;
      std::printf("%s{\"kernel\": \"%s\", \"host_enqueue_us\": %.2f}", i == first ? "" : ", ", steps[i].kernel.c_str(), host_us[i] / sequences);
    }
    std::printf("], \"host_enqueue_us_per_sequence\": %.1f, \"host_enqueue_us_per_sequence_back_to_back\": %.1f, \"eager_sequence_us\": %.1f, \"graph_nodes\": %zu, \"graph_sequence_us\": %.1f, "
                "\"host_us_per_graph_launch\": %.1f, \"graph_matches_eager\": %s, \"pairs_joined\": %zu, \"pair_launch_sequence_us\": %.1f, \"pair_launch_host_enqueue_us_per_sequence\": %.1f, \"pair_launch_matches_eager\": %s}\n",
                host_sum, host_sequence_us, eager_us, nodes, graph_us, host_graph_us, graph_ok ? "true" : "false", pairs, pairs_us, pairs_host_us, pairs_ok ? "true" : "false");
    HIP_OK(hipGraphExecDestroy(exec));
    HIP_OK(hipGraphDestroy(graph));
    HIP_OK(hipEventDestroy(e0));
    HIP_OK(hipEventDestroy(e1));
    return graph_ok && pairs_ok ? 0 : 1;
  } catch (const FatalError& e) {
    std::fprintf(stderr, "fatal: %s\n", e.what());
    return 1;
  }
}
