// Command-line driver of the model-file code of this package, used by the
// tests: dumps a "<name>.nb" file as text, writes an example file, and runs
// round-trip and malformed-input checks.  The dump format and the example are
// the same as those of oracle/ref_model_file.cc, which drives the
// reference's own classes, so the two can be compared line by line.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <string>
#include <typeinfo>
#include <vector>

#include "lite/model_parser/model_parser.h"

using namespace paddle::lite;  // NOLINT

namespace {

uint64_t Fnv(const void* data, size_t n) {
  uint64_t h = 1469598103934665603ull;
  const uint8_t* p = static_cast<const uint8_t*>(data);
  for (size_t i = 0; i < n; ++i) h = (h ^ p[i]) * 1099511628211ull;
  return h;
}

const char* VarTypeName(VarDataType t) {
  switch (t) {
    case VarDataType::BOOL: return "BOOL";
    case VarDataType::INT8: return "INT8";
    case VarDataType::UINT8: return "UINT8";
    case VarDataType::INT16: return "INT16";
    case VarDataType::INT32: return "INT32";
    case VarDataType::INT64: return "INT64";
    case VarDataType::FP16: return "FP16";
    case VarDataType::FP32: return "FP32";
    case VarDataType::FP64: return "FP64";
    case VarDataType::LOD_TENSOR: return "LOD_TENSOR";
    case VarDataType::FEED_MINIBATCH: return "FEED_MINIBATCH";
    case VarDataType::FETCH_LIST: return "FETCH_LIST";
    default: return "OTHER";
  }
}

void PrintStrings(const std::vector<std::string>& v) {
  for (auto& s : v) std::printf(" \"%s\"", s.c_str());
  std::printf("\n");
}

void PrintAttr(const std::string& name, const std::any& a) {
  const std::type_info& t = a.type();
  std::printf(" attr %s kind ", name.c_str());
  if (t == typeid(int)) {
    std::printf("INT: %d\n", std::any_cast<int>(a));
  } else if (t == typeid(float)) {
    std::printf("FLOAT: %.9g\n", std::any_cast<float>(a));
  } else if (t == typeid(bool)) {
    std::printf("BOOLEAN: %d\n", std::any_cast<bool>(a) ? 1 : 0);
  } else if (t == typeid(int64_t)) {
    std::printf("LONG: %lld\n", static_cast<long long>(std::any_cast<int64_t>(a)));
  } else if (t == typeid(double)) {
    std::printf("FLOAT64: %.17g\n", std::any_cast<double>(a));
  } else if (t == typeid(std::string)) {
    std::printf("STRING: \"%s\"\n", std::any_cast<const std::string&>(a).c_str());
  } else if (t == typeid(std::vector<int>)) {
    std::printf("INTS:");
    for (int v : std::any_cast<const std::vector<int>&>(a)) std::printf(" %d", v);
    std::printf("\n");
  } else if (t == typeid(std::vector<float>)) {
    std::printf("FLOATS:");
    for (float v : std::any_cast<const std::vector<float>&>(a)) std::printf(" %.9g", v);
    std::printf("\n");
  } else if (t == typeid(std::vector<int64_t>)) {
    std::printf("LONGS:");
    for (int64_t v : std::any_cast<const std::vector<int64_t>&>(a)) std::printf(" %lld", static_cast<long long>(v));
    std::printf("\n");
  } else if (t == typeid(std::vector<double>)) {
    std::printf("FLOAT64S:");
    for (double v : std::any_cast<const std::vector<double>&>(a)) std::printf(" %.17g", v);
    std::printf("\n");
  } else if (t == typeid(std::vector<std::string>)) {
    std::printf("STRINGS:");
    PrintStrings(std::any_cast<const std::vector<std::string>&>(a));
  } else {
    std::printf("OTHER: ?\n");
  }
}

void DumpLoaded(uint16_t meta_version, const cpp::ProgramDesc& prog, const Scope& scope) {
  std::printf("meta_version %d\n", meta_version);
  if (prog.HasVersion()) std::printf("version %lld\n", static_cast<long long>(prog.Version()));
  for (size_t b = 0; b < prog.BlocksSize(); ++b) {
    const cpp::BlockDesc& block = *prog.GetBlock(b);
    std::printf("block %d parent %d forward %d\n", block.Idx(), block.ParentIdx(), block.ForwardBlockIdx());
    for (const cpp::VarDesc& var : block.vars()) {
      std::printf("var %s type %s persistable %d", var.Name().c_str(), VarTypeName(var.GetType()), var.Persistable() ? 1 : 0);
      if (var.GetType() == VarDataType::LOD_TENSOR) {
        std::printf(" dtype %s shape", VarTypeName(var.GetDataType()));
        for (int64_t d : var.GetShape()) std::printf(" %lld", static_cast<long long>(d));
      }
      std::printf("\n");
    }
    for (const OpInfo& op : block.ops()) {
      std::printf("op %s\n", op.Type().c_str());
      for (auto& kv : op.inputs()) {
        std::printf(" in %s:", kv.first.c_str());
        PrintStrings(kv.second);
      }
      for (auto& kv : op.outputs()) {
        std::printf(" out %s:", kv.first.c_str());
        PrintStrings(kv.second);
      }
      for (auto& kv : op.attrs()) PrintAttr(kv.first, kv.second);
    }
  }
  for (const std::string& name : scope.LocalVarNames()) {  // name order
    const Tensor& t = scope.FindVar(name)->Get<Tensor>();
    std::printf("tensor %s precision %d dims", name.c_str(), static_cast<int>(t.precision()));
    for (int64_t d : t.dims().Vectorize()) std::printf(" %lld", static_cast<long long>(d));
    std::printf(" bytes %zu fnv %016llx\n", t.memory_size(), static_cast<unsigned long long>(Fnv(t.raw_data(), t.memory_size())));
  }
}

std::string ReadFile(const std::string& path) {
  std::ifstream f(path, std::ios::binary);
  if (!f.good()) {
    std::fprintf(stderr, "cannot open %s\n", path.c_str());
    std::exit(2);
  }
  return std::string((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}

int Dump(const std::string& path) {
  const std::string bytes = ReadFile(path);
  cpp::ProgramDesc prog;
  Scope scope;
  std::string error;
  if (!TryLoadModelNaiveFromMemory(bytes, &scope, &prog, &error)) {
    std::printf("error: %s\n", error.c_str());
    return 1;
  }
  uint16_t meta_version;
  std::memcpy(&meta_version, bytes.data(), 2);
  DumpLoaded(meta_version, prog, scope);
  return 0;
}

template <typename T>
void Fill(Scope* scope, const std::string& name, const std::vector<int64_t>& dims, int mul, int mod, int sub) {
  Tensor* t = scope->NewTensor(name);
  t->Resize(dims);
  T* d = t->mutable_data<T>(TargetType::kHost);
  for (int64_t i = 0; i < t->numel(); ++i) d[i] = static_cast<T>((i * mul) % mod - sub);
  t->set_persistable(true);
}

void AddVar(cpp::BlockDesc* block, const std::string& name, VarDataType type, bool persistable, VarDataType dtype, const std::vector<int64_t>& shape) {
  cpp::VarDesc* var = block->AddVar();
  var->SetName(name);
  var->SetType(type);
  var->SetPersistable(persistable);
  var->SetDataType(dtype);
  var->SetShape(shape);
}

void BuildExample(cpp::ProgramDesc* prog, Scope* scope) {
  cpp::BlockDesc* block = prog->AddBlock();
  block->SetIdx(0);
  block->SetParentIdx(-1);
  prog->SetVersion(2012000);
  AddVar(block, "feed", VarDataType::FEED_MINIBATCH, true, VarDataType::FP32, {});
  AddVar(block, "x", VarDataType::LOD_TENSOR, false, VarDataType::FP32, {-1, 8, 4, 4});
  AddVar(block, "conv1_w_nonzeros_output", VarDataType::LOD_TENSOR, true, VarDataType::FP32, {12});
  AddVar(block, "conv1_w_oc_nonzeros", VarDataType::LOD_TENSOR, true, VarDataType::INT32, {6});
  AddVar(block, "conv1_w_ic_diffs", VarDataType::LOD_TENSOR, true, VarDataType::INT32, {12});
  AddVar(block, "conv1_b", VarDataType::LOD_TENSOR, true, VarDataType::FP32, {6});
  AddVar(block, "conv2_w_nonzeros_output", VarDataType::LOD_TENSOR, true, VarDataType::INT8, {9});
  AddVar(block, "y", VarDataType::LOD_TENSOR, false, VarDataType::FP32, {-1, 6, 4, 4});
  AddVar(block, "fetch", VarDataType::FETCH_LIST, true, VarDataType::FP32, {});
  Fill<float>(scope, "conv1_w_nonzeros_output", {12}, 7, 13, 6);
  Fill<int32_t>(scope, "conv1_w_oc_nonzeros", {6}, 2, 100, 0);
  Fill<int32_t>(scope, "conv1_w_ic_diffs", {12}, 64, 1000, 448);
  Fill<float>(scope, "conv1_b", {6}, 3, 5, 2);
  Fill<int8_t>(scope, "conv2_w_nonzeros_output", {9}, 37, 255, 127);
  {
    OpInfo op("feed");
    op.SetInput("X", {"feed"});
    op.SetOutput("Out", {"x"});
    op.SetAttr<int>("col", 0);
    *block->AddOp() = op;
  }
  {
    OpInfo op("sparse_conv2d");
    op.SetInput("Input", {"x"});
    op.SetInput("NonZeroWeights", {"conv1_w_nonzeros_output"});
    op.SetInput("OcNonZeros", {"conv1_w_oc_nonzeros"});
    op.SetInput("Diffs", {"conv1_w_ic_diffs"});
    op.SetInput("Bias", {"conv1_b"});
    op.SetOutput("Output", {"y"});
    op.SetAttr<std::vector<int>>("strides", {1, 1});
    op.SetAttr<std::vector<int>>("paddings", {0, 0});
    op.SetAttr<std::vector<int>>("dilations", {1, 1});
    op.SetAttr<int>("groups", 1);
    op.SetAttr<int>("first_ic", 3);
    op.SetAttr<int>("flag_semi", 1);
    op.SetAttr<bool>("with_act", true);
    op.SetAttr<bool>("enable_int8", false);
    op.SetAttr<std::string>("act_type", "leaky_relu");
    op.SetAttr<float>("leaky_relu_alpha", 0.1f);
    op.SetAttr<std::vector<float>>("Input0_scale", {0.0125f});
    op.SetAttr<std::vector<float>>("Filter0_scale", {0.5f, 0.25f, 0.125f, 1.5f, 2.5f, 3.0f});
    op.SetAttr<int64_t>("op_role", 4294967296ll + 5);
    op.SetAttr<std::vector<int64_t>>("shape64", {-1, 1099511627776ll});
    op.SetAttr<std::vector<std::string>>("op_callstack", {"a", "", "line three"});
    op.SetAttr<double>("eps64", 1e-12);
    op.SetAttr<std::vector<double>>("f64s", {0.5, -2.25});
    *block->AddOp() = op;
  }
  {
    OpInfo op("fetch");
    op.SetInput("X", {"y"});
    op.SetOutput("Out", {"fetch"});
    op.SetAttr<int>("col", 0);
    *block->AddOp() = op;
  }
}

int WriteExample(const std::string& path, uint16_t meta_version) {
  cpp::ProgramDesc prog;
  Scope scope;
  BuildExample(&prog, &scope);
  const std::string bytes = SerializeModelNaive(scope, prog, meta_version);
  std::ofstream f(path, std::ios::binary | std::ios::trunc);
  f.write(bytes.data(), static_cast<std::streamsize>(bytes.size()));
  return f.good() ? 0 : 1;
}

#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) {                                                          \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);         \
      ++failures;                                                           \
    }                                                                       \
  } while (0)

int SelfTest() {
  int failures = 0;
  for (uint16_t meta : {uint16_t(1), uint16_t(2)}) {
    cpp::ProgramDesc prog;
    Scope scope;
    BuildExample(&prog, &scope);
    const std::string bytes = SerializeModelNaive(scope, prog, meta);
    cpp::ProgramDesc back;
    Scope loaded;
    std::string error;
    EXPECT(TryLoadModelNaiveFromMemory(bytes, &loaded, &back, &error));
    // a second generation of the file is byte-identical to the first
    EXPECT(SerializeModelNaive(loaded, back, meta) == bytes);
    EXPECT(back.BlocksSize() == 1 && back.GetBlock(0)->OpsSize() == 3 && back.GetBlock(0)->VarsSize() == 9);
    const OpInfo& op = back.GetBlock(0)->GetOp(1);
    EXPECT(op.Type() == "sparse_conv2d");
    EXPECT(op.GetAttr<int>("first_ic") == 3 && op.GetAttr<int>("flag_semi") == 1);
    EXPECT(op.GetAttr<float>("leaky_relu_alpha") == 0.1f);
    EXPECT(op.GetAttr<std::vector<float>>("Filter0_scale").size() == 6);
    EXPECT(op.GetAttr<int64_t>("op_role") == 4294967301ll);
    EXPECT(op.Input("Diffs").front() == "conv1_w_ic_diffs");
    const Tensor* diffs = loaded.FindMutableTensor("conv1_w_ic_diffs");
    EXPECT(diffs && diffs->precision() == PrecisionType::kInt32 && diffs->numel() == 12 && diffs->persistable());
    EXPECT(diffs && diffs->data<int32_t>()[3] == (3 * 64) % 1000 - 448);
    EXPECT(loaded.FindVar("x") == nullptr);  // not a parameter
    // every truncation of the file is refused, never read past its end
    int refused = 0;
    for (size_t n = 0; n < bytes.size(); ++n) {
      cpp::ProgramDesc p2;
      Scope s2;
      if (!TryLoadModelNaiveFromMemory(bytes.substr(0, n), &s2, &p2, &error)) ++refused;
    }
    EXPECT(refused == static_cast<int>(bytes.size()));
    // offsets that point outside the buffer are refused
    std::string bad = bytes;
    const size_t root = 2 + 16 + 8;
    const uint32_t far = 0x7fffffff;
    std::memcpy(&bad[root], &far, 4);
    cpp::ProgramDesc p3;
    Scope s3;
    EXPECT(!TryLoadModelNaiveFromMemory(bad, &s3, &p3, &error));
  }
  {
    // meta version 0 (the format before v2.7) and unknown versions
    std::string old(64, '\0');
    cpp::ProgramDesc p;
    Scope s;
    std::string error;
    EXPECT(!TryLoadModelNaiveFromMemory(old, &s, &p, &error) && error.find("upgraded") != std::string::npos);
    old[0] = 9;
    EXPECT(!TryLoadModelNaiveFromMemory(old, &s, &p, &error) && error.find("cannot be recognized") != std::string::npos);
  }
  std::printf(failures ? "model file selftest: %d failure(s)\n" : "model file selftest: ok\n", failures);
  return failures ? 1 : 0;
}

}  // namespace

int main(int argc, char** argv) {
  const std::string cmd = argc >= 2 ? argv[1] : "";
  if (cmd == "dump" && argc >= 3) return Dump(argv[2]);
  if (cmd == "write-example" && argc >= 3) return WriteExample(argv[2], argc >= 4 ? static_cast<uint16_t>(std::atoi(argv[3])) : 2);
  if (cmd == "selftest") return SelfTest();
  std::fprintf(stderr, "usage: model_file_tool dump FILE | write-example FILE [META_VERSION] | selftest\n");
  return 2;
}
