// Test infrastructure: drives the REFERENCE's own model-file classes
// (lite/model_parser/flatbuffers/*, its checked-in flatc output under
// third-party/flatbuffers/pre-build, lite/core/{scope,tensor}) to write an
// example "<name>.nb" file and to dump any such file as text.  Built only
// where the reference checkout is present, into oracle/_ref/; the sequence of
// writes in WriteExample / reads in Dump restates
// lite/model_parser/model_parser.cc:470-535 (SaveModelNaive) and :838-905
// (LoadModelFbsFromFile), which cannot be compiled here themselves (they need
// protobuf and a generated version header).
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <set>
#include <string>
#include <vector>

#include "lite/core/model/base/io.h"
#include "lite/core/scope.h"
#include "lite/core/tensor.h"
#include "lite/model_parser/flatbuffers/io.h"
#include "lite/model_parser/flatbuffers/program_desc.h"

using namespace paddle::lite;  // NOLINT

namespace {

uint64_t Fnv(const void* data, size_t n) {
  uint64_t h = 1469598103934665603ull;
  const uint8_t* p = static_cast<const uint8_t*>(data);
  for (size_t i = 0; i < n; ++i) h = (h ^ p[i]) * 1099511628211ull;
  return h;
}

template <typename T>
void Fill(Scope* scope, const std::string& name, PrecisionType prec, const std::vector<int64_t>& dims, int mul, int mod, int sub) {
  auto* t = scope->Var(name)->GetMutable<Tensor>();
  t->Resize(dims);
  t->set_precision(prec);
  T* d = t->mutable_data<T>();
  for (int64_t i = 0; i < t->numel(); ++i) d[i] = static_cast<T>((i * mul) % mod - sub);
  t->set_persistable(true);
}

void AddVar(fbs::BlockDesc* block, const std::string& name, VarDataType type, bool persistable, VarDataType dtype, const std::vector<int64_t>& shape) {
  fbs::VarDesc var(block->AddVar<fbs::proto::VarDescT>());
  var.SetName(name);
  var.SetType(type);
  var.SetPersistable(persistable);
  var.SetDataType(dtype);
  var.SetShape(shape);
}

void BuildExample(fbs::ProgramDesc* prog, Scope* scope) {
  fbs::BlockDesc block(prog->AddBlock<fbs::proto::BlockDescT>());
  block.SetIdx(0);
  block.SetParentIdx(-1);
  prog->SetVersion(2012000);
  AddVar(&block, "feed", VarDataType::FEED_MINIBATCH, true, VarDataType::FP32, {});
  AddVar(&block, "x", VarDataType::LOD_TENSOR, false, VarDataType::FP32, {-1, 8, 4, 4});
  AddVar(&block, "conv1_w_nonzeros_output", VarDataType::LOD_TENSOR, true, VarDataType::FP32, {12});
  AddVar(&block, "conv1_w_oc_nonzeros", VarDataType::LOD_TENSOR, true, VarDataType::INT32, {6});
  AddVar(&block, "conv1_w_ic_diffs", VarDataType::LOD_TENSOR, true, VarDataType::INT32, {12});
  AddVar(&block, "conv1_b", VarDataType::LOD_TENSOR, true, VarDataType::FP32, {6});
  AddVar(&block, "conv2_w_nonzeros_output", VarDataType::LOD_TENSOR, true, VarDataType::INT8, {9});
  AddVar(&block, "y", VarDataType::LOD_TENSOR, false, VarDataType::FP32, {-1, 6, 4, 4});
  AddVar(&block, "fetch", VarDataType::FETCH_LIST, true, VarDataType::FP32, {});
  Fill<float>(scope, "conv1_w_nonzeros_output", PRECISION(kFloat), {12}, 7, 13, 6);
  Fill<int32_t>(scope, "conv1_w_oc_nonzeros", PRECISION(kInt32), {6}, 2, 100, 0);
  Fill<int32_t>(scope, "conv1_w_ic_diffs", PRECISION(kInt32), {12}, 64, 1000, 448);
  Fill<float>(scope, "conv1_b", PRECISION(kFloat), {6}, 3, 5, 2);
  Fill<int8_t>(scope, "conv2_w_nonzeros_output", PRECISION(kInt8), {9}, 37, 255, 127);
  {
    fbs::OpDesc op(block.AddOp<fbs::proto::OpDescT>());
    op.SetType("feed");
    op.SetInput("X", {"feed"});
    op.SetOutput("Out", {"x"});
    op.SetAttr<int32_t>("col", 0);
  }
  {
    fbs::OpDesc op(block.AddOp<fbs::proto::OpDescT>());
    op.SetType("sparse_conv2d");
    op.SetInput("Input", {"x"});
    op.SetInput("NonZeroWeights", {"conv1_w_nonzeros_output"});
    op.SetInput("OcNonZeros", {"conv1_w_oc_nonzeros"});
    op.SetInput("Diffs", {"conv1_w_ic_diffs"});
    op.SetInput("Bias", {"conv1_b"});
    op.SetOutput("Output", {"y"});
    op.SetAttr<std::vector<int>>("strides", {1, 1});
    op.SetAttr<std::vector<int>>("paddings", {0, 0});
    op.SetAttr<std::vector<int>>("dilations", {1, 1});
    op.SetAttr<int32_t>("groups", 1);
    op.SetAttr<int32_t>("first_ic", 3);
    op.SetAttr<int32_t>("flag_semi", 1);
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
  }
  {
    fbs::OpDesc op(block.AddOp<fbs::proto::OpDescT>());
    op.SetType("fetch");
    op.SetInput("X", {"y"});
    op.SetOutput("Out", {"fetch"});
    op.SetAttr<int32_t>("col", 0);
  }
}

// SaveModelNaive's sequence (model_parser.cc:470-535).
void WriteExample(const std::string& path, uint16_t meta_version) {
  fbs::ProgramDesc prog;
  Scope scope;
  BuildExample(&prog, &scope);
  model_parser::Buffer buffer;
  model_parser::BinaryFileWriter writer{path};
  writer.Write(&meta_version, sizeof(uint16_t));
  char version[16] = {0};
  std::strncpy(version, "ref-tool", 15);
  writer.Write(version, 16);
  prog.CopyDataToBuffer(&buffer);
  uint64_t topology_size = buffer.size();
  writer.Write(&topology_size, sizeof(uint64_t));
  writer.Write(buffer.data(), topology_size);
  std::set<std::string> names = {"conv1_w_nonzeros_output", "conv1_w_oc_nonzeros", "conv1_w_ic_diffs", "conv1_b", "conv2_w_nonzeros_output"};
  if (meta_version == 1) {
    fbs::CombinedParamsDesc params_prog;
    fbs::deprecated::SetCombinedParamsWithScope(scope, names, &params_prog);
    params_prog.CopyDataToBuffer(&buffer);
    writer.Write(buffer.data(), buffer.size());
  } else {
    fbs::ParamSerializer serializer{&writer};
    serializer.ForwardWrite(scope, names);
  }
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

const char* AttrKindName(OpAttrType t) {
  switch (t) {
    case OpAttrType::INT: return "INT";
    case OpAttrType::FLOAT: return "FLOAT";
    case OpAttrType::STRING: return "STRING";
    case OpAttrType::INTS: return "INTS";
    case OpAttrType::FLOATS: return "FLOATS";
    case OpAttrType::STRINGS: return "STRINGS";
    case OpAttrType::BOOLEAN: return "BOOLEAN";
    case OpAttrType::LONG: return "LONG";
    case OpAttrType::LONGS: return "LONGS";
    case OpAttrType::FLOAT64: return "FLOAT64";
    case OpAttrType::FLOAT64S: return "FLOAT64S";
    default: return "OTHER";
  }
}

void PrintStrings(const std::vector<std::string>& v) {
  for (auto& s : v) std::printf(" \"%s\"", s.c_str());
  std::printf("\n");
}

// LoadModelFbsFromFile's sequence (model_parser.cc:838-905).
int Dump(const std::string& path) {
  model_parser::BinaryFileReader reader(path, 0);
  uint16_t meta_version;
  reader.Read(&meta_version, sizeof(uint16_t));
  char opt_version[17] = {0};
  reader.Read(opt_version, 16);
  uint64_t topo_size;
  reader.Read(&topo_size, sizeof(uint64_t));
  model_parser::Buffer buf(topo_size);
  reader.Read(buf.data(), topo_size);
  fbs::ProgramDescView prog_view(std::move(buf));
  const fbs::ProgramDescView& prog = prog_view;  // the read accessors are the const ones
  Scope scope;
  if (meta_version == 1) {
    model_parser::Buffer pbuf(reader.length() - reader.current());
    reader.Read(pbuf.data(), reader.length() - reader.current());
    fbs::CombinedParamsDescView params(std::move(pbuf));
    fbs::deprecated::SetScopeWithCombinedParams(&scope, params);
  } else if (meta_version == 2) {
    fbs::ParamDeserializer deserializer(&reader);
    deserializer.ForwardRead(&scope);
  } else {
    std::printf("unsupported meta_version %d\n", meta_version);
    return 1;
  }
  std::printf("meta_version %d\n", meta_version);
  if (prog.HasVersion()) std::printf("version %lld\n", static_cast<long long>(prog.Version()));
  for (size_t b = 0; b < prog.BlocksSize(); ++b) {
    const auto* block = prog.GetBlock<fbs::BlockDescView>(b);
    std::printf("block %d parent %d forward %d\n", block->Idx(), block->ParentIdx(), block->ForwardBlockIdx());
    for (size_t i = 0; i < block->VarsSize(); ++i) {
      const auto* var = block->GetVar<fbs::VarDescView>(i);
      std::printf("var %s type %s persistable %d", var->Name().c_str(), VarTypeName(var->GetType()), var->Persistable() ? 1 : 0);
      if (var->GetType() == VarDataType::LOD_TENSOR) {
        std::printf(" dtype %s shape", VarTypeName(var->GetDataType()));
        for (int64_t d : var->GetShape()) std::printf(" %lld", static_cast<long long>(d));
      }
      std::printf("\n");
    }
    for (size_t i = 0; i < block->OpsSize(); ++i) {
      const auto* op = block->GetOp<fbs::OpDescView>(i);
      std::printf("op %s\n", op->Type().c_str());
      for (auto& arg : op->InputArgumentNames()) {
        std::printf(" in %s:", arg.c_str());
        PrintStrings(op->Input(arg));
      }
      for (auto& arg : op->OutputArgumentNames()) {
        std::printf(" out %s:", arg.c_str());
        PrintStrings(op->Output(arg));
      }
      for (auto& name : op->AttrNames()) {
        const auto type = op->GetAttrType(name);
        std::printf(" attr %s kind %s:", name.c_str(), AttrKindName(type));
        switch (type) {
          case OpAttrType::INT: std::printf(" %d\n", op->GetAttr<int32_t>(name)); break;
          case OpAttrType::FLOAT: std::printf(" %.9g\n", op->GetAttr<float>(name)); break;
          case OpAttrType::BOOLEAN: std::printf(" %d\n", op->GetAttr<bool>(name) ? 1 : 0); break;
          case OpAttrType::LONG: std::printf(" %lld\n", static_cast<long long>(op->GetAttr<int64_t>(name))); break;
          case OpAttrType::FLOAT64: std::printf(" %.17g\n", op->GetAttr<double>(name)); break;
          case OpAttrType::STRING: std::printf(" \"%s\"\n", op->GetAttr<std::string>(name).c_str()); break;
          case OpAttrType::INTS: {
            auto v = op->GetAttr<std::vector<int>>(name);
            for (size_t k = 0; k < v.size(); ++k) std::printf(" %d", v[k]);
            std::printf("\n");
            break;
          }
          case OpAttrType::FLOATS: {
            auto v = op->GetAttr<std::vector<float>>(name);
            for (size_t k = 0; k < v.size(); ++k) std::printf(" %.9g", v[k]);
            std::printf("\n");
            break;
          }
          case OpAttrType::LONGS: {
            auto v = op->GetAttr<std::vector<int64_t>>(name);
            for (size_t k = 0; k < v.size(); ++k) std::printf(" %lld", static_cast<long long>(v[k]));
            std::printf("\n");
            break;
          }
          case OpAttrType::FLOAT64S: {
            auto v = op->GetAttr<std::vector<double>>(name);
            for (size_t k = 0; k < v.size(); ++k) std::printf(" %.17g", v[k]);
            std::printf("\n");
            break;
          }
          case OpAttrType::STRINGS: {
            auto v = op->GetAttr<std::vector<std::string>>(name);
            std::vector<std::string> s;
            for (size_t k = 0; k < v.size(); ++k) s.push_back(v[k]);
            PrintStrings(s);
            break;
          }
          default: std::printf(" ?\n");
        }
      }
    }
  }
  std::vector<std::string> names = scope.LocalVarNames();
  std::sort(names.begin(), names.end());
  for (auto& name : names) {
    const auto& t = scope.FindVar(name)->Get<Tensor>();
    std::printf("tensor %s precision %d dims", name.c_str(), static_cast<int>(t.precision()));
    for (int64_t d : t.dims().Vectorize()) std::printf(" %lld", static_cast<long long>(d));
    std::printf(" bytes %zu fnv %016llx\n", t.memory_size(), static_cast<unsigned long long>(Fnv(t.raw_data(), t.memory_size())));
  }
  return 0;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc >= 3 && std::string(argv[1]) == "dump") return Dump(argv[2]);
  if (argc >= 3 && std::string(argv[1]) == "write-example") {
    WriteExample(argv[2], argc >= 4 ? static_cast<uint16_t>(std::atoi(argv[3])) : 2);
    return 0;
  }
  std::fprintf(stderr, "usage: ref_model_file dump FILE | write-example FILE [META_VERSION]\n");
  return 2;
}
