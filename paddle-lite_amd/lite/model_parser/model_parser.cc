#include "lite/model_parser/model_parser.h"

#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <typeinfo>

#include "lite/model_parser/flatbuffers/wire.h"

namespace paddle {
namespace lite {

namespace {

using fbs::wire::Builder;
using fbs::wire::FormatError;
using fbs::wire::Table;
using fbs::wire::View;

// Attribute kinds (framework.fbs AttrType).
enum AttrKind : int {
  kAttrInt = 0, kAttrFloat = 1, kAttrString = 2, kAttrInts = 3, kAttrFloats = 4, kAttrStrings = 5, kAttrBool = 6, kAttrBools = 7,
  kAttrBlock = 8, kAttrLong = 9, kAttrBlocks = 10, kAttrLongs = 11, kAttrFloat64s = 12, kAttrVar = 13, kAttrVars = 14, kAttrFloat64 = 15,
};

// Field slots, in schema order.
namespace slot {
enum { kProgBlocks = 0, kProgVersion = 1, kProgOpVersionMap = 2 };
enum { kBlockIdx = 0, kBlockParent = 1, kBlockVars = 2, kBlockOps = 3, kBlockForward = 4 };
enum { kVarName = 0, kVarType = 1, kVarPersistable = 2, kVarNeedCheckFeed = 3 };
enum { kVarTypeType = 0, kVarTypeLodTensor = 2 };
enum { kLodTensorTensor = 0, kLodTensorLevel = 1 };
enum { kTensorDataType = 0, kTensorDims = 1 };
enum { kOpType = 0, kOpInputs = 1, kOpOutputs = 2, kOpAttrs = 3, kOpIsTarget = 4 };
enum { kArgParameter = 0, kArgArguments = 1 };
enum {
  kAttrName = 0, kAttrType = 1, kAttrI = 2, kAttrF = 3, kAttrS = 4, kAttrIntsV = 5, kAttrFloatsV = 6, kAttrStringsV = 7, kAttrB = 8,
  kAttrBoolsV = 9, kAttrBlockIdx = 10, kAttrL = 11, kAttrBlocksIdx = 12, kAttrLongsV = 13, kAttrF64 = 14, kAttrF64sV = 15,
};
enum { kParamVersion = 0, kParamName = 1, kParamVariableType = 2, kParamVariable = 3 };
enum { kParamLodLevel = 0, kParamLod = 1, kParamDim = 2, kParamDataType = 3, kParamData = 4 };
enum { kCombinedParams = 0 };
}  // namespace slot

VarDataType ToVarType(PrecisionType p) {
  // lite/core/model/base/traits.h:81-102
  switch (p) {
    case PrecisionType::kBool: return VarDataType::BOOL;
    case PrecisionType::kInt8: return VarDataType::INT8;
    case PrecisionType::kUInt8: return VarDataType::UINT8;
    case PrecisionType::kInt16: return VarDataType::INT16;
    case PrecisionType::kInt32: return VarDataType::INT32;
    case PrecisionType::kInt64: return VarDataType::INT64;
    case PrecisionType::kFP16: return VarDataType::FP16;
    case PrecisionType::kFloat: return VarDataType::FP32;
    default: LOG(FATAL) << "Illegal flatbuffer VarType." << static_cast<int>(p);
  }
  return VarDataType::FP32;
}

PrecisionType ToPrecision(int var_type) {
  switch (static_cast<VarDataType>(var_type)) {
    case VarDataType::BOOL: return PrecisionType::kBool;
    case VarDataType::INT8: return PrecisionType::kInt8;
    case VarDataType::UINT8: return PrecisionType::kUInt8;
    case VarDataType::INT16: return PrecisionType::kInt16;
    case VarDataType::INT32: return PrecisionType::kInt32;
    case VarDataType::INT64: return PrecisionType::kInt64;
    case VarDataType::FP16: return PrecisionType::kFP16;
    case VarDataType::FP32: return PrecisionType::kFloat;
    default: throw FormatError("Illegal flatbuffer VarType: " + std::to_string(var_type));
  }
}

size_t ElementBytes(PrecisionType p) {
  switch (p) {
    case PrecisionType::kBool:
    case PrecisionType::kInt8:
    case PrecisionType::kUInt8: return 1;
    case PrecisionType::kInt16:
    case PrecisionType::kFP16: return 2;
    case PrecisionType::kInt64: return 8;
    default: return 4;
  }
}

// ------------------------------------------------------------- topology
Builder::Ref WriteAttr(Builder* b, const std::string& name, const std::any& value) {
  const std::type_info& t = value.type();
  const Builder::Ref name_ref = b->CreateString(name);
  Builder::Ref ref = 0;
  int kind = -1;
  if (t == typeid(std::string)) {
    kind = kAttrString;
    ref = b->CreateString(std::any_cast<const std::string&>(value));
  } else if (t == typeid(std::vector<int>)) {
    kind = kAttrInts;
    ref = b->CreateVector(std::any_cast<const std::vector<int>&>(value));
  } else if (t == typeid(std::vector<float>)) {
    kind = kAttrFloats;
    ref = b->CreateVector(std::any_cast<const std::vector<float>&>(value));
  } else if (t == typeid(std::vector<int64_t>)) {
    kind = kAttrLongs;
    ref = b->CreateVector(std::any_cast<const std::vector<int64_t>&>(value));
  } else if (t == typeid(std::vector<double>)) {
    kind = kAttrFloat64s;
    ref = b->CreateVector(std::any_cast<const std::vector<double>&>(value));
  } else if (t == typeid(std::vector<bool>)) {
    kind = kAttrBools;
    ref = b->CreateBoolVector(std::any_cast<const std::vector<bool>&>(value));
  } else if (t == typeid(std::vector<std::string>)) {
    kind = kAttrStrings;
    std::vector<Builder::Ref> refs;
    for (const std::string& s : std::any_cast<const std::vector<std::string>&>(value)) refs.push_back(b->CreateString(s));
    ref = b->CreateRefVector(refs);
  }
  b->StartTable();
  b->AddRef(slot::kAttrName, name_ref);
  if (kind >= 0) {
    const int vslot = kind == kAttrString ? slot::kAttrS
                      : kind == kAttrInts ? slot::kAttrIntsV
                      : kind == kAttrFloats ? slot::kAttrFloatsV
                      : kind == kAttrLongs ? slot::kAttrLongsV
                      : kind == kAttrFloat64s ? slot::kAttrF64sV
                      : kind == kAttrBools ? slot::kAttrBoolsV
                                           : slot::kAttrStringsV;
    b->AddRef(vslot, ref);
  } else if (t == typeid(int)) {
    kind = kAttrInt;
    b->AddScalar<int32_t>(slot::kAttrI, std::any_cast<int>(value), 0);
  } else if (t == typeid(float)) {
    kind = kAttrFloat;
    b->AddScalar<float>(slot::kAttrF, std::any_cast<float>(value), 0.0f);
  } else if (t == typeid(bool)) {
    kind = kAttrBool;
    b->AddScalar<uint8_t>(slot::kAttrB, std::any_cast<bool>(value) ? 1 : 0, 0);
  } else if (t == typeid(int64_t)) {
    kind = kAttrLong;
    b->AddScalar<int64_t>(slot::kAttrL, std::any_cast<int64_t>(value), 0);
  } else if (t == typeid(double)) {
    kind = kAttrFloat64;
    b->AddScalar<double>(slot::kAttrF64, std::any_cast<double>(value), 0.0);
  } else if (t == typeid(int16_t)) {
    kind = kAttrBlock;
    b->AddScalar<int32_t>(slot::kAttrBlockIdx, std::any_cast<int16_t>(value), 0);
  } else {
    LOG(FATAL) << "attribute " << name << " has a type the model file cannot hold";
  }
  b->AddScalar<int32_t>(slot::kAttrType, kind, 0);
  return b->EndTable();
}

Builder::Ref WriteArgs(Builder* b, const std::map<std::string, std::vector<std::string>>& args) {
  std::vector<Builder::Ref> tables;
  for (const auto& kv : args) {  // key order, as lookups by key need
    std::vector<Builder::Ref> names;
    for (const std::string& n : kv.second) names.push_back(b->CreateString(n));
    const Builder::Ref arguments = b->CreateRefVector(names);
    const Builder::Ref parameter = b->CreateString(kv.first);
    b->StartTable();
    b->AddRef(slot::kArgParameter, parameter);
    b->AddRef(slot::kArgArguments, arguments);
    tables.push_back(b->EndTable());
  }
  return b->CreateRefVector(tables);
}

Builder::Ref WriteOp(Builder* b, const OpInfo& op) {
  std::vector<Builder::Ref> attrs;
  for (const auto& kv : op.attrs()) attrs.push_back(WriteAttr(b, kv.first, kv.second));
  const Builder::Ref attrs_ref = b->CreateRefVector(attrs);
  const Builder::Ref outputs = WriteArgs(b, op.outputs());
  const Builder::Ref inputs = WriteArgs(b, op.inputs());
  const Builder::Ref type = b->CreateString(op.Type());
  b->StartTable();
  b->AddRef(slot::kOpType, type);
  b->AddRef(slot::kOpInputs, inputs);
  b->AddRef(slot::kOpOutputs, outputs);
  b->AddRef(slot::kOpAttrs, attrs_ref);
  return b->EndTable();
}

Builder::Ref WriteVar(Builder* b, const cpp::VarDesc& var) {
  const Builder::Ref dims = b->CreateVector(var.GetShape());
  b->StartTable();
  b->AddScalar<int32_t>(slot::kTensorDataType, static_cast<int32_t>(var.GetDataType()), 0);
  b->AddRef(slot::kTensorDims, dims);
  const Builder::Ref tensor = b->EndTable();
  b->StartTable();
  b->AddRef(slot::kLodTensorTensor, tensor);
  b->AddScalar<int32_t>(slot::kLodTensorLevel, var.LodLevel(), 0);
  const Builder::Ref lod_tensor = b->EndTable();
  b->StartTable();
  b->AddScalar<int32_t>(slot::kVarTypeType, static_cast<int32_t>(var.GetType()), 0);
  b->AddRef(slot::kVarTypeLodTensor, lod_tensor);
  const Builder::Ref type = b->EndTable();
  const Builder::Ref name = b->CreateString(var.Name());
  b->StartTable();
  b->AddRef(slot::kVarName, name);
  b->AddRef(slot::kVarType, type);
  b->AddScalar<uint8_t>(slot::kVarPersistable, var.Persistable() ? 1 : 0, 0);
  b->AddScalar<uint8_t>(slot::kVarNeedCheckFeed, var.NeedCheckFeed() ? 1 : 0, 0);
  return b->EndTable();
}

std::any ReadAttrValue(const Table& a, const std::string& name) {
  const int kind = a.Scalar<int32_t>(slot::kAttrType, 0);
  switch (kind) {
    case kAttrInt: return std::any(static_cast<int>(a.Scalar<int32_t>(slot::kAttrI, 0)));
    case kAttrFloat: return std::any(a.Scalar<float>(slot::kAttrF, 0.0f));
    case kAttrString: return std::any(a.String(slot::kAttrS));
    case kAttrInts: return std::any(a.Vector<int32_t>(slot::kAttrIntsV).ToVector());
    case kAttrFloats: return std::any(a.Vector<float>(slot::kAttrFloatsV).ToVector());
    case kAttrStrings: {
      std::vector<std::string> v;
      for (size_t i = 0; i < a.VectorSize(slot::kAttrStringsV); ++i) v.push_back(a.StringAt(slot::kAttrStringsV, i));
      return std::any(v);
    }
    case kAttrBool: return std::any(a.Scalar<uint8_t>(slot::kAttrB, 0) != 0);
    case kAttrBools: {
      const auto raw = a.Vector<uint8_t>(slot::kAttrBoolsV);
      std::vector<bool> v(raw.size());
      for (size_t i = 0; i < raw.size(); ++i) v[i] = raw[i] != 0;
      return std::any(v);
    }
    case kAttrBlock: return std::any(static_cast<int16_t>(a.Scalar<int32_t>(slot::kAttrBlockIdx, 0)));
    case kAttrLong: return std::any(a.Scalar<int64_t>(slot::kAttrL, 0));
    case kAttrLongs: return std::any(a.Vector<int64_t>(slot::kAttrLongsV).ToVector());
    case kAttrFloat64: return std::any(a.Scalar<double>(slot::kAttrF64, 0.0));
    case kAttrFloat64s: return std::any(a.Vector<double>(slot::kAttrF64sV).ToVector());
    default: throw FormatError("attribute " + name + " has unsupported type " + std::to_string(kind));
  }
}

void ReadArgs(const Table& op, int slot_id, bool inputs, OpInfo* out) {
  for (size_t i = 0; i < op.VectorSize(slot_id); ++i) {
    const Table arg = op.TableAt(slot_id, i);
    std::vector<std::string> names;
    for (size_t k = 0; k < arg.VectorSize(slot::kArgArguments); ++k) names.push_back(arg.StringAt(slot::kArgArguments, k));
    if (inputs) {
      out->SetInput(arg.String(slot::kArgParameter), names);
    } else {
      out->SetOutput(arg.String(slot::kArgParameter), names);
    }
  }
}

// ----------------------------------------------------------- parameters
void FillTensor(const Table& param, Scope* scope) {
  // lite/model_parser/flatbuffers/io.cc:60-69 and param_desc.h:33-80
  const std::string name = param.String(slot::kParamName);
  if (!param.Has(slot::kParamName)) throw FormatError("parameter without a name");
  if (param.Scalar<uint8_t>(slot::kParamVariableType, 0) != 1) throw FormatError("parameter " + name + " is not a LoDTensorDesc");
  const Table t = param.Sub(slot::kParamVariable);
  if (!t.valid() || !t.Has(slot::kParamData)) throw FormatError("parameter " + name + " has no data");
  const auto dim = t.Vector<int64_t>(slot::kParamDim);
  const auto data = t.Vector<uint8_t>(slot::kParamData);
  // the dimensions must describe exactly the bytes that are there: kernels size
  // their reads from the dimensions
  const PrecisionType precision = ToPrecision(t.Scalar<int32_t>(slot::kParamDataType, 0));
  const std::vector<int64_t> dims = dim.ToVector();
  uint64_t numel = 1;
  for (int64_t d : dims) {
    if (d < 0 || (d > 0 && numel > (uint64_t{1} << 40) / static_cast<uint64_t>(d))) throw FormatError("parameter " + name + " has illegal dimensions");
    numel *= static_cast<uint64_t>(d);
  }
  if (numel * ElementBytes(precision) != data.size())
    throw FormatError("parameter " + name + ": dimensions describe " + std::to_string(numel * ElementBytes(precision)) + " bytes, the record holds " + std::to_string(data.size()));
  Tensor* tensor = scope->Var(name)->GetMutable<Tensor>();
  tensor->Resize(dims);
  tensor->set_precision(precision);
  void* dst = tensor->mutable_data(TargetType::kHost, data.size());
  if (data.size()) std::memcpy(dst, data.bytes(), data.size());
  tensor->set_persistable(true);
}

Builder::Ref WriteParam(Builder* b, const std::string& name, const Tensor& tensor) {
  const Builder::Ref data = b->CreateVector(static_cast<const uint8_t*>(tensor.raw_data()), tensor.memory_size());
  const Builder::Ref dim = b->CreateVector(tensor.dims().Vectorize());
  b->StartTable();
  b->AddRef(slot::kParamDim, dim);
  b->AddScalar<int32_t>(slot::kParamDataType, static_cast<int32_t>(ToVarType(tensor.precision())), 0);
  b->AddRef(slot::kParamData, data);
  const Builder::Ref lod_tensor = b->EndTable();
  const Builder::Ref name_ref = b->CreateString(name);
  b->StartTable();
  b->AddRef(slot::kParamName, name_ref);
  b->AddScalar<uint8_t>(slot::kParamVariableType, 1, 0);
  b->AddRef(slot::kParamVariable, lod_tensor);
  return b->EndTable();
}

std::set<std::string> ParamNames(const cpp::ProgramDesc& prog) {
  std::set<std::string> names;  // each name once, in name order
  if (prog.BlocksSize() == 0) return names;
  for (const cpp::VarDesc& var : prog.GetBlock(0)->vars()) {
    if (cpp::IsParamVarDesc(var)) names.insert(var.Name());
  }
  return names;
}

template <typename T>
void Append(std::string* out, T v) {
  out->append(reinterpret_cast<const char*>(&v), sizeof(T));
}

class Cursor {
 public:
  explicit Cursor(const std::string& s) : s_(s) {}
  template <typename T>
  T Read() {
    T v;
    std::memcpy(&v, Bytes(sizeof(T)), sizeof(T));
    return v;
  }
  const uint8_t* Bytes(size_t n) {
    if (n > s_.size() - pos_) throw FormatError("model file ends early");
    const uint8_t* p = reinterpret_cast<const uint8_t*>(s_.data()) + pos_;
    pos_ += n;
    return p;
  }
  size_t left() const { return s_.size() - pos_; }

 private:
  const std::string& s_;
  size_t pos_ = 0;
};

void LoadFromMemory(const std::string& model_buffer, Scope* scope, cpp::ProgramDesc* cpp_prog) {
  Cursor in(model_buffer);
  const uint16_t meta_version = in.Read<uint16_t>();
  if (meta_version == 0) {
    throw FormatError("Paddle-Lite v2.7 has upgraded the naive-buffer model format. Please use the OPT to generate a new model.");
  }
  if (meta_version != 1 && meta_version != 2) {
    throw FormatError("The model format cannot be recognized. Please make sure you use the correct interface and model file.");
  }
  const uint8_t* opt_version = in.Bytes(16);
  const std::string opt_version_str(reinterpret_cast<const char*>(opt_version), strnlen(reinterpret_cast<const char*>(opt_version), 16));
  if (opt_version_str != version()) {
    LOG(WARNING) << "the version of opt that transformed this model (" << opt_version_str << ") is not this library's (" << version() << ")";
  }
  const uint64_t topo_size = in.Read<uint64_t>();
  if (topo_size > in.left()) throw FormatError("model file ends inside the topology");
  fbs::ParseProgramDesc(in.Bytes(static_cast<size_t>(topo_size)), static_cast<size_t>(topo_size), cpp_prog);
  if (meta_version == 1) {
    const size_t n = in.left();
    const View view(in.Bytes(n), n);
    const Table combined = Table::Root(view);
    for (size_t i = 0; i < combined.VectorSize(slot::kCombinedParams); ++i) FillTensor(combined.TableAt(slot::kCombinedParams, i), scope);
    return;
  }
  // meta version 2: lite/model_parser/flatbuffers/io.cc:112-148
  const uint16_t params_version = in.Read<uint16_t>();
  if (params_version != 0) throw FormatError("File format error: The version of params must be zero.");
  const uint16_t meta_size = in.Read<uint16_t>();
  in.Bytes(meta_size);
  const uint16_t header_size = in.Read<uint16_t>();
  if (header_size < 6) throw FormatError("parameter header too short");
  const uint8_t* header = in.Bytes(header_size);
  uint16_t params_size;
  std::memcpy(&params_size, header, 2);
  for (uint16_t i = 0; i < params_size; ++i) {
    const uint32_t total_size = in.Read<uint32_t>();
    const uint32_t offset = in.Read<uint32_t>();
    if (offset < 4 || offset > total_size) throw FormatError("bad parameter record");
    in.Bytes(offset - 4);
    const uint32_t param_bytes = total_size - offset;
    fbs::ParseParamDesc(in.Bytes(param_bytes), param_bytes, scope);
  }
}

}  // namespace

std::string version() { return "pl-hip"; }

namespace fbs {

std::vector<uint8_t> SerializeProgramDesc(const cpp::ProgramDesc& prog) {
  Builder b;
  std::vector<Builder::Ref> blocks;
  for (size_t bi = 0; bi < prog.BlocksSize(); ++bi) {
    const cpp::BlockDesc& block = *prog.GetBlock(bi);
    std::vector<Builder::Ref> ops, vars;
    for (const OpInfo& op : block.ops()) ops.push_back(WriteOp(&b, op));
    for (const cpp::VarDesc& var : block.vars()) vars.push_back(WriteVar(&b, var));
    const Builder::Ref ops_ref = b.CreateRefVector(ops);
    const Builder::Ref vars_ref = b.CreateRefVector(vars);
    b.StartTable();
    b.AddScalar<int32_t>(slot::kBlockIdx, block.Idx(), 0);
    b.AddScalar<int32_t>(slot::kBlockParent, block.ParentIdx(), 0);
    b.AddRef(slot::kBlockVars, vars_ref);
    b.AddRef(slot::kBlockOps, ops_ref);
    b.AddScalar<int32_t>(slot::kBlockForward, block.ForwardBlockIdx(), -1);
    blocks.push_back(b.EndTable());
  }
  Builder::Ref op_versions = 0;
  if (!prog.OpVersionMap().empty()) {
    std::vector<Builder::Ref> pairs;
    for (const auto& kv : prog.OpVersionMap()) {
      b.StartTable();
      b.AddScalar<int32_t>(0, kv.second, 0);
      const Builder::Ref v = b.EndTable();
      const Builder::Ref name = b.CreateString(kv.first);
      b.StartTable();
      b.AddRef(0, name);
      b.AddRef(1, v);
      pairs.push_back(b.EndTable());
    }
    const Builder::Ref pair_vec = b.CreateRefVector(pairs);
    b.StartTable();
    b.AddRef(0, pair_vec);
    op_versions = b.EndTable();
  }
  Builder::Ref version_ref = 0;
  if (prog.HasVersion()) {
    b.StartTable();
    b.AddScalar<int64_t>(0, prog.Version(), 0);
    version_ref = b.EndTable();
  }
  const Builder::Ref blocks_ref = b.CreateRefVector(blocks);
  b.StartTable();
  b.AddRef(slot::kProgBlocks, blocks_ref);
  b.AddRef(slot::kProgVersion, version_ref);
  b.AddRef(slot::kProgOpVersionMap, op_versions);
  b.Finish(b.EndTable());
  return b.Release();
}

void ParseProgramDesc(const uint8_t* data, size_t size, cpp::ProgramDesc* prog) {
  const View view(data, size);
  const Table root = Table::Root(view);
  prog->ClearBlocks();
  for (size_t bi = 0; bi < root.VectorSize(slot::kProgBlocks); ++bi) {
    const Table blk = root.TableAt(slot::kProgBlocks, bi);
    cpp::BlockDesc* out = prog->AddBlock();
    out->SetIdx(blk.Scalar<int32_t>(slot::kBlockIdx, 0));
    out->SetParentIdx(blk.Scalar<int32_t>(slot::kBlockParent, 0));
    out->SetForwardBlockIdx(blk.Scalar<int32_t>(slot::kBlockForward, -1));
    for (size_t i = 0; i < blk.VectorSize(slot::kBlockVars); ++i) {
      const Table v = blk.TableAt(slot::kBlockVars, i);
      cpp::VarDesc* var = out->AddVar();
      var->SetName(v.String(slot::kVarName));
      var->SetPersistable(v.Scalar<uint8_t>(slot::kVarPersistable, 0) != 0);
      var->SetNeedCheckFeed(v.Scalar<uint8_t>(slot::kVarNeedCheckFeed, 0) != 0);
      const Table type = v.Sub(slot::kVarType);
      if (!type.valid()) throw FormatError("variable " + var->Name() + " has no type");
      var->SetType(static_cast<VarDataType>(type.Scalar<int32_t>(slot::kVarTypeType, 0)));
      const Table lod_tensor = type.Sub(slot::kVarTypeLodTensor);
      if (lod_tensor.valid()) {
        var->SetLodLevel(lod_tensor.Scalar<int32_t>(slot::kLodTensorLevel, 0));
        const Table tensor = lod_tensor.Sub(slot::kLodTensorTensor);
        if (tensor.valid()) {
          var->SetDataType(static_cast<VarDataType>(tensor.Scalar<int32_t>(slot::kTensorDataType, 0)));
          var->SetShape(tensor.Vector<int64_t>(slot::kTensorDims).ToVector());
        }
      }
    }
    for (size_t i = 0; i < blk.VectorSize(slot::kBlockOps); ++i) {
      const Table o = blk.TableAt(slot::kBlockOps, i);
      OpInfo* op = out->AddOp();
      op->SetType(o.String(slot::kOpType));
      ReadArgs(o, slot::kOpInputs, true, op);
      ReadArgs(o, slot::kOpOutputs, false, op);
      for (size_t k = 0; k < o.VectorSize(slot::kOpAttrs); ++k) {
        const Table a = o.TableAt(slot::kOpAttrs, k);
        const std::string name = a.String(slot::kAttrName);
        const std::any value = ReadAttrValue(a, name);
        op->SetAttr<std::any>(name, value);
      }
    }
  }
  const Table ver = root.Sub(slot::kProgVersion);
  if (ver.valid()) prog->SetVersion(ver.Scalar<int64_t>(0, 0));
  const Table map = root.Sub(slot::kProgOpVersionMap);
  if (map.valid()) {
    std::vector<std::pair<std::string, int32_t>> pairs;
    for (size_t i = 0; i < map.VectorSize(0); ++i) {
      const Table pair = map.TableAt(0, i);
      const Table v = pair.Sub(1);
      pairs.emplace_back(pair.String(0), v.valid() ? v.Scalar<int32_t>(0, 0) : 0);
    }
    prog->SetOpVersionMap(pairs);
  }
}

std::vector<uint8_t> SerializeParamDesc(const std::string& name, const Tensor& tensor) {
  Builder b;
  b.Finish(WriteParam(&b, name, tensor));
  return b.Release();
}

void ParseParamDesc(const uint8_t* data, size_t size, Scope* scope) {
  const View view(data, size);
  FillTensor(Table::Root(view), scope);
}

}  // namespace fbs

bool TryLoadModelNaiveFromMemory(const std::string& model_buffer, Scope* scope, cpp::ProgramDesc* cpp_prog, std::string* error) {
  CHECK(cpp_prog);
  CHECK(scope);
  try {
    LoadFromMemory(model_buffer, scope, cpp_prog);
  } catch (const fbs::wire::FormatError& e) {
    if (error) *error = e.what();
    return false;
  }
  return true;
}

void LoadModelNaiveFromMemory(const std::string& model_buffer, Scope* scope, cpp::ProgramDesc* cpp_prog) {
  std::string error;
  if (!TryLoadModelNaiveFromMemory(model_buffer, scope, cpp_prog, &error)) LOG(FATAL) << error;
}

void LoadModelNaiveFromFile(const std::string& filename, Scope* scope, cpp::ProgramDesc* cpp_prog) {
  std::ifstream f(filename, std::ios::binary);
  CHECK(f.good()) << "Cannot open " << filename;
  const std::string bytes((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
  LoadModelNaiveFromMemory(bytes, scope, cpp_prog);
}

std::string SerializeModelNaive(const Scope& exec_scope, const cpp::ProgramDesc& cpp_prog, uint16_t meta_version) {
  CHECK(meta_version == 1 || meta_version == 2) << "Error: Unsupported opt meta_version, meta_version should be set as 1 or 2.";
  std::string out;
  Append<uint16_t>(&out, meta_version);
  char ver[16] = {0};
  std::strncpy(ver, version().c_str(), 15);
  out.append(ver, 16);
  const std::vector<uint8_t> topo = fbs::SerializeProgramDesc(cpp_prog);
  Append<uint64_t>(&out, topo.size());
  out.append(reinterpret_cast<const char*>(topo.data()), topo.size());
  const std::set<std::string> names = ParamNames(cpp_prog);
  auto tensor_of = [&](const std::string& name) -> const Tensor& {
    Variable* var = exec_scope.FindVar(name);
    CHECK(var) << "parameter " << name << " is not in the scope";
    return var->Get<Tensor>();
  };
  if (meta_version == 1) {
    Builder b;
    std::vector<Builder::Ref> params;
    for (const std::string& name : names) params.push_back(WriteParam(&b, name, tensor_of(name)));
    const Builder::Ref vec = b.CreateRefVector(params);
    b.StartTable();
    b.AddRef(slot::kCombinedParams, vec);
    b.Finish(b.EndTable());
    out.append(reinterpret_cast<const char*>(b.data()), b.size());
    return out;
  }
  // lite/model_parser/flatbuffers/io.cc:71-110
  Append<uint16_t>(&out, 0);  // version of the parameter section
  Append<uint16_t>(&out, 0);  // size of its (reserved) meta information
  uint32_t max_tensor_size = 0;
  for (const std::string& name : names) {
    const size_t bytes = tensor_of(name).memory_size();
    CHECK(bytes < 0xffffffffull) << "The size of param is out of range.";
    if (bytes > max_tensor_size) max_tensor_size = static_cast<uint32_t>(bytes);
  }
  Append<uint16_t>(&out, 6);
  Append<uint16_t>(&out, static_cast<uint16_t>(names.size()));
  Append<uint32_t>(&out, max_tensor_size);
  for (const std::string& name : names) {
    const std::vector<uint8_t> param = fbs::SerializeParamDesc(name, tensor_of(name));
    Append<uint32_t>(&out, static_cast<uint32_t>(param.size() + 4));
    Append<uint32_t>(&out, 4);
    out.append(reinterpret_cast<const char*>(param.data()), param.size());
  }
  return out;
}

int RebakeSparseConvDiffs(cpp::ProgramDesc* prog, Scope* scope, int64_t new_h, int64_t new_w) {
  CHECK(prog && scope);
  CHECK(new_h > 0 && new_w > 0) << "the new input size must be positive";
  if (prog->BlocksSize() == 0) return 0;
  cpp::BlockDesc* block = prog->GetBlock(0);
  auto find_var = [&](const std::string& name) -> cpp::VarDesc* {
    for (cpp::VarDesc& v : block->vars())
      if (v.Name() == name) return &v;
    return nullptr;
  };
  // sizes first: several ops may read one variable, whose shape changes below
  std::vector<std::pair<OpInfo*, int64_t>> todo;
  for (OpInfo& op : block->ops()) {
    if (op.Type() != "sparse_conv2d") continue;
    const cpp::VarDesc* x = find_var(op.Input("Input").front());
    if (!x || x->GetShape().size() != 4 || x->GetShape()[2] <= 0 || x->GetShape()[3] <= 0) continue;
    todo.emplace_back(&op, x->GetShape()[2] * x->GetShape()[3]);
  }
  const int64_t new_size = new_h * new_w;
  std::set<std::string> done;  // a Diffs tensor shared by two ops is rewritten once
  for (auto& item : todo) {
    const OpInfo& op = *item.first;
    const int64_t old_size = item.second;
    const std::string diffs_name = op.Input("Diffs").front();
    if (!done.insert(diffs_name).second) continue;
    Tensor* diffs = scope->FindMutableTensor(diffs_name);
    CHECK(diffs && diffs->precision() == PrecisionType::kInt32) << "sparse_conv2d without an int32 Diffs tensor";
    int32_t* d = diffs->mutable_data<int32_t>(TargetType::kHost);
    for (int64_t i = 0; i < diffs->numel(); ++i) {
      CHECK(d[i] % old_size == 0) << "Diffs entry " << i << " is not a multiple of the recorded input size " << old_size;
      const int64_t v = static_cast<int64_t>(d[i]) / old_size * new_size;
      CHECK(v >= INT32_MIN && v <= INT32_MAX) << "Diffs entry " << i << " does not fit 32 bits at the new input size";
      d[i] = static_cast<int32_t>(v);
    }
  }
  auto reshape = [&](cpp::VarDesc* v) {
    if (!v || v->GetShape().size() != 4) return;
    std::vector<int64_t> s = v->GetShape();
    s[2] = new_h;
    s[3] = new_w;
    v->SetShape(s);
  };
  for (auto& item : todo) {
    reshape(find_var(item.first->Input("Input").front()));
    reshape(find_var(item.first->Output("Output").front()));
  }
  return static_cast<int>(todo.size());
}

void SaveModelNaive(const std::string& model_file, const Scope& exec_scope, const cpp::ProgramDesc& cpp_prog) {
  const uint16_t meta_version = std::getenv("PADDLE_LITE_MODEL_VERSION1") != nullptr ? 1 : 2;
  const std::string bytes = SerializeModelNaive(exec_scope, cpp_prog, meta_version);
  const std::string path = model_file + ".nb";
  std::ofstream f(path, std::ios::binary | std::ios::trunc);
  CHECK(f.good()) << "Cannot write " << path;
  f.write(bytes.data(), static_cast<std::streamsize>(bytes.size()));
  CHECK(f.good()) << "Cannot write " << path;
}

}  // namespace lite
}  // namespace paddle
