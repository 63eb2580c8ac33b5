// Variable, block and program descriptions: what a model file's topology
// part holds (reference: lite/core/model/general/{var_desc,block_desc,
// program_desc}.h; the enum values are those of
// lite/model_parser/flatbuffers/framework.fbs).
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "lite/core/op_desc.h"

namespace paddle {
namespace lite {

enum class VarDataType : int {
  BOOL = 0, INT16 = 1, INT32 = 2, INT64 = 3, FP16 = 4, FP32 = 5, FP64 = 6, LOD_TENSOR = 7, SELECTED_ROWS = 8, FEED_MINIBATCH = 9,
  FETCH_LIST = 10, STEP_SCOPES = 11, LOD_RANK_TABLE = 12, LOD_TENSOR_ARRAY = 13, PLACE_LIST = 14, READER = 15, RAW = 17, TUPLE = 18,
  SIZE_T = 19, UINT8 = 20, INT8 = 21,
};

namespace cpp {

class VarDesc {
 public:
  VarDesc() = default;
  explicit VarDesc(const std::string& name) : name_(name) {}
  const std::string& Name() const { return name_; }
  void SetName(const std::string& n) { name_ = n; }
  VarDataType GetType() const { return type_; }
  void SetType(VarDataType t) { type_ = t; }
  bool Persistable() const { return persistable_; }
  void SetPersistable(bool p) { persistable_ = p; }
  // element type and shape of a LOD_TENSOR variable
  VarDataType GetDataType() const { return data_type_; }
  void SetDataType(VarDataType t) { data_type_ = t; }
  const std::vector<int64_t>& GetShape() const { return shape_; }
  void SetShape(const std::vector<int64_t>& s) { shape_ = s; }
  int32_t LodLevel() const { return lod_level_; }
  void SetLodLevel(int32_t l) { lod_level_ = l; }
  bool NeedCheckFeed() const { return need_check_feed_; }
  void SetNeedCheckFeed(bool v) { need_check_feed_ = v; }

 private:
  std::string name_;
  VarDataType type_ = VarDataType::LOD_TENSOR;
  bool persistable_ = false, need_check_feed_ = false;
  VarDataType data_type_ = VarDataType::FP32;
  std::vector<int64_t> shape_;
  int32_t lod_level_ = 0;
};

// A weight: a persistable tensor variable (lite/core/model/base/var_desc.h:62-64).
inline bool IsParamVarDesc(const VarDesc& var) { return var.GetType() == VarDataType::LOD_TENSOR && var.Persistable(); }

class BlockDesc {
 public:
  int32_t Idx() const { return idx_; }
  void SetIdx(int32_t i) { idx_ = i; }
  int32_t ParentIdx() const { return parent_idx_; }
  void SetParentIdx(int32_t i) { parent_idx_ = i; }
  int32_t ForwardBlockIdx() const { return forward_block_idx_; }
  void SetForwardBlockIdx(int32_t i) { forward_block_idx_ = i; }
  size_t VarsSize() const { return vars_.size(); }
  size_t OpsSize() const { return ops_.size(); }
  const VarDesc& GetVar(size_t i) const { return vars_.at(i); }
  const OpInfo& GetOp(size_t i) const { return ops_.at(i); }
  VarDesc* AddVar() {
    vars_.emplace_back();
    return &vars_.back();
  }
  OpInfo* AddOp() {
    ops_.emplace_back();
    return &ops_.back();
  }
  std::vector<VarDesc>& vars() { return vars_; }
  const std::vector<VarDesc>& vars() const { return vars_; }
  std::vector<OpInfo>& ops() { return ops_; }
  const std::vector<OpInfo>& ops() const { return ops_; }

 private:
  int32_t idx_ = 0, parent_idx_ = 0, forward_block_idx_ = -1;
  std::vector<VarDesc> vars_;
  std::vector<OpInfo> ops_;
};

class ProgramDesc {
 public:
  size_t BlocksSize() const { return blocks_.size(); }
  BlockDesc* GetBlock(size_t i) { return &blocks_.at(i); }
  const BlockDesc* GetBlock(size_t i) const { return &blocks_.at(i); }
  BlockDesc* AddBlock() {
    blocks_.emplace_back();
    return &blocks_.back();
  }
  void ClearBlocks() { blocks_.clear(); }
  bool HasVersion() const { return has_version_; }
  int64_t Version() const { return version_; }
  void SetVersion(int64_t v) {
    version_ = v;
    has_version_ = true;
  }
  // op type -> version, in the order of the file
  const std::vector<std::pair<std::string, int32_t>>& OpVersionMap() const { return op_versions_; }
  void SetOpVersionMap(const std::vector<std::pair<std::string, int32_t>>& m) { op_versions_ = m; }

 private:
  std::vector<BlockDesc> blocks_;
  int64_t version_ = 0;
  bool has_version_ = false;
  std::vector<std::pair<std::string, int32_t>> op_versions_;
};

}  // namespace cpp
}  // namespace lite
}  // namespace paddle
