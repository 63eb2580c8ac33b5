// Operator description: named input / output argument lists and typed
// attributes, plus the quantisation scales OpInfo carries
// (reference: lite/core/model/general/op_desc.h, lite/core/op_lite.h OpInfo).
#pragma once

#include <algorithm>
#include <any>
#include <map>
#include <string>
#include <vector>

#include "lite/utils/log.h"

namespace paddle {
namespace lite {
namespace cpp {

class OpDesc {
 public:
  OpDesc() = default;
  explicit OpDesc(const std::string& type) : type_(type) {}
  virtual ~OpDesc() = default;

  const std::string& Type() const { return type_; }
  void SetType(const std::string& t) { type_ = t; }

  std::vector<std::string> Input(const std::string& arg) const { return Find(inputs_, arg, "input"); }
  std::vector<std::string> Output(const std::string& arg) const { return Find(outputs_, arg, "output"); }
  void SetInput(const std::string& arg, const std::vector<std::string>& names) { inputs_[arg] = names; }
  void SetOutput(const std::string& arg, const std::vector<std::string>& names) { outputs_[arg] = names; }
  bool HasInput(const std::string& arg) const { return inputs_.count(arg) != 0; }
  bool HasOutput(const std::string& arg) const { return outputs_.count(arg) != 0; }
  std::vector<std::string> InputArgumentNames() const { return Keys(inputs_); }
  std::vector<std::string> OutputArgumentNames() const { return Keys(outputs_); }
  const std::map<std::string, std::vector<std::string>>& inputs() const { return inputs_; }
  const std::map<std::string, std::vector<std::string>>& outputs() const { return outputs_; }

  bool HasAttr(const std::string& name) const { return attrs_.count(name) != 0; }
  std::vector<std::string> AttrNames() const {
    std::vector<std::string> n;
    for (auto& kv : attrs_) n.push_back(kv.first);
    return n;
  }
  template <typename T>
  void SetAttr(const std::string& name, const T& v) {
    attrs_[name] = v;
  }
  template <typename T>
  T GetAttr(const std::string& name) const {
    auto it = attrs_.find(name);
    CHECK(it != attrs_.end()) << "No attributes called " << name << " found for " << type_;
    const T* v = std::any_cast<T>(&it->second);
    CHECK(v != nullptr) << "attribute " << name << " of " << type_ << " has another type";
    return *v;
  }
  const std::map<std::string, std::any>& attrs() const { return attrs_; }
  void CopyAttrsFrom(const OpDesc& other) {
    for (auto& kv : other.attrs_) attrs_[kv.first] = kv.second;
  }

 private:
  using ArgMap = std::map<std::string, std::vector<std::string>>;
  std::vector<std::string> Find(const ArgMap& m, const std::string& arg, const char* what) const {
    auto it = m.find(arg);
    CHECK(it != m.end()) << "No " << what << " called " << arg << " found for " << type_;
    return it->second;
  }
  static std::vector<std::string> Keys(const ArgMap& m) {
    std::vector<std::string> k;
    for (auto& kv : m) k.push_back(kv.first);
    return k;
  }

  std::string type_;
  ArgMap inputs_, outputs_;
  std::map<std::string, std::any> attrs_;
};

}  // namespace cpp

// OpDesc plus the per-argument quantisation scales, stored as attributes
// "<name>" with a vector<float> value like the reference does
// (lite/core/op_lite.h: OpInfo::{Has,Get,Set}{Input,Output}Scale).
class OpInfo : public cpp::OpDesc {
 public:
  OpInfo() = default;
  explicit OpInfo(const std::string& type) : cpp::OpDesc(type) {}
  explicit OpInfo(const cpp::OpDesc& d) : cpp::OpDesc(d) {}

  bool HasInputScale(const std::string& name, bool is_scale_name = false) const { return HasAttr(ScaleKey(name, is_scale_name)); }
  bool HasOutputScale(const std::string& name, bool is_scale_name = false) const { return HasAttr(ScaleKey(name, is_scale_name)); }
  std::vector<float> GetInputScale(const std::string& name, bool is_scale_name = false) const { return GetAttr<std::vector<float>>(ScaleKey(name, is_scale_name)); }
  std::vector<float> GetOutputScale(const std::string& name, bool is_scale_name = false) const { return GetAttr<std::vector<float>>(ScaleKey(name, is_scale_name)); }
  void SetInputScale(const std::string& name, const std::vector<float>& v, bool is_scale_name = false) { SetAttr(ScaleKey(name, is_scale_name), v); }
  void SetOutputScale(const std::string& name, const std::vector<float>& v, bool is_scale_name = false) { SetAttr(ScaleKey(name, is_scale_name), v); }

 private:
  // Scales are addressed by scale name ("Input0_scale") in this slice; a
  // variable name would first have to be mapped to "<Arg><index>_scale".
  static std::string ScaleKey(const std::string& name, bool is_scale_name) {
    CHECK(is_scale_name) << "scales are looked up by scale name here";
    return name;
  }
};

}  // namespace lite
}  // namespace paddle
