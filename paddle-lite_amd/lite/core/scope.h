// Variable and Scope: name -> tensor storage that operators attach to
// (reference: lite/core/variable.h, lite/core/scope.h).
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "lite/core/tensor.h"

namespace paddle {
namespace lite {

class Variable {
 public:
  template <typename T>
  const T& Get() const {
    static_assert(std::is_same<T, Tensor>::value, "only tensors are stored");
    CHECK(tensor_) << "variable holds no tensor";
    return *tensor_;
  }
  template <typename T>
  T* GetMutable() {
    static_assert(std::is_same<T, Tensor>::value, "only tensors are stored");
    if (!tensor_) tensor_.reset(new Tensor);
    return tensor_.get();
  }

 private:
  std::unique_ptr<Tensor> tensor_;
};

class Scope {
 public:
  Variable* Var(const std::string& name) {
    auto& slot = vars_[name];
    if (!slot) slot.reset(new Variable);
    return slot.get();
  }
  Variable* FindVar(const std::string& name) const {
    auto it = vars_.find(name);
    return it == vars_.end() ? nullptr : it->second.get();
  }
  Tensor* NewTensor(const std::string& name) { return Var(name)->GetMutable<Tensor>(); }
  Tensor* FindMutableTensor(const std::string& name) const {
    Variable* v = FindVar(name);
    return v ? v->GetMutable<Tensor>() : nullptr;
  }
  void Erase(const std::string& name) { vars_.erase(name); }
  std::vector<std::string> LocalVarNames() const {
    std::vector<std::string> n;
    for (auto& kv : vars_) n.push_back(kv.first);
    return n;
  }

 private:
  std::map<std::string, std::unique_ptr<Variable>> vars_;
};

}  // namespace lite
}  // namespace paddle
