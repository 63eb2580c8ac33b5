// Operator and kernel registries with the reference's registration macros
// (reference: lite/core/op_registry.h:38-291).
#pragma once

#include <functional>
#include <list>
#include <map>
#include <memory>
#include <string>
#include <tuple>
#include <vector>

#include "lite/core/kernel.h"
#include "lite/core/op_lite.h"

namespace paddle {
namespace lite {

class OpLiteFactory {
 public:
  using Creator = std::function<std::unique_ptr<OpLite>()>;
  static OpLiteFactory& Global() {
    static OpLiteFactory* f = new OpLiteFactory;
    return *f;
  }
  void RegisterCreator(const std::string& op_type, Creator c) { creators_[op_type] = std::move(c); }
  std::unique_ptr<OpLite> Create(const std::string& op_type) const {
    auto it = creators_.find(op_type);
    return it == creators_.end() ? nullptr : it->second();
  }
  std::vector<std::string> GetAllOps() const {
    std::vector<std::string> v;
    for (auto& kv : creators_) v.push_back(kv.first);
    return v;
  }

 private:
  std::map<std::string, Creator> creators_;
};
using LiteOpRegistry = OpLiteFactory;

struct OpLiteRegistrar {
  OpLiteRegistrar(const std::string& op_type, OpLiteFactory::Creator c) { OpLiteFactory::Global().RegisterCreator(op_type, std::move(c)); }
  void touch() {}
};

class KernelFactory {
 public:
  using Creator = std::function<std::unique_ptr<KernelBase>()>;
  using Key = std::tuple<lite_api::TargetType, lite_api::PrecisionType, lite_api::DataLayoutType>;
  static KernelFactory& Global() {
    static KernelFactory* f = new KernelFactory;
    return *f;
  }
  void RegisterCreator(const std::string& op_type, lite_api::TargetType t, lite_api::PrecisionType p, lite_api::DataLayoutType l, Creator c) {
    creators_[op_type][Key(t, p, l)].push_back(std::move(c));
  }
  // every kernel of an op
  std::list<std::unique_ptr<KernelBase>> Create(const std::string& op_type) const {
    std::list<std::unique_ptr<KernelBase>> out;
    auto it = creators_.find(op_type);
    if (it == creators_.end()) return out;
    for (auto& per_place : it->second)
      for (auto& c : per_place.second) out.emplace_back(c());
    return out;
  }
  // the kernels of one (target, precision, layout); a list because several
  // aliases may share a place (int8_fp32_out / int8_int8_out)
  std::list<std::unique_ptr<KernelBase>> Create(const std::string& op_type, lite_api::TargetType t, lite_api::PrecisionType p, lite_api::DataLayoutType l) const {
    std::list<std::unique_ptr<KernelBase>> out;
    auto it = creators_.find(op_type);
    if (it == creators_.end()) return out;
    auto jt = it->second.find(Key(t, p, l));
    if (jt == it->second.end()) return out;
    for (auto& c : jt->second) out.emplace_back(c());
    return out;
  }

 private:
  std::map<std::string, std::map<Key, std::list<Creator>>> creators_;
};
using KernelRegistry = KernelFactory;

struct KernelRegistrar {
  KernelRegistrar(const std::string& op_type, lite_api::TargetType t, lite_api::PrecisionType p, lite_api::DataLayoutType l, KernelFactory::Creator c) {
    KernelFactory::Global().RegisterCreator(op_type, t, p, l, std::move(c));
  }
  void touch() {}
};

// Declared type of one kernel argument
// (reference: lite/core/type_system.h LiteType::GetTensorTy).
struct TensorTy {
  lite_api::TargetType target;
  lite_api::PrecisionType precision;
  lite_api::DataLayoutType layout;
};
struct LiteType {
  static TensorTy GetTensorTy(lite_api::TargetType t, lite_api::PrecisionType p = lite_api::PrecisionType::kFloat, lite_api::DataLayoutType l = lite_api::DataLayoutType::kNCHW) {
    return TensorTy{t, p, l};
  }
};

// Argument types per "op_type/alias" and place: what type_target_cast_pass
// reads to decide where io_copy / calib ops are needed.
class ParamTypeRegistry {
 public:
  struct Entry {
    bool is_input;
    std::string arg;
    TensorTy type;
  };
  static ParamTypeRegistry& Global() {
    static ParamTypeRegistry* r = new ParamTypeRegistry;
    return *r;
  }
  class NewInstance {
   public:
    NewInstance(const std::string& kernel_key, lite_api::Place place) : key_(kernel_key + ":" + place.DebugString()) {}
    NewInstance& BindInput(const std::string& arg, const TensorTy& ty) {
      ParamTypeRegistry::Global().types_[key_].push_back(Entry{true, arg, ty});
      return *this;
    }
    NewInstance& BindOutput(const std::string& arg, const TensorTy& ty) {
      ParamTypeRegistry::Global().types_[key_].push_back(Entry{false, arg, ty});
      return *this;
    }
    bool Finalize() { return true; }

   private:
    std::string key_;
  };
  const std::vector<Entry>* Retrieve(const std::string& kernel_key, lite_api::Place place) const {
    auto it = types_.find(kernel_key + ":" + place.DebugString());
    return it == types_.end() ? nullptr : &it->second;
  }

 private:
  std::map<std::string, std::vector<Entry>> types_;
};

}  // namespace lite
}  // namespace paddle

#define REGISTER_LITE_OP(op_type__, OpClass)                                                           \
  static paddle::lite::OpLiteRegistrar op_type__##__registry(#op_type__, []() {                        \
    return std::unique_ptr<paddle::lite::OpLite>(new OpClass(#op_type__));                             \
  });                                                                                                  \
  int touch_op_##op_type__() {                                                                         \
    op_type__##__registry.touch();                                                                     \
    return 0;                                                                                          \
  }

#define REGISTER_LITE_KERNEL(op_type__, target__, precision__, layout__, KernelClass, alias__)                 \
  static paddle::lite::KernelRegistrar op_type__##target__##precision__##layout__##alias__##_kernel_registry(  \
      #op_type__, TARGET(target__), PRECISION(precision__), DATALAYOUT(layout__), []() {                      \
        std::unique_ptr<KernelClass> x(new KernelClass);                                                      \
        x->set_op_type(#op_type__);                                                                           \
        x->set_alias(#alias__);                                                                               \
        return std::unique_ptr<paddle::lite::KernelBase>(std::move(x));                                       \
      });                                                                                                     \
  int touch_##op_type__##target__##precision__##layout__##alias__() {                                         \
    op_type__##target__##precision__##layout__##alias__##_kernel_registry.touch();                            \
    return 0;                                                                                                 \
  }                                                                                                           \
  static bool op_type__##target__##precision__##layout__##alias__##_param_register __attribute__((unused)) =  \
      paddle::lite::ParamTypeRegistry::NewInstance(                                                           \
          #op_type__ "/" #alias__, paddle::lite_api::Place(TARGET(target__), PRECISION(precision__), DATALAYOUT(layout__)))
