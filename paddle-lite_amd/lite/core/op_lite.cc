#include "lite/core/op_lite.h"

#include "lite/core/op_registry.h"

namespace paddle {
namespace lite {

// reference: lite/core/op_lite.cc (OpLite::CreateKernels): kernels of the
// first valid place that has a registration; "op/alias" restricts the alias.
std::vector<std::unique_ptr<KernelBase>> OpLite::CreateKernels(const std::vector<lite_api::Place>& places, const std::string& kernel_type) {
  std::vector<std::unique_ptr<KernelBase>> out;
  std::string alias;
  const size_t slash = kernel_type.find('/');
  if (slash != std::string::npos) alias = kernel_type.substr(slash + 1);
  for (const lite_api::Place& place : places) {
    auto ks = KernelFactory::Global().Create(op_type_, place.target, place.precision, place.layout);
    for (auto& k : ks) {
      if (!alias.empty() && k->alias() != alias) continue;
      k->SetContext(ContextScheduler::Global().NewContext(k->target()));
      AttachKernel(k.get());
      out.emplace_back(std::move(k));
    }
    if (!out.empty()) break;
  }
  return out;
}

}  // namespace lite
}  // namespace paddle
