#include "lite/core/optimizer/mir/sparse_conv_detect_pass.h"

#include "lite/core/optimizer/mir/graph.h"

#include "pl_sparse_conv.h"
#include "lite/core/tensor.h"

namespace paddle {
namespace lite {
namespace mir {

namespace {

struct Counts {
  int zeros = 0, n_weights = 0, n_diffs = 0, flag_semi = 0;
};

// The counting step of the pass: semi analysis first; fp32 matrices that are
// not semi-structured get their rows padded to four entries
// (reference: sparse_conv_detect_pass.cc:654-683).
Counts Analyse(int dtype, const void* w, int oc, int ic) {
  Counts c;
  int32_t nnz = 0, channels = 0, blocks = 0, semi = 0;
  c.zeros = pl_sparse_count_semi(dtype, w, oc, ic, &nnz, &channels, &blocks, &semi);
  CHECK_GE(c.zeros, 0) << pl_last_error();
  c.flag_semi = semi;
  c.n_weights = nnz;
  c.n_diffs = semi ? blocks : nnz;
  if (dtype == 0 && !semi) {
    int32_t padded = 0;
    c.zeros = pl_sparse_count_zeros(dtype, w, oc, ic, &padded);
    c.n_weights = c.n_diffs = padded;
  }
  return c;
}

}  // namespace

int SparseConvDetectPass::Apply(std::vector<OpInfo>* ops, Scope* scope) const {
  Graph graph(*ops, *scope);
  const int replaced = Apply(&graph, scope);
  *ops = graph.TopologicalOps();
  return replaced;
}

int SparseConvDetectPass::Apply(Graph* graph, Scope* scope) const {
  int replaced = 0;
  for (Graph::Node* node : graph->OpNodes()) {
    OpInfo& conv = node->op;
    if (conv.Type() != "conv2d") continue;
    const std::string x = conv.Input("Input").front();
    const std::string w = conv.Input("Filter").front();
    const std::string y = conv.Output("Output").front();
    Tensor* xt = scope->FindMutableTensor(x);
    Tensor* wt = scope->FindMutableTensor(w);
    CHECK(xt && wt) << "conv2d input or filter is not in the scope";
    const DDim& xd = xt->dims();
    const DDim& wd = wt->dims();
    const int groups = conv.GetAttr<int>("groups");
    const auto strides = conv.GetAttr<std::vector<int>>("strides");
    const auto paddings = conv.GetAttr<std::vector<int>>("paddings");
    const bool int8 = wt->precision() == PrecisionType::kInt8;
    const bool fp32 = wt->precision() == PrecisionType::kFloat;
    const int oc = static_cast<int>(wd[0]), ic = static_cast<int>(wd[1]) * groups;
    // the conditions of sparse_conv_detect_pass.cc:627-652
    if (!(int8 || fp32)) continue;
    if (!(wd[2] == 1 && wd[3] == 1)) continue;
    if (groups != 1) continue;
    if (!(strides[0] == 1 && strides[1] == 1)) continue;
    if (!(paddings[0] == 0 && paddings[1] == 0)) continue;
    if (!(oc > 0 && ic > 0)) continue;

    const int dtype = int8 ? 1 : 0;
    const Counts c = Analyse(dtype, wt->raw_data(), oc, ic);
    const float zero_fraction = static_cast<float>(c.zeros) / static_cast<float>(oc * ic);
    if (zero_fraction < sparse_threshold_) continue;  // :684-692

    const int im_size = static_cast<int>(xd[2] * xd[3]);
    Tensor* nz = scope->NewTensor(w + "_nonzeros_output");
    Tensor* ocn = scope->NewTensor(w + "_oc_nonzeros");
    Tensor* dif = scope->NewTensor(w + "_ic_diffs");
    nz->Resize({c.n_weights});
    ocn->Resize({oc});
    dif->Resize({c.n_diffs});
    void* nz_data = int8 ? static_cast<void*>(nz->mutable_data<int8_t>(TargetType::kHost)) : static_cast<void*>(nz->mutable_data<float>(TargetType::kHost));
    uint32_t* ocn_data = ocn->mutable_data<uint32_t>(TargetType::kHost);
    int32_t* dif_data = dif->mutable_data<int32_t>(TargetType::kHost);
    const int first_ic = pl_sparse_pack(dtype, c.flag_semi, wt->raw_data(), oc, ic, im_size, nz_data, c.n_weights, ocn_data, dif_data, c.n_diffs);
    CHECK_GE(first_ic, 0) << pl_last_error();
    for (Tensor* t : {nz, ocn, dif}) t->set_persistable(true);
    nz->set_precision(int8 ? PrecisionType::kInt8 : PrecisionType::kFloat);
    ocn->set_precision(PrecisionType::kInt32);
    dif->set_precision(PrecisionType::kInt32);

    OpInfo sparse("sparse_conv2d");
    sparse.SetInput("Input", {x});
    sparse.SetInput("NonZeroWeights", {w + "_nonzeros_output"});
    sparse.SetInput("OcNonZeros", {w + "_oc_nonzeros"});
    sparse.SetInput("Diffs", {w + "_ic_diffs"});
    if (conv.HasInput("Bias") && !conv.Input("Bias").empty()) sparse.SetInput("Bias", {conv.Input("Bias").front()});
    if (conv.HasInput("Prelu_alpha")) sparse.SetInput("Prelu_alpha", conv.Input("Prelu_alpha"));
    sparse.SetOutput("Output", {y});
    // int8 weights force enable_int8 on the conv before its attributes
    // (scales included) are copied over (:806-827)
    if (int8) conv.SetAttr<bool>("enable_int8", true);
    sparse.CopyAttrsFrom(conv);
    sparse.SetAttr<int>("first_ic", first_ic);
    sparse.SetAttr<int>("flag_semi", c.flag_semi);

    // The rewrite on the graph (:828-857): the conv node goes, the sparse op
    // node takes over its links to the activation, the bias and the output,
    // the three new weight variables are linked in, and the dense filter's
    // node is dropped.  A filter that another op still reads keeps its node
    // and its tensor (the reference removes the node regardless and would
    // leave that op with a dangling link).
    const int order = node->order;
    Graph::Node* filter = graph->Var(w);
    graph->RemoveNode(node);  // `conv` is gone from here on
    for (const char* weight : {"_nonzeros_output", "_oc_nonzeros", "_ic_diffs"}) graph->RetrieveVarNode(w + weight, true);
    graph->CreateOpNode(sparse, order);
    if (filter != nullptr && filter->outlinks.empty() && filter->inlinks.empty()) {
      graph->RemoveNode(filter);
      scope->Erase(w);
    }
    ++replaced;
  }
  return replaced;
}

}  // namespace mir
}  // namespace lite
}  // namespace paddle
