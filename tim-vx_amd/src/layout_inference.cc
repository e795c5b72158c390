// Layout inference for the operators of this runtime.
// reference: src/tim/transform/layout_inference.cc:340-417 (driver),
// src/tim/transform/ops/conv2d_layout_inference.h:36-136, pool2d_layout_inference.h,
// fullyconnected_layout_inference.h:43-75, op_layout_inference.h:36-45 (the permutations).
//
// One walk over the source graph in dependency order. Every source tensor has a counterpart in
// the new graph and a permutation pv saying how the counterpart is laid out: its dimension i
// is the source tensor's dimension pv[i]. A convolution or pooling tagged CWHN wants its
// activations as pv = {1, 2, 0, 3} (WHCN) and gets a Transpose in front only when the
// producer delivers something else, so chains of CWHN operators run back to back in WHCN with
// one permute at the graph's input and one at its output. Constant kernels are permuted on
// the host; kernels that are graph inputs get a Transpose. Element-wise operators pass the
// permutation through, everything else (FullyConnected, Reshape, Transpose) takes its input
// in the source layout.
#include "tim/transform/layout_inference.h"

#include <algorithm>
#include <cstring>
#include <deque>
#include <set>

#include "runtime.h"
#include "tim/vx/ops.h"

namespace tim {
namespace transform {
namespace {

using vx::DataLayout;
using vx::OpImpl;
using vx::OpKind;
using vx::Operation;
using vx::Tensor;
using vx::TensorAttribute;
using vx::TensorImpl;
using vx::TensorSpec;
using Perm = std::vector<uint32_t>;

class PermuteVector : public IPermuteVector {
 public:
  explicit PermuteVector(Perm p) : p_(std::move(p)) {}
  uint32_t Rank() const override { return static_cast<uint32_t>(p_.size()); }
  Perm AsStdVec() const override { return p_; }
  bool IsAligned() const override {
    for (uint32_t i = 0; i < p_.size(); ++i)
      if (p_[i] != i) return false;
    return true;
  }

 private:
  Perm p_;
};

Perm Identity(size_t rank) {
  Perm p(rank);
  for (size_t i = 0; i < rank; ++i) p[i] = static_cast<uint32_t>(i);
  return p;
}
bool IsIdentity(const Perm& p) { return p == Identity(p.size()); }
bool IsPermutation(const Perm& p, size_t rank) {
  if (p.size() != rank) return false;
  std::vector<bool> seen(rank, false);
  for (uint32_t v : p) {
    if (v >= rank || seen[v]) return false;
    seen[v] = true;
  }
  return true;
}
// The Transpose that turns a tensor laid out as `have` into one laid out as `want`
// (both relative to the same source tensor): out dim i = in dim t[i].
Perm Between(const Perm& have, const Perm& want) {
  Perm t(want.size());
  for (size_t i = 0; i < want.size(); ++i)
    t[i] = static_cast<uint32_t>(std::find(have.begin(), have.end(), want[i]) - have.begin());
  return t;
}
vx::ShapeType Permuted(const vx::ShapeType& shape, const Perm& p) {
  vx::ShapeType out(p.size());
  for (size_t i = 0; i < p.size(); ++i) out[i] = shape[p[i]];
  return out;
}

Perm ActivationLayout(DataLayout l, size_t rank) {
  if (l == DataLayout::CWHN && rank == 4) return {1, 2, 0, 3};
  return Identity(rank);
}
Perm KernelLayout(DataLayout l, size_t rank) {
  if (rank != 4) return Identity(rank);
  switch (l) {
    case DataLayout::IcWHOc: return {1, 2, 0, 3};
    case DataLayout::OcIcWH: return {2, 3, 1, 0};
    case DataLayout::IcOcWH: return {2, 3, 0, 1};
    default: return Identity(rank);
  }
}

struct Walk {
  std::shared_ptr<vx::Graph> src, dst;
  std::map<Tensor*, std::shared_ptr<Tensor>> mapped;
  std::map<Tensor*, Perm> pv;
  bool ok = true;

  TensorSpec SpecFor(const std::shared_ptr<Tensor>& t_src, const Perm& p, TensorAttribute attr) {
    TensorSpec s = t_src->GetSpec();
    s.attr_ = attr;
    if (!s.shape_.empty() && s.shape_.size() == p.size()) s.shape_ = Permuted(s.shape_, p);
    vx::Quantization& q = s.quantization_;
    if (q.Type() == vx::QuantType::SYMMETRIC_PER_CHANNEL && q.ChannelDim() >= 0 &&
        static_cast<size_t>(q.ChannelDim()) < p.size())
      q.SetChannelDim(static_cast<int32_t>(std::find(p.begin(), p.end(), static_cast<uint32_t>(q.ChannelDim())) - p.begin()));
    return s;
  }

  // A constant of the source graph, laid out as p, created in the new graph (data permuted on the host).
  std::shared_ptr<Tensor> PermutedConstant(const std::shared_ptr<Tensor>& t_src, const Perm& p) {
    auto* ti = static_cast<TensorImpl*>(t_src.get());
    const vx::ShapeType& shape = ti->spec_.shape_;
    const size_t eb = static_cast<size_t>(ti->spec_.GetElementByteSize());
    const uint8_t* in = ti->HostData();
    std::vector<uint8_t> out(ti->HostBytes());
    if (!in || out.empty()) {
      VSILOGE("layout inference: constant tensor %u has no data", ti->id_);
      ok = false;
      return nullptr;
    }
    const size_t rank = shape.size();
    std::vector<size_t> in_stride(rank, 1);
    for (size_t i = 1; i < rank; ++i) in_stride[i] = in_stride[i - 1] * shape[i - 1];
    const vx::ShapeType oshape = Permuted(shape, p);
    std::vector<uint32_t> c(rank, 0);
    const size_t total = out.size() / eb;
    for (size_t o = 0; o < total; ++o) {
      size_t src_off = 0;
      for (size_t i = 0; i < rank; ++i) src_off += c[i] * in_stride[p[i]];
      std::memcpy(&out[o * eb], in + src_off * eb, eb);
      for (size_t i = 0; i < rank; ++i) {
        if (++c[i] < oshape[i]) break;
        c[i] = 0;
      }
    }
    return dst->CreateTensor(SpecFor(t_src, p, TensorAttribute::CONSTANT), out.data());
  }

  // The counterpart of t_src laid out as `want`: as it is, behind a Transpose, or (constants) permuted.
  std::shared_ptr<Tensor> InLayout(const std::shared_ptr<Tensor>& t_src, const Perm& want) {
    if (t_src->IsConstTensor()) {
      if (IsIdentity(want)) {
        auto it = mapped.find(t_src.get());
        if (it != mapped.end()) return it->second;  // shared constants are created once
        auto* ti = static_cast<TensorImpl*>(t_src.get());
        auto t = dst->CreateTensor(ti->spec_, ti->HostData());
        mapped[t_src.get()] = t;
        pv[t_src.get()] = want;
        return t;
      }
      return PermutedConstant(t_src, want);
    }
    auto cur = mapped.at(t_src.get());
    const Perm& have = pv.at(t_src.get());
    if (have == want) return cur;
    if (have.size() != want.size()) {
      VSILOGE("layout inference: tensor %u has rank %zu where an operator expects rank %zu", t_src->GetId(), have.size(), want.size());
      ok = false;
      return nullptr;
    }
    auto out = dst->CreateTensor(SpecFor(t_src, want, TensorAttribute::TRANSIENT));
    auto tr = dst->CreateOperation<vx::ops::Transpose>(Between(have, want));
    (*tr).BindInput(cur).BindOutput(out);
    // later consumers that want the same layout reuse the permuted tensor
    mapped[t_src.get()] = out;
    pv[t_src.get()] = want;
    return out;
  }

  // The tensor an operator of the new graph writes for t_src when it produces layout p. A graph
  // OUTPUT keeps the source shape: a Transpose back is put behind the operator when p is not the identity.
  std::shared_ptr<Tensor> OutLayout(const std::shared_ptr<Tensor>& t_src, const Perm& p) {
    const bool is_output = t_src->GetSpec().attr_ == TensorAttribute::OUTPUT;
    if (!is_output || IsIdentity(p)) {
      std::shared_ptr<Tensor> t;
      if (is_output) {
        t = mapped.at(t_src.get());  // created up front with the source spec
      } else {
        t = dst->CreateTensor(SpecFor(t_src, p, TensorAttribute::TRANSIENT));
        mapped[t_src.get()] = t;
      }
      pv[t_src.get()] = p;
      return t;
    }
    auto inner = dst->CreateTensor(SpecFor(t_src, p, TensorAttribute::TRANSIENT));
    auto tr = dst->CreateOperation<vx::ops::Transpose>(Between(p, Identity(p.size())));
    (*tr).BindInput(inner).BindOutput(mapped.at(t_src.get()));
    pv[t_src.get()] = Identity(p.size());
    return inner;
  }

  // TRANSIENT tensors are usually declared without a shape: their rank then comes from the permutation
  // recorded for them when their producer was handled.
  size_t RankOf(const std::shared_ptr<Tensor>& t) {
    if (!t->GetShape().empty()) return t->GetShape().size();
    auto it = pv.find(t.get());
    return it != pv.end() ? it->second.size() : 0;
  }

  void Handle(const std::shared_ptr<Operation>& op) {
    OpImpl* im = op->impl().get();
    const auto& ins = im->inputs_tensor_;
    const auto& outs = im->outputs_tensor_;
    if (ins.empty() || outs.size() != 1) {
      VSILOGE("layout inference: %s with %zu inputs / %zu outputs", vx::OpKindName(im->kind_), ins.size(), outs.size());
      ok = false;
      return;
    }
    std::vector<std::shared_ptr<Tensor>> new_ins;
    Perm out_pv;
    std::shared_ptr<Operation> clone;
    switch (im->kind_) {
      case OpKind::CONV2D: {
        const size_t rank = im->attrs_.conv_1d ? 3 : 4;
        const Perm act = im->attrs_.conv_1d ? Identity(rank) : ActivationLayout(im->layout_, rank);
        new_ins.push_back(InLayout(ins[0], act));
        if (ins.size() > 1)
          new_ins.push_back(InLayout(ins[1], im->attrs_.conv_1d ? Identity(3) : KernelLayout(im->attrs_.kernel_layout, 4)));
        for (size_t i = 2; i < ins.size(); ++i)
          new_ins.push_back(ins[i]->IsPlaceHolder() ? dst->CreateTensorPlaceHolder() : InLayout(ins[i], Identity(RankOf(ins[i]))));
        out_pv = act;
        clone = op->Clone(dst);
        if (!im->attrs_.conv_1d) clone->impl()->layout_ = DataLayout::WHCN;
        clone->impl()->attrs_.kernel_layout = DataLayout::WHIcOc;
        break;
      }
      case OpKind::POOL: {
        const Perm act = im->attrs_.pool_1d ? Identity(3) : ActivationLayout(im->layout_, 4);
        new_ins.push_back(InLayout(ins[0], act));
        out_pv = act;
        clone = op->Clone(dst);
        if (!im->attrs_.pool_1d) clone->impl()->layout_ = DataLayout::WHCN;
        break;
      }
      case OpKind::RELU:
      case OpKind::RELU6:
      case OpKind::DATACONVERT: {
        out_pv = ins[0]->IsConstTensor() ? Identity(RankOf(ins[0])) : pv.at(ins[0].get());
        new_ins.push_back(InLayout(ins[0], out_pv));
        clone = op->Clone(dst);
        break;
      }
      case OpKind::SOFTMAX: {
        out_pv = ins[0]->IsConstTensor() ? Identity(RankOf(ins[0])) : pv.at(ins[0].get());
        new_ins.push_back(InLayout(ins[0], out_pv));
        const int32_t rank = static_cast<int32_t>(out_pv.size());
        int32_t axis = im->attrs_.sm_axis;
        if (axis < 0) axis += rank;
        if (axis < 0 || axis >= rank) {
          VSILOGE("layout inference: SOFTMAX axis %d of a rank-%d tensor", im->attrs_.sm_axis, rank);
          ok = false;
          return;
        }
        const int32_t new_axis = static_cast<int32_t>(std::find(out_pv.begin(), out_pv.end(), static_cast<uint32_t>(axis)) - out_pv.begin());
        clone = dst->CreateOperation<vx::ops::Softmax>(im->attrs_.beta, new_axis);
        break;
      }
      case OpKind::ADD: {
        if (ins.size() != 2) { ok = false; return; }
        // follow the operand that is not a constant (the first, if neither is)
        const size_t lead = ins[0]->IsConstTensor() && !ins[1]->IsConstTensor() ? 1 : 0;
        out_pv = ins[lead]->IsConstTensor() ? Identity(RankOf(ins[lead])) : pv.at(ins[lead].get());
        new_ins.resize(2);
        new_ins[lead] = InLayout(ins[lead], out_pv);
        new_ins[1 - lead] = InLayout(ins[1 - lead], out_pv);
        clone = op->Clone(dst);
        break;
      }
      case OpKind::FCL:
      case OpKind::RESHAPE:
      case OpKind::DECONV2D:  // taken in the source layout (WHCN is what it accepts)
      case OpKind::TRANSPOSE: {
        for (const auto& t : ins)
          new_ins.push_back(t->IsPlaceHolder() ? dst->CreateTensorPlaceHolder() : InLayout(t, Identity(RankOf(t))));
        const size_t out_rank = im->kind_ == OpKind::FCL ? 2
                                : im->kind_ == OpKind::RESHAPE ? im->attrs_.new_shape.size()
                                : im->kind_ == OpKind::TRANSPOSE ? im->attrs_.perm.size()
                                : im->attrs_.conv_1d ? 3 : 4;  // (DeConv1d: {W, C, N})
        out_pv = Identity(out_rank);
        clone = op->Clone(dst);
        break;
      }
    }
    if (!ok || !clone) { ok = false; return; }
    if (!outs[0]->GetShape().empty() && outs[0]->GetShape().size() != out_pv.size()) {
      VSILOGE("layout inference: %s writes a rank-%zu tensor declared with rank %zu", vx::OpKindName(im->kind_),
              out_pv.size(), outs[0]->GetShape().size());
      ok = false;
      return;
    }
    auto out = OutLayout(outs[0], out_pv);
    for (auto& t : new_ins) {
      if (!t) { ok = false; return; }
      clone->BindInput(t);
    }
    clone->BindOutput(out);
  }
};

}  // namespace

std::shared_ptr<IPermuteVector> MakePermuteVector(const std::vector<uint32_t>& perm) {
  return std::make_shared<PermuteVector>(perm);
}

// The walk itself, into a graph the caller made. io_map may arrive holding counterparts for some
// of the source graph's INPUT / OUTPUT tensors (tensors of dst, with the source tensors' specs):
// those are used instead of new ones. On return it holds all of them.
bool RewriteInto(const std::shared_ptr<vx::Graph>& src_graph, const std::shared_ptr<vx::Graph>& dst_graph,
                 const std::map<std::shared_ptr<vx::Tensor>, std::shared_ptr<IPermuteVector>>& tensor_pv_map,
                 std::map<std::shared_ptr<vx::Tensor>, std::shared_ptr<vx::Tensor>>* io_map) {
  Walk w;
  w.src = src_graph;
  w.dst = dst_graph;
  auto stated = [&](const std::shared_ptr<Tensor>& t) {
    auto it = tensor_pv_map.find(t);
    Perm p = it != tensor_pv_map.end() && it->second ? it->second->AsStdVec() : Identity(t->GetShape().size());
    if (!IsPermutation(p, t->GetShape().size())) {
      VSILOGE("layout inference: the permute vector given for tensor %u is not a permutation of its dimensions", t->GetId());
      w.ok = false;
      p = Identity(t->GetShape().size());
    }
    return p;
  };
  auto counterpart = [&](const std::shared_ptr<Tensor>& t) {
    auto it = io_map->find(t);
    if (it != io_map->end() && it->second) return it->second;
    auto n = w.dst->CreateTensor(t->GetSpec());
    (*io_map)[t] = n;
    return n;
  };
  for (const auto& t : src_graph->InputsTensor()) {
    w.mapped[t.get()] = counterpart(t);
    w.pv[t.get()] = stated(t);
  }
  for (const auto& t : src_graph->OutputsTensor()) w.mapped[t.get()] = counterpart(t);
  // dependency order: an operator is handled once every non-constant input has a counterpart
  std::deque<std::shared_ptr<Operation>> pending(src_graph->OpVector().begin(), src_graph->OpVector().end());
  std::set<Tensor*> produced;
  for (const auto& t : src_graph->InputsTensor()) produced.insert(t.get());
  size_t stalled = 0;
  while (!pending.empty() && w.ok && stalled <= pending.size()) {
    auto op = pending.front();
    pending.pop_front();
    bool ready = true;
    for (const auto& t : op->impl()->inputs_tensor_)
      if (!t->IsPlaceHolder() && !t->IsConstTensor() && !produced.count(t.get())) ready = false;
    if (!ready) {
      pending.push_back(op);
      ++stalled;
      continue;
    }
    stalled = 0;
    w.Handle(op);
    for (const auto& t : op->impl()->outputs_tensor_) produced.insert(t.get());
  }
  if (!pending.empty() && w.ok) {
    VSILOGE("layout inference: %zu operators wait for tensors nothing produces", pending.size());
    w.ok = false;
  }
  if (!w.ok) VSILOGE("layout inference failed; the rewritten graph is incomplete and will not compile");
  return w.ok;
}

std::pair<std::shared_ptr<vx::Graph>, std::map<std::shared_ptr<vx::Tensor>, std::shared_ptr<vx::Tensor>>>
LayoutInference(const std::shared_ptr<vx::Graph>& src_graph, std::shared_ptr<vx::Context>& ctx,
                std::map<std::shared_ptr<vx::Tensor>, std::shared_ptr<IPermuteVector>> tensor_pv_map) {
  std::map<std::shared_ptr<Tensor>, std::shared_ptr<Tensor>> io_map;
  auto dst = ctx->CreateGraph();
  RewriteInto(src_graph, dst, tensor_pv_map, &io_map);
  return std::make_pair(dst, io_map);
}

}  // namespace transform
}  // namespace tim
