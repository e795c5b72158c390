// Host-side compile passes: execution order, operand checks, padding and
// shape inference. The rules restate ovxlib's per-operator check/setup:
//   padding / output size  src/tim/vx/internal/src/utils/vsi_nn_util.c:203-235,483-588
//   conv2d                 src/tim/vx/internal/src/ops/vsi_nn_op_conv2d.c:80-287
//   pool                   src/tim/vx/internal/src/ops/vsi_nn_op_pool.c:210-427
//   fully connected        src/tim/vx/internal/src/ops/vsi_nn_op_fullconnect2.c:45-196
//   bias-scale consistency src/tim/vx/internal/src/quantization/vsi_nn_asymmetric_affine.c:62-112
//                          src/tim/vx/internal/src/utils/vsi_nn_dtype_util.c:368-420
#include <algorithm>
#include <cmath>
#include <set>

#include "runtime.h"

namespace tim {
namespace vx {

uint32_t ComputeFilterSize(uint32_t in, uint32_t ksize, const uint32_t pad[2],
                           uint32_t stride, uint32_t dilation, RoundType rnd) {
  if (stride == 0) {
    if (in == ksize) {
      stride = 1;
    } else {
      VSILOGE("Error stride value: 0.");
      return 0;
    }
  }
  if (dilation > 1) ksize = dilation * (ksize - 1) + 1;
  int64_t span = static_cast<int64_t>(in) + pad[0] + pad[1] - ksize;
  if (span < 0) return 0;
  uint32_t out = static_cast<uint32_t>(span);
  out = rnd == RoundType::CEILING ? (out + stride - 1) / stride : out / stride;
  return out + 1;
}

void ComputePaddingPerAxis(uint32_t in, uint32_t ksize, uint32_t stride,
                           uint32_t dilation, PadType type, uint32_t out_pad[2]) {
  if (dilation == 0) dilation = 1;
  if (stride == 0) stride = 1;
  int64_t eff = static_cast<int64_t>(ksize - 1) * dilation + 1;
  int64_t out = 0;
  if (type == PadType::SAME)
    out = (static_cast<int64_t>(in) + stride - 1) / stride;
  else if (type == PadType::VALID)
    out = (static_cast<int64_t>(in) + stride - eff) / stride;
  int64_t total = (out - 1) * stride + eff - in;
  if (total < 0) total = 0;
  out_pad[0] = static_cast<uint32_t>(total / 2);
  out_pad[1] = static_cast<uint32_t>(total - out_pad[0]);
}

namespace {

TensorImpl* Impl(const std::shared_ptr<Tensor>& t) {
  return static_cast<TensorImpl*>(t.get());
}

bool IsQuantInt(DataType d) {
  return d == DataType::UINT8 || d == DataType::INT8;
}

// Conv / FC operand pairs this runtime executes. The reference accepts more
// (int16 dynamic fixed point, int4, bf16 ...); those are rejected here.
bool WeightPairSupported(const TensorSpec& in, const TensorSpec& w) {
  DataType a = in.datatype_, b = w.datatype_;
  QuantType qa = in.quantization_.Type(), qb = w.quantization_.Type();
  if (a == DataType::FLOAT32 && b == DataType::FLOAT32) return true;
  if (a == DataType::FLOAT16 && b == DataType::FLOAT16) return true;
  if (qa != QuantType::ASYMMETRIC) return false;
  if (a == DataType::UINT8 && b == DataType::UINT8 && qb == QuantType::ASYMMETRIC) return true;
  if (a == DataType::INT8 && b == DataType::INT8 && qb == QuantType::ASYMMETRIC) return true;
  if (IsQuantInt(a) && b == DataType::INT8 && qb == QuantType::SYMMETRIC_PER_CHANNEL) return true;
  return false;
}

bool BiasScaleConsistent(const TensorSpec& in, const TensorSpec& w,
                         const TensorSpec* bias) {
  // Checked only when input, weight and bias share one quantization kind and
  // input/weight share a data type; mixed combinations pass unchecked.
  const Quantization &qi = in.quantization_, &qw = w.quantization_;
  if (in.datatype_ != w.datatype_ || qi.Type() != qw.Type()) return true;
  if (bias && bias->quantization_.Type() != qi.Type()) return true;
  if (!IsQuantInt(in.datatype_) || qi.Type() != QuantType::ASYMMETRIC) return true;
  if (!bias || bias->quantization_.Scales().empty() ||
      bias->quantization_.Scales()[0] == 0.f)
    return true;
  if (qi.Scales().empty() || qw.Scales().empty()) return true;
  double product = static_cast<double>(qi.Scales()[0]) * static_cast<double>(qw.Scales()[0]);
  double bs = bias->quantization_.Scales()[0];
  double diff = std::fabs(product - bs);
  double tol = std::max(std::min(product, bs) * 1e-5, 1e-8);
  if (diff <= tol) return true;
  VSILOGE("bias scale %g != input scale * weight scale %g", bs, product);
  return false;
}

// A TRANSIENT tensor created without a shape takes the inferred one. A shape
// the caller declared is kept, as ovxlib only infers when the rank is "auto"
// (vsi_nn_op_conv2d.c:253): spatial extents (the first `spatial` dims) may
// differ from the inferred ones - the operator then produces exactly the
// declared window positions, which is what
// depthwiseConv_test.cc:268 (SAME padding, output declared 1x1) relies on -
// while the remaining dims must match.
bool AssignShape(TensorImpl* t, const ShapeType& inferred, const char* what,
                 size_t spatial = 0) {
  if (t->spec_.shape_.empty()) {
    t->spec_.shape_ = inferred;
    return true;
  }
  const ShapeType& have = t->spec_.shape_;
  bool same_rank = have.size() == inferred.size();
  if (same_rank) {
    bool ok = true;
    for (size_t i = 0; i < have.size(); ++i) {
      if (have[i] == inferred[i]) continue;
      if (i < spatial) {
        VSILOGW("%s: declared output dim %zu = %u, inferred %u; keeping the declared one",
                what, i, have[i], inferred[i]);
      } else {
        ok = false;
      }
    }
    if (ok) return true;
  }
  int64_t n_have = 1, n_want = 1;
  for (auto d : have) n_have *= d;
  for (auto d : inferred) n_want *= d;
  if (spatial == 0 && n_have == n_want) return true;  // same data, other view
  VSILOGE("%s: output tensor %u holds %lld elements, operator produces %lld",
          what, t->id_, static_cast<long long>(n_have),
          static_cast<long long>(n_want));
  return false;
}

bool SetupConv(OpImpl* op) {
  if (op->inputs_tensor_.size() < 2 || op->outputs_tensor_.size() != 1) {
    VSILOGE("CONV2D needs {input, weight[, bias]} and one output");
    return false;
  }
  TensorImpl *x = Impl(op->inputs_tensor_[0]), *w = Impl(op->inputs_tensor_[1]);
  TensorImpl* b = op->inputs_tensor_.size() > 2 && !op->inputs_tensor_[2]->IsPlaceHolder()
                      ? Impl(op->inputs_tensor_[2]) : nullptr;
  TensorImpl* y = Impl(op->outputs_tensor_[0]);
  const bool one_d = op->attrs_.conv_1d;
  if (one_d ? (op->layout_ != DataLayout::WCN && op->layout_ != DataLayout::ANY)
            : (op->layout_ != DataLayout::WHCN && op->layout_ != DataLayout::ANY)) {
    VSILOGE("%s", one_d ? "CONV1D: only WCN activations are supported" : "CONV2D: only WHCN activations are supported");
    return false;
  }
  if (one_d ? (x->spec_.shape_.size() != 3 || w->spec_.shape_.size() != 3)
            : (x->spec_.shape_.size() != 4 || w->spec_.shape_.size() != 4)) {
    VSILOGE("%s", one_d ? "CONV1D: input and weight must be 3-D" : "CONV2D: input and weight must be 4-D");
    return false;
  }
  if (!BiasScaleConsistent(x->spec_, w->spec_, b ? &b->spec_ : nullptr)) return false;
  if (!WeightPairSupported(x->spec_, w->spec_)) {
    VSILOGE("Inputs/Outputs data type not support: %s x %s",
            DataTypeName(x->spec_.datatype_), DataTypeName(w->spec_.datatype_));
    return false;
  }
  OpAttrs& a = op->attrs_;
  // Conv1d: {W, C, N} x {Kw, Ic, Oc} is the 2-D operator on {W, 1, C, N} x {Kw, 1, Ic, Oc}; the
  // depthwise weight {Kw, 1, Ic*m} is the 2-D depthwise weight {Kw, 1, Ic*m, 1}
  // (src/tim/vx/internal/src/ops/vsi_nn_op_conv1d.c reshapes the same way)
  ShapeType xs = x->spec_.shape_, ws = w->spec_.shape_;
  if (one_d) {
    xs = {xs[0], 1, xs[1], xs[2]};
    ws = a.multiplier > 0 ? ShapeType{ws[0], 1, ws[2], 1} : ShapeType{ws[0], 1, ws[1], ws[2]};
    if (a.multiplier > 0 && w->spec_.shape_[1] != 1) {
      VSILOGE("CONV1D: depthwise weight must be {Kw, 1, Ic*multiplier}");
      return false;
    }
  }
  for (int i = 0; i < 2; ++i)
    if (a.dilation[i] == 0) a.dilation[i] = 1;
  if (a.pad_type != PadType::AUTO) {
    ComputePaddingPerAxis(xs[0], ws[0], a.stride[0], a.dilation[0], a.pad_type, &a.pad[0]);
    ComputePaddingPerAxis(xs[1], ws[1], a.stride[1], a.dilation[1], a.pad_type, &a.pad[2]);
  }
  a.ksize[0] = ws[0];
  a.ksize[1] = ws[1];
  uint32_t oc;
  if (a.multiplier > 0) {
    oc = xs[2] * a.multiplier;
    if (ws[2] != oc || ws[3] != 1) {
      VSILOGE("depthwise weight must be {Kw, Kh, Ic*multiplier, 1}");
      return false;
    }
  } else if (a.groups > 1) {
    const uint32_t g = static_cast<uint32_t>(a.groups);
    oc = ws[3];
    if (xs[2] % g != 0 || oc % g != 0 || ws[2] != xs[2] / g) {
      VSILOGE("GROUPED_CONV2D: %u groups need input C %u and weight Oc %u divisible and weight Ic %u == C / groups",
              g, xs[2], oc, ws[2]);
      return false;
    }
  } else {
    oc = ws[3];
    if (ws[2] != xs[2]) {
      VSILOGE("CONV2D: weight Ic %u != input C %u", ws[2], xs[2]);
      return false;
    }
  }
  if (b && static_cast<uint32_t>(b->spec_.GetElementNum()) != oc) {
    VSILOGE("CONV2D: bias has %lld elements, expected %u",
            static_cast<long long>(b->spec_.GetElementNum()), oc);
    return false;
  }
  ShapeType out = {
      ComputeFilterSize(xs[0], ws[0], &a.pad[0], a.stride[0], a.dilation[0], RoundType::FLOOR),
      ComputeFilterSize(xs[1], ws[1], &a.pad[2], a.stride[1], a.dilation[1], RoundType::FLOOR),
      oc, xs[3]};
  // A declared output that is longer than the pads make it reads padding behind the input's end: the reference
  // hands the declared size to the driver as it is (its GroupedConv1d "PaddingTest": a two-column input under a
  // three-tap VALID kernel with two declared output columns, golden = the window sliding over trailing zeros).
  {
    const ShapeType& have = y->spec_.shape_;
    const size_t rank = one_d ? 3 : 4;
    if (have.size() == rank) {
      const uint32_t declared[2] = {have[0], one_d ? 1u : have[1]};
      for (int i = 0; i < 2; ++i) {
        if (declared[i] <= out[i]) continue;
        const uint64_t reach = static_cast<uint64_t>(declared[i] - 1) * a.stride[i] + static_cast<uint64_t>(ws[i] - 1) * a.dilation[i] + 1;
        const uint64_t span = static_cast<uint64_t>(xs[i]) + a.pad[2 * i] + a.pad[2 * i + 1];
        if (reach > span) a.pad[2 * i + 1] += static_cast<uint32_t>(reach - span);
        VSILOGW("%s: declared output dim %d = %u, the pads give %u; the last windows read padding behind the input",
                one_d ? "CONV1D" : "CONV2D", i, declared[i], out[i]);
        out[i] = declared[i];
      }
    }
  }
  if (out[0] == 0 || out[1] == 0) {
    VSILOGE("CONV2D: empty output");
    return false;
  }
  if (one_d) return AssignShape(y, ShapeType{out[0], out[2], out[3]}, "CONV1D", 1);
  return AssignShape(y, out, "CONV2D", 2);
}

// reference: src/tim/vx/internal/src/ops/vsi_nn_op_deconvolution.c:217-218, 456-497
bool SetupDeconv(OpImpl* op) {
  if (op->inputs_tensor_.size() < 2 || op->outputs_tensor_.size() != 1) {
    VSILOGE("DECONV2D needs {input, weight[, bias]} and one output");
    return false;
  }
  TensorImpl *x = Impl(op->inputs_tensor_[0]), *w = Impl(op->inputs_tensor_[1]);
  TensorImpl* b = op->inputs_tensor_.size() > 2 && !op->inputs_tensor_[2]->IsPlaceHolder()
                      ? Impl(op->inputs_tensor_[2]) : nullptr;
  TensorImpl* y = Impl(op->outputs_tensor_[0]);
  const bool one_d = op->attrs_.conv_1d;
  if (op->layout_ != DataLayout::WHCN && op->layout_ != DataLayout::ANY && !(one_d && op->layout_ == DataLayout::WCN)) {
    VSILOGE("DECONV2D: only WHCN (1-D: WCN) activations are supported");
    return false;
  }
  // DeConv1d: {W, C, N} x {Kw, Ic, Oc} is the 2-D operator on {W, 1, C, N} x {Kw, 1, Ic, Oc}
  // (src/tim/vx/internal/src/ops/vsi_nn_op_deconvolution1d.c:62-72 reshapes the weight the same way)
  ShapeType xs = x->spec_.shape_, ws = w->spec_.shape_;
  if (one_d ? (xs.size() != 3 || ws.size() != 3) : (xs.size() != 4 || ws.size() != 4)) {
    VSILOGE("%s", one_d ? "DECONV1D: input and weight must be 3-D" : "DECONV2D: input and weight must be 4-D");
    return false;
  }
  if (one_d) {
    xs = {xs[0], 1, xs[1], xs[2]};
    ws = {ws[0], 1, ws[1], ws[2]};
  }
  if (!BiasScaleConsistent(x->spec_, w->spec_, b ? &b->spec_ : nullptr)) return false;
  if (!WeightPairSupported(x->spec_, w->spec_)) {
    VSILOGE("Inputs/Outputs data type not support: %s x %s", DataTypeName(x->spec_.datatype_),
            DataTypeName(w->spec_.datatype_));
    return false;
  }
  OpAttrs& a = op->attrs_;
  if (a.groups == 0) a.groups = 1;
  const uint32_t g = static_cast<uint32_t>(a.groups);
  uint32_t oc;
  if (g > 1 && g == xs[2] && ws[3] == 1) {
    oc = ws[2];  // depthwise form {Kw, Kh, C, 1}
    if (oc != xs[2]) {
      VSILOGE("DECONV2D: depthwise weight must be {Kw, Kh, C, 1} with C = input channels %u", xs[2]);
      return false;
    }
  } else {
    oc = ws[3];
    if (xs[2] % g != 0 || oc % g != 0 || ws[2] != xs[2] / g) {
      VSILOGE("DECONV2D: weight Ic %u != input C %u / group %u", ws[2], xs[2], g);
      return false;
    }
  }
  if (b && static_cast<uint32_t>(b->spec_.GetElementNum()) != oc) {
    VSILOGE("DECONV2D: bias has %lld elements, expected %u", static_cast<long long>(b->spec_.GetElementNum()), oc);
    return false;
  }
  a.ksize[0] = ws[0];
  a.ksize[1] = ws[1];
  const int64_t ow = (static_cast<int64_t>(xs[0]) - 1) * a.stride[0] + ws[0] - a.pad[0] - a.pad[1] + a.output_padding[0];
  const int64_t oh = (static_cast<int64_t>(xs[1]) - 1) * a.stride[1] + ws[1] - a.pad[2] - a.pad[3] + a.output_padding[1];
  if (ow <= 0 || oh <= 0 || !a.stride[0] || !a.stride[1]) {
    VSILOGE("DECONV2D: empty output");
    return false;
  }
  if (one_d) return AssignShape(y, ShapeType{static_cast<uint32_t>(ow), oc, xs[3]}, "DECONV1D", 1);
  return AssignShape(y, ShapeType{static_cast<uint32_t>(ow), static_cast<uint32_t>(oh), oc, xs[3]}, "DECONV2D", 2);
}

bool SetupFcl(OpImpl* op) {
  if (op->inputs_tensor_.size() < 2 || op->outputs_tensor_.size() != 1) {
    VSILOGE("FCL needs {input, weight[, bias]} and one output");
    return false;
  }
  TensorImpl *x = Impl(op->inputs_tensor_[0]), *w = Impl(op->inputs_tensor_[1]);
  TensorImpl* b = op->inputs_tensor_.size() > 2 && !op->inputs_tensor_[2]->IsPlaceHolder()
                      ? Impl(op->inputs_tensor_[2]) : nullptr;
  TensorImpl* y = Impl(op->outputs_tensor_[0]);
  if (!BiasScaleConsistent(x->spec_, w->spec_, b ? &b->spec_ : nullptr)) return false;
  if (!WeightPairSupported(x->spec_, w->spec_)) {
    VSILOGE("FCL: unsupported operand types %s x %s",
            DataTypeName(x->spec_.datatype_), DataTypeName(w->spec_.datatype_));
    return false;
  }
  const OpAttrs& a = op->attrs_;
  const ShapeType& xs = x->spec_.shape_;
  if (a.axis >= xs.size()) {
    VSILOGE("FCL: axis %u out of range", a.axis);
    return false;
  }
  uint64_t k = 1, m = 1;
  for (uint32_t i = 0; i <= a.axis; ++i) k *= xs[i];
  for (size_t i = a.axis + 1; i < xs.size(); ++i) m *= xs[i];
  uint32_t n = w->spec_.shape_.back();
  if (static_cast<uint64_t>(w->spec_.GetElementNum()) != k * n) {
    VSILOGE("FCL: weight holds %lld elements, expected K*N = %llu",
            static_cast<long long>(w->spec_.GetElementNum()),
            static_cast<unsigned long long>(k * n));
    return false;
  }
  if (b && static_cast<uint32_t>(b->spec_.GetElementNum()) != n) {
    VSILOGE("FCL: bias size mismatch");
    return false;
  }
  ShapeType out = {a.weights ? a.weights : n};
  for (size_t i = a.axis + 1; i < xs.size(); ++i) out.push_back(xs[i]);
  if (out.size() == 1) out.push_back(static_cast<uint32_t>(m));
  if (out[0] != n) {
    VSILOGE("FCL: weights attribute %u != weight rows %u", out[0], n);
    return false;
  }
  return AssignShape(y, out, "FCL");
}

bool SetupPool(OpImpl* op) {
  if (op->inputs_tensor_.size() != 1 || op->outputs_tensor_.size() != 1) {
    VSILOGE("POOL needs one input and one output");
    return false;
  }
  TensorImpl *x = Impl(op->inputs_tensor_[0]), *y = Impl(op->outputs_tensor_[0]);
  const TensorSpec &xi = x->spec_, &yo = y->spec_;
  bool ok = (xi.datatype_ == yo.datatype_) &&
            (xi.datatype_ == DataType::FLOAT32 || xi.datatype_ == DataType::FLOAT16 ||
             (IsQuantInt(xi.datatype_) &&
              xi.quantization_.Type() == QuantType::ASYMMETRIC &&
              yo.quantization_.Type() == QuantType::ASYMMETRIC));
  if (!ok) {
    VSILOGE("Inputs/Outputs data type not support: %s -> %s",
            DataTypeName(xi.datatype_), DataTypeName(yo.datatype_));
    return false;
  }
  OpAttrs& a = op->attrs_;
  const ShapeType& xs = xi.shape_;
  size_t want_rank = a.pool_1d ? 3 : 4;
  if (xs.size() != want_rank) {
    VSILOGE("POOL: input must be %zu-D", want_rank);
    return false;
  }
  uint32_t in_w = xs[0], in_h = a.pool_1d ? 1 : xs[1];
  if (a.pad_type != PadType::AUTO) {
    ComputePaddingPerAxis(in_w, a.ksize[0], a.stride[0], 1, a.pad_type, &a.pad[0]);
    if (!a.pool_1d)
      ComputePaddingPerAxis(in_h, a.ksize[1], a.stride[1], 1, a.pad_type, &a.pad[2]);
  }
  ShapeType out;
  out.push_back(ComputeFilterSize(in_w, a.ksize[0], &a.pad[0], a.stride[0], 1, a.round_type));
  if (!a.pool_1d)
    out.push_back(ComputeFilterSize(in_h, a.ksize[1], &a.pad[2], a.stride[1], 1, a.round_type));
  for (size_t i = a.pool_1d ? 1 : 2; i < xs.size(); ++i) out.push_back(xs[i]);
  if (out[0] == 0 || (!a.pool_1d && out[1] == 0)) {
    VSILOGE("POOL: empty output");
    return false;
  }
  return AssignShape(y, out, "POOL", a.pool_1d ? 1 : 2);
}

bool SetupSameShape(OpImpl* op, const char* what, size_t n_in) {
  if (op->inputs_tensor_.size() != n_in || op->outputs_tensor_.size() != 1) {
    VSILOGE("%s: wrong operand count", what);
    return false;
  }
  TensorImpl* x = Impl(op->inputs_tensor_[0]);
  if (n_in == 2) {
    TensorImpl* x2 = Impl(op->inputs_tensor_[1]);
    if (x2->spec_.shape_ != x->spec_.shape_) {
      VSILOGE("%s: broadcasting is not supported", what);
      return false;
    }
  }
  return AssignShape(Impl(op->outputs_tensor_[0]), x->spec_.shape_, what);
}

bool SetupReshape(OpImpl* op) {
  if (op->inputs_tensor_.size() != 1 || op->outputs_tensor_.size() != 1) return false;
  return AssignShape(Impl(op->outputs_tensor_[0]), op->attrs_.new_shape, "RESHAPE");
}

// reference: src/tim/vx/internal/src/ops/vsi_nn_op_permute.c:219-230 (out.size[i] = in.size[perm[i]])
bool SetupTranspose(OpImpl* op) {
  if (op->inputs_tensor_.size() != 1 || op->outputs_tensor_.size() != 1) {
    VSILOGE("TRANSPOSE: wrong operand count");
    return false;
  }
  TensorImpl* x = Impl(op->inputs_tensor_[0]);
  TensorImpl* y = Impl(op->outputs_tensor_[0]);
  const ShapeType& xs = x->spec_.shape_;
  const std::vector<uint32_t>& perm = op->attrs_.perm;
  if (perm.size() != xs.size() || xs.empty() || xs.size() > 6) {
    VSILOGE("TRANSPOSE: perm of %zu entries for a rank-%zu input (ranks 1..6)", perm.size(), xs.size());
    return false;
  }
  std::vector<bool> seen(xs.size(), false);
  ShapeType out(xs.size());
  for (size_t i = 0; i < perm.size(); ++i) {
    if (perm[i] >= xs.size() || seen[perm[i]]) {
      VSILOGE("TRANSPOSE: perm is not a permutation of the input's dimensions");
      return false;
    }
    seen[perm[i]] = true;
    out[i] = xs[perm[i]];
  }
  if (y->spec_.datatype_ != x->spec_.datatype_) {
    VSILOGE("TRANSPOSE: output type differs from the input's");
    return false;
  }
  return AssignShape(y, out, "TRANSPOSE");
}

}  // namespace

bool GraphImpl::VerifyAndInfer() {
  // ---- execution order: an operator is ready once all non-constant inputs
  // that have a producer have been produced ---------------------------------
  sorted_ops_.clear();
  std::set<Tensor*> ready;
  std::vector<Operation*> pending;
  for (auto& op : op_vector_) pending.push_back(op.get());
  auto produced_elsewhere = [&](Tensor* t) {
    for (auto& op : op_vector_)
      for (auto& o : op->impl()->outputs_tensor_)
        if (o.get() == t) return true;
    return false;
  };
  while (!pending.empty()) {
    bool progressed = false;
    for (auto it = pending.begin(); it != pending.end();) {
      OpImpl* im = (*it)->impl().get();
      bool ok = true;
      for (auto& t : im->inputs_tensor_) {
        if (t->IsPlaceHolder() || t->IsConstTensor()) continue;
        if (ready.count(t.get())) continue;
        if (produced_elsewhere(t.get())) { ok = false; break; }
      }
      if (ok) {
        sorted_ops_.push_back(*it);
        for (auto& o : im->outputs_tensor_) ready.insert(o.get());
        it = pending.erase(it);
        progressed = true;
      } else {
        ++it;
      }
    }
    if (!progressed) {
      VSILOGE("graph has a cycle");
      return false;
    }
  }

  // ---- per-operator check + setup ------------------------------------------
  for (Operation* op : sorted_ops_) {
    OpImpl* im = op->impl().get();
    for (auto& t : im->inputs_tensor_) {
      if (t->IsPlaceHolder()) continue;
      if (t->GetShape().empty()) {
        VSILOGE("%s (uid %u): input tensor %u has no shape", OpKindName(im->kind_),
                im->uid_, t->GetId());
        return false;
      }
    }
    bool ok = false;
    switch (im->kind_) {
      case OpKind::CONV2D: ok = SetupConv(im); break;
      case OpKind::FCL: ok = SetupFcl(im); break;
      case OpKind::POOL: ok = SetupPool(im); break;
      case OpKind::RELU: ok = SetupSameShape(im, "RELU", 1); break;
      case OpKind::RELU6: ok = SetupSameShape(im, "RELU6", 1); break;
      case OpKind::ADD: ok = SetupSameShape(im, "ADD", 2); break;
      case OpKind::SOFTMAX: ok = SetupSameShape(im, "SOFTMAX", 1); break;
      case OpKind::RESHAPE: ok = SetupReshape(im); break;
      case OpKind::TRANSPOSE: ok = SetupTranspose(im); break;
      case OpKind::DATACONVERT: ok = SetupSameShape(im, "DATACONVERT", 1); break;
      case OpKind::DECONV2D: ok = SetupDeconv(im); break;
    }
    if (!ok) {
      VSILOGE("setup of %s (uid %u) failed", OpKindName(im->kind_), im->uid_);
      return false;
    }
  }
  return true;
}

}  // namespace vx
}  // namespace tim
