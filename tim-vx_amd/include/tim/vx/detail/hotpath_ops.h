// Operator classes of the quantized-convolution path and the glue operators
// the LeNet / MobileNet graphs need around it. Constructor signatures and
// protected data members follow the reference headers cited per class.
#pragma once

#include "tim/vx/detail/core_api.h"

namespace tim {
namespace vx {
namespace ops {

// Dense, 1x1 and depthwise (multiplier > 0) 2-D convolution.
// reference: include/tim/vx/ops/conv2d.h:59-104, src/tim/vx/ops/conv2d.cc:34-82
// Inputs: activation WHCN, weight WHIcOc (depthwise: {Kw, Kh, Ic*multiplier, 1}),
// optional bias {Oc}. `weights` and `ksize` are stored, never forwarded; the
// kernel size always comes from the weight tensor.
class Conv2d : public BuiltinOp {
 public:
  Conv2d(Graph* graph, PadType padding, const std::array<uint32_t, 2>& stride,
         const std::array<uint32_t, 2>& dilation, int32_t multiplier = 0,
         DataLayout input_layout = DataLayout::WHCN,
         DataLayout kernel_layout = DataLayout::WHIcOc);
  Conv2d(Graph* graph, const std::array<uint32_t, 4> pad,
         const std::array<uint32_t, 2>& stride,
         const std::array<uint32_t, 2>& dilation, int32_t multiplier = 0,
         DataLayout input_layout = DataLayout::WHCN,
         DataLayout kernel_layout = DataLayout::WHIcOc);
  Conv2d(Graph* graph, int32_t weights, PadType padding,
         const std::array<uint32_t, 2>& ksize,
         const std::array<uint32_t, 2>& stride,
         const std::array<uint32_t, 2>& dilation, int32_t multiplier = 0,
         DataLayout input_layout = DataLayout::WHCN,
         DataLayout kernel_layout = DataLayout::WHIcOc);
  Conv2d(Graph* graph, int32_t weights, PadType padding,
         const std::array<uint32_t, 2>& ksize,
         const std::array<uint32_t, 2>& stride,
         const std::array<uint32_t, 2>& dilation,
         const std::array<uint32_t, 4>& pad, int32_t multiplier = 0,
         DataLayout input_layout = DataLayout::WHCN,
         DataLayout kernel_layout = DataLayout::WHIcOc);

  DataLayout KernelDataLayout() { return kernel_layout_; }
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;
  const std::vector<std::shared_ptr<Tensor>> ConstantInputsTensor()
      const override;

 protected:
  const uint32_t weights_;
  const PadType padding_;
  const std::array<uint32_t, 2> ksize_;
  const std::array<uint32_t, 2> stride_;
  const std::array<uint32_t, 2> dilation_;
  const std::array<uint32_t, 4> pad_;  // left, right, top, bottom
  const int32_t multiplier_;
  const DataLayout kernel_layout_;

 private:
  void OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor,
                           int32_t input_idx) override;
};

// 1-D convolution: activation {W, C, N}, weight {Kw, Ic, Oc} (depthwise: {Kw, 1, Ic*multiplier}),
// optional bias {Oc}, output {W', Oc, N} - the 2-D operator on rows of height one.
// reference: include/tim/vx/ops/conv1d.h:35-70, src/tim/vx/ops/conv1d.cc:34-84
class Conv1d : public BuiltinOp {
 public:
  Conv1d(Graph* graph, PadType padding, uint32_t stride, uint32_t dilation, int32_t multiplier = 0,
         DataLayout input_layout = DataLayout::WCN, DataLayout kernel_layout = DataLayout::WIcOc);
  Conv1d(Graph* graph, const std::array<uint32_t, 2>& pad, uint32_t stride, uint32_t dilation,
         int32_t multiplier = 0, DataLayout input_layout = DataLayout::WCN,
         DataLayout kernel_layout = DataLayout::WIcOc);
  Conv1d(Graph* graph, int32_t weights, PadType padding, uint32_t ksize, uint32_t stride,
         uint32_t dilation, int32_t multiplier = 0, DataLayout input_layout = DataLayout::WCN,
         DataLayout kernel_layout = DataLayout::WIcOc);
  Conv1d(Graph* graph, int32_t weights, PadType padding, uint32_t ksize, uint32_t stride,
         uint32_t dilation, const std::array<uint32_t, 2>& pad, int32_t multiplier = 0,
         DataLayout input_layout = DataLayout::WCN, DataLayout kernel_layout = DataLayout::WIcOc);

  DataLayout KernelDataLayout() { return kernel_layout_; }
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;

 protected:
  const uint32_t weights_;
  const PadType padding_;
  const uint32_t ksize_;
  const uint32_t stride_;
  const uint32_t dilation_;
  const std::array<uint32_t, 2> pad_;
  const int32_t multiplier_;
  const DataLayout kernel_layout_;

 private:
  void OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor,
                           int32_t input_idx) override;
};

// Grouped 1-D convolution: the grouped operator on {W, C, N} tensors, weight {Kw, Ic / groups, Oc}.
// reference: include/tim/vx/ops/groupedconv1d.h:56-80, src/tim/vx/ops/groupedconv1d.cc:34-66
class GroupedConv1d : public BuiltinOp {
 public:
  GroupedConv1d(Graph* graph, PadType padding, std::array<uint32_t, 2> pad, uint32_t stride, uint32_t dilation,
                uint32_t group, DataLayout input_layout = DataLayout::WCN,
                DataLayout kernel_layout = DataLayout::WIcOc);
  GroupedConv1d(Graph* graph, PadType padding, const uint32_t stride, const uint32_t dilation, uint32_t group,
                DataLayout input_layout = DataLayout::WCN, DataLayout kernel_layout = DataLayout::WIcOc);

  DataLayout KernelDataLayout() { return kernel_layout_; }
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;

 protected:
  const PadType padding_;
  const std::array<uint32_t, 2> pad_;
  const uint32_t stride_;
  const uint32_t dilation_;
  const uint32_t group_;
  const DataLayout kernel_layout_;

 private:
  void OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor,
                           int32_t input_idx) override;
};

// Grouped 2-D convolution: output channel block j (Oc / groups channels) reads input
// channel block j (Ic / groups channels); weight {Kw, Kh, Ic / groups, Oc}, optional bias {Oc}.
// reference: include/tim/vx/ops/groupedconv2d.h:56-82, src/tim/vx/ops/groupedconv2d.cc
class GroupedConv2d : public BuiltinOp {
 public:
  GroupedConv2d(Graph* graph, PadType padding, const std::array<uint32_t, 2>& strides,
                const std::array<uint32_t, 2>& dilation, int32_t grouped_number,
                DataLayout input_layout = DataLayout::WHCN,
                DataLayout kernel_layout = DataLayout::WHIcOc);
  GroupedConv2d(Graph* graph, const std::array<uint32_t, 4>& pad,
                const std::array<uint32_t, 2>& strides,
                const std::array<uint32_t, 2>& dilation, int32_t group_number,
                DataLayout input_layout = DataLayout::WHCN,
                DataLayout kernel_layout = DataLayout::WHIcOc);

  DataLayout KernelDataLayout() { return kernel_layout_; }
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;

 protected:
  const PadType padding_;
  const std::array<uint32_t, 2> strides_;
  const std::array<uint32_t, 2> dilation_;
  const std::array<uint32_t, 4> pad_;
  const int32_t group_number_;
  const DataLayout kernel_layout_;

 private:
  void OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor,
                           int32_t input_idx) override;
};

// out[n, m] = sum_k in[k, m] * w[k, n] + bias[n]; input dims 0..axis flatten
// into k. reference: include/tim/vx/ops/fullyconnected.h:42-56
class FullyConnected : public BuiltinOp {
 public:
  FullyConnected(Graph* graph, uint32_t axis);
  FullyConnected(Graph* graph, uint32_t axis, uint32_t weights);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;

 protected:
  uint32_t axis_;
  uint32_t weights_;

 private:
  void OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor,
                           int32_t input_idx) override;
};

// MAX / AVG / AVG_ANDROID / L2 window reduction.
// reference: include/tim/vx/ops/pool2d.h:67-108, src/tim/vx/ops/pool2d.cc:34-115
class Pool2d : public BuiltinOp {
 public:
  Pool2d(Graph* graph, PoolType type, PadType padding,
         const std::array<uint32_t, 2>& ksize,
         const std::array<uint32_t, 2>& stride,
         RoundType round_type = RoundType::FLOOR,
         DataLayout layout = DataLayout::WHCN);
  Pool2d(Graph* graph, PoolType type, const std::array<uint32_t, 4>& pad,
         const std::array<uint32_t, 2>& ksize,
         const std::array<uint32_t, 2>& stride,
         RoundType round_type = RoundType::FLOOR,
         DataLayout layout = DataLayout::WHCN);
  // global pooling: window = stride = input_size
  Pool2d(Graph* graph, PoolType type, const std::array<uint32_t, 2>& input_size,
         RoundType round_type = RoundType::FLOOR,
         DataLayout layout = DataLayout::WHCN);
  // adaptive pooling: stride = floor(in / out), window = in - (out - 1) * stride
  Pool2d(Graph* graph, PoolType type, const std::array<uint32_t, 2>& input_size,
         const std::array<uint32_t, 2>& output_size,
         RoundType round_type = RoundType::FLOOR,
         DataLayout layout = DataLayout::WHCN);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;
  void Init();

 protected:
  const PoolType type_;
  const PadType padding_;
  std::array<uint32_t, 2> ksize_;
  std::array<uint32_t, 2> stride_;
  const RoundType round_type_;
  const std::array<uint32_t, 4> pad_;
};

// 1-D form of Pool2d over {W, C, N}; executed as a Pool2d with H = 1.
// reference: include/tim/vx/ops/pool1d.h
class Pool1d : public BuiltinOp {
 public:
  Pool1d(Graph* graph, PoolType type, PadType padding, uint32_t ksize,
         uint32_t stride, RoundType round_type = RoundType::FLOOR,
         DataLayout layout = DataLayout::WCN);
  Pool1d(Graph* graph, PoolType type, const std::array<uint32_t, 2>& pad,
         uint32_t ksize, uint32_t stride,
         RoundType round_type = RoundType::FLOOR,
         DataLayout layout = DataLayout::WCN);
  Pool1d(Graph* graph, PoolType type, uint32_t input_size,
         RoundType round_type = RoundType::FLOOR,
         DataLayout layout = DataLayout::WCN);
  Pool1d(Graph* graph, PoolType type, uint32_t input_size, uint32_t output_size,
         RoundType round_type = RoundType::FLOOR,
         DataLayout layout = DataLayout::WCN);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;
  void Init();

 protected:
  const PoolType type_;
  const PadType padding_;
  uint32_t ksize_;
  uint32_t stride_;
  const RoundType round_type_;
  const std::array<uint32_t, 2> pad_;
};

// reference: include/tim/vx/ops/activations.h (Relu, Relu6 only)
class Relu : public BuiltinOp {
 public:
  Relu(Graph* graph);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;
};
class Relu6 : public BuiltinOp {
 public:
  Relu6(Graph* graph);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;
};

// reference: include/tim/vx/ops/elementwise.h (Add only)
class Add : public BuiltinOp {
 public:
  Add(Graph* graph);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;
};

// reference: include/tim/vx/ops/softmax.h
class Softmax : public BuiltinOp {
 public:
  Softmax(Graph* graph, float beta, int32_t axis);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;

 protected:
  float beta_;
  int32_t axis_;
};

// reference: include/tim/vx/ops/reshape.h
class Reshape : public BuiltinOp {
 public:
  Reshape(Graph* graph, const std::vector<uint32_t>& target_shape);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;

 protected:
  std::vector<uint32_t> size_;
};

// reference: include/tim/vx/ops/deconv.h:54-86
// The transpose of Conv2d: weights {Kw, Kh, Ic, Oc}, or {Kw, Kh, C, 1} for the depthwise form
// (group == channel count); out = (in - 1) * stride + k - pads + output_padding.
class DeConv2d : public BuiltinOp {
 public:
  DeConv2d(Graph* graph, int32_t oc_count_, PadType pad_type,
           const std::array<uint32_t, 2>& ksize,
           const std::array<uint32_t, 2>& stride,
           const std::array<uint32_t, 2>& output_padding,
           DataLayout input_layout = DataLayout::WHCN,
           DataLayout kernel_layout = DataLayout::WHIcOc);
  DeConv2d(Graph* graph, int32_t oc_count_, PadType pad_type,
           const std::array<uint32_t, 2>& ksize,
           const std::array<uint32_t, 2>& stride,
           const std::array<uint32_t, 2>& output_padding,
           const std::array<uint32_t, 4>& pad, const uint32_t group = 1,
           DataLayout input_layout = DataLayout::WHCN,
           DataLayout kernel_layout = DataLayout::WHIcOc);
  DataLayout KernelDataLayout() { return kernel_layout_; }
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;

 protected:
  void OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor, int32_t input_idx) override;
  const uint32_t oc_count_;
  const PadType pad_type_;
  const std::array<uint32_t, 2> ksize_;
  const std::array<uint32_t, 2> stride_;
  const std::array<uint32_t, 2> output_padding_;
  const std::array<uint32_t, 4> pad_;
  const uint32_t group_;
  const DataLayout kernel_layout_;
};

// Transposed 1-D convolution: DeConv2d on {W, C, N} tensors, weight {Kw, Ic / groups, Oc} (the 2-D operator on rows
// of height one, as ovxlib reshapes it: src/tim/vx/internal/src/ops/vsi_nn_op_deconvolution1d.c:62-72).
// reference: include/tim/vx/ops/deconv1d.h:53-90, src/tim/vx/ops/deconv1d.cc:36-98
class DeConv1d : public BuiltinOp {
 public:
  DeConv1d(Graph* graph, PadType pad_type, uint32_t stride, uint32_t output_padding, uint32_t group = 1,
           DataLayout input_layout = DataLayout::WHCN, DataLayout kernel_layout = DataLayout::WHIcOc);
  DeConv1d(Graph* graph, const std::array<uint32_t, 2>& pad, uint32_t stride, uint32_t output_padding,
           uint32_t group = 1, DataLayout input_layout = DataLayout::WHCN,
           DataLayout kernel_layout = DataLayout::WHIcOc);
  DeConv1d(Graph* graph, int32_t oc_count_, PadType pad_type, uint32_t ksize, uint32_t stride,
           uint32_t output_padding);
  DeConv1d(Graph* graph, int32_t oc_count_, PadType pad_type, uint32_t ksize, uint32_t stride,
           uint32_t output_padding, const std::array<uint32_t, 2>& pad, uint32_t group = 1);
  DeConv1d(Graph* graph, PadType pad_type, uint32_t stride, uint32_t output_padding,
           const std::array<uint32_t, 2>& pad, uint32_t group, DataLayout input_layout,
           DataLayout kernel_layout);

  DataLayout KernelDataLayout() { return kernel_layout_; }
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;

 protected:
  void OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor, int32_t input_idx) override;
  const uint32_t oc_count_;
  const PadType pad_type_;
  const uint32_t ksize_;
  const uint32_t stride_;
  const uint32_t output_padding_;
  const std::array<uint32_t, 2> pad_;
  const uint32_t group_;
  const DataLayout kernel_layout_;
};

// reference: include/tim/vx/ops/simple_operations.h:118 (DataConvert only)
// Converts between tensor types and quantizations: quantize, dequantize, requantize.
class DataConvert : public BuiltinOp {
 public:
  DataConvert(Graph* graph);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;
};

// reference: include/tim/vx/ops/transpose.h
// Output dimension i is input dimension perm[i], dimension 0 fastest.
class Transpose : public BuiltinOp {
 public:
  Transpose(Graph* graph, const std::vector<uint32_t>& perm);
  std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const override;

 protected:
  std::vector<uint32_t> perm_;
};

}  // namespace ops
}  // namespace vx
}  // namespace tim
