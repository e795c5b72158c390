// Host-side probe of the tim::vx runtime for the CPU test tier: the front end, the compile passes
// (ordering, verification, shape inference) and layout inference, linked with an executor that does
// nothing, so that Compile() succeeds without a GPU. Builds a few graphs and prints, per graph, the
// operators in execution order with the shapes inferred for their outputs. tests/test_host_runtime.py
// compiles it and checks the output. Nothing here computes tensor values.
#include <cstdio>
#include <string>

#include "runtime.h"
#include "tim/transform/layout_inference.h"
#include "tim/vx/context.h"
#include "tim/vx/graph.h"
#include "tim/vx/ops.h"

using namespace tim::vx;

namespace {
class NoopExecutor : public Executor {
 public:
  bool Realize(GraphImpl*) override { return true; }
  bool Execute(GraphImpl* graph) override {
    for (auto& t : graph->outputs_tensor_) static_cast<TensorImpl*>(t.get())->EnsureHostBuffer();
    return true;
  }
};

void Dump(const char* name, const std::shared_ptr<Graph>& graph, bool compiled) {
  std::printf("graph %s compile=%d\n", name, compiled ? 1 : 0);
  if (!compiled) return;
  auto* g = static_cast<GraphImpl*>(graph.get());
  for (Operation* op : g->sorted_ops_) {
    OpImpl* im = op->impl().get();
    std::printf("  %s", OpKindName(im->kind_));
    if (im->kind_ == OpKind::TRANSPOSE) {
      std::printf(" perm");
      for (auto p : im->attrs_.perm) std::printf(" %u", p);
    }
    if (im->kind_ == OpKind::SOFTMAX) std::printf(" axis %d", im->attrs_.sm_axis);
    if (im->kind_ == OpKind::CONV2D || im->kind_ == OpKind::POOL || im->kind_ == OpKind::DECONV2D)
      std::printf(" pad %u %u %u %u", im->attrs_.pad[0], im->attrs_.pad[1], im->attrs_.pad[2], im->attrs_.pad[3]);
    std::printf(" ->");
    for (auto d : im->outputs_tensor_[0]->GetShape()) std::printf(" %u", d);
    std::printf("\n");
  }
}

TensorSpec U8(const ShapeType& s, TensorAttribute a, float scale = 0.5f, int32_t zp = 128) {
  return TensorSpec(DataType::UINT8, s, a, Quantization(QuantType::ASYMMETRIC, scale, zp));
}
TensorSpec I32(const ShapeType& s, float scale) {
  return TensorSpec(DataType::INT32, s, TensorAttribute::CONSTANT, Quantization(QuantType::ASYMMETRIC, scale, 0));
}

// An NHWC classifier head: CWHN conv 3x3 SAME + Relu6 -> CWHN max pool 2x2/2 -> Reshape -> FullyConnected -> Softmax,
// TRANSIENT tensors declared without shapes.
void NhwcNet(const std::shared_ptr<Context>& ctx_in) {
  auto ctx = ctx_in;
  auto g = ctx->CreateGraph();
  std::vector<uint8_t> w(8 * 3 * 3 * 16, 130), fw(16 * 6 * 5 * 10, 127);
  std::vector<int32_t> b(16, 1), fb(10, 2);
  auto x = g->CreateTensor(U8({8, 12, 10, 2}, TensorAttribute::INPUT));
  auto wt = g->CreateTensor(U8({8, 3, 3, 16}, TensorAttribute::CONSTANT, 0.25f, 120), w.data());
  auto bt = g->CreateTensor(I32({16}, 0.125f), b.data());
  auto t0 = g->CreateTensor(U8({}, TensorAttribute::TRANSIENT, 2.f, 0));
  auto t1 = g->CreateTensor(U8({}, TensorAttribute::TRANSIENT, 2.f, 0));
  auto t2 = g->CreateTensor(U8({}, TensorAttribute::TRANSIENT, 2.f, 0));
  auto t3 = g->CreateTensor(U8({}, TensorAttribute::TRANSIENT, 2.f, 0));
  auto fwt = g->CreateTensor(U8({16 * 6 * 5, 10}, TensorAttribute::CONSTANT, 0.01f, 128), fw.data());
  auto fbt = g->CreateTensor(I32({10}, 0.02f), fb.data());
  auto t4 = g->CreateTensor(U8({}, TensorAttribute::TRANSIENT, 1.f, 128));
  auto y = g->CreateTensor(TensorSpec(DataType::FLOAT32, {10, 2}, TensorAttribute::OUTPUT));
  g->CreateOperation<ops::Conv2d>(16, PadType::SAME, std::array<uint32_t, 2>{3, 3}, std::array<uint32_t, 2>{1, 1},
                                  std::array<uint32_t, 2>{1, 1}, std::array<uint32_t, 4>{0, 0, 0, 0}, 0,
                                  DataLayout::CWHN, DataLayout::IcWHOc)
      ->BindInputs({x, wt, bt}).BindOutputs({t0});
  g->CreateOperation<ops::Relu6>()->BindInputs({t0}).BindOutputs({t1});
  g->CreateOperation<ops::Pool2d>(PoolType::MAX, PadType::VALID, std::array<uint32_t, 2>{2, 2},
                                  std::array<uint32_t, 2>{2, 2}, RoundType::FLOOR, DataLayout::CWHN)
      ->BindInputs({t1}).BindOutputs({t2});
  g->CreateOperation<ops::Reshape>(std::vector<uint32_t>{16 * 6 * 5, 2})->BindInputs({t2}).BindOutputs({t3});
  g->CreateOperation<ops::FullyConnected>(0, 10)->BindInputs({t3, fwt, fbt}).BindOutputs({t4});
  g->CreateOperation<ops::Softmax>(1.0f, 0)->BindInputs({t4}).BindOutputs({y});
  auto r = tim::transform::LayoutInference(g, ctx);
  const bool ok = r.first->Compile();
  Dump("nhwc_net", r.first, ok);
  std::printf("  io_map %zu input_shape", r.second.size());
  for (auto d : r.second[x]->GetShape()) std::printf(" %u", d);
  std::printf(" output_shape");
  for (auto d : r.second[y]->GetShape()) std::printf(" %u", d);
  std::printf("\n");
  // the source graph itself is not runnable: its operators are tagged CWHN
  Dump("nhwc_net_source", g, g->Compile());
}

// Softmax over the channels of a CWHN tensor that sits between two CWHN poolings: the axis follows the layout.
void SoftmaxAxis(const std::shared_ptr<Context>& ctx_in) {
  auto ctx = ctx_in;
  auto g = ctx->CreateGraph();
  auto x = g->CreateTensor(TensorSpec(DataType::FLOAT32, {6, 8, 8, 1}, TensorAttribute::INPUT));
  auto t0 = g->CreateTensor(TensorSpec(DataType::FLOAT32, {}, TensorAttribute::TRANSIENT));
  auto y = g->CreateTensor(TensorSpec(DataType::FLOAT32, {6, 4, 4, 1}, TensorAttribute::OUTPUT));
  g->CreateOperation<ops::Pool2d>(PoolType::AVG, PadType::VALID, std::array<uint32_t, 2>{2, 2},
                                  std::array<uint32_t, 2>{2, 2}, RoundType::FLOOR, DataLayout::CWHN)
      ->BindInputs({x}).BindOutputs({t0});
  g->CreateOperation<ops::Softmax>(1.0f, 0)->BindInputs({t0}).BindOutputs({y});
  auto r = tim::transform::LayoutInference(g, ctx);
  Dump("softmax_axis", r.first, r.first->Compile());
}

// Shape inference of the operators added around the convolution path.
void Shapes(const std::shared_ptr<Context>& ctx) {
  {
    auto g = ctx->CreateGraph();
    std::vector<float> w(3 * 3 * 4 * 6, 1.f);
    auto x = g->CreateTensor(TensorSpec(DataType::FLOAT32, {5, 7, 4, 2}, TensorAttribute::INPUT));
    auto wt = g->CreateTensor(TensorSpec(DataType::FLOAT32, {3, 3, 4, 6}, TensorAttribute::CONSTANT), w.data());
    auto t = g->CreateTensor(TensorSpec(DataType::FLOAT32, {}, TensorAttribute::TRANSIENT));
    auto u = g->CreateTensor(TensorSpec(DataType::FLOAT32, {}, TensorAttribute::TRANSIENT));
    auto y = g->CreateTensor(TensorSpec(DataType::FLOAT16, {}, TensorAttribute::OUTPUT));
    g->CreateOperation<ops::DeConv2d>(6, PadType::AUTO, std::array<uint32_t, 2>{3, 3}, std::array<uint32_t, 2>{2, 2},
                                      std::array<uint32_t, 2>{1, 1}, std::array<uint32_t, 4>{1, 1, 1, 1}, 1)
        ->BindInputs({x, wt}).BindOutputs({t});
    g->CreateOperation<ops::Transpose>(std::vector<uint32_t>{2, 0, 1, 3})->BindInputs({t}).BindOutputs({u});
    g->CreateOperation<ops::DataConvert>()->BindInputs({u}).BindOutputs({y});
    Dump("deconv_transpose_convert", g, g->Compile());
  }
  {
    auto g = ctx->CreateGraph();
    auto x = g->CreateTensor(TensorSpec(DataType::FLOAT32, {5, 7, 4}, TensorAttribute::INPUT));
    auto y = g->CreateTensor(TensorSpec(DataType::FLOAT32, {}, TensorAttribute::OUTPUT));
    g->CreateOperation<ops::Transpose>(std::vector<uint32_t>{0, 0, 1})->BindInputs({x}).BindOutputs({y});
    Dump("bad_perm", g, g->Compile());
  }
  {
    auto g = ctx->CreateGraph();
    std::vector<float> w(3 * 3 * 2 * 8, 1.f);
    auto x = g->CreateTensor(TensorSpec(DataType::FLOAT32, {9, 9, 4, 1}, TensorAttribute::INPUT));
    auto wt = g->CreateTensor(TensorSpec(DataType::FLOAT32, {3, 3, 2, 8}, TensorAttribute::CONSTANT), w.data());
    auto y = g->CreateTensor(TensorSpec(DataType::FLOAT32, {}, TensorAttribute::OUTPUT));
    g->CreateOperation<ops::GroupedConv2d>(PadType::SAME, std::array<uint32_t, 2>{2, 2}, std::array<uint32_t, 2>{1, 1}, 2)
        ->BindInputs({x, wt}).BindOutputs({y});
    Dump("grouped_same_stride2", g, g->Compile());
  }
}
}  // namespace

namespace tim {
namespace vx {
std::unique_ptr<Executor> CreateExecutor() { return std::unique_ptr<Executor>(new NoopExecutor()); }
}  // namespace vx
}  // namespace tim

int main() {
  auto ctx = Context::Create();
  NhwcNet(ctx);
  SoftmaxAxis(ctx);
  Shapes(ctx);
  return 0;
}
