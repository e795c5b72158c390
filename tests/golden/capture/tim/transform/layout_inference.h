// Fixture-generator shim in front of the real header: the reference's layout-inference tests
// call LayoutInference(src_graph, ctx); the recorder needs to know which graph was the source,
// because what a fixture holds is the SOURCE graph (layouts as the test states them) with the
// expected output, not the rewritten graph.
#pragma once
#include_next "tim/transform/layout_inference.h"

namespace tvxcap {
void NoteLayoutInference(
    const std::shared_ptr<tim::vx::Graph>& src,
    const std::pair<std::shared_ptr<tim::vx::Graph>,
                    std::map<std::shared_ptr<tim::vx::Tensor>, std::shared_ptr<tim::vx::Tensor>>>& result);
}
namespace tim {
namespace transform {
inline auto LayoutInferenceRecorded(const std::shared_ptr<vx::Graph>& src, std::shared_ptr<vx::Context>& ctx) {
  auto r = LayoutInference(src, ctx);
  ::tvxcap::NoteLayoutInference(src, r);
  return r;
}
}  // namespace transform
}  // namespace tim
#define LayoutInference LayoutInferenceRecorded
