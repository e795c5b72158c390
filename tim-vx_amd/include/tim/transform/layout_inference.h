// Layout inference: rewrites a graph whose operators carry channel-fastest (CWHN) activations
// and IcWHOc / OcIcWH / IcOcWH kernels - what NHWC front ends hand over - into an equivalent
// graph on the WHCN / WHIcOc layouts the kernels run on.
// reference: include/tim/transform/layout_inference.h:42-54 (same entry point and result).
#pragma once
#include <map>
#include <memory>
#include <utility>
#include <vector>

namespace tim {
namespace vx {
class Context;
class Graph;
class Tensor;
class Operation;
}  // namespace vx

namespace transform {

// How a tensor of the rewritten graph relates to the tensor of the source graph it stands for:
// its dimension i is the source tensor's dimension AsStdVec()[i] (dimension 0 fastest).
class IPermuteVector {
 public:
  virtual ~IPermuteVector() {}
  virtual uint32_t Rank() const = 0;
  virtual std::vector<uint32_t> AsStdVec() const = 0;
  virtual bool IsAligned() const = 0;  // the identity
};
std::shared_ptr<IPermuteVector> MakePermuteVector(const std::vector<uint32_t>& perm);

// Returns the rewritten graph and the map from the source graph's INPUT / OUTPUT tensors to
// their counterparts, which keep the source tensors' shapes (permutes are inserted behind the
// inputs and in front of the outputs where an operator wants another layout). tensor_pv_map
// may state that the data fed to an input is already permuted.
std::pair<std::shared_ptr<vx::Graph>,
          std::map<std::shared_ptr<vx::Tensor>, std::shared_ptr<vx::Tensor>>>
LayoutInference(const std::shared_ptr<vx::Graph>& src_graph, std::shared_ptr<vx::Context>& ctx,
                std::map<std::shared_ptr<vx::Tensor>, std::shared_ptr<IPermuteVector>> tensor_pv_map =
                    std::map<std::shared_ptr<vx::Tensor>, std::shared_ptr<IPermuteVector>>());

}  // namespace transform
}  // namespace tim
