// Private object model behind the tim::vx API: tensors, operator records,
// the graph container and the executor interface the graph hands its
// compiled plan to. Nothing here is visible to applications.
#pragma once

#include <cstdio>
#include <cstdlib>
#include <memory>
#include <string>
#include <vector>

#include "tim/vx/detail/hotpath_ops.h"

namespace tim {
namespace vx {

// ---- logging: same levels and env switch as ovxlib's VSILOG*
// (reference: src/tim/vx/internal/src/vsi_nn_log.c:32-78) --------------------
enum TvxLogLevel { TVX_LOG_ERROR = 1, TVX_LOG_WARN = 2, TVX_LOG_INFO = 3, TVX_LOG_DEBUG = 4 };
int TvxLogThreshold();
#define TVX_LOG(level, tag, ...)                                  \
  do {                                                            \
    if ((level) <= ::tim::vx::TvxLogThreshold()) {                \
      std::fprintf(stderr, tag "[%s:%d] ", __func__, __LINE__);   \
      std::fprintf(stderr, __VA_ARGS__);                          \
      std::fprintf(stderr, "\n");                                 \
    }                                                             \
  } while (0)
#define VSILOGE(...) TVX_LOG(::tim::vx::TVX_LOG_ERROR, "E ", __VA_ARGS__)
#define VSILOGW(...) TVX_LOG(::tim::vx::TVX_LOG_WARN, "W ", __VA_ARGS__)
#define VSILOGI(...) TVX_LOG(::tim::vx::TVX_LOG_INFO, "I ", __VA_ARGS__)
#define VSILOGD(...) TVX_LOG(::tim::vx::TVX_LOG_DEBUG, "D ", __VA_ARGS__)

enum class OpKind : uint32_t {
  CONV2D = 1, FCL, POOL, RELU, RELU6, ADD, SOFTMAX, RESHAPE, TRANSPOSE, DATACONVERT, DECONV2D
};
const char* OpKindName(OpKind k);

// Attributes of every operator kind in one flat record; each kind reads only
// its own fields.
struct OpAttrs {
  // conv2d / pool
  PadType pad_type = PadType::AUTO;
  uint32_t pad[4] = {0, 0, 0, 0};  // left, right, top, bottom
  uint32_t stride[2] = {1, 1};
  uint32_t dilation[2] = {1, 1};
  uint32_t ksize[2] = {0, 0};
  int32_t multiplier = 0;
  int32_t groups = 0;  // GroupedConv2d: > 1
  DataLayout kernel_layout = DataLayout::WHIcOc;  // read by layout inference only
  uint32_t output_padding[2] = {0, 0};  // DeConv2d
  bool conv_1d = false;  // Conv1d: {W, C, N} tensors, the 2-D operator on rows of height one
  uint32_t weights = 0;
  // pool
  PoolType pool_type = PoolType::MAX;
  RoundType round_type = RoundType::FLOOR;
  bool pool_1d = false;
  // fully connected
  uint32_t axis = 0;
  // softmax
  float beta = 1.0f;
  int32_t sm_axis = 0;
  // reshape
  std::vector<uint32_t> new_shape;
  // transpose
  std::vector<uint32_t> perm;
  // rounding policy (Operation::SetRoundingPolicy)
  OverflowPolicy overflow = OverflowPolicy::SATURATE;
  RoundingPolicy rounding = RoundingPolicy::RTNE;
  RoundType down_scale_rounding = RoundType::FLOOR;
  uint32_t accumulator_bits = 0;
};

class GraphImpl;

class OpImpl {
 public:
  OpImpl(Graph* graph, OpKind kind, int in_cnt, int out_cnt, DataLayout layout);
  GraphImpl* graph_;
  OpKind kind_;
  int input_cnt_;
  int output_cnt_;
  DataLayout layout_;
  uint32_t uid_;
  OpAttrs attrs_;
  std::vector<std::shared_ptr<Tensor>> inputs_tensor_;
  std::vector<std::shared_ptr<Tensor>> outputs_tensor_;
};

class TensorImpl : public Tensor {
 public:
  TensorImpl(GraphImpl* graph, const TensorSpec& spec, const void* data,
             void* user_io_ptr);
  ~TensorImpl() override;

  const ShapeType& GetShape() override { return spec_.shape_; }
  DataType GetDataType() override { return spec_.datatype_; }
  const Quantization& GetQuantization() override { return spec_.quantization_; }
  TensorSpec& GetSpec() override { return spec_; }
  uint32_t GetId() override { return id_; }
  bool CopyDataToTensor(const void* data, uint32_t size_in_bytes = 0) override;
  bool CopyDataFromTensor(void* data) override;
  bool SwapHandle(void* new_ptr, bool is_new_ptr_malloc_by_ovxlib,
                  void** old_ptr) override;
  bool SwapHandle(std::shared_ptr<tim::vx::Tensor> tensor) override;
  bool SwapHandleWithCache(std::shared_ptr<tim::vx::Tensor> tensor) override;
  bool FlushCacheForHandle() override;
  bool InvalidateCacheForHandle() override;
  void* map(bool invalidate_cpu_cache = false) override;
  void unmap() override;
  bool IsPlaceHolder() override { return false; }
  bool IsConstTensor() override {
    return (spec_.attr_ & TensorAttribute::CONSTANT) != 0;
  }
  bool IsScalar() override { return is_scalar_ != 0; }
  bool SaveTensorToTextByFp32(std::string filename) override;
  void SetScalar(int8_t is_scalar) override { is_scalar_ = is_scalar; }
  void* ConvertTensorToData(uint8_t* tensorData) override;
  float* ConvertTensorToFloat32Data() override;

  bool IsWriteable() const { return spec_.attr_ != TensorAttribute::TRANSIENT; }
  bool IsReadable() const { return spec_.attr_ != TensorAttribute::TRANSIENT; }
  // Host image of the tensor: constant data, or the staging buffer of an
  // INPUT / OUTPUT / VARIABLE tensor. Empty for TRANSIENT tensors.
  uint8_t* HostData();
  size_t HostBytes() const;
  void EnsureHostBuffer();

  GraphImpl* graph_;
  uint32_t id_;
  TensorSpec spec_;
  // The tensor's own host image: page-locked memory for INPUT / OUTPUT tensors when the executor offers
  // it (g_host_alloc), ordinary memory otherwise.
  uint8_t* owned_ = nullptr;
  size_t owned_bytes_ = 0;
  void (*owned_free_)(void*) = nullptr;
  void ReleaseOwned();
  uint8_t* user_ptr_ = nullptr;  // CreateIOTensor(spec, ptr) / SwapHandle
  bool host_dirty_ = false;      // host image newer than the device copy
  int8_t is_scalar_ = 0;
};

class TensorPlaceholder : public TensorImpl {
 public:
  explicit TensorPlaceholder(GraphImpl* graph);
  bool IsPlaceHolder() override { return true; }
};

// What a graph is compiled into and run by. One implementation drives the
// GPU through the C ABI of include/tvx_hip.h; test tooling may link another.
class Executor {
 public:
  virtual ~Executor() {}
  // Called once after verification, shape inference and ordering succeeded.
  virtual bool Realize(GraphImpl* graph) = 0;
  // Blocking: results are visible in OUTPUT tensors' host images on return.
  virtual bool Execute(GraphImpl* graph) = 0;
};
std::unique_ptr<Executor> CreateExecutor();
// Host memory the executor can copy from / to fastest (null: none on offer). Set by the executor's module.
extern void* (*g_host_alloc)(size_t bytes);
extern void (*g_host_free)(void* p);

class ContextImpl : public Context {
 public:
  std::shared_ptr<Graph> CreateGraph() override;
  std::shared_ptr<Graph> CreateGraph(const CompileOption& options) override;
  bool isClOnly() override { return false; }
  bool hasSP() override { return false; }
};

class GraphImpl : public Graph {
 public:
  GraphImpl(ContextImpl* context, const CompileOption& options);
  ~GraphImpl() override;

  void SetCompileOption(const CompileOption&) override;
  std::shared_ptr<Tensor> CreateTensor(const TensorSpec& spec,
                                       const void* data = nullptr) override;
  std::shared_ptr<Tensor> CreateTensor(const TensorSpec& spec,
                                       const DmaBufferDesc& dmafd) override;
  std::shared_ptr<Tensor> CreateIOTensor(const TensorSpec& spec,
                                         void* data = nullptr) override;
  std::shared_ptr<Tensor> CreateTensorPlaceHolder() override;
  bool Compile() override;
  bool CompileToBinary(void* buf, size_t* size) override;
  bool Run() override;
  const std::vector<std::shared_ptr<Tensor>> InputsTensor() const override;
  const std::vector<std::shared_ptr<Tensor>> OutputsTensor() const override;
  void UpdateTensorConsumersMap(const std::shared_ptr<Tensor>& tensor,
                                const Operation* op) override;
  void RenewTensorConsumersMap(const std::shared_ptr<Tensor>& org_tensor,
                               const std::shared_ptr<Tensor>& dst_tensor,
                               const Operation* op) override;
  void UpdateTensorProducerMap(const std::shared_ptr<Tensor>& tensor,
                               const Operation* op) override;
  const std::vector<std::shared_ptr<Operation>> GetConsumersOp(
      std::shared_ptr<Tensor> tensor) const override;
  std::shared_ptr<Operation> GetProducerOp(
      std::shared_ptr<Tensor> tensor) override;
  void PrintGraph() const override;
  std::vector<std::shared_ptr<Operation>>& OpVector() override;
  std::map<std::shared_ptr<Tensor>, std::vector<std::shared_ptr<Operation>>>&
  TensorConsumer() override;
  std::map<std::shared_ptr<Tensor>, std::shared_ptr<Operation>>&
  TensorProducer() override;

  uint32_t NextTensorId() { return next_tensor_id_++; }
  uint32_t NextOpUid() { return ++cur_nid_; }
  void ConsumeInput() { --not_consumed_input_cnt_; }
  void ConsumeOutput() { --not_consumed_output_cnt_; }

  // Host-side compile passes (graph_passes.cc). Each returns false and logs
  // on the first violation.
  bool VerifyAndInfer();
  // Operators in execution (topological) order; valid after VerifyAndInfer().
  std::vector<Operation*> sorted_ops_;

  ContextImpl* context_;
  CompileOption options_;
  std::shared_ptr<Tensor> tensor_placeholder_;
  std::vector<std::shared_ptr<Tensor>> inputs_tensor_;
  std::vector<std::shared_ptr<Tensor>> outputs_tensor_;
  std::map<std::shared_ptr<Tensor>, std::vector<std::shared_ptr<Operation>>>
      tensor_consumers_;
  std::map<std::shared_ptr<Tensor>, std::shared_ptr<Operation>> tensor_producer_;
  int32_t not_consumed_input_cnt_ = 0;
  int32_t not_consumed_output_cnt_ = 0;
  uint32_t next_tensor_id_ = 0;
  uint32_t cur_nid_ = 0;
  int compile_state_ = 0;  // 0 = not attempted, 1 = ok, -1 = failed
  std::unique_ptr<Executor> executor_;
};

// ---- shape / padding arithmetic shared by the passes and the tests --------
// reference: src/tim/vx/internal/src/utils/vsi_nn_util.c:203-235,483-588
uint32_t ComputeFilterSize(uint32_t in, uint32_t ksize, const uint32_t pad[2],
                           uint32_t stride, uint32_t dilation, RoundType rnd);
void ComputePaddingPerAxis(uint32_t in, uint32_t ksize, uint32_t stride,
                           uint32_t dilation, PadType type, uint32_t out_pad[2]);

size_t DataTypeBytes(DataType t);
const char* DataTypeName(DataType t);

}  // namespace vx
}  // namespace tim

#include "tim/transform/layout_inference.h"
namespace tim {
namespace transform {
// Rebuilds src_graph (layouts resolved) inside dst_graph; see layout_inference.cc.
bool RewriteInto(const std::shared_ptr<vx::Graph>& src_graph, const std::shared_ptr<vx::Graph>& dst_graph,
                 const std::map<std::shared_ptr<vx::Tensor>, std::shared_ptr<IPermuteVector>>& tensor_pv_map,
                 std::map<std::shared_ptr<vx::Tensor>, std::shared_ptr<vx::Tensor>>* io_map);
}  // namespace transform
}  // namespace tim
