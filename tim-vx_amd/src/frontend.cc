// Object model of the tim::vx API: specs, tensors, graph bookkeeping,
// operator construction and binding. Host-only; the compiled graph is handed
// to an Executor (runtime.h).
//
// Behaviour follows the reference's pimpl layer:
//   src/tim/vx/tensor.cc (specs, host copies, TRANSIENT access rules),
//   src/tim/vx/graph.cc (IO registration, producer/consumer maps, compile-once),
//   src/tim/vx/operation.cc + builtin_op_impl.cc (positional binding),
//   src/tim/vx/ops/{conv2d,fullyconnected,pool2d,pool1d,activations}.cc.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <fstream>

#include "runtime.h"

namespace tim {
namespace vx {

int TvxLogThreshold() {
  static int level = [] {
    const char* e = std::getenv("VSI_NN_LOG_LEVEL");
    return e ? std::atoi(e) : static_cast<int>(TVX_LOG_WARN);
  }();
  return level;
}

const char* OpKindName(OpKind k) {
  switch (k) {
    case OpKind::CONV2D: return "CONV2D";
    case OpKind::FCL: return "FCL";
    case OpKind::POOL: return "POOL";
    case OpKind::RELU: return "RELU";
    case OpKind::RELU6: return "RELU6";
    case OpKind::ADD: return "ADD";
    case OpKind::SOFTMAX: return "SOFTMAX";
    case OpKind::RESHAPE: return "RESHAPE";
    case OpKind::TRANSPOSE: return "TRANSPOSE";
    case OpKind::DATACONVERT: return "DATACONVERT";
    case OpKind::DECONV2D: return "DECONV2D";
  }
  return "?";
}

size_t DataTypeBytes(DataType t) {
  switch (t) {
    case DataType::INT16: case DataType::UINT16: case DataType::FLOAT16: return 2;
    case DataType::INT32: case DataType::UINT32: case DataType::FLOAT32: return 4;
    case DataType::INT64: return 8;
    default: return 1;
  }
}

const char* DataTypeName(DataType t) {
  switch (t) {
    case DataType::INT8: return "INT8";
    case DataType::UINT8: return "UINT8";
    case DataType::INT16: return "INT16";
    case DataType::UINT16: return "UINT16";
    case DataType::INT32: return "INT32";
    case DataType::UINT32: return "UINT32";
    case DataType::INT64: return "INT64";
    case DataType::FLOAT16: return "FLOAT16";
    case DataType::FLOAT32: return "FLOAT32";
    case DataType::BOOL8: return "BOOL8";
    case DataType::INT4: return "INT4";
    case DataType::UINT4: return "UINT4";
    default: return "UNKNOWN";
  }
}

// ---------------------------------------------------------------------------
// TensorSpec / Quantization (reference: src/tim/vx/tensor.cc:471-560)
// ---------------------------------------------------------------------------
TensorSpec::TensorSpec(const TensorSpec& o)
    : datatype_(o.datatype_), shape_(o.shape_), attr_(o.attr_),
      quantization_(o.quantization_) {}

TensorSpec& TensorSpec::operator=(const TensorSpec& o) {
  datatype_ = o.datatype_;
  shape_ = o.shape_;
  attr_ = o.attr_;
  quantization_ = o.quantization_;
  return *this;
}

bool TensorSpec::operator==(const TensorSpec& o) const {
  return datatype_ == o.datatype_ && shape_ == o.shape_ && attr_ == o.attr_ &&
         quantization_ == o.quantization_;
}

TensorSpec& TensorSpec::SetDataType(DataType d) { datatype_ = d; return *this; }
TensorSpec& TensorSpec::SetShape(const ShapeType& s) { shape_ = s; return *this; }
TensorSpec& TensorSpec::SetAttribute(TensorAttribute a) { attr_ = a; return *this; }
TensorSpec& TensorSpec::SetQuantization(Quantization& q) {
  quantization_ = q;
  return *this;
}

TensorSpec TensorSpec::AsTransientSpec() const {
  return TensorSpec(datatype_, ShapeType({}), TensorAttribute::TRANSIENT,
                    quantization_);
}

int64_t TensorSpec::GetElementNum() const {
  int64_t n = 1;
  for (auto d : shape_) n *= d;
  return n;
}

int64_t TensorSpec::GetElementByteSize() const {
  // INT64 counts as 1 here exactly as in the reference (tensor.cc:515-532).
  return datatype_ == DataType::INT64 ? 1
                                      : static_cast<int64_t>(DataTypeBytes(datatype_));
}

int64_t TensorSpec::GetByteSize() const {
  return GetElementNum() * GetElementByteSize();
}

bool Quantization::operator==(const Quantization& o) const {
  if (type_ != QuantType::DYNAMIC_FIXED_POINT) {
    return type_ == o.type_ && scales_ == o.scales_ &&
           zero_points_ == o.zero_points_ && channel_dim_ == o.channel_dim_;
  }
  return fl_ == o.fl_;
}

// ---------------------------------------------------------------------------
// CompileOption (reference: src/tim/vx/compile_option.cc:32-72)
// ---------------------------------------------------------------------------
struct CompileOptionImpl {
  bool relax_mode = false;
  uint32_t device_id = 0;
};
CompileOption::CompileOption() : impl_(std::make_shared<CompileOptionImpl>()) {}
bool CompileOption::isRelaxMode() const { return impl_->relax_mode; }
bool CompileOption::setRelaxMode(bool enable) {
  impl_->relax_mode = enable;
  return true;
}
void CompileOption::setDeviceId(uint32_t device) { impl_->device_id = device; }
uint32_t CompileOption::getDeviceId() { return impl_->device_id; }
CompileOption CompileOption::DefaultOptions;

// ---------------------------------------------------------------------------
// fp16 <-> fp32 on the host (round-to-nearest-even)
// ---------------------------------------------------------------------------
static float HalfBitsToFloat(uint16_t h) {
  uint32_t sign = (h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, man = h & 0x3ff;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = -1;
      do { ++e; man <<= 1; } while (!(man & 0x400));
      bits = sign | ((112 - e) << 23) | ((man & 0x3ff) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

static uint16_t FloatToHalfBits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  int32_t exp = static_cast<int32_t>((x >> 23) & 0xff) - 127 + 15;
  uint32_t man = x & 0x7fffffu;
  if (((x >> 23) & 0xff) == 0xff) return sign | 0x7c00u | (man ? 0x200u : 0);
  if (exp >= 31) return sign | 0x7c00u;
  if (exp <= 0) {
    if (exp < -10) return sign;
    man |= 0x800000u;
    uint32_t shift = 14 - exp;
    uint32_t half = man >> shift, rem = man & ((1u << shift) - 1);
    uint32_t mid = 1u << (shift - 1);
    if (rem > mid || (rem == mid && (half & 1))) ++half;
    return sign | half;
  }
  uint32_t half = (exp << 10) | (man >> 13);
  uint32_t rem = man & 0x1fff;
  if (rem > 0x1000 || (rem == 0x1000 && (half & 1))) ++half;
  return sign | half;
}

// ---------------------------------------------------------------------------
// Tensor
// ---------------------------------------------------------------------------
TensorImpl::TensorImpl(GraphImpl* graph, const TensorSpec& spec,
                       const void* data, void* user_io_ptr)
    : graph_(graph), id_(graph ? graph->NextTensorId() : 0xffffffffu),
      spec_(spec), user_ptr_(static_cast<uint8_t*>(user_io_ptr)) {
  // Initial data is copied at creation into any host-visible tensor, so the
  // caller may free its buffer (reference: src/tim/vx/tensor.cc:451-456; an
  // INPUT-attribute weight filled this way: conv2d_test.cc:1980-2052).
  if (data && IsWriteable() && !spec_.shape_.empty()) {
    EnsureHostBuffer();
    std::memcpy(HostData(), data, HostBytes());
    host_dirty_ = true;
  }
}

void* (*g_host_alloc)(size_t bytes) = nullptr;
void (*g_host_free)(void* p) = nullptr;

TensorImpl::~TensorImpl() { ReleaseOwned(); }

void TensorImpl::ReleaseOwned() {
  if (owned_ && owned_free_) owned_free_(owned_);
  owned_ = nullptr;
  owned_bytes_ = 0;
  owned_free_ = nullptr;
}

size_t TensorImpl::HostBytes() const {
  size_t n = DataTypeBytes(spec_.datatype_);
  for (auto d : spec_.shape_) n *= d;
  return n;
}

void TensorImpl::EnsureHostBuffer() {
  if (user_ptr_) return;
  size_t n = HostBytes();
  if (owned_bytes_ == n && (owned_ || n == 0)) return;
  ReleaseOwned();
  if (n == 0) return;
  const bool io = (spec_.attr_ & (TensorAttribute::INPUT | TensorAttribute::OUTPUT)) != 0;
  if (io && g_host_alloc && g_host_free) {
    owned_ = static_cast<uint8_t*>(g_host_alloc(n));
    if (owned_) owned_free_ = g_host_free;
  }
  if (!owned_) {
    owned_ = static_cast<uint8_t*>(std::malloc(n));
    owned_free_ = std::free;
  }
  if (owned_) {
    owned_bytes_ = n;
    std::memset(owned_, 0, n);
  }
}

uint8_t* TensorImpl::HostData() {
  if (user_ptr_) return user_ptr_;
  return owned_;
}

bool TensorImpl::CopyDataToTensor(const void* data, uint32_t size_in_bytes) {
  (void)size_in_bytes;  // ignored, as in the reference
  if (!IsWriteable()) return false;
  if (!data) return true;
  if (spec_.shape_.empty()) {
    VSILOGE("tensor %u has no shape yet", id_);
    return false;
  }
  EnsureHostBuffer();
  std::memcpy(HostData(), data, HostBytes());
  host_dirty_ = true;
  return true;
}

bool TensorImpl::CopyDataFromTensor(void* data) {
  if (!IsReadable()) return false;
  if (!data) return true;
  if (!HostData()) {
    VSILOGE("tensor %u holds no data", id_);
    return false;
  }
  std::memcpy(data, HostData(), HostBytes());
  return true;
}

bool TensorImpl::SwapHandle(void* new_ptr, bool, void** old_ptr) {
  if (!(spec_.attr_ & (TensorAttribute::INPUT | TensorAttribute::OUTPUT)))
    return false;
  if (old_ptr) *old_ptr = user_ptr_;
  user_ptr_ = static_cast<uint8_t*>(new_ptr);
  host_dirty_ = true;
  return true;
}

bool TensorImpl::SwapHandle(std::shared_ptr<tim::vx::Tensor> tensor) {
  auto* other = dynamic_cast<TensorImpl*>(tensor.get());
  if (!other || !user_ptr_ || !other->user_ptr_) return false;
  std::swap(user_ptr_, other->user_ptr_);
  host_dirty_ = other->host_dirty_ = true;
  return true;
}

bool TensorImpl::SwapHandleWithCache(std::shared_ptr<tim::vx::Tensor> tensor) {
  return SwapHandle(tensor);
}

bool TensorImpl::FlushCacheForHandle() {
  if (!(spec_.attr_ & TensorAttribute::INPUT)) return false;
  host_dirty_ = true;
  return true;
}

bool TensorImpl::InvalidateCacheForHandle() {
  return (spec_.attr_ & TensorAttribute::OUTPUT) != 0;
}

void* TensorImpl::map(bool) {
  if (!(spec_.attr_ & (TensorAttribute::INPUT | TensorAttribute::OUTPUT)))
    return nullptr;
  EnsureHostBuffer();
  return HostData();
}

void TensorImpl::unmap() {
  if (spec_.attr_ & TensorAttribute::INPUT) host_dirty_ = true;
}

float* TensorImpl::ConvertTensorToFloat32Data() {
  // Caller frees with free(), as with vsi_nn_ConvertTensorToFloat32Data.
  size_t n = static_cast<size_t>(spec_.GetElementNum());
  float* out = static_cast<float*>(std::malloc(n * sizeof(float)));
  uint8_t* src = HostData();
  if (!out || !src) {
    std::free(out);
    return nullptr;
  }
  const Quantization& q = spec_.quantization_;
  float scale = q.Scales().empty() ? 1.0f : q.Scales()[0];
  int32_t zp = q.ZeroPoints().empty() ? 0 : q.ZeroPoints()[0];
  bool affine = q.Type() == QuantType::ASYMMETRIC;
  for (size_t i = 0; i < n; ++i) {
    switch (spec_.datatype_) {
      case DataType::FLOAT32: out[i] = reinterpret_cast<float*>(src)[i]; break;
      case DataType::FLOAT16:
        out[i] = HalfBitsToFloat(reinterpret_cast<uint16_t*>(src)[i]);
        break;
      case DataType::UINT8:
        out[i] = affine ? scale * (static_cast<int32_t>(src[i]) - zp) : src[i];
        break;
      case DataType::INT8: {
        int32_t v = reinterpret_cast<int8_t*>(src)[i];
        out[i] = affine ? scale * (v - zp) : v;
        break;
      }
      case DataType::INT32: {
        int32_t v = reinterpret_cast<int32_t*>(src)[i];
        out[i] = affine ? scale * (v - zp) : static_cast<float>(v);
        break;
      }
      default: out[i] = 0.f;
    }
  }
  return out;
}

void* TensorImpl::ConvertTensorToData(uint8_t* tensorData) {
  if (!HostData()) return nullptr;
  if (!tensorData) tensorData = static_cast<uint8_t*>(std::malloc(HostBytes()));
  if (tensorData) std::memcpy(tensorData, HostData(), HostBytes());
  return tensorData;
}

bool TensorImpl::SaveTensorToTextByFp32(std::string filename) {
  float* f = ConvertTensorToFloat32Data();
  if (!f) return false;
  std::ofstream os(filename);
  size_t n = static_cast<size_t>(spec_.GetElementNum());
  for (size_t i = 0; i < n; ++i) os << f[i] << "\n";
  std::free(f);
  return static_cast<bool>(os);
}

TensorPlaceholder::TensorPlaceholder(GraphImpl* graph)
    : TensorImpl(nullptr, TensorSpec(), nullptr, nullptr) {
  graph_ = graph;
}

namespace utils {
bool Float32ToDtype(std::shared_ptr<tim::vx::Tensor> tensor,
                    std::vector<float> fval, uint8_t* tensorData) {
  // Host quantiser: round-half-even, then add the zero point, then saturate
  // (reference: src/tim/vx/internal/include/utils/vsi_nn_dtype_util_prv.h:228-252).
  if (!tensor || !tensorData) return false;
  const Quantization& q = tensor->GetQuantization();
  float scale = q.Scales().empty() ? 1.0f : q.Scales()[0];
  int32_t zp = q.ZeroPoints().empty() ? 0 : q.ZeroPoints()[0];
  for (size_t i = 0; i < fval.size(); ++i) {
    switch (tensor->GetDataType()) {
      case DataType::FLOAT32: reinterpret_cast<float*>(tensorData)[i] = fval[i]; break;
      case DataType::FLOAT16:
        reinterpret_cast<uint16_t*>(tensorData)[i] = FloatToHalfBits(fval[i]);
        break;
      case DataType::UINT8: {
        long v = std::lrint(std::nearbyint(fval[i] / scale)) + zp;
        tensorData[i] = static_cast<uint8_t>(std::min(255l, std::max(0l, v)));
        break;
      }
      case DataType::INT8: {
        long v = std::lrint(std::nearbyint(fval[i] / scale)) + zp;
        reinterpret_cast<int8_t*>(tensorData)[i] =
            static_cast<int8_t>(std::min(127l, std::max(-128l, v)));
        break;
      }
      case DataType::INT32:
        reinterpret_cast<int32_t*>(tensorData)[i] =
            static_cast<int32_t>(std::lrint(std::nearbyint(fval[i] / scale)) + zp);
        break;
      default: return false;
    }
  }
  return true;
}

bool DtypeToFloat32(std::shared_ptr<tim::vx::Tensor> tensor,
                    uint8_t* tensorData, float* data) {
  if (!tensor || !tensorData || !data) return false;
  const Quantization& q = tensor->GetQuantization();
  float scale = q.Scales().empty() ? 1.0f : q.Scales()[0];
  int32_t zp = q.ZeroPoints().empty() ? 0 : q.ZeroPoints()[0];
  switch (tensor->GetDataType()) {
    case DataType::FLOAT32: *data = *reinterpret_cast<float*>(tensorData); break;
    case DataType::FLOAT16:
      *data = HalfBitsToFloat(*reinterpret_cast<uint16_t*>(tensorData));
      break;
    case DataType::UINT8: *data = scale * (static_cast<int32_t>(*tensorData) - zp); break;
    case DataType::INT8:
      *data = scale * (static_cast<int32_t>(*reinterpret_cast<int8_t*>(tensorData)) - zp);
      break;
    case DataType::INT32:
      *data = scale * (*reinterpret_cast<int32_t*>(tensorData) - zp);
      break;
    default: return false;
  }
  return true;
}
}  // namespace utils

// ---------------------------------------------------------------------------
// Context / Graph
// ---------------------------------------------------------------------------
std::shared_ptr<Context> Context::Create() {
  return std::make_shared<ContextImpl>();
}

std::shared_ptr<Graph> ContextImpl::CreateGraph() {
  return std::make_shared<GraphImpl>(this, CompileOption::DefaultOptions);
}

std::shared_ptr<Graph> ContextImpl::CreateGraph(const CompileOption& options) {
  return std::make_shared<GraphImpl>(this, options);
}

const std::vector<std::shared_ptr<Tensor>> Graph::GetConstantInputs() const {
  std::vector<std::shared_ptr<Tensor>> out;
  for (auto& op : op_vector_) {
    auto c = op->ConstantInputsTensor();
    out.insert(out.end(), c.begin(), c.end());
  }
  return out;
}

GraphImpl::GraphImpl(ContextImpl* context, const CompileOption& options)
    : context_(context), options_(options) {}

GraphImpl::~GraphImpl() {
  // Executors may hold device memory keyed by tensors: drop them first.
  executor_.reset();
}

void GraphImpl::SetCompileOption(const CompileOption& o) { options_ = o; }

std::shared_ptr<Tensor> GraphImpl::CreateTensor(const TensorSpec& spec,
                                                const void* data) {
  auto tensor = std::make_shared<TensorImpl>(this, spec, data, nullptr);
  if (spec.attr_ & TensorAttribute::INPUT) {
    if (std::find(inputs_tensor_.begin(), inputs_tensor_.end(), tensor) ==
        inputs_tensor_.end())
      inputs_tensor_.push_back(tensor);
    ++not_consumed_input_cnt_;
  }
  if (spec.attr_ & TensorAttribute::OUTPUT) {
    outputs_tensor_.push_back(tensor);
    ++not_consumed_output_cnt_;
  }
  return tensor;
}

std::shared_ptr<Tensor> GraphImpl::CreateTensor(const TensorSpec& spec,
                                                const DmaBufferDesc&) {
  VSILOGW("dma-buf backed tensors are not supported; using a host buffer");
  return CreateTensor(spec, static_cast<const void*>(nullptr));
}

std::shared_ptr<Tensor> GraphImpl::CreateIOTensor(const TensorSpec& spec,
                                                  void* data) {
  auto tensor = std::make_shared<TensorImpl>(this, spec, nullptr, data);
  if (spec.attr_ & TensorAttribute::INPUT) {
    inputs_tensor_.push_back(tensor);
    ++not_consumed_input_cnt_;
  }
  if (spec.attr_ & TensorAttribute::OUTPUT) {
    outputs_tensor_.push_back(tensor);
    ++not_consumed_output_cnt_;
  }
  return tensor;
}

std::shared_ptr<Tensor> GraphImpl::CreateTensorPlaceHolder() {
  if (!tensor_placeholder_)
    tensor_placeholder_ = std::make_shared<TensorPlaceholder>(this);
  return tensor_placeholder_;
}

const std::vector<std::shared_ptr<Tensor>> GraphImpl::InputsTensor() const {
  return inputs_tensor_;
}
const std::vector<std::shared_ptr<Tensor>> GraphImpl::OutputsTensor() const {
  return outputs_tensor_;
}
std::vector<std::shared_ptr<Operation>>& GraphImpl::OpVector() {
  return op_vector_;
}
std::map<std::shared_ptr<Tensor>, std::vector<std::shared_ptr<Operation>>>&
GraphImpl::TensorConsumer() {
  return tensor_consumers_;
}
std::map<std::shared_ptr<Tensor>, std::shared_ptr<Operation>>&
GraphImpl::TensorProducer() {
  return tensor_producer_;
}

void GraphImpl::UpdateTensorConsumersMap(const std::shared_ptr<Tensor>& tensor,
                                         const Operation* op) {
  for (const auto& added : op_vector_)
    if (added.get() == op) tensor_consumers_[tensor].push_back(added);
}

void GraphImpl::RenewTensorConsumersMap(
    const std::shared_ptr<Tensor>& org_tensor,
    const std::shared_ptr<Tensor>& dst_tensor, const Operation* op) {
  auto it = std::find_if(op_vector_.begin(), op_vector_.end(),
                         [op](const std::shared_ptr<Operation>& o) {
                           return o.get() == op;
                         });
  if (it == op_vector_.end()) return;
  tensor_consumers_.erase(org_tensor);
  tensor_consumers_[dst_tensor].push_back(*it);
}

void GraphImpl::UpdateTensorProducerMap(const std::shared_ptr<Tensor>& tensor,
                                        const Operation* op) {
  for (const auto& added : op_vector_)
    if (added.get() == op) tensor_producer_[tensor] = added;
}

const std::vector<std::shared_ptr<Operation>> GraphImpl::GetConsumersOp(
    std::shared_ptr<Tensor> tensor) const {
  auto it = tensor_consumers_.find(tensor);
  if (it != tensor_consumers_.end()) return it->second;
  VSILOGD("Tensor has no consumers, may be graph output.");
  return {};
}

std::shared_ptr<Operation> GraphImpl::GetProducerOp(
    std::shared_ptr<Tensor> tensor) {
  auto it = tensor_producer_.find(tensor);
  if (it != tensor_producer_.end()) return it->second;
  VSILOGD("Tensor has no producer, may be graph input.");
  return {};
}

void GraphImpl::PrintGraph() const {
  std::fprintf(stderr, "graph: %zu ops\n", op_vector_.size());
  for (auto& op : op_vector_) {
    const OpImpl* im = op->impl().get();
    std::fprintf(stderr, "  [%u] %s in(", im->uid_, OpKindName(im->kind_));
    for (auto& t : im->inputs_tensor_) std::fprintf(stderr, " %u", t->GetId());
    std::fprintf(stderr, " ) out(");
    for (auto& t : im->outputs_tensor_) std::fprintf(stderr, " %u", t->GetId());
    std::fprintf(stderr, " )\n");
  }
}

bool GraphImpl::Compile() {
  // Compiled at most once; later calls report the first outcome.
  if (compile_state_ != 0) return compile_state_ > 0;
  if (not_consumed_input_cnt_ > 0)
    VSILOGW("Graph has free input, INPUT tensor may be created but not consumed.");
  if (not_consumed_output_cnt_ != 0)
    VSILOGW("Graph has free output, OUTPUT tensor may be created but not consumed.");
  compile_state_ = -1;
  if (!VerifyAndInfer()) return false;
  executor_ = CreateExecutor();
  if (!executor_ || !executor_->Realize(this)) {
    executor_.reset();
    return false;
  }
  compile_state_ = 1;
  return true;
}

bool GraphImpl::CompileToBinary(void*, size_t*) {
  VSILOGE("binary graph export is not supported by this runtime");
  return false;
}

bool GraphImpl::Run() { return Compile() && executor_->Execute(this); }

// ---------------------------------------------------------------------------
// Operation / BuiltinOp
// ---------------------------------------------------------------------------
OpImpl::OpImpl(Graph* graph, OpKind kind, int in_cnt, int out_cnt,
               DataLayout layout)
    : graph_(static_cast<GraphImpl*>(graph)), kind_(kind), input_cnt_(in_cnt),
      output_cnt_(out_cnt), layout_(layout), uid_(graph_->NextOpUid()) {}

Operation::Operation() {}
Operation::~Operation() {}
std::unique_ptr<OpImpl>& Operation::impl() { return impl_; }
const std::unique_ptr<OpImpl>& Operation::impl() const { return impl_; }
const uint32_t& Operation::uid() const { return impl_->uid_; }

Operation& Operation::BindInput(const std::shared_ptr<Tensor>& tensor) {
  impl_->inputs_tensor_.push_back(tensor);
  if (!tensor->IsPlaceHolder() && (tensor->GetSpec().attr_ & TensorAttribute::INPUT))
    impl_->graph_->ConsumeInput();
  impl_->graph_->UpdateTensorConsumersMap(tensor, this);
  OnBindInputPostProc(tensor,
                      static_cast<int32_t>(impl_->inputs_tensor_.size()) - 1);
  return *this;
}

Operation& Operation::BindOutput(const std::shared_ptr<Tensor>& tensor) {
  impl_->outputs_tensor_.push_back(tensor);
  if (tensor->GetSpec().attr_ & TensorAttribute::OUTPUT)
    impl_->graph_->ConsumeOutput();
  impl_->graph_->UpdateTensorProducerMap(tensor, this);
  return *this;
}

Operation& Operation::BindInputs(
    const std::vector<std::shared_ptr<Tensor>>& tensors) {
  for (auto& t : tensors) BindInput(t);
  return *this;
}

Operation& Operation::BindOutputs(
    const std::vector<std::shared_ptr<Tensor>>& tensors) {
  for (auto& t : tensors) BindOutput(t);
  return *this;
}

Operation& Operation::SetRoundingPolicy(OverflowPolicy overflow_policy,
                                        RoundingPolicy rounding_policy,
                                        RoundType down_scale_size_rounding,
                                        uint32_t accumulator_bits) {
  impl_->attrs_.overflow = overflow_policy;
  impl_->attrs_.rounding = rounding_policy;
  impl_->attrs_.down_scale_rounding = down_scale_size_rounding;
  impl_->attrs_.accumulator_bits = accumulator_bits;
  return *this;
}

bool Operation::IsAllInputsConst() const {
  for (auto& t : impl_->inputs_tensor_)
    if (!t->IsConstTensor()) return false;
  return true;
}

const std::vector<std::shared_ptr<Tensor>> Operation::ConstantInputsTensor() const {
  if (IsAllInputsConst()) return impl_->inputs_tensor_;
  return {};
}

void Operation::OnBindInputPostProc(const std::shared_ptr<Tensor>&, int32_t) {}

BuiltinOp::BuiltinOp(Graph* graph, uint32_t kind, int in_cnt, int out_cnt,
                     DataLayout layout) {
  impl_.reset(new OpImpl(graph, static_cast<OpKind>(kind), in_cnt, out_cnt, layout));
}

// An fp16 constant bias is replaced by an fp32 constant at bind time
// (reference: src/tim/vx/ops/conv2d.cc:101-118, fullyconnected.cc:48-63).
static void PromoteHalfBias(Operation* op, OpImpl* impl,
                            const std::shared_ptr<Tensor>& tensor) {
  if (tensor->GetDataType() != DataType::FLOAT16 || !tensor->IsConstTensor() ||
      impl->inputs_tensor_.size() != 3)
    return;
  float* f32 = tensor->ConvertTensorToFloat32Data();
  if (!f32) return;
  TensorSpec spec(DataType::FLOAT32, tensor->GetShape(), TensorAttribute::CONSTANT);
  auto promoted = impl->graph_->CreateTensor(spec, f32);
  std::free(f32);
  impl->inputs_tensor_[2] = promoted;
  impl->graph_->RenewTensorConsumersMap(tensor, promoted, op);
}

namespace ops {

static constexpr uint32_t K(OpKind k) { return static_cast<uint32_t>(k); }

// ---- Conv2d ---------------------------------------------------------------
Conv2d::Conv2d(Graph* graph, PadType padding,
               const std::array<uint32_t, 2>& stride,
               const std::array<uint32_t, 2>& dilation, int32_t multiplier,
               DataLayout input_layout, DataLayout kernel_layout)
    : Conv2d(graph, 0, padding, {0, 0}, stride, dilation, {0, 0, 0, 0},
             multiplier, input_layout, kernel_layout) {}

Conv2d::Conv2d(Graph* graph, const std::array<uint32_t, 4> pad,
               const std::array<uint32_t, 2>& stride,
               const std::array<uint32_t, 2>& dilation, int32_t multiplier,
               DataLayout input_layout, DataLayout kernel_layout)
    : Conv2d(graph, 0, PadType::AUTO, {0, 0}, stride, dilation, pad, multiplier,
             input_layout, kernel_layout) {}

Conv2d::Conv2d(Graph* graph, int32_t weights, PadType padding,
               const std::array<uint32_t, 2>& ksize,
               const std::array<uint32_t, 2>& stride,
               const std::array<uint32_t, 2>& dilation, int32_t multiplier,
               DataLayout input_layout, DataLayout kernel_layout)
    : Conv2d(graph, weights, padding, ksize, stride, dilation, {0, 0, 0, 0},
             multiplier, input_layout, kernel_layout) {}

Conv2d::Conv2d(Graph* graph, int32_t weights, PadType padding,
               const std::array<uint32_t, 2>& ksize,
               const std::array<uint32_t, 2>& stride,
               const std::array<uint32_t, 2>& dilation,
               const std::array<uint32_t, 4>& pad, int32_t multiplier,
               DataLayout input_layout, DataLayout kernel_layout)
    : BuiltinOp(graph, K(OpKind::CONV2D), 0, 0, input_layout),
      weights_(weights), padding_(padding), ksize_(ksize), stride_(stride),
      dilation_(dilation), pad_(pad), multiplier_(multiplier),
      kernel_layout_(kernel_layout) {
  OpAttrs& a = impl_->attrs_;
  a.kernel_layout = kernel_layout_;
  if (padding_ == PadType::NONE)
    VSILOGW("PadType::NONE is treated as AUTO (explicit pad)");
  a.pad_type = padding_ == PadType::NONE ? PadType::AUTO : padding_;
  for (int i = 0; i < 4; ++i) a.pad[i] = pad_[i];
  for (int i = 0; i < 2; ++i) {
    a.stride[i] = stride_[i];
    a.dilation[i] = dilation_[i];
  }
  a.multiplier = multiplier_;
  // `weights` and `ksize` are kept on the object only; shape inference reads
  // the weight tensor (reference: src/tim/vx/ops/conv2d.cc:57-82).
}

std::shared_ptr<Operation> Conv2d::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Conv2d>(
      static_cast<int32_t>(weights_), padding_, ksize_, stride_, dilation_, pad_,
      multiplier_, impl_->layout_, kernel_layout_);
}

const std::vector<std::shared_ptr<Tensor>> Conv2d::ConstantInputsTensor() const {
  if (IsAllInputsConst()) return {impl_->inputs_tensor_[0]};
  return {};
}

void Conv2d::OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor, int32_t) {
  PromoteHalfBias(this, impl_.get(), tensor);
}

// ---- Conv1d -----------------------------------------------------------------
Conv1d::Conv1d(Graph* graph, PadType padding, uint32_t stride, uint32_t dilation,
               int32_t multiplier, DataLayout input_layout, DataLayout kernel_layout)
    : Conv1d(graph, 0, padding, 0, stride, dilation, {0, 0}, multiplier, input_layout, kernel_layout) {}

Conv1d::Conv1d(Graph* graph, const std::array<uint32_t, 2>& pad, uint32_t stride, uint32_t dilation,
               int32_t multiplier, DataLayout input_layout, DataLayout kernel_layout)
    : Conv1d(graph, 0, PadType::AUTO, 0, stride, dilation, pad, multiplier, input_layout, kernel_layout) {}

Conv1d::Conv1d(Graph* graph, int32_t weights, PadType padding, uint32_t ksize, uint32_t stride,
               uint32_t dilation, int32_t multiplier, DataLayout input_layout, DataLayout kernel_layout)
    : Conv1d(graph, weights, padding, ksize, stride, dilation, {0, 0}, multiplier, input_layout,
             kernel_layout) {}

Conv1d::Conv1d(Graph* graph, int32_t weights, PadType padding, uint32_t ksize, uint32_t stride,
               uint32_t dilation, const std::array<uint32_t, 2>& pad, int32_t multiplier,
               DataLayout input_layout, DataLayout kernel_layout)
    : BuiltinOp(graph, K(OpKind::CONV2D), 0, 0, input_layout),
      weights_(weights), padding_(padding), ksize_(ksize), stride_(stride), dilation_(dilation),
      pad_(pad), multiplier_(multiplier), kernel_layout_(kernel_layout) {
  OpAttrs& a = impl_->attrs_;
  a.kernel_layout = kernel_layout_;
  a.conv_1d = true;
  a.pad_type = padding_ == PadType::NONE ? PadType::AUTO : padding_;
  a.pad[0] = pad_[0];
  a.pad[1] = pad_[1];
  a.stride[0] = stride_;
  a.stride[1] = 1;
  a.dilation[0] = dilation_;
  a.dilation[1] = 1;
  a.multiplier = multiplier_;
}

std::shared_ptr<Operation> Conv1d::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Conv1d>(static_cast<int32_t>(weights_), padding_, ksize_, stride_,
                                        dilation_, pad_, multiplier_, impl_->layout_, kernel_layout_);
}

void Conv1d::OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor, int32_t) {
  PromoteHalfBias(this, impl_.get(), tensor);
}

// ---- GroupedConv1d (reference: src/tim/vx/ops/groupedconv1d.cc:34-66) -------
GroupedConv1d::GroupedConv1d(Graph* graph, PadType padding, const uint32_t stride, const uint32_t dilation,
                             uint32_t group, DataLayout input_layout, DataLayout kernel_layout)
    : GroupedConv1d(graph, padding, {0, 0}, stride, dilation, group, input_layout, kernel_layout) {}

GroupedConv1d::GroupedConv1d(Graph* graph, PadType padding, std::array<uint32_t, 2> pad, uint32_t stride,
                             uint32_t dilation, uint32_t group, DataLayout input_layout, DataLayout kernel_layout)
    : BuiltinOp(graph, K(OpKind::CONV2D), 0, 0, input_layout),
      padding_(padding), pad_(pad), stride_(stride), dilation_(dilation), group_(group),
      kernel_layout_(kernel_layout) {
  OpAttrs& a = impl_->attrs_;
  a.kernel_layout = kernel_layout_;
  a.conv_1d = true;
  a.pad_type = padding_ == PadType::NONE ? PadType::AUTO : padding_;
  a.pad[0] = pad_[0];
  a.pad[1] = pad_[1];
  a.stride[0] = stride_;
  a.stride[1] = 1;
  a.dilation[0] = dilation_;
  a.dilation[1] = 1;
  a.groups = static_cast<int32_t>(group_);
}

std::shared_ptr<Operation> GroupedConv1d::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<GroupedConv1d>(padding_, pad_, stride_, dilation_, group_, impl_->layout_,
                                               kernel_layout_);
}

void GroupedConv1d::OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor, int32_t) {
  PromoteHalfBias(this, impl_.get(), tensor);
}

// ---- GroupedConv2d ----------------------------------------------------------
// The same operator kind as Conv2d with a group count (the reference has a kind of its own,
// VSI_NN_OP_GROUPED_CONV2D, whose setup splits into per-group convolutions:
// src/tim/vx/internal/src/ops/vsi_nn_op_grouped_conv2d.c).
GroupedConv2d::GroupedConv2d(Graph* graph, PadType padding,
                             const std::array<uint32_t, 2>& strides,
                             const std::array<uint32_t, 2>& dilation, int32_t grouped_number,
                             DataLayout input_layout, DataLayout kernel_layout)
    : BuiltinOp(graph, K(OpKind::CONV2D), 0, 0, input_layout),
      padding_(padding), strides_(strides), dilation_(dilation), pad_({0, 0, 0, 0}),
      group_number_(grouped_number), kernel_layout_(kernel_layout) {
  OpAttrs& a = impl_->attrs_;
  a.kernel_layout = kernel_layout_;
  a.pad_type = padding_ == PadType::NONE ? PadType::AUTO : padding_;
  for (int i = 0; i < 2; ++i) {
    a.stride[i] = strides_[i];
    a.dilation[i] = dilation_[i];
  }
  a.groups = group_number_;
}

GroupedConv2d::GroupedConv2d(Graph* graph, const std::array<uint32_t, 4>& pad,
                             const std::array<uint32_t, 2>& strides,
                             const std::array<uint32_t, 2>& dilation, int32_t group_number,
                             DataLayout input_layout, DataLayout kernel_layout)
    : BuiltinOp(graph, K(OpKind::CONV2D), 0, 0, input_layout),
      padding_(PadType::AUTO), strides_(strides), dilation_(dilation), pad_(pad),
      group_number_(group_number), kernel_layout_(kernel_layout) {
  OpAttrs& a = impl_->attrs_;
  a.kernel_layout = kernel_layout_;
  a.pad_type = PadType::AUTO;
  for (int i = 0; i < 4; ++i) a.pad[i] = pad_[i];
  for (int i = 0; i < 2; ++i) {
    a.stride[i] = strides_[i];
    a.dilation[i] = dilation_[i];
  }
  a.groups = group_number_;
}

std::shared_ptr<Operation> GroupedConv2d::Clone(std::shared_ptr<Graph>& graph) const {
  if (padding_ != PadType::AUTO)
    return graph->CreateOperation<GroupedConv2d>(padding_, strides_, dilation_, group_number_,
                                                 impl_->layout_, kernel_layout_);
  return graph->CreateOperation<GroupedConv2d>(pad_, strides_, dilation_, group_number_,
                                               impl_->layout_, kernel_layout_);
}

void GroupedConv2d::OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor, int32_t) {
  PromoteHalfBias(this, impl_.get(), tensor);
}

// ---- FullyConnected -------------------------------------------------------
FullyConnected::FullyConnected(Graph* graph, uint32_t axis)
    : FullyConnected(graph, axis, 0) {}

FullyConnected::FullyConnected(Graph* graph, uint32_t axis, uint32_t weights)
    : BuiltinOp(graph, K(OpKind::FCL)), axis_(axis), weights_(weights) {
  impl_->attrs_.axis = axis;
  impl_->attrs_.weights = weights;
}

std::shared_ptr<Operation> FullyConnected::Clone(
    std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<FullyConnected>(axis_, weights_);
}

void FullyConnected::OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor,
                                         int32_t) {
  PromoteHalfBias(this, impl_.get(), tensor);
}

// ---- Pool2d ---------------------------------------------------------------
Pool2d::Pool2d(Graph* graph, PoolType type, PadType padding,
               const std::array<uint32_t, 2>& ksize,
               const std::array<uint32_t, 2>& stride, RoundType round_type,
               DataLayout layout)
    : BuiltinOp(graph, K(OpKind::POOL), 1, 1, layout), type_(type),
      padding_(padding), ksize_(ksize), stride_(stride), round_type_(round_type),
      pad_({0, 0, 0, 0}) {
  Init();
}

Pool2d::Pool2d(Graph* graph, PoolType type, const std::array<uint32_t, 4>& pad,
               const std::array<uint32_t, 2>& ksize,
               const std::array<uint32_t, 2>& stride, RoundType round_type,
               DataLayout layout)
    : BuiltinOp(graph, K(OpKind::POOL), 1, 1, layout), type_(type),
      padding_(PadType::AUTO), ksize_(ksize), stride_(stride),
      round_type_(round_type), pad_(pad) {
  Init();
}

Pool2d::Pool2d(Graph* graph, PoolType type,
               const std::array<uint32_t, 2>& input_size, RoundType round_type,
               DataLayout layout)
    : BuiltinOp(graph, K(OpKind::POOL), 1, 1, layout), type_(type),
      padding_(PadType::AUTO), ksize_(input_size), stride_(input_size),
      round_type_(round_type), pad_({0, 0, 0, 0}) {
  Init();
}

Pool2d::Pool2d(Graph* graph, PoolType type,
               const std::array<uint32_t, 2>& input_size,
               const std::array<uint32_t, 2>& output_size, RoundType round_type,
               DataLayout layout)
    : BuiltinOp(graph, K(OpKind::POOL), 1, 1, layout), type_(type),
      padding_(PadType::AUTO), round_type_(round_type), pad_({0, 0, 0, 0}) {
  for (int i = 0; i < 2; ++i) {
    stride_[i] = input_size[i] / output_size[i];
    ksize_[i] = input_size[i] - (output_size[i] - 1) * stride_[i];
  }
  Init();
}

void Pool2d::Init() {
  OpAttrs& a = impl_->attrs_;
  a.pool_type = type_;
  a.round_type = round_type_;
  a.pad_type = padding_ == PadType::NONE ? PadType::AUTO : padding_;
  for (int i = 0; i < 2; ++i) {
    a.ksize[i] = ksize_[i];
    a.stride[i] = stride_[i];
  }
  for (int i = 0; i < 4; ++i) a.pad[i] = pad_[i];
  SetRoundingPolicy(OverflowPolicy::SATURATE, RoundingPolicy::RTNE, round_type_);
}

std::shared_ptr<Operation> Pool2d::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Pool2d>(type_, pad_, ksize_, stride_,
                                        round_type_, impl_->layout_);
}

// ---- Pool1d: a Pool2d over {W, 1, C, N} -----------------------------------
Pool1d::Pool1d(Graph* graph, PoolType type, PadType padding, uint32_t ksize,
               uint32_t stride, RoundType round_type, DataLayout layout)
    : BuiltinOp(graph, K(OpKind::POOL), 1, 1, layout), type_(type),
      padding_(padding), ksize_(ksize), stride_(stride), round_type_(round_type),
      pad_({0, 0}) {
  Init();
}

Pool1d::Pool1d(Graph* graph, PoolType type, const std::array<uint32_t, 2>& pad,
               uint32_t ksize, uint32_t stride, RoundType round_type,
               DataLayout layout)
    : BuiltinOp(graph, K(OpKind::POOL), 1, 1, layout), type_(type),
      padding_(PadType::AUTO), ksize_(ksize), stride_(stride),
      round_type_(round_type), pad_(pad) {
  Init();
}

Pool1d::Pool1d(Graph* graph, PoolType type, uint32_t input_size,
               RoundType round_type, DataLayout layout)
    : BuiltinOp(graph, K(OpKind::POOL), 1, 1, layout), type_(type),
      padding_(PadType::AUTO), ksize_(input_size), stride_(input_size),
      round_type_(round_type), pad_({0, 0}) {
  Init();
}

Pool1d::Pool1d(Graph* graph, PoolType type, uint32_t input_size,
               uint32_t output_size, RoundType round_type, DataLayout layout)
    : BuiltinOp(graph, K(OpKind::POOL), 1, 1, layout), type_(type),
      padding_(PadType::AUTO), round_type_(round_type), pad_({0, 0}) {
  stride_ = input_size / output_size;
  ksize_ = input_size - (output_size - 1) * stride_;
  Init();
}

void Pool1d::Init() {
  OpAttrs& a = impl_->attrs_;
  a.pool_1d = true;
  a.pool_type = type_;
  a.round_type = round_type_;
  a.pad_type = padding_ == PadType::NONE ? PadType::AUTO : padding_;
  a.ksize[0] = ksize_;
  a.ksize[1] = 1;
  a.stride[0] = stride_;
  a.stride[1] = 1;
  a.pad[0] = pad_[0];
  a.pad[1] = pad_[1];
  a.pad[2] = a.pad[3] = 0;
  SetRoundingPolicy(OverflowPolicy::SATURATE, RoundingPolicy::RTNE, round_type_);
}

std::shared_ptr<Operation> Pool1d::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Pool1d>(type_, pad_, ksize_, stride_,
                                        round_type_, impl_->layout_);
}

// ---- parameterless / small ops ---------------------------------------------
Relu::Relu(Graph* graph) : BuiltinOp(graph, K(OpKind::RELU)) {}
std::shared_ptr<Operation> Relu::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Relu>();
}

Relu6::Relu6(Graph* graph) : BuiltinOp(graph, K(OpKind::RELU6)) {}
std::shared_ptr<Operation> Relu6::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Relu6>();
}

Add::Add(Graph* graph) : BuiltinOp(graph, K(OpKind::ADD), 2, 1) {}
std::shared_ptr<Operation> Add::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Add>();
}

Softmax::Softmax(Graph* graph, float beta, int32_t axis)
    : BuiltinOp(graph, K(OpKind::SOFTMAX)), beta_(beta), axis_(axis) {
  impl_->attrs_.beta = beta;
  impl_->attrs_.sm_axis = axis;
}
std::shared_ptr<Operation> Softmax::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Softmax>(beta_, axis_);
}

Reshape::Reshape(Graph* graph, const std::vector<uint32_t>& target_shape)
    : BuiltinOp(graph, K(OpKind::RESHAPE), 1, 1), size_(target_shape) {
  impl_->attrs_.new_shape = target_shape;
}
std::shared_ptr<Operation> Reshape::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Reshape>(size_);
}

// ---- DeConv2d (reference: src/tim/vx/ops/deconv.cc:36-88) ------------------------------------
DeConv2d::DeConv2d(Graph* graph, int32_t oc_count, PadType pad_type, const std::array<uint32_t, 2>& ksize,
                   const std::array<uint32_t, 2>& stride, const std::array<uint32_t, 2>& output_padding,
                   DataLayout input_layout, DataLayout kernel_layout)
    : DeConv2d(graph, oc_count, pad_type, ksize, stride, output_padding, {0, 0, 0, 0}, 1, input_layout,
               kernel_layout) {}

DeConv2d::DeConv2d(Graph* graph, int32_t oc_count, PadType pad_type, const std::array<uint32_t, 2>& ksize,
                   const std::array<uint32_t, 2>& stride, const std::array<uint32_t, 2>& output_padding,
                   const std::array<uint32_t, 4>& pad, const uint32_t group, DataLayout input_layout,
                   DataLayout kernel_layout)
    : BuiltinOp(graph, K(OpKind::DECONV2D), 0, 0, input_layout),
      oc_count_(oc_count), pad_type_(pad_type), ksize_(ksize), stride_(stride),
      output_padding_(output_padding), pad_(pad), group_(group), kernel_layout_(kernel_layout) {
  OpAttrs& a = impl_->attrs_;
  a.kernel_layout = kernel_layout_;
  // the pad type is carried along but the explicit pads are what sizes the output, as in the
  // reference (vsi_nn_op_deconvolution.c:463-481)
  a.pad_type = PadType::AUTO;
  for (int i = 0; i < 4; ++i) a.pad[i] = pad_[i];
  for (int i = 0; i < 2; ++i) {
    a.stride[i] = stride_[i];
    a.ksize[i] = ksize_[i];
    a.output_padding[i] = output_padding_[i];
  }
  a.weights = oc_count_;
  a.groups = static_cast<int32_t>(group_);
}

std::shared_ptr<Operation> DeConv2d::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<DeConv2d>(static_cast<int32_t>(oc_count_), pad_type_, ksize_, stride_,
                                          output_padding_, pad_, group_, impl_->layout_, kernel_layout_);
}

void DeConv2d::OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor, int32_t) {
  PromoteHalfBias(this, impl_.get(), tensor);
}

// ---- DeConv1d (reference: src/tim/vx/ops/deconv1d.cc:36-98) ------------------------------------
DeConv1d::DeConv1d(Graph* graph, PadType pad_type, uint32_t stride, uint32_t output_padding, uint32_t group,
                   DataLayout input_layout, DataLayout kernel_layout)
    : DeConv1d(graph, pad_type, stride, output_padding, {0, 0}, group, input_layout, kernel_layout) {}

DeConv1d::DeConv1d(Graph* graph, const std::array<uint32_t, 2>& pad, uint32_t stride, uint32_t output_padding,
                   uint32_t group, DataLayout input_layout, DataLayout kernel_layout)
    : DeConv1d(graph, PadType::AUTO, stride, output_padding, pad, group, input_layout, kernel_layout) {}

DeConv1d::DeConv1d(Graph* graph, int32_t, PadType pad_type, uint32_t, uint32_t stride, uint32_t output_padding)
    : DeConv1d(graph, pad_type, stride, output_padding, {0, 0}, 1, DataLayout::WHCN, DataLayout::WHIcOc) {}

DeConv1d::DeConv1d(Graph* graph, int32_t, PadType pad_type, uint32_t, uint32_t stride, uint32_t output_padding,
                   const std::array<uint32_t, 2>& pad, uint32_t group)
    : DeConv1d(graph, pad_type, stride, output_padding, pad, group, DataLayout::WHCN, DataLayout::WHIcOc) {}

// (as in the reference, the channel count and kernel size arguments are not forwarded: the weight tensor has them)
DeConv1d::DeConv1d(Graph* graph, PadType pad_type, uint32_t stride, uint32_t output_padding,
                   const std::array<uint32_t, 2>& pad, uint32_t group, DataLayout input_layout,
                   DataLayout kernel_layout)
    : BuiltinOp(graph, K(OpKind::DECONV2D), 0, 0, input_layout),
      oc_count_(0), pad_type_(pad_type), ksize_(0), stride_(stride), output_padding_(output_padding), pad_(pad),
      group_(group), kernel_layout_(kernel_layout) {
  OpAttrs& a = impl_->attrs_;
  a.kernel_layout = kernel_layout_;
  a.conv_1d = true;
  a.pad_type = PadType::AUTO;  // the explicit pads size the output (vsi_nn_op_deconvolution1d.c:250-259)
  a.pad[0] = pad_[0];
  a.pad[1] = pad_[1];
  a.stride[0] = stride_;
  a.stride[1] = 1;
  a.output_padding[0] = output_padding_;
  a.output_padding[1] = 0;
  a.groups = static_cast<int32_t>(group_);
}

std::shared_ptr<Operation> DeConv1d::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<DeConv1d>(pad_type_, stride_, output_padding_, pad_, group_, impl_->layout_,
                                          kernel_layout_);
}

void DeConv1d::OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor, int32_t) {
  PromoteHalfBias(this, impl_.get(), tensor);
}

DataConvert::DataConvert(Graph* graph) : BuiltinOp(graph, K(OpKind::DATACONVERT), 1, 1) {}
std::shared_ptr<Operation> DataConvert::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<DataConvert>();
}

Transpose::Transpose(Graph* graph, const std::vector<uint32_t>& perm)
    : BuiltinOp(graph, K(OpKind::TRANSPOSE), 1, 1), perm_(perm) {
  impl_->attrs_.perm = perm;
}
std::shared_ptr<Operation> Transpose::Clone(std::shared_ptr<Graph>& graph) const {
  return graph->CreateOperation<Transpose>(perm_);
}

}  // namespace ops
}  // namespace vx
}  // namespace tim
