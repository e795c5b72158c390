// tim::vx core object model (Context / Graph / Tensor / Operation) as seen by
// applications. One translation unit of declarations; the per-name headers
// next to this directory only forward here.
//
// The class names, member signatures and the order of virtual functions are
// the contract applications compile against in the reference
// (include/tim/vx/{types,tensor,graph,context,operation,builtin_op,
// compile_option}.h); everything behind OpImpl / the concrete Graph and
// Tensor classes belongs to this runtime.
#pragma once

#include <array>
#include <cstddef>
#include <cstdint>
#include <iostream>
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace tim {
namespace vx {

// ---- enumerations (reference: include/tim/vx/types.h:30-89) ---------------
enum class DataType {
  UNKNOWN, INT8, UINT8, INT16, UINT16, INT32, UINT32, INT64,
  FLOAT16, FLOAT32, BOOL8, INT4, UINT4
};
enum class QuantType {
  NONE, ASYMMETRIC, SYMMETRIC_PER_CHANNEL, ASYMMETRIC_PER_CHANNEL,
  DYNAMIC_FIXED_POINT
};
enum TensorAttribute {
  CONSTANT = 1 << 0, TRANSIENT = 1 << 1, VARIABLE = 1 << 2,
  INPUT = 1 << 3, OUTPUT = 1 << 4
};
enum class PadType { NONE = -1, AUTO, VALID, SAME };
enum class PoolType { MAX, AVG, L2, AVG_ANDROID };
enum class RoundType { CEILING, FLOOR };
enum class OverflowPolicy { WRAP, SATURATE };
enum class RoundingPolicy { TO_ZERO, RTNE };
enum class ResizeType { NEAREST_NEIGHBOR, BILINEAR, AREA };
enum class DataLayout {
  ANY, WHCN, CWHN, IcWHOc, OcIcWH, IcOcWH, WHIcOc, WCN, WIcOc,
  WHDCN, WHDIcOc, CWHDN, OcIcWHD
};

// dim 0 is the fastest-varying one (W of WHCN).
using ShapeType = std::vector<uint32_t>;

// ---- Quantization (reference: include/tim/vx/tensor.h:40-89) --------------
class Quantization {
 public:
  Quantization() : type_(QuantType::NONE) {}
  Quantization(QuantType type, float scale, int32_t zero_point)
      : type_(type), scales_({scale}), zero_points_({zero_point}) {}
  Quantization(QuantType type, int32_t channel_dim, std::vector<float> scales,
               std::vector<int32_t> zero_points)
      : type_(type), channel_dim_(channel_dim), scales_(std::move(scales)),
        zero_points_(std::move(zero_points)) {}
  Quantization(QuantType type, int8_t fl) : type_(type), fl_(fl) {}

  QuantType& Type() { return type_; }
  const QuantType& Type() const { return type_; }
  Quantization& SetType(QuantType t) { type_ = t; return *this; }

  int32_t& ChannelDim() { return channel_dim_; }
  const int32_t& ChannelDim() const { return channel_dim_; }
  Quantization& SetChannelDim(int32_t d) { channel_dim_ = d; return *this; }

  std::vector<float>& Scales() { return scales_; }
  const std::vector<float>& Scales() const { return scales_; }
  Quantization& SetScales(std::vector<float> s) { scales_ = s; return *this; }

  std::vector<int32_t>& ZeroPoints() { return zero_points_; }
  const std::vector<int32_t>& ZeroPoints() const { return zero_points_; }
  Quantization& SetZeroPoints(std::vector<int32_t> z) {
    zero_points_ = z;
    return *this;
  }

  const std::int8_t& Fl() const { return fl_; }
  bool operator==(const Quantization& rhs) const;

 protected:
  QuantType type_{QuantType::NONE};
  int32_t channel_dim_{-1};
  std::vector<float> scales_;
  std::vector<int32_t> zero_points_;
  int8_t fl_ = 0;
};

// ---- TensorSpec (reference: include/tim/vx/tensor.h:91-137) ---------------
struct TensorSpec {
  TensorSpec() {}
  TensorSpec(DataType datatype, const ShapeType& shape, TensorAttribute attr)
      : datatype_(datatype), shape_(shape), attr_(attr) {}
  TensorSpec(DataType datatype, const ShapeType& shape, TensorAttribute attr,
             const Quantization& quantization)
      : TensorSpec(datatype, shape, attr) {
    quantization_ = quantization;
  }
  TensorSpec(const TensorSpec& other);
  bool operator==(const TensorSpec& rhs) const;
  TensorSpec& operator=(const TensorSpec& other);

  TensorSpec& SetDataType(DataType datatype);
  TensorSpec& SetShape(const ShapeType& shape);
  TensorSpec& SetAttribute(TensorAttribute attr);
  TensorSpec& SetQuantization(Quantization& quantization);
  TensorSpec AsTransientSpec() const;
  int64_t GetElementNum() const;
  int64_t GetElementByteSize() const;
  int64_t GetByteSize() const;

  inline DataType& GetDataType() { return datatype_; }
  inline ShapeType& GetShapeType() { return shape_; }
  inline TensorAttribute& GetTensorAttribute() { return attr_; }
  inline Quantization& GetQuantization() { return quantization_; }

  DataType datatype_;
  ShapeType shape_;
  TensorAttribute attr_;
  Quantization quantization_;
};

struct DmaBufferDesc {
  int64_t fd;
};

// ---- Tensor (reference: include/tim/vx/tensor.h:143-169) ------------------
class Tensor {
 public:
  virtual ~Tensor() {}
  virtual const ShapeType& GetShape() = 0;
  virtual DataType GetDataType() = 0;
  virtual const Quantization& GetQuantization() = 0;
  virtual TensorSpec& GetSpec() = 0;
  virtual uint32_t GetId() = 0;
  // size_in_bytes is accepted and ignored: the whole tensor is always copied
  // (reference: src/tim/vx/tensor.cc:154-166).
  virtual bool CopyDataToTensor(const void* data,
                                uint32_t size_in_bytes = 0) = 0;
  virtual bool CopyDataFromTensor(void* data) = 0;
  virtual bool SwapHandle(void* new_ptr, bool is_new_ptr_malloc_by_ovxlib,
                          void** old_ptr) = 0;
  virtual bool SwapHandle(std::shared_ptr<tim::vx::Tensor> tensor) = 0;
  virtual bool SwapHandleWithCache(std::shared_ptr<tim::vx::Tensor> tensor) = 0;
  virtual bool FlushCacheForHandle() = 0;
  virtual bool InvalidateCacheForHandle() = 0;
  virtual void* map(bool invalidate_cpu_cache = false) = 0;
  virtual void unmap() = 0;
  virtual bool IsPlaceHolder() = 0;
  virtual bool IsConstTensor() = 0;
  virtual bool IsScalar() = 0;
  virtual bool SaveTensorToTextByFp32(std::string filename) = 0;
  virtual void SetScalar(int8_t is_scalar) = 0;
  virtual void* ConvertTensorToData(uint8_t* tensorData) = 0;
  virtual float* ConvertTensorToFloat32Data() = 0;
};

namespace utils {
bool Float32ToDtype(std::shared_ptr<tim::vx::Tensor> tensor,
                    std::vector<float> fval, uint8_t* tensorData);
bool DtypeToFloat32(std::shared_ptr<tim::vx::Tensor> tensor,
                    uint8_t* tensorData, float* data);
}  // namespace utils

// ---- CompileOption (reference: include/tim/vx/compile_option.h:37-57) -----
struct CompileOptionImpl;
class CompileOption {
 public:
  CompileOption();
  ~CompileOption() {}
  bool isRelaxMode() const;
  bool setRelaxMode(bool enable = false);
  // The GPU a graph compiles for (platform::IDevice::device_id_t, the index IDevice::Enumerate() numbers devices
  // by; reference: compile_option.h:45-48, consumed at graph.cc:345-348). A graph whose index names no GPU of the
  // machine does not compile.
  void setDeviceId(uint32_t device);
  uint32_t getDeviceId();
  static CompileOption DefaultOptions;

 private:
  std::shared_ptr<CompileOptionImpl> impl_;
};

class Operation;

// ---- Graph (reference: include/tim/vx/graph.h:48-116) ---------------------
class Graph {
 public:
  virtual ~Graph() {}
  virtual void SetCompileOption(const CompileOption&) = 0;
  virtual std::shared_ptr<Tensor> CreateTensor(const TensorSpec& spec,
                                               const void* data = nullptr) = 0;
  virtual std::shared_ptr<Tensor> CreateTensor(const TensorSpec& spec,
                                               const DmaBufferDesc& dmafd) = 0;
  virtual std::shared_ptr<Tensor> CreateIOTensor(const TensorSpec& spec,
                                                 void* data = nullptr) = 0;
  virtual std::shared_ptr<Tensor> CreateTensorPlaceHolder() = 0;
  virtual bool Compile() = 0;
  virtual bool CompileToBinary(void* buf, size_t* size) = 0;
  virtual bool Run() = 0;

  template <typename OpType, typename... Params>
  std::shared_ptr<OpType> CreateOperation(Params... parameters) {
    auto op = std::make_shared<OpType>(this, parameters...);
    op_vector_.push_back(op);
    return op;
  }

  virtual const std::vector<std::shared_ptr<Tensor>> InputsTensor() const = 0;
  virtual const std::vector<std::shared_ptr<Tensor>> OutputsTensor() const = 0;
  virtual void UpdateTensorConsumersMap(const std::shared_ptr<Tensor>& tensor,
                                        const Operation* op) = 0;
  virtual void RenewTensorConsumersMap(
      const std::shared_ptr<Tensor>& org_tensor,
      const std::shared_ptr<Tensor>& dst_tensor, const Operation* op) = 0;
  virtual void UpdateTensorProducerMap(const std::shared_ptr<Tensor>& tensor,
                                       const Operation* op) = 0;
  virtual const std::vector<std::shared_ptr<Operation>> GetConsumersOp(
      std::shared_ptr<Tensor> tensor) const = 0;
  virtual std::shared_ptr<Operation> GetProducerOp(
      std::shared_ptr<Tensor> tensor) = 0;
  virtual void PrintGraph() const = 0;
  const std::vector<std::shared_ptr<Tensor>> GetConstantInputs() const;
  virtual std::vector<std::shared_ptr<Operation>>& OpVector() = 0;
  virtual std::map<std::shared_ptr<Tensor>,
                   std::vector<std::shared_ptr<Operation>>>&
  TensorConsumer() = 0;
  virtual std::map<std::shared_ptr<Tensor>, std::shared_ptr<Operation>>&
  TensorProducer() = 0;

 protected:
  std::vector<std::shared_ptr<tim::vx::Operation>> op_vector_;
};

// ---- Context (reference: include/tim/vx/context.h:34-44) ------------------
class Context {
 public:
  virtual ~Context() {}
  virtual std::shared_ptr<Graph> CreateGraph() = 0;
  virtual std::shared_ptr<Graph> CreateGraph(const CompileOption& options) = 0;
  virtual bool isClOnly() = 0;
  virtual bool hasSP() = 0;
  static std::shared_ptr<Context> Create();
};

// ---- Operation / BuiltinOp (reference: include/tim/vx/operation.h:35-64,
//      include/tim/vx/builtin_op.h:32-36) -----------------------------------
class OpImpl;

class Operation {
 public:
  Operation();
  virtual ~Operation();
  virtual std::shared_ptr<Operation> Clone(
      std::shared_ptr<Graph>& graph) const = 0;
  // Inputs are positional: activation, weight, optional bias.
  Operation& BindInput(const std::shared_ptr<Tensor>& tensor);
  Operation& BindOutput(const std::shared_ptr<Tensor>& tensor);
  Operation& BindInputs(const std::vector<std::shared_ptr<Tensor>>& tensors);
  Operation& BindOutputs(const std::vector<std::shared_ptr<Tensor>>& tensors);
  Operation& SetRoundingPolicy(
      OverflowPolicy overflow_policy = OverflowPolicy::SATURATE,
      RoundingPolicy rounding_policy = RoundingPolicy::RTNE,
      RoundType down_scale_size_rounding = RoundType::FLOOR,
      uint32_t accumulator_bits = 0);
  std::unique_ptr<OpImpl>& impl();
  const std::unique_ptr<OpImpl>& impl() const;
  const uint32_t& uid() const;
  virtual const std::vector<std::shared_ptr<Tensor>> ConstantInputsTensor()
      const;

 protected:
  bool IsAllInputsConst() const;
  std::unique_ptr<OpImpl> impl_;

 private:
  virtual void OnBindInputPostProc(const std::shared_ptr<Tensor>& tensor,
                                   int32_t input_idx);
};

#define DirectMapOp BuiltinOp
class BuiltinOp : public Operation {
 public:
  BuiltinOp(Graph* graph, uint32_t kind, int in_cnt = 0, int out_cnt = 0,
            DataLayout layout = DataLayout::ANY);
};

}  // namespace vx
}  // namespace tim
