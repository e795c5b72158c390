// Whole-graph scheduling interfaces: tensor handle, executable, executor, device.
// reference: include/tim/vx/platform/platform.h:56-145 (same names, signatures and protected members,
// so code written against the reference compiles unchanged). Here a device is one GPU, an executor an
// ordered queue of executables on it, an executable a graph compiled for that GPU whose inputs and
// outputs are the tensors behind handles the caller got from AllocateTensor().
#pragma once
#include <functional>
#include <memory>
#include <vector>

#include "tim/vx/context.h"
#include "tim/vx/graph.h"
#include "tim/vx/tensor.h"

namespace tim {
namespace vx {
namespace platform {

class IDevice;
class IExecutor;
class IExecutable;

// A tensor of an executable's graph, as the caller sees it.
class ITensorHandle {
 public:
  virtual ~ITensorHandle() {}
  virtual bool CopyDataToTensor(const void* data, uint32_t size_in_bytes) = 0;
  virtual bool CopyDataFromTensor(void* data) = 0;
  virtual std::shared_ptr<Tensor> GetTensor() const { return tensor_; }
  virtual TensorSpec& GetSpec() { return spec_; }

 protected:
  std::shared_ptr<Tensor> tensor_;
  TensorSpec spec_;
};

// A compiled graph. Handles bind in the order of the source graph's InputsTensor() / OutputsTensor().
class IExecutable : public std::enable_shared_from_this<IExecutable> {
 public:
  virtual ~IExecutable() {}
  virtual void SetInput(const std::shared_ptr<ITensorHandle>& th) = 0;
  virtual void SetOutput(const std::shared_ptr<ITensorHandle>& th) = 0;
  virtual void SetInputs(const std::vector<std::shared_ptr<ITensorHandle>>& ths) = 0;
  virtual void SetOutputs(const std::vector<std::shared_ptr<ITensorHandle>>& ths) = 0;
  virtual std::vector<std::shared_ptr<ITensorHandle>> GetOutputs() { return output_handles_; }
  virtual std::vector<std::shared_ptr<ITensorHandle>> Getinputs() { return input_handles_; }
  // queue this executable on its executor relative to `ref` (see IExecutor::Submit)
  virtual bool Submit(const std::shared_ptr<IExecutable>& ref, bool after = true) = 0;
  virtual bool Trigger(bool async = false) = 0;  // run now
  virtual bool Verify() = 0;                     // bind the handles and compile (once)
  std::shared_ptr<Graph> NBGraph() const { return nb_graph_; }
  virtual std::shared_ptr<ITensorHandle> AllocateTensor(const TensorSpec& tensor_spec, void* data = nullptr,
                                                        uint32_t size = 0) = 0;

 protected:
  std::weak_ptr<IExecutor> executor_;
  std::shared_ptr<Context> context_;
  std::shared_ptr<Graph> nb_graph_;  // the graph that runs (a rebuilt copy of the source graph, not a binary)
  std::vector<std::shared_ptr<ITensorHandle>> input_handles_;
  std::vector<std::shared_ptr<ITensorHandle>> output_handles_;
};

// An ordered queue of executables on one device.
class IExecutor {
 public:
  using task = std::weak_ptr<IExecutable>;
  virtual ~IExecutor() {}
  // executable == ref appends; otherwise it goes right behind (after) or in front of `ref`
  virtual bool Submit(const std::shared_ptr<IExecutable>& executable, const std::shared_ptr<IExecutable>& ref,
                      bool after = true) = 0;
  virtual bool Trigger(bool async = false) = 0;  // runs the queue front to back and empties it
  virtual std::shared_ptr<IExecutable> Compile(const std::shared_ptr<Graph>& graph) = 0;
  virtual std::shared_ptr<IDevice> Device() const { return device_; }
  virtual std::shared_ptr<Context> Contex() const { return context_; }
  virtual uint32_t CoreIndex() const { return core_index_; }
  virtual uint32_t CoreCount() const { return core_count_; }

 protected:
  std::vector<task> tasks_;
  std::shared_ptr<IDevice> device_;
  std::shared_ptr<Context> context_;
  uint32_t core_index_ = 0;
  uint32_t core_count_ = 0;
};

// One GPU.
class IDevice {
 public:
  using device_id_t = uint32_t;
  using async_callback = std::function<bool(const void*)>;
  using data_t = const void*;
  virtual ~IDevice() {}
  static std::vector<std::shared_ptr<IDevice>> Enumerate();
  device_id_t Id() const { return device_id_; }
  uint32_t CoreCount() const { return core_count_; }
  // whole graphs queued on the device itself: Trigger compiles (first time) and runs them in order
  // (virtual functions keep the reference's order)
  virtual bool Submit(const std::shared_ptr<Graph>& graph) = 0;
  virtual bool Trigger(bool async = false, async_callback cb = NULL) = 0;
  virtual void WaitDeviceIdle() = 0;
  virtual bool DeviceExit() = 0;
  virtual void RemoteReset() {}
  virtual std::shared_ptr<IExecutor> CreateExecutor(const int32_t core_index = 0, const int32_t core_count = -1,
                                                    const std::shared_ptr<Context>& context = nullptr) = 0;

 protected:
  device_id_t device_id_ = 0;
  uint32_t core_count_ = 0;
};

// executor->Compile(graph)
std::shared_ptr<IExecutable> Compile(const std::shared_ptr<Graph>& graph, const std::shared_ptr<IExecutor>& executor);

}  // namespace platform
}  // namespace vx
}  // namespace tim
