// The platform interfaces on this runtime (reference: src/tim/vx/platform/native.cc:43-330).
// The reference compiles a graph to a driver binary and replays it through an NBG node; here
// an executable keeps the source graph and, once its handles are bound, rebuilds it into a
// graph of its own whose inputs and outputs ARE the handles' tensors (the same walk layout
// inference does, so CWHN sources are accepted as well), compiles that and runs it.
#include <algorithm>

#include "runtime.h"
#include "tim/vx/platform/native.h"
#include "tvx_hip.h"

namespace tim {
namespace vx {
namespace platform {
namespace {

class TensorHandleImpl : public NativeTensorHandle {
 public:
  explicit TensorHandleImpl(const std::shared_ptr<Tensor>& tensor) {
    tensor_ = tensor;
    spec_ = tensor->GetSpec();
  }
  bool CopyDataToTensor(const void* data, uint32_t size_in_bytes) override {
    return tensor_->CopyDataToTensor(data, size_in_bytes);
  }
  bool CopyDataFromTensor(void* data) override { return tensor_->CopyDataFromTensor(data); }
};

class ExecutorImpl;

class ExecutableImpl : public NativeExecutable {
 public:
  ExecutableImpl(const std::shared_ptr<IExecutor>& executor, const std::shared_ptr<Graph>& source)
      : source_(source) {
    executor_ = executor;
    context_ = executor->Contex();
    // (reference: native.cc:300-303 - the executable's graph is compiled for the executor's device)
    CompileOption option;
    option.setDeviceId(executor->Device()->Id());
    nb_graph_ = context_->CreateGraph(option);
  }
  void SetInput(const std::shared_ptr<ITensorHandle>& th) override { input_handles_.push_back(th); }
  void SetOutput(const std::shared_ptr<ITensorHandle>& th) override { output_handles_.push_back(th); }
  void SetInputs(const std::vector<std::shared_ptr<ITensorHandle>>& ths) override {
    for (auto& t : ths) SetInput(t);
  }
  void SetOutputs(const std::vector<std::shared_ptr<ITensorHandle>>& ths) override {
    for (auto& t : ths) SetOutput(t);
  }
  bool Submit(const std::shared_ptr<IExecutable>& ref, bool after) override {
    auto ex = executor_.lock();
    return ex && ex->Submit(shared_from_this(), ref, after);
  }
  bool Trigger(bool) override { return Verify() && nb_graph_->Run(); }
  std::shared_ptr<ITensorHandle> AllocateTensor(const TensorSpec& spec, void* data, uint32_t) override {
    return std::make_shared<TensorHandleImpl>(nb_graph_->CreateTensor(spec, data));
  }
  // Binds the handles (in the order of the source graph's inputs / outputs) and compiles, once.
  bool Verify() override {
    if (state_ != 0) return state_ > 0;
    state_ = -1;
    const auto ins = source_->InputsTensor(), outs = source_->OutputsTensor();
    if (ins.size() != input_handles_.size() || outs.size() != output_handles_.size()) {
      VSILOGE("executable: %zu / %zu handles bound for a graph with %zu inputs / %zu outputs",
              input_handles_.size(), output_handles_.size(), ins.size(), outs.size());
      return false;
    }
    std::map<std::shared_ptr<Tensor>, std::shared_ptr<Tensor>> io;
    auto bind = [&](const std::shared_ptr<Tensor>& t, const std::shared_ptr<ITensorHandle>& h, const char* what) {
      auto ht = h->GetTensor();
      if (!ht || static_cast<TensorImpl*>(ht.get())->graph_ != static_cast<GraphImpl*>(nb_graph_.get())) {
        VSILOGE("executable: an %s handle was not allocated by this executable", what);
        return false;
      }
      if (ht->GetSpec().datatype_ != t->GetSpec().datatype_ ||
          ht->GetSpec().GetElementNum() != t->GetSpec().GetElementNum()) {
        VSILOGE("executable: an %s handle does not match tensor %u of the graph", what, t->GetId());
        return false;
      }
      io[t] = ht;
      return true;
    };
    for (size_t i = 0; i < ins.size(); ++i)
      if (!bind(ins[i], input_handles_[i], "input")) return false;
    for (size_t i = 0; i < outs.size(); ++i)
      if (!bind(outs[i], output_handles_[i], "output")) return false;
    if (!transform::RewriteInto(source_, nb_graph_, {}, &io)) return false;
    if (!nb_graph_->Compile()) return false;
    state_ = 1;
    return true;
  }

 private:
  std::shared_ptr<Graph> source_;
  int state_ = 0;  // 0 = not verified, 1 = compiled, -1 = failed
};

class ExecutorImpl : public NativeExecutor, public std::enable_shared_from_this<ExecutorImpl> {
 public:
  ExecutorImpl(const std::shared_ptr<IDevice>& device, int32_t core_index, int32_t core_count,
               const std::shared_ptr<Context>& context) {
    device_ = device;
    context_ = context ? context : Context::Create();
    const int32_t total = static_cast<int32_t>(device->CoreCount());
    core_index_ = static_cast<uint32_t>(std::min(std::max(core_index, 0), std::max(total - 1, 0)));
    core_count_ = static_cast<uint32_t>(core_count <= 0 ? total - static_cast<int32_t>(core_index_)
                                                         : std::min(core_count, total - static_cast<int32_t>(core_index_)));
  }
  bool Submit(const std::shared_ptr<IExecutable>& executable, const std::shared_ptr<IExecutable>& ref,
              bool after) override {
    if (!executable || !executable->Verify()) {
      VSILOGE("executor: the executable does not compile");
      return false;
    }
    if (executable == ref) {
      tasks_.push_back(executable);
      return true;
    }
    for (size_t i = 0; i < tasks_.size(); ++i)
      if (tasks_[i].lock() == ref) {
        tasks_.insert(tasks_.begin() + i + (after ? 1 : 0), executable);
        return true;
      }
    return false;
  }
  bool Trigger(bool) override {
    bool ok = !tasks_.empty();
    while (!tasks_.empty()) {
      auto t = tasks_.front().lock();
      tasks_.erase(tasks_.begin());
      if (!t) {
        VSILOGE("executor: a submitted executable no longer exists");
        return false;
      }
      ok = t->Trigger() && ok;
    }
    device_->WaitDeviceIdle();
    return ok;
  }
  std::shared_ptr<IExecutable> Compile(const std::shared_ptr<Graph>& graph) override {
    if (!graph) return nullptr;
    if (device_->Id() != 0) {
      VSILOGE("executor: running on a GPU other than the process's current one is not implemented");
      return nullptr;
    }
    return std::make_shared<ExecutableImpl>(shared_from_this(), graph);
  }
};

class DeviceImpl : public NativeDevice, public std::enable_shared_from_this<DeviceImpl> {
 public:
  explicit DeviceImpl(device_id_t id) {
    device_id_ = id;
    core_count_ = 1;  // a GPU is handed out whole
  }
  bool Submit(const std::shared_ptr<Graph>& graph) override {
    if (!graph) return false;
    queue_.push_back(graph);
    return true;
  }
  bool Trigger(bool, async_callback) override {
    bool ok = !queue_.empty();
    for (auto& g : queue_) ok = g->Compile() && g->Run() && ok;
    queue_.clear();
    return ok;
  }
  void WaitDeviceIdle() override {}  // Graph::Run() returns with the results on the host
  bool DeviceExit() override { return true; }
  std::shared_ptr<IExecutor> CreateExecutor(const int32_t core_index, const int32_t core_count,
                                            const std::shared_ptr<Context>& context) override {
    return std::make_shared<ExecutorImpl>(shared_from_this(), core_index, core_count, context);
  }

 private:
  std::vector<std::shared_ptr<Graph>> queue_;
};

}  // namespace

std::shared_ptr<IExecutable> Compile(const std::shared_ptr<Graph>& graph, const std::shared_ptr<IExecutor>& executor) {
  return executor ? executor->Compile(graph) : nullptr;
}

std::vector<std::shared_ptr<IDevice>> NativeDevice::Enumerate() {
  std::vector<std::shared_ptr<IDevice>> out;
  const int n = tvx_device_count();
  for (int i = 0; i < n; ++i) out.push_back(std::make_shared<DeviceImpl>(static_cast<uint32_t>(i)));
  return out;
}

std::vector<std::shared_ptr<IDevice>> IDevice::Enumerate() { return NativeDevice::Enumerate(); }

}  // namespace platform
}  // namespace vx
}  // namespace tim
