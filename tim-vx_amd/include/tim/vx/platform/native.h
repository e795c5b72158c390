// The in-process back end of the platform interfaces: the GPUs of this machine
// (reference: include/tim/vx/platform/native.h:33-83).
#pragma once
#include "tim/vx/platform/platform.h"

namespace tim {
namespace vx {
namespace platform {

class NativeDevice : public IDevice {
 public:
  // one device per GPU the runtime sees; empty without a GPU
  static std::vector<std::shared_ptr<IDevice>> Enumerate();
};
class NativeExecutable : public IExecutable {};
class NativeExecutor : public IExecutor {};
class NativeTensorHandle : public ITensorHandle {};

}  // namespace platform
}  // namespace vx
}  // namespace tim
