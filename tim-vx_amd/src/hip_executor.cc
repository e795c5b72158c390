// Executor of a compiled tim::vx graph on the GPU, reaching it only through the
// C ABI of include/tvx_hip.h (this file needs no HIP header).
//
// Realize() is the counterpart of vsi_nn_SetupGraph's compute_node pass plus
// vxVerifyGraph (src/tim/vx/internal/src/vsi_nn_graph.c:389-467,1591-1603): every
// operator becomes one tvx_op (the vx_node analogue), constants are uploaded and
// re-packed, and Conv2d / FullyConnected followed by Relu / Relu6 through a
// single-consumer TRANSIENT tensor with the same quantization are fused into the
// producer's epilogue - the fusion the closed driver performs itself.
// Execute() is vsi_nn_RunGraph -> vxProcessGraph (vsi_nn_graph.c:1605-1639):
// inputs go host -> device, operators run in order on one stream, outputs come
// back, and the call returns when everything is visible to the host.
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>

#include "runtime.h"
#include <utility>

#include "tvx_hip.h"

namespace tim {
namespace vx {
namespace {

double g_last_device_ms = 0.0;
// Profiling of Graph::Run(): -1 follows TVX_RUNTIME_PROFILE in the environment (unset: off, "ops": per operator, anything
// else: the operator sequence as a whole); 0 / 1 / 2 are set by tvx_runtime_set_profile().
std::atomic<int> g_profile_mode{-1};
// Per-operator device time of the most recent Graph::Run() (TVX_RUNTIME_PROFILE=ops): name and microseconds.
std::vector<std::pair<std::string, double>> g_last_op_us;
std::vector<uint64_t> g_last_op_bytes;

int DtypeCode(DataType t) {
  switch (t) {
    case DataType::UINT8: return TVX_U8;
    case DataType::INT8: return TVX_I8;
    case DataType::FLOAT16: return TVX_F16;
    case DataType::FLOAT32: return TVX_F32;
    default: return -1;
  }
}

float ScaleOf(const TensorSpec& s) {
  return s.quantization_.Scales().empty() ? 1.0f : s.quantization_.Scales()[0];
}
int32_t ZpOf(const TensorSpec& s) {
  return s.quantization_.ZeroPoints().empty() ? 0 : s.quantization_.ZeroPoints()[0];
}
bool IsQuantSpec(const TensorSpec& s) {
  return s.datatype_ == DataType::UINT8 || s.datatype_ == DataType::INT8;
}

struct Step {
  tvx_op* op = nullptr;
  TensorImpl* in0 = nullptr;
  TensorImpl* in1 = nullptr;  // run-time weights / second Add operand
  TensorImpl* in2 = nullptr;  // run-time bias
  TensorImpl* out = nullptr;
  // a channel-blocked copy of a tensor that stays in WHCN order for its other readers stands in for in0 / in1 / out
  void* blocked_in0 = nullptr;
  void* blocked_in1 = nullptr;
  void* blocked_out = nullptr;
  std::string name;
  uint64_t bytes = 0;  // tensor bytes the step has to move: its operands and its result
};

class HipExecutor : public Executor {
 public:
  ~HipExecutor() override {
    for (auto& s : steps_) tvx_op_destroy(s.op);
    for (void* e : events_) (void)tvx_event_destroy(e);
    for (auto& kv : owned_) tvx_free(kv.second);
    for (auto& kv : blocked_copy_) tvx_free(kv.second);
    if (stream_) tvx_stream_destroy(stream_);
  }

  bool Realize(GraphImpl* graph) override {
    if (tvx_device_count() <= 0) {
      VSILOGE("no GPU: this runtime has no CPU execution path");
      return false;
    }
    // the device the graph was compiled for (reference: graph.cc:345-348, VX_GRAPH_DEVICE_INDEX_VIV): this runtime
    // drives the process's current GPU, index 0
    const uint32_t device = graph->options_.getDeviceId();
    if (device >= static_cast<uint32_t>(tvx_device_count()) || device != 0) {
      VSILOGE("graph compiled for device %u: this runtime runs on device 0 of %d", device, tvx_device_count());
      return false;
    }
    if (tvx_stream_create(&stream_) != TVX_OK) return Fail("stream");
    // ---- activation fusion plan ------------------------------------------------
    std::map<Operation*, Operation*> fused_act;  // producer -> activation folded into it
    std::map<Operation*, bool> skipped;
    for (Operation* op : graph->sorted_ops_) {
      OpImpl* im = op->impl().get();
      if (im->kind_ != OpKind::CONV2D && im->kind_ != OpKind::FCL) continue;
      auto mid = im->outputs_tensor_[0];
      if (!(mid->GetSpec().attr_ & TensorAttribute::TRANSIENT)) continue;
      auto consumers = graph->GetConsumersOp(mid);
      if (consumers.size() != 1) continue;
      OpImpl* act = consumers[0]->impl().get();
      if (act->kind_ != OpKind::RELU && act->kind_ != OpKind::RELU6) continue;
      const TensorSpec &ms = mid->GetSpec(), &os = act->outputs_tensor_[0]->GetSpec();
      if (ms.datatype_ != os.datatype_) continue;
      if (IsQuantSpec(ms) && (ScaleOf(ms) != ScaleOf(os) || ZpOf(ms) != ZpOf(os))) continue;
      fused_act[op] = consumers[0].get();
      skipped[consumers[0].get()] = true;
    }
    // ---- residual fusion plan: a convolution whose TRANSIENT result only feeds a same-type Add, the
    // Add's other operand being there before the convolution runs, may become one operator
    std::map<Operation*, AddFusion> fused_add;  // convolution -> the Add folded into it
    std::map<Tensor*, size_t> produced_at;  // position of the operator that writes a tensor
    for (size_t i = 0; i < graph->sorted_ops_.size(); ++i)
      for (auto& t : graph->sorted_ops_[i]->impl()->outputs_tensor_) produced_at[t.get()] = i;
    if (!std::getenv("TVX_NO_RESIDUAL_FUSION")) {  // tuning aid: keep the Adds as operators of their own
      for (size_t i = 0; i < graph->sorted_ops_.size(); ++i) {
        Operation* add = graph->sorted_ops_[i];
        OpImpl* aim = add->impl().get();
        if (aim->kind_ != OpKind::ADD || aim->inputs_tensor_.size() != 2) continue;
        for (int k = 0; k < 2; ++k) {
          auto mid = aim->inputs_tensor_[k];
          auto other = aim->inputs_tensor_[1 - k];
          auto pit = produced_at.find(mid.get());
          if (pit == produced_at.end() || !(mid->GetSpec().attr_ & TensorAttribute::TRANSIENT)) continue;
          Operation* conv = graph->sorted_ops_[pit->second];
          OpImpl* cim = conv->impl().get();
          if (cim->kind_ != OpKind::CONV2D || cim->attrs_.conv_1d || fused_act.count(conv) || fused_add.count(conv)) continue;
          if (graph->GetConsumersOp(mid).size() != 1 || mid == other) continue;
          auto oit = produced_at.find(other.get());
          if (oit != produced_at.end() && oit->second >= pit->second) continue;  // not there yet when the convolution runs
          fused_add[conv] = AddFusion{add, k + 1};
          break;
        }
      }
    }
    // ---- depthwise -> pointwise plan: a depthwise convolution (with the activation folded into it) whose
    // TRANSIENT result only feeds a 1x1 convolution may become one operator with it
    std::map<Operation*, Operation*> fused_dwpw;  // depthwise convolution -> the pointwise one folded into it
    if (!std::getenv("TVX_NO_DWPW_FUSION")) {  // tuning aid: keep the two convolutions apart
      for (Operation* op : graph->sorted_ops_) {
        OpImpl* im = op->impl().get();
        if (im->kind_ != OpKind::CONV2D || im->attrs_.multiplier != 1 || im->attrs_.conv_1d || fused_add.count(op)) continue;
        auto fa = fused_act.find(op);
        auto mid = fa != fused_act.end() ? fa->second->impl()->outputs_tensor_[0] : im->outputs_tensor_[0];
        if (!(mid->GetSpec().attr_ & TensorAttribute::TRANSIENT)) continue;
        auto consumers = graph->GetConsumersOp(mid);
        if (consumers.size() != 1) continue;
        OpImpl* pim = consumers[0]->impl().get();
        if (pim->kind_ != OpKind::CONV2D || pim->attrs_.multiplier != 0 || pim->attrs_.conv_1d ||
            pim->inputs_tensor_[0] != mid)
          continue;
        // The merged kernel's strength is latency, not throughput: from about 26 M depthwise outputs at stride 1
        // the two kernels on their own are faster (MobileNetV2 at batch 64, 56 x 56 x 144: 37 us against 43;
        // 112 x 112 x 32, 25.7 M outputs: the same either way; everything smaller and every stride-2 stage: merged).
        {
          uint64_t outputs = 1;
          for (uint32_t e : mid->GetShape()) outputs *= e;
          if (im->attrs_.stride[0] == 1 && im->attrs_.stride[1] == 1 && outputs >= 26000000ull && !std::getenv("TVX_DWPW_ANY_SIZE")) continue;
        }
        // the merged operator runs where the depthwise convolution stands: a residual operand of the pointwise
        // convolution's Add has to exist by then
        auto pad = fused_add.find(consumers[0].get());
        if (pad != fused_add.end()) {
          auto other = pad->second.add->impl()->inputs_tensor_[pad->second.conv_operand == 1 ? 1 : 0];
          auto oit = produced_at.find(other.get());
          if (oit != produced_at.end() && oit->second >= produced_at[im->outputs_tensor_[0].get()]) continue;
        }
        fused_dwpw[op] = consumers[0].get();
      }
    }
    // ---- inverted-residual plan: a 1x1 convolution (with its activation) whose TRANSIENT result only feeds the
    // depthwise convolution of such a pair may become one operator with both
    std::map<Operation*, Operation*> fused_block;  // expansion -> the depthwise convolution behind it
    if (!std::getenv("TVX_NO_BLOCK_FUSION")) {  // tuning aid
      for (Operation* op : graph->sorted_ops_) {
        OpImpl* im = op->impl().get();
        if (im->kind_ != OpKind::CONV2D || im->attrs_.multiplier != 0 || im->attrs_.conv_1d || fused_add.count(op)) continue;
        auto fa = fused_act.find(op);
        auto mid = fa != fused_act.end() ? fa->second->impl()->outputs_tensor_[0] : im->outputs_tensor_[0];
        if (!(mid->GetSpec().attr_ & TensorAttribute::TRANSIENT)) continue;
        auto consumers = graph->GetConsumersOp(mid);
        if (consumers.size() != 1) continue;
        Operation* dw = consumers[0].get();
        auto fd = fused_dwpw.find(dw);
        if (fd == fused_dwpw.end() || dw->impl()->inputs_tensor_[0] != mid) continue;
        // the merged operator runs where the expansion stands: the residual operand has to exist by then
        auto pad = fused_add.find(fd->second);
        if (pad != fused_add.end()) {
          auto other = pad->second.add->impl()->inputs_tensor_[pad->second.conv_operand == 1 ? 1 : 0];
          auto oit = produced_at.find(other.get());
          if (oit != produced_at.end() && oit->second >= produced_at[im->outputs_tensor_[0].get()]) continue;
        }
        fused_block[op] = dw;
      }
    }
    // ---- convolution -> 2x2 max pooling, FullyConnected -> Softmax: a TRANSIENT result with that one reader may
    // never reach memory (whether a kernel takes the pair is decided when the operators are created)
    std::map<Operation*, Operation*> fused_pool, fused_softmax;
    if (!std::getenv("TVX_NO_POOL_FUSION")) {  // tuning aid
      for (Operation* op : graph->sorted_ops_) {
        OpImpl* im = op->impl().get();
        const bool conv = im->kind_ == OpKind::CONV2D && !im->attrs_.conv_1d && im->attrs_.multiplier == 0;
        if (!conv && im->kind_ != OpKind::FCL) continue;
        if (fused_add.count(op) || fused_dwpw.count(op) || fused_block.count(op)) continue;
        auto fa = fused_act.find(op);
        auto mid = fa != fused_act.end() ? fa->second->impl()->outputs_tensor_[0] : im->outputs_tensor_[0];
        if (!(mid->GetSpec().attr_ & TensorAttribute::TRANSIENT)) continue;
        auto consumers = graph->GetConsumersOp(mid);
        if (consumers.size() != 1) continue;
        OpImpl* next = consumers[0]->impl().get();
        if (next->inputs_tensor_[0] != mid) continue;
        if (conv && next->kind_ == OpKind::POOL && !next->attrs_.pool_1d) fused_pool[op] = consumers[0].get();
        if (!conv && next->kind_ == OpKind::SOFTMAX) fused_softmax[op] = consumers[0].get();
      }
      // a pointwise convolution folded into the depthwise one in front of it is not there to take a pooling
      for (auto& kv : fused_dwpw) fused_pool.erase(kv.second);
    }
    // ---- channel-blocked plan: runs of convolutions over small planes between TRANSIENT tensors kept 16 channels to
    // a unit; the operators of the plan are no longer there for the other fusions
    std::map<Operation*, BlockedOp> blocked, blocked_writers;  // (writers: WHCN in, blocked out, in front of the plan)
    {
      const char* lever = std::getenv("TVX_BLOCKED_LAYOUT");  // tuning aid: 0 keeps every tensor in WHCN order
      if (!lever || std::atoi(lever) != 0) PlanBlocked(graph, fused_act, fused_add, &blocked, &blocked_writers);
      for (auto it = fused_block.begin(); it != fused_block.end();) {
        Operation* dw = it->second;
        auto pair = fused_dwpw.find(dw);
        const bool hit = blocked.count(it->first) || blocked.count(dw) || blocked_writers.count(dw) ||
                         (pair != fused_dwpw.end() && blocked.count(pair->second));
        it = hit ? fused_block.erase(it) : std::next(it);
      }
      for (auto it = fused_dwpw.begin(); it != fused_dwpw.end();) {
        if (blocked.count(it->first) || blocked.count(it->second) || blocked_writers.count(it->first)) {
          for (auto fb = fused_block.begin(); fb != fused_block.end();) fb = fb->second == it->first ? fused_block.erase(fb) : std::next(fb);
          it = fused_dwpw.erase(it);
        } else {
          ++it;
        }
      }
      for (auto it = fused_pool.begin(); it != fused_pool.end();)
        it = blocked.count(it->first) || blocked.count(it->second) ? fused_pool.erase(it) : std::next(it);
    }
    // ---- device storage: one buffer per tensor, Reshape outputs alias their input --
    for (Operation* op : graph->sorted_ops_) {
      OpImpl* im = op->impl().get();
      for (auto& t : im->inputs_tensor_)
        if (!t->IsPlaceHolder() && !EnsureBuffer(static_cast<TensorImpl*>(t.get()))) return false;
      if (im->kind_ == OpKind::RESHAPE) {
        dev_[static_cast<TensorImpl*>(im->outputs_tensor_[0].get())] =
            dev_[static_cast<TensorImpl*>(im->inputs_tensor_[0].get())];
        continue;
      }
      for (auto& t : im->outputs_tensor_)
        if (!EnsureBuffer(static_cast<TensorImpl*>(t.get()))) return false;
    }
    // ---- operators ---------------------------------------------------------------
    for (Operation* op : graph->sorted_ops_) {
      if (skipped.count(op)) continue;
      OpImpl* im = op->impl().get();
      if (im->attrs_.overflow != OverflowPolicy::SATURATE || im->attrs_.rounding != RoundingPolicy::RTNE) {
        VSILOGE("%s: only SATURATE + RTNE rounding policy is implemented", OpKindName(im->kind_));
        return false;
      }
      auto writer = blocked_writers.find(op);
      if (writer != blocked_writers.end()) {
        Push(writer->second.op, im, writer->second.in0, nullptr, static_cast<TensorImpl*>(writer->second.out.get()));
        continue;
      }
      auto planned = blocked.find(op);
      if (planned != blocked.end()) {
        if (!AddBlocked(im, &planned->second)) return false;
        if (planned->second.add) skipped[planned->second.add] = true;
        continue;
      }
      int act = TVX_ACT_NONE;
      TensorImpl* out = static_cast<TensorImpl*>(im->outputs_tensor_[0].get());
      auto f = fused_act.find(op);
      if (f != fused_act.end()) {
        OpImpl* a = f->second->impl().get();
        act = a->kind_ == OpKind::RELU ? TVX_ACT_RELU : TVX_ACT_RELU6;
        out = static_cast<TensorImpl*>(a->outputs_tensor_[0].get());
      }
      bool ok = true;
      switch (im->kind_) {
        case OpKind::CONV2D: {
          // folded activation and output tensor of a convolution of the plan
          auto folded = [&](Operation* c, int* c_act) {
            *c_act = TVX_ACT_NONE;
            TensorImpl* c_out = static_cast<TensorImpl*>(c->impl()->outputs_tensor_[0].get());
            auto cf = fused_act.find(c);
            if (cf != fused_act.end()) {
              OpImpl* ca = cf->second->impl().get();
              *c_act = ca->kind_ == OpKind::RELU ? TVX_ACT_RELU : TVX_ACT_RELU6;
              c_out = static_cast<TensorImpl*>(ca->outputs_tensor_[0].get());
            }
            return c_out;
          };
          auto fb = fused_block.find(op);
          if (fb != fused_block.end()) {
            Operation* dw = fb->second;
            Operation* pw = fused_dwpw[dw];
            int dw_act, pw_act;
            TensorImpl* dw_out = folded(dw, &dw_act);
            TensorImpl* pw_out = folded(pw, &pw_act);
            auto pad = fused_add.find(pw);
            bool all = false;
            ok = AddBlock(im, out, act, dw->impl().get(), dw_out, dw_act, pw->impl().get(), pw_out, pw_act,
                          pad != fused_add.end() ? pad->second.add->impl().get() : nullptr,
                          pad != fused_add.end() ? pad->second.conv_operand : 0, &all);
            if (!ok) break;
            if (all) {
              skipped[dw] = true;  // (the activations folded into the three are skipped already)
              skipped[pw] = true;
              if (pad != fused_add.end()) skipped[pad->second.add] = true;
              break;
            }
          }
          auto fd = fused_dwpw.find(op);
          if (fd != fused_dwpw.end()) {
            Operation* pw = fd->second;
            OpImpl* pim = pw->impl().get();
            int pw_act = TVX_ACT_NONE;
            TensorImpl* pw_out = static_cast<TensorImpl*>(pim->outputs_tensor_[0].get());
            auto pf = fused_act.find(pw);
            if (pf != fused_act.end()) {
              OpImpl* pa = pf->second->impl().get();
              pw_act = pa->kind_ == OpKind::RELU ? TVX_ACT_RELU : TVX_ACT_RELU6;
              pw_out = static_cast<TensorImpl*>(pa->outputs_tensor_[0].get());
            }
            auto pad = fused_add.find(pw);
            bool both = false;
            ok = AddDwPw(im, out, act, pim, pw_out, pw_act, pad != fused_add.end() ? pad->second.add->impl().get() : nullptr,
                         pad != fused_add.end() ? pad->second.conv_operand : 0, &both);
            if (!ok) break;
            if (both) {
              skipped[pw] = true;  // (the activation folded into it is skipped already)
              if (pad != fused_add.end()) skipped[pad->second.add] = true;
              break;
            }
          }
          auto fp = fused_pool.find(op);
          if (fp != fused_pool.end()) {
            bool both = false;
            ok = AddConvPool(im, out, act, fp->second->impl().get(), &both);
            if (!ok) break;
            if (both) {
              skipped[fp->second] = true;
              break;
            }
          }
          auto fa = fused_add.find(op);
          bool fused = false;
          if (fa != fused_add.end()) {
            ok = AddConv(im, out, act, false, fa->second.add->impl().get(), fa->second.conv_operand, &fused);
            if (fused) skipped[fa->second.add] = true;
          }
          if (ok && !fused) ok = AddConv(im, out, act);
          break;
        }
        case OpKind::FCL: {
          bool both = false;
          auto fs = fused_softmax.find(op);
          if (fs != fused_softmax.end()) {
            ok = AddFcSoftmax(im, out, act, fs->second->impl().get(), &both);
            if (both) skipped[fs->second] = true;
          }
          if (ok && !both) ok = AddFc(im, out, act);
          break;
        }
        case OpKind::POOL: ok = AddPool(im, out); break;
        case OpKind::RELU: ok = AddActivation(im, out, TVX_ACT_RELU); break;
        case OpKind::RELU6: ok = AddActivation(im, out, TVX_ACT_RELU6); break;
        case OpKind::ADD: ok = AddAdd(im, out); break;
        case OpKind::SOFTMAX: ok = AddSoftmax(im, out); break;
        case OpKind::RESHAPE: break;  // aliased
        case OpKind::TRANSPOSE: ok = AddTranspose(im, out); break;
        case OpKind::DATACONVERT: ok = AddConvert(im, out); break;
        case OpKind::DECONV2D: ok = AddConv(im, out, TVX_ACT_NONE, true); break;
      }
      if (!ok) return false;
    }
    // constants that are read at run time (weights bound as non-constant tensors are
    // uploaded in Execute); constant activations are uploaded once here
    for (auto& kv : dev_) {
      TensorImpl* t = kv.first;
      if (t->IsConstTensor() && t->HostData() && owned_.count(t)) {
        if (tvx_memcpy_h2d(kv.second, t->HostData(), t->HostBytes(), stream_) != TVX_OK) return Fail("upload");
        t->host_dirty_ = false;
      }
    }
    return tvx_stream_synchronize(stream_) == TVX_OK || Fail("sync");
  }

  bool Execute(GraphImpl* graph) override {
    // host -> device: every host-visible non-output tensor whose host image changed
    for (auto& kv : dev_) {
      TensorImpl* t = kv.first;
      if (!owned_.count(t) || (t->spec_.attr_ & TensorAttribute::OUTPUT)) continue;
      if (t->host_dirty_ && t->HostData()) {
        if (tvx_memcpy_h2d(kv.second, t->HostData(), t->HostBytes(), stream_) != TVX_OK) return Fail("input upload");
        t->host_dirty_ = false;
      }
    }
    // With TVX_RUNTIME_PROFILE set, the operator sequence is timed on its own
    // (uploads drained first), for tools that report device time per Run().
    std::chrono::steady_clock::time_point t0;
    const int profile_mode = ProfileMode();
    const bool profile_ = profile_mode >= 1, profile_ops_ = profile_mode == 2;
    if (profile_) {
      if (tvx_stream_synchronize(stream_) != TVX_OK) return Fail("sync");
      t0 = std::chrono::steady_clock::now();
    }
    // TVX_RUNTIME_PROFILE=ops: a time stamp on the stream in front of every operator and behind the last
    // (what vxQueryNode(VX_NODE_PERFORMANCE) reports per node in the reference's driver)
    if (profile_ops_ && events_.size() != steps_.size() + 1) {
      while (events_.size() < steps_.size() + 1) {
        void* e = nullptr;
        if (tvx_event_create(&e) != TVX_OK) return Fail("event");
        events_.push_back(e);
      }
    }
    size_t step_index = 0;
    for (auto& s : steps_) {
      if (profile_ops_ && tvx_event_record(events_[step_index], stream_) != TVX_OK) return Fail("event");
      ++step_index;
      const int st = tvx_op_run3(s.op, s.blocked_in0 ? s.blocked_in0 : dev_[s.in0],
                                 s.blocked_in1 ? s.blocked_in1 : (s.in1 ? dev_[s.in1] : nullptr),
                                 s.in2 ? dev_[s.in2] : nullptr, s.blocked_out ? s.blocked_out : dev_[s.out], stream_);
      if (st != TVX_OK) {
        VSILOGE("%s failed: %s", s.name.c_str(), tvx_last_error());
        return false;
      }
    }
    if (profile_ops_ && tvx_event_record(events_[steps_.size()], stream_) != TVX_OK) return Fail("event");
    if (profile_) {
      if (tvx_stream_synchronize(stream_) != TVX_OK) return Fail("sync");
      g_last_device_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    }
    if (profile_ops_) {
      g_last_op_us.clear();
      g_last_op_bytes.clear();
      for (size_t i = 0; i < steps_.size(); ++i) {
        float ms = 0.f;
        if (tvx_event_elapsed_ms(events_[i], events_[i + 1], &ms) != TVX_OK) return Fail("event");
        g_last_op_us.emplace_back(steps_[i].name, static_cast<double>(ms) * 1e3);
        g_last_op_bytes.push_back(steps_[i].bytes);
      }
    }
    for (auto& t : graph->outputs_tensor_) {
      TensorImpl* ti = static_cast<TensorImpl*>(t.get());
      auto it = dev_.find(ti);
      if (it == dev_.end()) continue;  // an OUTPUT tensor no operator writes
      ti->EnsureHostBuffer();
      if (tvx_memcpy_d2h(ti->HostData(), it->second, ti->HostBytes(), stream_) != TVX_OK) return Fail("output download");
    }
    return tvx_stream_synchronize(stream_) == TVX_OK || Fail("sync");
  }

 private:
  struct AddFusion { Operation* add; int conv_operand; };  // conv_operand: 1 or 2, which operand of the Add the convolution is

  // An operator of the channel-blocked plan.
  struct BlockedOp {
    tvx_op* op = nullptr;       // created when the plan is made; owned by steps_ once placed
    TensorImpl* in0 = nullptr;
    TensorImpl* res = nullptr;  // the other operand of the Add folded into a convolution
    std::shared_ptr<Tensor> out;  // what it writes: its own output, its activation's or its Add's
    Operation* add = nullptr;
    bool pool = false;
    bool convert[2] = {false, false};  // in0 / res come in WHCN order and need a blocked copy
  };

  bool Fail(const char* what) {
    VSILOGE("%s: %s", what, tvx_last_error());
    return false;
  }

  bool EnsureBuffer(TensorImpl* t) {
    if (dev_.count(t)) return true;
    void* p = nullptr;
    if (tvx_malloc(&p, t->HostBytes() ? t->HostBytes() : 16) != TVX_OK) return Fail("device allocation");
    dev_[t] = p;
    owned_[t] = p;
    return true;
  }

  void Push(tvx_op* op, OpImpl* im, TensorImpl* in0, TensorImpl* in1, TensorImpl* out, TensorImpl* in2 = nullptr) {
    Step s;
    s.op = op;
    s.in0 = in0;
    s.in1 = in1;
    s.in2 = in2;
    s.out = out;
    s.name = std::string(OpKindName(im->kind_)) + " (" + tvx_op_kernel_name(op) + ")";
    for (TensorImpl* t : {in0, in1, in2, out})
      if (t) s.bytes += t->HostBytes();
    VSILOGI("uid %u -> %s", im->uid_, s.name.c_str());
    steps_.push_back(s);
  }

  // Weight quantization -> descriptor fields; per-channel scales stay alive in `scales`.
  static void WeightQuant(const TensorSpec& w, float* scale, int32_t* zp, const float** scales) {
    *scales = nullptr;
    *scale = 1.0f;
    *zp = 0;
    if (w.quantization_.Type() == QuantType::SYMMETRIC_PER_CHANNEL) {
      *scales = w.quantization_.Scales().data();
    } else if (w.quantization_.Type() == QuantType::ASYMMETRIC) {
      *scale = ScaleOf(w);
      *zp = ZpOf(w);
    }
  }

  // With add_im: tries the Conv2d + Add operator (conv_operand: which operand of the Add the convolution is);
  // *fused says whether it exists for this convolution - if not, nothing has been added and the caller goes on
  // with the two operators.
  // The convolution `im` writing `out` (its own output tensor or that of the activation folded into it) as a descriptor.
  static tvx_conv2d_desc ConvDesc(OpImpl* im, TensorImpl* out, int act, bool transposed) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    TensorImpl* w = static_cast<TensorImpl*>(im->inputs_tensor_[1].get());
    const OpAttrs& a = im->attrs_;
    ShapeType xs = x->spec_.shape_, ws = w->spec_.shape_, os = out->spec_.shape_;
    if (a.conv_1d) {  // {W, C, N} tensors viewed as {W, 1, C, N}; only the kernel extents of `ws` are read
      xs = {xs[0], 1, xs[1], xs[2]};
      ws = {ws[0], 1, 0, 0};
      os = {os[0], 1, os[1], os[2]};
    }
    tvx_conv2d_desc d{};
    d.in_w = xs[0]; d.in_h = xs[1]; d.in_c = xs[2]; d.batch = xs[3];
    d.k_w = ws[0]; d.k_h = ws[1];
    d.out_w = os[0]; d.out_h = os[1]; d.out_c = os[2];
    d.stride_w = a.stride[0]; d.stride_h = a.stride[1];
    d.dilation_w = transposed ? 1 : a.dilation[0]; d.dilation_h = transposed ? 1 : a.dilation[1];
    d.pad_left = a.pad[0]; d.pad_top = a.pad[2];
    d.multiplier = a.multiplier;
    d.groups = a.groups;
    d.in_dtype = DtypeCode(x->spec_.datatype_);
    d.w_dtype = DtypeCode(w->spec_.datatype_);
    d.out_dtype = DtypeCode(out->spec_.datatype_);
    d.in_scale = ScaleOf(x->spec_); d.in_zp = ZpOf(x->spec_);
    WeightQuant(w->spec_, &d.w_scale, &d.w_zp, &d.w_scales);
    d.out_scale = ScaleOf(out->spec_); d.out_zp = ZpOf(out->spec_);
    d.activation = act;
    return d;
  }

  static bool AddDesc(OpImpl* add_im, tvx_eltwise_desc* e) {
    TensorImpl* a0 = static_cast<TensorImpl*>(add_im->inputs_tensor_[0].get());
    TensorImpl* a1 = static_cast<TensorImpl*>(add_im->inputs_tensor_[1].get());
    TensorImpl* sum = static_cast<TensorImpl*>(add_im->outputs_tensor_[0].get());
    if (a0->spec_.datatype_ != a1->spec_.datatype_ || a0->spec_.datatype_ != sum->spec_.datatype_ ||
        a0->spec_.shape_ != a1->spec_.shape_)
      return false;
    *e = tvx_eltwise_desc{};
    e->count = static_cast<uint64_t>(sum->spec_.GetElementNum());
    e->dtype = DtypeCode(sum->spec_.datatype_);
    e->a_scale = ScaleOf(a0->spec_); e->a_zp = ZpOf(a0->spec_);
    e->b_scale = ScaleOf(a1->spec_); e->b_zp = ZpOf(a1->spec_);
    e->out_scale = ScaleOf(sum->spec_); e->out_zp = ZpOf(sum->spec_);
    return true;
  }

  // Expansion, depthwise convolution and projection (+ residual Add) as one operator (tvx_mbconv_create). *fused
  // says whether a kernel took the block; if not, nothing has been added and the caller goes on operator by operator.
  bool AddBlock(OpImpl* ex_im, TensorImpl* ex_out, int ex_act, OpImpl* dw_im, TensorImpl* dw_out, int dw_act,
                OpImpl* pw_im, TensorImpl* pw_out, int pw_act, OpImpl* add_im, int conv_operand, bool* fused) {
    *fused = false;
    TensorImpl* w[3];
    TensorImpl* b[3];
    OpImpl* ims[3] = {ex_im, dw_im, pw_im};
    for (int i = 0; i < 3; ++i) {
      w[i] = static_cast<TensorImpl*>(ims[i]->inputs_tensor_[1].get());
      b[i] = ims[i]->inputs_tensor_.size() > 2 && !ims[i]->inputs_tensor_[2]->IsPlaceHolder()
                 ? static_cast<TensorImpl*>(ims[i]->inputs_tensor_[2].get()) : nullptr;
      if (!w[i]->IsConstTensor() || !w[i]->HostData() || (b[i] && (!b[i]->IsConstTensor() || !b[i]->HostData()))) return true;
    }
    const tvx_conv2d_desc ex = ConvDesc(ex_im, ex_out, ex_act, false);
    const tvx_conv2d_desc dw = ConvDesc(dw_im, dw_out, dw_act, false);
    const tvx_conv2d_desc pw = ConvDesc(pw_im, pw_out, pw_act, false);
    tvx_eltwise_desc e{};
    if (add_im && !AddDesc(add_im, &e)) return true;
    tvx_op* op = nullptr;
    const int st = tvx_mbconv_create(&ex, w[0]->HostData(), b[0] ? b[0]->HostData() : nullptr, &dw, w[1]->HostData(),
                                     b[1] ? b[1]->HostData() : nullptr, &pw, w[2]->HostData(),
                                     b[2] ? b[2]->HostData() : nullptr, add_im ? &e : nullptr, conv_operand, &op);
    if (st == TVX_E_UNSUPPORTED) return true;
    if (st != TVX_OK) return Fail("tvx_mbconv_create");
    *fused = true;
    TensorImpl* x = static_cast<TensorImpl*>(ex_im->inputs_tensor_[0].get());
    if (add_im) {
      TensorImpl* other = static_cast<TensorImpl*>(add_im->inputs_tensor_[conv_operand == 1 ? 1 : 0].get());
      Push(op, ex_im, x, other, static_cast<TensorImpl*>(add_im->outputs_tensor_[0].get()));
    } else {
      Push(op, ex_im, x, nullptr, pw_out);
    }
    return true;
  }

  // A depthwise convolution and the pointwise convolution that alone reads its result as one operator
  // (tvx_conv2d_dw_pw_create), the pointwise one possibly with the residual Add behind it. *fused says whether a
  // kernel took the pair; if not, the caller adds the operators one by one.
  bool AddDwPw(OpImpl* dw_im, TensorImpl* dw_out, int dw_act, OpImpl* pw_im, TensorImpl* pw_out, int pw_act,
               OpImpl* add_im, int conv_operand, bool* fused) {
    *fused = false;
    auto constant = [](OpImpl* im, TensorImpl** w, TensorImpl** b) {
      *w = static_cast<TensorImpl*>(im->inputs_tensor_[1].get());
      *b = im->inputs_tensor_.size() > 2 && !im->inputs_tensor_[2]->IsPlaceHolder()
               ? static_cast<TensorImpl*>(im->inputs_tensor_[2].get()) : nullptr;
      return (*w)->IsConstTensor() && (*w)->HostData() && (!*b || ((*b)->IsConstTensor() && (*b)->HostData()));
    };
    TensorImpl *dw_w, *dw_b, *pw_w, *pw_b;
    if (!constant(dw_im, &dw_w, &dw_b) || !constant(pw_im, &pw_w, &pw_b)) return true;
    const tvx_conv2d_desc dw = ConvDesc(dw_im, dw_out, dw_act, false);
    const tvx_conv2d_desc pw = ConvDesc(pw_im, pw_out, pw_act, false);
    tvx_eltwise_desc e{};
    if (add_im && !AddDesc(add_im, &e)) return true;
    tvx_op* op = nullptr;
    const int st = tvx_conv2d_dw_pw_create(&dw, dw_w->HostData(), dw_b ? dw_b->HostData() : nullptr, &pw, pw_w->HostData(),
                                           pw_b ? pw_b->HostData() : nullptr, add_im ? &e : nullptr, conv_operand, &op);
    if (st == TVX_E_UNSUPPORTED) return true;
    if (st != TVX_OK) return Fail("tvx_conv2d_dw_pw_create");
    *fused = true;
    TensorImpl* x = static_cast<TensorImpl*>(dw_im->inputs_tensor_[0].get());
    if (add_im) {
      TensorImpl* other = static_cast<TensorImpl*>(add_im->inputs_tensor_[conv_operand == 1 ? 1 : 0].get());
      Push(op, dw_im, x, other, static_cast<TensorImpl*>(add_im->outputs_tensor_[0].get()));
    } else {
      Push(op, dw_im, x, nullptr, pw_out);
    }
    return true;
  }

  // Channel-blocked plan. Planes of a few pixels (7 x 7 at the end of a MobileNet) make WHCN rows no 16-byte load is
  // aligned to; 1x1 and depthwise 3x3 convolutions over them are faster between tensors kept 16 channels to a unit
  // (tvx_conv2d_blocked_create). A TRANSIENT tensor has no host image, so its order in memory is this runtime's
  // choice. An operator joins the plan if a blocked kernel takes it and every reader of its result is in the plan too;
  // a tensor that comes in from outside gets a blocked copy, made by a step of its own (tvx_layout_create), and the
  // plan ends at an average pooling over whole planes, whose result is one pixel per plane in WHCN order. A plan of
  // fewer than three convolutions does not pay for the copy and is dropped.
  void PlanBlocked(GraphImpl* graph, const std::map<Operation*, Operation*>& fused_act,
                   const std::map<Operation*, AddFusion>& fused_add, std::map<Operation*, BlockedOp>* plan,
                   std::map<Operation*, BlockedOp>* writers) {
    // pixels of a plane; from 14 x 14 up the WHCN kernels and the block kernel are as fast or faster (MobileNetV2 at
    // batch 64: 19.5 us for the three blocked operators of a 64 -> 384 -> 64 block against 15.7 us)
    uint64_t kMaxPlane = 64;
    if (const char* v = std::getenv("TVX_BLOCKED_MAX_PLANE")) kMaxPlane = std::strtoull(v, nullptr, 10);  // tuning aid
    std::map<Operation*, Operation*> add_owner;  // Add -> the convolution it is folded into
    for (auto& kv : fused_add) add_owner[kv.second.add] = kv.first;
    auto constant = [](OpImpl* im, TensorImpl** w, TensorImpl** b) {
      *w = static_cast<TensorImpl*>(im->inputs_tensor_[1].get());
      *b = im->inputs_tensor_.size() > 2 && !im->inputs_tensor_[2]->IsPlaceHolder()
               ? static_cast<TensorImpl*>(im->inputs_tensor_[2].get()) : nullptr;
      return (*w)->IsConstTensor() && (*w)->HostData() && (!*b || ((*b)->IsConstTensor() && (*b)->HostData()));
    };
    for (Operation* op : graph->sorted_ops_) {
      OpImpl* im = op->impl().get();
      if (im->attrs_.overflow != OverflowPolicy::SATURATE || im->attrs_.rounding != RoundingPolicy::RTNE) continue;
      TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
      const ShapeType& xs = x->spec_.shape_;
      if (xs.size() != 4 || static_cast<uint64_t>(xs[0]) * xs[1] > kMaxPlane || !IsQuantSpec(x->spec_)) continue;
      BlockedOp b;
      b.in0 = x;
      if (im->kind_ == OpKind::CONV2D && !im->attrs_.conv_1d) {
        TensorImpl *w, *bias;
        if (!constant(im, &w, &bias)) continue;
        int act = TVX_ACT_NONE;
        b.out = im->outputs_tensor_[0];
        tvx_conv2d_desc d = ConvDesc(im, static_cast<TensorImpl*>(b.out.get()), act, false);
        tvx_eltwise_desc e{};
        int conv_operand = 0;
        auto fa = fused_act.find(op);
        auto fd = fused_add.find(op);
        if (fa != fused_act.end()) {
          OpImpl* a = fa->second->impl().get();
          act = a->kind_ == OpKind::RELU ? TVX_ACT_RELU : TVX_ACT_RELU6;
          b.out = a->outputs_tensor_[0];
          d = ConvDesc(im, static_cast<TensorImpl*>(b.out.get()), act, false);
        } else if (fd != fused_add.end()) {
          OpImpl* a = fd->second.add->impl().get();
          if (!AddDesc(a, &e)) continue;
          conv_operand = fd->second.conv_operand;
          b.add = fd->second.add;
          b.res = static_cast<TensorImpl*>(a->inputs_tensor_[conv_operand == 1 ? 1 : 0].get());
          b.out = a->outputs_tensor_[0];
        }
        if (!(b.out->GetSpec().attr_ & TensorAttribute::TRANSIENT)) continue;
        if (tvx_conv2d_blocked_create(&d, b.add ? &e : nullptr, conv_operand, w->HostData(), bias ? bias->HostData() : nullptr,
                                      &b.op) != TVX_OK)
          continue;
      } else if (im->kind_ == OpKind::POOL && !im->attrs_.pool_1d) {
        b.pool = true;
        b.out = im->outputs_tensor_[0];
        const tvx_pool2d_desc d = PoolDesc(im, x, static_cast<TensorImpl*>(b.out.get()));
        if (tvx_pool2d_blocked_create(&d, &b.op) != TVX_OK) continue;
      } else {
        continue;
      }
      (*plan)[op] = b;
    }
    // closure: what a convolution of the plan writes is blocked, so every reader has to be in the plan, as its input
    // or as the residual operand of its Add; a pooling of the plan reads what a convolution of the plan wrote
    for (bool changed = true; changed;) {
      changed = false;
      std::map<Tensor*, Operation*> written;  // blocked tensor -> the convolution of the plan that writes it
      for (auto& kv : *plan)
        if (!kv.second.pool) written[kv.second.out.get()] = kv.first;
      for (auto it = plan->begin(); it != plan->end();) {
        BlockedOp& b = it->second;
        bool keep = true;
        if (b.pool) {
          keep = written.count(b.in0) != 0;
        } else {
          for (auto& reader : graph->GetConsumersOp(b.out)) {
            auto r = plan->find(reader.get());
            if (r != plan->end() && r->second.in0 == b.out.get()) continue;
            auto owner = add_owner.find(reader.get());
            if (owner != add_owner.end()) {
              auto o = plan->find(owner->second);
              if (o != plan->end() && o->second.add == reader.get() && o->second.res == b.out.get()) continue;
            }
            keep = false;
            break;
          }
        }
        if (keep) {
          ++it;
        } else {
          tvx_op_destroy(b.op);
          it = plan->erase(it);
          changed = true;
        }
      }
    }
    size_t convolutions = 0;
    std::map<Tensor*, Operation*> written;
    for (auto& kv : *plan)
      if (!kv.second.pool) {
        written[kv.second.out.get()] = kv.first;
        ++convolutions;
      }
    if (convolutions < 3) {
      for (auto& kv : *plan) tvx_op_destroy(kv.second.op);
      plan->clear();
      return;
    }
    for (auto& kv : *plan) {
      kv.second.convert[0] = !written.count(kv.second.in0);
      kv.second.convert[1] = kv.second.res && !written.count(kv.second.res);
    }
    // a TRANSIENT tensor that enters the plan from a depthwise convolution and is read by nothing else: where a kernel
    // can, that convolution writes it blocked itself (tvx_conv2d_to_blocked_create) and the copy falls away
    if (std::getenv("TVX_NO_BLOCKED_WRITERS")) return;  // tuning aid
    for (Operation* prod : graph->sorted_ops_) {
      OpImpl* pim = prod->impl().get();
      if (pim->kind_ != OpKind::CONV2D || pim->attrs_.conv_1d || pim->attrs_.multiplier != 1 || plan->count(prod) || fused_add.count(prod)) continue;
      if (pim->attrs_.overflow != OverflowPolicy::SATURATE || pim->attrs_.rounding != RoundingPolicy::RTNE) continue;
      int act = TVX_ACT_NONE;
      std::shared_ptr<Tensor> out = pim->outputs_tensor_[0];
      auto fa = fused_act.find(prod);
      if (fa != fused_act.end()) {
        OpImpl* a = fa->second->impl().get();
        act = a->kind_ == OpKind::RELU ? TVX_ACT_RELU : TVX_ACT_RELU6;
        out = a->outputs_tensor_[0];
      }
      if (!(out->GetSpec().attr_ & TensorAttribute::TRANSIENT)) continue;
      auto readers = graph->GetConsumersOp(out);
      bool all_in_plan = !readers.empty();
      for (auto& r : readers) {
        auto pr = plan->find(r.get());
        all_in_plan = all_in_plan && pr != plan->end() && pr->second.in0 == out.get() && pr->second.convert[0] && pr->second.res != out.get();
      }
      TensorImpl *w, *bias;
      if (!all_in_plan || !constant(pim, &w, &bias)) continue;
      BlockedOp b;
      b.in0 = static_cast<TensorImpl*>(pim->inputs_tensor_[0].get());
      b.out = out;
      const tvx_conv2d_desc d = ConvDesc(pim, static_cast<TensorImpl*>(out.get()), act, false);
      if (tvx_conv2d_to_blocked_create(&d, w->HostData(), bias ? bias->HostData() : nullptr, &b.op) != TVX_OK) continue;
      (*writers)[prod] = b;
      for (auto& r : readers) (*plan)[r.get()].convert[0] = false;
    }
  }

  // Places an operator of the channel-blocked plan, behind the steps that make the blocked copies it reads.
  bool AddBlocked(OpImpl* im, BlockedOp* b) {
    void* copy[2] = {nullptr, nullptr};
    TensorImpl* ins[2] = {b->in0, b->res};
    for (int i = 0; i < 2; ++i) {
      if (!ins[i] || !b->convert[i]) continue;
      auto it = blocked_copy_.find(ins[i]);
      if (it == blocked_copy_.end()) {
        const ShapeType& s = ins[i]->spec_.shape_;
        tvx_op* to_blocked = nullptr;
        if (s.size() != 4 || tvx_layout_create(s[0], s[1], s[2], s[3], 1, &to_blocked) != TVX_OK) return Fail("tvx_layout_create");
        void* p = nullptr;
        if (tvx_malloc(&p, ins[i]->HostBytes()) != TVX_OK) {
          tvx_op_destroy(to_blocked);
          return Fail("device allocation");
        }
        it = blocked_copy_.emplace(ins[i], p).first;
        Push(to_blocked, im, ins[i], nullptr, ins[i]);
        steps_.back().blocked_out = p;
      }
      copy[i] = it->second;
    }
    Push(b->op, im, b->in0, b->res, static_cast<TensorImpl*>(b->out.get()));
    steps_.back().blocked_in0 = copy[0];
    steps_.back().blocked_in1 = copy[1];
    b->op = nullptr;
    return true;
  }

  bool AddConv(OpImpl* im, TensorImpl* out, int act, bool transposed = false, OpImpl* add_im = nullptr,
               int conv_operand = 0, bool* fused = nullptr) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    TensorImpl* w = static_cast<TensorImpl*>(im->inputs_tensor_[1].get());
    TensorImpl* b = im->inputs_tensor_.size() > 2 && !im->inputs_tensor_[2]->IsPlaceHolder()
                        ? static_cast<TensorImpl*>(im->inputs_tensor_[2].get()) : nullptr;
    tvx_conv2d_desc d = ConvDesc(im, out, act, transposed);
    // a bias that is not a constant is read at run time, which the kernels with packed weights
    // cannot do: weights and bias then both go in as operands of the generic kernel
    const bool bias_at_run = b && !b->IsConstTensor();
    const bool const_w = w->IsConstTensor() && w->HostData() && !bias_at_run;
    tvx_op* op = nullptr;
    if (add_im) {
      *fused = false;
      TensorImpl* a0 = static_cast<TensorImpl*>(add_im->inputs_tensor_[0].get());
      TensorImpl* a1 = static_cast<TensorImpl*>(add_im->inputs_tensor_[1].get());
      TensorImpl* sum = static_cast<TensorImpl*>(add_im->outputs_tensor_[0].get());
      tvx_eltwise_desc e{};
      if (!const_w || !AddDesc(add_im, &e)) return true;
      const int st = tvx_conv2d_add_create(&d, &e, conv_operand, w->HostData(), b ? b->HostData() : nullptr, &op);
      if (st == TVX_E_UNSUPPORTED) return true;
      if (st != TVX_OK) return Fail("tvx_conv2d_add_create");
      *fused = true;
      Push(op, im, x, conv_operand == 1 ? a1 : a0, sum);
      return true;
    }
    if ((transposed ? tvx_deconv2d_create : tvx_conv2d_create)(&d, const_w ? w->HostData() : nullptr,
                                                                 b && !bias_at_run ? b->HostData() : nullptr, &op) != TVX_OK)
      return Fail(transposed ? "tvx_deconv2d_create" : "tvx_conv2d_create");
    Push(op, im, x, const_w ? nullptr : w, out, bias_at_run ? b : nullptr);
    return true;
  }

  static tvx_fc_desc FcDesc(OpImpl* im, TensorImpl* out, int act) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    TensorImpl* w = static_cast<TensorImpl*>(im->inputs_tensor_[1].get());
    const ShapeType& xs = x->spec_.shape_;
    uint64_t k = 1, m = 1;
    for (uint32_t i = 0; i <= im->attrs_.axis; ++i) k *= xs[i];
    for (size_t i = im->attrs_.axis + 1; i < xs.size(); ++i) m *= xs[i];
    tvx_fc_desc d{};
    d.m = static_cast<uint32_t>(m);
    d.k = static_cast<uint32_t>(k);
    d.n = w->spec_.shape_.back();
    d.in_dtype = DtypeCode(x->spec_.datatype_);
    d.w_dtype = DtypeCode(w->spec_.datatype_);
    d.out_dtype = DtypeCode(out->spec_.datatype_);
    d.in_scale = ScaleOf(x->spec_); d.in_zp = ZpOf(x->spec_);
    WeightQuant(w->spec_, &d.w_scale, &d.w_zp, &d.w_scales);
    d.out_scale = ScaleOf(out->spec_); d.out_zp = ZpOf(out->spec_);
    d.activation = act;
    return d;
  }

  bool AddFc(OpImpl* im, TensorImpl* out, int act) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    TensorImpl* w = static_cast<TensorImpl*>(im->inputs_tensor_[1].get());
    TensorImpl* b = im->inputs_tensor_.size() > 2 && !im->inputs_tensor_[2]->IsPlaceHolder()
                        ? static_cast<TensorImpl*>(im->inputs_tensor_[2].get()) : nullptr;
    const tvx_fc_desc d = FcDesc(im, out, act);
    const bool bias_at_run = b && !b->IsConstTensor();  // as for Conv2d
    const bool const_w = w->IsConstTensor() && w->HostData() && !bias_at_run;
    tvx_op* op = nullptr;
    if (tvx_fully_connected_create(&d, const_w ? w->HostData() : nullptr, b && !bias_at_run ? b->HostData() : nullptr, &op) != TVX_OK)
      return Fail("tvx_fully_connected_create");
    Push(op, im, x, const_w ? nullptr : w, out, bias_at_run ? b : nullptr);
    return true;
  }

  // A FullyConnected layer and the Softmax that alone reads its codes as one operator (tvx_fully_connected_softmax_create).
  // *fused says whether a kernel took the pair; if not, nothing has been added.
  bool AddFcSoftmax(OpImpl* im, TensorImpl* out, int act, OpImpl* sm_im, bool* fused) {
    *fused = false;
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    TensorImpl* w = static_cast<TensorImpl*>(im->inputs_tensor_[1].get());
    TensorImpl* b = im->inputs_tensor_.size() > 2 && !im->inputs_tensor_[2]->IsPlaceHolder()
                        ? static_cast<TensorImpl*>(im->inputs_tensor_[2].get()) : nullptr;
    TensorImpl* y = static_cast<TensorImpl*>(sm_im->outputs_tensor_[0].get());
    if (!w->IsConstTensor() || !w->HostData() || (b && (!b->IsConstTensor() || !b->HostData()))) return true;
    tvx_softmax_desc sd{};
    if (y->spec_.datatype_ != DataType::FLOAT32 || !SoftmaxDesc(sm_im, out, &sd)) return true;
    const tvx_fc_desc d = FcDesc(im, out, act);
    if (sd.inner > 1 || sd.channels != d.n || sd.rows != d.m) return true;
    tvx_op* op = nullptr;
    const int st = tvx_fully_connected_softmax_create(&d, &sd, w->HostData(), b ? b->HostData() : nullptr, &op);
    if (st == TVX_E_UNSUPPORTED) return true;
    if (st != TVX_OK) return Fail("tvx_fully_connected_softmax_create");
    *fused = true;
    Push(op, im, x, nullptr, y);
    return true;
  }

  // A convolution and the pooling that alone reads its result as one operator (tvx_conv2d_pool_create).
  bool AddConvPool(OpImpl* im, TensorImpl* out, int act, OpImpl* pool_im, bool* fused) {
    *fused = false;
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    TensorImpl* w = static_cast<TensorImpl*>(im->inputs_tensor_[1].get());
    TensorImpl* b = im->inputs_tensor_.size() > 2 && !im->inputs_tensor_[2]->IsPlaceHolder()
                        ? static_cast<TensorImpl*>(im->inputs_tensor_[2].get()) : nullptr;
    TensorImpl* y = static_cast<TensorImpl*>(pool_im->outputs_tensor_[0].get());
    if (!w->IsConstTensor() || !w->HostData() || (b && (!b->IsConstTensor() || !b->HostData()))) return true;
    if (out->spec_.datatype_ != y->spec_.datatype_) return true;
    const tvx_conv2d_desc d = ConvDesc(im, out, act, false);
    const tvx_pool2d_desc pd = PoolDesc(pool_im, out, y);
    tvx_op* op = nullptr;
    const int st = tvx_conv2d_pool_create(&d, &pd, w->HostData(), b ? b->HostData() : nullptr, &op);
    if (st == TVX_E_UNSUPPORTED || st == TVX_E_INVALID) return true;  // (a pooling the fused form does not describe)
    if (st != TVX_OK) return Fail("tvx_conv2d_pool_create");
    *fused = true;
    Push(op, im, x, nullptr, y);
    return true;
  }

  static tvx_pool2d_desc PoolDesc(OpImpl* im, TensorImpl* x, TensorImpl* out) {
    const OpAttrs& a = im->attrs_;
    const ShapeType &xs = x->spec_.shape_, &os = out->spec_.shape_;
    tvx_pool2d_desc d{};
    if (a.pool_1d) {  // {W, C, N} viewed as {W, 1, C, N}
      d.in_w = xs[0]; d.in_h = 1; d.channels = xs[1]; d.batch = xs[2];
      d.out_w = os[0]; d.out_h = 1;
    } else {
      d.in_w = xs[0]; d.in_h = xs[1]; d.channels = xs[2]; d.batch = xs[3];
      d.out_w = os[0]; d.out_h = os[1];
    }
    d.k_w = a.ksize[0]; d.k_h = a.pool_1d ? 1 : a.ksize[1];
    d.stride_w = a.stride[0] ? a.stride[0] : 1;
    d.stride_h = a.pool_1d ? 1 : (a.stride[1] ? a.stride[1] : 1);
    d.pad_left = a.pad[0]; d.pad_top = a.pool_1d ? 0 : a.pad[2];
    d.pool_type = static_cast<int>(a.pool_type);
    d.dtype = DtypeCode(x->spec_.datatype_);
    d.in_scale = ScaleOf(x->spec_); d.in_zp = ZpOf(x->spec_);
    d.out_scale = ScaleOf(out->spec_); d.out_zp = ZpOf(out->spec_);
    return d;
  }

  bool AddPool(OpImpl* im, TensorImpl* out) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    const tvx_pool2d_desc d = PoolDesc(im, x, out);
    tvx_op* op = nullptr;
    if (tvx_pool2d_create(&d, &op) != TVX_OK) return Fail("tvx_pool2d_create");
    Push(op, im, x, nullptr, out);
    return true;
  }

  bool AddActivation(OpImpl* im, TensorImpl* out, int act) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    if (x->spec_.datatype_ != out->spec_.datatype_) {
      VSILOGE("activation: input and output data types differ");
      return false;
    }
    tvx_eltwise_desc d{};
    d.count = static_cast<uint64_t>(x->spec_.GetElementNum());
    d.dtype = DtypeCode(x->spec_.datatype_);
    d.activation = act;
    d.a_scale = ScaleOf(x->spec_); d.a_zp = ZpOf(x->spec_);
    d.out_scale = ScaleOf(out->spec_); d.out_zp = ZpOf(out->spec_);
    tvx_op* op = nullptr;
    if (tvx_activation_create(&d, &op) != TVX_OK) return Fail("tvx_activation_create");
    Push(op, im, x, nullptr, out);
    return true;
  }

  bool AddAdd(OpImpl* im, TensorImpl* out) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    TensorImpl* z = static_cast<TensorImpl*>(im->inputs_tensor_[1].get());
    if (x->spec_.datatype_ != z->spec_.datatype_ || x->spec_.datatype_ != out->spec_.datatype_) {
      VSILOGE("ADD: operand data types differ");
      return false;
    }
    tvx_eltwise_desc d{};
    d.count = static_cast<uint64_t>(x->spec_.GetElementNum());
    d.dtype = DtypeCode(x->spec_.datatype_);
    d.a_scale = ScaleOf(x->spec_); d.a_zp = ZpOf(x->spec_);
    d.b_scale = ScaleOf(z->spec_); d.b_zp = ZpOf(z->spec_);
    d.out_scale = ScaleOf(out->spec_); d.out_zp = ZpOf(out->spec_);
    tvx_op* op = nullptr;
    if (tvx_add_create(&d, &op) != TVX_OK) return Fail("tvx_add_create");
    Push(op, im, x, z, out);
    return true;
  }

  // The Softmax `im` over tensor x as a descriptor; false when its axis lies outside the tensor.
  static bool SoftmaxDesc(OpImpl* im, TensorImpl* x, tvx_softmax_desc* d) {
    const ShapeType& xs = x->spec_.shape_;
    const int32_t rank = static_cast<int32_t>(xs.size());
    int32_t axis = im->attrs_.sm_axis;
    if (axis < 0) axis += rank;  // negative axes count from the slowest dimension
    if (axis < 0 || axis >= rank) return false;
    *d = tvx_softmax_desc{};
    d->channels = xs[axis];
    d->inner = 1;
    for (int32_t i = 0; i < axis; ++i) d->inner *= xs[i];
    d->rows = static_cast<uint64_t>(x->spec_.GetElementNum()) / (d->channels * d->inner);
    d->beta = im->attrs_.beta;
    d->in_dtype = DtypeCode(x->spec_.datatype_);
    d->in_scale = ScaleOf(x->spec_); d->in_zp = ZpOf(x->spec_);
    return true;
  }

  bool AddSoftmax(OpImpl* im, TensorImpl* out) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    tvx_softmax_desc d{};
    if (out->spec_.datatype_ != DataType::FLOAT32 || !SoftmaxDesc(im, x, &d)) {
      VSILOGE("SOFTMAX: axis %d of a rank-%zu tensor with a FLOAT32 output is what is implemented", im->attrs_.sm_axis,
              x->spec_.shape_.size());
      return false;
    }
    tvx_op* op = nullptr;
    if (tvx_softmax_create(&d, &op) != TVX_OK) return Fail("tvx_softmax_create");
    Push(op, im, x, nullptr, out);
    return true;
  }

  bool AddConvert(OpImpl* im, TensorImpl* out) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    const int in_code = DtypeCode(x->spec_.datatype_), out_code = DtypeCode(out->spec_.datatype_);
    if (in_code < 0 || out_code < 0) {
      VSILOGE("DATACONVERT: UINT8, INT8, FLOAT16 and FLOAT32 tensors are what is implemented");
      return false;
    }
    tvx_convert_desc d{};
    d.count = static_cast<uint64_t>(x->spec_.GetElementNum());
    d.in_dtype = in_code; d.in_scale = ScaleOf(x->spec_); d.in_zp = ZpOf(x->spec_);
    d.out_dtype = out_code; d.out_scale = ScaleOf(out->spec_); d.out_zp = ZpOf(out->spec_);
    tvx_op* op = nullptr;
    if (tvx_convert_create(&d, &op) != TVX_OK) return Fail("tvx_convert_create");
    Push(op, im, x, nullptr, out);
    return true;
  }

  bool AddTranspose(OpImpl* im, TensorImpl* out) {
    TensorImpl* x = static_cast<TensorImpl*>(im->inputs_tensor_[0].get());
    tvx_transpose_desc d{};
    d.rank = static_cast<uint32_t>(x->spec_.shape_.size());
    for (uint32_t i = 0; i < d.rank; ++i) {
      d.in_dims[i] = x->spec_.shape_[i];
      d.perm[i] = im->attrs_.perm[i];
    }
    d.elem_bytes = static_cast<uint32_t>(x->spec_.GetElementByteSize());
    tvx_op* op = nullptr;
    if (tvx_transpose_create(&d, &op) != TVX_OK) return Fail("tvx_transpose_create");
    Push(op, im, x, nullptr, out);
    return true;
  }

  void* stream_ = nullptr;
  static int ProfileMode() {
    static const int from_env = [] {
      const char* e = std::getenv("TVX_RUNTIME_PROFILE");
      return !e ? 0 : (std::string(e) == "ops" ? 2 : 1);
    }();
    const int m = g_profile_mode.load(std::memory_order_relaxed);
    return m >= 0 ? m : from_env;
  }
  std::vector<void*> events_;
  std::vector<Step> steps_;
  std::map<TensorImpl*, void*> dev_;    // tensor -> device pointer (possibly an alias)
  std::map<TensorImpl*, void*> owned_;  // tensors that own their buffer
  std::map<TensorImpl*, void*> blocked_copy_;  // WHCN tensor -> its channel-blocked copy, written by a step of the plan
};

}  // namespace

std::unique_ptr<Executor> CreateExecutor() {
  return std::unique_ptr<Executor>(new HipExecutor());
}

// Host images of INPUT / OUTPUT tensors in page-locked memory (falls back to ordinary memory without a GPU).
namespace {
void* PinnedAlloc(size_t bytes) {
  void* p = nullptr;
  return tvx_host_malloc(&p, bytes) == TVX_OK ? p : nullptr;
}
void PinnedFree(void* p) { (void)tvx_host_free(p); }
struct OfferPinnedMemory {
  OfferPinnedMemory() {
    g_host_alloc = PinnedAlloc;
    g_host_free = PinnedFree;
  }
} g_offer_pinned_memory;
}  // namespace

}  // namespace vx
}  // namespace tim

// Milliseconds the operator sequence of the most recent Graph::Run() took on the
// device (0 unless TVX_RUNTIME_PROFILE is set). No counterpart in the reference.
extern "C" double tvx_runtime_last_device_ms(void) { return tim::vx::g_last_device_ms; }
// Profiling of the following Graph::Run() calls: 0 off (no synchronisation inside a Run() beyond its last one), 1 the
// operator sequence as a whole, 2 per operator, -1 back to what TVX_RUNTIME_PROFILE says. No counterpart in the reference.
extern "C" void tvx_runtime_set_profile(int mode) { tim::vx::g_profile_mode.store(mode < -1 || mode > 2 ? -1 : mode); }
// Operators of the most recent Graph::Run() with their device time (TVX_RUNTIME_PROFILE=ops): count, then
// name and microseconds of operator i. No counterpart in the reference's API (its driver keeps such numbers
// per vx_node).
extern "C" int tvx_runtime_last_op_count(void) { return static_cast<int>(tim::vx::g_last_op_us.size()); }
// (an index outside [0, count) answers with nothing / zero)
extern "C" const char* tvx_runtime_last_op_name(int i) {
  return i >= 0 && static_cast<size_t>(i) < tim::vx::g_last_op_us.size() ? tim::vx::g_last_op_us[static_cast<size_t>(i)].first.c_str() : nullptr;
}
extern "C" double tvx_runtime_last_op_us(int i) {
  return i >= 0 && static_cast<size_t>(i) < tim::vx::g_last_op_us.size() ? tim::vx::g_last_op_us[static_cast<size_t>(i)].second : 0.0;
}
extern "C" unsigned long long tvx_runtime_last_op_bytes(int i) {
  return i >= 0 && static_cast<size_t>(i) < tim::vx::g_last_op_bytes.size() ? tim::vx::g_last_op_bytes[static_cast<size_t>(i)] : 0ull;
}
