// tvx_graph_runner: builds graphs through the public tim::vx API from a plain-text
// description, runs them, and writes what each graph produced.
//
//   tvx_graph_runner <graphs.txt> <blob.bin> <out.bin>
//
// graphs.txt, one record per line, fields separated by blanks:
//   graph <name>
//   t <id> <dtype> <attr> <rank> <dims..> <quant> <channel_dim> <ns> <scales..> <nz> <zps..> <off> <len>
//       bytes [off, off+len) of blob.bin are the tensor's data; len 0 = no data.
//       CONSTANT tensors get theirs at creation, INPUT tensors by CopyDataToTensor.
//   op <KIND> <n_in> <ids..> <n_out> <ids..> <pad_type> <pl> <pr> <pt> <pb> <sw> <sh> <dw> <dh>
//      <kw> <kh> <multiplier> <weights> <pool_type> <round_type> <pool_1d> <axis> <beta> <sm_axis>
//      <n_shape> <shape..> <groups> <conv_1d>
//       id -1 = the graph's placeholder tensor (no bias); <pool_1d>: 0 = Pool2d by pad / pad type, 1 = Pool1d,
//       2 = Pool2d's global-pooling constructor (<kw> <kh> = input size), 3 = its adaptive constructor
//       (<kw> <kh> = input size, <sw> <sh> = output size)
//   device <index>            (before the tensors) the graph is created with CompileOption::setDeviceId(index)
//   clone                     operators are created in a second graph and arrive through Operation::Clone()
//   run <tensor id>           compile (first time) + run; append the tensor to out.bin
//   feed <tensor id> <off> <len>   an INPUT tensor takes these blob bytes from the next run on
//   bench <warmup> <iters>    time Graph::Run() (after a `run`)
//   end
// For every `run` one line goes to stdout: "ok <name> <offset> <bytes>" or
// "fail <name> <stage>"; for every `bench`: "bench <name> <ms per Run> <ms per Run, device part>" and, with
// TVX_RUNTIME_PROFILE=ops in the environment, "opbench <name> <index> <operator> <microseconds> <operand + result bytes>" per operator.
#include <algorithm>
#include <memory>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <map>
#include <mutex>
#include <thread>
#include <sstream>
#include <string>
#include <vector>

#include "tim/vx/context.h"
#include "tim/vx/graph.h"
#include "tim/transform/layout_inference.h"
#include "tim/vx/ops.h"
#include "tim/vx/platform/platform.h"
#include "tim/vx/tensor.h"

extern "C" double tvx_runtime_last_device_ms(void);
extern "C" void tvx_runtime_set_profile(int mode);
extern "C" int tvx_runtime_last_op_count(void);
extern "C" const char* tvx_runtime_last_op_name(int i);
extern "C" double tvx_runtime_last_op_us(int i);
extern "C" unsigned long long tvx_runtime_last_op_bytes(int i);

using namespace tim::vx;

namespace {

DataType ParseDtype(const std::string& s) {
  static const std::map<std::string, DataType> m = {
      {"UINT8", DataType::UINT8},     {"INT8", DataType::INT8},       {"INT16", DataType::INT16},
      {"INT32", DataType::INT32},     {"FLOAT16", DataType::FLOAT16}, {"FLOAT32", DataType::FLOAT32},
      {"UINT32", DataType::UINT32},   {"BOOL8", DataType::BOOL8}};
  auto it = m.find(s);
  if (it == m.end()) { std::fprintf(stderr, "unknown dtype %s\n", s.c_str()); std::exit(2); }
  return it->second;
}
TensorAttribute ParseAttr(const std::string& s) {
  if (s == "CONSTANT") return TensorAttribute::CONSTANT;
  if (s == "INPUT") return TensorAttribute::INPUT;
  if (s == "OUTPUT") return TensorAttribute::OUTPUT;
  if (s == "TRANSIENT") return TensorAttribute::TRANSIENT;
  return TensorAttribute::VARIABLE;
}
QuantType ParseQuant(const std::string& s) {
  if (s == "ASYMMETRIC") return QuantType::ASYMMETRIC;
  if (s == "SYMMETRIC_PER_CHANNEL") return QuantType::SYMMETRIC_PER_CHANNEL;
  if (s == "ASYMMETRIC_PER_CHANNEL") return QuantType::ASYMMETRIC_PER_CHANNEL;
  if (s == "DYNAMIC_FIXED_POINT") return QuantType::DYNAMIC_FIXED_POINT;
  return QuantType::NONE;
}
PadType ParsePad(const std::string& s) {
  if (s == "VALID") return PadType::VALID;
  if (s == "SAME") return PadType::SAME;
  if (s == "NONE") return PadType::NONE;
  return PadType::AUTO;
}
DataLayout ParseLayout(const std::string& s, DataLayout fallback) {
  static const std::map<std::string, DataLayout> m = {
      {"WHCN", DataLayout::WHCN}, {"CWHN", DataLayout::CWHN}, {"IcWHOc", DataLayout::IcWHOc},
      {"OcIcWH", DataLayout::OcIcWH}, {"IcOcWH", DataLayout::IcOcWH}, {"WHIcOc", DataLayout::WHIcOc},
      {"WCN", DataLayout::WCN}, {"WIcOc", DataLayout::WIcOc}};
  auto it = m.find(s);
  return it == m.end() ? fallback : it->second;
}
PoolType ParsePool(const std::string& s) {
  if (s == "AVG") return PoolType::AVG;
  if (s == "L2") return PoolType::L2;
  if (s == "AVG_ANDROID") return PoolType::AVG_ANDROID;
  return PoolType::MAX;
}

struct Pending {
  std::shared_ptr<Tensor> tensor;
  size_t off = 0, len = 0;
  bool is_input = false;
  // `handles` graphs: the caller-owned buffer behind a CreateIOTensor tensor, and whether the next
  // run must bring a fresh one in through SwapHandle
  std::vector<char>* handle = nullptr;
  bool swap_next = false;
  std::shared_ptr<platform::ITensorHandle> th;  // `platform` graphs: the executable's handle for this tensor
};

}  // namespace

// Processes one graph file; result lines go to `log` (stdout for the plain invocation).
static int RunFile(const char* graphs_path, const char* blob_path, const char* out_path, FILE* log);

// With --threads N the file is processed by N threads, each from Context::Create() on, one after the other under one
// mutex - the reference's multi-thread sample does the same with its LeNet
// (samples/multi_thread_test/multi_thread_test.cc:330-372) - or, with --no-lock, all at once (a context per thread).
// Thread i writes <out>.<i>; the results must be the same bytes and the same result lines.
static int RunThreads(int n_threads, bool lock, const char* graphs_path, const char* blob_path, const char* out_path) {
  std::mutex mutex;
  std::vector<std::thread> threads;
  std::vector<int> status(static_cast<size_t>(n_threads), -1);
  std::vector<std::string> logs(static_cast<size_t>(n_threads)), outs(static_cast<size_t>(n_threads));
  for (int i = 0; i < n_threads; ++i) {
    outs[static_cast<size_t>(i)] = std::string(out_path) + "." + std::to_string(i);
    threads.emplace_back([&, i]() {
      std::unique_lock<std::mutex> guard(mutex, std::defer_lock);
      if (lock) guard.lock();
      char* text = nullptr;
      size_t size = 0;
      FILE* log = open_memstream(&text, &size);
      status[static_cast<size_t>(i)] = RunFile(graphs_path, blob_path, outs[static_cast<size_t>(i)].c_str(), log);
      std::fclose(log);
      logs[static_cast<size_t>(i)].assign(text, size);
      std::free(text);
    });
  }
  for (auto& t : threads) t.join();
  auto slurp = [](const std::string& path) {
    std::ifstream f(path, std::ios::binary);
    return std::string((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
  };
  const std::string first = slurp(outs[0]);
  bool same = status[0] == 0;
  for (int i = 1; i < n_threads; ++i)
    same = same && status[static_cast<size_t>(i)] == 0 && logs[static_cast<size_t>(i)] == logs[0] && slurp(outs[static_cast<size_t>(i)]) == first;
  std::fputs(logs[0].c_str(), stdout);
  std::printf("threads %d %s %zu\n", n_threads, same ? "identical" : "different", first.size());
  return same ? 0 : 1;
}

int main(int argc, char** argv) {
  if (argc >= 2 && std::string(argv[1]) == "--threads") {
    const bool lock = !(argc >= 4 && std::string(argv[3]) == "--no-lock");
    const int first = lock ? 3 : 4;
    if (argc != first + 3) {
      std::fprintf(stderr, "usage: tvx_graph_runner --threads N [--no-lock] graphs.txt blob.bin out.bin\n");
      return 2;
    }
    return RunThreads(std::max(1, atoi(argv[2])), lock, argv[first], argv[first + 1], argv[first + 2]);
  }
  if (argc != 4) {
    std::fprintf(stderr, "usage: tvx_graph_runner graphs.txt blob.bin out.bin\n");
    return 2;
  }
  return RunFile(argv[1], argv[2], argv[3], stdout);
}

static int RunFile(const char* graphs_path, const char* blob_path, const char* out_path, FILE* log) {
  std::ifstream txt(graphs_path);
  std::ifstream blobf(blob_path, std::ios::binary);
  if (!txt || !blobf) { std::fprintf(stderr, "cannot open inputs\n"); return 2; }
  std::vector<char> blob((std::istreambuf_iterator<char>(blobf)), std::istreambuf_iterator<char>());
  FILE* out = std::fopen(out_path, "wb");
  if (!out) { std::fprintf(stderr, "cannot open %s\n", out_path); return 2; }
  size_t out_off = 0;

  auto context = Context::Create();
  std::shared_ptr<Graph> graph, source_graph;
  std::map<int, Pending> tensors;
  std::string name, line;
  bool compiled = false, compile_ok = false, use_handles = false, use_platform = false, use_clone = false;
  std::shared_ptr<Graph> donor;  // with `clone`: operators are created here and Clone()d into the graph
  std::shared_ptr<platform::IExecutor> executor;
  std::shared_ptr<platform::IExecutable> executable;
  std::vector<std::unique_ptr<std::vector<char>>> handle_bufs;

  while (std::getline(txt, line)) {
    std::istringstream ss(line);
    std::string rec;
    if (!(ss >> rec)) continue;
    if (rec == "graph") {
      ss >> name;
      graph = context->CreateGraph();
      tensors.clear();
      compiled = compile_ok = false;
      use_handles = false;
      handle_bufs.clear();
      use_platform = false;
      use_clone = false;
      donor.reset();
      executable.reset();
      executor.reset();
    } else if (rec == "platform") {
      // the graph runs as an executable of the platform API: device -> executor -> Compile(graph),
      // tensor handles allocated by the executable for every graph input / output, Submit + Trigger
      use_platform = true;
    } else if (rec == "device") {
      // the graph is created with a CompileOption that names the GPU it compiles for
      uint32_t id = 0;
      ss >> id;
      CompileOption option;
      option.setDeviceId(id);
      if (option.getDeviceId() != id) { std::fprintf(stderr, "CompileOption lost the device id\n"); return 2; }
      graph = context->CreateGraph(option);
    } else if (rec == "clone") {
      // every operator is created in a second graph and arrives in this one through Operation::Clone()
      use_clone = true;
      donor = context->CreateGraph();
    } else if (rec == "handles") {
      // graph inputs and outputs live in buffers of the caller (Graph::CreateIOTensor), are handed over
      // with FlushCacheForHandle / InvalidateCacheForHandle and exchanged with SwapHandle between runs
      use_handles = true;
    } else if (rec == "t") {
      int id, rank, chdim, ns, nz;
      std::string dt, attr, qt;
      ss >> id >> dt >> attr >> rank;
      ShapeType shape(rank);
      for (auto& d : shape) ss >> d;
      ss >> qt >> chdim >> ns;
      std::vector<float> scales(ns);
      for (auto& s : scales) ss >> s;
      ss >> nz;
      std::vector<int32_t> zps(nz);
      for (auto& z : zps) ss >> z;
      Pending p;
      ss >> p.off >> p.len;
      if (p.off + p.len > blob.size()) { std::fprintf(stderr, "blob range\n"); return 2; }
      const QuantType q = ParseQuant(qt);
      Quantization quant = q == QuantType::NONE ? Quantization() : Quantization(q, chdim, scales, zps);
      TensorSpec spec(ParseDtype(dt), shape, ParseAttr(attr), quant);
      p.is_input = attr == "INPUT";
      const bool at_create = p.len && !p.is_input;
      if (use_handles && (attr == "INPUT" || attr == "OUTPUT")) {
        handle_bufs.emplace_back(new std::vector<char>(static_cast<size_t>(spec.GetByteSize())));
        p.handle = handle_bufs.back().get();
        p.tensor = graph->CreateIOTensor(spec, p.handle->data());
      } else {
        p.tensor = graph->CreateTensor(spec, at_create ? blob.data() + p.off : nullptr);
      }
      tensors[id] = p;
    } else if (rec == "op") {
      std::string kind, pad_type, pool_type, round_type;
      int n_in, n_out;
      ss >> kind >> n_in;
      std::vector<std::shared_ptr<Tensor>> ins, outs;
      for (int i = 0; i < n_in; ++i) {
        int id;
        ss >> id;
        ins.push_back(id < 0 ? graph->CreateTensorPlaceHolder() : tensors.at(id).tensor);
      }
      ss >> n_out;
      for (int i = 0; i < n_out; ++i) {
        int id;
        ss >> id;
        outs.push_back(tensors.at(id).tensor);
      }
      std::array<uint32_t, 4> pad;
      std::array<uint32_t, 2> stride, dil, ksize;
      int32_t multiplier, weights, pool_1d, axis, sm_axis, n_shape;
      float beta;
      ss >> pad_type >> pad[0] >> pad[1] >> pad[2] >> pad[3] >> stride[0] >> stride[1] >> dil[0] >> dil[1] >>
          ksize[0] >> ksize[1] >> multiplier >> weights >> pool_type >> round_type >> pool_1d >> axis >> beta >>
          sm_axis >> n_shape;
      std::vector<uint32_t> new_shape(n_shape);
      for (auto& d : new_shape) ss >> d;
      int32_t groups = 0, conv_1d = 0;
      ss >> groups >> conv_1d;
      int32_t n_perm = 0;
      ss >> n_perm;
      std::vector<uint32_t> perm(n_perm > 0 ? n_perm : 0);
      for (auto& d : perm) ss >> d;
      std::string layout_s = "ANY", klayout_s = "ANY";
      ss >> layout_s >> klayout_s;
      std::array<uint32_t, 2> out_pad = {0, 0};
      ss >> out_pad[0] >> out_pad[1];
      if (!ss) { std::fprintf(stderr, "malformed op record in %s\n", name.c_str()); return 2; }
      const DataLayout layout = ParseLayout(layout_s, DataLayout::WHCN), klayout = ParseLayout(klayout_s, DataLayout::WHIcOc);
      const RoundType rnd = round_type == "CEILING" ? RoundType::CEILING : RoundType::FLOOR;
      std::shared_ptr<Operation> op;
      std::shared_ptr<Graph> target = graph;
      if (use_clone) graph = donor;
      if (kind == "CONV2D" && conv_1d && groups > 1) {
        op = graph->CreateOperation<ops::GroupedConv1d>(ParsePad(pad_type), std::array<uint32_t, 2>{pad[0], pad[1]},
                                                        stride[0], dil[0], static_cast<uint32_t>(groups));
      } else if (kind == "DECONV2D" && conv_1d) {
        op = graph->CreateOperation<ops::DeConv1d>(weights, ParsePad(pad_type), ksize[0], stride[0], out_pad[0],
                                                   std::array<uint32_t, 2>{pad[0], pad[1]},
                                                   static_cast<uint32_t>(groups > 0 ? groups : 1));
      } else if (kind == "CONV2D" && conv_1d) {
        op = graph->CreateOperation<ops::Conv1d>(weights, ParsePad(pad_type), ksize[0], stride[0], dil[0],
                                                 std::array<uint32_t, 2>{pad[0], pad[1]}, multiplier);
      } else if (kind == "CONV2D" && groups > 1) {
        if (ParsePad(pad_type) == PadType::AUTO)
          op = graph->CreateOperation<ops::GroupedConv2d>(pad, stride, dil, groups, layout, klayout);
        else
          op = graph->CreateOperation<ops::GroupedConv2d>(ParsePad(pad_type), stride, dil, groups, layout, klayout);
      } else if (kind == "CONV2D") {
        op = graph->CreateOperation<ops::Conv2d>(weights, ParsePad(pad_type), ksize, stride, dil, pad, multiplier, layout, klayout);
      } else if (kind == "FCL") {
        op = graph->CreateOperation<ops::FullyConnected>(static_cast<uint32_t>(axis), static_cast<uint32_t>(weights));
      } else if (kind == "POOL") {
        if (pool_1d == 1) {
          op = graph->CreateOperation<ops::Pool1d>(ParsePool(pool_type), std::array<uint32_t, 2>{pad[0], pad[1]},
                                                   ksize[0], stride[0], rnd);
        } else if (pool_1d == 2) {  // the global-pooling constructor: ksize carries the input size
          op = graph->CreateOperation<ops::Pool2d>(ParsePool(pool_type), ksize, rnd, layout);
        } else if (pool_1d == 3) {  // the adaptive constructor: ksize = input size, stride = output size
          op = graph->CreateOperation<ops::Pool2d>(ParsePool(pool_type), ksize, stride, rnd, layout);
        } else if (ParsePad(pad_type) == PadType::AUTO) {
          op = graph->CreateOperation<ops::Pool2d>(ParsePool(pool_type), pad, ksize, stride, rnd, layout);
        } else {
          op = graph->CreateOperation<ops::Pool2d>(ParsePool(pool_type), ParsePad(pad_type), ksize, stride, rnd, layout);
        }
      } else if (kind == "RELU") {
        op = graph->CreateOperation<ops::Relu>();
      } else if (kind == "RELU6") {
        op = graph->CreateOperation<ops::Relu6>();
      } else if (kind == "ADD") {
        op = graph->CreateOperation<ops::Add>();
      } else if (kind == "SOFTMAX") {
        op = graph->CreateOperation<ops::Softmax>(beta, sm_axis);
      } else if (kind == "RESHAPE") {
        op = graph->CreateOperation<ops::Reshape>(new_shape);
      } else if (kind == "DECONV2D") {
        op = graph->CreateOperation<ops::DeConv2d>(weights, ParsePad(pad_type), ksize, stride, out_pad, pad,
                                                   static_cast<uint32_t>(groups > 0 ? groups : 1), layout, klayout);
      } else if (kind == "DATACONVERT") {
        op = graph->CreateOperation<ops::DataConvert>();
      } else if (kind == "TRANSPOSE") {
        op = graph->CreateOperation<ops::Transpose>(perm);
      } else {
        std::fprintf(stderr, "unknown op kind %s\n", kind.c_str());
        return 2;
      }
      if (use_clone) {
        graph = target;
        op = op->Clone(graph);
      }
      op->BindInputs(ins).BindOutputs(outs);
    } else if (rec == "infer") {
      // layout inference: the rewritten graph replaces the one built so far; INPUT / OUTPUT
      // tensors are looked up through the map it returns
      auto r = tim::transform::LayoutInference(graph, context);
      for (auto& kv : tensors) {
        auto it = r.second.find(kv.second.tensor);
        if (it != r.second.end()) kv.second.tensor = it->second;
      }
      source_graph = graph;
      graph = r.first;
    } else if (rec == "run") {
      int id;
      ss >> id;
      if (!compiled && use_platform) {
        compiled = true;
        auto devices = platform::IDevice::Enumerate();
        if (!devices.empty()) executor = devices[0]->CreateExecutor(0, -1, context);
        if (executor) executable = platform::Compile(graph, executor);
        if (executable) {
          auto handle_for = [&](const std::shared_ptr<Tensor>& t) {
            auto th = executable->AllocateTensor(t->GetSpec());
            for (auto& kv : tensors)
              if (kv.second.tensor == t) kv.second.th = th;
            return th;
          };
          for (auto& t : graph->InputsTensor()) executable->SetInput(handle_for(t));
          for (auto& t : graph->OutputsTensor()) executable->SetOutput(handle_for(t));
          compile_ok = executable->Verify();
        }
      }
      if (!compiled) {
        compile_ok = graph->Compile();
        compiled = true;
      }
      const char* stage = nullptr;
      if (!compile_ok) stage = "compile";
      if (!stage)
        for (auto& kv : tensors) {
          Pending& p = kv.second;
          if (!p.is_input || !p.len) continue;
          if (use_platform) {
            if (!p.th || !p.th->CopyDataToTensor(blob.data() + p.off, static_cast<uint32_t>(p.len))) stage = "copy_in";
          } else if (p.handle) {
            if (p.swap_next) {  // a new buffer of the caller's takes the old one's place
              handle_bufs.emplace_back(new std::vector<char>(p.handle->size()));
              std::vector<char>* fresh = handle_bufs.back().get();
              void* old = nullptr;
              if (!p.tensor->SwapHandle(fresh->data(), false, &old) || old != p.handle->data()) stage = "swap_handle";
              std::memset(p.handle->data(), 0xA5, p.handle->size());  // the old buffer must not be read again
              p.handle = fresh;
              p.swap_next = false;
            }
            std::memcpy(p.handle->data(), blob.data() + p.off, std::min(p.len, p.handle->size()));
            if (!p.tensor->FlushCacheForHandle()) stage = "flush_handle";
          } else if (!p.tensor->CopyDataToTensor(blob.data() + p.off, static_cast<uint32_t>(p.len))) {
            stage = "copy_in";
          }
        }
      if (!stage && !(use_platform ? executable->Submit(executable) && executor->Trigger() : graph->Run())) stage = "run";
      std::vector<char> result;
      if (!stage) {
        Pending& po = tensors.at(id);
        auto& t = po.tensor;
        result.resize(t->GetSpec().GetByteSize());
        if (use_platform) {
          if (!po.th || !po.th->CopyDataFromTensor(result.data())) stage = "copy_out";
        } else if (po.handle) {
          if (!t->InvalidateCacheForHandle()) stage = "invalidate_handle";
          else std::memcpy(result.data(), po.handle->data(), result.size());  // straight out of the caller's buffer
        } else if (!t->CopyDataFromTensor(result.data())) {
          stage = "copy_out";
        }
      }
      if (stage) {
        std::fprintf(log, "fail %s %s\n", name.c_str(), stage);
      } else {
        std::fwrite(result.data(), 1, result.size(), out);
        std::fprintf(log, "ok %s %zu %zu\n", name.c_str(), out_off, result.size());
        out_off += result.size();
      }
      std::fflush(log);
    } else if (rec == "feed") {
      // the input tensor takes other bytes of the blob from the next `run` on
      int id;
      size_t off, len;
      ss >> id >> off >> len;
      auto it = tensors.find(id);
      if (it == tensors.end() || !it->second.is_input || off + len > blob.size()) {
        std::fprintf(stderr, "bad feed record\n");
        return 2;
      }
      it->second.off = off;
      it->second.len = len;
      it->second.swap_next = it->second.handle != nullptr;
    } else if (rec == "bench") {
      int warmup, iters;
      ss >> warmup >> iters;
      if (!compile_ok) { std::fprintf(log, "fail %s bench\n", name.c_str()); continue; }
      // every iteration hands the inputs over again, as an application with new data would: the time per
      // Run() then holds the host -> device copy of the inputs as well as the download of the output
      auto feed = [&]() {
        for (auto& kv : tensors)
          if (kv.second.is_input && kv.second.len && !kv.second.handle && !kv.second.th)
            kv.second.tensor->CopyDataToTensor(blob.data() + kv.second.off, static_cast<uint32_t>(kv.second.len));
      };
      // two passes: Run() as an application calls it (no profiling: one synchronisation, at its end) for the time per
      // Run(); then with the operator sequence timed on its own (a synchronisation in front of it and behind it)
      tvx_runtime_set_profile(0);
      for (int i = 0; i < warmup; ++i) { feed(); graph->Run(); }
      auto t0 = std::chrono::steady_clock::now();
      for (int i = 0; i < iters; ++i) { feed(); graph->Run(); }
      auto t1 = std::chrono::steady_clock::now();
      const char* env_profile = std::getenv("TVX_RUNTIME_PROFILE");
      tvx_runtime_set_profile(env_profile && std::string(env_profile) == "ops" ? 2 : 1);
      for (int i = 0; i < warmup; ++i) { feed(); graph->Run(); }
      double dev_ms = 0;
      std::vector<double> op_us;
      for (int i = 0; i < iters; ++i) {
        feed();
        graph->Run();
        dev_ms += tvx_runtime_last_device_ms();
        const int n_ops = tvx_runtime_last_op_count();  // only with TVX_RUNTIME_PROFILE=ops
        op_us.resize(static_cast<size_t>(n_ops), 0.0);
        for (int o = 0; o < n_ops; ++o) op_us[static_cast<size_t>(o)] += tvx_runtime_last_op_us(o);
      }
      tvx_runtime_set_profile(-1);
      std::fprintf(log, "bench %s %.6f %.6f\n", name.c_str(),
                  std::chrono::duration<double, std::milli>(t1 - t0).count() / iters, dev_ms / iters);
      for (size_t o = 0; o < op_us.size(); ++o) {
        const char* raw_name = tvx_runtime_last_op_name(static_cast<int>(o));
        std::string op_name = raw_name ? raw_name : "?";
        for (char& c : op_name) if (c == ' ') c = '_';
        std::fprintf(log, "opbench %s %zu %s %.3f %llu\n", name.c_str(), o, op_name.c_str(), op_us[o] / iters,
                    tvx_runtime_last_op_bytes(static_cast<int>(o)));
      }
      std::fflush(log);
    } else if (rec == "end") {
      graph.reset();
      source_graph.reset();
      tensors.clear();
    }
  }
  std::fclose(out);
  return 0;
}
