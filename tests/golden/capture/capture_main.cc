// Fixture recorder. Linked with the runtime's host-side front end and with
// one of the reference's *_test.cc files (compiled where it lies, never
// copied), it runs every TEST body with an Executor that computes nothing and
// writes, for each comparison the test makes, one JSON case:
// the graph (tensors with inferred shapes, operator attributes with resolved
// padding), constant and input data, the expected vector and its tolerance.
//
// Usage: capture_<name> <out.json>
#include <cinttypes>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "gtest/gtest.h"
#include "runtime.h"

using namespace tim::vx;

namespace {
struct TestEntry {
  std::string suite, name;
  void (*body)();
};
std::vector<TestEntry>& Tests() {
  static std::vector<TestEntry> t;
  return t;
}
GraphImpl* g_last_graph = nullptr;
std::string g_current;
int g_case_in_test = 0;
FILE* g_out = nullptr;
bool g_first_case = true;
bool g_compile_failed = false;

class NullExecutor : public Executor {
 public:
  bool Realize(GraphImpl* graph) override {
    g_last_graph = graph;
    return true;
  }
  bool Execute(GraphImpl* graph) override {
    g_last_graph = graph;
    for (auto& t : graph->outputs_tensor_)
      static_cast<TensorImpl*>(t.get())->EnsureHostBuffer();
    return true;
  }
};

float HalfToFloat(uint16_t h) {
  uint32_t sign = (h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, man = h & 0x3ff, bits;
  if (exp == 0) {
    if (!man) bits = sign;
    else {
      int e = -1;
      do { ++e; man <<= 1; } while (!(man & 0x400));
      bits = sign | ((112 - e) << 23) | ((man & 0x3ff) << 13);
    }
  } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
  else bits = sign | ((exp + 112) << 23) | (man << 13);
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

void EmitNumbers(const std::vector<double>& v, bool integral) {
  bool all_same = !v.empty();
  for (double x : v) if (x != v[0]) { all_same = false; break; }
  if (all_same && v.size() > 16) {
    if (integral) std::fprintf(g_out, "{\"fill\": %lld, \"n\": %zu}", (long long)v[0], v.size());
    else std::fprintf(g_out, "{\"fill\": %.9g, \"n\": %zu}", v[0], v.size());
    return;
  }
  std::fputc('[', g_out);
  for (size_t i = 0; i < v.size(); ++i) {
    if (i) std::fputc(',', g_out);
    if (integral) std::fprintf(g_out, "%lld", (long long)v[i]);
    else std::fprintf(g_out, "%.9g", v[i]);
  }
  std::fputc(']', g_out);
}

bool IsIntegral(DataType t) {
  return !(t == DataType::FLOAT16 || t == DataType::FLOAT32);
}

std::vector<double> TensorValues(TensorImpl* t) {
  std::vector<double> v;
  uint8_t* p = t->HostData();
  if (!p) return v;
  size_t n = static_cast<size_t>(t->spec_.GetElementNum());
  v.reserve(n);
  for (size_t i = 0; i < n; ++i) {
    switch (t->spec_.datatype_) {
      case DataType::UINT8: v.push_back(p[i]); break;
      case DataType::INT8: v.push_back(reinterpret_cast<int8_t*>(p)[i]); break;
      case DataType::INT16: v.push_back(reinterpret_cast<int16_t*>(p)[i]); break;
      case DataType::UINT16: v.push_back(reinterpret_cast<uint16_t*>(p)[i]); break;
      case DataType::INT32: v.push_back(reinterpret_cast<int32_t*>(p)[i]); break;
      case DataType::UINT32: v.push_back(reinterpret_cast<uint32_t*>(p)[i]); break;
      case DataType::FLOAT32: v.push_back(reinterpret_cast<float*>(p)[i]); break;
      case DataType::FLOAT16: v.push_back(HalfToFloat(reinterpret_cast<uint16_t*>(p)[i])); break;
      default: v.push_back(0);
    }
  }
  return v;
}

const char* QuantName(QuantType q) {
  switch (q) {
    case QuantType::NONE: return "NONE";
    case QuantType::ASYMMETRIC: return "ASYMMETRIC";
    case QuantType::SYMMETRIC_PER_CHANNEL: return "SYMMETRIC_PER_CHANNEL";
    case QuantType::ASYMMETRIC_PER_CHANNEL: return "ASYMMETRIC_PER_CHANNEL";
    case QuantType::DYNAMIC_FIXED_POINT: return "DYNAMIC_FIXED_POINT";
  }
  return "?";
}

const char* AttrName(TensorAttribute a) {
  if (a & TensorAttribute::CONSTANT) return "CONSTANT";
  if (a & TensorAttribute::INPUT) return "INPUT";
  if (a & TensorAttribute::OUTPUT) return "OUTPUT";
  if (a & TensorAttribute::TRANSIENT) return "TRANSIENT";
  return "VARIABLE";
}

void EmitTensor(TensorImpl* t, TensorImpl* data_from = nullptr) {
  if (!data_from) data_from = t;
  std::fprintf(g_out, "{\"id\": %u, \"dtype\": \"%s\", \"attr\": \"%s\", \"shape\": [",
               t->id_, DataTypeName(t->spec_.datatype_), AttrName(t->spec_.attr_));
  for (size_t i = 0; i < t->spec_.shape_.size(); ++i)
    std::fprintf(g_out, "%s%u", i ? "," : "", t->spec_.shape_[i]);
  const Quantization& q = t->spec_.quantization_;
  std::fprintf(g_out, "], \"quant\": {\"type\": \"%s\", \"channel_dim\": %d, \"scales\": [",
               QuantName(q.Type()), q.ChannelDim());
  for (size_t i = 0; i < q.Scales().size(); ++i)
    std::fprintf(g_out, "%s%.9g", i ? "," : "", q.Scales()[i]);
  std::fprintf(g_out, "], \"zero_points\": [");
  for (size_t i = 0; i < q.ZeroPoints().size(); ++i)
    std::fprintf(g_out, "%s%d", i ? "," : "", q.ZeroPoints()[i]);
  std::fprintf(g_out, "]}, \"data\": ");
  bool has = (t->spec_.attr_ & (TensorAttribute::CONSTANT | TensorAttribute::INPUT)) &&
             data_from->HostData();
  if (has) EmitNumbers(TensorValues(data_from), IsIntegral(t->spec_.datatype_));
  else std::fprintf(g_out, "null");
  std::fputc('}', g_out);
}

const char* PadName(PadType p) {
  switch (p) {
    case PadType::NONE: return "NONE";
    case PadType::AUTO: return "AUTO";
    case PadType::VALID: return "VALID";
    case PadType::SAME: return "SAME";
  }
  return "?";
}

const char* LayoutName(DataLayout l) {
  switch (l) {
    case DataLayout::WHCN: return "WHCN";
    case DataLayout::CWHN: return "CWHN";
    case DataLayout::IcWHOc: return "IcWHOc";
    case DataLayout::OcIcWH: return "OcIcWH";
    case DataLayout::IcOcWH: return "IcOcWH";
    case DataLayout::WHIcOc: return "WHIcOc";
    case DataLayout::WCN: return "WCN";
    case DataLayout::WIcOc: return "WIcOc";
    default: return "ANY";
  }
}

void EmitOp(OpImpl* op) {
  const OpAttrs& a = op->attrs_;
  std::fprintf(g_out, "{\"kind\": \"%s\", \"inputs\": [", OpKindName(op->kind_));
  bool first = true;
  for (auto& t : op->inputs_tensor_) {
    if (t->IsPlaceHolder()) continue;
    std::fprintf(g_out, "%s%u", first ? "" : ",", t->GetId());
    first = false;
  }
  std::fprintf(g_out, "], \"outputs\": [");
  for (size_t i = 0; i < op->outputs_tensor_.size(); ++i)
    std::fprintf(g_out, "%s%u", i ? "," : "", op->outputs_tensor_[i]->GetId());
  static const char* pool_names[] = {"MAX", "AVG", "L2", "AVG_ANDROID"};
  std::fprintf(g_out,
               "], \"attrs\": {\"pad_type\": \"%s\", \"pad\": [%u,%u,%u,%u], "
               "\"stride\": [%u,%u], \"dilation\": [%u,%u], \"ksize\": [%u,%u], "
               "\"multiplier\": %d, \"weights\": %u, \"pool_type\": \"%s\", "
               "\"round_type\": \"%s\", \"pool_1d\": %s, \"axis\": %u, \"groups\": %d, \"conv_1d\": %s, \"beta\": %.9g, \"sm_axis\": %d, \"layout\": \"%s\", \"kernel_layout\": \"%s\", \"output_padding\": [%u,%u], \"perm\": [",
               PadName(a.pad_type), a.pad[0], a.pad[1], a.pad[2], a.pad[3],
               a.stride[0], a.stride[1], a.dilation[0], a.dilation[1], a.ksize[0],
               a.ksize[1], a.multiplier, a.weights,
               pool_names[static_cast<int>(a.pool_type)],
               a.round_type == RoundType::CEILING ? "CEILING" : "FLOOR",
               a.pool_1d ? "true" : "false", a.axis, a.groups, a.conv_1d ? "true" : "false", a.beta, a.sm_axis, LayoutName(op->layout_), LayoutName(a.kernel_layout), a.output_padding[0], a.output_padding[1]);
  for (size_t i = 0; i < a.perm.size(); ++i) std::fprintf(g_out, "%s%u", i ? "," : "", a.perm[i]);
  std::fprintf(g_out, "]}}");
}
}  // namespace

namespace tim {
namespace vx {
std::unique_ptr<Executor> CreateExecutor() {
  return std::unique_ptr<Executor>(new NullExecutor());
}
}  // namespace vx
}  // namespace tim

namespace tvxcap {
Reg::Reg(const char* suite, const char* name, void (*body)()) {
  Tests().push_back({suite, name, body});
}

Sink Check(bool ok, const char* expr) {
  if (!ok) {
    std::fprintf(stderr, "  [%s] EXPECT_TRUE(%s) is false\n", g_current.c_str(), expr);
    if (std::strstr(expr, "Compile")) g_compile_failed = true;
  }
  return Sink();
}

static GraphImpl* g_li_source = nullptr;
static GraphImpl* g_li_result = nullptr;
static std::map<TensorImpl*, TensorImpl*> g_li_map;
static std::shared_ptr<Graph> g_li_keep_src, g_li_keep_dst;
void NoteLayoutInference(
    const std::shared_ptr<Graph>& src,
    const std::pair<std::shared_ptr<Graph>, std::map<std::shared_ptr<Tensor>, std::shared_ptr<Tensor>>>& r) {
  g_li_keep_src = src;
  g_li_keep_dst = r.first;
  g_li_source = static_cast<GraphImpl*>(src.get());
  g_li_result = static_cast<GraphImpl*>(r.first.get());
  g_li_map.clear();
  for (auto& kv : r.second)
    g_li_map[static_cast<TensorImpl*>(kv.first.get())] = static_cast<TensorImpl*>(kv.second.get());
}

void ForgetLayoutInference() {
  g_li_source = g_li_result = nullptr;
  g_li_map.clear();
  g_li_keep_src.reset();
  g_li_keep_dst.reset();
}

std::vector<double> g_near;
void RecordGolden(const std::vector<double>& golden, double tol, const char* how);
int RecordMem(const void*, const void* expected, size_t bytes) {
  if (g_last_graph && g_last_graph->outputs_tensor_.size() == 1) {
    auto* out = static_cast<TensorImpl*>(g_last_graph->outputs_tensor_[0].get());
    if (out->spec_.datatype_ == DataType::FLOAT32 && bytes == static_cast<size_t>(out->spec_.GetByteSize())) {
      const float* f = static_cast<const float*>(expected);
      RecordGolden(std::vector<double>(f, f + bytes / 4), 0.0, "eq");
    }
  }
  return 0;
}
void RecordGolden(const std::vector<double>& golden, double tol, const char* how);
Sink RecordNear(double golden, double tol) {
  g_near.push_back(golden);
  // the graph is alive only inside the test body: emit as soon as every output element has its scalar
  if (g_last_graph && !g_compile_failed && g_last_graph->outputs_tensor_.size() == 1 &&
      static_cast<int64_t>(g_near.size()) == g_last_graph->outputs_tensor_[0]->GetSpec().GetElementNum()) {
    RecordGolden(g_near, tol, "near");
    g_near.clear();
  }
  return Sink();
}

void RecordGolden(const std::vector<double>& golden, double tol, const char* how) {
  if (!g_last_graph || g_compile_failed) {
    std::fprintf(stderr, "  [%s] no compiled graph: case skipped\n", g_current.c_str());
    return;
  }
  GraphImpl* g = g_last_graph;
  // a graph that came out of layout inference: the fixture holds the SOURCE graph, with the data
  // the test fed to the rewritten graph's inputs
  const bool from_li = g_li_result == g && g_li_source;
  if (from_li) g = g_li_source;
  if (g->outputs_tensor_.size() != 1) {
    std::fprintf(stderr, "  [%s] %zu graph outputs: case skipped\n", g_current.c_str(),
                 g->outputs_tensor_.size());
    return;
  }
  auto* out = static_cast<TensorImpl*>(g->outputs_tensor_[0].get());
  std::fprintf(g_out, "%s\n{\"test\": \"%s\", \"index\": %d, \"tensors\": [",
               g_first_case ? "" : ",", g_current.c_str(), g_case_in_test++);
  g_first_case = false;
  // every tensor an operator touches
  std::vector<TensorImpl*> seen;
  auto add = [&](const std::shared_ptr<Tensor>& t) {
    if (t->IsPlaceHolder()) return;
    auto* ti = static_cast<TensorImpl*>(t.get());
    for (auto* s : seen) if (s == ti) return;
    seen.push_back(ti);
  };
  std::vector<Operation*> ops = g->sorted_ops_;
  if (from_li) {  // never compiled: creation order (the tests build their graphs front to back)
    ops.clear();
    for (auto& op : g->OpVector()) ops.push_back(op.get());
  }
  for (Operation* op : ops) {
    for (auto& t : op->impl()->inputs_tensor_) add(t);
    for (auto& t : op->impl()->outputs_tensor_) add(t);
  }
  for (size_t i = 0; i < seen.size(); ++i) {
    if (i) std::fputc(',', g_out);
    auto it = g_li_map.find(seen[i]);
    EmitTensor(seen[i], from_li && it != g_li_map.end() ? it->second : nullptr);
  }
  std::fprintf(g_out, "], \"ops\": [");
  for (size_t i = 0; i < ops.size(); ++i) {
    if (i) std::fputc(',', g_out);
    EmitOp(ops[i]->impl().get());
  }
  std::fprintf(g_out, "], \"layout_inference\": %s, \"output\": %u, \"compare\": \"%s\", \"tol\": %.9g, \"golden\": ",
               from_li ? "true" : "false", out->id_, how, tol);
  EmitNumbers(golden, IsIntegral(out->spec_.datatype_));
  std::fputc('}', g_out);
}
}  // namespace tvxcap

int main(int argc, char** argv) {
  if (argc < 2) {
    std::fprintf(stderr, "usage: %s out.json\n", argv[0]);
    return 2;
  }
  g_out = std::fopen(argv[1], "w");
  if (!g_out) return 2;
  std::fprintf(g_out, "[");
  for (auto& t : Tests()) {
    g_current = t.suite + "." + t.name;
    g_case_in_test = 0;
    g_last_graph = nullptr;
    g_compile_failed = false;
    tvxcap::g_near.clear();
    t.body();
    tvxcap::ForgetLayoutInference();
    g_last_graph = nullptr;
    std::fprintf(stderr, "%s: %d case(s)\n", g_current.c_str(), g_case_in_test);
  }
  std::fprintf(g_out, "\n]\n");
  std::fclose(g_out);
  return 0;
}
