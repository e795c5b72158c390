// C ABI of include/tvx_hip.h: library/device helpers, descriptor validation,
// requantization tables, and the walk over kernel variants that picks the
// first one claiming an operator (the counterpart of ovxlib's
// vsi_nn_kernel_selector priority walk, src/tim/vx/internal/src/kernel/vsi_nn_kernel.c:1178-1299).
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <new>

#include "tvx_internal.h"
#include "variants.h"

namespace tvx {

static thread_local char g_error[512] = "";

int SetError(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return status;
}

int DeviceBuffer::Alloc(size_t n) {
  if (ptr) { (void)hipFree(ptr); ptr = nullptr; }
  bytes = n;
  if (n == 0) return TVX_OK;
  TVX_HIP_CHECK(hipMalloc(&ptr, n));
  return TVX_OK;
}

int DeviceBuffer::Upload(const void* host, size_t n) {
  int s = Alloc(n);
  if (s != TVX_OK) return s;
  if (n) TVX_HIP_CHECK(hipMemcpy(ptr, host, n, hipMemcpyHostToDevice));
  return TVX_OK;
}

static void QuantizeMultiplier(double m, int32_t* mult, int32_t* shift) {
  if (!(m > 0.0) || !std::isfinite(m)) {
    *mult = 0;
    *shift = 1;
    return;
  }
  int e = 0;
  const double q = std::frexp(m, &e);
  int64_t qi = std::llround(q * 2147483648.0);
  if (qi == (int64_t{1} << 31)) {
    qi >>= 1;
    ++e;
  }
  *mult = static_cast<int32_t>(qi);
  *shift = 31 - e;
}

int BuildRequantTables(uint32_t channels, float in_scale, float w_scale,
                       const float* w_scales, float out_scale,
                       std::vector<int32_t>* mult, std::vector<int32_t>* shift) {
  mult->resize(channels);
  shift->resize(channels);
  if (!(out_scale > 0.f) || !(in_scale > 0.f))
    return SetError(TVX_E_INVALID, "scales must be positive (in %g, out %g)", in_scale, out_scale);
  for (uint32_t c = 0; c < channels; ++c) {
    const double ws = w_scales ? static_cast<double>(w_scales[c]) : static_cast<double>(w_scale);
    if (!(ws > 0.0)) return SetError(TVX_E_INVALID, "weight scale of channel %u is %g", c, ws);
    int32_t m, s;
    QuantizeMultiplier(static_cast<double>(in_scale) * ws / static_cast<double>(out_scale), &m, &s);
    if (s < 1)
      return SetError(TVX_E_UNSUPPORTED, "requantization multiplier of channel %u is >= 2^30", c);
    if (s > 62) {  // underflows to 0 for every int32 accumulator
      m = 0;
      s = 1;
    }
    (*mult)[c] = m;
    (*shift)[c] = s;
  }
  return TVX_OK;
}

int64_t AccumulatorBound(uint64_t reduction, const void* bias_host, uint32_t channels) {
  // |sum (x - zx)(w - zw)| <= reduction * 255 * 255 for 8-bit operands
  int64_t b = static_cast<int64_t>(reduction) * 255 * 255;
  const int32_t* bias = static_cast<const int32_t*>(bias_host);
  int64_t mx = 0;
  for (uint32_t c = 0; bias && c < channels; ++c) mx = std::max<int64_t>(mx, std::llabs(static_cast<long long>(bias[c])));
  return b + mx;
}

int BuildRequantRecords(const std::vector<int32_t>& mult, const std::vector<int32_t>& shift,
                        int channels, int alloc, int out_zp, std::vector<int32_t>* records,
                        int64_t acc_bound) {
  int rq = kRqFastNoTie;
  for (int c = 0; c < channels; ++c) {
    const int32_t m = mult[c], s = shift[c];
    if (m == 0) continue;
    // (zp << t) + 2^30 must stay inside int32
    if (s < 33 || s - 32 > 20) { rq = kRqGeneric; break; }
    // a tie needs an accumulator v with v * m = 2^(s-1) (mod 2^s): ctz(v) = s - 1 - ctz(m), which
    // no 32-bit v has when that exceeds 31, and no accumulator of this operator has when
    // 2^(s - 1 - ctz(m)) is beyond the largest magnitude it can reach
    const int need = s - 1 - __builtin_ctz(static_cast<uint32_t>(m));
    const bool reachable = need <= 31 && (acc_bound < 0 || (int64_t{1} << need) <= acc_bound);
    if (reachable) rq = kRqFast;
  }
  records->assign(static_cast<size_t>(alloc) * 4, 0);
  for (int c = 0; c < alloc; ++c) {
    int32_t m = c < channels ? mult[c] : 0, s = c < channels ? shift[c] : 33;
    if (m == 0) s = 33;
    int32_t* q = &(*records)[static_cast<size_t>(c) * 4];
    q[0] = m;
    if (rq == kRqGeneric) {
      q[1] = s;
    } else {
      const int t = s - 32;
      const int ctz = m ? __builtin_ctz(static_cast<uint32_t>(m)) : 0;
      q[1] = t;
      q[2] = (1 << (t - 1)) + (out_zp << t);
      q[3] = ctz == 0 ? -1 : static_cast<int32_t>((uint32_t{1} << (32 - ctz)) - 1);
    }
  }
  return rq;
}

void ActRange(int out_dtype, float out_scale, int32_t out_zp, int act, int32_t* lo, int32_t* hi) {
  *lo = out_dtype == TVX_U8 ? 0 : -128;
  *hi = out_dtype == TVX_U8 ? 255 : 127;
  if (act == TVX_ACT_RELU || act == TVX_ACT_RELU6) {
    if (out_zp > *lo) *lo = out_zp;
  }
  if (act == TVX_ACT_RELU6) {
    const double six = std::nearbyint(6.0 / static_cast<double>(out_scale));
    if (six < 1e9) {
      const int64_t top = static_cast<int64_t>(out_zp) + static_cast<int64_t>(six);
      if (top < *hi) *hi = static_cast<int32_t>(top);
    }
  }
  if (*lo > *hi) *lo = *hi;
}

static bool ValidDtype(int d) { return d >= TVX_U8 && d <= TVX_F32; }

static int CheckOperandTypes(int in, int w, int out, const char* what) {
  if (!ValidDtype(in) || !ValidDtype(w) || !ValidDtype(out))
    return SetError(TVX_E_INVALID, "%s: unknown dtype", what);
  if (IsQuant(in)) {
    // u8 x u8, i8 x i8, and either activation with int8 per-channel weights
    if (!IsQuant(w) || !IsQuant(out) || out != in)
      return SetError(TVX_E_UNSUPPORTED, "%s: dtype combination in=%d w=%d out=%d", what, in, w, out);
    if (in == TVX_I8 && w == TVX_U8)
      return SetError(TVX_E_UNSUPPORTED, "%s: int8 activations with uint8 weights", what);
  } else if (w != in || out != in) {
    return SetError(TVX_E_UNSUPPORTED, "%s: dtype combination in=%d w=%d out=%d", what, in, w, out);
  }
  return TVX_OK;
}

// A zero point is a code of its tensor's type. The kernels' accumulator bounds (|x - zx|, |w - zw| <= 255)
// and the 32-bit requantization records (out_zp << t) rely on it.
static int CheckZeroPoint(int dtype, int32_t zp, const char* what, const char* which) {
  if (!IsQuant(dtype)) return TVX_OK;
  const int32_t lo = dtype == TVX_U8 ? 0 : -128, hi = dtype == TVX_U8 ? 255 : 127;
  if (zp < lo || zp > hi)
    return SetError(TVX_E_INVALID, "%s: %s zero point %d outside [%d, %d]", what, which, zp, lo, hi);
  return TVX_OK;
}

static int CheckConvZeroPoints(int in_dtype, int32_t in_zp, int w_dtype, int32_t w_zp, bool per_channel,
                               int out_dtype, int32_t out_zp, const char* what) {
  int s = CheckZeroPoint(in_dtype, in_zp, what, "input");
  if (s == TVX_OK && !per_channel) s = CheckZeroPoint(w_dtype, w_zp, what, "weight");
  if (s == TVX_OK) s = CheckZeroPoint(out_dtype, out_zp, what, "output");
  return s;
}

}  // namespace tvx

using namespace tvx;

extern "C" {

const char* tvx_version(void) { return "tvx-hip 0.1 (gfx950)"; }
const char* tvx_last_error(void) { return g_error; }

const char* tvx_status_string(int status) {
  switch (status) {
    case TVX_OK: return "ok";
    case TVX_E_INVALID: return "invalid argument";
    case TVX_E_UNSUPPORTED: return "unsupported";
    case TVX_E_DEVICE: return "device error";
    case TVX_E_NOMEM: return "out of memory";
  }
  return "unknown status";
}

int tvx_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

int tvx_malloc(void** dev_ptr, size_t bytes) {
  if (!dev_ptr) return SetError(TVX_E_INVALID, "tvx_malloc: null result pointer");
  *dev_ptr = nullptr;
  if (bytes == 0) return TVX_OK;
  hipError_t e = hipMalloc(dev_ptr, bytes);
  if (e == hipErrorOutOfMemory) return SetError(TVX_E_NOMEM, "hipMalloc(%zu) out of memory", bytes);
  if (e != hipSuccess) return SetError(TVX_E_DEVICE, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
  return TVX_OK;
}

int tvx_host_malloc(void** host_ptr, size_t bytes) {
  if (!host_ptr) return SetError(TVX_E_INVALID, "tvx_host_malloc: null result pointer");
  *host_ptr = nullptr;
  if (bytes == 0) return TVX_OK;
  if (tvx_device_count() <= 0) return SetError(TVX_E_DEVICE, "no HIP device: page-locked memory needs one");
  hipError_t e = hipHostMalloc(host_ptr, bytes, hipHostMallocDefault);
  if (e == hipErrorOutOfMemory) return SetError(TVX_E_NOMEM, "hipHostMalloc(%zu) out of memory", bytes);
  if (e != hipSuccess) return SetError(TVX_E_DEVICE, "hipHostMalloc(%zu): %s", bytes, hipGetErrorString(e));
  return TVX_OK;
}

int tvx_host_free(void* host_ptr) {
  if (host_ptr) TVX_HIP_CHECK(hipHostFree(host_ptr));
  return TVX_OK;
}

int tvx_free(void* dev_ptr) {
  if (dev_ptr) TVX_HIP_CHECK(hipFree(dev_ptr));
  return TVX_OK;
}

int tvx_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return TVX_OK;
  if (!dst || !src) return SetError(TVX_E_INVALID, "tvx_memcpy_h2d: null pointer");
  TVX_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)));
  return TVX_OK;
}

int tvx_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return TVX_OK;
  if (!dst || !src) return SetError(TVX_E_INVALID, "tvx_memcpy_d2h: null pointer");
  TVX_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
  return TVX_OK;
}

int tvx_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
  if (bytes == 0) return TVX_OK;
  if (!dst || !src) return SetError(TVX_E_INVALID, "tvx_memcpy_d2d: null pointer");
  TVX_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream)));
  return TVX_OK;
}

int tvx_stream_create(void** stream) {
  if (!stream) return SetError(TVX_E_INVALID, "tvx_stream_create: null result pointer");
  hipStream_t s = nullptr;
  TVX_HIP_CHECK(hipStreamCreate(&s));  // default priority
  *stream = s;
  return TVX_OK;
}

int tvx_stream_destroy(void* stream) {
  if (stream) TVX_HIP_CHECK(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return TVX_OK;
}

int tvx_stream_synchronize(void* stream) {
  TVX_HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return TVX_OK;
}

int tvx_event_create(void** event) {
  if (!event) return SetError(TVX_E_INVALID, "tvx_event_create: null result pointer");
  hipEvent_t e = nullptr;
  TVX_HIP_CHECK(hipEventCreate(&e));
  *event = e;
  return TVX_OK;
}

int tvx_event_destroy(void* event) {
  if (event) TVX_HIP_CHECK(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return TVX_OK;
}

int tvx_event_record(void* event, void* stream) {
  if (!event) return SetError(TVX_E_INVALID, "tvx_event_record: null event");
  TVX_HIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
  return TVX_OK;
}

int tvx_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!start || !stop || !ms) return SetError(TVX_E_INVALID, "tvx_event_elapsed_ms: null argument");
  TVX_HIP_CHECK(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return TVX_OK;
}

int tvx_quantize_multiplier(double m, int32_t* mult, int32_t* shift) {
  if (!mult || !shift) return SetError(TVX_E_INVALID, "tvx_quantize_multiplier: null pointer");
  QuantizeMultiplier(m, mult, shift);
  return TVX_OK;
}

int64_t tvx_requantize(int32_t acc, int32_t mult, int32_t shift) {
  const int64_t p = static_cast<int64_t>(acc) * static_cast<int64_t>(mult);
  if (shift < 1) return p > 0 ? (int64_t{1} << 40) : (p < 0 ? -(int64_t{1} << 40) : 0);
  if (shift > 62) return 0;
  int64_t fl = p >> shift;
  const int64_t rem = p & ((int64_t{1} << shift) - 1);
  const int64_t half = int64_t{1} << (shift - 1);
  if (rem > half || (rem == half && (fl & 1))) ++fl;
  return fl;
}

static int NoGpu() {
  if (tvx_device_count() <= 0)
    return SetError(TVX_E_DEVICE, "no HIP device: this library has no CPU path");
  return TVX_OK;
}

// tvx_conv2d_create, and (fused_pool) the convolution half of tvx_conv2d_pool_create: then only the kernels with
// a pooled epilogue are asked.
static int CreateConv(const tvx_conv2d_desc* d, const void* weights_host, const void* bias_host, bool fused_pool,
                      tvx_op** out) {
  if (!d->in_w || !d->in_h || !d->in_c || !d->batch || !d->k_w || !d->k_h || !d->out_w ||
      !d->out_h || !d->out_c || !d->stride_w || !d->stride_h || !d->dilation_w || !d->dilation_h)
    return SetError(TVX_E_INVALID, "tvx_conv2d_create: zero extent, stride or dilation");
  if (d->multiplier < 0) return SetError(TVX_E_INVALID, "tvx_conv2d_create: negative multiplier");
  if (d->groups < 0 || (d->groups > 1 && (d->multiplier != 0 || d->in_c % d->groups || d->out_c % d->groups)))
    return SetError(TVX_E_INVALID, "tvx_conv2d_create: %d groups do not divide in_c %u / out_c %u (or multiplier set)",
                    d->groups, d->in_c, d->out_c);
  if (d->multiplier > 0 && d->out_c != d->in_c * static_cast<uint32_t>(d->multiplier))
    return SetError(TVX_E_INVALID, "tvx_conv2d_create: depthwise out_c %u != in_c %u * multiplier %d",
                    d->out_c, d->in_c, d->multiplier);
  // the last window row/column must start inside the padded input
  if (static_cast<uint64_t>(d->out_w - 1) * d->stride_w >= static_cast<uint64_t>(d->in_w) + d->pad_left ||
      static_cast<uint64_t>(d->out_h - 1) * d->stride_h >= static_cast<uint64_t>(d->in_h) + d->pad_top)
    return SetError(TVX_E_INVALID, "tvx_conv2d_create: output extent reaches past the input");
  int s = CheckOperandTypes(d->in_dtype, d->w_dtype, d->out_dtype, "tvx_conv2d_create");
  if (s == TVX_OK) s = CheckConvZeroPoints(d->in_dtype, d->in_zp, d->w_dtype, d->w_zp, d->w_scales != nullptr,
                                           d->out_dtype, d->out_zp, "tvx_conv2d_create");
  if (s != TVX_OK) return s;
  if ((s = NoGpu()) != TVX_OK) return s;

  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_conv2d_create: host allocation failed");
  op->kind = OP_CONV2D;
  op->conv = *d;
  op->fused_pool = fused_pool ? 1 : 0;
  // one input channel per group is a depthwise convolution in other words: same weight image
  // ({k_w, k_h, 1, out_c} = {k_w, k_h, in_c * m, 1}), same channel map (oc / m), and the
  // depthwise kernels apply
  if (d->groups > 1 && static_cast<uint32_t>(d->groups) == d->in_c) {
    op->conv.multiplier = static_cast<int32_t>(d->out_c / d->in_c);
    op->conv.groups = 0;
  }
  const tvx_conv2d_desc norm = op->conv;
  d = &norm;
  op->conv.w_scales = nullptr;  // host pointer is not kept (`norm` still has it for the setup functions)
  op->quantized = IsQuant(d->in_dtype);
  op->has_const_weights = weights_host != nullptr;
  op->w_zp = d->w_scales ? 0 : d->w_zp;
  if (op->quantized) {
    std::vector<int32_t>&mult = op->h_mult, &shift = op->h_shift;
    s = BuildRequantTables(d->out_c, d->in_scale, d->w_scale, d->w_scales, d->out_scale, &mult, &shift);
    if (s == TVX_OK) s = op->mult.Upload(mult.data(), mult.size() * 4);
    if (s == TVX_OK) s = op->shift.Upload(shift.data(), shift.size() * 4);
    ActRange(d->out_dtype, d->out_scale, d->out_zp, d->activation, &op->act_lo, &op->act_hi);
    if (s != TVX_OK) { delete op; return s; }
  }
  s = TVX_E_UNSUPPORTED;
  if (fused_pool) {
    s = ConvIm2colSetup(op, d, weights_host, bias_host);
    if (s == TVX_E_UNSUPPORTED) s = ConvIgemmSetup(op, d, weights_host, bias_host);
  } else {
    for (ConvSetupFn fn : ConvVariants()) {
      s = fn(op, d, weights_host, bias_host);
      if (s != TVX_E_UNSUPPORTED) break;
    }
  }
  if (s != TVX_OK) { delete op; return s; }
  *out = op;
  return TVX_OK;
}

int tvx_conv2d_create(const tvx_conv2d_desc* d, const void* weights_host,
                      const void* bias_host, tvx_op** out) {
  if (!d || !out) return SetError(TVX_E_INVALID, "tvx_conv2d_create: null argument");
  *out = nullptr;
  return CreateConv(d, weights_host, bias_host, false, out);
}

int tvx_conv2d_pool_create(const tvx_conv2d_desc* d, const tvx_pool2d_desc* pool, const void* weights_host,
                           const void* bias_host, tvx_op** out) {
  if (!d || !pool || !out) return SetError(TVX_E_INVALID, "tvx_conv2d_pool_create: null argument");
  *out = nullptr;
  if (pool->in_w != d->out_w || pool->in_h != d->out_h || pool->channels != d->out_c || pool->batch != d->batch ||
      pool->dtype != d->out_dtype)
    return SetError(TVX_E_INVALID, "tvx_conv2d_pool_create: the pooling's input is not the convolution's output");
  const bool fusable = IsQuant(d->in_dtype) && IsQuant(d->out_dtype) && weights_host && pool->pool_type == TVX_POOL_MAX &&
                       pool->k_w == 2 && pool->k_h == 2 && pool->stride_w == 2 && pool->stride_h == 2 &&
                       pool->pad_left == 0 && pool->pad_top == 0 && d->out_w % 2 == 0 && d->out_h % 2 == 0 &&
                       pool->out_w == d->out_w / 2 && pool->out_h == d->out_h / 2 &&
                       pool->in_scale == d->out_scale && pool->in_zp == d->out_zp &&
                       pool->out_scale == d->out_scale && pool->out_zp == d->out_zp;
  if (!fusable)
    return SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_pool_create: quantized convolution with constant weights and a 2 x 2 / stride-2 "
                    "max pooling without padding that keeps the quantization are what is fused");
  const int s = CreateConv(d, weights_host, bias_host, true, out);
  if (s == TVX_E_UNSUPPORTED) return SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_pool_create: no fused kernel for this convolution");
  if (s == TVX_OK) (*out)->pool = *pool;
  return s;
}

int tvx_conv2d_add_create(const tvx_conv2d_desc* d, const tvx_eltwise_desc* add, int conv_operand,
                          const void* weights_host, const void* bias_host, tvx_op** out) {
  if (!d || !add || !out) return SetError(TVX_E_INVALID, "tvx_conv2d_add_create: null argument");
  *out = nullptr;
  if (conv_operand != 1 && conv_operand != 2)
    return SetError(TVX_E_INVALID, "tvx_conv2d_add_create: conv_operand must be 1 or 2");
  if (!IsQuant(d->in_dtype) || !IsQuant(d->out_dtype) || add->dtype != d->out_dtype || !weights_host ||
      !(add->a_scale > 0.f) || !(add->b_scale > 0.f) || !(add->out_scale > 0.f))
    return SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_add_create: quantized tensors of one type and constant weights only");
  // the convolution's own output quantization is the Add's for that operand
  const float conv_scale = conv_operand == 1 ? add->a_scale : add->b_scale;
  const int32_t conv_zp = conv_operand == 1 ? add->a_zp : add->b_zp;
  if (conv_scale != d->out_scale || conv_zp != d->out_zp)
    return SetError(TVX_E_INVALID, "tvx_conv2d_add_create: the Add's operand %d is not quantized like the convolution's output", conv_operand);
  if (!d->in_w || !d->in_h || !d->in_c || !d->batch || !d->out_c)
    return SetError(TVX_E_INVALID, "tvx_conv2d_add_create: zero extent");
  int s = CheckOperandTypes(d->in_dtype, d->w_dtype, d->out_dtype, "tvx_conv2d_add_create");
  if (s == TVX_OK) s = CheckConvZeroPoints(d->in_dtype, d->in_zp, d->w_dtype, d->w_zp, d->w_scales != nullptr,
                                           d->out_dtype, d->out_zp, "tvx_conv2d_add_create");
  if (s == TVX_OK) s = CheckZeroPoint(add->dtype, add->a_zp, "tvx_conv2d_add_create", "Add operand");
  if (s == TVX_OK) s = CheckZeroPoint(add->dtype, add->b_zp, "tvx_conv2d_add_create", "Add operand");
  if (s == TVX_OK) s = CheckZeroPoint(add->dtype, add->out_zp, "tvx_conv2d_add_create", "Add output");
  if (s != TVX_OK) return s;
  if ((s = NoGpu()) != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_conv2d_add_create: host allocation failed");
  op->kind = OP_CONV2D;
  op->conv = *d;
  op->elt = *add;
  op->fused_add = conv_operand;
  const tvx_conv2d_desc norm = op->conv;
  op->conv.w_scales = nullptr;
  op->quantized = true;
  op->has_const_weights = true;
  op->w_zp = d->w_scales ? 0 : d->w_zp;
  s = BuildRequantTables(d->out_c, d->in_scale, d->w_scale, d->w_scales, d->out_scale, &op->h_mult, &op->h_shift);
  ActRange(d->out_dtype, d->out_scale, d->out_zp, d->activation, &op->act_lo, &op->act_hi);
  if (s == TVX_OK) s = PwConvSetup(op, &norm, weights_host, bias_host);  // the kernel that has the fused form
  if (s != TVX_OK) {
    delete op;
    return s == TVX_E_UNSUPPORTED ? SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_add_create: no fused kernel for this convolution") : s;
  }
  *out = op;
  return TVX_OK;
}

// ---- channel-blocked tensors (an order the runtime may give TRANSIENT tensors of small planes) ----
int tvx_conv2d_blocked_create(const tvx_conv2d_desc* d, const tvx_eltwise_desc* add, int conv_operand,
                              const void* weights_host, const void* bias_host, tvx_op** out) {
  if (!d || !out) return SetError(TVX_E_INVALID, "tvx_conv2d_blocked_create: null argument");
  *out = nullptr;
  if (add && conv_operand != 1 && conv_operand != 2)
    return SetError(TVX_E_INVALID, "tvx_conv2d_blocked_create: conv_operand must be 1 or 2");
  if (!d->in_w || !d->in_h || !d->in_c || !d->batch || !d->k_w || !d->k_h || !d->out_w || !d->out_h || !d->out_c ||
      !d->stride_w || !d->stride_h || !d->dilation_w || !d->dilation_h)
    return SetError(TVX_E_INVALID, "tvx_conv2d_blocked_create: zero extent, stride or dilation");
  if (static_cast<uint64_t>(d->out_w - 1) * d->stride_w >= static_cast<uint64_t>(d->in_w) + d->pad_left ||
      static_cast<uint64_t>(d->out_h - 1) * d->stride_h >= static_cast<uint64_t>(d->in_h) + d->pad_top)
    return SetError(TVX_E_INVALID, "tvx_conv2d_blocked_create: output extent reaches past the input");
  if (!IsQuant(d->in_dtype) || !weights_host)
    return SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_blocked_create: quantized tensors and constant weights only");
  int s = CheckOperandTypes(d->in_dtype, d->w_dtype, d->out_dtype, "tvx_conv2d_blocked_create");
  if (s == TVX_OK) s = CheckConvZeroPoints(d->in_dtype, d->in_zp, d->w_dtype, d->w_zp, d->w_scales != nullptr,
                                           d->out_dtype, d->out_zp, "tvx_conv2d_blocked_create");
  if (s == TVX_OK && add) {
    if (add->dtype != d->out_dtype || !(add->a_scale > 0.f) || !(add->b_scale > 0.f) || !(add->out_scale > 0.f))
      return SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_blocked_create: the Add must be quantized like the convolution's output type");
    const float conv_scale = conv_operand == 1 ? add->a_scale : add->b_scale;
    const int32_t conv_zp = conv_operand == 1 ? add->a_zp : add->b_zp;
    if (conv_scale != d->out_scale || conv_zp != d->out_zp)
      return SetError(TVX_E_INVALID, "tvx_conv2d_blocked_create: the Add's operand %d is not quantized like the convolution's output", conv_operand);
    s = CheckZeroPoint(add->dtype, add->a_zp, "tvx_conv2d_blocked_create", "Add operand");
    if (s == TVX_OK) s = CheckZeroPoint(add->dtype, add->b_zp, "tvx_conv2d_blocked_create", "Add operand");
    if (s == TVX_OK) s = CheckZeroPoint(add->dtype, add->out_zp, "tvx_conv2d_blocked_create", "Add output");
  }
  if (s != TVX_OK) return s;
  if ((s = NoGpu()) != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_conv2d_blocked_create: host allocation failed");
  op->kind = OP_CONV2D;
  op->conv = *d;
  if (add) {
    op->elt = *add;
    op->fused_add = conv_operand;
  }
  const tvx_conv2d_desc norm = op->conv;
  op->conv.w_scales = nullptr;
  op->quantized = true;
  op->has_const_weights = true;
  op->w_zp = d->w_scales ? 0 : d->w_zp;
  s = BuildRequantTables(d->out_c, d->in_scale, d->w_scale, d->w_scales, d->out_scale, &op->h_mult, &op->h_shift);
  ActRange(d->out_dtype, d->out_scale, d->out_zp, d->activation, &op->act_lo, &op->act_hi);
  if (s == TVX_OK) {
    s = BlockedPwSetup(op, &norm, weights_host, bias_host);
    if (s == TVX_E_UNSUPPORTED && !add) s = BlockedDwSetup(op, &norm, weights_host, bias_host);
  }
  if (s != TVX_OK) {
    delete op;
    return s == TVX_E_UNSUPPORTED ? SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_blocked_create: no kernel for this convolution on blocked tensors") : s;
  }
  *out = op;
  return TVX_OK;
}

int tvx_conv2d_to_blocked_create(const tvx_conv2d_desc* d, const void* weights_host, const void* bias_host, tvx_op** out) {
  static const char* const fn = "tvx_conv2d_to_blocked_create";
  if (!d || !out) return SetError(TVX_E_INVALID, "%s: null argument", fn);
  *out = nullptr;
  if (!d->in_w || !d->in_h || !d->in_c || !d->batch || !d->k_w || !d->k_h || !d->out_w || !d->out_h || !d->out_c ||
      !d->stride_w || !d->stride_h || !d->dilation_w || !d->dilation_h)
    return SetError(TVX_E_INVALID, "%s: zero extent, stride or dilation", fn);
  if (static_cast<uint64_t>(d->out_w - 1) * d->stride_w >= static_cast<uint64_t>(d->in_w) + d->pad_left ||
      static_cast<uint64_t>(d->out_h - 1) * d->stride_h >= static_cast<uint64_t>(d->in_h) + d->pad_top)
    return SetError(TVX_E_INVALID, "%s: output extent reaches past the input", fn);
  if (!IsQuant(d->in_dtype) || !weights_host) return SetError(TVX_E_UNSUPPORTED, "%s: quantized tensors and constant weights only", fn);
  if (d->multiplier != 1 || d->out_c != d->in_c) return SetError(TVX_E_UNSUPPORTED, "%s: depthwise convolutions with multiplier 1 only", fn);
  int s = CheckOperandTypes(d->in_dtype, d->w_dtype, d->out_dtype, fn);
  if (s == TVX_OK) s = CheckConvZeroPoints(d->in_dtype, d->in_zp, d->w_dtype, d->w_zp, d->w_scales != nullptr, d->out_dtype, d->out_zp, fn);
  if (s != TVX_OK) return s;
  if ((s = NoGpu()) != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "%s: host allocation failed", fn);
  op->kind = OP_CONV2D;
  op->conv = *d;
  const tvx_conv2d_desc norm = op->conv;
  op->conv.w_scales = nullptr;
  op->quantized = true;
  op->has_const_weights = true;
  op->out_blocked = 1;
  op->w_zp = d->w_scales ? 0 : d->w_zp;
  s = BuildRequantTables(d->out_c, d->in_scale, d->w_scale, d->w_scales, d->out_scale, &op->h_mult, &op->h_shift);
  ActRange(d->out_dtype, d->out_scale, d->out_zp, d->activation, &op->act_lo, &op->act_hi);
  if (s == TVX_OK) s = DwPlanesSetup(op, &norm, weights_host, bias_host);
  if (s != TVX_OK) {
    delete op;
    return s == TVX_E_UNSUPPORTED ? SetError(TVX_E_UNSUPPORTED, "%s: no kernel writes this convolution's result blocked", fn) : s;
  }
  *out = op;
  return TVX_OK;
}

int tvx_pool2d_blocked_create(const tvx_pool2d_desc* d, tvx_op** out) {
  if (!d || !out) return SetError(TVX_E_INVALID, "tvx_pool2d_blocked_create: null argument");
  *out = nullptr;
  if (!d->in_w || !d->in_h || !d->channels || !d->batch || !d->out_w || !d->out_h || !d->k_w || !d->k_h || !d->stride_w || !d->stride_h)
    return SetError(TVX_E_INVALID, "tvx_pool2d_blocked_create: zero extent or stride");
  if (!IsQuant(d->dtype) || !(d->in_scale > 0.f) || !(d->out_scale > 0.f))
    return SetError(TVX_E_UNSUPPORTED, "tvx_pool2d_blocked_create: quantized tensors with positive scales only");
  int s = CheckZeroPoint(d->dtype, d->in_zp, "tvx_pool2d_blocked_create", "input");
  if (s == TVX_OK) s = CheckZeroPoint(d->dtype, d->out_zp, "tvx_pool2d_blocked_create", "output");
  if (s == TVX_OK) s = NoGpu();
  if (s != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_pool2d_blocked_create: host allocation failed");
  op->kind = OP_POOL2D;
  op->pool = *d;
  op->quantized = true;
  s = BlockedAvgSetup(op);
  if (s != TVX_OK) {
    delete op;
    return s == TVX_E_UNSUPPORTED ? SetError(TVX_E_UNSUPPORTED, "tvx_pool2d_blocked_create: whole-plane average pooling only") : s;
  }
  *out = op;
  return TVX_OK;
}

int tvx_layout_create(uint32_t w, uint32_t h, uint32_t c, uint32_t n, int to_blocked, tvx_op** out) {
  if (!out) return SetError(TVX_E_INVALID, "tvx_layout_create: null argument");
  *out = nullptr;
  if (!w || !h || !c || !n) return SetError(TVX_E_INVALID, "tvx_layout_create: zero extent");
  int s = NoGpu();
  if (s != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_layout_create: host allocation failed");
  op->kind = OP_TRANSPOSE;
  s = LayoutSetup(op, w, h, c, n, to_blocked ? 1 : 0);
  if (s != TVX_OK) {
    delete op;
    return s == TVX_E_UNSUPPORTED ? SetError(TVX_E_UNSUPPORTED, "tvx_layout_create: channels must be a multiple of 16") : s;
  }
  *out = op;
  return TVX_OK;
}

int tvx_conv2d_dw_pw_create(const tvx_conv2d_desc* dw, const void* dw_w, const void* dw_b,
                            const tvx_conv2d_desc* pw, const void* pw_w, const void* pw_b,
                            const tvx_eltwise_desc* add, int conv_operand, tvx_op** out) {
  if (!dw || !pw || !out) return SetError(TVX_E_INVALID, "tvx_conv2d_dw_pw_create: null argument");
  *out = nullptr;
  if (add && conv_operand != 1 && conv_operand != 2)
    return SetError(TVX_E_INVALID, "tvx_conv2d_dw_pw_create: conv_operand must be 1 or 2");
  if (!IsQuant(dw->in_dtype) || !IsQuant(dw->out_dtype) || !IsQuant(pw->out_dtype) || !dw_w || !pw_w)
    return SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_dw_pw_create: quantized tensors and constant weights only");
  if (!dw->in_w || !dw->in_h || !dw->in_c || !dw->batch || !dw->out_w || !dw->out_h || !pw->out_c)
    return SetError(TVX_E_INVALID, "tvx_conv2d_dw_pw_create: zero extent");
  if (dw->multiplier < 1 || dw->out_c != dw->in_c * static_cast<uint32_t>(dw->multiplier))
    return SetError(TVX_E_INVALID, "tvx_conv2d_dw_pw_create: the first convolution must be depthwise");
  int s = CheckOperandTypes(dw->in_dtype, dw->w_dtype, dw->out_dtype, "tvx_conv2d_dw_pw_create");
  if (s == TVX_OK) s = CheckOperandTypes(pw->in_dtype, pw->w_dtype, pw->out_dtype, "tvx_conv2d_dw_pw_create");
  if (s == TVX_OK) s = CheckConvZeroPoints(dw->in_dtype, dw->in_zp, dw->w_dtype, dw->w_zp, dw->w_scales != nullptr,
                                           dw->out_dtype, dw->out_zp, "tvx_conv2d_dw_pw_create");
  if (s == TVX_OK) s = CheckConvZeroPoints(pw->in_dtype, pw->in_zp, pw->w_dtype, pw->w_zp, pw->w_scales != nullptr,
                                           pw->out_dtype, pw->out_zp, "tvx_conv2d_dw_pw_create");
  if (s != TVX_OK) return s;
  if (add) {
    if (add->dtype != pw->out_dtype || !(add->a_scale > 0.f) || !(add->b_scale > 0.f) || !(add->out_scale > 0.f))
      return SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_dw_pw_create: the Add must be of the convolution's output type");
    const float conv_scale = conv_operand == 1 ? add->a_scale : add->b_scale;
    const int32_t conv_zp = conv_operand == 1 ? add->a_zp : add->b_zp;
    if (conv_scale != pw->out_scale || conv_zp != pw->out_zp)
      return SetError(TVX_E_INVALID, "tvx_conv2d_dw_pw_create: the Add's operand %d is not quantized like the convolution's output", conv_operand);
    s = CheckZeroPoint(add->dtype, add->a_zp, "tvx_conv2d_dw_pw_create", "Add operand");
    if (s == TVX_OK) s = CheckZeroPoint(add->dtype, add->b_zp, "tvx_conv2d_dw_pw_create", "Add operand");
    if (s == TVX_OK) s = CheckZeroPoint(add->dtype, add->out_zp, "tvx_conv2d_dw_pw_create", "Add output");
    if (s != TVX_OK) return s;
  }
  if ((s = NoGpu()) != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_conv2d_dw_pw_create: host allocation failed");
  op->kind = OP_CONV2D;
  op->conv = *pw;
  op->conv.w_scales = nullptr;
  if (add) {
    op->elt = *add;
    op->fused_add = conv_operand;
  }
  op->quantized = true;
  op->has_const_weights = true;
  op->w_zp = pw->w_scales ? 0 : pw->w_zp;
  std::vector<int32_t> dw_mult, dw_shift;
  int32_t dw_lo = 0, dw_hi = 0;
  s = BuildRequantTables(pw->out_c, pw->in_scale, pw->w_scale, pw->w_scales, pw->out_scale, &op->h_mult, &op->h_shift);
  if (s == TVX_OK) s = BuildRequantTables(dw->out_c, dw->in_scale, dw->w_scale, dw->w_scales, dw->out_scale, &dw_mult, &dw_shift);
  ActRange(pw->out_dtype, pw->out_scale, pw->out_zp, pw->activation, &op->act_lo, &op->act_hi);
  ActRange(dw->out_dtype, dw->out_scale, dw->out_zp, dw->activation, &dw_lo, &dw_hi);
  if (s == TVX_OK) s = DwPwSetup(op, dw, dw_w, dw_b, dw_mult, dw_shift, dw_lo, dw_hi, pw, pw_w, pw_b);
  if (s != TVX_OK) {
    delete op;
    return s == TVX_E_UNSUPPORTED ? SetError(TVX_E_UNSUPPORTED, "tvx_conv2d_dw_pw_create: no fused kernel for this pair") : s;
  }
  *out = op;
  return TVX_OK;
}

int tvx_mbconv_create(const tvx_conv2d_desc* expand, const void* expand_w, const void* expand_b,
                      const tvx_conv2d_desc* dw, const void* dw_w, const void* dw_b,
                      const tvx_conv2d_desc* project, const void* project_w, const void* project_b,
                      const tvx_eltwise_desc* add, int conv_operand, tvx_op** out) {
  static const char* const fn = "tvx_mbconv_create";
  if (!expand || !dw || !project || !out) return SetError(TVX_E_INVALID, "%s: null argument", fn);
  *out = nullptr;
  if (add && conv_operand != 1 && conv_operand != 2) return SetError(TVX_E_INVALID, "%s: conv_operand must be 1 or 2", fn);
  const tvx_conv2d_desc* stages[3] = {expand, dw, project};
  const void* weights[3] = {expand_w, dw_w, project_w};
  for (int i = 0; i < 3; ++i) {
    const tvx_conv2d_desc* d = stages[i];
    if (!IsQuant(d->in_dtype) || !IsQuant(d->out_dtype) || !weights[i])
      return SetError(TVX_E_UNSUPPORTED, "%s: quantized tensors and constant weights only", fn);
    if (!d->in_w || !d->in_h || !d->in_c || !d->batch || !d->out_w || !d->out_h || !d->out_c)
      return SetError(TVX_E_INVALID, "%s: zero extent", fn);
    int s = CheckOperandTypes(d->in_dtype, d->w_dtype, d->out_dtype, fn);
    if (s == TVX_OK) s = CheckConvZeroPoints(d->in_dtype, d->in_zp, d->w_dtype, d->w_zp, d->w_scales != nullptr, d->out_dtype, d->out_zp, fn);
    if (s != TVX_OK) return s;
  }
  if (dw->multiplier != 1 || dw->out_c != dw->in_c)
    return SetError(TVX_E_INVALID, "%s: the second convolution must be depthwise with multiplier 1", fn);
  if (add) {
    if (add->dtype != project->out_dtype || !(add->a_scale > 0.f) || !(add->b_scale > 0.f) || !(add->out_scale > 0.f))
      return SetError(TVX_E_UNSUPPORTED, "%s: the Add must be of the block's output type", fn);
    const float conv_scale = conv_operand == 1 ? add->a_scale : add->b_scale;
    const int32_t conv_zp = conv_operand == 1 ? add->a_zp : add->b_zp;
    if (conv_scale != project->out_scale || conv_zp != project->out_zp)
      return SetError(TVX_E_INVALID, "%s: the Add's operand %d is not quantized like the projection's output", fn, conv_operand);
    int s = CheckZeroPoint(add->dtype, add->a_zp, fn, "Add operand");
    if (s == TVX_OK) s = CheckZeroPoint(add->dtype, add->b_zp, fn, "Add operand");
    if (s == TVX_OK) s = CheckZeroPoint(add->dtype, add->out_zp, fn, "Add output");
    if (s != TVX_OK) return s;
  }
  int s = NoGpu();
  if (s != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "%s: host allocation failed", fn);
  op->kind = OP_CONV2D;
  op->conv = *project;
  op->conv.w_scales = nullptr;
  if (add) {
    op->elt = *add;
    op->fused_add = conv_operand;
  }
  op->quantized = true;
  op->has_const_weights = true;
  op->w_zp = project->w_scales ? 0 : project->w_zp;
  std::vector<int32_t> mult[2], shift[2];
  MbStage st[2] = {{expand, expand_w, expand_b, &mult[0], &shift[0], 0, 0}, {dw, dw_w, dw_b, &mult[1], &shift[1], 0, 0}};
  s = BuildRequantTables(project->out_c, project->in_scale, project->w_scale, project->w_scales, project->out_scale, &op->h_mult, &op->h_shift);
  ActRange(project->out_dtype, project->out_scale, project->out_zp, project->activation, &op->act_lo, &op->act_hi);
  for (int i = 0; i < 2 && s == TVX_OK; ++i) {
    const tvx_conv2d_desc* d = st[i].desc;
    s = BuildRequantTables(d->out_c, d->in_scale, d->w_scale, d->w_scales, d->out_scale, &mult[i], &shift[i]);
    ActRange(d->out_dtype, d->out_scale, d->out_zp, d->activation, &st[i].lo, &st[i].hi);
  }
  if (s == TVX_OK) s = MbConvSetup(op, st[0], st[1], project, project_w, project_b);
  if (s != TVX_OK) {
    delete op;
    return s == TVX_E_UNSUPPORTED ? SetError(TVX_E_UNSUPPORTED, "%s: no fused kernel for this block", fn) : s;
  }
  *out = op;
  return TVX_OK;
}

int tvx_deconv2d_create(const tvx_conv2d_desc* d, const void* weights_host, const void* bias_host,
                        tvx_op** out) {
  if (!d || !out) return SetError(TVX_E_INVALID, "tvx_deconv2d_create: null argument");
  *out = nullptr;
  if (!d->in_w || !d->in_h || !d->in_c || !d->batch || !d->k_w || !d->k_h || !d->out_w || !d->out_h ||
      !d->out_c || !d->stride_w || !d->stride_h)
    return SetError(TVX_E_INVALID, "tvx_deconv2d_create: zero extent or stride");
  if (d->dilation_w != 1 || d->dilation_h != 1)
    return SetError(TVX_E_INVALID, "tvx_deconv2d_create: dilation must be 1");
  if (d->multiplier != 0 && (d->multiplier != 1 || d->out_c != d->in_c))
    return SetError(TVX_E_INVALID, "tvx_deconv2d_create: the depthwise form has multiplier 1 and out_c == in_c");
  if (d->groups < 0 || (d->groups > 1 && (d->multiplier != 0 || d->in_c % d->groups || d->out_c % d->groups)))
    return SetError(TVX_E_INVALID, "tvx_deconv2d_create: %d groups do not divide in_c %u / out_c %u (or multiplier set)",
                    d->groups, d->in_c, d->out_c);
  // Output pixels beyond what the last input pixel's window reaches hold the bias alone (output padding; the
  // reference's DeConv1d test pads one column at stride 1 and expects exactly that), but not without bound:
  // at most one more window and stride.
  if (static_cast<uint64_t>(d->out_w) + d->pad_left > static_cast<uint64_t>(d->in_w - 1) * d->stride_w + 2ull * d->k_w + d->stride_w ||
      static_cast<uint64_t>(d->out_h) + d->pad_top > static_cast<uint64_t>(d->in_h - 1) * d->stride_h + 2ull * d->k_h + d->stride_h)
    return SetError(TVX_E_INVALID, "tvx_deconv2d_create: output extent reaches far past the last input window");
  int s = CheckOperandTypes(d->in_dtype, d->w_dtype, d->out_dtype, "tvx_deconv2d_create");
  if (s == TVX_OK) s = CheckConvZeroPoints(d->in_dtype, d->in_zp, d->w_dtype, d->w_zp, d->w_scales != nullptr,
                                           d->out_dtype, d->out_zp, "tvx_deconv2d_create");
  if (s != TVX_OK) return s;
  if ((s = NoGpu()) != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_deconv2d_create: host allocation failed");
  op->kind = OP_DECONV2D;
  op->conv = *d;
  if (d->groups > 1 && static_cast<uint32_t>(d->groups) == d->in_c && d->out_c == d->in_c) {
    op->conv.multiplier = 1;  // one channel per group: the depthwise form
    op->conv.groups = 0;
  }
  const tvx_conv2d_desc norm = op->conv;
  op->conv.w_scales = nullptr;
  op->quantized = IsQuant(d->in_dtype);
  op->has_const_weights = weights_host != nullptr;
  op->w_zp = d->w_scales ? 0 : d->w_zp;
  if (op->quantized) {
    std::vector<int32_t>&mult = op->h_mult, &shift = op->h_shift;
    s = BuildRequantTables(d->out_c, d->in_scale, d->w_scale, d->w_scales, d->out_scale, &mult, &shift);
    if (s == TVX_OK) s = op->mult.Upload(mult.data(), mult.size() * 4);
    if (s == TVX_OK) s = op->shift.Upload(shift.data(), shift.size() * 4);
    ActRange(d->out_dtype, d->out_scale, d->out_zp, d->activation, &op->act_lo, &op->act_hi);
    if (s != TVX_OK) { delete op; return s; }
  }
  s = ConvGenericSetup(op, &norm, weights_host, bias_host);
  if (s != TVX_OK) { delete op; return s; }
  *out = op;
  return TVX_OK;
}

int tvx_fully_connected_create(const tvx_fc_desc* d, const void* weights_host,
                               const void* bias_host, tvx_op** out) {
  if (!d || !out) return SetError(TVX_E_INVALID, "tvx_fully_connected_create: null argument");
  *out = nullptr;
  if (!d->m || !d->k || !d->n) return SetError(TVX_E_INVALID, "tvx_fully_connected_create: zero extent");
  int s = CheckOperandTypes(d->in_dtype, d->w_dtype, d->out_dtype, "tvx_fully_connected_create");
  if (s == TVX_OK) s = CheckConvZeroPoints(d->in_dtype, d->in_zp, d->w_dtype, d->w_zp, d->w_scales != nullptr,
                                           d->out_dtype, d->out_zp, "tvx_fully_connected_create");
  if (s != TVX_OK) return s;
  if ((s = NoGpu()) != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_fully_connected_create: host allocation failed");
  op->kind = OP_FC;
  op->fc = *d;
  op->fc.w_scales = nullptr;
  op->quantized = IsQuant(d->in_dtype);
  op->has_const_weights = weights_host != nullptr;
  op->w_zp = d->w_scales ? 0 : d->w_zp;
  if (op->quantized) {
    std::vector<int32_t>&mult = op->h_mult, &shift = op->h_shift;
    s = BuildRequantTables(d->n, d->in_scale, d->w_scale, d->w_scales, d->out_scale, &mult, &shift);
    if (s == TVX_OK) s = op->mult.Upload(mult.data(), mult.size() * 4);
    if (s == TVX_OK) s = op->shift.Upload(shift.data(), shift.size() * 4);
    ActRange(d->out_dtype, d->out_scale, d->out_zp, d->activation, &op->act_lo, &op->act_hi);
    if (s != TVX_OK) { delete op; return s; }
  }
  s = TVX_E_UNSUPPORTED;
  for (FcSetupFn fn : FcVariants()) {
    s = fn(op, d, weights_host, bias_host);
    if (s != TVX_E_UNSUPPORTED) break;
  }
  if (s != TVX_OK) { delete op; return s; }
  *out = op;
  return TVX_OK;
}

int tvx_fully_connected_softmax_create(const tvx_fc_desc* d, const tvx_softmax_desc* sm, const void* weights_host,
                                       const void* bias_host, tvx_op** out) {
  if (!d || !sm || !out) return SetError(TVX_E_INVALID, "tvx_fully_connected_softmax_create: null argument");
  *out = nullptr;
  if (!d->m || !d->k || !d->n) return SetError(TVX_E_INVALID, "tvx_fully_connected_softmax_create: zero extent");
  if (sm->channels != d->n || sm->rows != d->m || sm->inner > 1 || sm->in_dtype != d->out_dtype)
    return SetError(TVX_E_INVALID, "tvx_fully_connected_softmax_create: the Softmax does not run along the FullyConnected's outputs");
  if (!IsQuant(d->in_dtype) || !IsQuant(d->out_dtype) || !weights_host || sm->in_scale != d->out_scale || sm->in_zp != d->out_zp)
    return SetError(TVX_E_UNSUPPORTED, "tvx_fully_connected_softmax_create: quantized tensors, constant weights and one quantization "
                    "of the intermediate codes are what is fused");
  int s = CheckOperandTypes(d->in_dtype, d->w_dtype, d->out_dtype, "tvx_fully_connected_softmax_create");
  if (s == TVX_OK) s = CheckConvZeroPoints(d->in_dtype, d->in_zp, d->w_dtype, d->w_zp, d->w_scales != nullptr,
                                           d->out_dtype, d->out_zp, "tvx_fully_connected_softmax_create");
  if (s != TVX_OK) return s;
  if ((s = NoGpu()) != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_fully_connected_softmax_create: host allocation failed");
  op->kind = OP_FC;
  op->fc = *d;
  op->fc.w_scales = nullptr;
  op->sm = *sm;
  op->fused_softmax = 1;
  op->quantized = true;
  op->has_const_weights = true;
  op->w_zp = d->w_scales ? 0 : d->w_zp;
  s = BuildRequantTables(d->n, d->in_scale, d->w_scale, d->w_scales, d->out_scale, &op->h_mult, &op->h_shift);
  if (s == TVX_OK) s = op->mult.Upload(op->h_mult.data(), op->h_mult.size() * 4);
  if (s == TVX_OK) s = op->shift.Upload(op->h_shift.data(), op->h_shift.size() * 4);
  ActRange(d->out_dtype, d->out_scale, d->out_zp, d->activation, &op->act_lo, &op->act_hi);
  if (s == TVX_OK) s = FcSoftmaxSetup(op, d, weights_host, bias_host);
  if (s != TVX_OK) {
    delete op;
    return s == TVX_E_UNSUPPORTED ? SetError(TVX_E_UNSUPPORTED, "tvx_fully_connected_softmax_create: no fused kernel for this layer") : s;
  }
  *out = op;
  return TVX_OK;
}

int tvx_pool2d_create(const tvx_pool2d_desc* d, tvx_op** out) {
  if (!d || !out) return SetError(TVX_E_INVALID, "tvx_pool2d_create: null argument");
  *out = nullptr;
  if (!d->in_w || !d->in_h || !d->channels || !d->batch || !d->out_w || !d->out_h || !d->k_w ||
      !d->k_h || !d->stride_w || !d->stride_h)
    return SetError(TVX_E_INVALID, "tvx_pool2d_create: zero extent or stride");
  if (!ValidDtype(d->dtype)) return SetError(TVX_E_INVALID, "tvx_pool2d_create: unknown dtype");
  if (d->pool_type != TVX_POOL_MAX && d->pool_type != TVX_POOL_AVG && d->pool_type != TVX_POOL_AVG_ANDROID && d->pool_type != TVX_POOL_L2)
    return SetError(TVX_E_UNSUPPORTED, "tvx_pool2d_create: pool type %d", d->pool_type);
  int s = CheckZeroPoint(d->dtype, d->in_zp, "tvx_pool2d_create", "input");
  if (s == TVX_OK) s = CheckZeroPoint(d->dtype, d->out_zp, "tvx_pool2d_create", "output");
  if (s == TVX_OK) s = NoGpu();
  if (s != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_pool2d_create: host allocation failed");
  op->kind = OP_POOL2D;
  op->pool = *d;
  op->quantized = IsQuant(d->dtype);
  if (op->quantized && (!(d->in_scale > 0.f) || !(d->out_scale > 0.f))) {
    delete op;
    return SetError(TVX_E_INVALID, "tvx_pool2d_create: scales must be positive");
  }
  s = TVX_E_UNSUPPORTED;
  for (SimpleSetupFn fn : PoolVariants()) {
    s = fn(op);
    if (s != TVX_E_UNSUPPORTED) break;
  }
  if (s != TVX_OK) { delete op; return s; }
  *out = op;
  return TVX_OK;
}

static int CreateSimple(int kind, const tvx_eltwise_desc* d, tvx_op** out, int (*setup)(tvx_op*),
                        const char* what) {
  if (!d || !out) return SetError(TVX_E_INVALID, "%s: null argument", what);
  *out = nullptr;
  if (!ValidDtype(d->dtype)) return SetError(TVX_E_INVALID, "%s: unknown dtype", what);
  if (IsQuant(d->dtype) && (!(d->a_scale > 0.f) || !(d->out_scale > 0.f) ||
                            (kind == OP_ADD && !(d->b_scale > 0.f))))
    return SetError(TVX_E_INVALID, "%s: scales must be positive", what);
  int s = CheckZeroPoint(d->dtype, d->a_zp, what, "input");
  if (s == TVX_OK && kind == OP_ADD) s = CheckZeroPoint(d->dtype, d->b_zp, what, "second input");
  if (s == TVX_OK) s = CheckZeroPoint(d->dtype, d->out_zp, what, "output");
  if (s == TVX_OK) s = NoGpu();
  if (s != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "%s: host allocation failed", what);
  op->kind = kind;
  op->elt = *d;
  op->quantized = IsQuant(d->dtype);
  s = setup(op);
  if (s != TVX_OK) { delete op; return s; }
  *out = op;
  return TVX_OK;
}

int tvx_activation_create(const tvx_eltwise_desc* d, tvx_op** out) {
  return CreateSimple(OP_ACTIVATION, d, out, ActivationSetup, "tvx_activation_create");
}

int tvx_add_create(const tvx_eltwise_desc* d, tvx_op** out) {
  return CreateSimple(OP_ADD, d, out, AddSetup, "tvx_add_create");
}

int tvx_softmax_create(const tvx_softmax_desc* d, tvx_op** out) {
  if (!d || !out) return SetError(TVX_E_INVALID, "tvx_softmax_create: null argument");
  *out = nullptr;
  if (!d->channels) return SetError(TVX_E_INVALID, "tvx_softmax_create: zero channels");
  if (!ValidDtype(d->in_dtype)) return SetError(TVX_E_INVALID, "tvx_softmax_create: unknown dtype");
  int s = NoGpu();
  if (s != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_softmax_create: host allocation failed");
  op->kind = OP_SOFTMAX;
  op->sm = *d;
  op->quantized = IsQuant(d->in_dtype);
  s = SoftmaxSetup(op);
  if (s != TVX_OK) { delete op; return s; }
  *out = op;
  return TVX_OK;
}

int tvx_convert_create(const tvx_convert_desc* d, tvx_op** out) {
  if (!d || !out) return SetError(TVX_E_INVALID, "tvx_convert_create: null argument");
  *out = nullptr;
  if (!ValidDtype(d->in_dtype) || !ValidDtype(d->out_dtype))
    return SetError(TVX_E_INVALID, "tvx_convert_create: unknown dtype");
  if ((IsQuant(d->in_dtype) && !(d->in_scale > 0.f)) || (IsQuant(d->out_dtype) && !(d->out_scale > 0.f)))
    return SetError(TVX_E_INVALID, "tvx_convert_create: a quantized tensor needs a positive scale");
  int s = NoGpu();
  if (s != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_convert_create: host allocation failed");
  op->kind = OP_CONVERT;
  op->cv = *d;
  s = ConvertSetup(op);
  if (s != TVX_OK) { delete op; return s; }
  *out = op;
  return TVX_OK;
}

int tvx_transpose_create(const tvx_transpose_desc* d, tvx_op** out) {
  if (!d || !out) return SetError(TVX_E_INVALID, "tvx_transpose_create: null argument");
  *out = nullptr;
  if (d->rank < 1 || d->rank > 6) return SetError(TVX_E_INVALID, "tvx_transpose_create: rank %u not in 1..6", d->rank);
  if (d->elem_bytes != 1 && d->elem_bytes != 2 && d->elem_bytes != 4)
    return SetError(TVX_E_INVALID, "tvx_transpose_create: element size %u", d->elem_bytes);
  uint32_t seen = 0;
  for (uint32_t i = 0; i < d->rank; ++i) {
    if (d->perm[i] >= d->rank || (seen >> d->perm[i] & 1u))
      return SetError(TVX_E_INVALID, "tvx_transpose_create: perm is not a permutation of 0..%u", d->rank - 1);
    seen |= 1u << d->perm[i];
    if (!d->in_dims[i]) return SetError(TVX_E_INVALID, "tvx_transpose_create: zero extent");
  }
  int s = NoGpu();
  if (s != TVX_OK) return s;
  tvx_op* op = new (std::nothrow) tvx_op();
  if (!op) return SetError(TVX_E_NOMEM, "tvx_transpose_create: host allocation failed");
  op->kind = OP_TRANSPOSE;
  op->tr = *d;
  s = TransposeSetup(op);
  if (s != TVX_OK) { delete op; return s; }
  *out = op;
  return TVX_OK;
}

int tvx_op_run(tvx_op* op, const void* in0, const void* in1, void* out_ptr, void* stream) {
  if (!op || !op->run) return SetError(TVX_E_INVALID, "tvx_op_run: null operator");
  if (!in0 || !out_ptr) return SetError(TVX_E_INVALID, "tvx_op_run: null tensor pointer");
  if ((op->kind == OP_CONV2D || op->kind == OP_DECONV2D || op->kind == OP_FC) && !op->has_const_weights && !in1)
    return SetError(TVX_E_INVALID, "tvx_op_run: operator was created without weights, pass them as in1");
  if ((op->kind == OP_ADD || op->fused_add) && !in1) return SetError(TVX_E_INVALID, "tvx_op_run: Add needs two operands");
  return op->run(op, in0, in1, out_ptr, static_cast<hipStream_t>(stream));
}

int tvx_op_run3(tvx_op* op, const void* in0, const void* in1, const void* in2, void* out_ptr, void* stream) {
  if (!in2) return tvx_op_run(op, in0, in1, out_ptr, stream);
  if (!op || !op->run) return SetError(TVX_E_INVALID, "tvx_op_run3: null operator");
  if ((op->kind != OP_CONV2D && op->kind != OP_DECONV2D && op->kind != OP_FC) || op->has_const_weights || op->bias.ptr)
    return SetError(TVX_E_UNSUPPORTED,
                    "tvx_op_run3: a run-time bias goes with a Conv2d / FullyConnected created without weights and bias");
  op->bias_at_run = in2;
  const int s = tvx_op_run(op, in0, in1, out_ptr, stream);
  op->bias_at_run = nullptr;
  return s;
}

const char* tvx_op_kernel_name(const tvx_op* op) { return op ? op->kernel_name : ""; }

void tvx_op_destroy(tvx_op* op) { delete op; }

}  // extern "C"
