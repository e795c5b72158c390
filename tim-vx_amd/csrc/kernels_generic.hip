// Generic kernels: one thread per output element, any shape / stride /
// dilation / padding / multiplier, every supported dtype. They are the
// variant of last resort and the on-GPU cross-check for the tuned variants.
#include <type_traits>

#include "variants.h"

namespace tvx {
namespace {

template <int DT> struct Elem;
template <> struct Elem<TVX_U8> { using type = uint8_t; };
template <> struct Elem<TVX_I8> { using type = int8_t; };
template <> struct Elem<TVX_F16> { using type = __half; };
template <> struct Elem<TVX_F32> { using type = float; };

__device__ __forceinline__ float ToFloat(float v) { return v; }
__device__ __forceinline__ float ToFloat(__half v) { return __half2float(v); }
__device__ __forceinline__ void FromFloat(float v, float* o) { *o = v; }
__device__ __forceinline__ void FromFloat(float v, __half* o) { *o = __float2half_rn(v); }

__device__ __forceinline__ float ApplyAct(float v, int act) {
  if (act == TVX_ACT_RELU || act == TVX_ACT_RELU6) v = v < 0.f ? 0.f : v;
  if (act == TVX_ACT_RELU6) v = v > 6.f ? 6.f : v;
  return v;
}

constexpr int kBlock = 256;
inline unsigned Blocks(uint64_t n) { return static_cast<unsigned>((n + kBlock - 1) / kBlock); }

// ---------------------------------------------------------------------------
// Conv2d
// ---------------------------------------------------------------------------
struct ConvArgs {
  int in_w, in_h, in_c, batch, k_w, k_h, out_w, out_h, out_c;
  int stride_w, stride_h, dil_w, dil_h, pad_left, pad_top, multiplier;
  int in_zp, w_zp, out_zp, lo, hi, act;
  int groups;  // >= 1
  int transposed;  // DeConv2d: every input pixel scatters a window (gathered here per output)
};

// Input row (column) that kernel tap k of output row o reads, or -1. Convolution:
// o * stride - pad + k * dil. Transposed convolution: the i with i * stride - pad + k = o.
__device__ __forceinline__ int TapSource(const ConvArgs& a, int o, int k, int stride, int dil, int pad, int extent) {
  int i;
  if (a.transposed) {
    const int t = o + pad - k;
    if (t < 0 || t % stride) return -1;
    i = t / stride;
  } else {
    i = o * stride - pad + k * dil;
  }
  return i >= 0 && i < extent ? i : -1;
}

// Input channels one output channel reads, and the first of them: all of them (dense), one
// (depthwise, oc = ic * multiplier + j) or the channels of its group.
__device__ __forceinline__ void ChannelRange(const ConvArgs& a, int oc, int* ic_per_oc, int* ic0) {
  if (a.multiplier > 0) {
    *ic_per_oc = 1;
    *ic0 = oc / a.multiplier;
  } else {
    *ic_per_oc = a.in_c / a.groups;
    *ic0 = (oc / (a.out_c / a.groups)) * *ic_per_oc;
  }
}

template <typename XT, typename WT>
__global__ void __launch_bounds__(kBlock)
ConvQuantKernel(ConvArgs a, const XT* __restrict__ x, const WT* __restrict__ w,
                const int32_t* __restrict__ bias, const int32_t* __restrict__ mult,
                const int32_t* __restrict__ shift, XT* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int ow = idx % a.out_w;
  const int oh = (idx / a.out_w) % a.out_h;
  const int oc = (idx / (static_cast<uint64_t>(a.out_w) * a.out_h)) % a.out_c;
  const int n = idx / (static_cast<uint64_t>(a.out_w) * a.out_h * a.out_c);
  int ic_per_oc, ic0;
  ChannelRange(a, oc, &ic_per_oc, &ic0);
  int32_t acc = 0;
  for (int ci = 0; ci < ic_per_oc; ++ci) {
    const XT* xp = x + (static_cast<uint64_t>(n) * a.in_c + ic0 + ci) * a.in_h * a.in_w;
    const WT* wp = w + (static_cast<uint64_t>(oc) * ic_per_oc + ci) * a.k_h * a.k_w;
    for (int ky = 0; ky < a.k_h; ++ky) {
      const int ih = TapSource(a, oh, ky, a.stride_h, a.dil_h, a.pad_top, a.in_h);
      if (ih < 0) continue;
      for (int kx = 0; kx < a.k_w; ++kx) {
        const int iw = TapSource(a, ow, kx, a.stride_w, a.dil_w, a.pad_left, a.in_w);
        if (iw < 0) continue;
        acc += (static_cast<int32_t>(xp[ih * a.in_w + iw]) - a.in_zp) *
               (static_cast<int32_t>(wp[ky * a.k_w + kx]) - a.w_zp);
      }
    }
  }
  if (bias) acc += bias[oc];
  y[idx] = static_cast<XT>(RequantClamp(acc, mult[oc], shift[oc], a.out_zp, a.lo, a.hi));
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
ConvFloatKernel(ConvArgs a, const T* __restrict__ x, const T* __restrict__ w,
                const float* __restrict__ bias, T* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int ow = idx % a.out_w;
  const int oh = (idx / a.out_w) % a.out_h;
  const int oc = (idx / (static_cast<uint64_t>(a.out_w) * a.out_h)) % a.out_c;
  const int n = idx / (static_cast<uint64_t>(a.out_w) * a.out_h * a.out_c);
  int ic_per_oc, ic0;
  ChannelRange(a, oc, &ic_per_oc, &ic0);
  float acc = 0.f;
  for (int ci = 0; ci < ic_per_oc; ++ci) {
    const T* xp = x + (static_cast<uint64_t>(n) * a.in_c + ic0 + ci) * a.in_h * a.in_w;
    const T* wp = w + (static_cast<uint64_t>(oc) * ic_per_oc + ci) * a.k_h * a.k_w;
    for (int ky = 0; ky < a.k_h; ++ky) {
      const int ih = TapSource(a, oh, ky, a.stride_h, a.dil_h, a.pad_top, a.in_h);
      if (ih < 0) continue;
      for (int kx = 0; kx < a.k_w; ++kx) {
        const int iw = TapSource(a, ow, kx, a.stride_w, a.dil_w, a.pad_left, a.in_w);
        if (iw < 0) continue;
        acc += ToFloat(xp[ih * a.in_w + iw]) * ToFloat(wp[ky * a.k_w + kx]);
      }
    }
  }
  if (bias) acc += bias[oc];
  FromFloat(ApplyAct(acc, a.act), &y[idx]);
}

int ConvGenericRun(tvx_op* op, const void* in0, const void* in1, void* out, hipStream_t st) {
  const tvx_conv2d_desc& d = op->conv;
  ConvArgs a{static_cast<int>(d.in_w), static_cast<int>(d.in_h), static_cast<int>(d.in_c),
             static_cast<int>(d.batch), static_cast<int>(d.k_w), static_cast<int>(d.k_h),
             static_cast<int>(d.out_w), static_cast<int>(d.out_h), static_cast<int>(d.out_c),
             static_cast<int>(d.stride_w), static_cast<int>(d.stride_h),
             static_cast<int>(d.dilation_w), static_cast<int>(d.dilation_h),
             static_cast<int>(d.pad_left), static_cast<int>(d.pad_top), d.multiplier,
             d.in_zp, op->w_zp, d.out_zp, op->act_lo, op->act_hi, d.activation, d.groups > 1 ? d.groups : 1,
             op->kind == OP_DECONV2D ? 1 : 0};
  const void* w = op->has_const_weights ? op->weights.ptr : in1;
  const uint64_t total = static_cast<uint64_t>(d.out_w) * d.out_h * d.out_c * d.batch;
  const dim3 grid(Blocks(total)), block(kBlock);
  const int32_t* bias_i = op->bias_at_run ? static_cast<const int32_t*>(op->bias_at_run) : op->bias.as<int32_t>();
  const float* bias_f = op->bias_at_run ? static_cast<const float*>(op->bias_at_run) : op->bias.as<float>();
  const int32_t *mu = op->mult.as<int32_t>(), *sh = op->shift.as<int32_t>();
  if (d.in_dtype == TVX_U8 && d.w_dtype == TVX_U8) {
    hipLaunchKernelGGL((ConvQuantKernel<uint8_t, uint8_t>), grid, block, 0, st, a,
                       static_cast<const uint8_t*>(in0), static_cast<const uint8_t*>(w), bias_i,
                       mu, sh, static_cast<uint8_t*>(out), total);
  } else if (d.in_dtype == TVX_U8 && d.w_dtype == TVX_I8) {
    hipLaunchKernelGGL((ConvQuantKernel<uint8_t, int8_t>), grid, block, 0, st, a,
                       static_cast<const uint8_t*>(in0), static_cast<const int8_t*>(w), bias_i, mu,
                       sh, static_cast<uint8_t*>(out), total);
  } else if (d.in_dtype == TVX_I8) {
    hipLaunchKernelGGL((ConvQuantKernel<int8_t, int8_t>), grid, block, 0, st, a,
                       static_cast<const int8_t*>(in0), static_cast<const int8_t*>(w), bias_i, mu,
                       sh, static_cast<int8_t*>(out), total);
  } else if (d.in_dtype == TVX_F32) {
    hipLaunchKernelGGL((ConvFloatKernel<float>), grid, block, 0, st, a,
                       static_cast<const float*>(in0), static_cast<const float*>(w),
                       bias_f, static_cast<float*>(out), total);
  } else {
    hipLaunchKernelGGL((ConvFloatKernel<__half>), grid, block, 0, st, a,
                       static_cast<const __half*>(in0), static_cast<const __half*>(w),
                       bias_f, static_cast<__half*>(out), total);
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

// ---------------------------------------------------------------------------
// FullyConnected
// ---------------------------------------------------------------------------
struct FcArgs {
  int m, k, n, in_zp, w_zp, out_zp, lo, hi, act;
};

template <typename XT, typename WT>
__global__ void __launch_bounds__(kBlock)
FcQuantKernel(FcArgs a, const XT* __restrict__ x, const WT* __restrict__ w,
              const int32_t* __restrict__ bias, const int32_t* __restrict__ mult,
              const int32_t* __restrict__ shift, XT* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int n = idx % a.n;
  const uint64_t m = idx / a.n;
  const XT* xp = x + m * a.k;
  const WT* wp = w + static_cast<uint64_t>(n) * a.k;
  int32_t acc = 0;
  for (int k = 0; k < a.k; ++k)
    acc += (static_cast<int32_t>(xp[k]) - a.in_zp) * (static_cast<int32_t>(wp[k]) - a.w_zp);
  if (bias) acc += bias[n];
  y[idx] = static_cast<XT>(RequantClamp(acc, mult[n], shift[n], a.out_zp, a.lo, a.hi));
}

// (x - zx) . (w - zw) over the sixteen bytes of two vectors
template <typename XT, typename WT>
__device__ __forceinline__ int32_t Dot16(const uint4& xv, const uint4& wv, int in_zp, int w_zp) {
  const uint32_t xd[4] = {xv.x, xv.y, xv.z, xv.w}, wd[4] = {wv.x, wv.y, wv.z, wv.w};
  int32_t acc = 0;
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int b = 0; b < 4; ++b)
      acc += (static_cast<int32_t>(static_cast<XT>(xd[d] >> (8 * b))) - in_zp) *
             (static_cast<int32_t>(static_cast<WT>(wd[d] >> (8 * b))) - w_zp);
  return acc;
}

// One wavefront per output: the lanes stride over K sixteen bytes at a time (consecutive lanes
// read consecutive chunks of both rows; rows start at any byte, the loads are unaligned) and the
// partial sums meet in a butterfly. For the small FullyConnected layers at the end of a network -
// a few thousand outputs with a long reduction - where one thread per output would walk its row
// alone. A row of up to 1024 bytes is one round trip to memory.
template <typename XT, typename WT>
__global__ void __launch_bounds__(kBlock)
FcQuantWaveKernel(FcArgs a, const XT* __restrict__ x, const WT* __restrict__ w,
                  const int32_t* __restrict__ bias, const int32_t* __restrict__ mult,
                  const int32_t* __restrict__ shift, XT* __restrict__ y, uint64_t total) {
  const int lane = threadIdx.x & 63;
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * (kBlock / 64) + (threadIdx.x >> 6);
  if (idx >= total) return;
  const int n = idx % a.n;
  const uint64_t m = idx / a.n;
  const XT* xp = x + m * a.k;
  const WT* wp = w + static_cast<uint64_t>(n) * a.k;
  int32_t acc = 0;
  const int k16 = a.k & ~15;
  for (int k = lane * 16; k < k16; k += 1024) {
    uint4 xv, wv;
    __builtin_memcpy(&xv, xp + k, 16);
    __builtin_memcpy(&wv, wp + k, 16);
    acc += Dot16<XT, WT>(xv, wv, a.in_zp, a.w_zp);
  }
  if (k16 + lane < a.k)
    acc += (static_cast<int32_t>(xp[k16 + lane]) - a.in_zp) * (static_cast<int32_t>(wp[k16 + lane]) - a.w_zp);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
  if (lane == 0) {
    if (bias) acc += bias[n];
    y[idx] = static_cast<XT>(RequantClamp(acc, mult[n], shift[n], a.out_zp, a.lo, a.hi));
  }
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
FcFloatKernel(FcArgs a, const T* __restrict__ x, const T* __restrict__ w,
              const float* __restrict__ bias, T* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int n = idx % a.n;
  const uint64_t m = idx / a.n;
  const T* xp = x + m * a.k;
  const T* wp = w + static_cast<uint64_t>(n) * a.k;
  float acc = 0.f;
  for (int k = 0; k < a.k; ++k) acc += ToFloat(xp[k]) * ToFloat(wp[k]);
  if (bias) acc += bias[n];
  FromFloat(ApplyAct(acc, a.act), &y[idx]);
}

int FcGenericRun(tvx_op* op, const void* in0, const void* in1, void* out, hipStream_t st) {
  const tvx_fc_desc& d = op->fc;
  FcArgs a{static_cast<int>(d.m), static_cast<int>(d.k), static_cast<int>(d.n), d.in_zp, op->w_zp,
           d.out_zp, op->act_lo, op->act_hi, d.activation};
  const void* w = op->has_const_weights ? op->weights.ptr : in1;
  const uint64_t total = static_cast<uint64_t>(d.m) * d.n;
  const dim3 grid(Blocks(total)), block(kBlock);
  const int32_t* bias_i = op->bias_at_run ? static_cast<const int32_t*>(op->bias_at_run) : op->bias.as<int32_t>();
  const float* bias_f = op->bias_at_run ? static_cast<const float*>(op->bias_at_run) : op->bias.as<float>();
  const int32_t *mu = op->mult.as<int32_t>(), *sh = op->shift.as<int32_t>();
  // few outputs with a long reduction: a wavefront per output
  const bool wave = total <= 16384 && d.k >= 128;
  const dim3 wgrid(static_cast<unsigned>((total + kBlock / 64 - 1) / (kBlock / 64)));
  if (d.in_dtype == TVX_U8 && d.w_dtype == TVX_U8) {
    if (wave)
      hipLaunchKernelGGL((FcQuantWaveKernel<uint8_t, uint8_t>), wgrid, block, 0, st, a,
                         static_cast<const uint8_t*>(in0), static_cast<const uint8_t*>(w), bias_i,
                         mu, sh, static_cast<uint8_t*>(out), total);
    else
      hipLaunchKernelGGL((FcQuantKernel<uint8_t, uint8_t>), grid, block, 0, st, a,
                         static_cast<const uint8_t*>(in0), static_cast<const uint8_t*>(w), bias_i,
                         mu, sh, static_cast<uint8_t*>(out), total);
  } else if (d.in_dtype == TVX_U8 && d.w_dtype == TVX_I8) {
    if (wave)
      hipLaunchKernelGGL((FcQuantWaveKernel<uint8_t, int8_t>), wgrid, block, 0, st, a,
                         static_cast<const uint8_t*>(in0), static_cast<const int8_t*>(w), bias_i, mu,
                         sh, static_cast<uint8_t*>(out), total);
    else
      hipLaunchKernelGGL((FcQuantKernel<uint8_t, int8_t>), grid, block, 0, st, a,
                         static_cast<const uint8_t*>(in0), static_cast<const int8_t*>(w), bias_i, mu,
                         sh, static_cast<uint8_t*>(out), total);
  } else if (d.in_dtype == TVX_I8) {
    if (wave)
      hipLaunchKernelGGL((FcQuantWaveKernel<int8_t, int8_t>), wgrid, block, 0, st, a,
                         static_cast<const int8_t*>(in0), static_cast<const int8_t*>(w), bias_i, mu,
                         sh, static_cast<int8_t*>(out), total);
    else
      hipLaunchKernelGGL((FcQuantKernel<int8_t, int8_t>), grid, block, 0, st, a,
                         static_cast<const int8_t*>(in0), static_cast<const int8_t*>(w), bias_i, mu,
                         sh, static_cast<int8_t*>(out), total);
  } else if (d.in_dtype == TVX_F32) {
    hipLaunchKernelGGL((FcFloatKernel<float>), grid, block, 0, st, a,
                       static_cast<const float*>(in0), static_cast<const float*>(w),
                       bias_f, static_cast<float*>(out), total);
  } else {
    hipLaunchKernelGGL((FcFloatKernel<__half>), grid, block, 0, st, a,
                       static_cast<const __half*>(in0), static_cast<const __half*>(w),
                       bias_f, static_cast<__half*>(out), total);
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

// ---------------------------------------------------------------------------
// Pool2d
// ---------------------------------------------------------------------------
struct PoolArgs {
  int in_w, in_h, out_w, out_h, k_w, k_h, stride_w, stride_h, pad_left, pad_top, type;
  int in_zp, out_zp, qmin, qmax, mult, shift;
  double ratio;
};

template <typename T>
__global__ void __launch_bounds__(kBlock)
PoolQuantKernel(PoolArgs a, const T* __restrict__ x, T* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int ow = idx % a.out_w;
  const int oh = (idx / a.out_w) % a.out_h;
  const uint64_t plane = idx / (static_cast<uint64_t>(a.out_w) * a.out_h);
  const T* xp = x + plane * a.in_w * a.in_h;
  int cnt = 0, vmax = INT32_MIN;
  int64_t sum = 0, sq = 0;
  for (int ky = 0; ky < a.k_h; ++ky) {
    const int ih = oh * a.stride_h - a.pad_top + ky;
    if (ih < 0 || ih >= a.in_h) continue;
    for (int kx = 0; kx < a.k_w; ++kx) {
      const int iw = ow * a.stride_w - a.pad_left + kx;
      if (iw < 0 || iw >= a.in_w) continue;
      const int v = static_cast<int>(xp[ih * a.in_w + iw]) - a.in_zp;
      ++cnt;
      sum += v;
      sq += static_cast<int64_t>(v) * v;
      vmax = v > vmax ? v : vmax;
    }
  }
  int64_t r = 0;
  if (a.type == TVX_POOL_MAX) {
    if (cnt) r = RequantRne(vmax, a.mult, a.shift);
  } else if (a.type == TVX_POOL_L2) {
    // root of the mean of the squares, the mean over the whole window (padding counts as zeros)
    r = static_cast<int64_t>(rint(a.ratio * __dsqrt_rn(static_cast<double>(sq) / static_cast<double>(a.k_w * a.k_h))));
  } else {
    const int div = a.type == TVX_POOL_AVG ? a.k_w * a.k_h : cnt;
    if (div) r = static_cast<int64_t>(rint(static_cast<double>(sum) * a.ratio / static_cast<double>(div)));
  }
  r += a.out_zp;
  r = r < a.qmin ? a.qmin : (r > a.qmax ? a.qmax : r);
  y[idx] = static_cast<T>(r);
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
PoolFloatKernel(PoolArgs a, const T* __restrict__ x, T* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  const int ow = idx % a.out_w;
  const int oh = (idx / a.out_w) % a.out_h;
  const uint64_t plane = idx / (static_cast<uint64_t>(a.out_w) * a.out_h);
  const T* xp = x + plane * a.in_w * a.in_h;
  int cnt = 0;
  float vmax = -INFINITY, sum = 0.f, sq = 0.f;
  for (int ky = 0; ky < a.k_h; ++ky) {
    const int ih = oh * a.stride_h - a.pad_top + ky;
    if (ih < 0 || ih >= a.in_h) continue;
    for (int kx = 0; kx < a.k_w; ++kx) {
      const int iw = ow * a.stride_w - a.pad_left + kx;
      if (iw < 0 || iw >= a.in_w) continue;
      const float v = ToFloat(xp[ih * a.in_w + iw]);
      ++cnt;
      sum += v;
      sq += v * v;
      vmax = v > vmax ? v : vmax;
    }
  }
  float r;
  if (a.type == TVX_POOL_MAX) {
    r = cnt ? vmax : 0.f;
  } else if (a.type == TVX_POOL_L2) {
    r = sqrtf(sq / static_cast<float>(a.k_w * a.k_h));
  } else {
    const int div = a.type == TVX_POOL_AVG ? a.k_w * a.k_h : cnt;
    r = div ? sum / static_cast<float>(div) : 0.f;
  }
  FromFloat(r, &y[idx]);
}

// Quantized average over a whole plane (global average pooling): L lanes share a plane, read it
// as dwords (the last one ending with the plane), sum the bytes with dot4 against ones and add
// up across the lanes; the result is formed exactly as in the kernel above.
template <typename T, int L>
__global__ void __launch_bounds__(kBlock)
PoolPlaneAvgKernel(PoolArgs a, const T* __restrict__ x, T* __restrict__ y, uint64_t planes) {
  const uint64_t plane = (static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x) / L;
  const int lane = threadIdx.x % L;
  const int hw = a.in_w * a.in_h;
  const int n_dw = plane < planes ? (hw + 3) / 4 : 0;  // lanes past the last plane stay for the shuffles
  const uint8_t* xp = reinterpret_cast<const uint8_t*>(x) + plane * hw;
  int sum = 0;
  for (int i = lane; i < n_dw; i += L) {
    const int at = min(4 * i, hw - 4);
    uint32_t v;
    __builtin_memcpy(&v, xp + at, 4);
    v >>= 8 * (4 * i - at);  // the bytes in front of a short last dword were counted already
    if constexpr (std::is_signed<T>::value) sum = __builtin_amdgcn_sdot4(static_cast<int>(v), 0x01010101, sum, false);
    else sum = static_cast<int>(__builtin_amdgcn_udot4(v, 0x01010101u, static_cast<uint32_t>(sum), false));
  }
#pragma unroll
  for (int o = L / 2; o; o >>= 1) sum += __shfl_xor(sum, o, 64);
  if (lane != 0 || plane >= planes) return;
  const int64_t total = static_cast<int64_t>(sum) - static_cast<int64_t>(hw) * a.in_zp;
  int64_t r = static_cast<int64_t>(rint(static_cast<double>(total) * a.ratio / static_cast<double>(hw)));
  r += a.out_zp;
  r = r < a.qmin ? a.qmin : (r > a.qmax ? a.qmax : r);
  y[plane] = static_cast<T>(r);
}

template <typename T>
static void LaunchPoolPlaneAvg(const PoolArgs& a, const void* in0, void* out, uint64_t planes, hipStream_t st) {
  const int n_dw = (a.in_w * a.in_h + 3) / 4;
  const T* x = static_cast<const T*>(in0);
  T* y = static_cast<T*>(out);
  const dim3 block(kBlock);
  if (n_dw <= 4) hipLaunchKernelGGL((PoolPlaneAvgKernel<T, 4>), dim3(Blocks(planes * 4)), block, 0, st, a, x, y, planes);
  else if (n_dw <= 16) hipLaunchKernelGGL((PoolPlaneAvgKernel<T, 16>), dim3(Blocks(planes * 16)), block, 0, st, a, x, y, planes);
  else hipLaunchKernelGGL((PoolPlaneAvgKernel<T, 64>), dim3(Blocks(planes * 64)), block, 0, st, a, x, y, planes);
}

// does the window of a quantized average pooling cover exactly the whole, unpadded plane?
static bool IsPlaneAverage(const tvx_op* op) {
  const tvx_pool2d_desc& d = op->pool;
  const uint64_t hw = static_cast<uint64_t>(d.in_w) * d.in_h;
  return op->quantized && (d.pool_type == TVX_POOL_AVG || d.pool_type == TVX_POOL_AVG_ANDROID) &&
         d.k_w == d.in_w && d.k_h == d.in_h && d.pad_left == 0 && d.pad_top == 0 && d.out_w == 1 && d.out_h == 1 &&
         hw >= 4 && hw <= (1u << 22);  // the byte sum of a plane stays below 2^31
}

int PoolGenericRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const tvx_pool2d_desc& d = op->pool;
  PoolArgs a{static_cast<int>(d.in_w), static_cast<int>(d.in_h), static_cast<int>(d.out_w),
             static_cast<int>(d.out_h), static_cast<int>(d.k_w), static_cast<int>(d.k_h),
             static_cast<int>(d.stride_w), static_cast<int>(d.stride_h),
             static_cast<int>(d.pad_left), static_cast<int>(d.pad_top), d.pool_type,
             d.in_zp, d.out_zp, d.dtype == TVX_U8 ? 0 : -128, d.dtype == TVX_U8 ? 255 : 127,
             op->geo[0], op->geo[1],
             op->quantized ? static_cast<double>(d.in_scale) / static_cast<double>(d.out_scale) : 1.0};
  const uint64_t total = static_cast<uint64_t>(d.out_w) * d.out_h * d.channels * d.batch;
  if (IsPlaneAverage(op)) {
    if (d.dtype == TVX_U8) LaunchPoolPlaneAvg<uint8_t>(a, in0, out, total, st);
    else LaunchPoolPlaneAvg<int8_t>(a, in0, out, total, st);
    TVX_HIP_CHECK(hipGetLastError());
    return TVX_OK;
  }
  const dim3 grid(Blocks(total)), block(kBlock);
  switch (d.dtype) {
    case TVX_U8:
      hipLaunchKernelGGL((PoolQuantKernel<uint8_t>), grid, block, 0, st, a,
                         static_cast<const uint8_t*>(in0), static_cast<uint8_t*>(out), total);
      break;
    case TVX_I8:
      hipLaunchKernelGGL((PoolQuantKernel<int8_t>), grid, block, 0, st, a,
                         static_cast<const int8_t*>(in0), static_cast<int8_t*>(out), total);
      break;
    case TVX_F32:
      hipLaunchKernelGGL((PoolFloatKernel<float>), grid, block, 0, st, a,
                         static_cast<const float*>(in0), static_cast<float*>(out), total);
      break;
    default:
      hipLaunchKernelGGL((PoolFloatKernel<__half>), grid, block, 0, st, a,
                         static_cast<const __half*>(in0), static_cast<__half*>(out), total);
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

// ---------------------------------------------------------------------------
// element-wise
// ---------------------------------------------------------------------------
struct EltArgs {
  int a_zp, b_zp, out_zp, lo, hi, mult, shift, act;
  double ra, rb;
};

template <typename T>
__global__ void __launch_bounds__(kBlock)
ActQuantKernel(EltArgs a, const T* __restrict__ x, T* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  y[idx] = static_cast<T>(
      RequantClamp(static_cast<int32_t>(x[idx]) - a.a_zp, a.mult, a.shift, a.out_zp, a.lo, a.hi));
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
ActFloatKernel(EltArgs a, const T* __restrict__ x, T* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  FromFloat(ApplyAct(ToFloat(x[idx]), a.act), &y[idx]);
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
AddQuantKernel(EltArgs a, const T* __restrict__ x, const T* __restrict__ z, T* __restrict__ y,
               uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  // rne(fma(a - za, sa/so, (b - zb) * (sb/so))) in double: one defined order.
  const double tb = __dmul_rn(static_cast<double>(static_cast<int32_t>(z[idx]) - a.b_zp), a.rb);
  const double t = fma(static_cast<double>(static_cast<int32_t>(x[idx]) - a.a_zp), a.ra, tb);
  int64_t r = static_cast<int64_t>(rint(t)) + a.out_zp;
  r = r < a.lo ? a.lo : (r > a.hi ? a.hi : r);
  y[idx] = static_cast<T>(r);
}

// The same arithmetic on 16 elements per thread (whole 16-byte chunks of both operands); the
// ragged tail of the tensor goes to the one-element kernel above.
template <typename T>
__global__ void __launch_bounds__(kBlock)
AddQuantVecKernel(EltArgs a, const uint4* __restrict__ x, const uint4* __restrict__ z, uint4* __restrict__ y,
                  uint64_t chunks) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= chunks) return;
  const uint4 xv = x[idx], zv = z[idx];
  const uint32_t xs[4] = {xv.x, xv.y, xv.z, xv.w}, zs[4] = {zv.x, zv.y, zv.z, zv.w};
  uint32_t out[4];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    int r4[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int xa = static_cast<int32_t>(static_cast<T>((xs[d] >> (8 * e)) & 0xff));
      const int zb = static_cast<int32_t>(static_cast<T>((zs[d] >> (8 * e)) & 0xff));
      const double tb = __dmul_rn(static_cast<double>(zb - a.b_zp), a.rb);
      const double t = fma(static_cast<double>(xa - a.a_zp), a.ra, tb);
      // |t| < 2^29 (8-bit operands, ratios bounded at creation): the 32-bit conversion is exact
      r4[e] = Med3(static_cast<int>(rint(t)) + a.out_zp, a.lo, a.hi);
    }
    out[d] = PackBytes(r4[0], r4[1], r4[2], r4[3]);
  }
  y[idx] = make_uint4(out[0], out[1], out[2], out[3]);
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
AddFloatKernel(const T* __restrict__ x, const T* __restrict__ z, T* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  FromFloat(ToFloat(x[idx]) + ToFloat(z[idx]), &y[idx]);
}

EltArgs MakeEltArgs(const tvx_op* op) {
  const tvx_eltwise_desc& d = op->elt;
  EltArgs a{};
  a.a_zp = d.a_zp;
  a.b_zp = d.b_zp;
  a.out_zp = d.out_zp;
  a.lo = op->act_lo;
  a.hi = op->act_hi;
  a.mult = op->geo[0];
  a.shift = op->geo[1];
  a.act = d.activation;
  if (op->quantized) {
    a.ra = static_cast<double>(d.a_scale) / static_cast<double>(d.out_scale);
    a.rb = static_cast<double>(d.b_scale) / static_cast<double>(d.out_scale);
  }
  return a;
}

int ActivationRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const EltArgs a = MakeEltArgs(op);
  const uint64_t total = op->elt.count;
  if (!total) return TVX_OK;
  const dim3 grid(Blocks(total)), block(kBlock);
  switch (op->elt.dtype) {
    case TVX_U8:
      hipLaunchKernelGGL((ActQuantKernel<uint8_t>), grid, block, 0, st, a,
                         static_cast<const uint8_t*>(in0), static_cast<uint8_t*>(out), total);
      break;
    case TVX_I8:
      hipLaunchKernelGGL((ActQuantKernel<int8_t>), grid, block, 0, st, a,
                         static_cast<const int8_t*>(in0), static_cast<int8_t*>(out), total);
      break;
    case TVX_F32:
      hipLaunchKernelGGL((ActFloatKernel<float>), grid, block, 0, st, a,
                         static_cast<const float*>(in0), static_cast<float*>(out), total);
      break;
    default:
      hipLaunchKernelGGL((ActFloatKernel<__half>), grid, block, 0, st, a,
                         static_cast<const __half*>(in0), static_cast<__half*>(out), total);
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

// 16 elements per thread where all three tensors are 16-byte aligned and the ratios are small
// enough for the 32-bit rounding conversion; the one-element kernel for the tail and otherwise.
template <typename T>
void AddQuantLaunch(const EltArgs& a, const void* in0, const void* in1, void* out, uint64_t total, bool small_ratios,
                    hipStream_t st) {
  const T* x = static_cast<const T*>(in0);
  const T* z = static_cast<const T*>(in1);
  T* y = static_cast<T*>(out);
  uint64_t done = 0;
  const bool aligned = ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(in1) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  if (aligned && small_ratios && total >= 16) {
    const uint64_t chunks = total / 16;
    hipLaunchKernelGGL((AddQuantVecKernel<T>), dim3(Blocks(chunks)), dim3(kBlock), 0, st, a,
                       reinterpret_cast<const uint4*>(x), reinterpret_cast<const uint4*>(z),
                       reinterpret_cast<uint4*>(y), chunks);
    done = chunks * 16;
  }
  if (done < total)
    hipLaunchKernelGGL((AddQuantKernel<T>), dim3(Blocks(total - done)), dim3(kBlock), 0, st, a, x + done, z + done,
                       y + done, total - done);
}

int AddRun(tvx_op* op, const void* in0, const void* in1, void* out, hipStream_t st) {
  const EltArgs a = MakeEltArgs(op);
  const uint64_t total = op->elt.count;
  if (!total) return TVX_OK;
  const dim3 grid(Blocks(total)), block(kBlock);
  switch (op->elt.dtype) {
    case TVX_U8:
      AddQuantLaunch<uint8_t>(a, in0, in1, out, total, op->geo[2] != 0, st);
      break;
    case TVX_I8:
      AddQuantLaunch<int8_t>(a, in0, in1, out, total, op->geo[2] != 0, st);
      break;
    case TVX_F32:
      hipLaunchKernelGGL((AddFloatKernel<float>), grid, block, 0, st,
                         static_cast<const float*>(in0), static_cast<const float*>(in1),
                         static_cast<float*>(out), total);
      break;
    default:
      hipLaunchKernelGGL((AddFloatKernel<__half>), grid, block, 0, st,
                         static_cast<const __half*>(in0), static_cast<const __half*>(in1),
                         static_cast<__half*>(out), total);
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

// ---------------------------------------------------------------------------
// Softmax: one thread per row (rows are short: class counts)
// ---------------------------------------------------------------------------
template <typename T, bool QUANT>
__global__ void __launch_bounds__(kBlock)
SoftmaxKernel(int c, uint64_t rows, uint64_t inner, float beta, float scale, int zp, const T* __restrict__ x,
              float* __restrict__ y) {
  // any axis: one thread per (row, inner position); the c elements of its group are `inner` apart
  const uint64_t t = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (t >= rows * inner) return;
  const uint64_t base = (t / inner) * c * inner + t % inner;
  const T* xp = x + base;
  float* yp = y + base;
  float mx = -INFINITY;
  for (int i = 0; i < c; ++i) {
    float v;
    if constexpr (QUANT) v = scale * static_cast<float>(static_cast<int>(xp[i * inner]) - zp);
    else v = ToFloat(xp[i * inner]);
    yp[i * inner] = v;
    mx = v > mx ? v : mx;
  }
  float sum = 0.f;
  for (int i = 0; i < c; ++i) {
    const float e = expf(beta * (yp[i * inner] - mx));
    yp[i * inner] = e;
    sum += e;
  }
  for (int i = 0; i < c; ++i) yp[i * inner] = yp[i * inner] / sum;
}

// Contiguous groups of at most 64 * kSmVals elements: G lanes share a group and keep its
// elements in registers between the three passes (maximum, exponentials and their sum,
// division), so that the group is read once and written once.
constexpr int kSmVals = 16;

template <typename T, bool QUANT, int G>
__global__ void __launch_bounds__(kBlock)
SoftmaxRowKernel(int c, uint64_t rows, float beta, float scale, int zp, const T* __restrict__ x,
                 float* __restrict__ y) {
  const uint64_t row = (static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x) / G;
  const int lane = threadIdx.x % G;
  // lanes past the last row stay for the shuffles and touch no memory
  const int live = row < rows ? c : 0;
  const T* xp = x + row * c;
  float* yp = y + row * c;
  float v[kSmVals];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < kSmVals; ++j) {
    const int i = lane + j * G;
    v[j] = -INFINITY;
    if (i < live) {
      if constexpr (QUANT) v[j] = scale * static_cast<float>(static_cast<int>(xp[i]) - zp);
      else v[j] = ToFloat(xp[i]);
    }
    mx = v[j] > mx ? v[j] : mx;
  }
#pragma unroll
  for (int o = G / 2; o; o >>= 1) {
    const float other = __shfl_xor(mx, o, 64);
    mx = other > mx ? other : mx;
  }
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < kSmVals; ++j) {
    const int i = lane + j * G;
    v[j] = i < live ? expf(beta * (v[j] - mx)) : 0.f;
    sum += v[j];
  }
#pragma unroll
  for (int o = G / 2; o; o >>= 1) sum += __shfl_xor(sum, o, 64);
#pragma unroll
  for (int j = 0; j < kSmVals; ++j) {
    const int i = lane + j * G;
    if (i < live) yp[i] = v[j] / sum;
  }
}

template <typename T, bool QUANT>
static void LaunchSoftmaxRows(const tvx_softmax_desc& d, int zp, float scale, const void* in0, float* y,
                              hipStream_t st) {
  const int c = static_cast<int>(d.channels);
  const T* x = static_cast<const T*>(in0);
  const dim3 block(kBlock);
  // the fewest lanes that leave at most four elements to each, 64 from there on
  const int g = c <= 4 ? 1 : (c <= 16 ? 4 : (c <= 64 ? 16 : 64));
  const dim3 grid(Blocks(d.rows * g));
  switch (g) {
    case 1: hipLaunchKernelGGL((SoftmaxRowKernel<T, QUANT, 1>), grid, block, 0, st, c, d.rows, d.beta, scale, zp, x, y); break;
    case 4: hipLaunchKernelGGL((SoftmaxRowKernel<T, QUANT, 4>), grid, block, 0, st, c, d.rows, d.beta, scale, zp, x, y); break;
    case 16: hipLaunchKernelGGL((SoftmaxRowKernel<T, QUANT, 16>), grid, block, 0, st, c, d.rows, d.beta, scale, zp, x, y); break;
    default: hipLaunchKernelGGL((SoftmaxRowKernel<T, QUANT, 64>), grid, block, 0, st, c, d.rows, d.beta, scale, zp, x, y);
  }
}

int SoftmaxRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const tvx_softmax_desc& d = op->sm;
  if (!d.rows) return TVX_OK;
  const uint64_t inner = d.inner ? d.inner : 1;
  if (inner == 1 && d.channels <= 64u * kSmVals) {
    float* yr = static_cast<float*>(out);
    switch (d.in_dtype) {
      case TVX_U8: LaunchSoftmaxRows<uint8_t, true>(d, d.in_zp, d.in_scale, in0, yr, st); break;
      case TVX_I8: LaunchSoftmaxRows<int8_t, true>(d, d.in_zp, d.in_scale, in0, yr, st); break;
      case TVX_F32: LaunchSoftmaxRows<float, false>(d, 0, 1.f, in0, yr, st); break;
      default: LaunchSoftmaxRows<__half, false>(d, 0, 1.f, in0, yr, st);
    }
    TVX_HIP_CHECK(hipGetLastError());
    return TVX_OK;
  }
  const dim3 grid(Blocks(d.rows * inner)), block(kBlock);
  float* y = static_cast<float*>(out);
  const int c = static_cast<int>(d.channels);
  switch (d.in_dtype) {
    case TVX_U8:
      hipLaunchKernelGGL((SoftmaxKernel<uint8_t, true>), grid, block, 0, st, c, d.rows, inner, d.beta,
                         d.in_scale, d.in_zp, static_cast<const uint8_t*>(in0), y);
      break;
    case TVX_I8:
      hipLaunchKernelGGL((SoftmaxKernel<int8_t, true>), grid, block, 0, st, c, d.rows, inner, d.beta,
                         d.in_scale, d.in_zp, static_cast<const int8_t*>(in0), y);
      break;
    case TVX_F32:
      hipLaunchKernelGGL((SoftmaxKernel<float, false>), grid, block, 0, st, c, d.rows, inner, d.beta, 1.f,
                         0, static_cast<const float*>(in0), y);
      break;
    default:
      hipLaunchKernelGGL((SoftmaxKernel<__half, false>), grid, block, 0, st, c, d.rows, inner, d.beta, 1.f,
                         0, static_cast<const __half*>(in0), y);
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

// ---------------------------------------------------------------------------
// FullyConnected + Softmax over its (at most 16) outputs: one wavefront per input row. The lanes stride over K sixteen
// bytes at a time for every output (the row of x is loaded once), the partial sums meet in a butterfly, lane n
// requantizes output n as the FullyConnected kernels do, and the Softmax runs across those lanes in the
// arithmetic - and the order of additions - of SoftmaxRowKernel on the stored codes.
// ---------------------------------------------------------------------------
constexpr int kFcSmMaxN = 16;

template <typename XT, typename WT>
__global__ void __launch_bounds__(kBlock)
FcSoftmaxKernel(FcArgs a, float beta, float sm_scale, const XT* __restrict__ x, const WT* __restrict__ w,
                const int32_t* __restrict__ bias, const int32_t* __restrict__ mult,
                const int32_t* __restrict__ shift, float* __restrict__ y) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (row >= a.m) return;  // whole wavefronts
  const XT* xp = x + static_cast<uint64_t>(row) * a.k;
  // this lane's table entries travel with the rows
  const int nl = min(lane, a.n - 1);
  const int my_bias = bias ? bias[nl] : 0, my_mult = mult[nl], my_shift = shift[nl];
  // Sixteen bytes of the row and of every weight row per lane and step; the loads stand under no branch
  // (outputs past the last read the last row again, lanes past the row's end read its start and add nothing),
  // so that all of a step travel together: a row of up to 1024 bytes is one round trip to memory.
  int32_t acc[kFcSmMaxN];
#pragma unroll
  for (int n = 0; n < kFcSmMaxN; ++n) acc[n] = 0;
  const int k16 = a.k & ~15;
  for (int k0 = 0; k0 < k16; k0 += 1024) {
    const int k = k0 + lane * 16;
    const bool ok = k < k16;
    const int kk = ok ? k : 0;
    uint4 xv, wv[kFcSmMaxN];
    __builtin_memcpy(&xv, xp + kk, 16);
#pragma unroll
    for (int n = 0; n < kFcSmMaxN; ++n) __builtin_memcpy(&wv[n], w + static_cast<uint64_t>(min(n, a.n - 1)) * a.k + kk, 16);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < kFcSmMaxN; ++n) {
      const int32_t d = Dot16<XT, WT>(xv, wv[n], a.in_zp, a.w_zp);
      acc[n] += ok ? d : 0;
    }
  }
  {
    const bool ok = k16 + lane < a.k;
    const int kk = ok ? k16 + lane : 0;
    const int32_t xe = static_cast<int32_t>(xp[kk]) - a.in_zp;
    int32_t we[kFcSmMaxN];
#pragma unroll
    for (int n = 0; n < kFcSmMaxN; ++n) we[n] = static_cast<int32_t>(w[static_cast<uint64_t>(min(n, a.n - 1)) * a.k + kk]) - a.w_zp;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int n = 0; n < kFcSmMaxN; ++n) acc[n] += ok ? xe * we[n] : 0;
  }
  int32_t mine = 0;  // output `lane` of the row
#pragma unroll
  for (int off = 32; off > 0; off >>= 1)
#pragma unroll
    for (int n = 0; n < kFcSmMaxN; ++n) acc[n] += __shfl_xor(acc[n], off);
#pragma unroll
  for (int n = 0; n < kFcSmMaxN; ++n)
    if (lane == n) mine = acc[n];
  const int code = RequantClamp(mine + my_bias, my_mult, my_shift, a.out_zp, a.lo, a.hi);
  // ---- Softmax over lanes 0 .. n-1 ----
  const bool live = lane < a.n;
  const float v = live ? sm_scale * static_cast<float>(code - a.out_zp) : -INFINITY;
  float mx = v;
#pragma unroll
  for (int o = 8; o; o >>= 1) {
    const float other = __shfl_xor(mx, o, 64);
    mx = other > mx ? other : mx;
  }
  const float e = live ? expf(beta * (v - mx)) : 0.f;
  float ee[kFcSmMaxN];
#pragma unroll
  for (int i = 0; i < kFcSmMaxN; ++i) ee[i] = __shfl(e, i, 64);
  float sum;
  if (a.n <= 4) {  // SoftmaxRowKernel with one lane per row: in index order
    sum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) sum += ee[i];
  } else {  // ... with four lanes per row: lane l sums elements l, l + 4, ..., the lanes meet in a butterfly
    float part[4];
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      part[l] = 0.f;
#pragma unroll
      for (int j = 0; j < kFcSmMaxN / 4; ++j) part[l] += ee[l + 4 * j];
    }
    sum = (part[0] + part[2]) + (part[1] + part[3]);
  }
  if (live) y[static_cast<uint64_t>(row) * a.n + lane] = e / sum;
}

int FcSoftmaxRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const tvx_fc_desc& d = op->fc;
  FcArgs a{static_cast<int>(d.m), static_cast<int>(d.k), static_cast<int>(d.n), d.in_zp, op->w_zp,
           d.out_zp, op->act_lo, op->act_hi, d.activation};
  const dim3 grid((d.m + kBlock / 64 - 1) / (kBlock / 64)), block(kBlock);
  const int32_t* bias = op->bias.as<int32_t>();
  const int32_t *mu = op->mult.as<int32_t>(), *sh = op->shift.as<int32_t>();
  float* y = static_cast<float*>(out);
  if (d.in_dtype == TVX_U8 && d.w_dtype == TVX_U8)
    hipLaunchKernelGGL((FcSoftmaxKernel<uint8_t, uint8_t>), grid, block, 0, st, a, op->sm.beta, op->sm.in_scale,
                       static_cast<const uint8_t*>(in0), op->weights.as<uint8_t>(), bias, mu, sh, y);
  else if (d.in_dtype == TVX_U8)
    hipLaunchKernelGGL((FcSoftmaxKernel<uint8_t, int8_t>), grid, block, 0, st, a, op->sm.beta, op->sm.in_scale,
                       static_cast<const uint8_t*>(in0), op->weights.as<int8_t>(), bias, mu, sh, y);
  else
    hipLaunchKernelGGL((FcSoftmaxKernel<int8_t, int8_t>), grid, block, 0, st, a, op->sm.beta, op->sm.in_scale,
                       static_cast<const int8_t*>(in0), op->weights.as<int8_t>(), bias, mu, sh, y);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

// ---------------------------------------------------------------------------
// Transpose: one thread per output element; output dimension i walks input dimension perm[i]
// ---------------------------------------------------------------------------
struct TransposeArgs {
  uint32_t rank;
  uint32_t out_dims[6];
  uint64_t in_stride[6];  // element stride of the input dimension each output dimension walks
};

template <typename T>
__global__ void __launch_bounds__(kBlock)
TransposeKernel(TransposeArgs a, const T* __restrict__ x, T* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  uint64_t rest = idx, src = 0;
  for (uint32_t i = 0; i < a.rank; ++i) {
    const uint64_t c = rest % a.out_dims[i];
    rest /= a.out_dims[i];
    src += c * a.in_stride[i];
  }
  y[idx] = x[src];
}

int TransposeRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const tvx_transpose_desc& d = op->tr;
  TransposeArgs a{};
  a.rank = d.rank;
  uint64_t stride[6], total = 1;
  for (uint32_t i = 0; i < d.rank; ++i) {
    stride[i] = total;
    total *= d.in_dims[i];
  }
  for (uint32_t i = 0; i < d.rank; ++i) {
    a.out_dims[i] = d.in_dims[d.perm[i]];
    a.in_stride[i] = stride[d.perm[i]];
  }
  const dim3 grid(Blocks(total)), block(kBlock);
  if (d.elem_bytes == 1)
    hipLaunchKernelGGL((TransposeKernel<uint8_t>), grid, block, 0, st, a, static_cast<const uint8_t*>(in0),
                       static_cast<uint8_t*>(out), total);
  else if (d.elem_bytes == 2)
    hipLaunchKernelGGL((TransposeKernel<uint16_t>), grid, block, 0, st, a, static_cast<const uint16_t*>(in0),
                       static_cast<uint16_t*>(out), total);
  else
    hipLaunchKernelGGL((TransposeKernel<uint32_t>), grid, block, 0, st, a, static_cast<const uint32_t*>(in0),
                       static_cast<uint32_t*>(out), total);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

// ---------------------------------------------------------------------------
// DataConvert: element -> float32 -> output type, one thread per element
// ---------------------------------------------------------------------------
struct ConvertArgs {
  float in_scale, out_scale;
  int in_zp, out_zp;
};

template <typename TI>
__device__ __forceinline__ float ConvertLoad(const TI* x, uint64_t i, const ConvertArgs& a) {
  if constexpr (std::is_same<TI, uint8_t>::value || std::is_same<TI, int8_t>::value)
    return (static_cast<float>(static_cast<int>(x[i])) - static_cast<float>(a.in_zp)) * a.in_scale;
  else
    return ToFloat(x[i]);
}

template <typename TI, typename TO>
__global__ void __launch_bounds__(kBlock)
ConvertKernel(ConvertArgs a, const TI* __restrict__ x, TO* __restrict__ y, uint64_t total) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx >= total) return;
  const float f = ConvertLoad(x, idx, a);
  if constexpr (std::is_same<TO, uint8_t>::value || std::is_same<TO, int8_t>::value) {
    const float lo = std::is_same<TO, uint8_t>::value ? 0.f : -128.f, hi = std::is_same<TO, uint8_t>::value ? 255.f : 127.f;
    // saturate in float (a NaN becomes the lower bound), then the conversion is exact
    float r = rintf(__fdiv_rn(f, a.out_scale)) + static_cast<float>(a.out_zp);
    r = fminf(fmaxf(r, lo), hi);
    y[idx] = static_cast<TO>(static_cast<int>(r));
  } else {
    FromFloat(f, &y[idx]);
  }
}

template <typename TI>
void ConvertLaunchOut(const tvx_convert_desc& d, const ConvertArgs& a, const void* in0, void* out, hipStream_t st) {
  const dim3 grid(Blocks(d.count)), block(kBlock);
  const TI* x = static_cast<const TI*>(in0);
  switch (d.out_dtype) {
    case TVX_U8: hipLaunchKernelGGL((ConvertKernel<TI, uint8_t>), grid, block, 0, st, a, x, static_cast<uint8_t*>(out), d.count); break;
    case TVX_I8: hipLaunchKernelGGL((ConvertKernel<TI, int8_t>), grid, block, 0, st, a, x, static_cast<int8_t*>(out), d.count); break;
    case TVX_F16: hipLaunchKernelGGL((ConvertKernel<TI, __half>), grid, block, 0, st, a, x, static_cast<__half*>(out), d.count); break;
    default: hipLaunchKernelGGL((ConvertKernel<TI, float>), grid, block, 0, st, a, x, static_cast<float*>(out), d.count); break;
  }
}

int ConvertRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const tvx_convert_desc& d = op->cv;
  if (!d.count) return TVX_OK;
  const ConvertArgs a{d.in_scale, d.out_scale, d.in_zp, d.out_zp};
  switch (d.in_dtype) {
    case TVX_U8: ConvertLaunchOut<uint8_t>(d, a, in0, out, st); break;
    case TVX_I8: ConvertLaunchOut<int8_t>(d, a, in0, out, st); break;
    case TVX_F16: ConvertLaunchOut<__half>(d, a, in0, out, st); break;
    default: ConvertLaunchOut<float>(d, a, in0, out, st); break;
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

int UploadWeightsAndBias(tvx_op* op, const void* w, size_t w_bytes, const void* b, size_t b_bytes) {
  int s = TVX_OK;
  if (w) s = op->weights.Upload(w, w_bytes);
  if (s == TVX_OK && b) s = op->bias.Upload(b, b_bytes);
  return s;
}

}  // namespace

int ConvGenericSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w, const void* b) {
  const uint64_t ic_per_oc = d->multiplier > 0 ? 1 : d->in_c / (d->groups > 1 ? d->groups : 1);
  const size_t w_bytes = static_cast<size_t>(d->k_w) * d->k_h * ic_per_oc * d->out_c * DtypeBytes(d->w_dtype);
  int s = UploadWeightsAndBias(op, w, w_bytes, b, static_cast<size_t>(d->out_c) * 4);
  if (s != TVX_OK) return s;
  op->run = ConvGenericRun;
  op->kernel_name = op->kind == OP_DECONV2D ? "deconv2d_generic" : "conv2d_generic";
  return TVX_OK;
}

int FcGenericSetup(tvx_op* op, const tvx_fc_desc* d, const void* w, const void* b) {
  const size_t w_bytes = static_cast<size_t>(d->k) * d->n * DtypeBytes(d->w_dtype);
  int s = UploadWeightsAndBias(op, w, w_bytes, b, static_cast<size_t>(d->n) * 4);
  if (s != TVX_OK) return s;
  op->run = FcGenericRun;
  op->kernel_name = "fc_generic";
  return TVX_OK;
}

// FullyConnected + Softmax (the caller has checked that the Softmax reads the FullyConnected's codes along its outputs)
int FcSoftmaxSetup(tvx_op* op, const tvx_fc_desc* d, const void* w, const void* b) {
  if (!op->quantized || !w || d->n > static_cast<uint32_t>(kFcSmMaxN) || d->m > 0x7fffffffu / 64) return TVX_E_UNSUPPORTED;
  if (d->in_dtype == TVX_I8 && d->w_dtype != TVX_I8) return TVX_E_UNSUPPORTED;
  int s = UploadWeightsAndBias(op, w, static_cast<size_t>(d->k) * d->n, b, static_cast<size_t>(d->n) * 4);
  if (s != TVX_OK) return s;
  op->run = FcSoftmaxRun;
  op->kernel_name = "fc_softmax_i8";
  return TVX_OK;
}

static int ScalarRequant(tvx_op* op, float in_scale, float out_scale) {
  std::vector<int32_t> mult, shift;
  int s = BuildRequantTables(1, in_scale, 1.0f, nullptr, out_scale, &mult, &shift);
  if (s != TVX_OK) return s;
  op->geo[0] = mult[0];
  op->geo[1] = shift[0];
  return TVX_OK;
}

int PoolGenericSetup(tvx_op* op) {
  if (op->quantized) {
    int s = ScalarRequant(op, op->pool.in_scale, op->pool.out_scale);
    if (s != TVX_OK) return s;
  }
  op->run = PoolGenericRun;
  op->kernel_name = IsPlaneAverage(op) ? "avgpool_plane_i8" : "pool2d_generic";
  return TVX_OK;
}

int ActivationSetup(tvx_op* op) {
  if (op->quantized) {
    int s = ScalarRequant(op, op->elt.a_scale, op->elt.out_scale);
    if (s != TVX_OK) return s;
    ActRange(op->elt.dtype, op->elt.out_scale, op->elt.out_zp, op->elt.activation, &op->act_lo,
             &op->act_hi);
  }
  op->run = ActivationRun;
  op->kernel_name = "activation_generic";
  return TVX_OK;
}

int AddSetup(tvx_op* op) {
  if (op->quantized)
    ActRange(op->elt.dtype, op->elt.out_scale, op->elt.out_zp, TVX_ACT_NONE, &op->act_lo, &op->act_hi);
  // the 16-element kernel rounds through a 32-bit conversion: fine while |a ra + b rb| stays far below 2^31
  const double ra = static_cast<double>(op->elt.a_scale) / static_cast<double>(op->elt.out_scale);
  const double rb = static_cast<double>(op->elt.b_scale) / static_cast<double>(op->elt.out_scale);
  op->geo[2] = op->quantized && ra < 1048576.0 && rb < 1048576.0 ? 1 : 0;
  op->run = AddRun;
  op->kernel_name = "add_generic";
  return TVX_OK;
}

int ConvertSetup(tvx_op* op) {
  op->run = ConvertRun;
  op->kernel_name = "convert_generic";
  return TVX_OK;
}

int TransposeSetup(tvx_op* op) {
  op->run = TransposeRun;
  op->kernel_name = "transpose_generic";
  return TVX_OK;
}

int SoftmaxSetup(tvx_op* op) {
  op->run = SoftmaxRun;
  op->kernel_name = "softmax_generic";
  return TVX_OK;
}

}  // namespace tvx
