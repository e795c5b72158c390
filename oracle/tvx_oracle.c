/*
 * CPU restatement of TIM-VX's quantized convolution path. TEST INFRASTRUCTURE:
 * only tests, the smoke check and the benchmark's cpu_baseline leg may call
 * it; the shipped library never does.
 *
 * The arithmetic of Conv2d / FullyConnected / Pool2d lives in VeriSilicon's
 * closed OpenVX driver (vxConvolutionLayer, vxFullyConnectedLayer,
 * vxPoolingLayer2: prebuilt-sdk/x86_64_linux/include/VX/vx_khr_nn.h:873,915,
 * 1739), whose binary is not part of the reference checkout. This file
 * restates the published semantics and is pinned by the reference's own
 * inline golden vectors (tests/golden/ *.json, recorded from
 * src/tim/vx/ops/{conv2d,depthwiseConv,groupedconv2d,conv1d,deconv2d,fullyconnected,max_pool,
 * avg_pool,softmax,transpose,simple_operations}_test.cc and
 * src/tim/transform/layout_inference_test.cc).
 *
 * What the goldens pin: indexing, padding, stride, dilation, depthwise channel
 * mapping, zero-point handling, per-channel scales, saturation, pooling
 * divisors. What they do NOT pin ("parity unpinned", chosen here and applied
 * identically on the GPU):
 *   - rounding of the requantization at exact .5 ties and its arithmetic
 *     form: here a Q31 multiplier and a single round-half-to-even right shift
 *     of the 64-bit product;
 *   - quantized FullyConnected, ReLU/ReLU6, Add and quantized AVG rounding
 *     (the reference compares AVG with +-1 tolerance);
 *   - DeConv2d with more than one channel per group: the reference's tests are
 *     single-channel or depthwise, so the channel order of the {Kw, Kh, Ic, Oc}
 *     weights follows include/tim/vx/ops/deconv.h:46-52 only;
 *   - DataConvert on exact .5 ties (round-half-to-even of f / scale, as
 *     vsi_nn_dtype_util_prv.h:228-252 computes it with the default rounding mode);
 *   - Transpose: the reference's two tests move a {1, 3} vector and cannot tell a
 *     permutation from its inverse; the direction follows the extent rule
 *     out.size[i] = in.size[perm[i]] (vsi_nn_op_permute.c:219-230) and is checked
 *     against numpy on non-involutive permutations.
 *
 * Layouts (dim 0 fastest): activations WHCN, weights WHIcOc, depthwise
 * weights {Kw,Kh,Ic*mult,1}, FC input {K,M}, weight {K,N}, output {N,M}
 * (src/tim/vx/ops/conv2d_test.cc:990-1040, depthwiseConv_test.cc:12-37,
 * fullyconnected_test.cc:36-59).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

enum { TVXO_U8 = 0, TVXO_I8 = 1, TVXO_F16 = 2, TVXO_F32 = 3 };
enum { TVXO_ACT_NONE = 0, TVXO_ACT_RELU = 1, TVXO_ACT_RELU6 = 2 };
enum { TVXO_POOL_MAX = 0, TVXO_POOL_AVG = 1, TVXO_POOL_L2 = 2, TVXO_POOL_AVG_ANDROID = 3 };

/* ---- fp16 <-> fp32 ------------------------------------------------------ */
static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ff, bits;
  if (e == 0) {
    if (m == 0) {
      bits = sign;
    } else {
      int s = -1;
      do { ++s; m <<= 1; } while (!(m & 0x400));
      bits = sign | (uint32_t)(112 - s) << 23 | (m & 0x3ff) << 13;
    }
  } else if (e == 31) {
    bits = sign | 0x7f800000u | m << 13;
  } else {
    bits = sign | (e + 112) << 23 | m << 13;
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u, man = x & 0x7fffffu;
  int32_t e = (int32_t)((x >> 23) & 0xff) - 127 + 15;
  if (((x >> 23) & 0xff) == 0xff) return (uint16_t)(sign | 0x7c00u | (man ? 0x200u : 0));
  if (e >= 31) return (uint16_t)(sign | 0x7c00u);
  if (e <= 0) {
    if (e < -10) return (uint16_t)sign;
    man |= 0x800000u;
    uint32_t sh = (uint32_t)(14 - e), half = man >> sh, rem = man & ((1u << sh) - 1), mid = 1u << (sh - 1);
    if (rem > mid || (rem == mid && (half & 1))) ++half;
    return (uint16_t)(sign | half);
  }
  uint32_t half = (uint32_t)e << 10 | man >> 13, rem = man & 0x1fff;
  if (rem > 0x1000 || (rem == 0x1000 && (half & 1))) ++half;
  return (uint16_t)(sign | half);
}

/* ---- requantization ------------------------------------------------------ */
/*
 * Real multiplier M = s_in * s_w / s_out (each float scale widened to double
 * first) as mult * 2^-shift with mult in [2^30, 2^31). API contract that
 * requests round-to-nearest-even + saturate: include/tim/vx/operation.h:44-48.
 */
void tvxo_quantize_multiplier(double m, int32_t* mult, int32_t* shift) {
  if (!(m > 0.0) || !isfinite(m)) {
    *mult = 0;
    *shift = 0;
    return;
  }
  int e;
  double q = frexp(m, &e); /* m = q * 2^e, q in [0.5, 1) */
  int64_t qi = llround(q * 2147483648.0);
  if (qi == 2147483648LL) {
    qi /= 2;
    ++e;
  }
  *mult = (int32_t)qi;
  *shift = 31 - e;
}

/* round_half_even(acc * mult / 2^shift), as a 64-bit integer */
int64_t tvxo_requant(int32_t acc, int32_t mult, int32_t shift) {
  int64_t p = (int64_t)acc * (int64_t)mult;
  /* multiplier >= 2^30: any non-zero accumulator saturates every 8-bit output */
  if (shift <= 0) return p > 0 ? ((int64_t)1 << 40) : (p < 0 ? -((int64_t)1 << 40) : 0);
  if (shift > 62) return 0;
  int64_t fl = p >> shift; /* arithmetic: floor */
  int64_t rem = p & (((int64_t)1 << shift) - 1);
  int64_t half = (int64_t)1 << (shift - 1);
  if (rem > half || (rem == half && (fl & 1))) ++fl;
  return fl;
}

static inline int64_t clamp64(int64_t v, int64_t lo, int64_t hi) {
  return v < lo ? lo : (v > hi ? hi : v);
}

static inline int32_t load_q(const void* p, int dtype, int64_t i) {
  return dtype == TVXO_U8 ? (int32_t)((const uint8_t*)p)[i] : (int32_t)((const int8_t*)p)[i];
}
static inline void store_q(void* p, int dtype, int64_t i, int64_t v) {
  if (dtype == TVXO_U8) ((uint8_t*)p)[i] = (uint8_t)v;
  else ((int8_t*)p)[i] = (int8_t)v;
}
static inline float load_f(const void* p, int dtype, int64_t i) {
  return dtype == TVXO_F32 ? ((const float*)p)[i] : half_to_float(((const uint16_t*)p)[i]);
}
static inline void store_f(void* p, int dtype, int64_t i, float v) {
  if (dtype == TVXO_F32) ((float*)p)[i] = v;
  else ((uint16_t*)p)[i] = float_to_half(v);
}

/* Output clamp of a quantized tensor with an optional fused activation:
 * relu -> lower bound at the quantized zero; relu6 -> additionally an upper
 * bound at zero_point + round_half_even(6 / scale). */
void tvxo_act_range(int out_dtype, float out_scale, int32_t out_zp, int act,
                    int32_t* lo, int32_t* hi) {
  int32_t qmin = out_dtype == TVXO_U8 ? 0 : -128, qmax = out_dtype == TVXO_U8 ? 255 : 127;
  *lo = qmin;
  *hi = qmax;
  if (act == TVXO_ACT_RELU || act == TVXO_ACT_RELU6) {
    if (out_zp > *lo) *lo = out_zp;
  }
  if (act == TVXO_ACT_RELU6) {
    double six = nearbyint(6.0 / (double)out_scale);
    if (six < 1e9) {
      int64_t top = (int64_t)out_zp + (int64_t)six;
      if (top < *hi) *hi = (int32_t)top;
    }
  }
  if (*lo > *hi) *lo = *hi;
}

typedef struct {
  /* shapes */
  int32_t in_w, in_h, in_c, batch;
  int32_t k_w, k_h, out_c;
  int32_t out_w, out_h;
  int32_t stride_w, stride_h, dil_w, dil_h;
  int32_t pad_left, pad_top;
  int32_t multiplier; /* 0: dense; >0: depthwise, oc = ic*multiplier + j */
  /* types and quantization */
  int32_t in_dtype, w_dtype, out_dtype;
  float in_scale;
  int32_t in_zp;
  float w_scale;          /* per-tensor */
  int32_t w_zp;           /* per-tensor */
  const float* w_scales;  /* per-channel [out_c] or NULL */
  float out_scale;
  int32_t out_zp;
  int32_t act;
  int32_t groups; /* 0 or 1: ordinary; g > 1: grouped, weights {k_w, k_h, in_c/g, out_c} */
} tvxo_conv_desc;

/*
 * Conv2d, dense, depthwise or grouped (vxConvolutionLayer semantics,
 * vx_khr_nn.h:837-852; depthwise channel map vsi_nn_op_conv2d.c:275-278; grouped: output
 * channel block j of out_c/g channels reads input channel block j of in_c/g channels, weights
 * {k_w, k_h, in_c/g, out_c} - src/tim/vx/ops/groupedconv2d_test.cc:30-294 pins shapes and values).
 *   acc = sum (x - zx)(w - zw) + bias        (int32, wraps)
 *   y   = clamp(requant(acc) + zy)
 * Taps outside the input contribute nothing (padding with the real value 0).
 * bias: int32 for quantized, float for floating point; may be NULL.
 */
void tvxo_conv2d(const tvxo_conv_desc* d, const void* x, const void* w,
                 const void* bias, void* y) {
  const int quant = d->in_dtype == TVXO_U8 || d->in_dtype == TVXO_I8;
  const int64_t in_plane = (int64_t)d->in_w * d->in_h, out_plane = (int64_t)d->out_w * d->out_h;
  const int32_t groups = d->groups > 1 ? d->groups : 1;
  const int32_t ic_per_oc = d->multiplier > 0 ? 1 : d->in_c / groups;
  int32_t lo = 0, hi = 0;
  if (quant) tvxo_act_range(d->out_dtype, d->out_scale, d->out_zp, d->act, &lo, &hi);
  const int64_t total = (int64_t)d->batch * d->out_c;
#pragma omp parallel for schedule(static)
  for (int64_t job = 0; job < total; ++job) {
    const int32_t n = (int32_t)(job / d->out_c), oc = (int32_t)(job % d->out_c);
    const int32_t ic0 = d->multiplier > 0 ? oc / d->multiplier : (oc / (d->out_c / groups)) * ic_per_oc;
    int32_t mult = 0, shift = 0;
    if (quant) {
      double ws = d->w_scales ? (double)d->w_scales[oc] : (double)d->w_scale;
      tvxo_quantize_multiplier((double)d->in_scale * ws / (double)d->out_scale, &mult, &shift);
    }
    const int32_t zw = d->w_scales ? 0 : d->w_zp;
    for (int32_t oh = 0; oh < d->out_h; ++oh) {
      for (int32_t ow = 0; ow < d->out_w; ++ow) {
        int64_t acc = 0;
        float facc = 0.f;
        for (int32_t ci = 0; ci < ic_per_oc; ++ci) {
          const int32_t ic = ic0 + ci;
          const int64_t xb = ((int64_t)n * d->in_c + ic) * in_plane;
          const int64_t wb = ((int64_t)oc * ic_per_oc + ci) * d->k_h * d->k_w;
          for (int32_t ky = 0; ky < d->k_h; ++ky) {
            const int32_t ih = oh * d->stride_h - d->pad_top + ky * d->dil_h;
            if (ih < 0 || ih >= d->in_h) continue;
            for (int32_t kx = 0; kx < d->k_w; ++kx) {
              const int32_t iw = ow * d->stride_w - d->pad_left + kx * d->dil_w;
              if (iw < 0 || iw >= d->in_w) continue;
              const int64_t xi = xb + (int64_t)ih * d->in_w + iw, wi = wb + (int64_t)ky * d->k_w + kx;
              if (quant) {
                acc += (int64_t)(load_q(x, d->in_dtype, xi) - d->in_zp) *
                       (int64_t)(load_q(w, d->w_dtype, wi) - zw);
              } else {
                facc += load_f(x, d->in_dtype, xi) * load_f(w, d->w_dtype, wi);
              }
            }
          }
        }
        const int64_t yi = ((int64_t)n * d->out_c + oc) * out_plane + (int64_t)oh * d->out_w + ow;
        if (quant) {
          if (bias) acc += ((const int32_t*)bias)[oc];
          int64_t r = tvxo_requant((int32_t)(uint32_t)(uint64_t)acc, mult, shift);
          store_q(y, d->out_dtype, yi, clamp64(r + d->out_zp, lo, hi));
        } else {
          if (bias) facc += ((const float*)bias)[oc];
          if (d->act == TVXO_ACT_RELU || d->act == TVXO_ACT_RELU6) facc = facc < 0.f ? 0.f : facc;
          if (d->act == TVXO_ACT_RELU6) facc = facc > 6.f ? 6.f : facc;
          store_f(y, d->out_dtype, yi, facc);
        }
      }
    }
  }
}

/*
 * DeConv2d, the transposed convolution (vxDeconvolutionLayer; src/tim/vx/ops/deconv.cc:45-79,
 * extent rule src/tim/vx/internal/src/ops/vsi_nn_op_deconvolution.c:217-218; values pinned by
 * src/tim/vx/ops/deconv2d_test.cc:20-140: no kernel flip, out(0,0) = in(0,0) * w(0,0)).
 * Written as the scatter it is defined by: input pixel (ix, iy) of channel ic adds
 * (x - zx)(w[oc][ic][ky][kx] - zw) to output pixel (ix*stride - pad_left + kx, iy*stride - pad_top + ky);
 * then bias, requantization and clamp as for Conv2d. Weights {k_w, k_h, in_c/groups, out_c};
 * multiplier = 1 is the depthwise form ({k_w, k_h, c, 1}); dilation is not used.
 */
void tvxo_deconv2d(const tvxo_conv_desc* d, const void* x, const void* w, const void* bias, void* y) {
  const int quant = d->in_dtype == TVXO_U8 || d->in_dtype == TVXO_I8;
  const int64_t in_plane = (int64_t)d->in_w * d->in_h, out_plane = (int64_t)d->out_w * d->out_h;
  const int32_t groups = d->groups > 1 ? d->groups : 1;
  const int32_t ic_per_oc = d->multiplier > 0 ? 1 : d->in_c / groups;
  int32_t lo = 0, hi = 0;
  if (quant) tvxo_act_range(d->out_dtype, d->out_scale, d->out_zp, d->act, &lo, &hi);
  const int64_t total = (int64_t)d->batch * d->out_c;
#pragma omp parallel for schedule(static)
  for (int64_t job = 0; job < total; ++job) {
    const int32_t n = (int32_t)(job / d->out_c), oc = (int32_t)(job % d->out_c);
    const int32_t ic0 = d->multiplier > 0 ? oc / d->multiplier : (oc / (d->out_c / groups)) * ic_per_oc;
    const int32_t zw = d->w_scales ? 0 : d->w_zp;
    int64_t* acc = (int64_t*)calloc((size_t)out_plane, sizeof(int64_t));
    float* facc = (float*)calloc((size_t)out_plane, sizeof(float));
    for (int32_t ci = 0; ci < ic_per_oc; ++ci) {
      const int64_t xb = ((int64_t)n * d->in_c + ic0 + ci) * in_plane;
      const int64_t wb = ((int64_t)oc * ic_per_oc + ci) * d->k_h * d->k_w;
      for (int32_t iy = 0; iy < d->in_h; ++iy)
        for (int32_t ix = 0; ix < d->in_w; ++ix)
          for (int32_t ky = 0; ky < d->k_h; ++ky) {
            const int32_t oy = iy * d->stride_h - d->pad_top + ky;
            if (oy < 0 || oy >= d->out_h) continue;
            for (int32_t kx = 0; kx < d->k_w; ++kx) {
              const int32_t ox = ix * d->stride_w - d->pad_left + kx;
              if (ox < 0 || ox >= d->out_w) continue;
              const int64_t xi = xb + (int64_t)iy * d->in_w + ix, wi = wb + (int64_t)ky * d->k_w + kx;
              if (quant)
                acc[(int64_t)oy * d->out_w + ox] +=
                    (int64_t)(load_q(x, d->in_dtype, xi) - d->in_zp) * (int64_t)(load_q(w, d->w_dtype, wi) - zw);
              else
                facc[(int64_t)oy * d->out_w + ox] += load_f(x, d->in_dtype, xi) * load_f(w, d->w_dtype, wi);
            }
          }
    }
    int32_t mult = 0, shift = 0;
    if (quant) {
      double ws = d->w_scales ? (double)d->w_scales[oc] : (double)d->w_scale;
      tvxo_quantize_multiplier((double)d->in_scale * ws / (double)d->out_scale, &mult, &shift);
    }
    for (int64_t p = 0; p < out_plane; ++p) {
      const int64_t yi = ((int64_t)n * d->out_c + oc) * out_plane + p;
      if (quant) {
        int64_t a = acc[p] + (bias ? ((const int32_t*)bias)[oc] : 0);
        int64_t r = tvxo_requant((int32_t)(uint32_t)(uint64_t)a, mult, shift);
        store_q(y, d->out_dtype, yi, clamp64(r + d->out_zp, lo, hi));
      } else {
        float f = facc[p] + (bias ? ((const float*)bias)[oc] : 0.f);
        if (d->act == TVXO_ACT_RELU || d->act == TVXO_ACT_RELU6) f = f < 0.f ? 0.f : f;
        if (d->act == TVXO_ACT_RELU6) f = f > 6.f ? 6.f : f;
        store_f(y, d->out_dtype, yi, f);
      }
    }
    free(acc);
    free(facc);
  }
}

typedef struct {
  int32_t m, k, n;
  int32_t in_dtype, w_dtype, out_dtype;
  float in_scale;
  int32_t in_zp;
  float w_scale;
  int32_t w_zp;
  const float* w_scales; /* per output feature [n] or NULL */
  float out_scale;
  int32_t out_zp;
  int32_t act;
} tvxo_fc_desc;

/*
 * FullyConnected (vxFullyConnectedLayer; flattening
 * src/tim/vx/internal/src/ops/vsi_nn_op_fullconnect2.c:86-98):
 *   out[m*N + n] = requant(sum_k (x[m*K+k]-zx)(w[n*K+k]-zw[n]) + b[n])
 */
void tvxo_fully_connected(const tvxo_fc_desc* d, const void* x, const void* w,
                          const void* bias, void* y) {
  const int quant = d->in_dtype == TVXO_U8 || d->in_dtype == TVXO_I8;
  int32_t lo = 0, hi = 0;
  if (quant) tvxo_act_range(d->out_dtype, d->out_scale, d->out_zp, d->act, &lo, &hi);
  int32_t* mults = NULL;
  int32_t* shifts = NULL;
  if (quant) {
    mults = (int32_t*)malloc(sizeof(int32_t) * (size_t)d->n);
    shifts = (int32_t*)malloc(sizeof(int32_t) * (size_t)d->n);
    for (int32_t n = 0; n < d->n; ++n) {
      double ws = d->w_scales ? (double)d->w_scales[n] : (double)d->w_scale;
      tvxo_quantize_multiplier((double)d->in_scale * ws / (double)d->out_scale, &mults[n], &shifts[n]);
    }
  }
  const int32_t zw = d->w_scales ? 0 : d->w_zp;
#pragma omp parallel for schedule(static)
  for (int32_t m = 0; m < d->m; ++m) {
    for (int32_t n = 0; n < d->n; ++n) {
      const int64_t xb = (int64_t)m * d->k, wb = (int64_t)n * d->k, yi = (int64_t)m * d->n + n;
      if (quant) {
        int32_t acc = 0; /* int32: enough for K*255*255 < 2^31, wraps beyond like the GPU accumulators */
        if (d->in_dtype == TVXO_I8 && d->w_dtype == TVXO_I8 && d->in_zp == 0 && zw == 0) {
          const int8_t* xp = (const int8_t*)x + xb;
          const int8_t* wp = (const int8_t*)w + wb;
          for (int32_t k = 0; k < d->k; ++k) acc += (int32_t)xp[k] * (int32_t)wp[k];
        } else {
          uint32_t u = 0;
          for (int32_t k = 0; k < d->k; ++k)
            u += (uint32_t)((load_q(x, d->in_dtype, xb + k) - d->in_zp) *
                            (load_q(w, d->w_dtype, wb + k) - zw));
          acc = (int32_t)u;
        }
        if (bias) acc = (int32_t)((uint32_t)acc + (uint32_t)((const int32_t*)bias)[n]);
        int64_t r = tvxo_requant(acc, mults[n], shifts[n]);
        store_q(y, d->out_dtype, yi, clamp64(r + d->out_zp, lo, hi));
      } else {
        float facc = 0.f;
        for (int32_t k = 0; k < d->k; ++k)
          facc += load_f(x, d->in_dtype, xb + k) * load_f(w, d->w_dtype, wb + k);
        if (bias) facc += ((const float*)bias)[n];
        if (d->act == TVXO_ACT_RELU || d->act == TVXO_ACT_RELU6) facc = facc < 0.f ? 0.f : facc;
        if (d->act == TVXO_ACT_RELU6) facc = facc > 6.f ? 6.f : facc;
        store_f(y, d->out_dtype, yi, facc);
      }
    }
  }
  free(mults);
  free(shifts);
}

typedef struct {
  int32_t in_w, in_h, channels, batch; /* channels = C (planes per image) */
  int32_t out_w, out_h;
  int32_t k_w, k_h, stride_w, stride_h, pad_left, pad_top;
  int32_t pool_type;
  int32_t dtype; /* in == out */
  float in_scale;
  int32_t in_zp;
  float out_scale;
  int32_t out_zp;
} tvxo_pool_desc;

/*
 * Pool2d (vxPoolingLayer2; src/tim/vx/internal/src/ops/vsi_nn_op_pool.c:66-158).
 * MAX over in-bounds taps. AVG divides the in-bounds sum by k_w*k_h (padding
 * counts as real zeros, avg_pool_test.cc:428-455); AVG_ANDROID by the number
 * of in-bounds taps (avg_pool_test.cc:490-514). Quantized: operate on
 * (x - z_in), scale by s_in/s_out, round half to even, add z_out, saturate.
 * L2 (src/tim/vx/type_utils.cc:99-100 -> VX_NN_POOLING_L2): the root of the
 * mean of the squares, the mean taken over k_w*k_h like AVG's (padding counts
 * as zeros); no reference test holds an L2 vector: the divisor is this
 * restatement's choice (parity unpinned), the arithmetic is pinned by closed
 * forms. Quantized: ratio * sqrt(sum (x - z_in)^2 / div) in double.
 */
void tvxo_pool2d(const tvxo_pool_desc* d, const void* x, void* y) {
  const int quant = d->dtype == TVXO_U8 || d->dtype == TVXO_I8;
  const int32_t qmin = d->dtype == TVXO_U8 ? 0 : -128, qmax = d->dtype == TVXO_U8 ? 255 : 127;
  const double ratio = quant ? (double)d->in_scale / (double)d->out_scale : 1.0;
  int32_t mult = 0, shift = 0;
  if (quant) tvxo_quantize_multiplier(ratio, &mult, &shift);
  const int64_t planes = (int64_t)d->batch * d->channels;
#pragma omp parallel for schedule(static)
  for (int64_t p = 0; p < planes; ++p) {
    const int64_t xb = p * d->in_w * d->in_h, yb = p * d->out_w * d->out_h;
    for (int32_t oh = 0; oh < d->out_h; ++oh) {
      for (int32_t ow = 0; ow < d->out_w; ++ow) {
        int32_t cnt = 0, imax = INT32_MIN;
        int64_t isum = 0, isq = 0;
        float fmax = -INFINITY, fsum = 0.f, fsq = 0.f;
        for (int32_t ky = 0; ky < d->k_h; ++ky) {
          const int32_t ih = oh * d->stride_h - d->pad_top + ky;
          if (ih < 0 || ih >= d->in_h) continue;
          for (int32_t kx = 0; kx < d->k_w; ++kx) {
            const int32_t iw = ow * d->stride_w - d->pad_left + kx;
            if (iw < 0 || iw >= d->in_w) continue;
            const int64_t xi = xb + (int64_t)ih * d->in_w + iw;
            ++cnt;
            if (quant) {
              int32_t v = load_q(x, d->dtype, xi) - d->in_zp;
              isum += v;
              isq += (int64_t)v * v;
              if (v > imax) imax = v;
            } else {
              float v = load_f(x, d->dtype, xi);
              fsum += v;
              fsq += v * v;
              if (v > fmax) fmax = v;
            }
          }
        }
        const int64_t yi = yb + (int64_t)oh * d->out_w + ow;
        const int32_t div = d->pool_type == TVXO_POOL_AVG || d->pool_type == TVXO_POOL_L2 ? d->k_w * d->k_h : cnt;
        if (quant) {
          int64_t r;
          if (d->pool_type == TVXO_POOL_MAX) {
            r = cnt ? tvxo_requant(imax, mult, shift) : 0;
          } else if (d->pool_type == TVXO_POOL_L2) {
            r = (int64_t)nearbyint(ratio * sqrt((double)isq / (double)div));
          } else {
            r = div ? (int64_t)nearbyint((double)isum * ratio / (double)div) : 0;
          }
          store_q(y, d->dtype, yi, clamp64(r + d->out_zp, qmin, qmax));
        } else {
          float r = d->pool_type == TVXO_POOL_MAX ? (cnt ? fmax : 0.f) : (div ? fsum / (float)div : 0.f);
          if (d->pool_type == TVXO_POOL_L2) r = sqrtf(fsq / (float)div);
          store_f(y, d->dtype, yi, r);
        }
      }
    }
  }
}

/*
 * Standalone ReLU / ReLU6 (vxActivationLayer; src/tim/vx/ops/activations.cc:33-42):
 * clamp in the real domain, requantized to the output tensor's scale/zp.
 */
void tvxo_activation(int act, int dtype, int64_t count, const void* x, float in_scale,
                     int32_t in_zp, void* y, float out_scale, int32_t out_zp) {
  if (dtype == TVXO_U8 || dtype == TVXO_I8) {
    int32_t mult, shift, lo, hi;
    tvxo_quantize_multiplier((double)in_scale / (double)out_scale, &mult, &shift);
    tvxo_act_range(dtype, out_scale, out_zp, act, &lo, &hi);
    for (int64_t i = 0; i < count; ++i) {
      int64_t r = tvxo_requant(load_q(x, dtype, i) - in_zp, mult, shift);
      store_q(y, dtype, i, clamp64(r + out_zp, lo, hi));
    }
  } else {
    for (int64_t i = 0; i < count; ++i) {
      float v = load_f(x, dtype, i);
      if (act != TVXO_ACT_NONE) v = v < 0.f ? 0.f : v;
      if (act == TVXO_ACT_RELU6) v = v > 6.f ? 6.f : v;
      store_f(y, dtype, i, v);
    }
  }
}

/*
 * Quantized / float elementwise Add (vxTensorAddNode;
 * src/tim/vx/internal/src/kernel/vx/eltwise_vx.c:56-67), same-shape operands:
 *   y = clamp(rne(fma(a - za, sa/so, (b - zb) * (sb/so))) + zo)   in double.
 */
void tvxo_add(int dtype, int64_t count, const void* a, float a_scale, int32_t a_zp,
              const void* b, float b_scale, int32_t b_zp, void* y, float out_scale,
              int32_t out_zp) {
  if (dtype == TVXO_U8 || dtype == TVXO_I8) {
    const int32_t qmin = dtype == TVXO_U8 ? 0 : -128, qmax = dtype == TVXO_U8 ? 255 : 127;
    const double ra = (double)a_scale / (double)out_scale, rb = (double)b_scale / (double)out_scale;
    for (int64_t i = 0; i < count; ++i) {
      double tb = (double)(load_q(b, dtype, i) - b_zp) * rb;
      double t = fma((double)(load_q(a, dtype, i) - a_zp), ra, tb);
      store_q(y, dtype, i, clamp64((int64_t)nearbyint(t) + out_zp, qmin, qmax));
    }
  } else {
    for (int64_t i = 0; i < count; ++i) store_f(y, dtype, i, load_f(a, dtype, i) + load_f(b, dtype, i));
  }
}

/*
 * Softmax over dim 0 of a {C, rows} view, fp32 output
 * (vxSoftmaxLayer2; src/tim/vx/internal/src/kernel/vx/softmax_vx.c:88):
 * dequantize, subtract the row maximum, exp(beta * v), normalize.
 */
void tvxo_softmax(int dtype, int32_t c, int64_t rows, int64_t inner, float beta, const void* x,
                  float in_scale, int32_t in_zp, float* y) {
  /* the tensor is {inner, c, rows} with inner fastest: the axis' elements are `inner` apart
   * (src/tim/vx/ops/softmax_test.cc:30-290 pins axes 0, 1 and 2 of 2-D and 3-D tensors) */
  if (inner < 1) inner = 1;
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t in = 0; in < inner; ++in) {
      const int64_t base = r * c * inner + in;
      float mx = -INFINITY, sum = 0.f;
      for (int32_t i = 0; i < c; ++i) {
        int64_t idx = base + i * inner;
        float v = (dtype == TVXO_U8 || dtype == TVXO_I8) ? in_scale * (float)(load_q(x, dtype, idx) - in_zp)
                                                       : load_f(x, dtype, idx);
        y[idx] = v;
        if (v > mx) mx = v;
      }
      for (int32_t i = 0; i < c; ++i) {
        float e = expf(beta * (y[base + i * inner] - mx));
        y[base + i * inner] = e;
        sum += e;
      }
      for (int32_t i = 0; i < c; ++i) y[base + i * inner] /= sum;
    }
  }
}

/*
 * DataConvert (VSI_NN_OP_DATACONVERT; src/tim/vx/ops/simple_operations.cc:39): every element
 * goes through float32, as in ovxlib's type conversions
 * (src/tim/vx/internal/include/utils/vsi_nn_dtype_util_prv.h:228-266):
 *   f = (q - zp) * scale            for a quantized input, the value itself for a float one
 *   q = sat(rint(f / scale) + zp)   for a quantized output (round half to even)
 */
void tvxo_convert(int in_dtype, int64_t count, const void* x, float in_scale, int32_t in_zp,
                  int out_dtype, void* y, float out_scale, int32_t out_zp) {
  const int in_q = in_dtype == TVXO_U8 || in_dtype == TVXO_I8;
  const int out_q = out_dtype == TVXO_U8 || out_dtype == TVXO_I8;
  const double qmin = out_dtype == TVXO_U8 ? 0 : -128, qmax = out_dtype == TVXO_U8 ? 255 : 127;
  for (int64_t i = 0; i < count; ++i) {
    const float f = in_q ? ((float)load_q(x, in_dtype, i) - (float)in_zp) * in_scale : load_f(x, in_dtype, i);
    if (out_q) {
      double r = (double)rintf(f / out_scale) + (double)out_zp;
      r = r < qmin ? qmin : (r > qmax ? qmax : r);
      if (r != r) r = qmin;
      store_q(y, out_dtype, i, (int64_t)r);
    } else {
      store_f(y, out_dtype, i, f);
    }
  }
}

/*
 * Transpose (PERMUTE): output dimension i is input dimension perm[i], dimension 0 fastest
 * (src/tim/vx/internal/src/ops/vsi_nn_op_permute.c:219-230 sizes the output as
 * out.size[i] = in.size[perm[i]]; src/tim/vx/ops/transpose_test.cc:29-100). Elements are
 * moved byte for byte. Written as a walk over INPUT coordinates that scatters, the reverse
 * of the product's gather.
 */
void tvxo_transpose(int32_t rank, const uint32_t* in_dims, const uint32_t* perm, int32_t elem_bytes,
                    const void* x, void* y) {
  uint64_t out_stride_of_in[8], out_dims[8], total = 1, s = 1;
  for (int32_t i = 0; i < rank; ++i) out_dims[i] = in_dims[perm[i]];
  for (int32_t i = 0; i < rank; ++i) {
    out_stride_of_in[perm[i]] = s; /* input dimension perm[i] is output dimension i */
    s *= out_dims[i];
    total *= in_dims[i];
  }
  uint32_t coord[8] = {0};
  for (uint64_t idx = 0; idx < total; ++idx) {
    uint64_t dst = 0;
    for (int32_t i = 0; i < rank; ++i) dst += coord[i] * out_stride_of_in[i];
    memcpy((char*)y + dst * elem_bytes, (const char*)x + idx * elem_bytes, (size_t)elem_bytes);
    for (int32_t i = 0; i < rank; ++i) {
      if (++coord[i] < in_dims[i]) break;
      coord[i] = 0;
    }
  }
}

int tvxo_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
void tvxo_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}
