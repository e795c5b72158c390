// Depthwise 3x3 convolution and the pointwise (1x1) convolution it only feeds, as one kernel: the tensor
// between them - in a MobileNet block the widest of the block - never leaves the CU. In the reference the
// two are separate vxConvolutionLayer nodes that the closed driver merges when it verifies the graph
// (src/tim/vx/internal/src/vsi_nn_graph.c:1591-1603); here the runtime asks for the merged operator when
// the depthwise result has no other reader. Bit for bit the two operators one after the other: the
// depthwise result is requantized to its own tensor's scale and zero point (and clamped by its fused
// ReLU / ReLU6) before the pointwise convolution reads it.
//
// A workgroup owns RPT whole output rows of one image (at most 128 pixels) for every channel:
//   1. depthwise phase - the stencil of dwconv3x3_i8: a thread holds four columns x RPT rows of one
//      channel plane, loads only the dwords under its own columns (the neighbours' come by wavefront
//      shifts), cuts the windows with v_alignbyte and multiplies with v_dot4; the requantized dwords
//      (four pixels of one channel) go to an LDS tile in the tensor's own order [channel][pixel];
//   2. from there the pixel-major operand tile of the matrix cores is built exactly as pwconv_i8 builds
//      it from global memory (4 x 4 byte transposes in registers, 16-byte LDS stores);
//   3. pointwise phase - as in pwconv_i8's 32-pixel form: a wavefront owns 32 pixels and walks the 32-channel
//      output tiles, weights stream from L2 in MFMA-fragment order, results are staged per wavefront and
//      leave as 16-byte chunks of contiguous WHCN rows; the zero-point term of uint8 weights is a second MFMA
//      against a constant fragment; a residual Add behind the pointwise convolution rides on the copy-out.
#include <algorithm>
#include <cstdlib>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kMaxSlots = 512;      // most pixel slots of a tile (32-pixel MFMA tiles, a multiple of four of them)
constexpr int kStageStride = 40;    // bytes per staged output row of 32 pixels (8-byte aligned rows)
constexpr int kStageBytes = 32 * kStageStride;

struct DwPwArgs {
  const uint8_t* x;      // depthwise input {W, H, C, N}
  uint8_t* y;            // pointwise output {OW, OH, OC, N}
  // ---- depthwise part (tables as in dwconv3x3_i8)
  const int32_t* dw_wpk;
  const int32_t* dw_biasf;
  const tvx_v4i* dw_rq;
  int C, H, W, OH, OW;
  int pad_t;
  int ow4, lpr_shift;
  int dw_xor_mask, dw_pad_fill, dw_zws, dw_out_zp, dw_lo, dw_hi;
  int dw_box;            // the depthwise weights are packed unshifted: the window sum carries their zero point
  int dw_ties, pw_ties;  // whether an accumulator of the depthwise / pointwise convolution can land on an exact .5
  uint32_t c4n_magic;    // ceil(2^32 / (cp / 4)): a division by multiply-high
  // ---- pointwise part (tables as in pwconv_i8)
  const v4i* wpk;
  const int32_t* biasf;
  const v4i* rq;
  int OC, cp, ksteps, pix_stride, oc_tiles;
  int xor_mask, neg_zws4, zp;
  int out_zp, lo, hi;
  int P;                 // pixels of a tile: RPT * OW
  int slots;             // P rounded up to a multiple of 128
  int tiles_per_image;
  // ---- fused residual Add behind the pointwise convolution (0 = off), as in pwconv_i8
  const uint8_t* res;
  double add_ra, add_rb;
  int add_mode, add_signed;
  int add_za, add_zb, add_zo, add_lo, add_hi;
};

// Four columns x RPT output rows of one depthwise channel plane, in two steps so that the loads of several
// channels can be in flight together; S = stride, PL = left padding.
template <int S, int RPT>
struct PatchShape {
  static constexpr int kOwn = S;                    // input dwords under a thread's four outputs
  static constexpr int kRows = S * (RPT - 1) + 3;   // input rows behind its output rows
};

template <int S, int RPT>
__device__ __forceinline__ void PatchLoad(const DwPwArgs& a, const uint8_t* xn, uint32_t plane_off, int w4, int oh0,
                                          int (&raw)[PatchShape<S, RPT>::kRows][PatchShape<S, RPT>::kOwn + 2]) {
  constexpr int kOwn = PatchShape<S, RPT>::kOwn, kRows = PatchShape<S, RPT>::kRows;
  const int in_dwords = a.W / 4;
  const int d0 = S * w4;
  const int ih0 = oh0 * S - a.pad_t;
  // xn: the image (uniform), plane_off: the channel plane inside it; offsets inside an image fit 32 bits (checked at
  // creation): one scalar base + one vector offset per load. Rows outside the image read the nearest row inside.
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int ihc = min(max(ih0 + r, 0), a.H - 1);
    const uint32_t row_off = plane_off + __umul24(static_cast<uint32_t>(ihc), static_cast<uint32_t>(a.W));
#pragma unroll
    for (int i = 0; i < kOwn; ++i)  // unconditional: masked later
      raw[r][1 + i] = *reinterpret_cast<const int*>(xn + (row_off + static_cast<uint32_t>(min(d0 + i, in_dwords - 1)) * 4u));
  }
}

// A depthwise channel's constants: three rows of taps (a dword each), the folded bias, the requantization record.
struct ChannelConsts {
  v4i taps;  // (the fourth dword is not used here)
  int bias;
  v4i q;
};

__device__ __forceinline__ ChannelConsts LoadChannelConsts(const DwPwArgs& a, int c) {
  ChannelConsts k;
  k.taps = *reinterpret_cast<const v4i*>(a.dw_wpk + c * 4);
  k.bias = a.dw_biasf[c];
  k.q = a.dw_rq[c];
  return k;
}

template <int S, int PL, int RPT>
__device__ __forceinline__ void PatchCompute(const DwPwArgs& a, const ChannelConsts& k, int w4, int oh0,
                                             int (&raw)[PatchShape<S, RPT>::kRows][PatchShape<S, RPT>::kOwn + 2],
                                             uint32_t (&packed)[RPT]) {
  constexpr int kOwn = PatchShape<S, RPT>::kOwn, kRows = PatchShape<S, RPT>::kRows;
  const int wk0 = k.taps[0], wk1 = k.taps[1], wk2 = k.taps[2];
  const bool box = a.dw_box != 0;  // (wave-uniform: a branch, not a mask)
  const int bias = k.bias;
  const v4i q = k.q;
  const int in_dwords = a.W / 4;
  const int d0 = S * w4;
  const int ih0 = oh0 * S - a.pad_t;
  const bool has_left = w4 > 0;
  const bool has_right = d0 + kOwn < in_dwords;
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int ih = ih0 + r;
    const int keep_row = (ih >= 0 && ih < a.H) ? -1 : 0;
#pragma unroll
    for (int i = 0; i < kOwn; ++i) {
      const int keep = d0 + i < in_dwords ? keep_row : 0;
      raw[r][1 + i] = ((raw[r][1 + i] ^ a.dw_xor_mask) & keep) | (a.dw_pad_fill & ~keep);
    }
  }
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    // (the wavefront's first / last lane has no such neighbour; it is the first / last lane of an image row and takes the padding)
    const int l = __builtin_amdgcn_mov_dpp(raw[r][kOwn], 0x138, 0xf, 0xf, true);
    const int rr = __builtin_amdgcn_mov_dpp(raw[r][1], 0x130, 0xf, 0xf, true);
    raw[r][0] = has_left ? l : a.dw_pad_fill;
    raw[r][kOwn + 1] = has_right ? rr : a.dw_pad_fill;
  }
#pragma unroll
  for (int o = 0; o < RPT; ++o) {
    int win[3][4];
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      win[r][0] = Window<4 + S * 0 - PL>(raw[S * o + r]);
      win[r][1] = Window<4 + S * 1 - PL>(raw[S * o + r]);
      win[r][2] = Window<4 + S * 2 - PL>(raw[S * o + r]);
      win[r][3] = Window<4 + S * 3 - PL>(raw[S * o + r]);
    }
    int accs[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int acc = Dot4Add(win[0][i], wk0, bias);
      acc = __builtin_amdgcn_sdot4(win[1][i], wk1, acc, false);
      acc = __builtin_amdgcn_sdot4(win[2][i], wk2, acc, false);
      if (box) {
        int sx = __builtin_amdgcn_sdot4(win[0][i], 0x00010101, 0, false);
        sx = __builtin_amdgcn_sdot4(win[1][i], 0x00010101, sx, false);
        sx = __builtin_amdgcn_sdot4(win[2][i], 0x00010101, sx, false);
        acc -= a.dw_zws * sx;
      }
      accs[i] = acc;
    }
    packed[o] = Requant8x4Pack(accs, q, a.dw_out_zp, a.dw_lo, a.dw_hi, a.dw_ties);
  }
}

// S: stride of the depthwise convolution (left padding 1 at stride 1, 0 at stride 2: SAME);
// RPT: output rows of a tile.
// (two wavefronts per SIMD at least: within 256 registers the compiler keeps MFMA accumulators in ordinary vector
// registers, where the epilogue reads them, instead of moving every value out of the accumulation registers first)
template <int S, int RPT, bool ADD>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) DwPwKernel(DwPwArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  constexpr int PL = S == 1 ? 1 : 0;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // an XCD gets a contiguous run of tiles: vertically neighbouring tiles share input rows in its L2
  int wg = blockIdx.x;
  {
    const int per = gridDim.x >> 3, rem = gridDim.x & 7, xcd = wg & 7;
    wg = xcd * per + min(xcd, rem) + (wg >> 3);
  }
  const int n = wg / a.tiles_per_image;
  const int g = wg - n * a.tiles_per_image;
  const int oh0 = g * RPT;
  const int hw = a.OH * a.OW;
  const int mid_stride = a.slots + 4;              // bytes per channel row of the depthwise tile (+ 4: bank spread)
  int8_t* mid = lds;                               // [channel][slots + 4]: the depthwise result of the tile
  int8_t* xl = lds + a.cp * mid_stride;            // [pixel slot][pix_stride]: the MFMA operand tile
  int8_t* stage = xl + a.slots * a.pix_stride + wave * kStageBytes;
  int8_t* w_lds = xl + a.slots * a.pix_stride + 4 * kStageBytes;  // the pointwise weights, in fragment order
  const int oc_alloc = a.oc_tiles * 32;
  v4i* rq_lds = reinterpret_cast<v4i*>(w_lds + oc_alloc * a.cp);
  int* bias_lds = reinterpret_cast<int*>(rq_lds + oc_alloc);

  // ---- the pointwise weights and the epilogue's tables: global -> LDS by DMA, under the depthwise phase ----
  {
    typedef const __attribute__((address_space(1))) void* gptr;
    typedef __attribute__((address_space(3))) void* lptr;
    const int chunks = oc_alloc * a.cp >> 4;
    for (int i = wave * 64; i < chunks; i += kThreads)
      if (i + lane < chunks)
        __builtin_amdgcn_global_load_lds((gptr)(a.wpk + i + lane), (lptr)(w_lds + i * 16), 16, 0, 0);
    for (int i = wave * 64; i < oc_alloc; i += kThreads)
      if (i + lane < oc_alloc) {
        __builtin_amdgcn_global_load_lds((gptr)(a.rq + i + lane), (lptr)(rq_lds + i), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr)(a.biasf + i + lane), (lptr)(bias_lds + i), 4, 0, 0);
      }
  }

  // ---- 1. depthwise: (channel, four columns) per thread and pass, RPT rows; the loads of several passes
  // are issued together (a pass on its own would be one memory round trip each) ----
  {
    constexpr int kRows = PatchShape<S, RPT>::kRows, kOwn = PatchShape<S, RPT>::kOwn;
    constexpr int kBatch = (24 / (kRows * kOwn)) > 8 ? 8 : ((24 / (kRows * kOwn)) < 1 ? 1 : (24 / (kRows * kOwn)));
    const int w4 = tid & ((1 << a.lpr_shift) - 1);
    const int per_pass = kThreads >> a.lpr_shift;
    const size_t plane = static_cast<size_t>(a.H) * a.W;
    const uint32_t plane32 = static_cast<uint32_t>(plane);
    const uint8_t* xn = a.x + static_cast<size_t>(n) * a.C * plane;
    for (int c0 = tid >> a.lpr_shift; c0 < a.C; c0 += per_pass * kBatch) {
      int raw[kBatch][kRows][kOwn + 2];
      ChannelConsts consts[kBatch];
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const int c = min(c0 + b * per_pass, a.C - 1);
        PatchLoad<S, RPT>(a, xn, static_cast<uint32_t>(c) * plane32, w4, oh0, raw[b]);
        consts[b] = LoadChannelConsts(a, c);
      }
#pragma unroll
      for (int b = 0; b < kBatch; ++b) {
        const int c = c0 + b * per_pass;
        if (c < a.C) {  // whole image rows of lanes take this branch together
          uint32_t packed[RPT];
          PatchCompute<S, PL, RPT>(a, consts[b], w4, oh0, raw[b], packed);
          if (w4 < a.ow4) {
#pragma unroll
            for (int o = 0; o < RPT; ++o)
              *reinterpret_cast<uint32_t*>(mid + c * mid_stride + o * a.OW + w4 * 4) = packed[o];
          }
        }
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the DMA above)
  __syncthreads();
  // ---- 2. [channel][pixel] -> [pixel][channel]: a thread turns four channels of four pixels ----
  {
    const int c4n = a.cp >> 2;                 // (a multiple of 8)
    const int items = (a.slots >> 2) * c4n;
    for (int it = tid; it < items; it += kThreads) {
      const int pq = __umulhi(it, a.c4n_magic), c4 = it - pq * c4n;
      const bool live = pq * 4 < a.P;
      uint32_t raw[4], t[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int c = c4 * 4 + j;
        const uint32_t v = *reinterpret_cast<const uint32_t*>(mid + min(c, a.C - 1) * mid_stride + pq * 4);
        raw[j] = (live && c < a.C) ? v ^ a.xor_mask : 0u;
      }
      Transpose4x4(raw, t);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        *reinterpret_cast<uint32_t*>(xl + (pq * 4 + e) * a.pix_stride + c4 * 4) = t[e];
    }
  }
  __syncthreads();

  // ---- 3. pointwise: a wavefront takes 32 pixel slots at a time and walks every output tile ----
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const v4i fz = {a.neg_zws4, a.neg_zws4, a.neg_zws4, a.neg_zws4};
  for (int part0 = wave * 32; part0 < a.P; part0 += 128) {
    // copy-out mapping of a staged 32 x 32 patch: lane -> 16-pixel chunk lane & 1 of output-channel row lane >> 1
    const int px_in_row = part0 + (lane & 1) * 16;
    const bool out_live = px_in_row < a.P;
    const size_t out_off = static_cast<size_t>(n) * a.OC * hw + static_cast<size_t>(g) * a.P + px_in_row;
    const int8_t* xa = xl + (part0 + frag_row) * a.pix_stride + frag_half * 16;
    for (int tile = 0; tile < a.oc_tiles; ++tile) {
      const v4i q = rq_lds[tile * 32 + frag_row];
      const int nb = bias_lds[tile * 32 + frag_row];
      v16i acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = nb;
      const v4i* wf = reinterpret_cast<const v4i*>(w_lds) + tile * a.ksteps * 64 + lane;
      v4i fw = wf[0], fx = *reinterpret_cast<const v4i*>(xa);
      for (int k = 0; k < a.ksteps; ++k) {
        const int kn = min(k + 1, a.ksteps - 1);
        const v4i fw1 = wf[kn * 64];
        const v4i fx1 = *reinterpret_cast<const v4i*>(xa + kn * 32);
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx, fw, acc, 0, 0, 0);
        if (a.zp) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx, fz, acc, 0, 0, 0);
        fw = fw1; fx = fx1;
      }
      // ---- epilogue: the residual operand first (it travels while the results are requantized) ----
      const int rows = min(32, a.OC - tile * 32);
      const int row = lane >> 1;
      const size_t at = out_off + (static_cast<size_t>(tile) * 32 + row) * hw;
      uint4 res16 = make_uint4(0, 0, 0, 0);
      if (ADD && row < rows && out_live) res16 = *reinterpret_cast<const uint4*>(a.res + at);
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        const int pl = 8 * gq + 4 * frag_half;
        const int av[4] = {acc[gq * 4], acc[gq * 4 + 1], acc[gq * 4 + 2], acc[gq * 4 + 3]};
        *reinterpret_cast<uint32_t*>(stage + frag_row * kStageStride + pl) = Requant8x4Pack(av, q, a.out_zp, a.lo, a.hi, a.pw_ties);
      }
      __builtin_amdgcn_wave_barrier();
      {
        const int8_t* sp = stage + row * kStageStride + (lane & 1) * 16;
        const uint2 lo8 = *reinterpret_cast<const uint2*>(sp);
        const uint2 hi8 = *reinterpret_cast<const uint2*>(sp + 8);
        if (row < rows && out_live) {
          uint4 o = make_uint4(lo8.x, lo8.y, hi8.x, hi8.y);
          if (ADD)
            o = make_uint4(AddResidual4(a, o.x, res16.x), AddResidual4(a, o.y, res16.y), AddResidual4(a, o.z, res16.z),
                           AddResidual4(a, o.w, res16.w));
          *reinterpret_cast<uint4*>(a.y + at) = o;
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

struct Plan {
  DwPwArgs a;
  int lds_bytes, stride, rpt;
  dim3 grid;
};

typedef void (*DwPwFn)(DwPwArgs);

template <bool ADD>
DwPwFn KernelOf(int stride, int rpt) {
  if (stride == 1) return rpt == 4 ? DwPwKernel<1, 4, ADD> : (rpt == 2 ? DwPwKernel<1, 2, ADD> : DwPwKernel<1, 1, ADD>);
  return rpt == 4 ? DwPwKernel<2, 4, ADD> : (rpt == 2 ? DwPwKernel<2, 2, ADD> : DwPwKernel<2, 1, ADD>);
}
DwPwFn Kernel(int stride, int rpt, bool add) {
  return add ? KernelOf<true>(stride, rpt) : KernelOf<false>(stride, rpt);
}

int DwPwRun(tvx_op* op, const void* in0, const void* in1, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  DwPwArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  a.res = static_cast<const uint8_t*>(in1);
  if (a.add_mode && !in1) return SetError(TVX_E_INVALID, "dwpw_i8: the fused Add needs its second operand as in1");
  if ((reinterpret_cast<uintptr_t>(in0) & 3) | ((reinterpret_cast<uintptr_t>(out) | (a.add_mode ? reinterpret_cast<uintptr_t>(in1) : 0)) & 15))
    return SetError(TVX_E_INVALID, "dwpw_i8: the input must be 4-byte, the output (and the Add's operand) 16-byte aligned");
  hipLaunchKernelGGL(Kernel(plan->stride, plan->rpt, a.add_mode != 0), plan->grid, dim3(kThreads), plan->lds_bytes, st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

int RoundUp(int v, int m) { return (v + m - 1) / m * m; }

}  // namespace

// `op` carries the pointwise convolution (op->conv, requantization tables, clamp, fused Add); `dw` and its
// tables describe the depthwise convolution in front of it. Declines (TVX_E_UNSUPPORTED) what the kernel does
// not cover; the caller then creates the two operators.
int DwPwSetup(tvx_op* op, const tvx_conv2d_desc* dw, const void* dw_w, const void* dw_b,
              const std::vector<int32_t>& dw_mult, const std::vector<int32_t>& dw_shift, int dw_lo, int dw_hi,
              const tvx_conv2d_desc* pw, const void* pw_w, const void* pw_b) {
  if (!dw_w || !pw_w) return TVX_E_UNSUPPORTED;
  // ---- depthwise: 3x3, multiplier 1, SAME at stride 1 or 2, rows of whole dwords ----
  if (dw->multiplier != 1 || dw->k_w != 3 || dw->k_h != 3 || dw->dilation_w != 1 || dw->dilation_h != 1) return TVX_E_UNSUPPORTED;
  if (dw->stride_w != dw->stride_h || (dw->stride_w != 1 && dw->stride_w != 2)) return TVX_E_UNSUPPORTED;
  const int S = dw->stride_w;
  if (dw->pad_left != (S == 1 ? 1u : 0u) || dw->pad_top > 1 || (dw->in_w & 3) || (dw->out_w & 3)) return TVX_E_UNSUPPORTED;
  const int ow4 = dw->out_w / 4, in_dw = dw->in_w / 4;
  int lpr_shift = 0;
  while ((1 << lpr_shift) < ow4 || S * (1 << lpr_shift) < in_dw) ++lpr_shift;
  if (lpr_shift > 6) return TVX_E_UNSUPPORTED;
  if (static_cast<uint32_t>((dw->out_w - 1) * S + 2) >= dw->in_w + dw->pad_left + 4) return TVX_E_UNSUPPORTED;
  // ---- pointwise: 1x1, stride 1, unpadded, on the depthwise result ----
  if (pw->multiplier != 0 || pw->groups > 1 || pw->k_w != 1 || pw->k_h != 1 || pw->stride_w != 1 || pw->stride_h != 1 ||
      pw->pad_left != 0 || pw->pad_top != 0)
    return TVX_E_UNSUPPORTED;
  if (pw->in_w != dw->out_w || pw->in_h != dw->out_h || pw->in_c != dw->out_c || pw->batch != dw->batch ||
      pw->out_w != pw->in_w || pw->out_h != pw->in_h || pw->in_dtype != dw->out_dtype ||
      pw->in_scale != dw->out_scale || pw->in_zp != dw->out_zp)
    return TVX_E_UNSUPPORTED;
  // ---- tile: whole rows, at most kMaxSlots pixels, 16-byte chunks ----
  // (as many rows as keep the tile's LDS image - depthwise tile, operand tile, staging - within a third of a CU's)
  const int cp_ = RoundUp(static_cast<int>(dw->in_c), 32);
  const int oc_alloc_ = RoundUp(static_cast<int>(pw->out_c), 32);
  auto lds_of = [&](int r) {
    const int slots = RoundUp(r * static_cast<int>(dw->out_w), 128);
    return cp_ * (slots + 4) + slots * (cp_ + 16) + 4 * kStageBytes + oc_alloc_ * (cp_ + 20);
  };
  auto fits = [&](int r) {
    return r * dw->out_w <= static_cast<uint32_t>(kMaxSlots) && dw->out_h % r == 0 && (r * dw->out_w) % 16 == 0;
  };
  // Among the tiles that fit: the one with the least work on the busiest CU. A CU handles a whole number of
  // tiles; a tile's cost grows with its pixels, shorter tiles re-read more input rows per output row.
  int rpt = 0;
  {
    int cus = 256;
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0)
      cus = prop.multiProcessorCount;
    double best = 0;
    for (int r : {4, 2, 1}) {
      if (!fits(r) || lds_of(r) > 52 * 1024) continue;
      const uint64_t wgs = static_cast<uint64_t>(dw->batch) * (dw->out_h / r);
      const double per_cu = static_cast<double>((wgs + cus - 1) / cus);
      const double cost = per_cu * r * (r == 1 ? 1.3 : (r == 2 ? 1.08 : 1.0));
      if (!rpt || cost < best) { rpt = r; best = cost; }
    }
  }
  if (!rpt)  // (no tile that small: the fewest rows that make 16-byte chunks)
    for (int r : {1, 2, 4})
      if (fits(r)) { rpt = r; break; }
  if (const char* f = getenv("TVX_DWPW_ROWS")) {  // tuning aid
    const int r = atoi(f);
    if ((r == 1 || r == 2 || r == 4) && fits(r)) rpt = r;
  }
  if (!rpt) return TVX_E_UNSUPPORTED;
  const uint64_t tiles = static_cast<uint64_t>(dw->batch) * (dw->out_h / rpt);
  if (tiles > 0x7fffffffull || static_cast<uint64_t>(dw->in_h) * dw->in_w * dw->in_c >= (1ull << 32) - 16 || dw->in_h >= (1u << 24)) return TVX_E_UNSUPPORTED;  // (32-bit offsets inside an image)

  DwPwArgs a{};
  const int C = dw->in_c;
  a.C = C; a.H = dw->in_h; a.W = dw->in_w; a.OH = dw->out_h; a.OW = dw->out_w;
  a.pad_t = dw->pad_top;
  a.ow4 = ow4; a.lpr_shift = lpr_shift;
  const bool x_u8 = dw->in_dtype == TVX_U8, dww_u8 = dw->w_dtype == TVX_U8;
  const int dzxs = dw->in_zp - (x_u8 ? 128 : 0);
  const int dzws = (dw->w_scales ? 0 : dw->w_zp) - (dww_u8 ? 128 : 0);
  if (dzxs < -128 || dzxs > 127) return TVX_E_UNSUPPORTED;
  std::vector<int32_t> dwpk, dbiasf, drq;
  a.dw_box = PackDepthwise3x3(C, dw_w, dww_u8, dw_b, dzxs, dzws, true, &dwpk, &dbiasf);
  const int dw_rq = BuildRequantRecords(dw_mult, dw_shift, C, C, dw->out_zp, &drq, AccumulatorBound(9, dw_b, C));
  if (dw_rq == kRqGeneric) return TVX_E_UNSUPPORTED;
  a.dw_ties = dw_rq == kRqFast;
  a.dw_xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.dw_pad_fill = static_cast<int>(static_cast<uint32_t>(dzxs & 0xff) * 0x01010101u);
  a.dw_zws = dzws; a.dw_out_zp = dw->out_zp; a.dw_lo = dw_lo; a.dw_hi = dw_hi;

  a.OC = pw->out_c;
  a.cp = RoundUp(C, 32);
  a.ksteps = a.cp / 32;
  a.pix_stride = a.cp + 16;
  a.oc_tiles = (a.OC + 31) / 32;
  a.P = rpt * dw->out_w;
  a.slots = RoundUp(a.P, 128);
  a.tiles_per_image = dw->out_h / rpt;
  const bool m_u8 = pw->in_dtype == TVX_U8, pww_u8 = pw->w_dtype == TVX_U8;
  const int zxs = pw->in_zp - (m_u8 ? 128 : 0);
  const int zws = op->w_zp - (pww_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127 || zws < -127 || zws > 127) return TVX_E_UNSUPPORTED;
  a.xor_mask = m_u8 ? static_cast<int>(0x80808080u) : 0;
  a.neg_zws4 = static_cast<int>(static_cast<uint32_t>((-zws) & 0xff) * 0x01010101u);
  a.zp = zws != 0;
  a.out_zp = pw->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  if (op->fused_add) {
    const tvx_eltwise_desc& e = op->elt;
    const double ra = static_cast<double>(e.a_scale) / static_cast<double>(e.out_scale);
    const double rb = static_cast<double>(e.b_scale) / static_cast<double>(e.out_scale);
    if (!(ra < 1048576.0) || !(rb < 1048576.0)) return TVX_E_UNSUPPORTED;
    a.add_mode = op->fused_add;
    a.add_signed = pw->out_dtype == TVX_I8;
    a.add_ra = ra; a.add_rb = rb;
    a.add_za = e.a_zp; a.add_zb = e.b_zp; a.add_zo = e.out_zp;
    ActRange(pw->out_dtype, e.out_scale, e.out_zp, TVX_ACT_NONE, &a.add_lo, &a.add_hi);
  }
  const int lds_bytes = lds_of(rpt);
  if (lds_bytes > 160 * 1024) return TVX_E_UNSUPPORTED;
  // pointwise weights in fragment order, constants folded into the bias (as PwConvSetup packs them)
  const int oc_alloc = a.oc_tiles * 32;
  std::vector<int8_t> packed(static_cast<size_t>(a.oc_tiles) * a.ksteps * 1024, 0);
  std::vector<int32_t> biasf(oc_alloc, 0);
  const uint8_t* src = static_cast<const uint8_t*>(pw_w);
  const int32_t* b = static_cast<const int32_t*>(pw_b);
  for (int oc = 0; oc < a.OC; ++oc) {
    int64_t sw = 0;
    for (int c = 0; c < C; ++c) {
      const uint8_t raw = src[static_cast<size_t>(oc) * C + c];
      const int8_t v = static_cast<int8_t>(pww_u8 ? raw ^ 0x80 : raw);
      const int ks = c / 32, half = (c % 32) / 16, j = c % 16;
      packed[((static_cast<size_t>(oc / 32) * a.ksteps + ks) * 64 + half * 32 + oc % 32) * 16 + j] = v;
      sw += v;
    }
    const int64_t v = (b ? b[oc] : 0) - static_cast<int64_t>(zxs) * sw + static_cast<int64_t>(C) * zxs * zws;
    biasf[oc] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  std::vector<int32_t> rqt;
  const int pw_rq =
      BuildRequantRecords(op->h_mult, op->h_shift, a.OC, oc_alloc, pw->out_zp, &rqt, AccumulatorBound(C, pw_b, a.OC));
  if (pw_rq == kRqGeneric) return TVX_E_UNSUPPORTED;
  a.pw_ties = pw_rq == kRqFast;
  a.c4n_magic = static_cast<uint32_t>(((1ull << 32) + a.cp / 4 - 1) / (a.cp / 4));
  int s = op->packed.Upload(packed.data(), packed.size());
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s == TVX_OK) s = op->weights.Upload(dwpk.data(), dwpk.size() * 4);
  if (s == TVX_OK) s = op->bias.Upload(dbiasf.data(), dbiasf.size() * 4);
  if (s == TVX_OK) s = op->aux3.Upload(drq.data(), drq.size() * 4);
  if (s != TVX_OK) return s;
  a.wpk = op->packed.as<v4i>();
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<v4i>();
  a.dw_wpk = op->weights.as<int32_t>();
  a.dw_biasf = op->bias.as<int32_t>();
  a.dw_rq = op->aux3.as<tvx_v4i>();
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel(S, rpt, a.add_mode != 0)),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (e != hipSuccess) return SetError(TVX_E_DEVICE, "hipFuncSetAttribute(dynamic LDS %d): %s", lds_bytes, hipGetErrorString(e));
  Plan plan{};
  plan.a = a;
  plan.lds_bytes = lds_bytes;
  plan.stride = S;
  plan.rpt = rpt;
  plan.grid = dim3(static_cast<unsigned>(tiles));
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = DwPwRun;
  op->kernel_name = op->fused_add ? "dwconv3x3_pwconv_add_i8" : "dwconv3x3_pwconv_i8";
  return TVX_OK;
}

}  // namespace tvx
