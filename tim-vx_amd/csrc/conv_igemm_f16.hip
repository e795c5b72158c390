// conv2d_igemm_f16: dense float16 convolution as an implicit GEMM on the matrix cores - vxConvolutionLayer as ovxlib
// reaches it for float16 tensors (reference: src/tim/vx/internal/src/ops/vsi_nn_op_conv2d.c:35-118; data types
// src/tim/vx/internal/src/ops/vsi_nn_op_conv2d.c:96-105).
//
// A workgroup (four wavefronts) owns 128 consecutive output pixels of one image and up to 64 output channels. The
// input rows behind those pixels - with the halo the window needs, padding as zeros - are transposed into LDS ONCE as
// [row][column][channel] (a thread loads two pixels of eight channel planes, eight dwords, and stores two 16-byte
// units of eight channels each), so that the eight reduction halves a lane feeds to v_mfma_f32_32x32x16_f16 are one
// 16-byte LDS read at (window row, window column, channel group) for every tap: no gather per tap. The weights are
// packed in fragment order when the operator is created and read straight from global memory (they stay in L2), a
// tap's channel steps requested one round ahead. Activations are the A operand: a lane ends up with one output channel
// and four consecutive pixels per accumulator quad - float32 accumulation, bias and activation in float32, one rounding
// to float16 -, two swaps between the wavefront's halves make that sixteen consecutive pixels: 32 contiguous bytes.
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int kPixels = 128;   // output pixels of a workgroup: one 32-pixel tile per wavefront
constexpr int kMaxSteps = 8;   // 16-channel steps of a tap: at most 128 input channels (an LDS row of a pixel is 2 C + 16 bytes)

struct FcvArgs {
  const _Float16* x;
  _Float16* y;
  const v4i* wpk;        // [channel-tile pair][tap][channel step][OT tiles][64 lanes]: eight halves each
  const float* bias;     // or null
  int C, H, W, OC, OH, OW;
  int kh, kw, s, pad_t, pad_l;
  int csteps;            // C / 16
  int halo_w;            // columns of the staged rows: (OW - 1) * s + kw
  int pix_stride;        // bytes between two pixels in LDS: 2 C + 16 (bank spread)
  int tiles_per_image;
  int act;
  int aligned4;          // OH * OW is a multiple of four: four pixels of a channel are one aligned store
};

constexpr int kStageBatch = 4;  // staging units of a thread whose loads are requested together

// OT: 32-channel tiles of a workgroup (1 or 2); PT: 32-pixel tiles of a wavefront (1 or 2: 128 or 256 pixels a workgroup);
// CSB: 16-channel steps of one multiplication round (2 or 4; a tap takes ceil(csteps / CSB) rounds)
template <int OT, int PT, int CSB>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) ConvIgemmF16Kernel(FcvArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int kTile = kPixels * PT;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = blockIdx.x / a.tiles_per_image, tile = blockIdx.x - n * a.tiles_per_image;
  const int hw = a.OH * a.OW;
  const int p0 = tile * kTile;
  const int p_last = min(p0 + kTile, hw) - 1;
  const int y0 = p0 / a.OW, y1 = p_last / a.OW;           // output rows of the tile
  const int halo_rows = (y1 - y0) * a.s + a.kh;
  const int iy0 = y0 * a.s - a.pad_t;                     // image row of halo row 0

  // ---- the halo rows -> LDS as [row][column][channel]; a unit: two columns (an aligned dword) x eight channels ----
  {
    const int jlo = (-a.pad_l) >> 1, jhi = (a.halo_w - 1 - a.pad_l) >> 1;  // column pairs: image columns 2 j, 2 j + 1
    const int pairs = jhi - jlo + 1, cgroups = a.C / 8;
    const int units = halo_rows * cgroups * pairs;
    const size_t plane = static_cast<size_t>(a.H) * a.W;
    const _Float16* xn = a.x + static_cast<size_t>(n) * a.C * plane;
    for (int u0 = tid; u0 < units; u0 += kThreads * kStageBatch) {
      uint32_t d[kStageBatch][8];
      int to[kStageBatch];   // LDS byte offset of the unit's first pixel, or -1
      bool st0[kStageBatch], st1[kStageBatch];
#pragma unroll
      for (int b = 0; b < kStageBatch; ++b) {
        const int u = u0 + b * kThreads;
        const bool live = u < units;
        const int uc = live ? u : 0;
        const int j = uc % pairs, rest = uc / pairs;
        const int cg = rest % cgroups, hy = rest / cgroups;
        const int iy = iy0 + hy, ix = 2 * (jlo + j);
        // (W is even: a pair lies inside its row or outside it as a whole, and its dword is aligned)
        const bool inside = live && iy >= 0 && iy < a.H && ix >= 0 && ix < a.W;
        const _Float16* src = xn + (static_cast<size_t>(cg * 8) * plane + static_cast<size_t>(inside ? iy : 0) * a.W + (inside ? ix : 0));
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          const uint32_t v = *reinterpret_cast<const uint32_t*>(src + c * plane);  // (the address is selected, not the load)
          d[b][c] = inside ? v : 0u;
        }
        const int hx = ix + a.pad_l;
        to[b] = ((hy * a.halo_w + hx) * a.pix_stride) + cg * 16;
        st0[b] = live && hx >= 0 && hx < a.halo_w;
        st1[b] = live && hx + 1 >= 0 && hx + 1 < a.halo_w;
      }
#pragma unroll
      for (int b = 0; b < kStageBatch; ++b) {
        // low halves: the pixel at ix, high halves: at ix + 1
        v4i lo, hi;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          lo[q] = static_cast<int>(__builtin_amdgcn_perm(d[b][2 * q + 1], d[b][2 * q], 0x05040100));
          hi[q] = static_cast<int>(__builtin_amdgcn_perm(d[b][2 * q + 1], d[b][2 * q], 0x07060302));
        }
        if (st0[b]) *reinterpret_cast<v4i*>(lds + to[b]) = lo;
        if (st1[b]) *reinterpret_cast<v4i*>(lds + to[b] + a.pix_stride) = hi;
      }
    }
  }
  __syncthreads();

  // ---- multiply: activations x weights; a round = one tap x CSB channel steps, the next round's fragments requested
  // before this round is multiplied ----
  const int row = lane & 31, kg = lane >> 5;  // pixel of a tile / output channel of a tile; eight-channel half of a step
  const uint8_t* xb[PT];
#pragma unroll
  for (int t = 0; t < PT; ++t) {
    const int p = min(p0 + (wave * PT + t) * 32 + row, hw - 1);  // (pixels past the image's end repeat the last one and are not stored)
    const int oy = p / a.OW, ox = p - oy * a.OW;
    xb[t] = lds + (static_cast<size_t>((oy - y0) * a.s) * a.halo_w + ox * a.s) * a.pix_stride + kg * 16;
  }
  const v4i* wp = a.wpk + static_cast<size_t>(blockIdx.y) * (a.kh * a.kw) * a.csteps * OT * 64 + lane;
  const int cblocks = (a.csteps + CSB - 1) / CSB;
  const int rounds = a.kh * a.kw * cblocks;
  auto fetch = [&](int r, v4i (&fx)[PT][CSB], v4i (&fw)[CSB][OT]) {
    const int tap = r / cblocks, cb = r - tap * cblocks;
    const int ky = tap / a.kw, kx = tap - ky * a.kw;
    const size_t x_at = (static_cast<size_t>(ky) * a.halo_w + kx) * a.pix_stride;
    const v4i* wt = wp + static_cast<size_t>(tap) * a.csteps * OT * 64;
#pragma unroll
    for (int cs = 0; cs < CSB; ++cs) {
      const int c = min(cb * CSB + cs, a.csteps - 1);  // (past the end: the last step once more, not multiplied)
#pragma unroll
      for (int t = 0; t < PT; ++t) fx[t][cs] = *reinterpret_cast<const v4i*>(xb[t] + x_at + c * 32);
#pragma unroll
      for (int t = 0; t < OT; ++t) fw[cs][t] = wt[(c * OT + t) * 64];
    }
  };
  v16f acc[PT][OT];
#pragma unroll
  for (int t = 0; t < PT; ++t)
#pragma unroll
    for (int o = 0; o < OT; ++o)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[t][o][i] = 0.f;
  auto multiply = [&](int r, const v4i (&fx)[PT][CSB], const v4i (&fw)[CSB][OT]) {
    const int cb = r % cblocks;
#pragma unroll
    for (int cs = 0; cs < CSB; ++cs) {
      if (cb * CSB + cs < a.csteps) {  // uniform
#pragma unroll
        for (int t = 0; t < PT; ++t)
#pragma unroll
          for (int o = 0; o < OT; ++o)
            acc[t][o] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, fx[t][cs]), __builtin_bit_cast(v8h, fw[cs][o]), acc[t][o], 0, 0, 0);
      }
    }
  };
  v4i fxa[PT][CSB], fwa[CSB][OT], fxb[PT][CSB], fwb[CSB][OT];
  fetch(0, fxa, fwa);
  for (int r = 0; r < rounds; r += 2) {
    fetch(min(r + 1, rounds - 1), fxb, fwb);
    multiply(r, fxa, fwa);
    fetch(min(r + 2, rounds - 1), fxa, fwa);
    if (r + 1 < rounds) multiply(r + 1, fxb, fwb);
  }

  // ---- a lane holds output channel `row` of each tile and, per accumulator quad g, pixels 8 g + 4 kg + 0 .. 3 of a pixel
  // tile: behind two swaps between the wavefront's halves a lower lane holds pixels 0 .. 15, its partner 16 .. 31 ----
#pragma unroll
  for (int o = 0; o < OT; ++o) {
    const int oc = (blockIdx.y * OT + o) * 32 + row;
    const bool live = oc < a.OC;
    const float b = live && a.bias ? a.bias[oc] : 0.f;
    _Float16* yp = a.y + (static_cast<size_t>(n) * a.OC + (live ? oc : 0)) * hw;
#pragma unroll
    for (int t = 0; t < PT; ++t) {
      uint32_t q[4][2];  // quad g: four pixels as two dwords
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        _Float16 h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float v = acc[t][o][4 * g + e] + b;
          if (a.act == TVX_ACT_RELU || a.act == TVX_ACT_RELU6) v = v < 0.f ? 0.f : v;
          if (a.act == TVX_ACT_RELU6) v = v > 6.f ? 6.f : v;
          h[e] = static_cast<_Float16>(v);
        }
        __builtin_memcpy(q[g], h, 8);
      }
      // quads of the lower half: pixels 0-3, 8-11, 16-19, 24-27; of the upper half: 4-7, 12-15, 20-23, 28-31
      uint32_t run[8];  // sixteen consecutive pixels
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const auto s02 = __builtin_amdgcn_permlane32_swap(q[0][d], q[2][d], false, false);
        const auto s13 = __builtin_amdgcn_permlane32_swap(q[1][d], q[3][d], false, false);
        run[d] = s02[0]; run[2 + d] = s02[1]; run[4 + d] = s13[0]; run[6 + d] = s13[1];
      }
      const int pp = p0 + (wave * PT + t) * 32 + 16 * kg;
      if (!live) continue;
      if (a.aligned4) {  // (runs of four pixels lie inside the image or outside it as a whole)
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (pp + 4 * k < hw) *reinterpret_cast<uint2*>(yp + pp + 4 * k) = uint2{run[2 * k], run[2 * k + 1]};
      } else {
#pragma unroll
        for (int k = 0; k < 16; ++k)
          if (pp + k < hw) yp[pp + k] = __builtin_bit_cast(_Float16, static_cast<uint16_t>(run[k >> 1] >> (16 * (k & 1))));
      }
    }
  }
}

typedef void (*FcvFn)(FcvArgs);
FcvFn KernelOf(int ot, int pt, int csteps) {
  if (csteps <= 2) {
    if (pt == 1) return ot == 1 ? ConvIgemmF16Kernel<1, 1, 2> : ConvIgemmF16Kernel<2, 1, 2>;
    return ot == 1 ? ConvIgemmF16Kernel<1, 2, 2> : ConvIgemmF16Kernel<2, 2, 2>;
  }
  if (pt == 1) return ot == 1 ? ConvIgemmF16Kernel<1, 1, 4> : ConvIgemmF16Kernel<2, 1, 4>;
  return ot == 1 ? ConvIgemmF16Kernel<1, 2, 4> : ConvIgemmF16Kernel<2, 2, 4>;
}

struct Plan {
  FcvArgs a;
  int ot, pt;
  dim3 grid;
  unsigned lds_bytes;
};

int ConvIgemmF16Run(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  FcvArgs a = plan->a;
  a.x = static_cast<const _Float16*>(in0);
  a.y = static_cast<_Float16*>(out);
  if (reinterpret_cast<uintptr_t>(in0) & 3) return SetError(TVX_E_INVALID, "conv2d_igemm_f16: the input must be 4-byte aligned");
  if (reinterpret_cast<uintptr_t>(out) & (a.aligned4 ? 7 : 1)) {
    if (reinterpret_cast<uintptr_t>(out) & 1) return SetError(TVX_E_INVALID, "conv2d_igemm_f16: the result must be 2-byte aligned");
    a.aligned4 = 0;
  }
  hipLaunchKernelGGL(KernelOf(plan->ot, plan->pt, a.csteps), plan->grid, dim3(kThreads), plan->lds_bytes, st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

}  // namespace

// Claims dense float16 convolutions (one group, dilation 1, one stride for both axes, constant weights) whose input
// rows are whole dwords (even width) and whose channels are a multiple of 16, at most 128, where the halo rows of 128
// output pixels fit LDS. Declines (TVX_E_UNSUPPORTED) the rest: conv2d_gemm_f16 takes it.
int ConvIgemmF16Setup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (d->in_dtype != TVX_F16 || d->w_dtype != TVX_F16 || d->out_dtype != TVX_F16 || !w_host) return TVX_E_UNSUPPORTED;
  if (d->multiplier != 0 || d->groups > 1 || d->dilation_w != 1 || d->dilation_h != 1) return TVX_E_UNSUPPORTED;
  if (d->stride_w != d->stride_h || d->stride_w > 4) return TVX_E_UNSUPPORTED;
  if (d->in_c % 16 || d->in_c > 16 * kMaxSteps || (d->in_w & 1) || d->k_w > 11 || d->k_h > 11) return TVX_E_UNSUPPORTED;
  if (const char* f = getenv("TVX_NO_CONV_IGEMM_F16"))  // tuning aid: leaves float16 convolutions to conv2d_gemm_f16
    if (atoi(f)) return TVX_E_UNSUPPORTED;
  Plan plan{};
  FcvArgs& a = plan.a;
  a.C = d->in_c; a.H = d->in_h; a.W = d->in_w; a.OC = d->out_c; a.OH = d->out_h; a.OW = d->out_w;
  a.kh = d->k_h; a.kw = d->k_w; a.s = d->stride_w; a.pad_t = d->pad_top; a.pad_l = d->pad_left;
  a.csteps = a.C / 16;
  a.halo_w = (a.OW - 1) * a.s + a.kw;
  a.pix_stride = 2 * a.C + 16;
  a.act = d->activation;
  const int64_t hw = static_cast<int64_t>(a.OH) * a.OW;
  a.aligned4 = hw % 4 == 0;
  // 256-pixel workgroups (two pixel tiles a wavefront: every weight fragment multiplies twice) where that still leaves
  // two workgroups per CU and the rows behind them fit LDS
  int cus = 256;
  {
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
  }
  auto lds_of = [&](int pt) {
    const int rows = static_cast<int>(std::min<int64_t>(a.OH, (kPixels * pt + a.OW - 2) / a.OW + 1));  // most output rows the pixels of a tile touch
    return (static_cast<int64_t>(rows - 1) * a.s + a.kh) * a.halo_w * a.pix_stride;
  };
  plan.pt = 1;
  if (lds_of(2) <= 80 * 1024 && static_cast<int64_t>(d->batch) * ((hw + 2 * kPixels - 1) / (2 * kPixels)) * ((a.OC + 63) / 64) >= cus) plan.pt = 2;
  if (const char* f = getenv("TVX_CONV_F16_PIXEL_TILES")) if (atoi(f) == 1 || (atoi(f) == 2 && lds_of(2) <= 80 * 1024)) plan.pt = atoi(f);  // test lever
  a.tiles_per_image = static_cast<int>((hw + kPixels * plan.pt - 1) / (kPixels * plan.pt));
  const int64_t lds = lds_of(plan.pt);
  if (lds > 80 * 1024) return TVX_E_UNSUPPORTED;
  plan.lds_bytes = static_cast<unsigned>(lds);
  const uint64_t in_elems = static_cast<uint64_t>(d->batch) * a.C * a.H * a.W, out_elems = static_cast<uint64_t>(d->batch) * a.OC * hw;
  if (std::max(in_elems, out_elems) >= (1ull << 31)) return TVX_E_UNSUPPORTED;
  const int oc_tiles = (a.OC + 31) / 32;
  plan.ot = oc_tiles >= 2 ? 2 : 1;
  const int groups = (oc_tiles + plan.ot - 1) / plan.ot;
  const uint64_t grid_x = static_cast<uint64_t>(d->batch) * a.tiles_per_image;
  if (grid_x > 0x7fffffffull || groups > 65535) return TVX_E_UNSUPPORTED;
  plan.grid = dim3(static_cast<unsigned>(grid_x), groups);
  // weights {kw, kh, C, OC} (kw fastest) -> [tile group][tap][channel step][tile][lane]: lane = (eight-channel half, output channel)
  const int taps = a.kh * a.kw;
  std::vector<uint16_t> packed(static_cast<size_t>(groups) * taps * a.csteps * plan.ot * 64 * 8, 0);
  const uint16_t* src = static_cast<const uint16_t*>(w_host);
  for (int oc = 0; oc < a.OC; ++oc)
    for (int c = 0; c < a.C; ++c)
      for (int t = 0; t < taps; ++t) {
        const uint16_t v = src[(static_cast<size_t>(oc) * a.C + c) * taps + t];
        const int grp = (oc / 32) / plan.ot, tl = (oc / 32) % plan.ot, cs = c / 16, kg = (c % 16) / 8, j = c % 8;
        const size_t lane = static_cast<size_t>(kg) * 32 + oc % 32;
        packed[((((static_cast<size_t>(grp) * taps + t) * a.csteps + cs) * plan.ot + tl) * 64 + lane) * 8 + j] = v;
      }
  int s = op->packed.Upload(packed.data(), packed.size() * 2);
  if (s == TVX_OK && bias_host) s = op->bias.Upload(bias_host, static_cast<size_t>(a.OC) * 4);
  if (s != TVX_OK) return s;
  a.wpk = op->packed.as<v4i>();
  a.bias = bias_host ? op->bias.as<float>() : nullptr;
  if (plan.lds_bytes > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(KernelOf(plan.ot, plan.pt, a.csteps)),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(plan.lds_bytes));
    if (e != hipSuccess) return SetError(TVX_E_DEVICE, "hipFuncSetAttribute(dynamic LDS %u): %s", plan.lds_bytes, hipGetErrorString(e));
  }
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = ConvIgemmF16Run;
  op->kernel_name = "conv2d_igemm_f16";
  return TVX_OK;
}

}  // namespace tvx
