// Quantized 1x1 and depthwise 3x3 convolutions and the global average pooling on a channel-blocked layout for small
// planes: stands in for vxConvolutionLayer / vxPoolingLayer2 as src/tim/vx/internal/src/kernel/vx/convolutional.c:504-582
// and src/tim/vx/internal/src/ops/vsi_nn_op_pool.c:144-150 call them, where the runtime keeps a TRANSIENT tensor - whose
// bytes no host code ever sees - in an order of its own.
//
// WHCN planes of 7 x 7 pixels are 49-byte rows: no load of a pointwise convolution over them is aligned, every operand
// fragment of the matrix cores is sixteen bytes gathered from sixteen planes. The blocked order is
//   byte ((c / 16) * P + p) * 16 + c % 16,   p = n * H * W + y * W + x,   P = N * H * W
// (sixteen channels of a pixel side by side, pixels of the whole batch in a row, 16-channel blocks outermost): the sixteen
// reduction bytes a lane feeds to v_mfma_i32_32x32x32_i8 are one aligned 16-byte load, 32 lanes of a fragment read 512
// contiguous bytes, and nothing goes through LDS on the way in. With the weights as the A operand (packed in fragment
// order when the operator is created) a lane ends up with one pixel and, after two swaps between the wavefront's
// halves, sixteen consecutive output channels of it: one aligned 16-byte store into the blocked result.
//
//   pointwise   a wavefront owns 32 pixels x OCT 32-channel tiles; the four wavefronts of a workgroup either take four
//               pixel tiles (short reductions into many channels: the expansions) or split the reduction of one pixel
//               tile four ways and add up in LDS (long reductions into few channels: the projections). Operand
//               fragments of a batch of k-steps are requested together, straight from global memory.
//   depthwise   a lane owns one pixel and sixteen channels: nine aligned 16-byte loads (neighbouring pixels are
//               neighbouring 16-byte units), taps outside the image replaced by the input zero point; the three
//               bytes of a kernel row are brought side by side per channel (two v_perm) and meet the row's packed
//               weights in one v_dot4.
//   average     a lane owns one image and sixteen channels and adds up the plane's pixels, two bytes at a time in
//               16-bit halves.
// Zero points and requantization are those of the WHCN kernels (pwconv_i8.hip, dwconv3x3_i8.hip, kernels_generic.hip).
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;

// ---- WHCN planes <-> blocked ------------------------------------------------------------------------------------
struct LayoutArgs {
  const uint8_t* x;
  uint8_t* y;
  int HW, C, P;        // pixels of a plane, channels (a multiple of 16), pixels of the batch
  int to_blocked;
};

__global__ void __launch_bounds__(kThreads) LayoutKernel(LayoutArgs a) {
  // a thread owns one pixel of one 16-channel block: sixteen strided bytes on the planes' side, one 16-byte unit on the
  // blocked side
  const int p = blockIdx.x * kThreads + threadIdx.x;
  const int block = blockIdx.y;
  if (p >= a.P) return;
  const int n = p / a.HW, q = p - n * a.HW;
  const size_t plane0 = (static_cast<size_t>(n) * a.C + block * 16) * a.HW + q;
  const size_t unit = (static_cast<size_t>(block) * a.P + p) * 16;
  if (a.to_blocked) {
    uint32_t d[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 16; ++j) d[j >> 2] |= static_cast<uint32_t>(a.x[plane0 + static_cast<size_t>(j) * a.HW]) << (8 * (j & 3));
    *reinterpret_cast<v4i*>(a.y + unit) = v4i{static_cast<int>(d[0]), static_cast<int>(d[1]), static_cast<int>(d[2]), static_cast<int>(d[3])};
  } else {
    const v4i v = *reinterpret_cast<const v4i*>(a.x + unit);
#pragma unroll
    for (int j = 0; j < 16; ++j) a.y[plane0 + static_cast<size_t>(j) * a.HW] = static_cast<uint8_t>(static_cast<uint32_t>(v[j >> 2]) >> (8 * (j & 3)));
  }
}

// ---- pointwise ---------------------------------------------------------------------------------------------------
struct BpArgs {
  const uint8_t* x;
  uint8_t* y;
  const uint8_t* res;    // fused residual Add: the other operand, blocked like the result
  const v4i* wpk;        // [oc tile][k-step][lane]: 16 reduction bytes of channel tile * 32 + lane % 32 (pwconv_i8.hip's order)
  const int32_t* biasf;  // bias + per-channel zero-point terms
  const tvx_v4i* rq;     // per channel requantization record
  int P, C, OC;          // pixels of the batch, input channels (a multiple of 32), output channels (a multiple of 32)
  int ksteps;            // C / 32
  int xor_mask;          // 0x80808080 for uint8 activations
  int neg_zws4;          // -(weight zero point, int8 domain) in all four bytes
  int out_zp, lo, hi;
  int uni;               // one requantization record for every channel (per-tensor quantization): `u`, no record loads
  tvx_v4i u;
  // the fused Add, as in pwconv_i8.hip (add_mode 0 = off, 1: a = convolution, b = residual, 2: the other way round)
  int add_mode, add_signed, add_za, add_zb, add_zo, add_lo, add_hi;
  double add_ra, add_rb;
};

// OCT: 32-channel output tiles of a wavefront; KS: 1 = the workgroup's wavefronts take four pixel tiles, 4 = they split
// one pixel tile's reduction; BATCH: k-steps whose fragments are requested together; ZP: uniform weight zero point
template <int RQ, bool ZP, int OCT, int KS, int BATCH, bool ADD>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) BlockedPwKernel(BpArgs a) {
  __shared__ int red[KS == 4 ? 3 * OCT * 16 * 64 : 1];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n = lane & 31, h = lane >> 5;  // pixel inside the tile; which sixteen of a k-step's 32 channels
  const int pt = KS == 1 ? blockIdx.x * 4 + wave : blockIdx.x;
  const int p0 = pt * 32;
  if (KS == 1 && p0 >= a.P) return;  // (KS == 4: the workgroup's barrier needs everyone)
  const int p = min(p0 + n, a.P - 1);  // (pixels past the end repeat the last one and are dropped)
  const int tile0 = blockIdx.y * OCT;
  // this wavefront's k-steps: all of them, or every fourth
  const int ks0 = KS == 1 ? 0 : wave, ks_step = KS;
  const uint8_t* xp = a.x + (static_cast<size_t>(h) * a.P + p) * 16;
  const size_t x_step = static_cast<size_t>(a.P) * 32;  // a k-step is two 16-channel blocks
  const v4i* wp = a.wpk + static_cast<size_t>(tile0) * a.ksteps * 64 + lane;
  const v4i fz = {a.neg_zws4, a.neg_zws4, a.neg_zws4, a.neg_zws4};

  v16i acc[OCT];
#pragma unroll
  for (int j = 0; j < OCT; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0;
  for (int kb = ks0; kb < a.ksteps; kb += ks_step * BATCH) {
    v4i fx[BATCH], fw[BATCH][OCT];
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const int ks = min(kb + b * ks_step, a.ksteps - 1);  // (past the end: the last k-step once more, not multiplied)
      fx[b] = *reinterpret_cast<const v4i*>(xp + ks * x_step);
#pragma unroll
      for (int j = 0; j < OCT; ++j) fw[b][j] = wp[(static_cast<size_t>(j) * a.ksteps + ks) * 64];
    }
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      if (kb + b * ks_step < a.ksteps) {  // uniform
#pragma unroll
        for (int i = 0; i < 4; ++i) fx[b][i] ^= a.xor_mask;
#pragma unroll
        for (int j = 0; j < OCT; ++j) {
          acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[b][j], fx[b], acc[j], 0, 0, 0);
          if (ZP) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fz, fx[b], acc[j], 0, 0, 0);
        }
      }
    }
  }
  if constexpr (KS == 4) {
    // partial sums meet in LDS; the first wavefront goes on alone
    if (wave != 0) {
#pragma unroll
      for (int j = 0; j < OCT; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) red[(((wave - 1) * OCT + j) * 16 + i) * 64 + lane] = acc[j][i];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
      for (int j = 0; j < OCT; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[j][i] += red[((w * OCT + j) * 16 + i) * 64 + lane];
  }
  // ---- epilogue: a lane holds pixel n and, per accumulator quad g, channels 8 g + 4 h + 0 .. 3 of each tile ----
#pragma unroll
  for (int j = 0; j < OCT; ++j) {
    const int tile = tile0 + j;
    if (tile * 32 >= a.OC) break;  // uniform
    uint32_t quad[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int oc = tile * 32 + 8 * g + 4 * h;
      const v4i b4 = *reinterpret_cast<const v4i*>(a.biasf + oc);
      if (a.uni) {  // (uniform)
        const int v4[4] = {acc[j][4 * g] + b4[0], acc[j][4 * g + 1] + b4[1], acc[j][4 * g + 2] + b4[2], acc[j][4 * g + 3] + b4[3]};
        quad[g] = RequantPack4<RQ>(v4, a.u, a.out_zp, a.lo, a.hi);
      } else {
        int r4[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) r4[e] = Requant8<RQ>(acc[j][4 * g + e] + b4[e], a.rq[oc + e], a.out_zp, a.lo, a.hi);
        quad[g] = PackBytes(r4[0], r4[1], r4[2], r4[3]);
      }
    }
    // quad g of the lower half: channels 8 g .. 8 g + 3, of the upper half: 8 g + 4 .. 8 g + 7. Behind the swaps a lower
    // lane holds channels 0 .. 15 of the tile, its partner in the upper half channels 16 .. 31: one blocked unit each.
    const auto s02 = __builtin_amdgcn_permlane32_swap(quad[0], quad[2], false, false);
    const auto s13 = __builtin_amdgcn_permlane32_swap(quad[1], quad[3], false, false);
    uint32_t unit[4] = {s02[0], s02[1], s13[0], s13[1]};
    if (p0 + n < a.P) {
      const size_t at = (static_cast<size_t>(tile * 2 + h) * a.P + p) * 16;
      if (ADD) {
        const v4i r = *reinterpret_cast<const v4i*>(a.res + at);
#pragma unroll
        for (int i = 0; i < 4; ++i) unit[i] = AddResidual4(a, unit[i], static_cast<uint32_t>(r[i]));
      }
      *reinterpret_cast<v4i*>(a.y + at) = v4i{static_cast<int>(unit[0]), static_cast<int>(unit[1]), static_cast<int>(unit[2]), static_cast<int>(unit[3])};
    }
  }
}

// ---- depthwise 3x3, stride 1 ---------------------------------------------------------------------------------------
struct BdArgs {
  const uint8_t* x;
  uint8_t* y;
  const v4i* wpk;        // per channel: kernel row ky = bytes (w[ky][0], w[ky][1], w[ky][2], 0) int8 for ky = 0 .. 2, then the window-sum flag
  const int32_t* biasf;
  const tvx_v4i* rq;
  int P, C, H, W, OH, OW, PO;  // input pixels of the batch, channels, plane extents; output pixels of the batch
  int pad_t, pad_l;
  int xor_mask, pad_fill, zws, out_zp, lo, hi;
};

// BOX: the weights are not shifted by their zero point (they would not fit int8): the window sum carries that term
template <int RQ, bool BOX>
__global__ void __launch_bounds__(kThreads) BlockedDwKernel(BdArgs a) {
  const int po = blockIdx.x * kThreads + threadIdx.x;  // output pixel of the batch
  const int block = blockIdx.y;
  if (po >= a.PO) return;
  const int ohw = a.OH * a.OW;
  const int n = po / ohw, q = po - n * ohw;
  const int oy = q / a.OW, ox = q - oy * a.OW;
  const int iy0 = oy - a.pad_t, ix0 = ox - a.pad_l;
  const int base = n * (a.H * a.W);
  const uint8_t* xb = a.x + static_cast<size_t>(block) * a.P * 16;
  v4i tap[3][3];
#pragma unroll
  for (int ky = 0; ky < 3; ++ky)
#pragma unroll
    for (int kx = 0; kx < 3; ++kx) {
      const int iy = iy0 + ky, ix = ix0 + kx;
      const bool inside = iy >= 0 && iy < a.H && ix >= 0 && ix < a.W;
      const int at = inside ? base + iy * a.W + ix : base;  // (a tap outside the image reads a pixel that exists and is replaced)
      const v4i v = *reinterpret_cast<const v4i*>(xb + static_cast<size_t>(at) * 16);
#pragma unroll
      for (int i = 0; i < 4; ++i) tap[ky][kx][i] = inside ? (v[i] ^ a.xor_mask) : a.pad_fill;
    }
  uint32_t out[4];
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {  // four channels at a time: dword qd of every tap
    int r4[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int c = block * 16 + qd * 4 + e;
      const v4i k = a.wpk[c];
      int acc = a.biasf[c], sx = 0;
#pragma unroll
      for (int ky = 0; ky < 3; ++ky) {
        // bytes e of the row's three taps side by side: (t0, t1, t2, 0)
        const uint32_t t01 = __builtin_amdgcn_perm(static_cast<uint32_t>(tap[ky][1][qd]), static_cast<uint32_t>(tap[ky][0][qd]), 0x0c0c0400u + 0x0101u * e);
        const uint32_t row = __builtin_amdgcn_perm(static_cast<uint32_t>(tap[ky][2][qd]), t01, 0x0c040100u + (static_cast<uint32_t>(e) << 16));
        acc = __builtin_amdgcn_sdot4(static_cast<int>(row), k[ky], acc, false);
        if (BOX) sx = __builtin_amdgcn_sdot4(static_cast<int>(row), 0x00010101, sx, false);
      }
      if (BOX) acc -= a.zws * sx;
      r4[e] = Requant8<RQ>(acc, a.rq[c], a.out_zp, a.lo, a.hi);
    }
    out[qd] = PackBytes(r4[0], r4[1], r4[2], r4[3]);
  }
  *reinterpret_cast<v4i*>(a.y + (static_cast<size_t>(block) * a.PO + po) * 16) =
      v4i{static_cast<int>(out[0]), static_cast<int>(out[1]), static_cast<int>(out[2]), static_cast<int>(out[3])};
}

// ---- global average pooling: blocked in, one code per (image, channel) out ----------------------------------------
struct BaArgs {
  const uint8_t* x;
  uint8_t* y;            // [N][C]
  int HW, C, N, P;
  int is_signed, in_zp, out_zp, qmin, qmax;
  double ratio;          // in_scale / out_scale
};

__global__ void __launch_bounds__(kThreads) BlockedAvgKernel(BaArgs a) {
  // eight lanes share one (image, 16-channel block): every eighth pixel each, then three steps of a butterfly
  const int t = (blockIdx.x * kThreads + threadIdx.x) >> 3, part = threadIdx.x & 7;
  const int blocks = a.C / 16;
  const bool live = t < a.N * blocks;
  const int tc = live ? t : 0;
  const int n = tc / blocks, block = tc - n * blocks;
  const uint8_t* xp = a.x + (static_cast<size_t>(block) * a.P + static_cast<size_t>(n) * a.HW) * 16;
  // sums of bytes 0 / 2 and of bytes 1 / 3 of each dword in 16-bit halves (a plane has at most 256 pixels);
  // signed codes are added up as unsigned ones with the sign bit flipped
  uint32_t ev[4] = {0, 0, 0, 0}, od[4] = {0, 0, 0, 0};
  const uint32_t flip = a.is_signed ? 0x80808080u : 0u;
  for (int q = part; q < a.HW; q += 8) {
    const v4i v = *reinterpret_cast<const v4i*>(xp + static_cast<size_t>(q) * 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t d = static_cast<uint32_t>(v[i]) ^ flip;
      ev[i] += d & 0x00ff00ffu;
      od[i] += (d >> 8) & 0x00ff00ffu;
    }
  }
#pragma unroll
  for (int o = 1; o < 8; o <<= 1)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ev[i] += __shfl_xor(ev[i], o, 64);
      od[i] += __shfl_xor(od[i], o, 64);
    }
  if (!live || part >= 4) return;
  // lane `part` of the eight finishes dword `part`: channels 4 part .. 4 part + 3
  const uint32_t e = part == 0 ? ev[0] : (part == 1 ? ev[1] : (part == 2 ? ev[2] : ev[3]));
  const uint32_t o = part == 0 ? od[0] : (part == 1 ? od[1] : (part == 2 ? od[2] : od[3]));
  const int s4[4] = {static_cast<int>(e & 0xffff), static_cast<int>(o & 0xffff), static_cast<int>(e >> 16), static_cast<int>(o >> 16)};
  int r4[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int64_t sum = static_cast<int64_t>(s4[k]) - (a.is_signed ? 128ll * a.HW : 0ll);
    const int64_t total = sum - static_cast<int64_t>(a.HW) * a.in_zp;
    int64_t r = static_cast<int64_t>(rint(static_cast<double>(total) * a.ratio / static_cast<double>(a.HW)));
    r += a.out_zp;
    r4[k] = static_cast<int>(r < a.qmin ? a.qmin : (r > a.qmax ? a.qmax : r));
  }
  *reinterpret_cast<uint32_t*>(a.y + static_cast<size_t>(n) * a.C + block * 16 + part * 4) = PackBytes(r4[0], r4[1], r4[2], r4[3]);
}

// ---- host side -----------------------------------------------------------------------------------------------------
struct PwPlan {
  BpArgs a;
  int rq, zp, form;  // form 0: four pixel tiles per workgroup; 1: the reduction split over the workgroup, one channel tile
  int oct;           // form 0: 32-channel tiles of a wavefront (1, 2 or 4)
  dim3 grid;
};

template <int RQ, bool ZP, bool ADD>
void LaunchPwForm(const PwPlan* p, const BpArgs& a, hipStream_t st) {
  if (p->form == 1) hipLaunchKernelGGL((BlockedPwKernel<RQ, ZP, 1, 4, 8, ADD>), p->grid, dim3(kThreads), 0, st, a);
  else if (p->oct == 4) hipLaunchKernelGGL((BlockedPwKernel<RQ, ZP, 4, 1, 4, ADD>), p->grid, dim3(kThreads), 0, st, a);
  else if (p->oct == 2) hipLaunchKernelGGL((BlockedPwKernel<RQ, ZP, 2, 1, 8, ADD>), p->grid, dim3(kThreads), 0, st, a);
  else hipLaunchKernelGGL((BlockedPwKernel<RQ, ZP, 1, 1, 8, ADD>), p->grid, dim3(kThreads), 0, st, a);
}
template <int RQ, bool ZP>
void LaunchPwAdd(const PwPlan* p, const BpArgs& a, hipStream_t st) {
  if (a.add_mode) LaunchPwForm<RQ, ZP, true>(p, a, st);
  else LaunchPwForm<RQ, ZP, false>(p, a, st);
}
template <int RQ>
void LaunchPwZp(const PwPlan* p, const BpArgs& a, hipStream_t st) {
  if (p->zp) LaunchPwAdd<RQ, true>(p, a, st);
  else LaunchPwAdd<RQ, false>(p, a, st);
}

int BlockedPwRun(tvx_op* op, const void* in0, const void* in1, void* out, hipStream_t st) {
  const PwPlan* p = reinterpret_cast<const PwPlan*>(op->host_blob.data());
  BpArgs a = p->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  a.res = static_cast<const uint8_t*>(in1);
  if (a.add_mode && !in1) return SetError(TVX_E_INVALID, "pwconv_blocked_i8: the fused Add needs its second operand as in1");
  if ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(in1)) & 15)
    return SetError(TVX_E_INVALID, "pwconv_blocked_i8: blocked tensors must be 16-byte aligned");
  if (p->rq == kRqFastNoTie) LaunchPwZp<kRqFastNoTie>(p, a, st);
  else if (p->rq == kRqFast) LaunchPwZp<kRqFast>(p, a, st);
  else LaunchPwZp<kRqGeneric>(p, a, st);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

struct DwPlan {
  BdArgs a;
  int rq, box;
  dim3 grid;
};

int BlockedDwRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const DwPlan* p = reinterpret_cast<const DwPlan*>(op->host_blob.data());
  BdArgs a = p->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(out)) & 15)
    return SetError(TVX_E_INVALID, "dwconv3x3_blocked_i8: blocked tensors must be 16-byte aligned");
  const dim3 block(kThreads);
#define TVX_LAUNCH_DW(RQ) \
  if (p->box) hipLaunchKernelGGL((BlockedDwKernel<RQ, true>), p->grid, block, 0, st, a); \
  else hipLaunchKernelGGL((BlockedDwKernel<RQ, false>), p->grid, block, 0, st, a)
  if (p->rq == kRqFastNoTie) { TVX_LAUNCH_DW(kRqFastNoTie); }
  else if (p->rq == kRqFast) { TVX_LAUNCH_DW(kRqFast); }
  else { TVX_LAUNCH_DW(kRqGeneric); }
#undef TVX_LAUNCH_DW
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

struct AvgPlan {
  BaArgs a;
  dim3 grid;
};

int BlockedAvgRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const AvgPlan* p = reinterpret_cast<const AvgPlan*>(op->host_blob.data());
  BaArgs a = p->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if ((reinterpret_cast<uintptr_t>(in0) & 15) || (reinterpret_cast<uintptr_t>(out) & 3))
    return SetError(TVX_E_INVALID, "avgpool_blocked_i8: the blocked tensor must be 16-byte, the result 4-byte aligned");
  hipLaunchKernelGGL(BlockedAvgKernel, p->grid, dim3(kThreads), 0, st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

struct LayoutPlan {
  LayoutArgs a;
  dim3 grid;
};

int LayoutRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const LayoutPlan* p = reinterpret_cast<const LayoutPlan*>(op->host_blob.data());
  LayoutArgs a = p->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if (reinterpret_cast<uintptr_t>(a.to_blocked ? out : in0) & 15)
    return SetError(TVX_E_INVALID, "layout_blocked: the blocked tensor must be 16-byte aligned");
  hipLaunchKernelGGL(LayoutKernel, p->grid, dim3(kThreads), 0, st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

}  // namespace

// Claims a quantized 1x1 / stride-1 / unpadded convolution with constant weights between blocked tensors: input and
// output channels multiples of 32. `op->fused_add` / `op->elt` carry a residual Add as for pwconv_i8.
int BlockedPwSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || d->multiplier != 0 || d->groups > 1) return TVX_E_UNSUPPORTED;
  if (d->k_w != 1 || d->k_h != 1 || d->stride_w != 1 || d->stride_h != 1 || d->pad_left || d->pad_top) return TVX_E_UNSUPPORTED;
  if (d->out_w != d->in_w || d->out_h != d->in_h || d->in_c % 32 || d->out_c % 32) return TVX_E_UNSUPPORTED;
  const uint64_t pixels = static_cast<uint64_t>(d->in_w) * d->in_h * d->batch;
  if (pixels * std::max(d->in_c, d->out_c) >= (1ull << 31)) return TVX_E_UNSUPPORTED;
  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127 || zws < -127 || zws > 127) return TVX_E_UNSUPPORTED;
  PwPlan plan{};
  BpArgs& a = plan.a;
  a.P = static_cast<int>(pixels); a.C = d->in_c; a.OC = d->out_c;
  a.ksteps = a.C / 32;
  a.xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.neg_zws4 = static_cast<int>(static_cast<uint32_t>((-zws) & 0xff) * 0x01010101u);
  a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  if (op->fused_add) {
    const tvx_eltwise_desc& e = op->elt;
    const double ra = static_cast<double>(e.a_scale) / static_cast<double>(e.out_scale);
    const double rb = static_cast<double>(e.b_scale) / static_cast<double>(e.out_scale);
    if (!(ra < 1048576.0) || !(rb < 1048576.0)) return TVX_E_UNSUPPORTED;
    a.add_mode = op->fused_add;
    a.add_signed = d->out_dtype == TVX_I8;
    a.add_ra = ra; a.add_rb = rb;
    a.add_za = e.a_zp; a.add_zb = e.b_zp; a.add_zo = e.out_zp;
    ActRange(d->out_dtype, e.out_scale, e.out_zp, TVX_ACT_NONE, &a.add_lo, &a.add_hi);
  }
  const int oc_tiles = a.OC / 32;
  std::vector<int8_t> packed(static_cast<size_t>(oc_tiles) * a.ksteps * 1024, 0);
  std::vector<int32_t> biasf(a.OC, 0);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  for (int oc = 0; oc < a.OC; ++oc) {
    int64_t sw = 0;
    for (int c = 0; c < a.C; ++c) {
      const uint8_t raw = src[static_cast<size_t>(oc) * a.C + c];
      const int8_t v = static_cast<int8_t>(w_u8 ? raw ^ 0x80 : raw);
      const int ks = c / 32, half = (c % 32) / 16, j = c % 16;
      packed[((static_cast<size_t>(oc / 32) * a.ksteps + ks) * 64 + half * 32 + oc % 32) * 16 + j] = v;
      sw += v;
    }
    const int64_t v = (b ? b[oc] : 0) - static_cast<int64_t>(zxs) * sw + static_cast<int64_t>(a.C) * zxs * zws;
    biasf[oc] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  std::vector<int32_t> rqt;
  plan.rq = BuildRequantRecords(op->h_mult, op->h_shift, a.OC, a.OC, d->out_zp, &rqt, AccumulatorBound(a.C, bias_host, a.OC));
  int s = op->packed.Upload(packed.data(), packed.size());
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s != TVX_OK) return s;
  a.wpk = op->packed.as<v4i>();
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<tvx_v4i>();
  a.uni = 1;
  for (int oc = 1; oc < a.OC; ++oc)
    if (std::memcmp(&rqt[4 * oc], &rqt[0], 16) != 0) a.uni = 0;
  a.u = tvx_v4i{rqt[0], rqt[1], rqt[2], rqt[3]};
  if (const char* f = getenv("TVX_BLOCKED_UNIFORM_RQ")) if (!atoi(f)) a.uni = 0;  // test lever: keeps the per-channel record loads
  plan.zp = zws != 0;
  // few output channels behind a long reduction: split the reduction over the workgroup; else four pixel tiles a workgroup
  const int pix_tiles = (a.P + 31) / 32;
  plan.form = (a.ksteps >= 12 && oc_tiles <= 12) ? 1 : 0;
  if (const char* f = getenv("TVX_BLOCKED_PW_FORM")) if (atoi(f) == 0 || atoi(f) == 1) plan.form = atoi(f);  // test lever
  // (channel tiles per wavefront: as many as still leave the chip two wavefronts per SIMD)
  plan.oct = static_cast<long long>(pix_tiles) * oc_tiles >= 4 * 2048 ? 4 : (static_cast<long long>(pix_tiles) * oc_tiles >= 2 * 2048 ? 2 : 1);
  if (const char* f = getenv("TVX_BLOCKED_PW_TILES")) if (atoi(f) == 1 || atoi(f) == 2 || atoi(f) == 4) plan.oct = atoi(f);  // test lever
  if (plan.form == 0) plan.grid = dim3((pix_tiles + 3) / 4, (oc_tiles + plan.oct - 1) / plan.oct);
  else plan.grid = dim3(pix_tiles, oc_tiles);
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = BlockedPwRun;
  op->kernel_name = op->fused_add ? "pwconv_add_blocked_i8" : "pwconv_blocked_i8";
  return TVX_OK;
}

// Claims a quantized depthwise 3x3 convolution (multiplier 1, stride 1, dilation 1, constant weights) between blocked
// tensors: channels a multiple of 16.
int BlockedDwSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || d->multiplier != 1) return TVX_E_UNSUPPORTED;
  if (d->k_w != 3 || d->k_h != 3 || d->dilation_w != 1 || d->dilation_h != 1 || d->stride_w != 1 || d->stride_h != 1) return TVX_E_UNSUPPORTED;
  if (d->in_c % 16 || d->out_c != d->in_c) return TVX_E_UNSUPPORTED;
  const uint64_t pin = static_cast<uint64_t>(d->in_w) * d->in_h * d->batch, pout = static_cast<uint64_t>(d->out_w) * d->out_h * d->batch;
  if (std::max(pin, pout) * d->in_c >= (1ull << 31)) return TVX_E_UNSUPPORTED;
  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127) return TVX_E_UNSUPPORTED;
  const int C = d->in_c;
  std::vector<int32_t> wpk, biasf;
  const bool box = PackDepthwise3x3(C, w_host, w_u8, bias_host, zxs, zws, true, &wpk, &biasf);
  std::vector<int32_t> rqt;
  DwPlan plan{};
  plan.rq = BuildRequantRecords(op->h_mult, op->h_shift, C, C, d->out_zp, &rqt, AccumulatorBound(9, bias_host, C));
  int s = op->packed.Upload(wpk.data(), wpk.size() * 4);
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s != TVX_OK) return s;
  BdArgs& a = plan.a;
  a.wpk = op->packed.as<v4i>();
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<tvx_v4i>();
  a.P = static_cast<int>(pin); a.PO = static_cast<int>(pout); a.C = C;
  a.H = d->in_h; a.W = d->in_w; a.OH = d->out_h; a.OW = d->out_w;
  a.pad_t = d->pad_top; a.pad_l = d->pad_left;
  a.xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.pad_fill = static_cast<int>(static_cast<uint32_t>(zxs & 0xff) * 0x01010101u);
  a.zws = zws; a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  plan.box = box ? 1 : 0;
  plan.grid = dim3((a.PO + kThreads - 1) / kThreads, C / 16);
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = BlockedDwRun;
  op->kernel_name = "dwconv3x3_blocked_i8";
  return TVX_OK;
}

// Claims a quantized average pooling over whole unpadded planes of a blocked tensor (channels a multiple of 16); the
// result, one pixel per plane, is written in WHCN order (byte n * C + c).
int BlockedAvgSetup(tvx_op* op) {
  const tvx_pool2d_desc& d = op->pool;
  const uint64_t hw = static_cast<uint64_t>(d.in_w) * d.in_h;
  if (!op->quantized || (d.pool_type != TVX_POOL_AVG && d.pool_type != TVX_POOL_AVG_ANDROID)) return TVX_E_UNSUPPORTED;
  if (d.k_w != d.in_w || d.k_h != d.in_h || d.pad_left || d.pad_top || d.out_w != 1 || d.out_h != 1) return TVX_E_UNSUPPORTED;
  if (hw > 256 || d.channels % 16 || hw * d.channels * d.batch >= (1ull << 31)) return TVX_E_UNSUPPORTED;
  AvgPlan plan{};
  BaArgs& a = plan.a;
  a.HW = static_cast<int>(hw); a.C = d.channels; a.N = d.batch; a.P = static_cast<int>(hw * d.batch);
  a.is_signed = d.dtype == TVX_I8;
  a.in_zp = d.in_zp; a.out_zp = d.out_zp;
  a.qmin = d.dtype == TVX_U8 ? 0 : -128; a.qmax = d.dtype == TVX_U8 ? 255 : 127;
  a.ratio = static_cast<double>(d.in_scale) / static_cast<double>(d.out_scale);
  const int threads = a.N * (a.C / 16) * 8;
  plan.grid = dim3((threads + kThreads - 1) / kThreads);
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = BlockedAvgRun;
  op->kernel_name = "avgpool_blocked_i8";
  return TVX_OK;
}

// WHCN planes -> blocked (to_blocked) or back: one-byte codes, channels a multiple of 16.
int LayoutSetup(tvx_op* op, uint32_t w, uint32_t h, uint32_t c, uint32_t n, int to_blocked) {
  const uint64_t hw = static_cast<uint64_t>(w) * h, pixels = hw * n;
  if (!hw || !c || !n || c % 16 || pixels * c >= (1ull << 31)) return TVX_E_UNSUPPORTED;
  LayoutPlan plan{};
  plan.a.HW = static_cast<int>(hw); plan.a.C = c; plan.a.P = static_cast<int>(pixels); plan.a.to_blocked = to_blocked;
  plan.grid = dim3((plan.a.P + kThreads - 1) / kThreads, c / 16);
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = LayoutRun;
  op->kernel_name = to_blocked ? "layout_to_blocked" : "layout_from_blocked";
  return TVX_OK;
}

}  // namespace tvx
