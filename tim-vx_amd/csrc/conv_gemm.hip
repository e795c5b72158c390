// conv2d_gemm_i8 / conv2d_gemm_f16: convolution as a GEMM over gathered windows, for the shapes the
// specialised kernels leave: grouped convolutions (groups other than 1 and C), dilated and strided ones of
// any channel count, and every float16 convolution. Replaces vxConvolutionLayer as ovxlib reaches it for
// those (reference: src/tim/vx/internal/src/ops/vsi_nn_op_conv2d.c:35-118, vsi_nn_op_grouped_conv2d.c).
//
// A workgroup owns 128 consecutive output pixels of one image and 32 or 64 output channels of one group.
// The reduction runs tap by tap (a tap's channels padded to whole half-chunks) in chunks of 64 bytes per pixel
// row: every thread gathers its share of half a chunk - 32 bytes per pixel of one tap's channel planes, by pixel
// quads where rows allow it (four pixels x 8 channels from 8 loads, transposed in registers), else by elements
// (one pixel x 32 channels) - into registers (the next chunk's loads are in flight under the MFMAs),
// the chunk lands in LDS as [pixel][k], the weights - packed at creation into the very LDS image and fetched
// a chunk ahead like the activations - are copied beside it, and each wavefront multiplies its 32 pixels with all the workgroup's channels
// (v_mfma_i32_32x32x32_i8 / v_mfma_f32_32x32x16_f16: both read 16 bytes per lane and step 32 bytes of a row).
// Quantized tensors: activations and weights go to the signed domain (u8 ^ 0x80), padding holds the input's
// zero point, the weights' zero point is a second MFMA against a constant vector, everything constant is
// folded into the bias; the epilogue is the library's round-half-even requantization. float16: float32
// accumulation, bias and activation, one rounding to float16.
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int kPixels = 128;      // output pixels of a workgroup
constexpr int kChunkBytes = 64;   // bytes of a pixel's window per reduction step
constexpr int kRowStride = kChunkBytes + 16;  // LDS row stride: 20 dwords spread the 16-byte fragment reads over the banks

struct GemmArgs {
  const uint8_t* x;
  uint8_t* y;
  const uint8_t* wpk;    // [group][channel tile][chunk][32 * OT rows][64 bytes]
  const int2* tab;       // per half-chunk (32 bytes of one tap's channels): {element offset of its first channel at the tap, dy | dx << 8 | real channels << 16}
  const int32_t* biasf;  // quantized: bias with the zero-point terms folded in, per padded output channel
  const float* biasfl;   // float16: the bias
  const tvx_v4i* rq;
  int C, H, W, OC, OH, OW;
  int sh, sw, pad_t, pad_l;
  int icg, ocg;          // channels per group, in and out
  int chunks;            // reduction steps
  int tiles_per_group;   // channel tiles of a group
  int xor_mask4, pad_fill4, neg_zws4, zp;
  int out_zp, lo, hi, rq_mode;
  int act;
  int aligned4;          // OH * OW is a multiple of four: four pixels of a channel are one aligned store
};

template <bool F16>
__device__ __forceinline__ void StoreFour(const GemmArgs& a, uint8_t* y, size_t at, int p, int hw, const int (&q)[4],
                                          const float (&f)[4]) {
  if (F16) {
    _Float16 h[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) h[e] = static_cast<_Float16>(f[e]);
    _Float16* yp = reinterpret_cast<_Float16*>(y) + at;
    if (a.aligned4) {
      if (p < hw) *reinterpret_cast<uint2*>(yp) = *reinterpret_cast<const uint2*>(h);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (p + e < hw) yp[e] = h[e];
    }
  } else {
    if (a.aligned4) {
      if (p < hw) *reinterpret_cast<uint32_t*>(y + at) = PackBytes(q[0], q[1], q[2], q[3]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (p + e < hw) y[at + e] = static_cast<uint8_t>(q[e]);
    }
  }
}

// OT: 32-channel tiles of a workgroup (1 or 2). QUAD: the gather by pixel quads (see below) instead of by elements.
// (two wavefronts per SIMD at least: within 256 registers the compiler keeps MFMA accumulators in ordinary vector
// registers, where the epilogue reads them, instead of moving every value out of the accumulation registers first)
template <bool F16, int OT, bool QUAD>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) ConvGemmKernel(GemmArgs a) {
  __shared__ __attribute__((aligned(16))) uint8_t a_lds[kPixels * kRowStride];
  __shared__ __attribute__((aligned(16))) uint8_t b_lds[OT * 32 * kRowStride];
  constexpr int ESZ = F16 ? 2 : 1;
  constexpr int kPerHalf = kChunkBytes / 2 / ESZ;  // window elements a thread gathers per chunk
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = wave >> 1;                       // which 32 bytes of the chunk this thread gathers
  const int px = tid & (kPixels - 1);
  const int hw = a.OH * a.OW;
  const int p0 = blockIdx.x * kPixels;
  const int group = blockIdx.y / a.tiles_per_group;
  const int tile = blockIdx.y - group * a.tiles_per_group;
  const int n = blockIdx.z;

  const int p = p0 + px;
  const bool p_live = p < hw;
  const int oh = p / a.OW, ow = p - oh * a.OW;
  const int ih0 = oh * a.sh - a.pad_t, iw0 = ow * a.sw - a.pad_l;
  const size_t plane = static_cast<size_t>(a.H) * a.W;
  const uint8_t* xg = a.x + (static_cast<size_t>(n) * a.C + static_cast<size_t>(group) * a.icg) * plane * ESZ;
  const int origin = ih0 * a.W + iw0;  // may be negative: only added to offsets of taps inside the image
  const uint8_t* wsrc = a.wpk + (static_cast<size_t>(group) * a.tiles_per_group + tile) * a.chunks * (OT * 32 * kChunkBytes);

  // The reduction runs tap by tap, a tap's channels padded to whole half-chunks: the 32 bytes a thread gathers
  // belong to one tap (one validity test, one base address) and walk the channel planes.
  // The window table's entry of this wavefront's half of a chunk (the same for all its lanes), read through the
  // constant address space: a scalar load. As a vector load the compiler waits for it with every load in flight
  // counted - the whole round trip in front of every chunk's gather.
  auto table_entry = [&](int chunk) {
    const __attribute__((address_space(4))) int* tab4 =
        reinterpret_cast<const __attribute__((address_space(4))) int*>(reinterpret_cast<uintptr_t>(a.tab));
    int2 e;
    e.x = tab4[(chunk * 2 + half) * 2];
    e.y = tab4[(chunk * 2 + half) * 2 + 1];
    return e;
  };
  uint32_t g[8];  // the 32 bytes of this thread's pixel row and chunk half
  const int plane_i = a.H * a.W;
  auto gather = [&](int chunk) {
    const int2 e = table_entry(chunk);
    const int dy = e.y & 0xff, dx = (e.y >> 8) & 0xff;
    const int nreal = e.y >> 16;              // real channels in this half-chunk (the rest is padding)
    const bool inside = p_live && static_cast<unsigned>(ih0 + dy) < static_cast<unsigned>(a.H) &&
                        static_cast<unsigned>(iw0 + dx) < static_cast<unsigned>(a.W);
    const int base = inside ? origin + e.x : 0;  // (outside: any readable element, masked below)
#pragma unroll
    for (int i = 0; i < kPerHalf; i += 4 / ESZ) {
      uint32_t word = 0;
#pragma unroll
      for (int j = 0; j < 4 / ESZ; ++j) {
        const int c = max(0, min(i + j, nreal - 1));  // (padding channels re-read a real one, masked below)
        uint32_t v;
        if (F16) {
          v = reinterpret_cast<const uint16_t*>(xg)[base + c * plane_i];
          if (!inside || i + j >= nreal) v = 0;
          word |= v << (16 * j);
        } else {
          v = xg[base + c * plane_i] ^ (static_cast<uint32_t>(a.xor_mask4) & 0xff);
          if (!inside) v = static_cast<uint32_t>(a.pad_fill4) & 0xff;
          if (i + j >= nreal || !p_live) v = 0;
          word |= v << (8 * j);
        }
      }
      g[i * ESZ / 4] = word;
    }
  };

  // ---- the gather by pixel quads (unit column stride, output rows of whole quads) -------------------
  // Four consecutive output pixels of a row read four consecutive input columns at every tap: a thread owns one
  // quad and 8 (float16: 4) channels of its chunk half, loads per channel the 4 (8) bytes under the quad - one
  // unaligned load instead of four element loads, clamped into the row and shifted back into place at the
  // image's left and right edges -, transposes the channel x pixel block in registers and writes 8 bytes per
  // pixel into the LDS image. Per chunk: 8 (4) loads and ~45 vector instructions, against 32 (16) loads and ~200.
  constexpr int kQuadCh = F16 ? 4 : 8;  // channels of a thread
  const int q = lane & 31;
  const int cg = (wave & 1) * 2 + (lane >> 5);
  const int pq = p0 + 4 * q;
  const bool q_live = pq < hw;
  const int q_oh = pq / a.OW, q_ow = pq - q_oh * a.OW;
  const int q_ih0 = q_oh * a.sh - a.pad_t, q_iw0 = q_ow - a.pad_l;
  const int q_origin = q_ih0 * a.W + q_iw0;
  int q_shift = 0, q_s = 0, q_n = 0;  // of the chunk in flight: columns clamped away, first column, real channels from this thread's first
  bool q_row = false;
  auto gather_quad = [&](int chunk) {
    const int2 e = table_entry(chunk);
    const int dy = e.y & 0xff, dx = (e.y >> 8) & 0xff;
    const int nreal = e.y >> 16;
    q_row = q_live && static_cast<unsigned>(q_ih0 + dy) < static_cast<unsigned>(a.H);
    q_s = q_iw0 + dx;
    q_shift = q_s - max(0, min(q_s, a.W - 4));
    q_n = nreal - cg * kQuadCh;
    const int base = q_row ? q_origin + e.x - q_shift : 0;  // (rows outside the image: any readable place, replaced below)
#pragma unroll
    for (int j = 0; j < kQuadCh; ++j) {
      const int c = max(0, min(cg * kQuadCh + j, nreal - 1));  // (padding channels re-read a real one, masked below)
      if (F16) {
        uint2 v;
        __builtin_memcpy(&v, xg + (static_cast<size_t>(base) + static_cast<size_t>(c) * plane_i) * 2, 8);
        g[2 * j] = v.x;
        g[2 * j + 1] = v.y;
      } else {
        uint32_t v;
        __builtin_memcpy(&v, xg + base + static_cast<size_t>(c) * plane_i, 4);
        g[j] = v;
      }
    }
  };
  // the chunk in the registers -> the LDS image [pixel][k]
  auto commit_quad = [&] {
    uint32_t out[4][2];  // per pixel of the quad: this thread's 8 bytes
    bool ok[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) ok[i] = q_row && static_cast<unsigned>(q_s + i) < static_cast<unsigned>(a.W);
    if (F16) {
      // byte k of the shifted pair = byte (k + 2 shift) mod 8 of the eight loaded (added per byte, no carries: at most 7 + 7)
      const uint32_t turn = static_cast<uint32_t>((2 * q_shift) & 7) * 0x01010101u;
      const uint32_t sel0 = (0x03020100u + turn) & 0x07070707u;
      const uint32_t sel1 = (0x07060504u + turn) & 0x07070707u;
      uint32_t lo[4], hi[4];  // per channel: pixels 0, 1 and 2, 3
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        lo[j] = __builtin_amdgcn_perm(g[2 * j + 1], g[2 * j], sel0);
        hi[j] = __builtin_amdgcn_perm(g[2 * j + 1], g[2 * j], sel1);
      }
      const uint32_t m0 = q_n >= 2 ? ~0u : (q_n == 1 ? 0xffffu : 0u), m1 = q_n >= 4 ? ~0u : (q_n == 3 ? 0xffffu : 0u);
      out[0][0] = __builtin_amdgcn_perm(lo[1], lo[0], 0x05040100) & m0;
      out[0][1] = __builtin_amdgcn_perm(lo[3], lo[2], 0x05040100) & m1;
      out[1][0] = __builtin_amdgcn_perm(lo[1], lo[0], 0x07060302) & m0;
      out[1][1] = __builtin_amdgcn_perm(lo[3], lo[2], 0x07060302) & m1;
      out[2][0] = __builtin_amdgcn_perm(hi[1], hi[0], 0x05040100) & m0;
      out[2][1] = __builtin_amdgcn_perm(hi[3], hi[2], 0x05040100) & m1;
      out[3][0] = __builtin_amdgcn_perm(hi[1], hi[0], 0x07060302) & m0;
      out[3][1] = __builtin_amdgcn_perm(hi[3], hi[2], 0x07060302) & m1;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (!ok[i]) out[i][0] = out[i][1] = 0;
    } else {
      // pixel i = byte (i + shift) mod 4 of the four loaded (added per byte, no carries: at most 3 + 3)
      const uint32_t sel = (0x03020100u + static_cast<uint32_t>(q_shift & 3) * 0x01010101u) & 0x03030303u;
      uint32_t e8[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) e8[j] = __builtin_amdgcn_perm(g[j], g[j], sel) ^ static_cast<uint32_t>(a.xor_mask4);
      const int na = max(0, min(q_n, 4)), nb = max(0, min(q_n - 4, 4));
      const uint32_t ma = na >= 4 ? ~0u : (1u << (8 * na)) - 1u, mb = nb >= 4 ? ~0u : (1u << (8 * nb)) - 1u;
      const uint32_t pad = q_live ? static_cast<uint32_t>(a.pad_fill4) : 0u;
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const uint32_t lo01 = __builtin_amdgcn_perm(e8[4 * b + 1], e8[4 * b], 0x05010400);
        const uint32_t hi01 = __builtin_amdgcn_perm(e8[4 * b + 1], e8[4 * b], 0x07030602);
        const uint32_t lo23 = __builtin_amdgcn_perm(e8[4 * b + 3], e8[4 * b + 2], 0x05010400);
        const uint32_t hi23 = __builtin_amdgcn_perm(e8[4 * b + 3], e8[4 * b + 2], 0x07030602);
        out[0][b] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100);
        out[1][b] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302);
        out[2][b] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100);
        out[3][b] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302);
        const uint32_t m = b ? mb : ma;
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i][b] = (ok[i] ? out[i][b] : pad) & m;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<uint2*>(a_lds + (4 * q + i) * kRowStride + half * 32 + cg * 8) = make_uint2(out[i][0], out[i][1]);
  };

  const int row = lane & 31, fh = lane >> 5;
  v16i acc_i[OT];
  v16f acc_f[OT];
#pragma unroll
  for (int t = 0; t < OT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc_i[t][r] = 0;
      acc_f[t][r] = 0.f;
    }
  const v4i fz = {a.neg_zws4, a.neg_zws4, a.neg_zws4, a.neg_zws4};

  // the weights of a chunk travel like its activations: into registers under the MFMAs of the chunk before
  uint4 w16 = make_uint4(0, 0, 0, 0);
  auto fetch_weights = [&](int chunk) {
    if (tid < OT * 128)
      w16 = *reinterpret_cast<const uint4*>(wsrc + static_cast<size_t>(chunk) * (OT * 32 * kChunkBytes) + tid * 16);
  };
  if (QUAD) gather_quad(0);
  else gather(0);
  fetch_weights(0);
  for (int chunk = 0; chunk < a.chunks; ++chunk) {
    // registers -> LDS
    {
      if (QUAD) {
        commit_quad();
      } else {
        uint8_t* dst = a_lds + px * kRowStride + half * 32;
        *reinterpret_cast<uint4*>(dst) = make_uint4(g[0], g[1], g[2], g[3]);
        *reinterpret_cast<uint4*>(dst + 16) = make_uint4(g[4], g[5], g[6], g[7]);
      }
      if (tid < OT * 128) *reinterpret_cast<uint4*>(b_lds + (tid >> 2) * kRowStride + (tid & 3) * 16) = w16;
    }
    __syncthreads();
    if (chunk + 1 < a.chunks) {
      if (QUAD) gather_quad(chunk + 1);
      else gather(chunk + 1);
      fetch_weights(chunk + 1);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const uint8_t* ap = a_lds + (wave * 32 + row) * kRowStride + ks * 32 + fh * 16;
      if (F16) {
        const v8h fx = *reinterpret_cast<const v8h*>(ap);
#pragma unroll
        for (int t = 0; t < OT; ++t) {
          const v8h fw = *reinterpret_cast<const v8h*>(b_lds + (t * 32 + row) * kRowStride + ks * 32 + fh * 16);
          acc_f[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fx, fw, acc_f[t], 0, 0, 0);
        }
      } else {
        const v4i fx = *reinterpret_cast<const v4i*>(ap);
#pragma unroll
        for (int t = 0; t < OT; ++t) {
          const v4i fw = *reinterpret_cast<const v4i*>(b_lds + (t * 32 + row) * kRowStride + ks * 32 + fh * 16);
          acc_i[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx, fw, acc_i[t], 0, 0, 0);
          if (a.zp) acc_i[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx, fz, acc_i[t], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }

  // ---- epilogue: lane = output channel `row` of each tile, pixels 8 gq + 4 fh + e of the wavefront's 32 ----
#pragma unroll
  for (int t = 0; t < OT; ++t) {
    const int ocl = (tile * OT + t) * 32 + row;  // channel within the group
    if (ocl >= a.ocg) continue;
    const int oc = group * a.ocg + ocl;
    const int tab_at = (group * a.tiles_per_group + tile) * OT * 32 + t * 32 + row;
    const size_t plane_at = (static_cast<size_t>(n) * a.OC + oc) * hw;
    v4i q = {0, 0, 0, 0};
    int bi = 0;
    float bf = 0.f;
    if (F16) {
      bf = a.biasfl ? a.biasfl[oc] : 0.f;
    } else {
      q = a.rq[tab_at];
      bi = a.biasf[tab_at];
    }
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const int pp = p0 + wave * 32 + 8 * gq + 4 * fh;
      int qi[4] = {0, 0, 0, 0};
      float fo[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (F16) {
          float v = acc_f[t][gq * 4 + e] + bf;
          if (a.act == TVX_ACT_RELU || a.act == TVX_ACT_RELU6) v = v < 0.f ? 0.f : v;
          if (a.act == TVX_ACT_RELU6) v = v > 6.f ? 6.f : v;
          fo[e] = v;
        } else {
          const int v = acc_i[t][gq * 4 + e] + bi;
          qi[e] = a.rq_mode == kRqGeneric ? Requant8<kRqGeneric>(v, q, a.out_zp, a.lo, a.hi)
                                          : (a.rq_mode == kRqFast ? Requant8<kRqFast>(v, q, a.out_zp, a.lo, a.hi)
                                                                  : Requant8<kRqFastNoTie>(v, q, a.out_zp, a.lo, a.hi));
        }
      }
      StoreFour<F16>(a, a.y, plane_at + pp, pp, hw, qi, fo);
    }
  }
}

struct Plan {
  GemmArgs a;
  dim3 grid;
  int ot;
  bool f16;
  bool quad;  // unit column stride, output rows of whole pixel quads, at least four input columns
};

int ConvGemmRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  GemmArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  const uintptr_t need = plan->f16 ? 7 : 3;
  a.aligned4 = a.aligned4 && (reinterpret_cast<uintptr_t>(out) & need) == 0;
  if (plan->f16 && ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(out)) & 1))
    return SetError(TVX_E_INVALID, "conv2d_gemm_f16: tensors must be 2-byte aligned");
  const dim3 block(kThreads);
#define TVX_LAUNCH(F, O, Q) hipLaunchKernelGGL((ConvGemmKernel<F, O, Q>), plan->grid, block, 0, st, a)
  if (plan->f16) {
    if (plan->quad) { if (plan->ot == 2) TVX_LAUNCH(true, 2, true); else TVX_LAUNCH(true, 1, true); }
    else { if (plan->ot == 2) TVX_LAUNCH(true, 2, false); else TVX_LAUNCH(true, 1, false); }
  } else {
    if (plan->quad) { if (plan->ot == 2) TVX_LAUNCH(false, 2, true); else TVX_LAUNCH(false, 1, true); }
    else { if (plan->ot == 2) TVX_LAUNCH(false, 2, false); else TVX_LAUNCH(false, 1, false); }
  }
#undef TVX_LAUNCH
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

}  // namespace

// Claims convolutions with constant weights, quantized (u8 / i8 activations) or float16 throughout, whose
// groups are worth a matrix tile: at least 8 output channels and 32 bytes of window per group.
int ConvGemmSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!w_host || op->fused_add || op->kind != OP_CONV2D) return TVX_E_UNSUPPORTED;
  const bool f16 = d->in_dtype == TVX_F16 && d->w_dtype == TVX_F16 && d->out_dtype == TVX_F16;
  if (!f16 && !op->quantized) return TVX_E_UNSUPPORTED;
  if (const char* f = getenv("TVX_NO_CONV_GEMM"))  // tuning aid: leaves these shapes to the generic kernel
    if (atoi(f)) return TVX_E_UNSUPPORTED;
  const int esz = f16 ? 2 : 1;
  const int groups = d->multiplier > 0 ? static_cast<int>(d->in_c) : (d->groups > 1 ? d->groups : 1);
  const int icg = static_cast<int>(d->in_c) / groups, ocg = static_cast<int>(d->out_c) / groups;
  const int taps = static_cast<int>(d->k_w * d->k_h);
  const uint64_t K64 = static_cast<uint64_t>(icg) * taps;
  if (ocg < 8 || K64 * esz < 32 || K64 > (1u << 24)) return TVX_E_UNSUPPORTED;
  if ((d->k_h - 1) * d->dilation_h > 255 || (d->k_w - 1) * d->dilation_w > 255) return TVX_E_UNSUPPORTED;
  const uint64_t in_elems = static_cast<uint64_t>(d->in_c) * d->in_h * d->in_w;
  const uint64_t hw = static_cast<uint64_t>(d->out_h) * d->out_w;
  if (in_elems >= (1ull << 31) || hw >= (1ull << 31) || d->batch > 65535) return TVX_E_UNSUPPORTED;
  const int K = static_cast<int>(K64);
  const int kc = kChunkBytes / esz;  // window elements per chunk
  const int kh = kc / 2;             // ... per half-chunk: what one thread gathers, all of one tap
  const int cpt = (icg + kh - 1) / kh * kh;  // a tap's channels, padded to whole half-chunks
  const int halves = taps * cpt / kh;
  const int chunks = (halves + 1) / 2;
  const int ot = ocg <= 32 ? 1 : 2;
  const int tiles = (ocg + 32 * ot - 1) / (32 * ot);
  if (static_cast<uint64_t>(groups) * tiles > 65535) return TVX_E_UNSUPPORTED;

  Plan plan{};
  GemmArgs& a = plan.a;
  a.C = d->in_c; a.H = d->in_h; a.W = d->in_w; a.OC = d->out_c; a.OH = d->out_h; a.OW = d->out_w;
  a.sh = d->stride_h; a.sw = d->stride_w; a.pad_t = d->pad_top; a.pad_l = d->pad_left;
  a.icg = icg; a.ocg = ocg; a.chunks = chunks; a.tiles_per_group = tiles;
  a.act = d->activation;
  a.aligned4 = hw % 4 == 0;

  // ---- the window table, the same for all groups: per half-chunk its tap and first channel ----
  std::vector<int32_t> tab(static_cast<size_t>(chunks) * 2 * 2, 0);
  for (int h = 0; h < halves; ++h) {
    const int t = h * kh / cpt, c0 = h * kh % cpt;
    const int dy = (t / static_cast<int>(d->k_w)) * static_cast<int>(d->dilation_h);
    const int dx = (t % static_cast<int>(d->k_w)) * static_cast<int>(d->dilation_w);
    const int nreal = std::max(0, std::min(kh, icg - c0));
    tab[2 * h] = c0 * a.H * a.W + dy * a.W + dx;
    tab[2 * h + 1] = dy | dx << 8 | nreal << 16;
  }

  // ---- weights [oc][c][ky][kx] -> per group, channel tile and chunk the LDS image [32 * OT rows][64 bytes] ----
  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = f16 ? 0 : d->in_zp - (x_u8 ? 128 : 0);
  const int zws = f16 ? 0 : op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127 || zws < -127 || zws > 127) return TVX_E_UNSUPPORTED;
  const int rows = 32 * ot;
  const size_t alloc_oc = static_cast<size_t>(groups) * tiles * rows;
  std::vector<uint8_t> packed(alloc_oc * chunks * kChunkBytes, 0);
  std::vector<int32_t> biasf(alloc_oc, 0);
  // (slots past a group's channels: a real channel's record, so that they do not decide the requantization flavour)
  std::vector<int32_t> mult(alloc_oc, f16 ? 0 : op->h_mult[0]), shift(alloc_oc, f16 ? 1 : op->h_shift[0]);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  for (int g = 0; g < groups; ++g)
    for (int ocl = 0; ocl < ocg; ++ocl) {
      const int oc = g * ocg + ocl;
      const int tile = ocl / rows, r = ocl % rows;
      const size_t slot = (static_cast<size_t>(g) * tiles + tile) * rows + r;
      int64_t sw = 0;
      for (int k = 0; k < K; ++k) {  // the weight tensor's own order: [oc][c][ky][kx]
        const int kp = (k % taps) * cpt + k / taps;  // position in the tap-major, channel-padded reduction
        const size_t at = (((static_cast<size_t>(g) * tiles + tile) * chunks + kp / kc) * rows + r) * kChunkBytes +
                          static_cast<size_t>(kp % kc) * esz;
        if (f16) {
          std::memcpy(&packed[at], src + (static_cast<size_t>(oc) * K + k) * 2, 2);
        } else {
          const uint8_t raw = src[static_cast<size_t>(oc) * K + k];
          const int8_t v = static_cast<int8_t>(w_u8 ? raw ^ 0x80 : raw);
          packed[at] = static_cast<uint8_t>(v);
          sw += v;
        }
      }
      if (!f16) {
        const int64_t v = (b ? b[oc] : 0) - static_cast<int64_t>(zxs) * sw + static_cast<int64_t>(K) * zxs * zws;
        biasf[slot] = static_cast<int32_t>(static_cast<uint32_t>(v));
        mult[slot] = op->h_mult[oc];
        shift[slot] = op->h_shift[oc];
      }
    }
  int s = op->packed.Upload(packed.data(), packed.size());
  if (s == TVX_OK) s = op->aux3.Upload(tab.data(), tab.size() * 4);
  if (s != TVX_OK) return s;
  a.wpk = op->packed.as<uint8_t>();
  a.tab = op->aux3.as<int2>();
  if (f16) {
    if (bias_host) {
      s = op->bias.Upload(bias_host, static_cast<size_t>(d->out_c) * 4);
      if (s != TVX_OK) return s;
      a.biasfl = op->bias.as<float>();
    }
  } else {
    std::vector<int32_t> rqt;
    a.rq_mode = BuildRequantRecords(mult, shift, static_cast<int>(alloc_oc), static_cast<int>(alloc_oc), d->out_zp, &rqt,
                                    AccumulatorBound(static_cast<uint64_t>(K), bias_host, d->out_c));
    s = op->aux.Upload(biasf.data(), biasf.size() * 4);
    if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
    if (s != TVX_OK) return s;
    a.biasf = op->aux.as<int32_t>();
    a.rq = op->aux2.as<tvx_v4i>();
    a.xor_mask4 = x_u8 ? static_cast<int>(0x80808080u) : 0;
    a.pad_fill4 = static_cast<int>(static_cast<uint32_t>(zxs & 0xff) * 0x01010101u);
    a.neg_zws4 = static_cast<int>(static_cast<uint32_t>((-zws) & 0xff) * 0x01010101u);
    a.zp = zws != 0;
    a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  }
  plan.grid = dim3(static_cast<unsigned>((hw + kPixels - 1) / kPixels), static_cast<unsigned>(groups * tiles), d->batch);
  plan.ot = ot;
  plan.f16 = f16;
  plan.quad = d->stride_w == 1 && d->out_w % 4 == 0 && d->in_w >= 4;
  if (const char* f = getenv("TVX_CONV_GEMM_QUAD")) plan.quad = plan.quad && atoi(f) != 0;  // tuning aid: 0 = the gather by elements
  op->host_blob.resize(sizeof(Plan));
  std::memcpy(op->host_blob.data(), &plan, sizeof(Plan));
  op->run = ConvGemmRun;
  op->kernel_name = f16 ? "conv2d_gemm_f16" : "conv2d_gemm_i8";
  return TVX_OK;
}

}  // namespace tvx
