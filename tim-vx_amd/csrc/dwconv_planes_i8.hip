// Depthwise quantized convolution (multiplier 1) for small planes of any width.
//
// In WHCN every (image, channel) plane is contiguous, and so is a run of G
// consecutive planes - input and output alike. A workgroup therefore copies the
// G input planes into LDS as one linear, 16-byte-chunked stream (no row or
// alignment structure needed: widths like 14 or 7 are as good as any), computes
// the stencil out of LDS - a work item is four neighbouring outputs of one row,
// sharing the loaded input columns - into an LDS image of the G output planes,
// and copies that image out as another linear stream. Out-of-image taps read the
// input zero point, so with wz = w - zw every output is
//   bias - zx * sum(wz) + sum x * wz,
// the first two terms folded at creation. Any kernel size, stride, dilation
// and padding; 3x3 is unrolled.
#include <algorithm>

#include "variants.h"

namespace tvx {
namespace {

constexpr int kThreads = 256;

struct DwpArgs {
  const uint8_t* x;
  uint8_t* y;
  const int32_t* tab;  // per channel: kh*kw ints wz, then the folded bias; row stride tab_stride ints
  const tvx_v4i* rq;   // per channel requantization record
  int C, H, W, OH, OW;
  int kh, kw, sh, sw, dh, dw, pad_t, pad_l;
  int tab_stride;
  int G;               // planes per workgroup
  long long planes;    // batch * C
  int in_zp, out_zp, lo, hi;
  int ow4;             // work items per output row
};

// Linear copy of `len` bytes from global `src` into LDS so that byte i lands at
// dst[(src & 15) + i]: whole aligned 16-byte chunks, except that a chunk reaching
// past `limit` (the end of the tensor) is read byte by byte.
__device__ __forceinline__ void CopyIn(const uint8_t* src, size_t len, const uint8_t* limit, uint8_t* dst, int tid) {
  const uintptr_t s = reinterpret_cast<uintptr_t>(src);
  const uint8_t* base = reinterpret_cast<const uint8_t*>(s & ~uintptr_t{15});
  const int head = static_cast<int>(s & 15);
  const int chunks = static_cast<int>((head + len + 15) / 16);
  for (int i = tid; i < chunks; i += kThreads) {
    const uint8_t* p = base + static_cast<size_t>(i) * 16;
    if (p + 16 <= limit) {
      *reinterpret_cast<uint4*>(dst + i * 16) = *reinterpret_cast<const uint4*>(p);
    } else {
      for (int b = 0; b < 16; ++b)
        if (p + b < limit) dst[i * 16 + b] = p[b];
    }
  }
}

// Linear copy of `len` bytes from LDS (byte i at src[(dst & 15) + i]) to global `dst`.
__device__ __forceinline__ void CopyOut(uint8_t* dst, size_t len, const uint8_t* src, int tid) {
  const uintptr_t d = reinterpret_cast<uintptr_t>(dst);
  uint8_t* base = reinterpret_cast<uint8_t*>(d & ~uintptr_t{15});
  const int head = static_cast<int>(d & 15);
  const int end = head + static_cast<int>(len);
  const int chunks = (end + 15) / 16;
  for (int i = tid; i < chunks; i += kThreads) {
    const int lo = i * 16, hi = lo + 16;
    if (lo >= head && hi <= end) {
      *reinterpret_cast<uint4*>(base + lo) = *reinterpret_cast<const uint4*>(src + lo);
    } else {
      for (int b = max(lo, head); b < min(hi, end); ++b) base[b] = src[b];
    }
  }
}

template <typename XT, bool K3, int RQ>
__global__ void __launch_bounds__(kThreads) DwPlanesKernel(DwpArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  const int tid = threadIdx.x;
  const long long p0 = static_cast<long long>(blockIdx.x) * a.G;
  const int g_n = static_cast<int>(min(static_cast<long long>(a.G), a.planes - p0));
  const int hwi = a.H * a.W, hwo = a.OH * a.OW;
  const uint8_t* src = a.x + static_cast<size_t>(p0) * hwi;
  uint8_t* dst = a.y + static_cast<size_t>(p0) * hwo;
  const int in_head = static_cast<int>(reinterpret_cast<uintptr_t>(src) & 15);
  const int out_head = static_cast<int>(reinterpret_cast<uintptr_t>(dst) & 15);
  uint8_t* in_lds = lds_raw;
  uint8_t* out_lds = lds_raw + ((a.G * hwi + 15 + 16) & ~15);
  CopyIn(src, static_cast<size_t>(g_n) * hwi, a.x + static_cast<size_t>(a.planes) * hwi, in_lds, tid);
  __syncthreads();
  const XT* xin = reinterpret_cast<const XT*>(in_lds + in_head);
  uint8_t* yout = out_lds + out_head;

  const int kh = K3 ? 3 : a.kh, kw = K3 ? 3 : a.kw;
  const int items_per_plane = a.OH * a.ow4;
  const int items = g_n * items_per_plane;
  for (int it = tid; it < items; it += kThreads) {
    const int g = it / items_per_plane;
    const int r = it - g * items_per_plane;
    const int oy = r / a.ow4;
    const int ox0 = (r - oy * a.ow4) * 4;
    const int c = static_cast<int>((p0 + g) % a.C);
    const int32_t* t = a.tab + static_cast<size_t>(c) * a.tab_stride;
    const int bias = t[kh * kw];
    int acc[4] = {bias, bias, bias, bias};
    const XT* plane = xin + g * hwi;
    const int iy0 = oy * a.sh - a.pad_t;
    const int ix0 = ox0 * a.sw - a.pad_l;
    auto tap = [&](int ky, int kx) {
      const int iy = iy0 + ky * a.dh;
      const bool row_ok = iy >= 0 && iy < a.H;
      const XT* row = plane + (row_ok ? iy : 0) * a.W;
      const int wz = t[ky * kw + kx];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int ix = ix0 + j * a.sw + kx * a.dw;
        const bool ok = row_ok && ix >= 0 && ix < a.W;
        const int xv = ok ? static_cast<int>(row[ok ? ix : 0]) : a.in_zp;
        acc[j] += xv * wz;
      }
    };
    if (K3) {
#pragma unroll
      for (int ky = 0; ky < 3; ++ky)
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) tap(ky, kx);
    } else {
      for (int ky = 0; ky < kh; ++ky)
        for (int kx = 0; kx < kw; ++kx) tap(ky, kx);
    }
    const tvx_v4i q = a.rq[c];
    uint8_t* o = yout + g * hwo + oy * a.OW + ox0;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (ox0 + j < a.OW) o[j] = static_cast<uint8_t>(Requant8<RQ>(acc[j], q, a.out_zp, a.lo, a.hi));
  }
  __syncthreads();
  CopyOut(dst, static_cast<size_t>(g_n) * hwo, out_lds, tid);
}

struct Plan {
  DwpArgs a;
  int lds_bytes, x_u8, k3, rq;
  unsigned grid;
};

template <typename XT, bool K3>
void LaunchRq(const Plan* p, const DwpArgs& a, hipStream_t st) {
  const dim3 grid(p->grid), block(kThreads);
  if (p->rq == kRqFastNoTie)
    hipLaunchKernelGGL((DwPlanesKernel<XT, K3, kRqFastNoTie>), grid, block, p->lds_bytes, st, a);
  else if (p->rq == kRqFast)
    hipLaunchKernelGGL((DwPlanesKernel<XT, K3, kRqFast>), grid, block, p->lds_bytes, st, a);
  else
    hipLaunchKernelGGL((DwPlanesKernel<XT, K3, kRqGeneric>), grid, block, p->lds_bytes, st, a);
}

int DwPlanesRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* p = reinterpret_cast<const Plan*>(op->host_blob.data());
  DwpArgs a = p->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(out)) & 15)
    return SetError(TVX_E_INVALID, "dwconv_planes_i8: tensors must be 16-byte aligned");
  if (p->x_u8) {
    if (p->k3) LaunchRq<uint8_t, true>(p, a, st); else LaunchRq<uint8_t, false>(p, a, st);
  } else {
    if (p->k3) LaunchRq<int8_t, true>(p, a, st); else LaunchRq<int8_t, false>(p, a, st);
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

}  // namespace

// Claims quantized depthwise convolutions (multiplier 1, constant weights) whose planes
// are small enough for a few of them to sit in LDS.
int DwPlanesSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || d->multiplier != 1) return TVX_E_UNSUPPORTED;
  const uint64_t hwi = static_cast<uint64_t>(d->in_w) * d->in_h, hwo = static_cast<uint64_t>(d->out_w) * d->out_h;
  if (hwi == 0 || hwo == 0 || hwi + hwo > 40 * 1024) return TVX_E_UNSUPPORTED;
  const int taps = d->k_w * d->k_h;
  if (taps > 121) return TVX_E_UNSUPPORTED;
  const int C = d->in_c;
  const bool w_u8 = d->w_dtype == TVX_U8;
  Plan p{};
  DwpArgs& a = p.a;
  a.C = C; a.H = d->in_h; a.W = d->in_w; a.OH = d->out_h; a.OW = d->out_w;
  a.kh = d->k_h; a.kw = d->k_w; a.sh = d->stride_h; a.sw = d->stride_w;
  a.dh = d->dilation_h; a.dw = d->dilation_w; a.pad_t = d->pad_top; a.pad_l = d->pad_left;
  a.tab_stride = taps + 1;
  a.planes = static_cast<long long>(d->batch) * C;
  a.in_zp = d->in_zp; a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  a.ow4 = (a.OW + 3) / 4;
  // planes per workgroup: about 8 KiB of input + output, but leave a few workgroups per CU
  long long g = std::max<long long>(1, 8192 / static_cast<long long>(hwi + hwo));
  g = std::min<long long>(g, std::max<long long>(1, a.planes / 1024));
  a.G = static_cast<int>(std::min<long long>(g, 256));
  const long long grid = (a.planes + a.G - 1) / a.G;
  if (grid > 0x7fffffffll) return TVX_E_UNSUPPORTED;
  p.lds_bytes = static_cast<int>(((a.G * hwi + 15 + 16) & ~15ull) + ((a.G * hwo + 15 + 16) & ~15ull));
  std::vector<int32_t> tab(static_cast<size_t>(C) * a.tab_stride);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  for (int c = 0; c < C; ++c) {
    int64_t sum = 0;
    for (int t = 0; t < taps; ++t) {
      const uint8_t raw = src[static_cast<size_t>(c) * taps + t];
      const int wz = (w_u8 ? static_cast<int>(raw) : static_cast<int>(static_cast<int8_t>(raw))) - op->w_zp;
      tab[static_cast<size_t>(c) * a.tab_stride + t] = wz;
      sum += wz;
    }
    // padding taps are fed the zero point, so every output sums all taps
    const int64_t v = (b ? b[c] : 0) - static_cast<int64_t>(d->in_zp) * sum;
    tab[static_cast<size_t>(c) * a.tab_stride + taps] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  std::vector<int32_t> rqt;
  p.rq = BuildRequantRecords(op->h_mult, op->h_shift, C, C, d->out_zp, &rqt, AccumulatorBound(taps, bias_host, C));
  int s = op->packed.Upload(tab.data(), tab.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s != TVX_OK) return s;
  a.tab = op->packed.as<int32_t>();
  a.rq = op->aux2.as<tvx_v4i>();
  p.x_u8 = d->in_dtype == TVX_U8;
  p.k3 = d->k_w == 3 && d->k_h == 3;
  p.grid = static_cast<unsigned>(grid);
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&p), reinterpret_cast<const uint8_t*>(&p) + sizeof(p));
  op->run = DwPlanesRun;
  op->kernel_name = "dwconv_planes_i8";
  return TVX_OK;
}

}  // namespace tvx
