// Depthwise quantized convolution (multiplier 1) for small planes of any width.
//
// In WHCN every (image, channel) plane is contiguous, and so is a run of G
// consecutive planes - input and output alike. A workgroup therefore reads the
// G input planes as one linear stream of aligned 16-byte chunks (no row or
// alignment structure needed: widths like 14 or 7 are as good as any) and
// scatters the bytes into LDS images of the planes that carry their padding
// border, pre-filled with the input zero point: the stencil then runs without a
// single bounds check. A work item is four neighbouring outputs of one row; for
// 3x3 kernels of stride 1 or 2 they share the input columns they read. Results
// go to an LDS image of the G output planes, which leaves as another linear
// stream. With wz = w - zw every output is bias - zx * sum(wz) + sum x * wz, the
// first two terms folded at creation and kept, with the taps, in LDS per plane.
// 3x3 kernels of stride 1 or 2 on rows of at least four bytes take a second kernel that
// keeps the same plan but works on whole dwords (see DwRowsKernel below).
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
  int ph, pw;          // padded plane extent in LDS
  int off_out, off_tab;  // LDS carve-up (bytes): output image, per-plane tables
};

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

// MODE 0: any kernel; 1: 3x3, stride 1, dilation 1; 2: 3x3, stride 2, dilation 1.
template <typename XT, int MODE, int RQ>
__global__ void __launch_bounds__(kThreads) DwPlanesKernel(DwpArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  const int tid = threadIdx.x;
  const long long p0 = static_cast<long long>(blockIdx.x) * a.G;
  const int g_n = static_cast<int>(min(static_cast<long long>(a.G), a.planes - p0));
  const int hwi = a.H * a.W, hwo = a.OH * a.OW;
  const int pplane = a.ph * a.pw;
  const uint8_t* src = a.x + static_cast<size_t>(p0) * hwi;
  uint8_t* dst = a.y + static_cast<size_t>(p0) * hwo;
  uint8_t* in_lds = lds_raw;
  uint8_t* out_lds = lds_raw + a.off_out;
  int* tab_lds = reinterpret_cast<int*>(lds_raw + a.off_tab);
  const int taps = MODE ? 9 : a.kh * a.kw;
  const int tstride = taps + 5;  // taps, folded bias, 4-dword requantization record

  // ---- padded planes <- zero point; per-plane tables ----------------------------------
  {
    const uint32_t z4 = static_cast<uint32_t>(a.in_zp & 0xff) * 0x01010101u;
    const uint4 z16 = make_uint4(z4, z4, z4, z4);
    for (int i = tid; i < a.off_out / 16; i += kThreads) reinterpret_cast<uint4*>(in_lds)[i] = z16;
    for (int i = tid; i < g_n * tstride; i += kThreads) {
      const int g = i / tstride, e = i - g * tstride;
      const int c = static_cast<int>((p0 + g) % a.C);
      tab_lds[i] = e <= taps ? a.tab[static_cast<size_t>(c) * a.tab_stride + e]
                             : reinterpret_cast<const int*>(a.rq)[c * 4 + (e - taps - 1)];
    }
  }
  __syncthreads();
  // ---- input stream -> plane interiors ---------------------------------------------------
  {
    const uintptr_t sa = reinterpret_cast<uintptr_t>(src);
    const uint8_t* base = reinterpret_cast<const uint8_t*>(sa & ~uintptr_t{15});
    const int head = static_cast<int>(sa & 15);
    const int len = g_n * hwi;
    const int chunks = (head + len + 15) / 16;
    const uint8_t* limit = a.x + static_cast<size_t>(a.planes) * hwi;
    for (int i = tid; i < chunks; i += kThreads) {
      const uint8_t* pch = base + static_cast<size_t>(i) * 16;
      uint32_t w[4] = {0, 0, 0, 0};
      if (pch + 16 <= limit) {
        const uint4 v = *reinterpret_cast<const uint4*>(pch);
        w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
      } else {
        for (int b = 0; b < 16; ++b)
          if (pch + b < limit) w[b >> 2] |= static_cast<uint32_t>(pch[b]) << (8 * (b & 3));
      }
      // linear index of the chunk's first byte -> (plane, row, column), then walk
      int li = i * 16 - head;
      const int lj = max(li, 0);
      int g = lj / hwi;
      int rem = lj - g * hwi;
      int iy = rem / a.W, ix = rem - iy * a.W;
      uint8_t* o = in_lds + g * pplane + (iy + a.pad_t) * a.pw + a.pad_l + ix;
#pragma unroll
      for (int b = 0; b < 16; ++b, ++li) {
        if (li < 0 || li >= len) continue;
        *o = static_cast<uint8_t>(w[b >> 2] >> (8 * (b & 3)));
        ++o;
        if (++ix == a.W) {
          ix = 0;
          o += a.pw - a.W;
          if (++iy == a.H) { iy = 0; o += pplane - a.H * a.pw; }
        }
      }
    }
  }
  __syncthreads();

  // ---- stencil ------------------------------------------------------------------------------
  const int out_head = static_cast<int>(reinterpret_cast<uintptr_t>(dst) & 15);
  uint8_t* yout = out_lds + out_head;
  const int items_per_plane = a.OH * a.ow4;
  const int items = g_n * items_per_plane;
  for (int it = tid; it < items; it += kThreads) {
    const int g = it / items_per_plane;
    const int r = it - g * items_per_plane;
    const int oy = r / a.ow4;
    const int ox0 = (r - oy * a.ow4) * 4;
    const int* t = tab_lds + g * tstride;
    const int bias = t[taps];
    int acc[4] = {bias, bias, bias, bias};
    const XT* win = reinterpret_cast<const XT*>(in_lds) + g * pplane + (oy * a.sh) * a.pw + ox0 * a.sw;
    if (MODE) {
      constexpr int kCols = MODE == 1 ? 6 : 9;  // input columns behind four outputs
#pragma unroll
      for (int ky = 0; ky < 3; ++ky) {
        int col[kCols];
#pragma unroll
        for (int j = 0; j < kCols; ++j) col[j] = static_cast<int>(win[ky * a.pw + j]);
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) {
          const int wz = t[ky * 3 + kx];
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[j] += col[j * MODE + kx] * wz;
        }
      }
    } else {
      for (int ky = 0; ky < a.kh; ++ky)
        for (int kx = 0; kx < a.kw; ++kx) {
          const int wz = t[ky * a.kw + kx];
          const XT* px = win + (ky * a.dh) * a.pw + kx * a.dw;
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[j] += static_cast<int>(px[j * a.sw]) * wz;
        }
    }
    const tvx_v4i q = {t[taps + 1], t[taps + 2], t[taps + 3], t[taps + 4]};
    uint8_t* o = yout + g * hwo + oy * a.OW + ox0;
    const int lo = a.lo, hi = a.hi;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (ox0 + j < a.OW) o[j] = static_cast<uint8_t>(Requant8<RQ>(acc[j], q, a.out_zp, lo, hi));
  }
  __syncthreads();
  CopyOut(dst, static_cast<size_t>(g_n) * hwo, out_lds, tid);
}

struct Plan {
  DwpArgs a;
  int lds_bytes, x_u8, mode, rq;
  unsigned grid;
};

template <typename XT, int MODE>
void LaunchRq(const Plan* p, const DwpArgs& a, hipStream_t st) {
  const dim3 grid(p->grid), block(kThreads);
  if (p->rq == kRqFastNoTie)
    hipLaunchKernelGGL((DwPlanesKernel<XT, MODE, kRqFastNoTie>), grid, block, p->lds_bytes, st, a);
  else if (p->rq == kRqFast)
    hipLaunchKernelGGL((DwPlanesKernel<XT, MODE, kRqFast>), grid, block, p->lds_bytes, st, a);
  else
    hipLaunchKernelGGL((DwPlanesKernel<XT, MODE, kRqGeneric>), grid, block, p->lds_bytes, st, a);
}

template <typename XT>
void LaunchMode(const Plan* p, const DwpArgs& a, hipStream_t st) {
  if (p->mode == 1) LaunchRq<XT, 1>(p, a, st);
  else if (p->mode == 2) LaunchRq<XT, 2>(p, a, st);
  else LaunchRq<XT, 0>(p, a, st);
}

int DwPlanesRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* p = reinterpret_cast<const Plan*>(op->host_blob.data());
  DwpArgs a = p->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(out)) & 15)
    return SetError(TVX_E_INVALID, "dwconv_planes_i8: tensors must be 16-byte aligned");
  if (p->x_u8) LaunchMode<uint8_t>(p, a, st); else LaunchMode<int8_t>(p, a, st);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}


// ---- 3x3, stride 1 or 2: the same idea on dwords ------------------------------------------
// The padded planes live in LDS as rows of whole dwords in the int8 domain (uint8 inputs are
// re-biased on the way in). Every dword of a padded plane is composed in registers from one
// unaligned global dword and the zero point (v_alignbyte), so there is no fill pass and no
// byte store; a work item is four neighbouring outputs in each of two output rows: it reads
// two or three dwords of each input row behind them, cuts the windows with v_alignbyte,
// multiplies with v_dot4 against the packed kernel rows and stores its bytes straight to
// the output tensor (unaligned dword stores are legal on global memory; rows of width 14 or
// 7 need them). Index arithmetic uses 24-bit multiplies and reciprocals, no divisions.
struct DwrArgs {
  const uint8_t* x;
  uint8_t* y;
  const int32_t* wpk;    // per channel: three packed kernel rows (kx in bytes 0..2), one unused word
  const int32_t* biasf;  // per channel: bias with the constant zero-point terms folded in
  const tvx_v4i* rq;
  int C, H, W, OH, OW, pad_t, pad_l;
  int G, planes;
  int ow4, oh2;          // work items per output row pair, row pairs per plane
  int ph, pw4;           // padded plane: ph rows of pw4 dwords
  uint32_t m_c, m_plane4, m_pw4, m_ipp, m_ow4;  // reciprocals of C, ph*pw4, pw4, oh2*ow4, ow4
  int xor_mask, pad_fill, zws, out_zp, lo, hi;
  int off_tab;           // dword offset of the per-plane tables in LDS
  int out_blocked, PO;   // the result goes out channel-blocked (byte ((c / 16) * PO + p) * 16 + c % 16, PO pixels in the batch)
};

constexpr int kCopyBatch = 8;  // input dwords a thread has in flight
constexpr int kTabDwords = 8;  // per plane: {row0, row1, row2, bias}, requantization record

__device__ __forceinline__ int DivMagic(int u, uint32_t magic) {
  return magic ? static_cast<int>(__umulhi(static_cast<uint32_t>(u), magic)) : u;
}

// BOXSUM: the weights are not pre-shifted by their zero point; the window sum supplies the term.
template <int S, bool BOXSUM, int RQ>
__global__ void __launch_bounds__(kThreads) DwRowsKernel(DwrArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_raw[];
  uint32_t* lds32 = reinterpret_cast<uint32_t*>(lds_raw);
  int* tab = reinterpret_cast<int*>(lds32 + a.off_tab);
  const int tid = threadIdx.x;
  const int p0 = blockIdx.x * a.G;
  const int g_n = min(a.G, a.planes - p0);
  const int hwi = a.H * a.W, hwo = a.OH * a.OW;
  const int plane4 = a.ph * a.pw4;

  // ---- per-plane tables: one entry per thread (G * kTabDwords <= kThreads); the address is
  // selected, not the loaded value, so the load is unconditional and travels with the input's
  int tab_val;
  {
    const int i = min(tid, g_n * kTabDwords - 1);
    const int g = i / kTabDwords, e = i - g * kTabDwords;
    const int pl = p0 + g;
    const int c = pl - __mul24(DivMagic(pl, a.m_c), a.C);
    const int* from = e < 3 ? a.wpk + (c * 4 + e) : (e == 3 ? a.biasf + c : reinterpret_cast<const int*>(a.rq) + (c * 4 + (e - 4)));
    tab_val = *from;
  }
  // ---- input planes -> padded planes, one dword per step -----------------------------------
  {
    const uint8_t* src = a.x + static_cast<size_t>(p0) * hwi;
    const uint32_t z4 = static_cast<uint32_t>(a.pad_fill);
    const int n_in = g_n * plane4;
    // kCopyBatch loads of a thread travel together: all are issued (from clamped indices, so
    // none sits under a branch) before the first is composed and stored
    for (int i0 = tid; i0 < n_in; i0 += kThreads * kCopyBatch) {
      uint32_t v[kCopyBatch];
      int d[kCopyBatch];
      uint32_t keep[kCopyBatch];
#pragma unroll
      for (int b = 0; b < kCopyBatch; ++b) {
        const int i = min(i0 + b * kThreads, n_in - 1);
        const int g = DivMagic(i, a.m_plane4);
        const int r2 = i - __mul24(g, plane4);
        const int r = DivMagic(r2, a.m_pw4);
        const int j = r2 - __mul24(r, a.pw4);
        const int ih = r - a.pad_t;
        const int c0 = 4 * j - a.pad_l;  // input column of the dword's first byte
        const bool row_ok = static_cast<unsigned>(ih) < static_cast<unsigned>(a.H);
        // the load always lies inside the row: at the edges it is shifted against the zero point
        const int cl = min(max(c0, 0), a.W - 4);
        __builtin_memcpy(&v[b], src + (__mul24(g, hwi) + __mul24(row_ok ? ih : 0, a.W) + cl), 4);
        d[b] = c0 - cl;  // < 0: left edge, > 0: right edge (>= 4: beyond the row)
        keep[b] = (row_ok && d[b] < 4) ? ~0u : 0u;
      }
#pragma unroll
      for (int b = 0; b < kCopyBatch; ++b) {
        const uint32_t x = v[b] ^ static_cast<uint32_t>(a.xor_mask);
        const uint32_t left = __builtin_amdgcn_alignbyte(x, z4, static_cast<uint32_t>(4 + d[b]) & 3u);
        const uint32_t right = __builtin_amdgcn_alignbyte(z4, x, static_cast<uint32_t>(d[b]) & 3u);
        const uint32_t res = d[b] < 0 ? left : right;
        // mask arithmetic, not a select against the loaded value
        if (i0 + b * kThreads < n_in) lds32[i0 + b * kThreads] = (res & keep[b]) | (z4 & ~keep[b]);
      }
    }
  }
  if (tid < g_n * kTabDwords) tab[tid] = tab_val;
  __syncthreads();

  // ---- stencil ------------------------------------------------------------------------------
  const int ipp = a.oh2 * a.ow4;
  const int items = g_n * ipp;
  uint8_t* dst = a.y + static_cast<size_t>(p0) * hwo;
  const int lo = a.lo, hi = a.hi;
  constexpr int kRows = S + 3;  // input rows behind two output rows
  for (int it = tid; it < items; it += kThreads) {
    const int g = DivMagic(it, a.m_ipp);
    const int r = it - __mul24(g, ipp);
    const int oy2 = DivMagic(r, a.m_ow4);
    const int q = r - __mul24(oy2, a.ow4);
    const int oy = oy2 * 2;
    const tvx_v4i t0 = *reinterpret_cast<const tvx_v4i*>(tab + g * kTabDwords);
    const tvx_v4i rq = *reinterpret_cast<const tvx_v4i*>(tab + g * kTabDwords + 4);
    // the padded plane has rows for a second output row even when OH is odd (its result is dropped)
    const uint32_t* row = lds32 + (__mul24(g, plane4) + __mul24(oy * S, a.pw4) + q * S);
    uint32_t win[kRows][4];
#pragma unroll
    for (int ir = 0; ir < kRows; ++ir) {
      const uint32_t d0 = row[ir * a.pw4], d1 = row[ir * a.pw4 + 1];
      if (S == 1) {
        win[ir][0] = d0;
        win[ir][1] = __builtin_amdgcn_alignbyte(d1, d0, 1);
        win[ir][2] = __builtin_amdgcn_alignbyte(d1, d0, 2);
        win[ir][3] = __builtin_amdgcn_alignbyte(d1, d0, 3);
      } else {
        const uint32_t d2 = row[ir * a.pw4 + 2];
        win[ir][0] = d0;
        win[ir][1] = __builtin_amdgcn_alignbyte(d1, d0, 2);
        win[ir][2] = d1;
        win[ir][3] = __builtin_amdgcn_alignbyte(d2, d1, 2);
      }
    }
    uint8_t* o = dst + (__mul24(g, hwo) + __mul24(oy, a.OW) + 4 * q);
    const int n = min(4, a.OW - 4 * q);
#pragma unroll
    for (int orow = 0; orow < 2; ++orow) {
      int r4[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int acc = Dot4Add(static_cast<int>(win[orow * S][j]), t0[0], t0[3]);
#pragma unroll
        for (int ky = 1; ky < 3; ++ky) acc = __builtin_amdgcn_sdot4(static_cast<int>(win[orow * S + ky][j]), t0[ky], acc, false);
        if (BOXSUM) {
          int sx = 0;
#pragma unroll
          for (int ky = 0; ky < 3; ++ky) sx = __builtin_amdgcn_sdot4(static_cast<int>(win[orow * S + ky][j]), 0x00010101, sx, false);
          acc -= __mul24(a.zws, sx);
        }
        r4[j] = Requant8<RQ>(acc, rq, a.out_zp, lo, hi);
      }
      const uint32_t packed = PackBytes(r4[0], r4[1], r4[2], r4[3]);
      if (a.out_blocked) {  // (uniform) four pixels of one channel: four bytes sixteen apart
        if (oy + orow < a.OH) {
          const int pl = p0 + g;
          const int img = DivMagic(pl, a.m_c), c = pl - __mul24(img, a.C);
          const int pix = __mul24(img, hwo) + __mul24(oy + orow, a.OW) + 4 * q;
          uint8_t* ob = a.y + (static_cast<size_t>(c >> 4) * a.PO + pix) * 16 + (c & 15);
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (j < n) ob[j * 16] = static_cast<uint8_t>(packed >> (8 * j));
        }
      } else if (oy + orow < a.OH) {
        uint8_t* orw = o + orow * a.OW;
        if (n == 4) {
          __builtin_memcpy(orw, &packed, 4);
        } else {
          if (n & 2) {
            const uint16_t h = static_cast<uint16_t>(packed);
            __builtin_memcpy(orw, &h, 2);
          }
          if (n & 1) orw[n & 2] = static_cast<uint8_t>(packed >> (8 * (n & 2)));
        }
      }
    }
  }
}

struct RowsPlan {
  DwrArgs a;
  int lds_bytes, stride, boxsum, rq;
  unsigned grid;
};

template <int S, bool BOXSUM>
void LaunchRowsRq(const RowsPlan* p, const DwrArgs& a, hipStream_t st) {
  const dim3 grid(p->grid), block(kThreads);
  if (p->rq == kRqFastNoTie)
    hipLaunchKernelGGL((DwRowsKernel<S, BOXSUM, kRqFastNoTie>), grid, block, p->lds_bytes, st, a);
  else if (p->rq == kRqFast)
    hipLaunchKernelGGL((DwRowsKernel<S, BOXSUM, kRqFast>), grid, block, p->lds_bytes, st, a);
  else
    hipLaunchKernelGGL((DwRowsKernel<S, BOXSUM, kRqGeneric>), grid, block, p->lds_bytes, st, a);
}

int DwRowsRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const RowsPlan* p = reinterpret_cast<const RowsPlan*>(op->host_blob.data());
  DwrArgs a = p->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if (p->stride == 1) {
    if (p->boxsum) LaunchRowsRq<1, true>(p, a, st); else LaunchRowsRq<1, false>(p, a, st);
  } else {
    if (p->boxsum) LaunchRowsRq<2, true>(p, a, st); else LaunchRowsRq<2, false>(p, a, st);
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

uint32_t Reciprocal(int d) {
  return d <= 1 ? 0u : static_cast<uint32_t>(((uint64_t{1} << 32) + d - 1) / d);
}

// The dword form of the kernel: 3x3, dilation 1, one stride (1 or 2) for both axes, rows of at
// least four bytes. Declines (TVX_E_UNSUPPORTED) what it does not cover.
int DwRowsSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (d->k_w != 3 || d->k_h != 3 || d->dilation_w != 1 || d->dilation_h != 1) return TVX_E_UNSUPPORTED;
  if (d->stride_w != d->stride_h || (d->stride_w != 1 && d->stride_w != 2)) return TVX_E_UNSUPPORTED;
  if (d->in_w < 4 || d->pad_left > 3) return TVX_E_UNSUPPORTED;
  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127) return TVX_E_UNSUPPORTED;
  const int S = d->stride_w, C = d->in_c;
  const long long planes = static_cast<long long>(d->batch) * C;
  const long long hwi = static_cast<long long>(d->in_w) * d->in_h, hwo = static_cast<long long>(d->out_w) * d->out_h;
  if (planes * C >= (1ll << 32)) return TVX_E_UNSUPPORTED;  // the channel of a plane comes from a 32-bit reciprocal
  RowsPlan p{};
  DwrArgs& a = p.a;
  a.C = C; a.H = d->in_h; a.W = d->in_w; a.OH = d->out_h; a.OW = d->out_w;
  a.pad_t = d->pad_top; a.pad_l = d->pad_left;
  a.planes = static_cast<int>(planes);
  a.ow4 = (a.OW + 3) / 4;
  // padded plane: the stencil of every work item (the last one of a row may overhang) reads inside it
  const long long pw4 = std::max<long long>(S * a.ow4 + 1, (a.pad_l + a.W + 3) / 4);
  a.oh2 = (a.OH + 1) / 2;
  const long long ph = std::max<long long>(static_cast<long long>(2 * a.oh2 - 1) * S + 3, a.pad_t + a.H);
  const long long plane_bytes = pw4 * 4 * ph;
  if (plane_bytes > 32 * 1024) return TVX_E_UNSUPPORTED;
  a.pw4 = static_cast<int>(pw4);
  a.ph = static_cast<int>(ph);
  // planes per workgroup: about 8 KiB of padded planes, but keep a thousand workgroups when there are enough planes
  long long g = std::max<long long>(1, 8192 / plane_bytes);
  g = std::min<long long>(g, std::max<long long>(1, planes / 1024));
  a.G = static_cast<int>(std::min<long long>(g, kThreads / kTabDwords));
  const long long grid = (planes + a.G - 1) / a.G;
  if (grid > 0x7fffffffll) return TVX_E_UNSUPPORTED;
  a.off_tab = static_cast<int>((a.G * pw4 * ph + 3) & ~3ll);  // tables are read as 16-byte records
  p.lds_bytes = (a.off_tab + a.G * kTabDwords) * 4;
  // 32-bit offsets inside a workgroup's planes, exact reciprocal divisions
  // offsets inside a workgroup's planes are formed with 24-bit multiplies; reciprocal divisions are exact
  // while dividend * divisor < 2^32
  const long long max_items = std::max<long long>(a.G * pw4 * ph, static_cast<long long>(a.G) * a.oh2 * a.ow4);
  if (a.G * std::max(hwi, hwo) >= (1ll << 23) || planes >= (1ll << 23) || C >= (1 << 23) ||
      max_items * std::max<long long>(pw4 * ph, static_cast<long long>(a.oh2) * a.ow4) >= (1ll << 32))
    return TVX_E_UNSUPPORTED;
  a.m_c = Reciprocal(C);
  a.m_plane4 = Reciprocal(static_cast<int>(pw4 * ph));
  a.m_pw4 = Reciprocal(a.pw4);
  a.m_ipp = Reciprocal(a.oh2 * a.ow4);
  a.m_ow4 = Reciprocal(a.ow4);
  std::vector<int32_t> wpk, biasf, rqt;
  p.boxsum = PackDepthwise3x3(C, w_host, w_u8, bias_host, zxs, zws, true, &wpk, &biasf);
  a.zws = zws;
  p.rq = BuildRequantRecords(op->h_mult, op->h_shift, C, C, d->out_zp, &rqt, AccumulatorBound(9, bias_host, C));
  int s = op->packed.Upload(wpk.data(), wpk.size() * 4);
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s != TVX_OK) return s;
  a.wpk = op->packed.as<int32_t>();
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<tvx_v4i>();
  a.xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.pad_fill = static_cast<int>(static_cast<uint32_t>(zxs & 0xff) * 0x01010101u);
  a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  if (op->out_blocked) {
    if (C % 16 || d->batch * hwo * C >= (1ll << 31) || d->batch * hwo >= (1ll << 23)) return TVX_E_UNSUPPORTED;
    a.out_blocked = 1;
    a.PO = static_cast<int>(d->batch * hwo);
  }
  p.stride = S;
  p.grid = static_cast<unsigned>(grid);
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&p), reinterpret_cast<const uint8_t*>(&p) + sizeof(p));
  op->run = DwRowsRun;
  op->kernel_name = op->out_blocked ? "dwconv_planes_to_blocked_i8" : "dwconv_planes_i8";
  return TVX_OK;
}

}  // namespace

// Claims quantized depthwise convolutions (multiplier 1, constant weights) whose planes
// are small enough for a few of them to sit in LDS.
int DwPlanesSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || d->multiplier != 1) return TVX_E_UNSUPPORTED;
  {
    const int s = DwRowsSetup(op, d, w_host, bias_host);
    if (s != TVX_E_UNSUPPORTED || op->out_blocked) return s;  // (only the dword form writes blocked results)
  }
  const uint64_t hwi = static_cast<uint64_t>(d->in_w) * d->in_h, hwo = static_cast<uint64_t>(d->out_w) * d->out_h;
  if (hwi == 0 || hwo == 0) return TVX_E_UNSUPPORTED;
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
  // padded plane: every tap of every work item (four outputs, the last item of a row may
  // overhang) reads inside it
  const long long need_w = static_cast<long long>(a.ow4 * 4 - 1) * a.sw + static_cast<long long>(a.kw - 1) * a.dw + 1;
  const long long need_h = static_cast<long long>(a.OH - 1) * a.sh + static_cast<long long>(a.kh - 1) * a.dh + 1;
  const long long pw = std::max<long long>(need_w, a.pad_l + a.W), ph = std::max<long long>(need_h, a.pad_t + a.H);
  if (pw * ph + static_cast<long long>(hwo) > 48 * 1024) return TVX_E_UNSUPPORTED;
  a.pw = static_cast<int>(pw);
  a.ph = static_cast<int>(ph);
  // planes per workgroup: about 10 KiB of LDS images, but leave a few workgroups per CU
  long long g = std::max<long long>(1, 10240 / (pw * ph + static_cast<long long>(hwo)));
  g = std::min<long long>(g, std::max<long long>(1, a.planes / 1024));
  a.G = static_cast<int>(std::min<long long>(g, 256));
  const long long grid = (a.planes + a.G - 1) / a.G;
  if (grid > 0x7fffffffll) return TVX_E_UNSUPPORTED;
  a.off_out = static_cast<int>((a.G * pw * ph + 15) & ~15ll);
  a.off_tab = a.off_out + static_cast<int>((a.G * hwo + 15 + 16) & ~15ull);
  p.lds_bytes = a.off_tab + a.G * (taps + 5) * 4;
  if (p.lds_bytes > 64 * 1024) return TVX_E_UNSUPPORTED;
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
  const bool k3 = d->k_w == 3 && d->k_h == 3 && d->dilation_w == 1 && d->dilation_h == 1 &&
                  d->stride_w == d->stride_h;
  p.mode = k3 && d->stride_w == 1 ? 1 : (k3 && d->stride_w == 2 ? 2 : 0);
  p.grid = static_cast<unsigned>(grid);
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&p), reinterpret_cast<const uint8_t*>(&p) + sizeof(p));
  op->run = DwPlanesRun;
  op->kernel_name = "dwconv_planes_i8";
  return TVX_OK;
}

}  // namespace tvx
