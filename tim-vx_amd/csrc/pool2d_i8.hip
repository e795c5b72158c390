// Quantized Pool2d (MAX / AVG / AVG_ANDROID on uint8 and int8 planes) for windows two or three taps
// wide: stands in for vxPoolingLayer2 as src/tim/vx/internal/src/ops/vsi_nn_op_pool.c:144-150 calls it.
//
// Pooling moves bytes and does next to no arithmetic, so the kernel is built around memory:
//  * A workgroup takes a band of output rows of one plane, or several whole small planes. What it
//    needs from the input is one contiguous byte range per plane; the range is read exactly once,
//    as aligned dwords in lane order (a wavefront instruction fetches 256 contiguous bytes).
//  * The bytes go into an LDS image of the padded planes: row pitch a multiple of four, left /
//    top / right / bottom padding cells pre-filled with the operator's neutral code (the smallest
//    code for MAX, the input zero point for the averages), so that no tap is ever tested against
//    the image border.
//  * A thread produces four neighbouring outputs of a row. Their windows start at LDS columns
//    4 j * stride, always dword-aligned: it reads two or three aligned dwords per window row,
//    reduces them in registers with constant byte positions and stores one dword.
// The arithmetic is that of the generic kernel: MAX on codes, then the Q31 requantization of
// (max - z_in); averages as rint((double)(sum - n z_in) * (s_in / s_out) / divisor) + z_out.
#include <algorithm>
#include <cstdlib>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kBandBytesDefault = 16 * 1024;  // LDS image a workgroup aims for

struct PoolRowsArgs {
  const uint8_t* x;
  uint8_t* y;
  int W, H, OW, OH;
  int kh, sh, pad_l, pad_t;
  int planes;          // batch * channels
  int G;               // planes per workgroup
  int RB;              // output rows per workgroup (per plane)
  int bands;           // row bands per plane
  int rows_in;         // LDS rows per plane: (RB - 1) * sh + kh
  int pitch;           // LDS row pitch in bytes (multiple of 4)
  int ow4;             // groups of four outputs per row
  int fill;            // neutral code in all four bytes
  int in_zp, out_zp, qmin, qmax, mult, shift;
  int identity;        // input and output scales are equal: requantization only moves the zero point
  double ratio;
  uint32_t magic_w;    // ceil(2^32 / W)
  uint32_t magic_plane;  // ceil(2^32 / (W * H))
  uint32_t magic_ow4, magic_oh;
};

// maximum of the two unsigned 16-bit halves, each on its own
__device__ __forceinline__ uint32_t PkMaxU16(uint32_t x, uint32_t y) {
  uint32_t r;
  asm("v_pk_max_u16 %0, %1, %2" : "=v"(r) : "v"(x), "v"(y));
  return r;
}

__device__ __forceinline__ uint32_t DivMagic(uint32_t v, uint32_t magic, uint32_t d) {
  // floor(v / d) for v * d < 2^32 (magic = ceil(2^32 / d)); d == 1 has magic 0
  return d == 1 ? v : __umulhi(v, magic);
}

// Four neighbouring outputs per thread from the LDS image `lds` of g_n planes (rows oh0 .. oh0 + rb - 1 of each).
template <int KW, int SW, bool SIGNED, int TYPE>
__device__ __forceinline__ void PoolOutputs(const PoolRowsArgs& a, const uint8_t* lds, int p0, int g_n, int oh0, int rb,
                                            int plane_lds, int tid) {
  constexpr int NB = 3 * SW + KW;          // window bytes of four neighbouring outputs
  constexpr int NDW = (NB + 3) / 4;
  const int items = g_n * rb * a.ow4;
  for (int it = tid; it < items; it += kThreads) {
    // (several planes per workgroup only where a plane is one band: rb == OH then)
    const int row_all = static_cast<int>(DivMagic(it, a.magic_ow4, a.ow4));
    const int j = it - row_all * a.ow4;
    const int g = g_n > 1 ? static_cast<int>(DivMagic(row_all, a.magic_oh, a.OH)) : 0;
    const int orow = row_all - g * rb;
    const uint8_t* win = lds + g * plane_lds + orow * a.sh * a.pitch + j * 4 * SW;
    int acc[4];
    if (TYPE == TVX_POOL_MAX && SW == 2) {
      // Stride 2: output e takes bytes 2 e .. 2 e + KW - 1 of the window. The maximum down the window's rows is
      // taken on 16-bit halves, even and odd bytes apart (two bytes per instruction; signed codes are moved to
      // unsigned order first), then across: max(even[e], odd[e]) and, for three taps, even[e + 1].
      uint32_t ev[NDW], od[NDW];
#pragma unroll
      for (int q = 0; q < NDW; ++q) ev[q] = od[q] = 0;
      for (int ky = 0; ky < a.kh; ++ky) {
#pragma unroll
        for (int q = 0; q < NDW; ++q) {
          uint32_t d = reinterpret_cast<const uint32_t*>(win + ky * a.pitch)[q];
          if (SIGNED) d ^= 0x80808080u;
          ev[q] = PkMaxU16(ev[q], d & 0x00ff00ffu);
          od[q] = PkMaxU16(od[q], (d >> 8) & 0x00ff00ffu);
        }
      }
      // ev[q] = {byte 4 q, byte 4 q + 2} = even[2 q], even[2 q + 1]; od[q] likewise
      uint32_t m01 = PkMaxU16(ev[0], od[0]), m23 = PkMaxU16(ev[1], od[1]);
      if (KW == 3) {
        const uint32_t e12 = __builtin_amdgcn_alignbit(ev[1], ev[0], 16);          // even[1], even[2]
        const uint32_t e34 = __builtin_amdgcn_alignbit(NDW > 2 ? ev[NDW - 1] : 0u, ev[1], 16);  // even[3], even[4]
        m01 = PkMaxU16(m01, e12);
        m23 = PkMaxU16(m23, e34);
      }
      const int bias = SIGNED ? 128 : 0;
      acc[0] = static_cast<int>(m01 & 0xffffu) - bias;
      acc[1] = static_cast<int>(m01 >> 16) - bias;
      acc[2] = static_cast<int>(m23 & 0xffffu) - bias;
      acc[3] = static_cast<int>(m23 >> 16) - bias;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = TYPE == TVX_POOL_MAX ? INT32_MIN : 0;
      for (int ky = 0; ky < a.kh; ++ky) {
        uint32_t d[NDW];
#pragma unroll
        for (int q = 0; q < NDW; ++q) d[q] = reinterpret_cast<const uint32_t*>(win + ky * a.pitch)[q];
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int kx = 0; kx < KW; ++kx) {
            const int b = e * SW + kx;
            const uint32_t raw = (d[b >> 2] >> ((b & 3) * 8)) & 0xffu;
            const int v = SIGNED ? static_cast<int>(static_cast<int8_t>(raw)) : static_cast<int>(raw);
            acc[e] = TYPE == TVX_POOL_MAX ? max(acc[e], v) : acc[e] + v;
          }
      }
    }
    const int oh = oh0 + orow;
    int out[4];
    if (TYPE == TVX_POOL_MAX && a.identity) {
      // equal input and output scales: the requantization multiplies by one (every window holds a tap of the
      // image: the padding is narrower than the window)
#pragma unroll
      for (int e = 0; e < 4; ++e) out[e] = Med3(acc[e] - a.in_zp + a.out_zp, a.qmin, a.qmax);
    } else {
      const int ih0 = oh * a.sh - a.pad_t;
      const int ny = min(ih0 + a.kh, a.H) - max(ih0, 0);  // rows of the window inside the image
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        long long r = 0;
        if (TYPE == TVX_POOL_MAX) {
          r = RequantRne(acc[e] - a.in_zp, a.mult, a.shift);
        } else {
          int div = KW * a.kh;
          if (TYPE == TVX_POOL_AVG_ANDROID) {
            const int iw0 = (j * 4 + e) * SW - a.pad_l;
            div = max(min(iw0 + KW, a.W) - max(iw0, 0), 0) * max(ny, 0);
          }
          // the padding cells hold the zero point: the sum over all cells minus their zero points is the sum over the taps inside
          const int sum = acc[e] - KW * a.kh * a.in_zp;
          if (div) r = static_cast<long long>(rint(static_cast<double>(sum) * a.ratio / static_cast<double>(div)));
        }
        r += a.out_zp;
        out[e] = static_cast<int>(r < a.qmin ? a.qmin : (r > a.qmax ? a.qmax : r));
      }
    }
    uint8_t* dst = a.y + (static_cast<size_t>(p0 + g) * a.OH + oh) * a.OW + j * 4;
    if ((a.OW & 3) == 0) {
      *reinterpret_cast<uint32_t*>(dst) = PackBytes(out[0], out[1], out[2], out[3]);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (j * 4 + e < a.OW) dst[e] = static_cast<uint8_t>(out[e]);
    }
  }
}

template <int KW, int SW, bool SIGNED, int TYPE>
__global__ void __launch_bounds__(kThreads) PoolRowsKernel(PoolRowsArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x;
  const int band = blockIdx.x % a.bands;
  const int p0 = (blockIdx.x / a.bands) * a.G;
  const int g_n = min(a.G, a.planes - p0);
  const int oh0 = band * a.RB;
  const int rb = min(a.RB, a.OH - oh0);
  const int ih_first = oh0 * a.sh - a.pad_t;                 // input row of LDS row 0 (may be negative)
  const int rows_in = (rb - 1) * a.sh + a.kh;
  const int ih_lo = max(ih_first, 0), ih_hi = min(ih_first + rows_in, a.H);  // rows that exist
  const int plane_lds = a.rows_in * a.pitch;

  // ---- neutral fill of the whole LDS image ------------------------------------------------
  {
    const int chunks = (g_n * plane_lds + 15) >> 4;
    const v4i f = v4i{a.fill, a.fill, a.fill, a.fill};
    for (int c = tid; c < chunks; c += kThreads) reinterpret_cast<v4i*>(lds)[c] = f;
  }
  __syncthreads();
  // ---- the input rows: per plane one contiguous range, read as aligned dwords ---------------------
  const uint32_t plane_bytes = static_cast<uint32_t>(a.H) * static_cast<uint32_t>(a.W);
  if (ih_lo == 0 && ih_hi == a.H && (a.W & 3) == 0 && (a.pad_l & 3) == 0 && a.magic_plane != 0 &&
      ((reinterpret_cast<uintptr_t>(a.x) + static_cast<size_t>(p0) * plane_bytes) & 15) == 0 && ((static_cast<size_t>(g_n) * plane_bytes) & 15) == 0) {
    // Whole planes of whole dwords: the workgroup's planes are one contiguous range. It is read as 16-byte chunks
    // in lane order, every thread's loads issued before the first is used - plane by plane (below) small planes
    // cost one memory round trip each.
    const uint32_t row_bytes = static_cast<uint32_t>(a.W);
    const uint32_t n16 = static_cast<uint32_t>(g_n) * plane_bytes >> 4;
    const v4i* src16 = reinterpret_cast<const v4i*>(a.x + static_cast<size_t>(p0) * plane_bytes);
    uint8_t* dst0 = lds + (0 - ih_first) * a.pitch + a.pad_l;
    auto put16 = [&](uint32_t i, const v4i& v) {
      const uint32_t o = i << 4;
      const uint32_t g = __umulhi(o, a.magic_plane);
      const uint32_t po = o - g * plane_bytes;
      uint32_t r = DivMagic(po, a.magic_w, row_bytes);
      uint32_t c = po - r * row_bytes;
      uint8_t* dst_plane = dst0 + g * plane_lds;
      uint32_t gg = g;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        *reinterpret_cast<uint32_t*>(dst_plane + r * a.pitch + c) = static_cast<uint32_t>(v[q]);
        c += 4;
        if (c == row_bytes) {
          c = 0;
          if (++r == static_cast<uint32_t>(a.H)) { r = 0; ++gg; dst_plane = dst0 + gg * plane_lds; }  // (a chunk may run into the next plane)
        }
      }
    };
    constexpr int kInFlight = 4;
    for (uint32_t i0 = tid; i0 < n16; i0 += kInFlight * kThreads) {
      v4i v[kInFlight];
#pragma unroll
      for (int k = 0; k < kInFlight; ++k) v[k] = src16[min(i0 + k * kThreads, n16 - 1)];
#pragma unroll
      for (int k = 0; k < kInFlight; ++k)
        if (i0 + k * kThreads < n16) put16(i0 + k * kThreads, v[k]);
    }
  } else if (ih_hi > ih_lo) {
    const uint32_t row_bytes = static_cast<uint32_t>(a.W);
    const uint32_t range = static_cast<uint32_t>(ih_hi - ih_lo) * row_bytes;  // bytes per plane
    for (int g = 0; g < g_n; ++g) {
      const size_t start = (static_cast<size_t>(p0 + g) * a.H + ih_lo) * row_bytes;  // byte offset in the tensor
      const uint32_t head = static_cast<uint32_t>((4 - ((reinterpret_cast<uintptr_t>(a.x) + start) & 3)) & 3);  // bytes before the first aligned dword
      uint8_t* dst_plane = lds + g * plane_lds + (ih_lo - ih_first) * a.pitch + a.pad_l;
      auto put = [&](uint32_t o, uint32_t v) {  // byte at offset o of the range
        const uint32_t r = DivMagic(o, a.magic_w, row_bytes);
        dst_plane[r * a.pitch + (o - r * row_bytes)] = static_cast<uint8_t>(v);
      };
      // head and tail bytes one by one, whole dwords in between
      const uint32_t h = min(head, range);
      if (tid < static_cast<int>(h)) put(tid, a.x[start + tid]);
      const uint32_t ndw = (range - h) >> 2;
      const uint32_t tail0 = h + (ndw << 2);
      if (tid >= 32 && tid - 32 < static_cast<int>(range - tail0)) put(tail0 + (tid - 32), a.x[start + tail0 + (tid - 32)]);
      const uint32_t* src = reinterpret_cast<const uint32_t*>(a.x + start + h);
      if (h == 0 && (row_bytes & 3) == 0 && (a.pad_l & 3) == 0 && ((reinterpret_cast<uintptr_t>(a.x) + start) & 15) == 0) {
        // rows of whole dwords that land on LDS dwords: 16 bytes per lane and load, two loads in flight
        const uint32_t n16 = ndw >> 2;
        const v4i* src16 = reinterpret_cast<const v4i*>(src);
        auto put16 = [&](uint32_t i, const v4i& v) {
          const uint32_t o = i << 4;
          uint32_t r = DivMagic(o, a.magic_w, row_bytes);
          uint32_t c = o - r * row_bytes;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            *reinterpret_cast<uint32_t*>(dst_plane + r * a.pitch + c) = static_cast<uint32_t>(v[q]);
            c += 4;
            if (c == row_bytes) { c = 0; ++r; }
          }
        };
        uint32_t i = tid;
        for (; i + kThreads < n16; i += 2 * kThreads) {
          const v4i v0 = src16[i], v1 = src16[i + kThreads];
          put16(i, v0);
          put16(i + kThreads, v1);
        }
        if (i < n16) put16(i, src16[i]);
        for (uint32_t k = (n16 << 2) + tid; k < ndw; k += kThreads) {  // up to three dwords behind the last chunk
          const uint32_t o = k << 2;
          const uint32_t r = DivMagic(o, a.magic_w, row_bytes);
          *reinterpret_cast<uint32_t*>(dst_plane + r * a.pitch + (o - r * row_bytes)) = src[k];
        }
        continue;
      }
      for (uint32_t i = tid; i < ndw; i += kThreads) {
        const uint32_t v = src[i];
        const uint32_t o = h + (i << 2);
        uint32_t r = DivMagic(o, a.magic_w, row_bytes);
        uint32_t c = o - r * row_bytes;
        if (c + 3 < row_bytes && ((a.pad_l + c) & 3) == 0 && (a.pitch & 3) == 0) {
          *reinterpret_cast<uint32_t*>(dst_plane + r * a.pitch + c) = v;  // one row, aligned in LDS
        } else {
#pragma unroll
          for (int b = 0; b < 4; ++b) {
            dst_plane[r * a.pitch + c] = static_cast<uint8_t>(v >> (8 * b));
            if (++c == row_bytes) { c = 0; ++r; }
          }
        }
      }
    }
  }
  __syncthreads();
  PoolOutputs<KW, SW, SIGNED, TYPE>(a, lds, p0, g_n, oh0, rb, plane_lds, tid);
}

// Whole planes, several per step, with the loads of the next step in flight while this one is reduced: a
// workgroup walks its share of the plane groups through two LDS images. The padding cells are the same in
// every step and are filled once. Needs rows of whole dwords that land on LDS dwords and plane groups that
// start on 16-byte boundaries (at most kChunks 16-byte loads per thread and step).
constexpr int kChunks = 4;

template <int KW, int SW, bool SIGNED, int TYPE>
__global__ void __launch_bounds__(kThreads) PoolPlanesKernel(PoolRowsArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x;
  const int plane_lds = a.rows_in * a.pitch;
  const int image = (a.G * plane_lds + 15) / 16 * 16;
  const int steps = (a.planes + a.G - 1) / a.G;
  const uint32_t row_bytes = static_cast<uint32_t>(a.W);
  const uint32_t plane_bytes = static_cast<uint32_t>(a.H) * row_bytes;
  {
    const v4i f = v4i{a.fill, a.fill, a.fill, a.fill};
    for (int c = tid; c < (2 * image) >> 4; c += kThreads) reinterpret_cast<v4i*>(lds)[c] = f;
  }
  v4i d[kChunks];
  auto issue = [&](int step) {
    const int p0 = step * a.G;
    const uint32_t n16 = static_cast<uint32_t>(min(a.G, a.planes - p0)) * plane_bytes >> 4;
    const v4i* src = reinterpret_cast<const v4i*>(a.x + static_cast<size_t>(p0) * plane_bytes);
#pragma unroll
    for (int q = 0; q < kChunks; ++q) {
      const uint32_t i = tid + q * kThreads;
      d[q] = src[min(i, n16 - 1)];  // chunks past the end re-read the last one and are dropped
    }
  };
  auto scatter = [&](int step, uint8_t* img) {
    const int p0 = step * a.G;
    const uint32_t n16 = static_cast<uint32_t>(min(a.G, a.planes - p0)) * plane_bytes >> 4;
    uint8_t* dst = img + a.pad_t * a.pitch + a.pad_l;
#pragma unroll
    for (int q = 0; q < kChunks; ++q) {
      const uint32_t i = tid + q * kThreads;
      if (i >= n16) continue;
      const uint32_t o = i << 4;
      const uint32_t g = DivMagic(o, a.magic_plane, plane_bytes);
      const uint32_t in_plane = o - g * plane_bytes;
      uint32_t r = DivMagic(in_plane, a.magic_w, row_bytes);
      uint32_t c = in_plane - r * row_bytes;
      uint8_t* pl = dst + g * plane_lds;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        *reinterpret_cast<uint32_t*>(pl + r * a.pitch + c) = static_cast<uint32_t>(d[q][w]);
        c += 4;
        if (c == row_bytes) {
          c = 0;
          if (++r == static_cast<uint32_t>(a.H)) { r = 0; pl += plane_lds; }
        }
      }
    }
  };
  int step = blockIdx.x;
  if (step >= steps) return;
  issue(step);
  __syncthreads();  // the fill is complete
  int buf = 0;
  for (; step < steps; step += gridDim.x) {
    uint8_t* img = lds + buf * image;
    scatter(step, img);
    // this wavefront's LDS stores only: the previous step's global stores need not have completed
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const int next = step + gridDim.x;
    if (next < steps) issue(next);
    const int p0 = step * a.G;
    PoolOutputs<KW, SW, SIGNED, TYPE>(a, img, p0, min(a.G, a.planes - p0), 0, a.OH, plane_lds, tid);
    buf ^= 1;
  }
}

struct Plan {
  PoolRowsArgs a;
  int lds_bytes, kw, sw, type;
  bool is_signed;
  bool pipelined;  // PoolPlanesKernel
  dim3 grid;
};

typedef void (*PoolFn)(PoolRowsArgs);

template <int KW, int SW, bool SIGNED, int TYPE>
PoolFn KernelOf3(bool pipelined) {
  return pipelined ? PoolPlanesKernel<KW, SW, SIGNED, TYPE> : PoolRowsKernel<KW, SW, SIGNED, TYPE>;
}

template <int KW, int SW>
PoolFn KernelOf(bool is_signed, int type, bool pl) {
  if (type == TVX_POOL_MAX) return is_signed ? KernelOf3<KW, SW, true, TVX_POOL_MAX>(pl) : KernelOf3<KW, SW, false, TVX_POOL_MAX>(pl);
  if (type == TVX_POOL_AVG) return is_signed ? KernelOf3<KW, SW, true, TVX_POOL_AVG>(pl) : KernelOf3<KW, SW, false, TVX_POOL_AVG>(pl);
  return is_signed ? KernelOf3<KW, SW, true, TVX_POOL_AVG_ANDROID>(pl) : KernelOf3<KW, SW, false, TVX_POOL_AVG_ANDROID>(pl);
}

PoolFn Kernel(const Plan* p) {
  if (p->kw == 2 && p->sw == 1) return KernelOf<2, 1>(p->is_signed, p->type, p->pipelined);
  if (p->kw == 2 && p->sw == 2) return KernelOf<2, 2>(p->is_signed, p->type, p->pipelined);
  if (p->kw == 3 && p->sw == 1) return KernelOf<3, 1>(p->is_signed, p->type, p->pipelined);
  if (p->kw == 3 && p->sw == 2) return KernelOf<3, 2>(p->is_signed, p->type, p->pipelined);
  return nullptr;
}

int PoolRowsRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  PoolRowsArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if ((a.OW & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 3))
    return SetError(TVX_E_INVALID, "pool2d_rows_i8: the output tensor must be 4-byte aligned");
  if (plan->pipelined && (reinterpret_cast<uintptr_t>(in0) & 15))
    return SetError(TVX_E_INVALID, "pool2d_rows_i8: the input tensor must be 16-byte aligned");
  hipLaunchKernelGGL(Kernel(plan), plan->grid, dim3(kThreads), plan->lds_bytes, st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

}  // namespace

// Claims quantized pooling with windows two or three taps wide at stride one or two (the window height and
// the vertical stride are free).
int PoolRowsSetup(tvx_op* op) {
  const tvx_pool2d_desc& d = op->pool;
  if (!op->quantized || d.pool_type == TVX_POOL_L2) return TVX_E_UNSUPPORTED;  // (L2: the generic kernel)
  if ((d.k_w != 2 && d.k_w != 3) || (d.stride_w != 1 && d.stride_w != 2) || d.k_h > 16 || d.stride_h > 16)
    return TVX_E_UNSUPPORTED;
  if (d.pad_left >= d.k_w || d.pad_top >= d.k_h) return TVX_E_UNSUPPORTED;
  // an average over the whole plane has a kernel of its own (one wavefront share per plane)
  if (d.pool_type != TVX_POOL_MAX && d.out_w == 1 && d.out_h == 1 && d.k_w == d.in_w && d.k_h == d.in_h &&
      d.pad_left == 0 && d.pad_top == 0)
    return TVX_E_UNSUPPORTED;
  if (d.in_w >= (1u << 15) || d.in_h >= (1u << 15) || d.out_w >= (1u << 15)) return TVX_E_UNSUPPORTED;
  std::vector<int32_t> mult, shift;
  int s = BuildRequantTables(1, d.in_scale, 1.0f, nullptr, d.out_scale, &mult, &shift);
  if (s != TVX_OK) return s;
  PoolRowsArgs a{};
  a.W = d.in_w; a.H = d.in_h; a.OW = d.out_w; a.OH = d.out_h;
  a.kh = d.k_h; a.sh = d.stride_h; a.pad_l = d.pad_left; a.pad_t = d.pad_top;
  const uint64_t planes = static_cast<uint64_t>(d.channels) * d.batch;
  if (planes > 0x7fffffffull) return TVX_E_UNSUPPORTED;
  a.planes = static_cast<int>(planes);
  a.ow4 = (a.OW + 3) / 4;
  // LDS row: left padding, the row, and whatever the last group of four windows reaches
  const int reach = (a.ow4 * 4 - 1) * static_cast<int>(d.stride_w) + static_cast<int>(d.k_w);
  a.pitch = (std::max(reach, a.pad_l + a.W) + 3 + 4) / 4 * 4;  // + 4: the last window reads whole dwords
  int kBandBytes = kBandBytesDefault;
  if (const char* f = getenv("TVX_POOL_BAND_KB")) kBandBytes = std::max(4, std::min(60, atoi(f))) * 1024;  // tuning aid
  // rows per band: the whole plane if its padded image fits the budget, else as many rows as do
  const int rows_all = (a.OH - 1) * a.sh + a.kh;
  int rb = a.OH;
  if (rows_all * a.pitch > kBandBytes) rb = std::max(1, (kBandBytes / a.pitch - a.kh) / a.sh + 1);
  rb = std::min(rb, a.OH);
  a.RB = rb;
  a.bands = (a.OH + rb - 1) / rb;
  a.rows_in = (rb - 1) * a.sh + a.kh;
  const int plane_lds = a.rows_in * a.pitch;
  a.G = a.bands == 1 ? std::max(1, std::min<int>(kBandBytes / plane_lds, 64)) : 1;
  // enough workgroups for the chip before fattening them
  while (a.G > 1 && (planes + a.G - 1) / a.G < 1024) a.G = (a.G + 1) / 2;
  const int lds_bytes = (a.G * plane_lds + 15) / 16 * 16 + 16;
  if (lds_bytes > 64 * 1024) return TVX_E_UNSUPPORTED;
  const bool is_signed = d.dtype == TVX_I8;
  const int neutral = d.pool_type == TVX_POOL_MAX ? (is_signed ? 0x80 : 0x00) : (d.in_zp & 0xff);
  a.fill = static_cast<int>(static_cast<uint32_t>(neutral) * 0x01010101u);
  a.in_zp = d.in_zp; a.out_zp = d.out_zp;
  a.qmin = is_signed ? -128 : 0; a.qmax = is_signed ? 127 : 255;
  a.mult = mult[0]; a.shift = shift[0];
  a.identity = (mult[0] == (1 << 30) && shift[0] == 30) ? 1 : 0;
  a.ratio = static_cast<double>(d.in_scale) / static_cast<double>(d.out_scale);
  a.magic_w = a.W <= 1 ? 0u : static_cast<uint32_t>(((uint64_t{1} << 32) + a.W - 1) / a.W);
  a.magic_ow4 = a.ow4 <= 1 ? 0u : static_cast<uint32_t>(((uint64_t{1} << 32) + a.ow4 - 1) / a.ow4);
  a.magic_oh = a.OH <= 1 ? 0u : static_cast<uint32_t>(((uint64_t{1} << 32) + a.OH - 1) / a.OH);
  {
    // plane index of a byte offset inside a workgroup's planes (offsets below G * plane bytes; exact while offset * plane bytes < 2^32)
    const uint64_t pb = static_cast<uint64_t>(a.W) * a.H;
    a.magic_plane = (pb > 1 && pb * pb * static_cast<uint64_t>(a.G) < (1ull << 32)) ? static_cast<uint32_t>(((uint64_t{1} << 32) + pb - 1) / pb) : 0u;
  }
  // (a workgroup's items fit its LDS image, fewer than 2^14, and OH, ow4 < 2^15: the products stay below 2^32)
  // the byte offsets divided by W stay below 2^32 / W: a band holds at most rows_in * W < 2^30 bytes
  if (static_cast<uint64_t>(a.rows_in) * a.W * a.W >= (1ull << 32)) return TVX_E_UNSUPPORTED;
  const uint64_t wgs = ((planes + a.G - 1) / a.G) * a.bands;
  if (wgs > 0x7fffffffull) return TVX_E_UNSUPPORTED;
  Plan plan{};
  plan.lds_bytes = lds_bytes;
  plan.kw = d.k_w; plan.sw = d.stride_w; plan.type = d.pool_type;
  plan.is_signed = is_signed;
  plan.grid = dim3(static_cast<unsigned>(wgs));
  // Whole planes with dword-friendly rows: the pipelined kernel. Its plane groups hold at most kChunks 16-byte
  // chunks per thread and start on 16-byte boundaries.
  bool pipelined = a.bands == 1 && (a.W & 3) == 0 && (a.pad_l & 3) == 0;
  if (const char* f = getenv("TVX_POOL_PIPELINED")) pipelined = pipelined && atoi(f) != 0;  // tuning aid
  if (pipelined) {
    const uint64_t plane_bytes = static_cast<uint64_t>(a.W) * a.H;
    int g = static_cast<int>(std::min<uint64_t>(std::max<uint64_t>(1, kChunks * kThreads * 16 / plane_bytes), 64));
    g = std::min(g, std::max(1, kBandBytes / (std::max((a.OH - 1) * a.sh + a.kh, a.pad_t + a.H) * a.pitch)));
    while (g > 1 && ((plane_bytes * g) & 15)) --g;
    const uint64_t steps = (planes + g - 1) / g;
    pipelined = ((plane_bytes * g) & 15) == 0 && ((plane_bytes & 15) == 0 || planes % g == 0) &&
                plane_bytes * g <= static_cast<uint64_t>(kChunks) * kThreads * 16 &&
                plane_bytes * plane_bytes * g < (1ull << 32) && steps >= 512;
    // the pipelined plan is worked out aside and taken over only if it stands: its two LDS images must fit 64 KiB
    const int rows_in = std::max((a.OH - 1) * a.sh + a.kh, a.pad_t + a.H);  // every row of a plane is stored (with FLOOR rounding the last ones may lie below the last window)
    const int lds2 = 2 * ((g * rows_in * a.pitch + 15) / 16 * 16) + 16;
    if (pipelined && lds2 > 64 * 1024) pipelined = false;
    if (pipelined) {
      hipDeviceProp_t prop;
      int dev = 0;
      if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return SetError(TVX_E_DEVICE, "no device properties");
      int wg = 3 * prop.multiProcessorCount;
      if (const char* f = getenv("TVX_POOL_WGS")) wg = std::max(1, atoi(f));  // tuning aid
      a.G = g;
      a.magic_plane = plane_bytes <= 1 ? 0u : static_cast<uint32_t>(((uint64_t{1} << 32) + plane_bytes - 1) / plane_bytes);
      a.rows_in = rows_in;
      plan.grid = dim3(static_cast<unsigned>(std::min<uint64_t>(steps, wg)));
      plan.lds_bytes = lds2;
    }
  }
  plan.pipelined = pipelined;
  plan.a = a;
  if (!Kernel(&plan)) return TVX_E_UNSUPPORTED;
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = PoolRowsRun;
  op->kernel_name = "pool2d_rows_i8";
  return TVX_OK;
}

}  // namespace tvx
