// Quantized MAX pooling at stride 2 with windows of 2 or 3 taps (the pooling of ResNet / MobileNet stems and
// of LeNet) as a register stencil: stands in for vxPoolingLayer2 as
// src/tim/vx/internal/src/ops/vsi_nn_op_pool.c:144-150 calls it, for the shapes the LDS-staged kernel of
// pool2d_i8.hip spends most of its instructions on index arithmetic for.
//
// A thread owns eight input columns (one 64-bit load per input row) and two output rows of one plane, i.e.
// 2 x 4 outputs. Nothing goes through LDS; the one column a 3-tap window needs from the neighbouring eight
// comes from the neighbouring lane by a wavefront shift. The maximum of unsigned bytes is taken two at a
// time on the 16-bit halves of even and odd bytes (v_pk_max_u16; signed codes are moved to unsigned order
// by a flipped sign bit): per input row one split, per output row the maximum down the window's rows and
// then across. Rows and columns outside the image never take part: a row index is clamped into the image
// (the clamped row belongs to the same window, so the maximum does not change), the one padding column is
// the neutral 0. With equal input and output quantization - the usual case - the maximum is the result.
#include <algorithm>
#include <cstdlib>

#include "variants.h"

namespace tvx {
namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerThread = 2;  // output rows

struct PoolStencilArgs {
  const uint8_t* x;
  uint8_t* y;
  int W, H, OW, OH;
  int pad_t;
  int lanes;         // W / 8: threads of an image row
  int lpr_shift;     // log2 of the lanes of a row rounded up to a power of two
  int row_groups;    // groups of kRowsPerThread output rows of a plane
  uint32_t units;    // planes x row groups: a unit is one row group of one plane, 2^lpr_shift threads wide
  uint32_t rg_magic; // unit / row_groups as ((t + ((unit - t) >> rg_sh1)) >> rg_sh2, t = mulhi(unit, rg_magic)
  int rg_sh1, rg_sh2;
  int identity;      // equal quantization on both sides: the maximum is the result
  int in_zp, out_zp, qmin, qmax, mult, shift;
};

__device__ __forceinline__ uint32_t PkMax(uint32_t x, uint32_t y) {
  uint32_t r;
  asm("v_pk_max_u16 %0, %1, %2" : "=v"(r) : "v"(x), "v"(y));
  return r;
}

// KW, KH: window; PL: left padding (0 or 1)
template <int KW, int KH, int PL, bool SIGNED>
__global__ void __launch_bounds__(kThreads) PoolStencilKernel(PoolStencilArgs a) {
  constexpr int R = kRowsPerThread;
  constexpr int ROWS = 2 * (R - 1) + KH;  // input rows behind the thread's output rows
  const int tid = threadIdx.x;
  const int w8 = tid & ((1 << a.lpr_shift) - 1);
  const uint32_t unit = blockIdx.x * (kThreads >> a.lpr_shift) + (tid >> a.lpr_shift);
  // (whole units leave together; a lane past the row's end only ever is the neighbour of a lane that takes the
  // neutral column instead)
  if (unit >= a.units || w8 >= a.lanes) return;
  const uint32_t t = __umulhi(unit, a.rg_magic);
  const uint32_t plane = (t + ((unit - t) >> a.rg_sh1)) >> a.rg_sh2;
  const int oh0 = static_cast<int>(unit - plane * static_cast<uint32_t>(a.row_groups)) * R;
  const uint8_t* xp = a.x + static_cast<size_t>(plane) * a.H * a.W;
  uint8_t* yp = a.y + static_cast<size_t>(plane) * a.OH * a.OW;

  // ---- all rows of the thread are requested before the first is used ----
  const int ih0 = oh0 * 2 - a.pad_t;
  uint2 raw[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const int ih = min(max(ih0 + r, 0), a.H - 1);
    raw[r] = *reinterpret_cast<const uint2*>(xp + (__umul24(static_cast<uint32_t>(ih), static_cast<uint32_t>(a.W)) + static_cast<uint32_t>(w8) * 8u));
  }
  // ---- per input row: even and odd bytes as 16-bit halves: ev = {c0 c2 | c4 c6}, od = {c1 c3 | c5 c7} ----
  uint32_t ev[ROWS][2], od[ROWS][2];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    uint32_t lo = raw[r].x, hi = raw[r].y;
    if (SIGNED) {
      lo ^= 0x80808080u;
      hi ^= 0x80808080u;
    }
    ev[r][0] = lo & 0x00ff00ffu;
    ev[r][1] = hi & 0x00ff00ffu;
    od[r][0] = __builtin_amdgcn_perm(0u, lo, 0x0c030c01u);  // {byte 1, 0, byte 3, 0}
    od[r][1] = __builtin_amdgcn_perm(0u, hi, 0x0c030c01u);
  }
  const bool has_left = w8 > 0, has_right = w8 + 1 < a.lanes;
#pragma unroll
  for (int o = 0; o < R; ++o) {
    // the maximum down the window's rows
    uint32_t e0 = ev[2 * o][0], e1 = ev[2 * o][1], d0 = od[2 * o][0], d1 = od[2 * o][1];
#pragma unroll
    for (int k = 1; k < KH; ++k) {
      e0 = PkMax(e0, ev[2 * o + k][0]);
      e1 = PkMax(e1, ev[2 * o + k][1]);
      d0 = PkMax(d0, od[2 * o + k][0]);
      d1 = PkMax(d1, od[2 * o + k][1]);
    }
    // ... and across: output e takes columns 2 e - PL .. 2 e - PL + KW - 1
    uint32_t o01, o23;
    if (PL == 0) {
      o01 = PkMax(e0, d0);  // {max(c0, c1), max(c2, c3)}
      o23 = PkMax(e1, d1);
      if (KW == 3) {
        // the third tap: c2, c4 | c6, c8 - c8 is the right neighbour's c0 (wave_shl:1), or nothing at the row's end
        const uint32_t nb = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(e0), 0x130, 0xf, 0xf, true));
        o01 = PkMax(o01, __builtin_amdgcn_alignbit(e1, e0, 16));
        o23 = PkMax(o23, __builtin_amdgcn_alignbit(has_right ? nb : 0u, e1, 16));
      }
    } else {
      // columns -1 .. : output e takes c(2e - 1), c(2e) and, with three taps, c(2e + 1); c(-1) is the left
      // neighbour's c7 (wave_shr:1), or nothing at the row's start
      const uint32_t nb = static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(d1), 0x138, 0xf, 0xf, true));
      o01 = PkMax(e0, __builtin_amdgcn_alignbit(d0, has_left ? nb : 0u, 16));  // {c-1, c1} against {c0, c2}
      o23 = PkMax(e1, __builtin_amdgcn_alignbit(d1, d0, 16));                   // {c3, c5} against {c4, c6}
      if (KW == 3) {
        o01 = PkMax(o01, d0);  // {c1, c3}
        o23 = PkMax(o23, d1);
      }
    }
    if (oh0 + o >= a.OH) break;
    uint32_t packed = __builtin_amdgcn_perm(o23, o01, 0x06040200u);  // the four low bytes of the halves
    if (SIGNED) packed ^= 0x80808080u;
    if (!a.identity) {
      int out[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t code = (packed >> (8 * e)) & 0xffu;
        const int v = SIGNED ? static_cast<int>(static_cast<int8_t>(code)) : static_cast<int>(code);
        out[e] = RequantClamp(v - a.in_zp, a.mult, a.shift, a.out_zp, a.qmin, a.qmax);
      }
      packed = PackBytes(out[0], out[1], out[2], out[3]);
    }
    uint8_t* dst = yp + (__umul24(static_cast<uint32_t>(oh0 + o), static_cast<uint32_t>(a.OW)) + static_cast<uint32_t>(w8) * 4u);
    const int n_out = a.OW - w8 * 4;  // outputs of this lane in the row (a row may end inside a lane's four)
    if (n_out >= 4) {
      __builtin_memcpy(dst, &packed, 4);  // (rows of an odd width start at any byte)
    } else {
#pragma unroll
      for (int e = 0; e < 3; ++e)
        if (e < n_out) dst[e] = static_cast<uint8_t>(packed >> (8 * e));
    }
  }
}

struct Plan {
  PoolStencilArgs a;
  int kw, kh, pl;
  bool is_signed;
  dim3 grid;
};

typedef void (*Fn)(PoolStencilArgs);
template <int KW, int KH>
Fn KernelOf2(int pl, bool is_signed) {
  if (pl == 0) return is_signed ? PoolStencilKernel<KW, KH, 0, true> : PoolStencilKernel<KW, KH, 0, false>;
  return is_signed ? PoolStencilKernel<KW, KH, 1, true> : PoolStencilKernel<KW, KH, 1, false>;
}
Fn KernelOf(const Plan* p) {
  if (p->kw == 2 && p->kh == 2) return KernelOf2<2, 2>(p->pl, p->is_signed);
  if (p->kw == 2 && p->kh == 3) return KernelOf2<2, 3>(p->pl, p->is_signed);
  if (p->kw == 3 && p->kh == 2) return KernelOf2<3, 2>(p->pl, p->is_signed);
  return KernelOf2<3, 3>(p->pl, p->is_signed);
}

int PoolStencilRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  PoolStencilArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if (reinterpret_cast<uintptr_t>(in0) & 7)
    return SetError(TVX_E_INVALID, "pool2d_stencil_i8: the input tensor must be 8-byte aligned");
  hipLaunchKernelGGL(KernelOf(plan), plan->grid, dim3(kThreads), 0, st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

}  // namespace

// Claims quantized MAX pooling with 2 or 3 taps per direction at stride 2, at most one padding row / column in
// front, rows of whole 8-byte units and at most four outputs per eight input columns.
int PoolStencilSetup(tvx_op* op) {
  const tvx_pool2d_desc& d = op->pool;
  if (!op->quantized || d.pool_type != TVX_POOL_MAX) return TVX_E_UNSUPPORTED;
  if ((d.k_w != 2 && d.k_w != 3) || (d.k_h != 2 && d.k_h != 3) || d.stride_w != 2 || d.stride_h != 2) return TVX_E_UNSUPPORTED;
  if (d.pad_left > 1 || d.pad_top > 1) return TVX_E_UNSUPPORTED;
  if (d.in_w % 8 || d.in_w > 512 || d.out_w * 2 > d.in_w || d.in_h >= (1u << 15)) return TVX_E_UNSUPPORTED;
  // every window starts on a row of the image (rows past the end are clamped onto rows of the same window)
  if (static_cast<int64_t>(d.out_h - 1) * 2 - static_cast<int64_t>(d.pad_top) > static_cast<int64_t>(d.in_h) - 1) return TVX_E_UNSUPPORTED;
  // (four outputs per eight input columns: no window reaches past the one padding column behind a row)
  if (const char* f = getenv("TVX_POOL_STENCIL")) if (atoi(f) == 0) return TVX_E_UNSUPPORTED;  // test lever: the LDS-staged kernel instead
  const uint64_t planes = static_cast<uint64_t>(d.channels) * d.batch;
  if (planes > 0x7fffffffull) return TVX_E_UNSUPPORTED;
  std::vector<int32_t> mult, shift;
  int s = BuildRequantTables(1, d.in_scale, 1.0f, nullptr, d.out_scale, &mult, &shift);
  if (s != TVX_OK) return s;
  Plan plan{};
  PoolStencilArgs& a = plan.a;
  a.W = d.in_w; a.H = d.in_h; a.OW = d.out_w; a.OH = d.out_h;
  a.pad_t = d.pad_top;
  a.lanes = a.W / 8;
  a.lpr_shift = 0;
  while ((1 << a.lpr_shift) < a.lanes) ++a.lpr_shift;
  a.row_groups = (a.OH + kRowsPerThread - 1) / kRowsPerThread;
  if (planes * static_cast<uint64_t>(a.row_groups) > 0x7fffffffull) return TVX_E_UNSUPPORTED;
  a.units = static_cast<uint32_t>(planes) * static_cast<uint32_t>(a.row_groups);
  {
    // division by an invariant (Granlund & Montgomery): exact for every 32-bit numerator
    int l = 0;
    while ((1u << l) < static_cast<uint32_t>(a.row_groups)) ++l;
    a.rg_magic = static_cast<uint32_t>(((static_cast<uint64_t>(1) << 32) * ((static_cast<uint64_t>(1) << l) - a.row_groups)) / a.row_groups + 1);
    a.rg_sh1 = std::min(l, 1);
    a.rg_sh2 = std::max(l - 1, 0);
  }
  const bool is_signed = d.dtype == TVX_I8;
  a.in_zp = d.in_zp; a.out_zp = d.out_zp;
  a.qmin = is_signed ? -128 : 0; a.qmax = is_signed ? 127 : 255;
  a.mult = mult[0]; a.shift = shift[0];
  a.identity = (mult[0] == (1 << 30) && shift[0] == 30 && d.in_zp == d.out_zp) ? 1 : 0;
  plan.kw = d.k_w; plan.kh = d.k_h; plan.pl = d.pad_left;
  plan.is_signed = is_signed;
  const uint32_t units_per_block = kThreads >> a.lpr_shift;
  plan.grid = dim3((a.units + units_per_block - 1) / units_per_block);
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = PoolStencilRun;
  op->kernel_name = "pool2d_stencil_i8";
  return TVX_OK;
}

}  // namespace tvx
