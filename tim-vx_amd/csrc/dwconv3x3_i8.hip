// Depthwise 3x3 quantized convolution (multiplier 1) in WHCN: every (image,
// channel) plane is an independent 2-D stencil, so the kernel streams planes
// through registers at memory speed and never touches the matrix cores.
//
// A thread owns a 4-column x 4-row patch of one plane's output; it issues all
// loads of the input rows behind the patch up front: per row only the dword(s)
// under its own columns - the dword on either side comes from the neighbouring
// lane by a wavefront shift (DPP), an image row occupying a power-of-two number
// of lanes so that it never straddles two wavefronts. The thread cuts the four
// 3-byte windows out of them with v_alignbyte and feeds each window to three
// v_dot4 (one per kernel row, weights of a kernel row packed in one register). Rows above / below the image and columns left / right
// of it read as the input zero point, so the zero-point expansion
//   sum (x - zx)(w - zw) = sum xs ws - zws * Sx - zxs * Sw + 9 zxs zws
// only needs the window sum Sx when the weight zero point is non-zero (one
// more v_dot4 with ones per window and kernel row) - and then only for the few
// channels whose shifted weights ws - zws do not fit int8: for all others the
// shifted weights are packed instead and the Sx term vanishes. The channel
// constants are folded into the bias at creation. Requantization is the exact fixed-point
// one of the other kernels; four results are packed into one dword store.
#include <algorithm>

#include "variants.h"

namespace tvx {
namespace {

constexpr int kThreads = 256;

struct DwArgs {
  const uint8_t* x;
  uint8_t* y;
  const int32_t* wpk;    // per channel: 4 dwords: kernel row ky = bytes (w[ky][0], w[ky][1], w[ky][2], 0) int8 for
                         // ky = 0..2, then 1 when the channel needs the window sum (see the setup function)
  const int32_t* biasf;  // per channel: bias - zxs * Sw + 9 zxs zws
  const tvx_v4i* rq;     // per channel requantization record
  int C, H, W, OH, OW;
  int pad_t, pad_l;
  int ow4;               // output dwords per row
  int lpr_shift;         // log2 of the lanes an image row occupies (>= ow4 lanes, the rest idle)
  int rg_per_block;      // row groups (of RPT output rows) per workgroup
  int xor_mask, pad_fill, zws, out_zp, lo, hi;
};



// Four accumulators of the channel -> four codes in one dword. Where no accumulator can land on a tie the clamp
// comes in front of the shift (bounds shifted up: `lo_t`, `hi_t`), and the shift writes its byte of the dword: no
// packing instructions.
template <int RQ>
__device__ __forceinline__ uint32_t Requant4(const int (&acc)[4], const tvx_v4i& q, int t_v, int lo_t, int hi_t, int out_zp,
                                             int lo, int hi) {
  if (RQ == kRqFastNoTie) {
    int u[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) u[e] = Med3(__mulhi(acc[e], q[0]) + q[2], lo_t, hi_t);
    uint32_t d;
    ShiftIntoByte<0>(d, t_v, u[0]);
    ShiftIntoByte<1>(d, t_v, u[1]);
    ShiftIntoByte<2>(d, t_v, u[2]);
    ShiftIntoByte<3>(d, t_v, u[3]);
    return d;
  }
  int r[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] = Requant8<RQ>(acc[e], q, out_zp, lo, hi);
  return PackBytes(r[0], r[1], r[2], r[3]);
}

// S = stride (1 or 2, both directions), PL = left padding (0 or 1)
// RPT: output rows a thread produces (more rows: fewer, fatter workgroups and fewer halo rows re-read)
// CW: output columns a thread produces, 4 or 8 (8: one 64-bit load per input row, twice the bytes in flight
// per lane; stride 1 only, rows and pointers multiples of eight bytes)
template <int S, int PL, bool BOXSUM, int RQ, int RPT, int CW = 4>
__global__ void __launch_bounds__(kThreads) DwConv3x3Kernel(DwArgs a) {
  // grid: (channel, image, block of row groups) - the channel comes without a division
  const int c = blockIdx.x;
  const int plane = blockIdx.y * a.C + c;
  const int tid = threadIdx.x;
  const int rgl = tid >> a.lpr_shift;
  const int w4 = tid & ((1 << a.lpr_shift) - 1);
  const int oh0 = (blockIdx.z * a.rg_per_block + rgl) * RPT;
  // the channel's constants (scalar loads: the channel is the same for the whole workgroup)
  const int wk0 = a.wpk[c * 4 + 0], wk1 = a.wpk[c * 4 + 1], wk2 = a.wpk[c * 4 + 2];
  const bool box = BOXSUM && a.wpk[c * 4 + 3] != 0;  // a uniform branch, taken by few channels
  const int bias = a.biasf[c];
  const tvx_v4i q = a.rq[c];
  if (oh0 >= a.OH) return;  // whole rows of lanes leave together: neighbours stay consistent

  const uint8_t* xp = a.x + static_cast<size_t>(plane) * a.H * a.W;
  uint8_t* yp = a.y + static_cast<size_t>(plane) * a.OH * a.OW;
  const int in_dwords = a.W / 4;

  // input dwords under this thread's four outputs: S of them, starting at S * w4;
  // the byte array of a row is {left neighbour, own dwords, right neighbour}
  constexpr int kOwn = S * CW / 4;
  constexpr int kRows = S * (RPT - 1) + 3;  // input rows behind the thread's output rows
  const int d0 = kOwn * w4;
  const int ih0 = oh0 * S - a.pad_t;
  const bool has_left = w4 > 0;                      // else: left of the image
  const bool has_right = d0 + kOwn < in_dwords;      // else: right of the image

  // all loads of the thread are issued before the first use; a lane beyond the row's last
  // output still fetches its dwords when they exist (its left neighbour needs them)
  int raw[kRows][kOwn + 2];
  // (a row outside the image reads the nearest row inside and is replaced below; offsets inside a plane fit 32 bits:
  // one scalar base + one vector offset per load, no 64-bit vector arithmetic)
  const uint32_t col_off = static_cast<uint32_t>(CW == 8 ? min(d0, in_dwords - 2) : 0) * 4u;
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    const int ihc = min(max(ih0 + r, 0), a.H - 1);
    const uint32_t row_off = __umul24(static_cast<uint32_t>(ihc), static_cast<uint32_t>(a.W));
    if constexpr (CW == 8) {
      // (rows are whole 8-byte units here: a lane's unit lies inside the row or wholly past it)
      const int2 v2 = *reinterpret_cast<const int2*>(xp + (row_off + col_off));
      raw[r][1] = v2.x;
      raw[r][2] = v2.y;
    } else {
#pragma unroll
      for (int i = 0; i < kOwn; ++i)
        raw[r][1 + i] = *reinterpret_cast<const int*>(xp + (row_off + static_cast<uint32_t>(min(d0 + i, in_dwords - 1)) * 4u));
    }
  }
  // The channel's constants are needed from here on: their (scalar) loads are in flight together with the rows.
  // Left to the compiler they are requested where they are first used, behind the wait for the rows - a second
  // round trip.
  asm volatile("" ::"s"(wk0), "s"(wk1), "s"(wk2), "s"(bias), "s"(q[0]), "s"(q[1]), "s"(q[2]), "s"(q[3]));
  // Wavefronts whose rows and dwords all lie inside the image (one vote: most of them) only re-bias their bytes.
  const bool edge = ih0 < 0 || ih0 + kRows > a.H || d0 + kOwn > in_dwords;
  if (__builtin_amdgcn_ballot_w64(edge) != 0) {
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int ih = ih0 + r;
      const int keep_row = min(max(ih, 0), a.H - 1) == ih ? -1 : 0;
#pragma unroll
      for (int i = 0; i < kOwn; ++i) {
        const int keep = d0 + i < in_dwords ? keep_row : 0;
        // mask arithmetic, not a select: a select on the loaded value would be compiled into a
        // branch around the load, and then the loads would be waited for one at a time
        raw[r][1 + i] = ((raw[r][1 + i] ^ a.xor_mask) & keep) | (a.pad_fill & ~keep);
      }
    }
  } else if (a.xor_mask) {
#pragma unroll
    for (int r = 0; r < kRows; ++r)
#pragma unroll
      for (int i = 0; i < kOwn; ++i) raw[r][1 + i] ^= a.xor_mask;
  }
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    // lane l - 1 holds the dwords to the left, lane l + 1 those to the right (wave_shr:1, wave_shl:1); the
    // wavefront's first / last lane, which has no such neighbour, is the first / last lane of an image row
    // and takes the padding below
    const int l = __builtin_amdgcn_mov_dpp(raw[r][kOwn], 0x138, 0xf, 0xf, true);
    const int rr = __builtin_amdgcn_mov_dpp(raw[r][1], 0x130, 0xf, 0xf, true);
    raw[r][0] = has_left ? l : a.pad_fill;
    raw[r][kOwn + 1] = has_right ? rr : a.pad_fill;
  }
  if (w4 >= a.ow4) return;  // lanes that only fed their neighbour
  // Uniform operands that the instructions below take from vector registers (the three-address dot product, the
  // clamp) get one copy for all output rows: each row is a block of its own behind the bounds test, and the
  // compiler would copy them again in every block.
  int bias_v = bias, wk0_v = wk0, lo_v = a.lo, hi_v = a.hi, t_v = q[1];
  const int lo_t = a.lo << q[1];
  int hi_t = (a.hi << q[1]) | ((1 << q[1]) - 1);
  asm volatile("" : "+v"(bias_v), "+v"(wk0_v), "+v"(lo_v), "+v"(hi_v), "+v"(t_v), "+v"(hi_t));
  uint8_t* const yrow = yp;  // (uniform base; offsets inside a plane fit 32 bits)
  if constexpr (CW == 8) {
    // windows are cut per output row (three input rows x eight windows live at a time)
#pragma unroll
    for (int o = 0; o < RPT; ++o) {
      if (oh0 + o >= a.OH) break;
      int res[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int win3[3];
#pragma unroll
        for (int r = 0; r < 3; ++r) {
          const int (&rw)[kOwn + 2] = raw[o + r];
          win3[r] = i == 0 ? Window<4 + 0 - PL>(rw) : i == 1 ? Window<4 + 1 - PL>(rw) : i == 2 ? Window<4 + 2 - PL>(rw)
                  : i == 3 ? Window<4 + 3 - PL>(rw) : i == 4 ? Window<4 + 4 - PL>(rw) : i == 5 ? Window<4 + 5 - PL>(rw)
                  : i == 6 ? Window<4 + 6 - PL>(rw) : Window<4 + 7 - PL>(rw);
        }
        int acc = Dot4Add(win3[0], wk0_v, bias_v);
        acc = __builtin_amdgcn_sdot4(win3[1], wk1, acc, false);
        acc = __builtin_amdgcn_sdot4(win3[2], wk2, acc, false);
        if (BOXSUM && box) {
          int sx = __builtin_amdgcn_sdot4(win3[0], 0x00010101, 0, false);
          sx = __builtin_amdgcn_sdot4(win3[1], 0x00010101, sx, false);
          sx = __builtin_amdgcn_sdot4(win3[2], 0x00010101, sx, false);
          acc -= a.zws * sx;
        }
        res[i] = acc;
      }
      const int lo4[4] = {res[0], res[1], res[2], res[3]}, hi4[4] = {res[4], res[5], res[6], res[7]};
      *reinterpret_cast<uint2*>(yrow + (__umul24(static_cast<uint32_t>(oh0 + o), static_cast<uint32_t>(a.OW)) + static_cast<uint32_t>(w4) * 8u)) =
          make_uint2(Requant4<RQ>(lo4, q, t_v, lo_t, hi_t, a.out_zp, lo_v, hi_v), Requant4<RQ>(hi4, q, t_v, lo_t, hi_t, a.out_zp, lo_v, hi_v));
    }
  } else {
  int win[kRows][4];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    // output i of this thread reads input bytes [S i - PL, S i - PL + 3) of its own span
    win[r][0] = Window<4 + S * 0 - PL>(raw[r]);
    win[r][1] = Window<4 + S * 1 - PL>(raw[r]);
    win[r][2] = Window<4 + S * 2 - PL>(raw[r]);
    win[r][3] = Window<4 + S * 3 - PL>(raw[r]);
  }
#pragma unroll
  for (int o = 0; o < RPT; ++o) {
    if (oh0 + o >= a.OH) break;
    int res[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int acc = Dot4Add(win[S * o][i], wk0_v, bias_v);
      acc = __builtin_amdgcn_sdot4(win[S * o + 1][i], wk1, acc, false);
      acc = __builtin_amdgcn_sdot4(win[S * o + 2][i], wk2, acc, false);
      if (BOXSUM && box) {
        int sx = __builtin_amdgcn_sdot4(win[S * o][i], 0x00010101, 0, false);
        sx = __builtin_amdgcn_sdot4(win[S * o + 1][i], 0x00010101, sx, false);
        sx = __builtin_amdgcn_sdot4(win[S * o + 2][i], 0x00010101, sx, false);
        acc -= a.zws * sx;
      }
      res[i] = acc;
    }
    *reinterpret_cast<uint32_t*>(yrow + (__umul24(static_cast<uint32_t>(oh0 + o), static_cast<uint32_t>(a.OW)) + static_cast<uint32_t>(w4) * 4u)) =
        Requant4<RQ>(res, q, t_v, lo_t, hi_t, a.out_zp, lo_v, hi_v);
  }
  }
}

// Launch geometry for one patch width.
struct Shape {
  int ow4, lpr_shift, rg_per_block, threads, rows_per_thread;
  dim3 grid;
};

struct Plan {
  DwArgs a;
  int stride, pad_l, boxsum, rq;
  int lds_pad;      // dynamic LDS the launch asks for without using it: caps the workgroups a CU runs at a time
  int cols;         // output columns per thread of the preferred form: 4 or 8
  Shape shape;      // ... its geometry
  Shape fallback;   // four columns per thread: taken when the 8-column form is preferred but a pointer is not 8-byte aligned
};

template <int S, int PL, bool BOXSUM, int RPT, int CW>
void LaunchRq(const Plan* p, const Shape& sh, const DwArgs& a, hipStream_t st) {
  const dim3 block(sh.threads);
  if (p->rq == kRqFastNoTie) hipLaunchKernelGGL((DwConv3x3Kernel<S, PL, BOXSUM, kRqFastNoTie, RPT, CW>), sh.grid, block, p->lds_pad, st, a);
  else if (p->rq == kRqFast) hipLaunchKernelGGL((DwConv3x3Kernel<S, PL, BOXSUM, kRqFast, RPT, CW>), sh.grid, block, p->lds_pad, st, a);
  else hipLaunchKernelGGL((DwConv3x3Kernel<S, PL, BOXSUM, kRqGeneric, RPT, CW>), sh.grid, block, p->lds_pad, st, a);
}

template <int S, int PL, int CW>
void LaunchBox(const Plan* p, const Shape& sh, const DwArgs& a, hipStream_t st) {
  // eight rows per thread only exist for stride 1 (chosen for tall planes)
  if (S == 1 && sh.rows_per_thread == 8) {
    if (p->boxsum) LaunchRq<1, PL, true, 8, CW>(p, sh, a, st);
    else LaunchRq<1, PL, false, 8, CW>(p, sh, a, st);
  } else {
    if (p->boxsum) LaunchRq<S, PL, true, 4, CW>(p, sh, a, st);
    else LaunchRq<S, PL, false, 4, CW>(p, sh, a, st);
  }
}

int DwRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* p = reinterpret_cast<const Plan*>(op->host_blob.data());
  DwArgs a = p->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  const bool wide = p->cols == 8 && ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(out)) & 7) == 0;
  const Shape& sh = wide ? p->shape : (p->cols == 8 ? p->fallback : p->shape);
  a.ow4 = sh.ow4;
  a.lpr_shift = sh.lpr_shift;
  a.rg_per_block = sh.rg_per_block;
  if (p->stride == 1) {
    if (wide) {
      if (p->pad_l) LaunchBox<1, 1, 8>(p, sh, a, st); else LaunchBox<1, 0, 8>(p, sh, a, st);
    } else {
      if (p->pad_l) LaunchBox<1, 1, 4>(p, sh, a, st); else LaunchBox<1, 0, 4>(p, sh, a, st);
    }
  } else {
    if (p->pad_l) LaunchBox<2, 1, 4>(p, sh, a, st); else LaunchBox<2, 0, 4>(p, sh, a, st);
  }
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

}  // namespace

// Packs depthwise 3x3 weights for the signed dot4 stencils: per channel four dwords, the three
// kernel rows (kx in bytes 0..2, byte 3 zero) and a correction word. With xs, ws the int8-domain
// activations and weights and zxs, zws their zero points,
//   sum (xs - zxs)(ws - zws) = sum xs wz - zxs sum wz            when wz = ws - zws fits int8,
//                            = sum xs ws - zws Sx - zxs sum ws + 9 zxs zws   otherwise,
// with the window sum Sx taken in the kernel. The correction word is 1 for channels in the second
// form; with `all_or_none` every channel takes the second form as soon as one needs it (for
// kernels that decide per operator, not per channel). The constant terms are folded into
// `biasf`. Returns whether any channel needs the window sum.
bool PackDepthwise3x3(int C, const void* w_host, bool w_u8, const void* bias_host, int zxs, int zws,
                      bool all_or_none, std::vector<int32_t>* wpk_out, std::vector<int32_t>* biasf_out) {
  std::vector<int32_t>& wpk = *wpk_out;
  std::vector<int32_t>& biasf = *biasf_out;
  wpk.assign(static_cast<size_t>(C) * 4, 0);
  biasf.assign(C, 0);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  bool any_box = false, all_fit = true;
  for (size_t i = 0; i < static_cast<size_t>(C) * 9; ++i) {
    const int v = static_cast<int8_t>(w_u8 ? src[i] ^ 0x80 : src[i]);
    if (v - zws < -128 || v - zws > 127) all_fit = false;
  }
  for (int c = 0; c < C; ++c) {
    int ws[9];
    bool fits = true;  // do the shifted weights ws - zws fit int8?
    for (int t = 0; t < 9; ++t) {
      const uint8_t raw = src[static_cast<size_t>(c) * 9 + t];
      ws[t] = static_cast<int8_t>(w_u8 ? raw ^ 0x80 : raw);
      if (ws[t] - zws < -128 || ws[t] - zws > 127) fits = false;
    }
    if (all_or_none) fits = all_fit;
    int64_t sw = 0;
    for (int ky = 0; ky < 3; ++ky) {
      uint32_t pk = 0;
      for (int kx = 0; kx < 3; ++kx) {
        const int v = fits ? ws[ky * 3 + kx] - zws : ws[ky * 3 + kx];
        pk |= static_cast<uint32_t>(static_cast<uint8_t>(static_cast<int8_t>(v))) << (8 * kx);
        sw += v;
      }
      wpk[static_cast<size_t>(c) * 4 + ky] = static_cast<int32_t>(pk);
    }
    const bool box = !fits && zws != 0;
    wpk[static_cast<size_t>(c) * 4 + 3] = box ? 1 : 0;
    any_box |= box;
    const int64_t v = (b ? b[c] : 0) - static_cast<int64_t>(zxs) * sw + (fits ? 0 : 9ll * zxs * zws);
    biasf[c] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  return any_box;
}

// Claims quantized depthwise 3x3, multiplier 1, dilation 1, stride 1 or 2 (both
// directions), constant weights, row lengths that are multiples of four.
int DwConv3x3Setup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || d->multiplier != 1) return TVX_E_UNSUPPORTED;
  if (d->k_w != 3 || d->k_h != 3 || d->dilation_w != 1 || d->dilation_h != 1) return TVX_E_UNSUPPORTED;
  if (d->stride_w != d->stride_h || (d->stride_w != 1 && d->stride_w != 2)) return TVX_E_UNSUPPORTED;
  if (d->pad_left > 1 || (d->in_w & 3) || (d->out_w & 3)) return TVX_E_UNSUPPORTED;
  const int S = d->stride_w;
  // an image row takes a power-of-two number of lanes (at most a wavefront) that covers both its
  // output patches and the input dwords behind them
  auto lanes_shift = [&](int cols) {
    const int out_patches = d->out_w / cols, own = S * cols / 4, in_dw = d->in_w / 4;
    int shift = 0;
    while ((1 << shift) < out_patches || own * (1 << shift) < in_dw) ++shift;
    return shift;
  };
  if (lanes_shift(4) > 6) return TVX_E_UNSUPPORTED;
  if (d->batch > 65535 || (d->out_h + 3) / 4 > 65535) return TVX_E_UNSUPPORTED;  // (grid.y, grid.z)
  if (d->in_h >= (1u << 24) || static_cast<uint64_t>(d->in_h) * d->in_w >= (1ull << 31)) return TVX_E_UNSUPPORTED;  // (32-bit offsets inside a plane)
  // every output's window must end inside {own dwords, right neighbour}
  if (static_cast<uint32_t>((d->out_w - 1) * S + 2) >= d->in_w + d->pad_left + 4) return TVX_E_UNSUPPORTED;
  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127) return TVX_E_UNSUPPORTED;
  const int C = d->in_c;
  std::vector<int32_t> wpk, biasf;
  const bool any_box = PackDepthwise3x3(C, w_host, w_u8, bias_host, zxs, zws, false, &wpk, &biasf);
  std::vector<int32_t> rqt;
  const int rq = BuildRequantRecords(op->h_mult, op->h_shift, C, C, d->out_zp, &rqt, AccumulatorBound(9, bias_host, C));
  int s = op->packed.Upload(wpk.data(), wpk.size() * 4);
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s != TVX_OK) return s;
  Plan p{};
  DwArgs& a = p.a;
  a.wpk = op->packed.as<int32_t>();
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<tvx_v4i>();
  a.C = C; a.H = d->in_h; a.W = d->in_w; a.OH = d->out_h; a.OW = d->out_w;
  a.pad_t = d->pad_top; a.pad_l = d->pad_left;
  // Eight columns per thread (stride 1, rows that are whole 8-byte units): one 64-bit load per input row and lane.
  int cols = (S == 1 && (d->in_w & 7) == 0 && (d->out_w & 7) == 0) ? 8 : 4;
  if (const char* f = getenv("TVX_DWCONV_COLS")) {  // tuning aid: output columns per thread
    if (atoi(f) == 4) cols = 4;
  }
  auto shape_for = [&](int cw) {
    Shape sh{};
    sh.ow4 = d->out_w / cw;
    sh.lpr_shift = lanes_shift(cw);
    // tall planes at stride 1: eight output rows per thread (a third of the workgroups to dispatch,
    // ten input rows read for eight instead of six for four)
    // (with eight columns per thread four rows measure faster: the patch is already 32 outputs)
    int rpt = S == 1 && cw == 4 && d->out_h >= 96 ? 8 : 4;
    if (const char* f = getenv("TVX_DWCONV_ROWS")) {  // tuning aid: output rows per thread
      if (atoi(f) == 4 || (atoi(f) == 8 && S == 1)) rpt = atoi(f);
    }
    sh.rows_per_thread = rpt;
    const int row_groups = (static_cast<int>(d->out_h) + rpt - 1) / rpt;
    // a workgroup is as many wavefronts as a plane's row groups fill, four at most: wavefronts
    // without rows would be dispatched only to leave at once
    sh.threads = std::min(kThreads, ((row_groups << sh.lpr_shift) + 63) / 64 * 64);
    if (const char* f = getenv("TVX_DWCONV_THREADS")) {  // tuning aid
      if (atoi(f) == 64 || atoi(f) == 128 || atoi(f) == 192 || atoi(f) == 256) sh.threads = std::max(atoi(f), 1 << sh.lpr_shift);
    }
    sh.rg_per_block = sh.threads >> sh.lpr_shift;
    sh.grid = dim3(C, d->batch, (row_groups + sh.rg_per_block - 1) / sh.rg_per_block);
    return sh;
  };
  p.lds_pad = 0;
  if (const char* f = getenv("TVX_DWCONV_LDS_KB")) p.lds_pad = std::max(0, std::min(64, atoi(f))) * 1024;  // tuning aid
  p.cols = cols;
  p.shape = shape_for(cols);
  p.fallback = shape_for(4);
  a.xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.pad_fill = static_cast<int>(static_cast<uint32_t>(zxs & 0xff) * 0x01010101u);
  a.zws = zws; a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  p.stride = S; p.pad_l = d->pad_left; p.boxsum = any_box; p.rq = rq;
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&p), reinterpret_cast<const uint8_t*>(&p) + sizeof(p));
  op->run = DwRun;
  op->kernel_name = "dwconv3x3_i8";
  return TVX_OK;
}

}  // namespace tvx
