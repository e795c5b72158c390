// pwconv_dwconv3x3_pwconv_i8: an inverted-residual block - 1x1 expansion, depthwise 3x3, 1x1 projection and the
// residual Add behind it - as one kernel, for the small feature maps (28, 14 and 7 columns) where three or four
// launches of a few microseconds of work each cost more than the arithmetic. The closed driver fuses such
// chains when it verifies the graph (reference: src/tim/vx/internal/src/vsi_nn_graph.c:1591-1603); the
// operators it fuses are the Conv2d nodes of src/tim/vx/internal/src/ops/vsi_nn_op_conv2d.c:35-118.
//
// The expanded tensor never leaves the CU. A workgroup (four wavefronts) owns a band of output rows of one
// image (at most 32 or 64 output pixels) and first transposes the band's input rows - with the halo the 3x3
// window needs - into LDS as the MFMA operand [pixel][channel]. The expanded channels are then walked in
// chunks of 32, wavefront w taking chunks w, w + 4, ...: expansion of all halo pixels for the chunk
// (v_mfma_i32_32x32x32_i8, requantized into a wavefront-private [channel][pixel] image), depthwise stencil on
// that image (signed dot4 over byte windows, requantized and transposed into the projection's operand), and
// the chunk's contribution to every output channel accumulated in registers. No barrier inside the walk: a
// wavefront only reads what it wrote. At the end the partial projections meet in LDS by integer atomics and
// every wavefront requantizes, adds the residual to and stores its share of the outputs.
#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
constexpr int kMStride = 48;      // bytes per pixel row of the projection operand (32 channels + 16: bank spread)
constexpr int kMaxCinSteps = 5;   // 32-channel steps of the expansion's reduction (160 input channels)

struct MbArgs {
  const uint8_t* x;    // block input {W, H, Cin, N}
  uint8_t* y;          // block output {OW, OH, Cout, N}
  const uint8_t* res;  // the residual Add's other operand (quantized like y's type), or null
  // expansion: fragments [chunk][cin step][64 lanes], folded bias and requantization records per expanded channel
  const v4i* w1;
  const int32_t* b1;
  const v4i* q1;
  // depthwise: {three tap rows, folded bias} and requantization records per expanded channel
  const v4i* dwk;
  const v4i* q2;
  // projection: fragments [output tile][chunk][64 lanes], folded bias and records per output channel
  const v4i* w2;
  const int32_t* b3;
  const v4i* q3;
  int Cin, H, Cexp, Cout, OH;
  int cin_steps, chunks, nt;
  int R, IR, bands, mh;           // output rows of a band, input rows behind them, bands per image, 32-pixel halo tiles
  int xs;                          // bytes per pixel row of the expansion operand
  int ep;                          // bytes per channel row of the expanded image
  int off_wave, wave_bytes;        // LDS: the wavefronts' private areas (expanded image, then projection operand)
  int off_red;                     // LDS: the projection's sums over all wavefronts, [tile][register][lane] (zeroed at the start)
  // quantization
  int x_xor;                       // 0x80 for uint8 input
  int zp1, neg_zws1_4;             // expansion weights' zero point as a second MFMA
  int e_zp, e_lo, e_hi, e_xor4, e_pad4, ties1;
  int dw_box, dw_zws, m_zp, m_lo, m_hi, m_xor, ties2;
  int zp3, neg_zws3_4;
  int out_zp, lo, hi, ties3;
  // residual Add (mode 0 = none; 1 / 2 = the block's result is the Add's first / second operand)
  double add_ra, add_rb;
  int add_mode, add_signed;
  int add_za, add_zb, add_zo, add_lo, add_hi;
  int aligned4;                    // output planes and bands are whole dwords: dword copy-out
};

// Window of output column J of a depthwise row: W input columns, stride S, SAME padding (one column left at
// stride 1, none at stride 2); byte 0 of `row` is the column under the first output's leftmost tap. Columns past
// the row's end recompute the last one (nobody stores them).
template <int W, int S, int J>
__device__ __forceinline__ int WindowOf(const int (&row)[(W + 5) / 4 + 1]) {
  constexpr int OW = (W + S - 1) / S;
  return Window<S * (J < OW ? J : OW - 1)>(row);
}

template <int W, int S, int J>
__device__ __forceinline__ int DwOne(const MbArgs& a, const int (&rows)[3][(W + 5) / 4 + 1], const v4i& k) {
  const int w0 = WindowOf<W, S, J>(rows[0]), w1 = WindowOf<W, S, J>(rows[1]), w2 = WindowOf<W, S, J>(rows[2]);
  int v = Dot4Add(w0, k[0], k[3]);
  v = __builtin_amdgcn_sdot4(w1, k[1], v, false);
  v = __builtin_amdgcn_sdot4(w2, k[2], v, false);
  if (a.dw_box) {  // (wave-uniform) weights packed unshifted: their zero point times the window sum
    int sx = __builtin_amdgcn_sdot4(w0, 0x00010101, 0, false);
    sx = __builtin_amdgcn_sdot4(w1, 0x00010101, sx, false);
    sx = __builtin_amdgcn_sdot4(w2, 0x00010101, sx, false);
    v -= a.dw_zws * sx;
  }
  return v;
}

// Four output columns J0 .. J0 + 3 of one channel's depthwise row, requantized.
template <int W, int S, int J0>
__device__ __forceinline__ void DwFour(const MbArgs& a, const int (&rows)[3][(W + 5) / 4 + 1], const v4i& k, const v4i& q,
                                       int (&out)[4]) {
  const int acc[4] = {DwOne<W, S, J0>(a, rows, k), DwOne<W, S, J0 + 1>(a, rows, k), DwOne<W, S, J0 + 2>(a, rows, k),
                      DwOne<W, S, J0 + 3>(a, rows, k)};
  Requant8x4(acc, q, a.m_zp, a.m_lo, a.m_hi, a.ties2, out);
}

template <int W, int S, int J0>
struct DwRow {
  static __device__ __forceinline__ void Run(const MbArgs& a, const int (&rows)[3][(W + 5) / 4 + 1], const v4i& k, const v4i& q,
                                              uint8_t* m_row, int ch_byte, bool ch_live) {
    constexpr int OW = (W + S - 1) / S;
    if constexpr (J0 < OW) {
      int out[4];
      DwFour<W, S, J0>(a, rows, k, q, out);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (J0 + i < OW) m_row[(J0 + i) * kMStride + ch_byte] = ch_live ? static_cast<uint8_t>(out[i] ^ a.m_xor) : uint8_t{0};
      DwRow<W, S, J0 + 4>::Run(a, rows, k, q, m_row, ch_byte, ch_live);
    }
  }
};

// W: columns of the input; S: stride of the depthwise convolution; MO: 32-pixel tiles of a band's output;
// NTMAX: most 32-channel output tiles; ADD: residual Add behind the projection.
// (the register budget follows the accumulators: two wavefronts per SIMD up to five output tiles - three with two
// tiles, 168 registers, spill 36 bytes per lane and measure slower -, one beyond)
template <int W, int S, int MO, int NTMAX, bool ADD>
__global__ void __launch_bounds__(kThreads, (MO * NTMAX <= 5 ? 2 : 1)) MbConvKernel(MbArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int PL = S == 1 ? 1 : 0;               // left (and top) padding of the depthwise convolution
  constexpr int OW = (W + S - 1) / S;
  constexpr int NW = (W + 5) / 4;                  // dwords of a normalized input row: bytes 0 .. W + PL
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = blockIdx.x / a.bands, band = blockIdx.x - n * a.bands;
  const int or0 = band * a.R;
  const int rows_out = min(a.R, a.OH - or0);
  const int po = rows_out * OW;                    // live output pixels of the band
  const int ir0 = or0 * S - PL;                    // image row of the band's first halo row (may be -1)
  const int hp = a.IR * W;                         // halo pixels
  uint8_t* xin = lds;
  uint8_t* e_w = lds + a.off_wave + wave * a.wave_bytes + 4;  // (+ 4: the byte in front of row 0 is read)
  uint8_t* m_w = lds + a.off_wave + wave * a.wave_bytes + 16 + 32 * a.ep;

  const int frow = lane & 31, fh = lane >> 5;
  // The expansion's operands of the next chunk (fragments, the lane's bias and requantization record) are fetched
  // while this one is computed; what the later phases need is fetched at the chunk's start and has arrived by then.
  struct ExpandOperands {
    v4i wf[kMaxCinSteps];
    int bias1;
    v4i rq1;
  };
  auto fetch = [&](int chunk, ExpandOperands& o) {
    const int c = min(chunk, a.chunks - 1);
#pragma unroll
    for (int k = 0; k < kMaxCinSteps; ++k) o.wf[k] = a.w1[(c * a.cin_steps + min(k, a.cin_steps - 1)) * 64 + lane];
    o.bias1 = a.b1[c * 32 + frow];
    o.rq1 = a.q1[c * 32 + frow];
  };
  ExpandOperands next;
  fetch(wave, next);  // (on its way while the input rows are loaded)

  // ---- the band's input rows as the expansion's operand: xin[halo pixel][channel], signed bytes ----
  // A channel's halo rows are consecutive bytes of its plane. A thread takes four of them for four channels (dwords
  // at any byte offset where all sixteen bytes exist, else byte by byte with zeros for what lies outside the image,
  // the band or the channels), transposes, and stores four pixels' channel quads.
  {
    const int quads = a.mh * 8;                        // pixel quads of the halo tiles
    const int units = a.cin_steps * 8 * quads;         // x channel quads
    const int plane = a.H * W;
    const uint8_t* xn = a.x + static_cast<size_t>(n) * a.Cin * plane;
    const int live_lo = max(0, -ir0) * W, live_hi = min(a.IR, a.H - ir0) * W;  // the live bytes of a channel's halo rows
    const uint32_t xor4 = static_cast<uint32_t>(a.x_xor) * 0x01010101u;
    for (int unit = tid; unit < units; unit += kThreads) {
      const int c4 = unit / quads, p0 = (unit - c4 * quads) * 4;
      const int c = c4 * 4;
      const int at = ir0 * W + p0;                     // byte offset in the plane (negative above the image)
      uint32_t d[4];
      if (p0 >= live_lo && p0 + 4 <= live_hi && c + 4 <= a.Cin) {
#pragma unroll
        for (int j = 0; j < 4; ++j) __builtin_memcpy(&d[j], xn + (c + j) * plane + at, 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) d[j] ^= xor4;
      } else {
        uint8_t b[4][4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const bool live = p0 + e >= live_lo && p0 + e < live_hi && c + j < a.Cin;
            b[j][e] = live ? static_cast<uint8_t>(xn[(c + j) * plane + at + e] ^ a.x_xor) : uint8_t{0};
          }
#pragma unroll
        for (int j = 0; j < 4; ++j) d[j] = b[j][0] | b[j][1] << 8 | b[j][2] << 16 | static_cast<uint32_t>(b[j][3]) << 24;
      }
      uint32_t px[4];
      Transpose4x4(d, px);
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<uint32_t*>(xin + (p0 + i) * a.xs + c) = px[i];
    }
  }
  for (int i = tid; i < a.nt * MO * 256; i += kThreads) reinterpret_cast<v4i*>(lds + a.off_red)[i] = v4i{0, 0, 0, 0};
  __syncthreads();

  v16i acc_out[MO][NTMAX];
#pragma unroll
  for (int mo = 0; mo < MO; ++mo)
#pragma unroll
    for (int t = 0; t < NTMAX; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc_out[mo][t][r] = 0;
  const v4i fz1 = {a.neg_zws1_4, a.neg_zws1_4, a.neg_zws1_4, a.neg_zws1_4};
  const v4i fz3 = {a.neg_zws3_4, a.neg_zws3_4, a.neg_zws3_4, a.neg_zws3_4};

  // one halo tile of the chunk: accumulate, requantize, store as [channel][halo pixel]
  auto expand_finish = [&](const v16i& acc, int mt, const v4i& rq1) {
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const int av[4] = {acc[gq * 4], acc[gq * 4 + 1], acc[gq * 4 + 2], acc[gq * 4 + 3]};
      *reinterpret_cast<uint32_t*>(e_w + frow * a.ep + mt * 32 + 8 * gq + 4 * fh) =
          Requant8x4Pack(av, rq1, a.e_zp, a.e_lo, a.e_hi, a.ties1) ^ static_cast<uint32_t>(a.e_xor4);
    }
  };
  for (int chunk = wave; chunk < a.chunks; chunk += kWaves) {
    const int ch = chunk * 32 + frow;  // this lane's expanded channel, in all three phases
    const ExpandOperands cur = next;
    fetch(chunk + kWaves, next);
    const v4i dk = a.dwk[ch];
    const v4i rq2 = a.q2[ch];
    v4i w2f[NTMAX];
#pragma unroll
    for (int t = 0; t < NTMAX; ++t) w2f[t] = a.w2[(min(t, a.nt - 1) * a.chunks + chunk) * 64 + lane];

    // ---- expansion of every halo pixel for this chunk: e_w[channel][halo pixel], signed bytes; two halo tiles
    // at a time, so that one tile's MFMA chain runs under the other's ----
    for (int mt = 0; mt < a.mh; mt += 2) {
      const bool two = mt + 1 < a.mh;  // (wave-uniform)
      const int mt1 = two ? mt + 1 : mt;
      v16i acc0, acc1;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc0[r] = acc1[r] = cur.bias1;
      const uint8_t* xa0 = xin + (mt * 32 + frow) * a.xs + fh * 16;
      const uint8_t* xa1 = xin + (mt1 * 32 + frow) * a.xs + fh * 16;
#pragma unroll
      for (int k = 0; k < kMaxCinSteps; ++k) {
        if (k < a.cin_steps) {
          const v4i fx0 = *reinterpret_cast<const v4i*>(xa0 + k * 32);
          const v4i fx1 = *reinterpret_cast<const v4i*>(xa1 + k * 32);
          acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx0, cur.wf[k], acc0, 0, 0, 0);
          if (two) acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx1, cur.wf[k], acc1, 0, 0, 0);
          if (a.zp1) {
            acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx0, fz1, acc0, 0, 0, 0);
            if (two) acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx1, fz1, acc1, 0, 0, 0);
          }
        }
      }
      expand_finish(acc0, mt, cur.rq1);
      if (two) expand_finish(acc1, mt1, cur.rq1);
    }
    __builtin_amdgcn_wave_barrier();

    // ---- depthwise 3x3: lane = (channel, every second output row) -> m_w[output pixel][channel] ----
    for (int orr = fh; orr < rows_out; orr += 2) {
      int rows[3][NW + 1];
#pragma unroll
      for (int t = 0; t < 3; ++t) {
        const int irr = orr * S + t;                 // halo row
        const int ih = ir0 + irr;
        const bool row_ok = ih >= 0 && ih < a.H;
        const int o = frow * a.ep + irr * W - PL;    // byte 0 of the normalized row (>= -1: e_w has room in front)
        const int shift = (o + 4) & 3;
        const uint32_t* src = reinterpret_cast<const uint32_t*>(e_w + ((o + 4) & ~3) - 4);
        uint32_t raw[NW + 1];
#pragma unroll
        for (int i = 0; i <= NW; ++i) raw[i] = src[i];
#pragma unroll
        for (int i = 0; i < NW; ++i)
          rows[t][i] = row_ok ? static_cast<int>(__builtin_amdgcn_alignbyte(raw[i + 1], raw[i], shift)) : a.e_pad4;
        rows[t][NW] = a.e_pad4;
        // the padding columns: byte 0 at stride 1 (column -1), byte W + PL (column W)
        if (PL) rows[t][0] = (rows[t][0] & ~0xff) | (a.e_pad4 & 0xff);
        constexpr int rb = W + PL;
        rows[t][rb / 4] = (rows[t][rb / 4] & ~(0xff << (8 * (rb % 4)))) | (a.e_pad4 & (0xff << (8 * (rb % 4))));
      }
      DwRow<W, S, 0>::Run(a, rows, dk, rq2, m_w + orr * OW * kMStride, frow, ch < a.Cexp);
    }
    __builtin_amdgcn_wave_barrier();

    // ---- this chunk's contribution to every output tile ----
#pragma unroll
    for (int mo = 0; mo < MO; ++mo) {
      const v4i fx = *reinterpret_cast<const v4i*>(m_w + (mo * 32 + frow) * kMStride + fh * 16);
#pragma unroll
      for (int t = 0; t < NTMAX; ++t) {
        if (t < a.nt) {
          acc_out[mo][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx, w2f[t], acc_out[mo][t], 0, 0, 0);
          if (a.zp3) acc_out[mo][t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx, fz3, acc_out[mo][t], 0, 0, 0);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  // ---- the wavefronts' partial projections meet in LDS (integer atomics on a zeroed image laid out like the
  // accumulators: [tile][register][lane]); then every wavefront finishes its share of the (output tile, pixel tile,
  // register quad) units: requantize, add the residual, store. A unit is four pixels of each of 32 channels.
  int* red = reinterpret_cast<int*>(lds + a.off_red);
  const size_t out_plane = static_cast<size_t>(a.OH) * OW;
  const int units = a.nt * MO * 4;
  constexpr int kMaxUnits = (NTMAX * MO * 4 + kWaves - 1) / kWaves;
  // what the units need from memory is requested first: the sums then form under these loads
  int bias3[kMaxUnits];
  v4i rq3[kMaxUnits];
  uint32_t resv[kMaxUnits];
  size_t at[kMaxUnits];
  int px0[kMaxUnits];
#pragma unroll
  for (int i = 0; i < kMaxUnits; ++i) {
    const int u = min(wave + i * kWaves, units - 1);
    const int t = u / (MO * 4), mo = (u >> 2) % MO, gq = u & 3;
    const int oc = t * 32 + frow;
    bias3[i] = a.b3[oc];
    rq3[i] = a.q3[oc];
    px0[i] = mo * 32 + 8 * gq + 4 * fh;
    at[i] = (static_cast<size_t>(n) * a.Cout + oc) * out_plane + static_cast<size_t>(or0) * OW + px0[i];
    resv[i] = 0;
    if (ADD && oc < a.Cout) {
      if (a.aligned4) {
        if (px0[i] < po) resv[i] = *reinterpret_cast<const uint32_t*>(a.res + at[i]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (px0[i] + e < po) resv[i] |= static_cast<uint32_t>(a.res[at[i] + e]) << (8 * e);
      }
    }
  }
  if (wave < a.chunks) {  // (a wavefront that walked no chunk has nothing to add)
#pragma unroll
    for (int t = 0; t < NTMAX; ++t)
      if (t < a.nt) {
#pragma unroll
        for (int mo = 0; mo < MO; ++mo)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            __hip_atomic_fetch_add(red + ((t * MO + mo) * 16 + r) * 64 + lane, acc_out[mo][t][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < kMaxUnits; ++i) {
    const int u = wave + i * kWaves;
    if (u >= units) break;
    const int t = u / (MO * 4), gq = u & 3;
    const int oc = t * 32 + frow;
    int av[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) av[e] = red[((u >> 2) * 16 + gq * 4 + e) * 64 + lane] + bias3[i];
    const uint32_t codes = Requant8x4Pack(av, rq3[i], a.out_zp, a.lo, a.hi, a.ties3);
    if (oc >= a.Cout) continue;
    if (a.aligned4) {
      if (px0[i] < po) {
        uint32_t o = codes;
        if (ADD) o = AddResidual4(a, o, resv[i]);
        *reinterpret_cast<uint32_t*>(a.y + at[i]) = o;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (px0[i] + e < po) {
          int o = static_cast<int>((codes >> (8 * e)) & 0xff);
          if (ADD) o = AddResidual1(a, o, static_cast<int>((resv[i] >> (8 * e)) & 0xff));
          a.y[at[i] + e] = static_cast<uint8_t>(o);
        }
    }
  }
}

typedef void (*MbFn)(MbArgs);

template <int W, int S, int MO, bool ADD>
MbFn KernelNt(int nt) {
  if (nt <= 2) return MbConvKernel<W, S, MO, 2, ADD>;
  if (nt <= 5) return MbConvKernel<W, S, MO, 5, ADD>;
  if (MO == 1 && nt <= 10) return MbConvKernel<W, S, 1, 10, ADD>;
  return nullptr;
}

template <bool ADD>
MbFn KernelOf(int w, int s, int nt) {
  if (w == 28 && s == 1) return KernelNt<28, 1, 2, ADD>(nt);
  if (w == 28 && s == 2) return KernelNt<28, 2, 1, ADD>(nt);
  if (w == 14 && s == 1) return KernelNt<14, 1, 1, ADD>(nt);
  if (w == 14 && s == 2) return KernelNt<14, 2, 1, ADD>(nt);
  if (w == 7 && s == 1) return KernelNt<7, 1, 1, ADD>(nt);
  return nullptr;
}

struct Plan {
  MbArgs a;
  int w, s, lds_bytes;
  unsigned grid;
};

MbFn Kernel(const Plan& p) {
  return p.a.add_mode ? KernelOf<true>(p.w, p.s, p.a.nt) : KernelOf<false>(p.w, p.s, p.a.nt);
}

int MbConvRun(tvx_op* op, const void* in0, const void* in1, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  MbArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  a.res = static_cast<const uint8_t*>(in1);
  if (a.add_mode && !in1) return SetError(TVX_E_INVALID, "pwconv_dwconv3x3_pwconv_i8: the fused Add needs its second operand as in1");
  if (a.aligned4 && ((reinterpret_cast<uintptr_t>(out) | (a.add_mode ? reinterpret_cast<uintptr_t>(in1) : 0)) & 3))
    a.aligned4 = 0;
  hipLaunchKernelGGL(Kernel(*plan), dim3(plan->grid), dim3(kThreads), plan->lds_bytes, st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

int RoundUp(int v, int m) { return (v + m - 1) / m * m; }

// weights [oc][c] (uint8 re-biased to int8) -> MFMA fragments [oc tile][32-channel step][64 lanes][16 bytes];
// sums[oc] = sum of the signed weights
void PackPointwise(const void* w_host, bool w_u8, int OC, int C, std::vector<int8_t>* packed, std::vector<int64_t>* sums) {
  const int tiles = (OC + 31) / 32, steps = (C + 31) / 32;
  packed->assign(static_cast<size_t>(tiles) * steps * 1024, 0);
  sums->assign(static_cast<size_t>(tiles) * 32, 0);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  for (int oc = 0; oc < OC; ++oc)
    for (int c = 0; c < C; ++c) {
      const uint8_t raw = src[static_cast<size_t>(oc) * C + c];
      const int8_t v = static_cast<int8_t>(w_u8 ? raw ^ 0x80 : raw);
      const int ks = c / 32, half = (c % 32) / 16, j = c % 16;
      (*packed)[((static_cast<size_t>(oc / 32) * steps + ks) * 64 + half * 32 + oc % 32) * 16 + j] = v;
      (*sums)[oc] += v;
    }
}

bool IsPointwise(const tvx_conv2d_desc* d) {
  return d->multiplier == 0 && d->groups <= 1 && d->k_w == 1 && d->k_h == 1 && d->stride_w == 1 && d->stride_h == 1 &&
         d->dilation_w == 1 && d->dilation_h == 1 && d->pad_left == 0 && d->pad_top == 0 && d->out_w == d->in_w &&
         d->out_h == d->in_h;
}

bool Feeds(const tvx_conv2d_desc* a, const tvx_conv2d_desc* b) {
  return b->in_w == a->out_w && b->in_h == a->out_h && b->in_c == a->out_c && b->batch == a->batch &&
         b->in_dtype == a->out_dtype && b->in_scale == a->out_scale && b->in_zp == a->out_zp;
}

}  // namespace

// `op` carries the projection (op->conv, its requantization tables in h_mult / h_shift, clamp, fused Add);
// the expansion and the depthwise convolution come with their own tables. Declines (TVX_E_UNSUPPORTED) what
// the kernel does not cover; the caller then creates the operators one by one.
int MbConvSetup(tvx_op* op, const MbStage& ex, const MbStage& dw, const tvx_conv2d_desc* pr, const void* pr_w, const void* pr_b) {
  const tvx_conv2d_desc *e = ex.desc, *d = dw.desc;
  if (!IsPointwise(e) || !IsPointwise(pr) || !Feeds(e, d) || !Feeds(d, pr)) return TVX_E_UNSUPPORTED;
  if (d->multiplier != 1 || d->k_w != 3 || d->k_h != 3 || d->dilation_w != 1 || d->dilation_h != 1) return TVX_E_UNSUPPORTED;
  const int S = d->stride_w, W = d->in_w, H = d->in_h;
  if (d->stride_h != d->stride_w || (S != 1 && S != 2)) return TVX_E_UNSUPPORTED;
  const int PL = S == 1 ? 1 : 0;
  if (static_cast<int>(d->pad_left) != PL || static_cast<int>(d->pad_top) != PL) return TVX_E_UNSUPPORTED;
  const int OW = (W + S - 1) / S;
  if (static_cast<int>(d->out_w) != OW || static_cast<int>(d->out_h) != (H + S - 1) / S) return TVX_E_UNSUPPORTED;
  if (S == 2 && ((W | H) & 1)) return TVX_E_UNSUPPORTED;
  const int Cin = e->in_c, Cexp = e->out_c, Cout = pr->out_c;
  const int cin_steps = (Cin + 31) / 32, chunks = (Cexp + 31) / 32, nt = (Cout + 31) / 32;
  if (cin_steps > kMaxCinSteps) return TVX_E_UNSUPPORTED;
  Plan plan{};
  plan.w = W; plan.s = S;
  MbArgs& a = plan.a;
  a.nt = nt;
  a.add_mode = op->fused_add;
  if (!Kernel(plan)) return TVX_E_UNSUPPORTED;
  if (const char* f = getenv("TVX_NO_MBCONV"))  // tuning aid: leaves blocks to the single operators
    if (atoi(f)) return TVX_E_UNSUPPORTED;
  // Measured on MobileNetV2 at batch 64: the block kernel beats the single operators on the 14-column stride-1
  // blocks (25 against 32 us); on 28 columns their launches carry enough work, on 7 columns and at stride 2 the
  // block's work per wavefront is too long a chain. Those shapes are taken on request only.
  if (W != 14 || S != 1) {
    const char* f = getenv("TVX_MBCONV_ALL");
    if (!f || !atoi(f)) return TVX_E_UNSUPPORTED;
  }
  const int MO = (W == 28 && S == 1) ? 2 : 1;
  // rows of a band: what fills the output tiles; on 7-column planes two rows only, which doubles the bands (a batch
  // of 64 images then fills the chip) and needs a single halo tile
  int R = W == 7 ? 2 : MO * 32 / OW;
  R = std::min<int>(R, d->out_h);
  if (R < 1) return TVX_E_UNSUPPORTED;
  const int IR = (R - 1) * S + 3;
  const int mh = (IR * W + 31) / 32;
  if (static_cast<uint64_t>(e->in_c) * H * W >= (1ull << 31)) return TVX_E_UNSUPPORTED;

  a.Cin = Cin; a.H = H; a.Cexp = Cexp; a.Cout = Cout; a.OH = d->out_h;
  a.cin_steps = cin_steps; a.chunks = chunks;
  a.R = R; a.IR = IR; a.bands = (d->out_h + R - 1) / R; a.mh = mh;
  a.xs = cin_steps * 32 + 16;
  a.ep = mh * 32 + 4;
  a.off_wave = RoundUp(mh * 32 * a.xs, 16);
  a.wave_bytes = RoundUp(16 + 32 * a.ep + MO * 32 * kMStride, 16);
  a.off_red = a.off_wave + kWaves * a.wave_bytes;
  plan.lds_bytes = a.off_red + nt * MO * 4096;
  if (plan.lds_bytes > 160 * 1024) return TVX_E_UNSUPPORTED;
  const uint64_t grid = static_cast<uint64_t>(e->batch) * a.bands;
  if (grid > 0x7fffffffull) return TVX_E_UNSUPPORTED;
  plan.grid = static_cast<unsigned>(grid);

  // ---- expansion ----
  const bool x_u8 = e->in_dtype == TVX_U8, w1_u8 = e->w_dtype == TVX_U8;
  const int zxs = e->in_zp - (x_u8 ? 128 : 0);
  const int zws1 = (e->w_scales ? 0 : e->w_zp) - (w1_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127 || zws1 < -127 || zws1 > 127) return TVX_E_UNSUPPORTED;
  std::vector<int8_t> pk1, pk3;
  std::vector<int64_t> sw1, sw3;
  PackPointwise(ex.w, w1_u8, Cexp, Cin, &pk1, &sw1);
  const int exp_alloc = chunks * 32;
  std::vector<int32_t> b1(exp_alloc, 0), rq1, rq2, rq3;
  const int32_t* eb = static_cast<const int32_t*>(ex.b);
  for (int c = 0; c < Cexp; ++c) {
    const int64_t v = (eb ? eb[c] : 0) - static_cast<int64_t>(zxs) * sw1[c] + static_cast<int64_t>(Cin) * zxs * zws1;
    b1[c] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  const int f1 = BuildRequantRecords(*ex.mult, *ex.shift, Cexp, exp_alloc, e->out_zp, &rq1, AccumulatorBound(Cin, ex.b, Cexp));
  if (f1 == kRqGeneric) return TVX_E_UNSUPPORTED;
  a.x_xor = x_u8 ? 0x80 : 0;
  a.zp1 = zws1 != 0;
  a.neg_zws1_4 = static_cast<int>(static_cast<uint32_t>((-zws1) & 0xff) * 0x01010101u);
  const bool e_u8 = e->out_dtype == TVX_U8;
  a.e_zp = e->out_zp; a.e_lo = ex.lo; a.e_hi = ex.hi; a.ties1 = f1 == kRqFast;
  a.e_xor4 = e_u8 ? static_cast<int>(0x80808080u) : 0;
  const int zes = e->out_zp - (e_u8 ? 128 : 0);
  a.e_pad4 = static_cast<int>(static_cast<uint32_t>(zes & 0xff) * 0x01010101u);

  // ---- depthwise ----
  const bool wd_u8 = d->w_dtype == TVX_U8;
  const int zwd = (d->w_scales ? 0 : d->w_zp) - (wd_u8 ? 128 : 0);
  std::vector<int32_t> dwpk, dbias;
  a.dw_box = PackDepthwise3x3(Cexp, dw.w, wd_u8, dw.b, zes, zwd, true, &dwpk, &dbias);
  a.dw_zws = zwd;
  std::vector<int32_t> dwk(static_cast<size_t>(exp_alloc) * 4, 0);
  for (int c = 0; c < Cexp; ++c) {
    for (int t = 0; t < 3; ++t) dwk[4 * c + t] = dwpk[4 * c + t];
    dwk[4 * c + 3] = dbias[c];
  }
  const int f2 = BuildRequantRecords(*dw.mult, *dw.shift, Cexp, exp_alloc, d->out_zp, &rq2, AccumulatorBound(9, dw.b, Cexp));
  if (f2 == kRqGeneric) return TVX_E_UNSUPPORTED;
  const bool m_u8 = d->out_dtype == TVX_U8;
  a.m_zp = d->out_zp; a.m_lo = dw.lo; a.m_hi = dw.hi; a.ties2 = f2 == kRqFast;
  a.m_xor = m_u8 ? 0x80 : 0;
  const int zms = d->out_zp - (m_u8 ? 128 : 0);

  // ---- projection ----
  const bool w3_u8 = pr->w_dtype == TVX_U8;
  const int zws3 = op->w_zp - (w3_u8 ? 128 : 0);
  if (zms < -128 || zms > 127 || zws3 < -127 || zws3 > 127) return TVX_E_UNSUPPORTED;
  PackPointwise(pr_w, w3_u8, Cout, Cexp, &pk3, &sw3);
  const int out_alloc = nt * 32;
  std::vector<int32_t> b3(out_alloc, 0);
  const int32_t* pb = static_cast<const int32_t*>(pr_b);
  for (int c = 0; c < Cout; ++c) {
    const int64_t v = (pb ? pb[c] : 0) - static_cast<int64_t>(zms) * sw3[c] + static_cast<int64_t>(Cexp) * zms * zws3;
    b3[c] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  const int f3 = BuildRequantRecords(op->h_mult, op->h_shift, Cout, out_alloc, pr->out_zp, &rq3, AccumulatorBound(Cexp, pr_b, Cout));
  if (f3 == kRqGeneric) return TVX_E_UNSUPPORTED;
  a.zp3 = zws3 != 0;
  a.neg_zws3_4 = static_cast<int>(static_cast<uint32_t>((-zws3) & 0xff) * 0x01010101u);
  a.out_zp = pr->out_zp; a.lo = op->act_lo; a.hi = op->act_hi; a.ties3 = f3 == kRqFast;
  if (op->fused_add) {
    const tvx_eltwise_desc& el = op->elt;
    const double ra = static_cast<double>(el.a_scale) / static_cast<double>(el.out_scale);
    const double rb = static_cast<double>(el.b_scale) / static_cast<double>(el.out_scale);
    if (!(ra < 1048576.0) || !(rb < 1048576.0)) return TVX_E_UNSUPPORTED;
    a.add_signed = pr->out_dtype == TVX_I8;
    a.add_ra = ra; a.add_rb = rb;
    a.add_za = el.a_zp; a.add_zb = el.b_zp; a.add_zo = el.out_zp;
    ActRange(pr->out_dtype, el.out_scale, el.out_zp, TVX_ACT_NONE, &a.add_lo, &a.add_hi);
  }
  const uint64_t out_plane = static_cast<uint64_t>(d->out_h) * OW;
  a.aligned4 = out_plane % 4 == 0 && (R * OW) % 4 == 0 && (static_cast<int>(d->out_h) % R * OW) % 4 == 0;

  // ---- one device image: [w1 | w2 | b1 | q1 | dwk | q2 | b3 | q3], every part 16-byte aligned ----
  std::vector<uint8_t> blob;
  auto append = [&](const void* p, size_t n) {
    const size_t at = blob.size();
    blob.resize(at + (n + 15) / 16 * 16, 0);
    std::memcpy(blob.data() + at, p, n);
    return at;
  };
  // the projection's fragments are read [output tile][chunk]: PackPointwise's order
  const size_t o_w1 = append(pk1.data(), pk1.size()), o_w2 = append(pk3.data(), pk3.size());
  const size_t o_b1 = append(b1.data(), b1.size() * 4), o_q1 = append(rq1.data(), rq1.size() * 4);
  const size_t o_dk = append(dwk.data(), dwk.size() * 4), o_q2 = append(rq2.data(), rq2.size() * 4);
  const size_t o_b3 = append(b3.data(), b3.size() * 4), o_q3 = append(rq3.data(), rq3.size() * 4);
  int s = op->packed.Upload(blob.data(), blob.size());
  if (s != TVX_OK) return s;
  const uint8_t* base = op->packed.as<uint8_t>();
  a.w1 = reinterpret_cast<const v4i*>(base + o_w1);
  a.w2 = reinterpret_cast<const v4i*>(base + o_w2);
  a.b1 = reinterpret_cast<const int32_t*>(base + o_b1);
  a.q1 = reinterpret_cast<const v4i*>(base + o_q1);
  a.dwk = reinterpret_cast<const v4i*>(base + o_dk);
  a.q2 = reinterpret_cast<const v4i*>(base + o_q2);
  a.b3 = reinterpret_cast<const int32_t*>(base + o_b3);
  a.q3 = reinterpret_cast<const v4i*>(base + o_q3);

  const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel(plan)),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, plan.lds_bytes);
  if (err != hipSuccess) return SetError(TVX_E_DEVICE, "hipFuncSetAttribute(dynamic LDS %d): %s", plan.lds_bytes, hipGetErrorString(err));
  op->host_blob.resize(sizeof(Plan));
  std::memcpy(op->host_blob.data(), &plan, sizeof(Plan));
  op->run = MbConvRun;
  op->kernel_name = op->fused_add ? "pwconv_dwconv3x3_pwconv_add_i8" : "pwconv_dwconv3x3_pwconv_i8";
  return TVX_OK;
}

}  // namespace tvx
