// Dense quantized Conv2d as an implicit GEMM, one fat workgroup per compute unit.
//
// The same GEMM view as conv_igemm_i8.hip (rows = output pixels, columns = output channels,
// reduction = (ky, kx, c) with the channel fastest, operands re-biased to int8, the zero-point
// expansion folded into the bias plus a per-pixel sum), for layers whose whole weight block
// fits LDS next to two halo tiles (3x3x64 -> 64, 3x3x32 -> 64): a workgroup of sixteen
// wavefronts - four per SIMD, so that one wavefront's vector work runs under another's matrix
// instructions - walks bands of whole output rows of one image.
//
//   loader   every thread owns one (8 input columns x 4 channels) patch of the band's halo
//            rows: four 8-byte loads, two 4 x 4 byte transposes in registers, eight dword
//            stores into a channel-innermost halo tile. The loads of the NEXT band are issued
//            before the present band is multiplied and stored into the other halo buffer
//            behind it: one workgroup barrier per band.
//   weights  global -> LDS once per workgroup by DMA; B fragments are read from there per
//            k-step (no weight lives in a register, which is what lets four wavefronts share
//            a SIMD).
//   multiply wavefront w owns the band's 32-pixel tile w and both 32-channel tiles: per
//            k-step one A and two B fragment reads feed two v_mfma_i32_32x32x32_i8.
//   epilogue requantization from the wavefront's own accumulators into a wavefront-private
//            staging tile, from there 16 bytes per lane to the WHCN output: no second barrier.
#include <algorithm>
#include <cstdlib>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBandThreads = 1024;
constexpr int kBandWaves = kBandThreads / 64;
constexpr int kStageStride = 40;  // bytes per channel row of a wavefront's staging tile (32 pixels + bank spread)

struct BandArgs {
  const uint8_t* x;
  const int8_t* w;       // packed [64][kstride]
  uint8_t* y;
  const int32_t* biasf;  // bias + per-channel zero-point terms
  const v4i* rq;         // per channel {mult, t, rounding constant, tie mask}
  int C, H, W, OC, OH, OW;
  int sh, sw, pad_t, pad_l, khe;  // khe: rows a kernel column spans, (kh - 1) * dh + 1
  int rows;              // output rows of a band
  int PT;                // 32-pixel tiles of a full band
  int tiles_per_image, total_tiles;
  uint32_t magic_tpi, magic_ow, magic_gpr, magic_gblocks;
  int gpr;               // 8-column groups per input row
  int n_g8;              // ... per band (all halo rows)
  int gblocks;           // blocks of sixteen such groups
  int iwt, pix_stride;
  int kstride, w_chunks;
  int xor_mask, pad_fill, zws, out_zp, lo, hi;
  int halo_rows, pad_cols;
  int off_sx, off_rq, off_bias, off_w, off_stage, off_halo0, off_halo1;
  int tap_off[20];       // halo byte offset of k-step ks (its two 16-byte halves lie side by side)
};

// u / d by the host-made reciprocal ceil(2^32 / d); 0 stands for d = 1
__device__ __forceinline__ int FastDiv(int u, uint32_t magic) {
  return magic ? static_cast<int>(__umulhi(static_cast<uint32_t>(u), magic)) : u;
}

template <int KSTEPS, int RQ, bool ZP>
__global__ void __launch_bounds__(kBandThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
ConvBandKernel(BandArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int hw = a.OH * a.OW;

  // An XCD gets a contiguous run of bands (neighbouring bands of an image share halo rows and meet in that
  // XCD's L2); inside the run the XCD's workgroups interleave.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const int t_first = static_cast<int>(static_cast<long long>(a.total_tiles) * xcd / 8);
  const int t_end = static_cast<int>(static_cast<long long>(a.total_tiles) * (xcd + 1) / 8);
  int t = t_first + slot;
  if (t >= t_end) return;

  int* sx_lds = reinterpret_cast<int*>(lds + a.off_sx) + wave * 32;  // wavefront-private
  const v4i* rq_lds = reinterpret_cast<const v4i*>(lds + a.off_rq);
  const int* bias_lds = reinterpret_cast<const int*>(lds + a.off_bias);
  int8_t* stage = lds + a.off_stage + wave * (32 * kStageStride);  // wavefront-private

  // ---- this thread's patch: 8 input columns x 4 channels of one halo row. Sixteen consecutive lanes read
  // 128 contiguous bytes of a channel plane, the next sixteen the next channel group.
  const size_t plane = static_cast<size_t>(a.H) * a.W;
  const uint32_t plane32 = static_cast<uint32_t>(plane);
  const int cb = FastDiv(wave, a.magic_gblocks);
  const int gb = wave - cb * a.gblocks;
  const int g8 = gb * 16 + (lane & 15);
  const int c4 = cb * 4 + (lane >> 4);
  const bool has_patch = g8 < a.n_g8 && c4 * 4 < a.C;
  const int hr = has_patch ? FastDiv(g8, a.magic_gpr) : 0;
  const int col0 = has_patch ? (g8 - hr * a.gpr) * 8 : 0;
  uint32_t ch_off[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) ch_off[j] = has_patch ? static_cast<uint32_t>(c4 * 4 + j) * plane32 + static_cast<uint32_t>(col0) : 0u;
  const int dst0 = (hr * a.iwt + a.pad_l + col0) * a.pix_stride + c4 * 4;

  auto tile_geometry = [&](int tile_index, int* n, int* tl) {
    const int img = FastDiv(tile_index, a.magic_tpi);
    *n = img;
    *tl = tile_index - img * a.tiles_per_image;
  };
  // Is this thread's halo row inside the image for band `tl`? (wavefront-varying: lanes hold different rows)
  auto row_of = [&](int tl, bool* inside) {
    const int r0 = tl * a.rows;
    const int rows_here = min(a.rows, a.OH - r0);
    const int ih = r0 * a.sh - a.pad_t + hr;
    *inside = hr < (rows_here - 1) * a.sh + a.khe && ih >= 0 && ih < a.H;
    return *inside ? ih : 0;  // rows outside read row 0 and are replaced by the zero point behind the load
  };
  auto issue_loads = [&](int2 (&d)[4], int tile_index) {
    int n, tl;
    tile_geometry(tile_index, &n, &tl);
    bool inside;
    const uint32_t row_off = __umul24(static_cast<uint32_t>(row_of(tl, &inside)), static_cast<uint32_t>(a.W));
    const uint8_t* img = a.x + static_cast<size_t>(n) * a.C * plane;
#pragma unroll
    for (int j = 0; j < 4; ++j) d[j] = *reinterpret_cast<const int2*>(img + (ch_off[j] + row_off));
  };
  auto store_halo = [&](const int2 (&d)[4], int tile_index, int8_t* halo) {
    int n, tl;
    tile_geometry(tile_index, &n, &tl);
    bool inside;
    (void)row_of(tl, &inside);
    const int keep = inside ? -1 : 0;
    uint32_t lo4[4], hi4[4], px[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lo4[j] = static_cast<uint32_t>(((d[j].x ^ a.xor_mask) & keep) | (a.pad_fill & ~keep));
      hi4[j] = static_cast<uint32_t>(((d[j].y ^ a.xor_mask) & keep) | (a.pad_fill & ~keep));
    }
    Transpose4x4(lo4, px);
    Transpose4x4(hi4, px + 4);
    if (has_patch) {
      int8_t* dst = halo + dst0;
#pragma unroll
      for (int i = 0; i < 8; ++i) *reinterpret_cast<uint32_t*>(dst + i * a.pix_stride) = px[i];
    }
  };
  auto lds_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  // ---- prologue: the first band's rows on their way, weights and tables by DMA, the padding columns of both
  // halo buffers (no band ever writes them again) ----
  int2 d0[4];
  issue_loads(d0, t);
  {
    typedef const __attribute__((address_space(1))) void* gptr;
    typedef __attribute__((address_space(3))) void* lptr;
    for (int i = wave * 64; i < a.w_chunks; i += kBandThreads)
      __builtin_amdgcn_global_load_lds((gptr)(a.w + static_cast<size_t>(i + lane) * 16), (lptr)(lds + a.off_w + i * 16), 16, 0, 0);
    if (wave == kBandWaves - 1) {
      __builtin_amdgcn_global_load_lds((gptr)(a.rq + lane), (lptr)(lds + a.off_rq), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((gptr)(a.biasf + lane), (lptr)(lds + a.off_bias), 4, 0, 0);
    }
  }
  {
    const int right0 = a.pad_l + a.W;
    const int cpc = a.C >> 4;
    const int units = a.halo_rows * a.pad_cols * cpc;
    const v4i fill = v4i{a.pad_fill, a.pad_fill, a.pad_fill, a.pad_fill};
    for (int u = tid; u < 2 * units; u += kBandThreads) {
      const int b = u >= units ? 1 : 0, v = u - b * units;
      const int cell = v / cpc, c = (v - cell * cpc) * 16;
      const int r = cell / a.pad_cols, pcol = cell - r * a.pad_cols;
      const int col = pcol < a.pad_l ? pcol : right0 + (pcol - a.pad_l);
      *reinterpret_cast<v4i*>(lds + (b ? a.off_halo1 : a.off_halo0) + (r * a.iwt + col) * a.pix_stride + c) = fill;
    }
  }
  store_halo(d0, t, lds + a.off_halo0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the DMA has landed
  lds_barrier();

  int buf = 0;
  for (; t < t_end; t += per_xcd) {
    const int tn = t + per_xcd;
    const bool has_next = tn < t_end;
    int2 dn[4];
    if (has_next) issue_loads(dn, tn);
    int n, tl;
    tile_geometry(t, &n, &tl);
    const int r0 = tl * a.rows;
    const int valid = min(a.rows, a.OH - r0) * a.OW;  // pixels of this band
    const int8_t* halo = lds + (buf ? a.off_halo1 : a.off_halo0);

    if (wave < a.PT && wave * 32 < valid) {
      const int pl = min(wave * 32 + frag_row, valid - 1);  // rows past the band's end recompute its last pixel
      const int ohl = FastDiv(pl, a.magic_ow), ow = pl - ohl * a.OW;
      const int8_t* frag = halo + (ohl * a.sh * a.iwt + ow * a.sw) * a.pix_stride + frag_half * 16;
      const int8_t* w_row = lds + a.off_w + frag_row * a.kstride + frag_half * 16;
      v16i acc[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int bias = bias_lds[j * 32 + frag_row];
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = bias;
      }
      int sx = 0;
      constexpr int RING = 3;
      v4i fa[RING], fb[RING][2];
      auto fetch = [&](int ks, int slot_) {
        fa[slot_] = *reinterpret_cast<const v4i*>(frag + a.tap_off[ks]);
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[slot_][j] = *reinterpret_cast<const v4i*>(w_row + j * 32 * a.kstride + ks * 32);
      };
#pragma unroll
      for (int q = 0; q < RING - 1; ++q)
        if (q < KSTEPS) fetch(q, q);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        if (ks + RING - 1 < KSTEPS) fetch(ks + RING - 1, (ks + RING - 1) % RING);
        const v4i f = fa[ks % RING];
        if (ZP) {
#pragma unroll
          for (int q = 0; q < 4; ++q) sx = __builtin_amdgcn_sdot4(f[q], 0x01010101, sx, false);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f, fb[ks % RING][j], acc[j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (ZP) {
        sx += __shfl_xor(sx, 32);
        __builtin_amdgcn_wave_barrier();
        if (frag_half == 0) sx_lds[frag_row] = a.zws * sx;
        __builtin_amdgcn_wave_barrier();
      }
      // ---- requantize one 32-channel tile at a time into the wavefront's staging tile, copy it out ----
      const int nvalid = min(32, valid - wave * 32);  // a multiple of 8
      uint8_t* ytile = a.y + static_cast<size_t>(n) * a.OC * hw + static_cast<size_t>(r0) * a.OW + wave * 32;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const v4i rq = rq_lds[j * 32 + frag_row];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          v4i s4 = v4i{0, 0, 0, 0};
          if (ZP) s4 = *reinterpret_cast<const v4i*>(sx_lds + 8 * g + 4 * frag_half);
          int r4[4];
#pragma unroll
          for (int e = 0; e < 4; ++e)
            r4[e] = Requant8<RQ>(ZP ? acc[j][g * 4 + e] - s4[e] : acc[j][g * 4 + e], rq, a.out_zp, a.lo, a.hi);
          *reinterpret_cast<uint32_t*>(stage + frag_row * kStageStride + 8 * g + 4 * frag_half) = PackBytes(r4[0], r4[1], r4[2], r4[3]);
        }
        __builtin_amdgcn_wave_barrier();
        // lane -> (channel lane / 2, 16-byte half lane % 2) of the 32 x 32 tile
        const int ocl = lane >> 1, h16 = (lane & 1) * 16;
        const int2 v0 = *reinterpret_cast<const int2*>(stage + ocl * kStageStride + h16);
        const int2 v1 = *reinterpret_cast<const int2*>(stage + ocl * kStageStride + h16 + 8);
        const int oc = j * 32 + ocl;
        uint8_t* dst = ytile + static_cast<size_t>(oc) * hw + h16;
        if (oc < a.OC) {
          if (h16 + 16 <= nvalid) *reinterpret_cast<v4i*>(dst) = v4i{v0.x, v0.y, v1.x, v1.y};
          else if (h16 + 8 <= nvalid) *reinterpret_cast<int2*>(dst) = v0;
        }
        __builtin_amdgcn_wave_barrier();  // the staging tile is read before the next channel tile overwrites it
      }
    }
    if (has_next) {
      store_halo(dn, tn, lds + (buf ? a.off_halo0 : a.off_halo1));
      lds_barrier();  // the next band's halo tile is complete; everyone is done reading the present one
    }
    buf ^= 1;
  }
}

struct BandPlan {
  BandArgs a;
  int lds_bytes;
  int ksteps, rq;
  bool zp;
  unsigned grid;
};

typedef void (*BandFn)(BandArgs);
template <int KSTEPS>
BandFn BandKernelOf(int rq, bool zp) {
  if (rq == kRqFastNoTie) return zp ? ConvBandKernel<KSTEPS, kRqFastNoTie, true> : ConvBandKernel<KSTEPS, kRqFastNoTie, false>;
  return zp ? ConvBandKernel<KSTEPS, kRqFast, true> : ConvBandKernel<KSTEPS, kRqFast, false>;
}
BandFn BandKernel(int ksteps, int rq, bool zp) {
  if (rq == kRqGeneric) return nullptr;
  switch (ksteps) {
    case 9: return BandKernelOf<9>(rq, zp);
    case 18: return BandKernelOf<18>(rq, zp);
  }
  return nullptr;
}

int ConvBandRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const BandPlan* plan = reinterpret_cast<const BandPlan*>(op->host_blob.data());
  BandArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if (reinterpret_cast<uintptr_t>(in0) & 3 || reinterpret_cast<uintptr_t>(out) & 7)
    return SetError(TVX_E_INVALID, "conv2d_band_i8: the input must be 4-byte aligned, the output 8-byte aligned");
  hipLaunchKernelGGL(BandKernel(plan->ksteps, plan->rq, plan->zp), dim3(plan->grid), dim3(kBandThreads), plan->lds_bytes, st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

int RoundUp(int v, int m) { return (v + m - 1) / m * m; }
uint32_t Magic(int d) { return d <= 1 ? 0u : static_cast<uint32_t>(((uint64_t{1} << 32) + d - 1) / d); }
// Is floor(u * Magic(d) / 2^32) == u / d for every 0 <= u <= umax?
bool MagicExact(int d, uint64_t umax) {
  // the error of ceil(2^32 / d) is below d / 2^32 per unit of u: exact while umax * d < 2^32
  return umax * static_cast<uint64_t>(d) < (uint64_t{1} << 32);
}

}  // namespace

// Claims dense quantized convolutions with constant weights, 32 or 64 input channels, 33 to 64 output channels and
// rows of whole 8-byte units, whose weights and two halo tiles of a band of output rows fit one workgroup's LDS.
int ConvBandSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || d->multiplier != 0 || d->groups > 1) return TVX_E_UNSUPPORTED;
  bool forced = false;
  if (const char* f = getenv("TVX_CONV_BAND")) {  // test lever: 0 declines, 1 claims also where few bands make it the slower choice
    if (atoi(f) == 0) return TVX_E_UNSUPPORTED;
    forced = true;
  }
  BandArgs a{};
  a.C = d->in_c; a.H = d->in_h; a.W = d->in_w; a.OC = d->out_c; a.OH = d->out_h; a.OW = d->out_w;
  a.sh = d->stride_h; a.sw = d->stride_w; a.pad_t = d->pad_top; a.pad_l = d->pad_left;
  const int kh = d->k_h, kw = d->k_w, dh = d->dilation_h, dw = d->dilation_w;
  const int taps = kh * kw;
  if (a.C % 32 || a.C > 64 || a.OC <= 32 || a.OC > 64 || a.W % 8 || a.OW % 8) return TVX_E_UNSUPPORTED;
  const int cpc = a.C / 16;
  const int ksteps = taps * cpc / 2;
  if (ksteps > 20) return TVX_E_UNSUPPORTED;
  a.khe = (kh - 1) * dh + 1;
  a.iwt = std::max((a.OW - 1) * a.sw + (kw - 1) * dw + 1, a.pad_l + a.W);
  a.pad_cols = a.iwt - a.W;
  a.pix_stride = (cpc & 1) ? a.C : a.C + 16;  // an odd number of 16-byte chunks: consecutive pixels fall into different bank groups
  a.kstride = ksteps * 32 + 16;
  const int w_bytes = RoundUp(64 * a.kstride, 1024);
  a.w_chunks = w_bytes / 16;
  a.gpr = a.W / 8;

  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127) return TVX_E_UNSUPPORTED;
  a.xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.pad_fill = static_cast<int>(static_cast<uint32_t>(zxs & 0xff) * 0x01010101u);
  a.zws = zws;
  a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;

  std::vector<int32_t> rqt;
  const int rq = BuildRequantRecords(op->h_mult, op->h_shift, a.OC, 64, d->out_zp, &rqt,
                                     AccumulatorBound(static_cast<uint64_t>(taps) * a.C, bias_host, a.OC));
  BandFn fn = BandKernel(ksteps, rq, zws != 0);
  if (!fn) return TVX_E_UNSUPPORTED;

  hipDeviceProp_t prop;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return TVX_E_UNSUPPORTED;
  const int cus = std::max(8, prop.multiProcessorCount / 8 * 8);

  // ---- rows of a band: what the loader (one patch per thread), the wavefronts (one 32-pixel tile each) and LDS
  // allow; among those the choice that needs the fewest rounds of bands, each priced by its rows plus a fixed part
  int best_rows = 0, best_lds = 0;
  long long best_cost = 0;
  int want_rows = 0;
  if (const char* f = getenv("TVX_BAND_ROWS")) want_rows = atoi(f);  // test lever
  for (int r = 1; r <= a.OH; ++r) {
    const int halo_rows = (r - 1) * a.sh + a.khe;
    const int n_g8 = halo_rows * a.gpr;
    const int gblocks = (n_g8 + 15) / 16;
    if (gblocks * (a.C / 16) > kBandWaves) break;
    if ((r * a.OW + 31) / 32 > kBandWaves) break;
    const int halo_bytes = RoundUp(halo_rows * a.iwt * a.pix_stride + 64, 16);
    const int lds_bytes = kBandWaves * 128 + 64 * 16 + 64 * 4 + w_bytes + kBandWaves * 32 * kStageStride + 2 * halo_bytes;
    if (lds_bytes > 160 * 1024) break;
    const long long tiles = static_cast<long long>(d->batch) * ((a.OH + r - 1) / r);
    const long long cost = (tiles + cus - 1) / cus * (r + 2);
    if (best_rows == 0 || cost <= best_cost || r == want_rows) { best_rows = r; best_cost = cost; best_lds = lds_bytes; }
    if (r == want_rows) break;
  }
  if (best_rows == 0) return TVX_E_UNSUPPORTED;
  a.rows = best_rows;
  a.halo_rows = (a.rows - 1) * a.sh + a.khe;
  a.n_g8 = a.halo_rows * a.gpr;
  a.gblocks = (a.n_g8 + 15) / 16;
  a.PT = (a.rows * a.OW + 31) / 32;
  a.tiles_per_image = (a.OH + a.rows - 1) / a.rows;
  const uint64_t total = static_cast<uint64_t>(d->batch) * a.tiles_per_image;
  if (total > 0x7fffffffull) return TVX_E_UNSUPPORTED;
  a.total_tiles = static_cast<int>(total);
  // a handful of bands cannot fill the chip this way: the one-tile-per-workgroup kernel spreads them wider
  if (a.total_tiles < cus * 3 / 4 && !forced) return TVX_E_UNSUPPORTED;
  if (!MagicExact(a.tiles_per_image, total) || !MagicExact(a.OW, static_cast<uint64_t>(a.rows) * a.OW) ||
      !MagicExact(a.gpr, 1024) || !MagicExact(a.gblocks, kBandWaves))
    return TVX_E_UNSUPPORTED;
  a.magic_tpi = Magic(a.tiles_per_image);
  a.magic_ow = Magic(a.OW);
  a.magic_gpr = Magic(a.gpr);
  a.magic_gblocks = Magic(a.gblocks);
  // the loader's 24-bit multiplies and 32-bit offsets inside one image
  if (static_cast<uint64_t>(a.H) * a.W >= (1ull << 24) || static_cast<uint64_t>(a.H) * a.W * a.C >= (1ull << 31)) return TVX_E_UNSUPPORTED;

  const int halo_bytes = RoundUp(a.halo_rows * a.iwt * a.pix_stride + 64, 16);
  a.off_sx = 0;
  a.off_rq = kBandWaves * 128;
  a.off_bias = a.off_rq + 64 * 16;
  a.off_w = a.off_bias + 64 * 4;
  a.off_stage = a.off_w + w_bytes;
  a.off_halo0 = a.off_stage + kBandWaves * 32 * kStageStride;
  a.off_halo1 = a.off_halo0 + halo_bytes;
  const int lds_bytes = a.off_halo1 + halo_bytes;
  if (lds_bytes != best_lds) return SetError(TVX_E_INVALID, "conv2d_band_i8: LDS plan mismatch (%d, %d)", lds_bytes, best_lds);
  for (int ks = 0; ks < ksteps; ++ks) {
    const int q = 2 * ks, tp = q / cpc, cc = q % cpc;  // chunk 2 * ks; cpc is even, so chunk 2 * ks + 1 is the same tap's next chunk
    a.tap_off[ks] = ((tp / kw) * dh * a.iwt + (tp % kw) * dw) * a.pix_stride + cc * 16;
  }

  // ---- pack weights [oc][(ky, kx, c)] int8 with zero padding, fold constants into the bias ----
  std::vector<int8_t> packed(static_cast<size_t>(w_bytes) + 1024, 0);
  std::vector<int32_t> biasf(64, 0);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  for (int oc = 0; oc < a.OC; ++oc) {
    int64_t sw = 0;
    for (int tp = 0; tp < taps; ++tp)
      for (int c = 0; c < a.C; ++c) {
        const uint8_t raw = src[(static_cast<size_t>(oc) * a.C + c) * taps + tp];
        const int8_t v = static_cast<int8_t>(w_u8 ? raw ^ 0x80 : raw);
        packed[static_cast<size_t>(oc) * a.kstride + tp * a.C + c] = v;
        sw += v;
      }
    const int64_t v = (b ? b[oc] : 0) - static_cast<int64_t>(zxs) * sw + static_cast<int64_t>(taps) * a.C * zxs * zws;
    biasf[oc] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  int s = op->packed.Upload(packed.data(), packed.size());
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s != TVX_OK) return s;
  a.w = op->packed.as<int8_t>();
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<v4i>();
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) {
    (void)hipGetLastError();
    return TVX_E_UNSUPPORTED;
  }
  BandPlan plan;
  plan.a = a;
  plan.lds_bytes = lds_bytes;
  plan.ksteps = ksteps;
  plan.rq = rq;
  plan.zp = zws != 0;
  int wgs = cus;
  if (const char* f = getenv("TVX_BAND_WGS")) wgs = std::max(8, atoi(f) / 8 * 8);  // test lever
  plan.grid = static_cast<unsigned>(std::min(wgs, RoundUp(a.total_tiles, 8)));
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = ConvBandRun;
  op->kernel_name = "conv2d_band_i8";
  return TVX_OK;
}

}  // namespace tvx
