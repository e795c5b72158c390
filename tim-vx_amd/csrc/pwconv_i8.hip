// Pointwise (1x1, stride 1, unpadded) quantized Conv2d on the int8 matrix cores.
//
// With a 1x1 kernel there is no window: the pixels of the whole batch form one
// flat axis q = n * HW + p, and the op is Y[oc][q] = requant(sum_c W[oc][c] X[c][q]).
// It moves far more bytes than it multiplies, so the kernel is organised around
// the memory system, not the MFMA pipe:
//   * a workgroup owns 128 consecutive flat pixels and keeps their activations
//     for ALL input channels in LDS, channel-innermost (the WHCN input is
//     pixel-innermost; 4x4 byte transposes happen in registers on the way in, with
//     every global load of a thread in flight at once) - the input is read once;
//   * each wavefront owns whole 32-channel output tiles for all 128 pixels, so
//     its results are full 128-byte rows of the WHCN output: it stages them in a
//     private LDS patch and writes them itself - no workgroup barrier after the
//     input tile is built, and every global store is a complete cache line;
//   * weights are pre-packed in MFMA fragment order and stream global -> registers
//     (1 KiB contiguous per wavefront load, prefetched two steps ahead across tile
//     boundaries); they are small and live in L2.
// Zero points: sum (x - zx)(w - zw) = sum xs ws - zws Sx - zxs Sw + C zxs zws with
// xs, ws the operands moved to the signed int8 domain; Sx per pixel comes from
// v_dot4 on the fragments, the per-channel constants are folded into the bias.
#include <algorithm>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kPix = 128;          // flat pixels per workgroup
constexpr int kPixTiles = kPix / 32;
constexpr int kStageStride = 136;  // bytes per staged output row: 34 dwords spread 32 rows over all banks
constexpr int kStageBytes = 32 * kStageStride;
constexpr int kWaveLds = kStageBytes + kPix * 4;  // staging patch + per-pixel sums

struct PwArgs {
  const uint8_t* x;
  uint8_t* y;
  const v4i* wpk;        // [oc tile][k-step][lane]: 16 reduction bytes of channel tile*32 + lane%32
  const int32_t* biasf;  // bias + per-channel zero-point terms
  const v4i* rq;         // per channel requantization record
  int C, OC, HW;
  long long Q;           // batch * HW
  int cp;                // channels padded to 32
  int ksteps;            // cp / 32
  int pix_stride;        // LDS bytes per pixel: cp + 16 (an odd number of 16-byte chunks)
  int oc_tiles;          // ceil(OC / 32)
  int tiles_per_wg;      // output tiles one workgroup walks (grid.y covers the rest)
  int xor_mask;          // 0x80808080 for uint8 activations
  int zws, out_zp, lo, hi;
};

// 4 dwords = 4 channels x 4 pixels (pixel in the byte lanes) -> 4 dwords = 4 pixels x 4 channels.
__device__ __forceinline__ void Transpose4x4(const uint32_t in[4], uint32_t out[4]) {
  const uint32_t ab_lo = __builtin_amdgcn_perm(in[1], in[0], 0x05010400);  // a0 b0 a1 b1
  const uint32_t ab_hi = __builtin_amdgcn_perm(in[1], in[0], 0x07030602);  // a2 b2 a3 b3
  const uint32_t cd_lo = __builtin_amdgcn_perm(in[3], in[2], 0x05010400);
  const uint32_t cd_hi = __builtin_amdgcn_perm(in[3], in[2], 0x07030602);
  out[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100);  // a0 b0 c0 d0
  out[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302);  // a1 b1 c1 d1
  out[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100);
  out[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302);
}

// GRAN: pixels that are guaranteed to stay inside one image and to be aligned:
// 16 (HW % 16 == 0), 4 (HW % 4 == 0) or 1.
template <int GRAN, bool SX, int RQ>
__global__ void __launch_bounds__(kThreads) PwConvKernel(PwArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const long long q_base = static_cast<long long>(blockIdx.x) * kPix;
  int8_t* xl = lds;
  int8_t* stage = lds + kPix * a.pix_stride + wave * kWaveLds;
  int* sx_lds = reinterpret_cast<int*>(stage + kStageBytes);

  // ---- activations of the 128 pixels, all channels: global (pixel-innermost) -> LDS
  if (GRAN >= 4) {
    const int pq = tid & 31, cg0 = tid >> 5;  // 4-pixel group, first 16-channel group
    const long long q0 = q_base + pq * 4;
    const bool live = q0 < a.Q;
    const long long n = live ? q0 / a.HW : 0;
    const int p = live ? static_cast<int>(q0 - n * a.HW) : 0;
    const uint8_t* src = a.x + (static_cast<size_t>(n) * a.C) * a.HW + p;
    for (int cg = cg0; cg < a.cp / 16; cg += 8) {
      uint32_t raw[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int c = cg * 16 + j;
        raw[j] = (live && c < a.C)
                     ? *reinterpret_cast<const uint32_t*>(src + static_cast<size_t>(c) * a.HW) ^ a.xor_mask
                     : 0u;
      }
      uint32_t t[4][4];
#pragma unroll
      for (int b = 0; b < 4; ++b) Transpose4x4(raw + 4 * b, t[b]);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v4i v = {static_cast<int>(t[0][e]), static_cast<int>(t[1][e]), static_cast<int>(t[2][e]),
                 static_cast<int>(t[3][e])};
        *reinterpret_cast<v4i*>(xl + (pq * 4 + e) * a.pix_stride + cg * 16) = v;
      }
    }
  } else {
    const int px = tid & 127, cg0 = tid >> 7;
    const long long q0 = q_base + px;
    const bool live = q0 < a.Q;
    const long long n = live ? q0 / a.HW : 0;
    const int p = live ? static_cast<int>(q0 - n * a.HW) : 0;
    const uint8_t* src = a.x + (static_cast<size_t>(n) * a.C) * a.HW + p;
    for (int cg = cg0; cg < a.cp / 16; cg += 2) {
      uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int c = cg * 16 + j;
        const uint32_t b = (live && c < a.C) ? (src[static_cast<size_t>(c) * a.HW] ^ (a.xor_mask & 0xff)) : 0u;
        w[j >> 2] |= b << (8 * (j & 3));
      }
      v4i v = {static_cast<int>(w[0]), static_cast<int>(w[1]), static_cast<int>(w[2]), static_cast<int>(w[3])};
      *reinterpret_cast<v4i*>(xl + px * a.pix_stride + cg * 16) = v;
    }
  }

  // ---- where this lane's output groups live (the same for every output tile) -----
  // Copy-out mapping: GRAN 16: lane -> (row lane/8 + 8 i, 16-pixel chunk lane%8);
  // GRAN 4: lane -> (row lane/32 + 2 i, dword lane%32); GRAN 1: lane -> pixels lane, lane+64.
  constexpr int kGroups = GRAN == 1 ? 2 : 1;
  size_t out_off[kGroups];
  bool out_live[kGroups];
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    const int px = GRAN == 16 ? (lane & 7) * 16 : (GRAN == 4 ? (lane & 31) * 4 : lane + 64 * g);
    const long long q0 = q_base + px;
    out_live[g] = q0 < a.Q;
    const long long n = out_live[g] ? q0 / a.HW : 0;
    out_off[g] = static_cast<size_t>(n) * a.OC * a.HW + static_cast<size_t>(q0 - n * a.HW);
  }

  // ---- output tiles of this wavefront ------------------------------------------------
  const int t_begin = blockIdx.y * a.tiles_per_wg;
  const int t_end = min(t_begin + a.tiles_per_wg, a.oc_tiles);
  const int n_tiles = (t_end - t_begin - wave + 3) / 4;  // tiles t_begin + wave + 4 j
  __syncthreads();  // the input tile is complete; nothing below needs the other wavefronts
  if (n_tiles <= 0) return;

  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int8_t* xa = xl + frag_row * a.pix_stride + frag_half * 16;
  const int total = n_tiles * a.ksteps;

  // weight fragment stream, in consumption order
  int pf_tile = t_begin + wave, pf_ks = 0, pf_left = total;
  auto next_frag = [&]() -> v4i {
    const v4i f = a.wpk[(static_cast<size_t>(pf_tile) * a.ksteps + pf_ks) * 64 + lane];
    if (--pf_left > 0) {  // past the end: keep re-reading the last fragment
      if (++pf_ks == a.ksteps) { pf_ks = 0; pf_tile += 4; }
    }
    return f;
  };

  v16i acc[kPixTiles];
  int sx[kPixTiles] = {0, 0, 0, 0};
  int tile = t_begin + wave, ks = 0;
  bool first = true;
  auto init_acc = [&]() {
    const int b = a.biasf[tile * 32 + frag_row];
#pragma unroll
    for (int i = 0; i < kPixTiles; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][r] = b;
  };

  auto epilogue = [&]() {
    if (SX && first) {
#pragma unroll
      for (int i = 0; i < kPixTiles; ++i) {
        sx[i] += __shfl_xor(sx[i], 32);
        if (frag_half == 0) sx_lds[i * 32 + frag_row] = a.zws * sx[i];
      }
    }
    first = false;
    __builtin_amdgcn_wave_barrier();
    const int oc = tile * 32 + frag_row;
    const v4i q = a.rq[oc];
#pragma unroll
    for (int i = 0; i < kPixTiles; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int pl = i * 32 + 8 * g + 4 * frag_half;
        v4i s4 = {0, 0, 0, 0};
        if (SX) s4 = *reinterpret_cast<const v4i*>(sx_lds + pl);
        uint32_t packed = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int v = acc[i][g * 4 + e] - s4[e];
          packed |= static_cast<uint32_t>(Requant8<RQ>(v, q, a.out_zp, a.lo, a.hi) & 0xff) << (8 * e);
        }
        *reinterpret_cast<uint32_t*>(stage + frag_row * kStageStride + pl) = packed;
      }
    __builtin_amdgcn_wave_barrier();
    // copy-out: rows of the staging patch -> WHCN output
    const int rows = min(32, a.OC - tile * 32);
    uint8_t* ybase = a.y + static_cast<size_t>(tile) * 32 * a.HW;
    if (GRAN == 16) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = (lane >> 3) + 8 * i;
        const int8_t* s = stage + row * kStageStride + (lane & 7) * 16;
        const uint2 lo = *reinterpret_cast<const uint2*>(s);
        const uint2 hi = *reinterpret_cast<const uint2*>(s + 8);
        if (row < rows && out_live[0])
          *reinterpret_cast<uint4*>(ybase + out_off[0] + static_cast<size_t>(row) * a.HW) =
              make_uint4(lo.x, lo.y, hi.x, hi.y);
      }
    } else if (GRAN == 4) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = (lane >> 5) + 2 * i;
        const uint32_t v = *reinterpret_cast<const uint32_t*>(stage + row * kStageStride + (lane & 31) * 4);
        if (row < rows && out_live[0])
          *reinterpret_cast<uint32_t*>(ybase + out_off[0] + static_cast<size_t>(row) * a.HW) = v;
      }
    } else {
      for (int row = 0; row < rows; ++row)
#pragma unroll
        for (int g = 0; g < kGroups; ++g)
          if (out_live[g])
            ybase[out_off[g] + static_cast<size_t>(row) * a.HW] =
                static_cast<uint8_t>(stage[row * kStageStride + lane + 64 * g]);
    }
    __builtin_amdgcn_wave_barrier();
  };

  auto step = [&](const v4i& fw) {
    v4i fx[kPixTiles];
#pragma unroll
    for (int i = 0; i < kPixTiles; ++i)
      fx[i] = *reinterpret_cast<const v4i*>(xa + i * 32 * a.pix_stride + ks * 32);
    if (SX && first) {
#pragma unroll
      for (int i = 0; i < kPixTiles; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) sx[i] = __builtin_amdgcn_sdot4(fx[i][j], 0x01010101, sx[i], false);
    }
#pragma unroll
    for (int i = 0; i < kPixTiles; ++i)
      acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx[i], fw, acc[i], 0, 0, 0);
    if (++ks == a.ksteps) {
      epilogue();
      ks = 0;
      tile += 4;
      if (tile < t_end) init_acc();
    }
  };

  v4i f0 = next_frag();
  v4i f1 = next_frag();
  init_acc();
  for (int idx = 0; idx < total; idx += 2) {
    const v4i g0 = f0;
    f0 = next_frag();
    step(g0);
    if (idx + 1 < total) {
      const v4i g1 = f1;
      f1 = next_frag();
      step(g1);
    }
  }
}

struct Plan {
  PwArgs a;
  int lds_bytes, gran, sx, rq;
  dim3 grid;
};

template <int GRAN, bool SX, int RQ>
int Launch(const Plan* plan, const PwArgs& a, hipStream_t st, bool configure) {
  if (configure) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&PwConvKernel<GRAN, SX, RQ>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, plan->lds_bytes);
    if (e != hipSuccess)
      return SetError(TVX_E_DEVICE, "hipFuncSetAttribute(dynamic LDS %d): %s", plan->lds_bytes, hipGetErrorString(e));
    return TVX_OK;
  }
  hipLaunchKernelGGL((PwConvKernel<GRAN, SX, RQ>), plan->grid, dim3(kThreads), plan->lds_bytes, st, a);
  return TVX_OK;
}

template <int GRAN, bool SX>
int DispatchRq(const Plan* plan, const PwArgs& a, hipStream_t st, bool configure) {
  if (plan->rq == kRqFastNoTie) return Launch<GRAN, SX, kRqFastNoTie>(plan, a, st, configure);
  if (plan->rq == kRqFast) return Launch<GRAN, SX, kRqFast>(plan, a, st, configure);
  return Launch<GRAN, SX, kRqGeneric>(plan, a, st, configure);
}

template <int GRAN>
int DispatchSx(const Plan* plan, const PwArgs& a, hipStream_t st, bool configure) {
  return plan->sx ? DispatchRq<GRAN, true>(plan, a, st, configure) : DispatchRq<GRAN, false>(plan, a, st, configure);
}

int Dispatch(const Plan* plan, const PwArgs& a, hipStream_t st, bool configure) {
  if (plan->gran == 16) return DispatchSx<16>(plan, a, st, configure);
  if (plan->gran == 4) return DispatchSx<4>(plan, a, st, configure);
  return DispatchSx<1>(plan, a, st, configure);
}

int PwConvRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  PwArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(out)) & (plan->gran - 1))
    return SetError(TVX_E_INVALID, "pwconv_i8: tensors must be %d-byte aligned", plan->gran);
  const int s = Dispatch(plan, a, st, false);
  if (s != TVX_OK) return s;
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

int RoundUp(int v, int m) { return (v + m - 1) / m * m; }

}  // namespace

// Claims dense quantized 1x1 convolutions with unit stride, no padding and constant
// weights whose 128-pixel input tile fits the CU's LDS.
int PwConvSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || d->multiplier != 0) return TVX_E_UNSUPPORTED;
  if (d->k_w != 1 || d->k_h != 1 || d->stride_w != 1 || d->stride_h != 1 || d->pad_left != 0 ||
      d->pad_top != 0 || d->out_w != d->in_w || d->out_h != d->in_h)
    return TVX_E_UNSUPPORTED;
  PwArgs a{};
  a.C = d->in_c;
  a.OC = d->out_c;
  const uint64_t hw = static_cast<uint64_t>(d->in_w) * d->in_h;
  if (hw >= (1ull << 30)) return TVX_E_UNSUPPORTED;
  a.HW = static_cast<int>(hw);
  a.Q = static_cast<long long>(hw) * d->batch;
  a.cp = RoundUp(a.C, 32);
  a.ksteps = a.cp / 32;
  a.pix_stride = a.cp + 16;
  a.oc_tiles = (a.OC + 31) / 32;
  const int lds_bytes = kPix * a.pix_stride + 4 * kWaveLds;
  if (lds_bytes > 160 * 1024) return TVX_E_UNSUPPORTED;
  const long long gx = (a.Q + kPix - 1) / kPix;
  if (gx > 0x7fffffffll) return TVX_E_UNSUPPORTED;
  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127) return TVX_E_UNSUPPORTED;  // zero point outside the tensor's range
  a.xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.zws = zws;
  a.out_zp = d->out_zp;
  a.lo = op->act_lo;
  a.hi = op->act_hi;
  // few pixel tiles: spread the output tiles over grid.y (in units of one tile per
  // wavefront) until the launch has a few workgroups per CU
  const int quads = (a.oc_tiles + 3) / 4;
  int gy = static_cast<int>(std::min<long long>(quads, std::max<long long>(1, 1024 / gx)));
  a.tiles_per_wg = ((quads + gy - 1) / gy) * 4;
  gy = (a.oc_tiles + a.tiles_per_wg - 1) / a.tiles_per_wg;

  // ---- weights in fragment order, constants folded into the bias -------------------
  const int oc_alloc = a.oc_tiles * 32;
  std::vector<int8_t> packed(static_cast<size_t>(a.oc_tiles) * a.ksteps * 1024, 0);
  std::vector<int32_t> biasf(oc_alloc, 0);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  for (int oc = 0; oc < a.OC; ++oc) {
    int64_t sw = 0;
    for (int c = 0; c < a.C; ++c) {
      const uint8_t raw = src[static_cast<size_t>(oc) * a.C + c];
      const int8_t v = static_cast<int8_t>(w_u8 ? raw ^ 0x80 : raw);
      const int ks = c / 32, half = (c % 32) / 16, j = c % 16;
      const int lane = half * 32 + oc % 32;
      packed[((static_cast<size_t>(oc / 32) * a.ksteps + ks) * 64 + lane) * 16 + j] = v;
      sw += v;
    }
    const int64_t v = (b ? b[oc] : 0) - static_cast<int64_t>(zxs) * sw + static_cast<int64_t>(a.C) * zxs * zws;
    biasf[oc] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  std::vector<int32_t> rqt;
  const int rq = BuildRequantRecords(op->h_mult, op->h_shift, a.OC, oc_alloc, d->out_zp, &rqt);
  int s = op->packed.Upload(packed.data(), packed.size());
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s != TVX_OK) return s;
  a.wpk = op->packed.as<v4i>();
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<v4i>();

  Plan plan;
  plan.a = a;
  plan.lds_bytes = lds_bytes;
  plan.gran = (a.HW % 16 == 0) ? 16 : ((a.HW % 4 == 0) ? 4 : 1);
  plan.sx = zws != 0;
  plan.rq = rq;
  plan.grid = dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy));
  s = Dispatch(&plan, a, nullptr, true);
  if (s != TVX_OK) return s;
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = PwConvRun;
  op->kernel_name = "pwconv_i8";
  return TVX_OK;
}

}  // namespace tvx
