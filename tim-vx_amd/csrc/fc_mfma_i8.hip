// FullyConnected on the int8 matrix cores: out[m][n] = requant(sum_k x[m][k] w[n][k] ...).
// Both operands are K-contiguous (an "NT" GEMM), which is exactly the operand
// shape v_mfma_i32_32x32x32_i8 wants: every lane feeds 16 consecutive K bytes.
//
// Tiling: one 256-thread workgroup (4 wavefronts, 2 x 2) owns a TM x TN = 256 x 256
// output tile and walks K in steps of 128 bytes; each wavefront accumulates a
// 128 x 128 sub-tile as 4 x 4 MFMA tiles (256 accumulator registers per lane).
// Global -> registers -> LDS, double buffered (2 x 64 KiB of the CU's 160 KiB);
// rows are 128 B in LDS and their 16 B chunks are XOR-swizzled with the row
// number so that the 32 lanes of a fragment read hit 8 different bank groups.
//
// The MFMA "A" operand is the weight fragment and "B" the activation fragment,
// so a lane ends up with one activation row m and, per accumulator quad, four
// consecutive features n: four requantized bytes make one dword of the row-major
// output, and the per-row correction term of the zero-point expansion
//   sum (x - zx)(w - zw) = sum xs ws - zws * sum_k xs - zxs * sum_k ws + K zxs zws
// (xs = x - 128 for uint8, zxs likewise) is per lane, with no exchange needed.
// The per-feature terms are folded into the bias at creation.
#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int TM = 256, TN = 256, TK = 128;
constexpr int kThreads = 256;
constexpr int kTileBytes = TM * TK;             // 32 KiB per operand tile
constexpr int kLdsBytes = 4 * kTileBytes;       // X and W, two stages
constexpr int kOutStride = TN + 16;             // epilogue staging row stride (bytes)

struct FcArgs {
  const int8_t* x;      // [M][K] (uint8 is re-biased to int8 on the fly)
  const int8_t* w;      // [N][K] int8 (uint8 weights are re-biased when packed)
  int8_t* y;            // [M][N]
  const int32_t* biasf; // [N] bias + per-feature zero-point terms
  const int32_t* mult;  // [N]
  const int32_t* shift; // [N]
  int M, N, K;
  int zws;              // weight zero point in the int8 domain (0 for per-channel)
  int out_zp, lo, hi;
  int tiles_m, tiles_n;
};

__device__ __forceinline__ int SwizzledOffset(int row, int chunk) {
  return row * TK + ((chunk ^ (row & 7)) << 4);
}

template <bool X_U8, bool ROWSUM>
__global__ void __launch_bounds__(kThreads, 1) FcMfmaKernel(FcArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
  // run of tiles so that neighbours in its L2 share operand panels.
  int tile = blockIdx.x;
  const int total = a.tiles_m * a.tiles_n;
  if ((total & 7) == 0) tile = (tile & 7) * (total >> 3) + (tile >> 3);
  // inside a run, walk 8 tiles along n before stepping m
  const int tn_idx = tile % a.tiles_n, tm_idx = tile / a.tiles_n;
  const int m0 = tm_idx * TM, n0 = tn_idx * TN;

  // ---- global -> register staging: thread t carries chunk (t % 8) of rows t/8 + 32 i
  const int ld_chunk = tid & 7;
  const int ld_row = tid >> 3;
  v4i stage_x[8], stage_w[8];

  auto load_global = [&](int k0) {
    const int kc = k0 + ld_chunk * 16;
    const bool k_ok = kc < a.K;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = ld_row + 32 * i;
      v4i vx = {0, 0, 0, 0}, vw = {0, 0, 0, 0};
      if (k_ok && m0 + r < a.M) {
        vx = *reinterpret_cast<const v4i*>(a.x + static_cast<size_t>(m0 + r) * a.K + kc);
        if (X_U8) vx ^= static_cast<int>(0x80808080);
      }
      if (k_ok && n0 + r < a.N)
        vw = *reinterpret_cast<const v4i*>(a.w + static_cast<size_t>(n0 + r) * a.K + kc);
      stage_x[i] = vx;
      stage_w[i] = vw;
    }
  };
  auto store_lds = [&](int stage) {
    int8_t* xs = lds + stage * 2 * kTileBytes;
    int8_t* ws = xs + kTileBytes;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = ld_row + 32 * i;
      const int off = SwizzledOffset(r, ld_chunk);
      *reinterpret_cast<v4i*>(xs + off) = stage_x[i];
      *reinterpret_cast<v4i*>(ws + off) = stage_w[i];
    }
  };

  v16i acc[4][4];  // [tn][tm]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  int rowsum[4] = {0, 0, 0, 0};

  const int frag_row = lane & 31;   // row inside a 32-row MFMA tile
  const int frag_half = lane >> 5;  // which 16-byte half of a 32-byte k-step

  const int k_tiles = (a.K + TK - 1) / TK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int kt = 0; kt < k_tiles; ++kt) {
    const int stage = kt & 1;
    if (kt + 1 < k_tiles) load_global((kt + 1) * TK);
    const int8_t* xs = lds + stage * 2 * kTileBytes;
    const int8_t* ws = xs + kTileBytes;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int chunk = kk * 2 + frag_half;
      v4i fx[4], fw[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        fx[t] = *reinterpret_cast<const v4i*>(xs + SwizzledOffset(wm * 128 + t * 32 + frag_row, chunk));
        fw[t] = *reinterpret_cast<const v4i*>(ws + SwizzledOffset(wn * 128 + t * 32 + frag_row, chunk));
      }
      if (ROWSUM) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            rowsum[t] = __builtin_amdgcn_sdot4(fx[t][q], 0x01010101, rowsum[t], false);
      }
#pragma unroll
      for (int tn = 0; tn < 4; ++tn)
#pragma unroll
        for (int tm = 0; tm < 4; ++tm)
          acc[tn][tm] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[tn], fx[tm], acc[tn][tm], 0, 0, 0);
    }
    if (kt + 1 < k_tiles) store_lds(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue: requantize, stage the int8 tile in LDS, store 16-byte rows ----
  if (ROWSUM) {
#pragma unroll
    for (int t = 0; t < 4; ++t) rowsum[t] += __shfl_xor(rowsum[t], 32);
  }
  int8_t* out_tile = lds;  // TM rows x kOutStride bytes (the loop's last barrier freed the LDS)
#pragma unroll
  for (int tn = 0; tn < 4; ++tn) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      // accumulator rows 8g + 4*(lane/32) + 0..3 of this MFMA tile = 4 consecutive features
      const int nl = wn * 128 + tn * 32 + 8 * g + 4 * frag_half;
      const int n = n0 + nl;
      int b4[4], m4[4], s4[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int nn = n + q < a.N ? n + q : a.N - 1;
        b4[q] = a.biasf[nn];
        m4[q] = a.mult[nn];
        s4[q] = a.shift[nn];
      }
#pragma unroll
      for (int tm = 0; tm < 4; ++tm) {
        const int ml = wm * 128 + tm * 32 + frag_row;
        uint32_t packed = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          int v = acc[tn][tm][g * 4 + q] + b4[q];
          if (ROWSUM) v -= a.zws * rowsum[tm];
          const int r = RequantClamp(v, m4[q], s4[q], a.out_zp, a.lo, a.hi);
          packed |= static_cast<uint32_t>(r & 0xff) << (8 * q);
        }
        *reinterpret_cast<uint32_t*>(out_tile + ml * kOutStride + nl) = packed;
      }
    }
  }
  __syncthreads();
  const bool vec_ok = (a.N & 15) == 0;
  for (int c = tid; c < TM * (TN / 16); c += kThreads) {
    const int ml = c / (TN / 16), nc = (c % (TN / 16)) * 16;
    const int m = m0 + ml, n = n0 + nc;
    if (m >= a.M || n >= a.N) continue;
    const v4i v = *reinterpret_cast<const v4i*>(out_tile + ml * kOutStride + nc);
    int8_t* dst = a.y + static_cast<size_t>(m) * a.N + n;
    if (vec_ok) {
      *reinterpret_cast<v4i*>(dst) = v;
    } else {
      const int8_t* src = out_tile + ml * kOutStride + nc;
      for (int q = 0; q < 16 && n + q < a.N; ++q) dst[q] = src[q];
    }
  }
}

int FcMfmaRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const tvx_fc_desc& d = op->fc;
  FcArgs a;
  a.x = static_cast<const int8_t*>(in0);
  a.w = op->packed.as<int8_t>();
  a.y = static_cast<int8_t*>(out);
  a.biasf = op->aux.as<int32_t>();
  a.mult = op->mult.as<int32_t>();
  a.shift = op->shift.as<int32_t>();
  a.M = static_cast<int>(d.m);
  a.N = static_cast<int>(d.n);
  a.K = static_cast<int>(d.k);
  a.zws = op->geo[0];
  a.out_zp = d.out_zp;
  a.lo = op->act_lo;
  a.hi = op->act_hi;
  a.tiles_m = (a.M + TM - 1) / TM;
  a.tiles_n = (a.N + TN - 1) / TN;
  const dim3 grid(a.tiles_m * a.tiles_n), block(kThreads);
  const bool x_u8 = d.in_dtype == TVX_U8, rowsum = a.zws != 0;
  if (x_u8 && rowsum) hipLaunchKernelGGL((FcMfmaKernel<true, true>), grid, block, kLdsBytes, st, a);
  else if (x_u8) hipLaunchKernelGGL((FcMfmaKernel<true, false>), grid, block, kLdsBytes, st, a);
  else if (rowsum) hipLaunchKernelGGL((FcMfmaKernel<false, true>), grid, block, kLdsBytes, st, a);
  else hipLaunchKernelGGL((FcMfmaKernel<false, false>), grid, block, kLdsBytes, st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

}  // namespace

// Claims quantized FullyConnected with constant weights and K a multiple of 16
// (every 16-byte operand chunk is then whole and aligned).
int FcMfmaSetup(tvx_op* op, const tvx_fc_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || (d->k & 15) != 0) return TVX_E_UNSUPPORTED;
  if (static_cast<uint64_t>(d->m) * d->n >= (1ull << 31) || d->k > (1u << 24)) return TVX_E_UNSUPPORTED;
  const size_t wn = static_cast<size_t>(d->n) * d->k;
  const bool w_u8 = d->w_dtype == TVX_U8;
  // int8-domain operands: uint8 tensors are shifted by 128, zero points follow
  const int zxs = d->in_zp - (d->in_dtype == TVX_U8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  std::vector<int8_t> ws(wn);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  for (size_t i = 0; i < wn; ++i) ws[i] = static_cast<int8_t>(w_u8 ? src[i] ^ 0x80 : src[i]);
  std::vector<int32_t> biasf(d->n);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  for (uint32_t n = 0; n < d->n; ++n) {
    int64_t sw = 0;
    const int8_t* row = ws.data() + static_cast<size_t>(n) * d->k;
    for (uint32_t k = 0; k < d->k; ++k) sw += row[k];
    const int64_t v = (b ? b[n] : 0) - static_cast<int64_t>(zxs) * sw +
                      static_cast<int64_t>(d->k) * zxs * zws;
    biasf[n] = static_cast<int32_t>(static_cast<uint32_t>(v));  // int32 accumulators wrap
  }
  int s = op->packed.Upload(ws.data(), wn);
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s != TVX_OK) return s;
  hipError_t e = hipSuccess;
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(&FcMfmaKernel<true, true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&FcMfmaKernel<true, false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&FcMfmaKernel<false, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&FcMfmaKernel<false, false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (e != hipSuccess)
    return SetError(TVX_E_DEVICE, "hipFuncSetAttribute(dynamic LDS %d): %s", kLdsBytes, hipGetErrorString(e));
  op->geo[0] = zws;
  op->run = FcMfmaRun;
  op->kernel_name = "fc_mfma_i8_256x256x128";
  return TVX_OK;
}

}  // namespace tvx
