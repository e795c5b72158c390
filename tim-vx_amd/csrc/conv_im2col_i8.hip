// Quantized Conv2d with a short reduction (C * Kh * Kw <= 64) on the int8 matrix cores: the first
// layers of image networks (3 x 3 x 3 = 27, 1 x 5 x 5 = 25). The implicit-GEMM kernel pads the
// channels of every tap to 16 and would multiply mostly zeros there; here the whole window of an
// output pixel - its (c, ky, kx) bytes, padded to 32 or 64 - is one row of the MFMA A operand.
//
// Workgroup = 256 output pixels of one image x all output channels (<= 128). Each thread
// gathers the window of one pixel with byte loads (16 in flight, no branches: out-of-image taps
// read a safe address and are replaced by the input zero point), keeps the window sum for the
// zero-point expansion
//   sum (x - zx)(w - zw) = sum xs ws - zws * Sx - zxs * Sw + K zxs zws
// and stores the row to LDS. One or two v_mfma_i32_32x32x32_i8 steps per (pixel tile, channel
// tile) follow; the epilogue is the implicit-GEMM kernel's: requantize, pack four pixels per
// dword, stage [oc][pixel] in LDS, copy out as contiguous runs of the WHCN output.
#include <algorithm>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kPixels = 256;  // per workgroup: eight 32-pixel MFMA tiles, two per wavefront

struct ImArgs {
  const uint8_t* x;
  const int8_t* w;       // packed [oct][row_stride] (the LDS image), reduction order (c, ky, kx), zero padded
  uint8_t* y;
  const int32_t* biasf;  // bias + per-channel zero-point terms
  const v4i* rq;         // per channel {mult, shift | t, half, lowmask}
  int C, H, W, OC, OH, OW;
  int sh, sw, pad_t, pad_l;
  int kp;                // reduction length padded to 32 or 64
  int row_stride;        // bytes per LDS row of A and of the weights: kp + 16 (an odd number of 16-byte chunks)
  int oct;               // output channels padded to 32
  int xor_mask;          // 0x80 for uint8 activations, else 0
  int pad_fill;          // input zero point in the int8 domain (one byte)
  int zws, out_zp, lo, hi;
  int out_stride;        // epilogue staging row stride in bytes (odd number of dwords)
  int off_a, off_w, off_sx, off_rq, off_bias;  // LDS carve-up
  // The window, per reduction index: dy | dx << 8 | 1 << 16 (zero past the end) and the input offset
  // c * H * W + dy * W + dx. They travel in the kernel arguments so that the (wavefront-uniform) reads
  // are scalar loads of memory nothing can write; a table in global memory is read per lane, one round
  // trip a tap.
  // In row mode (kernels three or five taps wide, unit dilation along the row) entry r stands for a whole
  // kernel row of a channel: dy | 1 << 16 and c * H * W + dy * W; the taps are one or two dword loads.
  int taps[64];
  int offs[64];
  int rows;              // row mode: C * Kh
  int rows_mask;         // row mode: the window rows in use (bit dy), all of them inside the image for most pixels
  int total_bytes;       // row mode: size of the input tensor (< 2^31)
  int pool;              // 1: a 2 x 2 / stride-2 max pooling rides on the epilogue (the result has OH / 2 x OW / 2 pixels)
};

// KW: 0 = any window, one byte load per tap; 3 / 5 = row mode for kernels three / five taps wide
// (two wavefronts per SIMD at least: within 256 registers the compiler keeps MFMA accumulators in ordinary vector
// registers, where the epilogue reads them, instead of moving every value out of the accumulation registers first)
template <int OT, int RQ, int KW>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2))) ConvIm2colKernel(ImArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = blockIdx.y;
  const int hw = a.OH * a.OW;
  const int p0 = blockIdx.x * kPixels;
  const int valid = min(kPixels, hw - p0);

  int8_t* a_lds = lds + a.off_a;
  int8_t* w_lds = lds + a.off_w;
  int* sx_lds = reinterpret_cast<int*>(lds + a.off_sx);
  v4i* rq_lds = reinterpret_cast<v4i*>(lds + a.off_rq);
  int* bias_lds = reinterpret_cast<int*>(lds + a.off_bias);

  // weights (already laid out as their LDS image) and the epilogue's tables: global -> LDS by DMA,
  // waited for together with the window loads
  {
    typedef const __attribute__((address_space(1))) void* gptr;
    typedef __attribute__((address_space(3))) void* lptr;
    const int chunks = a.oct * a.row_stride >> 4;
    for (int i = wave * 64; i < chunks; i += kThreads)
      if (i + lane < chunks)
        __builtin_amdgcn_global_load_lds((gptr)(a.w + static_cast<size_t>(i + lane) * 16), (lptr)(w_lds + i * 16), 16, 0, 0);
    for (int i = wave * 64; i < a.oct; i += kThreads)
      if (i + lane < a.oct) {
        __builtin_amdgcn_global_load_lds((gptr)(a.rq + i + lane), (lptr)(rq_lds + i), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr)(a.biasf + i + lane), (lptr)(bias_lds + i), 4, 0, 0);
      }
  }

  // ---- the window of this thread's pixel ------------------------------------------------
  int sx = 0;
  {
    const int p = min(p0 + tid, hw - 1);  // threads past the end redo the last pixel; nobody reads their row
    int oh = p / a.OW, ow = p - oh * a.OW;
    if (a.pool) {
      // pixels in pooling order: four consecutive ones are a 2 x 2 window (row-major), windows row-major over
      // the pooled image - the four accumulators a lane holds per quad then are one pooled pixel's candidates
      const int q = p >> 2, e = p & 3, pw = a.OW >> 1;
      const int qh = q / pw, qw = q - qh * pw;
      oh = 2 * qh + (e >> 1);
      ow = 2 * qw + (e & 1);
    }
    const int ih0 = oh * a.sh - a.pad_t, iw0 = ow * a.sw - a.pad_l;
    const uint8_t* img = a.x + static_cast<size_t>(n) * a.C * a.H * a.W;
    const int origin = ih0 * a.W + iw0;  // may be negative; only added to offsets of taps inside the image
    // Which window rows / columns (offsets 0..31 from the window's origin) lie inside the image, as bit
    // masks: a tap's validity is then two shifts and an AND instead of two additions and two compares.
    auto span_mask = [](int first, int extent) {  // bits d with 0 <= first + d < extent, d in 0..31
      const int lo = max(0, -first), hi = min(32, extent - first);
      const int n = hi - lo;
      return n <= 0 ? 0u : ((n >= 32 ? 0xffffffffu : ((1u << n) - 1u)) << lo);
    };
    const uint32_t row_ok = span_mask(ih0, a.H), col_ok = span_mask(iw0, a.W);
    if constexpr (KW == 3 || KW == 5) {
      // Row mode: byte loads cost the L1 a tag lookup for every few lanes, and those lookups bound the
      // gather; the taps of a kernel row are adjacent bytes, so one (unaligned) dword fetches three of
      // them, two dwords five. A dword may begin in front of the tensor (left padding of its first row)
      // or end behind it: it is moved inside and shifted back. A row with no tap inside the image reads
      // the tensor's first dword(s) and is not used.
      constexpr int kMaxRows = 64 / KW;
      constexpr uint32_t kColMask = (1u << KW) - 1u;
      const int img_at = n * (a.C * a.H * a.W) + origin;
      auto place = [&](int r, int which, bool* row_in, int* moved) {  // -> byte index of the row's dword `which` in the tensor
        const int t = a.taps[r];
        *row_in = ((row_ok >> (t & 0xff)) & static_cast<uint32_t>(t >> 16) & 1u) != 0;
        const bool any = *row_in & ((col_ok & kColMask) != 0);
        const int want = (any ? img_at + a.offs[r] : 0) + 4 * which;
        const int at = min(max(want, 0), a.total_bytes - 4);
        *moved = at - want;  // first dword: -3 .. 4; second: -7 .. 0
        return at;
      };
      uint32_t v[kMaxRows], v2[KW == 5 ? kMaxRows : 1];
      int dw[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) dw[i] = 0;
      // Nearly every wavefront holds only pixels whose window rows all lie inside the image and whose dwords all
      // lie inside the tensor (the exceptions: an image's first / last output rows under padding, the tensor's
      // first and last bytes). There a row's dword sits where it is expected, nothing is moved or shifted back,
      // and what is left of the border - the same one or two window columns outside the image in every row of a
      // pixel - is one mask and one XOR pattern per thread: (dword & inside) ^ (re-bias where inside, the input
      // zero point where not).
      const int first_at = img_at + a.offs[0], last_at = img_at + a.offs[a.rows - 1] + (KW == 5 ? 4 : 0);
      const bool plain = (row_ok & static_cast<uint32_t>(a.rows_mask)) == static_cast<uint32_t>(a.rows_mask) &&
                         first_at >= 0 && last_at + 4 <= a.total_bytes;
      if (__builtin_amdgcn_ballot_w64(!plain) == 0) {
#pragma unroll
        for (int r = 0; r < kMaxRows; ++r) {
          v[r] = 0;
          if (KW == 5) v2[r] = 0;
          if (r < a.rows) {  // uniform
            const uint32_t at = static_cast<uint32_t>(img_at + a.offs[r]);
            __builtin_memcpy(&v[r], a.x + at, 4);
            if constexpr (KW == 5) __builtin_memcpy(&v2[r], a.x + at + 4, 4);
          }
        }
        __builtin_amdgcn_sched_barrier(0);  // all loads travel together
        uint32_t keep = 0, flip = 0, keep2 = 0, flip2 = 0;  // per window column: 0xff where inside; re-bias or zero point
#pragma unroll
        for (int e = 0; e < KW; ++e) {
          const bool inside = ((col_ok >> e) & 1u) != 0;
          const uint32_t k8 = inside ? 0xffu : 0u, f8 = static_cast<uint32_t>(inside ? a.xor_mask : a.pad_fill) & 0xffu;
          if (e < 4) keep |= k8 << (8 * e), flip |= f8 << (8 * e);
          else keep2 = k8, flip2 = f8;
        }
#pragma unroll
        for (int r = 0; r < kMaxRows; ++r) {
          if (r < a.rows) {
            const int k = r * KW, i = k >> 2, pos = k & 3;  // (constants once unrolled)
            const uint32_t row = (v[r] & keep) ^ flip;  // KW == 3: the fourth byte is masked away
            dw[i] |= static_cast<int>(row << (8 * pos));
            if (pos + (KW == 3 ? 3 : 4) > 4) dw[i + 1] |= static_cast<int>(row >> (8 * (4 - pos)));
            if constexpr (KW == 5) {
              const int k5 = k + 4;
              dw[k5 >> 2] |= static_cast<int>(((v2[r] & keep2) ^ flip2) << (8 * (k5 & 3)));
            }
          }
        }
      } else {
#pragma unroll
      for (int r = 0; r < kMaxRows; ++r) {
        v[r] = 0;
        if (KW == 5) v2[r] = 0;
        if (r < a.rows) {  // uniform
          bool row_in;
          int moved;
          const int at = place(r, 0, &row_in, &moved);
          __builtin_memcpy(&v[r], a.x + static_cast<uint32_t>(at), 4);
          if constexpr (KW == 5) {
            const int at2 = place(r, 1, &row_in, &moved);
            __builtin_memcpy(&v2[r], a.x + static_cast<uint32_t>(at2), 4);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);  // all loads travel together
#pragma unroll
      for (int r = 0; r < kMaxRows; ++r) {
        if (r < a.rows) {
          bool row_in;
          int moved;
          (void)place(r, 0, &row_in, &moved);
          // (moved by a whole dword - a five-tap row four columns in front of the tensor: every tap is masked)
          const uint32_t got = moved >= 4 ? 0u : (moved >= 0 ? v[r] << (8 * moved) : v[r] >> (-8 * moved));
          uint32_t got2 = 0;  // (fifth tap: the second dword's first byte)
          if constexpr (KW == 5) {
            (void)place(r, 1, &row_in, &moved);
            got2 = moved <= -4 ? 0u : v2[r] >> (-8 * moved);  // (moved by four bytes or more: the tap lies behind the tensor and is masked)
          }
#pragma unroll
          for (int e = 0; e < KW; ++e) {
            const bool inside = row_in & (((col_ok >> e) & 1u) != 0);
            const uint32_t raw = e < 4 ? (got >> (8 * e)) & 0xffu : got2 & 0xffu;
            const int byte = inside ? static_cast<int>(raw ^ static_cast<uint32_t>(a.xor_mask)) : a.pad_fill;
            const int k = r * KW + e;
            dw[k >> 2] |= byte << (8 * (k & 3));
          }
        }
      }
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) sx = __builtin_amdgcn_sdot4(dw[i], 0x01010101, sx, false);
      for (int k0 = 0; k0 < a.kp; k0 += 16) {
        const int i = k0 >> 2;
        const v4i out = i == 0 ? v4i{dw[0], dw[1], dw[2], dw[3]} : (i == 4 ? v4i{dw[4], dw[5], dw[6], dw[7]} : (i == 8 ? v4i{dw[8], dw[9], dw[10], dw[11]} : v4i{dw[12], dw[13], dw[14], dw[15]}));
        *reinterpret_cast<v4i*>(a_lds + tid * a.row_stride + k0) = out;
      }
    } else
    for (int k0 = 0; k0 < a.kp; k0 += 16) {
      int b[16];
      bool inside[16];
      int fill[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int t = a.taps[k0 + j];  // scalar: dy | dx << 8 | real << 16
        const int dy = t & 0xff, dx = (t >> 8) & 0xff;
        const uint32_t real = 0u - static_cast<uint32_t>(t >> 16);  // all ones or zero
        fill[j] = a.pad_fill & static_cast<int>(real);
        // bitwise, not short-circuit: no branch may stand between the loads
        inside[j] = ((row_ok >> dy) & (col_ok >> dx) & real & 1u) != 0;
        b[j] = img[static_cast<uint32_t>(inside[j] ? origin + a.offs[k0 + j] : 0)];  // uniform base + 32-bit lane offset
      }
      __builtin_amdgcn_sched_barrier(0);  // all sixteen loads travel together
      int dw[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int v = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int j = q * 4 + e;
          const int byte = inside[j] ? (b[j] ^ a.xor_mask) : fill[j];  // both below 256
          v |= byte << (8 * e);
        }
        dw[q] = v;
        sx = __builtin_amdgcn_sdot4(v, 0x01010101, sx, false);
      }
      *reinterpret_cast<v4i*>(a_lds + tid * a.row_stride + k0) = v4i{dw[0], dw[1], dw[2], dw[3]};
    }
  }
  sx_lds[tid] = a.zws * sx;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the table DMA has landed
  __syncthreads();

  // ---- MFMA: wave w owns pixel tiles w and w + 4, all channel tiles ---------------------------
  const int frag_row = lane & 31, frag_half = lane >> 5;
  v16i acc[2][OT];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < OT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  for (int ks = 0; ks < a.kp; ks += 32) {
    v4i fa[2], fb[OT];
#pragma unroll
    for (int i = 0; i < 2; ++i)
      fa[i] = *reinterpret_cast<const v4i*>(a_lds + ((wave + 4 * i) * 32 + frag_row) * a.row_stride + ks + frag_half * 16);
#pragma unroll
    for (int j = 0; j < OT; ++j)
      fb[j] = *reinterpret_cast<const v4i*>(w_lds + (j * 32 + frag_row) * a.row_stride + ks + frag_half * 16);
#pragma unroll
    for (int j = 0; j < OT; ++j)
#pragma unroll
      for (int i = 0; i < 2; ++i) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
  }
  __syncthreads();  // everyone is done with the A rows and the weights: the staging tile takes their place

  // ---- epilogue ---------------------------------------------------------------------------
  int8_t* out_tile = lds + a.off_a;  // [oct][out_stride]
  const int lo = a.lo, hi = a.hi;
#pragma unroll
  for (int j = 0; j < OT; ++j) {
    const int ocl = j * 32 + frag_row;
    const v4i q = rq_lds[ocl];
    const int bias = bias_lds[ocl];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int pt = wave + 4 * i;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int pl = pt * 32 + 8 * g + 4 * frag_half;
        const v4i s4 = *reinterpret_cast<const v4i*>(sx_lds + pl);
        if (a.pool) {
          // requantization is monotone: the window's largest accumulator gives its largest code
          const int m = max(max(acc[i][j][g * 4] - s4[0], acc[i][j][g * 4 + 1] - s4[1]),
                            max(acc[i][j][g * 4 + 2] - s4[2], acc[i][j][g * 4 + 3] - s4[3]));
          out_tile[ocl * a.out_stride + (pl >> 2)] = static_cast<int8_t>(Requant8<RQ>(m + bias, q, a.out_zp, lo, hi));
          continue;
        }
        int r4[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) r4[e] = acc[i][j][g * 4 + e] + (bias - s4[e]);
        *reinterpret_cast<uint32_t*>(out_tile + ocl * a.out_stride + pl) = RequantPack4<RQ>(r4, q, a.out_zp, lo, hi);
      }
    }
  }
  __syncthreads();
  // what leaves: the tile's pixels, or its pooled pixels (a quarter as many)
  const int hw_y = a.pool ? hw >> 2 : hw, valid_y = a.pool ? valid >> 2 : valid;
  uint8_t* ybase = a.y + static_cast<size_t>(n) * a.OC * hw_y + (a.pool ? p0 >> 2 : p0);
  if ((hw_y & 3) == 0) {
    const int per_row = valid_y >> 2;  // the tile's first pixel and the plane are multiples of 4: whole dwords
    for (int o = wave; o < a.OC; o += 4)
      for (int dwi = lane; dwi < per_row; dwi += 64)
        *reinterpret_cast<uint32_t*>(ybase + static_cast<size_t>(o) * hw_y + dwi * 4) =
            *reinterpret_cast<const uint32_t*>(out_tile + o * a.out_stride + dwi * 4);
  } else {
    for (int o = wave; o < a.OC; o += 4)
      for (int pi = lane; pi < valid_y; pi += 64)
        ybase[static_cast<size_t>(o) * hw_y + pi] = static_cast<uint8_t>(out_tile[o * a.out_stride + pi]);
  }
}

struct Plan {
  ImArgs a;
  int lds_bytes;
  int ot, rq, row_mode;
  dim3 grid;
};

template <int OT, int KW>
void LaunchRq(const Plan* plan, const ImArgs& a, hipStream_t st) {
  const dim3 block(kThreads);
  if (plan->rq == kRqFastNoTie)
    hipLaunchKernelGGL((ConvIm2colKernel<OT, kRqFastNoTie, KW>), plan->grid, block, plan->lds_bytes, st, a);
  else if (plan->rq == kRqFast)
    hipLaunchKernelGGL((ConvIm2colKernel<OT, kRqFast, KW>), plan->grid, block, plan->lds_bytes, st, a);
  else
    hipLaunchKernelGGL((ConvIm2colKernel<OT, kRqGeneric, KW>), plan->grid, block, plan->lds_bytes, st, a);
}

template <int KW>
void LaunchOt(const Plan* plan, const ImArgs& a, hipStream_t st) {
  if (plan->ot == 1) LaunchRq<1, KW>(plan, a, st);
  else if (plan->ot == 2) LaunchRq<2, KW>(plan, a, st);
  else LaunchRq<4, KW>(plan, a, st);
}

int ConvIm2colRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  ImArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if (plan->row_mode == 5) LaunchOt<5>(plan, a, st);
  else if (plan->row_mode) LaunchOt<3>(plan, a, st);
  else LaunchOt<0>(plan, a, st);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

int RoundUp(int v, int m) { return (v + m - 1) / m * m; }

}  // namespace

// Claims dense quantized convolutions with constant weights whose whole window is at most 64
// bytes and whose channel count the implicit-GEMM kernel would have to pad (C % 16 != 0).
int ConvIm2colSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || d->multiplier != 0 || d->groups > 1) return TVX_E_UNSUPPORTED;
  const int taps = static_cast<int>(d->k_w * d->k_h);
  const uint64_t k_real = static_cast<uint64_t>(d->in_c) * taps;
  if (k_real > 64 || d->in_c % 16 == 0 || d->out_c > 128) return TVX_E_UNSUPPORTED;
  if (static_cast<uint64_t>(d->in_c) * d->in_h * d->in_w >= (1ull << 31) || d->batch > 65535) return TVX_E_UNSUPPORTED;
  ImArgs a{};
  a.C = d->in_c; a.H = d->in_h; a.W = d->in_w; a.OC = d->out_c; a.OH = d->out_h; a.OW = d->out_w;
  a.sh = d->stride_h; a.sw = d->stride_w; a.pad_t = d->pad_top; a.pad_l = d->pad_left;
  const int K = static_cast<int>(k_real);
  a.kp = K <= 32 ? 32 : 64;
  a.row_stride = a.kp + 16;
  const int ot = d->out_c <= 32 ? 1 : (d->out_c <= 64 ? 2 : 4);
  a.oct = 32 * ot;
  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127) return TVX_E_UNSUPPORTED;  // zero point outside the tensor's range
  a.xor_mask = x_u8 ? 0x80 : 0;
  a.pad_fill = zxs & 0xff;
  a.zws = zws;
  a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  a.pool = op->fused_pool;  // (the caller has checked the pooling: 2 x 2, stride 2, even output extents)
  a.out_stride = ((kPixels / 4) | 1) * 4;
  // LDS: window sums and tables first; A rows + weights behind them are reused as the staging tile
  a.off_sx = 0;
  a.off_rq = kPixels * 4;
  a.off_bias = a.off_rq + a.oct * 16;
  a.off_a = a.off_bias + a.oct * 4;
  a.off_w = a.off_a + kPixels * a.row_stride;
  const int lds_bytes = a.off_a + std::max(kPixels * a.row_stride + a.oct * a.row_stride, a.oct * a.out_stride);

  // ---- pack weights [oc][(c, ky, kx)] int8 with zero padding, fold constants ---------------
  std::vector<int8_t> packed(static_cast<size_t>(a.oct) * a.row_stride, 0);
  std::vector<int32_t> biasf(a.oct, 0);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  for (int oc = 0; oc < a.OC; ++oc) {
    int64_t sw = 0;
    for (int k = 0; k < K; ++k) {  // the weight tensor's own order: [oc][c][ky][kx]
      const uint8_t raw = src[static_cast<size_t>(oc) * K + k];
      const int8_t v = static_cast<int8_t>(w_u8 ? raw ^ 0x80 : raw);
      packed[static_cast<size_t>(oc) * a.row_stride + k] = v;
      sw += v;
    }
    const int64_t v = (b ? b[oc] : 0) - static_cast<int64_t>(zxs) * sw + static_cast<int64_t>(K) * zxs * zws;
    biasf[oc] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  std::vector<int32_t> rqt;
  const int rq = BuildRequantRecords(op->h_mult, op->h_shift, a.OC, a.oct, d->out_zp, &rqt,
                                     AccumulatorBound(static_cast<uint64_t>(K), bias_host, a.OC));
  if ((d->k_h - 1) * d->dilation_h > 31 || (d->k_w - 1) * d->dilation_w > 31) return TVX_E_UNSUPPORTED;  // window offsets index 32-bit masks
  const uint64_t total_bytes = static_cast<uint64_t>(d->batch) * d->in_c * d->in_h * d->in_w;
  bool row_mode = (d->k_w == 3 || d->k_w == 5) && d->dilation_w == 1 && total_bytes >= 4 && total_bytes < (1ull << 31);
  if (const char* f = getenv("TVX_IM2COL_ROWS")) row_mode = row_mode && atoi(f) != 0;  // tuning aid
  if (row_mode) {
    a.rows = static_cast<int>(d->in_c * d->k_h);
    a.total_bytes = static_cast<int>(total_bytes);
    for (int r = 0; r < a.rows; ++r) {
      const int c = r / static_cast<int>(d->k_h);
      const int dy = (r % static_cast<int>(d->k_h)) * static_cast<int>(d->dilation_h);
      a.taps[r] = dy | 1 << 16;
      a.offs[r] = c * a.H * a.W + dy * a.W;
      a.rows_mask |= 1 << dy;
    }
  } else {
    for (int k = 0; k < K; ++k) {
      const int c = k / taps, t = k % taps;
      const int dy = (t / static_cast<int>(d->k_w)) * static_cast<int>(d->dilation_h);
      const int dx = (t % static_cast<int>(d->k_w)) * static_cast<int>(d->dilation_w);
      a.taps[k] = dy | dx << 8 | 1 << 16;
      a.offs[k] = c * a.H * a.W + dy * a.W + dx;
    }
  }
  int s = op->packed.Upload(packed.data(), packed.size());
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s != TVX_OK) return s;
  a.w = op->packed.as<int8_t>();
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<v4i>();

  Plan plan;
  plan.a = a;
  plan.lds_bytes = lds_bytes;
  plan.ot = ot;
  plan.rq = rq;
  plan.row_mode = row_mode ? static_cast<int>(d->k_w) : 0;  // 0, or the taps of a kernel row (3 / 5)
  const int hw = a.OH * a.OW;
  plan.grid = dim3(static_cast<unsigned>((hw + kPixels - 1) / kPixels), static_cast<unsigned>(d->batch));
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = ConvIm2colRun;
  op->kernel_name = op->fused_pool ? "conv2d_im2col_maxpool_i8" : "conv2d_im2col_i8";
  return TVX_OK;
}

}  // namespace tvx
