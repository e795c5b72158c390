// Dense quantized Conv2d as an implicit GEMM on the int8 matrix cores.
//
// GEMM view: rows = output pixels of one image, columns = output channels,
// reduction = (ky, kx, c) with the channel fastest. Activations arrive WHCN
// (W fastest, channel planes H*W apart) but v_mfma_i32_32x32x32_i8 wants 16
// consecutive reduction bytes per lane, so the workgroup first builds a
// channel-innermost halo tile of its input window in LDS (4 x 4 byte
// transposes in registers on the way in, all global loads of a thread in
// flight at once). Out-of-image positions of the tile hold the input zero
// point, so every window sums over all taps and the zero-point expansion
//   sum (x - zx)(w - zw) = sum xs ws - zws * Sx - zxs * Sw + K zxs zws
// needs one per-pixel sum Sx (taken with v_dot4 from the fragments already in
// registers) and per-channel constants folded into the bias at creation.
// The MFMA A operand of tap (ky, kx) is read straight out of the halo tile -
// no im2col copy exists anywhere. The packed weights of the channel block are
// DMA-ed global -> LDS (no registers) while the halo tile is being built and
// stay there for the whole tile.
//
// Epilogue: requantize with 32-bit arithmetic where the shifts allow it, pack
// four pixels per dword, stage [oc][pixel] in LDS, copy out as contiguous
// runs of the WHCN output.
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kMaxPtw = 2;     // 32-pixel MFMA tiles per wavefront (tile <= 256 pixels)

struct ConvArgs {
  const uint8_t* x;
  const int8_t* w;       // packed [oc_alloc][kstride]
  uint8_t* y;
  const int32_t* biasf;  // bias + per-channel zero-point terms
  const v4i* rq;         // per channel {mult, shift | t, half, lowmask}
  const int2* tapt;      // per (k-step, fragment half): {halo byte offset of the chunk, dot4 multiplier}
  int C, H, W, OC, OH, OW;
  int kh, kw, sh, sw, dh, dw, pad_t, pad_l;
  int cp, cpc;           // channels of one reduction group padded to 16, and 16-byte chunks per pixel
  int groups;            // reduction groups: the input channels are walked cp at a time
  int w_group_stride;    // bytes between the packed weights of consecutive groups
  int ksteps, kstride;
  int P, PT, tiles_per_image, oct;
  int iht, iwt;          // halo tile extent
  int pix_stride;        // bytes per halo pixel: cp, plus 16 when cp/16 is even (bank spread)
  int xor_mask;          // 0x80808080 for uint8 activations, else 0
  int pad_fill;          // input zero point (int8 domain) in all four bytes
  int zws, out_zp, lo, hi;
  int out_stride;        // epilogue staging row stride in bytes (odd number of dwords)
  int w_chunks;          // 16-byte chunks of one channel block's weights
  int w4_blocks;         // ceil(W / 64): blocks of 16 four-column patches per channel row
  int off_w, off_halo, off_sx, off_tap, off_rq, off_bias;  // LDS carve-up
  // persistent variant only
  int total_tiles;       // batch * tiles_per_image
  int halo_bytes;        // one of the two halo buffers
  int off_halo1;         // the second halo buffer (persistent variant: the staging tile lies between the two)
  uint32_t magic_ow;     // persistent variant: ceil(2^32 / OW), exact for every pixel index of an image (the host checks)
  uint32_t magic_tpi;    // ... ceil(2^32 / tiles_per_image), exact for every tile index (0: one tile per image)
  int rows;              // ... output rows of a tile
  uint32_t blk_col, blk_chan;  // ... per wavefront w (byte w): w % w4_blocks and w / w4_blocks
  int off_out;           // epilogue staging tile
  int pool;              // one-tile-per-workgroup kernel: a 2 x 2 / stride-2 max pooling rides on the epilogue
  int tap_off[40];       // halo byte offset of k-step ks (both fragment halves lie in one tap: + 16 * half)
};

__device__ __forceinline__ int FastDiv(int u, uint32_t magic) {
  return magic ? static_cast<int>(__umulhi(static_cast<uint32_t>(u), magic)) : u;
}

__device__ __forceinline__ int HaloOffset(const ConvArgs& a, int hp, int c) {
  return hp * a.pix_stride + c;
}

__device__ __forceinline__ int ChannelFill(const ConvArgs& a, int c, int c_real) {
  // zero-point bytes for real channels, zero for the padding up to 16
  const int n = c_real - c;  // real channels left in this group of four
  if (n >= 4) return a.pad_fill;
  if (n <= 0) return 0;
  return a.pad_fill & ((1 << (8 * n)) - 1);
}

template <int OT, int RQ>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(OT == 1 ? 4 : 2, OT == 1 ? 4 : 2))) ConvIgemmKernel(ConvArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // Workgroups go to the eight XCDs round-robin in launch order and each XCD has its own L2:
  // renumber them so that an XCD gets a contiguous run of tiles. Neighbouring tiles of an image,
  // whose halo rows overlap, then meet in one L2 instead of fetching the rows from HBM twice.
  int bx = blockIdx.x;
  if (gridDim.y == 1) {
    const int per = gridDim.x >> 3, rem = gridDim.x & 7, xcd = bx & 7;
    bx = xcd * per + min(xcd, rem) + (bx >> 3);
  }
  const int tile = bx % a.tiles_per_image;
  const int n = bx / a.tiles_per_image;
  const int oc0 = blockIdx.y * a.oct;
  const int hw = a.OH * a.OW;
  const int p0 = tile * a.P;
  const int p_end = min(p0 + a.P, hw);
  // With pooling the pixels run in pooling order: four consecutive ones are a 2 x 2 window (row-major), windows
  // row-major over the pooled image - the four accumulators a lane holds per quad are one pooled pixel's candidates.
  const int pool_w = a.OW >> 1;
  const int r0 = a.pool ? 2 * ((p0 >> 2) / pool_w) : p0 / a.OW;
  const int r1 = a.pool ? 2 * (((p_end - 1) >> 2) / pool_w) + 1 : (p_end - 1) / a.OW;
  const int ih0 = r0 * a.sh - a.pad_t;
  const int rows_needed = (r1 - r0) * a.sh + (a.kh - 1) * a.dh + 1;

  int8_t* w_lds = lds + a.off_w;
  int8_t* halo = lds + a.off_halo;
  int* sx_lds = reinterpret_cast<int*>(lds + a.off_sx);

  // The reduction order as a table (built once per operator: no index math in the main loop)
  // and the epilogue's per-channel tables go global -> LDS by DMA here, ahead of the input
  // loads, and are waited for together with the weights: no memory round trip of their own
  // stands in front of the halo loads or at the head of the epilogue, and no register is held.
  int2* tap_lds = reinterpret_cast<int2*>(lds + a.off_tap);
  v4i* rq_lds = reinterpret_cast<v4i*>(lds + a.off_rq);
  int* bias_lds = reinterpret_cast<int*>(lds + a.off_bias);
  {
    typedef const __attribute__((address_space(1))) void* gptr;
    typedef __attribute__((address_space(3))) void* lptr;
    const int tap_dwords = (a.ksteps * 2 + 2) * 2;
    const int* tap_src = reinterpret_cast<const int*>(a.tapt);
    for (int i = wave * 64; i < tap_dwords; i += kThreads)
      if (i + lane < tap_dwords)
        __builtin_amdgcn_global_load_lds((gptr)(tap_src + i + lane), (lptr)(reinterpret_cast<int*>(tap_lds) + i), 4, 0, 0);
    for (int i = wave * 64; i < a.oct; i += kThreads)  // tables cover the padded channel count
      if (i + lane < a.oct) {
        __builtin_amdgcn_global_load_lds((gptr)(a.rq + oc0 + i + lane), (lptr)(rq_lds + i), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr)(a.biasf + oc0 + i + lane), (lptr)(bias_lds + i), 4, 0, 0);
      }
  }
  // ---- main loop ---------------------------------------------------------------
  const int frag_row = lane & 31, frag_half = lane >> 5;
  int a_base[kMaxPtw];  // byte offset of each pixel's window origin in the halo tile (+ this lane's half)
  int n_ptw = 0;
#pragma unroll
  for (int i = 0; i < kMaxPtw; ++i) {
    const int pt = wave + 4 * i;
    a_base[i] = 0;
    if (pt < a.PT) {
      n_ptw = i + 1;
      int p = p0 + pt * 32 + frag_row;
      p = min(p, hw - 1);
      int oh = p / a.OW, ow = p - oh * a.OW;
      if (a.pool) {
        const int q = p >> 2, e = p & 3;
        const int qh = q / pool_w, qw = q - qh * pool_w;
        oh = 2 * qh + (e >> 1);
        ow = 2 * qw + (e & 1);
      }
      a_base[i] = ((oh - r0) * a.sh * a.iwt + ow * a.sw) * a.pix_stride;
    }
  }
  // accumulators start at zero; the folded bias is added in the epilogue
  v16i acc[kMaxPtw][OT];
#pragma unroll
  for (int j = 0; j < OT; ++j)
#pragma unroll
    for (int i = 0; i < kMaxPtw; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
  int sx[kMaxPtw] = {0, 0};

  // ---- reduction groups: (weights, halo tile) of cp input channels at a time ------------
  for (int g = 0; g < a.groups; ++g) {
    const int c_base = g * a.cp;
    const int c_real = min(a.C - c_base, a.cp);
    if (g > 0) __syncthreads();  // everyone is done with the previous group's tiles
    // ---- weights of this channel block: global -> LDS DMA, 1 KiB per wave instruction
    {
      const int8_t* src = a.w + static_cast<size_t>(g) * a.w_group_stride + static_cast<size_t>(oc0) * a.kstride;
      for (int i = wave * 64; i < a.w_chunks; i += kThreads) {
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(src + static_cast<size_t>(i + lane) * 16),
            (__attribute__((address_space(3))) void*)(w_lds + i * 16), 16, 0, 0);
      }
    }
    // ---- halo tile -------------------------------------------------------------
    const size_t plane = static_cast<size_t>(a.H) * a.W;
    const uint8_t* xin = a.x + static_cast<size_t>(n) * a.C * plane;
    const int c4n = a.cp / 4;
    // 256 zero bytes: the slack behind the last group's packed weights
    const uint8_t* zero_word =
        reinterpret_cast<const uint8_t*>(a.w) + static_cast<size_t>(a.groups) * a.w_group_stride - 256;
    if ((a.W & 3) == 0) {
      // A thread owns one (4 input columns, 4 channels) patch and walks the halo
      // rows with it, a batch of rows of loads in flight; lanes run over channel
      // groups first so that a wavefront's LDS stores spread over the banks.
      const int w4n = a.W / 4;
      const int patches = a.w4_blocks * ((c4n + 3) / 4) * 64;
      const uint32_t plane32 = static_cast<uint32_t>(plane);
      const int row_bytes = a.iwt * a.pix_stride;
      // Fewer patches than threads (small planes with few channels): the threads of a patch split its halo rows,
      // so that the rows of a tile are one batch of loads - one memory round trip - instead of several.
      const int row_groups = patches <= kThreads / 2 ? kThreads / patches : 1;  // (patches: 64 or 128 then)
      const int rows_per_group = (rows_needed + row_groups - 1) / row_groups;
      const int my_group = row_groups > 1 ? tid / patches : 0;
      const int hr_begin = my_group * rows_per_group, hr_end = min(rows_needed, hr_begin + rows_per_group);
      for (int pi = row_groups > 1 ? tid - my_group * patches : tid; pi < patches; pi += kThreads) {
        // patch index -> (column group, channel group): 16 consecutive lanes read 64
        // contiguous bytes of one channel row, the next 16 lanes the next channel group
        const int blk = pi >> 6, in_blk = pi & 63;
        int w4 = (blk % a.w4_blocks) * 16 + (in_blk & 15);
        int c4 = (blk / a.w4_blocks) * 4 + (in_blk >> 4);
        if (w4 >= w4n || c4 >= c4n) continue;
        const int c = c4 * 4;
        const int hc = a.pad_l + w4 * 4;
        // byte offsets of the patch's four channel rows inside this image (< 2^31)
        // Where each of the patch's four channel rows starts. A channel beyond the real ones
        // reads a zero word behind the packed weights instead: the loaded value is then used
        // as it is, with no select that the compiler could turn into a branch around the load.
        const uint8_t* src_row[4];
        uint32_t row_mul[4];
        int fill[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bool real = c + j < c_real;
          src_row[j] = real ? xin + (static_cast<size_t>(c_base + c + j) * plane32 + static_cast<uint32_t>(w4 * 4))
                            : zero_word;
          row_mul[j] = real ? 1u : 0u;
          fill[j] = real ? a.pad_fill : 0;
        }
        const int xm = a.xor_mask;
        int xmask[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) xmask[j] = c + j < c_real ? xm : 0;
        const int dst0 = __mul24(hc, a.pix_stride) + c;
        // columns of this patch that exist in the halo tile (stride > 1 may cut the right edge)
        const int ncols = min(4, a.iwt - hc);
        // A batch of NB halo rows: all loads first, then masks, transposes and stores. The batch
        // size follows the rows that are left (4, 6 or 8) so that few loads go to rows nobody needs.
        auto batch = [&](auto nb_tag, int hr0) {
          constexpr int NB = decltype(nb_tag)::value;
          int d[NB][4];
          // Out-of-image rows load row 0 (in bounds) and are replaced by the zero point; the
          // replacement is a mask operation, not a select: a select on the wavefront-uniform
          // `inside` would be turned into a branch around the load, and loads under branches
          // are waited for one by one instead of travelling together. All loads of the batch are
          // issued before any of them is used (the scheduling fence keeps the compiler from
          // pulling uses, and with them waits, in between the loads).
#pragma unroll
          for (int b = 0; b < NB; ++b) {
            const int ih = ih0 + hr0 + b;
            const bool inside = hr0 + b < hr_end && ih >= 0 && ih < a.H;
            const uint32_t row_off = __umul24(static_cast<uint32_t>(inside ? ih : 0), static_cast<uint32_t>(a.W));
#pragma unroll
            for (int j = 0; j < 4; ++j) d[b][j] = *reinterpret_cast<const int*>(src_row[j] + row_off * row_mul[j]);
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int b = 0; b < NB; ++b) {
            const int ih = ih0 + hr0 + b;
            const bool inside = hr0 + b < hr_end && ih >= 0 && ih < a.H;
            const int keep = inside ? -1 : 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) d[b][j] = ((d[b][j] ^ xmask[j]) & keep) | (fill[j] & ~keep);
          }
#pragma unroll
          for (int b = 0; b < NB; ++b) {
            if (hr0 + b >= hr_end) continue;
            // 4 x 4 byte transpose: d[j] = 4 pixels of channel c+j  ->  px[i] = 4 channels of pixel i
            const int lo01 = __builtin_amdgcn_perm(d[b][1], d[b][0], 0x05010400);
            const int hi01 = __builtin_amdgcn_perm(d[b][1], d[b][0], 0x07030602);
            const int lo23 = __builtin_amdgcn_perm(d[b][3], d[b][2], 0x05010400);
            const int hi23 = __builtin_amdgcn_perm(d[b][3], d[b][2], 0x07030602);
            int px[4];
            px[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100);
            px[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302);
            px[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100);
            px[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302);
            int8_t* dst = halo + dst0 + __mul24(hr0 + b, row_bytes);
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (i < ncols) *reinterpret_cast<int*>(dst + __mul24(i, a.pix_stride)) = px[i];
          }
        };
        for (int hr0 = hr_begin; hr0 < hr_end;) {
          const int left = hr_end - hr0;
          if (left > 6) {
            batch(std::integral_constant<int, 8>{}, hr0);
            hr0 += 8;
          } else if (left > 4) {
            batch(std::integral_constant<int, 6>{}, hr0);
            hr0 += 6;
          } else {
            batch(std::integral_constant<int, 4>{}, hr0);
            hr0 += 4;
          }
        }
      }
    } else {
      // general width: one (halo row, column, 4 channels) dword at a time
      const int units = rows_needed * a.W * c4n;
      for (int u = tid; u < units; u += kThreads) {
        const int c4 = u % c4n;
        const int iw = (u / c4n) % a.W;
        const int hr = u / (c4n * a.W);
        if (a.pad_l + iw >= a.iwt) continue;
        const int ih = ih0 + hr;
        const int c = c4 * 4;
        int v = ChannelFill(a, c, c_real);
        if (ih >= 0 && ih < a.H) {
          v = 0;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            if (c + j >= c_real) continue;
            const int b = xin[(c_base + c + j) * plane + static_cast<size_t>(ih) * a.W + iw] ^ (a.xor_mask & 0xff);
            v |= b << (8 * j);
          }
        }
        *reinterpret_cast<int*>(halo + HaloOffset(a, hr * a.iwt + a.pad_l + iw, c)) = v;
      }
    }
    // left / right padding columns: one 16-channel chunk of a (halo row, pad column) per step of a thread
    {
      const int right0 = a.pad_l + a.W;
      const int pad_cols = a.pad_l + max(a.iwt - right0, 0);
      const int units = rows_needed * pad_cols * a.cpc;
      for (int u = tid; u < units; u += kThreads) {
        const int cell = u / a.cpc, c = (u - cell * a.cpc) * 16;
        const int hr = cell / pad_cols, pc = cell - hr * pad_cols;
        const int hc = pc < a.pad_l ? pc : right0 + (pc - a.pad_l);
        *reinterpret_cast<v4i*>(halo + (hr * a.iwt + hc) * a.pix_stride + c) =
            v4i{ChannelFill(a, c, c_real), ChannelFill(a, c + 4, c_real), ChannelFill(a, c + 8, c_real),
                ChannelFill(a, c + 12, c_real)};
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the weight DMA has landed
    __syncthreads();

    // Every wavefront runs the same instruction stream: a wavefront whose second
    // pixel tile lies beyond the workgroup's tile computes it anyway (on pixel 0)
    // and drops the result. A k-step's chunk position comes from the tap table; the
    // padding chunk of an odd chunk count meets zero weights and carries a zero dot4
    // multiplier, which keeps it out of the pixel sum.
    {
      const int8_t* w_row = w_lds + frag_row * a.kstride + frag_half * 16;
      const int2* my_tap = tap_lds + frag_half;

      // NP: pixel tiles per wavefront - two, or one where the workgroup's tile has at most four (small planes: the
      // second tile would multiply padding)
      auto kloop = [&](auto np_tag) {
        constexpr int NP = decltype(np_tag)::value;
        auto load_ab = [&](v4i* fa, v4i* fb, int ks, int2 t) {
#pragma unroll
          for (int i = 0; i < NP; ++i)
            fa[i] = *reinterpret_cast<const v4i*>(halo + a_base[i] + t.x);
          // one k-step past the end reads bytes that exist in LDS and are never used
#pragma unroll
          for (int j = 0; j < OT; ++j)
            fb[j] = *reinterpret_cast<const v4i*>(w_row + j * 32 * a.kstride + ks * 32);
        };
        auto step = [&](const v4i* fa, const v4i* fb, int ones) {
#pragma unroll
          for (int i = 0; i < NP; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) sx[i] = __builtin_amdgcn_sdot4(fa[i][q], ones, sx[i], false);
#pragma unroll
          for (int j = 0; j < OT; ++j)
#pragma unroll
            for (int i = 0; i < NP; ++i)
              acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        };

        v4i fa0[NP], fb0[OT], fa1[NP], fb1[OT];
        int2 t0 = my_tap[0], t1 = my_tap[2];  // the table has one spare k-step at its end
        load_ab(fa0, fb0, 0, t0);
        int ks = 0;
        for (; ks + 1 < a.ksteps; ks += 2) {
          const int2 t2 = my_tap[(ks + 2) * 2];
          load_ab(fa1, fb1, ks + 1, t1);
          step(fa0, fb0, t0.y);
          const int2 t3 = my_tap[(ks + 3) * 2];
          load_ab(fa0, fb0, ks + 2, t2);
          step(fa1, fb1, t1.y);
          t0 = t2;
          t1 = t3;
        }
        if (ks < a.ksteps) step(fa0, fb0, t0.y);
      };
      if (a.PT <= 4) kloop(std::integral_constant<int, 1>{});
      else kloop(std::integral_constant<int, 2>{});
    }

  }

  // ---- epilogue ----------------------------------------------------------------
#pragma unroll
  for (int i = 0; i < kMaxPtw; ++i) {
    sx[i] += __shfl_xor(sx[i], 32);
    if (i < n_ptw && frag_half == 0) sx_lds[(wave + 4 * i) * 32 + frag_row] = a.zws * sx[i];
  }
  __syncthreads();  // everyone is done reading weights and halo; sx_lds is visible
  int8_t* out_tile = lds + a.off_w;  // [oct][out_stride], aliases weights + halo
  const int lo = a.lo, hi = a.hi;
#pragma unroll
  for (int j = 0; j < OT; ++j) {
    const int ocl = j * 32 + frag_row;
    const v4i q = rq_lds[ocl];
    const int bias = bias_lds[ocl];
#pragma unroll
    for (int i = 0; i < kMaxPtw; ++i) {
      if (i >= n_ptw) continue;
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
  const int valid = a.pool ? (p_end - p0) >> 2 : p_end - p0;
  const int hw_y = a.pool ? hw >> 2 : hw;
  const int oc_n = min(a.oct, a.OC - oc0);
  uint8_t* ybase = a.y + (static_cast<size_t>(n) * a.OC + oc0) * hw_y + (a.pool ? p0 >> 2 : p0);
  if ((hw_y & 3) == 0 && (valid & 3) == 0) {
    const int per_row = valid >> 2;  // the tile's first pixel and the plane are multiples of 4: whole dwords
    for (int o = wave; o < oc_n; o += 4)
      for (int dwi = lane; dwi < per_row; dwi += 64)
        *reinterpret_cast<uint32_t*>(ybase + static_cast<size_t>(o) * hw_y + dwi * 4) =
            *reinterpret_cast<const uint32_t*>(out_tile + o * a.out_stride + dwi * 4);
  } else {
    for (int o = wave; o < oc_n; o += 4)
      for (int pi = lane; pi < valid; pi += 64)
        ybase[static_cast<size_t>(o) * hw_y + pi] = static_cast<uint8_t>(out_tile[o * a.out_stride + pi]);
  }
}

// ---- persistent variant ----------------------------------------------------------------
// The same implicit GEMM for layers whose whole weight block fits the register file: every
// wavefront keeps all KSTEPS x OT weight fragments of the operator in VGPRs for its whole life
// (they reach the CU once per workgroup, by DMA into LDS, and are read into registers from
// there; afterwards no weight travels through LDS and one 1 KiB activation fragment read feeds
// OT MFMAs), and a workgroup walks many pixel tiles. While a tile is being multiplied the next
// tile's input rows are pulled into L2 by loads whose results nobody reads; behind the tile's
// epilogue they are loaded for real (the accumulators' registers are free then), transposed and
// stored into the second halo buffer. Two such workgroups share a CU and drift out of phase, so
// that one's requantization and stores run under the other's MFMA loop. Needs W % 4 == 0, all
// input channels in one reduction group with an even number of 16-byte chunks, at most six halo
// rows per tile and one (4 columns x 4 channels) patch per thread.
constexpr int kPersistRows = 6;  // most halo rows of a tile

// Behind a tile's epilogue its successor's halo rows go through registers in PHASES batches of NBP rows.
template <int KSTEPS, int OT, int RQ, bool ZP, int NBP, int PHASES>
__global__ void __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2)))
ConvPersistKernel(ConvArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int hw = a.OH * a.OW;

  // ---- this workgroup's tiles: an XCD gets a contiguous run of tiles (neighbouring tiles of an
  // image share halo rows and meet in that XCD's L2); inside the run the XCD's workgroups
  // interleave, so that at any time they work on neighbours.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const int t_first = static_cast<int>(static_cast<long long>(a.total_tiles) * xcd / 8);
  const int t_end = static_cast<int>(static_cast<long long>(a.total_tiles) * (xcd + 1) / 8);
  int t = t_first + slot;
  if (t >= t_end) return;

  int8_t* out_tile = lds + a.off_out;
  int* sx_lds = reinterpret_cast<int*>(lds + a.off_sx) + wave * 32;  // wavefront-private
  v4i* rq_lds = reinterpret_cast<v4i*>(lds + a.off_rq);
  int* bias_lds = reinterpret_cast<int*>(lds + a.off_bias);

  // ---- this thread's patch of the halo tile: 4 input columns x 4 channels, every halo row ------
  const size_t plane = static_cast<size_t>(a.H) * a.W;
  const uint32_t plane32 = static_cast<uint32_t>(plane);
  const int w4n = a.W / 4, c4n = a.cp / 4;
  const int row_bytes = a.iwt * a.pix_stride;
  const int blk = tid >> 6, in_blk = tid & 63;
  const int w4 = static_cast<int>((a.blk_col >> (8 * blk)) & 0xff) * 16 + (in_blk & 15);
  const int c4 = static_cast<int>((a.blk_chan >> (8 * blk)) & 0xff) * 4 + (in_blk >> 4);
  const bool has_patch = w4 < w4n && c4 < c4n;
  const int pc = c4 * 4;
  const int hc = a.pad_l + w4 * 4;
  const int dst0 = __mul24(hc, a.pix_stride) + pc;
  const int ncols = min(4, a.iwt - hc);
  uint32_t ch_off[4];  // byte offset of the patch's four channel rows inside an image
#pragma unroll
  for (int j = 0; j < 4; ++j) ch_off[j] = has_patch ? static_cast<uint32_t>(pc + j) * plane32 + static_cast<uint32_t>(w4 * 4) : 0u;
  const int xm = a.xor_mask;

  auto tile_geometry = [&](int tile_index, int* n, int* p0, int* p_end, int* r0, int* ih0, int* rows_needed) {
    const int img = a.magic_tpi ? static_cast<int>(__umulhi(static_cast<uint32_t>(tile_index), a.magic_tpi)) : tile_index;
    const int tl = tile_index - img * a.tiles_per_image;
    *n = img;
    *p0 = tl * a.P;
    *p_end = min(*p0 + a.P, hw);
    *r0 = tl * a.rows;  // (tiles are whole output rows)
    const int r1 = min(*r0 + a.rows, a.OH) - 1;
    *ih0 = *r0 * a.sh - a.pad_t;
    *rows_needed = (r1 - *r0) * a.sh + (a.kh - 1) * a.dh + 1;
  };
  // address of halo row b of a tile (wavefront-uniform); rows outside the image read row 0 and are replaced later
  auto row_pointer = [&](int n, int ih0, int rows_needed, int b) {
    const int ih = ih0 + b;
    const bool inside = b < rows_needed && ih >= 0 && ih < a.H;
    return a.x + static_cast<size_t>(n) * a.C * plane + __umul24(static_cast<uint32_t>(inside ? ih : 0), static_cast<uint32_t>(a.W));
  };
  // all loads of a tile's patch at once
  auto issue_loads = [&](int (&d)[NBP][4], int tile_index, int row_begin) {
    int n, p0, p_end, r0, ih0, rows_needed;
    tile_geometry(tile_index, &n, &p0, &p_end, &r0, &ih0, &rows_needed);
#pragma unroll
    for (int b = 0; b < NBP; ++b) {
      const uint8_t* row = row_pointer(n, ih0, rows_needed, row_begin + b);
#pragma unroll
      for (int j = 0; j < 4; ++j) d[b][j] = *reinterpret_cast<const int*>(row + ch_off[j]);
    }
  };
  // The same loads with nobody waiting for them: they bring the rows into L2 while the matrix cores work. All
  // write one register, which stays allocated (it is an operand of every one of them and of the wait below)
  // until they have landed.
  int landing = 0;
  auto pull_into_l2 = [&](int tile_index) {
    int n, p0, p_end, r0, ih0, rows_needed;
    tile_geometry(tile_index, &n, &p0, &p_end, &r0, &ih0, &rows_needed);
#pragma unroll
    for (int b = 0; b < NBP * PHASES; ++b) {
      const uint8_t* row = row_pointer(n, ih0, rows_needed, b);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        asm volatile("global_load_dword %0, %1, %2" : "+v"(landing) : "v"(ch_off[j]), "s"(row) : "memory");
    }
  };
  // masks, 4 x 4 byte transposes, stores into halo buffer `halo`
  auto store_halo = [&](const int (&d)[NBP][4], int tile_index, int8_t* halo, int row_begin) {
    int n, p0, p_end, r0, ih0, rows_needed;
    tile_geometry(tile_index, &n, &p0, &p_end, &r0, &ih0, &rows_needed);
    if (has_patch) {
#pragma unroll
      for (int b = 0; b < NBP; ++b) {
        if (row_begin + b >= rows_needed) continue;
        const int ih = ih0 + row_begin + b;
        const int keep = (ih >= 0 && ih < a.H) ? -1 : 0;
        int e[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) e[j] = ((d[b][j] ^ xm) & keep) | (a.pad_fill & ~keep);
        const int lo01 = __builtin_amdgcn_perm(e[1], e[0], 0x05010400);
        const int hi01 = __builtin_amdgcn_perm(e[1], e[0], 0x07030602);
        const int lo23 = __builtin_amdgcn_perm(e[3], e[2], 0x05010400);
        const int hi23 = __builtin_amdgcn_perm(e[3], e[2], 0x07030602);
        int px[4];
        px[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100);
        px[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302);
        px[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100);
        px[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302);
        int8_t* dst = halo + dst0 + __mul24(row_begin + b, row_bytes);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (i < ncols) *reinterpret_cast<int*>(dst + __mul24(i, a.pix_stride)) = px[i];
      }
    }
  };
  auto store_pad_columns = [&](int tile_index, int8_t* halo) {
    int n, p0, p_end, r0, ih0, rows_needed;
    tile_geometry(tile_index, &n, &p0, &p_end, &r0, &ih0, &rows_needed);
    const int right0 = a.pad_l + a.W;
    const int pad_cols = a.pad_l + max(a.iwt - right0, 0);
    const int units = rows_needed * pad_cols * a.cpc;
    const v4i fill = v4i{a.pad_fill, a.pad_fill, a.pad_fill, a.pad_fill};
    for (int u = tid; u < units; u += kThreads) {
      const int cell = u / a.cpc, c = (u - cell * a.cpc) * 16;
      const int hr = cell / pad_cols, pcol = cell - hr * pad_cols;
      const int col = pcol < a.pad_l ? pcol : right0 + (pcol - a.pad_l);
      *reinterpret_cast<v4i*>(halo + (hr * a.iwt + col) * a.pix_stride + c) = fill;
    }
  };
  // Barriers here wait for this wavefront's LDS traffic only: __syncthreads() would also wait for
  // the global stores of the tile just copied out.
  auto lds_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  // ---- prologue: the first tile's rows on their way, the weights by DMA into the (still empty) staging tile and second
  // halo buffer, which lie side by side; from there into every wavefront's registers - 288 KB per CU through LDS,
  // a microsecond of LDS bandwidth with the vector units idle - while the rows are transposed into the first halo
  // buffer - vector work with LDS nearly idle: half of the weight reads are issued in front of each half of the rows ----
  int d0[PHASES][NBP][4];
#pragma unroll
  for (int ph = 0; ph < PHASES; ++ph)
    if (has_patch) issue_loads(d0[ph], t, ph * NBP);
  for (int i = wave * 64; i < a.w_chunks; i += kThreads)
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void*)(a.w + static_cast<size_t>(i + lane) * 16),
        (__attribute__((address_space(3))) void*)(lds + a.off_out + i * 16), 16, 0, 0);
  if (tid < 32 * OT) {
    rq_lds[tid] = a.rq[tid];
    bias_lds[tid] = a.biasf[tid];
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the DMA has landed (and the rows have arrived)
  lds_barrier();
  v4i wr[KSTEPS][OT];
  {
    const int8_t* w_row = lds + a.off_out + frag_row * a.kstride + frag_half * 16;
    constexpr int kPerPhase = (KSTEPS + PHASES - 1) / PHASES;
#pragma unroll
    for (int ph = 0; ph < PHASES; ++ph) {
#pragma unroll
      for (int ks = ph * kPerPhase; ks < (ph + 1) * kPerPhase; ++ks)
        if (ks < KSTEPS) {
#pragma unroll
          for (int j = 0; j < OT; ++j) wr[ks][j] = *reinterpret_cast<const v4i*>(w_row + j * 32 * a.kstride + ks * 32);
        }
      store_halo(d0[ph], t, lds + a.off_halo, ph * NBP);
    }
  }
  store_pad_columns(t, lds + a.off_halo);
  lds_barrier();  // the first halo tile is complete, every wavefront has its weights: staging tile and second buffer are free

  int buf = 0;
  for (; t < t_end; t += per_xcd) {
    const int tn = t + per_xcd;
    const bool has_next = tn < t_end;
    if (has_next && has_patch) pull_into_l2(tn);
    int n, p0, p_end, r0, ih0, rows_needed;
    tile_geometry(t, &n, &p0, &p_end, &r0, &ih0, &rows_needed);
    const int8_t* halo = lds + (buf ? a.off_halo1 : a.off_halo);

    // ---- one 32-pixel MFMA tile at a time: reduction, then requantization into the staging tile ----
#pragma unroll
    for (int i = 0; i < kMaxPtw; ++i) {
      const int pt = wave + 4 * i;
      if (pt < a.PT && p0 + pt * 32 < p_end) {
        const int p = min(p0 + pt * 32 + frag_row, p_end - 1);  // rows past the tile's end recompute its last pixel
        const int oh = static_cast<int>(__umulhi(static_cast<uint32_t>(p), a.magic_ow)), ow = p - oh * a.OW;  // p / OW
        const int8_t* frag = halo + ((oh - r0) * a.sh * a.iwt + ow * a.sw) * a.pix_stride + frag_half * 16;
        // a lane's accumulators belong to one output channel per tile: they start from its folded bias
        v16i acc[OT];
#pragma unroll
        for (int j = 0; j < OT; ++j) {
          const int bias = bias_lds[j * 32 + frag_row];
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[j][r] = bias;
        }
        int sx = 0;
        // fragments RING - 1 k-steps ahead: LDS latency, not bandwidth, is what the loop would wait for
        constexpr int RING = ZP ? 3 : 4;  // (the pixel sums' registers cost the zero-point form one stage)
        v4i fa[RING];
#pragma unroll
        for (int q = 0; q < RING - 1; ++q)
          if (q < KSTEPS) fa[q] = *reinterpret_cast<const v4i*>(frag + a.tap_off[q]);
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          if (ks + RING - 1 < KSTEPS) fa[(ks + RING - 1) % RING] = *reinterpret_cast<const v4i*>(frag + a.tap_off[ks + RING - 1]);
          const v4i f = fa[ks % RING];
          if (ZP) {
#pragma unroll
            for (int q = 0; q < 4; ++q) sx = __builtin_amdgcn_sdot4(f[q], 0x01010101, sx, false);
          }
#pragma unroll
          for (int j = 0; j < OT; ++j) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(f, wr[ks][j], acc[j], 0, 0, 0);
          // a k-step's instructions stay in their k-step: the scheduler otherwise pulls the pixel sums of the fragment
          // just requested in front of the MFMAs on the older ones, and every k-step waits out a whole LDS round trip
          __builtin_amdgcn_sched_barrier(0);
        }
        if (ZP) {
          sx += __shfl_xor(sx, 32);
          __builtin_amdgcn_wave_barrier();
          if (frag_half == 0) sx_lds[frag_row] = a.zws * sx;
          __builtin_amdgcn_wave_barrier();
        }
        // the lane's requantization records, read before the first store into the staging tile (behind a store the
        // compiler has to read them again, and each read is a round trip the wavefront waits out)
        // (not in the tie-testing form, whose extra temporaries leave no registers for them)
        constexpr bool kRecordsAhead = RQ != kRqFast;
        v4i rqj[OT];
#pragma unroll
        for (int j = 0; j < OT; ++j) rqj[j] = kRecordsAhead ? rq_lds[j * 32 + frag_row] : v4i{0, 0, 0, 0};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int pl = pt * 32 + 8 * g + 4 * frag_half;
          v4i s4 = v4i{0, 0, 0, 0};
          if (ZP) s4 = *reinterpret_cast<const v4i*>(sx_lds + 8 * g + 4 * frag_half);
#pragma unroll
          for (int j = 0; j < OT; ++j) {
            const int ocl = j * 32 + frag_row;
            const v4i rq = kRecordsAhead ? rqj[j] : rq_lds[ocl];
            int r4[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              r4[e] = ZP ? acc[j][g * 4 + e] - s4[e] : acc[j][g * 4 + e];
            *reinterpret_cast<uint32_t*>(out_tile + ocl * a.out_stride + pl) = RequantPack4<RQ>(r4, rq, a.out_zp, a.lo, a.hi);
          }
        }
        if (ZP) __builtin_amdgcn_wave_barrier();  // the sums are read before the next MFMA tile's are written
      }
    }
    // ---- the next tile's rows: L2 -> registers -> the other halo buffer ----
    if (has_next) {
      int8_t* halo_next = lds + (buf ? a.off_halo : a.off_halo1);
      if (has_patch) asm volatile("s_waitcnt vmcnt(0)" : "+v"(landing)::"memory");
#pragma unroll
      for (int ph = 0; ph < PHASES; ++ph) {
        int d[NBP][4];
        if (has_patch) issue_loads(d, tn, ph * NBP);
        store_halo(d, tn, halo_next, ph * NBP);
      }
      store_pad_columns(tn, halo_next);
    }
    lds_barrier();  // staging tile complete, next halo complete
    // ---- copy out: contiguous runs of the WHCN output ----
    {
      const int valid = p_end - p0;
      const int oc_n = min(a.oct, a.OC);
      uint8_t* ybase = a.y + static_cast<size_t>(n) * a.OC * hw + p0;
      if ((((hw | p0 | valid) & 15) | (reinterpret_cast<uintptr_t>(a.y) & 15)) == 0) {
        // 16 bytes per lane, four output-channel rows per wavefront instruction
        const int chunk = lane & 15, chunks = valid >> 4;
        for (int o = wave * 4 + (lane >> 4); o < oc_n; o += 16) {
          if (chunk < chunks) {
            const int* src = reinterpret_cast<const int*>(out_tile + o * a.out_stride + chunk * 16);
            const v4i v = v4i{src[0], src[1], src[2], src[3]};
            *reinterpret_cast<v4i*>(ybase + static_cast<size_t>(o) * hw + chunk * 16) = v;
          }
        }
      } else {
        const int per_row = valid >> 2;  // p0 and hw are multiples of 4: whole dwords
        for (int o = wave; o < oc_n; o += 4)
          for (int dwi = lane; dwi < per_row; dwi += 64)
            *reinterpret_cast<uint32_t*>(ybase + static_cast<size_t>(o) * hw + dwi * 4) =
                *reinterpret_cast<const uint32_t*>(out_tile + o * a.out_stride + dwi * 4);
      }
    }
    lds_barrier();  // everyone has read the staging tile before the next tile's results go in
    buf ^= 1;
  }
  asm volatile("" ::"v"(landing));
}

struct Plan {
  ConvArgs a;
  int lds_bytes;
  int ot, rq;
  dim3 grid;
  int persist_ksteps;  // 0: one tile per workgroup (ConvIgemmKernel); else the persistent variant
  bool zp, small;
};

typedef void (*PersistFn)(ConvArgs);
// The persistent variant exists for these reduction lengths (k-steps of 32 bytes) with two output-channel tiles.
template <int KSTEPS, int NBP, int PHASES>
PersistFn PersistKernelOf(int rq, bool zp) {
  if (rq == kRqFastNoTie)
    return zp ? ConvPersistKernel<KSTEPS, 2, kRqFastNoTie, true, NBP, PHASES> : ConvPersistKernel<KSTEPS, 2, kRqFastNoTie, false, NBP, PHASES>;
  return zp ? ConvPersistKernel<KSTEPS, 2, kRqFast, true, NBP, PHASES> : ConvPersistKernel<KSTEPS, 2, kRqFast, false, NBP, PHASES>;
}
// small: tiles of at most four halo rows (two batches of two rows); else two batches of three
PersistFn PersistKernel(int ksteps, int rq, bool zp, bool small) {
  if (rq == kRqGeneric) return nullptr;
  switch (ksteps) {
    case 9: return small ? PersistKernelOf<9, 2, 2>(rq, zp) : PersistKernelOf<9, 3, 2>(rq, zp);
    case 18: return small ? PersistKernelOf<18, 2, 2>(rq, zp) : PersistKernelOf<18, 3, 2>(rq, zp);
  }
  return nullptr;
}

template <int OT>
void LaunchRq(const Plan* plan, const ConvArgs& a, hipStream_t st) {
  const dim3 block(kThreads);
  if (plan->rq == kRqFastNoTie)
    hipLaunchKernelGGL((ConvIgemmKernel<OT, kRqFastNoTie>), plan->grid, block, plan->lds_bytes, st, a);
  else if (plan->rq == kRqFast)
    hipLaunchKernelGGL((ConvIgemmKernel<OT, kRqFast>), plan->grid, block, plan->lds_bytes, st, a);
  else
    hipLaunchKernelGGL((ConvIgemmKernel<OT, kRqGeneric>), plan->grid, block, plan->lds_bytes, st, a);
}

int ConvIgemmRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  ConvArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if (plan->persist_ksteps) {
    if (reinterpret_cast<uintptr_t>(in0) & 3 || reinterpret_cast<uintptr_t>(out) & 3)
      return SetError(TVX_E_INVALID, "conv2d_igemm_i8: tensors must be 4-byte aligned");
    hipLaunchKernelGGL(PersistKernel(plan->persist_ksteps, plan->rq, plan->zp, plan->small), plan->grid, dim3(kThreads), plan->lds_bytes, st, a);
  } else if (plan->ot == 1) LaunchRq<1>(plan, a, st);
  else if (plan->ot == 2) LaunchRq<2>(plan, a, st);
  else LaunchRq<4>(plan, a, st);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

int RoundUp(int v, int m) { return (v + m - 1) / m * m; }

uint32_t Magic(int d) {
  return d <= 1 ? 0u : static_cast<uint32_t>(((uint64_t{1} << 32) + d - 1) / d);
}

template <int OT, int RQ>
hipError_t AllowLds(int bytes) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(&ConvIgemmKernel<OT, RQ>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
}

}  // namespace

// Claims dense quantized convolutions with constant weights whose weight block
// and halo tile fit the CU's LDS.
int ConvIgemmSetup(tvx_op* op, const tvx_conv2d_desc* d, const void* w_host, const void* bias_host) {
  if (!op->quantized || !w_host || d->multiplier != 0 || d->groups > 1) return TVX_E_UNSUPPORTED;
  ConvArgs a{};
  a.C = d->in_c; a.H = d->in_h; a.W = d->in_w; a.OC = d->out_c; a.OH = d->out_h; a.OW = d->out_w;
  a.kh = d->k_h; a.kw = d->k_w; a.sh = d->stride_h; a.sw = d->stride_w;
  a.dh = d->dilation_h; a.dw = d->dilation_w; a.pad_t = d->pad_top; a.pad_l = d->pad_left;
  const int taps = a.kh * a.kw;
  const int oc_pad = RoundUp(a.OC, 32);
  int ot = oc_pad <= 32 ? 1 : (oc_pad <= 64 ? 2 : 4);
  // pixel tile: the multiple of 32 (<= 256) wasting the fewest MFMA rows
  const int hw = a.OH * a.OW;
  int best_p = 32;
  double best_eff = 0;
  for (int p = 256; p >= 32; p -= 32) {
    const int tiles = (hw + p - 1) / p;
    const double eff = static_cast<double>(hw) / (static_cast<double>(tiles) * p);
    if (eff > best_eff + 1e-9) { best_eff = eff; best_p = p; }
  }
  // Few pixels and many channels (256 -> 256 on 14 x 14, batch 32: 64 such workgroups on 256 CUs): when that
  // choice fills less than half of the chip's workgroup slots, trade tile size for workgroups. A workgroup's
  // critical path is modelled as its MFMA blocks per wavefront (32-pixel tiles / 4 wavefronts x 32-channel
  // tiles) plus two blocks' worth of loads and barriers, the launch as that times the rounds the workgroups
  // need on two slots per CU; ties go to the larger tiles (fewer halo copies).
  {
    int cus = 256;
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
    const long long slots = 2ll * cus;
    auto workgroups = [&](int ot_, int p_) {
      return static_cast<long long>(d->batch) * ((hw + p_ - 1) / p_) * ((oc_pad + 32 * ot_ - 1) / (32 * ot_));
    };
    // (up to 64 output channels the choice above also decides the persistent variant: there only a launch of a
    // few workgroups - LeNet's second convolution at batch 1 is one - is re-cut)
    const char* persist_lever = getenv("TVX_IGEMM_PERSIST");  // (forcing the persistent variant keeps its tile choice)
    const bool tiny = ot < 4 && workgroups(ot, best_p) < cus / 8 && !(persist_lever && atoi(persist_lever) > 0);
    if ((ot == 4 && workgroups(ot, best_p) < slots / 2) || tiny) {
      auto cost = [&](int ot_, int p_) {
        const long long rounds = (workgroups(ot_, p_) + slots - 1) / slots;
        return rounds * (((p_ / 32 + 3) / 4) * ot_ + 2);
      };
      long long best_cost = cost(ot, best_p);
      const int ot_max = ot;
      for (int ot_ = ot_max; ot_ >= 1; ot_ /= 2)
        for (int p_ = 256; p_ >= 32; p_ -= 32) {
          if (p_ - 32 >= hw) continue;  // (a tile larger than the image needs)
          const long long c = cost(ot_, p_);
          if (c < best_cost) { best_cost = c; ot = ot_; best_p = p_; }
        }
    }
  }
  if (const char* f = getenv("TVX_IGEMM_OT")) { const int v = atoi(f); if ((v == 1 || v == 2 || v == 4) && 32 * v <= std::max(oc_pad, 32) * 2) ot = v; }  // tuning aid
  if (const char* f = getenv("TVX_IGEMM_P")) { const int v = atoi(f); if (v >= 32 && v <= 256 && v % 32 == 0) best_p = v; }  // tuning aid
  a.oct = 32 * ot;
  const int oc_blocks = (oc_pad + a.oct - 1) / a.oct;
  const int oc_alloc = oc_blocks * a.oct;
  a.P = best_p;
  a.PT = a.P / 32;
  a.tiles_per_image = (hw + a.P - 1) / a.P;
  // halo extent: the most output rows any tile touches
  a.pool = op->fused_pool;  // (the caller has checked the pooling: 2 x 2, stride 2, even output extents)
  int max_rows = 1;
  for (int t = 0; t < a.tiles_per_image; ++t) {
    const int p0 = t * a.P, pe = std::min(p0 + a.P, hw);
    if (a.pool) {  // pixels in pooling order: pairs of rows
      const int pw = a.OW / 2;
      max_rows = std::max(max_rows, 2 * (((pe - 1) / 4) / pw - (p0 / 4) / pw + 1));
    } else {
      max_rows = std::max(max_rows, (pe - 1) / a.OW - p0 / a.OW + 1);
    }
  }
  a.iht = (max_rows - 1) * a.sh + (a.kh - 1) * a.dh + 1;
  a.iwt = std::max((a.OW - 1) * a.sw + (a.kw - 1) * a.dw + 1, 1);
  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127) return TVX_E_UNSUPPORTED;  // zero point outside the tensor's range
  a.xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.pad_fill = static_cast<int>(static_cast<uint32_t>(zxs & 0xff) * 0x01010101u);
  a.zws = zws;
  a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  a.out_stride = ((a.P / 4) | 1) * 4;
  a.w4_blocks = (a.W / 4 + 15) / 16;
  // Reduction groups: the weights of one output-channel block and the halo tile must sit in
  // LDS together. All input channels at once when that fits next to a second workgroup on
  // the CU; otherwise the largest channel group that does (the kernel then walks the groups,
  // accumulating), and as a last resort whatever fits at all.
  const int sx_bytes = a.P * 4;
  const int out_bytes = a.oct * a.out_stride;
  int lds_bytes = 0, w_bytes = 0, kchunks = 0;
  auto plan_group = [&](int cp) {
    a.cp = cp;
    a.cpc = cp / 16;
    kchunks = taps * a.cpc;
    a.ksteps = (kchunks + 1) / 2;
    a.kstride = a.ksteps * 32 + 16;
    // Consecutive pixels of a fragment read must fall into different 16-byte bank
    // groups: that holds when the pixel stride is an odd number of 16-byte chunks.
    a.pix_stride = (a.cpc & 1) ? a.cp : a.cp + 16;
    w_bytes = RoundUp(a.oct * a.kstride, 1024);  // whole 1 KiB DMA bursts
    a.w_chunks = w_bytes / 16;
    const int halo_bytes = RoundUp(a.iht * a.iwt * a.pix_stride + 16, 16);
    const int tap_bytes = RoundUp((a.ksteps * 2 + 4) * 8, 16);
    const int rq_bytes = a.oct * 16, bias_bytes = a.oct * 4;
    // LDS carve-up: the per-pixel sums first; the weight + halo region behind them
    // is reused as the epilogue's staging tile
    a.off_sx = 0;
    a.off_tap = sx_bytes;
    a.off_rq = a.off_tap + tap_bytes;
    a.off_bias = a.off_rq + rq_bytes;
    a.off_w = a.off_bias + bias_bytes;
    a.off_halo = a.off_w + w_bytes;
    lds_bytes = a.off_w + std::max(w_bytes + halo_bytes, RoundUp(out_bytes, 16));
    a.groups = (a.C + cp - 1) / cp;
  };
  const int c_pad = RoundUp(a.C, 16);
  bool planned = false;
  for (int limit : {76 * 1024, 150 * 1024}) {
    for (int cp = c_pad; cp >= 16 && !planned; cp = cp > 256 ? 256 : cp / 2) {
      const int c16 = RoundUp(cp, 16);
      plan_group(c16);
      if (lds_bytes <= limit) planned = true;
    }
    if (planned) break;
  }
  if (!planned) return TVX_E_UNSUPPORTED;
  a.w_group_stride = oc_alloc * a.kstride + 1024;  // slack: the last block's DMA reads whole bursts
  // the loader's index split is exact while units * divisor < 2^32
  if (static_cast<uint64_t>(a.W) * a.cp >= (1ull << 24)) return TVX_E_UNSUPPORTED;
  // the loader uses 24-bit multiplies and 32-bit offsets inside one image
  if (static_cast<uint64_t>(a.H) * a.W >= (1ull << 24) ||
      static_cast<uint64_t>(a.H) * a.W * a.C >= (1ull << 31) ||
      static_cast<uint64_t>(a.iht) * a.iwt * a.pix_stride >= (1ull << 23))
    return TVX_E_UNSUPPORTED;
  if (static_cast<uint64_t>(d->batch) * a.tiles_per_image > 0x7fffffffull) return TVX_E_UNSUPPORTED;
  if (static_cast<uint64_t>(a.w_group_stride) * a.groups >= (1ull << 31)) return TVX_E_UNSUPPORTED;

  // ---- pack weights [group][oc][(ky,kx,c)] int8 with zero padding, fold constants -------
  std::vector<int8_t> packed(static_cast<size_t>(a.w_group_stride) * a.groups, 0);
  std::vector<int32_t> biasf(oc_alloc, 0);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  for (int oc = 0; oc < a.OC; ++oc) {
    int64_t sw = 0;
    for (int t = 0; t < taps; ++t)
      for (int c = 0; c < a.C; ++c) {
        const uint8_t raw = src[(static_cast<size_t>(oc) * a.C + c) * taps + t];
        const int8_t v = static_cast<int8_t>(w_u8 ? raw ^ 0x80 : raw);
        const int g = c / a.cp, cl = c % a.cp;
        packed[static_cast<size_t>(g) * a.w_group_stride + static_cast<size_t>(oc) * a.kstride +
               (t * a.cpc + cl / 16) * 16 + cl % 16] = v;
        sw += v;
      }
    const int64_t v = (b ? b[oc] : 0) - static_cast<int64_t>(zxs) * sw +
                      static_cast<int64_t>(taps) * a.C * zxs * zws;
    biasf[oc] = static_cast<int32_t>(static_cast<uint32_t>(v));
  }
  // ---- requantization records: 32-bit arithmetic when every shift allows it -------
  std::vector<int32_t> rqt;
  const int rq = BuildRequantRecords(op->h_mult, op->h_shift, a.OC, oc_alloc, d->out_zp, &rqt,
                                     AccumulatorBound(static_cast<uint64_t>(taps) * a.C, bias_host, a.OC));
  // tap table: chunk q = 2 * kstep + half of the (ky, kx, chunk) order; two spare
  // k-steps at the end so that the loop's prefetch stays inside the table
  std::vector<int32_t> tapt(static_cast<size_t>(a.ksteps + 2) * 4, 0);
  for (int q = 0; q < kchunks; ++q) {
    const int t = q / a.cpc, cc = q % a.cpc;
    const int ky = t / a.kw, kx = t % a.kw;
    tapt[q * 2] = (ky * a.dh * a.iwt + kx * a.dw) * a.pix_stride + cc * 16;
    tapt[q * 2 + 1] = 0x01010101;
  }
  int s = op->packed.Upload(packed.data(), packed.size());
  if (s == TVX_OK) s = op->aux3.Upload(tapt.data(), tapt.size() * 4);
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  if (s != TVX_OK) return s;
  a.w = op->packed.as<int8_t>();
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<v4i>();
  a.tapt = op->aux3.as<int2>();

  hipError_t e = hipSuccess;
  if (ot == 1) {
    e = rq == kRqGeneric ? AllowLds<1, kRqGeneric>(lds_bytes)
        : (rq == kRqFast ? AllowLds<1, kRqFast>(lds_bytes) : AllowLds<1, kRqFastNoTie>(lds_bytes));
  } else if (ot == 2) {
    e = rq == kRqGeneric ? AllowLds<2, kRqGeneric>(lds_bytes)
        : (rq == kRqFast ? AllowLds<2, kRqFast>(lds_bytes) : AllowLds<2, kRqFastNoTie>(lds_bytes));
  } else {
    e = rq == kRqGeneric ? AllowLds<4, kRqGeneric>(lds_bytes)
        : (rq == kRqFast ? AllowLds<4, kRqFast>(lds_bytes) : AllowLds<4, kRqFastNoTie>(lds_bytes));
  }
  if (e != hipSuccess)
    return SetError(TVX_E_DEVICE, "hipFuncSetAttribute(dynamic LDS %d): %s", lds_bytes, hipGetErrorString(e));
  Plan plan;
  plan.a = a;
  plan.lds_bytes = lds_bytes;
  plan.ot = ot;
  plan.rq = rq;
  plan.persist_ksteps = 0;
  plan.zp = zws != 0;
  plan.small = false;
  plan.grid = dim3(static_cast<unsigned>(d->batch * a.tiles_per_image), static_cast<unsigned>(oc_blocks));

  // ---- the persistent variant, where it applies ------------------------------------------------
  do {
    if (a.pool) break;  // the pooled epilogue exists in the one-tile-per-workgroup kernel
    if (const char* f = getenv("TVX_IGEMM_PERSIST")) if (atoi(f) == 0) break;  // tuning aid
    if (a.groups != 1 || a.cp != a.C || (a.cpc & 1) || oc_blocks != 1 || ot != 2 || (a.W & 3)) break;  // two output-channel tiles
    const int ksteps = taps * a.cpc / 2;
    if (!PersistKernel(ksteps, rq, plan.zp, false) || ksteps > 40) break;
    if (a.w4_blocks * ((a.cp / 4 + 3) / 4) > kThreads / 64) break;  // one patch per thread
    // pixel tile: whole output rows, at most six halo rows and 256 pixels; as many tiles as keep a few in
    // every workgroup's queue
    int want_rows = 0;
    if (const char* f = getenv("TVX_IGEMM_TILE_ROWS")) want_rows = atoi(f);  // tuning aid
    int rows = 0;
    if ((a.OH * a.OW) & 3) break;  // the copy-out writes whole dwords
    for (int r = 1; r <= a.OH; ++r) {
      if ((r - 1) * a.sh + (a.kh - 1) * a.dh + 1 > kPersistRows || r * a.OW > 256) break;
      if (r * a.OW & 3) continue;
      rows = r;
      if (r == want_rows) break;
    }
    if (rows == 0) break;
    ConvArgs pa = a;
    // the reciprocal the kernel divides pixel indices by the row length with: exact while p * OW < 2^32
    if (a.OW < 2 || static_cast<uint64_t>(a.OH) * a.OW * a.OW >= (uint64_t{1} << 32)) break;
    pa.magic_ow = static_cast<uint32_t>(((uint64_t{1} << 32) + a.OW - 1) / a.OW);
    pa.P = rows * a.OW;
    pa.PT = (pa.P + 31) / 32;
    pa.tiles_per_image = (a.OH + rows - 1) / rows;
    pa.rows = rows;
    pa.blk_col = pa.blk_chan = 0;
    for (int wv = 0; wv < kThreads / 64; ++wv) {
      pa.blk_col |= static_cast<uint32_t>(wv % pa.w4_blocks) << (8 * wv);
      pa.blk_chan |= static_cast<uint32_t>(wv / pa.w4_blocks) << (8 * wv);
    }
    if (static_cast<uint64_t>(d->batch) * pa.tiles_per_image * pa.tiles_per_image >= (uint64_t{1} << 32)) break;
    pa.magic_tpi = pa.tiles_per_image > 1 ? static_cast<uint32_t>(((uint64_t{1} << 32) + pa.tiles_per_image - 1) / pa.tiles_per_image) : 0u;
    pa.iht = (rows - 1) * a.sh + (a.kh - 1) * a.dh + 1;
    plan.small = pa.iht <= 4;
    PersistFn fn = PersistKernel(ksteps, rq, plan.zp, plan.small);
    pa.out_stride = ((pa.PT * 32 / 4) | 1) * 4;
    const uint64_t total = static_cast<uint64_t>(d->batch) * pa.tiles_per_image;
    if (total > 0x7fffffffull) break;
    pa.total_tiles = static_cast<int>(total);
    pa.oct = 64;
    pa.halo_bytes = RoundUp(pa.iht * pa.iwt * pa.pix_stride + 64, 16);
    pa.off_sx = 0;
    pa.off_rq = 512;
    pa.off_bias = pa.off_rq + 64 * 16;
    // first halo buffer | staging tile | second halo buffer: the weights' DMA lands in the last two
    pa.off_halo = pa.off_bias + 64 * 4;
    pa.off_out = pa.off_halo + pa.halo_bytes;
    pa.off_halo1 = pa.off_out + RoundUp(pa.oct * pa.out_stride, 16);
    // (the weights pass through the staging tile and the halo buffers on their way into the registers)
    const int plds = std::max(pa.off_halo1 + pa.halo_bytes, pa.off_out + pa.w_chunks * 16);
    if (plds > 80 * 1024) break;  // two workgroups per CU
    for (int ks = 0; ks < ksteps; ++ks) pa.tap_off[ks] = tapt[ks * 4];  // chunk 2 * ks (chunk 2 * ks + 1 follows it)
    bool halves_adjacent = true;
    for (int ks = 0; ks < ksteps; ++ks) halves_adjacent = halves_adjacent && tapt[ks * 4 + 2] == tapt[ks * 4] + 16;
    if (!halves_adjacent) break;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(fn), hipFuncAttributeMaxDynamicSharedMemorySize, plds) != hipSuccess) {
      (void)hipGetLastError();
      break;
    }
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) break;
    int wgs = 2 * prop.multiProcessorCount;
    // Few tiles: one tile per workgroup on as many CUs as there are tiles is as fast, and the prologue above
    // (the weights into every wavefront's registers) is not free.
    bool forced = false;
    if (const char* f = getenv("TVX_IGEMM_PERSIST")) forced = atoi(f) > 0;  // tuning aid
    if (pa.total_tiles < wgs * 3 / 4 && !forced && !getenv("TVX_IGEMM_WGS")) break;
    if (const char* f = getenv("TVX_IGEMM_WGS")) wgs = std::max(8, atoi(f));  // tuning aid
    wgs = std::min<int>(wgs, RoundUp(pa.total_tiles, 8));
    wgs = std::max(8, wgs / 8 * 8);
    plan.a = pa;
    plan.lds_bytes = plds;
    plan.persist_ksteps = ksteps;
    plan.grid = dim3(static_cast<unsigned>(wgs));
  } while (false);
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = ConvIgemmRun;
  op->kernel_name = plan.persist_ksteps ? "conv2d_igemm_i8_persistent" : (a.pool ? "conv2d_igemm_maxpool_i8" : "conv2d_igemm_i8");
  return TVX_OK;
}

}  // namespace tvx
