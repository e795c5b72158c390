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
//   epilogue requantization from the wavefront's own accumulators; two lane swaps between the
//            wavefront's halves (v_permlane32_swap) give every lane sixteen consecutive pixels
//            of a channel, which go to the WHCN output as they are: no staging in LDS.
#include <algorithm>
#include <cstdlib>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kBandThreads = 1024;
constexpr int kBandWaves = kBandThreads / 64;

struct BandArgs {
  // what stands between a wavefront's start and its first loads comes first
  const uint8_t* x;
  int total_tiles, tiles_per_xcd;
  int tiles_per_image, gblocks, gpr, iwt_div;
  uint32_t magic_tpi, magic_gblocks, magic_gpr, magic_iwt, magic_ow, magic_padcols;
  int n_g8;              // 8-column groups of a band's halo rows
  int C, H, W, OC, OH, OW;
  int sh, sw, pad_t, pad_l, khe;  // khe: rows a kernel column spans, (kh - 1) * dh + 1
  int rows;              // output rows of a band
  int PT;                // 32-pixel tiles of a full band
  int iwt, pix_stride;
  const int8_t* w;       // packed [64][kstride]
  uint8_t* y;
  const int32_t* biasf;  // bias + per-channel zero-point terms
  const v4i* rq;         // per channel {mult, t, rounding constant, tie mask}
  int kstride, w_chunks;
  int row_step, col_step;  // halo bytes from a kernel row / column to the next
  int s_row_step, s_col_step;  // ... sum-plane cells
  int xor_mask, pad_fill, zws, out_zp, lo, hi;
  int halo_rows, pad_cols, s_pad;  // s_pad: channel sum of a padding pixel
  int off_sx, off_rq, off_bias, off_w, off_halo0, off_halo1, off_s, s_bytes;
};

// u / d by the host-made reciprocal ceil(2^32 / d); 0 stands for d = 1
__device__ __forceinline__ int FastDiv(int u, uint32_t magic) {
  return static_cast<int>(__umulhi(static_cast<uint32_t>(u), magic)) + (magic == 0 ? u : 0);
}

// KH x KW taps over CPC 16-channel chunks (an even number): a k-step is one tap's pair of chunks.
template <int KH, int KW, int CPC, int RQ, bool ZP>
__global__ void __launch_bounds__(kBandThreads) __attribute__((amdgpu_waves_per_eu(4, 4)))
ConvBandKernel(BandArgs a) {
  constexpr int KSTEPS = KH * KW * CPC / 2;
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frag_row = lane & 31, frag_half = lane >> 5;

  // An XCD gets a contiguous run of bands (neighbouring bands of an image share halo rows and meet in that
  // XCD's L2); inside the run the XCD's workgroups interleave.
  const int xcd = blockIdx.x & 7, per_xcd = gridDim.x >> 3;
  int t = xcd * a.tiles_per_xcd + (blockIdx.x >> 3);
  const int t_end = min((xcd + 1) * a.tiles_per_xcd, a.total_tiles);
  if (t >= t_end) return;

  // ---- this thread's patch: 8 input columns x 4 channels of one halo row. Sixteen consecutive lanes read
  // 128 contiguous bytes of a channel plane, the next sixteen the next channel group.
  const uint32_t plane32 = static_cast<uint32_t>(a.H * a.W);
  const int cb = FastDiv(wave, a.magic_gblocks);
  const int g8 = (wave - cb * a.gblocks) * 16 + (lane & 15);
  const int c4 = cb * 4 + (lane >> 4);
  const bool has_patch = g8 < a.n_g8 && c4 * 4 < a.C;
  const int hr = has_patch ? FastDiv(g8, a.magic_gpr) : 0;
  const int col0 = has_patch ? (g8 - hr * a.gpr) * 8 : 0;
  const uint32_t ch_off = has_patch ? static_cast<uint32_t>(c4 * 4) * plane32 + static_cast<uint32_t>(col0) : 0u;
  const int px0 = hr * a.iwt + a.pad_l + col0;  // the patch's first pixel in the halo tile
  // With the i-th store every lane would write its i-th pixel: pixels 8 apart, i.e. one LDS bank for all column
  // groups of a wavefront. The lanes therefore rotate their pixels by their column group (the loaded dwords'
  // bytes are the pixels: a byte rotation in front of the transposes), and the i-th store writes pixel
  // (i + rot) % 8: eight banks apart times four channel groups - every bank, twice.
  const int rot = lane & 7;
  int pxm[8];  // halo pixel of the i-th store
#pragma unroll
  for (int i = 0; i < 8; ++i) pxm[i] = px0 + ((i + rot) & 7);
  // v_perm selectors of the rotation: byte k of the low dword is byte (k + rot) % 8 of the row, the high dword follows
  const uint32_t sel_lo = (static_cast<uint32_t>(rot & 7) | static_cast<uint32_t>((rot + 1) & 7) << 8 |
                           static_cast<uint32_t>((rot + 2) & 7) << 16 | static_cast<uint32_t>((rot + 3) & 7) << 24);
  const uint32_t sel_hi = sel_lo ^ 0x04040404u;
  const uint32_t image_bytes = static_cast<uint32_t>(a.C) * plane32;

  // Is this thread's halo row inside the image for band `tile_index`? (lanes hold different rows)
  auto row_of = [&](int tile_index, int* n, bool* inside) {
    const int img = FastDiv(tile_index, a.magic_tpi);
    const int r0 = (tile_index - img * a.tiles_per_image) * a.rows;
    const int rows_here = min(a.rows, a.OH - r0);
    const int ih = r0 * a.sh - a.pad_t + hr;
    *n = img;
    *inside = hr < (rows_here - 1) * a.sh + a.khe && ih >= 0 && ih < a.H;
    return *inside ? ih : 0;  // rows outside read row 0 and are replaced by the zero point behind the load
  };
  // The loads are inline assembly and are waited for by hand (loads_landed): the compiler's own wait insertion
  // would also wait for the output stores issued in between. To the compiler d[] is defined here and next used
  // by loads_landed, so it keeps the registers untouched in between.
  auto issue_loads = [&](int2 (&d)[4], int tile_index) {
    int n;
    bool inside;
    const uint32_t row_off = __umul24(static_cast<uint32_t>(row_of(tile_index, &n, &inside)), static_cast<uint32_t>(a.W));
    const uint8_t* img = a.x + static_cast<size_t>(static_cast<uint32_t>(n)) * image_bytes;
    uint32_t off = ch_off + row_off;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(d[j]) : "v"(off), "s"(img) : "memory");
      off += plane32;
    }
  };
  auto loads_landed = [](int2 (&d)[4]) {
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3])::"memory");
  };
  // masks, two 4 x 4 byte transposes, eight dword stores; the patch's share of its pixels' channel sums goes
  // into the sum plane `splane` by LDS atomics
  auto store_halo = [&](const int2 (&d)[4], int tile_index, int8_t* halo, int* splane) {
    int n;
    bool inside;
    (void)row_of(tile_index, &n, &inside);
    uint32_t lo4[4], hi4[4], px[8];
    // a band whose halo rows all lie inside the image (wavefront-uniform: most bands) needs no masks
    const int tl = tile_index - n * a.tiles_per_image;
    const int ih0 = tl * a.rows * a.sh - a.pad_t;
    const bool all_inside = ih0 >= 0 && ih0 + a.halo_rows <= a.H && (tl + 1) * a.rows <= a.OH;
    if (all_inside) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = static_cast<uint32_t>(d[j].x ^ a.xor_mask), hi = static_cast<uint32_t>(d[j].y ^ a.xor_mask);
        lo4[j] = __builtin_amdgcn_perm(hi, lo, sel_lo);
        hi4[j] = __builtin_amdgcn_perm(hi, lo, sel_hi);
      }
    } else {
      const int keep = inside ? -1 : 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = static_cast<uint32_t>(((d[j].x ^ a.xor_mask) & keep) | (a.pad_fill & ~keep));
        const uint32_t hi = static_cast<uint32_t>(((d[j].y ^ a.xor_mask) & keep) | (a.pad_fill & ~keep));
        lo4[j] = __builtin_amdgcn_perm(hi, lo, sel_lo);
        hi4[j] = __builtin_amdgcn_perm(hi, lo, sel_hi);
      }
    }
    Transpose4x4(lo4, px);
    Transpose4x4(hi4, px + 4);
    if (has_patch) {
#pragma unroll
      for (int i = 0; i < 8; ++i) *reinterpret_cast<uint32_t*>(halo + c4 * 4 + __mul24(pxm[i], a.pix_stride)) = px[i];
      if (ZP) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
          __hip_atomic_fetch_add(splane + pxm[i], __builtin_amdgcn_sdot4(static_cast<int>(px[i]), 0x01010101, 0, false),
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      }
    }
  };
  // The sum plane of the band after next starts from zero, its padding columns from the padding pixel's sum.
  const int s_cells = a.halo_rows * a.iwt;
  const int s_col = tid - FastDiv(tid, a.magic_iwt) * a.iwt_div;
  const int s_init = (s_col < a.pad_l || s_col >= a.pad_l + a.W) ? a.s_pad : 0;
  auto clear_sums = [&](int* splane) {
    if (ZP && tid < s_cells) splane[tid] = s_init;
  };
  auto sum_plane = [&](int k) { return reinterpret_cast<int*>(lds + a.off_s + k * a.s_bytes); };
  auto lds_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  // ---- prologue: the first band's rows on their way, weights and tables by DMA, the padding columns of both
  // halo buffers (no band ever writes them again), the sum planes' start values ----
  int2 dn[4];
  issue_loads(dn, t);
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
  clear_sums(sum_plane(0));
  clear_sums(sum_plane(1));
  {
    // padding cells (halo row, padding column, 16-channel chunk) of both buffers, one per thread and step
    const int cpc = a.C >> 4;
    const int per_buf = a.halo_rows * a.pad_cols * cpc;
    const v4i fill = v4i{a.pad_fill, a.pad_fill, a.pad_fill, a.pad_fill};
    for (int u = tid; u < 2 * per_buf; u += kBandThreads) {
      const int b = u >= per_buf ? 1 : 0, v = u - b * per_buf;
      const int chunk = v & (cpc - 1), cell = v >> (cpc == 4 ? 2 : 1);  // cpc is 2 or 4
      const int r = FastDiv(cell, a.magic_padcols);
      const int pcol = cell - r * a.pad_cols;
      const int col = pcol < a.pad_l ? pcol : a.W + pcol;
      *reinterpret_cast<v4i*>(lds + (b ? a.off_halo1 : a.off_halo0) + (r * a.iwt + col) * a.pix_stride + chunk * 16) = fill;
    }
  }
  lds_barrier();  // the sum planes hold their start values
  // s_waitcnt vmcnt(0) as an instruction the compiler sees: it then knows that the DMA has landed (behind a wait in
  // inline assembly it would go on protecting every later LDS read with a wait for all memory operations)
  __builtin_amdgcn_s_waitcnt(0x0f70);
  loads_landed(dn);
  store_halo(dn, t, lds + a.off_halo0, sum_plane(0));
  if (t + per_xcd < t_end) issue_loads(dn, t + per_xcd);
  lds_barrier();

  // ---- the bands: multiply the present band; feed (the next band's rows into the other halo buffer, the loads of
  // the band after it); requantize and store the present band; one barrier ----
  const int hw = a.OH * a.OW;
  int buf = 0, sk = 0;  // halo buffer and sum plane of the present band
  for (; t < t_end; t += per_xcd) {
    const int tn = t + per_xcd;
    const bool has_next = tn < t_end;
    const int img = FastDiv(t, a.magic_tpi);
    const int r0 = (t - img * a.tiles_per_image) * a.rows;
    const int valid = min(a.rows, a.OH - r0) * a.OW;  // pixels of this band
    const bool mine = wave < a.PT && wave * 32 < valid;
    int* sx_lds = reinterpret_cast<int*>(lds + a.off_sx) + wave * 32;  // wavefront-private

    v16i acc[2];
    if (mine) {
      const int8_t* halo = lds + (buf ? a.off_halo1 : a.off_halo0);
      const int pl = min(wave * 32 + frag_row, valid - 1);  // rows past the band's end recompute its last pixel
      const int ohl = FastDiv(pl, a.magic_ow), ow = pl - ohl * a.OW;
      const int hp = ohl * a.sh * a.iwt + ow * a.sw;  // the window's first halo pixel
      const int8_t* frag = halo + hp * a.pix_stride + frag_half * 16;
      const int8_t* w_row = lds + a.off_w + frag_row * a.kstride + frag_half * 16;
      const int* bias_lds = reinterpret_cast<const int*>(lds + a.off_bias);
      // The zero-point term of the wavefront's 32 pixels: window sums of the sum plane, times the weights' zero
      // point (requested here, used behind the multiplication).
      int st[KH * KW];
      if (ZP) {
        const int* sp = sum_plane(sk) + hp;
#pragma unroll
        for (int ky = 0; ky < KH; ++ky)
#pragma unroll
          for (int kx = 0; kx < KW; ++kx) st[ky * KW + kx] = sp[ky * a.s_row_step + kx * a.s_col_step];
        int sx = 0;
#pragma unroll
        for (int i = 0; i < KH * KW; ++i) sx += st[i];
        if (frag_half == 0) sx_lds[frag_row] = a.zws * sx;
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int bias = bias_lds[j * 32 + frag_row];
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[j][r] = bias;
      }
      constexpr int RING = 3;
      v4i fa[RING], fb[RING][2];
      auto fetch = [&](int ks, int slot_) {
        const int tap = ks * 2 / CPC, cc = ks * 2 % CPC;
        fa[slot_] = *reinterpret_cast<const v4i*>(frag + ((tap / KW) * a.row_step + (tap % KW) * a.col_step + cc * 16));
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[slot_][j] = *reinterpret_cast<const v4i*>(w_row + j * 32 * a.kstride + ks * 32);
      };
#pragma unroll
      for (int q = 0; q < RING - 1; ++q)
        if (q < KSTEPS) fetch(q, q);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
        if (ks + RING - 1 < KSTEPS) fetch(ks + RING - 1, (ks + RING - 1) % RING);
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks % RING], fb[ks % RING][j], acc[j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- the next band's rows (loaded one band ago) into the other halo buffer; the loads of the band after it
    // leave now; the sum plane of that band gets its start values ----
    if (has_next) {
      loads_landed(dn);
      store_halo(dn, tn, lds + (buf ? a.off_halo0 : a.off_halo1), sum_plane(sk == 2 ? 0 : sk + 1));
      if (tn + per_xcd < t_end) issue_loads(dn, tn + per_xcd);
      clear_sums(sum_plane(sk == 0 ? 2 : sk - 1));
    }
    // ---- accumulators -> codes. A lane holds four pixels of a channel per accumulator quad; two lane swaps
    // between the wavefront's halves turn four quads into sixteen consecutive pixels.
    if (mine) {
      const v4i* rq_lds = reinterpret_cast<const v4i*>(lds + a.off_rq);
      const int nvalid = min(32, valid - wave * 32);  // a multiple of 8
      uint8_t* ytile = a.y + (static_cast<size_t>(img) * a.OC * hw + static_cast<size_t>(r0) * a.OW + wave * 32);
      v4i s4[4];
      if (ZP) {
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int g = 0; g < 4; ++g) s4[g] = *reinterpret_cast<const v4i*>(sx_lds + 8 * g + 4 * frag_half);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const v4i rq = rq_lds[j * 32 + frag_row];
        const int lo_t = a.lo << rq[1], hi_t = (a.hi << rq[1]) | ((1 << rq[1]) - 1);
        uint32_t quad[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          int v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = ZP ? acc[j][g * 4 + e] - s4[g][e] : acc[j][g * 4 + e];
          if (RQ == kRqFastNoTie) {
            // clamp in front of the shift (bounds shifted up), the shift writes its byte of the dword
            int u[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) u[e] = Med3(__mulhi(v[e], rq[0]) + rq[2], lo_t, hi_t);
            ShiftIntoByte<0>(quad[g], rq[1], u[0]);
            ShiftIntoByte<1>(quad[g], rq[1], u[1]);
            ShiftIntoByte<2>(quad[g], rq[1], u[2]);
            ShiftIntoByte<3>(quad[g], rq[1], u[3]);
          } else {
            int r4[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) r4[e] = Requant8<RQ>(v[e], rq, a.out_zp, a.lo, a.hi);
            quad[g] = PackBytes(r4[0], r4[1], r4[2], r4[3]);
          }
        }
        // quad g of the lower half: pixels 8g .. 8g+3, of the upper half: 8g+4 .. 8g+7. Behind the swaps a lower lane
        // holds pixels 0 .. 15 of its channel, its partner in the upper half pixels 16 .. 31.
        // (the builtin, not inline assembly: the compiler must know that the swap is a cross-lane operation, or it
        // may move it into a divergent region, where the idle lanes' halves stay behind)
        const auto s02 = __builtin_amdgcn_permlane32_swap(quad[0], quad[2], false, false);
        const auto s13 = __builtin_amdgcn_permlane32_swap(quad[1], quad[3], false, false);
        quad[0] = s02[0]; quad[2] = s02[1]; quad[1] = s13[0]; quad[3] = s13[1];
        const int oc = j * 32 + frag_row, h16 = frag_half * 16;
        uint8_t* dst = ytile + static_cast<size_t>(oc) * hw + h16;
        if (oc < a.OC) {
          if (h16 + 16 <= nvalid) *reinterpret_cast<v4i*>(dst) = v4i{static_cast<int>(quad[0]), static_cast<int>(quad[2]), static_cast<int>(quad[1]), static_cast<int>(quad[3])};
          else if (h16 + 8 <= nvalid) *reinterpret_cast<int2*>(dst) = int2{static_cast<int>(quad[0]), static_cast<int>(quad[2])};
        }
      }
    }
    if (has_next) lds_barrier();  // the next band's halo tile and sums are complete; everyone is done reading the present ones
    buf ^= 1;
    sk = sk == 2 ? 0 : sk + 1;
  }
}

struct BandPlan {
  BandArgs a;
  int lds_bytes;
  int kh, kw, cpc, rq;
  bool zp;
  unsigned grid;
};

typedef void (*BandFn)(BandArgs);
template <int KH, int KW, int CPC>
BandFn BandKernelOf(int rq, bool zp) {
  if (rq == kRqFastNoTie) return zp ? ConvBandKernel<KH, KW, CPC, kRqFastNoTie, true> : ConvBandKernel<KH, KW, CPC, kRqFastNoTie, false>;
  return zp ? ConvBandKernel<KH, KW, CPC, kRqFast, true> : ConvBandKernel<KH, KW, CPC, kRqFast, false>;
}
// The kernel exists for 3 x 3 taps over 32 or 64 input channels.
BandFn BandKernel(int kh, int kw, int cpc, int rq, bool zp) {
  if (rq == kRqGeneric || kh != 3 || kw != 3) return nullptr;
  if (cpc == 2) return BandKernelOf<3, 3, 2>(rq, zp);
  if (cpc == 4) return BandKernelOf<3, 3, 4>(rq, zp);
  return nullptr;
}

int ConvBandRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const BandPlan* plan = reinterpret_cast<const BandPlan*>(op->host_blob.data());
  BandArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  if (reinterpret_cast<uintptr_t>(in0) & 3 || reinterpret_cast<uintptr_t>(out) & 7)
    return SetError(TVX_E_INVALID, "conv2d_band_i8: the input must be 4-byte aligned, the output 8-byte aligned");
  hipLaunchKernelGGL(BandKernel(plan->kh, plan->kw, plan->cpc, plan->rq, plan->zp), dim3(plan->grid), dim3(kBandThreads), plan->lds_bytes, st, a);
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
  a.row_step = dh * a.iwt * a.pix_stride; a.col_step = dw * a.pix_stride;
  a.s_row_step = dh * a.iwt; a.s_col_step = dw;
  a.iwt_div = a.iwt;
  if (a.pad_cols < 0) return TVX_E_UNSUPPORTED;

  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127) return TVX_E_UNSUPPORTED;
  a.xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.pad_fill = static_cast<int>(static_cast<uint32_t>(zxs & 0xff) * 0x01010101u);
  a.zws = zws;
  a.out_zp = d->out_zp; a.lo = op->act_lo; a.hi = op->act_hi;
  a.s_pad = a.C * zxs;

  std::vector<int32_t> rqt;
  const int rq = BuildRequantRecords(op->h_mult, op->h_shift, a.OC, 64, d->out_zp, &rqt,
                                     AccumulatorBound(static_cast<uint64_t>(taps) * a.C, bias_host, a.OC));
  BandFn fn = BandKernel(kh, kw, cpc, rq, zws != 0);
  if (!fn) return TVX_E_UNSUPPORTED;

  hipDeviceProp_t prop;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return TVX_E_UNSUPPORTED;
  const int cus = std::max(8, prop.multiProcessorCount / 8 * 8);

  // ---- rows of a band: what the loader (one patch per thread), the wavefronts (one 32-pixel tile each) and LDS
  // allow; among those the choice that needs the fewest rounds of bands, each priced by its halo rows
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
    const int s_bytes = RoundUp(halo_rows * a.iwt * 4, 16);
    if (halo_rows * a.iwt > kBandThreads) break;  // a thread per cell gives the sum planes their start values
    const int lds_bytes = kBandWaves * 128 + 64 * 16 + 64 * 4 + w_bytes + 2 * halo_bytes + 3 * s_bytes;
    if (lds_bytes > 160 * 1024) break;
    const long long tiles = static_cast<long long>(d->batch) * ((a.OH + r - 1) / r);
    const long long cost = (tiles + cus - 1) / cus * (r + 2);  // (a band costs its rows plus the halo's two; equal cost: the shorter band)
    if (best_rows == 0 || cost < best_cost || r == want_rows) { best_rows = r; best_cost = cost; best_lds = lds_bytes; }
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
      !MagicExact(a.gpr, 1024) || !MagicExact(a.gblocks, kBandWaves) || !MagicExact(a.iwt, kBandThreads) ||
      !MagicExact(std::max(a.pad_cols, 1), 2 * kBandThreads))
    return TVX_E_UNSUPPORTED;
  a.tiles_per_xcd = (a.total_tiles + 7) / 8;
  a.magic_iwt = Magic(a.iwt);
  a.magic_padcols = Magic(std::max(a.pad_cols, 1));
  a.magic_tpi = Magic(a.tiles_per_image);
  a.magic_ow = Magic(a.OW);
  a.magic_gpr = Magic(a.gpr);
  a.magic_gblocks = Magic(a.gblocks);
  // the loader's 24-bit multiplies and 32-bit offsets inside one image
  if (static_cast<uint64_t>(a.H) * a.W >= (1ull << 24) || static_cast<uint64_t>(a.H) * a.W * a.C >= (1ull << 31)) return TVX_E_UNSUPPORTED;
  if (a.halo_rows * a.iwt * a.pix_stride >= (1 << 23)) return TVX_E_UNSUPPORTED;

  const int halo_bytes = RoundUp(a.halo_rows * a.iwt * a.pix_stride + 64, 16);
  a.off_sx = 0;
  a.off_rq = kBandWaves * 128;
  a.off_bias = a.off_rq + 64 * 16;
  a.off_w = a.off_bias + 64 * 4;
  a.off_halo0 = a.off_w + w_bytes;
  a.off_halo1 = a.off_halo0 + halo_bytes;
  a.off_s = a.off_halo1 + halo_bytes;
  a.s_bytes = RoundUp(a.halo_rows * a.iwt * 4, 16);
  const int lds_bytes = a.off_s + 3 * a.s_bytes;
  if (lds_bytes != best_lds) return SetError(TVX_E_INVALID, "conv2d_band_i8: LDS plan mismatch (%d, %d)", lds_bytes, best_lds);

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
  plan.kh = kh; plan.kw = kw; plan.cpc = cpc;
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
