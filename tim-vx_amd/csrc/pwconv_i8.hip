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
//     (1 KiB contiguous per wavefront load, prefetched up to four (deep inputs: eight) steps ahead, the
//     first ones of a tile during the previous tile's epilogue); they are small and live in L2.
// Zero points: sum (x - zx)(w - zw) = sum xs ws - zws Sx - zxs Sw + C zxs zws with
// xs, ws the operands moved to the signed int8 domain; the Sx term is one more MFMA
// against a constant fragment, the per-channel constants are folded into the bias.
#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kStageStride = 136;  // bytes per staged output row: 34 dwords spread 32 rows over all banks
constexpr int kStageBytes = 32 * kStageStride;

struct PwArgs {
  const uint8_t* x;
  uint8_t* y;
  const v4i* wpk;        // [oc tile][k-step][lane]: 16 reduction bytes of channel tile*32 + lane%32
  const int32_t* biasf;  // bias + per-channel zero-point terms
  const v4i* rq;         // per channel requantization record
  int C, OC, HW;
  int HWp;               // pixels per image on the flat pixel axis: HW, rounded up to 4 when HW % 4 != 0,
                         // so that a 4-pixel group never straddles two images (the padding pixels are
                         // computed and dropped)
  int Q;                 // batch * HWp (< 2^31 - 256: flat pixel indices are 32-bit)
  int cp;                // channels padded to 32
  int ksteps;            // cp / 32
  int pix_stride;        // LDS bytes per pixel: cp + 16 (an odd number of 16-byte chunks)
  int oc_tiles;          // ceil(OC / 32)
  int tiles_per_wg;      // output tiles one workgroup walks
  int tile_groups;       // workgroups that share a pixel tile (oc_tiles / tiles_per_wg, rounded up)
  int xcd_runs;          // renumber the workgroups so that each XCD gets a contiguous run of them
  int xor_mask;          // 0x80808080 for uint8 activations
  int neg_zws4;          // -(weight zero point, int8 domain) in all four bytes
  int out_zp, lo, hi;
  // Fused residual Add (0 = off): the convolution's quantized output t meets a tensor r of the output's
  // shape on the way out, y = clamp(rne(fma(a - za, ra, (b - zb) * rb)) + zo) in double, exactly the
  // stand-alone Add on the tensor the convolution would have written. add_mode 1: a = t, b = r; 2: a = r, b = t.
  const uint8_t* res;
  double add_ra, add_rb;
  int add_mode, add_signed;
  int add_za, add_zb, add_zo, add_lo, add_hi;
};


// KP: flat pixels per workgroup: 128, or 32 when the whole batch has few pixels and more,
//     smaller workgroups are needed to fill the chip.
// NW: wavefronts per workgroup (1: every wavefront is on its own - shallow inputs whose
//     tile is a few KiB, many tiles in flight per CU; 4: the tile is built cooperatively).
// PT: 32-pixel MFMA tiles per work item; an item is (output tile, 32*PT-pixel part), so
//     that a workgroup with fewer output tiles than wavefronts still keeps all of them busy.
// GRAN: pixels guaranteed to stay inside one image and to be aligned: 16, 4 or 1.
// ZP: the weights have a zero point (int8 domain): its term -zws * sum_c xs is taken by a
//     second MFMA against a constant fragment - the matrix cores idle here anyway.
template <int KP, int NW, int PT, int GRAN, bool ZP, int RQ>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu((PT == 4 && GRAN < 16) ? 3 : 4, (PT == 4 && GRAN < 16) ? 3 : 4))) PwConvKernel(PwArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  constexpr int kThreads = 64 * NW;
  constexpr int kPix = KP;
  constexpr int kParts = KP / (32 * PT);  // pixel parts per output tile
  constexpr int kRowBytes = 32 * PT;  // staged bytes per output row
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = NW == 1 ? 0 : __builtin_amdgcn_readfirstlane(tid >> 6);
  // Workgroups go to the eight XCDs round-robin in launch order and each XCD has its own L2:
  // renumber them so that an XCD gets a contiguous run of (pixel tile, output-tile group) pairs,
  // pixel tiles in order and the groups of one pixel tile next to each other. A 32-pixel row
  // segment is a quarter of a cache line and neighbouring pixel tiles take the other quarters;
  // spread over four XCDs, every line would cross the fabric four times.
  int wg = blockIdx.x;
  if (a.xcd_runs) {
    const int per = gridDim.x >> 3, rem = gridDim.x & 7, xcd = wg & 7;
    wg = xcd * per + min(xcd, rem) + (wg >> 3);
  }
  const int pix_tile = static_cast<int>(static_cast<uint32_t>(wg) / static_cast<uint32_t>(a.tile_groups));
  const int tile_group = wg - pix_tile * a.tile_groups;
  const int q_base = pix_tile * kPix;
  int8_t* xl = lds;
  int8_t* stage = lds + kPix * a.pix_stride + wave * kStageBytes;

  // ---- work items of this wavefront: (output tile, pixel part) ---------------------------
  const int t_begin = tile_group * a.tiles_per_wg;
  const int t_end = min(t_begin + a.tiles_per_wg, a.oc_tiles);
  // wavefront w takes items w, w + NW, ...; with kParts | NW its pixel part never changes
  const int part = wave % kParts;
  constexpr int tile_step = NW / kParts > 0 ? NW / kParts : 1;
  const int tile0 = t_begin + wave / kParts;
  const int n_tiles = tile0 < t_end ? (t_end - tile0 + tile_step - 1) / tile_step : 0;

  // Weight fragments stream global -> registers four k-steps ahead. The first four of a tile
  // are requested before the previous tile's epilogue (for the first tile: before the input
  // tile is built), so their latency hides behind work that does not need them.
  auto frag_ptr = [&](int t, int k) { return a.wpk + (static_cast<size_t>(t) * a.ksteps + k) * 64 + lane; };
  constexpr int kRing = PT == 4 ? 2 : ((KP == 32 && NW == 4) ? 8 : 4);  // fragments in flight; four pixel tiles leave room for two, deep inputs (the 32-pixel, four-wavefront shape) take eight
  v4i nf[kRing];
#pragma unroll
  for (int j = 0; j < kRing; ++j) nf[j] = *frag_ptr(n_tiles > 0 ? tile0 : 0, min(j, a.ksteps - 1));
  // The folded bias and the requantization record of a tile travel with its first fragments: asked
  // for inside a tile's own computation they would each be a round trip that also waits for the
  // previous tile's stores (loads and stores complete in issue order).
  int nb = a.biasf[(n_tiles > 0 ? tile0 : 0) * 32 + (lane & 31)];
  v4i nq = a.rq[(n_tiles > 0 ? tile0 : 0) * 32 + (lane & 31)];

  // ---- activations of the 128 pixels, all channels: global (pixel-innermost) -> LDS
  {
    // A thread takes a group of 4 consecutive flat pixels and 16 channels per pass: 16 dword
    // loads in flight, 4x4 byte transposes, four 16-byte LDS stores.
    constexpr int kQuads = KP / 4;
    const int pq = tid % kQuads, cg0 = tid / kQuads;  // 4-pixel group, first 16-channel group
    const int q0 = q_base + pq * 4;
    const bool live = q0 < a.Q;
    const int n = live ? static_cast<int>(static_cast<uint32_t>(q0) / static_cast<uint32_t>(a.HWp)) : 0;
    const int p = live ? static_cast<int>(q0 - n * a.HWp) : 0;
    // GRAN 1: the last group of an image holds fewer than four of its pixels
    const bool whole = GRAN >= 4 ? live : (live && p + 3 < a.HW);
    const uint8_t* src = a.x + (static_cast<size_t>(n) * a.C) * a.HW + p;
    // Every load below is unconditional - a load under a per-lane condition becomes a branch
    // and a full wait, sixteen round trips instead of one: lanes and channels with nothing to
    // fetch read a valid address (channel clamped, src at the tensor base) and are masked.
    // With GRAN 1 a group may start at any byte (the dword loads are then unaligned, which
    // global memory allows), and the dword of an image's last group reaches past the end of its
    // row into the next row of the tensor; only behind the very last row there is nothing:
    // there the dword is fetched 4 - k bytes early and shifted down.
    const bool last_row_tail = GRAN == 1 && live && !whole && static_cast<long long>(n + 1) * a.HWp >= a.Q;
    const int back = last_row_tail ? 4 - (a.HW - p) : 0;
    // lanes with nothing to fetch stay on the first dword of the tensor: with images of fewer than
    // four pixels a dword at a later row of the first image could end behind a one-image tensor
    const size_t row_stride = (GRAN == 1 && !live) ? 0 : static_cast<size_t>(a.HW);
    for (int cg = cg0; cg < a.cp / 16; cg += kThreads / kQuads) {
      uint32_t raw[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int c = cg * 16 + j;
        const uint8_t* row = src + static_cast<size_t>(min(c, a.C - 1)) * row_stride;
        if (GRAN >= 4) {
          raw[j] = *reinterpret_cast<const uint32_t*>(row);
        } else {
          const int bk = c >= a.C - 1 ? back : 0;  // padding channels re-read the last one
          __builtin_memcpy(&raw[j], row - bk, 4);
        }
      }
      // all sixteen loads are issued before the first one is used: left to itself the scheduler
      // sometimes pairs every load with its use, sixteen round trips instead of one
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int c = cg * 16 + j;
        uint32_t v = raw[j];
        if (GRAN == 1) v >>= 8 * (c >= a.C - 1 ? back : 0);
        raw[j] = (live && c < a.C) ? v ^ a.xor_mask : 0u;
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
  }

  if (NW > 1) __syncthreads();  // the input tile is complete; nothing below needs the other wavefronts
  if (n_tiles <= 0) return;

  // ---- where this lane's output groups live (the same for every output tile) -----
  // Copy-out mapping of a staged row of kRowBytes pixels: GRAN 16: lane -> 16-pixel chunk
  // lane % (kRowBytes/16); GRAN 4 and 1: 4-pixel group lane % (kRowBytes/4), which with
  // GRAN 1 may be unaligned or an image's short last group (then stored byte by byte).
  constexpr int kUnit = GRAN == 16 ? 16 : 4;
  constexpr int kPerRow = kRowBytes / kUnit;
  constexpr int kRowsPerIter = 64 / kPerRow;
  const int px_in_row = (lane % kPerRow) * kUnit;
  const int oq0 = q_base + part * kRowBytes + px_in_row;
  const bool out_live = oq0 < a.Q;
  const int on = out_live ? static_cast<int>(static_cast<uint32_t>(oq0) / static_cast<uint32_t>(a.HWp)) : 0;
  const int op0 = out_live ? static_cast<int>(oq0 - on * a.HWp) : 0;
  const size_t out_off = static_cast<size_t>(on) * a.OC * a.HW + static_cast<size_t>(op0);
  const bool out_whole = GRAN >= 4 ? out_live : (out_live && op0 + 3 < a.HW);
  size_t out_px_off[4] = {0, 0, 0, 0};
  bool out_px_live[4] = {false, false, false, false};
  if (GRAN == 1 && out_live && !out_whole) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      out_px_live[e] = op0 + e < a.HW;
      out_px_off[e] = out_off + e;
    }
  }

  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int8_t* xa = xl + (part * kRowBytes + frag_row) * a.pix_stride + frag_half * 16;
  v16i acc[PT];
  // The zero-point term -zws * sum_c xs is the same for every output channel of a pixel. With
  // at most two pixel tiles per item it gets accumulators of its own, filled while the first
  // output tile is computed (an independent MFMA chain) and added to every tile's result.
  constexpr bool kSplitZp = ZP && PT <= 2;
  v16i accz[kSplitZp ? PT : 1];
  if (kSplitZp) {
#pragma unroll
    for (int i = 0; i < PT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) accz[i][r] = 0;
  }
  int tile = tile0;
  v4i q;
  auto init_acc = [&]() {
    const int b = nb;
    q = nq;
#pragma unroll
    for (int i = 0; i < PT; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][r] = b;
  };
  const v4i fz = {a.neg_zws4, a.neg_zws4, a.neg_zws4, a.neg_zws4};

  auto epilogue = [&]() {
    // Fused Add: the other operand's bytes for this lane's output groups are fetched first, so that
    // the requantization below runs while they travel (a load next to the store that uses it would be
    // a round trip per copy-out iteration: the compiler cannot move it above earlier stores).
    constexpr int kIters = 32 / kRowsPerIter;
    uint4 res16[GRAN == 16 ? kIters : 1];
    uint32_t res4[GRAN == 16 ? 1 : kIters];
    if (a.add_mode) {
      const int rows_live = min(32, a.OC - tile * 32);
#pragma unroll
      for (int i = 0; i < kIters; ++i) {
        const int row = lane / kPerRow + kRowsPerIter * i;
        const size_t at = static_cast<size_t>(tile) * 32 * a.HW + out_off + static_cast<size_t>(row) * a.HW;
        if (GRAN == 16) {
          res16[i] = make_uint4(0, 0, 0, 0);
          if (row < rows_live && out_live) res16[i] = *reinterpret_cast<const uint4*>(a.res + at);
        } else {
          res4[i] = 0;
          if (row < rows_live && out_whole) {
            if (GRAN == 4) res4[i] = *reinterpret_cast<const uint32_t*>(a.res + at);
            else __builtin_memcpy(&res4[i], a.res + at, 4);
          }
        }
      }
    }
    const int lo = a.lo, hi = a.hi;
#pragma unroll
    for (int i = 0; i < PT; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int pl = i * 32 + 8 * g + 4 * frag_half;
        int v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][g * 4 + e] + (kSplitZp ? accz[i][g * 4 + e] : 0);
        *reinterpret_cast<uint32_t*>(stage + frag_row * kStageStride + pl) = RequantPack4<RQ>(v, q, a.out_zp, lo, hi);
      }
    __builtin_amdgcn_wave_barrier();
    // copy-out: rows of the staging patch -> WHCN output
    const int rows = min(32, a.OC - tile * 32);
    if (GRAN == 16) {
#pragma unroll
      for (int i = 0; i < 32 / kRowsPerIter; ++i) {
        const int row = lane / kPerRow + kRowsPerIter * i;
        const int8_t* s = stage + row * kStageStride + px_in_row;
        const uint2 lo8 = *reinterpret_cast<const uint2*>(s);
        const uint2 hi8 = *reinterpret_cast<const uint2*>(s + 8);
        if (row < rows && out_live) {
          uint4 o = make_uint4(lo8.x, lo8.y, hi8.x, hi8.y);
          const size_t at = static_cast<size_t>(tile) * 32 * a.HW + out_off + static_cast<size_t>(row) * a.HW;
          if (a.add_mode) {
            const uint4 r = res16[i];
            o = make_uint4(AddResidual4(a, o.x, r.x), AddResidual4(a, o.y, r.y), AddResidual4(a, o.z, r.z),
                           AddResidual4(a, o.w, r.w));
          }
          *reinterpret_cast<uint4*>(a.y + at) = o;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 32 / kRowsPerIter; ++i) {
        const int row = lane / kPerRow + kRowsPerIter * i;
        uint32_t v = *reinterpret_cast<const uint32_t*>(stage + row * kStageStride + px_in_row);
        const size_t row_at = static_cast<size_t>(tile) * 32 * a.HW + static_cast<size_t>(row) * a.HW;
        if (row < rows && out_whole) {
          uint8_t* o = a.y + row_at + out_off;
          if (a.add_mode) v = AddResidual4(a, v, res4[i]);
          if (GRAN == 4) *reinterpret_cast<uint32_t*>(o) = v;
          else __builtin_memcpy(o, &v, 4);
        } else if (GRAN == 1 && row < rows) {
          if (a.add_mode) {
            uint32_t r = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (out_px_live[e]) r |= static_cast<uint32_t>(a.res[row_at + out_px_off[e]]) << (8 * e);
            v = AddResidual4(a, v, r);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (out_px_live[e]) a.y[row_at + out_px_off[e]] = static_cast<uint8_t>(v >> (8 * e));
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  };

  auto step = [&](const v4i& fw, int ks, bool first_tile) {
    v4i fx[PT];
#pragma unroll
    for (int i = 0; i < PT; ++i)
      fx[i] = *reinterpret_cast<const v4i*>(xa + i * 32 * a.pix_stride + ks * 32);
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx[i], fw, acc[i], 0, 0, 0);
      if (kSplitZp) {
        if (first_tile) accz[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx[i], fz, accz[i], 0, 0, 0);
      } else if (ZP) {
        acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx[i], fz, acc[i], 0, 0, 0);
      }
    }
  };

  for (int ti = 0; ti < n_tiles; ++ti, tile += tile_step) {
    init_acc();
    v4i ring[kRing];
#pragma unroll
    for (int j = 0; j < kRing; ++j) ring[j] = nf[j];
    for (int k0 = 0; k0 < a.ksteps; k0 += kRing) {
#pragma unroll
      for (int j = 0; j < kRing; ++j) {
        if (k0 + j < a.ksteps) {
          const v4i g = ring[j];
          if (k0 + j + kRing < a.ksteps) ring[j] = *frag_ptr(tile, k0 + j + kRing);
          step(g, k0 + j, ti == 0);
        }
      }
    }
    const int next_tile = tile + tile_step < t_end ? tile + tile_step : tile;
#pragma unroll
    for (int j = 0; j < kRing; ++j) nf[j] = *frag_ptr(next_tile, min(j, a.ksteps - 1));
    nb = a.biasf[next_tile * 32 + frag_row];
    nq = a.rq[next_tile * 32 + frag_row];
    epilogue();
  }
}


// ---- shallow inputs (at most 32 channels), large pixel counts: one wavefront streams pixel tiles ----------------
// The general kernel gives every 128-pixel tile a wavefront of its own, and with a few thousand tiles all of them are
// resident at once: the whole launch loads, then computes, then stores, and memory idles while the vector units work.
// Here a wavefront walks several pixel tiles; the sixteen dwords of its next tile are requested before the present
// tile is multiplied and requantized, so that loads, vector work and stores of different tiles overlap. With one
// k-step per output tile the operand fragments of a pixel tile are read from LDS once and kept for all output tiles.
// Pixel groups of sixteen stay inside one image (HW % 16 == 0), no fused Add.
constexpr int kStreamPix = 128;
template <bool ZP, int RQ>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 2))) PwStreamKernel(PwArgs a) {
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int lane = threadIdx.x;
  int8_t* xl = lds;                                 // [128 pixels][pix_stride]
  int8_t* stage = lds + kStreamPix * a.pix_stride;  // [32 channels][kStageStride]
  const int n_pix_tiles = (a.Q + kStreamPix - 1) / kStreamPix;
  // an XCD gets a contiguous run of pixel tiles (the grid is a multiple of eight workgroups)
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const int t_first = static_cast<int>(static_cast<long long>(n_pix_tiles) * xcd / 8);
  const int t_end = static_cast<int>(static_cast<long long>(n_pix_tiles) * (xcd + 1) / 8);
  int pt = t_first + slot;
  if (pt >= t_end) return;

  const int pq = lane & 31, cg = lane >> 5;  // this lane's 4-pixel group and 16-channel group of the input tile
  const uint32_t hw = static_cast<uint32_t>(a.HW);
  const uint32_t last_row = static_cast<uint32_t>(a.C - 1) * hw;
  auto request = [&](int tile, uint32_t (&raw)[16]) {
    const int q0 = tile * kStreamPix + pq * 4;
    const bool live = q0 < a.Q;
    const uint32_t n = live ? static_cast<uint32_t>(q0) / hw : 0u;
    const uint32_t p = live ? static_cast<uint32_t>(q0) - n * hw : 0u;
    const uint32_t at0 = n * static_cast<uint32_t>(a.C) * hw + p;
#pragma unroll
    for (int j = 0; j < 16; ++j)  // channel min(c, C - 1); unconditional loads, masked when they are used
      raw[j] = *reinterpret_cast<const uint32_t*>(a.x + (at0 + min(static_cast<uint32_t>(cg * 16 + j) * hw, last_row)));
  };
  auto commit = [&](int tile, uint32_t (&raw)[16]) {
    const bool live = tile * kStreamPix + pq * 4 < a.Q;
#pragma unroll
    for (int j = 0; j < 16; ++j) raw[j] = (live && cg * 16 + j < a.C) ? raw[j] ^ a.xor_mask : 0u;
    uint32_t t[4][4];
#pragma unroll
    for (int b = 0; b < 4; ++b) Transpose4x4(raw + 4 * b, t[b]);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const v4i v = {static_cast<int>(t[0][e]), static_cast<int>(t[1][e]), static_cast<int>(t[2][e]), static_cast<int>(t[3][e])};
      *reinterpret_cast<v4i*>(xl + (pq * 4 + e) * a.pix_stride + cg * 16) = v;
    }
  };

  const int frag_row = lane & 31, frag_half = lane >> 5;
  const int px_in_row = (lane & 7) * 16, row0 = lane >> 3;  // copy-out: 16-pixel chunk lane % 8 of staged rows lane / 8 + 8 i
  const v4i fz = {a.neg_zws4, a.neg_zws4, a.neg_zws4, a.neg_zws4};
  const int lo = a.lo, hi = a.hi;

  uint32_t raw[16];
  request(pt, raw);
  // the first output tile's weights and tables travel with the first rows
  v4i nf = a.wpk[lane];
  int nb = a.biasf[frag_row];
  v4i nq = a.rq[frag_row];
  for (; pt < t_end; pt += per_xcd) {
    commit(pt, raw);
    const int next_pt = pt + per_xcd;
    if (next_pt < t_end) request(next_pt, raw);  // in flight until the next round's commit
    __builtin_amdgcn_wave_barrier();
    v4i fx[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      fx[i] = *reinterpret_cast<const v4i*>(xl + (i * 32 + frag_row) * a.pix_stride + frag_half * 16);
    // where this lane's output chunks live
    const int oq0 = pt * kStreamPix + px_in_row;
    const bool out_live = oq0 < a.Q;
    const uint32_t on = out_live ? static_cast<uint32_t>(oq0) / hw : 0u;
    const uint32_t op0 = out_live ? static_cast<uint32_t>(oq0) - on * hw : 0u;
    const size_t out_off = static_cast<size_t>(on) * a.OC * a.HW + op0;
    for (int tile = 0; tile < a.oc_tiles; ++tile) {
      const v4i fw = nf, q = nq;
      v16i acc[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = nb;
      const int next_tile = tile + 1 < a.oc_tiles ? tile + 1 : 0;  // (the next pixel tile starts at output tile 0 again)
      nf = a.wpk[next_tile * 64 + lane];
      nb = a.biasf[next_tile * 32 + frag_row];
      nq = a.rq[next_tile * 32 + frag_row];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx[i], fw, acc[i], 0, 0, 0);
        if (ZP) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fx[i], fz, acc[i], 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int v[4] = {acc[i][g * 4], acc[i][g * 4 + 1], acc[i][g * 4 + 2], acc[i][g * 4 + 3]};
          *reinterpret_cast<uint32_t*>(stage + frag_row * kStageStride + i * 32 + 8 * g + 4 * frag_half) = RequantPack4<RQ>(v, q, a.out_zp, lo, hi);
        }
      __builtin_amdgcn_wave_barrier();
      const int rows = min(32, a.OC - tile * 32);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = row0 + 8 * i;
        const int8_t* sp = stage + row * kStageStride + px_in_row;
        const uint2 lo8 = *reinterpret_cast<const uint2*>(sp);
        const uint2 hi8 = *reinterpret_cast<const uint2*>(sp + 8);
        if (row < rows && out_live)
          *reinterpret_cast<uint4*>(a.y + (out_off + (static_cast<size_t>(tile) * 32 + row) * a.HW)) = make_uint4(lo8.x, lo8.y, hi8.x, hi8.y);
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

struct Plan {
  PwArgs a;
  int lds_bytes, kp, nw, pt, gran, zp, rq;
  dim3 grid;
  int stream_wgs;  // > 0: PwStreamKernel with that many workgroups
};

template <int KP, int NW, int PT, int GRAN, bool ZP, int RQ>
int Launch(const Plan* plan, const PwArgs& a, hipStream_t st, bool configure) {
  if (configure) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&PwConvKernel<KP, NW, PT, GRAN, ZP, RQ>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, plan->lds_bytes);
    if (e != hipSuccess)
      return SetError(TVX_E_DEVICE, "hipFuncSetAttribute(dynamic LDS %d): %s", plan->lds_bytes, hipGetErrorString(e));
    return TVX_OK;
  }
  hipLaunchKernelGGL((PwConvKernel<KP, NW, PT, GRAN, ZP, RQ>), plan->grid, dim3(64 * NW), plan->lds_bytes, st, a);
  return TVX_OK;
}

template <int KP, int NW, int PT, int GRAN, bool ZP>
int DispatchRq(const Plan* plan, const PwArgs& a, hipStream_t st, bool configure) {
  if (plan->rq == kRqFastNoTie) return Launch<KP, NW, PT, GRAN, ZP, kRqFastNoTie>(plan, a, st, configure);
  if (plan->rq == kRqFast) return Launch<KP, NW, PT, GRAN, ZP, kRqFast>(plan, a, st, configure);
  return Launch<KP, NW, PT, GRAN, ZP, kRqGeneric>(plan, a, st, configure);
}

template <int KP, int NW, int PT, int GRAN>
int DispatchZp(const Plan* plan, const PwArgs& a, hipStream_t st, bool configure) {
  return plan->zp ? DispatchRq<KP, NW, PT, GRAN, true>(plan, a, st, configure)
                  : DispatchRq<KP, NW, PT, GRAN, false>(plan, a, st, configure);
}

template <int KP, int NW, int PT>
int DispatchGran(const Plan* plan, const PwArgs& a, hipStream_t st, bool configure) {
  if (plan->gran == 16) return DispatchZp<KP, NW, PT, 16>(plan, a, st, configure);
  if (plan->gran == 4) return DispatchZp<KP, NW, PT, 4>(plan, a, st, configure);
  return DispatchZp<KP, NW, PT, 1>(plan, a, st, configure);
}

template <bool ZP>
int LaunchStream(const Plan* plan, const PwArgs& a, hipStream_t st) {
  const dim3 grid(plan->stream_wgs), block(64);
  const int lds = kStreamPix * a.pix_stride + kStageBytes;
  if (plan->rq == kRqFastNoTie) hipLaunchKernelGGL((PwStreamKernel<ZP, kRqFastNoTie>), grid, block, lds, st, a);
  else if (plan->rq == kRqFast) hipLaunchKernelGGL((PwStreamKernel<ZP, kRqFast>), grid, block, lds, st, a);
  else hipLaunchKernelGGL((PwStreamKernel<ZP, kRqGeneric>), grid, block, lds, st, a);
  return TVX_OK;
}

int Dispatch(const Plan* plan, const PwArgs& a, hipStream_t st, bool configure) {
  if (plan->stream_wgs > 0) {
    if (configure) return TVX_OK;  // (a few KiB of LDS: no attribute to set)
    return plan->zp ? LaunchStream<true>(plan, a, st) : LaunchStream<false>(plan, a, st);
  }
  if (plan->kp == 32) {
    if (plan->nw == 1) return DispatchGran<32, 1, 1>(plan, a, st, configure);
    return DispatchGran<32, 4, 1>(plan, a, st, configure);
  }
  if (plan->nw == 1) return DispatchGran<128, 1, 4>(plan, a, st, configure);
  if (plan->pt == 4) return DispatchGran<128, 4, 4>(plan, a, st, configure);
  if (plan->pt == 2) return DispatchGran<128, 4, 2>(plan, a, st, configure);
  return DispatchGran<128, 4, 1>(plan, a, st, configure);
}

int PwConvRun(tvx_op* op, const void* in0, const void* in1, void* out, hipStream_t st) {
  const Plan* plan = reinterpret_cast<const Plan*>(op->host_blob.data());
  PwArgs a = plan->a;
  a.x = static_cast<const uint8_t*>(in0);
  a.y = static_cast<uint8_t*>(out);
  a.res = static_cast<const uint8_t*>(in1);
  if (a.add_mode && !in1) return SetError(TVX_E_INVALID, "pwconv_i8: the fused Add needs its second operand as in1");
  if ((reinterpret_cast<uintptr_t>(in0) | reinterpret_cast<uintptr_t>(out) | (a.add_mode ? reinterpret_cast<uintptr_t>(in1) : 0)) & (plan->gran - 1))
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
  if (!op->quantized || !w_host || d->multiplier != 0 || d->groups > 1) return TVX_E_UNSUPPORTED;
  if (d->k_w != 1 || d->k_h != 1 || d->stride_w != 1 || d->stride_h != 1 || d->pad_left != 0 ||
      d->pad_top != 0 || d->out_w != d->in_w || d->out_h != d->in_h)
    return TVX_E_UNSUPPORTED;
  PwArgs a{};
  a.C = d->in_c;
  a.OC = d->out_c;
  const uint64_t hw = static_cast<uint64_t>(d->in_w) * d->in_h;
  if (hw >= (1ull << 30) || hw * d->in_c * d->batch < 4) return TVX_E_UNSUPPORTED;  // the input is read as dwords
  a.HW = static_cast<int>(hw);
  const uint64_t hwp = (hw + 3) / 4 * 4;
  a.HWp = static_cast<int>(hwp);
  if (hwp * d->batch >= (1ull << 31) - 256) return TVX_E_UNSUPPORTED;
  a.Q = static_cast<int>(hwp * d->batch);
  a.cp = RoundUp(a.C, 32);
  a.ksteps = a.cp / 32;
  a.pix_stride = a.cp + 16;
  a.oc_tiles = (a.OC + 31) / 32;
  // few pixels in the whole batch: 32-pixel workgroups, four times as many
  int kp = a.Q < 128 * 1024 ? 32 : 128;
  // a shallow input (a single wavefront loads its tile in one pass, or two of a 128-pixel tile): one
  // wavefront per workgroup, no barrier, many tiles in flight per CU
  int nw = a.cp / 16 <= (kp == 128 ? 4 : 8) ? 1 : 4;
  if (const char* f = getenv("TVX_PWCONV_SHAPE")) {  // tuning aid: "<pixels per workgroup>,<wavefronts>"
    int fk = 0, fn = 0;
    if (sscanf(f, "%d,%d", &fk, &fn) == 2 && (fk == 32 || fk == 128) && (fn == 1 || fn == 4)) { kp = fk; nw = fn; }
  }
  const int lds_bytes = kp * a.pix_stride + nw * kStageBytes;
  if (lds_bytes > 160 * 1024) return TVX_E_UNSUPPORTED;
  const long long gx = (static_cast<long long>(a.Q) + kp - 1) / kp;
  if (gx > 0x7fffffffll) return TVX_E_UNSUPPORTED;
  const bool x_u8 = d->in_dtype == TVX_U8, w_u8 = d->w_dtype == TVX_U8;
  const int zxs = d->in_zp - (x_u8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  if (zxs < -128 || zxs > 127) return TVX_E_UNSUPPORTED;  // zero point outside the tensor's range
  if (zws < -127 || zws > 127) return TVX_E_UNSUPPORTED;  // -zws must be an int8
  a.xor_mask = x_u8 ? static_cast<int>(0x80808080u) : 0;
  a.neg_zws4 = static_cast<int>(static_cast<uint32_t>((-zws) & 0xff) * 0x01010101u);
  a.out_zp = d->out_zp;
  a.lo = op->act_lo;
  a.hi = op->act_hi;
  if (op->fused_add) {
    const tvx_eltwise_desc& e = op->elt;  // a_* / b_* are the Add's first / second operand
    const double ra = static_cast<double>(e.a_scale) / static_cast<double>(e.out_scale);
    const double rb = static_cast<double>(e.b_scale) / static_cast<double>(e.out_scale);
    // as for the stand-alone 16-element Add: the sum must stay far below 2^31 for the 32-bit conversion
    if (!(ra < 1048576.0) || !(rb < 1048576.0)) return TVX_E_UNSUPPORTED;
    a.add_mode = op->fused_add;
    a.add_signed = d->out_dtype == TVX_I8;
    a.add_ra = ra;
    a.add_rb = rb;
    a.add_za = e.a_zp;
    a.add_zb = e.b_zp;
    a.add_zo = e.out_zp;
    ActRange(d->out_dtype, e.out_scale, e.out_zp, TVX_ACT_NONE, &a.add_lo, &a.add_hi);
  }
  // few pixel tiles: spread the output tiles over grid.y (in units of one tile per
  // wavefront) until the launch has a few workgroups per CU
  const int quads = (a.oc_tiles + nw - 1) / nw;
  // enough workgroups to give every SIMD several wavefronts; re-reading the small input
  // tile per output-tile group is cheap next to walking many output tiles in sequence
  long long want_wgs = nw == 1 ? 4096 : 2048;
  if (const char* f = getenv("TVX_PWCONV_WGS")) want_wgs = std::max(1, atoi(f));  // tuning aid
  int gy = static_cast<int>(std::min<long long>(quads, std::max<long long>(1, want_wgs / gx)));
  a.tiles_per_wg = std::min(((quads + gy - 1) / gy) * nw, a.oc_tiles);
  gy = (a.oc_tiles + a.tiles_per_wg - 1) / a.tiles_per_wg;
  a.tile_groups = gy;
  // pixel tiles that are whole cache lines of every channel row and have a single workgroup each
  // share nothing: they keep the launch order, which spreads the stream over all memory channels
  a.xcd_runs = (kp % 128 != 0 || a.HW % 128 != 0 || gy > 1) ? 1 : 0;
  if (const char* f = getenv("TVX_PWCONV_XCD_RUNS")) a.xcd_runs = atoi(f) != 0;  // tuning aid
  if (gx * gy > 0x7fffffffll) return TVX_E_UNSUPPORTED;
  // fewer output tiles than wavefronts: split the pixels of a tile over wavefronts instead
  const int pt = kp == 32 ? 1 : (nw == 1 ? 4 : (a.tiles_per_wg >= 4 ? 4 : (a.tiles_per_wg >= 2 ? 2 : 1)));

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
  const int rq = BuildRequantRecords(op->h_mult, op->h_shift, a.OC, oc_alloc, d->out_zp, &rqt,
                                     AccumulatorBound(a.C, bias_host, a.OC));
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
  plan.kp = kp;
  plan.nw = nw;
  plan.pt = pt;
  plan.gran = (a.HW % 16 == 0) ? 16 : ((a.HW % 4 == 0) ? 4 : 1);
  plan.zp = zws != 0;
  plan.rq = rq;
  plan.grid = dim3(static_cast<unsigned>(gx * gy));
  // Shallow inputs with thousands of pixel tiles: wavefronts that stream several tiles each (see PwStreamKernel).
  plan.stream_wgs = 0;
  {
    const long long pix_tiles = (static_cast<long long>(a.Q) + kStreamPix - 1) / kStreamPix;
    // two tiles per wavefront once that still leaves two wavefronts per SIMD; below that one tile each (the form's
    // leaner per-tile code is then what it has to offer; from 1024 tiles up it measures faster than the general kernel)
    int tiles_per_wave = pix_tiles >= 4096 ? 2 : 1;
    if (const char* f = getenv("TVX_PWCONV_STREAM")) tiles_per_wave = atoi(f);  // tuning aid: pixel tiles per wavefront, 0 = off
    long long min_tiles = 1024;
    if (const char* f = getenv("TVX_PWCONV_STREAM_MIN_TILES")) min_tiles = atoll(f);  // tuning / test aid
    if (tiles_per_wave > 0 && !op->fused_add && a.cp == 32 && plan.gran == 16 && kp == 128 && nw == 1 && pix_tiles >= min_tiles &&
        hw * d->in_c * d->batch < (1ull << 32) - 16) {
      const long long wgs = (pix_tiles + tiles_per_wave - 1) / tiles_per_wave;
      plan.stream_wgs = static_cast<int>(std::min<long long>((wgs + 7) / 8 * 8, 1 << 20));
    }
  }
  s = Dispatch(&plan, a, nullptr, true);
  if (s != TVX_OK) return s;
  op->host_blob.assign(reinterpret_cast<const uint8_t*>(&plan), reinterpret_cast<const uint8_t*>(&plan) + sizeof(plan));
  op->run = PwConvRun;
  op->kernel_name = op->fused_add ? "pwconv_add_i8" : (plan.stream_wgs > 0 ? "pwconv_i8_stream" : "pwconv_i8");
  return TVX_OK;
}

}  // namespace tvx
