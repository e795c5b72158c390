// FullyConnected on the int8 matrix cores: out[m][n] = requant(sum_k x[m][k] w[n][k] ...).
// Both operands are K-contiguous (an "NT" GEMM), which is exactly the operand
// shape v_mfma_i32_32x32x32_i8 wants: every lane feeds 16 consecutive K bytes.
//
// Tiling: one 256-thread workgroup (4 wavefronts) owns a TM x TN = 256 x 256 output tile
// and walks K in steps of 128 bytes; wavefront w accumulates all 256 activation rows
// against features [64 w, 64 w + 64) as 2 x 8 MFMA tiles (256 accumulator registers per
// lane). The two operands take different roads. Activation tiles go global -> LDS by DMA
// (no registers), four stages of 32 KiB; rows are 128 B in LDS and their 16 B chunks are
// XOR-swizzled with the row number so that the 32 lanes of a fragment read hit 8 different
// bank groups. The constant weights are packed at creation in MFMA-fragment order and go
// global -> registers, three k-tiles deep, never through LDS: no wavefront needs another
// one's weight fragments. Both prefetches run three k-tiles ahead, their instructions
// spread evenly between the MFMAs (one every fourth). Measured on the 8192 x 4096 x 4096
// layer: the k-loop takes the same time with and without the operand feed (it is bound by
// the matrix cores, whose clock drops under random data, plus ~10 % for the barrier per
// k-tile); prologue and epilogue of a tile cost ~9 us next to ~60 us of k-loop.
//
// The quantized variants also have a 128 x 256 form (MB = 4 activation blocks instead of 8): half
// the accumulators and two weight slots instead of three fit two wavefronts per SIMD, i.e. two
// workgroups per CU, so that one tile's prologue, barriers, in-place pass and epilogue run under
// the other's MFMAs. It is taken when there are 1024 such tiles and more.
//
// The MFMA "A" operand is the weight fragment and "B" the activation fragment,
// so a lane ends up with one activation row m and, per accumulator quad, four
// consecutive features n: four requantized bytes make one dword of the row-major
// output, and the per-row correction term of the zero-point expansion
//   sum (x - zx)(w - zw) = sum xs ws - zws * sum_k xs - zxs * sum_k ws + K zxs zws
// (xs = x - 128 for uint8, zxs likewise) is per lane, with no exchange needed.
// The per-feature terms are folded into the bias at creation.
//
// The float16 variant is the same kernel with the other matrix instruction:
// v_mfma_f32_32x32x16_f16 also takes 16 operand bytes per lane (8 halves) and the
// two lane halves also cover 32 bytes of a row, so tiles, DMA, swizzle and fragment
// addresses are identical with K counted in bytes; accumulation is fp32, the
// epilogue adds the fp32 bias, clamps for ReLU / ReLU6 and rounds to float16.
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "variants.h"

namespace tvx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int TN = 256, TK = 128;
constexpr int kThreads = 256;
constexpr int kStages = 4;                      // activation tiles in LDS (a power of two)
// The tile's geometry by its count MB of 32-row activation blocks: 8 (256 rows, one workgroup per CU, three weight
// slots) or 4 (128 rows, two workgroups per CU whose prologues, barriers and epilogues hide behind each other's
// MFMAs, two weight slots: half the registers per wavefront).
template <int MB>
struct Geo {
  static constexpr int TM = MB * 32;
  static constexpr int kSlots = MB == 8 ? 3 : 2;            // k-tiles of weight fragments resident in registers = prefetch distance
  static constexpr int kOps = MB + 8;                        // memory operations a wavefront issues per k-tile (DMA pieces + weight fragments)
  static constexpr int kTileBytes = TM * TK;                 // per activation tile: 32 / 16 KiB
  static constexpr int kTabOffset = kStages * kTileBytes;    // behind the stages: the tile's epilogue tables
  static constexpr int kRowsumOffset = kTabOffset + TN * 4 + TN * 16;  // behind the folded bias (or fp32 bias) and the requantization records
  static constexpr int kLdsBytes = kRowsumOffset + TM * 4;   // the activation rows' sums, exchanged between the wavefronts
};
// k-tiles of the packed weights: whole rounds of the kernel's weight slots
__host__ __device__ constexpr int k_tiles_padded(int k_bytes, int slots) { return ((k_bytes + TK - 1) / TK + slots - 1) / slots * slots; }
constexpr int kOutStride = TN + 16;             // epilogue staging row stride (bytes)

struct FcArgs {
  const int8_t* x;      // [M][K] (uint8 is re-biased to int8 on the fly)
  const int8_t* w;      // [N][K] int8 (uint8 weights are re-biased when packed)
  int8_t* y;            // [M][N]
  const int32_t* biasf; // [N] bias + per-feature zero-point terms
  const tvx_v4i* rq;    // [N padded to the tile] requantization records
  const int8_t* zeros;  // 128 x 0x00 then 128 x 0x80: source of reduction chunks past K
  int M, N, K;          // K in bytes of a row (float16: twice the element count)
  const float* biasf32; // float16 variant: [N padded to the tile] fp32 bias
  float flo, fhi;       // float16 variant: activation clamp
  int zws;              // weight zero point in the int8 domain (0 for per-channel)
  int out_zp, lo, hi;
  int tiles_m, tiles_n;
  int group_m;          // tile rows per panel of the tile order
};


__device__ __forceinline__ v16i Mfma(const v4i& a, const v4i& b, const v16i& c) {
  return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ v16f Mfma(const v4i& a, const v4i& b, const v16f& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
}

template <int MB, bool X_U8, bool ROWSUM, int RQ, bool F16 = false>
__global__ void __launch_bounds__(kThreads, MB == 8 ? 1 : 2) FcMfmaKernel(FcArgs a) {
  typedef typename std::conditional<F16, v16f, v16i>::type acc_t;
  typedef Geo<MB> G;
  // The 128-row form holds 128 accumulator, 64 weight and 32 activation registers of the 256 a wavefront has at two
  // per SIMD; the in-place pass of the uint8 / row-sum variants fits beside them with one piece in flight at a time.
  // (A register the compiler spilled while one of this kernel's hand-waited loads is still writing it would be saved
  // too early: every variant must build without spills.)
  static_assert(MB == 8 || (MB == 4 && !F16), "128-row tiles: the quantized variants only");
  constexpr int TM = G::TM, S = G::kSlots, P = G::kOps;
  constexpr int kTileBytes = G::kTileBytes, kTabOffset = G::kTabOffset, kRowsumOffset = G::kRowsumOffset;
  constexpr int kWaveRows = TM / 4;  // activation rows a wavefront fetches (and rewrites in place)
  extern __shared__ __attribute__((aligned(16))) int8_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
  // run of tiles so that neighbours in its L2 share operand panels.
  int tile = blockIdx.x;
  const int total = a.tiles_m * a.tiles_n;
  if ((total & 7) == 0) tile = (tile & 7) * (total >> 3) + (tile >> 3);
  // Within that run, tiles go in panels of `group_m` tile rows, column by column: the
  // workgroups running at the same time on an XCD then form a near-square block of tiles and
  // share each operand panel between more of them (a 4 x 8 block re-reads 12 panels per
  // k-tile for 32 tiles, a 2 x 16 block 18).
  const int per_group = a.group_m * a.tiles_n;
  const int first_m = (tile / per_group) * a.group_m;
  const int gm = min(a.tiles_m - first_m, a.group_m);
  const int in_group = tile % per_group;
  const int tm_idx = first_m + in_group % gm, tn_idx = in_group / gm;
  const int m0 = tm_idx * TM, n0 = tn_idx * TN;

  // The epilogue's per-feature tables go to LDS now, one feature per thread: fetched in the
  // epilogue they would cost a chain of dependent round trips per tile.
  {
    // (stored and read back through the same types: the tables are plain arrays to the compiler)
    if constexpr (F16) {
      reinterpret_cast<float*>(lds + kTabOffset)[tid] = a.biasf32[n0 + tid];
    } else {
      reinterpret_cast<int*>(lds + kTabOffset)[tid] = a.biasf[n0 + tid];  // tables are allocated up to the padded feature count
      reinterpret_cast<tvx_v4i*>(lds + kTabOffset + TN * 4)[tid] = a.rq[n0 + tid];
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the in-flight counts below start from zero
    if constexpr (!F16) __syncthreads();  // the accumulators start from the folded bias
  }
  // ---- activations: global -> LDS DMA ---------------------------------------------
  // One wave instruction moves 64 x 16 bytes into 1 KiB of consecutive LDS: 8
  // rows x 128 bytes of the activation tile. The XOR swizzle of the LDS layout is
  // applied on the source side: lane l fetches chunk (l & 7) ^ (l >> 3) of row
  // l >> 3, a permutation inside one 128-byte line. A wavefront moves rows
  // [64 w, 64 w + 64) per k-tile (8 instructions).
  const int dma_row = lane >> 3;
  uint32_t off_x[MB];  // byte offsets from the tensor base (tensors are < 4 GiB)
  // LDS slot (row r, position lane & 7) holds chunk (lane & 7) ^ ((r >> 1) & 7) of the row (a wavefront's rows begin
  // at a multiple of 16: the chunk depends on the piece and the lane only)
  auto dma_chunk = [&](int i) { return (lane & 7) ^ (((i * 8 + dma_row) >> 1) & 7); };
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    const int r = wave * kWaveRows + i * 8 + dma_row;
    const int chunk = dma_chunk(i);
    const int xm = min(m0 + r, a.M - 1);  // rows past the edge are computed and dropped
    off_x[i] = static_cast<uint32_t>(xm) * static_cast<uint32_t>(a.K) + chunk * 16;
  }
  const int k_tiles = (a.K + TK - 1) / TK;
  const bool k_tail = (a.K % TK) != 0;
  // piece i of k-tile kt into its stage; tiles past the last one and reduction bytes past K
  // read the zero source (0x80 before the re-bias of uint8 activations) and meet zero weights
  auto dma_piece = [&](auto whole, int kt, int i) {
    int8_t* dst = lds + (kt & (kStages - 1)) * kTileBytes + wave_s * kWaveRows * TK + i * 1024;
    const int k0 = kt * TK;
    if constexpr (decltype(whole)::value) {
      // a k-tile that lies inside K: a scalar base (tensor + k0) and the lane's 32-bit offset, no address arithmetic
      // on the vector unit
      const int8_t* base = a.x + k0;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(base + off_x[i]),
                                       (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
      return;
    }
    // branch-free: the address is blended from the two candidates with a mask
    const bool past = (kt >= k_tiles) | (k_tail & (k0 + dma_chunk(i) * 16 >= a.K));
    const uintptr_t real = reinterpret_cast<uintptr_t>(a.x) + (off_x[i] + static_cast<uint32_t>(k0));
    const uintptr_t zero = reinterpret_cast<uintptr_t>(a.zeros) + (X_U8 ? 128 : 0);
    const uintptr_t take_zero = past ? ~uintptr_t{0} : uintptr_t{0};
    const int8_t* src = reinterpret_cast<const int8_t*>((zero & take_zero) | (real & ~take_zero));
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
  };

  // ---- weights: global -> registers, in fragment order -------------------------------
  // The packed weights hold, per 32-feature block and 32-byte k-step, the 64 x 16 bytes of
  // the MFMA operand in lane order: one fully coalesced 1 KiB load per fragment, no LDS.
  // Wavefront w owns feature blocks 2 w and 2 w + 1 of the tile's eight and every
  // activation row, so no fragment is fetched twice. Three k-tiles of fragments are
  // resident; slot kt % 3 is refilled for k-tile kt + 3 as its k-steps retire.
  const int8_t* wp[2];  // (wavefront-uniform: the lane's 16 bytes are the load's vector offset)
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
    wp[nb] = a.w + (static_cast<size_t>(n0 / 32 + wave_s * 2 + nb) * (k_tiles_padded(a.K, S) * 4)) * 1024;
  const uint32_t lane16 = lane * 16;
  v4i wr[S][8];  // [slot][nb * 4 + k-step]
#define TVX_W_LOAD(dst, ptr, off) \
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(lane16), "s"(ptr), "n"(off))
  // fragment (nb, kk) of k-tile kt (callers stay below the padded count of k-tiles)
  auto w_piece = [&](int kt, int nb, int kk, v4i& dst) {
    const int8_t* ptr = wp[nb] + static_cast<size_t>(kt) * 4096;
    if (kk == 0) TVX_W_LOAD(dst, ptr, 0);
    else if (kk == 1) TVX_W_LOAD(dst, ptr, 1024);
    else if (kk == 2) TVX_W_LOAD(dst, ptr, 2048);
    else TVX_W_LOAD(dst, ptr, 3072);
  };
#undef TVX_W_LOAD

  // [feature block][activation block]; a lane holds, per accumulator quad g, features 8 g + 4 (lane / 32) + 0..3 of its
  // wavefront's blocks. The integer accumulators start from the folded bias: one addition less per output in the epilogue.
  acc_t acc[2][MB];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      int b4[4] = {0, 0, 0, 0};
      if constexpr (!F16) {
        const v4i t = *reinterpret_cast<const v4i*>(lds + kTabOffset + (wave * 64 + i * 32 + 8 * g + 4 * (lane >> 5)) * 4);
        b4[0] = t[0], b4[1] = t[1], b4[2] = t[2], b4[3] = t[3];
      }
#pragma unroll
      for (int j = 0; j < MB; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) acc[i][j][g * 4 + q] = b4[q];
    }
  int rowsum[MB] = {};  // per piece of this wavefront's share of the activation tile (see the in-place pass below)

  const int frag_row = lane & 31;   // row inside a 32-row MFMA tile
  const int frag_half = lane >> 5;  // which 16-byte half of a 32-byte k-step
  const int row7 = (frag_row >> 1) & 7;  // fragment tiles start at multiples of 32 rows

  // Activation fragments are fetched by inline assembly and waited for with explicit
  // s_waitcnt, like the weight fragments above: the compiler's own wait insertion treats
  // values carried across the loop back-edge conservatively (it waits for everything in
  // flight), which would serialize the fetches with the MFMAs.
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<size_t>(lds));
  uint32_t frag_x[4];  // per k-step: LDS address of this lane's fragment in activation block 0, stage 0
#pragma unroll
  for (int kk = 0; kk < 4; ++kk)
    frag_x[kk] = lds_base + frag_row * TK + (((kk * 2 + frag_half) ^ row7) << 4);
#define TVX_DS_READ(dst, addr, off) \
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
  // fragment t (activation rows 32 t ..) of k-step kk of k-tile kt
  auto load_frag = [&](int kt, int kk, v4i* fx, int t) {
    const uint32_t ax = frag_x[kk] + (kt & (kStages - 1)) * kTileBytes;
    if (t == 0) TVX_DS_READ(fx[0], ax, 0);
    else if (t == 1) TVX_DS_READ(fx[1], ax, 32 * TK);
    else if (t == 2) TVX_DS_READ(fx[2], ax, 64 * TK);
    else if (t == 3) TVX_DS_READ(fx[3], ax, 96 * TK);
    else if (t == 4) TVX_DS_READ(fx[4], ax, 128 * TK);
    else if (t == 5) TVX_DS_READ(fx[5], ax, 160 * TK);
    else if (t == 6) TVX_DS_READ(fx[6], ax, 192 * TK);
    else TVX_DS_READ(fx[7], ax, 224 * TK);
  };
#undef TVX_DS_READ
  // ---- uint8 activations and row sums: one pass over the tile in LDS ---------------------
  // The MFMA is signed, so uint8 activations are re-biased (x ^ 0x80 = x - 128 as int8), and a uniform
  // weight zero point needs the sum of every activation row. Both are vector-unit work, and a wavefront's
  // vector instructions do not overlap its own MFMAs (measured: each costs its full issue time on top of
  // the MFMA time). Done on the fragments, the four wavefronts - which all read every row - would each do
  // all of it; done once on the tile in LDS it is a quarter: every wavefront rewrites the 64 rows it
  // fetched itself (eight pieces of 1 KiB, a lane's 16 bytes of one row each), one k-tile ahead of the
  // MFMAs, spread over the first three k-steps. The barrier that publishes k-tile kt + 1 also publishes
  // its rewritten form.
  constexpr bool kInPlace = X_U8 || ROWSUM;
  const uint32_t own_x = lds_base + wave * kWaveRows * TK + lane * 16;
#define TVX_DS_READ(dst, addr, off) \
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
#define TVX_DS_WRITE(addr, src, off) \
  asm volatile("ds_write_b128 %0, %1 offset:%2" : : "v"(addr), "v"(src), "n"(off))
  auto piece_read = [&](int kt, int i, v4i& t) {
    const uint32_t ax = own_x + (kt & (kStages - 1)) * kTileBytes;
    if (i == 0) TVX_DS_READ(t, ax, 0);
    else if (i == 1) TVX_DS_READ(t, ax, 1024);
    else if (i == 2) TVX_DS_READ(t, ax, 2048);
    else if (i == 3) TVX_DS_READ(t, ax, 3072);
    else if (i == 4) TVX_DS_READ(t, ax, 4096);
    else if (i == 5) TVX_DS_READ(t, ax, 5120);
    else if (i == 6) TVX_DS_READ(t, ax, 6144);
    else TVX_DS_READ(t, ax, 7168);
  };
  auto piece_finish = [&](int kt, int i, v4i& t) {
    if (X_U8) t ^= static_cast<int>(0x80808080);
    if (ROWSUM) {
#pragma unroll
      for (int q = 0; q < 4; ++q) rowsum[i] = __builtin_amdgcn_sdot4(t[q], 0x01010101, rowsum[i], false);
    }
    if (X_U8) {
      const uint32_t ax = own_x + (kt & (kStages - 1)) * kTileBytes;
      if (i == 0) TVX_DS_WRITE(ax, t, 0);
      else if (i == 1) TVX_DS_WRITE(ax, t, 1024);
      else if (i == 2) TVX_DS_WRITE(ax, t, 2048);
      else if (i == 3) TVX_DS_WRITE(ax, t, 3072);
      else if (i == 4) TVX_DS_WRITE(ax, t, 4096);
      else if (i == 5) TVX_DS_WRITE(ax, t, 5120);
      else if (i == 6) TVX_DS_WRITE(ax, t, 6144);
      else TVX_DS_WRITE(ax, t, 7168);
    }
  };
#undef TVX_DS_READ
#undef TVX_DS_WRITE
  v4i pc[MB == 8 ? 3 : 1];  // pieces on their way through the pass (128 rows: one at a time)
  // One k-step: 16 MFMAs of 32 cycles each, and everything else the k-step has to issue dealt out
  // between them, a few instructions at a time (the compiler, left to itself, gathers them into two
  // runs per k-step; memory instructions issued in a burst queue up with the wavefront waiting behind
  // them). Pair p multiplies activation block p with the wavefront's two weight fragments; behind its
  // MFMAs go: the LDS reads of the next k-step's fragments (two per pair, all eight issued by the
  // middle of the k-step), this k-step's share of the in-place pass over the next k-tile (three
  // pieces in k-steps 0 and 1, two in k-step 2: read behind pair 2, finished behind pairs 6 and 7),
  // and the k-step's four memory operations of the prefetch - the weight registers are refilled
  // (for k-tile kt + 3) right after the last MFMA that reads them.
  auto k_step = [&](auto prefetch, auto whole, auto fetch_next, auto in_place, auto newer, int kt, int kk, v4i* fx,
                    v4i* w_slot, int next_kt, int next_kk, v4i* fx_next) {
    constexpr bool kPrefetch = decltype(prefetch)::value;
    constexpr bool kNext = decltype(fetch_next)::value;
    constexpr bool kPass = kInPlace && decltype(in_place)::value;
    // MB = 8: pieces 0-2, 3-5, 6-7 in k-steps 0, 1, 2; MB = 4: pieces 0-1, 2, 3
    const int first = MB == 8 ? kk * 3 : (kk == 0 ? 0 : kk + 1);
    const int pieces = MB == 8 ? (kk < 2 ? 3 : (kk == 2 ? 2 : 0)) : (kk == 0 ? 2 : (kk < 3 ? 1 : 0));
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      acc[0][mb] = Mfma(w_slot[kk], fx[mb], acc[0][mb]);
      if (kNext && mb < MB / 2) load_frag(next_kt, next_kk, fx_next, 2 * mb);
      if (kPass && mb == MB / 4) {
        // this wavefront's own pieces of k-tile kt + 1 have landed when at most the memory operations of the
        // k-tiles behind it (one with three weight slots, none with two or in the last round) are still on their way
        if (kk == 0) {
          if constexpr (decltype(newer)::value != 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((S - 2) * P) : "memory");
          else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        if constexpr (MB == 8) {
#pragma unroll
          for (int j = 0; j < 3; ++j)
            if (j < pieces) piece_read(kt + 1, first + j, pc[j]);
        } else {
          if (pieces > 0) piece_read(kt + 1, first, pc[0]);
        }
      }
      if (kPrefetch && mb == MB / 2) dma_piece(whole, kt + S, MB == 8 ? kk * 2 : kk);
      if (kPass && mb == MB - 2 && pieces > 0) {
        // (the pieces are operands of the wait: nothing that uses them may be moved in front of it)
        if constexpr (MB == 8) {
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(pc[0]), "+v"(pc[1]), "+v"(pc[2])::"memory");
          piece_finish(kt + 1, first, pc[0]);
        } else {
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(pc[0])::"memory");
          piece_finish(kt + 1, first, pc[0]);
          if (pieces > 1) piece_read(kt + 1, first + 1, pc[0]);  // (the second piece of k-step 0 follows through the same registers)
        }
      }
      if constexpr (MB == 8) {
        if (kPass && mb == MB - 1 && pieces > 2) piece_finish(kt + 1, first + 2, pc[2]);
      } else {
        if (kPass && mb == MB - 1 && pieces > 1) {
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(pc[0])::"memory");
          piece_finish(kt + 1, first + 1, pc[0]);
        }
      }
      if (kPrefetch && mb == MB - 1) w_piece(kt + S, 0, kk, w_slot[kk]);
      __builtin_amdgcn_sched_barrier(0);
      acc[1][mb] = Mfma(w_slot[4 + kk], fx[mb], acc[1][mb]);
      if (kNext && mb < MB / 2) load_frag(next_kt, next_kk, fx_next, 2 * mb + 1);
      if (MB == 8 && kPrefetch && mb == MB / 2 + 1) dma_piece(whole, kt + S, kk * 2 + 1);
      if constexpr (MB == 8) {
        if (kPass && mb == MB - 2 && pieces > 1) piece_finish(kt + 1, first + 1, pc[1]);
      }
      if (kPrefetch && mb == MB - 1) w_piece(kt + S, 1, kk, w_slot[4 + kk]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // k-tile kt with its weight slot: the fragments of k-step kk + 1 are fetched while step kk
  // multiplies; the barrier that publishes the next k-tile sits before the last k-step, so
  // that the first fragments of the next tile are on their way while it runs. Every k-tile
  // issues 16 memory operations in the same order; "at most 28 in flight" at the barrier
  // (12 of this k-tile, 16 of the one before) means that everything issued two k-tiles ago
  // - the activations and weights of k-tile kt + 1 - has landed.
  v4i fxa[MB], fxb[MB];
  // `prefetch`: the k-tile issues its share of k-tile kt + 3 (all rounds but the last, which is peeled off so that
  // no fetch is in flight when the loop ends: registers named by an unfinished fetch would otherwise have to be
  // kept out of the epilogue's hands). `in_flight`: memory operations that may still be on their way at the
  // barrier (28 while prefetching; 16, 0, 0 in the last round). `last`: no fragments of a next k-tile.
  auto k_tile = [&](auto prefetch, auto whole, auto in_flight, auto last, int kt, v4i* w_slot) {
    const std::integral_constant<bool, true> yes;
    const std::integral_constant<bool, !decltype(last)::value> unless_last;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the fragments of k-step 0
    __builtin_amdgcn_sched_barrier(0);
    k_step(prefetch, whole, yes, unless_last, in_flight, kt, 0, fxa, w_slot, kt, 1, fxb);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    k_step(prefetch, whole, yes, unless_last, in_flight, kt, 1, fxb, w_slot, kt, 2, fxa);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    k_step(prefetch, whole, yes, unless_last, in_flight, kt, 2, fxa, w_slot, kt, 3, fxb);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(decltype(in_flight)::value) : "memory");
    // the bare barrier: __syncthreads() adds a fence that waits for every memory operation in
    // flight - the whole prefetch - at every k-tile
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    k_step(prefetch, whole, unless_last, unless_last, in_flight, kt, 3, fxb, w_slot, kt + 1, 0, fxa);
  };
  // prologue: k-tiles 0, 1, 2 in the order every later k-tile uses (8 x (activation piece,
  // weight fragment)), so that the in-flight counts line up from the first barrier on
#pragma unroll
  for (int t = 0; t < S; ++t)
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        if (MB == 8 || nb == 0) dma_piece(std::integral_constant<bool, false>(), t, MB == 8 ? kk * 2 + nb : kk);
        __builtin_amdgcn_sched_barrier(0);
        w_piece(t, nb, kk, wr[t][nb * 4 + kk]);
        __builtin_amdgcn_sched_barrier(0);
      }
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"((S - 1) * P) : "memory");  // k-tile 0 has landed
  if (kInPlace) {
    // the in-place pass over k-tile 0 (every later k-tile gets it while the one before multiplies)
#pragma unroll
    for (int i = 0; i < MB; i += 2) {
      if constexpr (MB == 8) {
        piece_read(0, i, pc[0]);
        piece_read(0, i + 1, pc[1]);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(pc[0]), "+v"(pc[1])::"memory");
        piece_finish(0, i, pc[0]);
        piece_finish(0, i + 1, pc[1]);
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          piece_read(0, i + j, pc[0]);
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(pc[0])::"memory");
          piece_finish(0, i + j, pc[0]);
        }
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int t = 0; t < MB; ++t) load_frag(0, 0, fxa, t);
  const int kt_max = k_tiles_padded(a.K, S) - 1;
  // the loop runs whole rounds of three k-tiles (the weight slots are named registers); the
  // packed weights are zero-padded to that count and the activations past K read zeros
  {
    using std::integral_constant;
    const integral_constant<bool, true> yes;
    const integral_constant<bool, false> no;
    int kt = 0;
    // rounds whose prefetch (k-tiles kt + 3 .. kt + 5) lies inside K, then those that reach past it
    const int whole_tiles = a.K / TK;
    // memory operations that may still be on their way at a k-tile's barrier when everything of k-tile kt + 1 has
    // landed: the k-tiles between it and the one being fetched, and the three k-steps' worth of that one
    const integral_constant<int, (S - 2) * P + 3 * P / 4> steady;
    for (; kt + 2 * S <= whole_tiles; kt += S) {
      k_tile(yes, yes, steady, no, kt, wr[0]);
      k_tile(yes, yes, steady, no, kt + 1, wr[1]);
      if constexpr (S == 3) k_tile(yes, yes, steady, no, kt + 2, wr[S - 1]);
    }
    for (; kt + S <= kt_max; kt += S) {
      k_tile(yes, no, steady, no, kt, wr[0]);
      k_tile(yes, no, steady, no, kt + 1, wr[1]);
      if constexpr (S == 3) k_tile(yes, no, steady, no, kt + 2, wr[S - 1]);
    }
    // the last round: its k-tiles were fetched by the round before (or the prologue); nothing new is fetched
    if constexpr (S == 3) {
      k_tile(no, no, integral_constant<int, P>(), no, kt, wr[0]);
      k_tile(no, no, integral_constant<int, 0>(), no, kt + 1, wr[1]);
      k_tile(no, no, integral_constant<int, 0>(), yes, kt + 2, wr[S - 1]);
    } else {
      k_tile(no, no, integral_constant<int, 0>(), no, kt, wr[0]);
      k_tile(no, no, integral_constant<int, 0>(), yes, kt + 1, wr[1]);
    }
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // (nothing is in flight here; the staging tile is about to be written)
  if (ROWSUM) {
    // piece i holds rows kWaveRows w + 8 i + lane / 8, a lane its 16 bytes of every k-tile: eight lanes make a row
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      int sum = rowsum[i];
      sum += __shfl_xor(sum, 1);
      sum += __shfl_xor(sum, 2);
      sum += __shfl_xor(sum, 4);
      if ((lane & 7) == 0) reinterpret_cast<int*>(lds + kRowsumOffset)[wave * kWaveRows + i * 8 + (lane >> 3)] = sum;
    }
  }
  __syncthreads();  // the epilogue reuses the LDS

  // ---- epilogue ---------------------------------------------------------------
  // A lane holds activation row mb * 32 + lane % 32 and, per accumulator quad g, the four
  // consecutive features 8 g + 4 (lane / 32) + 0..3 of its wavefront's blocks 2 w, 2 w + 1.
  if constexpr (F16) {
    // ---- float16: bias, activation clamp, round; the 256 x 256 x 2-byte tile is staged in two rounds of 128
    // columns (64 KiB + padding): round r stages both feature blocks of wavefronts 2 r and 2 r + 1, so that a
    // staged row is 256 contiguous output bytes - two whole lines (halves of a line written in different
    // rounds cost half as many bytes again at the memory)
    constexpr int kHalfStride = 128 * 2 + 16;  // bytes per staged row: 128 halves + padding
    int8_t* out_tile = lds;
#pragma unroll
    for (int round = 0; round < 2; ++round) {
      if (round) __syncthreads();
      if ((wave >> 1) == round) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            __builtin_amdgcn_sched_barrier(0);  // (one feature quad at a time, as below)
            const int nl = wave * 64 + nb * 32 + 8 * g + 4 * frag_half;  // feature within the tile
            float b4[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) b4[q] = reinterpret_cast<const float*>(lds + kTabOffset)[nl + q];
            const int col = nl - round * 128;  // staged column (halves)
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
              const int ml = mb * 32 + frag_row;
              _Float16 h[4];
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                float v = acc[nb][mb][g * 4 + q] + b4[q];
                v = fminf(fmaxf(v, a.flo), a.fhi);
                h[q] = static_cast<_Float16>(v);
              }
              uint2 pk;
              __builtin_memcpy(&pk, h, 8);
              *reinterpret_cast<uint2*>(out_tile + ml * kHalfStride + col * 2) = pk;
            }
          }
        }
      }
      __syncthreads();
      // a staged row holds features [128 round, 128 round + 128) of the tile: 16 chunks of 8 halves
      const bool vec_ok = (a.N & 7) == 0;
      for (int c = tid; c < TM * 16; c += kThreads) {
        const int ml = c >> 4, ch = c & 15;
        const int m = m0 + ml, n = n0 + round * 128 + ch * 8;
        if (m >= a.M || n >= a.N) continue;
        const int8_t* src = out_tile + ml * kHalfStride + ch * 16;
        int8_t* dst = a.y + (static_cast<size_t>(m) * a.N + n) * 2;
        if (vec_ok) {
          *reinterpret_cast<v4i*>(dst) = *reinterpret_cast<const v4i*>(src);
        } else {
          for (int q = 0; q < 8 && n + q < a.N; ++q)
            reinterpret_cast<uint16_t*>(dst)[q] = reinterpret_cast<const uint16_t*>(src)[q];
        }
      }
    }
  } else {
    int zp_term[MB];  // weight zero point x row sum, per activation block of this lane's row
#pragma unroll
    for (int t = 0; t < MB; ++t)
      zp_term[t] = ROWSUM ? a.zws * reinterpret_cast<const int*>(lds + kRowsumOffset)[t * 32 + frag_row] : 0;
    int8_t* out_tile = lds;  // TM rows x kOutStride bytes (the loop's last barrier freed the LDS)
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        // (one feature quad at a time: hoisting the table reads of all eight quads costs more registers than there are)
        __builtin_amdgcn_sched_barrier(0);
        const int nl = wave * 64 + nb * 32 + 8 * g + 4 * frag_half;
        const int n = n0 + nl;
        tvx_v4i q4[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) q4[q] = reinterpret_cast<const tvx_v4i*>(lds + kTabOffset + TN * 4)[nl + q];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const int ml = mb * 32 + frag_row;
          int r4[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            int v = acc[nb][mb][g * 4 + q];  // (bias included: the accumulators started from it)
            if (ROWSUM) v -= zp_term[mb];
            r4[q] = Requant8<RQ>(v, q4[q], a.out_zp, a.lo, a.hi);
          }
          *reinterpret_cast<uint32_t*>(out_tile + ml * kOutStride + nl) = PackBytes(r4[0], r4[1], r4[2], r4[3]);
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
}

// ---- few outputs: 16 x 16 tiles, the reduction split over the workgroup's wavefronts ---------
// A layer like 64 x 1280 -> 1000 holds four 256 x 256 tiles - four workgroups on a chip of 256
// CUs. Here a workgroup owns 16 x 16 outputs (v_mfma_i32_16x16x64_i8), its four wavefronts
// take every fourth 64-byte k-step with operand fragments loaded straight from global memory
// (eight k-steps in flight per wavefront, every load unconditional: positions past K read the
// zero source, k-steps past the end re-read the last one and are dropped), the partial sums
// meet in LDS and the first wavefront requantizes and stores. Same operands, tables and
// arithmetic as the big kernel.
constexpr int kSmallBatch = 8;

template <bool X_U8, bool ROWSUM, int RQ>
__global__ void __launch_bounds__(kThreads) FcSmallKernel(FcArgs a) {
  __shared__ int red[4][4][64];
  __shared__ int red_rs[4][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tiles_n = (a.N + 15) / 16;
  const int tn = blockIdx.x % tiles_n, tm = blockIdx.x / tiles_n;
  const int n0 = tn * 16, m0 = tm * 16;
  const int row = lane & 15, kq = lane >> 4;  // fragment row; 16-byte quarter of a 64-byte k-step
  const int8_t* xrow = a.x + static_cast<size_t>(min(m0 + row, a.M - 1)) * a.K + kq * 16;
  const int8_t* wrow = a.w + static_cast<size_t>(min(n0 + row, a.N - 1)) * a.K + kq * 16;
  const int ksteps = (a.K + 63) / 64;
  v4i acc = {0, 0, 0, 0};
  int rowsum = 0;
  for (int ks0 = wave; ks0 < ksteps; ks0 += 4 * kSmallBatch) {
    v4i fx[kSmallBatch], fw[kSmallBatch];
#pragma unroll
    for (int b = 0; b < kSmallBatch; ++b) {
      const int off = min(ks0 + 4 * b, ksteps - 1) * 64;
      const bool past = off + kq * 16 >= a.K;  // only in the last k-step, when K is not a multiple of 64
      // the address is selected, not the value: the load itself stays unconditional
      const int8_t* px = past ? a.zeros + (X_U8 ? 128 : 0) : xrow + off;
      const int8_t* pw = past ? a.zeros : wrow + off;
      fx[b] = *reinterpret_cast<const v4i*>(px);
      fw[b] = *reinterpret_cast<const v4i*>(pw);
    }
#pragma unroll
    for (int b = 0; b < kSmallBatch; ++b) {
      if (ks0 + 4 * b < ksteps) {  // uniform over the wavefront
        if (X_U8) fx[b] ^= static_cast<int>(0x80808080);
        if (ROWSUM) {
#pragma unroll
          for (int q = 0; q < 4; ++q) rowsum = __builtin_amdgcn_sdot4(fx[b][q], 0x01010101, rowsum, false);
        }
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(fw[b], fx[b], acc, 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) red[wave][r][lane] = acc[r];
  if (ROWSUM) red_rs[wave][lane] = rowsum;
  __syncthreads();
  if (wave != 0) return;
  // lane holds activation row m0 + lane % 16 and features n0 + 4 * (lane / 16) + 0..3
  const int m = m0 + row, n = n0 + 4 * kq;
  int rs = 0;
  if (ROWSUM) {
#pragma unroll
    for (int w = 0; w < 4; ++w)
#pragma unroll
      for (int qq = 0; qq < 4; ++qq) rs += red_rs[w][qq * 16 + row];
  }
  int r4[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    int v = red[0][r][lane] + red[1][r][lane] + red[2][r][lane] + red[3][r][lane] + a.biasf[n + r];
    if (ROWSUM) v -= a.zws * rs;
    r4[r] = Requant8<RQ>(v, a.rq[n + r], a.out_zp, a.lo, a.hi);  // tables cover the padded feature count
  }
  if (m >= a.M || n >= a.N) return;
  int8_t* dst = a.y + static_cast<size_t>(m) * a.N + n;
  if ((a.N & 3) == 0) {
    *reinterpret_cast<uint32_t*>(dst) = PackBytes(r4[0], r4[1], r4[2], r4[3]);
  } else {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      if (n + r < a.N) dst[r] = static_cast<int8_t>(r4[r]);
  }
}

template <bool X_U8, bool ROWSUM>
void LaunchSmallRq(int rq, dim3 grid, hipStream_t st, const FcArgs& a) {
  const dim3 block(kThreads);
  if (rq == kRqFastNoTie) hipLaunchKernelGGL((FcSmallKernel<X_U8, ROWSUM, kRqFastNoTie>), grid, block, 0, st, a);
  else if (rq == kRqFast) hipLaunchKernelGGL((FcSmallKernel<X_U8, ROWSUM, kRqFast>), grid, block, 0, st, a);
  else hipLaunchKernelGGL((FcSmallKernel<X_U8, ROWSUM, kRqGeneric>), grid, block, 0, st, a);
}

// Few enough outputs that 256 x 256 tiles would leave most of the chip idle.
bool UseSmallTiles(const tvx_fc_desc& d) { return static_cast<uint64_t>(d.m) * d.n <= (1u << 18); }

typedef void (*TileKernel)(FcArgs);
template <int MB, bool X_U8, bool ROWSUM>
TileKernel TileKernelOf(int rq) {
  if (rq == kRqFastNoTie) return FcMfmaKernel<MB, X_U8, ROWSUM, kRqFastNoTie>;
  if (rq == kRqFast) return FcMfmaKernel<MB, X_U8, ROWSUM, kRqFast>;
  return FcMfmaKernel<MB, X_U8, ROWSUM, kRqGeneric>;
}
// mb: the tile's 32-row activation blocks (8, or 4 for the quantized variants)
TileKernel TileKernelOf(int mb, bool f16, bool x_u8, bool rowsum, int rq) {
  if (f16) return FcMfmaKernel<8, false, false, kRqGeneric, true>;
  if (x_u8 && rowsum) return mb == 8 ? TileKernelOf<8, true, true>(rq) : TileKernelOf<4, true, true>(rq);
  if (x_u8) return mb == 8 ? TileKernelOf<8, true, false>(rq) : TileKernelOf<4, true, false>(rq);
  if (rowsum) return mb == 8 ? TileKernelOf<8, false, true>(rq) : TileKernelOf<4, false, true>(rq);
  return mb == 8 ? TileKernelOf<8, false, false>(rq) : TileKernelOf<4, false, false>(rq);
}
int TileLdsBytes(int mb) { return mb == 8 ? Geo<8>::kLdsBytes : Geo<4>::kLdsBytes; }
int TileSlots(int mb) { return mb == 8 ? Geo<8>::kSlots : Geo<4>::kSlots; }

// 128-row tiles (the quantized variants have them) where there are enough to give every CU two workgroups twice
// over; TVX_FC_TILE_M=128|256 overrides (a test lever, read when the operator is created).
int ChooseTileBlocks(uint32_t m, uint32_t n, bool quantized) {
  if (!quantized) return 8;
  int mb = static_cast<uint64_t>((m + 127) / 128) * ((n + TN - 1) / TN) >= 1024 ? 4 : 8;
  if (const char* f = getenv("TVX_FC_TILE_M")) {
    const int v = atoi(f);
    if (v == 128) mb = 4;
    if (v == 256) mb = 8;
  }
  return mb;
}

int FcMfmaRun(tvx_op* op, const void* in0, const void*, void* out, hipStream_t st) {
  const tvx_fc_desc& d = op->fc;
  FcArgs a{};
  a.x = static_cast<const int8_t*>(in0);
  a.w = op->packed.as<int8_t>();
  a.y = static_cast<int8_t*>(out);
  a.biasf = op->aux.as<int32_t>();
  a.rq = op->aux2.as<tvx_v4i>();
  a.zeros = op->aux3.as<int8_t>();
  a.M = static_cast<int>(d.m);
  a.N = static_cast<int>(d.n);
  a.K = static_cast<int>(d.k);
  a.zws = op->geo[0];
  a.out_zp = d.out_zp;
  a.lo = op->act_lo;
  a.hi = op->act_hi;
  const int mb = op->geo[3];
  a.tiles_m = (a.M + mb * 32 - 1) / (mb * 32);
  a.tiles_n = (a.N + TN - 1) / TN;
  a.group_m = mb == 8 ? 4 : 8;  // panels of 1024 activation rows
  const dim3 grid(a.tiles_m * a.tiles_n);
  const bool x_u8 = d.in_dtype == TVX_U8, rowsum = a.zws != 0;
  const int rq = op->geo[1];
  if (op->geo[2]) {  // float16
    a.K = static_cast<int>(d.k) * 2;
    a.biasf32 = op->aux.as<float>();
    a.flo = d.activation == TVX_ACT_NONE ? -3.402823466e38f : 0.0f;
    a.fhi = d.activation == TVX_ACT_RELU6 ? 6.0f : 3.402823466e38f;
    hipLaunchKernelGGL(TileKernelOf(mb, true, false, false, rq), grid, dim3(kThreads), TileLdsBytes(mb), st, a);
    TVX_HIP_CHECK(hipGetLastError());
    return TVX_OK;
  }
  if (UseSmallTiles(d)) {
    const dim3 small_grid(((a.M + 15) / 16) * ((a.N + 15) / 16));
    if (x_u8 && rowsum) LaunchSmallRq<true, true>(rq, small_grid, st, a);
    else if (x_u8) LaunchSmallRq<true, false>(rq, small_grid, st, a);
    else if (rowsum) LaunchSmallRq<false, true>(rq, small_grid, st, a);
    else LaunchSmallRq<false, false>(rq, small_grid, st, a);
    TVX_HIP_CHECK(hipGetLastError());
    return TVX_OK;
  }
  hipLaunchKernelGGL(TileKernelOf(mb, false, x_u8, rowsum, rq), grid, dim3(kThreads), TileLdsBytes(mb), st, a);
  TVX_HIP_CHECK(hipGetLastError());
  return TVX_OK;
}

}  // namespace

// Weights [N][k_bytes] (int8 domain or float16 bytes) -> MFMA-fragment order: for every block
// of 32 features and every 32-byte k-step, 64 lanes x 16 bytes where lane l holds feature
// 32 b + l % 32, bytes [32 ks + 16 (l / 32), + 16). Features are padded to the tile and the
// reduction to whole rounds of `slots` k-tiles (the kernel's weight slots), with zeros.
static std::vector<int8_t> PackFragments(const int8_t* w, uint32_t n, uint32_t k_bytes, int slots) {
  const size_t n_blocks = (n + TN - 1) / TN * (TN / 32);
  const size_t ksteps = static_cast<size_t>(k_tiles_padded(static_cast<int>(k_bytes), slots)) * 4;
  std::vector<int8_t> out(n_blocks * ksteps * 1024, 0);
  for (size_t b = 0; b < n_blocks; ++b)
    for (int r = 0; r < 32; ++r) {
      const size_t row = b * 32 + r;
      if (row >= n) break;
      const int8_t* src = w + row * k_bytes;
      for (size_t c = 0; c * 16 < k_bytes; ++c) {  // 16-byte chunks of the row (k_bytes % 16 == 0)
        const size_t ks = c >> 1, half = c & 1;
        std::memcpy(&out[((b * ksteps + ks) * 64 + half * 32 + r) * 16], src + c * 16, 16);
      }
    }
  return out;
}

// float16 x float16 -> float16 with constant weights and K a multiple of 8.
static int FcMfmaSetupF16(tvx_op* op, const tvx_fc_desc* d, const void* w_host, const void* bias_host) {
  if ((d->k & 7) != 0) return TVX_E_UNSUPPORTED;
  if (static_cast<uint64_t>(d->m) * d->n >= (1ull << 30) || d->k > (1u << 23)) return TVX_E_UNSUPPORTED;
  if (static_cast<uint64_t>(d->m) * d->k >= (1ull << 31) || static_cast<uint64_t>(d->n) * d->k >= (1ull << 31))
    return TVX_E_UNSUPPORTED;  // the operand DMA addresses rows with 32-bit byte offsets
  const uint32_t n_alloc = (d->n + TN - 1) / TN * TN;
  std::vector<float> bias(n_alloc, 0.0f);
  if (bias_host) std::memcpy(bias.data(), bias_host, sizeof(float) * d->n);
  const int mb = ChooseTileBlocks(d->m, d->n, false);
  const std::vector<int8_t> frags = PackFragments(static_cast<const int8_t*>(w_host), d->n, d->k * 2, TileSlots(mb));
  int s = op->packed.Upload(frags.data(), frags.size());
  if (s == TVX_OK) s = op->aux.Upload(bias.data(), bias.size() * 4);
  std::vector<int8_t> zeros(256, 0);
  if (s == TVX_OK) s = op->aux3.Upload(zeros.data(), zeros.size());
  if (s != TVX_OK) return s;
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(TileKernelOf(mb, true, false, false, kRqGeneric)),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, TileLdsBytes(mb));
  if (e != hipSuccess)
    return SetError(TVX_E_DEVICE, "hipFuncSetAttribute(dynamic LDS %d): %s", TileLdsBytes(mb), hipGetErrorString(e));
  op->geo[2] = 1;
  op->geo[3] = mb;
  op->run = FcMfmaRun;
  op->kernel_name = "fc_mfma_f16_256x256x64";
  return TVX_OK;
}

// Claims FullyConnected with constant weights: quantized with K a multiple of 16 (every
// 16-byte operand chunk is then whole and aligned), or all-float16.
int FcMfmaSetup(tvx_op* op, const tvx_fc_desc* d, const void* w_host, const void* bias_host) {
  if (w_host && d->in_dtype == TVX_F16 && d->w_dtype == TVX_F16 && d->out_dtype == TVX_F16)
    return FcMfmaSetupF16(op, d, w_host, bias_host);
  if (!op->quantized || !w_host || (d->k & 15) != 0) return TVX_E_UNSUPPORTED;
  // a handful of outputs does not fill one 256 x 256 tile: the wavefront-per-output kernel is quicker
  if (static_cast<uint64_t>(d->m) * d->n <= 8192) return TVX_E_UNSUPPORTED;
  if (static_cast<uint64_t>(d->m) * d->n >= (1ull << 31) || d->k > (1u << 24)) return TVX_E_UNSUPPORTED;
  if (static_cast<uint64_t>(d->m) * d->k >= (1ull << 32) || static_cast<uint64_t>(d->n) * d->k >= (1ull << 32))
    return TVX_E_UNSUPPORTED;  // the operand DMA addresses rows with 32-bit offsets
  const size_t wn = static_cast<size_t>(d->n) * d->k;
  const bool w_u8 = d->w_dtype == TVX_U8;
  // int8-domain operands: uint8 tensors are shifted by 128, zero points follow
  const int zxs = d->in_zp - (d->in_dtype == TVX_U8 ? 128 : 0);
  const int zws = op->w_zp - (w_u8 ? 128 : 0);
  std::vector<int8_t> ws(wn);
  const uint8_t* src = static_cast<const uint8_t*>(w_host);
  for (size_t i = 0; i < wn; ++i) ws[i] = static_cast<int8_t>(w_u8 ? src[i] ^ 0x80 : src[i]);
  const uint32_t n_alloc = (d->n + TN - 1) / TN * TN;
  std::vector<int32_t> biasf(n_alloc, 0);
  const int32_t* b = static_cast<const int32_t*>(bias_host);
  for (uint32_t n = 0; n < d->n; ++n) {
    int64_t sw = 0;
    const int8_t* row = ws.data() + static_cast<size_t>(n) * d->k;
    for (uint32_t k = 0; k < d->k; ++k) sw += row[k];
    const int64_t v = (b ? b[n] : 0) - static_cast<int64_t>(zxs) * sw +
                      static_cast<int64_t>(d->k) * zxs * zws;
    biasf[n] = static_cast<int32_t>(static_cast<uint32_t>(v));  // int32 accumulators wrap
  }
  std::vector<int32_t> rqt;
  const int rq = BuildRequantRecords(op->h_mult, op->h_shift, static_cast<int>(d->n),
                                     static_cast<int>(n_alloc), d->out_zp, &rqt,
                                     AccumulatorBound(d->k, bias_host, d->n));
  // the tiled kernel reads fragment order, the small-tile kernel plain rows
  const int mb = ChooseTileBlocks(d->m, d->n, true);
  int s;
  if (UseSmallTiles(*d)) {
    s = op->packed.Upload(ws.data(), wn);
  } else {
    const std::vector<int8_t> frags = PackFragments(ws.data(), d->n, d->k, TileSlots(mb));
    s = op->packed.Upload(frags.data(), frags.size());
  }
  if (s == TVX_OK) s = op->aux.Upload(biasf.data(), biasf.size() * 4);
  if (s == TVX_OK) s = op->aux2.Upload(rqt.data(), rqt.size() * 4);
  std::vector<int8_t> zeros(256, 0);
  for (int i = 128; i < 256; ++i) zeros[i] = static_cast<int8_t>(-128);
  if (s == TVX_OK) s = op->aux3.Upload(zeros.data(), zeros.size());
  if (s != TVX_OK) return s;
  const bool x_u8 = d->in_dtype == TVX_U8, rowsum = zws != 0;
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(TileKernelOf(mb, false, x_u8, rowsum, rq)),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, TileLdsBytes(mb));
  if (e != hipSuccess)
    return SetError(TVX_E_DEVICE, "hipFuncSetAttribute(dynamic LDS %d): %s", TileLdsBytes(mb), hipGetErrorString(e));
  op->geo[0] = zws;
  op->geo[1] = rq;
  op->geo[3] = mb;
  op->run = FcMfmaRun;
  op->kernel_name = UseSmallTiles(*d) ? "fc_mfma_i8_16x16_splitk" : (mb == 8 ? "fc_mfma_i8_256x256x128" : "fc_mfma_i8_128x256x128");
  return TVX_OK;
}

}  // namespace tvx
