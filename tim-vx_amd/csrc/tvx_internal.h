// Shared declarations of the HIP side: the operator object behind tvx_op,
// error reporting, and the device-side requantization every epilogue uses.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "tvx_hip.h"

namespace tvx {

int SetError(int status, const char* fmt, ...);

#define TVX_HIP_CHECK(expr)                                                     \
  do {                                                                          \
    hipError_t e_ = (expr);                                                     \
    if (e_ != hipSuccess)                                                       \
      return ::tvx::SetError(TVX_E_DEVICE, "%s failed: %s (%s:%d)", #expr,      \
                             hipGetErrorString(e_), __FILE__, __LINE__);        \
  } while (0)

enum OpKind { OP_CONV2D = 1, OP_FC, OP_POOL2D, OP_ACTIVATION, OP_ADD, OP_SOFTMAX, OP_TRANSPOSE, OP_CONVERT, OP_DECONV2D };

// Device buffer owned by an operator, released in its destructor.
struct DeviceBuffer {
  void* ptr = nullptr;
  size_t bytes = 0;
  ~DeviceBuffer() { if (ptr) (void)hipFree(ptr); }
  DeviceBuffer() = default;
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  int Upload(const void* host, size_t n);
  int Alloc(size_t n);
  template <typename T> T* as() const { return static_cast<T*>(ptr); }
};

}  // namespace tvx

// The object behind the opaque handle. One `run` function per kernel variant.
struct tvx_op {
  int kind = 0;
  const char* kernel_name = "";
  int (*run)(tvx_op*, const void* in0, const void* in1, void* out, hipStream_t) = nullptr;
  const void* bias_at_run = nullptr;  // set by tvx_op_run3 for the duration of one enqueue
  int fused_add = 0;  // Conv2d + Add in one kernel: 1 = the convolution is the Add's first operand, 2 = its second (elt holds the Add)
  int fused_pool = 0;  // Conv2d + 2x2 / stride-2 max pooling in one kernel: the result has a quarter of conv's output pixels
  int fused_softmax = 0;  // FullyConnected + Softmax over its outputs in one kernel (sm holds the Softmax): fp32 result
  int out_blocked = 0;  // the result is written channel-blocked (the input is WHCN): set before a variant is asked

  tvx_conv2d_desc conv{};
  tvx_fc_desc fc{};
  tvx_pool2d_desc pool{};
  tvx_eltwise_desc elt{};
  tvx_softmax_desc sm{};
  tvx_transpose_desc tr{};
  tvx_convert_desc cv{};

  bool quantized = false;
  bool has_const_weights = false;
  int32_t act_lo = 0, act_hi = 0;  // output clamp incl. fused activation
  int32_t w_zp = 0;                // 0 for per-channel weights

  tvx::DeviceBuffer weights;  // as given (WHIcOc / {K,N})
  tvx::DeviceBuffer packed;   // variant-specific re-packed weights
  tvx::DeviceBuffer bias;     // int32 or float [oc]
  tvx::DeviceBuffer mult;     // int32 [oc]
  tvx::DeviceBuffer shift;    // int32 [oc]
  tvx::DeviceBuffer aux;      // variant-specific tables (e.g. folded bias)
  tvx::DeviceBuffer aux2;     // variant-specific tables (e.g. requantization records)
  tvx::DeviceBuffer aux3;     // variant-specific tables (e.g. reduction-order table)
  std::vector<int32_t> h_mult, h_shift;  // host copies of mult / shift
  std::vector<uint8_t> host_blob;        // variant-specific launch plan

  // variant-specific launch geometry
  int32_t geo[8] = {0};
};

namespace tvx {

// ---- device-side arithmetic -------------------------------------------------

// round_half_even(acc * mult / 2^shift); shift in [1, 62] (host guarantees it,
// larger shifts are delivered as mult = 0).
__device__ __forceinline__ int64_t RequantRne(int32_t acc, int32_t mult, int32_t shift) {
  const int64_t p = static_cast<int64_t>(acc) * static_cast<int64_t>(mult);
  int64_t fl = p >> shift;
  const int64_t rem = p & ((int64_t{1} << shift) - 1);
  const int64_t half = int64_t{1} << (shift - 1);
  if (rem > half || (rem == half && (fl & 1))) ++fl;
  return fl;
}

__device__ __forceinline__ int32_t RequantClamp(int32_t acc, int32_t mult, int32_t shift,
                                                int32_t zp, int32_t lo, int32_t hi) {
  int64_t r = RequantRne(acc, mult, shift) + zp;
  r = r < lo ? lo : (r > hi ? hi : r);
  return static_cast<int32_t>(r);
}

// ---- 32-bit requantization for MFMA epilogues ----------------------------------
// When every channel's shift is 32 + t with 1 <= t <= 20, round_half_even(acc * mult
// / 2^shift) + zp only needs the high half of the product: r = (hi + 2^(t-1) +
// (zp << t)) >> t rounds half up and adds the zero point; the low half matters on
// exact ties alone, which are fixed up (or proven impossible at creation).
// Record per channel: {mult, t (or the full shift in generic mode), rounding
// constant, mask of the accumulator bits that decide whether the low half is 0}.
typedef int tvx_v4i __attribute__((ext_vector_type(4)));
constexpr int kRqGeneric = 0;    // any shift: 64-bit product
constexpr int kRqFast = 1;       // high half of the product + tie fix-up
constexpr int kRqFastNoTie = 2;  // additionally no accumulator can land on a tie

// clamp(v, lo, hi) for lo <= hi in one instruction
__device__ __forceinline__ int Med3(int v, int lo, int hi) {
  int r;
  asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "v"(lo), "v"(hi));
  return r;
}

// a . b (four signed bytes each) + c into a new register: the three-address form. The builtin becomes the
// two-address v_dot4c, which needs a copy of c in front of it whenever c stays live (a bias shared by many outputs).
__device__ __forceinline__ int Dot4Add(int a, int b, int c) {
  int r;
  asm("v_dot4_i32_i8 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// The low bytes of four ints as one dword (a in byte 0).
__device__ __forceinline__ uint32_t PackBytes(int a, int b, int c, int d) {
  const uint32_t ab = __builtin_amdgcn_perm(static_cast<uint32_t>(b), static_cast<uint32_t>(a), 0x0c0c0400);
  const uint32_t cd = __builtin_amdgcn_perm(static_cast<uint32_t>(d), static_cast<uint32_t>(c), 0x0c0c0400);
  return __builtin_amdgcn_perm(cd, ab, 0x05040100);
}

// (v >> t) into byte E of d (the other bytes stay): the shift writes its result where the packed dword wants it.
// With the clamp in front of the shift (bounds shifted up: lo << t and (hi << t) | ((1 << t) - 1)) a requantized
// byte of the no-tie record form costs four instructions and no packing: high multiply, rounding constant, clamp, this.
template <int E>
__device__ __forceinline__ void ShiftIntoByte(uint32_t& d, int t, int v) {
  if (E == 0) asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD" : "=v"(d) : "v"(t), "v"(v));
  if (E == 1) asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(d) : "v"(t), "v"(v));
  if (E == 2) asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(d) : "v"(t), "v"(v));
  if (E == 3) asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(d) : "v"(t), "v"(v));
}

template <int RQ>
__device__ __forceinline__ int Requant8(int v, const tvx_v4i& q, int zp, int lo, int hi) {
  if (RQ == kRqGeneric) return RequantClamp(v, q[0], q[1], zp, lo, hi);
  const int h = __mulhi(v, q[0]);
  int r = (h + q[2]) >> q[1];
  if (RQ == kRqFast) {
    const int half = 1 << (q[1] - 1);
    const bool tie = ((h & (2 * half - 1)) == half) && ((v & q[3]) == 0);
    if (tie && ((r - zp) & 1)) --r;
  }
  return Med3(r, lo, hi);
}

// Four accumulators of one channel -> their four codes in one dword. Where no accumulator can land on a tie the clamp
// comes in front of the shift (bounds shifted up; a loop over the channel's pixels hoists them) and the shift writes
// its byte of the dword: four instructions a code - high multiply, rounding constant, clamp, shift - and no packing.
template <int RQ>
__device__ __forceinline__ uint32_t RequantPack4(const int (&v)[4], const tvx_v4i& q, int zp, int lo, int hi) {
  if (RQ == kRqFastNoTie) {
    const int lo_t = lo << q[1], hi_t = ((hi + 1) << q[1]) - 1;
    int u[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) u[e] = Med3(__mulhi(v[e], q[0]) + q[2], lo_t, hi_t);
    uint32_t d;
    ShiftIntoByte<0>(d, q[1], u[0]);
    ShiftIntoByte<1>(d, q[1], u[1]);
    ShiftIntoByte<2>(d, q[1], u[2]);
    ShiftIntoByte<3>(d, q[1], u[3]);
    return d;
  }
  int r[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) r[e] = Requant8<RQ>(v[e], q, zp, lo, hi);
  return PackBytes(r[0], r[1], r[2], r[3]);
}

// Four accumulators of one channel requantized together (the 32-bit record forms). `ties` (wave-uniform: a kernel
// argument) tells whether any accumulator of the operator can land on an exact .5: only then is the round-half-even
// fix-up executed.
__device__ __forceinline__ void Requant8x4(const int (&v)[4], const tvx_v4i& q, int zp, int lo, int hi, int ties,
                                           int (&out)[4]) {
  int h[4], r[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    h[e] = __mulhi(v[e], q[0]);
    r[e] = (h[e] + q[2]) >> q[1];
  }
  if (ties) {
    const int half = 1 << (q[1] - 1);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool tie = ((h[e] & (2 * half - 1)) == half) && ((v[e] & q[3]) == 0);
      if (tie && ((r[e] - zp) & 1)) --r[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) out[e] = Med3(r[e], lo, hi);
}

// ... and into one dword (`ties` as above: without ties the clamp-before-shift form, which needs no packing)
__device__ __forceinline__ uint32_t Requant8x4Pack(const int (&v)[4], const tvx_v4i& q, int zp, int lo, int hi, int ties) {
  if (!ties) return RequantPack4<kRqFastNoTie>(v, q, zp, lo, hi);
  int out[4];
  Requant8x4(v, q, zp, lo, hi, ties, out);
  return PackBytes(out[0], out[1], out[2], out[3]);
}

// The quantized Add fused behind a convolution: one code of the convolution's result (t) and one of the residual
// (r) -> the code of their sum, in the arithmetic of the stand-alone Add. `Args` carries add_mode (1: a = t, b = r;
// 2: a = r, b = t), add_signed, the zero points add_za / add_zb / add_zo, the ratios add_ra / add_rb and the clamp.
template <class Args>
__device__ __forceinline__ int AddResidual1(const Args& a, int t, int r) {
  if (a.add_signed) {
    t = static_cast<int8_t>(t);
    r = static_cast<int8_t>(r);
  }
  const int av = a.add_mode == 1 ? t : r, bv = a.add_mode == 1 ? r : t;
  const double tb = __dmul_rn(static_cast<double>(bv - a.add_zb), a.add_rb);
  const double s = fma(static_cast<double>(av - a.add_za), a.add_ra, tb);
  return Med3(static_cast<int>(rint(s)) + a.add_zo, a.add_lo, a.add_hi);
}
// ... on four codes in the bytes of a dword
template <class Args>
__device__ __forceinline__ uint32_t AddResidual4(const Args& a, uint32_t t4, uint32_t r4) {
  int out[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) out[e] = AddResidual1(a, static_cast<int>((t4 >> (8 * e)) & 0xff), static_cast<int>((r4 >> (8 * e)) & 0xff));
  return PackBytes(out[0], out[1], out[2], out[3]);
}

// 4 dwords = 4 channels x 4 pixels (pixel in the byte lanes) -> 4 dwords = 4 pixels x 4 channels.
__device__ __forceinline__ void Transpose4x4(const uint32_t in[4], uint32_t out[4]) {
  const uint32_t ab_lo = __builtin_amdgcn_perm(in[1], in[0], 0x05010400);  // a0 b0 a1 b1
  const uint32_t ab_hi = __builtin_amdgcn_perm(in[1], in[0], 0x07030602);  // a2 b2 a3 b3
  const uint32_t cd_lo = __builtin_amdgcn_perm(in[3], in[2], 0x05010400);
  const uint32_t cd_hi = __builtin_amdgcn_perm(in[3], in[2], 0x07030602);
  out[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100);  // a0 b0 c0 d0
  out[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302);
  out[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100);
  out[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302);
}

// bytes [IDX, IDX + 4) of the little-endian byte array formed by arr[0], arr[1], ...
template <int IDX, int N>
__device__ __forceinline__ int Window(const int (&arr)[N]) {
  constexpr int d = IDX / 4, sh = IDX % 4;
  static_assert(d + (sh ? 1 : 0) < N, "window outside the loaded dwords");
  if (sh == 0) return arr[d];
  return __builtin_amdgcn_alignbyte(arr[d + 1], arr[d], sh);
}

// ---- host helpers ------------------------------------------------------------
// Builds the records above for `alloc` channels (the first `channels` from the
// operator's mult/shift tables, the rest neutral) and returns the flavour.
// `acc_bound` (if >= 0) is the largest accumulator magnitude the operator can produce: ties
// that would need a larger accumulator are ruled out.
int BuildRequantRecords(const std::vector<int32_t>& mult, const std::vector<int32_t>& shift,
                        int channels, int alloc, int out_zp, std::vector<int32_t>* records,
                        int64_t acc_bound = -1);
// reduction length * 255 * 255 + max |bias|: bound of sum (x - zx)(w - zw) + bias for 8-bit operands
int64_t AccumulatorBound(uint64_t reduction, const void* bias_host, uint32_t channels);
// Per-output-channel requantization tables (mult/shift) for a conv / FC.
int BuildRequantTables(uint32_t channels, float in_scale, float w_scale,
                       const float* w_scales, float out_scale,
                       std::vector<int32_t>* mult, std::vector<int32_t>* shift);
void ActRange(int out_dtype, float out_scale, int32_t out_zp, int act, int32_t* lo, int32_t* hi);
inline bool IsQuant(int dtype) { return dtype == TVX_U8 || dtype == TVX_I8; }
inline size_t DtypeBytes(int dtype) {
  return dtype == TVX_F32 ? 4 : (dtype == TVX_F16 ? 2 : 1);
}

int ActivationSetup(tvx_op* op);
int AddSetup(tvx_op* op);
int SoftmaxSetup(tvx_op* op);

}  // namespace tvx
