// Measurement aids: what this very GPU sustains on the two resources the kernels are
// priced against, measured with the simplest possible kernels.
//
//  * tvx_calibrate_mfma_i8: v_mfma_i32_32x32x32_i8 issued back to back from registers
//    (16 independent accumulators per wavefront, one wavefront per SIMD, every CU busy).
//    With all-zero operands the loop runs at the nominal rate; with random operands the
//    chip lowers its clock under the switching power of the multipliers, and that lower
//    figure is what any real int8 GEMM on this device can approach.
//  * tvx_calibrate_copy: a plain 16-bytes-per-lane streaming copy, read + write bytes per
//    second.
//
// Built as its own small library (libtvx_calibrate.so) for the benchmark: it is not part of
// the operator library or of its C ABI. Both functions return 0, or -1 after printing the
// reason to stderr.
#include <cstdint>
#include <vector>

#include <hip/hip_runtime.h>

#include <cstdio>

namespace {

int Fail(const char* what) {
  std::fprintf(stderr, "tvx_calibrate: %s\n", what);
  return -1;
}


typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kMfmaPerIter = 64;

__global__ void __launch_bounds__(256, 1) MfmaRateKernel(const v4i* operands, int* sink, int iters) {
  const int lane = threadIdx.x & 63;
  v4i fa[4], fb[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    fa[t] = operands[(t * 64 + lane) & 1023];
    fb[t] = operands[(256 + t * 64 + lane) & 1023];
  }
  v16i acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int rep = 0; rep < kMfmaPerIter / 16; ++rep)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i * 4 + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i * 4 + j], 0, 0, 0);
  }
  int s = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

__global__ void __launch_bounds__(256) CopyKernel(const v4i* __restrict__ src, v4i* __restrict__ dst, size_t n16) {
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// Runs `launch` once untimed and then `launches` times between two events on the null stream.
template <typename F>
int TimeLaunches(int launches, F launch, double* ms_per_launch) {
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)
    return Fail("calibration: hipEventCreate failed");
  launch();
  hipError_t err = hipDeviceSynchronize();
  if (err == hipSuccess) err = hipEventRecord(e0, nullptr);
  for (int i = 0; i < launches; ++i) launch();
  if (err == hipSuccess) err = hipEventRecord(e1, nullptr);
  if (err == hipSuccess) err = hipEventSynchronize(e1);
  float ms = 0;
  if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (err != hipSuccess || hipGetLastError() != hipSuccess) return Fail("calibration: launch or timing failed");
  *ms_per_launch = ms / launches;
  return 0;
}

}  // namespace

extern "C" int tvx_calibrate_mfma_i8(int random_operands, int launches, double* tops) {
  if (!tops || launches < 1 || launches > 1000) return Fail("tvx_calibrate_mfma_i8: bad argument");
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return Fail("tvx_calibrate_mfma_i8: no GPU");
  const int wgs = prop.multiProcessorCount, iters = 500;
  std::vector<uint32_t> host(4096, 0u);
  if (random_operands) {
    uint64_t s = 0x9E3779B97F4A7C15ull;  // xorshift64*: any fixed non-trivial bit pattern will do
    for (auto& v : host) {
      s ^= s >> 12; s ^= s << 25; s ^= s >> 27;
      v = static_cast<uint32_t>((s * 0x2545F4914F6CDD1Dull) >> 32);
    }
  }
  void *ops = nullptr, *sink = nullptr;
  if (hipMalloc(&ops, host.size() * 4) != hipSuccess || hipMalloc(&sink, static_cast<size_t>(wgs) * 256 * 4) != hipSuccess) {
    (void)hipFree(ops);
    return Fail("tvx_calibrate_mfma_i8: allocation failed");
  }
  int st = hipMemcpy(ops, host.data(), host.size() * 4, hipMemcpyHostToDevice) == hipSuccess ? 0
                                                                                                : Fail("tvx_calibrate_mfma_i8: upload failed");
  double ms = 0;
  if (st == 0)
    st = TimeLaunches(launches, [&] {
      hipLaunchKernelGGL(MfmaRateKernel, dim3(wgs), dim3(256), 0, nullptr, static_cast<const v4i*>(ops), static_cast<int*>(sink), iters);
    }, &ms);
  (void)hipFree(ops);
  (void)hipFree(sink);
  if (st != 0) return st;
  const double ops_per_launch = 2.0 * 32 * 32 * 32 * kMfmaPerIter * iters * 4.0 * wgs;
  *tops = ops_per_launch / (ms * 1e-3) / 1e12;
  return 0;
}

extern "C" int tvx_calibrate_copy(size_t bytes, int launches, double* gb_per_s) {
  if (!gb_per_s || launches < 1 || launches > 1000 || bytes < 4096 || (bytes & 15))
    return Fail("tvx_calibrate_copy: bad argument");
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return Fail("tvx_calibrate_copy: no GPU");
  void *src = nullptr, *dst = nullptr;
  if (hipMalloc(&src, bytes) != hipSuccess || hipMalloc(&dst, bytes) != hipSuccess) {
    (void)hipFree(src);
    return Fail("tvx_calibrate_copy: allocation failed");
  }
  int st = hipMemset(src, 3, bytes) == hipSuccess ? 0 : Fail("tvx_calibrate_copy: memset failed");
  double ms = 0;
  const int wgs = prop.multiProcessorCount * 8;
  if (st == 0)
    st = TimeLaunches(launches, [&] {
      hipLaunchKernelGGL(CopyKernel, dim3(wgs), dim3(256), 0, nullptr, static_cast<const v4i*>(src), static_cast<v4i*>(dst), bytes / 16);
    }, &ms);
  (void)hipFree(src);
  (void)hipFree(dst);
  if (st != 0) return st;
  *gb_per_s = 2.0 * static_cast<double>(bytes) / (ms * 1e-3) / 1e9;
  return 0;
}
