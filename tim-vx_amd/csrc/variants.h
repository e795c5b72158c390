// Registry of kernel variants. Each setup function inspects the operator at
// creation and either claims it (TVX_OK: packs weights, fills op->run and
// op->kernel_name), declines (TVX_E_UNSUPPORTED: the next variant is asked),
// or fails (any other status aborts creation). Lists are ordered fastest
// first; the generic variant at the end accepts everything the descriptor
// checks let through.
#pragma once

#include <vector>

#include "tvx_internal.h"

namespace tvx {

typedef int (*ConvSetupFn)(tvx_op*, const tvx_conv2d_desc*, const void* weights_host,
                           const void* bias_host);
typedef int (*FcSetupFn)(tvx_op*, const tvx_fc_desc*, const void* weights_host,
                         const void* bias_host);
typedef int (*SimpleSetupFn)(tvx_op*);

const std::vector<ConvSetupFn>& ConvVariants();
const std::vector<FcSetupFn>& FcVariants();
const std::vector<SimpleSetupFn>& PoolVariants();

// int8 MFMA fully-connected (fc_mfma_i8.hip)
int FcMfmaSetup(tvx_op*, const tvx_fc_desc*, const void*, const void*);

// int8 MFMA implicit-GEMM convolution (conv_igemm_i8.hip)
int ConvIgemmSetup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);
// the same for layers whose weights and two halo tiles fit LDS: one sixteen-wavefront workgroup per CU (conv_band_i8.hip)
int ConvBandSetup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);
// Dense quantized conv whose whole window (C * Kh * Kw) is at most 64 bytes: im2col rows in LDS + MFMA.
int ConvIm2colSetup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);

// pointwise (1x1) convolution with the whole channel depth of a pixel tile in LDS (pwconv_i8.hip)
int PwConvSetup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);

// depthwise 3x3 stencil (dwconv3x3_i8.hip)
int DwConv3x3Setup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);

// convolutions, whole-plane average pooling and the layout change on channel-blocked tensors (blocked_i8.hip)
int BlockedPwSetup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);
int BlockedDwSetup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);
int BlockedAvgSetup(tvx_op*);
int LayoutSetup(tvx_op*, uint32_t w, uint32_t h, uint32_t c, uint32_t n, int to_blocked);

// depthwise, any kernel / width, planes staged through LDS (dwconv_planes_i8.hip)
int DwPlanesSetup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);
// shared by the two depthwise 3x3 stencils (defined in dwconv3x3_i8.hip)
bool PackDepthwise3x3(int C, const void* w_host, bool w_u8, const void* bias_host, int zxs, int zws,
                      bool all_or_none, std::vector<int32_t>* wpk, std::vector<int32_t>* biasf);

// depthwise 3x3 + pointwise convolution in one kernel (dwpw_i8.hip); `op` carries the pointwise half
int DwPwSetup(tvx_op* op, const tvx_conv2d_desc* dw, const void* dw_w, const void* dw_b,
              const std::vector<int32_t>& dw_mult, const std::vector<int32_t>& dw_shift, int dw_lo, int dw_hi,
              const tvx_conv2d_desc* pw, const void* pw_w, const void* pw_b);

// an inverted-residual block - 1x1 expansion, depthwise 3x3, 1x1 projection (+ Add) - in one kernel (mbconv_i8.hip);
// `op` carries the projection, the two stages in front of it come with their own tables
struct MbStage {
  const tvx_conv2d_desc* desc;
  const void* w;
  const void* b;
  const std::vector<int32_t>* mult;
  const std::vector<int32_t>* shift;
  int32_t lo, hi;  // output clamp incl. the stage's activation
};
int MbConvSetup(tvx_op* op, const MbStage& expand, const MbStage& depthwise, const tvx_conv2d_desc* project,
                const void* project_w, const void* project_b);

// convolution as a GEMM over gathered windows: grouped, dilated, float16 (conv_gemm.hip)
// dense float16 convolution, halo rows staged in LDS once (conv_igemm_f16.hip)
int ConvIgemmF16Setup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);
int ConvGemmSetup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);

// generic (kernels_generic.hip)
int ConvGenericSetup(tvx_op*, const tvx_conv2d_desc*, const void*, const void*);
int FcGenericSetup(tvx_op*, const tvx_fc_desc*, const void*, const void*);
// FullyConnected with at most 16 outputs + the Softmax over them, a wavefront per row (kernels_generic.hip)
int FcSoftmaxSetup(tvx_op*, const tvx_fc_desc*, const void*, const void*);
int PoolGenericSetup(tvx_op*);
// quantized pooling, windows two or three taps wide, planes staged through LDS (pool2d_i8.hip)
int PoolRowsSetup(tvx_op*);
// quantized MAX pooling at stride 2, windows of 2 or 3 taps, rows of whole 8-byte units: register stencil (pool2d_stencil_i8.hip)
int PoolStencilSetup(tvx_op*);
int TransposeSetup(tvx_op*);
int ConvertSetup(tvx_op*);

}  // namespace tvx
