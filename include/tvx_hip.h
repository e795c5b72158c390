/*
 * tvx_hip.h - C ABI between a TIM-VX graph runtime and the MI355X (gfx950)
 * kernels of the quantized convolution path.
 *
 * In the reference this seam is the OpenVX NN extension that ovxlib calls into
 * the closed Vivante driver. Each entry point below names the driver call it
 * stands in for. Like a vx_node, an operator is created once (weights are
 * re-packed, requantization tables are built, a kernel variant is chosen -
 * the work the driver does in vxVerifyGraph) and then run any number of times
 * (vxProcessGraph).
 *
 * Conventions: plain C, POD structs, device memory is passed as raw pointers,
 * `stream` is a hipStream_t passed as void* (NULL = the default stream).
 * Every function returns TVX_OK (0) or a negative tvx_status; tvx_last_error()
 * gives a text for the calling thread's last failure. *_run() only enqueues
 * work; the caller synchronizes. Nothing here allocates per run.
 *
 * Tensor layouts (dim 0 fastest, as everywhere in TIM-VX): activations WHCN,
 * convolution weights WHIcOc, depthwise weights {Kw, Kh, Ic*multiplier, 1},
 * fully-connected input {K, M}, weight {K, N}, output {N, M}.
 */
#ifndef TVX_HIP_H_
#define TVX_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum tvx_status {
  TVX_OK = 0,
  TVX_E_INVALID = -1,     /* bad argument / inconsistent descriptor */
  TVX_E_UNSUPPORTED = -2, /* valid request this library has no kernel for */
  TVX_E_DEVICE = -3,      /* HIP runtime failure, no usable GPU */
  TVX_E_NOMEM = -4
} tvx_status;

typedef enum tvx_dtype { TVX_U8 = 0, TVX_I8 = 1, TVX_F16 = 2, TVX_F32 = 3 } tvx_dtype;

/* Activation fused into the producing operator's epilogue
 * (stands in for the driver-side conv+relu fusion done inside vxVerifyGraph). */
typedef enum tvx_activation { TVX_ACT_NONE = 0, TVX_ACT_RELU = 1, TVX_ACT_RELU6 = 2 } tvx_activation;

/* vx_nn_pooling_type: include/VX/vx_khr_nn.h (VX_NN_POOLING_MAX/AVG/AVG_ANDROID);
 * numbering follows tim::vx::PoolType (include/tim/vx/types.h:62). */
typedef enum tvx_pool_type { TVX_POOL_MAX = 0, TVX_POOL_AVG = 1, TVX_POOL_L2 = 2, TVX_POOL_AVG_ANDROID = 3 } tvx_pool_type;

typedef struct tvx_op tvx_op; /* opaque operator (the vx_node analogue) */

/* ---- library / device ---------------------------------------------------- */
const char* tvx_version(void);
const char* tvx_last_error(void);
const char* tvx_status_string(int status);
/* Number of usable GPUs; 0 when there is none (never an error). */
int tvx_device_count(void);

/* Device memory and streams for runtimes that do not bring their own
 * (replaces the driver-owned tensor storage behind vxCreateTensor /
 * vxCopyTensorPatch: src/tim/vx/tensor.cc:154-228). */
int tvx_malloc(void** dev_ptr, size_t bytes);
int tvx_free(void* dev_ptr);
/* Page-locked host memory for tensors the application fills and reads (the host-visible buffers
 * behind vsi_nn_AddTensorFromHandle, src/tim/vx/tensor.cc:415-437): copies from and to it run at
 * the link's rate and without a staging copy. */
int tvx_host_malloc(void** host_ptr, size_t bytes);
int tvx_host_free(void* host_ptr);
int tvx_memcpy_h2d(void* dst_dev, const void* src_host, size_t bytes, void* stream);
int tvx_memcpy_d2h(void* dst_host, const void* src_dev, size_t bytes, void* stream);
int tvx_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream);
int tvx_stream_create(void** stream);
int tvx_stream_destroy(void* stream);
int tvx_stream_synchronize(void* stream);
/* Device-side time stamps on a stream, for per-node timing: what an OpenVX application reads back with
 * vxQueryNode(node, VX_NODE_PERFORMANCE, &vx_perf_t)
 * (prebuilt-sdk/x86_64_linux/include/VX/vx_types.h:1008,1692-1701). tvx_event_elapsed_ms needs both
 * events reached (synchronize the stream first). */
int tvx_event_create(void** event);
int tvx_event_destroy(void* event);
int tvx_event_record(void* event, void* stream);
int tvx_event_elapsed_ms(void* start, void* stop, float* ms);

/* ---- requantization (host side, no GPU needed) ---------------------------- */
/* real multiplier m (= s_in * s_w / s_out in double) -> mult * 2^-shift with
 * mult in [2^30, 2^31). The kernels apply it as one round-half-to-even right
 * shift of the 64-bit product acc * mult. */
int tvx_quantize_multiplier(double m, int32_t* mult, int32_t* shift);
/* The same fixed-point requantization the kernels' epilogues use, on the host:
 * round_half_even(acc * mult / 2^shift). */
int64_t tvx_requantize(int32_t acc, int32_t mult, int32_t shift);

/* ---- Conv2d (dense, 1x1, depthwise) --------------------------------------- */
/* Replaces vxConvolutionLayer(graph, inputs, weights, biases,
 * vx_nn_convolution_params_ext2_t{padding l/r/t/b, dilation, stride,
 * depth_multiplier, overflow/rounding policy}, outputs)
 * (prebuilt-sdk/x86_64_linux/include/VX/vx_khr_nn.h:738-824,835-873), as called
 * from src/tim/vx/internal/src/kernel/vx/convolutional.c:504-582. */
typedef struct tvx_conv2d_desc {
  uint32_t in_w, in_h, in_c, batch;
  uint32_t k_w, k_h;
  uint32_t out_w, out_h, out_c;
  uint32_t stride_w, stride_h;
  uint32_t dilation_w, dilation_h; /* >= 1 */
  uint32_t pad_left, pad_top;      /* right/bottom follow from out_w/out_h */
  int32_t multiplier;              /* 0 = dense; > 0 = depthwise, oc = ic*multiplier + j */
  int32_t in_dtype, w_dtype, out_dtype; /* tvx_dtype */
  float in_scale;
  int32_t in_zp;
  float w_scale;  /* per-tensor weight quantization ...                      */
  int32_t w_zp;
  const float* w_scales; /* ... or per-output-channel scales (host, out_c entries, zero point 0) */
  float out_scale;
  int32_t out_zp;
  int32_t activation; /* tvx_activation */
  /* grouped convolution (vx_nn_convolution_params_ext2_t has no such field: the reference
   * reaches it through its GROUPED_CONV2D operator, src/tim/vx/ops/groupedconv2d.cc): 0 or 1 =
   * ordinary; g > 1 = output channels [j*out_c/g, (j+1)*out_c/g) read input channels
   * [j*in_c/g, (j+1)*in_c/g) only and the weights are {k_w, k_h, in_c/g, out_c}. Needs
   * multiplier == 0 and g dividing in_c and out_c. */
  int32_t groups;
} tvx_conv2d_desc;

/* weights_host: WHIcOc image of the constant weights, or NULL when the weights
 * are a run-time tensor (then pass them to tvx_op_run as `in1`).
 * bias_host: int32 (quantized) or float (floating point) [out_c], or NULL. */
int tvx_conv2d_create(const tvx_conv2d_desc* desc, const void* weights_host,
                      const void* bias_host, tvx_op** op);

/* ---- FullyConnected ------------------------------------------------------- */
/* Replaces vxFullyConnectedLayer (vx_khr_nn.h:875-915) as called from
 * src/tim/vx/internal/src/ops/vsi_nn_op_fullconnect2.c:118-126:
 * out[m*N + n] = requant(sum_k (x[m*K+k]-zx)(w[n*K+k]-zw[n]) + bias[n]). */
typedef struct tvx_fc_desc {
  uint32_t m, k, n;
  int32_t in_dtype, w_dtype, out_dtype;
  float in_scale;
  int32_t in_zp;
  float w_scale;
  int32_t w_zp;
  const float* w_scales; /* per output feature (host, n entries) or NULL */
  float out_scale;
  int32_t out_zp;
  int32_t activation;
} tvx_fc_desc;

int tvx_fully_connected_create(const tvx_fc_desc* desc, const void* weights_host,
                               const void* bias_host, tvx_op** op);

/* ---- Pool2d ---------------------------------------------------------------- */
/* Replaces vxPoolingLayer2(graph, input, vx_nn_pooling_params_ext_t, output)
 * (vx_khr_nn.h:1696-1744) as called from
 * src/tim/vx/internal/src/ops/vsi_nn_op_pool.c:144-150. */
typedef struct tvx_pool2d_desc {
  uint32_t in_w, in_h, channels, batch;
  uint32_t out_w, out_h;
  uint32_t k_w, k_h, stride_w, stride_h, pad_left, pad_top;
  int32_t pool_type; /* tvx_pool_type */
  int32_t dtype;     /* input and output */
  float in_scale;
  int32_t in_zp;
  float out_scale;
  int32_t out_zp;
} tvx_pool2d_desc;

int tvx_pool2d_create(const tvx_pool2d_desc* desc, tvx_op** op);

/* ---- element-wise ---------------------------------------------------------- */
/* Standalone ReLU / ReLU6: replaces vxActivationLayer(RELU / RELU6)
 * (src/tim/vx/internal/src/ops/vsi_nn_op_relu.c:48-55,
 *  src/tim/vx/internal/src/kernel/vx/eltwise_unary_vx.c:333-352). */
typedef struct tvx_eltwise_desc {
  uint64_t count;
  int32_t dtype;
  int32_t activation; /* activation op: which clamp */
  float a_scale;
  int32_t a_zp;
  float b_scale; /* second operand (Add only) */
  int32_t b_zp;
  float out_scale;
  int32_t out_zp;
} tvx_eltwise_desc;

int tvx_activation_create(const tvx_eltwise_desc* desc, tvx_op** op);
/* Same-shape Add: replaces vxTensorAddNode
 * (src/tim/vx/internal/src/kernel/vx/eltwise_vx.c:56-67). */
int tvx_add_create(const tvx_eltwise_desc* desc, tvx_op** op);

/* Softmax along one axis of a tensor viewed as {inner, channels, rows} (inner fastest: the
 * product of the dimensions below the axis, 0 or 1 for axis 0), fp32 output: replaces
 * vxSoftmaxLayer2 (src/tim/vx/internal/src/kernel/vx/softmax_vx.c:88). */
typedef struct tvx_softmax_desc {
  uint32_t channels;
  uint64_t rows;
  float beta;
  int32_t in_dtype;
  float in_scale;
  int32_t in_zp;
  uint64_t inner;
} tvx_softmax_desc;

int tvx_softmax_create(const tvx_softmax_desc* desc, tvx_op** op);

/* ---- Conv2d + Add in one kernel -------------------------------------------------------- */
/* A convolution whose result only feeds a same-shape Add (the residual connection of an inverted
 * residual block): two nodes of the reference's graph (vxConvolutionLayer, then vxTensorAddNode:
 * src/tim/vx/internal/src/kernel/vx/eltwise_vx.c:56-67) as one operator whose result is, bit for
 * bit, what the two would give (the convolution's result quantized to its own output tensor
 * first). `conv` describes the convolution as for tvx_conv2d_create, `add` the Add (dtype,
 * a_* / b_* / out_* quantization; count and activation are ignored), conv_operand says which
 * operand of the Add the convolution is (1 or 2); the other operand goes in as in1 of
 * tvx_op_run. Returns TVX_E_UNSUPPORTED when no kernel fuses this convolution (the caller then
 * creates the two operators). */
int tvx_conv2d_add_create(const tvx_conv2d_desc* conv, const tvx_eltwise_desc* add, int conv_operand,
                          const void* weights_host, const void* bias_host, tvx_op** op);

/* ---- depthwise 3x3 Conv2d + the 1x1 Conv2d it only feeds, in one kernel ------------------- */
/* Two nodes of the reference's graph (vxConvolutionLayer twice: kernel/vx/convolutional.c:504-582, the
 * first through the "depthwise_conv2d" backend) whose intermediate tensor has no other reader: the closed
 * driver merges such layers when it verifies the graph (src/tim/vx/internal/src/vsi_nn_graph.c:1591-1603).
 * The result is, bit for bit, what the two operators give one after the other - the depthwise result is
 * quantized to its own tensor (dw->out_scale / out_zp, clamped by dw->activation) before the pointwise
 * convolution reads it - but that tensor never reaches memory. `dw` and `pw` describe the two convolutions
 * as for tvx_conv2d_create (pw's input is dw's output: same shape, type and quantization); `add` (may be
 * NULL) is a residual Add behind the pointwise convolution as in tvx_conv2d_add_create, its other operand
 * going in as in1 of tvx_op_run. Returns TVX_E_UNSUPPORTED when no kernel fuses this pair (the caller
 * then creates the operators one by one). */
int tvx_conv2d_dw_pw_create(const tvx_conv2d_desc* dw, const void* dw_weights_host, const void* dw_bias_host,
                            const tvx_conv2d_desc* pw, const void* pw_weights_host, const void* pw_bias_host,
                            const tvx_eltwise_desc* add, int conv_operand, tvx_op** op);

/* ---- an inverted-residual block: 1x1 Conv2d, depthwise 3x3 Conv2d, 1x1 Conv2d (+ Add) in one kernel ---- */
/* Three (four) nodes of the reference's graph (vxConvolutionLayer: kernel/vx/convolutional.c:504-582, and
 * vxTensorAdd behind them) whose two intermediate tensors have no other reader - the chain the closed driver
 * merges at verification (src/tim/vx/internal/src/vsi_nn_graph.c:1591-1603). The result is, bit for bit,
 * what the operators give one after the other: each intermediate is quantized to its own tensor (out_scale /
 * out_zp, clamped by the stage's activation) before the next stage reads it, but neither reaches memory.
 * `expand`, `dw` and `project` describe the convolutions as for tvx_conv2d_create (each stage's input is the
 * previous stage's output); `add` (may be NULL) is the residual Add behind the projection as in
 * tvx_conv2d_add_create, its other operand going in as in1 of tvx_op_run. Returns TVX_E_UNSUPPORTED when no
 * kernel fuses this block (the kernel covers feature maps 28, 14 or 7 columns wide, SAME depthwise padding,
 * at most 160 input and 320 output channels, and by default claims only the 14-column stride-1 blocks, where
 * it is faster than the three launches; the caller then creates the operators one by one). */
int tvx_mbconv_create(const tvx_conv2d_desc* expand, const void* expand_weights_host, const void* expand_bias_host,
                      const tvx_conv2d_desc* dw, const void* dw_weights_host, const void* dw_bias_host,
                      const tvx_conv2d_desc* project, const void* project_weights_host, const void* project_bias_host,
                      const tvx_eltwise_desc* add, int conv_operand, tvx_op** op);

/* ---- Conv2d + the 2x2 / stride-2 max pooling it only feeds, in one kernel ------------------------------ */
/* Two nodes of the reference's graph (vxConvolutionLayer: kernel/vx/convolutional.c:504-582, then
 * vxPoolingLayer2: src/tim/vx/internal/src/ops/vsi_nn_op_pool.c:144-150) whose intermediate tensor has no
 * other reader - LeNet's conv1 / pool1 and conv2 / pool2 (samples/lenet/lenet_asymu8.cc:248-272); the closed
 * driver merges such layers when it verifies the graph (src/tim/vx/internal/src/vsi_nn_graph.c:1591-1603).
 * The result is, bit for bit, what the two operators give one after the other (requantization is monotone, so
 * the maximum of the four accumulators is requantized once). `conv` describes the convolution as for
 * tvx_conv2d_create, `pool` the pooling as for tvx_pool2d_create: MAX, 2 x 2 window, stride 2, no padding,
 * input = the convolution's output (even extents) with the same type and quantization on both sides.
 * Returns TVX_E_UNSUPPORTED when no kernel fuses this pair (the caller then creates the two operators). */
int tvx_conv2d_pool_create(const tvx_conv2d_desc* conv, const tvx_pool2d_desc* pool, const void* weights_host,
                           const void* bias_host, tvx_op** op);

/* ---- FullyConnected + the Softmax over its outputs, in one kernel -------------------------------------- */
/* Two nodes of the reference's graph (vxFullyConnectedLayer: kernel/vx/convolutional.c:584-652, then
 * vxSoftmaxLayer2: src/tim/vx/internal/src/kernel/vx/softmax_vx.c:88) - the classifier head of LeNet
 * (samples/lenet/lenet_asymu8.cc:283-290): a quantized FullyConnected layer with at most 16 outputs whose
 * codes only feed a Softmax along that axis. The result (fp32) is, bit for bit, what the two operators give
 * one after the other. `fc` as for tvx_fully_connected_create (constant weights), `softmax` as for
 * tvx_softmax_create with channels = fc->n, rows = fc->m, inner <= 1 and the FullyConnected output's type and
 * quantization as its input's. Returns TVX_E_UNSUPPORTED otherwise (the caller then creates the two operators). */
int tvx_fully_connected_softmax_create(const tvx_fc_desc* fc, const tvx_softmax_desc* softmax,
                                       const void* weights_host, const void* bias_host, tvx_op** op);

/* ---- DeConv2d (transposed convolution) ----------------------------------------------- */
/* Replaces vxDeconvolutionLayer (src/tim/vx/ops/deconv.cc:45-79,
 * src/tim/vx/internal/src/ops/vsi_nn_op_deconvolution.c:217-218,398-497). Same descriptor as
 * Conv2d, read the other way round: input pixel (ix, iy) adds in * w[kx, ky] to output pixel
 * (ix * stride - pad_left + kx, iy * stride - pad_top + ky); weights {k_w, k_h, in_c / groups,
 * out_c} as the reference's WHIcOc deconvolution kernel, {k_w, k_h, out_c, 1} with
 * multiplier = 1 for the depthwise form (group == channels); dilation must be 1. The output
 * extent is the caller's: (in - 1) * stride + k - pads + output_padding, or anything smaller. */
int tvx_deconv2d_create(const tvx_conv2d_desc* desc, const void* weights_host, const void* bias_host,
                        tvx_op** op);

/* ---- DataConvert ------------------------------------------------------------------ */
/* Replaces the DATACONVERT operator (src/tim/vx/ops/simple_operations.cc:39 -> vxTensorCopyNode /
 * the conversions of src/tim/vx/internal/include/utils/vsi_nn_dtype_util_prv.h:228-266): every
 * element goes to float32 ((q - zp) * scale, or the float value) and from there to the output
 * type (rint(f / scale) + zp, saturated to the type's range; rounded to nearest even for
 * float16). Any pair of the four tensor types. */
typedef struct tvx_convert_desc {
  uint64_t count;
  int32_t in_dtype;
  float in_scale;
  int32_t in_zp;
  int32_t out_dtype;
  float out_scale;
  int32_t out_zp;
} tvx_convert_desc;

int tvx_convert_create(const tvx_convert_desc* desc, tvx_op** op);

/* ---- Transpose (permute) ----------------------------------------------------- */
/* Replaces the PERMUTE operator (src/tim/vx/ops/transpose.cc -> vxTensorPermuteNode):
 * output dimension i is input dimension perm[i] (out.size[i] = in.size[perm[i]],
 * src/tim/vx/internal/src/ops/vsi_nn_op_permute.c:219-230), dimension 0 fastest. Elements
 * are moved as they are (any type of elem_bytes 1, 2 or 4). */
typedef struct tvx_transpose_desc {
  uint32_t rank;       /* 1..6 */
  uint32_t in_dims[6];
  uint32_t perm[6];
  uint32_t elem_bytes;
} tvx_transpose_desc;

int tvx_transpose_create(const tvx_transpose_desc* desc, tvx_op** op);

/* ---- channel-blocked tensors ------------------------------------------------------------------- */
/* A TRANSIENT tensor of the reference's graph has no host image (src/tim/vx/tensor.cc: its data can neither
 * be written nor read by the application), so the order of its bytes is the runtime's own business, as it is
 * the closed driver's. For one-byte codes on small planes (7 x 7: 49-byte rows that no load is aligned to) this
 * library offers
 *   byte ((c / 16) * P + p) * 16 + c % 16,  p = n * H * W + y * W + x,  P = N * H * W   (channels a multiple of 16)
 * and operators between such tensors whose results are, code for code, those of the WHCN operators:
 *  - tvx_conv2d_blocked_create: vxConvolutionLayer (kernel/vx/convolutional.c:504-582) for a 1x1 / stride-1 /
 *    unpadded dense convolution (input and output channels multiples of 32), optionally with the same-shape Add
 *    behind it (`add` / `conv_operand` as for tvx_conv2d_add_create, the other operand - blocked - as in1; NULL:
 *    no Add), or for a depthwise 3x3 / stride-1 convolution (multiplier 1, `add` NULL); constant weights;
 *  - tvx_pool2d_blocked_create: vxPoolingLayer2 (ops/vsi_nn_op_pool.c:144-150) averaging whole unpadded planes of
 *    at most 256 pixels: blocked in, {1, 1, C, N} out in WHCN order (byte n * C + c);
 *  - tvx_conv2d_to_blocked_create: the same vxConvolutionLayer for a depthwise 3x3 convolution (multiplier 1, stride 1
 *    or 2, constant weights, channels a multiple of 16, planes that fit the LDS-staged kernel) that reads a WHCN tensor
 *    and writes its result blocked: the way into a run of blocked operators without a copy;
 *  - tvx_layout_create: WHCN -> blocked (to_blocked != 0) or back; no counterpart in the reference's API.
 * TVX_E_UNSUPPORTED: no blocked kernel for this operator (the caller keeps the tensor in WHCN). */
int tvx_conv2d_blocked_create(const tvx_conv2d_desc* conv, const tvx_eltwise_desc* add, int conv_operand,
                              const void* weights_host, const void* bias_host, tvx_op** op);
int tvx_conv2d_to_blocked_create(const tvx_conv2d_desc* conv, const void* weights_host, const void* bias_host, tvx_op** op);
int tvx_pool2d_blocked_create(const tvx_pool2d_desc* desc, tvx_op** op);
int tvx_layout_create(uint32_t w, uint32_t h, uint32_t c, uint32_t n, int to_blocked, tvx_op** op);

/* ---- running / inspecting operators ---------------------------------------- */
/* Enqueue one execution (the per-node share of vxProcessGraph).
 * in0: activation; in1: run-time weights (conv / FC created without constant
 * weights) or the second Add operand, else NULL; out: result. All device
 * pointers, sized by the operator's descriptor. */
int tvx_op_run(tvx_op* op, const void* in0, const void* in1, void* out, void* stream);
/* The same with a third operand: the bias of a Conv2d / FullyConnected whose weights are given
 * at run time too (created with weights_host == NULL and bias_host == NULL), int32 for quantized
 * tensors, float32 otherwise. This is the reference's convolution whose weight and bias tensors
 * are graph inputs (src/tim/transform/layout_inference_test.cc:65-121). in2 == NULL is
 * tvx_op_run. */
int tvx_op_run3(tvx_op* op, const void* in0, const void* in1, const void* in2, void* out, void* stream);
/* Name of the kernel variant chosen at creation, e.g. "conv2d_generic". */
const char* tvx_op_kernel_name(const tvx_op* op);
void tvx_op_destroy(tvx_op* op);

#ifdef __cplusplus
}
#endif
#endif /* TVX_HIP_H_ */
