/*
 * catchq.h -- C ABI of the MI355X (gfx950) fixed-point quantized-inference kernels.
 *
 * Drop-in boundary for the quantized hot path of Cambricon/catch (torch_mlu): each
 * entry point replaces one vendor-library call (or one group of small tensor ops)
 * that the reference's op wrappers make.  Citations are file:line in the
 * reference tree, below torch_mlu/csrc/aten/ unless a longer path is given.
 *
 * Conventions
 *   - plain pointers and sizes only; every device buffer (inputs, outputs,
 *     workspace) is owned by the caller; nothing here allocates or frees;
 *   - all device entry points are asynchronous on `stream` (a hipStream_t passed
 *     as void*; NULL = the null stream).  They are re-entrant and keep no state from call to
 *     call, with one documented exception: the fixed scratch memory of
 *     catchq_quantize_param_noalloc (per device, calls on one device must not overlap);
 *   - the return value is a status (0 = CATCHQ_OK); no exception crosses the
 *     boundary; catchq_status_string() names a status;
 *   - activations are NHWC, convolution weights [Co][kh][kw][Ci/groups]
 *     (= the memory of a channels-last [Co,Ci/g,kh,kw] tensor), GEMM operands
 *     row-major with K contiguous (A [M,K], B [N,K]).
 */
#ifndef CATCHQ_H_
#define CATCHQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *catchq_stream_t;

enum {
  CATCHQ_OK = 0,
  CATCHQ_ERR_ARG = 1,         /* null pointer, negative size, bad enum */
  CATCHQ_ERR_DTYPE = 2,       /* "quantify only support input float/half" (operators/cnnl/internal/quantify.cpp:73-74) */
  CATCHQ_ERR_BITWIDTH = 3,    /* "bitwidth not support" (operators/cnnl/internal/quantify.cpp:63) */
  CATCHQ_ERR_SHAPE = 4,       /* inconsistent shapes (groups, output extent <= 0, ...) */
  CATCHQ_ERR_LAUNCH = 5,      /* the HIP runtime refused the launch */
  CATCHQ_ERR_UNSUPPORTED = 6, /* combination not implemented */
  CATCHQ_ERR_TOO_LARGE = 7    /* input larger than the fixed scratch memory of a *_noalloc entry point serves */
};

enum { CATCHQ_F32 = 0, CATCHQ_F16 = 1 };
enum { CATCHQ_ACT_NONE = 0, CATCHQ_ACT_RELU = 1, CATCHQ_ACT_RELU6 = 2, CATCHQ_ACT_LEAKY = 3 };
/* cnnlQuantizeMode_t values used by the reference (operators/cnnl/internal/quantize_param.cpp:70-78) */
enum { CATCHQ_QUANTIZE_POSITION = 0, CATCHQ_QUANTIZE_POSITION_SCALE = 1, CATCHQ_QUANTIZE_POSITION_SCALE_OFFSET = 2 };

int catchq_version(void);
const char *catchq_status_string(int status);

/* ------------------------------------------------------------------ host q-param math */

/* get_pos_from_scale_data(bitwidth, scale_data)            cnnl/cnnl_util.cpp:337-347 */
int catchq_pos_from_scale(int bitwidth, float scale, int *position);

/* setQuantizedParams(scale, qmode, ...)                    torch_mlu/csrc/jit/utils/utils.cpp:81-105
 * position, fractional scale 2^pos*qmax/absmax and scale_factor 2^pos/scale_. */
int catchq_quant_params(int bitwidth, float scale, int *position, float *scale_frac, float *scale_factor);

/* the parameter part of cnnl_quantify_per_channel          operators/cnnl/quantify.cpp:55-98
 * scales[co] (= qmax/absmax_c) -> shared new_position, new_scale[co], scale_factor[co] (host arrays). */
int catchq_per_channel_params(int bitwidth, const float *scales, int co, int *new_position,
                              float *new_scale, float *scale_factor);

/* The same derivation for a model converted with .half(): scale_data is then a half tensor and every
 * tensor op of operators/cnnl/quantify.cpp:64-98 rounds to binary16 (absmax, log2, position, scale, new_scale,
 * scale_factor).  scales / new_scale / scale_factor hold binary16 bit patterns (host arrays).  A scale that is
 * not finite in binary16 (an int16 scale 32767/absmax above 65504) returns CATCHQ_ERR_ARG. */
int catchq_per_channel_params_f16(int bitwidth, const uint16_t *scales, int co, int *new_position,
                                  uint16_t *new_scale, uint16_t *scale_factor);

/* ------------------------------------------------------------------ quantize / dequantize */

/* cnnl_quantify_offline_internal(input, bitwidth, int position) -> cnnlQuantizeV1
 *                                                          operators/cnnl/internal/quantify.cpp:69-101
 * q[i] = sat(rne(x[i] * scale * 2^-position)); x fp32/fp16, q int8 / int16 / int32 (bitwidth 8/16/31).
 * The reference's eager path passes scale = 1. */
int catchq_quantize(const void *x, int x_dtype, void *q, int bitwidth, int64_t n, int position,
                    float scale, catchq_stream_t stream);

/* cnnl_quantify_offline_internal(input, bitwidth, Tensor position) -> cnnlQuantizeV2
 *                                                          operators/cnnl/internal/quantify.cpp:103-137
 * same, position (and optionally scale) read from device memory: no host sync. scale_dev may be NULL (=1). */
int catchq_quantize_devpos(const void *x, int x_dtype, void *q, int bitwidth, int64_t n,
                           const int32_t *position_dev, const float *scale_dev, catchq_stream_t stream);

/* cnnl_contiguous(input, ChannelsLast) followed by cnnl_quantify_offline
 *                                                          operators/cnnl/quantify_conv_forward.cpp:62-63,97
 * x [N,C,H,W] contiguous -> q [N,H,W,cpad] (channels C..cpad-1 zero), in one pass. */
int catchq_quantize_nchw_to_nhwc(const void *x, int x_dtype, void *q, int bitwidth, int n, int c, int h,
                                 int w, int cpad, int position, float scale, catchq_stream_t stream);

/* The same, written into a zero frame: q [N, out_h, out_w, cpad] holds the image at rows top.., columns
 * left.. and zeros elsewhere -- the zero padding of the convolution that follows
 * (convolution_forward_internal.cpp:150-153 passes it to the vendor descriptor), materialised once so that a
 * few-channel first layer can fetch whole filter rows with plain loads.  cpad 4 (int8) or 8. */
int catchq_quantize_nchw_to_nhwc_frame(const void *x, int x_dtype, void *q, int bitwidth, int n, int c, int h,
                                       int w, int cpad, int out_h, int out_w, int top, int left, int position,
                                       float scale, catchq_stream_t stream);

/* cnnlGetQuantizeParamWorkspaceSize + cnnl_quantize_param -> cnnlQuantizeParam
 *                                                          operators/cnnl/internal/quantize_param.cpp:39-96
 * max-abs reduction, then position (mode 0), + scale (1), + offset = 0 (2) written to device memory.
 * absmax_dev / scale_dev / offset_dev may be NULL.  The vendor formula is not in the reference tree;
 * defined as position = floor(log2(absmax)) - (bitwidth-2), scale = 2^position*qmax/absmax. */
int catchq_quantize_param_workspace_size(int64_t n, size_t *bytes);
int catchq_quantize_param(const void *x, int x_dtype, int64_t n, int bitwidth, int mode, void *workspace,
                          size_t workspace_bytes, float *absmax_dev, int32_t *position_dev,
                          float *scale_dev, float *offset_dev, catchq_stream_t stream);

/* catchq_quantize_param for callers that cannot allocate device memory or bring a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference, whose wrapper allocates the vendor workspace on every call (operators/cnnl/internal/quantize_param.cpp:67-83).
 * Same kernels, same results bit for bit; the per-block partial maxima go to a fixed 16 KiB array in
 * device memory that every device the library runs on holds until the process ends.  The call allocates
 * and frees nothing.  n above CATCHQ_QUANTIZE_PARAM_NOALLOC_MAX_N returns CATCHQ_ERR_TOO_LARGE.  All
 * calls on one device share that array: two calls whose kernels may run at the same time on one device
 * (different streams, different threads) race; calls on one stream are ordered and safe.  Nothing of an
 * earlier call's contents is read, so no clearing happens between calls.  The first call on a device
 * looks the array's address up (hipGetSymbolAddress); make that call outside a stream capture. */
#define CATCHQ_QUANTIZE_PARAM_NOALLOC_MAX_N (INT64_C(1) << 40)
int catchq_quantize_param_noalloc(const void *x, int x_dtype, int64_t n, int bitwidth, int mode,
                                  float *absmax_dev, int32_t *position_dev, float *scale_dev,
                                  float *offset_dev, catchq_stream_t stream);

/* the elementwise part of cnnl_quantify_per_channel        operators/cnnl/quantify.cpp:100-112
 * q[c, i] = sat(rne(w[c, i] / scale_factor[c])), w [co, inner] fp32/fp16, scale_factor on the device. */
int catchq_quantize_per_channel(const void *w, int w_dtype, void *q, int bitwidth, int co, int64_t inner,
                                const float *scale_factor_dev, catchq_stream_t stream);

/* The same with half tensors on both sides (weight and scale_factor binary16, as after .half()): the quotient
 * w / scale_factor is itself a half tensor in operators/cnnl/quantify.cpp:104, i.e. it is rounded to binary16
 * before round() and clamp() see it.  scale_factor_dev holds binary16 values. */
int catchq_quantize_per_channel_f16(const void *w, void *q, int bitwidth, int co, int64_t inner,
                                    const void *scale_factor_dev, catchq_stream_t stream);

/* explicit form of the dequantization the reference leaves to the vendor conv/matmul descriptors
 * (cnnl/cnnlTensorDescriptors.cpp:175-184) : y[i] = q[i] * 2^position / scale; q int8/int16/int32
 * (bits 8/16/32), y fp32/fp16. */
int catchq_dequantize(const void *q, int bits, void *y, int y_dtype, int64_t n, int position, float scale,
                      catchq_stream_t stream);

/* ------------------------------------------------------------------ integer contraction + epilogue */

/* What happens to each integer sum acc[r][c] (r = output row / pixel, c = output channel):
 *   v = float(acc) * 2^exp2                 positions of both operands (matmul_internal.cpp:93-96;
 *                                           convolution_forward_internal.cpp:85-88)
 *   v = v / chan_div[c]   if chan_div       "output / new_scale" (quantify_conv_forward.cpp:127; linear.cpp:56)
 *   v = v + bias[c]       if bias           (quantify_conv_forward.cpp:129; linear.cpp:57-59)
 *   v = v + resid[r][c]   if resid          residual branch of the caller's graph (fp32)
 *   v = act(v)                              ReLU, ReLU6, or leaky ReLU: v > 0 ? v : v * act_slope
 *   (with resid_after_act != 0 the residual is added after the activation instead of before it)
 * then any of: y[r][c] = v (fp32, or fp16 by one RNE conversion); acc_out[r][c] = acc;
 * q[r][c] = sat(rne(v * q_scale * 2^-q_position)) for the next layer (q_bitwidth 8/16).
 * All fp32, no fused multiply-add between the steps, true division.
 * chan_rcp (optional, only with chan_div) lets the kernels evaluate the division as
 *   q = v*r; e = fma(-q, d, v); v/d = fma(e, r, q)      (r = chan_rcp[c], d = chan_div[c])
 * which is the correctly rounded quotient, bit for bit the same as v / d, when r is the correctly
 * rounded reciprocal of d, d's significand is not all ones and nothing under/overflows
 * (Markstein's theorem).  The caller guarantees the first two; the kernels use the form only for
 * -64 <= exp2 <= 64 and divide otherwise. */
typedef struct catchq_epilogue {
  int exp2;
  const float *chan_div; /* device [co] or NULL */
  const float *chan_rcp; /* device [co] or NULL: 1/chan_div[c] rounded to nearest (see below) */
  const float *bias;     /* device [co] or NULL */
  const float *resid;    /* device [rows, co] fp32 or NULL */
  int act;               /* CATCHQ_ACT_* */
  void *y;               /* device [rows, co] or NULL */
  int y_dtype;           /* CATCHQ_F32 / CATCHQ_F16 */
  int32_t *acc_out;      /* device [rows, co] or NULL */
  void *q;               /* device [rows, co] int8/int16 or NULL */
  int q_bitwidth;
  int q_position;
  float q_scale;
  float act_slope;       /* CATCHQ_ACT_LEAKY: factor for v <= 0 */
  int resid_after_act;   /* 0: act(v + resid), otherwise act(v) + resid */
  const int32_t *exp2_dev[2]; /* device-resident positions added to exp2 when non-NULL (no host sync);
                                 the reciprocal form of the division is not used with them */
  int half_steps;        /* y_dtype CATCHQ_F16 only.  Non-zero: v is rounded to binary16 after the scaling by 2^exp2,
                            after the division by chan_div[c] and after the addition of bias[c] -- the values the
                            reference's per-channel branch produces for half tensors, where the vendor convolution
                            returns half and `output / new_scale` and `output + bias` are half tensor ops
                            (operators/cnnl/quantify_conv_forward.cpp:123-129); an intermediate beyond 65504 is inf,
                            as there.  Zero: all steps in fp32, one final conversion. */
  int sharing;           /* planning hint, per call: this many launches are expected to run on the device at the
                            same time (e.g. the parts of a batch on parallel streams), so the tile shapes are chosen
                            for 1/sharing of the compute units; 0 or 1: the launch has the device to itself.
                            Affects speed only, never a result.  (The reference plans per handle, one handle per
                            device re-bound to the calling thread's queue: torch_mlu/csrc/aten/cnnl/cnnlHandle.cpp:41-55;
                            it has no such hint.) */
} catchq_epilogue_t;

/* cnnl_mm(self, self_position, other, other_position, false, true) -> cnnlMatMul
 *                                                          operators/cnnl/matmul.cpp:69-75;
 *                                                          operators/cnnl/internal/matmul_internal.cpp:46-120
 * acc[m][n] = sum_k a[m][k] * b[n][k]; a [M,K], b [N,K]; a_bits/b_bits in {8,16}.
 * int8 x int8 and int16 x int8 accumulate in int32; int16 x int16 in int64 (acc_out unsupported there). */
int catchq_gemm_nt(const void *a, int a_bits, const void *b, int b_bits, int64_t m, int64_t n, int64_t k,
                   const catchq_epilogue_t *epilogue, catchq_stream_t stream);

typedef struct catchq_conv_desc {
  int n, h, w, ci;  /* input  [n,h,w,ci] */
  int co, kh, kw;   /* weight [co,kh,kw,ci/groups] */
  int pad_h, pad_w, stride_h, stride_w, dil_h, dil_w, groups;
} catchq_conv_desc_t;

/* conv_output_size()                                       operators/cnnl/internal/convolution_forward_internal.cpp:40-54 */
int catchq_conv_out_size(int in, int k, int pad, int stride, int dil);

/* cnnl_quantify_convolution_internal -> cnnlConvolutionForward
 *                                                          operators/cnnl/internal/convolution_forward_internal.cpp:56-180
 * integer cross-correlation with zero padding and groups; the output rows are the pixels
 * (n,ho,wo) in that order, so y/acc_out/q/resid are NHWC [n,ho,wo,co].
 * Depthwise layers (is_depthwise_conv, operators/cnnl/convolution_overrideable.cpp:41-54) run a
 * stencil kernel; dense layers an implicit GEMM on the int8 matrix cores: int8 x int8 with ci % 16 == 0,
 * int16 x int8 and int16 x int16 (the reference's quantized_mode 2 / 4, quantify_conv_forward.cpp:90-101) with
 * ci % 8 == 0 as two resp. four int8 digit products; grouped int8 layers (cnnlConvolutionForward takes every
 * group count, convolution_forward_internal.cpp:150-173) as one implicit GEMM per group when (ci / groups) % 16 == 0
 * and (co / groups) % 4 == 0; everything else (other grouped layers, odd channel counts) a direct kernel; the
 * arithmetic is the same in all of them. */
int catchq_conv2d_nhwc(const void *x, int x_bits, const void *w, int w_bits, const catchq_conv_desc_t *desc,
                       const catchq_epilogue_t *epilogue, catchq_stream_t stream);

/* cnnl_quantize_convolution_internal -> cnnlQuantizeConvolutionForward
 *                                                          operators/cnnl/internal/quantize_convolution.cpp:57-235
 * Convolution of floating tensors quantized on the fly with positions that live in device memory (int32[1]
 * each; scale 1, no offset, as the reference passes them): x [n,h,w,ci] and w [co,kh,kw,ci/groups] fp32/fp16,
 * q = sat(rne(v * 2^-position)) at x_bits / w_bits, integer convolution, y = acc * 2^(pos_x + pos_w) + bias
 * as fp32/fp16 NHWC.  No host synchronisation.  The caller supplies the workspace (the quantized copies of
 * both operands), as with the reference's cnnlGetConvolutionForwardWorkspaceSize (:160-169). */
int catchq_quantize_conv2d_workspace_size(const catchq_conv_desc_t *desc, int x_bits, int w_bits, size_t *bytes);
int catchq_quantize_conv2d_nhwc(const void *x, int x_dtype, const int32_t *x_position_dev, int x_bits,
                                const void *w, int w_dtype, const int32_t *w_position_dev, int w_bits,
                                const catchq_conv_desc_t *desc, const float *bias, void *y, int y_dtype,
                                void *workspace, size_t workspace_bytes, catchq_stream_t stream);

/* Last convolution of a residual block with the block's projection shortcut evaluated in the same launch.
 * In the reference a block with a projection ends in two torch_mlu::conv2d calls (cnnl_conv2d,
 * operators/cnnl/quantify_conv_forward.cpp:56-147: the 1x1 shortcut and the block's last convolution) and a
 * float add (cnnl_add, operators/cnnl/add.cpp), i.e. the shortcut's fp32 output is written and read back.  Here
 *   s[r][c] = float(acc_s[r][c]) * 2^shortcut.exp2 [/ shortcut.chan_div[c]] [+ shortcut.bias[c]]
 * (acc_s = the 1x1 convolution of shortcut.x [n, in_h, in_w, ci] with shortcut.w [co, ci], stride `stride`
 * in both directions, no padding; its output grid must equal the main convolution's) takes the place of
 * resid[r][c] in the epilogue above; epilogue->resid must be NULL.  s is computed by the same operations, in
 * the same order, as a catchq_conv2d_nhwc call of its own with fp32 output would store.
 * The workspace is only used when no fused kernel serves the shapes (then the shortcut runs as a launch of its
 * own into it): catchq_conv2d_shortcut_workspace_size returns 0 for int8 x int8 operands on both branches with
 * ci % 16 == 0 on both, groups == 1, at most 32 filter taps and co % 4 == 0 (all pointers 16-byte aligned, no
 * exp2_dev, no acc_out), and rows * co * 4 bytes otherwise. */
typedef struct catchq_shortcut {
  const void *x;         /* device [n, in_h, in_w, ci], x_bits wide */
  const void *w;         /* device [co, ci], w_bits wide */
  int x_bits, w_bits;
  int in_h, in_w, ci;    /* n and co are the main convolution's */
  int stride;
  int exp2;
  const float *chan_div; /* device [co] or NULL */
  const float *chan_rcp; /* device [co] or NULL, as in catchq_epilogue_t */
  const float *bias;     /* device [co] or NULL */
} catchq_shortcut_t;
int catchq_conv2d_shortcut_workspace_size(int x_bits, int w_bits, const catchq_conv_desc_t *desc,
                                          const catchq_shortcut_t *shortcut, size_t *bytes);
int catchq_conv2d_shortcut_nhwc(const void *x, int x_bits, const void *w, int w_bits, const catchq_conv_desc_t *desc,
                                const catchq_epilogue_t *epilogue, const catchq_shortcut_t *shortcut, void *workspace,
                                size_t workspace_bytes, catchq_stream_t stream);

/* First two convolutions of a bottleneck block in one launch.  In the reference a bottleneck block begins with two
 * torch_mlu::conv2d calls (cnnl_conv2d, operators/cnnl/quantify_conv_forward.cpp:56-147), each followed by ReLU
 * (operators/cnnl/activation.cpp): a 1x1 reduction whose output is quantized again for the 3x3 convolution behind
 * it.  Here `head` is that 1x1 convolution of x [n, h, w, head->ci] (int8) with head->w [desc->ci, head->ci] (int8),
 *   v1 = float(acc1) * 2^head->exp2 / head->chan_div[c] + head->bias[c]
 *   q1 = sat(rne(relu(v1) * 2^-head->q_position))                                  (int8, never stored)
 * and `desc` / `w` / `epilogue` describe the convolution of q1 [n, h, w, desc->ci] exactly as catchq_conv2d_nhwc takes
 * them (desc->n/h/w are x's; int8 x int8).  The values are those of two catchq_conv2d_nhwc calls, bit for bit.
 * The fused kernel serves 3x3 / stride 1 / padding 1 / 64 -> 64 channels behind a head of 64 or 256 input channels
 * on images cut into bands of rows (catchq_conv1x1_conv3x3_workspace_size reports 0 then); any other shape runs as
 * two launches with q1 in the caller's workspace (n * h * w * desc->ci bytes). */
typedef struct catchq_pointwise_head {
  const void *w;         /* device int8 [desc->ci, ci] */
  int ci;                /* input channels of the 1x1 convolution */
  int exp2;
  const float *chan_div; /* device [desc->ci] or NULL */
  const float *chan_rcp; /* device [desc->ci] or NULL, as in catchq_epilogue_t */
  const float *bias;     /* device [desc->ci] or NULL */
  int q_position;
} catchq_pointwise_head_t;
int catchq_conv1x1_conv3x3_workspace_size(const catchq_pointwise_head_t *head, const catchq_conv_desc_t *desc,
                                          const catchq_epilogue_t *epilogue, size_t *bytes);
int catchq_conv1x1_conv3x3_nhwc(const void *x, const catchq_pointwise_head_t *head, const void *w,
                                const catchq_conv_desc_t *desc, const catchq_epilogue_t *epilogue, void *workspace,
                                size_t workspace_bytes, catchq_stream_t stream);

/* An inverted-residual block in one launch: 1x1 expansion, 3x3 depthwise convolution, 1x1 linear projection.
 * In the reference the block is three torch_mlu::conv2d calls (cnnl_conv2d,
 * operators/cnnl/quantify_conv_forward.cpp:56-147; the middle one is depthwise by is_depthwise_conv,
 * operators/cnnl/convolution_overrideable.cpp:41-54), the first two each followed by ReLU6
 * (operators/cnnl/activation.cpp) and a quantization of the next convolution's input, the last one by the block's
 * float add (cnnl_add, operators/cnnl/add.cpp) where the block has a shortcut.  Here, for x [n, h, w, ci] (int8):
 *   q1 = sat(rne(act1(float(acc1) * 2^expand.exp2 / expand.chan_div[c] + expand.bias[c]) * 2^-expand.q_position))
 *        acc1 = the 1x1 convolution of x with expand.w [hid, ci]                         (int8 [n, h, w, hid], never stored)
 *   q2 = the same with acc2 = the depthwise 3x3 convolution (padding 1, stride `stride` in both directions) of q1
 *        with depthwise.w [hid, 3, 3] and depthwise's constants                          (int8 [n, ho, wo, hid], never stored)
 * and `epilogue` is applied to the 1x1 convolution of q2 with w_project [co, hid] exactly as catchq_conv2d_nhwc
 * applies it (rows = the pixels of [n, ho, wo]; resid, y, q as there).  act is CATCHQ_ACT_RELU or CATCHQ_ACT_RELU6.
 * The values are those of three catchq_conv2d_nhwc calls, bit for bit.
 * The fused kernel serves ci % 32 == 0 (ci <= 160), hid % 32 == 0 (hid >= 128), co % 32 == 0 (co <= 512), w <= 128,
 * stride 1 or 2, both inner stages with chan_div, chan_rcp and bias (-64 <= exp2 <= 64), no exp2_dev and no acc_out in
 * the epilogue, on images whose bands of output rows fit its tile (catchq_inverted_residual_workspace_size reports 0
 * then); any other shape runs as three launches with q1 and q2 in the caller's workspace
 * (n * (h * w + ho * wo) * hid bytes, each part rounded up to 256).  The one-launch kernel does the vector arithmetic of
 * the three launches and saves their start-up and the hidden tensors' traffic: it is the faster route for a lone
 * stream of launches from 14 x 14 outputs on, not for small images or beside other launches that fill the gaps. */
typedef struct catchq_requant_stage {
  const void *w;         /* device int8 */
  int exp2;
  const float *chan_div; /* device [hid] or NULL */
  const float *chan_rcp; /* device [hid] or NULL, as in catchq_epilogue_t */
  const float *bias;     /* device [hid] or NULL */
  int act;               /* CATCHQ_ACT_RELU or CATCHQ_ACT_RELU6 */
  int q_position;
} catchq_requant_stage_t;
int catchq_inverted_residual_workspace_size(int n, int h, int w, int ci, int hid, int co, int stride,
                                            const catchq_requant_stage_t *expand, const catchq_requant_stage_t *depthwise,
                                            const catchq_epilogue_t *epilogue, size_t *bytes);
int catchq_inverted_residual_nhwc(const void *x, int n, int h, int w, int ci, int hid, int co, int stride,
                                  const catchq_requant_stage_t *expand, const catchq_requant_stage_t *depthwise,
                                  const void *w_project, const catchq_epilogue_t *epilogue, void *workspace,
                                  size_t workspace_bytes, catchq_stream_t stream);

/* The first layers of an image network in one launch: input quantization, k x k convolution over a few channels,
 * ReLU / ReLU6, requantization, max pooling.  In the reference these are cnnl_quantify_offline on the channels-last
 * input (operators/cnnl/quantify_conv_forward.cpp:62-63,97), torch_mlu::conv2d (cnnl_conv2d,
 * operators/cnnl/quantify_conv_forward.cpp:56-147), ReLU (operators/cnnl/activation.cpp), the quantization of the
 * next convolution's input and cnnl_max_pool2d (operators/cnnl/pooling.cpp).  For x [n, c, h, w] (fp32, contiguous,
 * c <= 4):
 *   qx = sat(rne(x * x_scale * 2^-x_position))                  int8, inside the convolution's zero padding; never stored
 *   q1 = sat(rne(act(float(acc) * 2^conv.exp2 / conv.chan_div[o] + conv.bias[o]) * 2^-conv.q_position))
 *        acc = the kh x kw convolution (stride `stride`, padding `pad`, both directions) of qx with conv.w
 *        [co][kh][kw4][4] -- filter rows padded with zero taps to kw4 = kw rounded up to a multiple of 4, and to 4
 *        channels, the layout catchq_conv2d_nhwc takes for a framed 4-channel input          int8 [n, hc, wc, co]; never stored
 *   q  = max of q1 over windows pool_k x pool_k, stride pool_stride, padding pool_pad       int8 [n, hp, wp, co]
 * The values are those of catchq_quantize_nchw_to_nhwc_frame, catchq_conv2d_nhwc and catchq_maxpool_nhwc called one
 * after the other, bit for bit.  The fused kernel serves 7x7 / 2 / 3 convolutions of c <= 3 channels into 32, 64 or
 * 128 channels followed by 3x3 / 2 / 1 pooling, w % 4 == 0, x 16-byte aligned, the stage with chan_div, chan_rcp and
 * bias (-64 <= exp2 <= 64) (catchq_first_layers_workspace_size reports 0 then); anything else runs as the three
 * launches with qx and q1 in the caller's workspace.  `sharing` is the planning hint of catchq_epilogue_t::sharing. */
int catchq_first_layers_workspace_size(int n, int c, int h, int w, int co, int kh, int kw, int stride, int pad,
                                       const catchq_requant_stage_t *conv, int pool_k, int pool_stride, int pool_pad,
                                       int sharing, size_t *bytes);
int catchq_first_layers_nchw(const float *x, int n, int c, int h, int w, int x_position, float x_scale, int co,
                             int kh, int kw, int stride, int pad, const catchq_requant_stage_t *conv, int pool_k,
                             int pool_stride, int pool_pad, void *q, int sharing, void *workspace,
                             size_t workspace_bytes, catchq_stream_t stream);

/* A 1x1 convolution and the global average pooling behind it in one launch (the end of a classifier's feature
 * extractor).  In the reference: torch_mlu::conv2d (cnnl_conv2d, operators/cnnl/quantify_conv_forward.cpp:56-147), the
 * block's float add (cnnl_add, operators/cnnl/add.cpp) and ReLU (operators/cnnl/activation.cpp) where it has them,
 * adaptive_avg_pool2d((1,1)) (operators/cnnl/pooling.cpp), and the quantization of the classifier's input
 * (cnnl_linear, operators/cnnl/linear.cpp:40-167).  For x [n, hw, ci] (int8) and w [co, ci] (int8):
 *   v[i, p, c] = `epilogue` applied to the sums of the 1x1 convolution exactly as catchq_conv2d_nhwc applies it (exp2,
 *                chan_div, chan_rcp, bias, resid [n, hw, co] fp32, act none / ReLU / ReLU6; its y, q and acc_out must be
 *                NULL and resid_after_act 0: the convolution's output is never stored)
 *   mean[i, c] = (sum of v[i, p, c] over p in storage order, one fp32 addition each) / hw      fp32 [n, co], may be NULL
 *   q[i, c]    = sat(rne(mean[i, c] * q_scale * 2^-q_position))        int8 / int16 (q_bitwidth 8 / 16) [n, co], may be NULL
 * -- the values of catchq_conv2d_nhwc with an fp32 output followed by catchq_global_avgpool_nhwc /
 * catchq_global_avgpool_quantize_nhwc, bit for bit.  The fused kernel serves hw <= 64, ci % 32 == 0 (ci <= 4096),
 * co % 32 == 0, an epilogue with chan_div, chan_rcp and bias (-64 <= exp2 <= 64) and no exp2_dev
 * (catchq_conv1x1_avgpool_workspace_size reports 0 then); anything else runs as the two launches with the convolution's
 * fp32 output (n * hw * co * 4 bytes) in the caller's workspace. */
int catchq_conv1x1_avgpool_workspace_size(int n, int hw, int ci, int co, const catchq_epilogue_t *epilogue,
                                          size_t *bytes);
int catchq_conv1x1_avgpool_nhwc(const void *x, const void *w, int n, int hw, int ci, int co,
                                const catchq_epilogue_t *epilogue, float *mean, void *q, int q_bitwidth,
                                int q_position, float q_scale, void *workspace, size_t workspace_bytes,
                                catchq_stream_t stream);

/* Residual chain of a stage of bottleneck blocks, recomputed from its int8 inputs in one launch.
 * In the reference every residual block ends in torch_mlu::conv2d (cnnl_conv2d,
 * operators/cnnl/quantify_conv_forward.cpp:56-147) followed by a float add (cnnl_add, operators/cnnl/add.cpp)
 * and ReLU (operators/cnnl/activation.cpp): block b stores y_b = relu(conv_b + y_{b-1}) in fp32 and block
 * b+1 reads it back.  Here links[0] is the stage's 1x1 projection shortcut and links[1..] are the last 1x1
 * convolutions of the stage's blocks, in order:
 *   v_0 = float(acc_0) * 2^exp2_0 / chan_div_0[c] + bias_0[c]
 *   v_i = relu(float(acc_i) * 2^exp2_i / chan_div_i[c] + bias_i[c] + v_{i-1}),   i = 1 .. nlinks-1
 * with acc_i the 1x1 convolution of links[i].x [n, in_h, in_w, ci] (int8) with links[i].w [co, ci] (int8),
 * taps every `stride` pixels, no padding, on the output grid [n, ho, wo].  The launch stores
 * y = v_last (fp32, may be NULL) and q = sat(rne(v_last * 2^-q_position)) (int8, may be NULL) as NHWC
 * [n, ho, wo, co].  Every operation is the one catchq_conv2d_nhwc / catchq_conv2d_shortcut_nhwc calls of the
 * blocks, one after the other, would perform on the same integer sums in the same order, so y and q are
 * theirs bit for bit; the blocks' fp32 outputs in between are never stored.
 * Requirements (CATCHQ_ERR_UNSUPPORTED otherwise): 2 <= nlinks <= CATCHQ_CHAIN_MAX_LINKS, ci % 64 == 0,
 * co % 4 == 0, chan_div / chan_rcp / bias given for every link (chan_rcp as in catchq_epilogue_t),
 * -64 <= exp2 <= 64, every tensor below 2 GiB and 16-byte aligned.  `sharing` is the planning hint of
 * catchq_epilogue_t::sharing. */
#define CATCHQ_CHAIN_MAX_LINKS 8
typedef struct catchq_chain_link {
  const void *x;         /* device int8 [n, in_h, in_w, ci] */
  const void *w;         /* device int8 [co, ci] */
  int in_h, in_w, ci;
  int stride;
  int exp2;
  const float *chan_div; /* device [co] */
  const float *chan_rcp; /* device [co] */
  const float *bias;     /* device [co] */
} catchq_chain_link_t;
int catchq_conv1x1_chain_nhwc(const catchq_chain_link_t *links, int nlinks, int n, int ho, int wo, int co,
                              float *y, void *q, int q_position, int sharing, catchq_stream_t stream);

/* ------------------------------------------------------------------ neighbours of the convolutions */

/* Max pooling over an NHWC tensor whose elements are int8, int16 (quantized activations) or fp32
 * (elem_bits 8 / 16 / 32); windows k x k, zero-size padding never wins (2*pad <= k).  The reference
 * pools in float between its quantized ops (cnnl_max_pool2d, operators/cnnl/pooling.cpp); because
 * quantization is monotonic, pooling the integers gives the same integers. */
int catchq_maxpool_nhwc(const void *x, void *y, int elem_bits, int n, int h, int w, int c, int k, int stride,
                        int pad, catchq_stream_t stream);

/* Global average pooling of an fp32 NHWC tensor [n, hw, c] -> [n, c]: sequential fp32 sum over the
 * pixels in storage order, then one division by hw (adaptive_avg_pool2d((1,1)) in the reference's
 * models, operators/cnnl/pooling.cpp). */
int catchq_global_avgpool_nhwc(const float *x, float *y, int n, int hw, int c, catchq_stream_t stream);

/* The same pooling followed by the quantizer of the layer that consumes it, in one launch:
 * q[n, c] = sat(rne(mean * scale * 2^-position)), int8 / int16 (bitwidth 8 / 16) -- the values
 * catchq_global_avgpool_nhwc then catchq_quantize produce (adaptive_avg_pool2d, operators/cnnl/pooling.cpp,
 * followed by cnnl_quantify_offline_internal, operators/cnnl/internal/quantify.cpp:69-101, in the reference). */
int catchq_global_avgpool_quantize_nhwc(const float *x, void *q, int bitwidth, int n, int hw, int c, int position,
                                        float scale, catchq_stream_t stream);

/* Name of the kernel family catchq_conv2d_nhwc / catchq_gemm_nt would use ("mfma", "direct",
 * "depthwise", ...): for logs and tests; not part of the arithmetic. */
const char *catchq_conv2d_route(int x_bits, int w_bits, const catchq_conv_desc_t *desc);
const char *catchq_gemm_route(int a_bits, int b_bits, int64_t m, int64_t n, int64_t k);

/* ------------------------------------------------------------------ diagnostics */

/* Measurement aid, no counterpart in the reference: `blocks` blocks of four waves each run `iters` rounds of four
 * independent v_mfma_i32_32x32x32_i8 on operand fragments read once from `operands` (1 MiB of device memory,
 * 16-byte aligned; its contents decide how many bits toggle, which decides the clock the device sustains) with no
 * memory access inside the loop: 4 * blocks * iters * 4 * 65536 integer operations per call.  `sink` (one int32
 * of device memory) is only written if the sums take one improbable value.  Timed by the caller
 * (bench.py --probe mfma). */
int catchq_diag_mfma_i8_loop(const void *operands, int iters, int blocks, int32_t *sink, catchq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* CATCHQ_H_ */
