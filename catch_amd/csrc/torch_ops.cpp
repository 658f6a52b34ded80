// PyTorch-ROCm front end of the catchq C ABI.
//
// Registers the reference's two custom-op schemas unchanged
//   torch_mlu::conv2d(input, weight, bias, padding, stride, dilation, groups, q_scale, q_mode)
//   torch_mlu::linear(input, weight, bias, q_scale, q_mode)
// (torch_mlu/tools/mlu_functions.yaml:806-846, registered by tools/gen.py:38-43 in the reference)
// plus helper ops that mirror the reference's C++-internal kernels
// (tools/template/cnnl_kernel.h:48-72): quantize, quantize_per_channel, quantize_param, mm_q,
// and the integer-in/integer-out building blocks qconv2d / qlinear used by fused pipelines.
//
// Device tensors only: there is deliberately no CPU implementation behind these ops (the
// reference's own CPU fall-back for them returns its input, operators/op_methods.cpp:1019-1035).
#include <ATen/ATen.h>
#include <ATen/hip/HIPEvent.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>
#include <torch/library.h>

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "catchq.h"

namespace {

using at::Tensor;

void check_status(int st, const char *what) {
  TORCH_CHECK(st == CATCHQ_OK, what, ": ", catchq_status_string(st));
}

catchq_stream_t current_stream() {
  return reinterpret_cast<catchq_stream_t>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
}

int fp_dtype(const Tensor &t, const char *msg) {
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kHalf, msg);
  return t.scalar_type() == at::kHalf ? CATCHQ_F16 : CATCHQ_F32;
}

at::ScalarType int_type(int64_t bitwidth) {
  switch (bitwidth) {
    case 8: return at::kChar;
    case 16: return at::kShort;
    case 31: return at::kInt;
    default: TORCH_CHECK(false, "bitwidth not support");
  }
}

int bits_of(const Tensor &t) {
  switch (t.scalar_type()) {
    case at::kChar: return 8;
    case at::kShort: return 16;
    case at::kInt: return 32;
    default: TORCH_CHECK(false, "expected an int8/int16/int32 tensor, got ", t.scalar_type());
  }
}

bool has_bias(const Tensor &b) { return b.defined() && b.numel() != 0 && b.dim() != 0; }

// ------------------------------------------------------------------------------------------------
// quantize family
// ------------------------------------------------------------------------------------------------

// cnnl_quantify_offline(input, bitwidth, int position): same shape and memory format as the input.
Tensor quantize_op(const Tensor &x, int64_t bitwidth, int64_t position, double scale) {
  const int dt = fp_dtype(x, "quantify only support input float/half");
  c10::DeviceGuard guard(x.device());
  Tensor xi = x.is_non_overlapping_and_dense() ? x : x.contiguous();
  Tensor q = at::empty_like(xi, xi.options().dtype(int_type(bitwidth)));
  check_status(catchq_quantize(xi.data_ptr(), dt, q.data_ptr(), (int)bitwidth, xi.numel(), (int)position,
                               (float)scale, current_stream()),
               "torch_mlu::quantize");
  return q;
}

// cnnl_quantify_offline(input, bitwidth, Tensor position): position stays on the device.
Tensor quantize_dev_op(const Tensor &x, int64_t bitwidth, const Tensor &position) {
  const int dt = fp_dtype(x, "quantify only support input float/half");
  TORCH_CHECK(position.scalar_type() == at::kInt && position.numel() == 1 && position.device() == x.device(),
              "position must be a one-element int32 tensor on the input's device");
  c10::DeviceGuard guard(x.device());
  Tensor xi = x.is_non_overlapping_and_dense() ? x : x.contiguous();
  Tensor q = at::empty_like(xi, xi.options().dtype(int_type(bitwidth)));
  check_status(catchq_quantize_devpos(xi.data_ptr(), dt, q.data_ptr(), (int)bitwidth, xi.numel(),
                                      position.data_ptr<int32_t>(), nullptr, current_stream()),
               "torch_mlu::quantize_dev");
  return q;
}

// cnnl_quantize_param(input, bitwidth, mode) -> (position int32[1], scale fp32[1], offset fp32[1])
std::tuple<Tensor, Tensor, Tensor> quantize_param_op(const Tensor &x, int64_t bitwidth, int64_t mode) {
  const int dt = fp_dtype(x, "quantize_param only support input float/half");
  c10::DeviceGuard guard(x.device());
  Tensor xi = x.is_non_overlapping_and_dense() ? x : x.contiguous();
  size_t ws_bytes = 0;
  check_status(catchq_quantize_param_workspace_size(xi.numel(), &ws_bytes), "torch_mlu::quantize_param");
  Tensor ws = at::empty({(int64_t)ws_bytes}, xi.options().dtype(at::kChar));
  Tensor pos = at::empty({1}, xi.options().dtype(at::kInt));
  Tensor scale = at::ones({1}, xi.options().dtype(at::kFloat));
  Tensor offset = at::zeros({1}, xi.options().dtype(at::kFloat));
  check_status(catchq_quantize_param(xi.data_ptr(), dt, xi.numel(), (int)bitwidth, (int)mode, ws.data_ptr(),
                                     ws_bytes, nullptr, pos.data_ptr<int32_t>(), scale.data_ptr<float>(),
                                     offset.data_ptr<float>(), current_stream()),
               "torch_mlu::quantize_param");
  return std::make_tuple(pos, scale, offset);
}

struct PerChannel {
  int new_pos = 0;
  Tensor new_scale;     // device fp32 [Co]
  Tensor scale_factor;  // device fp32 [Co]
  Tensor scale_factor_h;  // device fp16 [Co]: set when the parameters were derived in binary16
};

PerChannel per_channel_params(const float *scales_host, int64_t co, int bw, const at::TensorOptions &dev_opts) {
  std::vector<float> ns(co), sf(co);
  PerChannel pc;
  check_status(catchq_per_channel_params(bw, scales_host, (int)co, &pc.new_pos, ns.data(), sf.data()),
               "per-channel parameters");
  auto host = at::TensorOptions().dtype(at::kFloat);
  pc.new_scale = at::from_blob(ns.data(), {co}, host).to(dev_opts.device(), /*non_blocking=*/false);
  pc.scale_factor = at::from_blob(sf.data(), {co}, host).to(dev_opts.device(), false);
  return pc;
}

// scales: a half tensor (any device).  The reference derives the parameters in the dtype of the scales
// (operators/cnnl/quantify.cpp:64-98), so a model converted with .half() gets them rounded to binary16 step
// by step; new_scale and scale_factor come back as the fp32 images of those binary16 values.
PerChannel per_channel_params_half(const Tensor &scales, int bw, const at::TensorOptions &dev_opts) {
  Tensor s_host = scales.to(at::kCPU).contiguous();
  const int64_t co = s_host.numel();
  Tensor ns = at::empty({co}, at::TensorOptions().dtype(at::kHalf));
  Tensor sf = at::empty({co}, at::TensorOptions().dtype(at::kHalf));
  PerChannel pc;
  const int st = catchq_per_channel_params_f16(bw, reinterpret_cast<const uint16_t *>(s_host.data_ptr<at::Half>()),
                                               (int)co, &pc.new_pos,
                                               reinterpret_cast<uint16_t *>(ns.data_ptr<at::Half>()),
                                               reinterpret_cast<uint16_t *>(sf.data_ptr<at::Half>()));
  TORCH_CHECK(st == CATCHQ_OK,
              "per-channel scales held in half precision must be finite and positive there (an int", bw,
              " scale ", bw == 16 ? "32767" : "127", "/absmax above 65504 is inf in half): keep q_scale in float");
  pc.new_scale = ns.to(at::kFloat).to(dev_opts.device(), false);
  pc.scale_factor = sf.to(at::kFloat).to(dev_opts.device(), false);
  pc.scale_factor_h = sf.to(dev_opts.device(), false);
  return pc;
}

// Whether the per-channel parameters are derived with half tensor ops like the reference does for a model
// converted with .half().  int8 only: every constant of the chain (127, the quotients up to 127 in steps of
// 1/16) is a half number.  For int16 half holds neither 32767 nor the integers above 2048, so what the
// reference's half chain yields there depends on how the device clamps and casts 32768.0; those scales are
// read as fp32 values and the derivation runs in fp32.  A half scale that is inf or NaN is refused either way.
bool half_chain(const Tensor &scales, int bw) {
  if (scales.scalar_type() != at::kHalf) return false;
  TORCH_CHECK(at::isfinite(scales).all().item<bool>(),
              "q_scale is held in half precision and is not finite there (an int16 scale 32767/absmax above 65504 "
              "becomes inf in half): keep q_scale in float");
  return bw == 8;
}

Tensor quantize_weight_per_channel(const Tensor &w_dense, const PerChannel &pc, int bw) {
  const int dt = fp_dtype(w_dense, "quantify only support input float/half");
  Tensor q = at::empty_like(w_dense, w_dense.options().dtype(int_type(bw)));
  const int64_t co = w_dense.size(0);
  if (pc.scale_factor_h.defined() && dt == CATCHQ_F16) {
    // half weight / half scale_factor: the quotient is a half tensor too (quantify.cpp:104)
    check_status(catchq_quantize_per_channel_f16(w_dense.data_ptr(), q.data_ptr(), bw, (int)co,
                                                 co ? w_dense.numel() / co : 0, pc.scale_factor_h.data_ptr(),
                                                 current_stream()),
                 "torch_mlu::quantize_per_channel");
    return q;
  }
  check_status(catchq_quantize_per_channel(w_dense.data_ptr(), dt, q.data_ptr(), bw, (int)co,
                                           co ? w_dense.numel() / co : 0, pc.scale_factor.data_ptr<float>(),
                                           current_stream()),
               "torch_mlu::quantize_per_channel");
  return q;
}

// cnnl_quantify_per_channel(input, scale_data, bitwidth) -> (quantized, new_position[1], new_scale[Co])
std::tuple<Tensor, Tensor, Tensor> quantize_per_channel_op(const Tensor &w, const Tensor &scales, int64_t bitwidth) {
  TORCH_CHECK(bitwidth == 8 || bitwidth == 16, "bitwidth not support");
  TORCH_CHECK(w.dim() >= 1 && scales.numel() == w.size(0), "one scale per output channel expected");
  c10::DeviceGuard guard(w.device());
  PerChannel pc;
  if (half_chain(scales, (int)bitwidth)) {
    pc = per_channel_params_half(scales, (int)bitwidth, w.options());
  } else {
    Tensor s_host = scales.to(at::kCPU, at::kFloat).contiguous();
    pc = per_channel_params(s_host.data_ptr<float>(), s_host.numel(), (int)bitwidth, w.options());
  }
  // dim 0 must be the slowest-varying dimension of the memory: true for contiguous and channels-last
  Tensor wd = w.is_non_overlapping_and_dense() && w.stride(0) * w.size(0) == w.numel() ? w : w.contiguous();
  Tensor q = quantize_weight_per_channel(wd, pc, (int)bitwidth);
  // new_position and new_scale in the dtype of the scales, as the reference's tensor ops leave them
  Tensor new_pos = at::full({1}, (double)pc.new_pos, w.options().dtype(scales.scalar_type() == at::kHalf ? at::kHalf : at::kFloat));
  return std::make_tuple(q, new_pos, scales.scalar_type() == at::kHalf ? pc.new_scale.to(at::kHalf) : pc.new_scale);
}

Tensor dequantize_op(const Tensor &q, int64_t position, double scale, bool half) {
  c10::DeviceGuard guard(q.device());
  Tensor qi = q.is_non_overlapping_and_dense() ? q : q.contiguous();
  Tensor y = at::empty_like(qi, qi.options().dtype(half ? at::kHalf : at::kFloat));
  check_status(catchq_dequantize(qi.data_ptr(), bits_of(qi), y.data_ptr(), half ? CATCHQ_F16 : CATCHQ_F32,
                                 qi.numel(), (int)position, (float)scale, current_stream()),
               "torch_mlu::dequantize");
  return y;
}

// ------------------------------------------------------------------------------------------------
// integer building blocks
// ------------------------------------------------------------------------------------------------

struct EpiArgs {
  int64_t exp2 = 0;
  c10::optional<Tensor> chan_div, bias, resid;
  int64_t act = 0;
  bool want_y = true, y_half = false, want_acc = false;
  int64_t q_bitwidth = 0, q_position = 0;
  double q_scale = 1.0;
  double act_slope = 0.0;
  bool resid_after_act = false;
  bool half_steps = false;  // fp16 output rounded after scaling, division and bias (the reference's half tensor ops)
};

struct EpiOut {
  Tensor y, acc, q;
};

// Planning hint of the calling thread: how many launches it expects to run on the device at the same time (a plan
// that records the parts of a batch on parallel streams sets it around the recording).  Thread-local, so two
// threads planning at once do not see each other's value; handed to the C ABI per call (catchq_epilogue_t::sharing).
thread_local int t_launch_sharing = 1;

// whether catchq_conv1x1_conv3x3_nhwc serves (1x1: k1 -> cm, then 3x3 / stride 1 / padding 1: cm -> co) over n images of
// h x w in one launch (per-channel constants with reciprocals and 16-byte aligned tensors assumed)
bool irb_fuses_op(int64_t n, int64_t h, int64_t w, int64_t ci, int64_t hid, int64_t co, int64_t stride) {
  float one = 1.0f;
  catchq_requant_stage_t st;
  std::memset(&st, 0, sizeof(st));
  st.w = &one; st.chan_div = st.chan_rcp = st.bias = &one;  // presence only: nothing is dereferenced
  st.act = CATCHQ_ACT_RELU6;
  catchq_epilogue_t e;
  std::memset(&e, 0, sizeof(e));
  e.q = &one; e.q_bitwidth = 8;
  e.sharing = t_launch_sharing;
  size_t bytes = 1;
  return catchq_inverted_residual_workspace_size((int)n, (int)h, (int)w, (int)ci, (int)hid, (int)co, (int)stride, &st, &st, &e,
                                                 &bytes) == CATCHQ_OK && bytes == 0;
}

bool first_layers_fuse_op(int64_t n, int64_t c, int64_t h, int64_t w, int64_t co, int64_t k, int64_t stride, int64_t pad,
                          int64_t pool_k, int64_t pool_stride, int64_t pool_pad) {
  float one = 1.0f;
  catchq_requant_stage_t st;
  std::memset(&st, 0, sizeof(st));
  st.w = &one; st.chan_div = st.chan_rcp = st.bias = &one;  // presence only: nothing is dereferenced
  st.act = CATCHQ_ACT_RELU;
  size_t bytes = 1;
  return catchq_first_layers_workspace_size((int)n, (int)c, (int)h, (int)w, (int)co, (int)k, (int)k, (int)stride, (int)pad, &st,
                                            (int)pool_k, (int)pool_stride, (int)pool_pad, t_launch_sharing,
                                            &bytes) == CATCHQ_OK && bytes == 0;
}

bool conv_avgpool_fuses_op(int64_t n, int64_t hw, int64_t ci, int64_t co) {
  float one = 1.0f;
  catchq_epilogue_t e;
  std::memset(&e, 0, sizeof(e));
  e.chan_div = e.chan_rcp = e.bias = &one;  // presence only: nothing is dereferenced
  e.act = CATCHQ_ACT_RELU;
  size_t bytes = 1;
  return catchq_conv1x1_avgpool_workspace_size((int)n, (int)hw, (int)ci, (int)co, &e, &bytes) == CATCHQ_OK && bytes == 0;
}

bool head_fuses_op(int64_t n, int64_t h, int64_t w, int64_t k1, int64_t cm, int64_t co) {
  float one = 1.0f;
  catchq_pointwise_head_t hd;
  std::memset(&hd, 0, sizeof(hd));
  hd.ci = (int)k1;
  hd.w = &one; hd.chan_div = hd.chan_rcp = hd.bias = &one;  // presence only: nothing is dereferenced
  catchq_conv_desc_t d = {(int)n, (int)h, (int)w, (int)cm, (int)co, 3, 3, 1, 1, 1, 1, 1, 1, 1};
  catchq_epilogue_t e;
  std::memset(&e, 0, sizeof(e));
  e.q = &one; e.q_bitwidth = 8;
  size_t bytes = 1;
  return catchq_conv1x1_conv3x3_workspace_size(&hd, &d, &e, &bytes) == CATCHQ_OK && bytes == 0;
}

int64_t set_launch_sharing_op(int64_t launches) {
  TORCH_CHECK(launches >= 1, "set_launch_sharing: at least one launch");
  const int before = t_launch_sharing;
  t_launch_sharing = (int)launches;
  return before;
}

Tensor as_f32_vec(const c10::optional<Tensor> &t, int64_t n, const char *name) {
  if (!t.has_value() || !t->defined()) return Tensor();
  TORCH_CHECK(t->numel() == n, name, ": expected ", n, " elements, got ", t->numel());
  return t->to(at::kFloat).contiguous();
}

uint32_t version_of(const Tensor &t);

// Correctly rounded reciprocals of a per-channel divisor vector, kept per divisor tensor (one
// device-to-host copy the first time a tensor is seen).  Undefined when some divisor has an
// all-ones significand: the kernels then divide (see catchq_epilogue_t::chan_rcp).
struct RcpEntry {
  c10::weak_intrusive_ptr<c10::TensorImpl> impl;
  uint32_t version;
  const void *ptr;
  Tensor rcp;
};
std::mutex g_rcp_mutex;
std::unordered_map<const c10::TensorImpl *, RcpEntry> g_rcp_cache;

Tensor reciprocals_for(const Tensor &div) {
  const c10::TensorImpl *key = div.unsafeGetTensorImpl();
  {
    std::lock_guard<std::mutex> lock(g_rcp_mutex);
    auto it = g_rcp_cache.find(key);
    if (it != g_rcp_cache.end()) {
      const RcpEntry &r = it->second;
      if (!r.impl.expired() && r.impl._unsafe_get_target() == key && r.version == version_of(div) &&
          r.ptr == div.data_ptr())
        return r.rcp;
      g_rcp_cache.erase(it);
    }
  }
  Tensor host = div.to(at::kCPU).contiguous();
  const float *d = host.data_ptr<float>();
  const int64_t n = host.numel();
  std::vector<float> r(n);
  bool usable = n > 0;
  for (int64_t i = 0; i < n; ++i) {
    uint32_t bits;
    std::memcpy(&bits, &d[i], 4);
    if ((bits & 0x7fffffu) == 0x7fffffu || !(d[i] > 0.0f) || !std::isfinite(d[i])) usable = false;
    r[i] = 1.0f / d[i];  // IEEE division: correctly rounded
  }
  Tensor rcp;
  if (usable) rcp = at::from_blob(r.data(), {n}, at::TensorOptions().dtype(at::kFloat)).to(div.device());
  std::lock_guard<std::mutex> lock(g_rcp_mutex);
  if (g_rcp_cache.size() > 4096) g_rcp_cache.clear();
  g_rcp_cache.insert_or_assign(key, RcpEntry{c10::weak_intrusive_ptr<c10::TensorImpl>(div.getIntrusivePtr()),
                                             version_of(div), div.data_ptr(), rcp});
  return rcp;
}

// fills a catchq_epilogue_t; `keep` holds the temporaries alive until the launch is enqueued
EpiOut prepare_epilogue(const EpiArgs &a, at::IntArrayRef out_shape, int64_t co, const at::TensorOptions &opts,
                        catchq_epilogue_t *e, std::vector<Tensor> *keep) {
  EpiOut o;
  std::memset(e, 0, sizeof(*e));
  TORCH_CHECK(a.exp2 >= -126 && a.exp2 <= 126, "position sum out of range");
  e->exp2 = (int)a.exp2;
  Tensor cd = as_f32_vec(a.chan_div, co, "chan_div"), bs = as_f32_vec(a.bias, co, "bias");
  if (cd.defined()) {
    e->chan_div = cd.data_ptr<float>();
    keep->push_back(cd);
    Tensor rcp = reciprocals_for(cd);
    if (rcp.defined()) { e->chan_rcp = rcp.data_ptr<float>(); keep->push_back(rcp); }
  }
  if (bs.defined()) { e->bias = bs.data_ptr<float>(); keep->push_back(bs); }
  if (a.resid.has_value() && a.resid->defined()) {
    TORCH_CHECK(a.resid->sizes() == out_shape && a.resid->scalar_type() == at::kFloat && a.resid->is_contiguous(),
                "resid must be a contiguous fp32 tensor of the output's shape");
    e->resid = a.resid->data_ptr<float>();
  }
  e->sharing = t_launch_sharing;
  e->half_steps = (a.half_steps && a.y_half) ? 1 : 0;
  e->act = (int)a.act;
  e->act_slope = (float)a.act_slope;
  e->resid_after_act = a.resid_after_act ? 1 : 0;
  if (a.want_y) {
    o.y = at::empty(out_shape, opts.dtype(a.y_half ? at::kHalf : at::kFloat));
    e->y = o.y.data_ptr();
    e->y_dtype = a.y_half ? CATCHQ_F16 : CATCHQ_F32;
  }
  if (a.want_acc) {
    o.acc = at::empty(out_shape, opts.dtype(at::kInt));
    e->acc_out = o.acc.data_ptr<int32_t>();
  }
  if (a.q_bitwidth != 0) {
    TORCH_CHECK(a.q_bitwidth == 8 || a.q_bitwidth == 16, "bitwidth not support");
    o.q = at::empty(out_shape, opts.dtype(int_type(a.q_bitwidth)));
    e->q = o.q.data_ptr();
    e->q_bitwidth = (int)a.q_bitwidth;
    e->q_position = (int)a.q_position;
    e->q_scale = (float)a.q_scale;
  }
  return o;
}

// qx [N,H,W,Ci] int8/int16 contiguous, qw [Co,kh,kw,Ci/g] contiguous -> outputs [N,Ho,Wo,Co]
EpiOut qconv2d_impl(const Tensor &qx, const Tensor &qw, at::IntArrayRef padding, at::IntArrayRef stride,
                    at::IntArrayRef dilation, int64_t groups, const EpiArgs &a) {
  TORCH_CHECK(qx.dim() == 4 && qw.dim() == 4 && qx.is_contiguous() && qw.is_contiguous(),
              "qconv2d expects contiguous NHWC activations and [Co,kh,kw,Ci/g] weights");
  TORCH_CHECK(padding.size() == 2 && stride.size() == 2 && dilation.size() == 2, "2-d conv parameters expected");
  TORCH_CHECK(groups > 0 && qx.size(3) == qw.size(3) * groups, "channel mismatch: input ", qx.size(3),
              ", weight ", qw.size(3), " x groups ", groups);
  catchq_conv_desc_t d;
  d.n = (int)qx.size(0); d.h = (int)qx.size(1); d.w = (int)qx.size(2); d.ci = (int)qx.size(3);
  d.co = (int)qw.size(0); d.kh = (int)qw.size(1); d.kw = (int)qw.size(2);
  d.pad_h = (int)padding[0]; d.pad_w = (int)padding[1];
  d.stride_h = (int)stride[0]; d.stride_w = (int)stride[1];
  d.dil_h = (int)dilation[0]; d.dil_w = (int)dilation[1];
  d.groups = (int)groups;
  TORCH_CHECK(d.stride_h > 0 && d.stride_w > 0, "non-positive stride is not supported");
  TORCH_CHECK(d.pad_h >= 0 && d.pad_w >= 0, "negative padding is not supported");
  const int ho = catchq_conv_out_size(d.h, d.kh, d.pad_h, d.stride_h, d.dil_h);
  const int wo = catchq_conv_out_size(d.w, d.kw, d.pad_w, d.stride_w, d.dil_w);
  TORCH_CHECK(ho > 0 && wo > 0, "Calculated output size is too small");
  catchq_epilogue_t e;
  std::vector<Tensor> keep;
  EpiOut o = prepare_epilogue(a, {d.n, ho, wo, d.co}, d.co, qx.options(), &e, &keep);
  if (d.n == 0 || d.co == 0) return o;  // nothing to compute: the empty outputs are the result
  check_status(catchq_conv2d_nhwc(qx.data_ptr(), bits_of(qx), qw.data_ptr(), bits_of(qw), &d, &e, current_stream()),
               "torch_mlu::conv2d");
  return o;
}

// The last convolution of a residual block with the block's 1x1 projection shortcut (sx [N,Hs,Ws,Cs],
// sw [Co,Cs] or [Co,1,1,Cs], stride s_stride, no padding) evaluated in the same launch; a.resid must be unset.
EpiOut qconv2d_shortcut_impl(const Tensor &qx, const Tensor &qw, at::IntArrayRef padding, at::IntArrayRef stride,
                             at::IntArrayRef dilation, const EpiArgs &a, const Tensor &sx, const Tensor &sw,
                             int64_t s_stride, int64_t s_exp2, const c10::optional<Tensor> &s_chan_div,
                             const c10::optional<Tensor> &s_bias) {
  TORCH_CHECK(qx.dim() == 4 && qw.dim() == 4 && qx.is_contiguous() && qw.is_contiguous(),
              "qconv2d expects contiguous NHWC activations and [Co,kh,kw,Ci/g] weights");
  TORCH_CHECK(sx.dim() == 4 && sx.is_contiguous() && sw.is_contiguous() && sw.numel() == qw.size(0) * sx.size(3) &&
                  sx.size(0) == qx.size(0),
              "shortcut: expected NHWC activations of the same batch and a [Co,Ci] filter");
  TORCH_CHECK(padding.size() == 2 && stride.size() == 2 && dilation.size() == 2, "2-d conv parameters expected");
  TORCH_CHECK(qx.size(3) == qw.size(3), "channel mismatch: input ", qx.size(3), ", weight ", qw.size(3));
  TORCH_CHECK(!(a.resid.has_value() && a.resid->defined()), "the shortcut is the residual: resid must not be given");
  catchq_conv_desc_t d;
  d.n = (int)qx.size(0); d.h = (int)qx.size(1); d.w = (int)qx.size(2); d.ci = (int)qx.size(3);
  d.co = (int)qw.size(0); d.kh = (int)qw.size(1); d.kw = (int)qw.size(2);
  d.pad_h = (int)padding[0]; d.pad_w = (int)padding[1];
  d.stride_h = (int)stride[0]; d.stride_w = (int)stride[1];
  d.dil_h = (int)dilation[0]; d.dil_w = (int)dilation[1];
  d.groups = 1;
  const int ho = catchq_conv_out_size(d.h, d.kh, d.pad_h, d.stride_h, d.dil_h);
  const int wo = catchq_conv_out_size(d.w, d.kw, d.pad_w, d.stride_w, d.dil_w);
  TORCH_CHECK(ho > 0 && wo > 0, "Calculated output size is too small");
  catchq_epilogue_t e;
  std::vector<Tensor> keep;
  EpiOut o = prepare_epilogue(a, {d.n, ho, wo, d.co}, d.co, qx.options(), &e, &keep);
  catchq_shortcut_t sc;
  std::memset(&sc, 0, sizeof(sc));
  sc.x = sx.data_ptr(); sc.w = sw.data_ptr();
  sc.x_bits = bits_of(sx); sc.w_bits = bits_of(sw);
  sc.in_h = (int)sx.size(1); sc.in_w = (int)sx.size(2); sc.ci = (int)sx.size(3);
  sc.stride = (int)s_stride;
  TORCH_CHECK(s_exp2 >= -126 && s_exp2 <= 126, "position sum out of range");
  sc.exp2 = (int)s_exp2;
  Tensor cd = as_f32_vec(s_chan_div, d.co, "shortcut chan_div"), bs = as_f32_vec(s_bias, d.co, "shortcut bias");
  if (cd.defined()) {
    sc.chan_div = cd.data_ptr<float>();
    keep.push_back(cd);
    Tensor rcp = reciprocals_for(cd);
    if (rcp.defined()) { sc.chan_rcp = rcp.data_ptr<float>(); keep.push_back(rcp); }
  }
  if (bs.defined()) { sc.bias = bs.data_ptr<float>(); keep.push_back(bs); }
  if (d.n == 0) return o;  // nothing to compute
  size_t ws_bytes = 0;
  check_status(catchq_conv2d_shortcut_workspace_size(bits_of(qx), bits_of(qw), &d, &sc, &ws_bytes),
               "torch_mlu::qconv2d_shortcut");
  Tensor ws = at::empty({(int64_t)std::max<size_t>(ws_bytes, 16)}, qx.options().dtype(at::kChar));
  check_status(catchq_conv2d_shortcut_nhwc(qx.data_ptr(), bits_of(qx), qw.data_ptr(), bits_of(qw), &d, &e, &sc,
                                           ws.data_ptr(), ws_bytes, current_stream()),
               "torch_mlu::qconv2d_shortcut");
  return o;
}

EpiOut qlinear_impl(const Tensor &qx, const Tensor &qw, const EpiArgs &a) {
  TORCH_CHECK(qx.dim() == 2 && qw.dim() == 2 && qx.is_contiguous() && qw.is_contiguous(), "dimension not support");
  TORCH_CHECK(qx.size(1) == qw.size(1), "size mismatch: ", qx.sizes(), " x ", qw.sizes(), "^T");
  catchq_epilogue_t e;
  std::vector<Tensor> keep;
  EpiOut o = prepare_epilogue(a, {qx.size(0), qw.size(0)}, qw.size(0), qx.options(), &e, &keep);
  if (qx.size(0) == 0 || qw.size(0) == 0) return o;  // nothing to compute
  check_status(catchq_gemm_nt(qx.data_ptr(), bits_of(qx), qw.data_ptr(), bits_of(qw), qx.size(0), qw.size(0),
                              qx.size(1), &e, current_stream()),
               "torch_mlu::linear");
  return o;
}

EpiArgs make_args(int64_t exp2, const c10::optional<Tensor> &chan_div, const c10::optional<Tensor> &bias,
                  const c10::optional<Tensor> &resid, int64_t act, bool want_y, bool y_half, bool want_acc,
                  int64_t q_bitwidth, int64_t q_position, double q_scale, double act_slope = 0.0,
                  bool resid_after_act = false) {
  EpiArgs a;
  a.act_slope = act_slope; a.resid_after_act = resid_after_act;
  a.exp2 = exp2; a.chan_div = chan_div; a.bias = bias; a.resid = resid; a.act = act;
  a.want_y = want_y; a.y_half = y_half; a.want_acc = want_acc;
  a.q_bitwidth = q_bitwidth; a.q_position = q_position; a.q_scale = q_scale;
  return a;
}

std::tuple<Tensor, Tensor, Tensor> tup(const EpiOut &o) { return std::make_tuple(o.y, o.q, o.acc); }

std::tuple<Tensor, Tensor, Tensor> qconv2d_op(const Tensor &qx, const Tensor &qw, int64_t exp2,
                                              const c10::optional<Tensor> &chan_div,
                                              const c10::optional<Tensor> &bias,
                                              const c10::optional<Tensor> &resid, at::IntArrayRef padding,
                                              at::IntArrayRef stride, at::IntArrayRef dilation, int64_t groups,
                                              int64_t act, bool want_y, bool y_half, bool want_acc,
                                              int64_t q_bitwidth, int64_t q_position, double q_scale,
                                              double act_slope, bool resid_after_act) {
  c10::DeviceGuard guard(qx.device());
  return tup(qconv2d_impl(qx, qw, padding, stride, dilation, groups,
                          make_args(exp2, chan_div, bias, resid, act, want_y, y_half, want_acc, q_bitwidth,
                                    q_position, q_scale, act_slope, resid_after_act)));
}

std::tuple<Tensor, Tensor> qconv2d_shortcut_op(const Tensor &qx, const Tensor &qw, int64_t exp2,
                                               const c10::optional<Tensor> &chan_div, const c10::optional<Tensor> &bias,
                                               const Tensor &sx, const Tensor &sw, int64_t s_stride, int64_t s_exp2,
                                               const c10::optional<Tensor> &s_chan_div,
                                               const c10::optional<Tensor> &s_bias, at::IntArrayRef padding,
                                               at::IntArrayRef stride, at::IntArrayRef dilation, int64_t act, bool want_y,
                                               bool y_half, int64_t q_bitwidth, int64_t q_position, double q_scale,
                                               double act_slope, bool resid_after_act) {
  c10::DeviceGuard guard(qx.device());
  EpiOut o = qconv2d_shortcut_impl(qx, qw, padding, stride, dilation,
                                   make_args(exp2, chan_div, bias, c10::nullopt, act, want_y, y_half, false, q_bitwidth,
                                             q_position, q_scale, act_slope, resid_after_act),
                                   sx, sw, s_stride, s_exp2, s_chan_div, s_bias);
  return std::make_tuple(o.y, o.q);
}

// First two convolutions of a bottleneck block (catchq_conv1x1_conv3x3_nhwc): qx [N,H,W,K1] int8 NHWC through the
// 1x1 filters w1 [Cm,K1] (or [Cm,1,1,K1]) + ReLU + int8 requantization at position q_position1, then qw [Co,kh,kw,Cm]
// with the usual epilogue arguments.
std::tuple<Tensor, Tensor> qconv2d_head_op(const Tensor &qx, const Tensor &w1, int64_t exp2_1,
                                           const c10::optional<Tensor> &chan_div1, const c10::optional<Tensor> &bias1,
                                           int64_t q_position1, const Tensor &qw, int64_t exp2,
                                           const c10::optional<Tensor> &chan_div, const c10::optional<Tensor> &bias,
                                           at::IntArrayRef padding, at::IntArrayRef stride, at::IntArrayRef dilation,
                                           int64_t act, bool want_y, bool y_half, int64_t q_bitwidth, int64_t q_position,
                                           double q_scale, double act_slope) {
  c10::DeviceGuard guard(qx.device());
  TORCH_CHECK(qx.dim() == 4 && qw.dim() == 4 && qx.is_contiguous() && qw.is_contiguous() && w1.is_contiguous(),
              "qconv2d_head expects contiguous NHWC activations and [Co,kh,kw,Ci] weights");
  TORCH_CHECK(qx.scalar_type() == at::kChar && qw.scalar_type() == at::kChar && w1.scalar_type() == at::kChar,
              "qconv2d_head: int8 operands expected");
  const int64_t cm = qw.size(3), k1 = qx.size(3);
  TORCH_CHECK(w1.size(0) == cm && w1.numel() == cm * k1, "qconv2d_head: the head's filters must be [", cm, ", ", k1, "]");
  TORCH_CHECK(w1.device() == qx.device() && qw.device() == qx.device(), "qconv2d_head: operands on different devices");
  TORCH_CHECK(padding.size() == 2 && stride.size() == 2 && dilation.size() == 2, "2-d conv parameters expected");
  catchq_conv_desc_t d;
  d.n = (int)qx.size(0); d.h = (int)qx.size(1); d.w = (int)qx.size(2); d.ci = (int)cm;
  d.co = (int)qw.size(0); d.kh = (int)qw.size(1); d.kw = (int)qw.size(2);
  d.pad_h = (int)padding[0]; d.pad_w = (int)padding[1];
  d.stride_h = (int)stride[0]; d.stride_w = (int)stride[1];
  d.dil_h = (int)dilation[0]; d.dil_w = (int)dilation[1];
  d.groups = 1;
  TORCH_CHECK(d.stride_h > 0 && d.stride_w > 0 && d.pad_h >= 0 && d.pad_w >= 0, "bad stride or padding");
  const int ho = catchq_conv_out_size(d.h, d.kh, d.pad_h, d.stride_h, d.dil_h);
  const int wo = catchq_conv_out_size(d.w, d.kw, d.pad_w, d.stride_w, d.dil_w);
  TORCH_CHECK(ho > 0 && wo > 0, "Calculated output size is too small");
  catchq_epilogue_t e;
  std::vector<Tensor> keep;
  EpiOut o = prepare_epilogue(make_args(exp2, chan_div, bias, c10::nullopt, act, want_y, y_half, false, q_bitwidth,
                                        q_position, q_scale, act_slope, false),
                              {d.n, ho, wo, d.co}, d.co, qx.options(), &e, &keep);
  catchq_pointwise_head_t hd;
  std::memset(&hd, 0, sizeof(hd));
  hd.w = w1.data_ptr();
  hd.ci = (int)k1;
  TORCH_CHECK(exp2_1 >= -126 && exp2_1 <= 126, "position sum out of range");
  hd.exp2 = (int)exp2_1;
  hd.q_position = (int)q_position1;
  Tensor cd = as_f32_vec(chan_div1, cm, "head chan_div"), bs = as_f32_vec(bias1, cm, "head bias");
  if (cd.defined()) {
    hd.chan_div = cd.data_ptr<float>();
    keep.push_back(cd);
    Tensor rcp = reciprocals_for(cd);
    if (rcp.defined()) { hd.chan_rcp = rcp.data_ptr<float>(); keep.push_back(rcp); }
  }
  if (bs.defined()) { hd.bias = bs.data_ptr<float>(); keep.push_back(bs); }
  if (d.n == 0) return std::make_tuple(o.y, o.q);
  size_t ws_bytes = 0;
  check_status(catchq_conv1x1_conv3x3_workspace_size(&hd, &d, &e, &ws_bytes), "torch_mlu::qconv2d_head");
  Tensor ws = at::empty({(int64_t)std::max<size_t>(ws_bytes, 16)}, qx.options().dtype(at::kChar));
  check_status(catchq_conv1x1_conv3x3_nhwc(qx.data_ptr(), &hd, qw.data_ptr(), &d, &e, ws.data_ptr(), ws_bytes,
                                           current_stream()),
               "torch_mlu::qconv2d_head");
  return std::make_tuple(o.y, o.q);
}

// An inverted-residual block (catchq_inverted_residual_nhwc): qx [N,H,W,Ci] int8 NHWC through the 1x1 expansion w1
// [hid,Ci] (or [hid,1,1,Ci]), the depthwise 3x3 filters wd [hid,3,3] (or [hid,3,3,1]; padding 1, `stride`), both with
// act1 / act2 (ReLU or ReLU6) and int8 requantization at q_position1 / q_position2, and the 1x1 projection w3 [Co,hid]
// with the usual epilogue arguments.
namespace {
struct StageKeep {
  catchq_requant_stage_t st;
  Tensor cd, rcp, bs;
};
void fill_stage(StageKeep *k, const Tensor &w, int64_t exp2, const c10::optional<Tensor> &chan_div,
                const c10::optional<Tensor> &bias, int64_t act, int64_t q_position, int64_t channels, const char *what) {
  std::memset(&k->st, 0, sizeof(k->st));
  TORCH_CHECK(exp2 >= -126 && exp2 <= 126, "position sum out of range");
  k->st.w = w.data_ptr();
  k->st.exp2 = (int)exp2;
  k->st.act = (int)act;
  k->st.q_position = (int)q_position;
  k->cd = as_f32_vec(chan_div, channels, what);
  k->bs = as_f32_vec(bias, channels, what);
  if (k->cd.defined()) {
    k->st.chan_div = k->cd.data_ptr<float>();
    k->rcp = reciprocals_for(k->cd);
    if (k->rcp.defined()) k->st.chan_rcp = k->rcp.data_ptr<float>();
  }
  if (k->bs.defined()) k->st.bias = k->bs.data_ptr<float>();
}
}  // namespace

std::tuple<Tensor, Tensor> qconv2d_irb_op(const Tensor &qx, const Tensor &w1, int64_t exp2_1,
                                          const c10::optional<Tensor> &chan_div1, const c10::optional<Tensor> &bias1,
                                          int64_t act1, int64_t q_position1, const Tensor &wd, int64_t stride, int64_t exp2_2,
                                          const c10::optional<Tensor> &chan_div2, const c10::optional<Tensor> &bias2,
                                          int64_t act2, int64_t q_position2, const Tensor &w3, int64_t exp2,
                                          const c10::optional<Tensor> &chan_div, const c10::optional<Tensor> &bias,
                                          const c10::optional<Tensor> &resid, bool want_y, bool y_half, int64_t q_bitwidth,
                                          int64_t q_position, double q_scale) {
  c10::DeviceGuard guard(qx.device());
  TORCH_CHECK(qx.dim() == 4 && qx.is_contiguous() && w1.is_contiguous() && wd.is_contiguous() && w3.is_contiguous(),
              "qconv2d_irb expects contiguous NHWC activations and contiguous filters");
  TORCH_CHECK(qx.scalar_type() == at::kChar && w1.scalar_type() == at::kChar && wd.scalar_type() == at::kChar &&
                  w3.scalar_type() == at::kChar,
              "qconv2d_irb: int8 operands expected");
  TORCH_CHECK(w1.device() == qx.device() && wd.device() == qx.device() && w3.device() == qx.device(),
              "qconv2d_irb: operands on different devices");
  const int64_t n = qx.size(0), h = qx.size(1), w = qx.size(2), ci = qx.size(3), hid = w1.size(0), co = w3.size(0);
  TORCH_CHECK(w1.numel() == hid * ci, "qconv2d_irb: the expansion's filters must be [", hid, ", ", ci, "]");
  TORCH_CHECK(wd.size(0) == hid && wd.numel() == hid * 9, "qconv2d_irb: the depthwise filters must be [", hid, ", 3, 3]");
  TORCH_CHECK(w3.numel() == co * hid, "qconv2d_irb: the projection's filters must be [", co, ", ", hid, "]");
  TORCH_CHECK(stride >= 1, "bad stride");
  const int ho = catchq_conv_out_size((int)h, 3, 1, (int)stride, 1), wo = catchq_conv_out_size((int)w, 3, 1, (int)stride, 1);
  TORCH_CHECK(ho > 0 && wo > 0, "Calculated output size is too small");
  catchq_epilogue_t e;
  std::vector<Tensor> keep;
  EpiOut o = prepare_epilogue(make_args(exp2, chan_div, bias, resid, 0, want_y, y_half, false, q_bitwidth, q_position,
                                        q_scale, 0.0, false),
                              {n, ho, wo, co}, co, qx.options(), &e, &keep);
  StageKeep k1, k2;
  fill_stage(&k1, w1, exp2_1, chan_div1, bias1, act1, q_position1, hid, "expansion constants");
  fill_stage(&k2, wd, exp2_2, chan_div2, bias2, act2, q_position2, hid, "depthwise constants");
  if (n == 0) return std::make_tuple(o.y, o.q);
  size_t ws_bytes = 0;
  check_status(catchq_inverted_residual_workspace_size((int)n, (int)h, (int)w, (int)ci, (int)hid, (int)co, (int)stride,
                                                       &k1.st, &k2.st, &e, &ws_bytes),
               "torch_mlu::qconv2d_irb");
  Tensor ws = at::empty({(int64_t)std::max<size_t>(ws_bytes, 16)}, qx.options().dtype(at::kChar));
  check_status(catchq_inverted_residual_nhwc(qx.data_ptr(), (int)n, (int)h, (int)w, (int)ci, (int)hid, (int)co, (int)stride,
                                             &k1.st, &k2.st, w3.data_ptr(), &e, ws.data_ptr(), ws_bytes, current_stream()),
               "torch_mlu::qconv2d_irb");
  return std::make_tuple(o.y, o.q);
}

// The first layers in one call (catchq_first_layers_nchw): x [N,C,H,W] fp32, w [Co,kh,kw4,4] int8 (filter rows padded
// with zero taps to a multiple of 4, and to 4 channels) -> the pooled int8 tensor [N,Hp,Wp,Co].
Tensor qconv2d_first_layers_op(const Tensor &x, int64_t x_position, double x_scale, const Tensor &w, int64_t exp2,
                               const c10::optional<Tensor> &chan_div, const c10::optional<Tensor> &bias, int64_t act,
                               int64_t q_position, int64_t kw, int64_t stride, int64_t pad, int64_t pool_k,
                               int64_t pool_stride, int64_t pool_pad) {
  c10::DeviceGuard guard(x.device());
  TORCH_CHECK(x.dim() == 4 && x.is_contiguous() && x.scalar_type() == at::kFloat,
              "qconv2d_first_layers expects a contiguous fp32 NCHW input");
  TORCH_CHECK(w.dim() == 4 && w.is_contiguous() && w.scalar_type() == at::kChar && w.device() == x.device(),
              "qconv2d_first_layers expects int8 filters [Co, kh, kw4, 4] on the input's device");
  const int64_t n = x.size(0), c = x.size(1), h = x.size(2), wd = x.size(3), co = w.size(0), kh = w.size(1);
  TORCH_CHECK(w.size(3) == 4 && w.size(2) == (kw + 3) / 4 * 4 && c <= 4,
              "qconv2d_first_layers: filter rows of ", (kw + 3) / 4 * 4, " taps x 4 channels expected");
  TORCH_CHECK(x_position >= -126 && x_position <= 126, "input position out of range");
  StageKeep k;
  fill_stage(&k, w, exp2, chan_div, bias, act, q_position, co, "first-layer constants");
  size_t ws_bytes = 0;
  check_status(catchq_first_layers_workspace_size((int)n, (int)c, (int)h, (int)wd, (int)co, (int)kh, (int)kw, (int)stride,
                                                  (int)pad, &k.st, (int)pool_k, (int)pool_stride, (int)pool_pad,
                                                  t_launch_sharing, &ws_bytes),
               "torch_mlu::qconv2d_first_layers");
  const int hc = catchq_conv_out_size((int)h, (int)kh, (int)pad, (int)stride, 1);
  const int wc = catchq_conv_out_size((int)wd, (int)kw, (int)pad, (int)stride, 1);
  const int hp = catchq_conv_out_size(hc, (int)pool_k, (int)pool_pad, (int)pool_stride, 1);
  const int wp = catchq_conv_out_size(wc, (int)pool_k, (int)pool_pad, (int)pool_stride, 1);
  Tensor q = at::empty({n, hp, wp, co}, x.options().dtype(at::kChar));
  if (n == 0) return q;
  Tensor ws = at::empty({(int64_t)std::max<size_t>(ws_bytes, 16)}, x.options().dtype(at::kChar));
  check_status(catchq_first_layers_nchw(x.data_ptr<float>(), (int)n, (int)c, (int)h, (int)wd, (int)x_position, (float)x_scale,
                                        (int)co, (int)kh, (int)kw, (int)stride, (int)pad, &k.st, (int)pool_k,
                                        (int)pool_stride, (int)pool_pad, q.data_ptr(), t_launch_sharing, ws.data_ptr(), ws_bytes,
                                        current_stream()),
               "torch_mlu::qconv2d_first_layers");
  return q;
}

// A 1x1 convolution and the global average pooling behind it (catchq_conv1x1_avgpool_nhwc): qx [N,H,W,Ci] int8 NHWC,
// qw [Co,Ci] or [Co,1,1,Ci] int8, resid [N,H,W,Co] fp32 -> (fp32 means [N,Co] or an undefined tensor,
// means quantized at (q_position, q_scale) [N,Co] or an undefined tensor)
std::tuple<Tensor, Tensor> qconv2d_avgpool_op(const Tensor &qx, const Tensor &qw, int64_t exp2,
                                              const c10::optional<Tensor> &chan_div, const c10::optional<Tensor> &bias,
                                              const c10::optional<Tensor> &resid, int64_t act, bool want_mean,
                                              int64_t q_bitwidth, int64_t q_position, double q_scale) {
  c10::DeviceGuard guard(qx.device());
  TORCH_CHECK(qx.dim() == 4 && qx.is_contiguous() && qw.is_contiguous() && qx.scalar_type() == at::kChar &&
                  qw.scalar_type() == at::kChar && qw.device() == qx.device(),
              "qconv2d_avgpool expects contiguous int8 NHWC activations and int8 filters on one device");
  const int64_t n = qx.size(0), hw = qx.size(1) * qx.size(2), ci = qx.size(3), co = qw.size(0);
  TORCH_CHECK(qw.numel() == co * ci, "qconv2d_avgpool: the filters must be [", co, ", ", ci, "]");
  TORCH_CHECK(want_mean || q_bitwidth != 0, "qconv2d_avgpool: no output requested");
  TORCH_CHECK(q_bitwidth == 0 || q_bitwidth == 8 || q_bitwidth == 16, "bitwidth not support");
  TORCH_CHECK(exp2 >= -126 && exp2 <= 126, "position sum out of range");
  catchq_epilogue_t e;
  std::memset(&e, 0, sizeof(e));
  e.exp2 = (int)exp2;
  e.act = (int)act;
  e.sharing = t_launch_sharing;
  Tensor cd = as_f32_vec(chan_div, co, "qconv2d_avgpool constants"), bs = as_f32_vec(bias, co, "qconv2d_avgpool constants"), rcp, rs;
  if (cd.defined()) {
    e.chan_div = cd.data_ptr<float>();
    rcp = reciprocals_for(cd);
    if (rcp.defined()) e.chan_rcp = rcp.data_ptr<float>();
  }
  if (bs.defined()) e.bias = bs.data_ptr<float>();
  if (resid.has_value() && resid->defined()) {
    rs = *resid;
    TORCH_CHECK(rs.scalar_type() == at::kFloat && rs.is_contiguous() && rs.numel() == n * hw * co && rs.device() == qx.device(),
                "qconv2d_avgpool: the residual must be a contiguous fp32 [N,H,W,Co] tensor on the input's device");
    e.resid = rs.data_ptr<float>();
  }
  Tensor mean, q;
  if (want_mean) mean = at::empty({n, co}, qx.options().dtype(at::kFloat));
  if (q_bitwidth) q = at::empty({n, co}, qx.options().dtype(int_type((int)q_bitwidth)));
  if (n == 0) return std::make_tuple(mean, q);
  size_t ws_bytes = 0;
  check_status(catchq_conv1x1_avgpool_workspace_size((int)n, (int)hw, (int)ci, (int)co, &e, &ws_bytes), "torch_mlu::qconv2d_avgpool");
  Tensor ws = at::empty({(int64_t)std::max<size_t>(ws_bytes, 16)}, qx.options().dtype(at::kChar));
  check_status(catchq_conv1x1_avgpool_nhwc(qx.data_ptr(), qw.data_ptr(), (int)n, (int)hw, (int)ci, (int)co, &e,
                                           mean.defined() ? mean.data_ptr<float>() : nullptr,
                                           q.defined() ? q.data_ptr() : nullptr, (int)q_bitwidth, (int)q_position,
                                           (float)q_scale, ws.data_ptr(), ws_bytes, current_stream()),
               "torch_mlu::qconv2d_avgpool");
  return std::make_tuple(mean, q);
}

// Residual chain (catchq_conv1x1_chain_nhwc): xs[i] [N,Hi,Wi,Ci] int8 NHWC, ws[i] [Co,Ci] or [Co,1,1,Ci] int8;
// link 0 is the projection shortcut, links 1.. the blocks' last 1x1 convolutions in order.
std::tuple<Tensor, Tensor> qconv2d_chain_op(at::TensorList xs, at::TensorList ws, at::IntArrayRef strides,
                                            at::IntArrayRef exp2s, at::TensorList chan_divs, at::TensorList biases,
                                            bool want_y, int64_t q_bitwidth, int64_t q_position) {
  const size_t nl = xs.size();
  TORCH_CHECK(nl >= 2 && nl <= CATCHQ_CHAIN_MAX_LINKS, "qconv2d_chain: 2 .. ", CATCHQ_CHAIN_MAX_LINKS, " links expected");
  TORCH_CHECK(ws.size() == nl && strides.size() == nl && exp2s.size() == nl && chan_divs.size() == nl && biases.size() == nl,
              "qconv2d_chain: one entry per link expected in every list");
  TORCH_CHECK(q_bitwidth == 0 || q_bitwidth == 8, "qconv2d_chain: int8 or no quantized output");
  TORCH_CHECK(want_y || q_bitwidth == 8, "qconv2d_chain: no output requested");
  c10::DeviceGuard guard(xs[0].device());
  const int64_t n = xs[0].size(0), co = ws[0].size(0);
  int ho = 0, wo = 0;
  catchq_chain_link_t links[CATCHQ_CHAIN_MAX_LINKS];
  std::vector<Tensor> keep;
  for (size_t i = 0; i < nl; ++i) {
    const Tensor &x = xs[i], &w = ws[i];
    TORCH_CHECK(x.dim() == 4 && x.is_contiguous() && x.scalar_type() == at::kChar && x.size(0) == n,
                "qconv2d_chain: int8 NHWC activations of one batch expected");
    TORCH_CHECK(w.is_contiguous() && w.scalar_type() == at::kChar && w.size(0) == co && w.numel() == co * x.size(3),
                "qconv2d_chain: int8 [Co,Ci] filters expected");
    TORCH_CHECK(x.device() == xs[0].device() && w.device() == xs[0].device() && chan_divs[i].device() == xs[0].device() &&
                    biases[i].device() == xs[0].device(),
                "qconv2d_chain: every link's tensors must live on one device");
    const int h = catchq_conv_out_size((int)x.size(1), 1, 0, (int)strides[i], 1);
    const int w_ = catchq_conv_out_size((int)x.size(2), 1, 0, (int)strides[i], 1);
    if (i == 0) { ho = h; wo = w_; }
    TORCH_CHECK(h == ho && w_ == wo && ho > 0 && wo > 0, "qconv2d_chain: the links' output grids differ");
    Tensor cd = as_f32_vec(chan_divs[i], co, "chan_div"), bs = as_f32_vec(biases[i], co, "bias");
    Tensor rcp = reciprocals_for(cd);
    TORCH_CHECK(rcp.defined(), "qconv2d_chain: a divisor without a usable reciprocal");
    keep.push_back(cd); keep.push_back(bs); keep.push_back(rcp);
    links[i].x = x.data_ptr(); links[i].w = w.data_ptr();
    links[i].in_h = (int)x.size(1); links[i].in_w = (int)x.size(2); links[i].ci = (int)x.size(3);
    links[i].stride = (int)strides[i];
    links[i].exp2 = (int)exp2s[i];
    links[i].chan_div = cd.data_ptr<float>(); links[i].chan_rcp = rcp.data_ptr<float>(); links[i].bias = bs.data_ptr<float>();
  }
  Tensor y, q;
  if (want_y) y = at::empty({n, ho, wo, co}, xs[0].options().dtype(at::kFloat));
  if (q_bitwidth == 8) q = at::empty({n, ho, wo, co}, xs[0].options().dtype(at::kChar));
  if (n == 0) return std::make_tuple(y, q);
  check_status(catchq_conv1x1_chain_nhwc(links, (int)nl, (int)n, ho, wo, (int)co, want_y ? y.data_ptr<float>() : nullptr,
                                         q.defined() ? q.data_ptr() : nullptr, (int)q_position, t_launch_sharing, current_stream()),
               "torch_mlu::qconv2d_chain");
  return std::make_tuple(y, q);
}

std::tuple<Tensor, Tensor, Tensor> qlinear_op(const Tensor &qx, const Tensor &qw, int64_t exp2,
                                              const c10::optional<Tensor> &chan_div,
                                              const c10::optional<Tensor> &bias, int64_t act, bool want_y,
                                              bool y_half, bool want_acc, int64_t q_bitwidth,
                                              int64_t q_position, double q_scale) {
  c10::DeviceGuard guard(qx.device());
  return tup(qlinear_impl(qx, qw,
                          make_args(exp2, chan_div, bias, c10::nullopt, act, want_y, y_half, want_acc, q_bitwidth,
                                    q_position, q_scale)));
}

// cnnl_mm(self, self_position, other, other_position, false, true): fp32 output
Tensor mm_q_op(const Tensor &a, int64_t pos_a, const Tensor &b, int64_t pos_b) {
  c10::DeviceGuard guard(a.device());
  EpiArgs args;
  args.exp2 = pos_a + pos_b;
  return qlinear_impl(a.contiguous(), b.contiguous(), args).y;
}

// fp NCHW (or channels-last) activations -> NHWC integer tensor [N,H,W,cpad]
Tensor quantize_to_nhwc(const Tensor &x, int bw, int pos, int64_t cpad, float scale = 1.0f) {
  const int dt = fp_dtype(x, "quantify only support input float/half");
  TORCH_CHECK(x.dim() == 4, "a 4-d activation tensor is expected");
  const int64_t n = x.size(0), c = x.size(1), h = x.size(2), w = x.size(3);
  if (cpad < c) cpad = c;
  Tensor q = at::empty({n, h, w, cpad}, x.options().dtype(int_type(bw)));
  if (cpad == c && x.is_contiguous(at::MemoryFormat::ChannelsLast)) {
    check_status(catchq_quantize(x.data_ptr(), dt, q.data_ptr(), bw, x.numel(), pos, scale, current_stream()),
                 "torch_mlu::quantize");
    return q;
  }
  Tensor xc = x.is_contiguous() ? x : x.contiguous();
  check_status(catchq_quantize_nchw_to_nhwc(xc.data_ptr(), dt, q.data_ptr(), bw, (int)n, (int)c, (int)h, (int)w,
                                            (int)cpad, pos, scale, current_stream()),
               "torch_mlu::quantize");
  return q;
}

Tensor quantize_nhwc_op(const Tensor &x, int64_t bitwidth, int64_t position, int64_t cpad, double scale) {
  c10::DeviceGuard guard(x.device());
  return quantize_to_nhwc(x, (int)bitwidth, (int)position, cpad, (float)scale);
}

// [N,C,H,W] floating -> [N, out_h, out_w, cpad] integers, the image at (top, left), zeros around it
Tensor quantize_nhwc_frame_op(const Tensor &x, int64_t bitwidth, int64_t position, int64_t cpad, int64_t out_h,
                              int64_t out_w, int64_t top, int64_t left, double scale) {
  c10::DeviceGuard guard(x.device());
  const int dt = fp_dtype(x, "quantify only support input float/half");
  TORCH_CHECK(x.dim() == 4, "a 4-d activation tensor is expected");
  Tensor xc = x.contiguous();
  Tensor q = at::empty({x.size(0), out_h, out_w, cpad}, x.options().dtype(int_type(bitwidth)));
  check_status(catchq_quantize_nchw_to_nhwc_frame(xc.data_ptr(), dt, q.data_ptr(), (int)bitwidth, (int)x.size(0),
                                                  (int)x.size(1), (int)x.size(2), (int)x.size(3), (int)cpad,
                                                  (int)out_h, (int)out_w, (int)top, (int)left, (int)position, (float)scale,
                                                  current_stream()),
               "torch_mlu::quantize");
  return q;
}

// ------------------------------------------------------------------------------------------------
// the two reference ops
// ------------------------------------------------------------------------------------------------

// Decoded q_scale / q_mode plus the quantized weight, kept per weight tensor so that steady-state
// calls neither copy the parameters to the host nor re-quantize the weight (the reference does both
// on every call: quantify_conv_forward.cpp:74-75,100-101,114,119-120).  An entry is valid while the
// same tensor objects, at the same versions, are passed again.
struct Prepared {
  c10::weak_intrusive_ptr<c10::TensorImpl> w_impl, s_impl, m_impl;
  uint32_t w_ver = 0, s_ver = 0, m_ver = 0;
  const void *w_ptr = nullptr, *s_ptr = nullptr, *m_ptr = nullptr;
  Tensor s_host, m_host;  // the q-params as read when the entry was made (compared by content when they live on the host)
  c10::StreamId made_on = 0;  // stream that allocated and filled qw / new_scale
  int bw_x = 8, bw_w = 8, pos_x = 0, pos_w = 0;
  bool per_channel = false;
  bool params_half = false;  // per-channel parameters derived with half tensor ops (half q_scale, int8)
  int variant = 0;   // caller's layout choice for qw (part of the cache key)
  Tensor qw;         // conv: [Co,kh,kw,Ci/g]; linear: [N,K]
  Tensor new_scale;  // device fp32 [Co] when per_channel
  // recorded on the stream that quantized the weight, behind those kernels: a later call on another stream
  // (another thread's, a side stream) waits for it before it reads qw / new_scale
  at::cuda::CUDAEvent ready;
  Prepared() : w_impl(c10::weak_intrusive_ptr<c10::TensorImpl>::reclaim(nullptr)),
               s_impl(c10::weak_intrusive_ptr<c10::TensorImpl>::reclaim(nullptr)),
               m_impl(c10::weak_intrusive_ptr<c10::TensorImpl>::reclaim(nullptr)) {}
};

uint32_t version_of(const Tensor &t) {
  // inference tensors carry no version counter
  return t.is_inference() ? 0u : t.unsafeGetTensorImpl()->version_counter().current_version();
}

bool cache_enabled() {
  static const bool on = [] {
    const char *v = std::getenv("CATCHQ_WEIGHT_CACHE");
    return !(v && v[0] == '0');
  }();
  return on;
}

std::mutex g_cache_mutex;
std::unordered_map<const c10::TensorImpl *, std::shared_ptr<Prepared>> g_cache;

bool still_valid(const Prepared &p, const Tensor &w, const Tensor &s, const Tensor &m) {
  auto same = [](const c10::weak_intrusive_ptr<c10::TensorImpl> &weak, const Tensor &t, uint32_t ver) {
    return !weak.expired() && weak._unsafe_get_target() == t.unsafeGetTensorImpl() && version_of(t) == ver;
  };
  if (!(same(p.w_impl, w, p.w_ver) && same(p.s_impl, s, p.s_ver) && same(p.m_impl, m, p.m_ver) &&
        p.w_ptr == w.data_ptr() && p.s_ptr == s.data_ptr() && p.m_ptr == m.data_ptr()))
    return false;
  // Tensors without a version counter (inference tensors) and `.data =` swaps that keep the storage cannot be
  // told apart by identity.  q-params that live on the host are compared by content (a few bytes); for device
  // tensors the storage address above is what is checked -- reading them back would be the host synchronisation
  // this cache exists to avoid (after writing into such a tensor in place, call torch_mlu::clear_weight_cache).
  auto same_content = [](const Tensor &now, const Tensor &then) {
    if (!now.device().is_cpu()) return true;
    return now.numel() == then.numel() && now.scalar_type() == then.scalar_type() && at::equal(now.contiguous(), then);
  };
  return same_content(s, p.s_host) && same_content(m, p.m_host);
}

c10::weak_intrusive_ptr<c10::TensorImpl> weak_of(const Tensor &t) {
  return c10::weak_intrusive_ptr<c10::TensorImpl>(t.getIntrusivePtr());
}

// Decode the two q-param encodings and quantize the weight (make_dense(weight, activation bit width)
// returns it dense, dim 0 slowest, in the layout the caller's kernel wants).
template <typename MakeDense>
std::shared_ptr<Prepared> prepare(MakeDense make_dense, const Tensor &weight, const Tensor &q_scale,
                                  const Tensor &q_mode) {
  auto p = std::make_shared<Prepared>();
  Tensor s_host = q_scale.to(at::kCPU).to(at::kFloat).contiguous();
  Tensor m_host = q_mode.to(at::kCPU).to(at::kInt).contiguous();
  const float *s = s_host.data_ptr<float>();
  const int32_t *m = m_host.data_ptr<int32_t>();
  int bw_act = 8;
  if (m_host.numel() == 1) {
    TORCH_CHECK(m[0] >= 1 && m[0] <= 4, "quantized_mode must be 1, 2, 3 or 4, got ", m[0]);
    bw_act = (m[0] == 1 || m[0] == 3) ? 8 : 16;
  } else {
    TORCH_CHECK(m_host.numel() == 2 && s_host.numel() == 2, "q_scale/q_mode must hold two values each");
    bw_act = (int)s[0];
  }
  const Tensor w_dense = make_dense(weight, bw_act);
  if (m_host.numel() == 1) {
    // CNML-compatible encoding: q_mode in {1:int8, 2:int16, 3:int8 per-channel, 4:int16 per-channel},
    // q_scale = [s_in, s_w | 0, s_c0 ...]   (quantify_conv_forward.cpp:77-131; linear.cpp:81-144)
    const int mode = m[0];
    TORCH_CHECK(mode >= 1 && mode <= 4, "quantized_mode must be 1, 2, 3 or 4, got ", mode);
    const int bw = (mode == 1 || mode == 3) ? 8 : 16;
    p->bw_x = p->bw_w = bw;
    p->per_channel = mode > 2;
    TORCH_CHECK(s_host.numel() >= 2, "q_scale needs at least [input_scale, weight_scale]");
    check_status(catchq_pos_from_scale(bw, s[0], &p->pos_x), "input position");
    if (!p->per_channel) {
      check_status(catchq_pos_from_scale(bw, s[1], &p->pos_w), "weight position");
      p->qw = quantize_op(w_dense, bw, p->pos_w, 1.0);
    } else {
      const int64_t co = w_dense.size(0);
      TORCH_CHECK(s_host.numel() == 2 + co, "per-channel q_scale must hold 2 + ", co, " values, got ", s_host.numel());
      p->params_half = half_chain(q_scale, bw);
      PerChannel pc = p->params_half
                          ? per_channel_params_half(q_scale.reshape({-1}).slice(0, 2), bw, w_dense.options())
                          : per_channel_params(s + 2, co, bw, w_dense.options());
      p->pos_w = pc.new_pos;
      p->new_scale = pc.new_scale;
      p->qw = quantize_weight_per_channel(w_dense, pc, bw);
    }
  } else {
    // CNNL encoding: q_scale = [bitwidth_in, bitwidth_w], q_mode = [pos_in, pos_w]
    // (quantify_conv_forward.cpp:132-145; linear.cpp:145-166)
    TORCH_CHECK(m_host.numel() == 2 && s_host.numel() == 2, "q_scale/q_mode must hold two values each");
    p->bw_x = (int)s[0];
    p->bw_w = (int)s[1];
    TORCH_CHECK((p->bw_x == 8 || p->bw_x == 16) && (p->bw_w == 8 || p->bw_w == 16), "bitwidth not support");
    p->pos_x = m[0];
    p->pos_w = m[1];
    p->qw = quantize_op(w_dense, p->bw_w, p->pos_w, 1.0);
  }
  p->w_impl = weak_of(weight); p->s_impl = weak_of(q_scale); p->m_impl = weak_of(q_mode);
  p->w_ver = version_of(weight); p->s_ver = version_of(q_scale); p->m_ver = version_of(q_mode);
  p->w_ptr = weight.data_ptr();
  p->s_ptr = q_scale.data_ptr();
  p->m_ptr = q_mode.data_ptr();
  p->s_host = q_scale.to(at::kCPU).contiguous().clone();
  p->m_host = q_mode.to(at::kCPU).contiguous().clone();
  return p;
}

template <typename MakeDense>
std::shared_ptr<Prepared> prepared_for(const Tensor &weight, const Tensor &q_scale, const Tensor &q_mode,
                                       MakeDense make_dense, int variant = 0) {
  const bool use_cache = cache_enabled();
  const c10::TensorImpl *key = weight.unsafeGetTensorImpl();
  if (use_cache) {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    auto it = g_cache.find(key);
    if (it != g_cache.end()) {
      if (it->second->variant == variant && still_valid(*it->second, weight, q_scale, q_mode)) {
        const auto cur = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
        if (!it->second->ready.query())  // still in flight on the stream that prepared it
          it->second->ready.block(cur);
        if (cur.id() != it->second->made_on) {
          // read on another stream than the one the caching allocator knows these blocks by: tell it, so that
          // an entry dropped while this stream's kernels still read it is not handed out again too early
          it->second->qw.record_stream(cur);
          if (it->second->new_scale.defined()) it->second->new_scale.record_stream(cur);
        }
        return it->second;
      }
      g_cache.erase(it);
    }
  }
  auto p = prepare(make_dense, weight, q_scale, q_mode);
  p->variant = variant;
  const auto made_on = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  p->made_on = made_on.id();
  p->ready.record(made_on);
  if (use_cache) {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    // every miss sweeps out the entries whose weight tensor is gone (their quantized copies are device memory;
    // misses are first uses of a weight, so the sweep is off the steady-state path)
    for (auto it = g_cache.begin(); it != g_cache.end();)
      it = it->second->w_impl.expired() ? g_cache.erase(it) : std::next(it);
    g_cache[key] = p;
  }
  return p;
}

int64_t cache_size_op() {
  std::lock_guard<std::mutex> lock(g_cache_mutex);
  return (int64_t)g_cache.size();
}

void clear_cache_op() {
  {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    g_cache.clear();
  }
  std::lock_guard<std::mutex> lock(g_rcp_mutex);
  g_rcp_cache.clear();
}

// quantized activations [N,H,W,Ci] x prepared weight -> floating [N,Ho,Wo,Co]
Tensor conv_prepared(const Tensor &qx, const Prepared &prep, const Tensor &bias, at::IntArrayRef padding,
                     at::IntArrayRef stride, at::IntArrayRef dilation, int64_t groups, bool half) {
  Tensor qw = prep.qw.permute({0, 2, 3, 1});  // view of the same memory as [Co,kh,kw,Ci/g], contiguous
  EpiArgs a;
  a.exp2 = prep.pos_x + prep.pos_w;
  if (prep.per_channel) a.chan_div = prep.new_scale;
  if (has_bias(bias)) a.bias = bias;
  a.y_half = half;
  // per-channel branch on half tensors: the vendor convolution's half output, then `/ new_scale` and `+ bias` as
  // half tensor ops (quantify_conv_forward.cpp:123-129); where the q-params stayed fp32 (int16), so does this
  a.half_steps = half && prep.per_channel && prep.params_half;
  return qconv2d_impl(qx, qw, padding, stride, dilation, groups, a).y;
}

Tensor conv2d_op(const Tensor &input, const Tensor &weight, const Tensor &bias, at::IntArrayRef padding,
                 at::IntArrayRef stride, at::IntArrayRef dilation, int64_t groups, const Tensor &q_scale,
                 const Tensor &q_mode) {
  TORCH_CHECK(input.dim() > 2, "Input's dim must greater than 2!");
  TORCH_CHECK(input.dim() == 4 && weight.dim() == 4, "torch_mlu::conv2d expects 4-d input and weight");
  const bool half = fp_dtype(input, "quantify only support input float/half") == CATCHQ_F16;
  c10::DeviceGuard guard(input.device());
  // Channel counts the matrix-core routes cannot take are padded with zero channels on both operands
  // (int8: multiples of 16, int16: multiples of 8); zeros on one side of every added product.  An image of
  // fewer than four channels (grey, RGB) takes four, and the int8 path also quantizes it into a zero frame
  // that holds the convolution's padding and pads the filter rows to whole groups of four taps -- the
  // shape of the streaming first-layer kernel (int16 activations take eight channels and stay unframed).
  const int64_t ci = input.size(1), kw = weight.size(3);
  const bool dense = groups == 1 && weight.size(1) == ci;
  const bool few = dense && ci < 4;
  auto device_channels = [&](int bw_act) -> int64_t {
    if (!dense) return ci;
    if (bw_act == 8) return ci < 4 ? 4 : (ci + 15) / 16 * 16;
    return (ci + 7) / 8 * 8;
  };
  const int64_t kw_extra = (kw + 3) / 4 * 4 - kw;
  const bool can_frame = few && dilation.size() == 2 && dilation[1] == 1 && padding.size() == 2;
  auto prep = prepared_for(weight, q_scale, q_mode, [&](const Tensor &w, int bw_act) {
    Tensor wd = w;
    const int64_t cpad = device_channels(bw_act) - ci;
    const int64_t taps = (few && bw_act == 8 && can_frame) ? kw_extra : 0;
    if (cpad > 0 || taps > 0) wd = at::constant_pad_nd(w, {0, taps, 0, 0, 0, cpad}, 0);
    // the memory of a channels-last [Co,Ci/g,kh,kw] tensor is [Co][kh][kw][Ci/g]
    return wd.contiguous(at::MemoryFormat::ChannelsLast);
  }, (few ? 1 : 0) | (can_frame ? 2 : 0));
  Tensor qx;
  std::vector<int64_t> pad(padding.begin(), padding.end());
  if (few && prep->bw_x == 8 && can_frame) {
    const Tensor xc = input.contiguous();
    const int64_t h = input.size(2), w_in = input.size(3);
    qx = at::empty({input.size(0), h + 2 * pad[0], w_in + 2 * pad[1] + kw_extra, 4}, input.options().dtype(at::kChar));
    check_status(catchq_quantize_nchw_to_nhwc_frame(xc.data_ptr(), half ? CATCHQ_F16 : CATCHQ_F32, qx.data_ptr(), 8,
                                                    (int)input.size(0), (int)ci, (int)h, (int)w_in, 4, (int)qx.size(1),
                                                    (int)qx.size(2), (int)pad[0], (int)pad[1], prep->pos_x, 1.0f,
                                                    current_stream()),
                 "torch_mlu::quantize");
    pad = {0, 0};
  } else {
    qx = quantize_to_nhwc(input, prep->bw_x, prep->pos_x, device_channels(prep->bw_x));
  }
  Tensor y = conv_prepared(qx, *prep, bias, pad, stride, dilation, groups, half);
  return y.permute({0, 3, 1, 2});  // logical NCHW over channels-last memory, like the reference
}

// [N,C,L] x [Co,Ci/g,k]: a convolution over images of one row (the reference's module calls
// torch.ops.torch_mlu.conv1d with the conv2d argument list: core/quantized/modules/conv.py:276-286)
Tensor conv1d_op(const Tensor &input, const Tensor &weight, const Tensor &bias, at::IntArrayRef padding,
                 at::IntArrayRef stride, at::IntArrayRef dilation, int64_t groups, const Tensor &q_scale,
                 const Tensor &q_mode) {
  TORCH_CHECK(input.dim() == 3 && weight.dim() == 3, "torch_mlu::conv1d expects 3-d input and weight");
  TORCH_CHECK(padding.size() == 1 && stride.size() == 1 && dilation.size() == 1, "1-d conv parameters expected");
  const bool half = fp_dtype(input, "quantify only support input float/half") == CATCHQ_F16;
  c10::DeviceGuard guard(input.device());
  auto prep = prepared_for(weight, q_scale, q_mode, [](const Tensor &w, int) {
    return w.unsqueeze(2).contiguous(at::MemoryFormat::ChannelsLast);  // memory [Co][1][k][Ci/g]
  });
  Tensor qx = quantize_to_nhwc(input.unsqueeze(2), prep->bw_x, prep->pos_x, input.size(1));
  Tensor y = conv_prepared(qx, *prep, bias, {0, padding[0]}, {1, stride[0]}, {1, dilation[0]}, groups, half);
  return y.squeeze(1).permute({0, 2, 1});  // [N,Lo,Co] memory seen as [N,Co,Lo]
}

// [N,C,D,H,W] x [Co,Ci/g,kd,kh,kw].  The depth taps are folded into the channel dimension of a 2-d
// convolution over the N*Do output depth slices: channel c*kd+t of slice (n, od) is input channel c at
// depth od*sd - pd + t*dd.  Quantization is per element, so folding the quantized integers gives the
// integers the 3-d convolution would read, and the int32 sums are the same.  With kd == 1 and depth
// stride 1 the fold is a view (the reference's pseudo-conv3d case, internal/quantize_util.cpp:57-139;
// module: core/quantized/modules/conv.py:345-354).
Tensor conv3d_op(const Tensor &input, const Tensor &weight, const Tensor &bias, at::IntArrayRef padding,
                 at::IntArrayRef stride, at::IntArrayRef dilation, int64_t groups, const Tensor &q_scale,
                 const Tensor &q_mode) {
  TORCH_CHECK(input.dim() == 5 && weight.dim() == 5, "torch_mlu::conv3d expects 5-d input and weight");
  TORCH_CHECK(padding.size() == 3 && stride.size() == 3 && dilation.size() == 3, "3-d conv parameters expected");
  const bool half = fp_dtype(input, "quantify only support input float/half") == CATCHQ_F16;
  c10::DeviceGuard guard(input.device());
  const int64_t n = input.size(0), c = input.size(1), dd_in = input.size(2), h = input.size(3), w = input.size(4);
  const int64_t kd = weight.size(2), pd = padding[0], sd = stride[0], dd = dilation[0];
  TORCH_CHECK(sd > 0 && dd > 0 && pd >= 0, "depth stride/dilation must be positive, padding non-negative");
  TORCH_CHECK(groups > 0 && c == weight.size(1) * groups, "channel mismatch: input ", c, ", weight ",
              weight.size(1), " x groups ", groups);
  const int64_t d_out = (dd_in + 2 * pd - dd * (kd - 1) - 1) / sd + 1;
  TORCH_CHECK(dd_in + 2 * pd >= dd * (kd - 1) + 1 && d_out > 0, "Calculated output size is too small");
  auto prep = prepared_for(weight, q_scale, q_mode, [](const Tensor &wt, int) {
    // [Co, (Ci/g)*kd, kh, kw] with the depth tap fastest inside a channel, stored [Co][kh][kw][(Ci/g)*kd]
    return wt.reshape({wt.size(0), wt.size(1) * wt.size(2), wt.size(3), wt.size(4)})
        .contiguous(at::MemoryFormat::ChannelsLast);
  });
  // [N,C,D*H,W] -> integers in [N,D,H,W,C] order
  Tensor q = quantize_to_nhwc(input.contiguous().view({n, c, dd_in * h, w}), prep->bw_x, prep->pos_x, c)
                 .view({n, dd_in, h, w, c});
  Tensor qx;
  if (kd == 1 && sd == 1 && pd == 0) {
    qx = q.view({n * dd_in, h, w, c});
  } else {
    if (pd > 0) q = at::constant_pad_nd(q, {0, 0, 0, 0, 0, 0, pd, pd}, 0);
    std::vector<Tensor> taps;
    for (int64_t t = 0; t < kd; ++t)
      taps.push_back(q.slice(1, t * dd, t * dd + (d_out - 1) * sd + 1, sd));  // [N,Do,H,W,C]
    qx = at::stack(taps, 5).view({n * d_out, h, w, c * kd});
  }
  Tensor y = conv_prepared(qx, *prep, bias, {padding[1], padding[2]}, {stride[1], stride[2]},
                           {dilation[1], dilation[2]}, groups, half);
  return y.view({n, d_out, y.size(1), y.size(2), y.size(3)}).permute({0, 4, 1, 2, 3});  // logical NCDHW
}

// cnnl_quantize_convolution_internal(input, input_position, weight, weight_position, bias, padding, stride,
// dilation, groups, bitwidth)      operators/cnnl/internal/quantize_convolution.cpp:57-235
// float tensors in, positions as int32 device tensors, nothing copied to the host
Tensor quantize_conv2d_op(const Tensor &input, const Tensor &input_position, const Tensor &weight,
                          const Tensor &weight_position, const Tensor &bias, at::IntArrayRef padding,
                          at::IntArrayRef stride, at::IntArrayRef dilation, int64_t groups, int64_t input_bitwidth,
                          int64_t weight_bitwidth) {
  TORCH_CHECK(input.dim() == 4 && weight.dim() == 4, "conv2d only support 4 dims.");
  TORCH_CHECK(padding.size() == 2 && stride.size() == 2 && dilation.size() == 2, "padding/stride/dilation: two values each");
  const int x_dt = fp_dtype(input, "quantify only support input float/half");
  const int w_dt = fp_dtype(weight, "quantify only support input float/half");
  TORCH_CHECK((input_bitwidth == 8 || input_bitwidth == 16) && (weight_bitwidth == 8 || weight_bitwidth == 16),
              "bitwidth not support");
  TORCH_CHECK(input_position.scalar_type() == at::kInt && weight_position.scalar_type() == at::kInt &&
                  input_position.numel() == 1 && weight_position.numel() == 1 &&
                  input_position.device() == input.device() && weight_position.device() == input.device(),
              "positions must be int32 tensors of one element on the input's device");
  if (has_bias(bias)) TORCH_CHECK(bias.dim() == 1 && bias.size(0) == weight.size(0), "currently only support 1-dim bias");
  c10::DeviceGuard guard(input.device());
  Tensor x = input.contiguous(at::MemoryFormat::ChannelsLast);   // memory [N][H][W][C]
  Tensor w = weight.contiguous(at::MemoryFormat::ChannelsLast);  // memory [Co][kh][kw][Ci/g]
  catchq_conv_desc_t d = {(int)x.size(0), (int)x.size(2), (int)x.size(3), (int)x.size(1), (int)w.size(0),
                          (int)w.size(2), (int)w.size(3), (int)padding[0], (int)padding[1], (int)stride[0],
                          (int)stride[1], (int)dilation[0], (int)dilation[1], (int)groups};
  TORCH_CHECK(groups > 0 && x.size(1) == w.size(1) * groups, "channel mismatch: input ", input.sizes(), ", weight ",
              weight.sizes(), ", groups ", groups);
  size_t ws_bytes = 0;
  check_status(catchq_quantize_conv2d_workspace_size(&d, (int)input_bitwidth, (int)weight_bitwidth, &ws_bytes),
               "torch_mlu::quantize_conv2d");
  const int ho = catchq_conv_out_size(d.h, d.kh, d.pad_h, d.stride_h, d.dil_h);
  const int wo = catchq_conv_out_size(d.w, d.kw, d.pad_w, d.stride_w, d.dil_w);
  Tensor workspace = at::empty({(int64_t)ws_bytes}, x.options().dtype(at::kChar));
  Tensor y = at::empty({d.n, ho, wo, d.co}, x.options());
  Tensor bs = has_bias(bias) ? bias.to(at::kFloat).contiguous() : Tensor();
  check_status(catchq_quantize_conv2d_nhwc(x.data_ptr(), x_dt, input_position.data_ptr<int32_t>(), (int)input_bitwidth,
                                           w.data_ptr(), w_dt, weight_position.data_ptr<int32_t>(),
                                           (int)weight_bitwidth, &d, bs.defined() ? bs.data_ptr<float>() : nullptr,
                                           y.data_ptr(), x_dt, workspace.data_ptr(), ws_bytes, current_stream()),
               "torch_mlu::quantize_conv2d");
  return y.permute({0, 3, 1, 2});
}

Tensor linear_op(const Tensor &input, const Tensor &weight, const Tensor &bias, const Tensor &q_scale,
                 const Tensor &q_mode) {
  TORCH_CHECK(weight.dim() == 2, "we only support the  dim of weight is 2");
  fp_dtype(input, "quantify only support input float/half");
  TORCH_CHECK(input.dim() >= 1 && input.size(-1) == weight.size(1), "size mismatch: input ", input.sizes(),
              ", weight ", weight.sizes());
  c10::DeviceGuard guard(input.device());
  // K is padded with zeros on both operands to what the matrix-core routes take (16 int8 / 8 int16 values)
  const int64_t k = weight.size(1);
  auto device_k = [&](int bw_act) { return bw_act == 8 ? (k + 15) / 16 * 16 : (k + 7) / 8 * 8; };
  auto prep = prepared_for(weight, q_scale, q_mode, [&](const Tensor &w, int bw_act) {
    const int64_t kpad = device_k(bw_act) - k;
    return kpad > 0 ? at::constant_pad_nd(w, {0, kpad}, 0).contiguous() : w.contiguous();
  });
  Tensor x2 = input.contiguous().view({-1, k});
  Tensor qx;
  if (device_k(prep->bw_x) != k && x2.size(0) > 0)  // rows as pixels of a [M, K, 1, 1] image, zero channels appended
    qx = quantize_to_nhwc(x2.view({x2.size(0), k, 1, 1}), prep->bw_x, prep->pos_x, device_k(prep->bw_x))
             .view({x2.size(0), device_k(prep->bw_x)});
  else if (device_k(prep->bw_x) != k)
    qx = at::empty({0, device_k(prep->bw_x)}, x2.options().dtype(int_type(prep->bw_x)));
  else
    qx = quantize_op(x2, prep->bw_x, prep->pos_x, 1.0);
  EpiArgs a;  // output is fp32 whatever the input type (operators/cnnl/matmul.cpp:72-74)
  a.exp2 = prep->pos_x + prep->pos_w;
  if (prep->per_channel) a.chan_div = prep->new_scale;
  if (has_bias(bias)) a.bias = bias;
  EpiOut o = qlinear_impl(qx, prep->qw, a);
  std::vector<int64_t> shape(input.sizes().begin(), input.sizes().end() - 1);
  shape.push_back(weight.size(0));
  return o.y.view(shape);
}

// x [N,H,W,C] contiguous int8 / int16 / fp32
Tensor maxpool_nhwc_op(const Tensor &x, int64_t k, int64_t stride, int64_t pad) {
  TORCH_CHECK(x.dim() == 4 && x.is_contiguous(), "maxpool_nhwc expects a contiguous [N,H,W,C] tensor");
  int bits = 0;
  switch (x.scalar_type()) {
    case at::kChar: bits = 8; break;
    case at::kShort: bits = 16; break;
    case at::kFloat: bits = 32; break;
    default: TORCH_CHECK(false, "maxpool_nhwc: int8, int16 or float32 expected");
  }
  c10::DeviceGuard guard(x.device());
  const int64_t ho = (x.size(1) + 2 * pad - k) / stride + 1, wo = (x.size(2) + 2 * pad - k) / stride + 1;
  TORCH_CHECK(ho > 0 && wo > 0, "Calculated output size is too small");
  Tensor y = at::empty({x.size(0), ho, wo, x.size(3)}, x.options());
  check_status(catchq_maxpool_nhwc(x.data_ptr(), y.data_ptr(), bits, (int)x.size(0), (int)x.size(1), (int)x.size(2),
                                   (int)x.size(3), (int)k, (int)stride, (int)pad, current_stream()),
               "torch_mlu::maxpool_nhwc");
  return y;
}

// x [N,H,W,C] contiguous fp32 -> [N,C]: the fp32 means, or (q_bitwidth 8 / 16) the means quantized at
// (q_position, q_scale) in the same launch
Tensor global_avgpool_nhwc_op(const Tensor &x, int64_t q_bitwidth, int64_t q_position, double q_scale) {
  TORCH_CHECK(x.dim() == 4 && x.is_contiguous() && x.scalar_type() == at::kFloat,
              "global_avgpool_nhwc expects a contiguous fp32 [N,H,W,C] tensor");
  c10::DeviceGuard guard(x.device());
  if (q_bitwidth != 0) {
    TORCH_CHECK(q_bitwidth == 8 || q_bitwidth == 16, "bitwidth not support");
    Tensor q = at::empty({x.size(0), x.size(3)}, x.options().dtype(int_type((int)q_bitwidth)));
    check_status(catchq_global_avgpool_quantize_nhwc(x.data_ptr<float>(), q.data_ptr(), (int)q_bitwidth, (int)x.size(0),
                                                     (int)(x.size(1) * x.size(2)), (int)x.size(3), (int)q_position,
                                                     (float)q_scale, current_stream()),
                 "torch_mlu::global_avgpool_nhwc");
    return q;
  }
  Tensor y = at::empty({x.size(0), x.size(3)}, x.options());
  check_status(catchq_global_avgpool_nhwc(x.data_ptr<float>(), y.data_ptr<float>(), (int)x.size(0),
                                          (int)(x.size(1) * x.size(2)), (int)x.size(3), current_stream()),
               "torch_mlu::global_avgpool_nhwc");
  return y;
}

std::string conv2d_route_op(int64_t x_bits, int64_t w_bits, at::IntArrayRef in_nhwc, at::IntArrayRef w_ohwi,
                            at::IntArrayRef padding, at::IntArrayRef stride, at::IntArrayRef dilation,
                            int64_t groups) {
  catchq_conv_desc_t d = {(int)in_nhwc[0], (int)in_nhwc[1], (int)in_nhwc[2], (int)in_nhwc[3], (int)w_ohwi[0],
                          (int)w_ohwi[1], (int)w_ohwi[2], (int)padding[0], (int)padding[1], (int)stride[0],
                          (int)stride[1], (int)dilation[0], (int)dilation[1], (int)groups};
  return catchq_conv2d_route((int)x_bits, (int)w_bits, &d);
}

}  // namespace

TORCH_LIBRARY(torch_mlu, m) {
  m.def("conv2d(Tensor input, Tensor weight, Tensor bias, int[] padding, int[] stride, int[] dilation, "
        "int groups, Tensor q_scale, Tensor q_mode) -> Tensor");
  m.def("conv1d(Tensor input, Tensor weight, Tensor bias, int[] padding, int[] stride, int[] dilation, "
        "int groups, Tensor q_scale, Tensor q_mode) -> Tensor");
  m.def("conv3d(Tensor input, Tensor weight, Tensor bias, int[] padding, int[] stride, int[] dilation, "
        "int groups, Tensor q_scale, Tensor q_mode) -> Tensor");
  m.def("linear(Tensor input, Tensor weight, Tensor bias, Tensor q_scale, Tensor q_mode) -> Tensor");
  m.def("quantize(Tensor x, int bitwidth, int position, float scale=1.0) -> Tensor");
  m.def("quantize_dev(Tensor x, int bitwidth, Tensor position) -> Tensor");
  m.def("quantize_nhwc(Tensor x, int bitwidth, int position, int cpad=0, float scale=1.0) -> Tensor");
  m.def("quantize_nhwc_frame(Tensor x, int bitwidth, int position, int cpad, int out_h, int out_w, int top, "
        "int left, float scale=1.0) -> Tensor");
  m.def("quantize_param(Tensor x, int bitwidth, int mode) -> (Tensor, Tensor, Tensor)");
  m.def("quantize_per_channel(Tensor w, Tensor scales, int bitwidth) -> (Tensor, Tensor, Tensor)");
  m.def("dequantize(Tensor q, int position, float scale=1.0, bool half=False) -> Tensor");
  m.def("mm_q(Tensor a, int pos_a, Tensor b, int pos_b) -> Tensor");
  m.def("qconv2d(Tensor qx, Tensor qw, int exp2, Tensor? chan_div, Tensor? bias, Tensor? resid, "
        "int[] padding, int[] stride, int[] dilation, int groups, int act=0, bool want_y=True, "
        "bool y_half=False, bool want_acc=False, int q_bitwidth=0, int q_position=0, float q_scale=1.0, "
        "float act_slope=0.0, bool resid_after_act=False) -> (Tensor, Tensor, Tensor)");
  m.def("qconv2d_shortcut(Tensor qx, Tensor qw, int exp2, Tensor? chan_div, Tensor? bias, Tensor sx, Tensor sw, "
        "int s_stride, int s_exp2, Tensor? s_chan_div, Tensor? s_bias, int[] padding, int[] stride, int[] dilation, "
        "int act=0, bool want_y=True, bool y_half=False, int q_bitwidth=0, int q_position=0, float q_scale=1.0, "
        "float act_slope=0.0, bool resid_after_act=False) -> (Tensor, Tensor)");
  m.def("qconv2d_head(Tensor qx, Tensor w1, int exp2_1, Tensor? chan_div1, Tensor? bias1, int q_position1, Tensor qw, "
        "int exp2, Tensor? chan_div, Tensor? bias, int[] padding, int[] stride, int[] dilation, int act=0, "
        "bool want_y=True, bool y_half=False, int q_bitwidth=0, int q_position=0, float q_scale=1.0, "
        "float act_slope=0.0) -> (Tensor, Tensor)");
  m.def("qconv2d_irb(Tensor qx, Tensor w1, int exp2_1, Tensor? chan_div1, Tensor? bias1, int act1, int q_position1, "
        "Tensor wd, int stride, int exp2_2, Tensor? chan_div2, Tensor? bias2, int act2, int q_position2, Tensor w3, "
        "int exp2, Tensor? chan_div, Tensor? bias, Tensor? resid, bool want_y=True, bool y_half=False, "
        "int q_bitwidth=0, int q_position=0, float q_scale=1.0) -> (Tensor, Tensor)");
  m.def("qconv2d_first_layers(Tensor x, int x_position, float x_scale, Tensor w, int exp2, Tensor? chan_div, Tensor? bias, "
        "int act, int q_position, int kw, int stride, int pad, int pool_k, int pool_stride, int pool_pad) -> Tensor");
  m.def("qconv2d_avgpool(Tensor qx, Tensor qw, int exp2, Tensor? chan_div, Tensor? bias, Tensor? resid, int act, "
        "bool want_mean=True, int q_bitwidth=0, int q_position=0, float q_scale=1.0) -> (Tensor, Tensor)");
  m.def("qconv2d_chain(Tensor[] xs, Tensor[] ws, int[] strides, int[] exp2s, Tensor[] chan_divs, Tensor[] biases, "
        "bool want_y=False, int q_bitwidth=8, int q_position=0) -> (Tensor, Tensor)");
  m.def("qlinear(Tensor qx, Tensor qw, int exp2, Tensor? chan_div, Tensor? bias, int act=0, "
        "bool want_y=True, bool y_half=False, bool want_acc=False, int q_bitwidth=0, int q_position=0, "
        "float q_scale=1.0) -> (Tensor, Tensor, Tensor)");
  m.def("quantize_conv2d(Tensor input, Tensor input_position, Tensor weight, Tensor weight_position, Tensor bias, "
        "int[] padding, int[] stride, int[] dilation, int groups, int input_bitwidth=8, int weight_bitwidth=8) -> Tensor");
  m.def("maxpool_nhwc(Tensor x, int k, int stride, int pad) -> Tensor");
  m.def("global_avgpool_nhwc(Tensor x, int q_bitwidth=0, int q_position=0, float q_scale=1.0) -> Tensor");
  m.def("set_launch_sharing(int launches) -> int", &set_launch_sharing_op);
  m.def("conv1x1_conv3x3_fuses(int n, int h, int w, int k1, int cm, int co) -> bool", &head_fuses_op);
  m.def("inverted_residual_fuses(int n, int h, int w, int ci, int hid, int co, int stride) -> bool", &irb_fuses_op);
  m.def("first_layers_fuse(int n, int c, int h, int w, int co, int k, int stride, int pad, int pool_k, int pool_stride, "
        "int pool_pad) -> bool", &first_layers_fuse_op);
  m.def("conv1x1_avgpool_fuses(int n, int hw, int ci, int co) -> bool", &conv_avgpool_fuses_op);
  m.def("clear_weight_cache() -> ()", &clear_cache_op);
  m.def("weight_cache_size() -> int", &cache_size_op);
  m.def("conv2d_route(int x_bits, int w_bits, int[] in_nhwc, int[] w_ohwi, int[] padding, int[] stride, "
        "int[] dilation, int groups) -> str", &conv2d_route_op);
}

TORCH_LIBRARY_IMPL(torch_mlu, CUDA, m) {  // ROCm tensors dispatch on the CUDA key
  m.impl("conv2d", &conv2d_op);
  m.impl("conv1d", &conv1d_op);
  m.impl("conv3d", &conv3d_op);
  m.impl("linear", &linear_op);
  m.impl("quantize", &quantize_op);
  m.impl("quantize_dev", &quantize_dev_op);
  m.impl("quantize_nhwc", &quantize_nhwc_op);
  m.impl("quantize_nhwc_frame", &quantize_nhwc_frame_op);
  m.impl("quantize_param", &quantize_param_op);
  m.impl("quantize_per_channel", &quantize_per_channel_op);
  m.impl("dequantize", &dequantize_op);
  m.impl("mm_q", &mm_q_op);
  m.impl("quantize_conv2d", &quantize_conv2d_op);
  m.impl("qconv2d", &qconv2d_op);
  m.impl("qconv2d_shortcut", &qconv2d_shortcut_op);
  m.impl("qconv2d_head", &qconv2d_head_op);
  m.impl("qconv2d_irb", &qconv2d_irb_op);
  m.impl("qconv2d_first_layers", &qconv2d_first_layers_op);
  m.impl("qconv2d_avgpool", &qconv2d_avgpool_op);
  m.impl("qconv2d_chain", &qconv2d_chain_op);
  m.impl("qlinear", &qlinear_op);
  m.impl("maxpool_nhwc", &maxpool_nhwc_op);
  m.impl("global_avgpool_nhwc", &global_avgpool_nhwc_op);
}
