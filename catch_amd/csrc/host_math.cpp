// Host-side quantization-parameter math (scalars and per-channel vectors; no device work).
#include <atomic>
#include <cmath>
#include <cstdint>
#include <vector>

#include "catchq.h"

#define CATCHQ_API extern "C" __attribute__((visibility("default")))

namespace {

struct Range {
  int n;
  int qmin, qmax;
};

bool range_for(int bitwidth, Range *r) {
  if (bitwidth == 8) {
    *r = {8, -128, 127};
    return true;
  }
  if (bitwidth == 16) {
    *r = {16, -32768, 32767};
    return true;
  }
  return false;
}

}  // namespace

CATCHQ_API int catchq_version(void) { return 104; }

CATCHQ_API const char *catchq_status_string(int status) {
  switch (status) {
    case CATCHQ_OK: return "ok";
    case CATCHQ_ERR_ARG: return "invalid argument";
    case CATCHQ_ERR_DTYPE: return "quantify only support input float/half";
    case CATCHQ_ERR_BITWIDTH: return "bitwidth not support";
    case CATCHQ_ERR_SHAPE: return "inconsistent shapes";
    case CATCHQ_ERR_LAUNCH: return "kernel launch failed";
    case CATCHQ_ERR_UNSUPPORTED: return "combination not supported";
    case CATCHQ_ERR_TOO_LARGE: return "input larger than the fixed scratch memory of this entry point serves";
    default: return "unknown status";
  }
}

// cnnl/cnnl_util.cpp:337-347 -- float absmax, float log over double log(2), floor, minus (bitwidth-2).
CATCHQ_API int catchq_pos_from_scale(int bitwidth, float scale, int *position) {
  Range r;
  if (!position) return CATCHQ_ERR_ARG;
  if (!range_for(bitwidth, &r)) return CATCHQ_ERR_BITWIDTH;
  if (!(scale > 0.0f) || std::isinf(scale)) return CATCHQ_ERR_ARG;  // the logarithm below needs a finite absmax > 0
  const float absmax = r.qmax / scale;
  *position = static_cast<int>(std::floor(std::log(absmax) / std::log(2)) - (bitwidth - 2));
  return CATCHQ_OK;
}

// jit/utils/utils.cpp:81-105 -- the intermediate values live in floats, the expressions in double.
CATCHQ_API int catchq_quant_params(int bitwidth, float scale, int *position, float *scale_frac,
                                   float *scale_factor) {
  Range r;
  if (!position || !scale_frac || !scale_factor) return CATCHQ_ERR_ARG;
  if (!range_for(bitwidth, &r)) return CATCHQ_ERR_BITWIDTH;
  if (!(scale > 0.0f) || std::isinf(scale)) return CATCHQ_ERR_ARG;
  const float absmax = r.qmax / scale;
  const float pos = std::floor(std::log(absmax) / std::log(2)) - (r.n - 2);
  const float frac = std::pow(2, pos) * (std::pow(2, (r.n - 1)) - 1) / absmax;
  const float factor = std::pow(2, pos) / frac;
  *position = static_cast<int>(pos);
  *scale_frac = frac;
  *scale_factor = factor;
  return CATCHQ_OK;
}

// operators/cnnl/quantify.cpp:55-98 -- every step is an fp32 tensor op there, so every step is
// an fp32 scalar op here.
CATCHQ_API int catchq_per_channel_params(int bitwidth, const float *scales, int co, int *new_position,
                                         float *new_scale, float *scale_factor) {
  Range r;
  if (!scales || !new_position || !new_scale || !scale_factor || co <= 0) return CATCHQ_ERR_ARG;
  if (!range_for(bitwidth, &r)) return CATCHQ_ERR_BITWIDTH;
  const float qmax = static_cast<float>(r.qmax);
  for (int c = 0; c < co; ++c)
    if (!(scales[c] > 0.0f) || std::isinf(scales[c])) return CATCHQ_ERR_ARG;
  std::vector<float> pos(co), chan_scale(co);
  float pos_hi = 0.f, pos_lo = 0.f;
  for (int c = 0; c < co; ++c) {
    const float absmax = qmax / scales[c];
    pos[c] = std::floor(std::log2(absmax)) - static_cast<float>(bitwidth - 2);
    chan_scale[c] = (std::exp2(pos[c]) * qmax) / absmax;
    pos_hi = (c == 0) ? pos[c] : std::fmax(pos_hi, pos[c]);
    pos_lo = (c == 0) ? pos[c] : std::fmin(pos_lo, pos[c]);
  }
  const float shared = std::nearbyint((pos_hi + pos_lo) / 2.0f);  // half-to-even
  for (int c = 0; c < co; ++c) {
    new_scale[c] = chan_scale[c] * std::exp2(shared - pos[c]);
    scale_factor[c] = std::exp2(shared) / new_scale[c];
  }
  *new_position = static_cast<int>(shared);
  return CATCHQ_OK;
}

namespace {
// one fp16 tensor op: evaluate in fp32, round the result to binary16
inline float h16(float v) { return static_cast<float>(static_cast<_Float16>(v)); }
inline float bits_to_float(uint16_t b) {
  _Float16 h;
  __builtin_memcpy(&h, &b, 2);
  return static_cast<float>(h);
}
inline uint16_t float_to_bits(float v) {
  const _Float16 h = static_cast<_Float16>(v);
  uint16_t b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}
}  // namespace

// operators/cnnl/quantify.cpp:55-98 when scale_data is a half tensor (a model converted with .half()):
// absmax_pc, log2, pos_pc, scale_pc, new_pos, new_scale and scale_factor are all half tensors there, so
// every step rounds to binary16.
CATCHQ_API int catchq_per_channel_params_f16(int bitwidth, const uint16_t *scales, int co, int *new_position,
                                             uint16_t *new_scale, uint16_t *scale_factor) {
  Range r;
  if (!scales || !new_position || !new_scale || !scale_factor || co <= 0) return CATCHQ_ERR_ARG;
  if (!range_for(bitwidth, &r)) return CATCHQ_ERR_BITWIDTH;
  const float qmax = static_cast<float>(r.qmax);
  std::vector<float> pos(co), chan_scale(co);
  float pos_hi = 0.f, pos_lo = 0.f;
  for (int c = 0; c < co; ++c) {
    const float s = bits_to_float(scales[c]);
    // an int16 scale 32767 / absmax above 65504 is +inf in binary16: no position can be derived from it
    if (!(s > 0.0f) || std::isinf(s)) return CATCHQ_ERR_ARG;
    // qmax / scale_data fills a half tensor with qmax first (32767 becomes 32768 there), then divides
    const float absmax = h16(h16(qmax) / s);
    if (!(absmax > 0.0f)) return CATCHQ_ERR_ARG;
    pos[c] = h16(std::floor(h16(std::log2(absmax))) - static_cast<float>(bitwidth - 2));
    chan_scale[c] = h16(h16(h16(std::exp2(pos[c])) * qmax) / absmax);
    pos_hi = (c == 0) ? pos[c] : std::fmax(pos_hi, pos[c]);
    pos_lo = (c == 0) ? pos[c] : std::fmin(pos_lo, pos[c]);
  }
  const float shared = std::nearbyint(h16(h16(pos_hi + pos_lo) / 2.0f));  // half-to-even
  for (int c = 0; c < co; ++c) {
    const float ns = h16(chan_scale[c] * h16(std::exp2(h16(shared - pos[c]))));
    const float sf = h16(h16(std::exp2(shared)) / ns);
    if (!(ns > 0.0f) || std::isinf(ns) || !(sf > 0.0f) || std::isinf(sf)) return CATCHQ_ERR_ARG;
    new_scale[c] = float_to_bits(ns);
    scale_factor[c] = float_to_bits(sf);
  }
  *new_position = static_cast<int>(shared);
  return CATCHQ_OK;
}

CATCHQ_API int catchq_conv_out_size(int in, int k, int pad, int stride, int dil) {
  const int kernel = dil * (k - 1) + 1;
  return (in + 2 * pad - kernel) / stride + 1;
}
