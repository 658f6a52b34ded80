// Shared device helpers of the catchq kernels (gfx950 only).
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <cstdlib>

#include "catchq.h"

#define CATCHQ_API extern "C" __attribute__((visibility("default")))

namespace catchq {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

inline hipStream_t as_stream(catchq_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status() { return hipGetLastError() == hipSuccess ? CATCHQ_OK : CATCHQ_ERR_LAUNCH; }

// compute units one launch should plan its tile shapes for: the device's 256, divided by the number of
// launches the caller says share the device (catchq_epilogue_t::sharing)
inline int planned_cus(int sharing) {
  const int cus = 256 / (sharing < 1 ? 1 : sharing);
  return cus < 1 ? 1 : cus;
}

// Allow `kern` more than the default 64 KiB of dynamic LDS: needed once per kernel and device.  `raised` is the
// call site's own flag array (one per kernel instance); setting the attribute twice is harmless, so relaxed
// atomics are all the synchronisation that concurrent first calls need.
inline int raise_lds_limit(const void *kern, int bytes, std::atomic<bool> (&raised)[64]) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return CATCHQ_ERR_LAUNCH;
  if (!raised[dev].load(std::memory_order_relaxed)) {
    if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
      (void)hipGetLastError();
      return CATCHQ_ERR_LAUNCH;
    }
    raised[dev].store(true, std::memory_order_relaxed);
  }
  return CATCHQ_OK;
}

// Tuning switches read from the environment exist only in builds made with -DCATCHQ_TUNING (A/B timing of tile
// shapes and load paths); the shipped kernel library reads no environment variable.  (The PyTorch extension on top
// of it has one run-time switch, CATCHQ_WEIGHT_CACHE=0, which turns its prepared-weight cache off.)
inline const char *tuning_env(const char *name) {
#ifdef CATCHQ_TUNING
  return std::getenv(name);
#else
  (void)name;
  return nullptr;
#endif
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- the quantize rule: q = sat(rne(x * scale * 2^-pos)), NaN -> 0 -------------------------
template <int BW>
struct QRange;
template <>
struct QRange<8> {
  typedef int8_t type;
  static constexpr float lo = -128.0f, hi = 127.0f;
};
template <>
struct QRange<16> {
  typedef int16_t type;
  static constexpr float lo = -32768.0f, hi = 32767.0f;
};
template <>
struct QRange<31> {
  typedef int32_t type;
  static constexpr float lo = -1073741824.0f, hi = 1073741823.0f;
};

// v_cvt_i32_f32 saturates out-of-range values and converts NaN to 0: with an integer clamp after
// it that is exactly "NaN -> 0, otherwise saturate".
__device__ __forceinline__ int cvt_i32_sat(float r) {
  int i;
  asm("v_cvt_i32_f32 %0, %1" : "=v"(i) : "v"(r));
  return i;
}

// x*scale is one fp32 rounding (exact for scale == 1), the scaling by 2^-pos is exact.
template <int BW>
__device__ __forceinline__ int quant1(float x, float scale, int neg_pos) {
  const float t = __builtin_ldexpf(x * scale, neg_pos);
  const int i = cvt_i32_sat(__builtin_rintf(t));
  constexpr int lo = (int)QRange<BW>::lo, hi = (int)QRange<BW>::hi;
  return min(max(i, lo), hi);
}

// same with scale == 1 known (x * 1.0f == x bit for bit, so the multiply is dropped)
template <int BW>
__device__ __forceinline__ int quant1_unit(float x, int neg_pos) {
  const int i = cvt_i32_sat(__builtin_rintf(__builtin_ldexpf(x, neg_pos)));
  constexpr int lo = (int)QRange<BW>::lo, hi = (int)QRange<BW>::hi;
  return min(max(i, lo), hi);
}

// v / d through the precomputed correctly rounded reciprocal r (see include/catchq.h)
__device__ __forceinline__ float div_by_rcp(float v, float d, float r) {
  const float q = v * r;
  const float err = __builtin_fmaf(-q, d, v);
  return __builtin_fmaf(err, r, q);
}

struct ConvDev {
  int N, H, W, Ci, Co, kh, kw, ph, pw, sh, sw, dh, dw, groups, Ho, Wo;
};

// ---- epilogue applied to one integer sum -----------------------------------------------------
struct EpiDev {
  int exp2;
  const float *chan_div;
  const float *chan_rcp;  // only set when the fused reciprocal form may be used
  const float *bias;
  const float *resid;
  int act;
  void *y;
  int y_f16;
  int32_t *acc_out;
  void *q;
  int q_bw;
  int q_neg_pos;
  float q_scale;
  float act_slope;
  int resid_after;
  const int *exp2_a, *exp2_b;  // device-resident positions added to exp2 (resolve_exp2)
  // the floating output / the residual is too large to stay cached until it is next used: written / read with
  // the non-temporal hint so that it does not push the operands and the int8 output out of the caches
  int y_stream, resid_stream;
  int cus;  // compute units the launch plans its tiles for (planned_cus of the caller's hint)
  int half_steps;  // fp16 output: round to binary16 after the scaling, the division and the bias (generic epilogues only)
};

// The second operand pair of a two-branch launch: the projection shortcut of a residual block.  Its
// integer sums are dequantized (divisor or reciprocal form, bias) exactly like a launch of their own
// with fp32 output would do, and the values serve as the residual of the main branch.
struct ShortcutDev {
  int exp2;
  const float *chan_div, *chan_rcp, *bias;
};

// An inner stage of a fused block: an int8 convolution whose ReLU / ReLU6 output is requantized to int8 at once
//   q = sat(rne(act(float(acc) * 2^exp2 / div[c] + bias[c]) * 2^q_neg_pos)),  rcp = correctly rounded reciprocals of div
struct IrbStageDev {
  const int8_t *w;
  const float *div, *rcp, *bias;
  int exp2, q_neg_pos, relu6;
};

// From which size on a floating output is written, and a residual read, with the non-temporal hint, for a launch that
// plans for `cus` of the 256 compute units.  Such a tensor is next used three launches later; kept in the caches it
// pushes out the int8 operands and the filters of the launches in between.  Measured end to end (same box,
// alternating): a residual read gains from the hint from 16 MiB on with the device to itself and from 8 MiB on as
// one of two parts (ResNet-50 two parts +0.9-1.5 %, MobileNetV2 +0.3 %); an output of 25 MB written by one of two
// parts gains as well (ResNet-50 +0.3-0.9 %, MobileNetV2 +1 %), while one of 51 MB written with the device to itself
// loses (MobileNetV2 on one stream -1.6 %): the output's limit falls with the square of the share -- a part has its
// share of the cache, and the other parts' traffic runs through that share too.
inline int64_t stream_limit_y(int cus) { return (64ll << 20) * cus / 256 * cus / 256; }
inline int64_t stream_limit_resid(int cus) { return (16ll << 20) * cus / 256; }

// out_elems: elements of the output tensor (0: unknown, nothing is streamed)
inline EpiDev make_epi(const catchq_epilogue_t *e, int64_t out_elems = 0) {
  EpiDev d;
  d.cus = planned_cus(e->sharing);
  const int64_t y_limit = stream_limit_y(d.cus), r_limit = stream_limit_resid(d.cus);
  d.y_stream = (e->y && out_elems * (e->y_dtype == CATCHQ_F16 ? 2 : 4) >= y_limit) ? 1 : 0;
  d.resid_stream = (e->resid && out_elems * 4 >= r_limit) ? 1 : 0;
  d.exp2 = e->exp2;
  d.chan_div = e->chan_div;
  const bool dev_exp = e->exp2_dev[0] || e->exp2_dev[1];
  d.half_steps = (e->half_steps && e->y && e->y_dtype == CATCHQ_F16) ? 1 : 0;
  // (the reciprocal form folds the power of two into the division: not with a rounding between the two)
  d.chan_rcp = (e->chan_div && e->chan_rcp && !dev_exp && !d.half_steps && e->exp2 >= -64 && e->exp2 <= 64) ? e->chan_rcp : nullptr;
  d.bias = e->bias;
  d.resid = e->resid;
  d.act = e->act;
  d.y = e->y;
  d.y_f16 = (e->y_dtype == CATCHQ_F16);
  d.acc_out = e->acc_out;
  d.q = e->q;
  d.q_bw = e->q_bitwidth;
  d.q_neg_pos = -e->q_position;
  d.q_scale = e->q_scale;
  d.act_slope = e->act_slope;
  d.resid_after = (e->resid && e->resid_after_act) ? 1 : 0;
  d.exp2_a = e->exp2_dev[0];
  d.exp2_b = e->exp2_dev[1];
  return d;
}

inline int check_epi(const catchq_epilogue_t *e) {
  if (!e) return CATCHQ_ERR_ARG;
  if (!e->y && !e->acc_out && !e->q) return CATCHQ_ERR_ARG;
  if (e->y && e->y_dtype != CATCHQ_F32 && e->y_dtype != CATCHQ_F16) return CATCHQ_ERR_DTYPE;
  if (e->q && e->q_bitwidth != 8 && e->q_bitwidth != 16) return CATCHQ_ERR_BITWIDTH;
  if (e->act < CATCHQ_ACT_NONE || e->act > CATCHQ_ACT_LEAKY) return CATCHQ_ERR_ARG;
  if (e->exp2 < -126 || e->exp2 > 126) return CATCHQ_ERR_ARG;
  if (e->q && (e->q_position < -126 || e->q_position > 126)) return CATCHQ_ERR_ARG;
  if (e->sharing < 0) return CATCHQ_ERR_ARG;
  return CATCHQ_OK;
}

// first statement of every kernel that takes an EpiDev: fold the device-resident positions into exp2
// (uniform scalar loads; the sum is clamped to what ldexpf handles without surprises)
__device__ __forceinline__ void resolve_exp2(EpiDev &e) {
  if (e.exp2_a || e.exp2_b) {
    int v = e.exp2;
    if (e.exp2_a) v += *e.exp2_a;
    if (e.exp2_b) v += *e.exp2_b;
    e.exp2 = v < -252 ? -252 : (v > 252 ? 252 : v);
  }
}

// value after dequant / bias / residual / activation; facc = float(acc) (one RNE conversion)
__device__ __forceinline__ float round_f16(float v) { return __half2float(__float2half_rn(v)); }

__device__ __forceinline__ float epi_value(float facc, int64_t idx, int c, const EpiDev &e) {
  float v = __builtin_ldexpf(facc, e.exp2);
  if (e.half_steps) v = round_f16(v);
  if (e.chan_div) {
    v = v / e.chan_div[c];
    if (e.half_steps) v = round_f16(v);
  }
  if (e.bias) {
    v = v + e.bias[c];
    if (e.half_steps) v = round_f16(v);
  }
  if (e.resid && !e.resid_after) v = v + e.resid[idx];
  if (e.act == CATCHQ_ACT_LEAKY) v = (v > 0.0f) ? v : v * e.act_slope;
  else if (e.act >= CATCHQ_ACT_RELU) v = (v > 0.0f) ? v : 0.0f;
  if (e.act == CATCHQ_ACT_RELU6) v = (v < 6.0f) ? v : 6.0f;
  if (e.resid && e.resid_after) v = v + e.resid[idx];
  return v;
}

__device__ __forceinline__ void epi_store(float v, int64_t idx, const EpiDev &e) {
  if (e.y) {
    if (e.y_f16) reinterpret_cast<__half *>(e.y)[idx] = __float2half_rn(v);
    else reinterpret_cast<float *>(e.y)[idx] = v;
  }
  if (e.q) {
    if (e.q_bw == 8) reinterpret_cast<int8_t *>(e.q)[idx] = (int8_t)quant1<8>(v, e.q_scale, e.q_neg_pos);
    else reinterpret_cast<int16_t *>(e.q)[idx] = (int16_t)quant1<16>(v, e.q_scale, e.q_neg_pos);
  }
}

}  // namespace catchq
