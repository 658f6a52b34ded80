/*
 * catchq_oracle.c -- CPU restatement of the fixed-point quantized-inference
 * arithmetic of Cambricon/catch (torch_mlu).  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the HIP kernels are compared with.  Nothing in
 * the shipped library links, imports or calls it: only the test-suite, the
 * smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Every function names the reference lines it restates (paths relative to the
 * reference tree).  The reference delegates the device arithmetic to the closed
 * vendor library CNNL 1.8.2 (script/release/build.property:5); where the tree
 * does not state a formula the choice made here is marked "unpinned".
 *
 * How each function is pinned (tests/test_oracle_pins.py):
 *   orc_pos_from_scale        closed form in source; exact powers of two; brute force
 *   orc_quant_params          scale_frac in (qmax/2^(n-1), qmax/2^(n-2)]; scale_factor*scale == 1
 *   orc_calib_scale           closed form in source (observer.py:113-140)
 *   orc_per_channel_params    fixture torch_mlu/csrc/test/data/test.txt (position +
 *                             per-channel scales are fixed points of the derivation)
 *   orc_quantize_*            scale=1,pos=0 == torch.round().clamp(); exhaustive fp16;
 *                             half-way ties; saturation
 *   orc_quantize_per_channel  torch.round(w/sf).clamp() (the reference's own op chain)
 *   orc_gemm_nt / orc_conv2d  torch int64 matmul / F.conv2d on int64 (textbook)
 *   orc_epilogue_*            numpy float32 evaluation of the same expression order
 *   orc_f32_to_f16 / f16_to_f32  numpy float16 (exhaustive one way, ties the other)
 *   orc_quantize_param        cnnlQuantizeParam's own formula is not in the tree
 *                             (internal/quantize_param.cpp:85-94 only calls it); defined as the
 *                             position rule of cnnl_util.cpp:337-347 and the scale of
 *                             jit/utils/utils.cpp:97-100; pinned by frexp (position), the exact
 *                             rational 2^pos*qmax/absmax rounded once (scale), agreement with
 *                             orc_quant_params, absmax -> +-qmax, zero / inf / NaN / denormals
 *   orc_maxpool_nhwc_f32      torch.nn.functional.max_pool2d over (k, stride, pad) grids
 *   orc_global_avgpool_nhwc_f32  numpy's sequential fp32 cumsum; float64 mean bound; an input on
 *                             which sequential, pairwise and reversed sums differ
 *   NaN -> 0 in quantize      PARITY UNPINNED (vendor behaviour not stated anywhere)
 *   float order of dequant+bias inside the vendor conv/matmul: PARITY UNPINNED;
 *                             fixed here as cvt(acc) * 2^e [/ new_scale_c] [+ bias] in fp32.
 *   position + fractional scale per tensor / per axis (oracle/ops.py decode_fractional, the
 *                             composition of orc_quant_params and orc_quantize_* with scale != 1):
 *                             parameters pinned (the step is absmax/qmax: extreme element -> +-qmax,
 *                             error <= half a step); what the reference's graph backend computes
 *                             from them is in a closed library: PARITY UNPINNED.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ helpers */

static inline void orc_qrange(int bw, float *qmin, float *qmax) {
  if (bw == 16) { *qmin = -32768.0f; *qmax = 32767.0f; }
  else if (bw == 31) { *qmin = -1073741824.0f; *qmax = 1073741823.0f; }
  else { *qmin = -128.0f; *qmax = 127.0f; }
}

ORC_API int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

ORC_API void orc_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* IEEE binary16 <-> binary32, round-to-nearest-even, written out so that the
 * oracle does not depend on compiler support for a half type. */
ORC_API float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; e++; } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

ORC_API uint16_t orc_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0u));
  }
  if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x33000001u) { /* < 2^-25 (or exactly 2^-25, a tie to even zero) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u;
  uint32_t shift, half_bits;
  if (e < -14) { /* subnormal half */
    shift = (uint32_t)(13 + (-14 - e));
    uint32_t r = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (r & 1u))) r++;
    return (uint16_t)(sign | r);
  }
  shift = 13;
  half_bits = ((uint32_t)(e + 15) << 10) | ((m >> shift) & 0x3ffu);
  {
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half_bits & 1u))) half_bits++;
  }
  return (uint16_t)(sign | half_bits);
}

/* ------------------------------------------------------------ q-param math */

/* scale -> position.  torch_mlu/csrc/aten/cnnl/cnnl_util.cpp:337-347:
 *   float absmax = qmax / scale_data;
 *   pos_ = std::floor(std::log(absmax) / std::log(2)) - (bitwidth - 2);
 * std::log(float) is the float overload, std::log(2) the double one, so the
 * quotient is formed in double and truncated to int after the subtraction. */
ORC_API int orc_pos_from_scale(int bw, float scale) {
  int qmax = (bw == 16) ? 32767 : 127;
  float absmax = (float)qmax / scale;
  double q = (double)logf(absmax) / log(2.0);
  return (int)(floor(q) - (double)(bw - 2));
}

/* position + fractional scale + scale_factor.
 * torch_mlu/csrc/jit/utils/utils.cpp:81-105 (setQuantizedParams):
 *   float absmax = qmax / scale;
 *   pos_   = floor(log(absmax)/log(2)) - (n-2)            (kept in a float)
 *   scale_ = pow(2,pos_) * (pow(2,n-1) - 1) / absmax      (double expr -> float)
 *   scale_factor_ = pow(2,pos_) / scale_                  (double expr -> float) */
ORC_API void orc_quant_params(int bw, float scale, int *pos, float *scale_frac,
                              float *scale_factor) {
  int n = (bw == 16) ? 16 : 8;
  int qmax = (bw == 16) ? 32767 : 127;
  float absmax = (float)qmax / scale;
  float pos_ = (float)(floor((double)logf(absmax) / log(2.0)) - (double)(n - 2));
  float scale_ = (float)(pow(2.0, (double)pos_) * (pow(2.0, (double)(n - 1)) - 1.0) / (double)absmax);
  float sf = (float)(pow(2.0, (double)pos_) / (double)scale_);
  *pos = (int)pos_;
  *scale_frac = scale_;
  *scale_factor = sf;
}

/* calibration scale from running min/max.
 * torch_mlu/core/quantized/observer.py:113-140 (_calculate_qparams): python
 * floats are doubles; scale = qmax/absmax, 1.0 when absmax==0 or NaN input. */
ORC_API double orc_calib_scale(int bw, double min_val, double max_val) {
  double qmax = (bw == 16) ? 32767.0 : 127.0;
  if (isnan(min_val) || isnan(max_val)) return 1.0;
  double absmax = (max_val > -min_val) ? max_val : -min_val;
  if (absmax != 0.0) return qmax / absmax;
  return 1.0;
}

/* per-channel parameter derivation, all in fp32 like the tensor ops it restates.
 * torch_mlu/csrc/aten/operators/cnnl/quantify.cpp:55-96:
 *   absmax_c = qmax / s_c                         (:64)
 *   pos_c    = floor(log2(absmax_c)) - (n-2)      (:71-84)
 *   scale_c  = 2^pos_c * (2^(n-1)-1) / absmax_c   (:87-88)
 *   new_pos  = round((max pos + min pos) / 2)     (:91-92, half-to-even: test_round.py:21-28)
 *   new_scale_c = scale_c * 2^(new_pos - pos_c)   (:95)
 *   sf_c     = 2^new_pos / new_scale_c            (:98) */
ORC_API void orc_per_channel_params(int bw, const float *s, int co, int *new_pos,
                                    float *new_scale, float *sf) {
  int n = (bw == 16) ? 16 : 8;
  float qmax = (bw == 16) ? 32767.0f : 127.0f;
  float *pos = (float *)malloc(sizeof(float) * (size_t)(co > 0 ? co : 1));
  float *sc = (float *)malloc(sizeof(float) * (size_t)(co > 0 ? co : 1));
  float pmax = -INFINITY, pmin = INFINITY;
  for (int c = 0; c < co; ++c) {
    float absmax = qmax / s[c];
    float p = floorf(log2f(absmax)) - (float)(n - 2);
    /* (scale_pc * qmax) / absmax_pc: left-to-right like the tensor expression */
    float t = exp2f(p) * (float)(pow(2.0, (double)(n - 1)) - 1.0);
    sc[c] = t / absmax;
    pos[c] = p;
    if (p > pmax) pmax = p;
    if (p < pmin) pmin = p;
  }
  float np = rintf((pmax + pmin) / 2.0f); /* default rounding mode = half-to-even */
  for (int c = 0; c < co; ++c) {
    float ns = sc[c] * exp2f(np - pos[c]);
    new_scale[c] = ns;
    sf[c] = exp2f(np) / ns;
  }
  *new_pos = (int)np;
  free(pos);
  free(sc);
}

/* position (+scale) from a tensor's max-abs: the role of cnnlQuantizeParam
 * (torch_mlu/csrc/aten/operators/cnnl/internal/quantize_param.cpp:39-96).
 * The vendor's own formula is not in the tree; defined here by the two formulas the tree does
 * state for the same quantities (cnnl_util.cpp:337-347; jit/utils/utils.cpp:97-100), in their
 * exact-exponent form:
 *   pos = floor(log2(absmax)) - (n-2) with floor(log2) taken from the exponent,
 *   scale = 2^pos * qmax / absmax rounded once to fp32, offset = 0.
 *   absmax 0, inf or NaN -> pos 0, scale 1. */
ORC_API void orc_quantize_param(float absmax, int bw, int *pos, float *scale, float *offset) {
  float qmax = (bw == 16) ? 32767.0f : 127.0f;
  int n = (bw == 16) ? 16 : 8;
  if (!(absmax > 0.0f) || isinf(absmax)) {
    *pos = 0; *scale = 1.0f; *offset = 0.0f;
    return;
  }
  int p = ilogbf(absmax) - (n - 2);
  *pos = p;
  /* absmax * 2^-p lies in [2^(n-2), 2^(n-1)): the scaling is exact even for a denormal absmax, so the
   * quotient is rounded once (2^p * qmax would underflow first for the smallest inputs) */
  *scale = qmax / ldexpf(absmax, -p);
  *offset = 0.0f;
}

ORC_API float orc_absmax_f32(const float *x, int64_t n) {
  float m = 0.0f;
#pragma omp parallel for reduction(max : m)
  for (int64_t i = 0; i < n; ++i) {
    float a = fabsf(x[i]);
    if (a > m) m = a; /* NaN compares false: ignored */
  }
  return m;
}

ORC_API float orc_absmax_f16(const uint16_t *x, int64_t n) {
  float m = 0.0f;
#pragma omp parallel for reduction(max : m)
  for (int64_t i = 0; i < n; ++i) {
    float a = fabsf(orc_f16_to_f32(x[i]));
    if (a > m) m = a;
  }
  return m;
}

/* ---------------------------------------------------------------- quantize */

/* q = clamp(rne(x * scale * 2^-pos), qmin, qmax).
 * Call sites: cnnlQuantizeV1/V2 with CNNL_QUANTIZE_POSITION
 * (internal/quantify.cpp:87-94,118-132); formula
 * docs/user_guide/source/pytorch_10_tools/Pytorch_tools.rst:157-161
 * ("qx = clamp(round(x*scale))"); rounding is half-to-even, saturating.
 * Order fixed here: t = x*scale in fp32, exact scaling by 2^-pos, rint, clamp.
 * NaN -> 0 (unpinned). */
static inline int32_t orc_q1(float x, float scale, int pos, float qmin, float qmax) {
  float t = x * scale;
  t = ldexpf(t, -pos);
  if (t != t) return 0;
  float r = rintf(t);
  if (r < qmin) r = qmin;
  if (r > qmax) r = qmax;
  return (int32_t)r;
}

static void orc_store(void *q, int bw, int64_t i, int32_t v) {
  if (bw == 8) ((int8_t *)q)[i] = (int8_t)v;
  else if (bw == 16) ((int16_t *)q)[i] = (int16_t)v;
  else ((int32_t *)q)[i] = v;
}

ORC_API void orc_quantize_f32(const float *x, void *q, int bw, int64_t n, int pos, float scale) {
  float qmin, qmax;
  orc_qrange(bw, &qmin, &qmax);
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) orc_store(q, bw, i, orc_q1(x[i], scale, pos, qmin, qmax));
}

ORC_API void orc_quantize_f16(const uint16_t *x, void *q, int bw, int64_t n, int pos, float scale) {
  float qmin, qmax;
  orc_qrange(bw, &qmin, &qmax);
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i)
    orc_store(q, bw, i, orc_q1(orc_f16_to_f32(x[i]), scale, pos, qmin, qmax));
}

/* NCHW fp32 -> NHWC int (channel count padded with zeros to cpad >= C).  The
 * reference makes the activation channels-last first and then quantizes
 * (quantify_conv_forward.cpp:62-63,97); elementwise, so the order is free. */
ORC_API void orc_quantize_nchw_to_nhwc_f32(const float *x, void *q, int bw, int N, int C, int H,
                                           int W, int cpad, int pos, float scale) {
  float qmin, qmax;
  orc_qrange(bw, &qmin, &qmax);
  int64_t hw = (int64_t)H * W;
#pragma omp parallel for
  for (int64_t np = 0; np < (int64_t)N * hw; ++np) {
    int64_t n = np / hw, p = np % hw;
    for (int c = 0; c < cpad; ++c) {
      int32_t v = 0;
      if (c < C) v = orc_q1(x[(n * C + c) * hw + p], scale, pos, qmin, qmax);
      orc_store(q, bw, np * cpad + c, v);
    }
  }
}

/* per-channel weight quantizer: q[c,...] = clamp(rne(w[c,...] / sf_c)).
 * quantify.cpp:100-105 (true fp32 division, round, clamp, cast). */
ORC_API void orc_quantize_per_channel_f32(const float *w, void *q, int bw, int co, int64_t inner,
                                          const float *sf) {
  float qmin, qmax;
  orc_qrange(bw, &qmin, &qmax);
#pragma omp parallel for
  for (int c = 0; c < co; ++c) {
    for (int64_t i = 0; i < inner; ++i) {
      float t = w[(int64_t)c * inner + i] / sf[c];
      int32_t v = 0;
      if (t == t) {
        float r = rintf(t);
        if (r < qmin) r = qmin;
        if (r > qmax) r = qmax;
        v = (int32_t)r;
      }
      orc_store(q, bw, (int64_t)c * inner + i, v);
    }
  }
}

/* explicit dequantize: x = q * 2^pos / scale  ("y = qy/scale1/scale2",
 * Pytorch_tools.rst:161; the reference has no standalone op for it). */
ORC_API void orc_dequantize_f32(const void *q, int bits, float *y, int64_t n, int pos, float scale) {
#pragma omp parallel for
  for (int64_t i = 0; i < n; ++i) {
    int32_t v = bits == 8 ? ((const int8_t *)q)[i] : bits == 16 ? ((const int16_t *)q)[i]
                                                                : ((const int32_t *)q)[i];
    float t = ldexpf((float)v, pos);
    y[i] = (scale == 1.0f) ? t : t / scale;
  }
}

/* --------------------------------------------------------- int contraction */

static inline int32_t orc_ld(const void *p, int bits, int64_t i) {
  return bits == 8 ? (int32_t)((const int8_t *)p)[i] : (int32_t)((const int16_t *)p)[i];
}

/* C[m][n] = sum_k A[m][k] * B[n][k]   (cnnlMatMul, transA=false, transB=true:
 * internal/matmul_internal.cpp:102-117; weight is [out,in]: linear.cpp:52-55).
 * Accumulates and stores int64, and reports how many results do not fit an
 * int32 accumulator (none may, where the device path accumulates in int32:
 * int8 x int8 and int16 x int8; int16 x int16 is defined on the exact sum). */
ORC_API int64_t orc_gemm_nt(const void *a, int a_bits, const void *b, int b_bits, int64_t M,
                            int64_t N, int64_t K, int64_t *acc) {
  int64_t overflow = 0;
  if (a_bits == 8 && b_bits == 8) {
    const int8_t *A = (const int8_t *)a, *B = (const int8_t *)b;
#pragma omp parallel for reduction(+ : overflow)
    for (int64_t m = 0; m < M; ++m) {
      for (int64_t n = 0; n < N; ++n) {
        const int8_t *ar = A + m * K, *br = B + n * K;
        int64_t s = 0;
        int32_t s32 = 0;
        /* |a*b| <= 2^14, so 2^16 terms cannot overflow int32: sum in blocks */
        for (int64_t k0 = 0; k0 < K; k0 += 65536) {
          int64_t k1 = k0 + 65536 < K ? k0 + 65536 : K;
          s32 = 0;
          for (int64_t k = k0; k < k1; ++k) s32 += (int32_t)ar[k] * (int32_t)br[k];
          s += s32;
        }
        if (s > INT32_MAX || s < INT32_MIN) overflow++;
        acc[m * N + n] = s;
      }
    }
    return overflow;
  }
#pragma omp parallel for reduction(+ : overflow)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      int64_t s = 0;
      for (int64_t k = 0; k < K; ++k)
        s += (int64_t)orc_ld(a, a_bits, m * K + k) * (int64_t)orc_ld(b, b_bits, n * K + k);
      if (s > INT32_MAX || s < INT32_MIN) overflow++;
      acc[m * N + n] = s;
    }
  }
  return overflow;
}

/* output extent, internal/convolution_forward_internal.cpp:40-54 */
ORC_API int orc_conv_out_size(int in, int k, int pad, int stride, int dil) {
  int kernel = dil * (k - 1) + 1;
  return (in + 2 * pad - kernel) / stride + 1;
}

/* Direct integer convolution (cross-correlation, zero padding, groups).
 * cnnlConvolutionForward on int8/int16 tensors in NHWC layout
 * (internal/convolution_forward_internal.cpp:85-88,158-173).
 *   x  [N,H,W,Ci]           w  [Co,kh,kw,Ci/g]          acc [N,Ho,Wo,Co]
 * int64 accumulation and storage, with a count of sums outside int32. */
ORC_API int64_t orc_conv2d_nhwc(const void *x, int x_bits, const void *w, int w_bits, int N, int H,
                                int W, int Ci, int Co, int kh, int kw, int pad_h, int pad_w,
                                int stride_h, int stride_w, int dil_h, int dil_w, int groups,
                                int64_t *acc) {
  int Ho = orc_conv_out_size(H, kh, pad_h, stride_h, dil_h);
  int Wo = orc_conv_out_size(W, kw, pad_w, stride_w, dil_w);
  int cig = Ci / groups, cog = Co / groups;
  int64_t overflow = 0;
  int fast = (x_bits == 8 && w_bits == 8 && (int64_t)kh * kw * cig <= 65536);
#pragma omp parallel for collapse(2) reduction(+ : overflow)
  for (int n = 0; n < N; ++n) {
    for (int ho = 0; ho < Ho; ++ho) {
      for (int wo = 0; wo < Wo; ++wo) {
        for (int co = 0; co < Co; ++co) {
          int g = co / cog;
          int64_t s = 0;
          for (int r = 0; r < kh; ++r) {
            int hi = ho * stride_h - pad_h + r * dil_h;
            if (hi < 0 || hi >= H) continue;
            for (int q = 0; q < kw; ++q) {
              int wi = wo * stride_w - pad_w + q * dil_w;
              if (wi < 0 || wi >= W) continue;
              int64_t xo = (((int64_t)n * H + hi) * W + wi) * Ci + (int64_t)g * cig;
              int64_t wo_ = (((int64_t)co * kh + r) * kw + q) * cig;
              if (fast) {
                const int8_t *xp = (const int8_t *)x + xo, *wp = (const int8_t *)w + wo_;
                int32_t t = 0;
                for (int c = 0; c < cig; ++c) t += (int32_t)xp[c] * (int32_t)wp[c];
                s += t;
              } else {
                for (int c = 0; c < cig; ++c)
                  s += (int64_t)orc_ld(x, x_bits, xo + c) * (int64_t)orc_ld(w, w_bits, wo_ + c);
              }
            }
          }
          if (s > INT32_MAX || s < INT32_MIN) overflow++;
          acc[(((int64_t)n * Ho + ho) * Wo + wo) * Co + co] = s;
        }
      }
    }
  }
  return overflow;
}

/* ----------------------------------------------------------------- epilogue */

/* y[r][c] = act( cvt_f32(acc[r][c]) * 2^exp2   (one RNE conversion of the integer sum)
 * [ / chan_div[c] ] [ + bias[c] ] )
 * per-tensor: positions live in the vendor conv/matmul descriptors
 *   (convolution_forward_internal.cpp:85-88; matmul_internal.cpp:93-96), bias added inside;
 * per-channel: output / new_scale then + bias as separate fp ops
 *   (quantify_conv_forward.cpp:123-129; linear.cpp:54-59).
 * act: 0 none, 1 ReLU (x>0?x:0), 2 ReLU6.  All arithmetic fp32, no fused
 * multiply-add; fp16 output = one final RNE conversion. */
static inline float orc_epi1(int64_t a, int e, const float *chan_div, const float *bias,
                             const float *resid, int64_t idx, int64_t c, int act) {
  float v = ldexpf((float)a, e);
  if (chan_div) v = v / chan_div[c];
  if (bias) v = v + bias[c];
  if (resid) v = v + resid[idx];
  if (act >= 1) v = (v > 0.0f) ? v : 0.0f;
  if (act == 2) v = (v < 6.0f) ? v : 6.0f;
  return v;
}

ORC_API void orc_epilogue_f32(const int64_t *acc, int64_t rows, int64_t co, int exp2,
                              const float *chan_div, const float *bias, const float *resid,
                              int act, float *y) {
#pragma omp parallel for
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < co; ++c)
      y[r * co + c] = orc_epi1(acc[r * co + c], exp2, chan_div, bias, resid, r * co + c, c, act);
}

ORC_API void orc_epilogue_f16(const int64_t *acc, int64_t rows, int64_t co, int exp2,
                              const float *chan_div, const float *bias, const float *resid,
                              int act, uint16_t *y) {
#pragma omp parallel for
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t c = 0; c < co; ++c)
      y[r * co + c] =
          orc_f32_to_f16(orc_epi1(acc[r * co + c], exp2, chan_div, bias, resid, r * co + c, c, act));
}

/* Global average pooling of an NHWC fp32 tensor: sequential fp32 sum over the pixels in storage
 * order, one division.  The order is this build's definition (floating-point sums depend on it). */
ORC_API void orc_global_avgpool_nhwc_f32(const float *x, int N, int HW, int C, float *y) {
#pragma omp parallel for
  for (int64_t i = 0; i < (int64_t)N * C; ++i) {
    int64_t n = i / C, c = i % C;
    float s = 0.0f;
    for (int p = 0; p < HW; ++p) s = s + x[(n * HW + p) * C + c];
    y[i] = s / (float)HW;
  }
}

/* 2-D max pooling over an NHWC fp32 tensor (-inf padding), used by the model
 * level checks; not part of the quantized arithmetic itself. */
ORC_API void orc_maxpool_nhwc_f32(const float *x, int N, int H, int W, int C, int k, int stride,
                                  int pad, float *y) {
  int Ho = (H + 2 * pad - k) / stride + 1, Wo = (W + 2 * pad - k) / stride + 1;
#pragma omp parallel for collapse(2)
  for (int n = 0; n < N; ++n)
    for (int ho = 0; ho < Ho; ++ho)
      for (int wo = 0; wo < Wo; ++wo)
        for (int c = 0; c < C; ++c) {
          float m = -INFINITY;
          for (int r = 0; r < k; ++r) {
            int hi = ho * stride - pad + r;
            if (hi < 0 || hi >= H) continue;
            for (int q = 0; q < k; ++q) {
              int wi = wo * stride - pad + q;
              if (wi < 0 || wi >= W) continue;
              float v = x[(((int64_t)n * H + hi) * W + wi) * C + c];
              if (v > m) m = v;
            }
          }
          y[(((int64_t)n * Ho + ho) * Wo + wo) * C + c] = m;
        }
}
