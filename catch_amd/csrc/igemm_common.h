// Pieces shared by the int8 implicit-GEMM kernels: parameters, the LDS swizzle, and the epilogue.
#pragma once
#include <type_traits>

#include "catchq_common.h"

namespace catchq {

struct IgemmParams {
  int64_t M;
  int N, K;
  int H, W, Ci, Ho, Wo, kh, kw, ph, pw, sh, sw, dh, dw;
  int kwq;  // LOAD_C4: chunks (groups of 4 taps) per filter row
  // LDS-DMA im2col loader: element strides of the activation tensor (image, image row, output-column
  // step unit).  A plain NHWC tensor has H*W*Ci, W*Ci, Ci; the pixel-window form of a few-channel
  // input (a filter row = one contiguous run of kw*C elements) uses other values.
  unsigned img_stride, row_stride, pix_stride;
  int tiles_n;
  int nblocks;
  // Order in which consecutive block ids walk the tile grid: 0 = row by row (all column tiles of one row tile,
  // then the next row tile); g > 0 = in bands of g row tiles, column by column inside a band, so that the blocks
  // running at the same time cover a g x (concurrent / g) patch of tiles and share both operands' panels in L2
  // instead of streaming the whole B operand past every row tile.
  int group_m;
  int tiles_m;
  // Leading dimension of the output matrices (y, q, acc_out, resid); 0 = N.  A grouped convolution runs one GEMM per
  // group (grid dimension y) whose N is the group's share of the output channels while the rows stay Co apart.
  int ldc;
  // groups > 1: per-group offsets -- bytes into the activation tensor (a pixel's channel slice), bytes into the
  // weights (the group's filters) and output channels (columns of the outputs and entries of the per-channel vectors)
  int groups, a_group_bytes, n_group;
  int64_t b_group_bytes;
};

__device__ __forceinline__ int out_ld(const IgemmParams &p) { return p.ldc ? p.ldc : p.N; }

constexpr int BK = 64;  // bytes of K per pipeline step (one LDS row)
enum { LOAD_GEMM = 0, LOAD_CONV = 1, LOAD_C4 = 2 };

// LDS rows are 64 bytes = four 16-byte chunks; the chunk index is XOR-ed with (row>>2)&3 so that
// 16 consecutive rows at one logical chunk fall into 16 different 16-byte bank groups
// (measured: 176 B/clk/CU with the swizzle, 62 B/clk/CU without).
__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 2) & 3); }

// block id -> tile index, XCD-aware: ids that land on one XCD (id % 8) take a contiguous run of
// tiles, so neighbouring tiles (same A rows, same weights) share that XCD's L2.
__device__ __forceinline__ int xcd_remap(int bid, int nb) {
  const int xcd = bid & 7, local = bid >> 3;
  const int q = nb >> 3, rem = nb & 7;
  return xcd * q + (xcd < rem ? xcd : rem) + local;
}

inline bool vec_epilogue_ok(int N, const EpiDev &e) {
  // (N < 2^24: the per-lane part of an element index, at most 32 rows, fits 32 bits with room to spare)
  return N % 4 == 0 && N < (1 << 24) && aligned16(e.chan_div) && aligned16(e.chan_rcp) && aligned16(e.bias) && aligned16(e.resid) && aligned16(e.y) &&
         aligned16(e.acc_out) && aligned16(e.q);
}

// What an epilogue instance knows at compile time.  A field of -1 is decided at run time from the
// EpiDev (the generic instance); fixed fields let the compiler drop every untaken branch, which
// matters because the epilogue is VALU-bound (about a dozen fp32 operations per output element).
//   DIV  0 none, 1 reciprocal form, 2 true division      BIAS 0/1     RESID 0 none, 1 before, 2 after the activation
//   ACT  CATCHQ_ACT_*       YM  0 none, 1 fp32, 2 fp16     QM  0 none, 8, 16     ACC 0/1
template <int DIV, int BIAS, int RESID, int ACT, int YM, int QM, int ACC>
struct EpiSpec {
  static constexpr bool kGeneric = DIV < 0;
  static constexpr int kAct = ACT;
  static constexpr int kQ = QM;
  // ReLU / ReLU6 feeding nothing but an int8 requantization: the activation folds into the clamp of the
  // quantizer, 0 <= x <= min(6, 127 * 2^pos)
  static constexpr bool kFoldAct = DIV >= 0 && QM == 8 && YM == 0 && ACC == 0 && RESID != 2 &&
                                   (ACT == CATCHQ_ACT_RELU || ACT == CATCHQ_ACT_RELU6);
  // ... and with the reciprocal form and no residual the requantization's power of two folds into the per-channel
  // constants as well (scaling by 2^k is exact, so every intermediate is the scaled image of the unfolded one): the
  // value arrives in units of the output's step, and one instruction (v_cvt_pk_u8_f32: round to nearest even,
  // saturate to 0 .. 255, insert the byte) rounds and packs it
  static constexpr bool kFoldScale = kFoldAct && DIV == 1 && RESID == 0;
  static __device__ __forceinline__ bool rcp(const EpiDev &e) { return DIV < 0 ? e.chan_rcp != nullptr : DIV == 1; }
  static __device__ __forceinline__ bool truediv(const EpiDev &e) {
    return DIV < 0 ? (e.chan_div != nullptr && e.chan_rcp == nullptr) : DIV == 2;
  }
  static __device__ __forceinline__ bool bias(const EpiDev &e) { return BIAS < 0 ? e.bias != nullptr : BIAS == 1; }
  static __device__ __forceinline__ bool resid(const EpiDev &e) { return RESID < 0 ? e.resid != nullptr : RESID >= 1; }
  static __device__ __forceinline__ bool resid_after(const EpiDev &e) { return RESID < 0 ? e.resid_after != 0 : RESID == 2; }
  static __device__ __forceinline__ int act(const EpiDev &e) { return ACT < 0 ? e.act : ACT; }
  static __device__ __forceinline__ bool y32(const EpiDev &e) { return YM < 0 ? (e.y && !e.y_f16) : YM == 1; }
  static __device__ __forceinline__ bool y16(const EpiDev &e) { return YM < 0 ? (e.y && e.y_f16) : YM == 2; }
  static __device__ __forceinline__ bool q8(const EpiDev &e) { return QM < 0 ? (e.q && e.q_bw == 8) : QM == 8; }
  static __device__ __forceinline__ bool q16(const EpiDev &e) { return QM < 0 ? (e.q && e.q_bw == 16) : QM == 16; }
  static __device__ __forceinline__ bool acc(const EpiDev &e) { return ACC < 0 ? e.acc_out != nullptr : ACC == 1; }
};
typedef EpiSpec<-1, -1, -1, -1, -1, -1, -1> EpiGeneric;

// epilogue variants a kernel can be instantiated with
enum {
  EPI_SCALAR = 0,   // any N / alignment: one element at a time, straight from the accumulators
  EPI_VECTOR = 1,   // generic, vectorised through LDS (N % 4 == 0, 16-byte aligned pointers)
  EPI_Q8_RELU = 2,  // reciprocal-form dequant + bias + ReLU -> int8                 (conv feeding a conv)
  EPI_RES_Y_Q8 = 3, // ... + residual + ReLU -> fp32 and int8                         (end of a residual block)
  EPI_Y32 = 4,      // reciprocal-form dequant + bias -> fp32                         (projection shortcut)
  EPI_RES_Y = 5,    // ... + residual + ReLU -> fp32                                   (last block)
  EPI_Y16_RELU = 6, // reciprocal-form dequant + bias + ReLU -> fp16                  (standalone linear)
  EPI_Q8_RELU6 = 7, // reciprocal-form dequant + bias + ReLU6 -> int8
  EPI_RES_Q8 = 8,   // ... + residual + ReLU -> int8 only                             (last block of a stage)
  // linear bottlenecks (no activation), reciprocal-form dequant + bias:
  EPI_LIN_Q8 = 9,          // -> int8
  EPI_LIN_Y_Q8 = 10,       // -> fp32 and int8
  EPI_LIN_RES_Q8 = 11,     // + residual -> int8
  EPI_LIN_RES_Y_Q8 = 12,   // + residual -> fp32 and int8
  // per-tensor weights (no divisor), bias, leaky ReLU, int16 requantization:
  EPI_LK_Q16 = 13,         // -> int16
  EPI_LK_Y_Q16 = 14,       // -> fp32 and int16
  EPI_LK_RESA_Q16 = 15,    // residual added after the activation -> int16
  EPI_LK_RESA_Y_Q16 = 16,  // residual added after the activation -> fp32 and int16
  EPI_COUNT = 17
};
template <int EPI> struct EpiOf { typedef EpiGeneric type; };
template <> struct EpiOf<EPI_Q8_RELU> { typedef EpiSpec<1, 1, 0, CATCHQ_ACT_RELU, 0, 8, 0> type; };
template <> struct EpiOf<EPI_RES_Y_Q8> { typedef EpiSpec<1, 1, 1, CATCHQ_ACT_RELU, 1, 8, 0> type; };
template <> struct EpiOf<EPI_Y32> { typedef EpiSpec<1, 1, 0, CATCHQ_ACT_NONE, 1, 0, 0> type; };
template <> struct EpiOf<EPI_RES_Y> { typedef EpiSpec<1, 1, 1, CATCHQ_ACT_RELU, 1, 0, 0> type; };
template <> struct EpiOf<EPI_Y16_RELU> { typedef EpiSpec<1, 1, 0, CATCHQ_ACT_RELU, 2, 0, 0> type; };
template <> struct EpiOf<EPI_Q8_RELU6> { typedef EpiSpec<1, 1, 0, CATCHQ_ACT_RELU6, 0, 8, 0> type; };
template <> struct EpiOf<EPI_RES_Q8> { typedef EpiSpec<1, 1, 1, CATCHQ_ACT_RELU, 0, 8, 0> type; };
template <> struct EpiOf<EPI_LIN_Q8> { typedef EpiSpec<1, 1, 0, CATCHQ_ACT_NONE, 0, 8, 0> type; };
template <> struct EpiOf<EPI_LIN_Y_Q8> { typedef EpiSpec<1, 1, 0, CATCHQ_ACT_NONE, 1, 8, 0> type; };
template <> struct EpiOf<EPI_LIN_RES_Q8> { typedef EpiSpec<1, 1, 1, CATCHQ_ACT_NONE, 0, 8, 0> type; };
template <> struct EpiOf<EPI_LIN_RES_Y_Q8> { typedef EpiSpec<1, 1, 1, CATCHQ_ACT_NONE, 1, 8, 0> type; };
template <> struct EpiOf<EPI_LK_Q16> { typedef EpiSpec<0, 1, 0, CATCHQ_ACT_LEAKY, 0, 16, 0> type; };
template <> struct EpiOf<EPI_LK_Y_Q16> { typedef EpiSpec<0, 1, 0, CATCHQ_ACT_LEAKY, 1, 16, 0> type; };
template <> struct EpiOf<EPI_LK_RESA_Q16> { typedef EpiSpec<0, 1, 2, CATCHQ_ACT_LEAKY, 0, 16, 0> type; };
template <> struct EpiOf<EPI_LK_RESA_Y_Q16> { typedef EpiSpec<0, 1, 2, CATCHQ_ACT_LEAKY, 1, 16, 0> type; };

// which variant serves this launch (the specialised ones also need a unit requantization scale: a
// fractional one costs them 2-4 % end to end even when it is not used, measured); a kernel family
// that has no instance of the variant returned uses the generic EPI_VECTOR
inline int pick_epilogue(int N, const EpiDev &e) {
  if (!vec_epilogue_ok(N, e)) return EPI_SCALAR;
  if (e.acc_out || (e.q && e.q_scale != 1.0f) || (e.chan_div && !e.chan_rcp) || e.half_steps) return EPI_VECTOR;
  // (the instances that fold the requantization's power of two into the per-channel constants keep those in range)
  if (e.q && (e.q_neg_pos < -40 || e.q_neg_pos > 40)) return EPI_VECTOR;
  const int div = e.chan_rcp ? 1 : 0, bias = e.bias ? 1 : 0;
  const int res = !e.resid ? 0 : (e.resid_after ? 2 : 1);
  const int ym = !e.y ? 0 : (e.y_f16 ? 2 : 1);
  const int qm = !e.q ? 0 : e.q_bw;
  static const struct { int epi, div, bias, res, act, ym, qm; } rows[] = {
      {EPI_Q8_RELU, 1, 1, 0, CATCHQ_ACT_RELU, 0, 8},        {EPI_RES_Y_Q8, 1, 1, 1, CATCHQ_ACT_RELU, 1, 8},
      {EPI_Y32, 1, 1, 0, CATCHQ_ACT_NONE, 1, 0},            {EPI_RES_Y, 1, 1, 1, CATCHQ_ACT_RELU, 1, 0},
      {EPI_Y16_RELU, 1, 1, 0, CATCHQ_ACT_RELU, 2, 0},       {EPI_Q8_RELU6, 1, 1, 0, CATCHQ_ACT_RELU6, 0, 8},
      {EPI_RES_Q8, 1, 1, 1, CATCHQ_ACT_RELU, 0, 8},         {EPI_LIN_Q8, 1, 1, 0, CATCHQ_ACT_NONE, 0, 8},
      {EPI_LIN_Y_Q8, 1, 1, 0, CATCHQ_ACT_NONE, 1, 8},       {EPI_LIN_RES_Q8, 1, 1, 1, CATCHQ_ACT_NONE, 0, 8},
      {EPI_LIN_RES_Y_Q8, 1, 1, 1, CATCHQ_ACT_NONE, 1, 8},   {EPI_LK_Q16, 0, 1, 0, CATCHQ_ACT_LEAKY, 0, 16},
      {EPI_LK_Y_Q16, 0, 1, 0, CATCHQ_ACT_LEAKY, 1, 16},     {EPI_LK_RESA_Q16, 0, 1, 2, CATCHQ_ACT_LEAKY, 0, 16},
      {EPI_LK_RESA_Y_Q16, 0, 1, 2, CATCHQ_ACT_LEAKY, 1, 16}};
  for (const auto &r : rows)
    if (r.div == div && r.bias == bias && r.res == res && r.act == e.act && r.ym == ym && r.qm == qm) return r.epi;
  return EPI_VECTOR;
}

// per-channel constants of one lane's four consecutive channels
struct EpiLane {
  v4f div, rcp, bias;
  bool use_rcp, use_div, use_bias, use_res, res_after, unit_q, half_steps;
  int act;
};

template <class S>
__device__ __forceinline__ EpiLane epi_lane_setup(int n, bool n_ok, const EpiDev &e) {
  EpiLane L;
  L.use_rcp = S::rcp(e); L.use_div = S::truediv(e); L.use_bias = S::bias(e); L.use_res = S::resid(e);
  L.res_after = S::resid_after(e);
  L.act = S::act(e);
  L.unit_q = S::kGeneric ? (e.q_scale == 1.0f) : true;
  L.half_steps = S::kGeneric ? (e.half_steps != 0) : false;
  // Reciprocal form with the power of two folded in:
  //   v = (f*2^e)/d  ==  q = f*(r*2^e); err = fma(-q, d*2^-e, f); fma(err, r*2^e, q)
  // (scaling by 2^e is exact, so every intermediate is the scaled image of the unfolded one)
  L.div = v4f{1.f, 1.f, 1.f, 1.f}; L.rcp = v4f{1.f, 1.f, 1.f, 1.f}; L.bias = v4f{0.f, 0.f, 0.f, 0.f};
  if (n_ok && (L.use_rcp || L.use_div)) L.div = *reinterpret_cast<const v4f *>(e.chan_div + n);
  if (n_ok && L.use_rcp) {
    L.rcp = *reinterpret_cast<const v4f *>(e.chan_rcp + n);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      L.rcp[t] = __builtin_ldexpf(L.rcp[t], e.exp2 + (S::kFoldScale ? e.q_neg_pos : 0));
      L.div[t] = __builtin_ldexpf(L.div[t], -e.exp2 - (S::kFoldScale ? e.q_neg_pos : 0));
    }
  }
  if (n_ok && L.use_bias) {
    L.bias = *reinterpret_cast<const v4f *>(e.bias + n);
    if constexpr (S::kFoldScale) {
#pragma unroll
      for (int t = 0; t < 4; ++t) L.bias[t] = __builtin_ldexpf(L.bias[t], e.q_neg_pos);
    }
  }
  return L;
}

// dequantization and bias of one integer sum: channel t of the lane's four
__device__ __forceinline__ float epi_dequant1(int a, int t, const EpiLane &L, int exp2) {
  float x = (float)a;
  if (L.use_rcp) x = div_by_rcp(x, L.div[t], L.rcp[t]);
  else {
    x = __builtin_ldexpf(x, exp2);
    if (L.half_steps) x = round_f16(x);
    if (L.use_div) {
      x = x / L.div[t];
      if (L.half_steps) x = round_f16(x);
    }
  }
  if (L.use_bias) {
    x = x + L.bias[t];
    if (L.half_steps) x = round_f16(x);
  }
  return x;
}

// Where an output element lives: a 64-bit element index, or a wave-uniform 64-bit part plus a 32-bit
// per-lane part (then the uniform part stays in scalar registers and a store needs one vector add).
struct EpiAt64 {
  int64_t idx;
  template <class T> __device__ __forceinline__ T *at(T *base) const { return base + idx; }
};
struct EpiAtSplit {
  int64_t uni;   // same for every lane of the wave
  unsigned off;  // this lane's part
  template <class T> __device__ __forceinline__ T *at(T *base) const { return (base + uni) + off; }
};

// A store / load with or without the non-temporal hint, chosen by a wave-uniform flag.  The empty volatile
// statements keep the two branches apart: merged into one access, they would lose the hint.
template <class T>
__device__ __forceinline__ void store_stream(T *dst, const T v, bool stream) {
  if (stream) {
    asm volatile("");
    __builtin_nontemporal_store(v, dst);
    asm volatile("");
  } else {
    *dst = v;
  }
}
template <class T>
__device__ __forceinline__ T load_stream(const T *src, bool stream) {
  T v;
  if (stream) {
    asm volatile("");
    v = __builtin_nontemporal_load(src);
    asm volatile("");
  } else {
    v = *src;
  }
  return v;
}

// four integer sums of one pixel (channels n..n+3 at `where`) -> all requested outputs
template <class S, class At>
__device__ __forceinline__ void epi_vec4(const v4i a, const v4f res, const EpiLane &L, const At where, const EpiDev &e) {
  if (S::acc(e)) *reinterpret_cast<v4i *>(where.at(e.acc_out)) = a;
  float v[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    float x = epi_dequant1(a[t], t, L, e.exp2);
    if (L.use_res && !L.res_after) x = x + res[t];
    if constexpr (!S::kFoldAct) {
      if (L.act == CATCHQ_ACT_LEAKY) x = (x > 0.0f) ? x : x * e.act_slope;
      else if (L.act >= CATCHQ_ACT_RELU) x = (x > 0.0f) ? x : 0.0f;
      if (L.act == CATCHQ_ACT_RELU6) x = (x < 6.0f) ? x : 6.0f;
      if (L.use_res && L.res_after) x = x + res[t];
    }
    v[t] = x;
  }
  if (S::y16(e)) {
    // two values per conversion instruction (v_cvt_pk_f16_f32: round to nearest even, like the single conversion)
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f16x2 h01 = __builtin_convertvector(f32x2{v[0], v[1]}, f16x2), h23 = __builtin_convertvector(f32x2{v[2], v[3]}, f16x2);
    const v2i packed = {__builtin_bit_cast(int, h01), __builtin_bit_cast(int, h23)};
    store_stream(reinterpret_cast<v2i *>(where.at(reinterpret_cast<__half *>(e.y))), packed, e.y_stream != 0);
  } else if (S::y32(e)) {
    v4f o = {v[0], v[1], v[2], v[3]};
    store_stream(reinterpret_cast<v4f *>(where.at(reinterpret_cast<float *>(e.y))), o, e.y_stream != 0);
  }
  if constexpr (S::kFoldScale) {
    // v is already in units of the output's step: clamp to 0 .. min(127, 6 / step) (the median maps a NaN to 0, as
    // ReLU does), then round, saturate and insert byte by byte
    float hi = 127.0f;
    if constexpr (S::kAct == CATCHQ_ACT_RELU6) {
      const float six = __builtin_ldexpf(6.0f, e.q_neg_pos);
      hi = (six < hi) ? six : hi;
    }
    unsigned packed = 0;
#pragma unroll
    for (int t = 0; t < 4; ++t)
      packed = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(v[t], 0.0f, hi), (unsigned)t, packed);
    *reinterpret_cast<unsigned *>(where.at(reinterpret_cast<int8_t *>(e.q))) = packed;
  } else if constexpr (!S::kGeneric && S::kQ == 8 && (S::kAct == CATCHQ_ACT_RELU || S::kAct == CATCHQ_ACT_RELU6)) {
    // values are >= 0 and never NaN here (or, with the activation folded in, are made so by the median:
    // for a NaN operand it returns the smallest of the other two, 0, which is what ReLU makes of a NaN);
    // the requantization scale is 1:
    //   sat(rne(x * 2^-pos)) = low byte of the float  fma(min(x, 127 * 2^pos), 2^-pos, 1.5 * 2^23)
    // (the product is exact, so the fma rounds once, to an integer, ties to even; clamping before
    // the rounding equals clamping after it because the bound is an integer multiple of 2^pos; a ReLU6
    // bound of 6 below that one takes its place: min(min(x, 6), hi) = min(x, min(6, hi)))
    float hi = __builtin_ldexpf(127.0f, -e.q_neg_pos);
    const float sc = __builtin_ldexpf(1.0f, e.q_neg_pos);
    if constexpr (S::kFoldAct && S::kAct == CATCHQ_ACT_RELU6) hi = (hi < 6.0f) ? hi : 6.0f;
    unsigned b[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float x = __builtin_amdgcn_fmed3f(v[t], 0.0f, hi);  // one instruction for max(0, min(v, hi))
      b[t] = __builtin_bit_cast(unsigned, __builtin_fmaf(x, sc, 12582912.0f));
    }
    const unsigned lo = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
    const unsigned hi2 = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
    *reinterpret_cast<unsigned *>(where.at(reinterpret_cast<int8_t *>(e.q))) = lo | hi2;
  } else if (S::q8(e)) {
    int b[4];
    if (L.unit_q) {
#pragma unroll
      for (int t = 0; t < 4; ++t) b[t] = quant1_unit<8>(v[t], e.q_neg_pos);
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t) b[t] = quant1<8>(v[t], e.q_scale, e.q_neg_pos);
    }
    // four clamped values -> four bytes: two byte permutes and a merge
    const unsigned lo = __builtin_amdgcn_perm((unsigned)b[1], (unsigned)b[0], 0x0c0c0400u);
    const unsigned hi = __builtin_amdgcn_perm((unsigned)b[3], (unsigned)b[2], 0x04000c0cu);
    *reinterpret_cast<unsigned *>(where.at(reinterpret_cast<int8_t *>(e.q))) = lo | hi;
  } else if (S::q16(e)) {
    // rounded to an integer and converted (NaN -> 0, out-of-range values saturate to the int32 range), then
    // v_cvt_pk_i16_i32 saturates two of them to int16 and packs them: no clamp, mask or shift of our own
    int i32[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const float x = L.unit_q ? v[t] : v[t] * e.q_scale;
      i32[t] = cvt_i32_sat(__builtin_rintf(__builtin_ldexpf(x, e.q_neg_pos)));
    }
    v2i pk;
    pk[0] = __builtin_bit_cast(int, __builtin_amdgcn_cvt_pk_i16(i32[0], i32[1]));
    pk[1] = __builtin_bit_cast(int, __builtin_amdgcn_cvt_pk_i16(i32[2], i32[3]));
    *reinterpret_cast<v2i *>(where.at(reinterpret_cast<int16_t *>(e.q))) = pk;
  }
}
template <class S>
__device__ __forceinline__ void epi_vec4(const v4i a, const v4f res, const EpiLane &L, int64_t idx, const EpiDev &e) {
  epi_vec4<S, EpiAt64>(a, res, L, EpiAt64{idx}, e);
}

// this lane's four channels within a wave tile of TN*32 columns starting at n_w
template <int TN>
__device__ __forceinline__ int epi_lane_channel(int n_w, int lane) { return n_w + (lane % (TN * 8)) * 4; }

// Vector epilogue of one wave with the lane's per-channel constants supplied by the caller (kernels
// that run many row groups against the same columns set them up once).  m_w and n_w are the same for
// every lane of the wave.  An element's index splits into the uniform (m_w + i*32) * N + n_w and a
// 32-bit per-lane rest, and a wave whose tile lies wholly inside the matrix (the usual case) runs
// without any per-lane bounds checks (FAST_PATH = false leaves that copy of the code out: kernels that
// unroll the epilogue several times over cannot afford the registers its free scheduling takes).
// BATCHES > 1 handles the 32 rows of a staged block in that many passes (residual loads, staged reads and
// arithmetic of one pass before the next): fewer values live at once, for instances that would otherwise lose a
// wave per SIMD to their register count.
template <int TM, int TN, int EPI, bool FAST_PATH = true, int BATCHES = 1>
__device__ __forceinline__ void igemm_epilogue_vec(v16i (&acc)[TM][TN], int *stage, int64_t m_w, int n_w, int lane,
                                                   const IgemmParams &p, const EpiDev &e, const EpiLane &L) {
  typedef typename EpiOf<EPI>::type S;
  constexpr int WN = TN * 32;
  constexpr int EPI_STRIDE = WN + 8;  // +8 ints: the two half-waves write different banks
  const int frow = lane & 31, fhalf = lane >> 5;
  constexpr int CPR = WN / 4;    // 4-channel groups per staged row
  constexpr int RPI = 64 / CPR;  // rows the wave moves per iteration
  constexpr int NIT = 32 / RPI;
  const int cg = lane % CPR, rsub = lane / CPR;
  const bool use_res = L.use_res;
  const unsigned lane_off0 = (unsigned)rsub * (unsigned)out_ld(p) + (unsigned)(cg * 4);
  const unsigned it_step = (unsigned)RPI * (unsigned)out_ld(p);
  auto tile = [&](auto full_c) {
    constexpr bool FULL = decltype(full_c)::value;
    const bool n_ok = FULL || (n_w + cg * 4 < p.N);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int64_t uni = (m_w + i * 32) * (int64_t)out_ld(p) + n_w;
      const int64_t left = p.M - (m_w + i * 32);
      const int rows = FULL ? 32 : (left < 0 ? 0 : (left > 32 ? 32 : (int)left));  // uniform
      // Opaque copy: a kernel that calls this in a loop would otherwise keep every iteration's byte
      // offsets (loop invariants) in registers across the whole loop; recomputing them costs one add each.
      unsigned lane_off = lane_off0;
      asm volatile("" : "+v"(lane_off));
      constexpr int NB = NIT / BATCHES;
      static_assert(NIT % BATCHES == 0, "the passes must divide the iterations");
      v4f resv[NB];
      auto load_resid = [&](int b) {
#pragma unroll
        for (int k = 0; k < NB; ++k) {
          const int it = b * NB + k;
          resv[k] = v4f{0.f, 0.f, 0.f, 0.f};
          if (FULL || (n_ok && it * RPI + rsub < rows))
            resv[k] = load_stream(reinterpret_cast<const v4f *>((e.resid + uni) + (lane_off + it * it_step)), e.resid_stream != 0);
        }
      };
      // residual rows of this 32-row block (of its first pass): all loads in flight before the staging below
      if (use_res) load_resid(0);
      // wave-private staging: stores then loads of the same wave, ordered by the LDS counter
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          stage[(8 * (r >> 2) + 4 * fhalf + (r & 3)) * EPI_STRIDE + j * 32 + frow] = acc[i][j][r];
#pragma unroll
      for (int b = 0; b < BATCHES; ++b) {
        if (b > 0 && use_res) load_resid(b);
        // all reads first: one LDS latency per pass instead of one per iteration
        v4i av[NB];
#pragma unroll
        for (int k = 0; k < NB; ++k)
          av[k] = *reinterpret_cast<const v4i *>(stage + ((b * NB + k) * RPI + rsub) * EPI_STRIDE + cg * 4);
#pragma unroll
        for (int k = 0; k < NB; ++k) {
          const int it = b * NB + k;
          if (!FULL && !(n_ok && it * RPI + rsub < rows)) continue;
          epi_vec4<S>(av[k], use_res ? resv[k] : v4f{0.f, 0.f, 0.f, 0.f}, L, EpiAtSplit{uni, lane_off + it * it_step}, e);
        }
      }
    }
  };
  // wave-uniform: the whole TM*32 x WN tile inside the matrix?
  if (FAST_PATH && m_w + TM * 32 <= p.M && n_w + WN <= p.N) tile(std::true_type{});
  else tile(std::false_type{});
}

// Vector epilogue of one wave whose residual comes from a second set of accumulators (same tile,
// same layout) instead of memory: both sets go through the wave's staging area, the shortcut's first.
template <int TM, int TN, int EPI>
__device__ __forceinline__ void igemm_epilogue_dual(v16i (&acc)[TM][TN], v16i (&acc_sc)[TM][TN], int *stage, int64_t m_w,
                                                    int n_w, int lane, const IgemmParams &p, const EpiDev &e,
                                                    const ShortcutDev &sc) {
  typedef typename EpiOf<EPI>::type S;
  static_assert(EPI != EPI_SCALAR, "the two-branch epilogue is the vector one");
  constexpr int WN = TN * 32;
  constexpr int EPI_STRIDE = WN + 8;
  const int frow = lane & 31, fhalf = lane >> 5;
  constexpr int CPR = WN / 4;
  constexpr int RPI = 64 / CPR;
  const int cg = lane % CPR, rsub = lane / CPR;
  const int n = n_w + cg * 4;
  const bool n_ok = n < p.N;
  EpiLane L = epi_lane_setup<S>(n, n_ok, e);
  L.use_res = true;
  L.res_after = e.resid_after != 0;
  EpiDev e_sc = {};
  e_sc.exp2 = sc.exp2; e_sc.chan_div = sc.chan_div; e_sc.chan_rcp = sc.chan_rcp; e_sc.bias = sc.bias;
  const EpiLane L_sc = epi_lane_setup<EpiGeneric>(n, n_ok, e_sc);
  const unsigned lane_off = (unsigned)rsub * (unsigned)out_ld(p) + (unsigned)(cg * 4);
  const unsigned it_step = (unsigned)RPI * (unsigned)out_ld(p);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    // shortcut sums -> fp32 residual values in the row-major layout of the stores
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        stage[(8 * (r >> 2) + 4 * fhalf + (r & 3)) * EPI_STRIDE + j * 32 + frow] = acc_sc[i][j][r];
    v4f resv[32 / RPI];
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
      const v4i a = *reinterpret_cast<const v4i *>(stage + (it * RPI + rsub) * EPI_STRIDE + cg * 4);
#pragma unroll
      for (int t = 0; t < 4; ++t) resv[it][t] = epi_dequant1(a[t], t, L_sc, sc.exp2);
    }
    // the wave's LDS operations complete in order: these stores cannot overtake the reads above
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        stage[(8 * (r >> 2) + 4 * fhalf + (r & 3)) * EPI_STRIDE + j * 32 + frow] = acc[i][j][r];
    const int64_t uni = (m_w + i * 32) * (int64_t)out_ld(p) + n_w;
    const int64_t left = p.M - (m_w + i * 32);
    const int rows = left < 0 ? 0 : (left > 32 ? 32 : (int)left);
    v4i av[32 / RPI];
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it)
      av[it] = *reinterpret_cast<const v4i *>(stage + (it * RPI + rsub) * EPI_STRIDE + cg * 4);
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
      if (!n_ok || it * RPI + rsub >= rows) continue;
      epi_vec4<S>(av[it], resv[it], L, EpiAtSplit{uni, lane_off + it * it_step}, e);
    }
  }
}

// Epilogue of one wave.  acc[i][j] is the 32x32 accumulator of rows m_w + i*32 .., columns
// n_w + j*32 ..; stage is this wave's private LDS area of 32 * (TN*32 + 8) ints.
template <int TM, int TN, int EPI, int BATCHES = 1>
__device__ __forceinline__ void igemm_epilogue(v16i (&acc)[TM][TN], int *stage, int64_t m_w, int n_w, int lane,
                                               const IgemmParams &p, const EpiDev &e) {
  typedef typename EpiOf<EPI>::type S;
  const int frow = lane & 31, fhalf = lane >> 5;
  if constexpr (EPI == EPI_SCALAR) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = n_w + j * 32 + frow;
        if (n >= p.N) continue;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t m = m_w + i * 32 + 8 * (r >> 2) + 4 * fhalf + (r & 3);
          if (m >= p.M) continue;
          const int64_t idx = m * out_ld(p) + n;
          const int a = acc[i][j][r];
          if (e.acc_out) e.acc_out[idx] = a;
          epi_store(epi_value((float)a, idx, n, e), idx, e);
        }
      }
    }
  } else {
    const int n = epi_lane_channel<TN>(n_w, lane);
    const EpiLane L = epi_lane_setup<S>(n, n < p.N, e);
    igemm_epilogue_vec<TM, TN, EPI, true, BATCHES>(acc, stage, m_w, n_w, lane, p, e, L);
  }
}

// 16 consecutive int16 (two 16-byte chunks) -> their high bytes and their biased low bytes
__device__ __forceinline__ void split_i16(const v4i c0, const v4i c1, v4i &hi, v4i &lo) {
  hi[0] = (int)__builtin_amdgcn_perm((unsigned)c0[1], (unsigned)c0[0], 0x07050301u);
  hi[1] = (int)__builtin_amdgcn_perm((unsigned)c0[3], (unsigned)c0[2], 0x07050301u);
  hi[2] = (int)__builtin_amdgcn_perm((unsigned)c1[1], (unsigned)c1[0], 0x07050301u);
  hi[3] = (int)__builtin_amdgcn_perm((unsigned)c1[3], (unsigned)c1[2], 0x07050301u);
  lo[0] = (int)(__builtin_amdgcn_perm((unsigned)c0[1], (unsigned)c0[0], 0x06040200u) ^ 0x80808080u);
  lo[1] = (int)(__builtin_amdgcn_perm((unsigned)c0[3], (unsigned)c0[2], 0x06040200u) ^ 0x80808080u);
  lo[2] = (int)(__builtin_amdgcn_perm((unsigned)c1[1], (unsigned)c1[0], 0x06040200u) ^ 0x80808080u);
  lo[3] = (int)(__builtin_amdgcn_perm((unsigned)c1[3], (unsigned)c1[2], 0x06040200u) ^ 0x80808080u);
}

// launchers of the LDS-DMA pipelined kernel (igemm_i8_dma.hip); return -1 when the shape is not
// eligible (operand of 2 GiB or more, four-channel stem) and the caller takes the register-staged kernel
int igemm_dma_launch(int load, const void *a, const void *b, IgemmParams p, const EpiDev &e, int64_t a_bytes,
                     int64_t b_bytes, hipStream_t s);


}  // namespace catchq
