// Streaming quantize / dequantize / max-abs kernels: HBM-bound, 16-byte loads per lane,
// lane-contiguous so every wave instruction touches whole cache lines.
#include <mutex>

#include "catchq_common.h"

namespace catchq {

constexpr int kThreads = 256;
constexpr int kMaxBlocks = 256 * 16;  // 256 CUs, enough resident waves to cover HBM latency

static inline int grid_for(int64_t work_items, int per_block) {
  int64_t b = (work_items + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > kMaxBlocks) b = kMaxBlocks;
  return (int)b;
}

__device__ __forceinline__ __half2 as_half2(int bits) {
  __half2 h;
  __builtin_memcpy(&h, &bits, 4);
  return h;
}

__device__ __forceinline__ float ld_f(const float *p, int64_t i) { return p[i]; }
__device__ __forceinline__ float ld_f(const __half *p, int64_t i) { return __half2float(p[i]); }

// ---- per-tensor quantize -------------------------------------------------------------------------
// Vector body: each lane converts VEC consecutive elements per step (one 16-byte load).
template <typename TIn, int BW>
__global__ __launch_bounds__(kThreads) void quantize_vec_kernel(const TIn *__restrict__ x,
                                                               typename QRange<BW>::type *__restrict__ q,
                                                               int64_t n, int pos, float scale,
                                                               const int32_t *__restrict__ pos_dev,
                                                               const float *__restrict__ scale_dev) {
  constexpr int VEC = 16 / sizeof(TIn);  // 4 floats or 8 halfs
  typedef typename QRange<BW>::type TQ;
  if (pos_dev) pos = *pos_dev;
  if (scale_dev) scale = *scale_dev;
  const int neg_pos = -pos;
  const int64_t nvec = n / VEC;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < nvec; i += stride) {
    v4i raw = __builtin_nontemporal_load(reinterpret_cast<const v4i *>(x) + i);
    TQ out[VEC];
    if constexpr (sizeof(TIn) == 4) {
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j] = (TQ)quant1<BW>(__int_as_float(raw[j]), scale, neg_pos);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const __half2 h = as_half2(raw[j]);
        out[2 * j] = (TQ)quant1<BW>(__low2float(h), scale, neg_pos);
        out[2 * j + 1] = (TQ)quant1<BW>(__high2float(h), scale, neg_pos);
      }
    }
    constexpr int OUT_BYTES = VEC * sizeof(TQ);
    if constexpr (OUT_BYTES == 4) {
      *reinterpret_cast<int *>(q + i * VEC) = *reinterpret_cast<int *>(out);
    } else if constexpr (OUT_BYTES == 8) {
      *reinterpret_cast<v2i *>(q + i * VEC) = *reinterpret_cast<v2i *>(out);
    } else if constexpr (OUT_BYTES == 16) {
      *reinterpret_cast<v4i *>(q + i * VEC) = *reinterpret_cast<v4i *>(out);
    } else {
      reinterpret_cast<v4i *>(q + i * VEC)[0] = reinterpret_cast<v4i *>(out)[0];
      reinterpret_cast<v4i *>(q + i * VEC)[1] = reinterpret_cast<v4i *>(out)[1];
    }
  }
  // tail (< VEC elements) by the first lanes of block 0
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - nvec * VEC)) {
    int64_t i = nvec * VEC + threadIdx.x;
    q[i] = (TQ)quant1<BW>(ld_f(x, i), scale, neg_pos);
  }
}

// Scalar body for unaligned pointers.
template <typename TIn, int BW>
__global__ __launch_bounds__(kThreads) void quantize_scalar_kernel(const TIn *__restrict__ x,
                                                                  typename QRange<BW>::type *__restrict__ q,
                                                                  int64_t n, int pos, float scale,
                                                                  const int32_t *__restrict__ pos_dev,
                                                                  const float *__restrict__ scale_dev) {
  typedef typename QRange<BW>::type TQ;
  if (pos_dev) pos = *pos_dev;
  if (scale_dev) scale = *scale_dev;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    q[i] = (TQ)quant1<BW>(ld_f(x, i), scale, -pos);
}

template <typename TIn, int BW>
static int launch_quantize(const void *x, void *q, int64_t n, int pos, float scale, const int32_t *pos_dev,
                           const float *scale_dev, hipStream_t s) {
  typedef typename QRange<BW>::type TQ;
  constexpr int VEC = 16 / sizeof(TIn);
  if (aligned16(x) && aligned16(q)) {
    quantize_vec_kernel<TIn, BW><<<grid_for(n / VEC, kThreads * 4), kThreads, 0, s>>>(
        (const TIn *)x, (TQ *)q, n, pos, scale, pos_dev, scale_dev);
  } else {
    quantize_scalar_kernel<TIn, BW><<<grid_for(n, kThreads * 4), kThreads, 0, s>>>(
        (const TIn *)x, (TQ *)q, n, pos, scale, pos_dev, scale_dev);
  }
  return launch_status();
}

static int quantize_dispatch(const void *x, int x_dtype, void *q, int bw, int64_t n, int pos, float scale,
                             const int32_t *pos_dev, const float *scale_dev, hipStream_t s) {
  if (n < 0 || (n > 0 && (!x || !q))) return CATCHQ_ERR_ARG;
  if (x_dtype != CATCHQ_F32 && x_dtype != CATCHQ_F16) return CATCHQ_ERR_DTYPE;
  if (bw != 8 && bw != 16 && bw != 31) return CATCHQ_ERR_BITWIDTH;
  if (!pos_dev && (pos < -126 || pos > 126)) return CATCHQ_ERR_ARG;
  if (n == 0) return CATCHQ_OK;
#define CATCHQ_Q(T, B) return launch_quantize<T, B>(x, q, n, pos, scale, pos_dev, scale_dev, s)
  if (x_dtype == CATCHQ_F32) {
    if (bw == 8) CATCHQ_Q(float, 8);
    if (bw == 16) CATCHQ_Q(float, 16);
    CATCHQ_Q(float, 31);
  }
  if (bw == 8) CATCHQ_Q(__half, 8);
  if (bw == 16) CATCHQ_Q(__half, 16);
  CATCHQ_Q(__half, 31);
#undef CATCHQ_Q
}

// ---- NCHW fp -> NHWC int (channels padded to cpad) ---------------------------------------------
// One thread per pixel: reads are coalesced along W for every channel plane, the store is one
// cpad-wide vector per pixel.  Meant for few-channel network inputs (cpad <= 16).
template <typename TIn, int BW, int CPAD>
__global__ __launch_bounds__(kThreads) void quantize_nchw_nhwc_kernel(const TIn *__restrict__ x,
                                                                     typename QRange<BW>::type *__restrict__ q,
                                                                     int n, int c, int64_t hw, int pos,
                                                                     float scale) {
  typedef typename QRange<BW>::type TQ;
  const int64_t total = (int64_t)n * hw;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t p = (int64_t)blockIdx.x * kThreads + threadIdx.x; p < total; p += stride) {
    int64_t img = p / hw, pix = p - img * hw;
    TQ out[CPAD];
#pragma unroll
    for (int ch = 0; ch < CPAD; ++ch) {
      out[ch] = 0;
      if (ch < c) out[ch] = (TQ)quant1<BW>(ld_f(x, (img * c + ch) * hw + pix), scale, -pos);
    }
    constexpr int BYTES = CPAD * sizeof(TQ);
    if constexpr (BYTES == 4) *reinterpret_cast<int *>(q + p * CPAD) = *reinterpret_cast<int *>(out);
    else if constexpr (BYTES == 8) *reinterpret_cast<v2i *>(q + p * CPAD) = *reinterpret_cast<v2i *>(out);
    else if constexpr (BYTES == 16) *reinterpret_cast<v4i *>(q + p * CPAD) = *reinterpret_cast<v4i *>(out);
    else {
#pragma unroll
      for (int ch = 0; ch < CPAD; ++ch) q[p * CPAD + ch] = out[ch];
    }
  }
}

// The same into a frame: output [n, oh, ow, CPAD] holds the image at (top, left) and zeros around it
// (a convolution's zero padding materialised once, so its loads need no border handling).
template <typename TIn, int BW, int CPAD>
__global__ __launch_bounds__(kThreads) void quantize_nchw_nhwc_frame_kernel(const TIn *__restrict__ x,
                                                                           typename QRange<BW>::type *__restrict__ q,
                                                                           int n, int c, int h, int w, int oh, int ow,
                                                                           int top, int left, int pos, float scale) {
  typedef typename QRange<BW>::type TQ;
  // A block is 64 lanes along a row x 4 rows; a lane owns PX pixels of its row, 64 apart (so that every load
  // and store instruction of the wave covers consecutive pixels), all of whose loads (PX pixels x c channel
  // planes) are requested before the first conversion.  The rows' coordinates are computed once per row: a
  // pixel costs no division.
  constexpr int PX = 4;
  const int64_t hw = (int64_t)h * w, rows = (int64_t)n * oh;
  const int lx = threadIdx.x & 63, ly = threadIdx.x >> 6;
  for (int64_t row = (int64_t)blockIdx.y * 4 + ly; row < rows; row += (int64_t)gridDim.y * 4) {
    const int64_t img = row / oh;
    const int oy = (int)(row - img * oh), iy = oy - top;
    const bool row_inside = (unsigned)iy < (unsigned)h;
    const TIn *src = x + img * c * hw + (int64_t)iy * w;
    TQ *dst = q + row * ow * CPAD;
    for (int ox0 = blockIdx.x * 64 * PX + lx; ox0 < ow; ox0 += gridDim.x * 64 * PX) {
      float v[PX][CPAD];
#pragma unroll
      for (int px = 0; px < PX; ++px) {
        const int ix = ox0 + px * 64 - left;
        const bool inside = row_inside && (unsigned)ix < (unsigned)w;
#pragma unroll
        for (int ch = 0; ch < CPAD; ++ch) {
          v[px][ch] = 0.0f;
          if (inside && ch < c) v[px][ch] = ld_f(src, ch * hw + ix);
        }
      }
#pragma unroll
      for (int px = 0; px < PX; ++px) {
        if (ox0 + px * 64 >= ow) break;
        TQ out[CPAD];
#pragma unroll
        for (int ch = 0; ch < CPAD; ++ch) out[ch] = (TQ)quant1<BW>(v[px][ch], scale, -pos);  // 0 -> 0
        constexpr int BYTES = CPAD * sizeof(TQ);
        TQ *o = dst + (ox0 + px * 64) * CPAD;
        if constexpr (BYTES == 4) *reinterpret_cast<int *>(o) = *reinterpret_cast<int *>(out);
        else if constexpr (BYTES == 8) *reinterpret_cast<v2i *>(o) = *reinterpret_cast<v2i *>(out);
        else *reinterpret_cast<v4i *>(o) = *reinterpret_cast<v4i *>(out);
      }
    }
  }
}

// General (any C) transpose-quantize through LDS: tile of 64 pixels x 64 channels.
template <typename TIn, int BW>
__global__ __launch_bounds__(kThreads) void quantize_nchw_nhwc_tile_kernel(const TIn *__restrict__ x,
                                                                          typename QRange<BW>::type *__restrict__ q,
                                                                          int n, int c, int64_t hw, int cpad,
                                                                          int pos, float scale) {
  typedef typename QRange<BW>::type TQ;
  __shared__ TQ tile[64][64 + 4];
  const int64_t ptiles = (hw + 63) / 64;
  const int ctiles = (cpad + 63) / 64;
  const int64_t total = (int64_t)n * ptiles * ctiles;
  for (int64_t t = blockIdx.x; t < total; t += gridDim.x) {
    int ct = (int)(t % ctiles);
    int64_t r = t / ctiles;
    int64_t pt = r % ptiles, img = r / ptiles;
    // read: lanes along pixels
    for (int i = threadIdx.x; i < 64 * 64; i += kThreads) {
      int ch = ct * 64 + i / 64;
      int64_t pix = pt * 64 + (i & 63);
      TQ v = 0;
      if (ch < c && pix < hw) v = (TQ)quant1<BW>(ld_f(x, (img * c + ch) * hw + pix), scale, -pos);
      tile[i & 63][i / 64] = v;
    }
    __syncthreads();
    // write: lanes along channels
    for (int i = threadIdx.x; i < 64 * 64; i += kThreads) {
      int ch = ct * 64 + (i & 63);
      int64_t pix = pt * 64 + i / 64;
      if (ch < cpad && pix < hw) q[(img * hw + pix) * cpad + ch] = tile[i / 64][i & 63];
    }
    __syncthreads();
  }
}

template <typename TIn, int BW>
static int launch_nchw_nhwc(const void *x, void *q, int n, int c, int h, int w, int cpad, int pos, float scale,
                            hipStream_t s) {
  typedef typename QRange<BW>::type TQ;
  const int64_t hw = (int64_t)h * w;
  const int64_t total = (int64_t)n * hw;
  const bool vec_ok = (reinterpret_cast<uintptr_t>(q) % (cpad * sizeof(TQ))) == 0;
  if (cpad == 4 && vec_ok) {
    quantize_nchw_nhwc_kernel<TIn, BW, 4><<<grid_for(total, kThreads), kThreads, 0, s>>>(
        (const TIn *)x, (TQ *)q, n, c, hw, pos, scale);
  } else if (cpad == 8 && vec_ok && BW == 8) {
    quantize_nchw_nhwc_kernel<TIn, BW, 8><<<grid_for(total, kThreads), kThreads, 0, s>>>(
        (const TIn *)x, (TQ *)q, n, c, hw, pos, scale);
  } else {
    int64_t tiles = (int64_t)n * ((hw + 63) / 64) * ((cpad + 63) / 64);
    quantize_nchw_nhwc_tile_kernel<TIn, BW><<<grid_for(tiles, 1), kThreads, 0, s>>>(
        (const TIn *)x, (TQ *)q, n, c, hw, cpad, pos, scale);
  }
  return launch_status();
}

// ---- per-channel weight quantize: q[c,i] = sat(rne(w[c,i] / sf[c])) ------------------------------
template <typename TIn, int BW>
__global__ __launch_bounds__(kThreads) void quantize_per_channel_kernel(const TIn *__restrict__ w,
                                                                       typename QRange<BW>::type *__restrict__ q,
                                                                       int64_t total, int64_t inner,
                                                                       const float *__restrict__ sf) {
  typedef typename QRange<BW>::type TQ;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    float t = ld_f(w, i) / sf[i / inner];  // correctly rounded fp32 division
    float r = __builtin_rintf(t);
    r = fminf(fmaxf(r, QRange<BW>::lo), QRange<BW>::hi);
    q[i] = (t != t) ? (TQ)0 : (TQ)(int)r;
  }
}

// the all-half form: weight, scale factor and their quotient are binary16 (the quotient of two halves,
// evaluated in fp32 and rounded to binary16, is the correctly rounded half quotient), then round + clamp
template <int BW>
__global__ __launch_bounds__(kThreads) void quantize_per_channel_f16_kernel(const __half *__restrict__ w,
                                                                           typename QRange<BW>::type *__restrict__ q,
                                                                           int64_t total, int64_t inner,
                                                                           const __half *__restrict__ sf) {
  typedef typename QRange<BW>::type TQ;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total; i += stride) {
    const float t = __half2float(__float2half_rn(__half2float(w[i]) / __half2float(sf[i / inner])));
    float r = __builtin_rintf(t);
    r = fminf(fmaxf(r, QRange<BW>::lo), QRange<BW>::hi);
    q[i] = (t != t) ? (TQ)0 : (TQ)(int)r;
  }
}

// ---- dequantize: y = q * 2^pos / scale ------------------------------------------------------------
template <typename TQ, typename TOut>
__global__ __launch_bounds__(kThreads) void dequantize_kernel(const TQ *__restrict__ q, TOut *__restrict__ y,
                                                             int64_t n, int pos, float scale) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride) {
    float t = __builtin_ldexpf((float)q[i], pos);
    if (scale != 1.0f) t = t / scale;
    if constexpr (sizeof(TOut) == 2) y[i] = __float2half_rn(t);
    else y[i] = t;
  }
}

// ---- max-abs reduction + position/scale finalize ---------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

template <typename TIn>
__global__ __launch_bounds__(kThreads) void absmax_partial_kernel(const TIn *__restrict__ x, int64_t n,
                                                                 float *__restrict__ partial, int vec_ok) {
  constexpr int VEC = 16 / sizeof(TIn);
  float m = 0.0f;  // fmaxf ignores NaN operands, like the oracle's comparison
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  int64_t done = 0;
  if (vec_ok) {
    const int64_t nvec = n / VEC;
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < nvec; i += stride) {
      v4i raw = reinterpret_cast<const v4i *>(x)[i];
      if constexpr (sizeof(TIn) == 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) m = fmaxf(m, fabsf(__int_as_float(raw[j])));
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const __half2 h = as_half2(raw[j]);
          m = fmaxf(m, fmaxf(fabsf(__low2float(h)), fabsf(__high2float(h))));
        }
      }
    }
    done = nvec * VEC;
  }
  for (int64_t i = done + (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    m = fmaxf(m, fabsf(ld_f(x, i)));
  __shared__ float wm[kThreads / 64];
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float r = wm[0];
    for (int i = 1; i < kThreads / 64; ++i) r = fmaxf(r, wm[i]);
    partial[blockIdx.x] = r;
  }
}

__global__ __launch_bounds__(kThreads) void absmax_finalize_kernel(const float *__restrict__ partial, int nparts,
                                                                  int bw, float *absmax_out, int32_t *pos_out,
                                                                  float *scale_out, float *offset_out) {
  float m = 0.0f;
  for (int i = threadIdx.x; i < nparts; i += kThreads) m = fmaxf(m, partial[i]);
  __shared__ float wm[kThreads / 64];
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0) wm[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    float absmax = wm[0];
    for (int i = 1; i < kThreads / 64; ++i) absmax = fmaxf(absmax, wm[i]);
    const float qmax = (bw == 16) ? 32767.0f : 127.0f;
    int pos = 0;
    float scale = 1.0f;
    if (absmax > 0.0f && absmax < __builtin_inff()) {
      // floor(log2(absmax)) from the exponent: exact, no transcendental
      pos = ilogbf(absmax) - (bw - 2);
      // absmax * 2^-pos is exact (also for a denormal absmax), so the quotient is rounded once
      scale = qmax / __builtin_ldexpf(absmax, -pos);
    }
    if (absmax_out) *absmax_out = absmax;
    if (pos_out) *pos_out = pos;
    if (scale_out) *scale_out = scale;
    if (offset_out) *offset_out = 0.0f;
  }
}

}  // namespace catchq

using namespace catchq;

CATCHQ_API int catchq_quantize(const void *x, int x_dtype, void *q, int bitwidth, int64_t n, int position,
                               float scale, catchq_stream_t stream) {
  return quantize_dispatch(x, x_dtype, q, bitwidth, n, position, scale, nullptr, nullptr, as_stream(stream));
}

CATCHQ_API int catchq_quantize_devpos(const void *x, int x_dtype, void *q, int bitwidth, int64_t n,
                                      const int32_t *position_dev, const float *scale_dev,
                                      catchq_stream_t stream) {
  if (!position_dev) return CATCHQ_ERR_ARG;
  return quantize_dispatch(x, x_dtype, q, bitwidth, n, 0, 1.0f, position_dev, scale_dev, as_stream(stream));
}

CATCHQ_API int catchq_quantize_nchw_to_nhwc(const void *x, int x_dtype, void *q, int bitwidth, int n, int c,
                                            int h, int w, int cpad, int position, float scale,
                                            catchq_stream_t stream) {
  if (n < 0 || c < 0 || h < 0 || w < 0 || cpad < c) return CATCHQ_ERR_SHAPE;
  if (x_dtype != CATCHQ_F32 && x_dtype != CATCHQ_F16) return CATCHQ_ERR_DTYPE;
  if (bitwidth != 8 && bitwidth != 16) return CATCHQ_ERR_BITWIDTH;
  if (position < -126 || position > 126) return CATCHQ_ERR_ARG;
  if ((int64_t)n * c * h * w == 0) return CATCHQ_OK;
  if (!x || !q) return CATCHQ_ERR_ARG;
  hipStream_t s = as_stream(stream);
  if (x_dtype == CATCHQ_F32)
    return bitwidth == 8 ? launch_nchw_nhwc<float, 8>(x, q, n, c, h, w, cpad, position, scale, s)
                         : launch_nchw_nhwc<float, 16>(x, q, n, c, h, w, cpad, position, scale, s);
  return bitwidth == 8 ? launch_nchw_nhwc<__half, 8>(x, q, n, c, h, w, cpad, position, scale, s)
                       : launch_nchw_nhwc<__half, 16>(x, q, n, c, h, w, cpad, position, scale, s);
}

template <typename TIn, int BW, int CPAD>
static int launch_frame(const void *x, void *q, int n, int c, int h, int w, int oh, int ow, int top, int left, int pos,
                        float scale, hipStream_t s) {
  typedef typename QRange<BW>::type TQ;
  const int64_t rows = (int64_t)n * oh;
  const int64_t row_groups = (rows + 3) / 4;  // a block takes 4 rows x 256 pixels
  const dim3 grid((unsigned)((ow + 255) / 256), (unsigned)(row_groups < 65535 ? row_groups : 65535));
  quantize_nchw_nhwc_frame_kernel<TIn, BW, CPAD><<<grid, kThreads, 0, s>>>((const TIn *)x, (TQ *)q, n, c, h, w, oh, ow,
                                                                          top, left, pos, scale);
  return launch_status();
}

CATCHQ_API int catchq_quantize_nchw_to_nhwc_frame(const void *x, int x_dtype, void *q, int bitwidth, int n, int c,
                                                  int h, int w, int cpad, int out_h, int out_w, int top, int left,
                                                  int position, float scale, catchq_stream_t stream) {
  if (n < 0 || c < 0 || h < 0 || w < 0 || cpad < c || top < 0 || left < 0 || out_h < h + top || out_w < w + left)
    return CATCHQ_ERR_SHAPE;
  if (x_dtype != CATCHQ_F32 && x_dtype != CATCHQ_F16) return CATCHQ_ERR_DTYPE;
  if (bitwidth != 8 && bitwidth != 16) return CATCHQ_ERR_BITWIDTH;
  if (position < -126 || position > 126) return CATCHQ_ERR_ARG;
  if (!((bitwidth == 8 && cpad == 4) || cpad == 8)) return CATCHQ_ERR_SHAPE;  // one 4/8/16-byte vector per pixel
  if ((int64_t)n * out_h * out_w == 0) return CATCHQ_OK;
  if (!x || !q || !aligned16(q)) return CATCHQ_ERR_ARG;
  hipStream_t s = as_stream(stream);
  const bool f32 = x_dtype == CATCHQ_F32;
#define CATCHQ_FRAME(T, BW, CP) launch_frame<T, BW, CP>(x, q, n, c, h, w, out_h, out_w, top, left, position, scale, s)
  if (bitwidth == 8 && cpad == 4) return f32 ? CATCHQ_FRAME(float, 8, 4) : CATCHQ_FRAME(__half, 8, 4);
  if (bitwidth == 8) return f32 ? CATCHQ_FRAME(float, 8, 8) : CATCHQ_FRAME(__half, 8, 8);
  return f32 ? CATCHQ_FRAME(float, 16, 8) : CATCHQ_FRAME(__half, 16, 8);
#undef CATCHQ_FRAME
}

static int absmax_blocks(int64_t n) { return grid_for(n / 4, kThreads * 4); }

CATCHQ_API int catchq_quantize_param_workspace_size(int64_t n, size_t *bytes) {
  if (!bytes || n < 0) return CATCHQ_ERR_ARG;
  *bytes = sizeof(float) * (size_t)absmax_blocks(n);
  return CATCHQ_OK;
}

CATCHQ_API int catchq_quantize_param(const void *x, int x_dtype, int64_t n, int bitwidth, int mode,
                                     void *workspace, size_t workspace_bytes, float *absmax_dev,
                                     int32_t *position_dev, float *scale_dev, float *offset_dev,
                                     catchq_stream_t stream) {
  if (n < 0 || (n > 0 && !x) || !workspace) return CATCHQ_ERR_ARG;
  if (x_dtype != CATCHQ_F32 && x_dtype != CATCHQ_F16) return CATCHQ_ERR_DTYPE;
  if (bitwidth != 8 && bitwidth != 16) return CATCHQ_ERR_BITWIDTH;
  if (mode < CATCHQ_QUANTIZE_POSITION || mode > CATCHQ_QUANTIZE_POSITION_SCALE_OFFSET) return CATCHQ_ERR_ARG;
  const int blocks = absmax_blocks(n);
  if (workspace_bytes < sizeof(float) * (size_t)blocks) return CATCHQ_ERR_ARG;
  hipStream_t s = as_stream(stream);
  float *partial = (float *)workspace;
  if (x_dtype == CATCHQ_F32)
    absmax_partial_kernel<float><<<blocks, kThreads, 0, s>>>((const float *)x, n, partial, aligned16(x) ? 1 : 0);
  else
    absmax_partial_kernel<__half><<<blocks, kThreads, 0, s>>>((const __half *)x, n, partial, aligned16(x) ? 1 : 0);
  if (launch_status() != CATCHQ_OK) return CATCHQ_ERR_LAUNCH;
  absmax_finalize_kernel<<<1, kThreads, 0, s>>>(partial, blocks, bitwidth, absmax_dev, position_dev,
                                               mode >= CATCHQ_QUANTIZE_POSITION_SCALE ? scale_dev : nullptr,
                                               mode >= CATCHQ_QUANTIZE_POSITION_SCALE_OFFSET ? offset_dev : nullptr);
  return launch_status();
}

// ---- the same reduction for callers that cannot allocate ---------------------------------------------------
// The per-block partial maxima live in a file-scope device array instead of a caller's workspace.  Each
// device holds its own copy of the array at its own address; host code never uses the array's name as a
// pointer, only the address hipGetSymbolAddress reports for the current device, looked up once per device.
static __device__ __align__(256) float scratch[kMaxBlocks];

static constexpr int kMaxDevices = 64;
static std::mutex scratch_mutex;
static float *scratch_ptr[kMaxDevices];  // guarded by scratch_mutex

static int scratch_for_current_device(float **out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return CATCHQ_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return CATCHQ_ERR_LAUNCH;
    }
    scratch_ptr[dev] = static_cast<float *>(p);
  }
  *out = scratch_ptr[dev];
  return CATCHQ_OK;
}

CATCHQ_API int catchq_quantize_param_noalloc(const void *x, int x_dtype, int64_t n, int bitwidth, int mode,
                                             float *absmax_dev, int32_t *position_dev, float *scale_dev,
                                             float *offset_dev, catchq_stream_t stream) {
  if (n < 0 || (n > 0 && !x)) return CATCHQ_ERR_ARG;
  if (n > CATCHQ_QUANTIZE_PARAM_NOALLOC_MAX_N) return CATCHQ_ERR_TOO_LARGE;
  float *partial = nullptr;
  const int st = scratch_for_current_device(&partial);
  if (st != CATCHQ_OK) return st;
  // every block writes its own slot before the finalize kernel reads exactly those slots: nothing of an
  // earlier call's contents is ever read, so nothing needs clearing
  return catchq_quantize_param(x, x_dtype, n, bitwidth, mode, partial, sizeof(float) * (size_t)kMaxBlocks,
                               absmax_dev, position_dev, scale_dev, offset_dev, stream);
}

CATCHQ_API int catchq_quantize_per_channel(const void *w, int w_dtype, void *q, int bitwidth, int co,
                                           int64_t inner, const float *scale_factor_dev,
                                           catchq_stream_t stream) {
  if (co < 0 || inner < 0) return CATCHQ_ERR_SHAPE;
  if (w_dtype != CATCHQ_F32 && w_dtype != CATCHQ_F16) return CATCHQ_ERR_DTYPE;
  if (bitwidth != 8 && bitwidth != 16) return CATCHQ_ERR_BITWIDTH;
  const int64_t total = (int64_t)co * inner;
  if (total == 0) return CATCHQ_OK;
  if (!w || !q || !scale_factor_dev) return CATCHQ_ERR_ARG;
  hipStream_t s = as_stream(stream);
  const int g = grid_for(total, kThreads * 4);
  if (w_dtype == CATCHQ_F32) {
    if (bitwidth == 8) quantize_per_channel_kernel<float, 8><<<g, kThreads, 0, s>>>((const float *)w, (int8_t *)q, total, inner, scale_factor_dev);
    else quantize_per_channel_kernel<float, 16><<<g, kThreads, 0, s>>>((const float *)w, (int16_t *)q, total, inner, scale_factor_dev);
  } else {
    if (bitwidth == 8) quantize_per_channel_kernel<__half, 8><<<g, kThreads, 0, s>>>((const __half *)w, (int8_t *)q, total, inner, scale_factor_dev);
    else quantize_per_channel_kernel<__half, 16><<<g, kThreads, 0, s>>>((const __half *)w, (int16_t *)q, total, inner, scale_factor_dev);
  }
  return launch_status();
}

CATCHQ_API int catchq_quantize_per_channel_f16(const void *w, void *q, int bitwidth, int co, int64_t inner,
                                               const void *scale_factor_dev, catchq_stream_t stream) {
  if (co < 0 || inner < 0) return CATCHQ_ERR_SHAPE;
  if (bitwidth != 8 && bitwidth != 16) return CATCHQ_ERR_BITWIDTH;
  const int64_t total = (int64_t)co * inner;
  if (total == 0) return CATCHQ_OK;
  if (!w || !q || !scale_factor_dev) return CATCHQ_ERR_ARG;
  hipStream_t s = as_stream(stream);
  const int g = grid_for(total, kThreads * 4);
  if (bitwidth == 8)
    quantize_per_channel_f16_kernel<8><<<g, kThreads, 0, s>>>((const __half *)w, (int8_t *)q, total, inner,
                                                              (const __half *)scale_factor_dev);
  else
    quantize_per_channel_f16_kernel<16><<<g, kThreads, 0, s>>>((const __half *)w, (int16_t *)q, total, inner,
                                                               (const __half *)scale_factor_dev);
  return launch_status();
}

CATCHQ_API int catchq_dequantize(const void *q, int bits, void *y, int y_dtype, int64_t n, int position,
                                 float scale, catchq_stream_t stream) {
  if (n < 0) return CATCHQ_ERR_ARG;
  if (bits != 8 && bits != 16 && bits != 32) return CATCHQ_ERR_BITWIDTH;
  if (y_dtype != CATCHQ_F32 && y_dtype != CATCHQ_F16) return CATCHQ_ERR_DTYPE;
  if (position < -126 || position > 126) return CATCHQ_ERR_ARG;
  if (n == 0) return CATCHQ_OK;
  if (!q || !y) return CATCHQ_ERR_ARG;
  hipStream_t s = as_stream(stream);
  const int g = grid_for(n, kThreads * 4);
#define CATCHQ_DQ(TQ, TO) dequantize_kernel<TQ, TO><<<g, kThreads, 0, s>>>((const TQ *)q, (TO *)y, n, position, scale)
  if (y_dtype == CATCHQ_F32) {
    if (bits == 8) CATCHQ_DQ(int8_t, float);
    else if (bits == 16) CATCHQ_DQ(int16_t, float);
    else CATCHQ_DQ(int32_t, float);
  } else {
    if (bits == 8) CATCHQ_DQ(int8_t, __half);
    else if (bits == 16) CATCHQ_DQ(int16_t, __half);
    else CATCHQ_DQ(int32_t, __half);
  }
#undef CATCHQ_DQ
  return launch_status();
}
