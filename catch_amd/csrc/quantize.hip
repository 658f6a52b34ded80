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

// The frame kernel for the usual network input: fp32 planes of a width that is a multiple of 4, int8 output with
// 4 channels per pixel.  A lane owns 4 consecutive image pixels of one output row: one 16-byte load per channel
// plane, one 16-byte store (4 pixels x 4 channels; the frame shifts it off 16-byte alignment, 4-byte alignment is
// what the store needs); the lanes behind the image's groups write the row's border pixels, one each.  A wave
// takes ROWS output rows at once, all their loads requested before the first conversion.
struct __attribute__((aligned(4))) frame_px4 { int v[4]; };
template <int ROWS>
__global__ __launch_bounds__(kThreads) void quantize_frame_f32_i8c4_kernel(const float *__restrict__ x, int8_t *__restrict__ q,
                                                                          int n, int c, int h, int w, int oh, int ow,
                                                                          int top, int left, int pos, float scale) {
  const int64_t hw = (int64_t)h * w, rows = (int64_t)n * oh;
  const int groups = w >> 2, border = ow - w, per_row = groups + border;
  const int lane = threadIdx.x & 63;
  const int64_t wave0 = ((int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6)) * ROWS;
  const int64_t wstride = (int64_t)gridDim.x * (kThreads / 64) * ROWS;
  for (int64_t row0 = wave0; row0 < rows; row0 += wstride) {
    for (int t = lane; t < per_row; t += 64) {
      v4f v[ROWS][3];
      bool inside[ROWS];
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int64_t row = row0 + r;
        const int64_t img = row / oh;
        const int iy = (int)(row - img * oh) - top;
        inside[r] = row < rows && (unsigned)iy < (unsigned)h && t < groups;
#pragma unroll
        for (int ch = 0; ch < 3; ++ch) {
          v[r][ch] = v4f{0.f, 0.f, 0.f, 0.f};
          if (inside[r] && ch < c)
            v[r][ch] = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(x + (img * c + ch) * hw + (int64_t)iy * w) + t);
        }
      }
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int64_t row = row0 + r;
        if (row >= rows) break;
        int8_t *dst = q + row * ow * 4;
        if (t < groups) {
          frame_px4 o;
#pragma unroll
          for (int px = 0; px < 4; ++px) {
            unsigned b = 0;
#pragma unroll
            for (int ch = 0; ch < 3; ++ch) b |= ((unsigned)quant1<8>(v[r][ch][px], scale, -pos) & 0xffu) << (8 * ch);  // 0 -> 0
            o.v[px] = (int)b;
          }
          // a row outside the image: inside[r] is false, every value above is the quantized zero
          *reinterpret_cast<frame_px4 *>(dst + (left + 4 * t) * 4) = o;
        } else {
          const int bpx = t - groups;  // border pixels: the `left` ones in front of the image, then the ones behind it
          const int ox = bpx < left ? bpx : w + bpx;
          *reinterpret_cast<int *>(dst + ox * 4) = 0;
        }
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
// one value: exact scaling by the power of two, then the division (DIV 0: scale == 1, no division; 1: the
// reciprocal form, bit for bit the IEEE quotient under the conditions div_by_rcp states; 2: true division)
template <int DIV>
__device__ __forceinline__ float dequant1(float qf, int pos, float scale, float rcp) {
  const float t = __builtin_ldexpf(qf, pos);
  if constexpr (DIV == 0) return t;
  else if constexpr (DIV == 1) {
    float v = div_by_rcp(t, scale, rcp);
    // the fp32 quotient exists as a value of its own: a conversion to fp16 behind it must round that value, not be
    // merged with the last fused multiply-add into one mixed-precision operation that rounds once
    asm volatile("" : "+v"(v));
    return v;
  } else return t / scale;
}

// Scalar body: any alignment, any n.
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

// Vector body: a lane owns E consecutive elements per step, E chosen so that its store is 16 bytes (4 fp32 or
// 8 fp16 values); its load is then E * sizeof(TQ) bytes (4 .. 32).  Lanes are contiguous, so every load and store
// instruction of a wave covers one contiguous run of memory.  UNROLL steps (a grid stride apart) are requested
// before the first conversion.  NT bit 0: non-temporal loads (nothing is read twice), bit 1: non-temporal stores;
// measured on 51 M int8 -> fp32 elements with cold inputs: plain stores 5.5 TB/s, non-temporal stores 5.1 TB/s
// (the loads' hint makes no difference), and a grid of up to 2 * kMaxBlocks blocks 5.8 TB/s.
template <typename TQ, typename TOut, int DIV, int NT = 1>
__global__ __launch_bounds__(kThreads) void dequantize_vec_kernel(const TQ *__restrict__ q, TOut *__restrict__ y,
                                                                 int64_t n, int pos, float scale, float rcp) {
  constexpr int E = 16 / sizeof(TOut);
  constexpr int IN_BYTES = E * sizeof(TQ);
  constexpr int IN_DW = IN_BYTES / 4;
  constexpr int UNROLL = 4;
  const int64_t nvec = n / E;
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  const int64_t first = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  for (int64_t i0 = first; i0 < nvec; i0 += stride * UNROLL) {
    // the lane's input of one step as 16-byte registers (the last one partly used when the input is 4 or 8 bytes)
    constexpr int NV = (IN_DW + 3) / 4;
    v4i raw[UNROLL][NV];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t i = i0 + u * stride;
      if (i >= nvec) break;
      const int *src = reinterpret_cast<const int *>(q) + i * IN_DW;
      if constexpr (IN_DW == 1) {
        raw[u][0] = v4i{(NT & 1 ? __builtin_nontemporal_load(src) : *src), 0, 0, 0};
      } else if constexpr (IN_DW == 2) {
        const v2i t = (NT & 1 ? __builtin_nontemporal_load(reinterpret_cast<const v2i *>(src)) : *reinterpret_cast<const v2i *>(src));
        raw[u][0] = v4i{t[0], t[1], 0, 0};
      } else {
#pragma unroll
        for (int d = 0; d < NV; ++d) raw[u][d] = NT & 1 ? __builtin_nontemporal_load(reinterpret_cast<const v4i *>(src) + d) : reinterpret_cast<const v4i *>(src)[d];
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int64_t i = i0 + u * stride;
      if (i >= nvec) break;
      float v[E];
#pragma unroll
      for (int k = 0; k < E; ++k) {
        int iv;
        if constexpr (sizeof(TQ) == 1) iv = (int)(int8_t)((unsigned)raw[u][k / 16][(k / 4) % 4] >> (8 * (k % 4)));
        else if constexpr (sizeof(TQ) == 2) iv = (int)(int16_t)((unsigned)raw[u][k / 8][(k / 2) % 4] >> (16 * (k % 2)));
        else iv = raw[u][k / 4][k % 4];
        v[k] = dequant1<DIV>((float)iv, pos, scale, rcp);
      }
      v4i out;
      if constexpr (sizeof(TOut) == 4) {
#pragma unroll
        for (int k = 0; k < 4; ++k) out[k] = __float_as_int(v[k]);
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const __half2 h = __halves2half2(__float2half_rn(v[2 * k]), __float2half_rn(v[2 * k + 1]));
          int bits;
          __builtin_memcpy(&bits, &h, 4);
          out[k] = bits;
        }
      }
      if (NT & 2) __builtin_nontemporal_store(out, reinterpret_cast<v4i *>(y) + i);
      else reinterpret_cast<v4i *>(y)[i] = out;
    }
  }
  // tail (< E elements) by the first lanes of block 0
  if (blockIdx.x == 0 && threadIdx.x < (int)(n - nvec * E)) {
    const int64_t i = nvec * E + threadIdx.x;
    const float t = dequant1<DIV>((float)q[i], pos, scale, rcp);
    if constexpr (sizeof(TOut) == 2) y[i] = __float2half_rn(t);
    else y[i] = t;
  }
}

template <typename TQ, typename TOut>
static int launch_dequantize(const void *q, void *y, int64_t n, int pos, float scale, hipStream_t s) {
  constexpr int E = 16 / sizeof(TOut);
  if (!aligned16(q) || !aligned16(y)) {
    dequantize_kernel<TQ, TOut><<<grid_for(n, kThreads * 4), kThreads, 0, s>>>((const TQ *)q, (TOut *)y, n, pos, scale);
    return launch_status();
  }
  const int64_t want_blocks = (n / E + kThreads * 4 - 1) / (kThreads * 4);
  const int g = (int)(want_blocks < 1 ? 1 : (want_blocks > 2 * kMaxBlocks ? 2 * kMaxBlocks : want_blocks));
  // the reciprocal form needs the correctly rounded reciprocal (IEEE division on the host gives it), a divisor whose
  // significand is not all ones, and no under- or overflow on the way: |q * 2^pos| <= 2^31 * 2^pos, so positions and
  // scales of moderate exponent qualify; everything else divides
  uint32_t sb;
  __builtin_memcpy(&sb, &scale, 4);
  const int se = (int)((sb >> 23) & 0xff) - 127;
  const bool rcp_ok = (sb & 0x7fffffu) != 0x7fffffu && se >= -30 && se <= 30 && pos >= -60 && pos <= 30 && scale > 0.0f;
  const float rcp = rcp_ok ? 1.0f / scale : 0.0f;
  if (scale == 1.0f)
    dequantize_vec_kernel<TQ, TOut, 0><<<g, kThreads, 0, s>>>((const TQ *)q, (TOut *)y, n, pos, scale, rcp);
  else if (rcp_ok)
    dequantize_vec_kernel<TQ, TOut, 1><<<g, kThreads, 0, s>>>((const TQ *)q, (TOut *)y, n, pos, scale, rcp);
  else
    dequantize_vec_kernel<TQ, TOut, 2><<<g, kThreads, 0, s>>>((const TQ *)q, (TOut *)y, n, pos, scale, rcp);
  return launch_status();
}

// ---- max-abs reduction + position/scale finalize ---------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

template <typename TIn, int UNROLL = 4>
__global__ __launch_bounds__(kThreads) void absmax_partial_kernel(const TIn *__restrict__ x, int64_t n,
                                                                 float *__restrict__ partial, int vec_ok) {
  constexpr int VEC = 16 / sizeof(TIn);
  float m = 0.0f;  // fmaxf ignores NaN operands, like the oracle's comparison
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  int64_t done = 0;
  if (vec_ok) {
    // UNROLL 16-byte loads (a grid stride apart) in flight per lane; the data is read once: non-temporal
    const int64_t nvec = n / VEC;
    for (int64_t i0 = (int64_t)blockIdx.x * kThreads + threadIdx.x; i0 < nvec; i0 += stride * UNROLL) {
      v4i raw[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int64_t i = i0 + u * stride;
        raw[u] = v4i{0, 0, 0, 0};  // |+0| never wins
        if (i < nvec) raw[u] = __builtin_nontemporal_load(reinterpret_cast<const v4i *>(x) + i);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if constexpr (sizeof(TIn) == 4) {
#pragma unroll
          for (int j = 0; j < 4; ++j) m = fmaxf(m, fabsf(__int_as_float(raw[u][j])));
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const __half2 h = as_half2(raw[u][j]);
            m = fmaxf(m, fmaxf(fabsf(__low2float(h)), fabsf(__high2float(h))));
          }
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
  if constexpr (sizeof(TIn) == 4 && BW == 8 && CPAD == 4) {
    if (w % 4 == 0 && c <= 3 && aligned16(x)) {
      constexpr int ROWS = 2;  // (1 and 2 rows per wave measure the same, 4 is slower)
      const int64_t waves = (rows + ROWS - 1) / ROWS;
      const int64_t blocks = (waves + kThreads / 64 - 1) / (kThreads / 64);
      quantize_frame_f32_i8c4_kernel<ROWS><<<(unsigned)(blocks < 65535 * 16 ? blocks : 65535 * 16), kThreads, 0, s>>>(
          (const float *)x, (int8_t *)q, n, c, h, w, oh, ow, top, left, pos, scale);
      return launch_status();
    }
  }
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

// blocks of the max-abs reduction: at most two per compute unit, each lane with four 16-byte loads in flight
// (measured on 51 M fp32 elements, cold: 512 blocks 5.6 TB/s, 1024 blocks 5.05, 4096 blocks 4.6)
static int absmax_blocks(int64_t n) {
  const int b = grid_for(n / 4, kThreads * 4);
  return b < 512 ? b : 512;
}

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
#define CATCHQ_DQ(TQ, TO) return launch_dequantize<TQ, TO>(q, y, n, position, scale, s)
  if (y_dtype == CATCHQ_F32) {
    if (bits == 8) CATCHQ_DQ(int8_t, float);
    if (bits == 16) CATCHQ_DQ(int16_t, float);
    CATCHQ_DQ(int32_t, float);
  }
  if (bits == 8) CATCHQ_DQ(int8_t, __half);
  if (bits == 16) CATCHQ_DQ(int16_t, __half);
  CATCHQ_DQ(int32_t, __half);
#undef CATCHQ_DQ
}
