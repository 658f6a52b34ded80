// Pooling on NHWC tensors for pipelines that keep activations quantized between layers.
//   max pooling (int8 / int16 / fp32): quantization is monotonic, so pooling the integers equals
//     quantizing the pooled floats;
//   global average pooling (fp32): sequential sum over (h, w) in that order, then one division --
//     a fixed order, so the result is reproducible bit for bit.
#include "catchq_common.h"

namespace catchq {

template <typename T>
struct Lowest;
template <>
struct Lowest<int8_t> {
  static __device__ int8_t value() { return -128; }
};
template <>
struct Lowest<int16_t> {
  static __device__ int16_t value() { return -32768; }
};
template <>
struct Lowest<float> {
  static __device__ float value() { return -__builtin_inff(); }
};

// one thread = one output pixel x VEC consecutive channels (VEC * sizeof(T) = 16 bytes, or VEC = 1).
// K > 0: the window size is known, every load of the window is requested before the first comparison
// (taps outside the image read the centre tap again, which is always inside and changes nothing);
// K = 0: any window, tap by tap.
template <typename T, int VEC, int K>
__global__ __launch_bounds__(256) void maxpool_nhwc_kernel(const T *__restrict__ x, T *__restrict__ y, int N, int H,
                                                          int W, int C, int k, int stride, int pad, int Ho,
                                                          int Wo) {
  const int cv = C / VEC;
  const int64_t total = (int64_t)N * Ho * Wo * cv;
  const int64_t step = (int64_t)gridDim.x * blockDim.x;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += step) {
    const int c = (int)(idx % cv) * VEC;
    int64_t p = idx / cv;
    const int wo = (int)(p % Wo);
    p /= Wo;
    const int ho = (int)(p % Ho);
    const int n = (int)(p / Ho);
    T m[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) m[j] = Lowest<T>::value();
    const T *img = x + (int64_t)n * H * W * C + c;
    if constexpr (K > 0) {
      // a window of K x K with pad <= K/2 always contains the pixel (ho*stride, wo*stride) clamped into the image
      const int hc = min(ho * stride, H - 1), wc = min(wo * stride, W - 1);
      v4i raw[K * K];
      T one[K * K];
#pragma unroll
      for (int r = 0; r < K; ++r)
#pragma unroll
        for (int q = 0; q < K; ++q) {
          int hi = ho * stride - pad + r, wi = wo * stride - pad + q;
          const bool in = (unsigned)hi < (unsigned)H && (unsigned)wi < (unsigned)W;
          hi = in ? hi : hc;
          wi = in ? wi : wc;
          const T *src = img + ((int64_t)hi * W + wi) * C;
          if constexpr (VEC == 1) one[r * K + q] = src[0];
          else raw[r * K + q] = *reinterpret_cast<const v4i *>(src);
        }
      if constexpr (VEC == 16) {
        // sixteen int8 per tap, four to a dword: flipping the sign bits turns the signed order into the unsigned
        // one, and the even / odd bytes of a dword, each alone in a 16-bit half, compare as 16-bit unsigned
        // numbers -- two packed 16-bit maxima per dword instead of four extract-and-compare pairs
        typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
        u16x2 even[4], odd[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) even[d] = odd[d] = u16x2{0, 0};
#pragma unroll
        for (int t = 0; t < K * K; ++t)
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const unsigned u = (unsigned)raw[t][d] ^ 0x80808080u;
            even[d] = __builtin_elementwise_max(even[d], __builtin_bit_cast(u16x2, u & 0x00ff00ffu));
            odd[d] = __builtin_elementwise_max(odd[d], __builtin_bit_cast(u16x2, u & 0xff00ff00u));
          }
        v4i packed;
#pragma unroll
        for (int d = 0; d < 4; ++d)
          packed[d] = (int)((__builtin_bit_cast(unsigned, even[d]) | __builtin_bit_cast(unsigned, odd[d])) ^ 0x80808080u);
        *reinterpret_cast<v4i *>(m) = packed;
      } else
#pragma unroll
      for (int t = 0; t < K * K; ++t) {
        if constexpr (VEC == 1) m[0] = (one[t] > m[0]) ? one[t] : m[0];
        else {
          T v[VEC];
          *reinterpret_cast<v4i *>(v) = raw[t];
#pragma unroll
          for (int j = 0; j < VEC; ++j) m[j] = (v[j] > m[j]) ? v[j] : m[j];
        }
      }
    } else {
      for (int r = 0; r < k; ++r) {
        const int hi = ho * stride - pad + r;
        if ((unsigned)hi >= (unsigned)H) continue;
        for (int q = 0; q < k; ++q) {
          const int wi = wo * stride - pad + q;
          if ((unsigned)wi >= (unsigned)W) continue;
          const T *src = img + ((int64_t)hi * W + wi) * C;
          T v[VEC];
          if constexpr (VEC == 1) v[0] = src[0];
          else *reinterpret_cast<v4i *>(v) = *reinterpret_cast<const v4i *>(src);
#pragma unroll
          for (int j = 0; j < VEC; ++j) m[j] = (v[j] > m[j]) ? v[j] : m[j];
        }
      }
    }
    T *dst = y + (((int64_t)n * Ho + ho) * Wo + wo) * C + c;
    if constexpr (VEC == 1) dst[0] = m[0];
    else *reinterpret_cast<v4i *>(dst) = *reinterpret_cast<v4i *>(m);
  }
}

template <typename T>
static int launch_maxpool(const void *x, void *y, int N, int H, int W, int C, int k, int stride, int pad, int Ho,
                          int Wo, hipStream_t s) {
  constexpr int VEC = 16 / sizeof(T);
  const bool vec = (C % VEC == 0) && aligned16(x) && aligned16(y);
  const int64_t total = (int64_t)N * Ho * Wo * (vec ? C / VEC : C);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (blocks < 1) blocks = 1;
#define CATCHQ_POOL(V, K) \
  maxpool_nhwc_kernel<T, V, K><<<(int)blocks, 256, 0, s>>>((const T *)x, (T *)y, N, H, W, C, k, stride, pad, Ho, Wo)
  // the unrolled windows rely on the clamped corner pixel lying inside the window: pad <= k/2 and a window
  // that starts inside the image
  const bool corner_ok = 2 * pad <= k && (int64_t)(Ho - 1) * stride - pad < H && (int64_t)(Wo - 1) * stride - pad < W;
  if (vec && k == 3 && corner_ok) CATCHQ_POOL(VEC, 3);
  else if (vec && k == 2 && corner_ok) CATCHQ_POOL(VEC, 2);
  else if (vec) CATCHQ_POOL(VEC, 0);
  else CATCHQ_POOL(1, 0);
#undef CATCHQ_POOL
  return launch_status();
}

// QBW = 0: the fp32 mean; 8 / 16: the mean quantized at (position, scale)
template <int QBW>
__global__ __launch_bounds__(256) void global_avgpool_nhwc_kernel(const float *__restrict__ x, void *__restrict__ yv,
                                                                 int N, int HW, int C, int neg_pos, float scale) {
  const int64_t total = (int64_t)N * C;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(idx % C);
    const int64_t n = idx / C;
    const float *src = x + n * HW * C + c;
    // the sum runs over the pixels in order (one fp32 addition each: the order is part of the result);
    // 25 loads are requested before their additions (a 7x7 map is two such batches): with one wave per SIMD the
    // kernel's time is the number of memory round trips a thread makes
    float s = 0.0f;
    int p = 0;
    constexpr int U = 25;
    for (; p + U <= HW; p += U) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = src[(int64_t)(p + u) * C];
#pragma unroll
      for (int u = 0; u < U; ++u) s = s + v[u];
    }
    for (; p < HW; ++p) s = s + src[(int64_t)p * C];
    const float mean = s / (float)HW;
    if constexpr (QBW == 0) reinterpret_cast<float *>(yv)[idx] = mean;
    else if constexpr (QBW == 8) reinterpret_cast<int8_t *>(yv)[idx] = (int8_t)quant1<8>(mean, scale, neg_pos);
    else reinterpret_cast<int16_t *>(yv)[idx] = (int16_t)quant1<16>(mean, scale, neg_pos);
  }
}

}  // namespace catchq

using namespace catchq;

CATCHQ_API int catchq_maxpool_nhwc(const void *x, void *y, int elem_bits, int n, int h, int w, int c, int k,
                                   int stride, int pad, catchq_stream_t stream) {
  if (n < 0 || h <= 0 || w <= 0 || c <= 0 || k <= 0 || stride <= 0 || pad < 0 || 2 * pad > k) return CATCHQ_ERR_SHAPE;
  const int ho = (h + 2 * pad - k) / stride + 1, wo = (w + 2 * pad - k) / stride + 1;
  if (ho <= 0 || wo <= 0) return CATCHQ_ERR_SHAPE;
  if (n == 0) return CATCHQ_OK;
  if (!x || !y) return CATCHQ_ERR_ARG;
  hipStream_t s = as_stream(stream);
  switch (elem_bits) {
    case 8: return launch_maxpool<int8_t>(x, y, n, h, w, c, k, stride, pad, ho, wo, s);
    case 16: return launch_maxpool<int16_t>(x, y, n, h, w, c, k, stride, pad, ho, wo, s);
    case 32: return launch_maxpool<float>(x, y, n, h, w, c, k, stride, pad, ho, wo, s);
    default: return CATCHQ_ERR_BITWIDTH;
  }
}

CATCHQ_API int catchq_global_avgpool_nhwc(const float *x, float *y, int n, int hw, int c, catchq_stream_t stream) {
  if (n < 0 || hw <= 0 || c <= 0) return CATCHQ_ERR_SHAPE;
  if (n == 0) return CATCHQ_OK;
  if (!x || !y) return CATCHQ_ERR_ARG;
  const int64_t total = (int64_t)n * c;
  int blocks = (int)((total + 255) / 256);
  if (blocks > 65536) blocks = 65536;
  global_avgpool_nhwc_kernel<0><<<blocks, 256, 0, as_stream(stream)>>>(x, y, n, hw, c, 0, 1.0f);
  return launch_status();
}

CATCHQ_API int catchq_global_avgpool_quantize_nhwc(const float *x, void *q, int bitwidth, int n, int hw, int c,
                                                   int position, float scale, catchq_stream_t stream) {
  if (n < 0 || hw <= 0 || c <= 0) return CATCHQ_ERR_SHAPE;
  if (bitwidth != 8 && bitwidth != 16) return CATCHQ_ERR_BITWIDTH;
  if (position < -126 || position > 126) return CATCHQ_ERR_ARG;
  if (n == 0) return CATCHQ_OK;
  if (!x || !q) return CATCHQ_ERR_ARG;
  const int64_t total = (int64_t)n * c;
  int blocks = (int)((total + 255) / 256);
  if (blocks > 65536) blocks = 65536;
  if (bitwidth == 8) global_avgpool_nhwc_kernel<8><<<blocks, 256, 0, as_stream(stream)>>>(x, q, n, hw, c, -position, scale);
  else global_avgpool_nhwc_kernel<16><<<blocks, 256, 0, as_stream(stream)>>>(x, q, n, hw, c, -position, scale);
  return launch_status();
}
