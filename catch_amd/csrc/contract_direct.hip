// Direct (one thread per output) integer GEMM / convolution: the route for every shape and
// bit-width combination that the MFMA and stencil kernels do not take (odd channel counts,
// grouped non-depthwise layers, int16 x int16).  Correctness path, not a fast path.
#include "catchq_common.h"

namespace catchq {

template <int BITS>
struct IntOf;
template <>
struct IntOf<8> {
  typedef int8_t type;
};
template <>
struct IntOf<16> {
  typedef int16_t type;
};

// int16 x int16 sums do not fit int32 for realistic K: accumulate those in int64.
template <int AB, int BB>
struct AccOf {
  typedef int32_t type;
};
template <>
struct AccOf<16, 16> {
  typedef int64_t type;
};

template <int AB, int BB>
__global__ __launch_bounds__(256) void gemm_nt_direct_kernel(const typename IntOf<AB>::type *__restrict__ a,
                                                            const typename IntOf<BB>::type *__restrict__ b,
                                                            int64_t M, int64_t N, int64_t K, EpiDev e) {
  resolve_exp2(e);
  typedef typename AccOf<AB, BB>::type TAcc;
  const int64_t total = M * N;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const int64_t m = idx / N, n = idx - m * N;
    const typename IntOf<AB>::type *ar = a + m * K;
    const typename IntOf<BB>::type *br = b + n * K;
    TAcc s = 0;
    for (int64_t k = 0; k < K; ++k) s += (TAcc)ar[k] * (TAcc)br[k];
    if constexpr (sizeof(TAcc) == 4) {
      if (e.acc_out) e.acc_out[idx] = s;
    }
    epi_store(epi_value((float)s, idx, (int)n, e), idx, e);
  }
}

template <int AB, int BB>
__global__ __launch_bounds__(256) void conv2d_direct_kernel(const typename IntOf<AB>::type *__restrict__ x,
                                                           const typename IntOf<BB>::type *__restrict__ w,
                                                           ConvDev d, EpiDev e) {
  resolve_exp2(e);
  typedef typename AccOf<AB, BB>::type TAcc;
  const int cig = d.Ci / d.groups, cog = d.Co / d.groups;
  const int64_t total = (int64_t)d.N * d.Ho * d.Wo * d.Co;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const int co = (int)(idx % d.Co);
    int64_t p = idx / d.Co;
    const int wo = (int)(p % d.Wo);
    p /= d.Wo;
    const int ho = (int)(p % d.Ho);
    const int n = (int)(p / d.Ho);
    const int g = co / cog;
    TAcc s = 0;
    for (int r = 0; r < d.kh; ++r) {
      const int hi = ho * d.sh - d.ph + r * d.dh;
      if (hi < 0 || hi >= d.H) continue;
      for (int q = 0; q < d.kw; ++q) {
        const int wi = wo * d.sw - d.pw + q * d.dw;
        if (wi < 0 || wi >= d.W) continue;
        const typename IntOf<AB>::type *xp = x + (((int64_t)n * d.H + hi) * d.W + wi) * d.Ci + (int64_t)g * cig;
        const typename IntOf<BB>::type *wp = w + (((int64_t)co * d.kh + r) * d.kw + q) * cig;
        for (int c = 0; c < cig; ++c) s += (TAcc)xp[c] * (TAcc)wp[c];
      }
    }
    if constexpr (sizeof(TAcc) == 4) {
      if (e.acc_out) e.acc_out[idx] = s;
    }
    epi_store(epi_value((float)s, idx, co, e), idx, e);
  }
}

static inline int direct_grid(int64_t total) {
  int64_t b = (total + 255) / 256;
  if (b > 65536) b = 65536;
  if (b < 1) b = 1;
  return (int)b;
}

int gemm_nt_direct(const void *a, int a_bits, const void *b, int b_bits, int64_t M, int64_t N, int64_t K,
                   const EpiDev &e, hipStream_t s) {
  const int g = direct_grid(M * N);
  if (a_bits == 8 && b_bits == 8)
    gemm_nt_direct_kernel<8, 8><<<g, 256, 0, s>>>((const int8_t *)a, (const int8_t *)b, M, N, K, e);
  else if (a_bits == 16 && b_bits == 8)
    gemm_nt_direct_kernel<16, 8><<<g, 256, 0, s>>>((const int16_t *)a, (const int8_t *)b, M, N, K, e);
  else if (a_bits == 16 && b_bits == 16) {
    if (e.acc_out) return CATCHQ_ERR_UNSUPPORTED;
    gemm_nt_direct_kernel<16, 16><<<g, 256, 0, s>>>((const int16_t *)a, (const int16_t *)b, M, N, K, e);
  } else
    return CATCHQ_ERR_BITWIDTH;
  return launch_status();
}

int conv2d_direct(const void *x, int x_bits, const void *w, int w_bits, const ConvDev &d, const EpiDev &e,
                  hipStream_t s) {
  const int g = direct_grid((int64_t)d.N * d.Ho * d.Wo * d.Co);
  if (x_bits == 8 && w_bits == 8)
    conv2d_direct_kernel<8, 8><<<g, 256, 0, s>>>((const int8_t *)x, (const int8_t *)w, d, e);
  else if (x_bits == 16 && w_bits == 8)
    conv2d_direct_kernel<16, 8><<<g, 256, 0, s>>>((const int16_t *)x, (const int8_t *)w, d, e);
  else if (x_bits == 16 && w_bits == 16) {
    if (e.acc_out) return CATCHQ_ERR_UNSUPPORTED;
    conv2d_direct_kernel<16, 16><<<g, 256, 0, s>>>((const int16_t *)x, (const int16_t *)w, d, e);
  } else
    return CATCHQ_ERR_BITWIDTH;
  return launch_status();
}

}  // namespace catchq
