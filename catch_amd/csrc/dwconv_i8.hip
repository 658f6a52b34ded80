// Depthwise int8 convolution (groups == Ci == Co) on NHWC tensors: a stencil, not a contraction,
// so no matrix cores.  A block owns a strip of output pixels of one image row and all channels of a
// 64-channel slab; the input rows the strip needs are staged in LDS once and every tap is read
// from there, the filter taps of the slab sit in LDS transposed to [tap][channel].
#include "catchq_common.h"

namespace catchq {

struct DwParams {
  int N, H, W, C, kh, kw, ph, pw, sh, sw, dh, dw, Ho, Wo;
  int strips;  // strips per output row
  int slabs;   // channel slabs
};

constexpr int DW_TW = 16;      // output pixels per strip
constexpr int DW_CS = 64;      // channels per slab
constexpr int DW_MAXTAPS = 25;  // up to 5x5
constexpr int DW_LDS_BYTES = 32 * 1024;

// threads: 256 = 16 channel-quads (x4 channels) x 16 pixels
__global__ __launch_bounds__(256) void dwconv_i8_kernel(const int8_t *__restrict__ x,
                                                       const int8_t *__restrict__ w, DwParams p, EpiDev e) {
  __shared__ __attribute__((aligned(16))) int8_t tile[DW_LDS_BYTES];
  __shared__ __attribute__((aligned(16))) int8_t wt[DW_MAXTAPS * DW_CS];

  int b = blockIdx.x;
  const int slab = b % p.slabs;
  b /= p.slabs;
  const int strip = b % p.strips;
  b /= p.strips;
  const int ho = b % p.Ho;
  const int img = b / p.Ho;

  const int c0 = slab * DW_CS;
  const int cs = min(DW_CS, p.C - c0);  // multiple of 4
  const int wo0 = strip * DW_TW;
  const int taps = p.kh * p.kw;

  // input window of the strip
  const int in_w = (DW_TW - 1) * p.sw + (p.kw - 1) * p.dw + 1;
  const int wi0 = wo0 * p.sw - p.pw;
  const int hi0 = ho * p.sh - p.ph;

  // filter slab -> LDS [tap][channel]
  for (int i = threadIdx.x; i < taps * DW_CS; i += 256) {
    const int t = i / DW_CS, c = i % DW_CS;
    wt[i] = (c < cs) ? w[(int64_t)(c0 + c) * taps + t] : (int8_t)0;
  }
  // input rows -> LDS [r][col][channel] as dwords (4 channels), zero outside the image
  const int quads = DW_CS / 4;
  const int total = p.kh * in_w * quads;
  int *tile32 = reinterpret_cast<int *>(tile);
  for (int i = threadIdx.x; i < total; i += 256) {
    const int cq = i % quads;
    const int col = (i / quads) % in_w;
    const int r = i / (quads * in_w);
    const int hi = hi0 + r * p.dh, wi = wi0 + col;
    int v = 0;
    if (cq * 4 < cs && (unsigned)hi < (unsigned)p.H && (unsigned)wi < (unsigned)p.W)
      v = *reinterpret_cast<const int *>(x + (((int64_t)img * p.H + hi) * p.W + wi) * p.C + c0 + cq * 4);
    tile32[i] = v;
  }
  __syncthreads();

  const int cq = threadIdx.x & 15;
  const int px = threadIdx.x >> 4;
  const int wo = wo0 + px;
  if (cq * 4 >= cs || wo >= p.Wo) return;

  int acc[4] = {0, 0, 0, 0};
  for (int r = 0; r < p.kh; ++r) {
    for (int q = 0; q < p.kw; ++q) {
      const int col = px * p.sw + q * p.dw;
      const int xv = tile32[(r * in_w + col) * quads + cq];
      const int wv = *reinterpret_cast<const int *>(wt + (r * p.kw + q) * DW_CS + cq * 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] += (int)(int8_t)(xv >> (8 * j)) * (int)(int8_t)(wv >> (8 * j));
    }
  }
  const int64_t pix = ((int64_t)img * p.Ho + ho) * p.Wo + wo;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = c0 + cq * 4 + j;
    const int64_t idx = pix * p.C + c;
    if (e.acc_out) e.acc_out[idx] = acc[j];
    epi_store(epi_value((float)acc[j], idx, c, e), idx, e);
  }
}

bool dwconv_i8_supported(int C, int kh, int kw, int sw, int dw) {
  if (C % 4 != 0 || kh * kw > DW_MAXTAPS) return false;
  const int in_w = (DW_TW - 1) * sw + (kw - 1) * dw + 1;
  return (int64_t)kh * in_w * DW_CS <= DW_LDS_BYTES;
}

int dwconv_i8(const void *x, const void *w, int N, int H, int W, int C, int kh, int kw, int ph, int pw, int sh,
              int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  DwParams p = {N, H, W, C, kh, kw, ph, pw, sh, sw, dh, dw, Ho, Wo, 0, 0};
  p.strips = (Wo + DW_TW - 1) / DW_TW;
  p.slabs = (C + DW_CS - 1) / DW_CS;
  const int64_t nb = (int64_t)N * Ho * p.strips * p.slabs;
  if (nb > 0x7fffffff) return CATCHQ_ERR_SHAPE;
  dwconv_i8_kernel<<<(int)nb, 256, 0, s>>>((const int8_t *)x, (const int8_t *)w, p, e);
  return launch_status();
}

}  // namespace catchq
