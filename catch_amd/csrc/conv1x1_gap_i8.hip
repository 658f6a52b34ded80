// The last 1x1 convolution of an image classifier and the global average pooling behind it in one launch.
//
// Run layer by layer the convolution writes its fp32 output (ResNet-50: 7 x 7 x 2048 floats per image, the largest
// tensor of the last stage) and the pooling reads it back to keep one value per channel -- two launches whose time
// is their start-up and the round trip of that tensor.  Here a block owns one image and 32 channels per wave:
//
//   1  the image's pixels (at most 64, int8) are copied to LDS once per block;
//   2  every wave multiplies on the matrix cores with the operands swapped (filters as A, straight from global
//      memory through a ring of registers, pixels as B from LDS), so that a lane ends up with four consecutive
//      channels of one pixel, and applies the convolution's epilogue (reciprocal-form division, bias, optional fp32
//      residual, activation) -- the arithmetic of the stand-alone launch, value for value;
//   3  the fp32 values go to a tile in LDS, and one lane per channel adds the pixels up in storage order, one fp32
//      addition each, divides once by the pixel count and stores the mean and / or its quantized form -- the
//      arithmetic of the stand-alone pooling kernel.
//
// The convolution's output never reaches memory; mean and quantized mean are those of the two launches bit for bit.
#include "igemm_common.h"

namespace catchq {

struct GapConvDev {
  const float *div, *rcp, *bias, *resid;
  int exp2, act;
  float *mean;  // [N, Co] or null
  void *q;      // [N, Co] int8 / int16 or null
  int q_bw, q_neg_pos;
  float q_scale;
};

struct GapConvParams {
  int N, HW, K, Co;
  int xs;      // bytes of a pixel row in LDS
  int groups;  // 32-pixel groups: 1 or 2
};

constexpr int GC_YP = 36;   // floats per pixel row of a wave's output tile
constexpr int GC_RING = 16;  // filter fragments in flight per lane (a K of 512 is requested whole)

template <int NW, bool RES>
__global__ __launch_bounds__(64 * NW) void conv1x1_gap_kernel(const int8_t *__restrict__ X, const int8_t *__restrict__ Wt,
                                                             GapConvDev e, GapConvParams p) {
  constexpr int NT = 64 * NW;
  extern __shared__ __attribute__((aligned(1024))) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int img = blockIdx.x;
  const int c_own = (blockIdx.y * NW + wave) * 32;
  const bool live = c_own < p.Co;  // wave-uniform; a wave past the last channel repeats the first channels' work and stores nothing
  const int c0 = live ? c_own : 0;
  const int nk = p.K >> 5;

  // The block's requests go out in the order their data is needed, and nothing waits before all are out: the image's
  // pixels (the wait counter retires loads in order, so these can be waited for alone), the filter fragments of the
  // first steps, the residual, the constants.
  constexpr int XU = 4;  // 16-byte chunks per lane in the first round: a 7 x 7 x 512 image whole
  const int cpr = p.K >> 4;  // chunks per pixel
  const int total = p.HW * cpr;
  const int8_t *xi = X + (int64_t)img * p.HW * p.K;  // the image's pixels are contiguous
  v4i xv[XU];
#pragma unroll
  for (int u = 0; u < XU; ++u) {
    const int i = tid + u * NT < total ? tid + u * NT : total - 1;
    xv[u] = *reinterpret_cast<const v4i *>(xi + (int64_t)i * 16);
  }
  v4i ring[GC_RING];
  const int8_t *wsrc = Wt + (int64_t)(c0 + frow) * p.K + fhalf * 16;
#pragma unroll
  for (int d = 0; d < GC_RING; ++d) {
    // straight-line requests (steps past K repeat the last one): with branches around them the wait counters would be
    // set for the worst case and the first use would wait for every request of the block
    ring[d] = *reinterpret_cast<const v4i *>(wsrc + (d < nk ? d : nk - 1) * 32);
  }
  // the residual of this lane's values
  v4f res[2][4];
  const int ch_l = c0 + 4 * fhalf;  // + 8 * i: the four channel quads of this lane
#pragma unroll
  for (int g = 0; g < 2; ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      res[g][i] = v4f{0.f, 0.f, 0.f, 0.f};
      const int px = g * 32 + frow;
      const int pc = px < p.HW ? px : p.HW - 1;  // lanes past the image read its last pixel
      if constexpr (RES)
        res[g][i] = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(e.resid + ((int64_t)img * p.HW + pc) * p.Co + ch_l + 8 * i));
    }
  // the channels' constants, the power of two folded into the reciprocal form
  v4f dv[4], rc[4], bs[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    dv[i] = *reinterpret_cast<const v4f *>(e.div + ch_l + 8 * i);
    rc[i] = *reinterpret_cast<const v4f *>(e.rcp + ch_l + 8 * i);
    bs[i] = *reinterpret_cast<const v4f *>(e.bias + ch_l + 8 * i);
  }
  // ---- 1: the image's pixels: requested first (see above), written to LDS now ----------------------------------------
#pragma unroll
  for (int u = 0; u < XU; ++u) {
    const int i = tid + u * NT;
    const int px = i / cpr, k = i - px * cpr;
    if (i < total) *reinterpret_cast<v4i *>(lds + px * p.xs + k * 16) = xv[u];
  }
  for (int i = tid + XU * NT; i < total; i += NT) {  // images beyond the first round's 64 KiB
    const int px = i / cpr, k = i - px * cpr;
    *reinterpret_cast<v4i *>(lds + px * p.xs + k * 16) = *reinterpret_cast<const v4i *>(xi + (int64_t)i * 16);
  }
  __syncthreads();

  // ---- 2: the convolution ---------------------------------------------------------------------------------------------
  v16i acc[2];
#pragma unroll
  for (int g = 0; g < 2; ++g)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[g][r] = 0;
  {
    const int8_t *xrow[2];
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const int px = g * 32 + frow;
      xrow[g] = lds + (px < p.HW ? px : p.HW - 1) * p.xs + fhalf * 16;  // lanes past the image repeat its last pixel
    }
    // pixel fragments one step ahead of the matrix instructions that read them
    v4i fb0 = *reinterpret_cast<const v4i *>(xrow[0]), fb1 = *reinterpret_cast<const v4i *>(xrow[1]);
    for (int ks0 = 0; ks0 < nk; ks0 += GC_RING) {
#pragma unroll
      for (int d = 0; d < GC_RING; ++d) {
        const int ks = ks0 + d;
        if (ks < nk) {  // wave-uniform
          const v4i fa = ring[d], b0 = fb0, b1 = fb1;
          if (ks + GC_RING < nk) ring[d] = *reinterpret_cast<const v4i *>(wsrc + (ks + GC_RING) * 32);
          const int kn = ks + 1 < nk ? ks + 1 : ks;
          fb0 = *reinterpret_cast<const v4i *>(xrow[0] + kn * 32);
          fb1 = *reinterpret_cast<const v4i *>(xrow[1] + kn * 32);
          acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, b0, acc[0], 0, 0, 0);
          if (p.groups > 1) acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, b1, acc[1], 0, 0, 0);
        }
      }
    }
  }
  __syncthreads();  // every wave is done with the pixels: the output tiles overlay them

  // ---- 3: epilogue into the wave's tile, then the ordered sum over the pixels -----------------------------------------
  float *yt = reinterpret_cast<float *>(lds) + wave * (p.HW * GC_YP);
  {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dv[i][j] = __builtin_ldexpf(dv[i][j], -e.exp2);
        rc[i][j] = __builtin_ldexpf(rc[i][j], e.exp2);
      }
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        if (g >= p.groups) break;
        const int px = g * 32 + frow;
        v4f y;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float v = div_by_rcp((float)acc[g][4 * i + j], dv[i][j], rc[i][j]) + bs[i][j];
          if constexpr (RES) v = v + res[g][i][j];
          if (e.act >= CATCHQ_ACT_RELU) v = (v > 0.0f) ? v : 0.0f;
          if (e.act == CATCHQ_ACT_RELU6) v = (v < 6.0f) ? v : 6.0f;
          y[j] = v;
        }
        if (px < p.HW) *reinterpret_cast<v4f *>(yt + px * GC_YP + 8 * i + 4 * fhalf) = y;
      }
    }
  }
  __syncthreads();
  if (live && lane < 32) {
    // in storage order, one addition per pixel: the order is part of the result; eight reads are requested at a time
    float s = 0.0f;
    int px = 0;
    for (; px + 8 <= p.HW; px += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = yt[(px + u) * GC_YP + lane];
#pragma unroll
      for (int u = 0; u < 8; ++u) s = s + v[u];
    }
    for (; px < p.HW; ++px) s = s + yt[px * GC_YP + lane];
    const float mean = s / (float)p.HW;
    const int64_t idx = (int64_t)img * p.Co + c_own + lane;
    if (e.mean) e.mean[idx] = mean;
    if (e.q) {
      if (e.q_bw == 8) reinterpret_cast<int8_t *>(e.q)[idx] = (int8_t)quant1<8>(mean, e.q_scale, e.q_neg_pos);
      else reinterpret_cast<int16_t *>(e.q)[idx] = (int16_t)quant1<16>(mean, e.q_scale, e.q_neg_pos);
    }
  }
}

// waves per block and LDS bytes; false: not this kernel's shape (images of at most 64 pixels, K a multiple of 32, Co a
// multiple of 32, pixels and output tiles within the LDS of a compute unit)
static bool gap_plan(int N, int HW, int K, int Co, int &nw, int &lds_bytes) {
  if (!(N > 0 && HW >= 1 && HW <= 64 && K >= 32 && K % 32 == 0 && K <= 4096 && Co >= 32 && Co % 32 == 0 &&
        (int64_t)N * HW * K < (1ll << 31) && (int64_t)N * HW * Co < (1ll << 31) && (int64_t)Co * K < (1ll << 31)))
    return false;
  // eight waves (256 channels) per block, four where that leaves compute units without a block
  nw = ((int64_t)N * ((Co + 255) / 256) >= 256) ? 8 : 4;
  const int tile_x = HW * (K + 16), tile_y = nw * HW * GC_YP * 4;
  lds_bytes = ((tile_x > tile_y ? tile_x : tile_y) + 255) / 256 * 256;
  return lds_bytes <= 160 * 1024;
}

bool conv1x1_gap_i8_ok(int N, int HW, int K, int Co) {
  int nw, lds;
  return gap_plan(N, HW, K, Co, nw, lds);
}

// x [N, HW, K] int8, w [Co, K] int8; mean / q [N, Co].  -1: not this kernel's shape.
int conv1x1_gap_i8(const void *x, const void *w, int N, int HW, int K, int Co, const GapConvDev &e, hipStream_t st) {
  int nw, lds_bytes;
  if (!gap_plan(N, HW, K, Co, nw, lds_bytes)) return -1;
  GapConvParams p = {};
  p.N = N; p.HW = HW; p.K = K; p.Co = Co;
  p.xs = K + 16;
  p.groups = (HW + 31) / 32;
  auto launch = [&](auto kern) {
    if (lds_bytes > 64 * 1024) {
      static std::atomic<bool> raised[64];
      if (raise_lds_limit((const void *)kern, 160 * 1024, raised) != CATCHQ_OK) return (int)CATCHQ_ERR_LAUNCH;
    }
    kern<<<dim3(N, (Co + 32 * nw - 1) / (32 * nw)), 64 * nw, lds_bytes, st>>>((const int8_t *)x, (const int8_t *)w, e, p);
    return launch_status();
  };
  if (e.resid) return nw == 8 ? launch(conv1x1_gap_kernel<8, true>) : launch(conv1x1_gap_kernel<4, true>);
  return nw == 8 ? launch(conv1x1_gap_kernel<8, false>) : launch(conv1x1_gap_kernel<4, false>);
}

}  // namespace catchq
