// The first layers of an image network in one launch: quantize the fp32 input, 7x7 stride-2 convolution over three
// (or fewer) channels, ReLU / ReLU6, requantize to int8, 3x3 stride-2 max pooling.
//
// Run layer by layer this is three launches: the quantizer writes a framed int8 image and the convolution reads it
// back, the convolution writes 64 channels for every second pixel -- the largest activation of the network -- and
// the pooling reads that to keep a quarter of it.  Here a block of eight waves owns a band of PR pooled rows of
// one image over its whole width:
//
//   1  input      the 4*PR + 7 image rows under the band (fewer at the image's edges) are read as fp32 planes,
//                 quantized with the quantizer's own arithmetic and written to LDS as 4-channel int8 pixels inside
//                 the convolution's zero frame -- the layout the stand-alone first-layer kernel reads from memory;
//   2  convolve   for every 32 convolution pixels x 32 output channels one wave multiplies on the matrix cores
//                 with the operands swapped (filter rows as A, image rows as B: a K step of 32 bytes is one filter
//                 row of 8 taps x 4 channels, the eighth tap and the fourth channel zero), so that a lane ends up
//                 with four consecutive channels of one pixel, applies the layer's epilogue arithmetic
//                 (reciprocal-form division, bias, the activation folded into the requantizer's clamp) and
//                 writes one dword into the band's convolution tile in LDS.  The 2*PR + 1 convolution rows of a
//                 band share one row with the band above: that row is computed twice;
//   3  pool       a lane takes four channels of one pooled column and walks down the band: three dwords of a
//                 convolution row give the row's maximum, shared by the two windows that contain the row; bytes are
//                 compared two at a time as 16-bit halves (the activation leaves 0..127, unsigned order is the
//                 signed one).  Window taps in the padding read a neighbour inside the window instead.
//
// Neither the framed int8 image nor the convolution's output reaches memory.  Every integer is the one the three
// separate launches produce: the same quantizer, the same sums, the same float operations in the same order, and
// the maximum of the same values.
#include "igemm_common.h"

namespace catchq {

struct StemPoolParams {
  int N, C, H, W;      // fp32 input [N, C, H, W], C <= 3
  int Hc, Wc, Co;      // convolution output
  int Hp, Wp;          // pooled output
  int PR, bands;       // pooled rows per block, blocks per image
  int in_pitch;        // bytes of a framed input row in LDS: (W + 8) * 4
  int off_in, off_tile;  // LDS regions behind the constants
  int x_neg_pos;
  float x_scale;
};

constexpr int SP_KH = 7, SP_PAD = 3, SP_TP_EXTRA = 4;

template <int NW>
__global__ __launch_bounds__(64 * NW) void stem_pool_kernel(const float *__restrict__ X, IrbStageDev s,
                                                           int8_t *__restrict__ Q, StemPoolParams p) {
  constexpr int NT = 64 * NW, KH = SP_KH;
  extern __shared__ __attribute__((aligned(1024))) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int img = blockIdx.x / p.bands, band = blockIdx.x - img * p.bands;
  const int pr0 = band * p.PR;
  const int prn = p.Hp - pr0 < p.PR ? p.Hp - pr0 : p.PR;
  const int cr0 = 2 * pr0 - 1 > 0 ? 2 * pr0 - 1 : 0;  // first and last convolution row of the band
  const int cr1 = 2 * (pr0 + prn - 1) + 1 < p.Hc - 1 ? 2 * (pr0 + prn - 1) + 1 : p.Hc - 1;
  const int nrows = cr1 - cr0 + 1;
  const int iy0 = 2 * cr0 - SP_PAD;     // image row of LDS row 0
  const int nin = 2 * (nrows - 1) + KH;  // framed input rows in use
  const int tp = p.Co + SP_TP_EXTRA;     // bytes of a tile pixel: the odd dword stride spreads a wave's stores over the banks

  // this wave's 32 output channels: filter rows stay in registers
  const int ncg = p.Co >> 5;
  const int chg = wave % ncg;
  v4i fw[KH];
  {
    const int8_t *src = s.w + (int64_t)(chg * 32 + frow) * (KH * 32) + fhalf * 16;
#pragma unroll
    for (int r = 0; r < KH; ++r) fw[r] = *reinterpret_cast<const v4i *>(src + r * 32);
  }
  float *cst = reinterpret_cast<float *>(lds);
  float cv[3] = {1.0f, 1.0f, 0.0f};
  if (tid < p.Co) { cv[0] = s.div[tid]; cv[1] = s.rcp[tid]; cv[2] = s.bias[tid]; }

  // ---- 1: the band's input rows, quantized into their frame ---------------------------------------------------------
  {
    const int groups = p.W >> 2, per_row = groups + 8;  // 4-pixel groups of a row, then 3 + 5 border pixels
    const int items = nin * per_row;
    const int64_t hw = (int64_t)p.H * p.W;
    const float *xi = X + (int64_t)img * p.C * hw;
    constexpr int U = 3;
    for (int it0 = tid; it0 < items; it0 += U * NT) {
      v4f v[U][3];
      int row[U], t[U];
      bool inside[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int it = it0 + u * NT;
        row[u] = it / per_row;
        t[u] = it - row[u] * per_row;
        const int iy = iy0 + row[u];
        inside[u] = it < items && t[u] < groups && (unsigned)iy < (unsigned)p.H;
#pragma unroll
        for (int ch = 0; ch < 3; ++ch) {
          v[u][ch] = v4f{0.f, 0.f, 0.f, 0.f};
          if (inside[u] && ch < p.C)
            v[u][ch] = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(xi + ch * hw + (int64_t)iy * p.W) + t[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (it0 + u * NT >= items) break;
        int *dst = reinterpret_cast<int *>(lds + p.off_in + row[u] * p.in_pitch);
        if (t[u] < groups) {
#pragma unroll
          for (int px = 0; px < 4; ++px) {
            unsigned b = 0;
#pragma unroll
            for (int ch = 0; ch < 3; ++ch)
              b |= ((unsigned)quant1<8>(v[u][ch][px], p.x_scale, p.x_neg_pos) & 0xffu) << (8 * ch);  // 0 -> 0
            dst[SP_PAD + 4 * t[u] + px] = (int)b;
          }
        } else {
          const int bpx = t[u] - groups;
          dst[bpx < SP_PAD ? bpx : p.W + bpx] = 0;
        }
      }
    }
  }
  if (tid < p.Co) {
    cst[tid] = __builtin_ldexpf(cv[0], -s.exp2);
    cst[p.Co + tid] = __builtin_ldexpf(cv[1], s.exp2);
    cst[2 * p.Co + tid] = cv[2];
  }
  float q_hi = __builtin_ldexpf(127.0f, -s.q_neg_pos);
  if (s.relu6) q_hi = q_hi < 6.0f ? q_hi : 6.0f;
  const float q_sc = __builtin_ldexpf(1.0f, s.q_neg_pos);
  __syncthreads();

  // ---- 2: convolution of the band, requantized into the tile --------------------------------------------------------
  {
    const int npix = nrows * p.Wc;
    const int ngroups = (npix + 31) >> 5;
    const int8_t *in = lds + p.off_in + fhalf * 16;
    int8_t *tile = lds + p.off_tile;
    auto load_px = [&](int g, v4i (&fx)[KH]) {
      const int t = g * 32 + frow;
      const int tc = t < npix ? t : npix - 1;  // lanes past the band repeat its last pixel; their results are dropped
      const int lr = tc / p.Wc, cc = tc - lr * p.Wc;
      const int8_t *src = in + 2 * lr * p.in_pitch + cc * 8;
#pragma unroll
      for (int r = 0; r < KH; ++r) {
        const v2i a = *reinterpret_cast<const v2i *>(src + r * p.in_pitch);
        const v2i b = *reinterpret_cast<const v2i *>(src + r * p.in_pitch + 8);
        fx[r] = v4i{a[0], a[1], b[0], b[1]};
      }
    };
    const int g_step = NW / ncg;
    int g = wave / ncg;
    v4i fxn[KH];
    if (g < ngroups) load_px(g, fxn);
    for (; g < ngroups; g += g_step) {
      v16i acc;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[r] = 0;
#pragma unroll
      for (int r = 0; r < KH; ++r) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[r], fxn[r], acc, 0, 0, 0);
      if (g + g_step < ngroups) load_px(g + g_step, fxn);
      const int t = g * 32 + frow;
      const float *cb = cst + chg * 32 + 4 * fhalf;
      int8_t *cell = tile + t * tp + chg * 32 + 4 * fhalf;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const v4f dv = *reinterpret_cast<const v4f *>(cb + 8 * i);
        const v4f rc = *reinterpret_cast<const v4f *>(cb + p.Co + 8 * i);
        const v4f bs = *reinterpret_cast<const v4f *>(cb + 2 * p.Co + 8 * i);
        unsigned b[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float x = div_by_rcp((float)acc[4 * i + j], dv[j], rc[j]) + bs[j];
          x = __builtin_amdgcn_fmed3f(x, 0.0f, q_hi);  // the activation and the upper clamp; NaN -> 0
          b[j] = __builtin_bit_cast(unsigned, __builtin_fmaf(x, q_sc, 12582912.0f));  // round to even into the low byte
        }
        const unsigned lo = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
        const unsigned hi = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
        if (t < npix) *reinterpret_cast<unsigned *>(cell + 8 * i) = lo | hi;
      }
    }
  }
  __syncthreads();

  // ---- 3: 3x3 stride-2 maximum over the tile -------------------------------------------------------------------------
  // A lane owns four channels of one pooled column and walks down the band's pooled rows: the maximum over the three
  // columns of a convolution row is taken once and shared by the two windows that contain the row.  Bytes are compared
  // two at a time as 16-bit halves: the even bytes masked out, the odd bytes in place (the byte below them only
  // breaks ties).
  {
    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
    const int quads = p.Co >> 2;
    const int items = p.Wp * quads;
    const int8_t *tile = lds + p.off_tile;
    int8_t *out = Q + ((int64_t)img * p.Hp + pr0) * p.Wp * p.Co;
    for (int it = tid; it < items; it += NT) {
      const int j = it / quads, q = it - j * quads;
      int cofs[3];
#pragma unroll
      for (int b = 0; b < 3; ++b) {
        int c = 2 * j - 1 + b;
        c = c < 0 ? 0 : (c > p.Wc - 1 ? p.Wc - 1 : c);  // a tap in the padding reads a neighbour inside the window
        cofs[b] = c * tp + 4 * q;
      }
      u16x2 even_r, odd_r;
      auto row_max = [&](int conv_row) {
        const int r = (conv_row < 0 ? 0 : (conv_row > p.Hc - 1 ? p.Hc - 1 : conv_row)) - cr0;
        const int8_t *base = tile + r * p.Wc * tp;
        const unsigned a = *reinterpret_cast<const unsigned *>(base + cofs[0]);
        const unsigned b = *reinterpret_cast<const unsigned *>(base + cofs[1]);
        const unsigned c = *reinterpret_cast<const unsigned *>(base + cofs[2]);
        even_r = __builtin_elementwise_max(__builtin_elementwise_max(__builtin_bit_cast(u16x2, a & 0x00ff00ffu),
                                                                     __builtin_bit_cast(u16x2, b & 0x00ff00ffu)),
                                           __builtin_bit_cast(u16x2, c & 0x00ff00ffu));
        odd_r = __builtin_elementwise_max(__builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)),
                                          __builtin_bit_cast(u16x2, c));
      };
      row_max(2 * pr0 - 1);
      u16x2 even_p = even_r, odd_p = odd_r;  // the row shared with the window above
      for (int i = 0; i < prn; ++i) {
        row_max(2 * (pr0 + i));
        u16x2 even = __builtin_elementwise_max(even_p, even_r), odd = __builtin_elementwise_max(odd_p, odd_r);
        row_max(2 * (pr0 + i) + 1);
        even = __builtin_elementwise_max(even, even_r);
        odd = __builtin_elementwise_max(odd, odd_r);
        even_p = even_r;
        odd_p = odd_r;
        *reinterpret_cast<unsigned *>(out + ((int64_t)i * p.Wp + j) * p.Co + 4 * q) =
            __builtin_bit_cast(unsigned, even) | (__builtin_bit_cast(unsigned, odd) & 0xff00ff00u);
      }
    }
  }
}

// 7x7 / 2 / pad 3 convolution of up to three channels followed by 3x3 / 2 / pad 1 max pooling; 32, 64 or 128 output
// channels; fp32 planes of a width that is a multiple of 4.
// Band height: a block's work grows with its 2 * PR + 1 convolution rows plus a fixed part (set-up, barriers, the
// latency of its input rows), the launch takes as many rounds of blocks as the busiest compute unit gets, and a
// compute unit that holds one block at a time (more than 80 KiB of LDS) cannot hide one block's input latency behind
// another's arithmetic.  Measured on 32 x 3 x 224 x 224 (us): PR 2 25.6, 3 25.7, 4 25.7, 5 28.9, 6 30.3 and, with one
// block of sixteen waves per compute unit, 7 20.0 (64 images: 3 42.0, 7 39.3) -- the estimate below ranks them in that
// order.  Blocks that are alone on their compute unit run sixteen waves.
static bool stem_pool_plan(int N, int C, int H, int W, int Co, StemPoolParams &p, int &lds_bytes, int &waves) {
  if (N <= 0 || C < 1 || C > 3 || H < 7 || W < 8 || W % 4 != 0 || W > 2048) return false;
  if (Co != 32 && Co != 64 && Co != 128) return false;
  p = StemPoolParams{};
  p.N = N; p.C = C; p.H = H; p.W = W; p.Co = Co;
  p.Hc = (H + 2 * SP_PAD - SP_KH) / 2 + 1;
  p.Wc = (W + 2 * SP_PAD - SP_KH) / 2 + 1;
  p.Hp = (p.Hc + 2 - 3) / 2 + 1;
  p.Wp = (p.Wc + 2 - 3) / 2 + 1;
  if (p.Hc < 2 || p.Wc < 2) return false;
  if ((int64_t)N * C * H * W >= (1ll << 31) || (int64_t)N * p.Hp * p.Wp * Co >= (1ll << 31)) return false;
  p.in_pitch = (W + 8) * 4;
  auto up = [](int v) { return (v + 255) / 256 * 256; };
  auto lds_of = [&](int pr) {
    return up(Co * 12) + up((4 * pr + SP_KH) * p.in_pitch) + up((2 * pr + 1) * p.Wc * (Co + SP_TP_EXTRA));
  };
  int want = 0;
  if (const char *t = tuning_env("CATCHQ_STEM_PR")) want = atoi(t);
  constexpr int kDeviceCUs = 256;
  int best = 0;
  int64_t best_cost = 0;
  for (int pr = 1; pr <= p.Hp && pr <= 16; ++pr) {
    const int lds = lds_of(pr);
    if (lds > 160 * 1024) break;
    const int bands = (p.Hp + pr - 1) / pr;
    const int64_t rounds = ((int64_t)N * bands + kDeviceCUs - 1) / kDeviceCUs;
    const int64_t cost = rounds * (4 * pr + 5) * (lds > 80 * 1024 ? 140 : 115);
    if (want > 0 ? (pr == want || !best) : (!best || cost < best_cost)) { best = pr; best_cost = cost; }
  }
  if (!best) return false;
  p.PR = best;
  p.bands = (p.Hp + best - 1) / best;
  if ((int64_t)N * p.bands > 0x7fffffff) return false;
  p.off_in = up(Co * 12);
  p.off_tile = p.off_in + up((4 * best + SP_KH) * p.in_pitch);
  lds_bytes = lds_of(best);
  waves = lds_bytes > 80 * 1024 ? 16 : 8;
  if (const char *t = tuning_env("CATCHQ_STEM_NW")) waves = atoi(t) == 16 ? 16 : 8;
  return true;
}

bool stem_pool_i8_ok(int N, int C, int H, int W, int Co) {
  StemPoolParams p;
  int lds, waves;
  return stem_pool_plan(N, C, H, W, Co, p, lds, waves);
}

// x fp32 [N, C, H, W]; s.w the filters [Co][7][8][4] (the eighth tap and the channels from C on zero); q int8
// [N, Hp, Wp, Co].  -1: not this kernel's shape.
int stem_pool_i8(const void *x, int N, int C, int H, int W, int x_pos, float x_scale, const IrbStageDev &s, int Co,
                 void *q, hipStream_t st) {
  StemPoolParams p;
  int lds_bytes, waves;
  if (!stem_pool_plan(N, C, H, W, Co, p, lds_bytes, waves)) return -1;
  p.x_neg_pos = -x_pos;
  p.x_scale = x_scale;
  auto launch = [&](auto kern, int nw) {
    if (lds_bytes > 64 * 1024) {
      static std::atomic<bool> raised[64];
      if (raise_lds_limit((const void *)kern, 160 * 1024, raised) != CATCHQ_OK) return (int)CATCHQ_ERR_LAUNCH;
    }
    kern<<<N * p.bands, 64 * nw, lds_bytes, st>>>((const float *)x, s, (int8_t *)q, p);
    return launch_status();
  };
  return waves == 16 ? launch(stem_pool_kernel<16>, 16) : launch(stem_pool_kernel<8>, 8);
}

}  // namespace catchq
