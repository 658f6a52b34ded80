// Depthwise int8 convolution (groups == Ci == Co) on NHWC tensors: a stencil, not a contraction,
// so no matrix cores.  Two kernels:
//  * dw3x3_kernel: 3x3, dilation 1, stride 1 or 2 (every depthwise layer of the MobileNet family).
//    A lane owns 4 channels x (2 rows x 4 columns) of output pixels, transposes the input window in
//    registers so that v_dot4_i32_i8 sums the taps of a filter row, and finishes with the vector epilogue of the GEMM kernels; adjacent lanes hold adjacent
//    channel quads, so loads and stores of a wave are contiguous runs of the NHWC row.
//  * dwconv_i8_kernel: any filter up to 5x5, any stride/dilation.  A block owns a strip of output pixels of one image row and all channels of a
// 64-channel slab; the input rows the strip needs are staged in LDS once and every tap is read
// from there, the filter taps of the slab sit in LDS transposed to [tap][channel].
#include "catchq_common.h"
#include "igemm_common.h"

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
  resolve_exp2(e);
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

struct Dw3Params {
  int N, H, W, C, ph, pw, Ho, Wo;
  int CQ;     // channel quads
  int WG;     // column groups per output row
  int HG;     // row groups per image
  int items;  // HG * WG * CQ: work items of one image
};

constexpr int DW3_PW = 4, DW3_PH = 2;

template <int S, int EPI>
__global__ __launch_bounds__(256) void dw3x3_kernel(const int8_t *__restrict__ x, const int8_t *__restrict__ w,
                                                   Dw3Params p, EpiDev e) {
  resolve_exp2(e);
  typedef typename EpiOf<EPI>::type Sp;
  constexpr int PW = DW3_PW, PH = DW3_PH;
  constexpr int NR = (PH - 1) * S + 3;  // input rows of the window
  const int item = blockIdx.x * 256 + threadIdx.x;  // (row group, column group, channel quad), channels fastest
  if (item >= p.items) return;
  const int t0 = item / p.CQ, cq = item - t0 * p.CQ;
  const int hg = t0 / p.WG, wg = t0 - hg * p.WG;
  const int ho0 = hg * PH, img = blockIdx.y;
  const int c = cq * 4;

  // The multiply-accumulate runs on v_dot4_i32_i8, which sums four byte products: the four bytes of
  // an operand must be four taps of ONE channel.  A pixel's dword holds four channels, so groups of
  // four horizontally adjacent pixels are transposed (4x4 bytes, 8 byte permutes, the first stage
  // shared between overlapping groups) into one dword per channel; a filter row is the byte vector
  // (w0, w1, w2, 0) or, for the output one pixel to the right within the same group, (0, w0, w1, w2).
  // 36 filter bytes of the four channels ([channel][tap]):
  int wraw[9];
#pragma unroll
  for (int i = 0; i < 9; ++i) wraw[i] = *reinterpret_cast<const int *>(w + (int64_t)c * 9 + 4 * i);
  int wa[4][3], wb[4][3];  // [channel][filter row]
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      unsigned v = 0;
#pragma unroll
      for (int q = 0; q < 3; ++q) {
        const int b = j * 9 + r * 3 + q;
        v |= (((unsigned)wraw[b >> 2] >> (8 * (b & 3))) & 0xffu) << (8 * q);
      }
      wa[j][r] = (int)v;
      wb[j][r] = (int)(v << 8);
    }

  int acc[PH][PW][4];  // every sum starts with filter row 0 (accumulator operand 0), no zeroing pass

  constexpr int NG = (S == 1) ? 2 : 4;  // transposed groups per input row: pixels 0-3, 2-5 [, 4-7, 6-9]
  constexpr int NCL = 2 * NG + 2;       // input columns loaded (stride 2: one more than the window, weight 0)
  const int hi0 = ho0 * S - p.ph, wi0 = wg * PW * S - p.pw;
  // addresses = a per-image base (the same for the whole block: scalar registers) + a 32-bit offset
  const int8_t *xi = x + (int64_t)img * p.H * p.W * p.C;
#pragma unroll
  for (int ri = 0; ri < NR; ++ri) {
    const int hi = hi0 + ri;
    const bool row_ok = (unsigned)hi < (unsigned)p.H;
    unsigned xr[NCL];
    const unsigned rowo = (unsigned)((hi * p.W + wi0) * p.C + c);  // column 0 of the window (may lie outside: masked below)
#pragma unroll
    for (int col = 0; col < NCL; ++col) {
      xr[col] = 0;
      if (row_ok && (unsigned)(wi0 + col) < (unsigned)p.W)
        xr[col] = *reinterpret_cast<const unsigned *>(xi + (rowo + (unsigned)(col * p.C)));
    }
    // first transposition stage on pixel pairs (2m, 2m+1): bytes (a0,b0,a1,b1) and (a2,b2,a3,b3)
    unsigned lo[NG + 1], hi2[NG + 1];
#pragma unroll
    for (int m = 0; m <= NG; ++m) {
      lo[m] = __builtin_amdgcn_perm(xr[2 * m + 1], xr[2 * m], 0x05010400u);
      hi2[m] = __builtin_amdgcn_perm(xr[2 * m + 1], xr[2 * m], 0x07030602u);
    }
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      // second stage: group g = pixels 2g .. 2g+3, one dword per channel
      int t[4];
      t[0] = (int)__builtin_amdgcn_perm(lo[g + 1], lo[g], 0x05040100u);
      t[1] = (int)__builtin_amdgcn_perm(lo[g + 1], lo[g], 0x07060302u);
      t[2] = (int)__builtin_amdgcn_perm(hi2[g + 1], hi2[g], 0x05040100u);
      t[3] = (int)__builtin_amdgcn_perm(hi2[g + 1], hi2[g], 0x07060302u);
#pragma unroll
      for (int py = 0; py < PH; ++py) {
        const int r = ri - py * S;
        if (r < 0 || r > 2) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (S == 1) {  // group g serves outputs 2g (taps at bytes 0..2) and 2g+1 (bytes 1..3)
            acc[py][2 * g][j] = __builtin_amdgcn_sdot4(t[j], wa[j][r], r == 0 ? 0 : acc[py][2 * g][j], false);
            acc[py][2 * g + 1][j] = __builtin_amdgcn_sdot4(t[j], wb[j][r], r == 0 ? 0 : acc[py][2 * g + 1][j], false);
          } else {                 // stride 2: group g starts at input pixel 2g = the window of output g
            acc[py][g][j] = __builtin_amdgcn_sdot4(t[j], wa[j][r], r == 0 ? 0 : acc[py][g][j], false);
          }
        }
      }
    }
  }

  const EpiLane L = epi_lane_setup<Sp>(c, true, e);
#pragma unroll
  for (int py = 0; py < PH; ++py) {
    const int ho = ho0 + py;
    if (ho >= p.Ho) continue;
#pragma unroll
    for (int px = 0; px < PW; ++px) {
      const int wo = wg * PW + px;
      if (wo >= p.Wo) continue;
      const EpiAtSplit at = {(int64_t)img * p.Ho * p.Wo * p.C, (unsigned)((ho * p.Wo + wo) * p.C + c)};
      v4f res = {0.f, 0.f, 0.f, 0.f};
      if (L.use_res) res = load_stream(reinterpret_cast<const v4f *>(at.at(e.resid)), e.resid_stream != 0);
      const v4i a = {acc[py][px][0], acc[py][px][1], acc[py][px][2], acc[py][px][3]};
      epi_vec4<Sp>(a, res, L, at, e);
    }
  }
}

template <int S, int EPI>
static void dw3x3_launch(const void *x, const void *w, const Dw3Params &p, dim3 grid, const EpiDev &e, hipStream_t s) {
  dw3x3_kernel<S, EPI><<<grid, 256, 0, s>>>((const int8_t *)x, (const int8_t *)w, p, e);
}

// 0 when launched, -1 when the shape is not this kernel's
static int dw3x3(const void *x, const void *w, int N, int H, int W, int C, int kh, int kw, int ph, int pw, int sh,
                 int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  if (kh != 3 || kw != 3 || dh != 1 || dw != 1 || sh != sw || (sh != 1 && sh != 2)) return -1;
  const int epi = pick_epilogue(C, e);
  if (epi == EPI_SCALAR) return -1;
  Dw3Params p = {N, H, W, C, ph, pw, Ho, Wo, C / 4, (Wo + DW3_PW - 1) / DW3_PW, (Ho + DW3_PH - 1) / DW3_PH, 0};
  const int64_t items = (int64_t)p.HG * p.WG * p.CQ;
  if (items > 0x7fffff00 || N > 65535) return -1;
  if ((int64_t)H * W * C >= (1ll << 31) || (int64_t)Ho * Wo * C >= (1ll << 31)) return -1;  // 32-bit offsets within an image
  p.items = (int)items;
  const dim3 grid((unsigned)((items + 255) / 256), (unsigned)N);
  const bool s2 = sh == 2;
  switch (epi) {
    case EPI_Q8_RELU6: s2 ? dw3x3_launch<2, EPI_Q8_RELU6>(x, w, p, grid, e, s) : dw3x3_launch<1, EPI_Q8_RELU6>(x, w, p, grid, e, s); break;
    case EPI_Q8_RELU: s2 ? dw3x3_launch<2, EPI_Q8_RELU>(x, w, p, grid, e, s) : dw3x3_launch<1, EPI_Q8_RELU>(x, w, p, grid, e, s); break;
    default: s2 ? dw3x3_launch<2, EPI_VECTOR>(x, w, p, grid, e, s) : dw3x3_launch<1, EPI_VECTOR>(x, w, p, grid, e, s); break;
  }
  return 0;
}

bool dwconv_i8_supported(int C, int kh, int kw, int sw, int dw) {
  if (C % 4 != 0 || kh * kw > DW_MAXTAPS) return false;
  const int in_w = (DW_TW - 1) * sw + (kw - 1) * dw + 1;
  return (int64_t)kh * in_w * DW_CS <= DW_LDS_BYTES;
}

int dwconv_i8(const void *x, const void *w, int N, int H, int W, int C, int kh, int kw, int ph, int pw, int sh,
              int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  if (dw3x3(x, w, N, H, W, C, kh, kw, ph, pw, sh, sw, dh, dw, Ho, Wo, e, s) == 0) return launch_status();
  DwParams p = {N, H, W, C, kh, kw, ph, pw, sh, sw, dh, dw, Ho, Wo, 0, 0};
  p.strips = (Wo + DW_TW - 1) / DW_TW;
  p.slabs = (C + DW_CS - 1) / DW_CS;
  const int64_t nb = (int64_t)N * Ho * p.strips * p.slabs;
  if (nb > 0x7fffffff) return CATCHQ_ERR_SHAPE;
  dwconv_i8_kernel<<<(int)nb, 256, 0, s>>>((const int8_t *)x, (const int8_t *)w, p, e);
  return launch_status();
}

}  // namespace catchq
