// C ABI entry points of the integer contractions: argument checks, then the route.
#include <cstring>

#include "catchq_common.h"

namespace catchq {

int gemm_nt_direct(const void *a, int a_bits, const void *b, int b_bits, int64_t M, int64_t N, int64_t K,
                   const EpiDev &e, hipStream_t s);
int conv2d_direct(const void *x, int x_bits, const void *w, int w_bits, const ConvDev &d, const EpiDev &e,
                  hipStream_t s);
int gemm_nt_mfma_i8(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e,
                    hipStream_t s);
int conv2d_mfma_i8(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph,
                   int pw, int sh, int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s);
int conv2d_mfma_i8_grouped(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph, int pw,
                           int sh, int sw, int dh, int dw, int Ho, int Wo, int groups, const EpiDev &e, hipStream_t s);
int gemm_nt_mfma_a16(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e, hipStream_t s);
int conv2d_mfma_a16(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph, int pw,
                    int sh, int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s);
int gemm_nt_mfma_a16w16(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e, hipStream_t s);
int conv2d_mfma_a16w16(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph, int pw,
                       int sh, int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s);
int conv2d_dual_i8(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph, int pw,
                   int sh, int sw, int dh, int dw, int Ho, int Wo, const void *xs, const void *ws, int Hs, int Ws, int Cs,
                   int ss, const EpiDev &e, const ShortcutDev &sc, hipStream_t s);
struct ChainLinkDev {  // igemm_i8_chain.hip
  const int8_t *x, *w;
  unsigned x_bytes, w_bytes;
  int K;
  unsigned img_stride, row_stride, pix_stride;
  int dense, k_shift;
  int exp2;
  const float *chan_div, *chan_rcp, *bias;
};
int conv1x1_chain_i8(const ChainLinkDev *links, int nlinks, int N, int Ho, int Wo, int Co, float *y, int8_t *q,
                     int q_position, int sharing, hipStream_t s);
bool conv2d_head_halo_i8_ok(int N, int H, int W, int K1, int Cm, int Co);
int conv2d_head_halo_i8(const void *x, int K1, const void *w1, const float *div1, const float *rcp1, const float *bias1,
                        int exp2_1, int q_position1, const void *w, int N, int H, int W, int Cm, int Co, const EpiDev &e,
                        hipStream_t s);
bool irb_i8_ok(int N, int H, int W, int Cin, int hid, int Co, int S, int cus);
int irb_i8(const void *x, int N, int H, int W, int Cin, int hid, int Co, int S, const IrbStageDev &s1, const IrbStageDev &s2,
           const void *w3, const EpiDev &e, hipStream_t s);
bool stem_pool_i8_ok(int N, int C, int H, int W, int Co);
int stem_pool_i8(const void *x, int N, int C, int H, int W, int x_pos, float x_scale, const IrbStageDev &s, int Co,
                 void *q, hipStream_t st);
struct GapConvDev {
  const float *div, *rcp, *bias, *resid;
  int exp2, act;
  float *mean;
  void *q;
  int q_bw, q_neg_pos;
  float q_scale;
};
bool conv1x1_gap_i8_ok(int N, int HW, int K, int Co);
int conv1x1_gap_i8(const void *x, const void *w, int N, int HW, int K, int Co, const GapConvDev &e, hipStream_t st);
bool dwconv_i8_supported(int C, int kh, int kw, int sw, int dw);
int dwconv_i8(const void *x, const void *w, int N, int H, int W, int C, int kh, int kw, int ph, int pw, int sh,
              int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s);

enum Route { kDirect, kMfma, kMfmaGrouped, kMfmaA16, kMfmaA16W16, kDepthwise, kBad };

static Route gemm_route(int a_bits, int b_bits, int64_t m, int64_t n, int64_t k, const void *a, const void *b) {
  if (a_bits == 8 && b_bits == 8 && k % 16 == 0 && k >= 16 && m > 0 && n > 0 && k < (1ll << 31) &&
      n < (1ll << 31) && (!a || aligned16(a)) && (!b || aligned16(b)))
    return kMfma;
  // int16 activations x int8 weights: two int8 passes over the split operand (buffer offsets are 32-bit)
  if (a_bits == 16 && b_bits == 8 && k % 8 == 0 && k >= 8 && m > 0 && n > 0 && m * k < (1ll << 30) &&
      n * k < (1ll << 31) && (!a || aligned16(a)) && (!b || aligned16(b)))
    return kMfmaA16;
  // int16 x int16: four digit products per K step, exact 64-bit sums
  if (a_bits == 16 && b_bits == 16 && k % 8 == 0 && k >= 8 && k < (1 << 16) && m > 0 && n > 0 && m * k < (1ll << 30) &&
      n * k < (1ll << 30) && (!a || aligned16(a)) && (!b || aligned16(b)))
    return kMfmaA16W16;
  return kDirect;
}

static Route conv_route(int x_bits, int w_bits, const catchq_conv_desc_t *d, const void *x, const void *w) {
  if (x_bits == 8 && w_bits == 8) {
    // is_depthwise_conv: groups != 1, co % groups == 0, one input channel per group, groups == ci
    if (d->groups != 1 && d->groups == d->ci && d->co == d->ci &&
        dwconv_i8_supported(d->ci, d->kh, d->kw, d->stride_w, d->dil_w) && (!x || aligned16(x)))
      return kDepthwise;
    if (d->groups == 1 && d->ci % 16 == 0 && (!x || aligned16(x)) && (!w || aligned16(w))) return kMfma;
    // grouped, not depthwise: one implicit GEMM per group when a group's channels fill whole 16-byte K chunks
    if (d->groups > 1 && d->groups < 65536 && (d->ci / d->groups) % 16 == 0 && (d->co / d->groups) % 4 == 0 &&
        d->kh * d->kw <= 32 && (int64_t)d->n * d->h * d->w * d->ci < (1ll << 31) &&
        (int64_t)d->co * d->kh * d->kw * (d->ci / d->groups) < (1ll << 31) && (!x || aligned16(x)) && (!w || aligned16(w)))
      return kMfmaGrouped;
    // four-channel inputs (an RGB image padded to 4): one pixel per dword
    if (d->groups == 1 && d->ci == 4 && d->dil_w == 1 && (!x || aligned16(x)) && (!w || aligned16(w))) return kMfma;
  }
  if (x_bits == 16 && w_bits == 8 && d->groups == 1 && d->ci % 8 == 0 && d->kh * d->kw <= 32 &&
      (int64_t)d->n * d->h * d->w * d->ci < (1ll << 30) && (int64_t)d->co * d->kh * d->kw * d->ci < (1ll << 31) &&
      (!x || aligned16(x)) && (!w || aligned16(w)))
    return kMfmaA16;
  if (x_bits == 16 && w_bits == 16 && d->groups == 1 && d->ci % 8 == 0 && d->kh * d->kw <= 32 &&
      (int64_t)d->kh * d->kw * d->ci < (1 << 16) && (int64_t)d->n * d->h * d->w * d->ci < (1ll << 30) &&
      (int64_t)d->co * d->kh * d->kw * d->ci < (1ll << 30) && (!x || aligned16(x)) && (!w || aligned16(w)))
    return kMfmaA16W16;
  return kDirect;
}

static const char *route_name(Route r) {
  switch (r) {
    case kMfma: return "mfma";
    case kMfmaGrouped: return "mfma_grouped";
    case kMfmaA16: return "mfma_a16";
    case kMfmaA16W16: return "mfma_a16w16";
    case kDepthwise: return "depthwise";
    case kDirect: return "direct";
    default: return "invalid";
  }
}

static int check_conv(const catchq_conv_desc_t *d, int *ho, int *wo) {
  if (!d) return CATCHQ_ERR_ARG;
  if (d->n < 0 || d->h <= 0 || d->w <= 0 || d->ci <= 0 || d->co <= 0 || d->kh <= 0 || d->kw <= 0)
    return CATCHQ_ERR_SHAPE;
  if (d->pad_h < 0 || d->pad_w < 0 || d->stride_h <= 0 || d->stride_w <= 0 || d->dil_h <= 0 || d->dil_w <= 0)
    return CATCHQ_ERR_SHAPE;
  if (d->groups <= 0 || d->ci % d->groups != 0 || d->co % d->groups != 0) return CATCHQ_ERR_SHAPE;
  *ho = catchq_conv_out_size(d->h, d->kh, d->pad_h, d->stride_h, d->dil_h);
  *wo = catchq_conv_out_size(d->w, d->kw, d->pad_w, d->stride_w, d->dil_w);
  if (*ho <= 0 || *wo <= 0) return CATCHQ_ERR_SHAPE;
  return CATCHQ_OK;
}

}  // namespace catchq

using namespace catchq;

CATCHQ_API const char *catchq_gemm_route(int a_bits, int b_bits, int64_t m, int64_t n, int64_t k) {
  return route_name(gemm_route(a_bits, b_bits, m, n, k, nullptr, nullptr));
}

CATCHQ_API const char *catchq_conv2d_route(int x_bits, int w_bits, const catchq_conv_desc_t *desc) {
  int ho, wo;
  if (check_conv(desc, &ho, &wo) != CATCHQ_OK) return route_name(kBad);
  return route_name(conv_route(x_bits, w_bits, desc, nullptr, nullptr));
}

CATCHQ_API int catchq_gemm_nt(const void *a, int a_bits, const void *b, int b_bits, int64_t m, int64_t n,
                              int64_t k, const catchq_epilogue_t *epilogue, catchq_stream_t stream) {
  if (m < 0 || n < 0 || k < 0) return CATCHQ_ERR_SHAPE;
  if ((a_bits != 8 && a_bits != 16) || (b_bits != 8 && b_bits != 16)) return CATCHQ_ERR_BITWIDTH;
  int st = check_epi(epilogue);
  if (st != CATCHQ_OK) return st;
  if (m == 0 || n == 0) return CATCHQ_OK;
  if (k > 0 && (!a || !b)) return CATCHQ_ERR_ARG;
  const EpiDev e = make_epi(epilogue, m * n);
  hipStream_t s = as_stream(stream);
  const Route route = gemm_route(a_bits, b_bits, m, n, k, a, b);
  if (route == kMfma) return gemm_nt_mfma_i8(a, b, m, n, k, e, s);
  if (route == kMfmaA16) {
    const int st = gemm_nt_mfma_a16(a, b, m, n, k, e, s);
    if (st >= 0) return st;
  }
  if (route == kMfmaA16W16) {
    const int st = gemm_nt_mfma_a16w16(a, b, m, n, k, e, s);
    if (st >= 0) return st;
  }
  return gemm_nt_direct(a, a_bits, b, b_bits, m, n, k, e, s);
}

CATCHQ_API int catchq_conv2d_nhwc(const void *x, int x_bits, const void *w, int w_bits,
                                  const catchq_conv_desc_t *desc, const catchq_epilogue_t *epilogue,
                                  catchq_stream_t stream) {
  int ho, wo;
  int st = check_conv(desc, &ho, &wo);
  if (st != CATCHQ_OK) return st;
  if ((x_bits != 8 && x_bits != 16) || (w_bits != 8 && w_bits != 16)) return CATCHQ_ERR_BITWIDTH;
  st = check_epi(epilogue);
  if (st != CATCHQ_OK) return st;
  if (desc->n == 0) return CATCHQ_OK;
  if (!x || !w) return CATCHQ_ERR_ARG;
  const EpiDev e = make_epi(epilogue, (int64_t)desc->n * ho * wo * desc->co);
  hipStream_t s = as_stream(stream);
  const catchq_conv_desc_t &d = *desc;
  switch (conv_route(x_bits, w_bits, desc, x, w)) {
    case kDepthwise:
      return dwconv_i8(x, w, d.n, d.h, d.w, d.ci, d.kh, d.kw, d.pad_h, d.pad_w, d.stride_h, d.stride_w, d.dil_h,
                       d.dil_w, ho, wo, e, s);
    case kMfma:
      return conv2d_mfma_i8(x, w, d.n, d.h, d.w, d.ci, d.co, d.kh, d.kw, d.pad_h, d.pad_w, d.stride_h,
                            d.stride_w, d.dil_h, d.dil_w, ho, wo, e, s);
    case kMfmaGrouped: {
      const int st2 = conv2d_mfma_i8_grouped(x, w, d.n, d.h, d.w, d.ci, d.co, d.kh, d.kw, d.pad_h, d.pad_w, d.stride_h,
                                             d.stride_w, d.dil_h, d.dil_w, ho, wo, d.groups, e, s);
      if (st2 >= 0) return st2;
      break;  // not eligible after all (e.g. 2^31 output pixels): the direct kernel
    }
    case kMfmaA16: {
      const int st2 = conv2d_mfma_a16(x, w, d.n, d.h, d.w, d.ci, d.co, d.kh, d.kw, d.pad_h, d.pad_w, d.stride_h,
                                      d.stride_w, d.dil_h, d.dil_w, ho, wo, e, s);
      if (st2 >= 0) return st2;
      break;  // not eligible after all: the direct kernel
    }
    case kMfmaA16W16: {
      const int st2 = conv2d_mfma_a16w16(x, w, d.n, d.h, d.w, d.ci, d.co, d.kh, d.kw, d.pad_h, d.pad_w, d.stride_h,
                                         d.stride_w, d.dil_h, d.dil_w, ho, wo, e, s);
      if (st2 >= 0) return st2;
      break;
    }
    default: break;
  }
  ConvDev cd = {d.n, d.h, d.w, d.ci, d.co, d.kh, d.kw, d.pad_h, d.pad_w, d.stride_h, d.stride_w,
                d.dil_h, d.dil_w, d.groups, ho, wo};
  return conv2d_direct(x, x_bits, w, w_bits, cd, e, s);
}

// shapes the two-branch kernel serves (pointer alignment is checked at the call)
static bool shortcut_fusable(int x_bits, int w_bits, const catchq_conv_desc_t *d, const catchq_shortcut_t *sc) {
  return x_bits == 8 && w_bits == 8 && sc->x_bits == 8 && sc->w_bits == 8 && d->groups == 1 && d->ci % 16 == 0 &&
         sc->ci % 16 == 0 && d->kh * d->kw <= 32 && d->co % 4 == 0 &&
         (int64_t)d->n * d->h * d->w * d->ci < (1ll << 31) && (int64_t)d->co * d->kh * d->kw * d->ci < (1ll << 31) &&
         (int64_t)d->n * sc->in_h * sc->in_w * sc->ci < (1ll << 31) && (int64_t)d->co * sc->ci < (1ll << 31);
}

static int check_shortcut(const catchq_conv_desc_t *d, const catchq_shortcut_t *sc, int ho, int wo) {
  if (!sc) return CATCHQ_ERR_ARG;
  if ((sc->x_bits != 8 && sc->x_bits != 16) || (sc->w_bits != 8 && sc->w_bits != 16)) return CATCHQ_ERR_BITWIDTH;
  if (sc->in_h <= 0 || sc->in_w <= 0 || sc->ci <= 0 || sc->stride <= 0) return CATCHQ_ERR_SHAPE;
  if (catchq_conv_out_size(sc->in_h, 1, 0, sc->stride, 1) != ho || catchq_conv_out_size(sc->in_w, 1, 0, sc->stride, 1) != wo)
    return CATCHQ_ERR_SHAPE;
  if (sc->exp2 < -126 || sc->exp2 > 126) return CATCHQ_ERR_ARG;
  return CATCHQ_OK;
}

CATCHQ_API int catchq_conv2d_shortcut_workspace_size(int x_bits, int w_bits, const catchq_conv_desc_t *desc,
                                                     const catchq_shortcut_t *shortcut, size_t *bytes) {
  int ho, wo;
  int st = check_conv(desc, &ho, &wo);
  if (st != CATCHQ_OK) return st;
  if (!bytes) return CATCHQ_ERR_ARG;
  if ((x_bits != 8 && x_bits != 16) || (w_bits != 8 && w_bits != 16)) return CATCHQ_ERR_BITWIDTH;
  st = check_shortcut(desc, shortcut, ho, wo);
  if (st != CATCHQ_OK) return st;
  *bytes = shortcut_fusable(x_bits, w_bits, desc, shortcut) ? 0 : (size_t)desc->n * ho * wo * desc->co * 4;
  return CATCHQ_OK;
}

CATCHQ_API int catchq_conv2d_shortcut_nhwc(const void *x, int x_bits, const void *w, int w_bits,
                                           const catchq_conv_desc_t *desc, const catchq_epilogue_t *epilogue,
                                           const catchq_shortcut_t *shortcut, void *workspace, size_t workspace_bytes,
                                           catchq_stream_t stream) {
  int ho, wo;
  int st = check_conv(desc, &ho, &wo);
  if (st != CATCHQ_OK) return st;
  if ((x_bits != 8 && x_bits != 16) || (w_bits != 8 && w_bits != 16)) return CATCHQ_ERR_BITWIDTH;
  st = check_epi(epilogue);
  if (st != CATCHQ_OK) return st;
  st = check_shortcut(desc, shortcut, ho, wo);
  if (st != CATCHQ_OK) return st;
  if (epilogue->resid) return CATCHQ_ERR_ARG;  // the shortcut is the residual
  if (desc->n == 0) return CATCHQ_OK;
  if (!x || !w || !shortcut->x || !shortcut->w) return CATCHQ_ERR_ARG;
  const catchq_conv_desc_t &d = *desc;
  const catchq_shortcut_t &sc = *shortcut;
  if (shortcut_fusable(x_bits, w_bits, desc, shortcut) && !epilogue->exp2_dev[0] && !epilogue->exp2_dev[1]) {
    EpiDev e = make_epi(epilogue, (int64_t)d.n * ho * wo * d.co);
    e.resid_after = epilogue->resid_after_act ? 1 : 0;
    ShortcutDev sd;
    sd.exp2 = sc.exp2;
    sd.chan_div = sc.chan_div;
    sd.chan_rcp = (sc.chan_div && sc.chan_rcp && sc.exp2 >= -64 && sc.exp2 <= 64) ? sc.chan_rcp : nullptr;
    sd.bias = sc.bias;
    const int st2 = conv2d_dual_i8(x, w, d.n, d.h, d.w, d.ci, d.co, d.kh, d.kw, d.pad_h, d.pad_w, d.stride_h, d.stride_w,
                                   d.dil_h, d.dil_w, ho, wo, sc.x, sc.w, sc.in_h, sc.in_w, sc.ci, sc.stride, e, sd,
                                   as_stream(stream));
    if (st2 >= 0) return st2;
  }
  // two launches: the shortcut's fp32 output goes through the workspace
  const size_t need = (size_t)d.n * ho * wo * d.co * 4;
  if (!workspace || workspace_bytes < need || !aligned16(workspace)) return CATCHQ_ERR_ARG;
  catchq_conv_desc_t ds = {d.n, sc.in_h, sc.in_w, sc.ci, d.co, 1, 1, 0, 0, sc.stride, sc.stride, 1, 1, 1};
  catchq_epilogue_t es;
  memset(&es, 0, sizeof(es));
  es.exp2 = sc.exp2;
  es.chan_div = sc.chan_div;
  es.chan_rcp = sc.chan_rcp;
  es.bias = sc.bias;
  es.y = workspace;
  es.y_dtype = CATCHQ_F32;
  st = catchq_conv2d_nhwc(sc.x, sc.x_bits, sc.w, sc.w_bits, &ds, &es, stream);
  if (st != CATCHQ_OK) return st;
  catchq_epilogue_t em = *epilogue;
  em.resid = (const float *)workspace;
  return catchq_conv2d_nhwc(x, x_bits, w, w_bits, desc, &em, stream);
}

CATCHQ_API int catchq_conv1x1_chain_nhwc(const catchq_chain_link_t *links, int nlinks, int n, int ho, int wo, int co,
                                         float *y, void *q, int q_position, int sharing, catchq_stream_t stream) {
  if (!links || n < 0 || ho <= 0 || wo <= 0 || co <= 0 || (!y && !q) || sharing < 0) return CATCHQ_ERR_ARG;
  if (nlinks < 2 || nlinks > CATCHQ_CHAIN_MAX_LINKS) return CATCHQ_ERR_UNSUPPORTED;
  if (q && (q_position < -126 || q_position > 126)) return CATCHQ_ERR_ARG;
  ChainLinkDev dev[CATCHQ_CHAIN_MAX_LINKS];
  for (int i = 0; i < nlinks; ++i) {
    const catchq_chain_link_t &l = links[i];
    if (l.in_h <= 0 || l.in_w <= 0 || l.ci <= 0 || l.stride <= 0) return CATCHQ_ERR_SHAPE;
    if (catchq_conv_out_size(l.in_h, 1, 0, l.stride, 1) != ho || catchq_conv_out_size(l.in_w, 1, 0, l.stride, 1) != wo)
      return CATCHQ_ERR_SHAPE;
    if (n > 0 && (!l.x || !l.w)) return CATCHQ_ERR_ARG;
    const int64_t xb = (int64_t)n * l.in_h * l.in_w * l.ci, wb = (int64_t)co * l.ci;
    if (xb >= (1ll << 31) || wb >= (1ll << 31) || l.ci % 64 != 0) return CATCHQ_ERR_UNSUPPORTED;
    // element strides of the taps, in 64 bits first: a huge stride on a one-pixel output grid passes the size checks
    const int64_t row_stride = (int64_t)l.stride * l.in_w * l.ci, pix_stride = (int64_t)l.stride * l.ci;
    if (row_stride >= (1ll << 31) || pix_stride >= (1ll << 31)) return CATCHQ_ERR_UNSUPPORTED;
    if (!l.chan_div || !l.chan_rcp || !l.bias || l.exp2 < -64 || l.exp2 > 64) return CATCHQ_ERR_UNSUPPORTED;
    dev[i].x = (const int8_t *)l.x;
    dev[i].w = (const int8_t *)l.w;
    dev[i].x_bytes = (unsigned)xb;
    dev[i].w_bytes = (unsigned)wb;
    dev[i].K = l.ci;
    dev[i].img_stride = (unsigned)(l.in_h * l.in_w * l.ci);
    dev[i].row_stride = (unsigned)row_stride;
    dev[i].pix_stride = (unsigned)pix_stride;
    dev[i].dense = (l.stride == 1 && l.in_h == ho && l.in_w == wo) ? 1 : 0;
    dev[i].k_shift = -1;
    dev[i].exp2 = l.exp2;
    dev[i].chan_div = l.chan_div;
    dev[i].chan_rcp = l.chan_rcp;
    dev[i].bias = l.bias;
  }
  if (n == 0) return CATCHQ_OK;
  const int st = conv1x1_chain_i8(dev, nlinks, n, ho, wo, co, y, (int8_t *)q, q_position, sharing, as_stream(stream));
  return st < 0 ? CATCHQ_ERR_UNSUPPORTED : st;
}

// shapes the head kernel serves (pointer alignment and the epilogue variant are checked at the call)
static bool head_fusable(const catchq_pointwise_head_t *hd, const catchq_conv_desc_t *d, const catchq_epilogue_t *e) {
  return d->groups == 1 && d->kh == 3 && d->kw == 3 && d->pad_h == 1 && d->pad_w == 1 && d->stride_h == 1 && d->stride_w == 1 &&
         d->dil_h == 1 && d->dil_w == 1 && hd->chan_div && hd->chan_rcp && hd->bias && hd->exp2 >= -64 && hd->exp2 <= 64 &&
         !e->exp2_dev[0] && !e->exp2_dev[1] && conv2d_head_halo_i8_ok(d->n, d->h, d->w, hd->ci, d->ci, d->co);
}

static int check_head(const catchq_pointwise_head_t *hd, const catchq_conv_desc_t *d) {
  if (!hd) return CATCHQ_ERR_ARG;
  if (hd->ci <= 0) return CATCHQ_ERR_SHAPE;
  if (hd->exp2 < -126 || hd->exp2 > 126 || hd->q_position < -126 || hd->q_position > 126) return CATCHQ_ERR_ARG;
  if (d->groups != 1) return CATCHQ_ERR_UNSUPPORTED;
  return CATCHQ_OK;
}

CATCHQ_API int catchq_conv1x1_conv3x3_workspace_size(const catchq_pointwise_head_t *head, const catchq_conv_desc_t *desc,
                                                     const catchq_epilogue_t *epilogue, size_t *bytes) {
  int ho, wo;
  int st = check_conv(desc, &ho, &wo);
  if (st != CATCHQ_OK) return st;
  if (!bytes) return CATCHQ_ERR_ARG;
  st = check_epi(epilogue);
  if (st != CATCHQ_OK) return st;
  st = check_head(head, desc);
  if (st != CATCHQ_OK) return st;
  *bytes = head_fusable(head, desc, epilogue) ? 0 : (size_t)desc->n * desc->h * desc->w * desc->ci;
  return CATCHQ_OK;
}

CATCHQ_API int catchq_conv1x1_conv3x3_nhwc(const void *x, const catchq_pointwise_head_t *head, const void *w,
                                           const catchq_conv_desc_t *desc, const catchq_epilogue_t *epilogue,
                                           void *workspace, size_t workspace_bytes, catchq_stream_t stream) {
  int ho, wo;
  int st = check_conv(desc, &ho, &wo);
  if (st != CATCHQ_OK) return st;
  st = check_epi(epilogue);
  if (st != CATCHQ_OK) return st;
  st = check_head(head, desc);
  if (st != CATCHQ_OK) return st;
  if (desc->n == 0) return CATCHQ_OK;
  if (!x || !w || !head->w) return CATCHQ_ERR_ARG;
  const catchq_conv_desc_t &d = *desc;
  if (head_fusable(head, desc, epilogue)) {
    const EpiDev e = make_epi(epilogue, (int64_t)d.n * ho * wo * d.co);
    const int st2 = conv2d_head_halo_i8(x, head->ci, head->w, head->chan_div, head->chan_rcp, head->bias, head->exp2,
                                        head->q_position, w, d.n, d.h, d.w, d.ci, d.co, e, as_stream(stream));
    if (st2 >= 0) return st2;
  }
  // two launches: the head's int8 output goes through the workspace
  const size_t need = (size_t)d.n * d.h * d.w * d.ci;
  if (!workspace || workspace_bytes < need || !aligned16(workspace)) return CATCHQ_ERR_ARG;
  catchq_conv_desc_t dh = {d.n, d.h, d.w, head->ci, d.ci, 1, 1, 0, 0, 1, 1, 1, 1, 1};
  catchq_epilogue_t eh;
  memset(&eh, 0, sizeof(eh));
  eh.exp2 = head->exp2;
  eh.chan_div = head->chan_div;
  eh.chan_rcp = head->chan_rcp;
  eh.bias = head->bias;
  eh.act = CATCHQ_ACT_RELU;
  eh.q = workspace;
  eh.q_bitwidth = 8;
  eh.q_position = head->q_position;
  eh.q_scale = 1.0f;
  eh.sharing = epilogue->sharing;
  st = catchq_conv2d_nhwc(x, 8, head->w, 8, &dh, &eh, stream);
  if (st != CATCHQ_OK) return st;
  return catchq_conv2d_nhwc(workspace, 8, w, 8, desc, epilogue, stream);
}

static size_t round256(size_t v) { return (v + 255) / 256 * 256; }

// shapes and constants the inverted-residual kernel serves (pointer alignment and the epilogue are checked at the call)
static bool irb_fusable(int n, int h, int w, int ci, int hid, int co, int stride, const catchq_requant_stage_t *s1,
                        const catchq_requant_stage_t *s2, const catchq_epilogue_t *e) {
  auto stage_ok = [](const catchq_requant_stage_t *s) {
    return s->chan_div && s->chan_rcp && s->bias && s->exp2 >= -64 && s->exp2 <= 64;
  };
  return stage_ok(s1) && stage_ok(s2) && !e->exp2_dev[0] && !e->exp2_dev[1] && !e->acc_out &&
         irb_i8_ok(n, h, w, ci, hid, co, stride, planned_cus(e->sharing));
}

static int check_irb(int n, int h, int w, int ci, int hid, int co, int stride, const catchq_requant_stage_t *s1,
                     const catchq_requant_stage_t *s2, const catchq_epilogue_t *e) {
  if (!s1 || !s2) return CATCHQ_ERR_ARG;
  if (n < 0 || h <= 0 || w <= 0 || ci <= 0 || hid <= 0 || co <= 0 || stride <= 0) return CATCHQ_ERR_SHAPE;
  const int st = check_epi(e);
  if (st != CATCHQ_OK) return st;
  for (const catchq_requant_stage_t *s : {s1, s2}) {
    if (s->act != CATCHQ_ACT_RELU && s->act != CATCHQ_ACT_RELU6) return CATCHQ_ERR_ARG;
    if (s->exp2 < -126 || s->exp2 > 126 || s->q_position < -126 || s->q_position > 126) return CATCHQ_ERR_ARG;
  }
  return CATCHQ_OK;
}

CATCHQ_API int catchq_inverted_residual_workspace_size(int n, int h, int w, int ci, int hid, int co, int stride,
                                                       const catchq_requant_stage_t *expand,
                                                       const catchq_requant_stage_t *depthwise,
                                                       const catchq_epilogue_t *epilogue, size_t *bytes) {
  const int st = check_irb(n, h, w, ci, hid, co, stride, expand, depthwise, epilogue);
  if (st != CATCHQ_OK) return st;
  if (!bytes) return CATCHQ_ERR_ARG;
  const int ho = catchq_conv_out_size(h, 3, 1, stride, 1), wo = catchq_conv_out_size(w, 3, 1, stride, 1);
  if (ho <= 0 || wo <= 0) return CATCHQ_ERR_SHAPE;
  *bytes = irb_fusable(n, h, w, ci, hid, co, stride, expand, depthwise, epilogue)
               ? 0 : round256((size_t)n * h * w * hid) + round256((size_t)n * ho * wo * hid);
  return CATCHQ_OK;
}

CATCHQ_API int catchq_inverted_residual_nhwc(const void *x, int n, int h, int w, int ci, int hid, int co, int stride,
                                             const catchq_requant_stage_t *expand, const catchq_requant_stage_t *depthwise,
                                             const void *w_project, const catchq_epilogue_t *epilogue, void *workspace,
                                             size_t workspace_bytes, catchq_stream_t stream) {
  int st = check_irb(n, h, w, ci, hid, co, stride, expand, depthwise, epilogue);
  if (st != CATCHQ_OK) return st;
  const int ho = catchq_conv_out_size(h, 3, 1, stride, 1), wo = catchq_conv_out_size(w, 3, 1, stride, 1);
  if (ho <= 0 || wo <= 0) return CATCHQ_ERR_SHAPE;
  if (n == 0) return CATCHQ_OK;
  if (!x || !w_project || !expand->w || !depthwise->w) return CATCHQ_ERR_ARG;
  if (irb_fusable(n, h, w, ci, hid, co, stride, expand, depthwise, epilogue) && aligned16(x) && aligned16(expand->w) &&
      aligned16(depthwise->w) && aligned16(w_project) && aligned16(expand->chan_div) && aligned16(expand->chan_rcp) &&
      aligned16(expand->bias) && aligned16(depthwise->chan_div) && aligned16(depthwise->chan_rcp) && aligned16(depthwise->bias)) {
    const EpiDev e = make_epi(epilogue, (int64_t)n * ho * wo * co);
    const IrbStageDev s1 = {(const int8_t *)expand->w, expand->chan_div, expand->chan_rcp, expand->bias, expand->exp2,
                            -expand->q_position, expand->act == CATCHQ_ACT_RELU6 ? 1 : 0};
    const IrbStageDev s2 = {(const int8_t *)depthwise->w, depthwise->chan_div, depthwise->chan_rcp, depthwise->bias,
                            depthwise->exp2, -depthwise->q_position, depthwise->act == CATCHQ_ACT_RELU6 ? 1 : 0};
    const int st2 = irb_i8(x, n, h, w, ci, hid, co, stride, s1, s2, w_project, e, as_stream(stream));
    if (st2 >= 0) return st2;
  }
  // three launches: the two hidden tensors go through the workspace
  const size_t b1 = round256((size_t)n * h * w * hid), b2 = round256((size_t)n * ho * wo * hid);
  if (!workspace || workspace_bytes < b1 + b2 || !aligned16(workspace)) return CATCHQ_ERR_ARG;
  void *q1 = workspace, *q2 = (char *)workspace + b1;
  auto stage_epi = [&](const catchq_requant_stage_t *s, void *q) {
    catchq_epilogue_t es;
    memset(&es, 0, sizeof(es));
    es.exp2 = s->exp2;
    es.chan_div = s->chan_div;
    es.chan_rcp = s->chan_rcp;
    es.bias = s->bias;
    es.act = s->act;
    es.q = q;
    es.q_bitwidth = 8;
    es.q_position = s->q_position;
    es.q_scale = 1.0f;
    es.sharing = epilogue->sharing;
    return es;
  };
  const catchq_conv_desc_t d1 = {n, h, w, ci, hid, 1, 1, 0, 0, 1, 1, 1, 1, 1};
  const catchq_epilogue_t e1 = stage_epi(expand, q1);
  st = catchq_conv2d_nhwc(x, 8, expand->w, 8, &d1, &e1, stream);
  if (st != CATCHQ_OK) return st;
  const catchq_conv_desc_t d2 = {n, h, w, hid, hid, 3, 3, 1, 1, stride, stride, 1, 1, hid};
  const catchq_epilogue_t e2 = stage_epi(depthwise, q2);
  st = catchq_conv2d_nhwc(q1, 8, depthwise->w, 8, &d2, &e2, stream);
  if (st != CATCHQ_OK) return st;
  const catchq_conv_desc_t d3 = {n, ho, wo, hid, co, 1, 1, 0, 0, 1, 1, 1, 1, 1};
  return catchq_conv2d_nhwc(q2, 8, w_project, 8, &d3, epilogue, stream);
}

// ---- first layers: quantizer + few-channel convolution + max pooling ------------------------------------------------
struct FirstLayersShape {
  int kw4, fh, fw, hc, wc, hp, wp;
};

static int check_first_layers(int n, int c, int h, int w, int co, int kh, int kw, int stride, int pad,
                              const catchq_requant_stage_t *conv, int pool_k, int pool_stride, int pool_pad,
                              FirstLayersShape *sh) {
  if (!conv) return CATCHQ_ERR_ARG;
  if (n < 0 || c <= 0 || c > 4 || h <= 0 || w <= 0 || co <= 0 || kh <= 0 || kw <= 0 || stride <= 0 || pad < 0 ||
      pool_k <= 0 || pool_stride <= 0 || pool_pad < 0 || 2 * pool_pad > pool_k)
    return CATCHQ_ERR_SHAPE;
  if (conv->act != CATCHQ_ACT_RELU && conv->act != CATCHQ_ACT_RELU6) return CATCHQ_ERR_ARG;
  if (conv->exp2 < -126 || conv->exp2 > 126 || conv->q_position < -126 || conv->q_position > 126) return CATCHQ_ERR_ARG;
  sh->kw4 = (kw + 3) / 4 * 4;
  sh->fh = h + 2 * pad;
  sh->fw = w + 2 * pad + sh->kw4 - kw;
  sh->hc = catchq_conv_out_size(h, kh, pad, stride, 1);
  sh->wc = catchq_conv_out_size(w, kw, pad, stride, 1);
  if (sh->hc <= 0 || sh->wc <= 0) return CATCHQ_ERR_SHAPE;
  sh->hp = catchq_conv_out_size(sh->hc, pool_k, pool_pad, pool_stride, 1);
  sh->wp = catchq_conv_out_size(sh->wc, pool_k, pool_pad, pool_stride, 1);
  if (sh->hp <= 0 || sh->wp <= 0) return CATCHQ_ERR_SHAPE;
  return CATCHQ_OK;
}

static bool first_layers_fusable(int n, int c, int h, int w, int co, int kh, int kw, int stride, int pad,
                                 const catchq_requant_stage_t *conv, int pool_k, int pool_stride, int pool_pad,
                                 int sharing) {
  return kh == 7 && kw == 7 && stride == 2 && pad == 3 && pool_k == 3 && pool_stride == 2 && pool_pad == 1 &&
         conv->chan_div && conv->chan_rcp && conv->bias && conv->exp2 >= -64 && conv->exp2 <= 64 &&
         stem_pool_i8_ok(n, c, h, w, co);
}

CATCHQ_API int catchq_first_layers_workspace_size(int n, int c, int h, int w, int co, int kh, int kw, int stride,
                                                  int pad, const catchq_requant_stage_t *conv, int pool_k,
                                                  int pool_stride, int pool_pad, int sharing, size_t *bytes) {
  FirstLayersShape sh;
  const int st = check_first_layers(n, c, h, w, co, kh, kw, stride, pad, conv, pool_k, pool_stride, pool_pad, &sh);
  if (st != CATCHQ_OK) return st;
  if (!bytes) return CATCHQ_ERR_ARG;
  *bytes = first_layers_fusable(n, c, h, w, co, kh, kw, stride, pad, conv, pool_k, pool_stride, pool_pad, sharing)
               ? 0 : round256((size_t)n * sh.fh * sh.fw * 4) + round256((size_t)n * sh.hc * sh.wc * co);
  return CATCHQ_OK;
}

CATCHQ_API int catchq_first_layers_nchw(const float *x, int n, int c, int h, int w, int x_position, float x_scale,
                                        int co, int kh, int kw, int stride, int pad,
                                        const catchq_requant_stage_t *conv, int pool_k, int pool_stride, int pool_pad,
                                        void *q, int sharing, void *workspace, size_t workspace_bytes,
                                        catchq_stream_t stream) {
  FirstLayersShape sh;
  int st = check_first_layers(n, c, h, w, co, kh, kw, stride, pad, conv, pool_k, pool_stride, pool_pad, &sh);
  if (st != CATCHQ_OK) return st;
  if (x_position < -126 || x_position > 126) return CATCHQ_ERR_ARG;
  if (n == 0) return CATCHQ_OK;
  if (!x || !q || !conv->w) return CATCHQ_ERR_ARG;
  if (first_layers_fusable(n, c, h, w, co, kh, kw, stride, pad, conv, pool_k, pool_stride, pool_pad, sharing) &&
      aligned16(x) && aligned16(conv->w) && aligned16(q)) {
    const IrbStageDev s = {(const int8_t *)conv->w, conv->chan_div, conv->chan_rcp, conv->bias, conv->exp2,
                           -conv->q_position, conv->act == CATCHQ_ACT_RELU6 ? 1 : 0};
    const int st2 = stem_pool_i8(x, n, c, h, w, x_position, x_scale, s, co, q, as_stream(stream));
    if (st2 >= 0) return st2;
  }
  // three launches: the framed int8 image and the convolution's output go through the workspace
  const size_t b1 = round256((size_t)n * sh.fh * sh.fw * 4), b2 = round256((size_t)n * sh.hc * sh.wc * co);
  if (!workspace || workspace_bytes < b1 + b2 || !aligned16(workspace)) return CATCHQ_ERR_ARG;
  void *qx = workspace, *q1 = (char *)workspace + b1;
  st = catchq_quantize_nchw_to_nhwc_frame(x, CATCHQ_F32, qx, 8, n, c, h, w, 4, sh.fh, sh.fw, pad, pad, x_position, x_scale,
                                          stream);
  if (st != CATCHQ_OK) return st;
  catchq_epilogue_t es;
  memset(&es, 0, sizeof(es));
  es.exp2 = conv->exp2;
  es.chan_div = conv->chan_div;
  es.chan_rcp = conv->chan_rcp;
  es.bias = conv->bias;
  es.act = conv->act;
  es.q = q1;
  es.q_bitwidth = 8;
  es.q_position = conv->q_position;
  es.q_scale = 1.0f;
  es.sharing = sharing;
  const catchq_conv_desc_t d = {n, sh.fh, sh.fw, 4, co, kh, sh.kw4, 0, 0, stride, stride, 1, 1, 1};
  st = catchq_conv2d_nhwc(qx, 8, conv->w, 8, &d, &es, stream);
  if (st != CATCHQ_OK) return st;
  return catchq_maxpool_nhwc(q1, q, 8, n, sh.hc, sh.wc, co, pool_k, pool_stride, pool_pad, stream);
}

// ---- 1x1 convolution + global average pooling ---------------------------------------------------------------------------
static int check_conv_avgpool(int n, int hw, int ci, int co, const catchq_epilogue_t *e) {
  if (n < 0 || hw <= 0 || ci <= 0 || co <= 0) return CATCHQ_ERR_SHAPE;
  if (!e || e->y || e->q || e->acc_out || (e->resid && e->resid_after_act)) return CATCHQ_ERR_ARG;  // the output is not stored
  if (e->act < CATCHQ_ACT_NONE || e->act > CATCHQ_ACT_LEAKY || e->exp2 < -126 || e->exp2 > 126 || e->sharing < 0)
    return CATCHQ_ERR_ARG;
  return CATCHQ_OK;
}

static bool conv_avgpool_fusable(int n, int hw, int ci, int co, const catchq_epilogue_t *e) {
  return e->chan_div && e->chan_rcp && e->bias && e->exp2 >= -64 && e->exp2 <= 64 && !e->exp2_dev[0] && !e->exp2_dev[1] &&
         !e->half_steps && (e->act == CATCHQ_ACT_NONE || e->act == CATCHQ_ACT_RELU || e->act == CATCHQ_ACT_RELU6) &&
         conv1x1_gap_i8_ok(n, hw, ci, co);
}

CATCHQ_API int catchq_conv1x1_avgpool_workspace_size(int n, int hw, int ci, int co, const catchq_epilogue_t *epilogue,
                                                     size_t *bytes) {
  const int st = check_conv_avgpool(n, hw, ci, co, epilogue);
  if (st != CATCHQ_OK) return st;
  if (!bytes) return CATCHQ_ERR_ARG;
  *bytes = conv_avgpool_fusable(n, hw, ci, co, epilogue) ? 0 : (size_t)n * hw * co * 4;
  return CATCHQ_OK;
}

CATCHQ_API int catchq_conv1x1_avgpool_nhwc(const void *x, const void *w, int n, int hw, int ci, int co,
                                           const catchq_epilogue_t *epilogue, float *mean, void *q, int q_bitwidth,
                                           int q_position, float q_scale, void *workspace, size_t workspace_bytes,
                                           catchq_stream_t stream) {
  int st = check_conv_avgpool(n, hw, ci, co, epilogue);
  if (st != CATCHQ_OK) return st;
  if (q && q_bitwidth != 8 && q_bitwidth != 16) return CATCHQ_ERR_BITWIDTH;
  if (q_position < -126 || q_position > 126) return CATCHQ_ERR_ARG;
  if (!mean && !q) return CATCHQ_ERR_ARG;
  if (n == 0) return CATCHQ_OK;
  if (!x || !w) return CATCHQ_ERR_ARG;
  if (conv_avgpool_fusable(n, hw, ci, co, epilogue) && aligned16(x) && aligned16(w) && aligned16(epilogue->chan_div) &&
      aligned16(epilogue->chan_rcp) && aligned16(epilogue->bias) && aligned16(epilogue->resid)) {
    const GapConvDev e = {epilogue->chan_div, epilogue->chan_rcp, epilogue->bias, epilogue->resid, epilogue->exp2,
                          epilogue->act, mean, q, q_bitwidth, -q_position, q_scale};
    const int st2 = conv1x1_gap_i8(x, w, n, hw, ci, co, e, as_stream(stream));
    if (st2 >= 0) return st2;
  }
  // two launches: the convolution's fp32 output goes through the workspace
  const size_t need = (size_t)n * hw * co * 4;
  if (!workspace || workspace_bytes < need || !aligned16(workspace)) return CATCHQ_ERR_ARG;
  catchq_epilogue_t ec = *epilogue;
  ec.y = workspace;
  ec.y_dtype = CATCHQ_F32;
  const catchq_conv_desc_t d = {n, hw, 1, ci, co, 1, 1, 0, 0, 1, 1, 1, 1, 1};
  st = catchq_conv2d_nhwc(x, 8, w, 8, &d, &ec, stream);
  if (st != CATCHQ_OK) return st;
  if (mean) {
    st = catchq_global_avgpool_nhwc((const float *)workspace, mean, n, hw, co, stream);
    if (st != CATCHQ_OK) return st;
  }
  if (q) return catchq_global_avgpool_quantize_nhwc((const float *)workspace, q, q_bitwidth, n, hw, co, q_position, q_scale, stream);
  return CATCHQ_OK;
}

CATCHQ_API int catchq_quantize_conv2d_workspace_size(const catchq_conv_desc_t *desc, int x_bits, int w_bits,
                                                     size_t *bytes) {
  int ho, wo;
  int st = check_conv(desc, &ho, &wo);
  if (st != CATCHQ_OK) return st;
  if (!bytes) return CATCHQ_ERR_ARG;
  if ((x_bits != 8 && x_bits != 16) || (w_bits != 8 && w_bits != 16)) return CATCHQ_ERR_BITWIDTH;
  const size_t xe = (size_t)desc->n * desc->h * desc->w * desc->ci;
  const size_t we = (size_t)desc->co * desc->kh * desc->kw * (desc->ci / desc->groups);
  *bytes = round256(xe * (x_bits / 8)) + round256(we * (w_bits / 8));
  return CATCHQ_OK;
}

CATCHQ_API int catchq_quantize_conv2d_nhwc(const void *x, int x_dtype, const int32_t *x_position_dev, int x_bits,
                                           const void *w, int w_dtype, const int32_t *w_position_dev, int w_bits,
                                           const catchq_conv_desc_t *desc, const float *bias, void *y, int y_dtype,
                                           void *workspace, size_t workspace_bytes, catchq_stream_t stream) {
  size_t need = 0;
  int st = catchq_quantize_conv2d_workspace_size(desc, x_bits, w_bits, &need);
  if (st != CATCHQ_OK) return st;
  if (desc->n == 0) return CATCHQ_OK;
  if (!x || !w || !y || !x_position_dev || !w_position_dev || !workspace) return CATCHQ_ERR_ARG;
  if (workspace_bytes < need || !aligned16(workspace)) return CATCHQ_ERR_ARG;
  const int64_t xe = (int64_t)desc->n * desc->h * desc->w * desc->ci;
  const int64_t we = (int64_t)desc->co * desc->kh * desc->kw * (desc->ci / desc->groups);
  void *qx = workspace;
  void *qw = (char *)workspace + round256((size_t)xe * (x_bits / 8));
  st = catchq_quantize_devpos(x, x_dtype, qx, x_bits, xe, x_position_dev, nullptr, stream);
  if (st != CATCHQ_OK) return st;
  st = catchq_quantize_devpos(w, w_dtype, qw, w_bits, we, w_position_dev, nullptr, stream);
  if (st != CATCHQ_OK) return st;
  catchq_epilogue_t e;
  memset(&e, 0, sizeof(e));
  e.exp2_dev[0] = x_position_dev;
  e.exp2_dev[1] = w_position_dev;
  e.bias = bias;
  e.y = y;
  e.y_dtype = y_dtype;
  return catchq_conv2d_nhwc(qx, x_bits, qw, w_bits, desc, &e, stream);
}
