// Last convolution of a residual block together with the block's projection shortcut, one launch:
//
//     out = act( dequant(conv(x, w)) + bias  +  [ dequant(conv1x1(x_sc, w_sc)) + bias_sc ] )
//
// Run as two launches, the shortcut writes an fp32 tensor of the output's size and the main
// convolution reads it back: 8 bytes per output element next to the 5 (fp32 + int8) the block's result
// itself costs.  Here both integer contractions run over the same output tile, one after the other
// through the same LDS ring, into two sets of accumulators; the epilogue dequantizes the shortcut's
// sums with the shortcut's own constants (the arithmetic of a stand-alone launch, so the values are
// the ones it would have stored) and uses them as the residual.  Nothing of the shortcut touches HBM
// except its operands.
#include "igemm_i8_dma.inc"

namespace catchq {

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int EPI>
__global__ __launch_bounds__(64 * WAVES_M *WAVES_N, 2) void igemm_i8_dual_kernel(
    const int8_t *__restrict__ X, const int8_t *__restrict__ W, IgemmParams p, unsigned x_bytes, unsigned w_bytes,
    const int8_t *__restrict__ XS, const int8_t *__restrict__ WS, IgemmParams ps, unsigned xs_bytes, unsigned ws_bytes,
    EpiDev e, ShortcutDev sc) {
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int EPI_STRIDE = WN + 8;
  extern __shared__ __attribute__((aligned(16))) int8_t lds_dyn[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;

  const int logical = xcd_remap(blockIdx.x, p.nblocks);
  const int tile_n = logical % p.tiles_n;
  const int tile_m = logical / p.tiles_n;
  const int64_t m0 = (int64_t)tile_m * BM;
  const int n0 = tile_n * BN;

  v16i acc_sc[TM][TN], acc[TM][TN];
  dma_mainloop<BM, BN, WAVES_M, WAVES_N, STAGES, LOAD_CONV, 64>(XS, WS, ps, xs_bytes, ws_bytes, m0, n0, lane, wave,
                                                                 lds_dyn, acc_sc);
  dma_mainloop<BM, BN, WAVES_M, WAVES_N, STAGES, LOAD_CONV, 64>(X, W, p, x_bytes, w_bytes, m0, n0, lane, wave, lds_dyn,
                                                                 acc);
  int *stage = reinterpret_cast<int *>(lds_dyn) + wave * 32 * EPI_STRIDE;
  igemm_epilogue_dual<TM, TN, EPI>(acc, acc_sc, stage, m0 + wave_m * WM, n0 + wave_n * WN, lane, p, e, sc);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int EPI>
static int launch_dual_epi(const void *x, const void *w, const IgemmParams &p, int64_t x_bytes, int64_t w_bytes,
                           const void *xs, const void *ws, const IgemmParams &ps, int64_t xs_bytes, int64_t ws_bytes,
                           const EpiDev &e, const ShortcutDev &sc, hipStream_t s) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int PIPE_BYTES = STAGES * (BM + BN) * 64;
  constexpr int EPI_BYTES = NW * 32 * (BN / WAVES_N + 8) * 4;
  constexpr int LDS_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;
  static_assert(LDS_BYTES <= 64 * 1024, "these tiles stay within the default dynamic LDS limit");
  igemm_i8_dual_kernel<BM, BN, WAVES_M, WAVES_N, STAGES, EPI><<<p.nblocks, 64 * NW, LDS_BYTES, s>>>(
      (const int8_t *)x, (const int8_t *)w, p, (unsigned)x_bytes, (unsigned)w_bytes, (const int8_t *)xs,
      (const int8_t *)ws, ps, (unsigned)xs_bytes, (unsigned)ws_bytes, e, sc);
  return launch_status();
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES>
static int launch_dual(const void *x, const void *w, IgemmParams p, int64_t x_bytes, int64_t w_bytes, const void *xs,
                       const void *ws, const IgemmParams &ps, int64_t xs_bytes, int64_t ws_bytes, const EpiDev &e,
                       const ShortcutDev &sc, hipStream_t s) {
  const int64_t tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const int64_t nb = tiles_m * p.tiles_n;
  if (nb > 0x7fffffff) return CATCHQ_ERR_SHAPE;
  p.nblocks = (int)nb;
  // the end of a residual block (reciprocal-form dequant, bias, ReLU, fp32 + int8 out) has its own instance
  EpiDev probe = e;
  probe.resid = reinterpret_cast<const float *>(e.y ? e.y : e.q);  // any 16-byte aligned non-null pointer
  if (pick_epilogue(p.N, probe) == EPI_RES_Y_Q8)
    return launch_dual_epi<BM, BN, WAVES_M, WAVES_N, STAGES, EPI_RES_Y_Q8>(x, w, p, x_bytes, w_bytes, xs, ws, ps, xs_bytes,
                                                                          ws_bytes, e, sc, s);
  return launch_dual_epi<BM, BN, WAVES_M, WAVES_N, STAGES, EPI_VECTOR>(x, w, p, x_bytes, w_bytes, xs, ws, ps, xs_bytes,
                                                                      ws_bytes, e, sc, s);
}

// Main convolution [N,H,W,Ci] x [Co,kh,kw,Ci] plus a 1x1 shortcut [N,Hs,Ws,Cs] x [Co,Cs] with stride ss and
// no padding, whose output grid must be the main one's.  -1 when the shapes are not this kernel's.
int conv2d_dual_i8(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph, int pw,
                   int sh, int sw, int dh, int dw, int Ho, int Wo, const void *xs, const void *ws, int Hs, int Ws, int Cs,
                   int ss, const EpiDev &e, const ShortcutDev &sc, hipStream_t s) {
  if (Ci % 16 != 0 || Cs % 16 != 0 || kh * kw > 32) return -1;  // 16-byte chunks within one tap; one validity bit per tap
  if (e.exp2_a || e.exp2_b || e.resid || e.acc_out) return -1;
  const int64_t x_bytes = (int64_t)N * H * W * Ci, w_bytes = (int64_t)Co * kh * kw * Ci;
  const int64_t xs_bytes = (int64_t)N * Hs * Ws * Cs, ws_bytes = (int64_t)Co * Cs;
  // buffer offsets are 32-bit and 0x80000000 must stay out of range
  for (int64_t b : {x_bytes, w_bytes, xs_bytes, ws_bytes})
    if (b <= 0 || b >= (1ll << 31)) return -1;
  if (!aligned16(x) || !aligned16(w) || !aligned16(xs) || !aligned16(ws)) return -1;
  if (!vec_epilogue_ok(Co, e) || !aligned16(sc.chan_div) || !aligned16(sc.chan_rcp) || !aligned16(sc.bias)) return -1;
  IgemmParams p = {};
  p.M = (int64_t)N * Ho * Wo;
  p.N = Co;
  p.K = kh * kw * Ci;
  p.H = H; p.W = W; p.Ci = Ci; p.Ho = Ho; p.Wo = Wo;
  p.kh = kh; p.kw = kw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
  p.img_stride = (unsigned)(H * W * Ci); p.row_stride = (unsigned)(W * Ci); p.pix_stride = (unsigned)Ci;
  IgemmParams ps = {};
  ps.M = p.M;
  ps.N = Co;
  ps.K = Cs;
  ps.H = Hs; ps.W = Ws; ps.Ci = Cs; ps.Ho = Ho; ps.Wo = Wo;
  ps.kh = 1; ps.kw = 1; ps.ph = 0; ps.pw = 0; ps.sh = ss; ps.sw = ss; ps.dh = 1; ps.dw = 1;
  ps.img_stride = (unsigned)(Hs * Ws * Cs); ps.row_stride = (unsigned)(Ws * Cs); ps.pix_stride = (unsigned)Cs;

  // Measured on the four projection blocks of ResNet-50 (32 and 64 images, timed inside a HIP graph): the 64x128
  // tile is 1-7 % faster than 64x64 on every one of them (half the activation fetches per output; two accumulator
  // sets of a 128x128 tile would leave a single block per CU, which was 2x slower).
  int tile = p.N >= 128 ? 64128 : 64064;
  if (const char *t = tuning_env("CATCHQ_DUAL_TILE")) {  // tuning aid: BMxBN
    int bm = 0, bn = 0;
    if (sscanf(t, "%dx%d", &bm, &bn) == 2) tile = bm * 1000 + bn;
  }
  switch (tile) {
    case 64128: return launch_dual<64, 128, 2, 2, 3>(x, w, p, x_bytes, w_bytes, xs, ws, ps, xs_bytes, ws_bytes, e, sc, s);
    default: return launch_dual<64, 64, 2, 2, 3>(x, w, p, x_bytes, w_bytes, xs, ws, ps, xs_bytes, ws_bytes, e, sc, s);
  }
}

}  // namespace catchq
