// Streaming int8 GEMM for short K and narrow N: the pointwise (1x1) convolutions at the head of
// MobileNet-style networks, K = Ci <= 96 and N = Co <= 160, millions of rows.  Such a launch moves
// every byte once and does a few hundred operations per row, so it is bound by HBM, not by the
// matrix cores, and the tile machinery of the implicit-GEMM kernels (LDS ring, barriers, one block
// per tile) only adds latency.  Here
//   * the whole weight matrix lives in the registers of every wave as MFMA B fragments;
//   * a wave walks over groups of 32 rows; a lane loads its A fragment (16 bytes of one row)
//     straight from global memory -- rows are K contiguous bytes, so a wave reads 32 full rows --
//     and keeps the fragments of the next DEPTH groups in flight;
//   * no block-level synchronisation at all; the epilogue is the shared one (wave-private LDS
//     transposition, 4 consecutive channels per lane).
#include "igemm_common.h"

namespace catchq {

constexpr int PW_MAX_KS = 3;  // K <= 96; supported (K steps, N fragments) pairs: KS * NF <= 6
constexpr int PW_DEPTH = 3;   // row groups whose loads are in flight per wave
constexpr bool PW_FAST = false;  // the check-free copy of the epilogue costs occupancy here and gains nothing (measured)

// widest power-of-two run of 32-column fragments the epilogue handles in one go
constexpr int pw_part(int nf) { return nf >= 4 ? 4 : nf >= 2 ? 2 : 1; }

// the shared epilogue wants a power-of-two number of column fragments: NF = 3 goes as 2 + 1, 5 as 4 + 1
template <int NF, int EPI>
__device__ __forceinline__ void pw_epilogue(v16i (&acc)[1][NF], int *stage, int64_t m, int lane, const IgemmParams &p,
                                            const EpiDev &e, const EpiLane &l_head, const EpiLane &l_tail) {
  constexpr int P = pw_part(NF);
  if constexpr (P == NF) {
    igemm_epilogue_vec<1, NF, EPI, PW_FAST>(acc, stage, m, 0, lane, p, e, l_head);
  } else {
    v16i head[1][P], tail[1][NF - P];
#pragma unroll
    for (int j = 0; j < P; ++j) head[0][j] = acc[0][j];
#pragma unroll
    for (int j = P; j < NF; ++j) tail[0][j - P] = acc[0][j];
    igemm_epilogue_vec<1, P, EPI, PW_FAST>(head, stage, m, 0, lane, p, e, l_head);
    igemm_epilogue_vec<1, NF - P, EPI, PW_FAST>(tail, stage, m, P * 32, lane, p, e, l_tail);
  }
}

template <int KS, int NF, int EPI>
__global__ __launch_bounds__(256, 2) void pw_i8_kernel(const int8_t *__restrict__ A, const int8_t *__restrict__ B,
                                                   IgemmParams p, EpiDev e, int ngroups) {
  resolve_exp2(e);
  constexpr int EPI_STRIDE = pw_part(NF) * 32 + 8;
  extern __shared__ __attribute__((aligned(16))) int pw_lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int kofs = fhalf * 16;

  // weights -> B fragments: lane (n = j*32 + frow, K half = fhalf)
  v4i fb[KS][NF];  // KS = ceil(K / 32); the last step may be half empty
#pragma unroll
  for (int s = 0; s < KS; ++s)
#pragma unroll
    for (int j = 0; j < NF; ++j) {
      const int n = j * 32 + frow, k = s * 32 + kofs;
      fb[s][j] = v4i{0, 0, 0, 0};
      if (n < p.N && k < p.K) fb[s][j] = *reinterpret_cast<const v4i *>(B + (int64_t)n * p.K + k);
    }

  auto load_a = [&](int g, v4i (&fa)[KS]) {
    const int64_t m = (int64_t)g * 32 + frow;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int k = s * 32 + kofs;
      fa[s] = v4i{0, 0, 0, 0};
      if (g < ngroups && m < p.M && k < p.K) fa[s] = *reinterpret_cast<const v4i *>(A + m * p.K + k);
    }
  };

  // per-channel constants of this lane's four channels, for both column runs of the epilogue
  typedef typename EpiOf<EPI>::type S;
  constexpr int P = pw_part(NF), T = (NF > P) ? NF - P : 1;
  const int n_head = epi_lane_channel<P>(0, lane), n_tail = epi_lane_channel<T>(P * 32, lane);
  const EpiLane l_head = epi_lane_setup<S>(n_head, n_head < p.N, e);
  const EpiLane l_tail = epi_lane_setup<S>(n_tail, NF > P && n_tail < p.N, e);

  const int gw = blockIdx.x * 4 + wave, nw = gridDim.x * 4;
  v4i ring[PW_DEPTH][KS];
#pragma unroll
  for (int d = 0; d < PW_DEPTH; ++d) load_a(gw + d * nw, ring[d]);

  int *stage = pw_lds + wave * 32 * EPI_STRIDE;
  for (int g0 = gw; g0 < ngroups; g0 += PW_DEPTH * nw) {
#pragma unroll
    for (int d = 0; d < PW_DEPTH; ++d) {
      const int g = g0 + d * nw;
      if (g >= ngroups) break;  // wave-uniform
      v4i fa[KS];
#pragma unroll
      for (int s = 0; s < KS; ++s) fa[s] = ring[d][s];
      load_a(g + PW_DEPTH * nw, ring[d]);
      v16i acc[1][NF];
      const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < NF; ++j) acc[0][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0], fb[0][j], zero, 0, 0, 0);
#pragma unroll
      for (int s = 1; s < KS; ++s)
#pragma unroll
        for (int j = 0; j < NF; ++j)
          acc[0][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[s], fb[s][j], acc[0][j], 0, 0, 0);
      pw_epilogue<NF, EPI>(acc, stage, (int64_t)g * 32, lane, p, e, l_head, l_tail);
    }
  }
}

template <int KS, int NF, int EPI>
static int pw_launch(const void *a, const void *b, const IgemmParams &p, const EpiDev &e, hipStream_t s) {
  constexpr int LDS_BYTES = 4 * 32 * (pw_part(NF) * 32 + 8) * 4;
  const int64_t ngroups = (p.M + 31) / 32;
  if (ngroups > 0x7fffffff) return -1;
  int blocks = (int)((ngroups + 3) / 4);
  const int resident = 256 * (pw_part(NF) == 1 ? 8 : pw_part(NF) == 2 ? 4 : 2);  // blocks resident at once (LDS-limited)
  if (blocks > resident) blocks = resident;
  auto kern = pw_i8_kernel<KS, NF, EPI>;
  if (LDS_BYTES > 64 * 1024) {
    static std::atomic<bool> raised[64];
    if (raise_lds_limit((const void *)kern, LDS_BYTES, raised) != CATCHQ_OK) return CATCHQ_ERR_LAUNCH;
  }
  kern<<<blocks, 256, LDS_BYTES, s>>>((const int8_t *)a, (const int8_t *)b, p, e, (int)ngroups);
  return launch_status();
}

template <int KS, int NF>
static int pw_pick_epi(const void *a, const void *b, const IgemmParams &p, const EpiDev &e, hipStream_t s) {
  switch (pick_epilogue(p.N, e)) {
    case EPI_SCALAR: return -1;
    case EPI_Q8_RELU6: return pw_launch<KS, NF, EPI_Q8_RELU6>(a, b, p, e, s);
    case EPI_Q8_RELU: return pw_launch<KS, NF, EPI_Q8_RELU>(a, b, p, e, s);
    case EPI_LIN_Q8: return pw_launch<KS, NF, EPI_LIN_Q8>(a, b, p, e, s);
    case EPI_LIN_Y_Q8: return pw_launch<KS, NF, EPI_LIN_Y_Q8>(a, b, p, e, s);
    default: return pw_launch<KS, NF, EPI_VECTOR>(a, b, p, e, s);
  }
}

// acc[m][n] = sum_k a[m][k] * b[n][k] for short K and narrow N (K % 16 == 0, 16-byte aligned operands);
// -1 when the shape is not this kernel's
int gemm_nt_stream_i8(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e, hipStream_t s) {
  if (K > PW_MAX_KS * 32 || K % 16 != 0 || N > 160 || M < 4096) return -1;
  const int ks = (int)((K + 31) / 32), nf = (int)((N + 31) / 32);
  if (ks * nf > 6) return -1;
  IgemmParams p = {};
  p.M = M;
  p.N = (int)N;
  p.K = (int)K;
  switch (ks * 8 + nf) {
    case 1 * 8 + 1: return pw_pick_epi<1, 1>(a, b, p, e, s);
    case 1 * 8 + 2: return pw_pick_epi<1, 2>(a, b, p, e, s);
    case 1 * 8 + 3: return pw_pick_epi<1, 3>(a, b, p, e, s);
    case 1 * 8 + 4: return pw_pick_epi<1, 4>(a, b, p, e, s);
    case 1 * 8 + 5: return pw_pick_epi<1, 5>(a, b, p, e, s);
    case 2 * 8 + 1: return pw_pick_epi<2, 1>(a, b, p, e, s);
    case 2 * 8 + 2: return pw_pick_epi<2, 2>(a, b, p, e, s);
    case 2 * 8 + 3: return pw_pick_epi<2, 3>(a, b, p, e, s);
    case 3 * 8 + 1: return pw_pick_epi<3, 1>(a, b, p, e, s);
    case 3 * 8 + 2: return pw_pick_epi<3, 2>(a, b, p, e, s);
    default: return -1;
  }
}


// ---- few-channel first layer ----------------------------------------------------------------------
// Input [N, H, W, 4] int8 already framed by its zero padding, filter rows padded to KW4*4 taps
// (weights [Co][kh][KW4*4][4], the extra taps zero).  A filter row is then one contiguous run of
// KW4*16 bytes of an image row, and an MFMA K step of 32 bytes is one filter row (KW4 = 2) or two
// (KW4 = 1; the K half a lane owns selects the row).  Same streaming scheme as above: weights in
// registers, 32 consecutive output pixels per wave step, A fragments loaded straight from global
// memory (neighbouring pixels overlap, the L1 serves that), loads of the next group in flight.
typedef int v4i_a4 __attribute__((ext_vector_type(4), aligned(4)));

// STEPS = K steps of 32 bytes: kh for KW4 = 2, ceil(kh / 2) for KW4 = 1
template <int KW4, int STEPS, int EPI>
__global__ __launch_bounds__(256, 2) void stem_i8_kernel(const int8_t *__restrict__ X, const int8_t *__restrict__ B,
                                                        IgemmParams p, EpiDev e, int ngroups) {
  resolve_exp2(e);
  typedef typename EpiOf<EPI>::type S;
  constexpr int EPI_STRIDE = 32 + 8;
  constexpr int DEPTH = 2;
  extern __shared__ __attribute__((aligned(16))) int pw_lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int n_base = blockIdx.y * 32;  // 32 output channels per wave; blockIdx.y selects the group
  const int rowbytes = p.W * 4;
  // this lane's filter row in step s and its byte offset within the row's taps
  auto frag_row = [&](int s) { return (KW4 == 2) ? s : 2 * s + fhalf; };
  const int tapofs = (KW4 == 2) ? fhalf * 16 : 0;
  const bool last_ok = frag_row(STEPS - 1) < p.kh;  // odd kh with two rows per step: no row for the upper K half

  v4i fb[STEPS];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int n = n_base + frow, r = frag_row(s);
    fb[s] = v4i{0, 0, 0, 0};
    if (n < p.N && r < p.kh) fb[s] = *reinterpret_cast<const v4i *>(B + (int64_t)n * p.K + r * (KW4 * 16) + tapofs);
  }
  const int n_lane = epi_lane_channel<1>(n_base, lane);
  const EpiLane L = epi_lane_setup<S>(n_lane, n_lane < p.N, e);

  auto load_a = [&](int g, v4i (&fa)[STEPS]) {
    // 32-bit index arithmetic (the launcher checks M and the image size): 64-bit divisions would
    // cost more than the rest of the step
    const unsigned m = (unsigned)g * 32u + (unsigned)frow;
    const bool ok = g < ngroups && m < (unsigned)p.M;
    const unsigned mm = ok ? m : 0u;
    const unsigned t = mm / (unsigned)p.Wo, wo = mm - t * (unsigned)p.Wo;
    const unsigned img = t / (unsigned)p.Ho, ho = t - img * (unsigned)p.Ho;
    const int8_t *base = X + (size_t)((img * (unsigned)p.H + ho * (unsigned)p.sh) * (unsigned)p.W + wo * (unsigned)p.sw) * 4 + tapofs;
    // rows of lanes that are out of range read the first pixel's rows: harmless, their results are not stored
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      if (s == STEPS - 1 && KW4 == 1) {
        fa[s] = v4i{0, 0, 0, 0};
        if (last_ok) fa[s] = *reinterpret_cast<const v4i_a4 *>(base + (int64_t)frag_row(s) * p.dh * rowbytes);
      } else {
        fa[s] = *reinterpret_cast<const v4i_a4 *>(base + (int64_t)frag_row(s) * p.dh * rowbytes);
      }
    }
  };

  const int gw = blockIdx.x * 4 + wave, nw = gridDim.x * 4;
  v4i ring[DEPTH][STEPS];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load_a(gw + d * nw, ring[d]);

  int *stage = pw_lds + wave * 32 * EPI_STRIDE;
  for (int g0 = gw; g0 < ngroups; g0 += DEPTH * nw) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int g = g0 + d * nw;
      if (g >= ngroups) break;  // wave-uniform
      v16i acc[1][1];
      const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[d][0], fb[0], zero, 0, 0, 0);
#pragma unroll
      for (int s = 1; s < STEPS; ++s)
        acc[0][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ring[d][s], fb[s], acc[0][0], 0, 0, 0);
      load_a(g + DEPTH * nw, ring[d]);  // the matrix cores have read the old fragments by now
      igemm_epilogue_vec<1, 1, EPI>(acc, stage, (int64_t)g * 32, n_base, lane, p, e, L);
    }
  }
}

template <int KW4, int STEPS, int EPI>
static int stem_launch(const void *x, const void *w, const IgemmParams &p, const EpiDev &e, hipStream_t s) {
  constexpr int LDS_BYTES = 4 * 32 * (32 + 8) * 4;
  const int64_t ngroups = (p.M + 31) / 32;
  if (ngroups > 0x7fffffff) return -1;
  int blocks = (int)((ngroups + 3) / 4);
  const int ngrp = (p.N + 31) / 32;
  if (blocks > 256 * 4 / ngrp) blocks = 256 * 4 / ngrp;
  stem_i8_kernel<KW4, STEPS, EPI><<<dim3(blocks, ngrp), 256, LDS_BYTES, s>>>((const int8_t *)x, (const int8_t *)w, p, e, (int)ngroups);
  return launch_status();
}

template <int KW4, int STEPS>
static int stem_pick_epi(const void *x, const void *w, const IgemmParams &p, const EpiDev &e, hipStream_t s) {
  switch (pick_epilogue(p.N, e)) {
    case EPI_SCALAR: return -1;
    case EPI_Q8_RELU6: return stem_launch<KW4, STEPS, EPI_Q8_RELU6>(x, w, p, e, s);
    case EPI_Q8_RELU: return stem_launch<KW4, STEPS, EPI_Q8_RELU>(x, w, p, e, s);
    default: return stem_launch<KW4, STEPS, EPI_VECTOR>(x, w, p, e, s);
  }
}

// convolution of a framed 4-channel int8 image (no padding left to apply), kw in {4, 8} (zero taps
// included), Co <= 128; -1 when the shape is not this kernel's
int conv2d_stem_i8(const void *x, const void *w, int N, int H, int W, int Co, int kh, int kw, int sh, int sw, int dh,
                   int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  if ((kw != 4 && kw != 8) || Co > 128 || (int64_t)N * Ho * Wo < 4096) return -1;
  if ((int64_t)N * Ho * Wo >= (1ll << 31) - 64 || (int64_t)N * H * W >= (1ll << 30)) return -1;  // 32-bit indices
  const int steps = (kw == 8) ? kh : (kh + 1) / 2;
  IgemmParams p = {};
  p.M = (int64_t)N * Ho * Wo;
  p.N = Co;
  p.K = kh * kw * 4;
  p.H = H; p.W = W; p.Ho = Ho; p.Wo = Wo; p.kh = kh; p.kw = kw; p.sh = sh; p.sw = sw; p.dh = dh;
  // the instantiated shapes: 3x3 and 5x5 (rows of 4 or 8 taps), 7x7 (rows of 8 taps)
  if (kw == 4 && steps == 2) return stem_pick_epi<1, 2>(x, w, p, e, s);
  if (kw == 8 && steps == 5) return stem_pick_epi<2, 5>(x, w, p, e, s);
  if (kw == 8 && steps == 7) return stem_pick_epi<2, 7>(x, w, p, e, s);
  return -1;
}

}  // namespace catchq
