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

// widest power-of-two run of 32-column fragments the epilogue handles in one go
constexpr int pw_part(int nf) { return nf >= 4 ? 4 : nf >= 2 ? 2 : 1; }

// the shared epilogue wants a power-of-two number of column fragments: NF = 3 goes as 2 + 1, 5 as 4 + 1
template <int NF, int EPI>
__device__ __forceinline__ void pw_epilogue(v16i (&acc)[1][NF], int *stage, int64_t m, int lane, const IgemmParams &p,
                                            const EpiDev &e) {
  constexpr int P = pw_part(NF);
  if constexpr (P == NF) {
    igemm_epilogue<1, NF, EPI>(acc, stage, m, 0, lane, p, e);
  } else {
    v16i head[1][P], tail[1][NF - P];
#pragma unroll
    for (int j = 0; j < P; ++j) head[0][j] = acc[0][j];
#pragma unroll
    for (int j = P; j < NF; ++j) tail[0][j - P] = acc[0][j];
    igemm_epilogue<1, P, EPI>(head, stage, m, 0, lane, p, e);
    igemm_epilogue<1, NF - P, EPI>(tail, stage, m, P * 32, lane, p, e);
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
#pragma unroll
      for (int j = 0; j < NF; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[0][j][r] = 0;
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int j = 0; j < NF; ++j)
          acc[0][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[s], fb[s][j], acc[0][j], 0, 0, 0);
      pw_epilogue<NF, EPI>(acc, stage, (int64_t)g * 32, lane, p, e);
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
    static bool raised[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return CATCHQ_ERR_LAUNCH;
    if (!raised[dev]) {
      if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES) != hipSuccess)
        return CATCHQ_ERR_LAUNCH;
      raised[dev] = true;
    }
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

}  // namespace catchq
