// int8 x int8 -> int32 implicit GEMM on gfx950 matrix cores (v_mfma_i32_32x32x32_i8).
//
//   C[m][n] = sum_k A[m][k] * B[n][k]       B = weights [Co][K], K contiguous
//   GEMM:  A = activations [M][K]
//   CONV:  A = im2col view of an NHWC int8 tensor, m = (img,ho,wo), k = (r,q,ci); gathered on the
//          fly into LDS, never materialised.  Needs Ci % 16 == 0 so that a 16-byte K chunk stays
//          inside one filter tap.
//
// Block = 256 threads = 4 waves (2 x 2); block tile BM x BN, K step 64 bytes; LDS double
// buffered, global loads for step s+1 are in flight while step s is multiplied.  LDS rows are
// 64 bytes = four 16-byte chunks, chunk index XOR-swizzled with (row>>2)&3 so that both the
// ds_write_b128 of the loaders and the ds_read_b128 of the MFMA operand fetch are conflict free.
#include "catchq_common.h"

namespace catchq {

struct IgemmParams {
  int64_t M;
  int N, K;
  int H, W, Ci, Ho, Wo, kh, kw, ph, pw, sh, sw, dh, dw;
  int tiles_n;
  int nblocks;
};

constexpr int BK = 64;

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 2) & 3); }

template <int BM, int BN, bool CONV>
__global__ __launch_bounds__(256) void igemm_i8_kernel(const int8_t *__restrict__ A,
                                                      const int8_t *__restrict__ B, IgemmParams p,
                                                      EpiDev e) {
  constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int LA = BM / 64, LB = BN / 64;  // 16-byte chunks each thread loads per K step
  __shared__ __attribute__((aligned(16))) int8_t lds[2][(BM + BN) * BK];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;

  // block id -> tile, XCD-aware: ids that land on one XCD (id % 8) take a contiguous run of
  // tiles, so neighbouring tiles (same A rows, same weights) share that XCD's L2.
  int logical;
  {
    const int bid = blockIdx.x, nb = p.nblocks;
    const int xcd = bid & 7, local = bid >> 3;
    const int q = nb >> 3, rem = nb & 7;
    logical = xcd * q + (xcd < rem ? xcd : rem) + local;
  }
  const int tile_n = logical % p.tiles_n;
  const int tile_m = logical / p.tiles_n;
  const int64_t m0 = (int64_t)tile_m * BM;
  const int n0 = tile_n * BN;

  // ---- loader state -------------------------------------------------------------------------
  const int lc = tid & 3;    // chunk column 0..3 within the 64-byte K step
  const int lr = tid >> 2;   // row 0..63 (+64*i)
  const int8_t *a_ptr[LA];
  int a_hi0[LA], a_wi0[LA];
  bool a_ok[LA];
#pragma unroll
  for (int i = 0; i < LA; ++i) {
    const int64_t m = m0 + lr + 64 * i;
    a_ok[i] = m < p.M;
    if constexpr (CONV) {
      const int64_t mm = a_ok[i] ? m : 0;
      const int wo = (int)(mm % p.Wo);
      const int64_t t = mm / p.Wo;
      const int ho = (int)(t % p.Ho);
      const int64_t img = t / p.Ho;
      a_hi0[i] = ho * p.sh - p.ph;
      a_wi0[i] = wo * p.sw - p.pw;
      a_ptr[i] = A + img * p.H * p.W * p.Ci;
    } else {
      a_hi0[i] = a_wi0[i] = 0;
      a_ptr[i] = A + (a_ok[i] ? m : 0) * p.K;
    }
  }
  const int8_t *b_ptr[LB];
  bool b_ok[LB];
#pragma unroll
  for (int i = 0; i < LB; ++i) {
    const int n = n0 + lr + 64 * i;
    b_ok[i] = n < p.N;
    b_ptr[i] = B + (int64_t)(b_ok[i] ? n : 0) * p.K;
  }
  // position of this thread's chunk along K: k = step*64 + lc*16 = (r, q, ci)
  int k_lin = lc * 16;
  int kr = 0, kq = 0, kci = lc * 16;
  if constexpr (CONV) {
    while (kci >= p.Ci) {
      kci -= p.Ci;
      if (++kq == p.kw) { kq = 0; ++kr; }
    }
  }

  v4i ra[LA], rb[LB];
  auto load_global = [&]() {
    const bool k_ok = k_lin < p.K;
#pragma unroll
    for (int i = 0; i < LA; ++i) {
      v4i v = {0, 0, 0, 0};
      if constexpr (CONV) {
        const int hi = a_hi0[i] + kr * p.dh, wi = a_wi0[i] + kq * p.dw;
        if (k_ok && a_ok[i] && (unsigned)hi < (unsigned)p.H && (unsigned)wi < (unsigned)p.W)
          v = *reinterpret_cast<const v4i *>(a_ptr[i] + ((int64_t)hi * p.W + wi) * p.Ci + kci);
      } else {
        if (k_ok && a_ok[i]) v = *reinterpret_cast<const v4i *>(a_ptr[i] + k_lin);
      }
      ra[i] = v;
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      v4i v = {0, 0, 0, 0};
      if (k_ok && b_ok[i]) v = *reinterpret_cast<const v4i *>(b_ptr[i] + k_lin);
      rb[i] = v;
    }
  };
  auto advance_k = [&]() {
    k_lin += BK;
    if constexpr (CONV) {
      kci += BK;
      while (kci >= p.Ci) {
        kci -= p.Ci;
        if (++kq == p.kw) { kq = 0; ++kr; }
      }
    }
  };
  auto store_lds = [&](int buf) {
    int8_t *la = lds[buf];
    int8_t *lb = lds[buf] + BM * BK;
#pragma unroll
    for (int i = 0; i < LA; ++i) {
      const int row = lr + 64 * i;
      *reinterpret_cast<v4i *>(la + row * BK + swz(row, lc) * 16) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      const int row = lr + 64 * i;
      *reinterpret_cast<v4i *>(lb + row * BK + swz(row, lc) * 16) = rb[i];
    }
  };

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  const int nsteps = (p.K + BK - 1) / BK;
  load_global();
  advance_k();
  store_lds(0);
  __syncthreads();

  const int frow = lane & 31;   // operand row within a 32-row MFMA tile
  const int fhalf = lane >> 5;  // which 16-byte half of the 32-byte K slice

  for (int step = 0; step < nsteps; ++step) {
    const int buf = step & 1;
    if (step + 1 < nsteps) {
      load_global();
      advance_k();
    }
    const int8_t *la = lds[buf];
    const int8_t *lb = lds[buf] + BM * BK;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      v4i fa[TM], fb[TN];
      const int chunk = ks * 2 + fhalf;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = wave_m * WM + i * 32 + frow;
        fa[i] = *reinterpret_cast<const v4i *>(la + row * BK + swz(row, chunk) * 16);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int row = wave_n * WN + j * 32 + frow;
        fb[j] = *reinterpret_cast<const v4i *>(lb + row * BK + swz(row, chunk) * 16);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (step + 1 < nsteps) store_lds(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: lane holds column (lane&31), rows 8*(r/4) + 4*(lane>>5) + (r&3) ---------------
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wave_n * WN + j * 32 + frow;
      if (n >= p.N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = m0 + wave_m * WM + i * 32 + 8 * (r >> 2) + 4 * fhalf + (r & 3);
        if (m >= p.M) continue;
        const int64_t idx = m * p.N + n;
        const int a = acc[i][j][r];
        if (e.acc_out) e.acc_out[idx] = a;
        epi_store(epi_value((float)a, idx, n, e), idx, e);
      }
    }
  }
}

template <int BM, int BN, bool CONV>
static int launch_igemm(const void *a, const void *b, IgemmParams p, const EpiDev &e, hipStream_t s) {
  const int64_t tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const int64_t nb = tiles_m * p.tiles_n;
  if (nb > 0x7fffffff) return CATCHQ_ERR_SHAPE;
  p.nblocks = (int)nb;
  igemm_i8_kernel<BM, BN, CONV><<<(int)nb, 256, 0, s>>>((const int8_t *)a, (const int8_t *)b, p, e);
  return launch_status();
}

template <bool CONV>
static int pick_tile(const void *a, const void *b, const IgemmParams &p, const EpiDev &e, hipStream_t s) {
  if (p.N <= 64) return launch_igemm<128, 64, CONV>(a, b, p, e, s);
  return launch_igemm<128, 128, CONV>(a, b, p, e, s);
}

int gemm_nt_mfma_i8(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e,
                    hipStream_t s) {
  IgemmParams p = {};
  p.M = M;
  p.N = (int)N;
  p.K = (int)K;
  return pick_tile<false>(a, b, p, e, s);
}

int conv2d_mfma_i8(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph,
                   int pw, int sh, int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  IgemmParams p = {};
  p.M = (int64_t)N * Ho * Wo;
  p.N = Co;
  p.K = kh * kw * Ci;
  p.H = H; p.W = W; p.Ci = Ci; p.Ho = Ho; p.Wo = Wo;
  p.kh = kh; p.kw = kw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
  return pick_tile<true>(x, w, p, e, s);
}

}  // namespace catchq
