// int8 x int8 -> int32 implicit GEMM on gfx950 matrix cores (v_mfma_i32_32x32x32_i8).
//
//   C[m][n] = sum_k A[m][k] * B[n][k]       B = weights [Co][K], K contiguous
//   LOAD_GEMM:  A = activations [M][K]
//   LOAD_CONV:  A = im2col view of an NHWC int8 tensor, m = (img,ho,wo), k = (r,q,ci); gathered on
//               the fly into LDS, never materialised.  Needs Ci % 16 == 0 so that a 16-byte K chunk
//               stays inside one filter tap.
//   LOAD_C4:    the same for Ci == 4 (an RGB input padded to four channels): one pixel is one
//               dword, a 16-byte chunk is four horizontally adjacent taps of one filter row, and
//               k = (r, q padded to a multiple of 4, ci).  Taps beyond kw read zero weights.
//
// Block = 256 threads = 4 waves (2 x 2); block tile BM x BN, K step 64 bytes; LDS double
// buffered, global loads for step s+1 are in flight while step s is multiplied.  LDS rows are
// 64 bytes = four 16-byte chunks, chunk index XOR-swizzled with (row>>2)&3 so that both the
// ds_write_b128 of the loaders and the ds_read_b128 of the MFMA operand fetch are conflict free.
//
// Epilogue: each wave transposes its accumulators through LDS (32 rows at a time) so that a lane
// owns four consecutive output channels of one pixel; residual loads and all stores are then
// 16-byte (fp32) / 4-byte (int8) vectors and whole output rows are written contiguously.
#include "catchq_common.h"

namespace catchq {

struct IgemmParams {
  int64_t M;
  int N, K;
  int H, W, Ci, Ho, Wo, kh, kw, ph, pw, sh, sw, dh, dw;
  int kwq;  // LOAD_C4: chunks (groups of 4 taps) per filter row
  int tiles_n;
  int nblocks;
};

constexpr int BK = 64;
enum { LOAD_GEMM = 0, LOAD_CONV = 1, LOAD_C4 = 2 };

__device__ __forceinline__ int swz(int row, int chunk) { return chunk ^ ((row >> 2) & 3); }

// 16 bytes from a 4-byte aligned address
__device__ __forceinline__ v4i load16_a4(const int8_t *p) {
  struct __attribute__((packed, aligned(4))) P { v4i v; };
  return reinterpret_cast<const P *>(p)->v;
}

template <int BM, int BN, int LOAD, bool VEC_EPI>
__global__ __launch_bounds__(256) void igemm_i8_kernel(const int8_t *__restrict__ A,
                                                      const int8_t *__restrict__ B, IgemmParams p,
                                                      EpiDev e) {
  constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int LA = BM / 64, LB = BN / 64;  // 16-byte chunks each thread loads per K step
  constexpr int EPI_STRIDE = WN + 8;         // ints per staged row (+8: the two half-waves hit different banks)
  constexpr int PIPE_BYTES = 2 * (BM + BN) * BK;
  constexpr int EPI_BYTES = VEC_EPI ? 4 * 32 * EPI_STRIDE * 4 : 0;
  constexpr int LDS_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;
  __shared__ __attribute__((aligned(16))) int8_t lds_raw[LDS_BYTES];
  int8_t(*lds)[(BM + BN) * BK] = reinterpret_cast<int8_t(*)[(BM + BN) * BK]>(lds_raw);

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
  const int lc = tid & 3;   // chunk column 0..3 within the 64-byte K step
  const int lr = tid >> 2;  // row 0..63 (+64*i)
  const int8_t *a_ptr[LA];
  int a_hi0[LA], a_wi0[LA];
  bool a_ok[LA];
#pragma unroll
  for (int i = 0; i < LA; ++i) {
    const int64_t m = m0 + lr + 64 * i;
    a_ok[i] = m < p.M;
    if constexpr (LOAD != LOAD_GEMM) {
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
    if constexpr (LOAD == LOAD_C4) b_ptr[i] = B + (int64_t)(b_ok[i] ? n : 0) * p.kh * p.kw * 4;
    else b_ptr[i] = B + (int64_t)(b_ok[i] ? n : 0) * p.K;
  }
  // position of this thread's chunk along K: k = step*64 + lc*16 = (r, q, ci)   [LOAD_C4: (r, q0)]
  int k_lin = lc * 16;
  int kr = 0, kq = 0, kci = lc * 16;
  if constexpr (LOAD == LOAD_CONV) {
    while (kci >= p.Ci) {
      kci -= p.Ci;
      if (++kq == p.kw) { kq = 0; ++kr; }
    }
  } else if constexpr (LOAD == LOAD_C4) {
    kq = lc;  // chunk index within the filter row; one chunk = 4 taps
    while (kq >= p.kwq) { kq -= p.kwq; ++kr; }
  }

  v4i ra[LA], rb[LB];
  auto load_global = [&]() {
    const bool k_ok = k_lin < p.K;
#pragma unroll
    for (int i = 0; i < LA; ++i) {
      v4i v = {0, 0, 0, 0};
      if constexpr (LOAD == LOAD_CONV) {
        const int hi = a_hi0[i] + kr * p.dh, wi = a_wi0[i] + kq * p.dw;
        if (k_ok && a_ok[i] && (unsigned)hi < (unsigned)p.H && (unsigned)wi < (unsigned)p.W)
          v = *reinterpret_cast<const v4i *>(a_ptr[i] + ((int64_t)hi * p.W + wi) * p.Ci + kci);
      } else if constexpr (LOAD == LOAD_C4) {
        const int hi = a_hi0[i] + kr * p.dh, wi = a_wi0[i] + kq * 4;  // horizontal dilation 1 on this path
        if (k_ok && a_ok[i] && (unsigned)hi < (unsigned)p.H) {
          const int8_t *row = a_ptr[i] + (int64_t)hi * p.W * 4;
          if (wi >= 0 && wi + 3 < p.W) {
            v = load16_a4(row + wi * 4);
          } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
              if ((unsigned)(wi + t) < (unsigned)p.W) v[t] = *reinterpret_cast<const int *>(row + (wi + t) * 4);
          }
        }
      } else {
        if (k_ok && a_ok[i]) v = *reinterpret_cast<const v4i *>(a_ptr[i] + k_lin);
      }
      ra[i] = v;
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      v4i v = {0, 0, 0, 0};
      if constexpr (LOAD == LOAD_C4) {
        if (k_ok && b_ok[i]) {
          const int8_t *row = b_ptr[i] + (kr * p.kw + kq * 4) * 4;
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (kq * 4 + t < p.kw) v[t] = *reinterpret_cast<const int *>(row + t * 4);
        }
      } else {
        if (k_ok && b_ok[i]) v = *reinterpret_cast<const v4i *>(b_ptr[i] + k_lin);
      }
      rb[i] = v;
    }
  };
  auto advance_k = [&]() {
    k_lin += BK;
    if constexpr (LOAD == LOAD_CONV) {
      kci += BK;
      while (kci >= p.Ci) {
        kci -= p.Ci;
        if (++kq == p.kw) { kq = 0; ++kr; }
      }
    } else if constexpr (LOAD == LOAD_C4) {
      kq += 4;
      while (kq >= p.kwq) { kq -= p.kwq; ++kr; }
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

  // ---- epilogue -------------------------------------------------------------------------------
  // accumulator layout: lane holds column (lane&31), rows 8*(r/4) + 4*(lane>>5) + (r&3)
  if constexpr (!VEC_EPI) {
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
  } else {
    // N % 4 == 0 and all pointers 16-byte aligned (checked on the host)
    constexpr int CPR = WN / 4;    // 4-channel groups per staged row
    constexpr int RPI = 64 / CPR;  // rows the wave moves per iteration
    int *stage = reinterpret_cast<int *>(lds_raw) + wave * 32 * EPI_STRIDE;
    const int cg = lane % CPR, rsub = lane / CPR;
    const int n = n0 + wave_n * WN + cg * 4;
    const bool n_ok = n < p.N;
    v4f div = {1.f, 1.f, 1.f, 1.f}, bias = {0.f, 0.f, 0.f, 0.f};
    if (n_ok && e.chan_div) div = *reinterpret_cast<const v4f *>(e.chan_div + n);
    if (n_ok && e.bias) bias = *reinterpret_cast<const v4f *>(e.bias + n);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      // wave-private staging: stores then loads of the same wave, ordered by the LDS counter
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          stage[(8 * (r >> 2) + 4 * fhalf + (r & 3)) * EPI_STRIDE + j * 32 + frow] = acc[i][j][r];
      const int64_t mbase = m0 + wave_m * WM + i * 32;
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int row = it * RPI + rsub;
        const int64_t m = mbase + row;
        const v4i a = *reinterpret_cast<const v4i *>(stage + row * EPI_STRIDE + cg * 4);
        if (!n_ok || m >= p.M) continue;
        const int64_t idx = m * p.N + n;
        if (e.acc_out) *reinterpret_cast<v4i *>(e.acc_out + idx) = a;
        v4f res = {0.f, 0.f, 0.f, 0.f};
        if (e.resid) res = *reinterpret_cast<const v4f *>(e.resid + idx);
        float v[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          float x = __builtin_ldexpf((float)a[t], e.exp2);
          if (e.chan_div) x = x / div[t];
          if (e.bias) x = x + bias[t];
          if (e.resid) x = x + res[t];
          if (e.act >= CATCHQ_ACT_RELU) x = (x > 0.0f) ? x : 0.0f;
          if (e.act == CATCHQ_ACT_RELU6) x = (x < 6.0f) ? x : 6.0f;
          v[t] = x;
        }
        if (e.y) {
          if (e.y_f16) {
            __half2 h[2] = {__halves2half2(__float2half_rn(v[0]), __float2half_rn(v[1])),
                            __halves2half2(__float2half_rn(v[2]), __float2half_rn(v[3]))};
            *reinterpret_cast<v2i *>(reinterpret_cast<__half *>(e.y) + idx) = *reinterpret_cast<v2i *>(h);
          } else {
            v4f o = {v[0], v[1], v[2], v[3]};
            *reinterpret_cast<v4f *>(reinterpret_cast<float *>(e.y) + idx) = o;
          }
        }
        if (e.q) {
          if (e.q_bw == 8) {
            unsigned pk = 0;
#pragma unroll
            for (int t = 0; t < 4; ++t) pk |= (unsigned)(quant1<8>(v[t], e.q_scale, e.q_neg_pos) & 0xff) << (8 * t);
            *reinterpret_cast<unsigned *>(reinterpret_cast<int8_t *>(e.q) + idx) = pk;
          } else {
            v2i pk;
            unsigned h[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) h[t] = (unsigned)quant1<16>(v[t], e.q_scale, e.q_neg_pos) & 0xffffu;
            pk[0] = (int)(h[0] | (h[1] << 16));
            pk[1] = (int)(h[2] | (h[3] << 16));
            *reinterpret_cast<v2i *>(reinterpret_cast<int16_t *>(e.q) + idx) = pk;
          }
        }
      }
    }
  }
}

static bool vec_epilogue_ok(int N, const EpiDev &e) {
  return N % 4 == 0 && aligned16(e.chan_div) && aligned16(e.bias) && aligned16(e.resid) && aligned16(e.y) &&
         aligned16(e.acc_out) && aligned16(e.q);
}

template <int BM, int BN, int LOAD>
static int launch_igemm(const void *a, const void *b, IgemmParams p, const EpiDev &e, hipStream_t s) {
  const int64_t tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const int64_t nb = tiles_m * p.tiles_n;
  if (nb > 0x7fffffff) return CATCHQ_ERR_SHAPE;
  p.nblocks = (int)nb;
  if (vec_epilogue_ok(p.N, e))
    igemm_i8_kernel<BM, BN, LOAD, true><<<(int)nb, 256, 0, s>>>((const int8_t *)a, (const int8_t *)b, p, e);
  else
    igemm_i8_kernel<BM, BN, LOAD, false><<<(int)nb, 256, 0, s>>>((const int8_t *)a, (const int8_t *)b, p, e);
  return launch_status();
}

// Tile choice: the largest tile that still gives every CU a few blocks; narrow outputs take a
// narrow tile so that no matrix-core work is spent on padding columns.
template <int LOAD>
static int pick_tile(const void *a, const void *b, const IgemmParams &p, const EpiDev &e, hipStream_t s) {
  auto blocks = [&](int bm, int bn) { return ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn); };
  constexpr int64_t kEnough = 2 * 256;
  if (p.N <= 64) {
    if (blocks(128, 64) >= kEnough) return launch_igemm<128, 64, LOAD>(a, b, p, e, s);
    return launch_igemm<64, 64, LOAD>(a, b, p, e, s);
  }
  if (blocks(128, 128) >= kEnough) return launch_igemm<128, 128, LOAD>(a, b, p, e, s);
  if (blocks(64, 128) >= kEnough) return launch_igemm<64, 128, LOAD>(a, b, p, e, s);
  return launch_igemm<64, 64, LOAD>(a, b, p, e, s);
}

int gemm_nt_mfma_i8(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e,
                    hipStream_t s) {
  IgemmParams p = {};
  p.M = M;
  p.N = (int)N;
  p.K = (int)K;
  return pick_tile<LOAD_GEMM>(a, b, p, e, s);
}

int conv2d_mfma_i8(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph,
                   int pw, int sh, int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  IgemmParams p = {};
  p.M = (int64_t)N * Ho * Wo;
  p.N = Co;
  p.H = H; p.W = W; p.Ci = Ci; p.Ho = Ho; p.Wo = Wo;
  p.kh = kh; p.kw = kw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
  if (Ci == 4) {
    p.kwq = (kw + 3) / 4;
    p.K = kh * p.kwq * 16;
    return pick_tile<LOAD_C4>(x, w, p, e, s);
  }
  p.K = kh * kw * Ci;
  return pick_tile<LOAD_CONV>(x, w, p, e, s);
}

}  // namespace catchq
