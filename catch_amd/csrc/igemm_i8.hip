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
#include <cstdlib>

#include "igemm_common.h"

namespace catchq {

// 16 bytes from a 4-byte aligned address
__device__ __forceinline__ v4i load16_a4(const int8_t *p) {
  struct __attribute__((packed, aligned(4))) P { v4i v; };
  return reinterpret_cast<const P *>(p)->v;
}

template <int BM, int BN, int LOAD, int EPI>
__global__ __launch_bounds__(256) void igemm_i8_kernel(const int8_t *__restrict__ A,
                                                      const int8_t *__restrict__ B, IgemmParams p,
                                                      EpiDev e) {
  resolve_exp2(e);
  constexpr int WM = BM / 2, WN = BN / 2;  // wave tile
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int LA = BM / 64, LB = BN / 64;  // 16-byte chunks each thread loads per K step
  constexpr int EPI_STRIDE = WN + 8;         // ints per staged row (+8: the two half-waves hit different banks)
  constexpr int PIPE_BYTES = 2 * (BM + BN) * BK;
  constexpr int EPI_BYTES = EPI != EPI_SCALAR ? 4 * 32 * EPI_STRIDE * 4 : 0;
  constexpr int LDS_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;
  __shared__ __attribute__((aligned(16))) int8_t lds_raw[LDS_BYTES];
  int8_t(*lds)[(BM + BN) * BK] = reinterpret_cast<int8_t(*)[(BM + BN) * BK]>(lds_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave >> 1, wave_n = wave & 1;

  const int logical = xcd_remap(blockIdx.x, p.nblocks);
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

  // Register ring: the loads of step s+D are issued while step s is multiplied, so D-1 whole steps
  // of work cover the memory latency of every load.
  constexpr int D = 4;
  v4i ra[D][LA], rb[D][LB];
  auto load_global = [&](auto slot_c) {
    constexpr int slot = decltype(slot_c)::value;
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
      ra[slot][i] = v;
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
      rb[slot][i] = v;
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
  auto store_lds = [&](int buf, auto slot_c) {
    constexpr int slot = decltype(slot_c)::value;
    int8_t *la = lds[buf];
    int8_t *lb = lds[buf] + BM * BK;
#pragma unroll
    for (int i = 0; i < LA; ++i) {
      const int row = lr + 64 * i;
      *reinterpret_cast<v4i *>(la + row * BK + swz(row, lc) * 16) = ra[slot][i];
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      const int row = lr + 64 * i;
      *reinterpret_cast<v4i *>(lb + row * BK + swz(row, lc) * 16) = rb[slot][i];
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
  const int frow = lane & 31;   // operand row within a 32-row MFMA tile
  const int fhalf = lane >> 5;  // which 16-byte half of the 32-byte K slice

  auto compute = [&](int buf) {
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
  };

  // prologue: steps 0..D-1 in flight, step 0 into LDS
  {
    auto issue = [&](auto slot_c) {
      if (decltype(slot_c)::value < nsteps) {
        load_global(slot_c);
        advance_k();
      }
    };
    issue(std::integral_constant<int, 0>{});
    issue(std::integral_constant<int, 1>{});
    issue(std::integral_constant<int, 2>{});
    issue(std::integral_constant<int, 3>{});
    store_lds(0, std::integral_constant<int, 0>{});
    __syncthreads();
  }
  // one ring position: slot d held step `step` (already in LDS), so it is free for step+D
  auto ring_step = [&](int step, auto d_c) {
    constexpr int d = decltype(d_c)::value;
    if (step >= nsteps) return;
    if (step + D < nsteps) {
      load_global(d_c);
      advance_k();
    }
    compute(d & 1);
    if (step + 1 < nsteps) store_lds((d + 1) & 1, std::integral_constant<int, (d + 1) % D>{});
    __syncthreads();
  };
  for (int base = 0; base < nsteps; base += D) {
    ring_step(base + 0, std::integral_constant<int, 0>{});
    ring_step(base + 1, std::integral_constant<int, 1>{});
    ring_step(base + 2, std::integral_constant<int, 2>{});
    ring_step(base + 3, std::integral_constant<int, 3>{});
  }

  // ---- epilogue -------------------------------------------------------------------------------
  int *stage = reinterpret_cast<int *>(lds_raw) + wave * 32 * EPI_STRIDE;
  igemm_epilogue<TM, TN, EPI>(acc, stage, m0 + wave_m * WM, n0 + wave_n * WN, lane, p, e);
}

template <int BM, int BN, int LOAD>
static int launch_igemm(const void *a, const void *b, IgemmParams p, const EpiDev &e, hipStream_t s) {
  const int64_t tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const int64_t nb = tiles_m * p.tiles_n;
  if (nb > 0x7fffffff) return CATCHQ_ERR_SHAPE;
  p.nblocks = (int)nb;
  const int epi = pick_epilogue(p.N, e);
  if (epi == EPI_SCALAR)
    igemm_i8_kernel<BM, BN, LOAD, EPI_SCALAR><<<(int)nb, 256, 0, s>>>((const int8_t *)a, (const int8_t *)b, p, e);
  else if (LOAD == LOAD_C4 && epi == EPI_Q8_RELU)  // the network stem: conv + ReLU feeding the next conv
    igemm_i8_kernel<BM, BN, LOAD, (LOAD == LOAD_C4 ? EPI_Q8_RELU : EPI_VECTOR)><<<(int)nb, 256, 0, s>>>(
        (const int8_t *)a, (const int8_t *)b, p, e);
  else
    igemm_i8_kernel<BM, BN, LOAD, EPI_VECTOR><<<(int)nb, 256, 0, s>>>((const int8_t *)a, (const int8_t *)b, p, e);
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

// CATCHQ_NO_DMA=1 keeps every shape on the register-staged kernel (for A/B timing)
static bool dma_enabled() {
  static const bool on = [] {
    const char *v = tuning_env("CATCHQ_NO_DMA");
    return !(v && v[0] == '1');
  }();
  return on;
}

// CATCHQ_NO_HALO=1 (tuning builds) keeps 3x3 layers on the implicit-GEMM kernel
static bool halo_enabled() {
  static const bool on = [] {
    const char *v = tuning_env("CATCHQ_NO_HALO");
    return !(v && v[0] == '1');
  }();
  return on;
}
int conv2d_halo_i8(const void *x, const void *w, int N, int Hi, int Wi, int Ci, int Co, int stride, const EpiDev &e,
                   hipStream_t s);

int gemm_nt_stream_i8(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e, hipStream_t s);
int conv2d_stem_i8(const void *x, const void *w, int N, int H, int W, int Co, int kh, int kw, int sh, int sw, int dh,
                   int Ho, int Wo, const EpiDev &e, hipStream_t s);

int gemm_nt_mfma_i8(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e,
                    hipStream_t s) {
  if (dma_enabled()) {  // short K, narrow N, many rows: the streaming kernel
    const int st = gemm_nt_stream_i8(a, b, M, N, K, e, s);
    if (st >= 0) return st;
  }
  IgemmParams p = {};
  p.M = M;
  p.N = (int)N;
  p.K = (int)K;
  if (dma_enabled()) {
    const int st = igemm_dma_launch(LOAD_GEMM, a, b, p, e, M * K, N * K, s);
    if (st >= 0) return st;
  }
  return pick_tile<LOAD_GEMM>(a, b, p, e, s);
}

// Grouped convolution (groups > 1, a multiple of 16 input channels and of 4 output channels per group): one implicit
// GEMM per group, the group index on the grid's second dimension; -1 when the shape is not eligible
int conv2d_mfma_i8_grouped(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph, int pw,
                           int sh, int sw, int dh, int dw, int Ho, int Wo, int groups, const EpiDev &e, hipStream_t s) {
  const int cig = Ci / groups, cog = Co / groups;
  if (groups < 2 || groups > 65535 || cig % 16 != 0 || cog % 4 != 0 || kh * kw > 32) return -1;
  IgemmParams p = {};
  p.M = (int64_t)N * Ho * Wo;
  p.N = cog;
  p.H = H; p.W = W; p.Ci = cig; p.Ho = Ho; p.Wo = Wo;
  p.kh = kh; p.kw = kw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
  p.K = kh * kw * cig;
  p.img_stride = (unsigned)(H * W * Ci); p.row_stride = (unsigned)(W * Ci); p.pix_stride = (unsigned)Ci;
  p.ldc = Co;
  p.groups = groups;
  p.a_group_bytes = cig;
  p.b_group_bytes = (int64_t)cog * p.K;
  p.n_group = cog;
  return igemm_dma_launch(LOAD_CONV, x, w, p, e, (int64_t)N * H * W * Ci, (int64_t)Co * p.K, s);
}

int conv2d_mfma_i8(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph,
                   int pw, int sh, int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  IgemmParams p = {};
  p.M = (int64_t)N * Ho * Wo;
  p.N = Co;
  p.H = H; p.W = W; p.Ci = Ci; p.Ho = Ho; p.Wo = Wo;
  p.kh = kh; p.kw = kw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
  if (Ci == 4 && ph == 0 && pw == 0 && dw == 1 && dma_enabled()) {  // framed few-channel image: streaming kernel
    const int st = conv2d_stem_i8(x, w, N, H, W, Co, kh, kw, sh, sw, dh, Ho, Wo, e, s);
    if (st >= 0) return st;
  }
  if (Ci == 4 && pw == 0 && dw == 1 && kw % 4 == 0 && kh <= 32 && dma_enabled()) {
    // Few-channel input already padded horizontally, filter rows padded to whole 16-byte chunks:
    // a filter row is one contiguous run of kw*4 bytes of an image row, starting sw*4 bytes further
    // for every output column.  To the loader that is a convolution with kh x 1 taps of kw*4
    // "channels" over an image whose "pixels" are sw*4 bytes apart and whose width is Wo.
    IgemmParams q = p;
    q.K = kh * kw * 4;
    q.Ci = kw * 4;
    q.kw = 1; q.sw = 1; q.pw = 0; q.dw = 1;
    q.W = Wo;
    q.img_stride = (unsigned)(H * W * 4); q.row_stride = (unsigned)(W * 4); q.pix_stride = (unsigned)(sw * 4);
    const int st = igemm_dma_launch(LOAD_CONV, x, w, q, e, (int64_t)N * H * W * 4, (int64_t)Co * q.K, s);
    if (st >= 0) return st;
  }
  if (Ci == 4) {
    p.kwq = (kw + 3) / 4;
    p.K = kh * p.kwq * 16;
    return pick_tile<LOAD_C4>(x, w, p, e, s);
  }
  p.K = kh * kw * Ci;
  if (dma_enabled() && kh == 1 && kw == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0) {
    // a pointwise convolution is a plain GEMM over the pixels
    int st = gemm_nt_stream_i8(x, w, p.M, Co, Ci, e, s);
    if (st >= 0) return st;
    // ... and takes the GEMM loader of the pipelined kernel: a row's address is its index times K, with no
    // (image, row, column) split and no tap masks in front of the first load
    const char *as_gemm = tuning_env("CATCHQ_PW_AS_GEMM");
    if (Ci % 16 == 0 && !(as_gemm && atoi(as_gemm) == 0)) {
      st = igemm_dma_launch(LOAD_GEMM, x, w, p, e, p.M * Ci, (int64_t)Co * Ci, s);
      if (st >= 0) return st;
    }
  }
  if (dma_enabled() && halo_enabled() && kh == 3 && kw == 3 && sh == sw && ph == 1 && pw == 1 && dh == 1 && dw == 1) {
    // the input patch of a band of output rows stays in LDS for all nine taps
    const int st = conv2d_halo_i8(x, w, N, H, W, Ci, Co, sh, e, s);
    if (st >= 0) return st;
  }
  p.img_stride = (unsigned)(H * W * Ci); p.row_stride = (unsigned)(W * Ci); p.pix_stride = (unsigned)Ci;
  if (dma_enabled() && kh * kw <= 32) {  // the DMA loader keeps one validity bit per filter tap
    const int st = igemm_dma_launch(LOAD_CONV, x, w, p, e, (int64_t)N * H * W * Ci, (int64_t)Co * p.K, s);
    if (st >= 0) return st;
  }
  return pick_tile<LOAD_CONV>(x, w, p, e, s);
}

}  // namespace catchq
