// int16 activations x int8 weights on the int8 matrix cores, LDS-DMA pipelined.
//
// An int16 value splits exactly into two int8 digits and a constant:
//     x = 256*hi + lo_s + 128,    hi = x >> 8  (signed high byte),   lo_s = (x & 255) - 128,
// so   sum_k x_k*w_k = 256 * sum hi_k*w_k  +  sum lo_s_k*w_k  +  128 * sum_k w_k.
// The two digit sums are int8 x int8 MFMA accumulations, the last term is a per-output-channel
// constant that a wave collects from the weight fragments it loads anyway (v_dot4 with all-ones).
// A zero written by the hardware for an out-of-image tap or a row beyond M decodes to
// (hi, lo_s) = (0, -128), i.e. to x = 0 after the constant is added, so the convolution's zero
// padding needs no special case; the same identity makes whatever the weight operand holds beyond
// K irrelevant.  All three terms are accumulated modulo 2^32, so the result is exact whenever the
// true sum fits an int32 (the precondition of the int16 x int8 contraction).
//
// The split happens in registers, between the LDS fetch and the MFMA: activations stay plain
// int16 NHWC in memory.  A-tile rows are 128 bytes (64 int16 of K) = eight 16-byte chunks, the
// chunk index XOR-ed with row&7; weight rows keep the 64-byte layout of the int8 kernel.  (row&7
// leaves a two-way bank conflict on the A fetches; the conflict-free (row>>1)&7 needs a second K
// position per lane in the loader and measured 8 % slower end to end: the loop is bound by the
// address arithmetic and issue of the loads, not by the LDS reads.)
#include "igemm_i8_dma.inc"

namespace catchq {

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int LOAD, int EPI>
__global__ __launch_bounds__(64 * WAVES_M *WAVES_N) void igemm_a16_dma_kernel(const int16_t *__restrict__ A,
                                                                            const int8_t *__restrict__ B,
                                                                            IgemmParams p, EpiDev e,
                                                                            unsigned a_bytes, unsigned b_bytes) {
  resolve_exp2(e);
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_STAGE = BM * BK * 2, B_STAGE = BN * BK;
  constexpr int STAGE_BYTES = A_STAGE + B_STAGE;
  constexpr int PIPE_BYTES = STAGES * STAGE_BYTES;
  constexpr int NIA = BM / 8, NIB = BN / 16;  // DMA instructions (1 KiB each) per stage: A, B
  constexpr int NI = (NIA + NIB) / NW;        // per wave
  static_assert((NIA + NIB) % NW == 0, "tile rows must split evenly over the waves");
  static_assert(STAGES >= 3, "the ring needs at least three stages");
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

  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void *)A, 0, (int)a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void *)B, 0, (int)b_bytes, 0x00020000);
  constexpr unsigned OOB = 0x80000000u;

  // ---- loader state -----------------------------------------------------------------------------
  // A instruction: 8 tile rows x 8 chunks (lane -> row lane/8, physical chunk lane%8);
  // B instruction: 16 tile rows x 4 chunks (lane -> row lane/4, physical chunk lane%4).
  unsigned rowbase[NI];  // byte offset of the row's K origin
  unsigned vmask[NI];    // A: bit t = filter tap t inside the image; B / plain GEMM: bit 0 = row exists
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int slot = wave * NI + j;
    if (slot < NIA) {
      const int64_t m = m0 + slot * 8 + (lane >> 3);
      const bool ok = m < p.M;
      const int64_t mm = ok ? m : 0;
      if constexpr (LOAD == LOAD_CONV) {
        // fewer than 2^31 output pixels (checked by the launcher): 32-bit divisions
        const unsigned mu = (unsigned)mm;
        const unsigned t = mu / (unsigned)p.Wo;
        const int wo = (int)(mu - t * (unsigned)p.Wo);
        const unsigned img = t / (unsigned)p.Ho;
        const int ho = (int)(t - img * (unsigned)p.Ho);
        const int hi0 = ho * p.sh - p.ph, wi0 = wo * p.sw - p.pw;
        rowbase[j] = 2u * ((unsigned)((int64_t)img * p.H * p.W * p.Ci) + (unsigned)((hi0 * p.W + wi0) * p.Ci));  // mod 2^32
        unsigned mask = 0;
        for (int r = 0; r < p.kh; ++r)
          for (int q = 0; q < p.kw; ++q)
            if ((unsigned)(hi0 + r * p.dh) < (unsigned)p.H && (unsigned)(wi0 + q * p.dw) < (unsigned)p.W)
              mask |= 1u << (r * p.kw + q);
        vmask[j] = ok ? mask : 0u;
      } else {
        rowbase[j] = (unsigned)(mm * p.K * 2);
        vmask[j] = ok ? 1u : 0u;
      }
    } else {
      const int n = n0 + (slot - NIA) * 16 + (lane >> 2);
      const bool ok = n < p.N;
      rowbase[j] = (unsigned)((int64_t)(ok ? n : 0) * p.K);
      vmask[j] = ok ? 1u : 0u;
    }
  }
  // this lane's position along K, in elements: as a loader of A (8-element chunks) and of B (16)
  int ka_lin = ((lane & 7) ^ (lane >> 3)) * 8;
  int kb_lin = ((lane & 3) ^ ((lane >> 4) & 3)) * 16;
  int kr = 0, kq = 0, kci = ka_lin, tap = 0;
  unsigned tapbase = 0;  // (kr*dh*W + kq*dw)*Ci elements
  auto normalise_tap = [&]() {
    while (kci >= p.Ci) {
      kci -= p.Ci;
      ++tap;
      if (++kq == p.kw) { kq = 0; ++kr; }
      tapbase = (unsigned)((kr * p.dh * p.W + kq * p.dw) * p.Ci);
    }
  };
  if constexpr (LOAD == LOAD_CONV) normalise_tap();

  auto issue_stage = [&](int stage_off) {
    const bool ka_ok = ka_lin < p.K, kb_ok = kb_lin < p.K;
    const unsigned a_koff = 2u * ((LOAD == LOAD_CONV) ? tapbase + (unsigned)kci : (unsigned)ka_lin);
    const unsigned a_bit = (LOAD == LOAD_CONV) ? (1u << tap) : 1u;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int slot = wave * NI + j;
      const bool is_a = slot < NIA;  // wave-uniform
      lds_ptr_t dst = (lds_ptr_t)(lds_dyn + stage_off + slot * 1024);  // B slots follow the A slots
      if (is_a) {
        const unsigned voff = select_u32(ka_ok && (vmask[j] & a_bit), rowbase[j] + a_koff, OOB);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, (int)voff, 0, 0, 0);
      } else {
        const unsigned voff = select_u32(kb_ok && vmask[j], rowbase[j] + (unsigned)kb_lin, OOB);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, (int)voff, 0, 0, 0);
      }
    }
    ka_lin += BK;
    kb_lin += BK;
    if constexpr (LOAD == LOAD_CONV) {
      kci += BK;
      normalise_tap();
    }
  };

  v16i acc_hi[TM][TN], acc_lo[TM][TN];
  int wsum[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) wsum[j] = 0;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) { acc_hi[i][j][r] = 0; acc_lo[i][j][r] = 0; }

  // ---- operand fetch addresses (LDS byte offsets) ------------------------------------------------
  const int frow = lane & 31, fhalf = lane >> 5;
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int8_t *)lds_dyn;
  // A: elements [ks*32 + fhalf*16, +16) of the step = logical chunks ks*4 + fhalf*2 and the next one
  const unsigned a_c0 = (unsigned)(((fhalf * 2) ^ (frow & 7)) * 16);
  const unsigned a_row = lds_base + (unsigned)((wave_m * WM + frow) * (BK * 2));
  // B: as in the int8 kernel
  const int swb = (frow >> 2) & 3;
  const unsigned b_k0 = (unsigned)((fhalf ^ swb) * 16), b_k1 = (unsigned)(((fhalf ^ swb) ^ 2) * 16);
  const unsigned b_row = lds_base + (unsigned)(A_STAGE + (wave_n * WN + frow) * BK);

  // one half of a K step (32 int16 activations x 32 int8 weights per tile): fetch, then multiply
  auto fetch_half = [&](v4i (&fa)[TM][2], v4i (&fb)[TN], unsigned a_base, unsigned a_chunk, unsigned b_addr) {
    const unsigned a_first = a_base + a_chunk, a_second = a_base + (a_chunk ^ 16u);
    // tile i of this wave sits 32 rows further: 4096 bytes for A, 2048 for B
    fa[0][0] = ds_read_b128<0>(a_first);
    fa[0][1] = ds_read_b128<0>(a_second);
    if constexpr (TM > 1) {
      fa[1][0] = ds_read_b128<4096>(a_first);
      fa[1][1] = ds_read_b128<4096>(a_second);
    }
    fb[0] = ds_read_b128<0>(b_addr);
    if constexpr (TN > 1) fb[1] = ds_read_b128<2048>(b_addr);
  };
  auto multiply_half = [&](v4i (&fa)[TM][2], v4i (&fb)[TN]) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int d = 0; d < 4; ++d) wsum[j] = __builtin_amdgcn_sdot4(fb[j][d], 0x01010101, wsum[j], false);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      v4i hi, lo;
      split_i16(fa[i][0], fa[i][1], hi, lo);
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc_hi[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(hi, fb[j], acc_hi[i][j], 0, 0, 0);
        acc_lo[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(lo, fb[j], acc_lo[i][j], 0, 0, 0);
      }
    }
  };
  static_assert(TM <= 2 && TN <= 2, "wave tile larger than 64x64");

  // both halves are requested up front: the second half's fragments arrive while the first half is multiplied
  auto compute = [&](unsigned stage_off) {
    constexpr int NF = 2 * TM + TN;  // LDS reads per half
    v4i fa0[TM][2], fb0[TN], fa1[TM][2], fb1[TN];
    fetch_half(fa0, fb0, a_row + stage_off, a_c0, b_row + stage_off + b_k0);
    fetch_half(fa1, fb1, a_row + stage_off, a_c0 ^ 64u, b_row + stage_off + b_k1);
#pragma unroll
    for (int i = 0; i < TM; ++i) { lgkm_wait<NF>(fa0[i][0]); lgkm_wait<NF>(fa0[i][1]); }
#pragma unroll
    for (int j = 0; j < TN; ++j) lgkm_wait<NF>(fb0[j]);
    multiply_half(fa0, fb0);
#pragma unroll
    for (int i = 0; i < TM; ++i) { lgkm_wait<0>(fa1[i][0]); lgkm_wait<0>(fa1[i][1]); }
#pragma unroll
    for (int j = 0; j < TN; ++j) lgkm_wait<0>(fb1[j]);
    multiply_half(fa1, fb1);
  };

  // ---- pipeline (same schedule as the int8 kernel) ---------------------------------------------------
  const int nsteps = (p.K + BK - 1) / BK;
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue_stage(s * STAGE_BYTES);
  int rd_off = 0, wr_off = (STAGES - 1) * STAGE_BYTES;
  for (int step = 0; step < nsteps; ++step) {
    CATCHQ_VMCNT(NI * (STAGES - 2));
    __builtin_amdgcn_s_barrier();
    issue_stage(wr_off);
    compute((unsigned)rd_off);
    rd_off = (rd_off + STAGE_BYTES == PIPE_BYTES) ? 0 : rd_off + STAGE_BYTES;
    wr_off = (wr_off + STAGE_BYTES == PIPE_BYTES) ? 0 : wr_off + STAGE_BYTES;
  }
  CATCHQ_VMCNT(0);
  __syncthreads();

  // the two K halves of a column's weight sum sit in lanes l and l^32; the accumulator layout has
  // column = lane & 31, the same as the weight fragment's row
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const unsigned ws = (unsigned)(wsum[j] + __shfl_xor(wsum[j], 32, 64)) << 7;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc_lo[i][j][r] = (int)(((unsigned)acc_hi[i][j][r] << 8) + (unsigned)acc_lo[i][j][r] + ws);
  }
  int *stage = reinterpret_cast<int *>(lds_dyn) + wave * 32 * EPI_STRIDE;
  // the residual epilogues of the wide tile in two passes: 104 registers or fewer keep three waves per SIMD
  constexpr int EPI_PASSES = (WN == 64 && (EPI == EPI_LK_RESA_Q16 || EPI == EPI_LK_RESA_Y_Q16)) ? 2 : 1;
  igemm_epilogue<TM, TN, EPI, EPI_PASSES>(acc_lo, stage, m0 + wave_m * WM, n0 + wave_n * WN, lane, p, e);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int LOAD, int EPI>
static int launch_a16_epi(const void *a, const void *b, const IgemmParams &p, const EpiDev &e, int64_t a_bytes,
                          int64_t b_bytes, hipStream_t s) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int PIPE_BYTES = STAGES * (2 * BM + BN) * BK;
  constexpr int EPI_BYTES = NW * 32 * (BN / WAVES_N + 8) * 4;
  constexpr int LDS_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;
  static_assert(LDS_BYTES <= 160 * 1024, "tile does not fit the LDS");
  auto kern = igemm_a16_dma_kernel<BM, BN, WAVES_M, WAVES_N, STAGES, LOAD, EPI>;
  if (LDS_BYTES > 64 * 1024) {
    static std::atomic<bool> raised[64];
    if (raise_lds_limit((const void *)kern, LDS_BYTES, raised) != CATCHQ_OK) return CATCHQ_ERR_LAUNCH;
  }
  kern<<<p.nblocks, 64 * NW, LDS_BYTES, s>>>((const int16_t *)a, (const int8_t *)b, p, e, (unsigned)a_bytes,
                                             (unsigned)b_bytes);
  return launch_status();
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int LOAD>
static int launch_a16(const void *a, const void *b, IgemmParams p, const EpiDev &e, int64_t a_bytes, int64_t b_bytes,
                      hipStream_t s) {
  const int64_t tiles_m = (p.M + BM - 1) / BM;
  p.tiles_n = (p.N + BN - 1) / BN;
  const int64_t nb = tiles_m * p.tiles_n;
  if (nb > 0x7fffffff) return CATCHQ_ERR_SHAPE;
  p.nblocks = (int)nb;
  const int epi = pick_epilogue(p.N, e);
  if (epi == EPI_SCALAR)
    return launch_a16_epi<BM, BN, WAVES_M, WAVES_N, STAGES, LOAD, EPI_SCALAR>(a, b, p, e, a_bytes, b_bytes, s);
  if constexpr (BM == 64) {  // the tiles of the detector layers: leaky ReLU, int16 requantization
    switch (epi) {
      case EPI_LK_Q16: return launch_a16_epi<BM, BN, WAVES_M, WAVES_N, STAGES, LOAD, EPI_LK_Q16>(a, b, p, e, a_bytes, b_bytes, s);
      case EPI_LK_Y_Q16: return launch_a16_epi<BM, BN, WAVES_M, WAVES_N, STAGES, LOAD, EPI_LK_Y_Q16>(a, b, p, e, a_bytes, b_bytes, s);
      case EPI_LK_RESA_Q16: return launch_a16_epi<BM, BN, WAVES_M, WAVES_N, STAGES, LOAD, EPI_LK_RESA_Q16>(a, b, p, e, a_bytes, b_bytes, s);
      case EPI_LK_RESA_Y_Q16: return launch_a16_epi<BM, BN, WAVES_M, WAVES_N, STAGES, LOAD, EPI_LK_RESA_Y_Q16>(a, b, p, e, a_bytes, b_bytes, s);
      default: break;
    }
  }
  return launch_a16_epi<BM, BN, WAVES_M, WAVES_N, STAGES, LOAD, EPI_VECTOR>(a, b, p, e, a_bytes, b_bytes, s);
}

template <int LOAD>
static int pick_a16_tile(const void *a, const void *b, const IgemmParams &p, const EpiDev &e, int64_t a_bytes,
                         int64_t b_bytes, hipStream_t s) {
  auto blocks = [&](int bm, int bn) { return ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn); };
  const int64_t kCUs = e.cus;
  int tile = forced_tile();
  if (!tile) {
    // Measured on every Darknet-53 layer (bs16, 416x416): the 64x64 tile is the default -- two accumulator
    // sets and the digit split keep a wave busy enough, and small tiles mean more resident blocks per CU.
    // Only GEMMs far beyond those sizes take the widest tile.
    if (p.N >= 256 && p.K >= 256 && (int64_t)p.M * p.N * p.K >= (1ll << 34)) tile = 128256;
    else {
      tile = 64064;
      // Twice the columns per block halve the fetches of the int16 operand.  It pays where the launch still has
      // two blocks per CU and the kernel keeps three waves per SIMD, which the detector's epilogue instances do
      // (the residual ones by working through a staged block in two passes): the 3x3 and 1x1 layers of
      // Darknet-53 with 128 or more output channels gain 5-25 %, 7.6 % end to end; with fewer blocks or narrower
      // outputs the same tile loses a few percent (all measured).
      const int epi = pick_epilogue(p.N, e);
      const bool detector = epi == EPI_LK_Q16 || epi == EPI_LK_Y_Q16 || epi == EPI_LK_RESA_Q16 || epi == EPI_LK_RESA_Y_Q16;
      if (detector && p.N % 128 == 0 && blocks(64, 128) >= 2 * kCUs) tile = 64128;
    }
  }
  switch (tile) {
    case 128256: return launch_a16<128, 256, 2, 4, 4, LOAD>(a, b, p, e, a_bytes, b_bytes, s);
    case 128128: return launch_a16<128, 128, 2, 2, 3, LOAD>(a, b, p, e, a_bytes, b_bytes, s);
    case 64128: return launch_a16<64, 128, 2, 2, 3, LOAD>(a, b, p, e, a_bytes, b_bytes, s);
    default: return launch_a16<64, 64, 2, 2, 3, LOAD>(a, b, p, e, a_bytes, b_bytes, s);
  }
}

// int16 x int8 contractions on the matrix cores; -1 when the shape is not eligible
int igemm_a16_launch(int load, const void *a, const void *b, IgemmParams p, const EpiDev &e, int64_t a_bytes,
                     int64_t b_bytes, hipStream_t s) {
  if (a_bytes >= (1ll << 31) || b_bytes >= (1ll << 31) || a_bytes <= 0 || b_bytes <= 0) return -1;
  if (load == LOAD_GEMM) return pick_a16_tile<LOAD_GEMM>(a, b, p, e, a_bytes, b_bytes, s);
  if (load == LOAD_CONV) return pick_a16_tile<LOAD_CONV>(a, b, p, e, a_bytes, b_bytes, s);
  return -1;
}

int gemm_nt_mfma_a16(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e, hipStream_t s) {
  IgemmParams p = {};
  p.M = M;
  p.N = (int)N;
  p.K = (int)K;
  return igemm_a16_launch(LOAD_GEMM, a, b, p, e, M * K * 2, N * K, s);
}

// ---- int16 x int16 ------------------------------------------------------------------------------------------
// Both operands split into digits:  x = 256*xh + xl + 128,  w = 256*wh + wl + 128  (high byte signed, low byte
// biased into int8), so
//   sum x*w = 65536*S_hh + 256*(S_hl + S_lh) + S_ll + 32768*(sum xh + sum wh) + 128*(sum xl + sum wl) + 16384*Kp
// with four int8 x int8 MFMA sums S_.. , the digit sums of the row (activations) and of the column (weights), which
// the wave collects from the fragments it loads anyway, and Kp the number of K positions walked (whole steps: a
// position beyond K, a row beyond M or N and an out-of-image tap all read as zeros, which decode to the value 0 on
// either side, so the identity covers them).  Every partial sum fits an int32 (|S| <= Kp * 2^14); the combination
// is done in 64-bit integers and is the exact sum, which is what the int16 x int16 contraction is defined on.
// One tile shape (64 x 64, four waves of 32 x 32), element-wise epilogue from the accumulators.
template <int LOAD>
__global__ __launch_bounds__(256) void igemm_a16w16_kernel(const int16_t *__restrict__ A, const int16_t *__restrict__ B,
                                                          IgemmParams p, EpiDev e, unsigned a_bytes, unsigned b_bytes) {
  resolve_exp2(e);
  constexpr int BM = 64, BN = 64, STAGES = 3;
  constexpr int A_STAGE = BM * BK * 2, STAGE_BYTES = (BM + BN) * BK * 2;
  constexpr int PIPE_BYTES = STAGES * STAGE_BYTES;
  constexpr int NIA = BM / 8;                 // DMA instructions (1 KiB: 8 rows x 128 bytes) per stage and operand
  constexpr int NI = (BM + BN) / 8 / 4;       // per wave
  extern __shared__ __attribute__((aligned(16))) int8_t lds_dyn[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave_m = wave >> 1, wave_n = wave & 1;
  const int logical = xcd_remap(blockIdx.x, p.nblocks);
  const int tile_n = logical % p.tiles_n;
  const int tile_m = logical / p.tiles_n;
  const int64_t m0 = (int64_t)tile_m * BM;
  const int n0 = tile_n * BN;

  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void *)A, 0, (int)a_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void *)B, 0, (int)b_bytes, 0x00020000);
  constexpr unsigned OOB = 0x80000000u;

  unsigned rowbase[NI];
  unsigned vmask[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int slot = wave * NI + j;
    if (slot < NIA) {
      const int64_t m = m0 + slot * 8 + (lane >> 3);
      const bool ok = m < p.M;
      const int64_t mm = ok ? m : 0;
      if constexpr (LOAD == LOAD_CONV) {
        const unsigned mu = (unsigned)mm;
        const unsigned t = mu / (unsigned)p.Wo;
        const int wo = (int)(mu - t * (unsigned)p.Wo);
        const unsigned img = t / (unsigned)p.Ho;
        const int ho = (int)(t - img * (unsigned)p.Ho);
        const int hi0 = ho * p.sh - p.ph, wi0 = wo * p.sw - p.pw;
        rowbase[j] = 2u * ((unsigned)((int64_t)img * p.H * p.W * p.Ci) + (unsigned)((hi0 * p.W + wi0) * p.Ci));  // mod 2^32
        unsigned mask = 0;
        for (int r = 0; r < p.kh; ++r)
          for (int q = 0; q < p.kw; ++q)
            if ((unsigned)(hi0 + r * p.dh) < (unsigned)p.H && (unsigned)(wi0 + q * p.dw) < (unsigned)p.W)
              mask |= 1u << (r * p.kw + q);
        vmask[j] = ok ? mask : 0u;
      } else {
        rowbase[j] = (unsigned)(mm * p.K * 2);
        vmask[j] = ok ? 1u : 0u;
      }
    } else {
      const int n = n0 + (slot - NIA) * 8 + (lane >> 3);
      const bool ok = n < p.N;
      rowbase[j] = (unsigned)((int64_t)(ok ? n : 0) * p.K * 2);
      vmask[j] = ok ? 1u : 0u;
    }
  }
  int k_lin = ((lane & 7) ^ (lane >> 3)) * 8;  // this lane's K position (elements) in either operand
  int kr = 0, kq = 0, kci = k_lin, tap = 0;
  unsigned tapbase = 0;
  auto normalise_tap = [&]() {
    while (kci >= p.Ci) {
      kci -= p.Ci;
      ++tap;
      if (++kq == p.kw) { kq = 0; ++kr; }
      tapbase = (unsigned)((kr * p.dh * p.W + kq * p.dw) * p.Ci);
    }
  };
  if constexpr (LOAD == LOAD_CONV) normalise_tap();

  auto issue_stage = [&](int stage_off) {
    const bool k_ok = k_lin < p.K;
    const unsigned a_koff = 2u * ((LOAD == LOAD_CONV) ? tapbase + (unsigned)kci : (unsigned)k_lin);
    const unsigned a_bit = (LOAD == LOAD_CONV) ? (1u << tap) : 1u;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int slot = wave * NI + j;
      const bool is_a = slot < NIA;  // wave-uniform
      lds_ptr_t dst = (lds_ptr_t)(lds_dyn + stage_off + slot * 1024);
      if (is_a) {
        const unsigned voff = select_u32(k_ok && (vmask[j] & a_bit), rowbase[j] + a_koff, OOB);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, (int)voff, 0, 0, 0);
      } else {
        const unsigned voff = select_u32(k_ok && vmask[j], rowbase[j] + 2u * (unsigned)k_lin, OOB);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, (int)voff, 0, 0, 0);
      }
    }
    k_lin += BK;
    if constexpr (LOAD == LOAD_CONV) {
      kci += BK;
      normalise_tap();
    }
  };

  v16i s_hh, s_hl, s_lh, s_ll;
#pragma unroll
  for (int r = 0; r < 16; ++r) { s_hh[r] = 0; s_hl[r] = 0; s_lh[r] = 0; s_ll[r] = 0; }
  int xh_sum = 0, xl_sum = 0, wh_sum = 0, wl_sum = 0;

  const int frow = lane & 31, fhalf = lane >> 5;
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int8_t *)lds_dyn;
  const unsigned c0 = (unsigned)(((fhalf * 2) ^ (frow & 7)) * 16);
  const unsigned a_row = lds_base + (unsigned)((wave_m * 32 + frow) * (BK * 2));
  const unsigned b_row = lds_base + (unsigned)(A_STAGE + (wave_n * 32 + frow) * (BK * 2));

  auto half_step = [&](unsigned a_base, unsigned b_base, unsigned chunk) {
    v4i fa0 = ds_read_b128<0>(a_base + chunk), fa1 = ds_read_b128<0>(a_base + (chunk ^ 16u));
    v4i fb0 = ds_read_b128<0>(b_base + chunk), fb1 = ds_read_b128<0>(b_base + (chunk ^ 16u));
    lgkm_wait<0>(fa0, fa1, fb0, fb1);
    v4i xh, xl, wh, wl;
    split_i16(fa0, fa1, xh, xl);
    split_i16(fb0, fb1, wh, wl);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      xh_sum = __builtin_amdgcn_sdot4(xh[d], 0x01010101, xh_sum, false);
      xl_sum = __builtin_amdgcn_sdot4(xl[d], 0x01010101, xl_sum, false);
      wh_sum = __builtin_amdgcn_sdot4(wh[d], 0x01010101, wh_sum, false);
      wl_sum = __builtin_amdgcn_sdot4(wl[d], 0x01010101, wl_sum, false);
    }
    s_hh = __builtin_amdgcn_mfma_i32_32x32x32_i8(xh, wh, s_hh, 0, 0, 0);
    s_hl = __builtin_amdgcn_mfma_i32_32x32x32_i8(xh, wl, s_hl, 0, 0, 0);
    s_lh = __builtin_amdgcn_mfma_i32_32x32x32_i8(xl, wh, s_lh, 0, 0, 0);
    s_ll = __builtin_amdgcn_mfma_i32_32x32x32_i8(xl, wl, s_ll, 0, 0, 0);
  };

  const int nsteps = (p.K + BK - 1) / BK;
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue_stage(s * STAGE_BYTES);
  int rd_off = 0, wr_off = (STAGES - 1) * STAGE_BYTES;
  for (int step = 0; step < nsteps; ++step) {
    CATCHQ_VMCNT(NI * (STAGES - 2));
    __builtin_amdgcn_s_barrier();
    issue_stage(wr_off);
    half_step(a_row + (unsigned)rd_off, b_row + (unsigned)rd_off, c0);
    half_step(a_row + (unsigned)rd_off, b_row + (unsigned)rd_off, c0 ^ 64u);
    rd_off = (rd_off + STAGE_BYTES == PIPE_BYTES) ? 0 : rd_off + STAGE_BYTES;
    wr_off = (wr_off + STAGE_BYTES == PIPE_BYTES) ? 0 : wr_off + STAGE_BYTES;
  }
  CATCHQ_VMCNT(0);

  // a lane holds the digit sums of A row / B row (lane & 31) over its half of every K step: add the halves
  xh_sum += __shfl_xor(xh_sum, 32, 64);
  xl_sum += __shfl_xor(xl_sum, 32, 64);
  wh_sum += __shfl_xor(wh_sum, 32, 64);
  wl_sum += __shfl_xor(wl_sum, 32, 64);
  // accumulator register r of a lane is row 8*(r>>2) + 4*(lane>>5) + (r&3), column lane & 31 of the 32 x 32 tile
  const int64_t col_part = 32768ll * wh_sum + 128ll * wl_sum + 16384ll * ((int64_t)nsteps * BK);
  const int n = n0 + wave_n * 32 + frow;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int row = 8 * (r >> 2) + 4 * fhalf + (r & 3);
    const int rxh = __shfl(xh_sum, row, 64), rxl = __shfl(xl_sum, row, 64);
    const int64_t m = m0 + wave_m * 32 + row;
    if (n >= p.N || m >= p.M) continue;
    const int64_t total = ((int64_t)s_hh[r] << 16) + (((int64_t)s_hl[r] + (int64_t)s_lh[r]) << 8) + (int64_t)s_ll[r] +
                          32768ll * rxh + 128ll * rxl + col_part;
    const int64_t idx = m * p.N + n;
    epi_store(epi_value((float)total, idx, n, e), idx, e);
  }
}

template <int LOAD>
static int launch_a16w16(const void *a, const void *b, IgemmParams p, const EpiDev &e, int64_t a_bytes, int64_t b_bytes,
                         hipStream_t s) {
  if (a_bytes >= (1ll << 31) || b_bytes >= (1ll << 31) || a_bytes <= 0 || b_bytes <= 0) return -1;
  if (e.acc_out) return -1;  // the exact sum is a 64-bit integer: no int32 accumulator output
  if (p.M >= (1ll << 31) - 64 || p.K >= (1 << 16)) return -1;  // 32-bit pixel index; partial sums within int32
  p.tiles_n = (p.N + 63) / 64;
  const int64_t nb = ((p.M + 63) / 64) * p.tiles_n;
  if (nb > 0x7fffffff) return -1;
  p.nblocks = (int)nb;
  igemm_a16w16_kernel<LOAD><<<p.nblocks, 256, 3 * 128 * BK * 2, s>>>((const int16_t *)a, (const int16_t *)b, p, e,
                                                                     (unsigned)a_bytes, (unsigned)b_bytes);
  return launch_status();
}

// int16 x int16 contractions on the matrix cores; -1 when the shape is not eligible
int gemm_nt_mfma_a16w16(const void *a, const void *b, int64_t M, int64_t N, int64_t K, const EpiDev &e, hipStream_t s) {
  IgemmParams p = {};
  p.M = M;
  p.N = (int)N;
  p.K = (int)K;
  return launch_a16w16<LOAD_GEMM>(a, b, p, e, M * K * 2, N * K * 2, s);
}

int conv2d_mfma_a16w16(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph, int pw,
                       int sh, int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  IgemmParams p = {};
  p.M = (int64_t)N * Ho * Wo;
  p.N = Co;
  p.H = H; p.W = W; p.Ci = Ci; p.Ho = Ho; p.Wo = Wo;
  p.kh = kh; p.kw = kw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
  p.K = kh * kw * Ci;
  return launch_a16w16<LOAD_CONV>(x, w, p, e, (int64_t)N * H * W * Ci * 2, (int64_t)Co * p.K * 2, s);
}

// ---- few-channel first layer, int16 activations -------------------------------------------------
// Input [N, H, W, 8] int16 already framed by its zero padding, filter rows padded to 4 taps (weights
// [Co][kh][4][8] int8, the extra tap zero).  A filter row is 64 contiguous bytes of an image row and
// exactly one MFMA K step (32 elements); the K half a lane owns is two adjacent pixels.  Weights and
// their column sums live in registers, A fragments come straight from global memory, a wave handles
// 32 consecutive output pixels x 32 output channels (blockIdx.y selects the channel group).
typedef int v4i_a4 __attribute__((ext_vector_type(4), aligned(4)));

template <int STEPS, int EPI>
__global__ __launch_bounds__(256, 2) void stem_a16_kernel(const int16_t *__restrict__ X, const int8_t *__restrict__ B,
                                                         IgemmParams p, EpiDev e, int ngroups) {
  resolve_exp2(e);
  typedef typename EpiOf<EPI>::type S;
  constexpr int EPI_STRIDE = 32 + 8;
  constexpr int DEPTH = 2;
  extern __shared__ __attribute__((aligned(16))) int stem_lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int n_base = blockIdx.y * 32;
  const int rowbytes = p.W * 16;

  v4i fb[STEPS];
  int wsum = 0;
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int n = n_base + frow;
    fb[s] = v4i{0, 0, 0, 0};
    if (n < p.N) fb[s] = *reinterpret_cast<const v4i *>(B + (int64_t)n * p.K + s * 32 + fhalf * 16);
#pragma unroll
    for (int d = 0; d < 4; ++d) wsum = __builtin_amdgcn_sdot4(fb[s][d], 0x01010101, wsum, false);
  }
  const unsigned wcorr = (unsigned)(wsum + __shfl_xor(wsum, 32, 64)) << 7;  // 128 * sum_k w[n][k], n = column of this lane
  const int n_lane = epi_lane_channel<1>(n_base, lane);
  const EpiLane L = epi_lane_setup<S>(n_lane, n_lane < p.N, e);

  auto load_a = [&](int g, v4i (&fa)[STEPS][2]) {
    const unsigned m = (unsigned)g * 32u + (unsigned)frow;
    const bool ok = g < ngroups && m < (unsigned)p.M;
    const unsigned mm = ok ? m : 0u;
    const unsigned t = mm / (unsigned)p.Wo, wo = mm - t * (unsigned)p.Wo;
    const unsigned img = t / (unsigned)p.Ho, ho = t - img * (unsigned)p.Ho;
    const int8_t *base = reinterpret_cast<const int8_t *>(X) +
                         (size_t)((img * (unsigned)p.H + ho * (unsigned)p.sh) * (unsigned)p.W + wo * (unsigned)p.sw) * 16 + fhalf * 32;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int8_t *row = base + (int64_t)s * p.dh * rowbytes;
      fa[s][0] = *reinterpret_cast<const v4i_a4 *>(row);
      fa[s][1] = *reinterpret_cast<const v4i_a4 *>(row + 16);
    }
  };

  const int gw = blockIdx.x * 4 + wave, nw = gridDim.x * 4;
  v4i ring[DEPTH][STEPS][2];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load_a(gw + d * nw, ring[d]);

  int *stage = stem_lds + wave * 32 * EPI_STRIDE;
  for (int g0 = gw; g0 < ngroups; g0 += DEPTH * nw) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      const int g = g0 + d * nw;
      if (g >= ngroups) break;  // wave-uniform
      v16i acc_hi, acc_lo;
      const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        v4i hi, lo;
        split_i16(ring[d][s][0], ring[d][s][1], hi, lo);
        acc_hi = __builtin_amdgcn_mfma_i32_32x32x32_i8(hi, fb[s], s == 0 ? zero : acc_hi, 0, 0, 0);
        acc_lo = __builtin_amdgcn_mfma_i32_32x32x32_i8(lo, fb[s], s == 0 ? zero : acc_lo, 0, 0, 0);
      }
      load_a(g + DEPTH * nw, ring[d]);
      v16i acc[1][1];
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[0][0][r] = (int)(((unsigned)acc_hi[r] << 8) + (unsigned)acc_lo[r] + wcorr);
      igemm_epilogue_vec<1, 1, EPI>(acc, stage, (int64_t)g * 32, n_base, lane, p, e, L);
    }
  }
}

// convolution of a framed 8-channel int16 image with 3-row filters of 4 taps (zero tap included);
// -1 when the shape is not this kernel's
static int conv2d_stem_a16(const void *x, const void *w, int N, int H, int W, int Co, int kh, int kw, int sh, int sw,
                           int dh, int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  if (kw != 4 || kh != 3 || Co > 128 || (int64_t)N * Ho * Wo < 4096) return -1;
  if ((int64_t)N * Ho * Wo >= (1ll << 31) - 64 || (int64_t)N * H * W >= (1ll << 27)) return -1;  // 32-bit indices
  IgemmParams p = {};
  p.M = (int64_t)N * Ho * Wo;
  p.N = Co;
  p.K = kh * kw * 8;
  p.H = H; p.W = W; p.Ho = Ho; p.Wo = Wo; p.kh = kh; p.kw = kw; p.sh = sh; p.sw = sw; p.dh = dh;
  if (pick_epilogue(p.N, e) == EPI_SCALAR) return -1;
  constexpr int LDS_BYTES = 4 * 32 * (32 + 8) * 4;
  const int64_t ngroups = (p.M + 31) / 32;
  const int ngrp = (p.N + 31) / 32;
  int blocks = (int)((ngroups + 3) / 4);
  if (blocks > 256 * 4 / ngrp) blocks = 256 * 4 / ngrp;
  if (pick_epilogue(p.N, e) == EPI_LK_Q16)  // a detector's first layer: leaky ReLU, int16 out
    stem_a16_kernel<3, EPI_LK_Q16><<<dim3(blocks, ngrp), 256, LDS_BYTES, s>>>((const int16_t *)x, (const int8_t *)w, p, e,
                                                                             (int)ngroups);
  else
    stem_a16_kernel<3, EPI_VECTOR><<<dim3(blocks, ngrp), 256, LDS_BYTES, s>>>((const int16_t *)x, (const int8_t *)w, p, e,
                                                                             (int)ngroups);
  return launch_status();
}

int conv2d_mfma_a16(const void *x, const void *w, int N, int H, int W, int Ci, int Co, int kh, int kw, int ph, int pw,
                    int sh, int sw, int dh, int dw, int Ho, int Wo, const EpiDev &e, hipStream_t s) {
  IgemmParams p = {};
  p.M = (int64_t)N * Ho * Wo;
  p.N = Co;
  p.H = H; p.W = W; p.Ci = Ci; p.Ho = Ho; p.Wo = Wo;
  p.kh = kh; p.kw = kw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
  p.K = kh * kw * Ci;
  if (p.M >= (1ll << 31)) return -1;  // the loaders split a pixel index with 32-bit divisions
  if (Ci == 8 && ph == 0 && pw == 0 && dw == 1) {  // framed few-channel image: streaming kernel
    const int st = conv2d_stem_a16(x, w, N, H, W, Co, kh, kw, sh, sw, dh, Ho, Wo, e, s);
    if (st >= 0) return st;
  }
  // a pointwise convolution is a plain GEMM over the pixels: row address = index x K, no pixel split and no
  // tap masks in front of the first load
  const char *as_gemm = tuning_env("CATCHQ_PW_AS_GEMM");
  if (kh == 1 && kw == 1 && sh == 1 && sw == 1 && ph == 0 && pw == 0 && !(as_gemm && atoi(as_gemm) == 0)) {
    const int st = igemm_a16_launch(LOAD_GEMM, x, w, p, e, p.M * Ci * 2, (int64_t)Co * Ci, s);
    if (st >= 0) return st;
  }
  return igemm_a16_launch(LOAD_CONV, x, w, p, e, (int64_t)N * H * W * Ci * 2, (int64_t)Co * p.K, s);
}

}  // namespace catchq
