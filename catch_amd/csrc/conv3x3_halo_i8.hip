// 3x3 int8 convolution (stride 1 or 2, padding 1) with the input patch resident in LDS.
//
// The implicit-GEMM kernel fetches every input pixel nine times (once per filter tap) and synchronises
// its block once per 64 bytes of K, which leaves a 3x3 layer bound by the load path when the image is
// large and by the per-step latency chain when it is small.  Here a block owns a band of whole output
// rows of one image (or a few whole small images): it loads the band's input rows plus a one-pixel
// frame into LDS ONCE -- rows and columns outside the image arrive as zeros from the out-of-range
// buffer loads, which is the convolution's padding -- and every filter tap then reads the A fragments
// of its pixels from that patch at a shifted address.  Only the weights stream: stages of 256 bytes of
// K for the block's output channels through a three-slot LDS ring, one barrier per stage, so a wave
// issues 16 to 32 MFMAs per synchronisation instead of two.
//
//   patch        PR x PC pixels of CI bytes; the 16-byte chunks of a pixel are XOR-swizzled (on the source
//                side of the LDS-DMA) with a key that counts output pixels, so that the ds_read_b128 of
//                32 consecutive output pixels at one tap and one logical chunk spread over all banks
//   output tile  P = TR * Wo consecutive output pixels (rows m0 .. m0 + P of the GEMM view), split
//                into 32-row MFMA sub-tiles; wave w owns sub-tiles w and w + 4; BN = 32 * TN channels
//   K order      (tap, channel), as the weight tensor [Co][3][3][Ci] stores it; a stage may end past
//                K: weights beyond K read as zeros, the patch address of a tap >= 9 is clamped
//
// The integer sums are those of any other route (exact), the epilogue is the shared one.
//
// With a head (HEAD = true) the patch is not loaded but computed: the block input goes through the 1x1
// convolution + ReLU + int8 requantization that precedes the 3x3 layer in a bottleneck block, for the band's rows
// plus the one-pixel halo, and the requantized values are written straight into the LDS patch; that convolution's
// output never reaches memory and its launch disappears.  A lane loads the A fragments of its pixels (rows of K1
// contiguous bytes) straight from global memory, the 1x1 filters sit in the ring slot that the 3x3 weights need
// last, and the two operands are swapped in the MFMA so that a lane ends up with four consecutive channels of one
// pixel: one dword of the patch.  Halo rows are computed by the bands on both sides: (TR + 2) / TR of a cheap
// convolution.  Pixels outside the image are zeros in the patch (the 3x3 layer's padding is applied to the head's
// output, not to its input).
#include <type_traits>

#include "conv3x3_halo.h"

namespace catchq {

// The 1x1 convolution + ReLU + int8 requantization in front of the 3x3 layer (HEAD kernels):
//   q1[p][c] = sat(rne(relu(float(acc1) * 2^exp2 / div[c] + bias[c]) * 2^-q_position)),  acc1 = sum_k x[p][k] * w[c][k]
struct HeadDev {
  const int8_t *w;                 // [CI][K1]
  const float *div, *rcp, *bias;   // [CI] each; rcp = correctly rounded reciprocals of div
  int exp2, q_neg_pos;
  unsigned w_bytes;
};

// K1 = 0: the patch is loaded from X [N, Hi, Wi, CI]; K1 > 0: X is the head's input [N, H, W, K1] and the patch
// is computed (stride 1, band mode, one block over all output channels, four waves, TMA = sub-tiles of the
// head's rows per wave)
template <int CI, int TN, int TMW, int S, int EPI, int NW = 4, int K1 = 0, int TMA = 1>
__global__ __launch_bounds__(64 * NW) void conv3x3_halo_kernel(const int8_t *__restrict__ X, const int8_t *__restrict__ Wt,
                                                          HaloParams hp, EpiDev e, HeadDev hd) {
  resolve_exp2(e);
  constexpr bool HEAD = K1 > 0;
  constexpr int CH = CI / 16;         // 16-byte chunks per pixel
  constexpr int LOG_CI = CI == 64 ? 6 : CI == 128 ? 7 : CI == 256 ? 8 : 9;
  constexpr int BN = 32 * TN;
  constexpr int KS = 256;             // bytes of K per weight stage
  constexpr int STAGES = 3;
  constexpr int B_STAGE = BN * KS;
  constexpr int NIB = BN / 4 / NW;    // weight DMA instructions (4 rows x 256 bytes) per wave and stage
  constexpr int K = 9 * CI;
  constexpr int NSTAGES = (K + KS - 1) / KS;
  constexpr int SUBS_PER_TAP = CI / 32;  // MFMA K steps (32 bytes) per filter tap
  constexpr int SUBS_PER_STAGE = KS / 32;
  static_assert(NW == 4 || NW == 8, "four or eight waves");
  static_assert(BN / 4 % NW == 0, "the weight rows must split evenly over the waves");
  static_assert(TMW == 1 || TMW == 2, "one or two sub-tiles per wave");
  // 1 KiB alignment: fragment addresses are formed by XOR-ing chunk bits into a precomputed address
  extern __shared__ __attribute__((aligned(1024))) int8_t lds_dyn[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int logical = xcd_remap(blockIdx.x, hp.nblocks);
  const int tile_n = logical % hp.tiles_n;
  const int tile_m = logical / hp.tiles_n;
  const int n0 = tile_n * BN;
  // first image, first output row and output pixel count of the tile
  int img0, ho0, p_tile;
  if (hp.image_mode) {
    img0 = tile_m * (hp.TR / hp.H);
    ho0 = 0;
    p_tile = hp.P;
  } else {
    img0 = tile_m / hp.bands;
    ho0 = (tile_m - img0 * hp.bands) * hp.TR;
    const int rows = hp.H - ho0 < hp.TR ? hp.H - ho0 : hp.TR;
    p_tile = rows * hp.W;
  }
  const int64_t m0 = ((int64_t)img0 * hp.H + ho0) * hp.W;
  const int patch_bytes = (hp.PR * hp.PC * CI + 1023) / 1024 * 1024;
  int8_t *ring = lds_dyn + patch_bytes;

  const __amdgpu_buffer_rsrc_t rsrc_x = __builtin_amdgcn_make_buffer_rsrc((void *)X, 0, (int)hp.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_w = __builtin_amdgcn_make_buffer_rsrc((void *)Wt, 0, (int)hp.w_bytes, 0x00020000);
  constexpr unsigned OOB = 0x80000000u;

  // ---- the input patch: every 16-byte chunk once ------------------------------------------------------------
  if constexpr (!HEAD) {
    const int npix = hp.PR * hp.PC;
    const int ninstr = patch_bytes / 1024;
    constexpr int PPI = 64 / CH > 0 ? 64 / CH : 1;  // pixels per DMA instruction (CH <= 32)
    // this lane's pixel in the wave's first instruction, then PPI * 4 pixels further per round
    unsigned pix = (unsigned)(wave * 64 + lane) / CH;  // (NW waves: instruction i of the patch belongs to wave i % NW)
    const unsigned phys = (unsigned)lane % CH;
    unsigned pr = pix / (unsigned)hp.PC, pc = pix - pr * (unsigned)hp.PC;
    for (int i = wave; i < ninstr; i += NW) {
      int img = img0, hi;
      if (hp.image_mode) {
        const unsigned g = pr / (unsigned)hp.img_rows;
        img += (int)g;
        hi = (int)(pr - g * (unsigned)hp.img_rows) - 1;
      } else {
        hi = ho0 * S - 1 + (int)pr;
      }
      const int wi = (int)pc - 1;
      const bool ok = (int)pix < npix && img < hp.N && (unsigned)hi < (unsigned)hp.Hi && (unsigned)wi < (unsigned)hp.Wi;
      const unsigned src = (unsigned)((img * hp.Hi + hi) * hp.Wi + wi) * (unsigned)CI + ((phys ^ halo_swz<CH>(halo_key<S>(pr, pc, (unsigned)hp.W))) << 4);
      const unsigned voff = select_u32(ok, src, OOB);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_ptr_t)(lds_dyn + i * 1024), 16, (int)voff, 0, 0, 0);
      pix += PPI * NW;
      pc += PPI * NW;
      while (pc >= (unsigned)hp.PC) { pc -= (unsigned)hp.PC; ++pr; }
    }
  }

  // ---- the weight ring ---------------------------------------------------------------------------------------
  // instruction b of a stage: rows 4b .. 4b+3 of the block's BN weight rows, 16 chunks each
  unsigned wbase[NIB];
  bool wrow_ok[NIB];
#pragma unroll
  for (int t = 0; t < NIB; ++t) {
    const int rb = (wave * NIB + t) * 4 + (lane >> 4);
    wrow_ok[t] = n0 + rb < hp.Co;
    wbase[t] = (unsigned)(n0 + rb) * (unsigned)K + ((((unsigned)lane & 15u) ^ ((unsigned)rb & 15u)) << 4);
  }
  auto issue_weights = [&](int stage, int slot_off) {
    const unsigned k0 = (unsigned)stage * KS;
#pragma unroll
    for (int t = 0; t < NIB; ++t) {
      const unsigned kk = k0 + ((((unsigned)lane & 15u) ^ ((unsigned)((wave * NIB + t) * 4 + (lane >> 4)) & 15u)) << 4);
      const unsigned voff = select_u32(wrow_ok[t] && kk < (unsigned)K, wbase[t] + k0, OOB);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (lds_ptr_t)(ring + slot_off + (wave * NIB + t) * 1024), 16, (int)voff, 0,
                                               0, 0);
    }
  };
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int8_t *)lds_dyn;
  if constexpr (!HEAD) {
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue_weights(s, s * B_STAGE);
  } else {
    // ---- the head: patch = requantized ReLU of the 1x1 convolution of the block input ------------------------------
    static_assert(S == 1 && (NW == 4 || NW == 8) && (K1 == 64 || K1 == 256) && CI * K1 <= B_STAGE, "head shapes");
    constexpr int KS1 = K1 / 32;   // MFMA K steps of the head
    constexpr int TN1 = CI / 32;   // its output channel tiles
    constexpr int CHW = K1 / 16;   // 16-byte chunks per filter row
    constexpr int W1_INSTR = CI * K1 / 1024;             // filter DMA instructions of the block
    constexpr int NI1 = (W1_INSTR + NW - 1) / NW;        // ... per wave (the last waves may have none)
    const unsigned w1_slot = (unsigned)patch_bytes + (STAGES - 1) * B_STAGE;  // the ring slot filled last
    const unsigned const_off = (unsigned)patch_bytes + STAGES * B_STAGE;      // div', rcp', bias: CI floats each
    {  // filters -> LDS, chunk index XOR-ed with a row key so that the fragment reads of 16 rows spread over the banks
      const __amdgpu_buffer_rsrc_t rsrc_w1 = __builtin_amdgcn_make_buffer_rsrc((void *)hd.w, 0, (int)hd.w_bytes, 0x00020000);
#pragma unroll
      for (int t = 0; t < NI1; ++t) {
        const int b = wave * NI1 + t;
        if (b >= W1_INSTR) break;  // wave-uniform
        unsigned row, phys, key;
        if constexpr (CHW >= 16) { row = (unsigned)b * (64 / CHW) + ((unsigned)lane / CHW); phys = (unsigned)lane % CHW; key = row & 15u; }
        else { row = (unsigned)b * 16 + ((unsigned)lane >> 2); phys = (unsigned)lane & 3u; key = (row >> 2) & 3u; }
        const unsigned voff = row * (unsigned)K1 + ((phys ^ key) << 4);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w1, (lds_ptr_t)(lds_dyn + w1_slot + b * 1024), 16, (int)voff, 0, 0, 0);
      }
    }
    // the rows of the head: patch rows 0 .. PR-1 of W pixels each (the patch's border columns are zeros), i.e. the
    // contiguous input pixels base_pix .. base_pix + PR * W; rows above / below the image are not computed
    const int m_a = hp.PR * hp.W;
    const int row_lo = (ho0 == 0) ? hp.W : 0;
    const int rows_in = hp.H - ho0 + 1 < hp.PR ? hp.H - ho0 + 1 : hp.PR;
    const int row_hi = rows_in * hp.W;
    const int base_pix = (img0 * hp.H + ho0 - 1) * hp.W;
    v4i fa[TMA][KS1];
    bool pvalid[TMA];
#pragma unroll
    for (int i = 0; i < TMA; ++i) {
      const int r_a = (wave + NW * i) * 32 + frow;
      pvalid[i] = r_a >= row_lo && r_a < row_hi;
      const int8_t *src = X + (int64_t)(base_pix + r_a) * K1 + fhalf * 16;
#pragma unroll
      for (int ks = 0; ks < KS1; ++ks) {
        fa[i][ks] = v4i{0, 0, 0, 0};
        if (pvalid[i]) fa[i][ks] = *reinterpret_cast<const v4i *>(src + ks * 32);
      }
    }
    // per-channel constants with the power of two folded in (as epi_lane_setup does), staged once per block
    if (threadIdx.x < CI) {
      const int c = threadIdx.x;
      float *cst = reinterpret_cast<float *>(lds_dyn + const_off);
      cst[c] = __builtin_ldexpf(hd.div[c], -hd.exp2);
      cst[CI + c] = __builtin_ldexpf(hd.rcp[c], hd.exp2);
      cst[2 * CI + c] = hd.bias[c];
    }
    // the patch's border columns
    for (int t = threadIdx.x; t < hp.PR * 2 * CH; t += 64 * NW) {
      const int pr = t / (2 * CH), rest = t - pr * (2 * CH);
      const int pc = (rest < CH) ? 0 : hp.PC - 1;
      *reinterpret_cast<v4i *>(lds_dyn + (pr * hp.PC + pc) * CI + (rest % CH) * 16) = v4i{0, 0, 0, 0};
    }
    CATCHQ_VMCNT(0);
    __syncthreads();  // filters, constants and border columns are in place
    // the 3x3 layer's first weight stages travel while the head is computed
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue_weights(s, s * B_STAGE);

    // filter fragment of channel tile j, K step ks: row j*32 + frow, logical chunk 2*ks + fhalf
    unsigned w1_addr[TN1];
#pragma unroll
    for (int j = 0; j < TN1; ++j) {
      const unsigned n = (unsigned)(j * 32 + frow);
      const unsigned key = (CHW >= 16) ? (n & 15u) : ((n >> 2) & 3u);
      w1_addr[j] = lds_base + w1_slot + n * (unsigned)K1 + ((((unsigned)fhalf) ^ key) << 4);
    }
    const float q_hi = __builtin_ldexpf(127.0f, -hd.q_neg_pos), q_sc = __builtin_ldexpf(1.0f, hd.q_neg_pos);
#pragma unroll
    for (int i = 0; i < TMA; ++i) {
      const int sub = wave + NW * i;
      if (sub * 32 >= m_a) break;  // wave-uniform
      v16i acc1[TN1];
#pragma unroll
      for (int j = 0; j < TN1; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc1[j][r] = 0;
      // operands swapped: the 32x32 result has channels down the rows, so a lane holds channels
      // 8g + 4*fhalf .. + 3 (g = 0 .. 3) of pixel frow
#pragma unroll
      for (int ks = 0; ks < KS1; ++ks) {
        v4i fw[TN1];
#pragma unroll
        for (int j = 0; j < TN1; ++j) fw[j] = ds_read_b128<0>(w1_addr[j] ^ (unsigned)(ks << 5));
#pragma unroll
        for (int j = 0; j < TN1; ++j) lgkm_wait<0>(fw[j]);
#pragma unroll
        for (int j = 0; j < TN1; ++j) acc1[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw[j], fa[i][ks], acc1[j], 0, 0, 0);
      }
      const int r_a = sub * 32 + frow;
      const unsigned pr = (unsigned)r_a / (unsigned)hp.W, pc = (unsigned)r_a - pr * (unsigned)hp.W + 1u;
      const unsigned pix_addr = lds_base + (pr * (unsigned)hp.PC + pc) * (unsigned)CI;
      const unsigned sw = halo_swz<CH>(halo_key<1>(pr, pc, (unsigned)hp.W));
#pragma unroll
      for (int j = 0; j < TN1; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const unsigned c0 = (unsigned)(j * 32 + 8 * g + 4 * fhalf);
          const unsigned caddr = lds_base + const_off + c0 * 4;
          v4i dv = ds_read_b128<0>(caddr), rc = ds_read_b128<CI * 4>(caddr), bs = ds_read_b128<CI * 8>(caddr);
          lgkm_wait<0>(dv, rc, bs);
          unsigned b[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            float x = div_by_rcp((float)acc1[j][4 * g + t], __int_as_float(dv[t]), __int_as_float(rc[t])) + __int_as_float(bs[t]);
            x = __builtin_amdgcn_fmed3f(x, 0.0f, q_hi);  // ReLU and the upper clamp; NaN -> 0
            b[t] = __builtin_bit_cast(unsigned, __builtin_fmaf(x, q_sc, 12582912.0f));
          }
          const unsigned lo = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
          const unsigned hi2 = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
          const unsigned packed = pvalid[i] ? (lo | hi2) : 0u;
          const unsigned dst = pix_addr + (((c0 >> 4) ^ sw) << 4) + (c0 & 15u);
          if (r_a < m_a) asm volatile("ds_write_b32 %0, %1" ::"v"(dst), "v"(packed) : "memory");
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }

  // ---- this lane's fragment addresses: one per sub-tile and filter tap ------------------------------------------
  // The A fragment of K step c (32 bytes: chunks 2c and 2c+1, this lane takes chunk 2c + fhalf) of a pixel sits at
  //   pixel * CI + (((2c + fhalf) ^ swz(pixel)) << 4)  =  [pixel * CI + ((fhalf ^ swz(pixel)) << 4)]  ^  (c << 5):
  // the bracket is fixed per (sub-tile, tap), the XOR mask is the same for every lane.
  unsigned a0[TMW][9];
#pragma unroll
  for (int i = 0; i < TMW; ++i) {
    int idx = (wave + NW * i) * 32 + frow;
    if (idx >= p_tile) idx = p_tile - 1;
    const unsigned tr = (unsigned)idx / (unsigned)hp.W, wo = (unsigned)idx - tr * (unsigned)hp.W;
    unsigned prow = tr;
    if (hp.image_mode) {
      const unsigned g = tr / (unsigned)hp.H;
      prow = g * (unsigned)hp.img_rows + (tr - g * (unsigned)hp.H) * S;
    } else {
      prow *= S;
    }
    const unsigned pcol = wo * S;
#pragma unroll
    for (int t = 0; t < 9; ++t) {
      const unsigned pr_t = prow + (unsigned)(t / 3), pc_t = pcol + (unsigned)(t % 3);
      const unsigned pix = pr_t * (unsigned)hp.PC + pc_t;
      a0[i][t] = lds_base + pix * (unsigned)CI + ((((unsigned)fhalf) ^ halo_swz<CH>(halo_key<S>(pr_t, pc_t, (unsigned)hp.W))) << 4);
    }
  }
  // weights: row frow of a 32-row block, chunk (2c + fhalf) ^ (frow & 15) of the stage's 16
  const unsigned ring_base = lds_base + (unsigned)patch_bytes;
  const unsigned b0 = ring_base + (unsigned)frow * KS + ((((unsigned)fhalf) ^ ((unsigned)frow & 15u)) << 4);

  v16i acc[TMW][TN];
#pragma unroll
  for (int i = 0; i < TMW; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  auto multiply = [&](v4i (&fa)[TMW], v4i (&fb)[TN]) {
#pragma unroll
    for (int i = 0; i < TMW; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
  };

  // the patch and the first weight stages: everything issued so far has landed, for every wave
  CATCHQ_VMCNT(0);
  __syncthreads();

  // The whole K loop is unrolled: tap and chunk of every step are compile-time constants, a step costs one XOR
  // per fragment address.  g counts 32-byte K steps; every SUBS_PER_STAGE of them a new weight stage begins.
  constexpr int NSUB_K = 9 * SUBS_PER_TAP;
  unsigned bslot = b0;  // this lane's weight fragment address in the stage being read
  int wr_off = (STAGES - 1) * B_STAGE, rd_off = 0;
  v4i fa[2][TMW], fb[2][TN];
  auto fetch = [&](v4i (&xa)[TMW], v4i (&xb)[TN], int tap, int c, int cb) {
#pragma unroll
    for (int i = 0; i < TMW; ++i) xa[i] = ds_read_b128<0>(a0[i][tap] ^ (unsigned)(c << 5));
    xb[0] = ds_read_b128<0>(bslot ^ (unsigned)(cb << 5));
    if constexpr (TN > 1) xb[1] = ds_read_b128<32 * KS>(bslot ^ (unsigned)(cb << 5));
  };
  static_for<0, NSUB_K>([&](auto gc) {
    constexpr int g = decltype(gc)::value;
    constexpr int in_stage = g % SUBS_PER_STAGE;
    if constexpr (in_stage == 0) {
      constexpr int stage = g / SUBS_PER_STAGE;
      if constexpr (stage > 0) {
        CATCHQ_VMCNT(NIB * (STAGES - 2));  // this wave's part of the stage has landed
        __builtin_amdgcn_s_barrier();      // ... and everyone's; the slot refilled below is no longer read
      }
      issue_weights(stage + STAGES - 1, wr_off);
      bslot = b0 + (unsigned)rd_off;
      rd_off = (rd_off + B_STAGE == STAGES * B_STAGE) ? 0 : rd_off + B_STAGE;
      wr_off = (wr_off + B_STAGE == STAGES * B_STAGE) ? 0 : wr_off + B_STAGE;
      fetch(fa[g & 1], fb[g & 1], g / SUBS_PER_TAP, g % SUBS_PER_TAP, in_stage);
    }
    // the next step's fragments are requested before this step's are waited for, inside a stage
    constexpr bool more = (g + 1 < NSUB_K) && ((g + 1) % SUBS_PER_STAGE != 0);
    if constexpr (more) {
      fetch(fa[(g + 1) & 1], fb[(g + 1) & 1], (g + 1) / SUBS_PER_TAP, (g + 1) % SUBS_PER_TAP, (g + 1) % SUBS_PER_STAGE);
      lgkm_wait_frags<TMW + TN, TMW, TN>(fa[g & 1], fb[g & 1]);
    } else {
      lgkm_wait_frags<0, TMW, TN>(fa[g & 1], fb[g & 1]);
    }
    multiply(fa[g & 1], fb[g & 1]);
  });
  CATCHQ_VMCNT(0);
  __syncthreads();  // the ring is dead: it becomes the epilogue's staging area

  IgemmParams p = {};
  p.N = hp.Co;
  p.M = (m0 + p_tile < hp.M) ? m0 + p_tile : hp.M;  // rows past the tile belong to the next one
  constexpr int EPI_STRIDE = 32 * TN + 8;
  // four staging areas: eight waves take turns in two groups, so that the epilogue needs no more LDS than the
  // weight ring did and two blocks still fit a compute unit where the patch is small
  int *stage_w = reinterpret_cast<int *>(ring) + (wave & 3) * 32 * EPI_STRIDE;
  auto finish = [&]() {
#pragma unroll
    for (int i = 0; i < TMW; ++i) {
      const int si = wave + NW * i;
      if (si * 32 >= p_tile) break;  // wave-uniform
      igemm_epilogue<1, TN, EPI>(reinterpret_cast<v16i(&)[1][TN]>(acc[i]), stage_w, m0 + si * 32, n0, lane, p, e);
    }
  };
  if constexpr (NW == 4) {
    finish();
  } else {
    if (wave < 4) finish();
    __syncthreads();
    if (wave >= 4) finish();
  }
}

template <int CI, int TN, int TMW, int S, int EPI, int NW, int K1 = 0, int TMA = 1>
static int launch_halo_epi(const void *x, const void *w, const HaloParams &hp, const EpiDev &e, int lds_bytes, hipStream_t s,
                           const HeadDev &hd = HeadDev{}) {
  auto kern = conv3x3_halo_kernel<CI, TN, TMW, S, EPI, NW, K1, TMA>;
  if (lds_bytes > 64 * 1024) {
    static std::atomic<bool> raised[64];
    if (raise_lds_limit((const void *)kern, 160 * 1024, raised) != CATCHQ_OK) return CATCHQ_ERR_LAUNCH;
  }
  kern<<<hp.nblocks, 64 * NW, lds_bytes, s>>>((const int8_t *)x, (const int8_t *)w, hp, e, hd);
  return launch_status();
}

template <int CI, int TN, int TMW, int S, int NW = 4>
static int launch_halo_tm(const void *x, const void *w, const HaloParams &hp, const EpiDev &e, int lds_bytes, hipStream_t s) {
  switch (pick_epilogue(hp.Co, e)) {
    case EPI_SCALAR: return -1;
    case EPI_Q8_RELU: return launch_halo_epi<CI, TN, TMW, S, EPI_Q8_RELU, NW>(x, w, hp, e, lds_bytes, s);
    default: return launch_halo_epi<CI, TN, TMW, S, EPI_VECTOR, NW>(x, w, hp, e, lds_bytes, s);
  }
}

template <int CI, int S>
static int launch_halo(const void *x, const void *w, const HaloParams &hp, const EpiDev &e, int tn, int lds_bytes, int waves,
                       hipStream_t s) {
  // five to eight sub-tiles on eight waves: one each, two waves per SIMD that overlap each other's fragment
  // fetches and multiplications
  if (waves == 8)
    return tn == 2 ? launch_halo_tm<CI, 2, 1, S, 8>(x, w, hp, e, lds_bytes, s) : launch_halo_tm<CI, 1, 1, S, 8>(x, w, hp, e, lds_bytes, s);
  // four or fewer sub-tiles: one per wave, no second set of accumulators
  if (hp.nsub <= 4)
    return tn == 2 ? launch_halo_tm<CI, 2, 1, S>(x, w, hp, e, lds_bytes, s) : launch_halo_tm<CI, 1, 1, S>(x, w, hp, e, lds_bytes, s);
  return tn == 2 ? launch_halo_tm<CI, 2, 2, S>(x, w, hp, e, lds_bytes, s) : launch_halo_tm<CI, 1, 2, S>(x, w, hp, e, lds_bytes, s);
}

// 3x3, stride 1 or 2 (both directions alike), padding 1, no dilation, Ci in {64, 128, 256, 512} (stride 2: not 64);
// input [N, Hi, Wi, Ci]; -1: not this kernel's shape
int conv2d_halo_i8(const void *x, const void *w, int N, int Hi, int Wi, int Ci, int Co, int stride, const EpiDev &e,
                   hipStream_t s) {
  HaloParams hp;
  int tn, lds_bytes, waves;
  if (!halo_plan(N, Hi, Wi, Ci, Co, stride, hp, tn, lds_bytes, waves, 0, 1, e.cus)) return -1;
  if (stride == 2) {
    switch (Ci) {
      case 128: return launch_halo<128, 2>(x, w, hp, e, tn, lds_bytes, waves, s);
      case 256: return launch_halo<256, 2>(x, w, hp, e, tn, lds_bytes, waves, s);
      default: return launch_halo<512, 2>(x, w, hp, e, tn, lds_bytes, waves, s);
    }
  }
  switch (Ci) {
    case 64: return launch_halo<64, 1>(x, w, hp, e, tn, lds_bytes, waves, s);
    case 128: return launch_halo<128, 1>(x, w, hp, e, tn, lds_bytes, waves, s);
    case 256: return launch_halo<256, 1>(x, w, hp, e, tn, lds_bytes, waves, s);
    default: return launch_halo<512, 1>(x, w, hp, e, tn, lds_bytes, waves, s);
  }
}

// The head's shapes: 1x1 convolution K1 -> 64 channels (+ ReLU, int8 requantization with unit scale) feeding a 3x3
// layer 64 -> 64, stride 1, padding 1, whose tiles are bands of rows; K1 in {64, 256}.
bool conv2d_head_halo_i8_ok(int N, int H, int W, int K1, int Cm, int Co) {
  if (Cm != 64 || Co != 64 || (K1 != 64 && K1 != 256)) return false;
  if ((int64_t)N * H * W * K1 >= (1ll << 31)) return false;
  HaloParams hp;
  int tn, lds_bytes, waves;
  if (!halo_plan(N, H, W, Cm, Co, 1, hp, tn, lds_bytes, waves, Co / 32)) return false;
  return hp.image_mode == 0 && waves == 4 && hp.tiles_n == 1 && (hp.PR * hp.W + 31) / 32 <= 12;
}

// x [N, H, W, K1] int8, head filters [Cm, K1], w [Co, 3, 3, Cm]; -1: not this kernel's shape
int conv2d_head_halo_i8(const void *x, int K1, const void *w1, const float *div1, const float *rcp1, const float *bias1,
                        int exp2_1, int q_position1, const void *w, int N, int H, int W, int Cm, int Co, const EpiDev &e,
                        hipStream_t s) {
  if (!conv2d_head_halo_i8_ok(N, H, W, K1, Cm, Co)) return -1;
  if (!div1 || !rcp1 || !bias1 || exp2_1 < -64 || exp2_1 > 64 || !aligned16(x) || !aligned16(w1) || !aligned16(w)) return -1;
  HaloParams hp;
  int tn, lds_bytes, waves;
  halo_plan(N, H, W, Cm, Co, 1, hp, tn, lds_bytes, waves, Co / 32);
  hp.x_bytes = (unsigned)((int64_t)N * H * W * K1);
  lds_bytes += 1024;  // the head's per-channel constants behind the ring
  if (lds_bytes > 160 * 1024) return -1;
  HeadDev hd = {(const int8_t *)w1, div1, rcp1, bias1, exp2_1, -q_position1, (unsigned)(Cm * K1)};
  const int epi = pick_epilogue(Co, e);
  if (epi == EPI_SCALAR) return -1;
#define CATCHQ_HEAD(K1_, TMW_)                                                                                                  \
  return epi == EPI_Q8_RELU ? launch_halo_epi<64, 2, TMW_, 1, EPI_Q8_RELU, 4, K1_, 3>(x, w, hp, e, lds_bytes, s, hd)             \
                            : launch_halo_epi<64, 2, TMW_, 1, EPI_VECTOR, 4, K1_, 3>(x, w, hp, e, lds_bytes, s, hd)
#define CATCHQ_HEAD8(K1_)                                                                                                       \
  return epi == EPI_Q8_RELU ? launch_halo_epi<64, 2, 1, 1, EPI_Q8_RELU, 8, K1_, 2>(x, w, hp, e, lds_bytes, s, hd)                \
                            : launch_halo_epi<64, 2, 1, 1, EPI_VECTOR, 8, K1_, 2>(x, w, hp, e, lds_bytes, s, hd)
  // Five to eight sub-tiles behind a head of 256 channels run on eight waves: the head's eleven or twelve sub-tiles of
  // matrix and epilogue work spread over twice the waves and need two thirds of the fragment registers (measured on
  // ResNet-50's first stage, 32 images: 20.7 -> 18.7 us per launch, +0.6 % end to end; the 64-channel head gains nothing)
  int head_waves = (K1 == 256 && hp.nsub > 4 && hp.nsub <= 8) ? 8 : 4;
  if (const char *t = tuning_env("CATCHQ_HEAD_WAVES")) head_waves = (atoi(t) == 8 && hp.nsub <= 8) ? 8 : 4;
  if (head_waves == 8) {
    if (K1 == 64) CATCHQ_HEAD8(64);
    CATCHQ_HEAD8(256);
  }
#undef CATCHQ_HEAD8
  if (K1 == 64) {
    if (hp.nsub <= 4) CATCHQ_HEAD(64, 1);
    CATCHQ_HEAD(64, 2);
  }
  if (hp.nsub <= 4) CATCHQ_HEAD(256, 1);
  CATCHQ_HEAD(256, 2);
#undef CATCHQ_HEAD
}

}  // namespace catchq
