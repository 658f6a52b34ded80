// Residual chain of a stage of bottleneck blocks, recomputed from int8 tensors in one launch.
//
// Block b of a stage ends in   y_b = relu(dequant(conv1x1(x_b, w_b)) + bias_b + y_{b-1}),   and the first
// block's y_{-1} is the projection shortcut dequant(conv1x1(x_s, w_s)) + bias_s.  Run block by block, every
// y_b travels through HBM in fp32 (4 bytes written, 4 read back, per output element and block) although it
// is a function of a few int8 tensors that are 4 to 16 times smaller: the blocks' 1x1 inputs x_s, x_0 .. x_b
// (K = a quarter of the output channels each).  This kernel evaluates the whole chain for its output tile:
// link after link it runs the integer contraction on the matrix cores, dequantizes the sums in the
// accumulator layout (a lane holds one output channel of 16 pixels per 32x32 tile: three per-channel
// constants per link, read from LDS) and folds them into the running fp32 values it keeps in registers.
// Only the last link's result leaves the chip, as int8 for the next convolution and / or as fp32.  Every
// fp32 operation is the one the block-by-block launches perform, in the same order, on the same integer
// sums, so the values are theirs bit for bit; what changes is that HBM traffic (8 bytes per element and
// block) is traded for matrix-core work (2K operations per element and link) and ~7 vector operations.
//
// All links' K steps form one sequence that streams through one LDS ring (LDS-DMA, 64-byte steps, three
// stages, or two when every link is a single step and the fold between two steps covers the next load):
// while the last step of a link is multiplied, the first steps of the next link are already on their way,
// so a link costs no pipeline drain of its own.
#include "igemm_i8_dma.inc"

namespace catchq {

constexpr int kChainMaxLinks = 8;

struct ChainLinkDev {
  const int8_t *x, *w;
  unsigned x_bytes, w_bytes;
  int K;                                        // bytes per input pixel = channels (multiple of 64)
  unsigned img_stride, row_stride, pix_stride;  // bytes per image / per OUTPUT row / per OUTPUT column of x
  int dense;    // stride 1 on an input of the output's extent: pixel m sits at m * K, no (image, row, column) split
  int k_shift;  // log2(K) when K is a power of two, else -1
  int exp2;
  const float *chan_div, *chan_rcp, *bias;
};

struct ChainParams {
  int64_t M;  // output pixels
  int N;      // output channels
  int Ho, Wo;
  int nlinks;
  int tiles_n, nblocks;
  float *y;
  int8_t *q;
  int q_neg_pos;
  int y_stream;
  int any_strided;  // some link is not dense
  ChainLinkDev link[kChainMaxLinks];
};

template <int BM, int BN, int STAGES, int MINW>
__global__ __launch_bounds__(256, MINW) void igemm_i8_chain_kernel(ChainParams cp) {
  constexpr int WAVES_M = 2, WAVES_N = 2, NW = 4;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  static_assert(TM == 1, "one 32-row accumulator block per wave");
  constexpr int STAGE_BYTES = (BM + BN) * 64;
  constexpr int PIPE_BYTES = STAGES * STAGE_BYTES;
  constexpr int NI = (BM + BN) / 16 / NW;  // DMA instructions (16 rows x 64 bytes) per wave and stage
  static_assert((BM + BN) / 16 % NW == 0, "tile rows must split evenly over the waves");
  constexpr int EPI_STRIDE = WN + 8;
  constexpr int EPI_BYTES = NW * 16 * EPI_STRIDE * 4;  // the staging area holds 16 rows of a wave's 32 at a time
  constexpr int FRONT_BYTES = PIPE_BYTES > EPI_BYTES ? PIPE_BYTES : EPI_BYTES;  // ring, later the staging area
  extern __shared__ __attribute__((aligned(16))) int8_t lds_dyn[];
  float *consts = reinterpret_cast<float *>(lds_dyn + FRONT_BYTES);  // [link][div' | rcp' | bias][BN]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
  const int logical = xcd_remap(blockIdx.x, cp.nblocks);
  const int tile_n = logical % cp.tiles_n;
  const int tile_m = logical / cp.tiles_n;
  const int64_t m0 = (int64_t)tile_m * BM;
  const int n0 = tile_n * BN;
  const int L = cp.nlinks;
  constexpr unsigned OOB = 0x80000000u;

  // ---- loader: NI rows per lane; an A row is an output pixel, a B row an output channel --------------------
  const int lrow = lane >> 2;
  const unsigned lchunk16 = (unsigned)(((lane & 3) ^ ((lane >> 4) & 3)) * 16);
  bool row_ok[NI];
  unsigned r_idx[NI];                      // A rows: the pixel index; B rows: the channel
  unsigned r_img[NI], r_ho[NI], r_wo[NI];  // A rows, only when some link is strided: the pixel split up
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int trow = (wave * NI + j) * 16 + lrow;
    r_img[j] = r_ho[j] = r_wo[j] = 0;
    if ((wave * NI + j) * 16 < BM) {  // wave-uniform
      const int64_t m = m0 + trow;
      row_ok[j] = m < cp.M;
      r_idx[j] = row_ok[j] ? (unsigned)m : 0u;
      if (cp.any_strided) {
        const unsigned t = r_idx[j] / (unsigned)cp.Wo;
        r_wo[j] = r_idx[j] - t * (unsigned)cp.Wo;
        r_img[j] = t / (unsigned)cp.Ho;
        r_ho[j] = t - r_img[j] * (unsigned)cp.Ho;
      }
    } else {
      const int n = n0 + trow - BM;
      row_ok[j] = n < cp.N;
      r_idx[j] = row_ok[j] ? (unsigned)n : 0u;
    }
  }
  // the issuing side of the ring: link and K offset of the next step to request
  int il = 0, ik = 0;
  unsigned base[NI];
  __amdgpu_buffer_rsrc_t rsrc_a, rsrc_b;
  auto bind_link = [&](int i) {
    const ChainLinkDev &ln = cp.link[i < L ? i : L - 1];
    rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void *)ln.x, 0, (int)ln.x_bytes, 0x00020000);
    rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void *)ln.w, 0, (int)ln.w_bytes, 0x00020000);
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const bool is_a = (wave * NI + j) * 16 < BM;  // wave-uniform
      unsigned b;
      if (is_a && !ln.dense) b = r_img[j] * ln.img_stride + r_ho[j] * ln.row_stride + r_wo[j] * ln.pix_stride;
      else b = ln.k_shift >= 0 ? r_idx[j] << ln.k_shift : r_idx[j] * (unsigned)ln.K;
      // an offset at or above 2^31 is out of range for every buffer here and stays so when a K offset is added
      base[j] = (row_ok[j] && i < L) ? b + lchunk16 : OOB;
    }
  };
  bind_link(0);
  // past the last link the slots are refilled with all-zero loads, so that the number of DMA instructions in
  // flight is the same at every step and one constant vmcnt serves all of them
  auto issue_step = [&](int stage_off) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int slot = wave * NI + j;
      const bool is_a = slot * 16 < BM;
      const unsigned voff = base[j] + (unsigned)ik;
      lds_ptr_t dst = (lds_ptr_t)(lds_dyn + stage_off + slot * 1024);
      if (is_a) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, dst, 16, (int)voff, 0, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, dst, 16, (int)voff, 0, 0, 0);
    }
    ik += 64;
    if (il < L && ik >= cp.link[il].K) {
      ++il;
      ik = 0;
      bind_link(il);
    }
  };

#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue_step(s * STAGE_BYTES);

  // ---- per-channel constants of every link -> LDS, with the power of two folded in (see epi_lane_setup) -----
  for (int idx = threadIdx.x; idx < L * BN; idx += 256) {
    const int i = idx / BN, c = idx - i * BN;
    const ChainLinkDev &ln = cp.link[i];
    float d = 1.0f, r = 1.0f, b = 0.0f;
    if (n0 + c < cp.N) {
      d = __builtin_ldexpf(ln.chan_div[n0 + c], -ln.exp2);
      r = __builtin_ldexpf(ln.chan_rcp[n0 + c], ln.exp2);
      b = ln.bias[n0 + c];
    }
    consts[(i * 3 + 0) * BN + c] = d;
    consts[(i * 3 + 1) * BN + c] = r;
    consts[(i * 3 + 2) * BN + c] = b;
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the stores above are in LDS before the first barrier below

  // ---- operand fetch addresses (LDS byte offsets), as in dma_mainloop with 64-byte rows --------------------
  const int frow = lane & 31, fhalf = lane >> 5;
  const int sw = (frow >> 2) & 3;
  const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int8_t *)lds_dyn;
  const unsigned off_k = (unsigned)((fhalf ^ sw) * 16);
  const unsigned a_row = lds_base + (unsigned)((wave_m * WM + frow) * 64);
  const unsigned b_row = lds_base + (unsigned)(BM * 64 + (wave_n * WN + frow) * 64);

  v16i acc[TN];
  float prev[TN][16];

  auto fetch = [&](v4i &fa, v4i (&fb)[TN], unsigned a_addr, unsigned b_addr) {
    fa = ds_read_b128<0>(a_addr);
    fb[0] = ds_read_b128<0>(b_addr);
    if constexpr (TN > 1) fb[1] = ds_read_b128<32 * 64>(b_addr);
    if constexpr (TN > 2) fb[2] = ds_read_b128<64 * 64>(b_addr);
    if constexpr (TN > 3) fb[3] = ds_read_b128<96 * 64>(b_addr);
  };

  int rd_off = 0, wr_off = (STAGES - 1) * STAGE_BYTES;
  // one K step of 64 bytes; FIRST: the link's sums start from zero (the matrix instruction takes the constant)
  auto step = [&](auto first_c) {
    constexpr bool FIRST = decltype(first_c)::value;
    CATCHQ_VMCNT(NI * (STAGES - 2));  // this wave's part of the stage has landed
    __builtin_amdgcn_s_barrier();     // ... and everyone's; the slot refilled below is no longer read
    const unsigned a0 = a_row + (unsigned)rd_off, b0 = b_row + (unsigned)rd_off;
    v4i fa[2], fb[2][TN];
    fetch(fa[0], fb[0], a0 + off_k, b0 + off_k);
    fetch(fa[1], fb[1], a0 + (off_k ^ 32u), b0 + (off_k ^ 32u));
    issue_step(wr_off);
    {
      v4i(&one)[1] = reinterpret_cast<v4i(&)[1]>(fa[0]);
      lgkm_wait_frags<1 + TN, 1, TN>(one, fb[0]);
    }
    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < TN; ++j)
      acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[0], fb[0][j], FIRST ? zero : acc[j], 0, 0, 0);
    {
      v4i(&one)[1] = reinterpret_cast<v4i(&)[1]>(fa[1]);
      lgkm_wait_frags<0, 1, TN>(one, fb[1]);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[1], fb[1][j], acc[j], 0, 0, 0);
    rd_off = (rd_off + STAGE_BYTES == PIPE_BYTES) ? 0 : rd_off + STAGE_BYTES;
    wr_off = (wr_off + STAGE_BYTES == PIPE_BYTES) ? 0 : wr_off + STAGE_BYTES;
  };
  // one link: its K steps, then its sums are folded into the running values: v = acc / d + bias (reciprocal
  // form), and relu(v + previous) for every link after the shortcut
  auto link = [&](int i, auto shortcut_c) {
    constexpr bool SHORTCUT = decltype(shortcut_c)::value;
    const int nsteps = cp.link[i].K >> 6;
    step(std::true_type{});
    for (int s = 1; s < nsteps; ++s) step(std::false_type{});
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int c = wave_n * WN + j * 32 + frow;
      const float d = consts[(i * 3 + 0) * BN + c], rc = consts[(i * 3 + 1) * BN + c], b = consts[(i * 3 + 2) * BN + c];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float v = div_by_rcp((float)acc[j][r], d, rc) + b;
        if constexpr (!SHORTCUT) {
          v = v + prev[j][r];
          v = (v > 0.0f) ? v : 0.0f;
        }
        prev[j][r] = v;
      }
    }
  };
  link(0, std::true_type{});
  for (int i = 1; i < L; ++i) link(i, std::false_type{});
  CATCHQ_VMCNT(0);
  __syncthreads();  // the ring is dead: it becomes the staging area

  // ---- the last link's values leave through the wave's staging area, 16 of its 32 rows at a time: a lane then
  // owns 4 consecutive channels of one pixel (16-byte fp32 / 4-byte int8 stores, rows contiguous).  The small area
  // keeps the block's LDS low enough for four blocks per compute unit with a two-stage ring. -------------------
  float *stage = reinterpret_cast<float *>(lds_dyn) + wave * 16 * EPI_STRIDE;
  constexpr int CPR = WN / 4;    // 4-channel groups per staged row
  constexpr int RPI = 64 / CPR;  // rows the wave moves per iteration
  constexpr int NIT = 16 / RPI;  // iterations per pass of 16 rows
  const int cg = lane % CPR, rsub = lane / CPR;
  const int n_w = n0 + wave_n * WN;
  const float hi = __builtin_ldexpf(127.0f, -cp.q_neg_pos);
  const float sc = __builtin_ldexpf(1.0f, cp.q_neg_pos);
  const unsigned lane_off = (unsigned)rsub * (unsigned)cp.N + (unsigned)(cg * 4);
  const unsigned it_step = (unsigned)RPI * (unsigned)cp.N;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    // rows 16h .. 16h+15 of the accumulator block are its registers 8h .. 8h+7 (row = 8 (r / 4) + 4 fhalf + r % 4);
    // the wave's LDS operations complete in order, so these writes cannot overtake the previous pass's reads
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 8; ++r) stage[(8 * (r >> 2) + 4 * fhalf + (r & 3)) * EPI_STRIDE + j * 32 + frow] = prev[j][8 * h + r];
    v4f vv[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) vv[it] = *reinterpret_cast<const v4f *>(stage + (it * RPI + rsub) * EPI_STRIDE + cg * 4);
    // an element's index: a wave-uniform 64-bit part plus a 32-bit per-lane part
    const int64_t m_w = m0 + wave_m * WM + 16 * h;
    const int64_t uni = m_w * (int64_t)cp.N + n_w;
    auto emit = [&](auto full_c) {
      constexpr bool FULL = decltype(full_c)::value;
      const bool n_ok = FULL || n_w + cg * 4 < cp.N;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        if (!FULL && !(n_ok && m_w + it * RPI + rsub < cp.M)) continue;
        const unsigned off = lane_off + it * it_step;
        if (cp.y) store_stream(reinterpret_cast<v4f *>((cp.y + uni) + off), vv[it], cp.y_stream != 0);
        if (cp.q) {
          // values are >= 0 and never NaN (the ReLU above): sat(rne(x * 2^-pos)) = low byte of the float
          // fma(min(x, 127 * 2^pos), 2^-pos, 1.5 * 2^23), as in the shared epilogue
          unsigned b[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const float x = __builtin_amdgcn_fmed3f(vv[it][t], 0.0f, hi);
            b[t] = __builtin_bit_cast(unsigned, __builtin_fmaf(x, sc, 12582912.0f));
          }
          const unsigned lo = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
          const unsigned hi2 = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
          *reinterpret_cast<unsigned *>((cp.q + uni) + off) = lo | hi2;
        }
      }
    };
    if (m_w + 16 <= cp.M && n_w + WN <= cp.N) emit(std::true_type{});  // wave-uniform: the rows lie inside the matrix
    else emit(std::false_type{});
  }
}

template <int BM, int BN, int STAGES, int MINW>
static int launch_chain(ChainParams &cp, hipStream_t s) {
  const int64_t tiles_m = (cp.M + BM - 1) / BM;
  cp.tiles_n = (cp.N + BN - 1) / BN;
  const int64_t nb = tiles_m * cp.tiles_n;
  if (nb > 0x7fffffff) return CATCHQ_ERR_SHAPE;
  cp.nblocks = (int)nb;
  constexpr int PIPE = STAGES * (BM + BN) * 64, EPI = 4 * 16 * (BN / 2 + 8) * 4;
  const int lds_bytes = (PIPE > EPI ? PIPE : EPI) + cp.nlinks * 3 * BN * 4;
  igemm_i8_chain_kernel<BM, BN, STAGES, MINW><<<cp.nblocks, 256, lds_bytes, s>>>(cp);
  return launch_status();
}

// links[0] is the projection shortcut (no activation, nothing added), links[1..] the blocks' last 1x1
// convolutions in order; -1 when the shapes are not this kernel's
int conv1x1_chain_i8(const ChainLinkDev *links, int nlinks, int N, int Ho, int Wo, int Co, float *y, int8_t *q,
                     int q_position, int sharing, hipStream_t s) {
  if (nlinks < 2 || nlinks > kChainMaxLinks || Co % 4 != 0) return -1;
  ChainParams cp = {};
  cp.M = (int64_t)N * Ho * Wo;
  if (cp.M >= (1ll << 31) || cp.M * Co >= (1ll << 40)) return -1;
  cp.N = Co;
  cp.Ho = Ho;
  cp.Wo = Wo;
  cp.nlinks = nlinks;
  cp.y = y;
  cp.q = q;
  cp.q_neg_pos = -q_position;
  cp.y_stream = (y && cp.M * Co * 4 >= stream_limit_y(planned_cus(sharing))) ? 1 : 0;
  if (!aligned16(y) || !aligned16(q)) return -1;
  for (int i = 0; i < nlinks; ++i) {
    const ChainLinkDev &ln = links[i];
    if (ln.K % 64 != 0 || ln.K <= 0 || ln.x_bytes == 0 || ln.w_bytes == 0 || ln.x_bytes >= 0x80000000u || ln.w_bytes >= 0x80000000u)
      return -1;
    if (!ln.chan_div || !ln.chan_rcp || !ln.bias || ln.exp2 < -64 || ln.exp2 > 64) return -1;
    if (!aligned16(ln.x) || !aligned16(ln.w)) return -1;
    cp.link[i] = ln;
    cp.link[i].k_shift = -1;
    for (int sft = 6; sft < 31; ++sft)
      if (ln.K == (1 << sft)) cp.link[i].k_shift = sft;
    if (!ln.dense) cp.any_strided = 1;
  }
  int variant = 0;
  if (const char *v = tuning_env("CATCHQ_CHAIN_VARIANT")) variant = atoi(v);
  if (Co < 128 || variant == 4) return launch_chain<64, 64, 3, 1>(cp, s);
  switch (variant) {
    case 1: return launch_chain<64, 128, 2, 1>(cp, s);
    case 2: return launch_chain<64, 128, 2, 4>(cp, s);
    case 3: return launch_chain<64, 128, 3, 1>(cp, s);
    default: break;
  }
  // every link a single K step: the fold between two steps covers the load of the next, a two-stage ring is
  // enough and leaves LDS for four blocks per compute unit
  int max_k = 0;
  for (int i = 0; i < nlinks; ++i) max_k = links[i].K > max_k ? links[i].K : max_k;
  int k2 = 64;
  if (const char *v = tuning_env("CATCHQ_CHAIN_K2")) k2 = atoi(v);
  if (max_k <= k2) return launch_chain<64, 128, 2, 4>(cp, s);
  return launch_chain<64, 128, 3, 4>(cp, s);
}

}  // namespace catchq
