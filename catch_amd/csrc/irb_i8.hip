// An inverted-residual block (1x1 expansion -> 3x3 depthwise -> 1x1 linear projection, all int8) in one launch.
//
// Run layer by layer, the block writes the expanded tensor (six times the block input) and reads it back, then
// does the same with the depthwise output, and late in a network each of the three launches is bound by its own
// start-up.  Here a block of eight waves owns a band of TR output rows of one image (the last band of an image may be
// shorter) and works through the hidden channels in chunks of HC = 128, 192 or 256 (the last chunk may be shorter):
//
//   1  expansion      the band's input rows (plus one row of halo on either side) sit in LDS; for every 32 pixels x
//                     32 hidden channels one wave multiplies on the matrix cores with the operands swapped (filters
//                     as A, pixels as B), so that a lane ends up with four consecutive channels of one pixel, applies
//                     the layer's own epilogue arithmetic (reciprocal-form division, bias, ReLU / ReLU6 folded into
//                     the requantizer's clamp) and writes one dword into the hidden patch in LDS.  Patch cells outside
//                     the image stay zero: the depthwise layer's padding applies to the expansion's output.
//   2  depthwise      a lane owns four channels x 2 x 4 output pixels, reads its window from the patch, transposes
//                     4 x 4 byte blocks in registers so that one v_dot4 sums a filter row (the arithmetic of the
//                     stand-alone stencil kernel), requantizes and writes the MFMA operand tile of the projection.
//   3  projection     swapped operands again: filters straight from global memory (requested before phase 2, whose
//                     vector work hides their latency), pixels from LDS; the sums of all chunks stay in registers.
//
// and the projection's epilogue (bias, optional fp32 residual, fp32 and / or int8 output) runs once at the end.
// Neither hidden tensor reaches memory.  Every integer is the one the three separate launches produce: the same
// sums, the same float operations in the same order.
//
// The block does the vector arithmetic of the three launches' epilogues (about 10 instructions per expansion
// output, 17 per depthwise output) on two waves per SIMD; what it saves is two launch start-ups and the traffic of
// the hidden tensors.  Measured on MobileNetV2's blocks (64 images) it is the faster route for a lone stream of
// launches from 14 x 14 outputs on; 7 x 7 images leave it too few blocks.
#include "igemm_i8_dma.inc"

namespace catchq {

struct IrbParams {
  int N, H, W, Cin, hid, Co, Ho, Wo;
  int TR, bands;   // output rows per tile, tiles per image
  int PR;          // input rows of a tile: (TR - 1) * S + 3
  int PRA, PCA;    // rows / columns of the hidden patch as allocated (what the stencil's windows may touch)
  int m_a, nsa;    // input pixels of a tile (PR * W) and their 32-pixel sub-tiles
  int p_out, nso;  // output pixels of a tile and their sub-tiles
  int nch;         // chunks of hidden channels (the last one may be shorter)
  int ks1;         // Cin / 32
  int nws, nwj, ncol;  // projection: waves along the pixel sub-tiles x waves along the 32-channel column tiles; column tiles
  int HG, WG;      // stencil groups (2 rows x 4 columns of outputs) per tile
  int xs, hs, as;  // LDS pitches in bytes: input pixel, patch pixel, projection operand row
  int off_c3, off_x, off_wp, off_cst, off_hp, off_a3;  // LDS regions; the output staging area overlays everything behind c3
};

constexpr int IRB_KS1MAX = 5;  // up to 160 input channels
constexpr int IRB_NW = 8;

template <int S, int MAXJ, int KS3>
__global__ __launch_bounds__(64 * IRB_NW) void irb_kernel(const int8_t *__restrict__ X, IrbStageDev s1, IrbStageDev s2,
                                                          const int8_t *__restrict__ W3, IrbParams p, EpiDev e) {
  resolve_exp2(e);
  constexpr int HC = 32 * KS3, NW = IRB_NW, NT = 64 * NW;
  constexpr int PW = 4, PH = 2;
  constexpr int NR = (PH - 1) * S + 3;
  constexpr int NG = (S == 1) ? 2 : 4;
  constexpr int NCL = 2 * NG + 2;
  extern __shared__ __attribute__((aligned(1024))) int8_t lds[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int img = blockIdx.x / p.bands, band = blockIdx.x - img * p.bands;
  const int ho0 = band * p.TR;
  const int hi0 = ho0 * S - 1;  // input row of patch row 0
  const int rows = p.Ho - ho0 < p.TR ? p.Ho - ho0 : p.TR;  // the last band of an image may be shorter
  const int p_out = rows * p.Wo;
  const int64_t base_pix = ((int64_t)img * p.H + hi0) * p.W;

  // the expansion's work items: (pixel sub-tile, 32-channel tile of the chunk), channel tiles fastest
  auto load_w1 = [&](v4i (&f)[IRB_KS1MAX], int t, int c0, int kc) {
    const int cj = t % kc;
    const int8_t *src = s1.w + (int64_t)(c0 + cj * 32 + frow) * p.Cin + fhalf * 16;
#pragma unroll
    for (int ks = 0; ks < IRB_KS1MAX; ++ks) {
      f[ks] = v4i{0, 0, 0, 0};
      if (ks < p.ks1) f[ks] = *reinterpret_cast<const v4i *>(src + ks * 32);
    }
  };
  const int kc_first = p.hid / 32 < KS3 ? p.hid / 32 : KS3;
  v4i fw1n[IRB_KS1MAX];
  if (wave < kc_first * p.nsa) load_w1(fw1n, wave, 0, kc_first);

  // ---- set-up: input rows, depthwise filters, folded per-channel constants, a zero patch ---------------------------
  // All global loads of the first round go out before anything is waited for (one memory latency, not one per
  // table); what does not fit the first round's registers follows in plain loops.
  {
    constexpr int XI = 3, CI2 = 2;
    const int cpp = p.Cin >> 4;
    const int total = p.m_a * cpp;
    float *cst = reinterpret_cast<float *>(lds + p.off_cst);
    float *c3 = reinterpret_cast<float *>(lds + p.off_c3);
    auto x_chunk = [&](int i) {
      const int px = i / cpp, k = i - px * cpp;
      const int hi = hi0 + px / p.W;
      v4i v = {0, 0, 0, 0};
      if ((unsigned)hi < (unsigned)p.H) v = *reinterpret_cast<const v4i *>(X + (base_pix + px) * p.Cin + k * 16);
      return v;
    };
    auto x_store = [&](int i, v4i v) {
      const int px = i / cpp, k = i - px * cpp;
      *reinterpret_cast<v4i *>(lds + p.off_x + px * p.xs + k * 16) = v;
    };
    // 36 filter bytes of four channels -> twelve dwords, one per channel and filter row: bytes (w0, w1, w2, 0)
    auto pack_filters = [&](int q, const int (&wraw)[9]) {
      int *dst = reinterpret_cast<int *>(lds + p.off_wp) + q * 12;
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 3; ++r) {
          unsigned v = 0;
#pragma unroll
          for (int k = 0; k < 3; ++k) {
            const int b = j * 9 + r * 3 + k;
            v |= (((unsigned)wraw[b >> 2] >> (8 * (b & 3))) & 0xffu) << (8 * k);
          }
          dst[j * 3 + r] = (int)v;
        }
    };
    auto fold = [&](int c, const float (&v)[6]) {
      cst[c] = __builtin_ldexpf(v[0], -s1.exp2);
      cst[p.hid + c] = __builtin_ldexpf(v[1], s1.exp2);
      cst[2 * p.hid + c] = v[2];
      cst[3 * p.hid + c] = __builtin_ldexpf(v[3], -s2.exp2);
      cst[4 * p.hid + c] = __builtin_ldexpf(v[4], s2.exp2);
      cst[5 * p.hid + c] = v[5];
    };
    v4i xv[XI];
    int wv[9];
    float cv[CI2][6], pv[3] = {1.0f, 1.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < XI; ++u)
      if (tid + u * NT < total) xv[u] = x_chunk(tid + u * NT);
    if (tid < p.hid / 4) {
#pragma unroll
      for (int i = 0; i < 9; ++i) wv[i] = reinterpret_cast<const int *>(s2.w)[tid * 9 + i];
    }
#pragma unroll
    for (int u = 0; u < CI2; ++u) {
      const int c = tid + u * NT;
      if (c < p.hid) {
        cv[u][0] = s1.div[c]; cv[u][1] = s1.rcp[c]; cv[u][2] = s1.bias[c];
        cv[u][3] = s2.div[c]; cv[u][4] = s2.rcp[c]; cv[u][5] = s2.bias[c];
      }
    }
    // the projection's constants, as epi_lane_setup prepares them (the power of two folded into the reciprocal form)
    if (tid < p.Co) {
      if (e.chan_div) pv[0] = e.chan_div[tid];
      if (e.chan_rcp) pv[1] = e.chan_rcp[tid];
      if (e.bias) pv[2] = e.bias[tid];
    }
    const int hpv = (p.off_a3 - p.off_hp) / 16;  // the patch region, rounded up
    for (int i = tid; i < hpv; i += NT) reinterpret_cast<v4i *>(lds + p.off_hp)[i] = v4i{0, 0, 0, 0};
#pragma unroll
    for (int u = 0; u < XI; ++u)
      if (tid + u * NT < total) x_store(tid + u * NT, xv[u]);
    if (tid < p.hid / 4) pack_filters(tid, wv);
#pragma unroll
    for (int u = 0; u < CI2; ++u)
      if (tid + u * NT < p.hid) fold(tid + u * NT, cv[u]);
    if (tid < p.Co) {
      if (e.chan_rcp) { pv[0] = __builtin_ldexpf(pv[0], -e.exp2); pv[1] = __builtin_ldexpf(pv[1], e.exp2); }
      c3[tid] = pv[0]; c3[p.Co + tid] = pv[1]; c3[2 * p.Co + tid] = pv[2];
    }
    for (int i = tid + XI * NT; i < total; i += NT) x_store(i, x_chunk(i));
    for (int q = tid + NT; q < p.hid / 4; q += NT) {
      int wr[9];
#pragma unroll
      for (int i = 0; i < 9; ++i) wr[i] = reinterpret_cast<const int *>(s2.w)[q * 9 + i];
      pack_filters(q, wr);
    }
    for (int c = tid + CI2 * NT; c < p.hid; c += NT) {
      const float v[6] = {s1.div[c], s1.rcp[c], s1.bias[c], s2.div[c], s2.rcp[c], s2.bias[c]};
      fold(c, v);
    }
  }

  float q1_hi = __builtin_ldexpf(127.0f, -s1.q_neg_pos), q2_hi = __builtin_ldexpf(127.0f, -s2.q_neg_pos);
  if (s1.relu6) q1_hi = q1_hi < 6.0f ? q1_hi : 6.0f;
  if (s2.relu6) q2_hi = q2_hi < 6.0f ? q2_hi : 6.0f;
  const float q1_sc = __builtin_ldexpf(1.0f, s1.q_neg_pos), q2_sc = __builtin_ldexpf(1.0f, s2.q_neg_pos);

  // requantized ReLU of one lane's four channels: (acc / div + bias) clamped to [0, hi], scaled, rounded to even
  auto requant4 = [&](const int *a, const v4f dv, const v4f rc, const v4f bs, float hi, float sc) -> unsigned {
    unsigned b[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      float x = div_by_rcp((float)a[t], dv[t], rc[t]) + bs[t];
      x = __builtin_amdgcn_fmed3f(x, 0.0f, hi);  // ReLU and the upper clamp; NaN -> 0
      b[t] = __builtin_bit_cast(unsigned, __builtin_fmaf(x, sc, 12582912.0f));
    }
    const unsigned lo = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
    const unsigned hi2 = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
    return lo | hi2;
  };

  // the projection: this wave's pixel sub-tile and column tiles
  const int ws = wave % p.nws, wj = wave / p.nws;
  const bool p3 = ws < p.nso;
  v16i acc3[MAXJ];
#pragma unroll
  for (int b = 0; b < MAXJ; ++b)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc3[b][r] = 0;

  __syncthreads();

  for (int ch = 0; ch < p.nch; ++ch) {
    const int c0 = ch * HC;
    const int kc = (p.hid - c0) / 32 < KS3 ? (p.hid - c0) / 32 : KS3;  // 32-channel tiles of this chunk
    // ---- 1: expansion of the chunk into the patch -------------------------------------------------------------------
    const int T1 = kc * p.nsa;
    for (int t = wave; t < T1; t += NW) {
      v4i fw1[IRB_KS1MAX];
#pragma unroll
      for (int ks = 0; ks < IRB_KS1MAX; ++ks) fw1[ks] = fw1n[ks];
      if (t + NW < T1) load_w1(fw1n, t + NW, c0, kc);
      const int sa = t / kc, cj = t - sa * kc;
      const int r_a = sa * 32 + frow;
      const bool in_tile = r_a < p.m_a;
      const int r_c = in_tile ? r_a : p.m_a - 1;
      const int8_t *xrow = lds + p.off_x + r_c * p.xs + fhalf * 16;
      v16i acc1;
#pragma unroll
      for (int r = 0; r < 16; ++r) acc1[r] = 0;
#pragma unroll
      for (int ks = 0; ks < IRB_KS1MAX; ++ks)
        if (ks < p.ks1) {
          const v4i fx = *reinterpret_cast<const v4i *>(xrow + ks * 32);
          acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw1[ks], fx, acc1, 0, 0, 0);
        }
      const int pr = r_c / p.W, wi = r_c - pr * p.W;
      const bool valid = (unsigned)(hi0 + pr) < (unsigned)p.H;
      int8_t *cell = lds + p.off_hp + (pr * p.PCA + wi + 1) * p.hs + cj * 32 + 4 * fhalf;
      const float *cbase = reinterpret_cast<const float *>(lds + p.off_cst) + c0 + cj * 32 + 4 * fhalf;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int a[4] = {acc1[4 * g], acc1[4 * g + 1], acc1[4 * g + 2], acc1[4 * g + 3]};
        const float *cb = cbase + 8 * g;
        const unsigned packed = requant4(a, *reinterpret_cast<const v4f *>(cb), *reinterpret_cast<const v4f *>(cb + p.hid),
                                         *reinterpret_cast<const v4f *>(cb + 2 * p.hid), q1_hi, q1_sc);
        if (in_tile) *reinterpret_cast<unsigned *>(cell + 8 * g) = valid ? packed : 0u;
      }
    }
    __syncthreads();  // the patch of this chunk is complete; nobody reads the previous chunk's projection operand any more

    // requests whose latency the stencil hides: the next chunk's first expansion filters, this chunk's projection filters
    if (ch + 1 < p.nch) {
      const int kn = (p.hid - c0 - HC) / 32 < KS3 ? (p.hid - c0 - HC) / 32 : KS3;
      if (wave < kn * p.nsa) load_w1(fw1n, wave, c0 + HC, kn);
    }
    v4i fw3[MAXJ][KS3];
#pragma unroll
    for (int b = 0; b < MAXJ; ++b) {
      const int j = wj + p.nwj * b;
      const int8_t *src = W3 + (int64_t)(j * 32 + frow) * p.hid + c0 + fhalf * 16;
#pragma unroll
      for (int ks = 0; ks < KS3; ++ks) {
        fw3[b][ks] = v4i{0, 0, 0, 0};
        if (p3 && j < p.ncol && ks < kc) fw3[b][ks] = *reinterpret_cast<const v4i *>(src + ks * 32);
      }
    }

    // ---- 2: depthwise stencil on the patch -> operand tile of the projection ----------------------------------------
    const int qc = kc * 8;  // channel quads of the chunk
    const int items = p.HG * p.WG * qc;
    for (int item = tid; item < items; item += NT) {
      const int t0 = item / qc, q = item - t0 * qc;
      const int hg = t0 / p.WG, wg = t0 - hg * p.WG;
      const int cl = q * 4;
      const v4i *wsrc = reinterpret_cast<const v4i *>(lds + p.off_wp + (c0 + cl) * 12);
      const v4i wq[3] = {wsrc[0], wsrc[1], wsrc[2]};
      int wa[4][3], wb[4][3];  // [channel][filter row]: bytes (w0, w1, w2, 0) and (0, w0, w1, w2)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 3; ++r) {
          wa[j][r] = wq[(j * 3 + r) >> 2][(j * 3 + r) & 3];
          wb[j][r] = (int)((unsigned)wa[j][r] << 8);
        }
      int acc[PH][PW][4];
      const int8_t *win = lds + p.off_hp + ((hg * PH * S) * p.PCA + wg * PW * S) * p.hs + cl;
#pragma unroll
      for (int ri = 0; ri < NR; ++ri) {
        unsigned xr[NCL];
#pragma unroll
        for (int col = 0; col < NCL; ++col) xr[col] = *reinterpret_cast<const unsigned *>(win + (ri * p.PCA + col) * p.hs);
        unsigned lo[NG + 1], hi2[NG + 1];
#pragma unroll
        for (int m = 0; m <= NG; ++m) {
          lo[m] = __builtin_amdgcn_perm(xr[2 * m + 1], xr[2 * m], 0x05010400u);
          hi2[m] = __builtin_amdgcn_perm(xr[2 * m + 1], xr[2 * m], 0x07030602u);
        }
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          int tt[4];
          tt[0] = (int)__builtin_amdgcn_perm(lo[g + 1], lo[g], 0x05040100u);
          tt[1] = (int)__builtin_amdgcn_perm(lo[g + 1], lo[g], 0x07060302u);
          tt[2] = (int)__builtin_amdgcn_perm(hi2[g + 1], hi2[g], 0x05040100u);
          tt[3] = (int)__builtin_amdgcn_perm(hi2[g + 1], hi2[g], 0x07060302u);
#pragma unroll
          for (int py = 0; py < PH; ++py) {
            const int r = ri - py * S;
            if (r < 0 || r > 2) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              if constexpr (S == 1) {
                acc[py][2 * g][j] = __builtin_amdgcn_sdot4(tt[j], wa[j][r], r == 0 ? 0 : acc[py][2 * g][j], false);
                acc[py][2 * g + 1][j] = __builtin_amdgcn_sdot4(tt[j], wb[j][r], r == 0 ? 0 : acc[py][2 * g + 1][j], false);
              } else {
                acc[py][g][j] = __builtin_amdgcn_sdot4(tt[j], wa[j][r], r == 0 ? 0 : acc[py][g][j], false);
              }
            }
          }
        }
      }
      const float *cb = reinterpret_cast<const float *>(lds + p.off_cst) + 3 * p.hid + c0 + cl;
      const v4f dv = *reinterpret_cast<const v4f *>(cb), rc = *reinterpret_cast<const v4f *>(cb + p.hid);
      const v4f bs = *reinterpret_cast<const v4f *>(cb + 2 * p.hid);
#pragma unroll
      for (int py = 0; py < PH; ++py) {
        const int ho_l = hg * PH + py;
#pragma unroll
        for (int px = 0; px < PW; ++px) {
          const int wo = wg * PW + px;
          const unsigned packed = requant4(acc[py][px], dv, rc, bs, q2_hi, q2_sc);
          if (ho_l < rows && wo < p.Wo) *reinterpret_cast<unsigned *>(lds + p.off_a3 + (ho_l * p.Wo + wo) * p.as + cl) = packed;
        }
      }
    }
    __syncthreads();  // the projection's operand tile is complete

    // ---- 3: projection of the chunk ----------------------------------------------------------------------------------
    if (p3) {
      const int8_t *arow = lds + p.off_a3 + (ws * 32 + frow) * p.as + fhalf * 16;
#pragma unroll
      for (int ks = 0; ks < KS3; ++ks) {
        if (ks >= kc) break;
        const v4i fa = *reinterpret_cast<const v4i *>(arow + ks * 32);
#pragma unroll
        for (int b = 0; b < MAXJ; ++b)
          if (wj + p.nwj * b < p.ncol) acc3[b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fw3[b][ks], fa, acc3[b], 0, 0, 0);
      }
    }
  }

  // ---- the projection's epilogue ---------------------------------------------------------------------------------------
  // A lane holds channels 8g + 4 * fhalf .. + 3 of pixel frow: stored from there, 32 lanes would write 16 bytes each into
  // 32 different rows.  The sums go through LDS instead (int32 [pixel][Co + 4], over the regions nobody reads any
  // more), and the block stores them with the channel quads of a pixel on consecutive lanes: whole rows at a time.
  __syncthreads();
  int *stg = reinterpret_cast<int *>(lds + p.off_x);
  const int sp = p.Co + 4;
  if (p3) {
    const int pix = ws * 32 + frow;
#pragma unroll
    for (int b = 0; b < MAXJ; ++b) {
      const int j = wj + p.nwj * b;
      if (j >= p.ncol) continue;
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<v4i *>(stg + pix * sp + j * 32 + 8 * g + 4 * fhalf) =
            v4i{acc3[b][4 * g], acc3[b][4 * g + 1], acc3[b][4 * g + 2], acc3[b][4 * g + 3]};
    }
  }
  __syncthreads();
  {
    const int64_t m0 = ((int64_t)img * p.Ho + ho0) * p.Wo;
    EpiLane L;
    L.use_rcp = e.chan_rcp != nullptr;
    L.use_div = e.chan_div != nullptr && e.chan_rcp == nullptr;
    L.use_bias = e.bias != nullptr;
    L.use_res = e.resid != nullptr;
    L.res_after = e.resid_after != 0;
    L.act = e.act;
    L.unit_q = e.q_scale == 1.0f;
    L.half_steps = e.half_steps != 0;
    const float *c3 = reinterpret_cast<const float *>(lds + p.off_c3);
    const int cq = p.Co >> 2;
    for (int i = tid; i < p_out * cq; i += NT) {
      const int pix = i / cq, n = (i - pix * cq) * 4;
      const v4i a = *reinterpret_cast<const v4i *>(stg + pix * sp + n);
      L.div = *reinterpret_cast<const v4f *>(c3 + n);
      L.rcp = *reinterpret_cast<const v4f *>(c3 + p.Co + n);
      L.bias = *reinterpret_cast<const v4f *>(c3 + 2 * p.Co + n);
      const int64_t idx = (m0 + pix) * p.Co + n;
      v4f res = {0.f, 0.f, 0.f, 0.f};
      if (L.use_res) res = load_stream(reinterpret_cast<const v4f *>(e.resid + idx), e.resid_stream != 0);
      epi_vec4<EpiGeneric>(a, res, L, idx, e);
    }
  }
}

// Tile choice; false: not this kernel's shape.  ks3: 32-channel tiles per chunk of hidden channels (4, 6 or 8).
static bool irb_plan(int N, int H, int W, int Cin, int hid, int Co, int S, int cus, IrbParams &p, int &maxj, int &ks3,
                     int &lds_bytes) {
  if (S != 1 && S != 2) return false;
  if (Cin % 32 != 0 || Cin > 32 * IRB_KS1MAX || hid % 32 != 0 || Co % 32 != 0 || Co <= 0 || Co > 64 * IRB_NW || hid < 128) return false;
  if (H < 2 || W < 2 || W > 128) return false;
  const int Ho = (H - 1) / S + 1, Wo = (W - 1) / S + 1;
  if ((int64_t)N * H * W * Cin >= (1ll << 31) || (int64_t)N * Ho * Wo * Co >= (1ll << 29) || (int64_t)Co * hid >= (1ll << 31) ||
      (int64_t)hid * Cin >= (1ll << 31))
    return false;
  const int ncol = Co / 32;
  int best = 0;
  IrbParams bp = {};
  int best_lds = 0, best_maxj = 0, best_ks3 = 0;
  int want = 0, want_ks3 = 0;  // tuning builds: a band height / chunk width to take if it is one of the candidates
  if (const char *t = tuning_env("CATCHQ_IRB_TR")) want = atoi(t);
  if (const char *t = tuning_env("CATCHQ_IRB_KS3")) want_ks3 = atoi(t);
  // candidates: the balanced band heights ceil(Ho / bands), from many short bands to one (the last band of an image
  // may be shorter than the others)
  for (int nb = Ho; nb >= 1; --nb) {
    const int tr = (Ho + nb - 1) / nb;
    if ((Ho + tr - 1) / tr != nb) continue;
    if (S == 1 && tr < 3 && tr != Ho) continue;  // halo rows recomputed: at most two thirds of the band again
    IrbParams q = {};
    q.N = N; q.H = H; q.W = W; q.Cin = Cin; q.hid = hid; q.Co = Co; q.Ho = Ho; q.Wo = Wo;
    q.TR = tr; q.bands = nb;
    q.PR = (tr - 1) * S + 3;
    q.HG = (tr + 1) / 2; q.WG = (Wo + 3) / 4;
    q.PRA = (S == 1) ? 2 * q.HG + 2 : 4 * q.HG + 1;
    q.PCA = (S == 1) ? 4 * q.WG + 2 : 8 * q.WG + 2;
    if (q.PRA < q.PR) q.PRA = q.PR;
    if (q.PCA < W + 2) q.PCA = W + 2;
    q.m_a = q.PR * W; q.nsa = (q.m_a + 31) / 32;
    q.p_out = tr * Wo; q.nso = (q.p_out + 31) / 32;
    if (q.nso > 8) continue;
    q.ks1 = Cin / 32;
    q.nws = 1;
    while (q.nws < q.nso) q.nws *= 2;
    q.nwj = IRB_NW / q.nws;
    q.ncol = ncol;
    const int mj = (ncol + q.nwj - 1) / q.nwj;
    if (mj > 3) continue;
    // hidden channels per chunk: the width that keeps most of the stencil's lanes busy (a lane takes a 2 x 4 group of
    // pixels of four channels; 512 lanes per round), wider on a tie; the projection's filters of a chunk wait in
    // registers, which bounds the width by the column tiles a wave owns
    int k_best = 0, lds_best = 0;
    int64_t num_best = 0, den_best = 1;
    for (int k3 : {4, 6, 8}) {
      if (mj * k3 > 16) continue;
      if (want_ks3 > 0 && k3 != want_ks3) continue;
      const int hc = 32 * k3, groups = q.HG * q.WG;
      int64_t work = 0, rounds = 0;
      for (int c0 = 0; c0 < hid; c0 += hc) {
        const int items = groups * ((hid - c0 < hc ? hid - c0 : hc) / 4);
        work += items;
        rounds += (items + 64 * IRB_NW - 1) / (64 * IRB_NW);
      }
      auto up = [](int v) { return (v + 255) / 256 * 256; };
      int lds = up(Co * 12) + up(q.m_a * (Cin + 16)) + up(hid * 12) + up(hid * 24) + up(q.PRA * q.PCA * (hc + 4)) +
                up(q.nso * 32 * (hc + 16));
      const int with_stage = up(Co * 12) + up(q.nso * 32 * (Co + 4) * 4);
      if (with_stage > lds) lds = with_stage;
      if (lds > 160 * 1024) continue;
      if (!k_best || work * den_best >= num_best * rounds) { k_best = k3; num_best = work; den_best = rounds; lds_best = lds; }
    }
    if (!k_best) continue;
    {
      const int hc = 32 * k_best;
      q.nch = (hid + hc - 1) / hc;
      q.xs = Cin + 16; q.hs = hc + 4; q.as = hc + 16;
      auto up = [](int v) { return (v + 255) / 256 * 256; };
      int off = up(Co * 12);  // off_c3 = 0
      q.off_x = off; off += up(q.m_a * q.xs);
      q.off_wp = off; off += up(hid * 12);
      q.off_cst = off; off += up(hid * 24);
      q.off_hp = off; off += up(q.PRA * q.PCA * q.hs);
      q.off_a3 = off; off += up(q.nso * 32 * q.as);
      if (off > lds_best) return false;
    }
    // the largest band that still gives every planned compute unit a block; otherwise the smallest that fits
    const int64_t blocks = (int64_t)N * q.bands;
    if (blocks > 0x7fffffff) continue;
    if (want > 0 ? (tr == want || !best) : (!best || blocks >= cus)) {
      best = tr; bp = q; best_lds = lds_best; best_maxj = mj; best_ks3 = k_best;
    }
  }
  if (!best) return false;
  p = bp; lds_bytes = best_lds; maxj = best_maxj; ks3 = best_ks3;
  return true;
}

bool irb_i8_ok(int N, int H, int W, int Cin, int hid, int Co, int S, int cus) {
  IrbParams p;
  int maxj, ks3, lds;
  return irb_plan(N, H, W, Cin, hid, Co, S, cus, p, maxj, ks3, lds);
}

template <int S, int MAXJ, int KS3>
static int irb_launch(const void *x, const IrbStageDev &s1, const IrbStageDev &s2, const void *w3, const IrbParams &p,
                      const EpiDev &e, int lds_bytes, hipStream_t s) {
  auto kern = irb_kernel<S, MAXJ, KS3>;
  if (lds_bytes > 64 * 1024) {
    static std::atomic<bool> raised[64];
    if (raise_lds_limit((const void *)kern, 160 * 1024, raised) != CATCHQ_OK) return CATCHQ_ERR_LAUNCH;
  }
  kern<<<p.N * p.bands, 64 * IRB_NW, lds_bytes, s>>>((const int8_t *)x, s1, s2, (const int8_t *)w3, p, e);
  return launch_status();
}

template <int S>
static int irb_launch_s(const void *x, const IrbStageDev &s1, const IrbStageDev &s2, const void *w3, const IrbParams &p,
                        const EpiDev &e, int maxj, int ks3, int lds_bytes, hipStream_t s) {
  switch (maxj * 10 + ks3) {
    case 14: return irb_launch<S, 1, 4>(x, s1, s2, w3, p, e, lds_bytes, s);
    case 16: return irb_launch<S, 1, 6>(x, s1, s2, w3, p, e, lds_bytes, s);
    case 18: return irb_launch<S, 1, 8>(x, s1, s2, w3, p, e, lds_bytes, s);
    case 24: return irb_launch<S, 2, 4>(x, s1, s2, w3, p, e, lds_bytes, s);
    case 26: return irb_launch<S, 2, 6>(x, s1, s2, w3, p, e, lds_bytes, s);
    case 28: return irb_launch<S, 2, 8>(x, s1, s2, w3, p, e, lds_bytes, s);
    case 34: return irb_launch<S, 3, 4>(x, s1, s2, w3, p, e, lds_bytes, s);
    default: return -1;
  }
}

// x [N, H, W, Cin] int8; w1 [hid][Cin]; wd [hid][3][3]; w3 [Co][hid]; the two inner stages requantize to int8 behind
// ReLU (relu6 = 0) or ReLU6; e is the projection's epilogue over [N, Ho, Wo, Co].  -1: not this kernel's shape.
int irb_i8(const void *x, int N, int H, int W, int Cin, int hid, int Co, int S, const IrbStageDev &s1, const IrbStageDev &s2,
           const void *w3, const EpiDev &e, hipStream_t s) {
  IrbParams p;
  int maxj, ks3, lds_bytes;
  if (!vec_epilogue_ok(Co, e)) return -1;
  if (!irb_plan(N, H, W, Cin, hid, Co, S, e.cus, p, maxj, ks3, lds_bytes)) return -1;
  return S == 1 ? irb_launch_s<1>(x, s1, s2, w3, p, e, maxj, ks3, lds_bytes, s)
                : irb_launch_s<2>(x, s1, s2, w3, p, e, maxj, ks3, lds_bytes, s);
}

}  // namespace catchq
