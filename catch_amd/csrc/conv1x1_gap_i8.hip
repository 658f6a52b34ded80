// The last 1x1 convolution of an image classifier and the global average pooling behind it in one launch.
//
// Run layer by layer the convolution writes its fp32 output (ResNet-50: 7 x 7 x 2048 floats per image, the largest
// tensor of the last stage) and the pooling reads it back to keep one value per channel -- two launches whose time
// is their start-up and the round trip of that tensor.  Here a block owns one image and 32 channels per wave:
//
//   1  the block's filter rows and the image's pixels (at most 64, int8) travel from global memory straight into
//      LDS (buffer_load ... lds, 16 bytes per lane, whole cache lines per instruction), K in chunks of at most 512
//      bytes; a row's 16-byte pieces are stored XOR-swizzled so that the fragment reads of 16 rows fall into 16
//      different pieces of an LDS line.  (Filter fragments fetched by the lanes themselves, 16 bytes per lane at a
//      stride of K bytes, cost one cache-line request per lane and made this kernel twice as slow.)
//   2  every wave multiplies on the matrix cores with the operands swapped (filters as A, pixels as B), so that a
//      lane ends up with four consecutive channels of one pixel; the integer sums go to the wave's tile in LDS;
//   3  the lanes take the tile row-wise -- eight lanes a pixel, four channels each, so that the fp32 residual is read
//      in whole cache lines -- and apply the convolution's epilogue (reciprocal-form division, bias, residual,
//      activation): the arithmetic of the stand-alone launch, value for value;
//   4  one lane per channel adds the pixels up in storage order, one fp32 addition each, divides once by the pixel
//      count and stores the mean and / or its quantized form -- the arithmetic of the stand-alone pooling kernel.
//
// The convolution's output never reaches memory; mean and quantized mean are those of the two launches bit for bit.
#include "igemm_i8_dma.inc"

namespace catchq {

struct GapConvDev {
  const float *div, *rcp, *bias, *resid;
  int exp2, act;
  float *mean;  // [N, Co] or null
  void *q;      // [N, Co] int8 / int16 or null
  int q_bw, q_neg_pos;
  float q_scale;
};

struct GapConvParams {
  int N, HW, K, Co;
  int KC;      // bytes of K per pass through LDS: a divisor of K, a multiple of 32, at most 512
  int sw;      // swizzle mask: (largest power of two that divides KC / 16, at most 16) - 1
  int groups;  // 32-pixel groups: 1 or 2
  int off_x;   // LDS offset of the pixels (behind the filter rows)
};

constexpr int GC_YP = 36;  // dwords per pixel row of a wave's output tile

template <int NW, bool RES>
__global__ __launch_bounds__(64 * NW) void conv1x1_gap_kernel(const int8_t *__restrict__ X, const int8_t *__restrict__ Wt,
                                                             GapConvDev e, GapConvParams p) {
  extern __shared__ __attribute__((aligned(1024))) int8_t lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int frow = lane & 31, fhalf = lane >> 5;
  const int img = blockIdx.x;
  const int cb = blockIdx.y * NW * 32;   // the block's first channel
  const int c_own = cb + wave * 32;      // this wave's
  const bool live = c_own < p.Co;        // wave-uniform; rows past the last channel are zero-filled by the loads
  const int chw = p.KC >> 4;             // 16-byte pieces per row of a pass
  const int w_rows = NW * 32;

  // epilogue operands in the row-wise layout: lane -> (pixel lane / 8 + 8 j, channels c_own + 4 (lane % 8) .. + 3)
  const int cc = lane & 7, pp = lane >> 3;
  const int ch_e = (live ? c_own : 0) + 4 * cc;
  v4f dv = *reinterpret_cast<const v4f *>(e.div + ch_e), rc = *reinterpret_cast<const v4f *>(e.rcp + ch_e);
  const v4f bs = *reinterpret_cast<const v4f *>(e.bias + ch_e);
  v4f res[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    res[j] = v4f{0.f, 0.f, 0.f, 0.f};
    const int px = pp + 8 * j < p.HW ? pp + 8 * j : p.HW - 1;  // rows past the image repeat its last pixel
    if constexpr (RES) res[j] = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(e.resid + ((int64_t)img * p.HW + px) * p.Co + ch_e));
  }

  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc((void *)(Wt + (int64_t)cb * p.K), 0, (int)((int64_t)(p.Co - cb) * p.K < (1 << 30) ? (int64_t)(p.Co - cb) * p.K : (1 << 30)), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_x =
      __builtin_amdgcn_make_buffer_rsrc((void *)(X + (int64_t)img * p.HW * p.K), 0, p.HW * p.K, 0x00020000);
  const int w_instr = w_rows * chw / 64;            // DMA instructions of a pass: filter rows ...
  const int x_instr = (p.HW * chw + 63) / 64;       // ... and pixels
  const int8_t *arow = lds + (wave * 32 + frow) * p.KC;
  const int a_key = frow & p.sw;
  const int8_t *xrow[2];
  int x_key[2];
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const int px = g * 32 + frow < p.HW ? g * 32 + frow : p.HW - 1;  // lanes past the image repeat its last pixel
    xrow[g] = lds + p.off_x + px * p.KC;
    x_key[g] = px & p.sw;
  }
  v16i acc[2];
#pragma unroll
  for (int g = 0; g < 2; ++g)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[g][r] = 0;

  for (int k0 = 0; k0 < p.K; k0 += p.KC) {
    if (k0 > 0) __syncthreads();  // the previous pass has been read
    // ---- 1: this pass of the filter rows and the pixels, straight into LDS ---------------------------------------------
    for (int b = wave; b < w_instr + x_instr; b += NW) {  // wave-uniform
      const bool is_w = b < w_instr;
      const int g = (is_w ? b : b - w_instr) * 64 + lane;  // piece index within the slab = LDS position
      const int row = g / chw, slot = g - row * chw;
      const int piece = slot ^ (row & p.sw);               // the swizzle is applied on the source side
      const int rows = is_w ? w_rows : p.HW;
      const unsigned voff = row < rows ? (unsigned)(row * p.K + k0 + piece * 16) : 0x80000000u;  // out of range: zeros
      lds_ptr_t dst = (lds_ptr_t)(lds + (is_w ? 0 : p.off_x) + (is_w ? b : b - w_instr) * 1024);
      if (is_w) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, dst, 16, (int)voff, 0, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, dst, 16, (int)voff, 0, 0, 0);
    }
    CATCHQ_VMCNT(0);  // this wave's transfers have landed; the barrier makes that true of every wave's
    __syncthreads();
    // ---- 2: the convolution over this pass -----------------------------------------------------------------------------
    const int steps = p.KC >> 5;
    v4i fa = *reinterpret_cast<const v4i *>(arow + ((fhalf ^ a_key) << 4));
    v4i fb0 = *reinterpret_cast<const v4i *>(xrow[0] + ((fhalf ^ x_key[0]) << 4));
    v4i fb1 = *reinterpret_cast<const v4i *>(xrow[1] + ((fhalf ^ x_key[1]) << 4));
    for (int s = 0; s < steps; ++s) {
      const v4i a = fa, b0 = fb0, b1 = fb1;
      const int cn = (s + 1 < steps ? s + 1 : s) * 2 + fhalf;  // fragments one step ahead of the matrix instructions
      fa = *reinterpret_cast<const v4i *>(arow + ((cn ^ a_key) << 4));
      fb0 = *reinterpret_cast<const v4i *>(xrow[0] + ((cn ^ x_key[0]) << 4));
      fb1 = *reinterpret_cast<const v4i *>(xrow[1] + ((cn ^ x_key[1]) << 4));
      acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b0, acc[0], 0, 0, 0);
      if (p.groups > 1) acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b1, acc[1], 0, 0, 0);
    }
  }
  __syncthreads();  // every wave is done with the operands: the output tiles overlay them

  // ---- 3: the sums into the wave's tile, the epilogue row-wise -----------------------------------------------------------
  int *yt = reinterpret_cast<int *>(lds) + wave * (p.HW * GC_YP);
#pragma unroll
  for (int g = 0; g < 2; ++g) {
    const int px = g * 32 + frow;
    if (g < p.groups && px < p.HW) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<v4i *>(yt + px * GC_YP + 8 * i + 4 * fhalf) =
            v4i{acc[g][4 * i], acc[g][4 * i + 1], acc[g][4 * i + 2], acc[g][4 * i + 3]};
    }
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {  // the power of two folded into the reciprocal form
    dv[j] = __builtin_ldexpf(dv[j], -e.exp2);
    rc[j] = __builtin_ldexpf(rc[j], e.exp2);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int px = pp + 8 * j;
    if (px < p.HW) {
      int *cell = yt + px * GC_YP + 4 * cc;
      const v4i a = *reinterpret_cast<const v4i *>(cell);
      v4f y;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        float v = div_by_rcp((float)a[t], dv[t], rc[t]) + bs[t];
        if constexpr (RES) v = v + res[j][t];
        if (e.act >= CATCHQ_ACT_RELU) v = (v > 0.0f) ? v : 0.0f;
        if (e.act == CATCHQ_ACT_RELU6) v = (v < 6.0f) ? v : 6.0f;
        y[t] = v;
      }
      *reinterpret_cast<v4f *>(cell) = y;
    }
  }
  __syncthreads();
  // ---- 4: the ordered sum over the pixels ----------------------------------------------------------------------------------
  if (live && lane < 32) {
    const float *yf = reinterpret_cast<const float *>(yt);
    // in storage order, one addition per pixel: the order is part of the result; eight reads are requested at a time
    float s = 0.0f;
    int px = 0;
    for (; px + 8 <= p.HW; px += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = yf[(px + u) * GC_YP + lane];
#pragma unroll
      for (int u = 0; u < 8; ++u) s = s + v[u];
    }
    for (; px < p.HW; ++px) s = s + yf[px * GC_YP + lane];
    const float mean = s / (float)p.HW;
    const int64_t idx = (int64_t)img * p.Co + c_own + lane;
    if (e.mean) e.mean[idx] = mean;
    if (e.q) {
      if (e.q_bw == 8) reinterpret_cast<int8_t *>(e.q)[idx] = (int8_t)quant1<8>(mean, e.q_scale, e.q_neg_pos);
      else reinterpret_cast<int16_t *>(e.q)[idx] = (int16_t)quant1<16>(mean, e.q_scale, e.q_neg_pos);
    }
  }
}

// waves per block, bytes of K per pass and LDS bytes; false: not this kernel's shape (images of at most 64 pixels, K a
// multiple of 32, Co a multiple of 32)
static bool gap_plan(int N, int HW, int K, int Co, int &nw, GapConvParams &p, int &lds_bytes) {
  if (!(N > 0 && HW >= 1 && HW <= 64 && K >= 32 && K % 32 == 0 && K <= 8192 && Co >= 32 && Co % 32 == 0 &&
        (int64_t)N * HW * K < (1ll << 31) && (int64_t)N * HW * Co < (1ll << 31) && (int64_t)Co * K < (1ll << 30)))
    return false;
  // eight waves (256 channels) per block, four where that leaves compute units without a block
  nw = ((int64_t)N * ((Co + 255) / 256) >= 256) ? 8 : 4;
  p = GapConvParams{};
  p.N = N; p.HW = HW; p.K = K; p.Co = Co;
  // K in passes of at most 512 bytes; of at most 256 where the launch has more blocks than the device has compute
  // units, so that two blocks share a unit and one's transfers run under the other's arithmetic (measured at 64 images,
  // 512 -> 2048 channels: 20.2 -> 16.2 us; 320 -> 1280: 16.4 -> 11.9 us; with one block per unit the second pass costs
  // 0.2 us instead)
  const int dmax = ((int64_t)N * ((Co + 32 * nw - 1) / (32 * nw)) > 256) ? 8 : 16;
  for (int d = dmax; d >= 1; --d)
    if ((K / 32) % d == 0) { p.KC = 32 * d; break; }
  int sw = 1;
  while (sw < 16 && (p.KC / 16) % (2 * sw) == 0) sw *= 2;
  p.sw = sw - 1;
  p.groups = (HW + 31) / 32;
  p.off_x = nw * 32 * p.KC;
  const int x_bytes = (HW * (p.KC / 16) + 63) / 64 * 1024;  // whole DMA instructions
  const int operands = p.off_x + x_bytes, tiles = nw * HW * GC_YP * 4;
  lds_bytes = ((operands > tiles ? operands : tiles) + 255) / 256 * 256;
  return lds_bytes <= 160 * 1024;
}

bool conv1x1_gap_i8_ok(int N, int HW, int K, int Co) {
  int nw, lds;
  GapConvParams p;
  return gap_plan(N, HW, K, Co, nw, p, lds);
}

// x [N, HW, K] int8, w [Co, K] int8; mean / q [N, Co].  -1: not this kernel's shape.
int conv1x1_gap_i8(const void *x, const void *w, int N, int HW, int K, int Co, const GapConvDev &e, hipStream_t st) {
  int nw, lds_bytes;
  GapConvParams p;
  if (!gap_plan(N, HW, K, Co, nw, p, lds_bytes)) return -1;
  auto launch = [&](auto kern) {
    if (lds_bytes > 64 * 1024) {
      static std::atomic<bool> raised[64];
      if (raise_lds_limit((const void *)kern, 160 * 1024, raised) != CATCHQ_OK) return (int)CATCHQ_ERR_LAUNCH;
    }
    kern<<<dim3(N, (Co + 32 * nw - 1) / (32 * nw)), 64 * nw, lds_bytes, st>>>((const int8_t *)x, (const int8_t *)w, e, p);
    return launch_status();
  };
  if (e.resid) return nw == 8 ? launch(conv1x1_gap_kernel<8, true>) : launch(conv1x1_gap_kernel<4, true>);
  return nw == 8 ? launch(conv1x1_gap_kernel<8, false>) : launch(conv1x1_gap_kernel<4, false>);
}

}  // namespace catchq
