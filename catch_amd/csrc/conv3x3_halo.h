// What the patch-resident 3x3 kernels (int8 and int16 activations) share: tile parameters, the patch swizzle and
// the host-side tile choice.
#pragma once
#include <type_traits>

#include "igemm_i8_dma.inc"

namespace catchq {

struct HaloParams {
  int N, H, W, Co;       // output [N, H, W, Co]
  int Hi, Wi;            // input [N, Hi, Wi, CI]
  int TR;                // output rows per tile
  int image_mode;        // 0: a band of TR rows of one image (the last band of an image may be shorter);
                         // 1: TR = G * H, G whole images
  int bands;             // bands per image (band mode)
  int PR, PC;            // patch rows / columns (stride 1: PC = W + 2)
  int img_rows;          // patch rows per image in image mode
  int P;                 // output pixels per tile = TR * W
  int nsub;              // 32-row sub-tiles per tile
  int tiles_n, nblocks;
  int64_t M;             // N * H * W
  unsigned x_bytes, w_bytes;
};

// f(integral_constant<int, G>) for G = 0 .. N-1, expanded at compile time (a #pragma unroll over this many large
// bodies is declined by the optimizer, and the fragment registers must never be indexed at run time)
template <int G, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (G < N) {
    f(std::integral_constant<int, G>{});
    static_for<G + 1, N>(f);
  }
}

// Swizzle of a pixel's 16-byte chunk index; CH = chunks per pixel.  The 32 lanes of an A fragment read the patch
// pixels of 32 consecutive OUTPUT pixels at one filter tap, and a ds_read_b128 is conflict-free when 16
// consecutive lanes fall into 16 different 16-byte slots of a 256-byte LDS line.  The key is therefore taken from
// h = (patch row / S) * Wo + (patch column / S): for a fixed tap h runs through consecutive integers with the
// output pixel index, across the ends of output rows as well (the patch pixel index itself jumps there).
template <int CH>
__device__ __forceinline__ unsigned halo_swz(unsigned h) {
  if constexpr (CH == 4) return (h >> 2) & 3u;
  else if constexpr (CH == 8) return (h >> 1) & 7u;
  else return h & 15u;
}
template <int S>
__device__ __forceinline__ unsigned halo_key(unsigned prow, unsigned pcol, unsigned wo_count) {
  constexpr int SH = S == 2 ? 1 : 0;
  return (prow >> SH) * wo_count + (pcol >> SH);
}

// Tile choice for a 3x3 layer over input [N, Hi, Wi, Ci] of elem_bytes-wide integers: fills hp, the column tiles per block (tn), the dynamic LDS
// size and the wave count; false: not this kernel's shape.  force_tn > 0 asks for that many column tiles (one block
// over all output channels) and for band mode; cus: the compute units the launch plans for.
inline bool halo_plan(int N, int Hi, int Wi, int Ci, int Co, int stride, HaloParams &hp, int &tn, int &lds_bytes, int &waves,
                      int force_tn = 0, int elem_bytes = 1, int cus = 256) {
  const int Cb = Ci * elem_bytes;  // bytes per input pixel
  if (Cb != 64 && Cb != 128 && Cb != 256 && Cb != 512) return false;
  if (stride != 1 && !(stride == 2 && Cb != 64)) return false;
  const int H = (Hi - 1) / stride + 1, W = (Wi - 1) / stride + 1;
  if (Co % 4 != 0 || Wi > 254 || (int64_t)N * Hi * Wi * Cb >= (1ll << 31) || (int64_t)Co * 9 * Ci >= (1ll << 31)) return false;
  if ((int64_t)N * Hi >= (1 << 24)) return false;
  hp = HaloParams{};
  hp.N = N; hp.H = H; hp.W = W; hp.Co = Co; hp.Hi = Hi; hp.Wi = Wi;
  hp.PC = (W - 1) * stride + 3;
  hp.img_rows = (H - 1) * stride + 3;
  hp.M = (int64_t)N * H * W;
  hp.x_bytes = (unsigned)((int64_t)N * Hi * Wi * Cb);
  hp.w_bytes = (unsigned)((int64_t)Co * 9 * Ci);
  constexpr int kLdsLimit = 160 * 1024, kMaxP = 256;
  const int kRing1 = 3 * 32 * 256 * (force_tn > 0 ? force_tn : 1);
  // Tile choice.  A tile of P pixels costs ceil(ceil(P / 32) / 4) rounds of MFMA work (four waves, one 32-row
  // sub-tile each per round) plus about half a round of patch loading and synchronisation; the patch must fit
  // beside the smaller weight ring.  Small images go whole, several per tile; larger ones are cut into bands of
  // rows of equal height, the last band of an image possibly shorter.  Twice the cost is compared, in integers.
  auto rounds2 = [](int pixels) { return 2 * (((pixels + 31) / 32 + 3) / 4) + 1; };
  int best = 0, lds = 0;
  tn = 2;
  int64_t tiles_m = 0;
  if (H * W <= kMaxP / 2 && force_tn == 0) {
    int g_max = kMaxP / (H * W);
    if (const char *t = tuning_env("CATCHQ_HALO_G")) g_max = atoi(t) < g_max ? atoi(t) : g_max;
    int64_t best_cost = 0;  // cost of `best_g` images' worth of work, cross-multiplied
    int best_g = 0;
    for (int g = g_max; g >= 1; --g) {
      const int patch = (g * hp.img_rows * hp.PC * Cb + 1023) / 1024 * 1024;
      if (patch + kRing1 > kLdsLimit) continue;
      const int64_t cost = rounds2(g * H * W);  // per g images
      if (!best_g || cost * best_g < best_cost * g) { best_g = g; best_cost = cost; lds = patch; }
    }
    if (!best_g) return false;
    best = best_g * H;
    hp.image_mode = 1;
    hp.PR = best_g * hp.img_rows;
    hp.bands = 1;
    tiles_m = ((int64_t)N + best_g - 1) / best_g;
  } else {
    // candidates: the balanced band heights ceil(H / bands), so that no tile is longer than it has to be
    int tr_max = H;
    if (const char *t = tuning_env("CATCHQ_HALO_TR")) tr_max = atoi(t) < tr_max ? atoi(t) : tr_max;
    int64_t best_cost = 0;
    for (int bands = 1; bands <= H; ++bands) {
      const int tr = (H + bands - 1) / bands;
      if (tr > tr_max || tr * W > kMaxP || (H + tr - 1) / tr != bands) continue;
      const int patch = (((tr - 1) * stride + 3) * hp.PC * Cb + 1023) / 1024 * 1024;
      if (patch + kRing1 > kLdsLimit) continue;
      const int64_t cost = (int64_t)bands * rounds2(tr * W);
      if (!best || cost < best_cost) { best = tr; best_cost = cost; lds = patch; hp.bands = bands; }
    }
    if (!best) return false;
    hp.image_mode = 0;
    hp.PR = (best - 1) * stride + 3;
    tiles_m = (int64_t)N * hp.bands;
  }
  hp.TR = best;
  hp.P = best * W;
  hp.nsub = (hp.P + 31) / 32;
  if (hp.nsub > 8) return false;
  // tiles that leave waves of the block without a sub-tile are the implicit-GEMM kernel's case
  if (hp.nsub < 3) return false;
  if (force_tn > 0) {
    tn = force_tn;
  } else {
    // 64 channels per block while that still gives every compute unit the launch plans for a block and the ring fits
    // (a launch that shares the device with another one plans for its share: measured on ResNet-50 as two parts,
    // 64-channel blocks in stages 3 and 4 are worth +0.5 % end to end)
    int64_t min_blocks = cus;
    if (const char *t = tuning_env("CATCHQ_HALO_MINBLK")) min_blocks = atoi(t);
    if (lds + 3 * 64 * 256 > kLdsLimit || tiles_m * ((Co + 63) / 64) < min_blocks) tn = 1;
    if (const char *t = tuning_env("CATCHQ_HALO_TN")) tn = atoi(t);
    if (lds + 3 * 32 * tn * 256 > kLdsLimit) tn = 1;
  }
  hp.tiles_n = (Co + 32 * tn - 1) / (32 * tn);
  const int64_t nb = tiles_m * hp.tiles_n;
  if (nb > 0x7fffffff) return false;
  // a stride-2 patch is four times its output and leaves room for one block per compute unit: past one round
  // of blocks the implicit-GEMM kernel is faster (measured on the ResNet-50 downsampling layers at 32 and 64 images)
  if (stride == 2 && nb > 256) return false;
  hp.nblocks = (int)nb;
  lds_bytes = lds + 3 * 32 * tn * 256;
  waves = 4;
  // (64-channel layers: K is 18 steps of 32 bytes, too short for a second wave per SIMD to repay its own set-up;
  // measured on ResNet-50's first stage, four waves end to end +0.9 %)
  if (hp.nsub > 4 && Cb >= 128) waves = 8;
  if (const char *t = tuning_env("CATCHQ_HALO_WAVES")) waves = (atoi(t) == 8 && hp.nsub > 4) ? 8 : 4;
  const int epi_bytes = lds + 4 * 32 * (32 * tn + 8) * 4;  // the epilogue's staging area lies where the ring was
  if (epi_bytes > lds_bytes) lds_bytes = epi_bytes;
  return lds_bytes <= kLdsLimit;
}

}  // namespace catchq
