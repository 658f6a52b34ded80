// LDS-DMA pipelined int8 implicit-GEMM convolution (Ci % 16 == 0) and the entry point that routes
// between the two loaders.
#include "igemm_i8_dma.inc"

namespace catchq {

int igemm_dma_launch_gemm(const void *a, const void *b, const IgemmParams &p, const EpiDev &e, int64_t a_bytes,
                          int64_t b_bytes, hipStream_t s);

int igemm_dma_launch(int load, const void *a, const void *b, IgemmParams p, const EpiDev &e, int64_t a_bytes,
                     int64_t b_bytes, hipStream_t s) {
  // buffer offsets are 32-bit and 0x80000000 must stay out of range
  if (a_bytes >= (1ll << 31) || b_bytes >= (1ll << 31) || a_bytes <= 0 || b_bytes <= 0) return -1;
  if (load == LOAD_GEMM) return igemm_dma_launch_gemm(a, b, p, e, a_bytes, b_bytes, s);
  if (load == LOAD_CONV) {
    if (p.M >= (1ll << 31)) return -1;  // the loader splits a pixel index with 32-bit divisions
    return pick_dma_tile<LOAD_CONV>(a, b, p, e, a_bytes, b_bytes, s);
  }
  return -1;
}

}  // namespace catchq
