// LDS-DMA pipelined int8 GEMM: instantiations for plain row-major A (linear layers).
#include "igemm_i8_dma.inc"

namespace catchq {

int igemm_dma_launch_gemm(const void *a, const void *b, const IgemmParams &p, const EpiDev &e, int64_t a_bytes,
                          int64_t b_bytes, hipStream_t s) {
  return pick_dma_tile<LOAD_GEMM>(a, b, p, e, a_bytes, b_bytes, s);
}

}  // namespace catchq
