// Measurement aid (not part of the library): the rate the int8 matrix cores sustain on this device when nothing
// else limits them -- a register-resident loop of v_mfma_i32_32x32x32_i8 with four independent accumulators per
// wave, eight waves per compute unit -- for operands of three kinds: all zero, uniformly random bytes, and
// bytes drawn from a clipped normal distribution (sigma 32, what quantized N(0,1) data looks like).  The rate
// depends on the operands: the device lowers its clock under high-toggle matrix work.
// Build:  hipcc --offload-arch=gfx950 -O3 -o probe_mfma probe_mfma.hip      Run:  ./probe_mfma [seconds per case]
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

#define CHECK(x)                                                                  \
  do {                                                                            \
    hipError_t err_ = (x);                                                        \
    if (err_ != hipSuccess) {                                                     \
      fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(err_));            \
      return 1;                                                                   \
    }                                                                             \
  } while (0)

__global__ __launch_bounds__(256) void mfma_loop(const v4i *__restrict__ operands, int iters, int *sink) {
  // eight operand fragments per lane, read once
  v4i a[4], b[4];
  const int lane = blockIdx.x * 256 + threadIdx.x;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operands[(lane * 8 + i) & 0xffff];
    b[i] = operands[(lane * 8 + 4 + i) & 0xffff];
  }
  v16i c[4] = {};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i) c[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[(i + it) & 3], c[i], 0, 0, 0);
  }
  int r = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) r += c[i][j];
  if (r == 0x7f123456) sink[0] = r;  // keeps the loop alive
}

int main(int argc, char **argv) {
  const double seconds = argc > 1 ? atof(argv[1]) : 1.0;
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int cus = prop.multiProcessorCount;
  printf("device %s, %d compute units, clock %d MHz\n", prop.name, cus, prop.clockRate / 1000);
  const int blocks = cus * 2;  // two blocks of four waves per compute unit: two waves per SIMD
  std::vector<int> host(65536 * 4);
  v4i *dev;
  int *sink;
  CHECK(hipMalloc(&dev, host.size() * 4));
  CHECK(hipMalloc(&sink, 4));
  const char *names[3] = {"zero operands", "uniform random bytes", "normal bytes, sigma 32"};
  for (int kind = 0; kind < 3; ++kind) {
    srand(1234);
    for (size_t i = 0; i < host.size(); ++i) {
      unsigned w = 0;
      for (int byte = 0; byte < 4; ++byte) {
        int v = 0;
        if (kind == 1) v = (rand() & 255) - 128;
        if (kind == 2) {
          const double u1 = (rand() + 1.0) / (RAND_MAX + 2.0), u2 = (rand() + 1.0) / (RAND_MAX + 2.0);
          v = (int)lrint(32.0 * sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2));
          v = v < -128 ? -128 : (v > 127 ? 127 : v);
        }
        w |= (unsigned)(v & 255) << (8 * byte);
      }
      host[i] = (int)w;
    }
    CHECK(hipMemcpy(dev, host.data(), host.size() * 4, hipMemcpyHostToDevice));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    int iters = 20000;
    mfma_loop<<<blocks, 256>>>(dev, 1000, sink);
    CHECK(hipDeviceSynchronize());
    double total_ms = 0, total_ops = 0;
    while (total_ms < seconds * 1e3) {
      CHECK(hipEventRecord(e0));
      mfma_loop<<<blocks, 256>>>(dev, iters, sink);
      CHECK(hipEventRecord(e1));
      CHECK(hipEventSynchronize(e1));
      float ms;
      CHECK(hipEventElapsedTime(&ms, e0, e1));
      total_ms += ms;
      total_ops += (double)blocks * 4 * iters * 4 * 65536.0;  // waves x iterations x MFMAs x 2*32*32*32
    }
    const double pops = total_ops / (total_ms * 1e-3) / 1e15;
    printf("%-24s %.3f POP/s  (%.0f int8 operations per clock and compute unit at the nominal clock)\n", names[kind], pops,
           pops * 1e15 / cus / (prop.clockRate * 1e3));
    fflush(stdout);
  }
  return 0;
}
