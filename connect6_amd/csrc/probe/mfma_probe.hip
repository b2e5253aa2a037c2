// Measurement aid for bench.py (not part of the drop-in library): the bf16 MFMA rate this GPU
// sustains when every CU runs back-to-back v_mfma_f32_32x32x16_bf16 with operands of random
// sign, exponent and mantissa, one wave per SIMD, and the shader clock it settles at.  The
// published peak assumes the top clock; under a dense matrix load the card's power management
// lowers it, and how far depends on the operand bits (all-zero operands barely lower it).
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int v4i __attribute__((ext_vector_type(4)));

namespace {

__device__ __forceinline__ unsigned mix(unsigned x) {
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}
// two bf16 values with random sign and mantissa and an exponent in [2^-7, 2^0]
__device__ __forceinline__ int random_pair(unsigned seed) {
  const unsigned r = mix(seed);
  const unsigned lo = (r & 0x807fu) | ((120u + ((r >> 8) & 7u)) << 7);
  const unsigned hi = ((r >> 16) & 0x807fu) | ((120u + ((r >> 28) & 7u)) << 7);
  return (int)(lo | (hi << 16));
}

constexpr int kPerIter = 12;

__global__ __launch_bounds__(256) void mfma_rate_kernel(float *sink, long long *stamps, int iters, int zero_operands) {
  const unsigned id = blockIdx.x * 256u + threadIdx.x;
  v4i a, b;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = zero_operands ? 0 : random_pair(8u * id + i);
    b[i] = zero_operands ? 0 : random_pair(8u * id + 4u + i);
  }
  f32x16 c[4] = {{0}, {0}, {0}, {0}};
  const long long t0 = clock64(), r0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < kPerIter; ++u)
      c[u & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                          __builtin_bit_cast(bf16x8, b), c[u & 3], 0, 0, 0);
  }
  const long long t1 = clock64(), r1 = wall_clock64();
  const f32x16 s = c[0] + c[1] + c[2] + c[3];
  sink[id] = s[0] + s[7];
  if (threadIdx.x == 0) {
    stamps[2 * blockIdx.x] = t1 - t0;      // shader clock cycles
    stamps[2 * blockIdx.x + 1] = r1 - r0;  // ticks of the constant 100 MHz counter
  }
}

}  // namespace

// Runs the loop on every CU and reports the rate over the whole launch (HIP events) and the mean
// shader clock inside it.  Returns 0, or a hipError_t value.
extern "C" int c6_probe_mfma_rate(int iters, int zero_operands, double *tflops, double *clock_ghz,
                                  double *cycles_per_mfma) {
  int dev = 0, cus = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return (int)e;
  float *sink = nullptr;
  long long *stamps = nullptr;
  e = hipMalloc(&sink, sizeof(float) * 256 * cus);
  if (e == hipSuccess) e = hipMalloc(&stamps, sizeof(long long) * 2 * cus);
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (e == hipSuccess) e = hipEventCreate(&e0);
  if (e == hipSuccess) e = hipEventCreate(&e1);
  float ms = 0.0f;
  if (e == hipSuccess) {
    hipLaunchKernelGGL(mfma_rate_kernel, dim3(cus), dim3(256), 0, 0, sink, stamps, iters / 8 + 1, zero_operands);  // warm-up
    hipEventRecord(e0, 0);
    hipLaunchKernelGGL(mfma_rate_kernel, dim3(cus), dim3(256), 0, 0, sink, stamps, iters, zero_operands);
    hipEventRecord(e1, 0);
    e = hipEventSynchronize(e1);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  }
  if (e == hipSuccess) {
    long long *h = new long long[2 * cus];
    e = hipMemcpy(h, stamps, sizeof(long long) * 2 * cus, hipMemcpyDeviceToHost);
    double cyc = 0.0, ticks = 0.0;
    for (int i = 0; i < cus; ++i) {
      cyc += (double)h[2 * i];
      ticks += (double)h[2 * i + 1];
    }
    delete[] h;
    const double mfmas = (double)iters * kPerIter;
    *tflops = 4.0 * cus * mfmas * 32768.0 / (ms * 1e-3) / 1e12;  // 4 waves per CU, 32x32x16x2 FLOP each
    *clock_ghz = ticks > 0.0 ? cyc / ticks * 0.1 : 0.0;
    *cycles_per_mfma = cyc / cus / mfmas;
  }
  if (e0) hipEventDestroy(e0);
  if (e1) hipEventDestroy(e1);
  if (sink) hipFree(sink);
  if (stamps) hipFree(stamps);
  return (int)e;
}
