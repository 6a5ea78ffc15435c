// Matrix-core ceiling probe (see mfma_ceiling.h): a measurement aid in a
// library of its own, outside the runtime's C-ABI.
//
// Four independent accumulators per wave, MFMAs back to back, operands that
// never leave their registers: the rate at which the matrix cores run when
// nothing feeds them.  RANDOM: operand bytes from a per-lane generator, two
// sets in alternation, so that the inputs toggle as a model's do; otherwise
// ones and zeros.  The accumulators are folded into a value that is stored
// only if it has one particular value, which keeps the loop alive.
#include <hip/hip_runtime.h>

#include "mfma_ceiling.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

namespace {
template <bool RANDOM>
__global__ __launch_bounds__(256) void k_mfma_probe(int iters,
    int *__restrict__ sink) {
  unsigned seed = threadIdx.x * 7919u + blockIdx.x * 104729u + 1u;
  auto next = [&]() {
    seed = seed * 1664525u + 1013904223u;
    return (int)(seed ^ (seed >> 15));
  };
  v4i a0 = {1, 1, 1, 1}, b0 = {1, 0, 1, 0}, a1 = a0, b1 = b0;
  if (RANDOM) {
    a0 = (v4i){next(), next(), next(), next()};
    b0 = (v4i){next(), next(), next(), next()};
    a1 = (v4i){next(), next(), next(), next()};
    b1 = (v4i){next(), next(), next(), next()};
  }
  asm volatile("" : "+v"(a0), "+v"(b0), "+v"(a1), "+v"(b1));
  v16i acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      acc[i][r] = 0;
  for (int it = 0; it < iters; ++it) {
    acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b0, acc[0], 0, 0, 0);
    acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b1, acc[1], 0, 0, 0);
    acc[2] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, b0, acc[2], 0, 0, 0);
    acc[3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, b1, acc[3], 0, 0, 0);
  }
  int fold = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      fold += acc[i][r];
  if (fold == 0x7fffffff)
    sink[0] = fold;
}
} // namespace


extern "C" int om_mi355x_measure_mfma_ceiling(int64_t random_operands,
    double *tops, double *clock_ghz) {
  if (!tops || !clock_ghz)
    return (int)hipErrorInvalidValue;
  hipDeviceProp_t prop;
  hipError_t e = hipSetDevice(0);
  if (e == hipSuccess)
    e = hipGetDeviceProperties(&prop, 0);
  if (e != hipSuccess)
    return (int)e;
  // Two blocks of four waves per CU (two waves per SIMD), 4 * kIters MFMAs
  // per wave: 5 to 15 ms, long enough for the clock to settle.  The first
  // launch brings the device to that state, the second is the one timed.
  const int kIters = 50000;
  const int blocks = 2 * prop.multiProcessorCount;
  int *sink = nullptr;
  hipStream_t st = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  float ms = 0.0f;
  e = hipMalloc((void **)&sink, 16);
  if (e == hipSuccess)
    e = hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
  if (e == hipSuccess)
    e = hipEventCreate(&e0);
  if (e == hipSuccess)
    e = hipEventCreate(&e1);
  auto launch = [&]() {
    if (random_operands)
      k_mfma_probe<true><<<(unsigned)blocks, 256, 0, st>>>(kIters, sink);
    else
      k_mfma_probe<false><<<(unsigned)blocks, 256, 0, st>>>(kIters, sink);
    return hipGetLastError();
  };
  if (e == hipSuccess)
    e = launch();
  if (e == hipSuccess)
    e = hipEventRecord(e0, st);
  if (e == hipSuccess)
    e = launch();
  if (e == hipSuccess)
    e = hipEventRecord(e1, st);
  if (e == hipSuccess)
    e = hipEventSynchronize(e1);
  if (e == hipSuccess)
    e = hipEventElapsedTime(&ms, e0, e1);
  if (e0)
    (void)hipEventDestroy(e0);
  if (e1)
    (void)hipEventDestroy(e1);
  if (st)
    (void)hipStreamDestroy(st);
  if (sink)
    (void)hipFree(sink);
  if (e != hipSuccess)
    return (int)e;
  if (ms <= 0.0f)
    return (int)hipErrorUnknown;
  // 4 waves a block, 4 * kIters MFMAs a wave, 32 * 32 * 32 multiply-adds each
  const double ops = (double)blocks * 4.0 * 4.0 * kIters * 32768.0 * 2.0;
  *tops = ops / ((double)ms * 1e-3) / 1e12;
  // A SIMD issues one of these MFMAs every 32 clocks when nothing holds it
  // up, which is the case here: the clock that this rate corresponds to.
  const double per_simd = (double)blocks * 4.0 * 4.0 * kIters /
                          ((double)prop.multiProcessorCount * 4.0);
  *clock_ghz = per_simd * 32.0 / ((double)ms * 1e6);
  return 0;
}
