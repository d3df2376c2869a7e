// Measurement aid: the rate at which this GPU retires v_mfma_f32_32x32x16_f16 when nothing else is in the
// way.  Every CU runs one workgroup of 8 waves (two per SIMD, the occupancy of the attention kernels); each
// wave issues back-to-back MFMAs on four independent accumulators from registers only -- no LDS, no memory,
// no other vector work.  The attention kernels cannot beat this figure, so it is the yardstick their
// roofline fraction is read against: with operands that differ from lane to lane it lies well below the
// nominal peak (the clock follows the power the operands' toggling draws), with identical operands in
// every lane close to it.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/acct_fa.h"

// Shader-clock and wall-clock (100 MHz) ticks that wave 0 of workgroup 0 spent in the MFMA loop of the last launch:
// their ratio is the shader clock while the matrix pipe runs flat out.
__device__ unsigned long long acct_probe_ticks[2];

// Target of a store that practically never executes (referenced from device code only).  External linkage: the
// compiler must not conclude that nobody reads it and drop the loop that feeds the store.
__device__ float acct_probe_sink[512];

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kItersPerLaunch = 1500, kMfmaPerIter = 16;

template <bool VARYING>
__global__ void __launch_bounds__(512) mfma_rate_kernel(int iters) {
  const int lane = threadIdx.x & 63;
  f16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    // VARYING: a hash of (lane, element) supplies sign and mantissa bits, magnitudes in [1/4, 4) -- every operand
    // bit toggles from lane to lane as with real data; otherwise one value everywhere
    uint32_t h = (uint32_t)(lane * 8 + e + 1) * 2654435761u;
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
    const uint16_t ba = VARYING ? (uint16_t)((h & 0x83ffu) | ((13u + ((h >> 10) & 3u)) << 10)) : (uint16_t)0x3400u;        // 0x3400 = 0.25
    const uint16_t bb = VARYING ? (uint16_t)(((h >> 16) & 0x83ffu) | ((13u + ((h >> 26) & 3u)) << 10)) : (uint16_t)0x3400u;
    a[e] = __builtin_bit_cast(_Float16, ba);
    b[e] = __builtin_bit_cast(_Float16, bb);
  }
  f32x16 c[4];
#pragma unroll
  for (int n = 0; n < 4; n++)
#pragma unroll
    for (int r = 0; r < 16; r++) c[n][r] = 0.f;
  const bool timed = blockIdx.x == 0 && threadIdx.x < 64;                  // wave-uniform
  unsigned long long t0 = 0, r0 = 0;
  if (timed) { t0 = __builtin_amdgcn_s_memtime(); r0 = __builtin_amdgcn_s_memrealtime(); }
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int n = 0; n < kMfmaPerIter; n++) c[n & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c[n & 3], 0, 0, 0);
  }
  float r = 0.f;
#pragma unroll
  for (int n = 0; n < 4; n++)
#pragma unroll
    for (int e = 0; e < 16; e++) r += c[n][e];                // (waits for the last MFMA)
  if (r == 123.456f) acct_probe_sink[threadIdx.x] = r;        // practically never true: keeps the loop alive without a store
  if (timed) {
    const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    if (lane == 0) { acct_probe_ticks[0] = t1 - t0; acct_probe_ticks[1] = r1 - r0; }
  }
}

}  // namespace

static int probe_mfma(int varying_operands, double* tflops, double* shader_ghz, void* stream) {
  if (!tflops) return ACCT_E_NULLPTR;
  *tflops = 0.0;
  if (shader_ghz) *shader_ghz = 0.0;
  int dev = 0, n_cu = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n_cu <= 0)
    return ACCT_E_LAUNCH;
  hipStream_t st = (hipStream_t)stream;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
    if (e0) (void)hipEventDestroy(e0);
    return ACCT_E_LAUNCH;
  }
  auto launch = [&]() {
    if (varying_operands) hipLaunchKernelGGL(mfma_rate_kernel<true>, dim3(n_cu), dim3(512), 0, st, kItersPerLaunch);
    else hipLaunchKernelGGL(mfma_rate_kernel<false>, dim3(n_cu), dim3(512), 0, st, kItersPerLaunch);
  };
  constexpr int kWarm = 40, kTimed = 10;              // ~60 ms of warm-up: the clock has settled under matrix load
  for (int i = 0; i < kWarm; i++) launch();
  hipError_t e = hipEventRecord(e0, st);
  for (int i = 0; i < kTimed; i++) launch();
  if (e == hipSuccess) e = hipEventRecord(e1, st);
  if (e == hipSuccess) e = hipEventSynchronize(e1);
  if (e == hipSuccess) e = hipGetLastError();
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (e != hipSuccess || !(ms > 0.f)) return ACCT_E_LAUNCH;
  const double flop = (double)kTimed * n_cu * 8.0 * kItersPerLaunch * kMfmaPerIter * (2.0 * 32 * 32 * 16);
  *tflops = flop / (ms * 1e-3) / 1e12;
  if (shader_ghz) {
    unsigned long long ticks[2] = {0, 0};
    if (hipMemcpyFromSymbol(ticks, HIP_SYMBOL(acct_probe_ticks), sizeof(ticks)) != hipSuccess || ticks[1] == 0) return ACCT_E_LAUNCH;
    *shader_ghz = (double)ticks[0] / ((double)ticks[1] * 10.0);            // the wall clock ticks every 10 ns
  }
  return ACCT_OK;
}

extern "C" int acct_probe_mfma_rate(int varying_operands, double* tflops, void* stream) {
  return probe_mfma(varying_operands, tflops, nullptr, stream);
}

extern "C" int acct_probe_mfma_clock(int varying_operands, double* tflops, double* shader_ghz, void* stream) {
  if (!shader_ghz) return ACCT_E_NULLPTR;
  return probe_mfma(varying_operands, tflops, shader_ghz, stream);
}
