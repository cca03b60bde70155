// Measures the vector issue rate this GPU sustains right now: chains of independent v_add_f32 (or v_fma_f64) on every
// SIMD, eight wavefronts each, for a given time. bench.py prints it beside the published peak, which is quoted at the
// nominal clock; under load the chip runs below it, box by box. Not part of the compiler's C-ABI: a library of its own.
#include <hip/hip_runtime.h>

namespace {

constexpr int CHAINS = 16, UNROLL = 8;

template <typename T>
__global__ void __launch_bounds__(256) issueChains(T* out, T x, unsigned long long rounds) {
  T acc[CHAINS];
  // The addend in a vector register: a vector instruction with a scalar-register operand issues at half the rate.
  x += T(threadIdx.x) * T(1e-30);
#pragma unroll
  for (int c = 0; c < CHAINS; ++c) acc[c] = T(threadIdx.x + c);
  for (unsigned long long r = 0; r < rounds; ++r) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int c = 0; c < CHAINS; ++c) {
        if constexpr (sizeof(T) == 4) acc[c] = acc[c] + x;   // one v_add_f32
        else acc[c] = __builtin_fma(acc[c], x, x);            // one v_fma_f64
      }
  }
  T s = T(0);
#pragma unroll
  for (int c = 0; c < CHAINS; ++c) s += acc[c];
  if (s == T(-1)) out[0] = s;  // never true for the arguments used; keeps the chains alive
}

template <typename T>
hipError_t timeLaunch(unsigned grid, unsigned long long rounds, T* out, float* ms) {
  hipEvent_t a, b;
  hipError_t e = hipEventCreate(&a);
  if (e != hipSuccess) return e;
  e = hipEventCreate(&b);
  if (e != hipSuccess) return e;
  (void)hipEventRecord(a, nullptr);
  hipLaunchKernelGGL(issueChains<T>, dim3(grid), dim3(256), 0, nullptr, out, T(1.0000001), rounds);
  (void)hipEventRecord(b, nullptr);
  e = hipEventSynchronize(b);
  if (e == hipSuccess) e = hipEventElapsedTime(ms, a, b);
  (void)hipEventDestroy(a);
  (void)hipEventDestroy(b);
  return e != hipSuccess ? e : hipGetLastError();
}

template <typename T>
int measure(double seconds, double* laneOpsPerSecond) {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 1;
  T* out = nullptr;
  if (hipMalloc(&out, sizeof(T)) != hipSuccess) return 1;
  const unsigned grid = unsigned(cus) * 8;  // 8 blocks of 4 wavefronts per CU: 8 wavefronts per SIMD
  const double opsPerRound = double(grid) * 256 * CHAINS * UNROLL;
  float ms = 0.f;
  unsigned long long rounds = 2000;
  int rc = 1;
  if (timeLaunch<T>(grid, rounds, out, &ms) == hipSuccess && ms > 0.f) {        // warm-up and a first estimate
    rounds = (unsigned long long)(rounds * (seconds * 1e3 / ms));
    if (rounds < 2000) rounds = 2000;
    if (timeLaunch<T>(grid, rounds, out, &ms) == hipSuccess && ms > 0.f) {
      *laneOpsPerSecond = opsPerRound * double(rounds) / (ms * 1e-3);
      rc = 0;
    }
  }
  (void)hipFree(out);
  return rc;
}

}  // namespace

// Lane-operations per second of independent float adds (f64 = 0) or double multiply-adds (f64 = 1) over a launch of
// about `seconds`; returns 0 on success. Uses the current device and the default stream.
extern "C" __attribute__((visibility("default"))) int spnc_issue_rate(int f64, double seconds, double* laneOpsPerSecond) {
  if (!laneOpsPerSecond || !(seconds > 0.0) || seconds > 5.0) return 2;
  return f64 ? measure<double>(seconds, laneOpsPerSecond) : measure<float>(seconds, laneOpsPerSecond);
}
