// Table-driven SPN interpreter kernel for gfx950.
//
// One sample per lane, 256-lane blocks, persistent over tiles of 256 samples. The instruction
// stream is wave-uniform and read through the constant address space (scalar loads); operands
// live in per-lane value slots laid out [slot][lane], so every LDS access is bank-conflict
// free and every spill access is fully coalesced. A lane only ever touches its own column of
// the slot file, so no barriers are needed.
//
// Arithmetic (log space): product = sum of child values; weighted sum over k children =
// m + log(sum_j w_j * exp(x_j - m)) with m = max_j x_j and linear weights w_j, which equals the
// reference's tree of pairwise log-adds (mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:216-240,
// mlir/lib/Conversion/HiSPNtoLoSPN/NodePatterns.cpp:49-88) up to rounding; sums sharing their
// child list share m and the exponentials. Gaussian and table leaves follow
// mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:306-374 and :440-529.
#include "interp_kernel.h"

#include "interp_program.h"
#include "spn_graph.h"

namespace spnc_hip {

namespace {

#define SPN_CONST __attribute__((address_space(4)))
typedef const SPN_CONST uint32_t* code_ptr;

constexpr unsigned B = INTERP_BLOCK;
constexpr uint32_t NONE = 0xFFFFFFFFu;

template <typename R, bool LOG2>
struct Math;
template <>
struct Math<float, true> {
  static __device__ __forceinline__ float exp(float x) { return __builtin_amdgcn_exp2f(x); }
  static __device__ __forceinline__ float log(float x) { return __builtin_amdgcn_logf(x); }
  static __device__ __forceinline__ float finish(float x) { return x * 0x1.62e43p-1f; }
  static __device__ __forceinline__ float lowest() { return -3.4028234663852886e38f; }
};
template <>
struct Math<float, false> {
  static __device__ __forceinline__ float exp(float x) { return expf(x); }
  static __device__ __forceinline__ float log(float x) { return logf(x); }
  static __device__ __forceinline__ float finish(float x) { return x; }
  static __device__ __forceinline__ float lowest() { return -3.4028234663852886e38f; }
};
template <>
struct Math<double, false> {
  static __device__ __forceinline__ double exp(double x) { return ::exp(x); }
  static __device__ __forceinline__ double log(double x) { return ::log(x); }
  static __device__ __forceinline__ double finish(double x) { return x; }
  static __device__ __forceinline__ double lowest() { return -1.7976931348623157e308; }
};

__device__ __forceinline__ float rmax(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double rmax(double a, double b) { return __builtin_fmax(a, b); }
__device__ __forceinline__ float rfma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double rfma(double a, double b, double c) { return __builtin_fma(a, b, c); }

template <typename R>
__device__ __forceinline__ R constAt(code_ptr code, uint32_t pc);
template <>
__device__ __forceinline__ float constAt<float>(code_ptr code, uint32_t pc) {
  return __uint_as_float(code[pc]);
}
template <>
__device__ __forceinline__ double constAt<double>(code_ptr code, uint32_t pc) {
  return __hiloint2double(int(code[pc + 1]), int(code[pc]));
}

template <typename R>
__device__ __forceinline__ R featureValue(const void* __restrict__ in, uint32_t type, unsigned long long idx) {
  switch (FeatureType(type)) {
    case FeatureType::U8: return R(static_cast<const unsigned char*>(in)[idx]);
    case FeatureType::U16: return R(static_cast<const unsigned short*>(in)[idx]);
    case FeatureType::U32: return R(static_cast<const unsigned int*>(in)[idx]);
    case FeatureType::U64: return R(static_cast<const unsigned long long*>(in)[idx]);
    case FeatureType::F32: return R(static_cast<const float*>(in)[idx]);
    default: return R(static_cast<const double*>(in)[idx]);
  }
}

// Clamped table index: values outside [0, L) select entry L ("impossible"), NaN selects
// entry L + 1 (marginal value) when marginalisation is supported.
__device__ __forceinline__ uint32_t featureIndex(const void* __restrict__ in, uint32_t type, unsigned long long idx, uint32_t L,
                                                 uint32_t marginal) {
  switch (FeatureType(type)) {
    case FeatureType::U8: {
      uint32_t v = static_cast<const unsigned char*>(in)[idx];
      return v < L ? v : L;
    }
    case FeatureType::U16: {
      uint32_t v = static_cast<const unsigned short*>(in)[idx];
      return v < L ? v : L;
    }
    case FeatureType::U32: {
      uint32_t v = static_cast<const unsigned int*>(in)[idx];
      return v < L ? v : L;
    }
    case FeatureType::U64: {
      unsigned long long v = static_cast<const unsigned long long*>(in)[idx];
      return v < L ? uint32_t(v) : L;
    }
    case FeatureType::F32: {
      float x = static_cast<const float*>(in)[idx];
      uint32_t t = (x > -1.0f && x < float(L)) ? uint32_t(x) : L;
      return (marginal && x != x) ? L + 1 : t;
    }
    default: {
      double x = static_cast<const double*>(in)[idx];
      uint32_t t = (x > -1.0 && x < double(L)) ? uint32_t(x) : L;
      return (marginal && x != x) ? L + 1 : t;
    }
  }
}

template <typename R>
struct Slots {
  R* lds;                    // this lane's column: slot s at lds[s * B]
  R* spill;                  // this lane's column: slot s at spill[(s - ldsSlots) * lanes]
  unsigned long long lanes;
  uint32_t ldsSlots;
  __device__ __forceinline__ R rd(uint32_t s) const { return s < ldsSlots ? lds[s * B] : spill[(unsigned long long)(s - ldsSlots) * lanes]; }
  __device__ __forceinline__ void wr(uint32_t s, R v) const {
    if (s < ldsSlots) lds[s * B] = v;
    else spill[(unsigned long long)(s - ldsSlots) * lanes] = v;
  }
};

template <typename R, bool LOG2, int M>
__device__ __forceinline__ uint32_t sumLayer(code_ptr code, uint32_t pc, uint32_t k, const Slots<R>& S) {
  typedef Math<R, LOG2> Mt;
  constexpr uint32_t RW = sizeof(R) / 4;
  const uint32_t dsts = pc + 2, kids = dsts + M, wts = kids + k;
  R m = R(-__builtin_huge_val());
#pragma unroll 4
  for (uint32_t j = 0; j < k; ++j) m = rmax(m, S.rd(code[kids + j]));
  const R ms = rmax(m, Mt::lowest());  // all children impossible: keep exp() arguments at -inf, not NaN
  R acc[M];
#pragma unroll
  for (int t = 0; t < M; ++t) acc[t] = R(0);
#pragma unroll 2
  for (uint32_t j = 0; j < k; ++j) {
    const R e = Mt::exp(S.rd(code[kids + j]) - ms);
#pragma unroll
    for (int t = 0; t < M; ++t) acc[t] = rfma(e, constAt<R>(code, wts + (j * M + t) * RW), acc[t]);
  }
#pragma unroll
  for (int t = 0; t < M; ++t) S.wr(code[dsts + t], ms + Mt::log(acc[t]));
  return wts + k * M * RW;
}

template <typename R, bool LOG2>
__global__ void __launch_bounds__(INTERP_BLOCK) spn_interp_kernel(const uint32_t* __restrict__ codeGlobal, InterpLaunch a) {
  typedef Math<R, LOG2> Mt;
  constexpr uint32_t RW = sizeof(R) / 4;
  extern __shared__ __align__(16) unsigned char ldsRaw[];
  code_ptr code = (code_ptr)codeGlobal;
  const SPN_CONST uint32_t* staged = (const SPN_CONST uint32_t*)a.staged;
  const R* __restrict__ tables = static_cast<const R*>(a.tables);
  R* __restrict__ out = static_cast<R*>(a.out);
  Slots<R> S;
  S.lds = reinterpret_cast<R*>(ldsRaw) + threadIdx.x;
  S.lanes = (unsigned long long)gridDim.x * B;
  S.spill = static_cast<R*>(a.spill) + (unsigned long long)blockIdx.x * B + threadIdx.x;
  S.ldsSlots = a.ldsSlots;
  const unsigned long long F = a.numFeatures;
  const bool stagedMode = a.featureMode == FEAT_STAGED;

  for (unsigned long long base = (unsigned long long)blockIdx.x * B; base < a.n; base += S.lanes) {
    const unsigned long long i = base + threadIdx.x;
    const bool valid = i < a.n;
    const unsigned long long row = (valid ? i : a.n - 1) * F;  // idle lanes recompute the last sample

    if (stagedMode) {
      for (uint32_t s = 0; s < a.numStaged; ++s) {
        const uint32_t col = staged[4 * s], vs = staged[4 * s + 1], is = staged[4 * s + 2], L = staged[4 * s + 3];
        if (vs != NONE) S.wr(vs, featureValue<R>(a.in, a.featureType, row + col));
        if (is != NONE) S.wr(is, R(featureIndex(a.in, a.featureType, row + col, L, a.marginal)));
      }
    }

    uint32_t pc = 0;
    R result;
    for (;;) {
      const uint32_t w0 = code[pc];
      const uint32_t op = w0 & 0xffu;
      if (op == OP_END) {
        result = S.rd(code[pc + 1]);
        break;
      }
      if (op == OP_PROD) {
        const uint32_t dst = code[pc + 1], ns = code[pc + 2], ng = code[pc + 3], nt = code[pc + 4];
        pc += 5;
        R acc = R(0);
#pragma unroll 4
        for (uint32_t j = 0; j < ns; ++j) acc += S.rd(code[pc + j]);
        pc += ns;
#pragma unroll 2
        for (uint32_t j = 0; j < ng; ++j) {
          const uint32_t fw = code[pc];
          const R mean = constAt<R>(code, pc + 1), coef = constAt<R>(code, pc + 1 + RW), den = constAt<R>(code, pc + 1 + 2 * RW);
          pc += 1 + 3 * RW;
          const R x = stagedMode ? S.rd(fw) : featureValue<R>(a.in, a.featureType, row + fw);
          const R d = x - mean;
          R v = coef + (d * d) * den;
          if (a.marginal) v = (x != x) ? R(0) : v;
          acc += v;
        }
        for (uint32_t j = 0; j < nt; ++j) {
          const uint32_t fw = code[pc], off = code[pc + 1], L = code[pc + 2];
          pc += 3;
          const uint32_t idx = stagedMode ? uint32_t(S.rd(fw)) : featureIndex(a.in, a.featureType, row + fw, L, a.marginal);
          acc += tables[off + idx];
        }
        S.wr(dst, acc);
      } else if (op == OP_SUM) {
        const uint32_t k = w0 >> 8, dst = code[pc + 1];
        pc += 2;
        if (k == 1) {
          S.wr(dst, S.rd(code[pc]) + constAt<R>(code, pc + 1));
          pc += 1 + RW;
        } else {
          R m = R(-__builtin_huge_val());
#pragma unroll 4
          for (uint32_t j = 0; j < k; ++j) m = rmax(m, S.rd(code[pc + j * (1 + RW)]));
          const R ms = rmax(m, Mt::lowest());
          R acc = R(0);
#pragma unroll 4
          for (uint32_t j = 0; j < k; ++j)
            acc = rfma(Mt::exp(S.rd(code[pc + j * (1 + RW)]) - ms), constAt<R>(code, pc + j * (1 + RW) + 1), acc);
          pc += k * (1 + RW);
          S.wr(dst, ms + Mt::log(acc));
        }
      } else {  // OP_SUMLAYER
        const uint32_t k = w0 >> 8, m = code[pc + 1];
        if (m == 8) pc = sumLayer<R, LOG2, 8>(code, pc, k, S);
        else if (m == 4) pc = sumLayer<R, LOG2, 4>(code, pc, k, S);
        else pc = sumLayer<R, LOG2, 2>(code, pc, k, S);
      }
    }
    if (valid) out[i] = Mt::finish(result);
  }
}

template <typename R, bool LOG2>
const void* kernelPtr() {
  return reinterpret_cast<const void*>(&spn_interp_kernel<R, LOG2>);
}

const void* pick(bool f64, bool log2Domain) {
  if (f64) return kernelPtr<double, false>();
  return log2Domain ? kernelPtr<float, true>() : kernelPtr<float, false>();
}

}  // namespace

hipError_t interpreterMaxLds(bool f64, bool log2Domain, size_t* bytes) {
  int dev = 0, maxLds = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  e = hipDeviceGetAttribute(&maxLds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
  if (e != hipSuccess) return e;
  (void)f64;
  (void)log2Domain;
  *bytes = size_t(maxLds);
  return hipSuccess;
}

hipError_t interpreterOccupancy(bool f64, bool log2Domain, size_t ldsBytes, int* blocksPerCU) {
  return hipOccupancyMaxActiveBlocksPerMultiprocessor(blocksPerCU, pick(f64, log2Domain), int(INTERP_BLOCK), ldsBytes);
}

hipError_t launchInterpreter(const InterpLaunch& args, bool f64, bool log2Domain, unsigned grid, size_t ldsBytes, hipStream_t stream) {
  const void* fn = pick(f64, log2Domain);
  if (ldsBytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, int(ldsBytes));
    if (e != hipSuccess) return e;
  }
  const uint32_t* code = args.code;
  InterpLaunch a = args;
  void* params[] = {(void*)&code, (void*)&a};
  return hipLaunchKernel(fn, dim3(grid), dim3(INTERP_BLOCK), params, ldsBytes, stream);
}

}  // namespace spnc_hip
