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

// Constants are read at a signed offset from a pointer, not at an unsigned index into the
// stream: only then may the compiler merge neighbouring reads into one wide scalar load.
template <typename R>
__device__ __forceinline__ R constAt(code_ptr code, long pc);
template <>
__device__ __forceinline__ float constAt<float>(code_ptr code, long pc) {
  return __uint_as_float(code[pc]);
}
template <>
__device__ __forceinline__ double constAt<double>(code_ptr code, long pc) {
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

// SPILL = false: every slot of the program lives in LDS, reads and writes are branch-free, so
// the compiler can batch the operand reads of an instruction.
template <typename R, bool SPILL>
struct Slots {
  R* lds;                    // this lane's column: slot s at lds[s * B]
  R* spill;                  // this lane's column: slot s at spill[(s - ldsSlots) * lanes]
  unsigned long long lanes;
  uint32_t ldsSlots;
  __device__ __forceinline__ R rd(uint32_t s) const {
    if (!SPILL) return lds[s * B];
    return s < ldsSlots ? lds[s * B] : spill[(unsigned long long)(s - ldsSlots) * lanes];
  }
  __device__ __forceinline__ void wr(uint32_t s, R v) const {
    if (!SPILL || s < ldsSlots) lds[s * B] = v;
    else spill[(unsigned long long)(s - ldsSlots) * lanes] = v;
  }
};

// All instruction decoding goes through a pointer to the current instruction (`ip`) and signed
// offsets from it, so that neighbouring words are fetched with wide scalar loads.

template <typename R, bool LOG2, bool SPILL, int M>
__device__ __forceinline__ code_ptr sumLayer(code_ptr ip, int k, const Slots<R, SPILL>& S) {
  typedef Math<R, LOG2> Mt;
  constexpr int RW = sizeof(R) / 4;
  code_ptr dsts = ip + 2, kids = dsts + M, w = kids + k;
  R m = R(-__builtin_huge_val());
#pragma unroll 8
  for (int j = 0; j < k; ++j) m = rmax(m, S.rd(kids[j]));
  const R ms = rmax(m, Mt::lowest());  // all children impossible: keep exp() arguments at -inf, not NaN
  R acc[M];
#pragma unroll
  for (int t = 0; t < M; ++t) acc[t] = R(0);
#pragma unroll 4
  for (int j = 0; j < k; ++j) {
    const R e = Mt::exp(S.rd(kids[j]) - ms);
#pragma unroll
    for (int t = 0; t < M; ++t) acc[t] = rfma(e, constAt<R>(w, (long(j) * M + t) * RW), acc[t]);
  }
#pragma unroll
  for (int t = 0; t < M; ++t) S.wr(dsts[t], ms + Mt::log(acc[t]));
  return w + long(k) * M * RW;
}

// M sums over the outer product of operand vectors a (NA slots) and b (NB slots):
// out_j = ma + mb + log(sum_{r,c} w_j[r][c] * exp(a_r - ma) * exp(b_c - mb)), ma = max a, mb = max b.
template <typename R, bool LOG2, bool SPILL, int M, int NB>
__device__ __forceinline__ code_ptr outerSum(code_ptr ip, int na, const Slots<R, SPILL>& S) {
  typedef Math<R, LOG2> Mt;
  constexpr int RW = sizeof(R) / 4;
  code_ptr dsts = ip + 2, as = dsts + M, bs = as + na, w = bs + NB;
  R eb[NB];
  R mb = R(-__builtin_huge_val());
#pragma unroll
  for (int c = 0; c < NB; ++c) {
    eb[c] = S.rd(bs[c]);
    mb = rmax(mb, eb[c]);
  }
  mb = rmax(mb, Mt::lowest());
#pragma unroll
  for (int c = 0; c < NB; ++c) eb[c] = Mt::exp(eb[c] - mb);
  R ma = R(-__builtin_huge_val());
#pragma unroll 8
  for (int r = 0; r < na; ++r) ma = rmax(ma, S.rd(as[r]));
  ma = rmax(ma, Mt::lowest());
  R acc[M];
#pragma unroll
  for (int t = 0; t < M; ++t) acc[t] = R(0);
  for (int r = 0; r < na; ++r) {
    const R ea = Mt::exp(S.rd(as[r]) - ma);
#pragma unroll
    for (int c = 0; c < NB; ++c) {
      const R e = ea * eb[c];
#pragma unroll
      for (int t = 0; t < M; ++t) acc[t] = rfma(e, constAt<R>(w, ((long(r) * NB + c) * M + t) * RW), acc[t]);
    }
  }
  const R base = ma + mb;
#pragma unroll
  for (int t = 0; t < M; ++t) S.wr(dsts[t], base + Mt::log(acc[t]));
  return w + long(na) * NB * M * RW;
}

// Fully unrolled form for operand vectors of a fixed, small size that all live in LDS: both
// vectors are read into registers first, so that the multiply-accumulate part contains no LDS
// access and its weights can stream in through wide scalar loads that overlap the arithmetic.
template <typename R, bool LOG2, int M, int NA, int NB>
__device__ __forceinline__ code_ptr outerSumFixed(code_ptr ip, const Slots<R, false>& S) {
  typedef Math<R, LOG2> Mt;
  constexpr int RW = sizeof(R) / 4;
  code_ptr dsts = ip + 2, as = dsts + M, bs = as + NA, w = bs + NB;
  R ea[NA], eb[NB];
  R ma = R(-__builtin_huge_val()), mb = R(-__builtin_huge_val());
#pragma unroll
  for (int r = 0; r < NA; ++r) ea[r] = S.rd(as[r]);
#pragma unroll
  for (int c = 0; c < NB; ++c) eb[c] = S.rd(bs[c]);
#pragma unroll
  for (int r = 0; r < NA; ++r) ma = rmax(ma, ea[r]);
#pragma unroll
  for (int c = 0; c < NB; ++c) mb = rmax(mb, eb[c]);
  ma = rmax(ma, Mt::lowest());
  mb = rmax(mb, Mt::lowest());
#pragma unroll
  for (int r = 0; r < NA; ++r) ea[r] = Mt::exp(ea[r] - ma);
#pragma unroll
  for (int c = 0; c < NB; ++c) eb[c] = Mt::exp(eb[c] - mb);
  R acc[M];
#pragma unroll
  for (int t = 0; t < M; ++t) acc[t] = R(0);
  // The weights arrive through scalar loads, whose wait counter is all-or-nothing: they are
  // requested two chunks of PAIRS (r,c) pairs ahead and the scheduler is kept from moving the
  // requests, so that two chunks of multiply-adds (and the other waves of the SIMD) cover the
  // latency of a chunk's loads.
  constexpr int PAIRS = (16 / RW) / M >= 1 ? (16 / RW) / M : 1, CHUNKS = NA * NB / PAIRS, AHEAD = 2;
  static_assert(NA * NB % PAIRS == 0, "chunking must divide the weight matrix");
  R wc[AHEAD + 1][PAIRS * M];
#pragma unroll
  for (int q = 0; q < AHEAD && q < CHUNKS; ++q)
#pragma unroll
    for (int j = 0; j < PAIRS * M; ++j) wc[q][j] = constAt<R>(w, (q * PAIRS * M + j) * RW);
#pragma unroll
  for (int q = 0; q < CHUNKS; ++q) {
    if (q + AHEAD < CHUNKS) {
#pragma unroll
      for (int j = 0; j < PAIRS * M; ++j) wc[(q + AHEAD) % (AHEAD + 1)][j] = constAt<R>(w, ((q + AHEAD) * PAIRS * M + j) * RW);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 0; k < PAIRS; ++k) {
      const int rc = q * PAIRS + k;
      const R e = ea[rc / NB] * eb[rc % NB];
#pragma unroll
      for (int t = 0; t < M; ++t) acc[t] = rfma(e, wc[q % (AHEAD + 1)][k * M + t], acc[t]);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  const R base = ma + mb;
#pragma unroll
  for (int t = 0; t < M; ++t) S.wr(dsts[t], base + Mt::log(acc[t]));
  return w + NA * NB * M * RW;
}

template <typename R, bool LOG2, bool SPILL, int M>
__device__ __forceinline__ code_ptr outerSumNB(code_ptr ip, int na, int nb, const Slots<R, SPILL>& S) {
  if constexpr (!SPILL && M == 8 && LOG2) {  // the unrolled form only where it pays: the float log2-domain kernel
    if (na == 8 && nb == 8) return outerSumFixed<R, LOG2, 8, 8, 8>(ip, S);
    if (na == 4 && nb == 4) return outerSumFixed<R, LOG2, 8, 4, 4>(ip, S);
  }
  if (nb == 8) return outerSum<R, LOG2, SPILL, M, 8>(ip, na, S);
  if (nb == 4) return outerSum<R, LOG2, SPILL, M, 4>(ip, na, S);
  if (nb == 16) return outerSum<R, LOG2, SPILL, M, 16>(ip, na, S);
  return outerSum<R, LOG2, SPILL, M, 2>(ip, na, S);
}

// Executes one instruction other than OP_END and returns the pointer to the next one.
template <typename R, bool LOG2, bool SPILL>
__device__ __forceinline__ code_ptr execute(code_ptr ip, uint32_t w0, const Slots<R, SPILL>& S, const InterpLaunch& a,
                                            const R* __restrict__ tables, unsigned long long row, bool stagedMode) {
  typedef Math<R, LOG2> Mt;
  constexpr int RW = sizeof(R) / 4;
  const uint32_t op = w0 & 0x7fu;
  if (op == OP_PROD) {
    const uint32_t dst = ip[1];
    const int ns = int(ip[2]), ng = int(ip[3]), nt = int(ip[4]);
    ip += 5;
    R acc = R(0);
#pragma unroll 4
    for (int j = 0; j < ns; ++j) acc += S.rd(ip[j]);
    ip += ns;
#pragma unroll 2
    for (int j = 0; j < ng; ++j) {
      const uint32_t fw = ip[0];
      const R mean = constAt<R>(ip, 1), coef = constAt<R>(ip, 1 + RW), den = constAt<R>(ip, 1 + 2 * RW);
      ip += 1 + 3 * RW;
      const R x = stagedMode ? S.rd(fw) : featureValue<R>(a.in, a.featureType, row + fw);
      const R d = x - mean;
      R v = coef + (d * d) * den;
      if (a.marginal) v = (x != x) ? R(0) : v;
      acc += v;
    }
    for (int j = 0; j < nt; ++j) {
      const uint32_t fw = ip[0], off = ip[1], L = ip[2];
      ip += 3;
      const uint32_t idx = stagedMode ? uint32_t(S.rd(fw)) : featureIndex(a.in, a.featureType, row + fw, L, a.marginal);
      acc += tables[off + idx];
    }
    S.wr(dst, acc);
    return ip;
  }
  if (op == OP_SUM) {
    const int k = int(w0 >> 8);
    const uint32_t dst = ip[1];
    ip += 2;
    if (k == 1) {
      S.wr(dst, S.rd(ip[0]) + constAt<R>(ip, 1));
      return ip + 1 + RW;
    }
    R m = R(-__builtin_huge_val());
#pragma unroll 4
    for (int j = 0; j < k; ++j) m = rmax(m, S.rd(ip[long(j) * (1 + RW)]));
    const R ms = rmax(m, Mt::lowest());
    R acc = R(0);
#pragma unroll 4
    for (int j = 0; j < k; ++j) acc = rfma(Mt::exp(S.rd(ip[long(j) * (1 + RW)]) - ms), constAt<R>(ip, long(j) * (1 + RW) + 1), acc);
    S.wr(dst, ms + Mt::log(acc));
    return ip + long(k) * (1 + RW);
  }
  if (op == OP_SUMLAYER) {
    const int k = int(w0 >> 8);
    const uint32_t m = ip[1];
    if (m == 8) return sumLayer<R, LOG2, SPILL, 8>(ip, k, S);
    if (m == 4) return sumLayer<R, LOG2, SPILL, 4>(ip, k, S);
    return sumLayer<R, LOG2, SPILL, 2>(ip, k, S);
  }
  // OP_OUTERSUM
  const int na = int((w0 >> 8) & 0xffu), nb = int(w0 >> 16);
  const uint32_t m = ip[1];
  if (m == 8) return outerSumNB<R, LOG2, SPILL, 8>(ip, na, nb, S);
  if (m == 4) return outerSumNB<R, LOG2, SPILL, 4>(ip, na, nb, S);
  return outerSumNB<R, LOG2, SPILL, 2>(ip, na, nb, S);
}

// MODE 0: every slot lives in LDS. MODE 1: slots below ldsSlots (the program's short pool) live
// in LDS, and only instructions flagged with bit 7 may touch the spill tier. MODE 2: any
// instruction may touch the spill tier (the short pool did not fit into LDS).
template <typename R, bool LOG2, int MODE>
__global__ void __launch_bounds__(INTERP_BLOCK) spn_interp_kernel(const uint32_t* __restrict__ codeGlobal, InterpLaunch a) {
  typedef Math<R, LOG2> Mt;
  extern __shared__ __align__(16) unsigned char ldsRaw[];
  code_ptr code = (code_ptr)codeGlobal;
  const SPN_CONST uint32_t* staged = (const SPN_CONST uint32_t*)a.staged;
  const R* __restrict__ tables = static_cast<const R*>(a.tables);
  R* __restrict__ out = static_cast<R*>(a.out);
  Slots<R, true> Sg;
  Sg.lds = reinterpret_cast<R*>(ldsRaw) + threadIdx.x;
  Sg.lanes = (unsigned long long)gridDim.x * B;
  Sg.spill = static_cast<R*>(a.spill) + (unsigned long long)blockIdx.x * B + threadIdx.x;
  Sg.ldsSlots = a.ldsSlots;
  Slots<R, false> Sl;
  Sl.lds = Sg.lds;
  Sl.lanes = Sg.lanes;
  Sl.spill = Sg.spill;
  Sl.ldsSlots = Sg.ldsSlots;
  const unsigned long long F = a.numFeatures;
  const bool stagedMode = a.featureMode == FEAT_STAGED;

  for (unsigned long long base = (unsigned long long)blockIdx.x * B; base < a.n; base += Sg.lanes) {
    const unsigned long long i = base + threadIdx.x;
    const bool valid = i < a.n;
    const unsigned long long row = (valid ? i : a.n - 1) * F;  // idle lanes recompute the last sample

    if (stagedMode) {
      for (int s = 0; s < int(a.numStaged); ++s) {
        const uint32_t col = staged[4 * s], vs = staged[4 * s + 1], is = staged[4 * s + 2], L = staged[4 * s + 3];
        if (MODE != 0) {
          if (vs != NONE) Sg.wr(vs, featureValue<R>(a.in, a.featureType, row + col));
          if (is != NONE) Sg.wr(is, R(featureIndex(a.in, a.featureType, row + col, L, a.marginal)));
        } else {
          if (vs != NONE) Sl.wr(vs, featureValue<R>(a.in, a.featureType, row + col));
          if (is != NONE) Sl.wr(is, R(featureIndex(a.in, a.featureType, row + col, L, a.marginal)));
        }
      }
    }

    code_ptr ip = code;
    R result;
    for (;;) {
      const uint32_t w0 = ip[0];
      const bool spillPath = MODE == 2 || (MODE == 1 && (w0 & 0x80u));
      if ((w0 & 0x7fu) == OP_END) {
        result = spillPath ? Sg.rd(ip[1]) : Sl.rd(ip[1]);
        break;
      }
      if (MODE != 0 && spillPath) ip = execute<R, LOG2, true>(ip, w0, Sg, a, tables, row, stagedMode);
      else ip = execute<R, LOG2, false>(ip, w0, Sl, a, tables, row, stagedMode);
    }
    if (valid) out[i] = Mt::finish(result);
  }
}

template <typename R, bool LOG2>
const void* kernelPtr(int mode) {
  if (mode == 0) return reinterpret_cast<const void*>(&spn_interp_kernel<R, LOG2, 0>);
  if (mode == 1) return reinterpret_cast<const void*>(&spn_interp_kernel<R, LOG2, 1>);
  return reinterpret_cast<const void*>(&spn_interp_kernel<R, LOG2, 2>);
}

const void* pick(bool f64, bool log2Domain, int mode) {
  if (f64) return kernelPtr<double, false>(mode);
  return log2Domain ? kernelPtr<float, true>(mode) : kernelPtr<float, false>(mode);
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

hipError_t interpreterOccupancy(bool f64, bool log2Domain, int mode, size_t ldsBytes, int* blocksPerCU) {
  const void* fn = pick(f64, log2Domain, mode);
  if (ldsBytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, int(ldsBytes));
    if (e != hipSuccess) return e;
  }
  return hipOccupancyMaxActiveBlocksPerMultiprocessor(blocksPerCU, fn, int(INTERP_BLOCK), ldsBytes);
}

hipError_t launchInterpreter(const InterpLaunch& args, bool f64, bool log2Domain, int mode, unsigned grid, size_t ldsBytes,
                             hipStream_t stream) {
  const void* fn = pick(f64, log2Domain, mode);
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
