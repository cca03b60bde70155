// Device code of the table-driven SPN interpreter (templates). Included by the translation units that instantiate the
// kernels, one flavour each (interp_kernel_inst.hip, built once per flavour), so that they compile in parallel.
#pragma once
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

// A wavefront that waits for memory between short bursts of arithmetic (leaf operands: constants, features, weights)
// runs at a higher priority than one inside a long matrix chain, so that its bursts go out when its data arrive and
// the chains of the other wavefronts fill the rest of the pipe.
#ifndef SPN_PRIO
#define SPN_PRIO 1
#endif
#if SPN_PRIO
#ifndef SPN_PRIO_HIGH
#define SPN_PRIO_HIGH 1
#endif
#define SPN_PRIO_LATENCY() __builtin_amdgcn_s_setprio(SPN_PRIO_HIGH)
#define SPN_PRIO_CHAIN() __builtin_amdgcn_s_setprio(0)
#else
#define SPN_PRIO_LATENCY()
#define SPN_PRIO_CHAIN()
#endif

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

// float64 in the log2 domain: base-2 exponential and logarithm by table and short polynomial, the routines that
// the straight-line float64 kernels carry (emit_hip.cpp): 2^x = 2^(n>>6) * T[n&63] * 2^r with n = rint(64 x),
// |r| <= 1/128 and a degree-5 polynomial; log2(2^e t) = e + G[j] + log2(1 + u), j = the top eight fraction bits of t,
// u = t R[j] - 1 in one fma, degree-7 polynomial. Within 1e-15 of libm. The tables (doubleMathTables()) are copied from
// behind the program's leaf tables into LDS when the kernel starts.
__shared__ double mathExp2[64];
__shared__ __align__(16) double mathLog2[512];
__shared__ double mathPoly[12];
template <>
struct Math<double, true> {
  static __device__ __forceinline__ double exp(double x) {
    x = x < -1100.0 ? -1100.0 : x;  // keeps NaN
    const double n = __builtin_rint(x * 64.0), r = __builtin_fma(n, -0x1p-6, x);
    const int ni = (int)n;
    const double t = mathExp2[ni & 63];
    double p = mathPoly[0];
    p = __builtin_fma(p, r, mathPoly[1]);
    p = __builtin_fma(p, r, mathPoly[2]);
    p = __builtin_fma(p, r, mathPoly[3]);
    p = __builtin_fma(p, r, mathPoly[4]);
    return __builtin_ldexp(__builtin_fma(t, p * r, t), ni >> 6);
  }
  static __device__ __forceinline__ double log(double x) {
    union { double d; unsigned long long u; } c;
    c.d = x;
    const unsigned hi = (unsigned)(c.u >> 32);
    const int e = (int)(hi >> 20) - 1023;
    const unsigned j = (hi >> 12) & 255u;
    c.u = (c.u & 0x000fffffffffffffull) | 0x3ff0000000000000ull;
    const double u = __builtin_fma(c.d, mathLog2[2 * j], -1.0);
    double p = mathPoly[5];
    p = __builtin_fma(p, u, mathPoly[6]);
    p = __builtin_fma(p, u, mathPoly[7]);
    p = __builtin_fma(p, u, mathPoly[8]);
    p = __builtin_fma(p, u, mathPoly[9]);
    p = __builtin_fma(p, u, mathPoly[10]);
    p = __builtin_fma(p, u, mathPoly[11]);
    const double r = __builtin_fma(u, p, mathLog2[2 * j + 1] + (double)e);
    return x == 0.0 ? -__builtin_huge_val() : (x != x ? x : r);  // 0: a sum whose terms are all impossible
  }
  static __device__ __forceinline__ double finish(double x) { return x * 0x1.62e42fefa39efp-1; }
  static __device__ __forceinline__ double lowest() { return -1.7976931348623157e308; }
};

__device__ __forceinline__ float rmax(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double rmax(double a, double b) { return __builtin_fmax(a, b); }
__device__ __forceinline__ float rfma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double rfma(double a, double b, double c) { return __builtin_fma(a, b, c); }

// A Gaussian leaf from its three constants and the neutral element / combination of a product, in log space
// (shift and den: den * ((x - mean)^2 + shift)) and in linear space (coef and den: coef * exp((x - mean)^2 * den)).
template <bool LINEAR, typename R>
__device__ __forceinline__ R gaussLeaf(R x, R mean, R c1, R c2) {
  const R d = x - mean;
  if constexpr (LINEAR) return c1 * ::exp(d * d * c2);
  else return rfma(d, d, c1) * c2;
}
template <bool LINEAR, typename R>
__device__ __forceinline__ R productStart() { return LINEAR ? R(1) : R(0); }
template <bool LINEAR, typename R>
__device__ __forceinline__ R productJoin(R acc, R v) { return LINEAR ? acc * v : acc + v; }

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

// The first 64 words of an instruction, length word included, held in one vector register: lane j
// holds word j, fetched with one coalesced load that the main loop issues for the next instruction
// before it executes the current one. A word becomes a scalar through a lane read, which costs a few
// cycles where a scalar load from the stream would cost a trip to the L2.
struct Head {
  static constexpr int WORDS = 64;
  uint32_t lanes;
  __device__ __forceinline__ uint32_t word(int j) const { return uint32_t(__builtin_amdgcn_readlane(int(lanes), j)); }
};
__device__ __forceinline__ Head loadHead(const uint32_t* codeGlobal, long at) {
  Head h;
  h.lanes = codeGlobal[at + (threadIdx.x & 63u)];
  return h;
}

// SPILL = false: every slot of the program lives in LDS, reads and writes are branch-free, so
// the compiler can batch the operand reads of an instruction.
template <typename R, bool SPILL>
struct Slots {
  R* lds;        // this lane's column in LDS: slot s at lds[s * B]
  R* spill;      // this lane's column in its block's part of the spill tier, moved back by ldsSlots slots:
                 // slot s >= ldsSlots at spill[s * B], so both tiers use the same stride
  R* spillBlock; // the same without the lane: wave-uniform, so spill accesses can take a scalar base and the lane as offset
  uint32_t ldsSlots;
  __device__ __forceinline__ R rdLds(uint32_t s) const { return lds[s * B]; }
  __device__ __forceinline__ R rdSpill(uint32_t s) const { return spillBlock[(unsigned long long)s * B + threadIdx.x]; }
  __device__ __forceinline__ void wrLds(uint32_t s, R v) const { lds[s * B] = v; }
  __device__ __forceinline__ void wrSpill(uint32_t s, R v) const { spillBlock[(unsigned long long)s * B + threadIdx.x] = v; }
  // With a spill tier the base pointer is selected, not the access: one generic load or store
  // per operand and no branch, so the operand accesses of an instruction can be in flight together.
  __device__ __forceinline__ R* at(uint32_t s) const {
    const unsigned long long inLds = (unsigned long long)(long long)(int32_t(s - ldsSlots) >> 31);  // all ones for LDS slots
    const unsigned long long base = ((unsigned long long)lds & inLds) | ((unsigned long long)spill & ~inLds);
    return reinterpret_cast<R*>(base) + s * B;
  }
  __device__ __forceinline__ R rd(uint32_t s) const {
    if (!SPILL) return lds[s * B];
    return *at(s);
  }
  __device__ __forceinline__ void wr(uint32_t s, R v) const {
    if (!SPILL) lds[s * B] = v;
    else *at(s) = v;
  }
};

// All instruction decoding goes through a pointer to the current instruction (`ip`) and signed
// offsets from it, so that neighbouring words are fetched with wide scalar loads.

// LINEAR (here and below): the program computes with probabilities, not their logarithms (the reference's
// computeInLogSpace=False, mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:242-304): products multiply, sums are plain
// weighted sums, a Gaussian leaf is coef * exp((x - mean)^2 * den), and only the root takes a logarithm.
template <typename R, bool LOG2, bool SPILL, int M, bool LINEAR = false>
__device__ __forceinline__ code_ptr sumLayer(code_ptr ip, int k, const Slots<R, SPILL>& S) {
  typedef Math<R, LOG2> Mt;
  constexpr int RW = sizeof(R) / 4;
  code_ptr dsts = ip + 2, kids = dsts + M, w = kids + k;
  if constexpr (LINEAR) {
    R sum[M];
#pragma unroll
    for (int t = 0; t < M; ++t) sum[t] = R(0);
#pragma unroll 4
    for (int j = 0; j < k; ++j) {
      const R x = S.rd(kids[j]);
#pragma unroll
      for (int t = 0; t < M; ++t) sum[t] = rfma(x, constAt<R>(w, (long(j) * M + t) * RW), sum[t]);
    }
#pragma unroll
    for (int t = 0; t < M; ++t) S.wr(dsts[t], sum[t]);
    return w + long(k) * M * RW;
  }
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
template <typename R, bool LOG2, bool SPILL, int M, int NB, bool LINEAR = false>
__device__ __forceinline__ code_ptr outerSum(code_ptr ip, int na, const Slots<R, SPILL>& S) {
  typedef Math<R, LOG2> Mt;
  constexpr int RW = sizeof(R) / 4;
  code_ptr dsts = ip + 2, as = dsts + M, bs = as + na, w = bs + NB;
  if constexpr (LINEAR) {
    R vb[NB], sum[M];
#pragma unroll
    for (int c = 0; c < NB; ++c) vb[c] = S.rd(bs[c]);
#pragma unroll
    for (int t = 0; t < M; ++t) sum[t] = R(0);
    for (int r = 0; r < na; ++r) {
      const R va = S.rd(as[r]);
#pragma unroll
      for (int c = 0; c < NB; ++c) {
        const R e = va * vb[c];
#pragma unroll
        for (int t = 0; t < M; ++t) sum[t] = rfma(e, constAt<R>(w, ((long(r) * NB + c) * M + t) * RW), sum[t]);
      }
    }
#pragma unroll
    for (int t = 0; t < M; ++t) S.wr(dsts[t], sum[t]);
    return w + long(na) * NB * M * RW;
  }
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

// Outer sum of eight double sums with the weights held in lanes. A double multiply-add takes its first factor from
// another lane of its row of sixteen at no cost (v_fmac_f64 with the DPP control row_newbcast; the float forms of that
// operand run at half rate, the double ones do not), so a register pair that every lane loaded 8 bytes of (lane l of a
// row the l-th of sixteen consecutive weights) feeds sixteen multiply-adds: the eight sums of two products, which is
// how the weights of this instruction lie in the stream (product-major, eight sums each). No scalar loads, no
// scalar operands; the vectors of operand row r + 1 are requested while row r is being added up.
struct __attribute__((packed, aligned(4))) StreamDouble {  // a double in the instruction stream: at a multiple of four bytes
  double value;
};
template <bool LOG2, bool SPILL, int NB, bool LINEAR = false>
__device__ __forceinline__ code_ptr outerSumLaneWeights(code_ptr ip, int na, const StreamDouble* wGlobal, const Slots<double, SPILL>& S) {
  typedef Math<double, LOG2> Mt;
  constexpr int M = 8, V = NB / 2;  // vectors of sixteen weights per operand row
  code_ptr dsts = ip + 2, as = dsts + M, bs = as + na;
  double eb[NB];
  double mb = -__builtin_huge_val();
#pragma unroll
  for (int c = 0; c < NB; ++c) {
    eb[c] = S.rd(bs[c]);
    mb = rmax(mb, eb[c]);
  }
  mb = LINEAR ? 0.0 : rmax(mb, Mt::lowest());
  const StreamDouble* wl = wGlobal + (threadIdx.x & 15u);
  double W[2][V];
#pragma unroll
  for (int v = 0; v < V; ++v) W[0][v] = wl[v * 16].value;
  double ma = 0.0;
  if constexpr (!LINEAR) {
#pragma unroll
    for (int c = 0; c < NB; ++c) eb[c] = Mt::exp(eb[c] - mb);
    ma = -__builtin_huge_val();
#pragma unroll 8
    for (int r = 0; r < na; ++r) ma = rmax(ma, S.rd(as[r]));
    ma = rmax(ma, Mt::lowest());
  }
  double acc[M];
#pragma unroll
  for (int t = 0; t < M; ++t) acc[t] = 0.0;
  // Two rows per round so that the two sets of vectors keep their registers.
  for (int r = 0; r < na; r += 2) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int row = r + half;
      // the next row's weights (past the last row: the words that follow the instruction, read and not used)
#pragma unroll
      for (int v = 0; v < V; ++v) W[half ^ 1][v] = wl[((row + 1) * V + v) * 16].value;
      const double ea = LINEAR ? S.rd(as[row]) : Mt::exp(S.rd(as[row]) - ma);
#pragma unroll
      for (int c = 0; c < NB; ++c) {
        const double e = ea * eb[c];
        if (c % 2 == 0)
          asm("v_fmac_f64_dpp %0, %8, %9 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %1, %8, %9 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %2, %8, %9 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %3, %8, %9 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %4, %8, %9 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %5, %8, %9 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %6, %8, %9 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %7, %8, %9 row_newbcast:7 row_mask:0xf bank_mask:0xf"
              : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
              : "v"(W[half][c / 2]), "v"(e));
        else
          asm("v_fmac_f64_dpp %0, %8, %9 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %1, %8, %9 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %2, %8, %9 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %3, %8, %9 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %4, %8, %9 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %5, %8, %9 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %6, %8, %9 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
              "v_fmac_f64_dpp %7, %8, %9 row_newbcast:15 row_mask:0xf bank_mask:0xf"
              : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
              : "v"(W[half][c / 2]), "v"(e));
      }
    }
  }
  const double base = ma + mb;
#pragma unroll
  for (int t = 0; t < M; ++t) S.wr(dsts[t], LINEAR ? acc[t] : base + Mt::log(acc[t]));
  return bs + NB + long(na) * NB * M * 2;
}

// Outer sum of eight float sums on the matrix cores. One 4x4x1 instruction multiplies, in every
// group of four lanes, four values of matrix A by four values of matrix B and accumulates the 16
// products; with the A-broadcast controls (cbsz = 4, abid = b) all sixteen groups take A from
// the four lanes of group b. So a vector register loaded with 64 consecutive weights (lane
// 4*b + i holds the weight of sum i for product b) serves sixteen products, B is simply every
// lane's own product exp(a_r - ma) * exp(b_c - mb), and accumulator register i of a lane ends up
// with sum i of that lane's sample: no data crosses lanes outside the instruction itself.
// The weights arrive through ordinary coalesced vector loads, requested before the operands.
typedef float float4v __attribute__((ext_vector_type(4)));

// Step K of the chain: both accumulators take product e_K, and the multiply that forms e_(K+2)
// sits between the two matrix instructions. One assembly statement per step keeps the two
// accumulator chains interleaved: left to the compiler they run one after the other, with every
// product held in a register in between (64 registers for an 8x8 region) and a stall between each
// pair of dependent instructions. Spacing rules, measured on gfx950 with a known-answer kernel:
// a matrix instruction that reads a register which a vector instruction has just written needs
// wait states in between and the hardware does not provide them (wrong results with none, and now
// and then with only another matrix instruction in between), hence products are formed two
// steps ahead and the first statement opens with s_nop; a matrix instruction may follow the one
// it accumulates onto after one independent matrix instruction; vector instructions that read a
// matrix result are held back by the hardware.
template <int K, int KEND, int NB>
struct MatrixSteps {
  // e: product of this step, e1: product of the next step (made one step ago, used one step from now).
  static __device__ __forceinline__ void run(const float* ea, const float* eb, const float (*A)[2], float4v& d0, float4v& d1, float e,
                                             float e1) {
    static_assert(K != 0 || KEND > 2, "the first step of a chain is the one that writes the accumulators whole");
    if constexpr (K + 2 < KEND) {
      float e2;
      if constexpr (K == 0) {
        // The two wait states in front separate the first matrix instruction from the vector instructions
        // that made its operands. The first step adds onto the constant 0, so the accumulators need no clearing.
        asm volatile(
            "s_nop 1\n\t"
            "v_mfma_f32_4x4x1_16b_f32 %0, %3, %5, 0 cbsz:4 abid:%8\n\t"
            "v_mul_f32 %2, %6, %7\n\t"
            "v_mfma_f32_4x4x1_16b_f32 %1, %4, %5, 0 cbsz:4 abid:%8"
            : "=&v"(d0), "=&v"(d1), "=&v"(e2)
            : "v"(A[K / 16][0]), "v"(A[K / 16][1]), "v"(e), "v"(ea[(K + 2) / NB]), "v"(eb[(K + 2) % NB]), "n"(K % 16), "v"(e1));
      } else {
        // No operand of this statement was written by the statement before it (the product comes from two
        // statements back), so the compiler has no reason to put wait states in between.
        asm volatile(
            "v_mfma_f32_4x4x1_16b_f32 %0, %3, %5, %0 cbsz:4 abid:%8\n\t"
            "v_mul_f32 %2, %6, %7\n\t"
            "v_mfma_f32_4x4x1_16b_f32 %1, %4, %5, %1 cbsz:4 abid:%8"
            : "+v"(d0), "+v"(d1), "=&v"(e2)
            : "v"(A[K / 16][0]), "v"(A[K / 16][1]), "v"(e), "v"(ea[(K + 2) / NB]), "v"(eb[(K + 2) % NB]), "n"(K % 16));
      }
      MatrixSteps<K + 1, KEND, NB>::run(ea, eb, A, d0, d1, e1, e2);
    } else {
      asm volatile(
          "v_mfma_f32_4x4x1_16b_f32 %0, %2, %4, %0 cbsz:4 abid:%5\n\t"
          "v_mfma_f32_4x4x1_16b_f32 %1, %3, %4, %1 cbsz:4 abid:%5"
          : "+v"(d0), "+v"(d1)
          : "v"(A[K / 16][0]), "v"(A[K / 16][1]), "v"(e), "n"(K % 16));
      if constexpr (K + 1 < KEND) MatrixSteps<K + 1, KEND, NB>::run(ea, eb, A, d0, d1, e1, e1);
    }
  }
};

// Reads / writes the N slots of a list whose slot numbers sit at head positions pos .. pos+N-1. tier: 0 all in
// LDS, 1 all in the spill tier, 2 either (select-the-base access). run: the slots are consecutive, so only the
// first number is read from the head and the others are constant offsets from its address.
template <int N, bool SPILL>
__device__ __forceinline__ void readList(const Slots<float, SPILL>& S, const Head& h, int pos, uint32_t tier, bool run, float* out) {
  if (run) {
    const uint32_t first = h.word(pos);
    if (!SPILL || tier == 0) {
#pragma unroll
      for (int j = 0; j < N; ++j) out[j] = S.rdLds(first + j);
    } else if (tier == 1) {
#pragma unroll
      for (int j = 0; j < N; ++j) out[j] = S.rdSpill(first + j);
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) out[j] = S.rd(first + j);
    }
  } else if (!SPILL || tier == 0) {
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = S.rdLds(h.word(pos + j));
  } else if (tier == 1) {
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = S.rdSpill(h.word(pos + j));
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) out[j] = S.rd(h.word(pos + j));
  }
}
template <int N, bool SPILL>
__device__ __forceinline__ void writeList(const Slots<float, SPILL>& S, const Head& h, int pos, uint32_t tier, bool run, const float* v) {
  if (run) {
    const uint32_t first = h.word(pos);
    if (!SPILL || tier == 0) {
#pragma unroll
      for (int j = 0; j < N; ++j) S.wrLds(first + j, v[j]);
    } else if (tier == 1) {
#pragma unroll
      for (int j = 0; j < N; ++j) S.wrSpill(first + j, v[j]);
    } else {
#pragma unroll
      for (int j = 0; j < N; ++j) S.wr(first + j, v[j]);
    }
  } else if (!SPILL || tier == 0) {
#pragma unroll
    for (int j = 0; j < N; ++j) S.wrLds(h.word(pos + j), v[j]);
  } else if (tier == 1) {
#pragma unroll
    for (int j = 0; j < N; ++j) S.wrSpill(h.word(pos + j), v[j]);
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) S.wr(h.word(pos + j), v[j]);
  }
}

// The matrix chain over the products ea[r] * eb[c] and what follows it: results as log2 values (base + log2 of
// each sum), or as a scaled vector, acc_t / max(acc) with base + log2(max) in the scale slot. dstPos / scalePos
// are the head positions of the eight destinations and of the scale slot.
template <bool LOG2, bool SPILL, int NA, int NB>
__device__ __forceinline__ void matrixChainAndStore(const float* ea, const float* eb, const float (*A)[2], float base, bool outScaled,
                                                    const Head& h, int dstPos, int scalePos, uint32_t tierD, bool dstRun,
                                                    const Slots<float, SPILL>& S) {
  typedef Math<float, LOG2> Mt;
  constexpr int M = 8, K = NA * NB;
  float4v d0, d1;   // written whole by the chain's first step
  SPN_PRIO_CHAIN();
  MatrixSteps<0, K, NB>::run(ea, eb, A, d0, d1, ea[0] * eb[0], ea[1 / NB] * eb[1 % NB]);
  SPN_PRIO_LATENCY();
  float res[M];
  if (outScaled) {
    // acc_t / max(acc) and one logarithm for the whole vector. All-zero accumulators (impossible evidence) give
    // zeros and a scale of -inf; the floor under the maximum only keeps the reciprocal finite.
    float m = rmax(rmax(rmax(d0[0], d0[1]), rmax(d0[2], d0[3])), rmax(rmax(d1[0], d1[1]), rmax(d1[2], d1[3])));
    const float inv = __builtin_amdgcn_rcpf(rmax(m, 0x1p-100f));
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      res[t] = d0[t] * inv;
      res[4 + t] = d1[t] * inv;
    }
    S.wr(h.word(scalePos), base + Mt::log(m));
  } else {
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      res[t] = base + Mt::log(d0[t]);
      res[4 + t] = base + Mt::log(d1[t]);
    }
  }
  writeList<M>(S, h, dstPos, tierD, dstRun, res);
}

template <bool LOG2, bool SPILL, bool TIERED, int NA, int NB>
__device__ __forceinline__ code_ptr outerSumMatrix(code_ptr ip, const Head& h, const float* wGlobal, const Slots<float, SPILL>& S) {
  typedef Math<float, LOG2> Mt;
  constexpr int M = 8, K = NA * NB, GROUPS = K / 16;
  // Positions in the head: length, opcode, M and format, then the slot lists and the three scale slots.
  constexpr int DST = 3, AS = DST + M, BS = AS + NA, SCALES = BS + NB;
  static_assert(SCALES + 3 <= Head::WORDS, "the slot lists must lie within the prefetched head");
  float A[GROUPS][2];
  const float* wl = wGlobal + (threadIdx.x & 63u);
#pragma unroll
  for (int g = 0; g < GROUPS; ++g) {
    A[g][0] = wl[g * 128];
    A[g][1] = wl[g * 128 + 64];
  }
  const uint32_t w0 = h.word(1), w1 = h.word(2);
  const bool aScaled = (w0 >> 30) & 1u, bScaled = (w0 >> 31) & 1u, outScaled = (w1 >> 8) & 1u;
  float ea[NA], eb[NB];
  // Flagged instructions: the tier bits say per slot list where it lives (valid when exactly the short pool is
  // in LDS), so a list is read with LDS instructions or with scalar-base global loads; mixed lists and other
  // LDS splits take the select-the-base form. A list that is a run of consecutive slots (bits 9-11 of the second
  // word) is addressed from its first slot with constant offsets: one lane read and one address for the list.
  const uint32_t tierA = TIERED ? (w0 >> 24) & 3u : 2u, tierB = TIERED ? (w0 >> 26) & 3u : 2u, tierD = TIERED ? (w0 >> 28) & 3u : 2u;
  readList<NA>(S, h, AS, tierA, (w1 >> 9) & 1u, ea);
  readList<NB>(S, h, BS, tierB, (w1 >> 10) & 1u, eb);
  // A scaled list already holds exp2(value - max) and brings max along in its scale slot; a list of log2
  // values is shifted by its maximum and exponentiated here. All slots are read before any is written.
  float base = 0.f;
  if (aScaled) {
    base += S.rd(h.word(SCALES + 1));
  } else {
    float ma = -__builtin_huge_valf();
#pragma unroll
    for (int r = 0; r < NA; ++r) ma = rmax(ma, ea[r]);
    ma = rmax(ma, Mt::lowest());
#pragma unroll
    for (int r = 0; r < NA; ++r) ea[r] = Mt::exp(ea[r] - ma);
    base += ma;
  }
  if (bScaled) {
    base += S.rd(h.word(SCALES + 2));
  } else {
    float mb = -__builtin_huge_valf();
#pragma unroll
    for (int c = 0; c < NB; ++c) mb = rmax(mb, eb[c]);
    mb = rmax(mb, Mt::lowest());
#pragma unroll
    for (int c = 0; c < NB; ++c) eb[c] = Mt::exp(eb[c] - mb);
    base += mb;
  }
  matrixChainAndStore<LOG2, SPILL, NA, NB>(ea, eb, A, base, outScaled, h, DST, SCALES, tierD, (w1 >> 11) & 1u, S);
  return ip + 2 + M + NA + NB + 3 + K * M;
}

// The operand counts the program builder emits the matrix form for (matrixFormShape in interp_program.cpp).
template <bool LOG2, bool SPILL, bool TIERED>
__device__ __forceinline__ code_ptr outerSumMatrixAny(code_ptr ip, const Head& h, int na, int nb, const float* wGlobal, const Slots<float, SPILL>& S) {
  if (na == 8 && nb == 8) return outerSumMatrix<LOG2, SPILL, TIERED, 8, 8>(ip, h, wGlobal, S);
  if (na == 4 && nb == 4) return outerSumMatrix<LOG2, SPILL, TIERED, 4, 4>(ip, h, wGlobal, S);
  if (na == 4 && nb == 8) return outerSumMatrix<LOG2, SPILL, TIERED, 4, 8>(ip, h, wGlobal, S);
  if (na == 8 && nb == 4) return outerSumMatrix<LOG2, SPILL, TIERED, 8, 4>(ip, h, wGlobal, S);
  if (na == 2 && nb == 8) return outerSumMatrix<LOG2, SPILL, TIERED, 2, 8>(ip, h, wGlobal, S);
  return outerSumMatrix<LOG2, SPILL, TIERED, 8, 2>(ip, h, wGlobal, S);
}

template <typename R, bool LOG2, bool SPILL, int M, bool LINEAR = false>
__device__ __forceinline__ code_ptr outerSumNB(code_ptr ip, int na, int nb, const Slots<R, SPILL>& S) {
  if (nb == 8) return outerSum<R, LOG2, SPILL, M, 8, LINEAR>(ip, na, S);
  if (nb == 4) return outerSum<R, LOG2, SPILL, M, 4, LINEAR>(ip, na, S);
  if (nb == 16) return outerSum<R, LOG2, SPILL, M, 16, LINEAR>(ip, na, S);
  return outerSum<R, LOG2, SPILL, M, 2, LINEAR>(ip, na, S);
}

// The operand vectors of a leaf region: NA + NB products of G Gaussian leaves, the first NA over the features
// x[0..G), the others over x[G..2G); constants (mean, shift, den per leaf) at ip[rec...]. Returns exp2(product -
// max) per list in ea / eb and the sum of the two maxima.
template <bool LOG2, int NA, int NB, int G, bool MARGINAL, typename R = float>
__device__ __forceinline__ R leafOperands(code_ptr ip, long rec, const R* x, R* ea, R* eb) {
  typedef Math<R, LOG2> Mt;
  constexpr int RW = sizeof(R) / 4;
  R e[NA + NB];
#pragma unroll
  for (int i = 0; i < NA + NB; ++i) {
    R acc = R(0);
#pragma unroll
    for (int j = 0; j < G; ++j) {
      const long at = rec + (i * G + j) * 3 * RW;
      const R xv = x[(i < NA ? 0 : G) + j];
      const R d = xv - constAt<R>(ip, at);
      R v = rfma(d, d, constAt<R>(ip, at + RW)) * constAt<R>(ip, at + 2 * RW);
      if (MARGINAL) v = (xv != xv) ? R(0) : v;
      acc += v;
    }
    e[i] = acc;
  }
  // The maxima start from the lowest finite value, which keeps them finite when every product is impossible.
  R ma = Mt::lowest(), mb = Mt::lowest();
#pragma unroll
  for (int r = 0; r < NA; ++r) ma = rmax(ma, e[r]);
#pragma unroll
  for (int c = 0; c < NB; ++c) mb = rmax(mb, e[NA + c]);
#pragma unroll
  for (int r = 0; r < NA; ++r) ea[r] = Mt::exp(e[r] - ma);
#pragma unroll
  for (int c = 0; c < NB; ++c) eb[c] = Mt::exp(e[NA + c] - mb);
  return ma + mb;
}

// Where the fused leaf instructions take their feature values from: staged slots (LDS, spill tier or either,
// as the tier says) or, when the program does not stage features, the columns of the sample's input row.
struct FeatureSource {
  const void* in;
  uint32_t type;
  unsigned long long row;
};
// Features held in registers for the whole tile (FEAT_REGISTER programs: the feature fields are register numbers). Always
// handed down as a reference to the kernel's own array and indexed directly, so that the array stays in registers.
typedef float FeatureRegs[INTERP_FEATURE_REGISTERS];
template <int COUNT, bool STAGED, bool SPILL>
__device__ __forceinline__ void readLeafFeatures(const Slots<float, SPILL>& S, const Head& h, int pos, uint32_t tier, const FeatureSource& fs,
                                                 bool useRegs, const FeatureRegs& regs, float* x) {
  if (!STAGED) {
#pragma unroll
    for (int j = 0; j < COUNT; ++j) x[j] = useRegs ? regs[h.word(pos + j) % INTERP_FEATURE_REGISTERS] : featureValue<float>(fs.in, fs.type, fs.row + h.word(pos + j));
  } else if (!SPILL || tier == 0) {
#pragma unroll
    for (int j = 0; j < COUNT; ++j) x[j] = S.rdLds(h.word(pos + j));
  } else if (tier == 1) {
#pragma unroll
    for (int j = 0; j < COUNT; ++j) x[j] = S.rdSpill(h.word(pos + j));
  } else {
#pragma unroll
    for (int j = 0; j < COUNT; ++j) x[j] = S.rd(h.word(pos + j));
  }
}

// OP_LEAFMM: the operand lists are products of G Gaussian leaves, all products of a list over the same G features.
// Weights, features and leaf constants are requested together; the products stay in registers.
template <bool LOG2, bool SPILL, bool TIERED, bool STAGED, int NA, int NB, int G, bool MARGINAL>
__device__ __forceinline__ code_ptr leafRegionMatrix(code_ptr ip, const Head& h, const float* wGlobal, const FeatureSource& fs,
                                                  bool useRegs, const FeatureRegs& regs, const Slots<float, SPILL>& S) {
  constexpr int M = 8, K = NA * NB, GROUPS = K / 16;
  // Head: length, opcode, format, eight destinations, the scale slot, 2 G feature slots. ip points at the opcode.
  constexpr int DST = 3, SCALE = DST + M, FEAT = SCALE + 1, REC = FEAT + 2 * G - 1;  // REC: offset of the constants from ip
  float A[GROUPS][2];
  const float* wl = wGlobal + (threadIdx.x & 63u);
#pragma unroll
  for (int g = 0; g < GROUPS; ++g) {
    A[g][0] = wl[g * 128];
    A[g][1] = wl[g * 128 + 64];
  }
  const uint32_t w0 = h.word(1), w1 = h.word(2);
  const uint32_t tierD = TIERED ? (w0 >> 28) & 3u : 2u, tierF = TIERED ? (w1 >> 16) & 3u : 2u;
  float x[2 * G];
  readLeafFeatures<2 * G, STAGED>(S, h, FEAT, tierF, fs, useRegs, regs, x);
  float ea[NA], eb[NB];
  const float base = leafOperands<LOG2, NA, NB, G, MARGINAL>(ip, REC, x, ea, eb);
  matrixChainAndStore<LOG2, SPILL, NA, NB>(ea, eb, A, base, (w1 >> 8) & 1u, h, DST, SCALE, tierD, (w1 >> 11) & 1u, S);
  return ip + 2 + M + 1 + 2 * G + (NA + NB) * G * 3 + K * M;
}
template <bool LOG2, bool SPILL, bool TIERED, bool STAGED, int NA, int NB>
__device__ __forceinline__ code_ptr leafRegionMatrixG(code_ptr ip, const Head& h, uint32_t leaves, bool marginal, const float* wGlobal,
                                                       const FeatureSource& fs, bool useRegs, const FeatureRegs& regs, const Slots<float, SPILL>& S) {
  if (!marginal) {
    if (leaves == 2) return leafRegionMatrix<LOG2, SPILL, TIERED, STAGED, NA, NB, 2, false>(ip, h, wGlobal, fs, useRegs, regs, S);
    if (leaves == 1) return leafRegionMatrix<LOG2, SPILL, TIERED, STAGED, NA, NB, 1, false>(ip, h, wGlobal, fs, useRegs, regs, S);
    return leafRegionMatrix<LOG2, SPILL, TIERED, STAGED, NA, NB, 4, false>(ip, h, wGlobal, fs, useRegs, regs, S);
  }
  if (leaves == 2) return leafRegionMatrix<LOG2, SPILL, TIERED, STAGED, NA, NB, 2, true>(ip, h, wGlobal, fs, useRegs, regs, S);
  if (leaves == 1) return leafRegionMatrix<LOG2, SPILL, TIERED, STAGED, NA, NB, 1, true>(ip, h, wGlobal, fs, useRegs, regs, S);
  return leafRegionMatrix<LOG2, SPILL, TIERED, STAGED, NA, NB, 4, true>(ip, h, wGlobal, fs, useRegs, regs, S);
}

// The matrix chain with the result left as it is: the linear sums, at most 1 each. For vectors that stay inside one
// instruction; the program builder fuses sums only where the weights keep the largest entry of such a vector above 2^-90.
template <int NA, int NB>
__device__ __forceinline__ void rawChain(const float* ea, const float* eb, const float (*A)[2], float* v) {
  float4v d0, d1;   // written whole by the chain's first step
  SPN_PRIO_CHAIN();
  MatrixSteps<0, NA * NB, NB>::run(ea, eb, A, d0, d1, ea[0] * eb[0], ea[1 / NB] * eb[1 % NB]);
  SPN_PRIO_LATENCY();
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    v[t] = d0[t];
    v[4 + t] = d1[t];
  }
}

// OP_LEAFPAIRMM: an 8x8 outer sum whose operand lists are the result vectors of two leaf regions (N x N products
// of G Gaussian leaves each, eight sums each; N = 4 is what the program builder emits). The two vectors stay in registers as they are; all weights,
// features and constants of the three sums are requested at the start.
template <bool LOG2, bool SPILL, bool TIERED, bool STAGED, int N, int G, bool MARGINAL>
__device__ __forceinline__ code_ptr leafPairMatrix(code_ptr ip, const Head& h, const float* wGlobal, const FeatureSource& fs,
                                                bool useRegs, const FeatureRegs& regs, const Slots<float, SPILL>& S) {
  constexpr int M = 8, KL = N * N, GL = KL / 16;
  // Head: length, opcode, format, eight destinations, the scale slot, 4 G feature slots. ip points at the opcode.
  constexpr int DST = 3, SCALE = DST + M, FEAT = SCALE + 1, REC = FEAT + 4 * G - 1, RECS = 2 * N * G * 3;
  float A1[GL][2], A2[GL][2], AT[4][2];
  const float* wl = wGlobal + (threadIdx.x & 63u);
#pragma unroll
  for (int g = 0; g < GL; ++g) {
    A1[g][0] = wl[g * 128];
    A1[g][1] = wl[g * 128 + 64];
  }
#pragma unroll
  for (int g = 0; g < GL; ++g) {
    A2[g][0] = wl[KL * M + g * 128];
    A2[g][1] = wl[KL * M + g * 128 + 64];
  }
  const uint32_t w0 = h.word(1), w1 = h.word(2);
  const uint32_t tierD = TIERED ? (w0 >> 28) & 3u : 2u, tierF = TIERED ? (w1 >> 16) & 3u : 2u;
  float x[4 * G];
  readLeafFeatures<4 * G, STAGED>(S, h, FEAT, tierF, fs, useRegs, regs, x);
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    AT[g][0] = wl[2 * KL * M + g * 128];
    AT[g][1] = wl[2 * KL * M + g * 128 + 64];
  }
  float va[M], vb[M], base = 0.f;
#pragma unroll
  for (int side = 0; side < 2; ++side) {
    float ea[N], eb[N];
    const float maxima = leafOperands<LOG2, N, N, G, MARGINAL>(ip, REC + side * RECS, x + side * 2 * G, ea, eb);
    base = side == 0 ? maxima : base + maxima;   // not 0 + maxima: that is an instruction (it turns -0 into +0)
    rawChain<N, N>(ea, eb, side == 0 ? A1 : A2, side == 0 ? va : vb);
  }
  matrixChainAndStore<LOG2, SPILL, 8, 8>(va, vb, AT, base, (w1 >> 8) & 1u, h, DST, SCALE, tierD, (w1 >> 11) & 1u, S);
  return ip + 2 + M + 1 + 4 * G + 2 * RECS + 2 * KL * M + 64 * M;
}
template <bool LOG2, bool SPILL, bool TIERED, bool STAGED, int N>
__device__ __forceinline__ code_ptr leafPairMatrixG(code_ptr ip, const Head& h, uint32_t leaves, bool marginal, const float* wGlobal,
                                                     const FeatureSource& fs, bool useRegs, const FeatureRegs& regs, const Slots<float, SPILL>& S) {
  if (!marginal) {
    if (leaves == 2) return leafPairMatrix<LOG2, SPILL, TIERED, STAGED, N, 2, false>(ip, h, wGlobal, fs, useRegs, regs, S);
    if (leaves == 1) return leafPairMatrix<LOG2, SPILL, TIERED, STAGED, N, 1, false>(ip, h, wGlobal, fs, useRegs, regs, S);
    return leafPairMatrix<LOG2, SPILL, TIERED, STAGED, N, 4, false>(ip, h, wGlobal, fs, useRegs, regs, S);
  }
  if (leaves == 2) return leafPairMatrix<LOG2, SPILL, TIERED, STAGED, N, 2, true>(ip, h, wGlobal, fs, useRegs, regs, S);
  if (leaves == 1) return leafPairMatrix<LOG2, SPILL, TIERED, STAGED, N, 1, true>(ip, h, wGlobal, fs, useRegs, regs, S);
  return leafPairMatrix<LOG2, SPILL, TIERED, STAGED, N, 4, true>(ip, h, wGlobal, fs, useRegs, regs, S);
}

// OP_LEAFQUADMM: two OP_LEAFPAIRMM over 4x4 leaf regions and the 8x8 outer sum over their two result vectors, i.e.
// seven sums over four leaf regions with every intermediate vector in registers. Weights are requested a stage
// ahead of the chain that uses them: those of the second pair while the first pair's 8x8 chain runs, those of
// the final sum while the second pair's runs.
template <bool LOG2, bool SPILL, bool TIERED, bool STAGED, int G, bool MARGINAL>
__device__ __forceinline__ code_ptr leafQuadMatrix(code_ptr ip, const Head& h, const float* wGlobal, const FeatureSource& fs,
                                                bool useRegs, const FeatureRegs& regs, const Slots<float, SPILL>& S) {
  constexpr int N = 4, M = 8;
  // Head: length, opcode, format, eight destinations, the scale slot, 8 G feature slots. ip points at the opcode.
  constexpr int DST = 3, SCALE = DST + M, FEAT = SCALE + 1, REC = FEAT + 8 * G - 1, RECS = 2 * N * G * 3;
  constexpr int LEAFW = N * N * M, PAIRW = 2 * LEAFW + 64 * M;  // weights: leaf, leaf, 8x8 per pair, then the final 8x8
  const float* wl = wGlobal + (threadIdx.x & 63u);
  auto loadLeaf = [&](int at, float (*A)[2]) {
    A[0][0] = wl[at];
    A[0][1] = wl[at + 64];
  };
  auto loadTop = [&](int at, float (*A)[2]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      A[g][0] = wl[at + g * 128];
      A[g][1] = wl[at + g * 128 + 64];
    }
  };
  float AL[4][1][2], AT[2][4][2], ATOP[4][2];
  loadLeaf(0, AL[0]);
  loadLeaf(LEAFW, AL[1]);
  const uint32_t w0 = h.word(1), w1 = h.word(2);
  const uint32_t tierD = TIERED ? (w0 >> 28) & 3u : 2u, tierF = TIERED ? (w1 >> 16) & 3u : 2u;
  float x[8 * G];
  readLeafFeatures<8 * G, STAGED>(S, h, FEAT, tierF, fs, useRegs, regs, x);
  loadTop(2 * LEAFW, AT[0]);
  float pv[2][M], base = 0.f;
#pragma unroll
  for (int pair = 0; pair < 2; ++pair) {
    float v[2][M];
#pragma unroll
    for (int side = 0; side < 2; ++side) {
      const int region = 2 * pair + side;
      float ea[N], eb[N];
      const float maxima = leafOperands<LOG2, N, N, G, MARGINAL>(ip, REC + region * RECS, x + region * 2 * G, ea, eb);
      base = region == 0 ? maxima : base + maxima;   // not 0 + maxima: that is an instruction (it turns -0 into +0)
      rawChain<N, N>(ea, eb, AL[region], v[side]);
    }
    if (pair == 0) {
      loadLeaf(PAIRW, AL[2]);
      loadLeaf(PAIRW + LEAFW, AL[3]);
      loadTop(PAIRW + 2 * LEAFW, AT[1]);
    } else {
      loadTop(2 * PAIRW, ATOP);
    }
    rawChain<8, 8>(v[0], v[1], AT[pair], pv[pair]);
  }
  matrixChainAndStore<LOG2, SPILL, 8, 8>(pv[0], pv[1], ATOP, base, (w1 >> 8) & 1u, h, DST, SCALE, tierD, (w1 >> 11) & 1u, S);
  return ip + 2 + M + 1 + 8 * G + 4 * RECS + 2 * PAIRW + 64 * M;
}

// ---- The fused leaf instructions in double precision ----
// No matrix instruction helps here (the double ones run at the rate of the vector unit and want four samples per group
// of lanes); what the matrix form buys the float kernels, weights that reach the arithmetic without scalar loads and
// scalar operands, the double kernels get from the cross-lane operand of v_fmac_f64 (outerSumLaneWeights above): the
// weights lie product-major in the stream, eight sums per product, so a register pair loaded with sixteen consecutive
// weights serves the eight sums of two products. Result vectors inside an instruction stay linear and unscaled, as in the
// float forms; an instruction's own result is written as log2 values (doubles have the range for the products of a
// whole instruction, and the consumer is an ordinary outer sum).

// The sixteen multiply-adds of one lane vector: the eight sums of two products.
__device__ __forceinline__ void laneVector(double* acc, double w, double e0, double e1) {
  asm("v_fmac_f64_dpp %0, %8, %9 row_newbcast:0 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %1, %8, %9 row_newbcast:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %2, %8, %9 row_newbcast:2 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %3, %8, %9 row_newbcast:3 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %4, %8, %9 row_newbcast:4 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %5, %8, %9 row_newbcast:5 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %6, %8, %9 row_newbcast:6 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %7, %8, %9 row_newbcast:7 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %0, %8, %10 row_newbcast:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %1, %8, %10 row_newbcast:9 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %2, %8, %10 row_newbcast:10 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %3, %8, %10 row_newbcast:11 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %4, %8, %10 row_newbcast:12 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %5, %8, %10 row_newbcast:13 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %6, %8, %10 row_newbcast:14 row_mask:0xf bank_mask:0xf\n\t"
      "v_fmac_f64_dpp %7, %8, %10 row_newbcast:15 row_mask:0xf bank_mask:0xf"
      : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]), "+v"(acc[4]), "+v"(acc[5]), "+v"(acc[6]), "+v"(acc[7])
      : "v"(w), "v"(e0), "v"(e1));
}

// acc[t] = sum over products k = r NB + c of w[k][t] ea[r] eb[c]. A loop over the operand rows, two per round with the
// vectors of the row after next requested meanwhile: unrolled over all products the chain of an 8x8 sum alone is 4.6 KiB of
// instructions that every wavefront would stream through the instruction cache once per use.
template <int NA, int NB>
__device__ __forceinline__ void laneChain(const double* ea, const double* eb, const StreamDouble* wGlobal, double* acc) {
  constexpr int V = NB / 2;  // vectors of sixteen weights per operand row
  static_assert(NA % 2 == 0, "operand rows are taken two at a time");
  const StreamDouble* wl = wGlobal + (threadIdx.x & 15u);
  double W[2][V];
#pragma unroll
  for (int v = 0; v < V; ++v) W[0][v] = wl[v * 16].value;
#pragma unroll
  for (int t = 0; t < 8; ++t) acc[t] = 0.0;
  SPN_PRIO_CHAIN();
#pragma unroll 1
  for (int r = 0; r < NA; r += 2) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int row = r + half;
      // the next row's weights (past the last row: the words that follow, read and not used)
#pragma unroll
      for (int v = 0; v < V; ++v) W[half ^ 1][v] = wl[((row + 1) * V + v) * 16].value;
      const double ear = ea[row];
#pragma unroll
      for (int v = 0; v < V; ++v) laneVector(acc, W[half][v], ear * eb[2 * v], ear * eb[2 * v + 1]);
    }
  }
  SPN_PRIO_LATENCY();
}

// One leaf region of N x N products of G Gaussian leaves: its eight sums, linear and unscaled, in v; returns the sum of the
// two operand maxima (log2). rec: offset of its constants from ip (in words), w: its weights.
template <bool LOG2, int N, int G, bool MARGINAL>
__device__ __forceinline__ double leafRegionLanes(code_ptr ip, long rec, const double* x, const StreamDouble* w, double* v) {
  double ea[N], eb[N];
  const double base = leafOperands<LOG2, N, N, G, MARGINAL, double>(ip, rec, x, ea, eb);
  laneChain<N, N>(ea, eb, w, v);
  return base;
}

template <int COUNT, bool SPILL>
__device__ __forceinline__ void readLeafFeaturesDouble(const Slots<double, SPILL>& S, const Head& h, int pos, bool staged, const FeatureSource& fs, double* x) {
  if (staged) {
#pragma unroll
    for (int j = 0; j < COUNT; ++j) x[j] = S.rd(h.word(pos + j));
  } else {
#pragma unroll
    for (int j = 0; j < COUNT; ++j) x[j] = featureValue<double>(fs.in, fs.type, fs.row + h.word(pos + j));
  }
}

template <bool LOG2, bool SPILL>
__device__ __forceinline__ void storeLogVector(const Slots<double, SPILL>& S, const Head& h, int dstPos, double base, const double* acc) {
  typedef Math<double, LOG2> Mt;
#pragma unroll
  for (int t = 0; t < 8; ++t) S.wr(h.word(dstPos + t), base + Mt::log(acc[t]));
}

// OP_LEAFMM, OP_LEAFPAIRMM and OP_LEAFQUADMM of a double program: REGIONS = 1, 2 or 4 leaf regions of N x N products.
// Words: opcode, format, eight destinations, a scale field (unused), 2 G feature fields per region, the regions'
// constants, then the weights (product-major): one region: its own; a pair: region, region, the 8x8 sum over them;
// a quad: pair, pair, the 8x8 sum over the pairs.
template <bool LOG2, bool SPILL, int REGIONS, int N, int G, bool MARGINAL>
__device__ __forceinline__ code_ptr leafLanes(code_ptr ip, const Head& h, const uint32_t* words, bool staged, const FeatureSource& fs,
                                               const Slots<double, SPILL>& S) {
  constexpr int M = 8, DST = 3, FEAT = DST + M + 1, NF = 2 * G * REGIONS, REC = FEAT + NF - 1;  // REC: offset of the constants from ip
  constexpr int RECW = 2 * N * G * 3 * 2;                          // words of one region's constants
  constexpr int LEAFW = N * N * M, TOPW = 64 * M, PAIRW = 2 * LEAFW + TOPW;  // weights (doubles) of a region, an 8x8 sum, a pair
  const StreamDouble* w = reinterpret_cast<const StreamDouble*>(words + REC + REGIONS * RECW);  // `words`: ip's word in global memory
  double x[NF];
  readLeafFeaturesDouble<NF>(S, h, FEAT, staged, fs, x);
  double out[M], base = 0.0;
  if constexpr (REGIONS == 1) {
    base = leafRegionLanes<LOG2, N, G, MARGINAL>(ip, REC, x, w, out);
  } else if constexpr (REGIONS == 2) {
    double va[M], vb[M];
    base = leafRegionLanes<LOG2, N, G, MARGINAL>(ip, REC, x, w, va);
    base += leafRegionLanes<LOG2, N, G, MARGINAL>(ip, REC + RECW, x + 2 * G, w + LEAFW, vb);
    laneChain<8, 8>(va, vb, w + 2 * LEAFW, out);
  } else {
    double pv[2][M];
#pragma unroll
    for (int pair = 0; pair < 2; ++pair) {
      double va[M], vb[M];
      base += leafRegionLanes<LOG2, N, G, MARGINAL>(ip, REC + (2 * pair) * RECW, x + (2 * pair) * 2 * G, w + pair * PAIRW, va);
      base += leafRegionLanes<LOG2, N, G, MARGINAL>(ip, REC + (2 * pair + 1) * RECW, x + (2 * pair + 1) * 2 * G, w + pair * PAIRW + LEAFW, vb);
      laneChain<8, 8>(va, vb, w + pair * PAIRW + 2 * LEAFW, pv[pair]);
    }
    laneChain<8, 8>(pv[0], pv[1], w + 2 * PAIRW, out);
  }
  storeLogVector<LOG2>(S, h, DST, base, out);
  constexpr int WEIGHTS = REGIONS == 1 ? LEAFW : (REGIONS == 2 ? PAIRW : 2 * PAIRW + TOPW);
  return ip + REC + REGIONS * RECW + WEIGHTS * 2;
}

template <bool LOG2, bool SPILL, int REGIONS, int N>
__device__ __forceinline__ code_ptr leafLanesG(code_ptr ip, const Head& h, uint32_t leaves, bool marginal, const uint32_t* stream, bool staged,
                                                const FeatureSource& fs, const Slots<double, SPILL>& S) {
  if (!marginal) {
    if (leaves == 2) return leafLanes<LOG2, SPILL, REGIONS, N, 2, false>(ip, h, stream, staged, fs, S);
    if (leaves == 1 || REGIONS == 4) return leafLanes<LOG2, SPILL, REGIONS, N, 1, false>(ip, h, stream, staged, fs, S);
    return leafLanes<LOG2, SPILL, REGIONS, N, REGIONS == 4 ? 1 : 4, false>(ip, h, stream, staged, fs, S);
  }
  if (leaves == 2) return leafLanes<LOG2, SPILL, REGIONS, N, 2, true>(ip, h, stream, staged, fs, S);
  if (leaves == 1 || REGIONS == 4) return leafLanes<LOG2, SPILL, REGIONS, N, 1, true>(ip, h, stream, staged, fs, S);
  return leafLanes<LOG2, SPILL, REGIONS, N, REGIONS == 4 ? 1 : 4, true>(ip, h, stream, staged, fs, S);
}

// The three fused leaf instructions. STAGED: their feature fields are slots of staged values, else input columns.
template <bool LOG2, bool SPILL, bool TIERED, bool STAGED>
__device__ __forceinline__ code_ptr leafInstruction(uint32_t op, code_ptr ip, const Head& h, int na, int nb, bool marginal, code_ptr code0,
                                                    const uint32_t* codeGlobal, const FeatureSource& fs, bool useRegs, const FeatureRegs& regs, const Slots<float, SPILL>& S) {
  const uint32_t leaves = (h.word(2) >> 12) & 0xfu;
  const float* code = reinterpret_cast<const float*>(codeGlobal) + (ip - code0);
  if (op == OP_LEAFQUADMM) {
    // One or two leaves per product (the program builder emits no others). The weights follow the header words,
    // destinations, scale slot, 8 G feature fields and the constants of 32 products of G leaves.
    const float* wGlobal = code + (11 + 8 * leaves + 32 * leaves * 3);
    if (!marginal) {
      if (leaves == 2) return leafQuadMatrix<LOG2, SPILL, TIERED, STAGED, 2, false>(ip, h, wGlobal, fs, useRegs, regs, S);
      return leafQuadMatrix<LOG2, SPILL, TIERED, STAGED, 1, false>(ip, h, wGlobal, fs, useRegs, regs, S);
    }
    if (leaves == 2) return leafQuadMatrix<LOG2, SPILL, TIERED, STAGED, 2, true>(ip, h, wGlobal, fs, useRegs, regs, S);
    return leafQuadMatrix<LOG2, SPILL, TIERED, STAGED, 1, true>(ip, h, wGlobal, fs, useRegs, regs, S);
  }
  if (op == OP_LEAFPAIRMM) {
    // na: operand count per list of the two leaf regions. The weights follow the header words, destinations, scale slot,
    // 4 G feature fields and the constants of 4 na products of G leaves. Leaf regions of 4x4 products only: with 8x8
    // the three sets of weights and the operands of two long chains would cost the whole kernel a wavefront per SIMD
    // in registers; those stay single OP_LEAFMM instructions.
    const float* wGlobal = code + (11 + 4 * leaves + 4 * na * leaves * 3);
    return leafPairMatrixG<LOG2, SPILL, TIERED, STAGED, 4>(ip, h, leaves, marginal, wGlobal, fs, useRegs, regs, S);
  }
  // OP_LEAFMM: the weights start after the two header words, eight destinations, the scale slot, the feature fields and the leaf constants.
  const float* wGlobal = code + (11 + 2 * leaves + (na + nb) * leaves * 3);
  if (na == 4) return leafRegionMatrixG<LOG2, SPILL, TIERED, STAGED, 4, 4>(ip, h, leaves, marginal, wGlobal, fs, useRegs, regs, S);
  return leafRegionMatrixG<LOG2, SPILL, TIERED, STAGED, 8, 8>(ip, h, leaves, marginal, wGlobal, fs, useRegs, regs, S);
}

// n products of G Gaussian leaves each. The records are independent, so they are taken four at
// a time: all constants of a group arrive in a few wide scalar loads and all feature reads of a
// group are in flight together, instead of one dependent load chain per product.
template <typename R, bool SPILL, int G, bool stagedMode, bool MARGINAL, bool LINEAR = false>
__device__ __forceinline__ code_ptr prodBatch(code_ptr ip, int n, const Slots<R, SPILL>& S, const InterpLaunch& a, unsigned long long row,
                                              bool useRegs, const FeatureRegs& regs) {
  constexpr int RW = sizeof(R) / 4, LEAF = 1 + 3 * RW, REC = 1 + G * LEAF, P = 4;
  ip += 2;
  int done = 0;
  for (; done + P <= n; done += P, ip += P * REC) {
    R x[P][G];
#pragma unroll
    for (int q = 0; q < P; ++q)
#pragma unroll
      for (int j = 0; j < G; ++j) {
        const uint32_t fw = ip[q * REC + 1 + j * LEAF];
        x[q][j] = stagedMode ? S.rd(fw) : (useRegs ? R(regs[fw % INTERP_FEATURE_REGISTERS]) : featureValue<R>(a.in, a.featureType, row + fw));
      }
#pragma unroll
    for (int q = 0; q < P; ++q) {
      R acc = productStart<LINEAR, R>();
#pragma unroll
      for (int j = 0; j < G; ++j) {
        const long at = q * REC + 1 + j * LEAF + 1;
        R v = gaussLeaf<LINEAR>(x[q][j], constAt<R>(ip, at), constAt<R>(ip, at + RW), constAt<R>(ip, at + 2 * RW));
        if (MARGINAL && a.marginal) v = (x[q][j] != x[q][j]) ? productStart<LINEAR, R>() : v;
        acc = productJoin<LINEAR>(acc, v);
      }
      S.wr(ip[q * REC], acc);
    }
  }
  for (; done < n; ++done, ip += REC) {
    R acc = productStart<LINEAR, R>();
#pragma unroll
    for (int j = 0; j < G; ++j) {
      const uint32_t fw = ip[1 + j * LEAF];
      const R xv = stagedMode ? S.rd(fw) : (useRegs ? R(regs[fw % INTERP_FEATURE_REGISTERS]) : featureValue<R>(a.in, a.featureType, row + fw));
      R v = gaussLeaf<LINEAR>(xv, constAt<R>(ip, 2 + j * LEAF), constAt<R>(ip, 2 + j * LEAF + RW), constAt<R>(ip, 2 + j * LEAF + 2 * RW));
      if (MARGINAL && a.marginal) v = (xv != xv) ? productStart<LINEAR, R>() : v;
      acc = productJoin<LINEAR>(acc, v);
    }
    S.wr(ip[0], acc);
  }
  return ip;
}

// The same for staged features when the program's short pool is exactly what lives in LDS: the second word
// says in which tier the feature slots (FT) and the destinations (DT) live, 0 LDS or 1 spill tier, so every
// access is an LDS instruction or a global access from a scalar base instead of a selected generic address.
// GROUPED: the j-th leaves of the four records of a group read the same feature, which is then read once.
template <typename R, int G, bool MARGINAL, int FT, int DT, bool GROUPED>
__device__ __forceinline__ code_ptr prodBatchTiered(code_ptr ip, int n, const Slots<R, true>& S, const InterpLaunch& a) {
  constexpr int RW = sizeof(R) / 4, LEAF = 1 + 3 * RW, REC = 1 + G * LEAF, P = 4;
  ip += 2;
  int done = 0;
  for (; done + P <= n; done += P, ip += P * REC) {
    R x[P][G];
#pragma unroll
    for (int q = 0; q < (GROUPED ? 1 : P); ++q)
#pragma unroll
      for (int j = 0; j < G; ++j) {
        const uint32_t fw = ip[q * REC + 1 + j * LEAF];
        x[q][j] = FT == 0 ? S.rdLds(fw) : S.rdSpill(fw);
      }
#pragma unroll
    for (int q = 0; q < P; ++q) {
      R acc = R(0);
#pragma unroll
      for (int j = 0; j < G; ++j) {
        const long at = q * REC + 1 + j * LEAF + 1;
        const R xv = x[GROUPED ? 0 : q][j];
        const R d = xv - constAt<R>(ip, at);
        R v = rfma(d, d, constAt<R>(ip, at + RW)) * constAt<R>(ip, at + 2 * RW);
        if (MARGINAL) v = (xv != xv) ? R(0) : v;
        acc += v;
      }
      if (DT == 0) S.wrLds(ip[q * REC], acc);
      else S.wrSpill(ip[q * REC], acc);
    }
  }
  for (; done < n; ++done, ip += REC) {
    R acc = R(0);
#pragma unroll
    for (int j = 0; j < G; ++j) {
      const uint32_t fw = ip[1 + j * LEAF];
      const R xv = FT == 0 ? S.rdLds(fw) : S.rdSpill(fw);
      const R d = xv - constAt<R>(ip, 2 + j * LEAF);
      R v = rfma(d, d, constAt<R>(ip, 2 + j * LEAF + RW)) * constAt<R>(ip, 2 + j * LEAF + 2 * RW);
      if (MARGINAL) v = (xv != xv) ? R(0) : v;
      acc += v;
    }
    if (DT == 0) S.wrLds(ip[0], acc);
    else S.wrSpill(ip[0], acc);
  }
  return ip;
}
template <typename R, int G, bool MARGINAL, int FT, int DT>
__device__ __forceinline__ code_ptr prodBatchTieredG(code_ptr ip, int n, bool grouped, const Slots<R, true>& S, const InterpLaunch& a) {
  if (grouped) return prodBatchTiered<R, G, MARGINAL, FT, DT, true>(ip, n, S, a);
  return prodBatchTiered<R, G, MARGINAL, FT, DT, false>(ip, n, S, a);
}
template <typename R, int G, bool MARGINAL>
__device__ __forceinline__ code_ptr prodBatchTieredAny(code_ptr ip, int n, uint32_t flags, const Slots<R, true>& S, const InterpLaunch& a) {
  const uint32_t ft = (flags >> 8) & 3u, dt = (flags >> 10) & 3u;
  const bool grouped = (flags >> 12) & 1u;
  if (ft == 0 && dt == 0) return prodBatchTieredG<R, G, MARGINAL, 0, 0>(ip, n, grouped, S, a);
  if (ft == 0) return prodBatchTieredG<R, G, MARGINAL, 0, 1>(ip, n, grouped, S, a);
  if (dt == 0) return prodBatchTieredG<R, G, MARGINAL, 1, 0>(ip, n, grouped, S, a);
  return prodBatchTieredG<R, G, MARGINAL, 1, 1>(ip, n, grouped, S, a);
}

// Executes one instruction other than OP_END and returns the pointer to the next one.
template <typename R, bool LOG2, bool SPILL, bool TIERED, bool LINEAR>
__device__ __forceinline__ code_ptr execute(code_ptr ip, const Head& h, const Slots<R, SPILL>& S, const InterpLaunch& a,
                                            const R* __restrict__ tables, unsigned long long row, bool stagedMode, code_ptr code0,
                                            const uint32_t* codeGlobal, bool useRegs, const FeatureRegs& regs) {
  typedef Math<R, LOG2> Mt;
  constexpr int RW = sizeof(R) / 4;
  const uint32_t w0 = h.word(1), op = w0 & 0x7fu;
  if (op == OP_PROD) {
    const uint32_t dst = h.word(2);
    const int ns = int(h.word(3)), ng = int(h.word(4)), nt = int(h.word(5));
    ip += 5;
    R acc = productStart<LINEAR, R>();
#pragma unroll 4
    for (int j = 0; j < ns; ++j) acc = productJoin<LINEAR>(acc, S.rd(ip[j]));
    ip += ns;
#pragma unroll 2
    for (int j = 0; j < ng; ++j) {
      const uint32_t fw = ip[0];
      const R mean = constAt<R>(ip, 1), shift = constAt<R>(ip, 1 + RW), den = constAt<R>(ip, 1 + 2 * RW);
      ip += 1 + 3 * RW;
      const R x = stagedMode ? S.rd(fw) : (useRegs ? R(regs[fw % INTERP_FEATURE_REGISTERS]) : featureValue<R>(a.in, a.featureType, row + fw));
      R v = gaussLeaf<LINEAR>(x, mean, shift, den);
      if (a.marginal) v = (x != x) ? productStart<LINEAR, R>() : v;
      acc = productJoin<LINEAR>(acc, v);
    }
    for (int j = 0; j < nt; ++j) {
      const uint32_t fw = ip[0], off = ip[1], L = ip[2];
      ip += 3;
      const uint32_t idx = stagedMode ? uint32_t(S.rd(fw)) : featureIndex(a.in, a.featureType, row + fw, L, a.marginal);
      acc = productJoin<LINEAR>(acc, tables[off + idx]);
    }
    S.wr(dst, acc);
    return ip;
  }
  if (op == OP_PRODBATCH) {
    const int n = int(w0 >> 8);
    const uint32_t flags = h.word(2), leaves = flags & 0xffu;
    if constexpr (SPILL && TIERED && !LINEAR) {
      // Tier flags are valid (exactly the short pool is in LDS): no generic accesses unless a list is mixed.
      if (stagedMode && ((flags >> 8) & 3u) != 2u && ((flags >> 10) & 3u) != 2u && leaves != 3) {
        if (!a.marginal) {
          if (leaves == 2) return prodBatchTieredAny<R, 2, false>(ip, n, flags, S, a);
          if (leaves == 1) return prodBatchTieredAny<R, 1, false>(ip, n, flags, S, a);
          return prodBatchTieredAny<R, 4, false>(ip, n, flags, S, a);
        }
        if (leaves == 2) return prodBatchTieredAny<R, 2, true>(ip, n, flags, S, a);
        if (leaves == 1) return prodBatchTieredAny<R, 1, true>(ip, n, flags, S, a);
        return prodBatchTieredAny<R, 4, true>(ip, n, flags, S, a);
      }
    }
    // Staged features make the whole batch straight-line code; the direct form decides the input type per read.
    // Without marginal support (the common staged case) the NaN select is not compiled in at all.
    if (stagedMode && !a.marginal) {
      if (leaves == 2) return prodBatch<R, SPILL, 2, true, false, LINEAR>(ip, n, S, a, row, useRegs, regs);
      if (leaves == 1) return prodBatch<R, SPILL, 1, true, false, LINEAR>(ip, n, S, a, row, useRegs, regs);
      if (leaves == 4) return prodBatch<R, SPILL, 4, true, false, LINEAR>(ip, n, S, a, row, useRegs, regs);
      return prodBatch<R, SPILL, 3, true, false, LINEAR>(ip, n, S, a, row, useRegs, regs);
    }
    if (stagedMode) {
      if (leaves == 2) return prodBatch<R, SPILL, 2, true, true, LINEAR>(ip, n, S, a, row, useRegs, regs);
      if (leaves == 1) return prodBatch<R, SPILL, 1, true, true, LINEAR>(ip, n, S, a, row, useRegs, regs);
      if (leaves == 4) return prodBatch<R, SPILL, 4, true, true, LINEAR>(ip, n, S, a, row, useRegs, regs);
      return prodBatch<R, SPILL, 3, true, true, LINEAR>(ip, n, S, a, row, useRegs, regs);
    }
    if (leaves == 2) return prodBatch<R, SPILL, 2, false, true, LINEAR>(ip, n, S, a, row, useRegs, regs);
    if (leaves == 1) return prodBatch<R, SPILL, 1, false, true, LINEAR>(ip, n, S, a, row, useRegs, regs);
    if (leaves == 4) return prodBatch<R, SPILL, 4, false, true, LINEAR>(ip, n, S, a, row, useRegs, regs);
    return prodBatch<R, SPILL, 3, false, true, LINEAR>(ip, n, S, a, row, useRegs, regs);
  }
  if (op == OP_SUM) {
    const int k = int(w0 >> 8);
    const uint32_t dst = h.word(2);
    ip += 2;
    if constexpr (LINEAR) {
      R sum = R(0);
#pragma unroll 4
      for (int j = 0; j < k; ++j) sum = rfma(S.rd(ip[long(j) * (1 + RW)]), constAt<R>(ip, long(j) * (1 + RW) + 1), sum);
      S.wr(dst, sum);
      return ip + long(k) * (1 + RW);
    }
    if (k == 1) {
      S.wr(dst, S.rd(ip[0]) + constAt<R>(ip, 1));
      return ip + 1 + RW;
    }
    // Terms are taken in chunks (sixteen, eight or four), all reads of a chunk in flight together; the running sum is kept
    // relative to the running maximum and rescaled when a chunk raises it, so every term is read once.
    constexpr int C = sizeof(R) == 8 ? 4 : (LOG2 ? 16 : 8);  // fewer values in registers where they or the exponentials are large
    R ms = Mt::lowest(), acc = R(0);
    int j = 0;
    for (; j + C <= k; j += C) {
      R v[C];
#pragma unroll
      for (int q = 0; q < C; ++q) v[q] = S.rd(ip[long(j + q) * (1 + RW)]);
      R cm = v[0];
#pragma unroll
      for (int q = 1; q < C; ++q) cm = rmax(cm, v[q]);
      const R mn = rmax(ms, cm);
      acc *= Mt::exp(ms - mn);
      ms = mn;
#pragma unroll
      for (int q = 0; q < C; ++q) acc = rfma(Mt::exp(v[q] - ms), constAt<R>(ip, long(j + q) * (1 + RW) + 1), acc);
    }
    if (j < k) {
      R cm = R(-__builtin_huge_val());
#pragma unroll 4
      for (int q = j; q < k; ++q) cm = rmax(cm, S.rd(ip[long(q) * (1 + RW)]));
      const R mn = rmax(ms, cm);
      acc *= Mt::exp(ms - mn);
      ms = mn;
#pragma unroll 4
      for (int q = j; q < k; ++q) acc = rfma(Mt::exp(S.rd(ip[long(q) * (1 + RW)]) - ms), constAt<R>(ip, long(q) * (1 + RW) + 1), acc);
    }
    S.wr(dst, ms + Mt::log(acc));
    return ip + long(k) * (1 + RW);
  }
  if (op == OP_SUMLAYER) {
    const int k = int(w0 >> 8);
    const uint32_t m = h.word(2);
    if (m == 8) return sumLayer<R, LOG2, SPILL, 8, LINEAR>(ip, k, S);
    if (m == 4) return sumLayer<R, LOG2, SPILL, 4, LINEAR>(ip, k, S);
    return sumLayer<R, LOG2, SPILL, 2, LINEAR>(ip, k, S);
  }
  const int na = int((w0 >> 8) & 0xffu), nb = int((w0 >> 16) & 0xffu);
  if constexpr (sizeof(R) == 4 && !LINEAR) {
    if (op == OP_LEAFQUADMM || op == OP_LEAFPAIRMM || op == OP_LEAFMM) {
      const FeatureSource fs{a.in, a.featureType, row};
      if (stagedMode) return leafInstruction<LOG2, SPILL, TIERED, true>(op, ip, h, na, nb, a.marginal != 0, code0, codeGlobal, fs, useRegs, regs, S);
      return leafInstruction<LOG2, SPILL, TIERED, false>(op, ip, h, na, nb, a.marginal != 0, code0, codeGlobal, fs, useRegs, regs, S);
    }
    if (op == OP_OUTERMM) {
      // The weights start after the two header words, eight destinations, na + nb operands and three scale slots.
      const float* wGlobal = reinterpret_cast<const float*>(codeGlobal) + ((ip - code0) + 13 + na + nb);
      return outerSumMatrixAny<LOG2, SPILL, TIERED>(ip, h, na, nb, wGlobal, S);
    }
  }
  if constexpr (sizeof(R) == 8 && !LINEAR) {
    if (op == OP_LEAFQUADMM || op == OP_LEAFPAIRMM || op == OP_LEAFMM) {
      const FeatureSource fs{a.in, a.featureType, row};
      const uint32_t leaves = (h.word(2) >> 12) & 0xfu;
      const uint32_t* stream = codeGlobal + (ip - code0);  // this instruction's words in global memory
      const bool marginal = a.marginal != 0;
      if (op == OP_LEAFQUADMM) return leafLanesG<LOG2, SPILL, 4, 4>(ip, h, leaves, marginal, stream, stagedMode, fs, S);
      if (op == OP_LEAFPAIRMM) return leafLanesG<LOG2, SPILL, 2, 4>(ip, h, leaves, marginal, stream, stagedMode, fs, S);
      if (na == 4) return leafLanesG<LOG2, SPILL, 1, 4>(ip, h, leaves, marginal, stream, stagedMode, fs, S);
      return leafLanesG<LOG2, SPILL, 1, 8>(ip, h, leaves, marginal, stream, stagedMode, fs, S);
    }
  }
  // OP_OUTERSUM
  const uint32_t m = h.word(2);
  if constexpr (sizeof(R) == 8) {
    // eight double sums over an even number of operand rows: the weights come through lanes (every lane of a
    // wavefront is at work here: idle lanes recompute the batch's last sample)
    if (m == 8 && (nb == 8 || nb == 4) && na % 2 == 0) {
      const StreamDouble* wGlobal = reinterpret_cast<const StreamDouble*>(codeGlobal + ((ip - code0) + 2 + 8 + na + nb));
      if (nb == 8) return outerSumLaneWeights<LOG2, SPILL, 8, LINEAR>(ip, na, wGlobal, S);
      return outerSumLaneWeights<LOG2, SPILL, 4, LINEAR>(ip, na, wGlobal, S);
    }
  }
  if (m == 8) return outerSumNB<R, LOG2, SPILL, 8, LINEAR>(ip, na, nb, S);
  if (m == 4) return outerSumNB<R, LOG2, SPILL, 4, LINEAR>(ip, na, nb, S);
  return outerSumNB<R, LOG2, SPILL, 2, LINEAR>(ip, na, nb, S);
}

// MODE 0: every slot lives in LDS. MODE 1: slots below ldsSlots (the program's short pool) live
// in LDS, and only instructions flagged with bit 7 may touch the spill tier. MODE 2: any
// instruction may touch the spill tier (the short pool did not fit into LDS).
// FEAT 1: the program stages its features in slots; 0: instructions read the input row themselves; 2: either,
// decided by the launch arguments (one kernel then carries both forms of every instruction that reads features);
// 3: the program keeps its (at most 32) features in registers: they are read from the input row once per tile and the
// feature fields of the instructions are register numbers, so no instruction fetches a feature from memory.
template <typename R, bool LOG2, int MODE, int FEAT_OR_LINEAR>
__global__ void __launch_bounds__(INTERP_BLOCK) spn_interp_kernel(const uint32_t* __restrict__ codeGlobal, InterpLaunch a) {
  typedef Math<R, LOG2> Mt;
  // Flavour 4 is the linear-space one: feature mode decided at run time like flavour 2, values are probabilities.
  constexpr bool LINEAR = FEAT_OR_LINEAR == 4;
  constexpr int FEAT = LINEAR ? 2 : FEAT_OR_LINEAR;
  extern __shared__ __align__(16) unsigned char ldsRaw[];
  code_ptr code = (code_ptr)codeGlobal;
  const SPN_CONST uint32_t* staged = (const SPN_CONST uint32_t*)a.staged;
  const R* __restrict__ tables = static_cast<const R*>(a.tables);
  R* __restrict__ out = static_cast<R*>(a.out);
  Slots<R, true> Sg;
  Sg.lds = reinterpret_cast<R*>(ldsRaw) + threadIdx.x;
  const unsigned long long lanes = (unsigned long long)gridDim.x * B;
  Sg.spillBlock = static_cast<R*>(a.spill) + (long long)blockIdx.x * a.spillSlots * B - (long long)a.ldsSlots * B;
  Sg.spill = Sg.spillBlock + threadIdx.x;
  Sg.ldsSlots = a.ldsSlots;
  Slots<R, false> Sl;
  Sl.lds = Sg.lds;
  Sl.spill = Sg.spill;
  Sl.spillBlock = Sg.spillBlock;
  Sl.ldsSlots = Sg.ldsSlots;
  if (sizeof(R) == 8 && LOG2) {
    const double* math = static_cast<const double*>(a.tables) + a.mathTables;
    for (unsigned t = threadIdx.x; t < 64; t += B) mathExp2[t] = math[t];
    for (unsigned t = threadIdx.x; t < 512; t += B) mathLog2[t] = math[64 + t];
    if (threadIdx.x < 12) mathPoly[threadIdx.x] = math[576 + threadIdx.x];
    __syncthreads();
  }
  const unsigned long long F = a.numFeatures;
  const bool stagedMode = FEAT == 2 ? a.featureMode == FEAT_STAGED : FEAT == 1;
  FeatureRegs regs;
  const bool useRegs = FEAT == 3;

  for (unsigned long long base = (unsigned long long)blockIdx.x * B; base < a.n; base += lanes) {
    const unsigned long long i = base + threadIdx.x;
    const bool valid = i < a.n;
    const unsigned long long row = (valid ? i : a.n - 1) * F;  // idle lanes recompute the last sample

    if (FEAT == 3) {
      // the staged list names the input column of every register; the register index is wave-uniform
      for (int s = 0; s < int(a.numStaged) && s < int(INTERP_FEATURE_REGISTERS); ++s) regs[s] = featureValue<float>(a.in, a.featureType, row + staged[4 * s]);
    }
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

    code_ptr ip = code;  // at the length word of the first instruction
    Head h = loadHead(codeGlobal, 0);
    R result;
    for (;;) {
      const uint32_t w0 = h.word(1);
      const bool spillPath = MODE == 2 || (MODE == 1 && (w0 & 0x80u));
      if ((w0 & 0x7fu) == OP_END) {
        result = spillPath ? Sg.rd(h.word(2)) : Sl.rd(h.word(2));
        break;
      }
      code_ptr next = ip + 1 + h.word(0);
      const Head hn = loadHead(codeGlobal, next - code);  // in flight while this instruction executes
      if (MODE != 0 && spillPath) execute<R, LOG2, true, MODE == 1, LINEAR>(ip + 1, h, Sg, a, tables, row, stagedMode, code, codeGlobal, useRegs, regs);
      else execute<R, LOG2, false, false, LINEAR>(ip + 1, h, Sl, a, tables, row, stagedMode, code, codeGlobal, useRegs, regs);
      ip = next;
      h = hn;
    }
    if (valid) out[i] = LINEAR ? R(::log(double(result))) : Mt::finish(result);
  }
}

template <typename R, bool LOG2, int FEAT>
const void* kernelPtr(int mode) {
  if (mode == 0) return reinterpret_cast<const void*>(&spn_interp_kernel<R, LOG2, 0, FEAT>);
  if (mode == 1) return reinterpret_cast<const void*>(&spn_interp_kernel<R, LOG2, 1, FEAT>);
  return reinterpret_cast<const void*>(&spn_interp_kernel<R, LOG2, 2, FEAT>);
}

}  // namespace
}  // namespace spnc_hip
