// Launch interface of the table-driven interpreter kernel (see interp_kernel.hip).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace spnc_hip {

constexpr unsigned INTERP_BLOCK = 256;
constexpr unsigned INTERP_FEATURE_REGISTERS = 32;  // features a float kernel can keep in registers (FEAT_REGISTER programs)

struct InterpLaunch {
  const uint32_t* code;      // device: instruction stream
  const void* in;            // device: [n, numFeatures] row-major, feature type below
  void* out;                 // device: [n] of the compute type
  unsigned long long n;
  const void* tables;        // device: leaf-table pool of the compute type
  void* spill;               // device: [gridDim.x][spillSlots][INTERP_BLOCK] of the compute type
  const uint32_t* staged;    // device: numStaged * 4 words (column, valueSlot, indexSlot, tableLen)
  uint32_t numStaged;
  uint32_t numFeatures;
  uint32_t featureType;      // spnc_hip::FeatureType as integer
  uint32_t featureMode;      // FEAT_STAGED / FEAT_DIRECT / FEAT_REGISTER
  uint32_t ldsSlots;         // slots [0, ldsSlots) live in LDS, the rest in the spill tier
  uint32_t spillSlots;       // number of slots in the spill tier
  uint32_t marginal;         // NaN features marginalise Gaussian leaves
  uint32_t mathTables;       // float64 in the log2 domain: index into `tables` of the exp2/log2 routines' tables
};

// Enqueues the interpreter on `stream`. ldsBytes = ldsSlots * INTERP_BLOCK * sizeof(compute type).
// linear: the program computes with probabilities (double), not logarithms.
// mode 0: all slots in LDS; 1: the program's short pool in LDS, flagged instructions may touch the spill tier;
// 2: any instruction may touch the spill tier.
hipError_t launchInterpreter(const InterpLaunch& args, bool f64, bool log2Domain, bool linear, int mode, unsigned grid, size_t ldsBytes,
                             hipStream_t stream);

// Device memory of the allocation-free entry point: one array per device inside the library's code object, held
// from library load to process end. Returns its address on the current device, its size and that device's ordinal.
// The first call on a device also creates the event through which calls on different streams take turns on the
// array (interpreterScratchEvent), so that no later call has anything left to create.
constexpr size_t INTERP_SCRATCH_BYTES = size_t(64) << 20;
hipError_t interpreterScratch(void** base, size_t* bytes, int* device);
hipEvent_t interpreterScratchEvent(int device);

// Largest LDS size a block may use on the current device, and the static LDS the kernel flavour for such a program
// takes of it (the dynamic size a launch may request is the difference).
hipError_t interpreterMaxLds(bool f64, bool log2Domain, bool linear, uint32_t featureMode, size_t* bytes, size_t* staticBytes);

// Resident blocks per CU for a given dynamic LDS size. featureMode: the program's (args.featureMode at launch);
// float kernels are built once per feature mode.
hipError_t interpreterOccupancy(bool f64, bool log2Domain, bool linear, int mode, uint32_t featureMode, size_t ldsBytes, int* blocksPerCU);

}  // namespace spnc_hip
