// Host side of the table-driven SPN interpreter kernel: picks the kernel flavour for a program, launches it, and owns
// the scratch array of the allocation-free entry point. The device code lives in interp_kernel_impl.h.
#include "interp_kernel.h"

#include <mutex>

#include "interp_program.h"
#include "spn_graph.h"

namespace spnc_hip {

// The kernels are instantiated in translation units of their own (interp_kernel_inst.hip), one per flavour.
const void* interpKernel_f32_log2_direct(int mode);
const void* interpKernel_f32_log2_staged(int mode);
const void* interpKernel_f32_log2_registers(int mode);
const void* interpKernel_f32_natural_direct(int mode);
const void* interpKernel_f32_natural_staged(int mode);
const void* interpKernel_f32_natural_registers(int mode);
const void* interpKernel_f64(int mode);
const void* interpKernel_f64_log2(int mode);
const void* interpKernel_f64_linear(int mode);

namespace {

// float kernels exist once per feature mode: the fused leaf instructions are long, and a kernel that held both
// of their forms would run the staged one slower (instruction fetch). double kernels decide at run time.
const void* pick(bool f64, bool log2Domain, bool linear, int mode, uint32_t featureMode) {
  if (linear) return interpKernel_f64_linear(mode);  // linear space computes in double, as the reference does
  if (f64) return log2Domain ? interpKernel_f64_log2(mode) : interpKernel_f64(mode);
  if (featureMode == FEAT_REGISTER) return log2Domain ? interpKernel_f32_log2_registers(mode) : interpKernel_f32_natural_registers(mode);
  if (featureMode == FEAT_STAGED) return log2Domain ? interpKernel_f32_log2_staged(mode) : interpKernel_f32_natural_staged(mode);
  return log2Domain ? interpKernel_f32_log2_direct(mode) : interpKernel_f32_natural_direct(mode);
}

}  // namespace

namespace {
// Scratch memory of the allocation-free entry point. The name is a host-side handle only: device code and every
// runtime call get the address that hipGetSymbolAddress returns for the current device.
static __device__ __align__(256) unsigned char scratch[INTERP_SCRATCH_BYTES];
std::mutex scratchMutex;
void* scratchAddress[64] = {};
hipEvent_t scratchEvent[64] = {};
}  // namespace

hipEvent_t interpreterScratchEvent(int device) { return device >= 0 && device < 64 ? scratchEvent[device] : nullptr; }

hipError_t interpreterScratch(void** base, size_t* bytes, int* device) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(scratchMutex);
  if (!scratchAddress[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    e = hipEventCreateWithFlags(&scratchEvent[dev], hipEventDisableTiming);
    if (e != hipSuccess) return e;
    scratchAddress[dev] = p;
  }
  *device = dev;
  *base = scratchAddress[dev];
  *bytes = INTERP_SCRATCH_BYTES;
  return hipSuccess;
}

hipError_t interpreterMaxLds(bool f64, bool log2Domain, bool linear, uint32_t featureMode, size_t* bytes, size_t* staticBytes) {
  int dev = 0, maxLds = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  e = hipDeviceGetAttribute(&maxLds, hipDeviceAttributeMaxSharedMemoryPerBlock, dev);
  if (e != hipSuccess) return e;
  hipFuncAttributes attr;
  e = hipFuncGetAttributes(&attr, pick(f64, log2Domain, linear, 1, featureMode));  // the three modes of a flavour hold the same static LDS
  if (e != hipSuccess) return e;
  *bytes = size_t(maxLds);
  *staticBytes = attr.sharedSizeBytes;
  return hipSuccess;
}

hipError_t interpreterOccupancy(bool f64, bool log2Domain, bool linear, int mode, uint32_t featureMode, size_t ldsBytes, int* blocksPerCU) {
  const void* fn = pick(f64, log2Domain, linear, mode, featureMode);
  if (ldsBytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, int(ldsBytes));
    if (e != hipSuccess) return e;
  }
  return hipOccupancyMaxActiveBlocksPerMultiprocessor(blocksPerCU, fn, int(INTERP_BLOCK), ldsBytes);
}

hipError_t launchInterpreter(const InterpLaunch& args, bool f64, bool log2Domain, bool linear, int mode, unsigned grid, size_t ldsBytes,
                             hipStream_t stream) {
  const void* fn = pick(f64, log2Domain, linear, mode, args.featureMode);
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
