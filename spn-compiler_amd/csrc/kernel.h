// Compiled-kernel handle and launcher for the HIP target.
//
// Stands in for the reference's Kernel descriptor (common/include/Kernel.h:29-126), its runtime
// (runtime/src/runtime.cpp:42-49, runtime/src/Executable.cpp:41-133) and the CUDA driver-API
// wrappers its generated host code calls (runtime/wrappers/cuda/CUDARuntimeWrappers.cpp:56-153):
// module loading, argument marshalling, streams, host<->device copies and the kernel launch all
// live here, directly on the HIP runtime.
#pragma once
#include <hip/hip_runtime.h>

#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/spnc_hip.h"
#include "emit_hip.h"
#include "interp_program.h"
#include "options.h"
#include "spn_graph.h"

namespace spnc_hip {

class Kernel {
 public:
  // Parses, validates and compiles a serialized query; writes the kernel file. Needs no GPU.
  static std::unique_ptr<Kernel> compile(const std::string& queryPath, const std::map<std::string, std::string>& options);
  // Restores a kernel from a kernel file written by compile().
  static std::unique_ptr<Kernel> load(const std::string& kernelFile);
  ~Kernel();

  void fillInfo(spnc_hip_info* info) const;
  const std::string& text() const { return text_; }

  // Host buffers in, host buffers out; returns when `out` is complete.
  void execute(size_t n, const void* in, void* out);
  // Device buffers; enqueues on `stream` and returns.
  void executeDevice(size_t n, const void* dIn, void* dOut, hipStream_t stream);

 private:
  Kernel() = default;
  void save(const std::string& path) const;
  void ensureDevice();
  void prepareDevice();
  void releaseDevice();
  void ensureStaging(size_t rows);
  void launch(size_t n, const void* dIn, void* dOut, hipStream_t stream);

  // ---- what is stored in the kernel file ----
  std::string fileName_, kernelName_;
  unsigned batchSize_ = 1, numFeatures_ = 0, bytesPerFeature_ = 0, bytesPerResult_ = 4;
  unsigned featureType_ = 0;
  bool marginal_ = false;
  unsigned kind_ = SPNC_HIP_KERNEL_JIT;
  GraphStats stats_;
  unsigned numNodes_ = 0;
  std::string text_;  // generated source or program listing
  // straight-line kernel
  std::vector<char> codeObject_;
  std::string entry_;
  unsigned blockSize_ = 256, samplesPerLane_ = 1, inputAlign_ = 4;
  int gridPolicy_ = 0;  // 0 = resident blocks, -1 = one tile per block, n = n blocks per CU
  // interpreter
  InterpProgram prog_;

  // ---- device state, created on first execute ----
  std::mutex mu_;
  bool deviceReady_ = false;
  int device_ = 0;
  int numCUs_ = 0;
  hipModule_t module_ = nullptr;
  hipFunction_t function_ = nullptr;
  int blocksPerCU_ = 1;
  uint32_t* dCode_ = nullptr;
  void* dTables_ = nullptr;
  uint32_t* dStaged_ = nullptr;
  void* dSpill_ = nullptr;
  size_t spillBytes_ = 0;
  uint32_t ldsSlots_ = 0;
  int interpMode_ = 0;
  size_t ldsBytes_ = 0;
  // double-buffered staging for host execute
  struct Stage {
    void *hIn = nullptr, *hOut = nullptr, *dIn = nullptr, *dOut = nullptr;
    hipStream_t stream = nullptr;
    size_t pendingRows = 0;   // rows whose results sit in hOut waiting to be copied out
    size_t pendingOffset = 0;
  } stage_[2];
  size_t stageRows_ = 0;
  hipEvent_t kernelDone_ = nullptr;
};

}  // namespace spnc_hip
