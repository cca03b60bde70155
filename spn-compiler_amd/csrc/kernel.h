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

// Whose turn it is on a device buffer that launches on several streams share.
struct Turn {
  hipEvent_t done = nullptr;   // recorded after the last launch that used the buffer
  hipStream_t last = nullptr;  // the stream of that launch
  bool used = false;
  void wait(hipStream_t stream);    // a launch on another stream than `last` waits for `done`
  void record(hipStream_t stream);  // creates `done` on first use
  void reset();
};

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
  // The same for interpreter kernels without any allocation: the kernel's device buffers come out of the library's
  // fixed scratch array (interp_kernel.h). Calls on different streams of one device take turns on that array.
  void executeDeviceStatic(size_t n, const void* dIn, void* dOut, hipStream_t stream);

 private:
  Kernel() = default;
  void save(const std::string& path) const;
  void ensureDevice();
  void queryDevice();
  void buildImages();
  void prepareDevice();
  void launchProgram(size_t n, const void* dIn, void* dOut, const uint32_t* code, const void* tables, const uint32_t* staged, void* spill,
                     size_t maxBlocks, hipStream_t stream);
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
  // A graph cut by "maxTaskSize": several kernels in the one code object, launched one after the other on the caller's
  // stream; values pass from task to task through an intermediate buffer of `taskSlots_` rows.
  struct Task {
    std::string entry;
    unsigned blockSize = 256;
    int gridPolicy = 0;
    hipFunction_t function = nullptr;
    int blocksPerCU = 1;
  };
  std::vector<Task> tasks_;
  unsigned taskSlots_ = 0;
  unsigned taskBufferMiB_ = 1024;
  // interpreter
  InterpProgram prog_;

  // ---- device state, created on first execute ----
  std::mutex mu_;
  bool deviceReady_ = false;   // module loaded / device buffers allocated
  bool deviceKnown_ = false;   // device facts and the kernel's launch shape queried
  uint64_t kernelId_ = 0;      // tag of this kernel's program in the shared scratch array
  std::vector<uint32_t> codeImage_, stagedImage_;  // what the device holds of the program (built once)
  std::vector<char> tableImage_;
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
  Turn spillTurn_;             // launches of this handle on different streams take turns on dSpill_
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
  // intermediate buffer of a partitioned kernel: [taskSlots_][interRows_] results, reused by every call (calls on
  // different streams wait for each other through interDone_)
  void* dInter_ = nullptr;
  size_t interRows_ = 0;
  hipEvent_t interDone_ = nullptr;
  bool interUsed_ = false;
};

}  // namespace spnc_hip
