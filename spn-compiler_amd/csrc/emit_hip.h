// Generator for the straight-line per-SPN HIP kernel (gfx950, one sample per lane).
//
// Replaces, for the HIP target, the reference's LoSPN->GPU lowering and cubin steps
// (mlir/lib/Conversion/LoSPNtoGPU/*, compiler/src/pipeline/steps/mlir/conversion/CUDA/*):
// instead of lowering MLIR it prints one HIP C++ translation unit per SPN, which jit.cpp
// compiles with hipRTC.
#pragma once
#include <string>
#include <vector>

#include "options.h"
#include "spn_graph.h"

namespace spnc_hip {

struct JitSource {
  std::string source;
  std::string entry;          // extern "C" kernel symbol
  unsigned blockSize = 256;
  unsigned samplesPerLane = 1;
  unsigned inputAlign = 4;    // required byte alignment of the input base pointer
  unsigned bytesPerResult = 4;
  unsigned tableEntries = 0;  // entries of the leaf-table pool (0 = none)
  bool tablesInLds = false;
  bool libraryMath = false;   // calls ocml exp/log (natural-log domain, linear space)
  bool doubleConstants = false;  // computes in double: constants live in registers, not in instruction literals
  bool oneTilePerBlock = false;
  bool waveTransposedInput = false;  // every wavefront copies its 64 rows with coalesced loads, packed to bytes, through its own LDS buffer
  bool packedRows = false;    // the kernel body works on rows packed to a byte per feature (sibling products evaluated together)
  bool stagedInput = false;   // rows reach the lanes through an LDS tile ("gpu-shared-mem")
};

// `entry` names the kernel. A task of a partitioned graph (g.isTask) takes two more arguments: the intermediate buffer to
// read from and to write to, [rows][n] values of the kernel's compute type.
JitSource emitHipSource(const Graph& g, const CompileOptions& o, const std::string& entry = "spn_kernel");

// The automatic choice behind "hip-inline-math": true if the library's exp/log are inlined at every call of this graph.
bool inlineLibraryMath(const Graph& g, const CompileOptions& o);

}  // namespace spnc_hip
