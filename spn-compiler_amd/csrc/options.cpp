#include "options.h"

#include <algorithm>
#include <cctype>
#include <set>
#include <stdexcept>

namespace spnc_hip {

namespace {

bool parseBool(const std::string& v) {
  std::string s = v;
  std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return char(std::tolower(c)); });
  return s == "true" || s == "yes";
}

int parseInt(const std::string& key, const std::string& v) {
  try {
    size_t pos = 0;
    int r = std::stoi(v, &pos);
    if (pos != v.size()) throw std::invalid_argument(v);
    return r;
  } catch (const std::exception&) {
    throw std::runtime_error("Could not parse option value " + v + " for " + key);
  }
}

// Options of the reference that steer only its CPU / MLIR / CUDA pipelines.
const std::set<std::string>& ignoredKeys() {
  static const std::set<std::string> k = {
      "irOptLevel", "mcOptLevel", "cpu-vectorize", "vector-library", "use-shuffle", "slp-max-attempts",
      "slp-max-successful-iterations", "slp-max-node-size", "slp-max-look-ahead", "slp-reorder-dfs",
      "slp-allow-duplicate-elements", "slp-allow-topological-mixing", "slp-use-xor-chains", "search-paths",
      "opt-repr", "stopAfter"};
  return k;
}

}  // namespace

CompileOptions parseOptions(const std::map<std::string, std::string>& kv) {
  CompileOptions o;
  bool haveTarget = false;
  for (const auto& e : kv) {
    const std::string& key = e.first;
    const std::string& val = e.second;
    if (key == "target") {
      if (val != "HIP") throw std::runtime_error("Target was '" + val + "', but this compiler only supports target 'HIP'");
      haveTarget = true;
    } else if (key == "use-log-space") {
      o.useLogSpace = parseBool(val);
    } else if (key == "gpu-shared-mem") {
      o.gpuSharedMem = parseBool(val) ? 1 : 0;
    } else if (key == "dump-ir") {
      o.dumpIR = parseBool(val);
    } else if (key == "collect-graph-stats") {
      o.collectGraphStats = parseBool(val);
    } else if (key == "graph-stats-file") {
      o.graphStatsFile = val;
    } else if (key == "maxTaskSize") {
      o.maxTaskSize = parseInt(key, val);
    } else if (key == "optLevel") {
      o.optLevel = parseInt(key, val);
      o.optLevelGiven = true;
    } else if (key == "delete-temps") {
      o.deleteTemps = parseBool(val);
    } else if (key == "hip-compute-type") {
      if (val == "float32") o.computeType = ComputeType::F32;
      else if (val == "float64") o.computeType = ComputeType::F64;
      else throw std::runtime_error("Could not parse option value " + val + " for " + key);
    } else if (key == "hip-kernel") {
      if (val == "auto") o.kernelMode = KernelMode::Auto;
      else if (val == "jit") o.kernelMode = KernelMode::Jit;
      else if (val == "interpreter") o.kernelMode = KernelMode::Interpreter;
      else throw std::runtime_error("Could not parse option value " + val + " for " + key);
    } else if (key == "hip-sum-form") {
      if (val == "nary") o.sumForm = SumForm::Nary;
      else if (val == "pairwise") o.sumForm = SumForm::Pairwise;
      else throw std::runtime_error("Could not parse option value " + val + " for " + key);
    } else if (key == "hip-log2-domain") {
      o.log2Domain = parseBool(val);
    } else if (key == "hip-interp-feature-registers") {
      o.interpFeatureRegisters = parseBool(val);
    } else if (key == "hip-interp-leaf-regions") {
      o.interpLeafRegions = parseBool(val);
    } else if (key == "hip-interp-vector-blocks") {
      o.interpVectorBlocks = parseBool(val);
    } else if (key == "hip-interp-scaled-vectors") {
      o.interpScaledVectors = parseBool(val);
    } else if (key == "hip-interp-matrix-core") {
      o.interpMatrixCore = parseBool(val);
    } else if (key == "hip-samples-per-lane") {
      o.samplesPerLane = parseInt(key, val);
      if (o.samplesPerLane < 0 || o.samplesPerLane > 16) throw std::runtime_error("hip-samples-per-lane must be in [0,16]");
    } else if (key == "hip-jit-max-ops") {
      o.jitMaxOps = parseInt(key, val);
    } else if (key == "hip-nan-masks") {
      o.nanMasks = parseBool(val);
    } else if (key == "hip-gauss-expanded") {
      o.gaussExpanded = val == "auto" ? -1 : (parseBool(val) ? 1 : 0);
    } else if (key == "hip-lane-constants") {
      o.laneConstants = parseBool(val);
    } else if (key == "hip-marginal-tables-kib") {
      o.marginalTablesKiB = parseInt(key, val);
      if (o.marginalTablesKiB < 0 || o.marginalTablesKiB > 60) throw std::runtime_error("hip-marginal-tables-kib must be in [0,60]");
    } else if (key == "hip-task-buffer-mib") {
      o.taskBufferMiB = parseInt(key, val);
      if (o.taskBufferMiB < 1 || o.taskBufferMiB > 65536) throw std::runtime_error("hip-task-buffer-mib must be in [1,65536]");
    } else if (key == "hip-prefetch-rows") {
      o.prefetchRows = parseBool(val) ? 1 : 0;
    } else if (key == "hip-hoist-feature-values") {
      o.hoistFeatureValues = parseBool(val);
    } else if (key == "hip-packed-rows") {
      o.packedRows = parseBool(val) ? 1 : 0;
    } else if (key == "hip-marginal-offsets") {
      o.marginalOffsets = parseBool(val);
    } else if (key == "hip-table-planes") {
      o.tablePlanes = parseBool(val);
    } else if (key == "hip-one-hot-max-domain") {
      o.oneHotMaxDomain = parseInt(key, val);
      if (o.oneHotMaxDomain < 0 || o.oneHotMaxDomain > 16) throw std::runtime_error("hip-one-hot-max-domain must be in [0,16]");
    } else if (key == "hip-fused-batch") {
      o.fusedBatch = parseInt(key, val);
      if (o.fusedBatch < 0 || o.fusedBatch > 16) throw std::runtime_error("hip-fused-batch must be in [0,16]");
    } else if (key == "hip-wave-transpose") {
      o.waveTranspose = parseBool(val) ? 1 : 0;
    } else if (key == "hip-nontemporal-loads") {
      o.nontemporalLoads = parseBool(val);
    } else if (key == "hip-eager-indices") {
      o.eagerIndices = parseBool(val);
    } else if (key == "hip-joint-tables") {
      o.jointTables = parseBool(val);
    } else if (key == "hip-grouped-tables") {
      o.groupedTables = parseBool(val);
    } else if (key == "hip-table-group-min-reads") {
      o.tableGroupMinReads = parseInt(key, val);
      if (o.tableGroupMinReads < 0) throw std::runtime_error("hip-table-group-min-reads must not be negative");
    } else if (key == "hip-table-group-window") {
      o.tableGroupWindow = parseInt(key, val);
      if (o.tableGroupWindow < 0) throw std::runtime_error("hip-table-group-window must not be negative");
    } else if (key == "hip-lds-ballast-kib") {
      o.ldsBallastKiB = parseInt(key, val);
      if (o.ldsBallastKiB < 0 || o.ldsBallastKiB > 150) throw std::runtime_error("hip-lds-ballast-kib must be in [0,150]");
    } else if (key == "hip-table-pad-kib") {
      o.tablePadKiB = parseInt(key, val);
      if (o.tablePadKiB < 0 || o.tablePadKiB > 64) throw std::runtime_error("hip-table-pad-kib must be in [0,64]");
    } else if (key == "hip-interp-short-slots") {
      o.interpShortSlots = parseInt(key, val);
      if (o.interpShortSlots < 0 || o.interpShortSlots > 160) throw std::runtime_error("hip-interp-short-slots must be in [0,160]");
    } else if (key == "hip-interp-lds-slots") {
      o.interpLdsSlots = parseInt(key, val);
      if (o.interpLdsSlots < 0 || o.interpLdsSlots > 160) throw std::runtime_error("hip-interp-lds-slots must be in [0,160]");
    } else if (key == "hip-interp-staged-features") {
      if (val == "lds") o.interpStagedLong = 0;
      else if (val == "spill") o.interpStagedLong = 1;
      else if (val == "auto") o.interpStagedLong = -1;
      else throw std::runtime_error("hip-interp-staged-features must be lds, spill or auto");
    } else if (key == "hip-interp-long-range") {
      o.interpLongRange = parseInt(key, val);
      if (o.interpLongRange < -1) throw std::runtime_error("hip-interp-long-range must be -1 or a count of instructions");
    } else if (key == "hip-machine-licm") {
      o.machineLicm = val == "auto" ? -1 : (parseBool(val) ? 1 : 0);
    } else if (key == "hip-inline-math") {
      o.inlineMath = val == "auto" ? -1 : (parseBool(val) ? 1 : 0);
    } else if (key == "hip-table-budget-kib") {
      o.tableBudgetKiB = parseInt(key, val);
      o.tableBudgetGiven = true;
      if (o.tableBudgetKiB < 0 || o.tableBudgetKiB > 140) throw std::runtime_error("hip-table-budget-kib must be in [0,140]");
    } else if (key == "hip-joint-max-entries") {
      o.jointMaxEntries = parseInt(key, val);
      if (o.jointMaxEntries < 0 || o.jointMaxEntries > 4096) throw std::runtime_error("hip-joint-max-entries must be in [0,4096]");
    } else if (key == "hip-min-blocks-per-cu") {
      o.minBlocksPerCU = parseInt(key, val);
      if (o.minBlocksPerCU < 0 || o.minBlocksPerCU > 8) throw std::runtime_error("hip-min-blocks-per-cu must be in [0,8]");
    } else if (key == "hip-blocks-per-cu") {
      o.blocksPerCU = parseInt(key, val);
      if (o.blocksPerCU < -1 || o.blocksPerCU > 64) throw std::runtime_error("hip-blocks-per-cu must be in [-1,64]");
    } else if (key == "hip-block-size") {
      o.blockSize = parseInt(key, val);
      if (o.blockSize < 0 || o.blockSize > 1024 || o.blockSize % 64 != 0)
        throw std::runtime_error("hip-block-size must be a multiple of 64 up to 1024");
    } else if (ignoredKeys().count(key)) {
      // accepted for compatibility, no effect on the HIP target
    } else {
      throw std::runtime_error("Unknown compile option " + key);
    }
  }
  if (!haveTarget) throw std::runtime_error("Could not verify configuration constraints!");
  if (o.collectGraphStats == false && kv.count("graph-stats-file"))
    throw std::runtime_error("Could not verify configuration constraints!");
  return o;
}

}  // namespace spnc_hip
