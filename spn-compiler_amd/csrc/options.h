// String-keyed compile options for the HIP target.
//
// Keeps the reference's option names and parsing rules (compiler/src/option/GlobalOptions.cpp:14-75;
// booleans are true for "true"/"yes" in any case, compiler/src/option/Options.cpp:78-82; an unknown key
// is fatal, compiler/src/option/Options.h:222-224; "target" is required). Options that only steer the
// reference's CPU/MLIR pipeline are accepted and ignored; options prefixed "hip-" are new.
#pragma once
#include <map>
#include <string>

namespace spnc_hip {

enum class KernelMode { Auto, Jit, Interpreter };
enum class SumForm { Nary, Pairwise };
enum class ComputeType { F32, F64 };

struct CompileOptions {
  bool useLogSpace = false;     // "use-log-space" (reference default false; the Python front passes true)
  int gpuSharedMem = -1;        // "gpu-shared-mem": stage the input tile through LDS (1), do not (0), decide from the SPN (-1, option absent)
  bool dumpIR = false;          // "dump-ir": print the generated device source / program
  bool collectGraphStats = false;
  std::string graphStatsFile = "/tmp/stats.json";
  int maxTaskSize = -1;
  int optLevel = 3;
  bool optLevelGiven = false;   // "optLevel" was passed explicitly
  bool deleteTemps = true;
  ComputeType computeType = ComputeType::F32;  // "hip-compute-type": float32 | float64 (log-space only)
  KernelMode kernelMode = KernelMode::Auto;    // "hip-kernel": auto | jit | interpreter
  SumForm sumForm = SumForm::Nary;             // "hip-sum-form": nary | pairwise
  bool log2Domain = true;                      // "hip-log2-domain": carry log2 values in f32 kernels
  int samplesPerLane = 0;                      // "hip-samples-per-lane": 0 = choose from SPN size
  int jitMaxOps = 20000;                       // "hip-jit-max-ops": above this, auto picks the interpreter
  int blockSize = 0;                           // "hip-block-size": 64, 128, 256 or 512 threads (0 = automatic)
  bool nontemporalLoads = true;                // "hip-nontemporal-loads": mark input loads as streaming
  bool eagerIndices = true;                    // "hip-eager-indices": compute table indices of all features first
  bool jointTables = true;                     // "hip-joint-tables": pair table leaves of a product into joint tables
  int machineLicm = -1;                        // "hip-machine-licm": machine LICM for generated kernels on (1), off (0) or decided per kernel (-1)
  int inlineMath = -1;                         // "hip-inline-math": exp/log routines inlined (1), called (0) or decided by graph size (-1)
  bool groupedTables = true;                   // "hip-grouped-tables": tables read with the same index are interleaved in blocks of four columns and fetched up to four per read
  int tableGroupMinReads = 200;                // "hip-table-group-min-reads": graphs with fewer table reads per sample keep plain tables
  int tableGroupWindow = 96;                   // "hip-table-group-window": tables of a group are used within this many table uses of each other
  int ldsBallastKiB = 0;                       // "hip-lds-ballast-kib": LDS a block claims without using it, which caps the blocks (and wavefronts) a CU holds; for measurement
  int tablePadKiB = 18;                        // "hip-table-pad-kib": LDS beyond the table budget that blocks of four columns may take (unused columns)
  int tableBudgetKiB = 62;                     // "hip-table-budget-kib": LDS the table pool may grow to when leaves are paired into joint tables
  bool tableBudgetGiven = false;               // without the option, kernels on packed rows pair up to 96 KiB (measured on the 100-feature discrete graph: 0.78 ms at 62 KiB, 0.75 ms at 80, 0.74 ms at 96 with leaves over three categories in tables too)
  int jointMaxEntries = 160;                   // "hip-joint-max-entries": largest joint table (entries) a pair of table leaves may get
  int interpShortSlots = 0;                    // "hip-interp-short-slots": LDS value slots per lane the interpreter program aims for (0 = automatic)
  bool interpLeafRegions = true;               // "hip-interp-leaf-regions": Gaussian leaf products read by one matrix-form outer sum are computed inside it
  bool interpVectorBlocks = true;              // "hip-interp-vector-blocks": results of a matrix-form outer sum occupy consecutive slots
  bool interpScaledVectors = true;             // "hip-interp-scaled-vectors": region vectors between matrix-form outer sums travel as scaled linear values
  bool interpMatrixCore = true;                // "hip-interp-matrix-core": float outer sums of eight sums run on the matrix cores
  bool interpFeatureRegisters = true;          // "hip-interp-feature-registers": float programs over at most 32 Gaussian-only features keep them in registers
  int interpLdsSlots = 0;                      // "hip-interp-lds-slots": upper bound on the value slots the launcher keeps in LDS (0 = automatic)
  int interpStagedLong = -1;                   // "hip-interp-staged-features": lds|spill (-1 = automatic): tier of the staged input features
  long interpLongRange = -1;                   // "hip-interp-long-range": values living longer than this many instructions go to the long-lived pool (-1 = automatic)
  int packedRows = -1;                         // "hip-packed-rows": wide rows of small integer features stay packed four to a register and the table leaves of sibling products are evaluated together (1), not (0), decided per kernel (-1)
  bool marginalOffsets = true;                 // "hip-marginal-offsets": float kernels replace a missing feature by a stand-in value, evaluate the Gaussian leaves of a product without selects and take what the leaves over missing features added off again with one table value per product
  bool tablePlanes = true;                     // "hip-table-planes": with packed rows, the tables of sibling products lie one after the other (4-byte reads, fewer LDS bank conflicts) instead of side by side per entry
  int oneHotMaxDomain = 2;                     // "hip-one-hot-max-domain": with packed rows, table leaves over at most this many categories are evaluated as multiply-adds on the vector unit instead of LDS reads
  bool nanMasks = true;                        // "hip-nan-masks": with marginalisation in log space, a Gaussian leaf of a missing (NaN) feature is zeroed by a bitwise AND with a per-feature mask instead of a select per leaf
  int gaussExpanded = -1;                      // "hip-gauss-expanded": float64 log-space kernels evaluate a Gaussian leaf inside a product as A x^2 + B x + C on per-feature x^2, x and 1 (zeroed for a missing feature): three multiply-adds per leaf and no mask, two without marginalisation (-1 = where the expansion keeps 1e-11, see emit_hip.cpp)
  bool laneConstants = true;                   // "hip-lane-constants": expanded Gaussian leaves take their constants from vector registers that hold sixteen constants each, one per lane of a row, through the cross-lane broadcast operand of the multiply-add (false = scalar moves with literals)
  int marginalTablesKiB = 40;                  // "hip-marginal-tables-kib": LDS for the tables from which expanded leaves of kernels with marginalisation read the sum of their constant terms by the pattern of missing features (0 = a third multiply-add per leaf instead)
  int taskBufferMiB = 1024;                    // "hip-task-buffer-mib": most device memory the values passing between the tasks of a partitioned graph may take; larger batches run in several passes
  int prefetchRows = -1;                       // "hip-prefetch-rows": with the per-wavefront transposed load, the loads of a wavefront's next 64 rows are issued before the current ones are evaluated and stay in registers meanwhile (-1 = with packed rows)
  bool hoistFeatureValues = true;              // "hip-hoist-feature-values": with packed rows, the values (and squares) of the features whose leaves are polynomials are computed once at the top of the kernel (false = again in every group of products that uses them: more arithmetic, fewer registers)
  int fusedBatch = -1;                         // "hip-fused-batch": with packed rows, LDS reads of this many table units are issued before the values of the batch before are added (0 = every unit on its own, no scheduling barriers; -1 = 2 when rows are prefetched, which leaves fewer registers, else 4)
  int waveTranspose = -1;                       // "hip-wave-transpose": rows of 32-bit integer features reach the lanes through a per-wave LDS transpose of packed bytes (1), not (0), decided per kernel (-1)
  int minBlocksPerCU = 0;                      // "hip-min-blocks-per-cu": register budget hint for the generated kernel (0 = none)
  int blocksPerCU = 0;                         // "hip-blocks-per-cu": 0 = resident blocks (persistent), -1 = one tile per block, n = n per CU
};

// Throws std::runtime_error("Unknown compile option <key>") etc.
CompileOptions parseOptions(const std::map<std::string, std::string>& kv);

}  // namespace spnc_hip
