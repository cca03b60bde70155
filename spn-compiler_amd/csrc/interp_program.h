// Node program for the table-driven interpreter kernel: the path for SPN DAGs too large to
// inline as one straight-line kernel. Plays the role the reference's task partitioner plays
// for large graphs (mlir/lib/Dialect/LoSPN/Passes/LoSPNTaskPartitioner.cpp), with a different
// mechanism: one resident kernel walks a wave-uniform instruction stream, operands live in
// per-lane value slots (LDS first, a coalesced global spill tier behind it).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#include "options.h"
#include "spn_graph.h"

namespace spnc_hip {

// The stream is a sequence of [length][instruction words...]: the length word counts the words of
// the instruction that follows it.
// Opcodes (low 7 bits of an instruction's first word; bit 7 is set when the instruction reads or
// writes a long-lived slot; the upper 24 bits hold counts).
enum InterpOp : uint32_t {
  OP_END = 0,       // [op][src]                       result = slot src
  OP_PROD = 1,      // [op][dst][ns][ng][nt] ns*slot, ng*(feat, mean, shift, den), nt*(feat, tableOffset, tableLen)
                    //   Gaussian leaf value = den * ((x - mean)^2 + shift), den = -1/(2 sigma^2) in the kernel's log unit
  OP_SUM = 2,       // [op|k<<8][dst] k*(slot, weight)                 one weighted sum
  OP_SUMLAYER = 3,  // [op|k<<8][M][dst*M] k*slot, k*M weights        M sums over the same k children (M in 2,4,8)
  OP_OUTERSUM = 4,  // [op|NA<<8|NB<<16][M][dst*M] NA*slot, NB*slot, NA*NB*M weights
                    //   M sums over all products a_r * b_c of two operand vectors, products never materialised
  OP_OUTERMM = 6,   // [op|NA<<8|NB<<16|tiers<<24|aScaled<<30|bScaled<<31][8|outScaled<<8][dst*8] NA*slot, NB*slot,
                    //   [scale slot of dst, of a, of b (0xFFFFFFFF where unused)], NA*NB*8 weights in matrix-core order
                    //   tiers: two bits each for the a, b and dst lists: 0 all short-pool slots, 1 all long-pool, 2 mixed
                    //   A scaled list holds v_i / max(v) (linear, in [0,1]) and its scale slot log2 max(v) plus the
                    //   scales it inherited: value_i = scale + log2(slot_i). Such vectors only travel between
                    //   matrix-form outer sums; they save the consumer's exponentials and the producer's logarithms.
                    //   OUTERSUM for float, eight sums and NA*NB a multiple of 16: weight of product k = r*NB + c and
                    //   sum t sits at word (k/16)*128 + (t/4)*64 + (k%16)*4 + t%4, i.e. 64-word rows that one
                    //   wavefront loads with one coalesced access and that feed sixteen 4x4x1 matrix instructions
  OP_LEAFMM = 7,    // [op|NA<<8|NB<<16|dstTier<<28][8|outScaled<<8|dstRun<<11|G<<12|featTier<<16] dst*8, scaleDst (or
                    //   0xFFFFFFFF), G feature slots of the a list, G of the b list, (NA+NB)*G*(mean, shift, den),
                    //   weights as in OP_OUTERMM: an OP_OUTERMM whose operand lists are products of G Gaussian leaves
                    //   each, all products of a list over the same features; they are computed in registers
  OP_LEAFPAIRMM = 8,// [op|N<<8|dstTier<<28][8|outScaled<<8|dstRun<<11|G<<12|featTier<<16] dst*8, scaleDst (or 0xFFFFFFFF),
                    //   feature slots (a and b list of the first leaf region, then of the second: 4 G), constants of the
                    //   first region's 2 N products and of the second's, weights of the first region (N*N*8), of the
                    //   second, of the 8x8 sum over the two result vectors (512), each as in OP_OUTERMM: two OP_LEAFMM
                    //   of N x N products and the OP_OUTERMM over their results in one instruction (emitted for N = 4)
  OP_LEAFQUADMM = 9,// [op|4<<8|dstTier<<28][8|outScaled<<8|dstRun<<11|G<<12|featTier<<16] dst*8, scaleDst (or 0xFFFFFFFF),
                    //   8 G feature slots (leaf regions 1 to 4, a list then b list), the constants of the four regions,
                    //   weights: region 1, region 2, the 8x8 sum over them, region 3, region 4, the 8x8 sum over them,
                    //   the 8x8 sum over the two pairs' results: two OP_LEAFPAIRMM and the OP_OUTERMM over their
                    //   results in one instruction (4x4 leaf regions, G = 1 or 2)
  OP_PRODBATCH = 5, // [op|n<<8][G|featTier<<8|dstTier<<10|grouped<<12] n*(dst, G*(feat, mean, shift, den))
                    //   n products of G Gaussian leaves each; the records are independent of each other.
                    //   Tiers as in OP_OUTERMM (0 short pool, 1 long pool, 2 mixed); grouped: in every full group
                    //   of four records the j-th leaves read the same feature
};

// How leaves obtain their feature value.
enum FeatureMode : uint32_t {
  FEAT_STAGED = 0,  // converted once per tile into reserved slots (feat fields hold slot numbers)
  FEAT_DIRECT = 1,  // read from the input row at each leaf (feat fields hold column numbers)
  FEAT_REGISTER = 2,  // converted once per tile into registers (feat fields hold register numbers; float programs whose
                      // features, at most 32, feed Gaussian leaves only). The staged list gives each register's column.
};

struct StagedFeature {
  uint32_t column;
  uint32_t valueSlot;  // slot of the value converted to the compute type (FEAT_REGISTER: the register number), or UINT32_MAX
  uint32_t indexSlot;  // slot of the clamped table index (raw u32 bits), or UINT32_MAX
  uint32_t tableLen;   // clamp bound L: indices >= L select the "impossible" entry, NaN selects L+1
};

struct InterpProgram {
  bool f64 = false;
  bool log2Domain = true;
  bool linear = false;                 // values are probabilities, not logarithms (the reference's computeInLogSpace=False); always f64
  FeatureMode featureMode = FEAT_STAGED;
  std::vector<uint32_t> code;
  std::vector<double> tables;          // pool of leaf tables in the kernel's log domain
  std::vector<uint32_t> directTableLen;  // FEAT_DIRECT: per column clamp bound (0 = none)
  std::vector<StagedFeature> staged;
  uint32_t numSlots = 0;      // value slots the program addresses, staged features included
  uint32_t shortSlots = 0;    // slots [0, shortSlots) are the busy ones; [shortSlots, numSlots) hold long-lived values
  uint32_t reservedSlots = 0; // leading slots pinned to staged features
  uint32_t numInstructions = 0;
  uint32_t mathTables = 0xFFFFFFFFu;  // float64 in the log2 domain: where in `tables` the 588 values of the exp2/log2 routines start
  uint32_t ldsSlotLimit = 0;  // "hip-interp-lds-slots": the launcher keeps at most this many slots in LDS (0 = as many as fit)
  uint32_t spillAccesses = 0; // slot words naming a long-lived slot: reads and writes of the spill tier per sample when only the short pool is in LDS
  std::string listing;        // human-readable form, for "dump-ir"
};

InterpProgram buildInterpProgram(const Graph& g, const CompileOptions& o);

// Throws std::runtime_error unless every slot, table, feature and weight access the kernel derives from the program
// stays in range (slot numbers and their tier flags, table offsets, feature columns, instruction lengths).
void checkInterpProgram(const InterpProgram& p, uint32_t numFeatures);

}  // namespace spnc_hip
