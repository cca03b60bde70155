// SPN query model: what the reader produces from a serialized query, and the validated,
// deduplicated, topologically scheduled DAG the kernel generators consume.
//
// Semantics follow the reference frontend
// (compiler/src/pipeline/steps/frontend/SPFlowToMLIRDeserializer.cpp:63-248) and the HiSPN
// verifiers (mlir/lib/Dialect/HiSPN/HiSPNOps.cpp:31-125).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace spnc_hip {

// External: inside one task of a partitioned graph, the value of a node that an earlier task computed (`feature` is its
// row in the intermediate buffer). Never appears in the graph of a whole query.
enum class NodeKind : uint8_t { Product = 0, Sum = 1, Histogram = 2, Gaussian = 3, Categorical = 4, External = 5 };

// A node exactly as serialized (ids, scope values).
struct RawNode {
  int32_t id = 0;
  NodeKind kind = NodeKind::Product;
  bool root = false;
  std::vector<int32_t> children;
  std::vector<double> weights;
  int32_t scope = -1;
  double mean = 0, stddev = 1;
  std::vector<double> probabilities;
  std::vector<int32_t> breaks;
  std::vector<double> densities;
};

struct RawModel {
  int32_t rootNode = 0;
  int32_t numFeatures = 0;
  std::string name, featureType;
  std::vector<int32_t> scope;
  std::vector<RawNode> nodes;
};

struct RawQuery {
  int32_t batchSize = 1;
  uint16_t errorKind = 0;
  double maxError = 0;
  bool supportMarginal = false;
  RawModel model;
};

// Reads a serialized query. Throws std::runtime_error with the reference's messages for raw
// models ("Cannot compile raw models"), queries without a joint ("Can only deserialize joint
// queries") and joints without a model ("No model attached to query").
RawQuery readQueryFile(const std::string& path);

enum class FeatureType : uint8_t { U8, U16, U32, U64, F32, F64 };

struct FeatureTypeInfo {
  FeatureType type;
  unsigned bytes;
  bool isFloat;
  const char* hipName;  // spelling of the type in generated device code
};
// Parses "[u]int<W>" / "float<W>"; integers are treated as unsigned of that width, as the
// reference does (uitofp / index_cast). Throws "Unsupported feature data type <text>".
FeatureTypeInfo parseFeatureType(const std::string& text);

// A DAG node after validation: children are indices into Graph::nodes (always smaller than
// the node's own index), leaves carry the input column and a flat linear-space table.
struct GraphNode {
  NodeKind kind;
  uint32_t feature = 0;            // input column (leaves)
  std::vector<uint32_t> children;  // inner nodes
  std::vector<double> weights;     // sums, linear space
  double mean = 0, stddev = 1;     // Gaussian
  std::vector<double> table;       // Categorical: probabilities; Histogram: flat [0,maxUB) densities, 0 in gaps
  uint32_t uses = 0;               // number of parents (root counts as one use)
};

struct GraphStats {
  uint32_t gaussians = 0, categoricals = 0, histograms = 0, products = 0, sums = 0;
  uint64_t productAdds = 0;   // sum over products of (k-1)
  uint64_t sumTerms = 0;      // sum over sums of k
  uint32_t maxFanIn = 0;
  uint32_t serializedNodes = 0;  // before dropping unreachable nodes and merging duplicates
  // Algorithmic work per sample: cheaper of pairwise tree (k==2) and n-ary LSE (k>=3) per sum,
  // 4 flops per Gaussian, 0 per table leaf, +1 select per leaf when marginal (Gaussian leaves that one product alone
  // reads: one add per four leaves and two selects per feature instead, which is what the float kernels do).
  uint64_t flopsMin = 0, transMin = 0, flopsPairwise = 0, transPairwise = 0;
  // Multiply-add pairs among flopsMin that one fused instruction computes in log space: a Gaussian leaf's
  // (d*d)*den + coef, and the add of a product for every Gaussian child that only this product reads
  // (den*(d*d + coef/den) + acc). Vector issue slots are priced without them, a transcendental at four slots.
  uint64_t fusedMin = 0;
  uint64_t issueSlotsMin() const { return flopsMin - fusedMin + 3 * transMin; }
};

// What the reference's "collect-graph-stats" pass reports (mlir/lib/Dialect/LoSPN/Passes/LoSPNGraphStatsCollection.cpp:44-97):
// operation counts of the binarised LoSPN graph right after the HiSPN lowering, i.e. before any merging of
// identical nodes, and the depths of its leaves.
struct LoSpnStats {
  uint64_t sumCount = 0;       // binary adds: k-1 per k-ary sum
  uint64_t productCount = 0;   // binary multiplies: k-1 per k-ary product and one per weighted sum term
  uint64_t constantCount = 0;  // weight constants: one per sum term
  uint64_t categoricalCount = 0, gaussianCount = 0, histogramCount = 0;
  uint64_t innerCount() const { return sumCount + productCount; }
  uint64_t leafCount() const { return categoricalCount + gaussianCount + histogramCount + constantCount; }  // constants count as leaves there
  int minDepth = 0, maxDepth = 0;
  double averageDepth = 0, medianDepth = 0;
  bool depthsExact = true;     // false: the graph shares so many nodes that the reference's path-by-path walk was replaced (see computeLoSpnStats)
};

// logSpace false adds the final log operation as the root of the depth count, as the reference's linear-space lowering does.
LoSpnStats computeLoSpnStats(const RawQuery& q, bool logSpace);

struct Graph {
  std::string name;
  FeatureTypeInfo ftype;
  uint32_t numFeatures = 0;
  bool supportMarginal = false;
  int32_t batchSize = 1;
  std::vector<GraphNode> nodes;  // children first; root is nodes.back()
  GraphStats stats;
  // Complete and decomposable: the children of every sum cover the same features, those of every product disjoint
  // ones. Then an input outside a table leaf's range makes the root's value log 0 whatever else the graph computes,
  // because every path from the root meets a leaf of that feature (what the kernels may rely on for such inputs).
  bool completeDecomposable = false;
  uint32_t root() const { return uint32_t(nodes.size() - 1); }
  // One task of a graph cut by "maxTaskSize": the values of `taskOutputs` go to rows `taskOutputSlots` of the intermediate
  // buffer ([rows][samples], value-major, so that the lanes of a wavefront touch consecutive addresses); the task that
  // holds the whole graph's root (`taskFinal`; the root is its last node) writes the result instead.
  bool isTask = false, taskFinal = false;
  std::vector<uint32_t> taskOutputs, taskOutputSlots;
};

// A graph cut into tasks that run one after the other, each a kernel of its own (the reference's
// mlir/lib/Dialect/LoSPN/Passes/LoSPNTaskPartitioner.cpp:36-148). `slots` rows of intermediate values are live at most.
struct TaskPlan {
  std::vector<Graph> tasks;
  uint32_t slots = 0;
};
// Operations of a node as the reference's partitioner counts them on the binarised graph: one per leaf, k-1 multiplies
// per k-ary product, k multiplies by the weights and k-1 adds per k-ary sum.
uint64_t taskWeight(const GraphNode& n);
uint64_t taskWeight(const Graph& g);
// Cuts `g` into tasks of at most `maxTaskSize` operations (plus 1 % slack, at least one). Sums and products that alone
// exceed the bound are first split into trees of smaller ones. One task (the graph itself, unmarked) if it fits.
TaskPlan partitionGraph(const Graph& g, int maxTaskSize);

// Validates the query and builds the scheduled DAG: only nodes reachable from the root,
// depth-first post-order (children first, left to right), structurally identical nodes merged.
// Throws std::runtime_error on every rule the reference rejects.
Graph buildGraph(const RawQuery& q);

}  // namespace spnc_hip
