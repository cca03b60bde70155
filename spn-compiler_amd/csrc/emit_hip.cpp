#include "emit_hip.h"

#include "math_tables.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <sstream>
#include <stdexcept>
#include <unordered_map>
#include <vector>

namespace spnc_hip {

namespace {

struct Emitter {
  const Graph& g;
  const CompileOptions& o;
  bool logSpace;
  bool f64;
  bool log2Dom;
  double scale;  // multiplies natural-log constants (log2(e) in the log2 domain)
  std::ostringstream body;
  std::vector<double> tablePool;
  std::vector<uint32_t> tableOffset;   // per node (for a paired leaf: offset of the joint table, held by the first of the pair)
  std::vector<uint32_t> partner;       // per node: the table leaf it shares a joint table with, or UINT32_MAX
  // Tables read with the same index (all leaves on one feature, all joint tables over one pair of features) are
  // interleaved in groups of four or two: entry i of the group holds the members' values for index i side by side,
  // and one 16- or 8-byte read fetches them all.
  struct TableGroup {
    uint32_t offset = 0, width = 1;      // pool offset in entries of the first member; members side by side per entry
    uint32_t stride = 1;                 // entries from one index value to the next: 4 in a block of four columns
    uint32_t fa = 0, fb = UINT32_MAX;    // index: t_fa, or t_fa * rowLen(fb) + t_fb for joint tables
    std::vector<uint32_t> members;       // table leaves (for a joint table: the first leaf of the pair), in node order
    bool loaded = false;
  };
  std::vector<TableGroup> groups;
  std::vector<uint32_t> groupOf, laneOf;  // per node (first leaf of a pair): its group and its position in the group's entries
  std::unordered_map<uint64_t, bool> jointIndexNamed;  // pairs of features whose joint index has been emitted
  std::vector<uint64_t> keyOrder;                                   // indices in order of first appearance
  std::unordered_map<uint64_t, std::vector<uint32_t>> unitsByKey;  // tables (joint tables: first leaf) per index
  bool packedIndices = false;                                       // blocks of four columns: byte offsets of the entries, four features to a register
  unsigned extractions = 0;                                         // numbers the statements that take a byte offset out of its register
  bool recording = false;                                           // first pass: only the order of table uses matters
  std::vector<uint32_t> useOrder, useRank;                          // tables in order of use; per table: its place in that order
  std::vector<uint32_t> featTableLen;  // per feature: longest table of any leaf on it (0 = none)
  std::vector<bool> featGauss;         // per feature: used by a Gaussian leaf
  // float64 log-space kernels: a Gaussian leaf inside a product is den (x - mean)^2 + coef = A x^2 + B x + C, evaluated
  // on per-feature x^2, x and 1 (all three zero for a missing feature) with one multiply-add per term, the constants as
  // scalar operands: three double-rate instructions per leaf where subtract, square-and-shift, mask (two registers)
  // and accumulate cost three double-rate and four single-rate ones; without marginalisation the C's of a product are
  // one constant and a leaf costs two. The expansion cancels where x is near the mean: its absolute error is about
  // 2^-52 |A| x^2 against 2^-52 |value| for the factored form, so it is used when, summed over the features, the
  // worst leaf of each feature keeps that below 1e-11 for inputs within eight standard deviations of the mean.
  bool expandedGauss = false;
  // Where the constants of the expanded leaves come from. A double constant as a scalar operand takes two scalar moves
  // with a literal each, and scalar instructions cost this kernel as much time as the multiply-adds they feed (measured:
  // 4.0 ns per term with them, 2.0 ns without, three wavefronts per SIMD). Instead a vector register pair holds sixteen
  // constants, lane l of every row of sixteen lanes the l-th (one coalesced 8-byte load per lane from a table in global
  // memory), and v_fmac_f64 reads the one it wants through its cross-lane operand (DPP row_newbcast:l), at the rate
  // of the plain instruction. All multiply-adds of a product sit in one assembler statement.
  bool laneConstants = false;
  std::vector<double> kPool;           // sixteen constants per vector, in order of use
  int kVectorsNamed = 0;               // vectors whose marker has been written into the body
  // With marginalisation the constant terms of a product's leaves depend on which of its features are missing. For
  // products of up to four expanded leaves the sum of the C's of the present features (plus the weight folded into the
  // product) is read from a table of 2^k entries in LDS, indexed by the pattern of present features, and is the
  // value the multiply-adds accumulate onto: one LDS read per product instead of one multiply-add per leaf.
  std::vector<double> cTables;
  std::vector<double> standIn;   // per feature: the value a missing input is replaced by when products take the leaves' offsets from a table
  bool marginalOffsets = false;
  std::map<std::vector<uint32_t>, std::string> patternNames;  // features of a product (in leaf order) -> variable with the pattern
  std::vector<bool> featUsed;
  std::vector<bool> featPrepared;
  std::vector<bool> emitted;
  std::unordered_map<uint32_t, double> foldedWeight;
  bool vectorRows = true;
  // Packed rows: the row reaches the kernel body as F/4 registers holding four features each, one byte per feature
  // (the value itself, saturated at 255). Table leaves that only their product reads are evaluated per group of sibling
  // products (the products under one sum that cover the same features), feature by feature: leaves over two or three
  // categories as polynomials in the feature's value (multiply-adds, no memory), the others from joint tables over pairs
  // of features in LDS, one index per pair for all siblings, whose entries lie side by side.
  bool packedRows = false;
  bool clampPacked = true;             // clamp the packed bytes to their tables' lengths before they index LDS
  std::vector<bool> featOneHot;        // per feature: its leaves are evaluated without memory accesses
  struct FusedUnit {
    uint32_t fa = 0, fb = UINT32_MAX;  // one feature, or a pair with a joint table
    uint32_t rowsA = 1, rowsB = 1;
    uint32_t base = 0, stride = 1;     // pool offset of the unit's table; entries per index (the siblings, padded to an even count)
    uint32_t plane = 0;                // sibling planes: elements from one sibling's table to the next (then stride is 1); 0 = siblings side by side
  };
  struct FusedGroup {
    std::vector<uint32_t> products;                    // the siblings
    std::vector<std::map<uint32_t, uint32_t>> leafOf;  // per sibling: feature -> leaf node
    std::vector<uint32_t> hot;                         // features evaluated from one-hot factors
    std::vector<FusedUnit> units;                      // features read from LDS
    bool emitted = false;
  };
  std::vector<FusedGroup> fusedGroups;
  std::vector<int> fusedGroupOf;       // per node: group of a product whose table leaves are evaluated this way, or -1
  std::vector<bool> fusedLeaf;         // per node: table leaf evaluated inside its product's group

  Emitter(const Graph& graph, const CompileOptions& opts) : g(graph), o(opts) {
    logSpace = o.useLogSpace;
    f64 = !logSpace || o.computeType == ComputeType::F64;
    log2Dom = logSpace && o.log2Domain;  // float: hardware exp2/log2; double: the short routines emitted with the kernel
    scale = log2Dom ? 1.4426950408889634074 : 1.0;
  }

  std::string lit(double v) const {
    if (std::isnan(v)) return f64 ? "__builtin_nan(\"\")" : "__builtin_nanf(\"\")";
    if (std::isinf(v)) {
      const char* inf = f64 ? "__builtin_huge_val()" : "__builtin_huge_valf()";
      return v < 0 ? std::string("(-") + inf + ")" : std::string(inf);
    }
    char buf[64];
    if (f64) {
      std::snprintf(buf, sizeof(buf), "%a", v);
    } else {
      std::snprintf(buf, sizeof(buf), "%af", double(float(v)));
    }
    std::string s(buf);
    return v < 0 ? "(" + s + ")" : s;
  }

  // log of a probability / weight, moved to the kernel's domain. Logs are taken in double and
  // rounded once to the compute type, as the reference does for its constants
  // (mlir/lib/Conversion/HiSPNtoLoSPN/NodePatterns.cpp:56-62,
  //  mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:120-138).
  double logConst(double p) const { return p > 0 ? std::log(p) * scale : -INFINITY; }

  static std::string v(uint32_t i) { return "v" + std::to_string(i); }

  template <typename Leaf, typename Comb>
  std::string tree(size_t lo, size_t hi, Leaf leaf, Comb comb) const {
    // Balanced binary tree with pivot ceil(k/2), left subtree first
    // (mlir/lib/Conversion/HiSPNtoLoSPN/NodePatterns.cpp:17-40,49-88).
    size_t k = hi - lo;
    if (k == 1) return leaf(lo);
    if (k == 2) {
      auto a = leaf(lo);  // sequenced: the callbacks emit code
      auto b = leaf(lo + 1);
      return comb(a, b);
    }
    size_t pivot = lo + (k + 1) / 2;
    auto l = tree(lo, pivot, leaf, comb);
    auto r = tree(pivot, hi, leaf, comb);
    return comb(l, r);
  }

  bool decideExpandedGauss() const {
    if (!(f64 && logSpace && log2Dom) || o.gaussExpanded == 0) return false;
    if (o.gaussExpanded == 1) return true;
    std::vector<double> worst(g.numFeatures, 0.0);
    for (const auto& n : g.nodes) {
      if (n.kind != NodeKind::Gaussian) continue;
      const double reach = std::fabs(n.mean) / n.stddev + 8.0;  // |x| / stddev at eight standard deviations
      worst[n.feature] = std::max(worst[n.feature], 0x1p-52 * 3.0 * 0.5 * scale * reach * reach);
    }
    double sum = 0.0;
    for (double w : worst) sum += w;
    return sum <= 1e-11;
  }

  // Missing features of float kernels, in products that evaluate their Gaussian leaves themselves ("hip-marginal-offsets"):
  // a missing value is replaced once per feature by a stand-in (the middle of the means of the feature's leaves), every
  // leaf is then evaluated without a select, and what the leaves over missing features added to the product, which
  // depends only on which of its features are missing, is taken off again with one value from a table in LDS (one
  // entry per pattern of missing features, four leaves to a table). A select per leaf is a quarter of such a
  // product's instructions. What is added and taken off again costs half an ulp of the running sum per leaf, so only
  // leaves whose value at the stand-in is small take part (at most 8 in magnitude, at most 32 per product together:
  // 1e-5 of error at worst); the others, narrow leaves far from the stand-in, keep their select.
  bool decideMarginalOffsets() {
    standIn.assign(g.numFeatures, 0.0);
    if (!(g.supportMarginal && logSpace && !f64 && o.marginalOffsets && o.marginalTablesKiB > 0)) return false;
    std::vector<double> lo(g.numFeatures, HUGE_VAL), hi(g.numFeatures, -HUGE_VAL);
    for (const auto& n : g.nodes)
      if (n.kind == NodeKind::Gaussian) lo[n.feature] = std::min(lo[n.feature], n.mean), hi[n.feature] = std::max(hi[n.feature], n.mean);
    for (uint32_t f = 0; f < g.numFeatures; ++f)
      if (lo[f] <= hi[f]) standIn[f] = double(float(0.5 * (lo[f] + hi[f])));
    return true;
  }
  // What a Gaussian leaf over a missing feature adds to its product when it is evaluated at the feature's stand-in,
  // from the constants as the kernel holds them (rounded to float: with a very narrow leaf next to the stand-in the
  // rounding of its mean alone moves the value by more than the results may differ). `folded`: the log-weight that rides
  // on this leaf's constant (the first leaf of a product); it stays in the product when the feature is missing.
  double offsetOf(const GraphNode& leaf, double folded = 0.0) const {
    const double den = -(1.0 / (2.0 * leaf.stddev * leaf.stddev)) * scale;
    const double coef = (-std::log(leaf.stddev) + -0.5 * std::log(2 * M_PI)) * scale;
    const double d = double(float(standIn[leaf.feature])) - double(float(leaf.mean));
    return double(float(den)) * (d * d + double(float(coef / den + folded / den))) - folded;
  }

  void prepare() {
    expandedGauss = decideExpandedGauss();
    laneConstants = expandedGauss && o.laneConstants;
    marginalOffsets = decideMarginalOffsets();
    featTableLen.assign(g.numFeatures, 0);
    featGauss.assign(g.numFeatures, false);
    featUsed.assign(g.numFeatures, false);
    featPrepared.assign(g.numFeatures, false);
    emitted.assign(g.nodes.size(), false);
    for (const auto& n : g.nodes) {
      if (n.kind == NodeKind::Gaussian) {
        featGauss[n.feature] = true;
        featUsed[n.feature] = true;
      } else if (n.kind == NodeKind::Categorical || n.kind == NodeKind::Histogram) {
        featTableLen[n.feature] = std::max<uint32_t>(featTableLen[n.feature], uint32_t(n.table.size()));
        featUsed[n.feature] = true;
      }
    }
    // Table pool: every table leaf on feature f owns L_f + 1 entries, its own values and then
    // "impossible" (log 0 / 0) up to index L_f for out-of-range inputs, plus, when the query
    // supports marginalisation, the marginal value (log 1 / 1) at L_f + 1 for NaN inputs.
    // The index is clamped once per feature.
    tableOffset.assign(g.nodes.size(), 0);
    partner.assign(g.nodes.size(), UINT32_MAX);
    fusedGroupOf.assign(g.nodes.size(), -1);
    fusedLeaf.assign(g.nodes.size(), false);
    featOneHot.assign(g.numFeatures, false);
    if (packedRows) planFusedGroups();
    auto isTable = [&](uint32_t c) { return g.nodes[c].kind == NodeKind::Categorical || g.nodes[c].kind == NodeKind::Histogram; };
    auto rowLen = [&](uint32_t feature) { return size_t(featTableLen[feature]) + (g.supportMarginal ? 2 : 1); };
    // Joint tables: two table leaves read only by the same product are replaced by one table over
    // the pair of indices, J[i][j] = T_a[i] (+ or *) T_b[j], combined in double. One LDS read and one
    // integer multiply-add then stand in for two LDS reads and one add; LDS reads are what bounds
    // table-heavy SPNs. Pairing stops when the pool would outgrow its LDS budget.
    const size_t realBytes = f64 ? 8 : 4, budget = size_t(o.tableBudgetKiB) * 1024;  // at most 62 KiB: LDS instruction offsets reach 64 KiB
    size_t plain = 0;
    for (uint32_t i = 0; i < g.nodes.size(); ++i)
      if (isTable(i)) plain += rowLen(g.nodes[i].feature);
    // Candidates: within a product, leaves ordered by table length and paired neighbour with
    // neighbour (small with small); globally the cheapest pairs are taken first.
    struct Candidate {
      size_t extra;
      uint32_t a, b;
    };
    std::vector<Candidate> candidates;
    for (uint32_t i = 0; i < g.nodes.size() && o.jointTables && !packedRows; ++i) {
      if (g.nodes[i].kind != NodeKind::Product) continue;
      std::vector<uint32_t> leaves;
      for (uint32_t c : g.nodes[i].children)
        if (isTable(c) && g.nodes[c].uses == 1) leaves.push_back(c);
      std::stable_sort(leaves.begin(), leaves.end(),
                       [&](uint32_t x, uint32_t y) { return rowLen(g.nodes[x].feature) < rowLen(g.nodes[y].feature); });
      for (size_t k = 0; k + 1 < leaves.size(); k += 2) {
        const size_t ra = rowLen(g.nodes[leaves[k]].feature), rb = rowLen(g.nodes[leaves[k + 1]].feature);
        if (ra * rb <= size_t(o.jointMaxEntries)) candidates.push_back({ra * rb - ra - rb, leaves[k], leaves[k + 1]});
      }
    }
    std::stable_sort(candidates.begin(), candidates.end(), [](const Candidate& x, const Candidate& y) { return x.extra < y.extra; });
    size_t projected = plain;
    for (const Candidate& c : candidates) {
      if ((projected + c.extra) * realBytes > budget) break;
      projected += c.extra;
      partner[c.a] = c.b;
      partner[c.b] = c.a;
    }
    // Units (single tables and joint tables) by index, in node order.
    for (uint32_t i = 0; i < g.nodes.size(); ++i) {
      if (!isTable(i) || fusedLeaf[i]) continue;
      if (partner[i] != UINT32_MAX && partner[i] < i) continue;  // second leaf of a pair: lives in the joint table
      const uint64_t fb = partner[i] == UINT32_MAX ? 0 : uint64_t(g.nodes[partner[i]].feature) + 1;
      const uint64_t key = o.groupedTables && !packedRows ? (uint64_t(g.nodes[i].feature) << 32) | fb : uint64_t(i);  // ungrouped: every table on its own
      if (!unitsByKey.count(key)) keyOrder.push_back(key);
      unitsByKey[key].push_back(i);
    }
    useRank.assign(g.nodes.size(), 0);
    if (o.groupedTables && !packedRows && !unitsByKey.empty()) recordUseOrder();
    buildPool();
    if (packedRows) appendFusedTables();
  }

  // ---- packed rows: groups of sibling products ----
  bool isTableLeaf(uint32_t c) const { return g.nodes[c].kind == NodeKind::Categorical || g.nodes[c].kind == NodeKind::Histogram; }
  // Entries per feature in the tables of the groups: no "impossible" entry. An input outside a feature's range is found
  // by a test of its own on the packed registers and makes the kernel return log 0; its clamped index reads one entry
  // past its table, inside the pool (which ends in padding), and whatever comes of that is dropped.
  uint32_t rowsOf(uint32_t feature) const { return featTableLen[feature]; }
  // Entries per index of a group's tables: the siblings' values side by side, padded to an even count so that two
  // of them are one aligned 8-byte (float) or 16-byte (double) LDS read.
  // The count of such reads per index is made odd: with an even count, entries 32 / count apart (or a fraction of
  // that) start in the same LDS bank, and lanes that read different entries of one table wait for each other (measured
  // on a graph with groups of four and eight siblings: 44 % of the LDS cycles were bank conflicts).
  static size_t fusedStride(size_t siblings) {
    if (siblings == 1) return 1;
    const size_t reads = (siblings + 1) / 2;
    return 2 * (reads | 1);
  }
  // The other layout, sibling planes ("hip-table-planes"): every sibling's table on its own, entry j of sibling s at
  // s * plane + j, read with one 4-byte (float) access per sibling, two siblings to an instruction. A wavefront's
  // 4-byte accesses are served 32 lanes at a time from 32 banks, so lanes that read different entries of a table wait
  // for each other only when the entries are a multiple of 32 apart; side by side, an 8-byte read covers 16 lanes at
  // a time and entries 16 / reads apart collide. Simulated on the 100-feature discrete graph with uniform inputs:
  // 41 % of the tables' LDS cycles are conflicts side by side (measured: 36 % of all LDS cycles), 24 % in planes.
  // The distance between planes keeps every sibling's offset within what one read instruction with two offsets can
  // name: 255 elements, or multiples of 64 elements.
  static size_t fusedPlane(size_t siblings, size_t entries) {
    if ((siblings - 1) * entries <= 255) return entries;
    return (entries + 63) / 64 * 64;
  }
  size_t fusedElements(size_t siblings, size_t entries) const {
    return o.tablePlanes && siblings > 1 ? siblings * fusedPlane(siblings, entries) : fusedStride(siblings) * entries;
  }

  void planFusedGroups() {
    std::vector<uint32_t> parent(g.nodes.size(), UINT32_MAX);
    for (uint32_t i = 0; i < g.nodes.size(); ++i)
      for (uint32_t c : g.nodes[i].children) parent[c] = i;
    // One-hot features: few categories, and every leaf on the feature has a finite value for each of them.
    for (uint32_t f = 0; f < g.numFeatures; ++f) featOneHot[f] = featTableLen[f] != 0 && featTableLen[f] <= uint32_t(o.oneHotMaxDomain);
    for (const auto& n : g.nodes) {
      if (n.kind != NodeKind::Categorical && n.kind != NodeKind::Histogram) continue;
      bool finite = n.table.size() == featTableLen[n.feature];
      for (double p : n.table) finite = finite && p > 0;
      if (!finite) featOneHot[n.feature] = false;
    }
    std::map<std::pair<uint32_t, std::vector<uint32_t>>, size_t> byKey;
    for (uint32_t i = 0; i < g.nodes.size(); ++i) {
      if (g.nodes[i].kind != NodeKind::Product) continue;
      std::map<uint32_t, uint32_t> own;  // feature -> leaf
      bool distinct = true;
      for (uint32_t c : g.nodes[i].children)
        if (isTableLeaf(c) && g.nodes[c].uses == 1) distinct = own.emplace(g.nodes[c].feature, c).second && distinct;
      if (own.empty() || !distinct) continue;
      std::vector<uint32_t> features;
      for (const auto& kv : own) features.push_back(kv.first);
      const bool underSum = g.nodes[i].uses == 1 && parent[i] != UINT32_MAX && g.nodes[parent[i]].kind == NodeKind::Sum;
      const auto key = std::make_pair(underSum ? parent[i] : uint32_t(g.nodes.size()) + i, features);
      auto it = byKey.find(key);
      if (it == byKey.end()) {
        it = byKey.emplace(key, fusedGroups.size()).first;
        FusedGroup G;
        std::vector<uint32_t> lds;
        for (uint32_t f : features) (featOneHot[f] ? G.hot : lds).push_back(f);
        std::stable_sort(lds.begin(), lds.end(), [&](uint32_t x, uint32_t y) { return rowsOf(x) < rowsOf(y); });
        for (size_t k = 0; k < lds.size();) {
          FusedUnit u;
          u.fa = lds[k];
          u.rowsA = rowsOf(lds[k]);
          if (o.jointTables && k + 1 < lds.size() && size_t(u.rowsA) * rowsOf(lds[k + 1]) <= size_t(o.jointMaxEntries)) {
            u.fb = lds[k + 1];
            u.rowsB = rowsOf(lds[k + 1]);
            k += 2;
          } else {
            k += 1;
          }
          G.units.push_back(u);
        }
        fusedGroups.push_back(std::move(G));
      }
      FusedGroup& G = fusedGroups[it->second];
      G.products.push_back(i);
      G.leafOf.push_back(own);
      fusedGroupOf[i] = int(it->second);
      for (const auto& kv : own) fusedLeaf[kv.second] = true;
    }
    // The joint tables must fit beside everything else in LDS: the largest pairs are split again until they do.
    size_t other = 0;
    for (uint32_t i = 0; i < g.nodes.size(); ++i)
      if (isTableLeaf(i) && !fusedLeaf[i]) other += rowsOf(g.nodes[i].feature);
    auto total = [&] {
      size_t t = other;
      for (const auto& G : fusedGroups)
        for (const auto& u : G.units) t += fusedElements(G.products.size(), size_t(u.rowsA) * u.rowsB);
      return t;
    };
    const size_t budget = size_t(o.tableBudgetGiven ? o.tableBudgetKiB : 96) * 1024 / (f64 ? 8 : 4);
    while (total() > budget) {
      FusedGroup* bestG = nullptr;
      size_t bestU = 0, bestGain = 0;
      for (auto& G : fusedGroups)
        for (size_t k = 0; k < G.units.size(); ++k) {
          const FusedUnit& u = G.units[k];
          if (u.fb == UINT32_MAX) continue;
          const size_t siblings = G.products.size();
          const size_t joint = fusedElements(siblings, size_t(u.rowsA) * u.rowsB), apart = fusedElements(siblings, u.rowsA) + fusedElements(siblings, u.rowsB);
          const size_t gain = joint > apart ? joint - apart : 0;
          if (gain > bestGain) bestGain = gain, bestG = &G, bestU = k;
        }
      if (!bestG) break;
      FusedUnit second;
      second.fa = bestG->units[bestU].fb;
      second.rowsA = bestG->units[bestU].rowsB;
      bestG->units[bestU].fb = UINT32_MAX;
      bestG->units[bestU].rowsB = 1;
      bestG->units.insert(bestG->units.begin() + bestU + 1, second);
    }
  }

  // Per unit one table whose entry `index` holds the values of all siblings side by side: one address serves them all
  // and two neighbours come with one read.
  void appendFusedTables() {
    auto padded = [&](uint32_t leaf) {
      const auto& n = g.nodes[leaf];
      std::vector<double> t;
      for (uint32_t j = 0; j < rowsOf(n.feature); ++j) t.push_back(logConst(j < n.table.size() ? n.table[j] : 0.0));
      return t;
    };
    // The bytes of a packed row are saturated at the longest table's length when the row is packed, so an index made of
    // unclamped bytes reaches at most `reach` entries past the start of its table. With that much padding behind the
    // pool no byte needs a clamp of its own: an input outside its feature's range makes the kernel return log 0
    // whatever the tables gave. When the padding would be large the bytes are clamped instead, and a clamped
    // out-of-range index reads at most one row of the first feature past its table.
    size_t largestRow = 0, reach = 0;
    for (auto& G : fusedGroups)
      for (auto& u : G.units) {
        const size_t k = G.products.size();
        const size_t entries = size_t(u.rowsA) * u.rowsB;
        const bool planes = o.tablePlanes && k > 1;
        u.stride = planes ? 1u : uint32_t(fusedStride(k));
        u.plane = planes ? uint32_t(fusedPlane(k, entries)) : 0u;
        if (tablePool.size() % 2) tablePool.push_back(0.0);
        u.base = uint32_t(tablePool.size());
        tablePool.resize(tablePool.size() + (planes ? k * u.plane : entries * u.stride), 0.0);
        for (size_t j = 0; j < k; ++j) {
          const std::vector<double> a = padded(G.leafOf[j].at(u.fa));
          const std::vector<double> b = u.fb == UINT32_MAX ? std::vector<double>{0.0} : padded(G.leafOf[j].at(u.fb));
          for (size_t x = 0; x < a.size(); ++x)
            for (size_t y = 0; y < b.size(); ++y)
              tablePool[planes ? u.base + j * u.plane + (x * b.size() + y) : u.base + (x * b.size() + y) * u.stride + j] = a[x] + b[y];
        }
        // how far past the pool's end an index made of unclamped (clamped) bytes can read, counted from the unit's last
        // element: with planes, the last sibling's table is the one at the end
        largestRow = std::max(largestRow, size_t(u.rowsB + 1) * u.stride);
        reach = std::max(reach, size_t(packedSaturation()) * size_t(u.rowsB + 1) * u.stride);
      }
    reach = std::max(reach, size_t(packedSaturation()) + 1);  // leaves outside the groups index their tables with the byte itself
    clampPacked = reach * (f64 ? 8 : 4) > 8192;
    if (!fusedGroups.empty()) tablePool.resize(tablePool.size() + (clampPacked ? largestRow : reach) + 2, 0.0);
  }
  // What a value is saturated at when a row is packed: the longest table's length, which is out of every feature's range.
  uint32_t packedSaturation() const {
    uint32_t longest = 1;
    for (uint32_t f = 0; f < g.numFeatures; ++f) longest = std::max(longest, featTableLen[f]);
    return longest;
  }

  unsigned extractions2 = 0;
  // The byte of feature f as a value of its own.
  // Written as a volatile statement: these stay in program order, so an index exists only from where the generator
  // put it. Left to the compiler, the extractions are merged or moved to the top of the kernel, and hundreds of
  // indices stay in registers (measured: 256 registers and 470 spilled ones against 140).
  std::string packedByte(uint32_t f) {
    const std::string name = "e" + std::to_string(extractions2++);
    body << "  unsigned " << name << ";\n  asm volatile(\"v_bfe_u32 %0, %1, " << 8 * (f % 4) << ", 8\" : \"=v\"(" << name << ") : \"v\"(PK" << f / 4 << "));\n";
    return name;
  }

  // What the kernel body starts with when rows are packed: the test for inputs outside their feature's range (in a
  // complete and decomposable graph such an input makes the result log 0, which the kernel returns at the end), the
  // clamp of the bytes where it is needed, and the values of the features whose leaves are polynomials.
  void emitPackedPrologue() {
    // Range test on the four bytes of a register at once: for a byte x and its length L <= 128,
    // ((x & 0x7f) + (0x80 - L)) | x has its top bit set exactly when x >= L (no carry leaves a byte).
    body << "  unsigned outsideBits = 0u;\n";
    for (uint32_t c = 0; c * 4 < g.numFeatures; ++c) {
      unsigned add = 0, keep = 0;
      for (uint32_t j = 0; j < 4 && c * 4 + j < g.numFeatures; ++j) {
        const uint32_t f = c * 4 + j;
        if (!featTableLen[f]) continue;
        keep |= 0xffu << (8 * j);
        add |= (0x80u - featTableLen[f]) << (8 * j);
      }
      if (!keep) continue;
      const std::string x = "R[" + std::to_string(c) + "]";
      body << "  outsideBits |= (((" << x << " & 0x7f7f7f7fu) + " << add << "u) | " << x << ")" << (keep != 0xffffffffu ? " & " + std::to_string(keep) + "u" : std::string())
           << ";\n";
    }
    body << "  const bool outside = (outsideBits & 0x80808080u) != 0u;\n";
    // Clamp: every byte to its feature's length, the register put together again. Written as instructions, and none
    // of them one that selects bytes by itself (SDWA): a SIMD overlaps nothing with those. Left out when even an index
    // made of arbitrary bytes stays inside the kernel's LDS: what such a read returns is dropped.
    for (uint32_t c = 0; c * 4 < g.numFeatures; ++c) {
      bool any = false;
      for (uint32_t j = 0; j < 4 && c * 4 + j < g.numFeatures; ++j) any = any || featTableLen[c * 4 + j];
      if (!any) continue;
      body << "  unsigned PK" << c << " = R[" << c << "];\n";
      if (!clampPacked) continue;
      std::string text, operands;
      unsigned operand = 3;
      for (int j = 3; j >= 0; --j) {   // %0 the result, %1 a byte, %2 the packed register
        const uint32_t f = c * 4 + uint32_t(j);
        const uint32_t len = f < g.numFeatures && featTableLen[f] ? featTableLen[f] : 255u;
        text += j == 3 ? "v_lshrrev_b32 %1, 24, %2\\n\\t" : j == 0 ? "v_and_b32 %1, 0xff, %2\\n\\t" : "v_bfe_u32 %1, %2, " + std::to_string(8 * j) + ", 8\\n\\t";
        std::string limit = std::to_string(len);
        if (len > 64) {
          limit = "%" + std::to_string(operand++);
          operands += ", \"s\"(" + std::to_string(len) + "u)";
        }
        text += std::string("v_min_u32 ") + (j == 3 ? "%0" : "%1") + ", " + limit + ", %1" + (j == 3 ? "" : "\\n\\tv_lshl_or_b32 %0, %0, 8, %1") + (j ? "\\n\\t" : "");
      }
      body << "  {\n    unsigned spn_q, spn_t;\n    asm(\"" << text << "\" : \"=&v\"(spn_q), \"=&v\"(spn_t) : \"v\"(PK" << c << ")" << operands << ");\n    PK" << c
           << " = spn_q;\n  }\n";
    }
    for (uint32_t f = 0; f < g.numFeatures && o.hoistFeatureValues; ++f)
      if (featOneHot[f]) emitFeatureValues(f, "");
  }

  // x (and x squared, or the 0/1 factors [x == c]) of a feature whose leaves are evaluated without memory accesses.
  void emitFeatureValues(uint32_t f, const std::string& suffix) {
    const char* one = f64 ? "1.0" : "1.0f";
    const char* zero = f64 ? "0.0" : "0.0f";
    const uint32_t d = featTableLen[f];
    const std::string v = "h" + std::to_string(f) + "_1" + suffix;
    if (!f64 && !suffix.empty())  // inside a group: as a volatile statement, or the compiler computes all of them at the top of the kernel again
      body << "  real_t " << v << ";\n  asm volatile(\"v_cvt_f32_ubyte" << f % 4 << " %0, %1\" : \"=v\"(" << v << ") : \"v\"(PK" << f / 4 << "));\n";
    else
      body << "  const real_t " << v << " = (real_t)((PK" << f / 4 << " >> " << 8 * (f % 4) << ") & 255u);\n";  // one instruction: byte to float
    if (d == 3) body << "  const real_t h" << f << "_2" << suffix << " = " << v << " * " << v << ";\n";
    for (uint32_t c = 2; d > 3 && c < d; ++c)
      body << "  const real_t h" << f << "_" << c << suffix << " = " << v << " == " << lit(double(c)) << " ? " << one << " : " << zero << ";\n";
  }

  // The table leaves of a group of sibling products, into one accumulator per sibling (named pt<product>).
  bool midpointHook = false;      // the body calls spn_mid() once, about half-way through its work (the row prefetch turns round there)
  bool midpointEmitted = false;
  size_t fusedWorkDone = 0;
  static size_t workOf(const FusedGroup& G) { return G.products.size() * (G.units.size() + 2 * G.hot.size()); }

  void emitFusedGroup(FusedGroup& G) {
    G.emitted = true;
    const size_t k = G.products.size();
    if (midpointHook && !midpointEmitted) {
      size_t total = 0;
      for (const auto& other : fusedGroups) total += workOf(other);
      if (2 * fusedWorkDone >= total) {
        body << "  spn_mid();\n";
        midpointEmitted = true;
      }
    }
    fusedWorkDone += workOf(G);
    const size_t realBytes = f64 ? 8 : 4;
    const char* fma = f64 ? "__builtin_fma(" : "__builtin_fmaf(";
    // Few siblings mean few independent chains of dependent adds, and with two wavefronts per SIMD nothing else hides
    // the latency of a vector instruction: each sibling's sum is then split over several partial accumulators.
    const size_t parts = k >= 4 ? 1 : (k == 3 ? 2 : (k == 2 ? 2 : 4));
    std::vector<std::vector<std::string>> acc(k);
    std::vector<std::string> allAcc;
    std::vector<size_t> turn(k, 0);
    for (size_t j = 0; j < k; ++j) {
      double base = 0;
      for (uint32_t f : G.hot) base += logConst(g.nodes[G.leafOf[j].at(f)].table[0]);
      for (size_t q = 0; q < parts; ++q) {
        acc[j].push_back("pt" + std::to_string(G.products[j]) + (q ? "_" + std::to_string(q) : std::string()));
        body << "  real_t " << acc[j].back() << " = " << lit(q ? 0.0 : base) << ";\n";
        allAcc.push_back(acc[j].back());
      }
      for (const auto& kv : G.leafOf[j]) emitted[kv.second] = true;
    }
    auto next = [&](size_t j) -> const std::string& { return acc[j][turn[j]++ % parts]; };
    // Work that needs no memory. A leaf over two or three categories is the polynomial through its values at x = 0, 1
    // (and 2): value(0) is part of the accumulator's start, the rest is one multiply-add per power of x. A leaf over
    // more categories (on request) is value(0) + (value(1) - value(0)) x plus one correction per category c >= 2,
    // multiplied with the 0/1 factor [x == c].
    std::vector<std::string> hotWork;
    const std::string suffix = o.hoistFeatureValues ? std::string() : "_g" + std::to_string(G.products[0]);
    for (uint32_t f : G.hot) {
      const uint32_t d = featTableLen[f];
      if (!o.hoistFeatureValues) emitFeatureValues(f, suffix);
      for (size_t j = 0; j < k; ++j) {
        const auto& t = g.nodes[G.leafOf[j].at(f)].table;
        const double v0 = logConst(t[0]), v1 = logConst(t[1]);
        std::vector<double> factor(d, 0.0);  // coefficient of h<f>_<c>
        if (d == 2) {
          factor[1] = v1 - v0;
        } else if (d == 3) {
          const double v2 = logConst(t[2]);
          factor[2] = (v2 - 2 * v1 + v0) / 2;
          factor[1] = v1 - v0 - factor[2];
        } else {
          // x = h_1 is the value itself: value(x) = v0 + (v1 - v0) * x + sum over c >= 2 of (v_c - v0 - c (v1 - v0)) [x == c]
          factor[1] = v1 - v0;
          for (uint32_t c = 2; c < d; ++c) factor[c] = logConst(t[c]) - v0 - double(c) * factor[1];
        }
        for (uint32_t c = 1; c < d; ++c) {
          const std::string& a = next(j);
          hotWork.push_back("  " + a + " = " + fma + "h" + std::to_string(f) + "_" + std::to_string(c) + suffix + ", " + lit(factor[c]) + ", " + a + ");\n");
        }
      }
    }
    // LDS reads in batches: the indices and reads of a batch are issued, then the values of the batch before are
    // added (and a share of the other work done) while they travel.
    const int fusedBatch = o.fusedBatch >= 0 ? o.fusedBatch : (midpointHook ? 2 : 4);
    const size_t batch = size_t(std::max(1, fusedBatch)), batches = (G.units.size() + batch - 1) / batch;
    const bool barriers = fusedBatch > 0;
    const size_t hotShare = batches ? (hotWork.size() + batches - 1) / batches : hotWork.size();
    size_t hotDone = 0;
    std::vector<std::string> pendingAdds;
    // Empty volatile statements that take the accumulators in and out: volatile statements keep their order (the
    // index computations are volatile too), so the adds between two of these pins stay between this batch's reads and
    // the next batch's indices. A scheduling barrier alone does not bind the compiler before instruction selection.
    auto pin = [&] {
      for (const std::string& a : allAcc) body << "  asm volatile(\"\" : \"+v\"(" << a << "));\n";
      body << "  __builtin_amdgcn_sched_barrier(0);\n";
    };
    for (size_t b0 = 0; b0 < G.units.size(); b0 += batch) {
      std::vector<std::string> adds;
      for (size_t q = b0; q < std::min(G.units.size(), b0 + batch); ++q) {
        const FusedUnit& u = G.units[q];
        // LDS address of the unit's entry: table + (a * rowsB + b) * stride * sizeof(real_t), as one statement: the bytes
        // of the two features are taken out of their packed registers, a 16-bit multiply-add makes the joint index and
        // another one scales it and brings in the table's address, so that every read of the unit is this register plus
        // a constant offset. (Left to the compiler, the address of nearly every read got an add of its own.)
        // None of these is an SDWA, DPP or 24-bit-multiply instruction: on gfx950 a SIMD issues one of those in the
        // time of about four plain instructions and overlaps nothing with it, while the ones used here issue every
        // other cycle when they alternate with the additions of the wavefront beside them (measured with two
        // wavefronts per SIMD: v_add_f32 alternating with v_mul_u32_u24_sdwa 2.2 ns per instruction, with v_bfe_u32
        // or v_mad_u32_u16 1.05 ns).
        const std::string idx = "a" + std::to_string(extractions2++);
        const size_t unitBytes = size_t(u.base) * realBytes;
        std::string operands;   // scalar operands of the statement, numbered from `next`
        unsigned nextOperand = u.fb != UINT32_MAX ? 4 : 2;
        // A small integer is written into the instruction; anything else takes a register of the kind asked for.
        auto constant = [&](size_t value, const char* kind) {
          if (value <= 64) return std::to_string(value);
          operands += std::string(", \"") + kind + "\"(" + std::to_string(value) + "u)";
          return "%" + std::to_string(nextOperand++);
        };
        auto extract = [&](const char* dst, const char* src, uint32_t f) {
          const unsigned byte = f % 4;
          if (byte == 0) return std::string("v_and_b32 ") + dst + ", 0xff, " + src + "\\n\\t";
          if (byte == 3) return std::string("v_lshrrev_b32 ") + dst + ", 24, " + src + "\\n\\t";
          return std::string("v_bfe_u32 ") + dst + ", " + src + ", " + std::to_string(8 * byte) + ", 8\\n\\t";
        };
        const size_t strideBytes = size_t(u.stride) * realBytes;
        if (u.fb != UINT32_MAX) {
          std::string text = extract("%0", "%2", u.fa) + extract("%1", "%3", u.fb);
          text += "v_mad_u32_u16 %0, %0, " + constant(u.rowsB, "s") + ", %1\\n\\t";
          const std::string scale = constant(strideBytes, "s");   // an instruction reads one scalar register at most
          operands += std::string(", \"") + (strideBytes <= 64 ? "s" : "v") + "\"(spn_tab_lds + " + std::to_string(unitBytes) + "u)";
          text += "v_mad_u32_u16 %0, %0, " + scale + ", %" + std::to_string(nextOperand++);
          body << "  unsigned " << idx << ", " << idx << "b;\n  asm volatile(\"" << text << "\" : \"=&v\"(" << idx << "), \"=&v\"(" << idx << "b) : \"v\"(PK"
               << u.fa / 4 << "), \"v\"(PK" << u.fb / 4 << ")" << operands << ");\n";
        } else {
          std::string text = extract("%0", "%1", u.fa);
          const std::string scale = constant(strideBytes, "s");
          operands += std::string(", \"") + (strideBytes <= 64 ? "s" : "v") + "\"(spn_tab_lds + " + std::to_string(unitBytes) + "u)";
          text += "v_mad_u32_u16 %0, %0, " + scale + ", %" + std::to_string(nextOperand++);
          body << "  unsigned " << idx << ";\n  asm volatile(\"" << text << "\" : \"=&v\"(" << idx << ") : \"v\"(PK" << u.fa / 4 << ")" << operands << ");\n";
        }
        for (size_t j = 0; j < k && u.plane; ++j) {   // sibling planes: one value per read (the compiler pairs the reads into instructions with two offsets)
          const std::string r = "r" + std::to_string(extractions2++);
          body << "  const real_t " << r << " = *reinterpret_cast<const __attribute__((address_space(3))) real_t*>(" << idx << " + " << j * u.plane * realBytes << "u);\n";
          adds.push_back("  " + next(j) + " += " + r + ";\n");
        }
        for (size_t j = 0; j < k && !u.plane; j += 2) {
          const std::string r = "r" + std::to_string(extractions2++);
          const std::string address = idx + " + " + std::to_string(j * realBytes) + "u";
          if (u.stride == 1) {
            body << "  const real_t " << r << " = *reinterpret_cast<const __attribute__((address_space(3))) real_t*>(" << address << ");\n";
            adds.push_back("  " + next(j) + " += " + r + ";\n");
          } else {
            body << "  const spn_r2 " << r << " = *reinterpret_cast<const __attribute__((address_space(3))) spn_r2*>(" << address << ");\n";
            adds.push_back("  " + next(j) + " += " + r + "[0];\n");
            if (j + 1 < k) adds.push_back("  " + next(j + 1) + " += " + r + "[1];\n");
          }
        }
      }
      if (!barriers) {  // plain order: every unit's values are added right after its reads
        for (const std::string& a : adds) body << a;
        for (size_t q = 0; q < hotShare && hotDone < hotWork.size(); ++q) body << hotWork[hotDone++];
        continue;
      }
      pin();
      for (const std::string& a : pendingAdds) body << a;
      for (size_t q = 0; q < hotShare && hotDone < hotWork.size(); ++q) body << hotWork[hotDone++];
      pin();
      pendingAdds = std::move(adds);
    }
    for (const std::string& a : pendingAdds) body << a;
    while (hotDone < hotWork.size()) body << hotWork[hotDone++];
    for (size_t j = 0; j < k; ++j)
      for (size_t q = 1; q < parts; ++q) body << "  " << acc[j][0] << " += " << acc[j][q] << ";\n";
  }

  std::vector<double> unitValues(uint32_t i) const {
    auto padded = [&](uint32_t c) {
      const auto& n = g.nodes[c];
      const uint32_t L = featTableLen[n.feature];
      std::vector<double> t;
      for (uint32_t j = 0; j <= L; ++j) {
        double p = j < n.table.size() ? n.table[j] : 0.0;
        t.push_back(logSpace ? logConst(p) : p);
      }
      if (g.supportMarginal) t.push_back(logSpace ? 0.0 : 1.0);
      return t;
    };
    std::vector<double> a = padded(i);
    if (partner[i] == UINT32_MAX) return a;
    std::vector<double> b = padded(partner[i]), joint;
    for (double x : a)
      for (double y : b) joint.push_back(logSpace ? x + y : x * y);
    return joint;
  }

  // Groups of four, two and one over the units of every index, in the order the lists hold them, and the pool.
  void buildPool() {
    const size_t realBytes = f64 ? 8 : 4, limit = (size_t(o.tableBudgetKiB) + size_t(o.tablePadKiB)) * 1024;
    bool shared = false;
    for (const auto& kv : unitsByKey) shared = shared || kv.second.size() > 1;
    // Blocks of four columns go with packed indices: the byte offset of a feature's entry, index * 4 * sizeof(real_t),
    // must fit into eight bits, and the indices must all be at hand when the kernel body starts.
    for (uint32_t f = 0; f < g.numFeatures; ++f)
      if (featTableLen[f] && (featTableLen[f] + (g.supportMarginal ? 1u : 0u)) * 4 * realBytes > 255) shared = false;
    if (!vectorRows || !o.eagerIndices) shared = false;
    size_t reads = 0;
    for (const auto& kv : unitsByKey) reads += kv.second.size();
    if (reads < size_t(o.tableGroupMinReads)) shared = false;  // too few reads for the LDS to matter
    packedIndices = false;
    for (int attempt = shared ? 0 : 1; attempt < 2; ++attempt) {
      const bool blocks = attempt == 0;  // else every table on its own, entries side by side
      groups.clear();
      tablePool.clear();
      groupOf.assign(g.nodes.size(), UINT32_MAX);
      laneOf.assign(g.nodes.size(), 0);
      for (uint64_t key : keyOrder) {
        const std::vector<uint32_t>& list = unitsByKey[key];
        const size_t rows = unitValues(list[0]).size(), firstGroup = groups.size();
        for (size_t pos = 0; pos < list.size();) {
          size_t count = 1;
          while (blocks && count < 4 && pos + count < list.size() &&
                 useRank[list[pos + count]] - useRank[list[pos]] <= uint32_t(o.tableGroupWindow))
            ++count;
          TableGroup G;
          G.width = uint32_t(count);
          G.stride = blocks ? 4 : 1;
          G.fa = g.nodes[list[pos]].feature;
          G.fb = partner[list[pos]] == UINT32_MAX ? UINT32_MAX : g.nodes[partner[list[pos]]].feature;
          for (size_t k = 0; k < count; ++k) {
            groupOf[list[pos + k]] = uint32_t(groups.size());
            laneOf[list[pos + k]] = uint32_t(k);
            G.members.push_back(list[pos + k]);
          }
          groups.push_back(G);
          pos += count;
        }
        // Columns: groups of four and three open a block of their own, pairs take a half, single tables whatever
        // is free (the fourth column beside three tables first).
        const size_t base = tablePool.size();
        std::vector<uint32_t> freeColumns;  // per block of this index: bit c set = column c is free
        auto place = [&](TableGroup& G, size_t block, uint32_t column) {
          if (block == freeColumns.size()) {
            freeColumns.push_back(0xfu);
            tablePool.resize(tablePool.size() + rows * G.stride, 0.0);
          }
          for (uint32_t c = 0; c < G.width; ++c) freeColumns[block] &= ~(1u << (column + c));
          G.offset = uint32_t(base + block * rows * G.stride + column);
          for (size_t m = 0; m < G.members.size(); ++m) {
            const std::vector<double> col = unitValues(G.members[m]);
            for (size_t r = 0; r < rows; ++r) tablePool[G.offset + r * G.stride + m] = col[r];
            tableOffset[G.members[m]] = G.offset;
          }
        };
        for (uint32_t width : {4u, 3u, 2u, 1u}) {
          for (size_t k = firstGroup; k < groups.size(); ++k) {
            TableGroup& G = groups[k];
            if (G.width != width) continue;
            if (!blocks) {
              G.offset = uint32_t(tablePool.size());
              tablePool.resize(tablePool.size() + rows, 0.0);
              const std::vector<double> col = unitValues(G.members[0]);
              std::copy(col.begin(), col.end(), tablePool.begin() + G.offset);
              tableOffset[G.members[0]] = G.offset;
              continue;
            }
            size_t block = freeColumns.size();
            uint32_t column = 0;
            for (size_t q = 0; q < freeColumns.size() && block == freeColumns.size() && width <= 2; ++q) {
              if (width == 2 && (freeColumns[q] & 0xcu) == 0xcu) block = q, column = 2;
              for (uint32_t c = 4; c-- > 0 && width == 1;)
                if (freeColumns[q] & (1u << c)) block = q, column = c;
            }
            place(G, block, column);
          }
        }
      }
      if (blocks && tablePool.size() * realBytes <= limit) packedIndices = true;
      if (!blocks || packedIndices) break;  // blocks that outgrow the LDS share: plain tables
    }
  }

  // A group's vector stays in registers from its read, at the first member's use, to the last member's use. The
  // members of a group are therefore tables of its index that the kernel needs shortly after one another (the
  // children of one sum, as a rule): a first pass over the graph records the order in which the tables are used.
  void recordUseOrder() {
    recording = true;
    emitNode(g.root());
    recording = false;
    useRank.assign(g.nodes.size(), UINT32_MAX);
    for (size_t k = 0; k < useOrder.size(); ++k)
      if (useRank[useOrder[k]] == UINT32_MAX) useRank[useOrder[k]] = uint32_t(k);
    for (auto& kv : unitsByKey)
      std::stable_sort(kv.second.begin(), kv.second.end(), [&](uint32_t x, uint32_t y) { return useRank[x] < useRank[y]; });
    body.str("");
    body.clear();
    kPool.clear();
    kVectorsNamed = 0;
    cTables.clear();
    patternNames.clear();
    std::fill(emitted.begin(), emitted.end(), false);
    std::fill(featPrepared.begin(), featPrepared.end(), false);
    foldedWeight.clear();
    jointIndexNamed.clear();
    useOrder.clear();
  }

  // Packed indices: register P<k> holds, for features 4k .. 4k+3, the byte offset of the feature's entry within a
  // block of four columns (index * 4 * sizeof(real_t)), eight bits each. An offset is taken out where a group is
  // read, by a statement of its own every time (the number in its comment keeps the compiler from merging them):
  // merged, a hundred offsets would stay in registers for the whole kernel, which is what the packing is there
  // to avoid.
  void emitPackedIndices() {
    const unsigned entryBytes = 4 * (f64 ? 8 : 4);
    for (uint32_t k = 0; k * 4 < g.numFeatures; ++k) {
      std::string expr;
      for (uint32_t j = 0; j < 4 && k * 4 + j < g.numFeatures; ++j) {
        const uint32_t f = k * 4 + j;
        if (!featUsed[f] || !featTableLen[f]) continue;
        expr += (expr.empty() ? "" : " | ") + std::string("((t") + std::to_string(f) + " * " + std::to_string(entryBytes) + "u) << " + std::to_string(8 * j) + ")";
      }
      if (!expr.empty()) body << "  const unsigned P" << k << " = " << expr << ";\n";
    }
  }
  std::string byteOffset(uint32_t f) {
    const std::string name = "b" + std::to_string(extractions);
    body << "  unsigned " << name << ";\n  asm(\"v_bfe_u32 %0, %1, " << 8 * (f % 4) << ", 8 ; " << extractions << "\" : \"=v\"(" << name << ") : \"v\"(P" << f / 4 << "));\n";
    ++extractions;
    return name;
  }

  // The index expression of a group: the clamped feature index, or the named joint index of its two features
  // (packed indices: the byte offset of the entry).
  std::string groupIndex(const TableGroup& G) {
    if (packedIndices) {
      const std::string a = byteOffset(G.fa);
      if (G.fb == UINT32_MAX) return a;
      const std::string b = byteOffset(G.fb);
      return "(" + a + " * " + std::to_string(featTableLen[G.fb] + (g.supportMarginal ? 2 : 1)) + "u + " + b + ")";
    }
    if (G.fb == UINT32_MAX) return "t" + std::to_string(G.fa);
    const std::string name = "k" + std::to_string(G.fa) + "_" + std::to_string(G.fb);
    const uint64_t key = (uint64_t(G.fa) << 32) | G.fb;
    if (!jointIndexNamed[key]) {
      jointIndexNamed[key] = true;
      body << "  const unsigned " << name << " = t" << G.fa << " * " << (featTableLen[G.fb] + (g.supportMarginal ? 2 : 1)) << "u + t" << G.fb << ";\n";
    }
    return name;
  }

  // The value of table unit i (a table leaf, or the first leaf of a pair): a plain read for a table on its own,
  // else a component of its group's vector, which is read where its first member is needed.
  std::string tableValue(uint32_t i) {
    if (recording) {
      useOrder.push_back(i);
      return "0";
    }
    TableGroup& G = groups[groupOf[i]];
    if (packedIndices) {
      const std::string q = "q" + std::to_string(groupOf[i]);
      if (!G.loaded) {
        G.loaded = true;
        const std::string idx = groupIndex(G);
        const char* type = G.width == 1 ? "real_t" : (G.width == 2 ? "spn_r2" : "spn_r4");  // three tables: the fourth column comes along unused
        body << "  const " << type << " " << q << " = *reinterpret_cast<const " << type << "*>(reinterpret_cast<const char*>(tab + " << G.offset
             << "u) + " << idx << ");\n";
      }
      return G.width == 1 ? q : q + "[" + std::to_string(laneOf[i]) + "]";
    }
    if (G.fb == UINT32_MAX) return "tab[" + std::to_string(G.offset) + "u + t" + std::to_string(G.fa) + "]";
    return "tab[" + std::to_string(G.offset) + "u + t" + std::to_string(G.fa) + " * " +
           std::to_string(featTableLen[G.fb] + (g.supportMarginal ? 2 : 1)) + "u + t" + std::to_string(G.fb) + "]";
  }

  // Emitted right before the first leaf that reads feature f, so that for wide rows the load
  // sits next to its first use instead of at the top of a very long basic block.
  void emitFeaturePrep(uint32_t f) {
    const bool isFloat = g.ftype.isFloat;
    {
      if (featPrepared[f]) return;
      featPrepared[f] = true;
      if (packedRows) {  // a leaf outside the groups: the clamped index itself
        const std::string x = packedByte(f);
        body << "  const unsigned t" << f << " = " << x << ";\n";
        return;
      }
      std::string x = "x[" + std::to_string(f) + "]";
      if (!vectorRows) {
        body << "  const feat_t x" << f << " = SPN_LOAD(row + " << f << ");\n";
        x = "x" + std::to_string(f);
      }
      if (featGauss[f]) body << "  const real_t g" << f << " = (real_t)" << x << ";\n";
      if (featGauss[f] && expandedGauss) {
        // x, x^2 and 1 of the expanded leaves; a missing feature zeroes all three, and with them every leaf over it
        if (g.supportMarginal)
          body << "  const bool gn" << f << " = g" << f << " != g" << f << ";\n  const real_t gx" << f << " = gn" << f << " ? 0.0 : g" << f
               << ";\n  const real_t go" << f << " = gn" << f << " ? 0.0 : 1.0;\n";
        else
          body << "  const real_t gx" << f << " = g" << f << ";\n";
        body << "  const real_t gq" << f << " = gx" << f << " * gx" << f << ";\n";
      }
      if (featGauss[f] && marginalOffsets)
        body << "  const bool gn" << f << " = g" << f << " != g" << f << ";\n  const real_t gz" << f << " = gn" << f << " ? " << lit(standIn[f]) << " : g" << f << ";\n";
      if (featGauss[f] && nanMasks()) {
        // All ones, or zero when the feature is missing. The empty assembler statement hides where the value came from:
        // otherwise the compiler turns every AND with it back into a select.
        body << "  unsigned gm" << f << " = (g" << f << " != g" << f << ") ? 0u : ~0u;\n  asm(\"\" : \"+v\"(gm" << f << "));\n";
      }
      if (featTableLen[f]) {
        uint32_t L = featTableLen[f];
        if (isFloat) {
          // fptoui-style truncation, guarded: anything outside [0, L) selects the "impossible" entry.
          body << "  unsigned t" << f << " = (" << x << " > (feat_t)-1 && " << x << " < (feat_t)" << L << ") ? (unsigned)"
               << x << " : " << L << "u;\n";
          if (g.supportMarginal) body << "  t" << f << " = (" << x << " != " << x << ") ? " << (L + 1) << "u : t" << f << ";\n";
        } else {
          // Compared in a type at least as wide as both sides: the table length cast to a narrow feature type
          // would wrap (256 entries on an 8-bit feature).
          const char* wide = g.ftype.bytes > 4 ? "(unsigned long long)" : "(unsigned)";
          body << "  const unsigned t" << f << " = (" << wide << x << " < " << L << (g.ftype.bytes > 4 ? "ull" : "u") << ") ? (unsigned)" << x
               << " : " << L << "u;\n";
        }
      }
    }
  }

  // The log2-domain f32 kernel uses the hardware exp2/log2 instructions directly. The other
  // flavours call the accurate library routines through out-of-line wrappers: inlining them
  // thousands of times into one basic block makes register allocation take minutes.
  std::string expOf(const std::string& a) const {
    return (log2Dom ? (f64 ? "spn_exp2(" : "__builtin_amdgcn_exp2f(") : "spn_exp(") + a + ")";
  }
  std::string logOf(const std::string& a) const {
    return (log2Dom ? (f64 ? "spn_log2(" : "__builtin_amdgcn_logf(") : "spn_log(") + a + ")";
  }
  std::string maxOf(const std::string& a, const std::string& b) const {
    // Values that come out of assembler statements (products with lane constants) are not known to be quieted NaNs to
    // the compiler, which then puts a canonicalising v_max_f64 x, x in front of every maximum that takes them; the
    // instruction itself has fmax semantics, so those kernels call it directly.
    if (laneConstants) return "spn_max(" + a + ", " + b + ")";
    return std::string(f64 ? "__builtin_fmax(" : "__builtin_fmaxf(") + a + ", " + b + ")";
  }

  void emitLeafMarginal(uint32_t i, const std::string& expr) {
    const auto& n = g.nodes[i];
    if (nanMasks()) {
      body << "  const real_t " << v(i) << " = " << masked(expr, n.feature) << ";\n";
    } else if (g.supportMarginal) {
      std::string x = "g" + std::to_string(n.feature);
      body << "  const real_t " << v(i) << " = (" << x << " != " << x << ") ? " << lit(logSpace ? 0.0 : 1.0) << " : (" << expr
           << ");\n";
    } else {
      body << "  const real_t " << v(i) << " = " << expr << ";\n";
    }
  }

  // Missing features in log space: the leaf's value becomes log 1 = +0.0 by clearing all its bits, one AND per register
  // (full rate) where a select costs a half-rate instruction per register plus moves for its constants.
  bool nanMasks() const { return g.supportMarginal && logSpace && f64 && o.nanMasks; }  // float kernels are faster with selects (measured: 2.07 against 2.58 ms on the 16-feature Gaussian tree)
  std::string masked(const std::string& expr, uint32_t feature) const { return "spn_mask(" + expr + ", gm" + std::to_string(feature) + ")"; }

  // A Gaussian leaf read by exactly one product is evaluated inside that product.
  bool inlineLeaf(uint32_t c) const { return g.nodes[c].kind == NodeKind::Gaussian && g.nodes[c].uses == 1; }
  bool fusableProduct(uint32_t i) const {
    if (g.nodes[i].kind != NodeKind::Product) return false;
    for (uint32_t c : g.nodes[i].children)
      if (inlineLeaf(c)) return true;
    return false;
  }

  // Names of the values a product combines, emitting whatever is not there yet. Two table
  // leaves that share a joint table count as one operand.
  std::vector<std::string> productOperands(const std::vector<uint32_t>& kids) {
    std::vector<std::string> ops;
    for (uint32_t c : kids) {
      if (fusedLeaf[c]) continue;  // part of pt<product>, which the caller adds
      const bool table = g.nodes[c].kind == NodeKind::Categorical || g.nodes[c].kind == NodeKind::Histogram;
      if (!table || partner[c] == UINT32_MAX) {
        emitNode(c);
        ops.push_back(v(c));
        continue;
      }
      const uint32_t a = std::min(c, partner[c]), b = std::max(c, partner[c]);
      if (c != a) continue;  // the pair was emitted with its first leaf
      const uint32_t fa = g.nodes[a].feature, fb = g.nodes[b].feature;
      emitFeaturePrep(fa);
      emitFeaturePrep(fb);
      emitted[a] = emitted[b] = true;
      const std::string name = "j" + std::to_string(a);
      const std::string value = tableValue(a);  // may emit the read of the group
      body << "  const real_t " << name << " = " << value << ";\n";
      ops.push_back(name);
    }
    return ops;
  }

  // Sixteen consecutive lanes of the constant pool for `values` (at most sixteen), all within one vector.
  std::pair<unsigned, unsigned> allocLanes(const std::vector<double>& values) {
    if (kPool.size() % 16 + values.size() > 16) kPool.resize((kPool.size() + 15) / 16 * 16, 0.0);
    const unsigned at = unsigned(kPool.size());
    kPool.insert(kPool.end(), values.begin(), values.end());
    // The vector is loaded where the marker stands; the markers are replaced by the loads of later vectors once the
    // whole body is there, so that a load is in flight for a few products before its first use.
    for (; kVectorsNamed <= int(at / 16); ++kVectorsNamed) body << "/*KV" << kVectorsNamed << "*/\n";
    return {at / 16, at % 16};
  }

  // The expanded leaves of product i on top of `rest` (the name of the sum of its other children, or empty).
  void emitExpandedLeaves(uint32_t i, const std::vector<uint32_t>& leaves, const std::string& rest, double fold) {
    const std::string p = "p" + std::to_string(i) + "_";
    const char* fma = "__builtin_fma(";
    const bool marginal = g.supportMarginal;
    struct Term { std::string input; double k; };
    std::string acc;
    double constants = fold;  // what does not depend on the inputs: the folded weight, and every leaf's C without marginalisation
    size_t chunk = 0;
    for (size_t lo = 0; lo < leaves.size(); ++chunk) {
      // Leaves in chunks: four when a pattern table holds their constant terms, eight otherwise (sixteen lanes, two or
      // three constants per leaf; an assembler statement takes thirty operands).
      const bool table = marginal && o.marginalTablesKiB > 0 && (cTables.size() + 16) * sizeof(double) <= size_t(o.marginalTablesKiB) * 1024;
      const size_t hi = std::min(leaves.size(), lo + (table ? 4 : (marginal ? 5 : 8)));
      std::vector<Term> terms;
      std::vector<uint32_t> feats;
      std::vector<double> cs;
      for (size_t j = lo; j < hi; ++j) {
        const auto& leaf = g.nodes[leaves[j]];
        emitFeaturePrep(leaf.feature);
        const std::string f = std::to_string(leaf.feature);
        const double den = -(1.0 / (2.0 * leaf.stddev * leaf.stddev)) * scale;
        const double coef = (-std::log(leaf.stddev) + -0.5 * std::log(2 * M_PI)) * scale;
        terms.push_back({"gq" + f, den});
        terms.push_back({"gx" + f, -2.0 * leaf.mean * den});
        const double C = den * leaf.mean * leaf.mean + coef;
        feats.push_back(leaf.feature);
        cs.push_back(C);
        if (!marginal) constants += C;
        else if (!table) terms.push_back({"go" + f, C});
      }
      // What the multiply-adds accumulate onto.
      const std::string a0 = p + "i" + std::to_string(chunk);
      std::string start;
      if (table) {
        auto it = patternNames.find(feats);
        if (it == patternNames.end()) {
          const std::string name = "pm" + std::to_string(patternNames.size());
          body << "  const unsigned " << name << " = ";
          for (size_t q = 0; q < feats.size(); ++q) body << (q ? " | " : "") << "(gn" << feats[q] << " ? 0u : " << (1u << q) << "u)";
          body << ";\n";
          it = patternNames.emplace(feats, name).first;
        }
        const size_t base = cTables.size();
        for (unsigned mask = 0; mask < (1u << feats.size()); ++mask) {
          double sum = chunk == 0 ? fold : 0.0;
          for (size_t q = 0; q < feats.size(); ++q)
            if (mask >> q & 1u) sum += cs[q];
          cTables.push_back(sum);
        }
        start = "SPN_CTAB[" + std::to_string(base) + "u + " + it->second + "]";
        if (chunk == 0) constants = 0.0;
      } else if (chunk == 0 && constants != 0.0) {
        start = lit(constants);
        constants = 0.0;
      }
      if (!acc.empty()) start = start.empty() ? acc : "(" + acc + " + " + start + ")";
      if (!laneConstants) {
        std::string cur = start;
        for (size_t t = 0; t < terms.size(); ++t) {
          const std::string name = p + "e" + std::to_string(chunk) + "_" + std::to_string(t);
          if (cur.empty()) body << "  const real_t " << name << " = " << terms[t].input << " * " << lit(terms[t].k) << ";\n";
          else body << "  const real_t " << name << " = " << fma << terms[t].input << ", " << lit(terms[t].k) << ", " << cur << ");\n";
          cur = name;
        }
        acc = cur;
      } else {
        std::vector<double> ks;
        for (const Term& t : terms) ks.push_back(t.k);
        const auto where = allocLanes(ks);
        body << "  real_t " << a0 << " = " << (start.empty() ? "0.0" : start) << ";\n";
        body << "  asm(\"";
        for (size_t t = 0; t < terms.size(); ++t)
          body << (t ? "\\n\\t" : "") << "v_fmac_f64_dpp %0, %1, %" << t + 2 << " row_newbcast:" << where.second + t << " row_mask:0xf bank_mask:0xf";
        body << "\"\n      : \"+v\"(" << a0 << ") : \"v\"(kv" << where.first << ")";
        for (const Term& t : terms) body << ", \"v\"(" << t.input << ")";
        body << ");\n";
        acc = a0;
      }
      lo = hi;
    }
    std::string value = acc;
    if (constants != 0.0) value = "(" + value + " + " + lit(constants) + ")";
    if (!rest.empty()) value = "(" + value + " + " + rest + ")";
    body << "  const real_t " << v(i) << " = " << value << ";\n";
  }

  // Log-space product with Gaussian leaves folded in. A leaf's value coef + d*d*den (d = x - mean)
  // is rewritten den * (d*d + coef/den), so that leaf plus accumulation cost three instructions
  // whose constants are all literals: d = x - mean; t = fma(d, d, coef/den); acc = fma(t, den, acc).
  // A log-weight handed down by the single parent sum is folded into the first leaf's constant.
  // With marginal support a NaN input selects the constant that makes the leaf contribute 0.
  void emitFusedProduct(uint32_t i) {
    const auto& n = g.nodes[i];
    std::vector<uint32_t> leaves, rest;
    for (uint32_t c : n.children) (inlineLeaf(c) ? leaves : rest).push_back(c);
    double fold = 0.0;
    auto it = foldedWeight.find(i);
    if (it != foldedWeight.end()) fold = it->second;
    std::string p = "p" + std::to_string(i) + "_";
    std::string acc;
    if (!rest.empty()) {
      const std::vector<std::string> ops = productOperands(rest);
      std::string e = tree(
          0, ops.size(), [&](size_t k) { return ops[k]; },
          [&](const std::string& a, const std::string& b) { return "(" + a + " + " + b + ")"; });
      acc = p + "r";
      body << "  const real_t " << acc << " = " << e << ";\n";
    }
    const char* fma = f64 ? "__builtin_fma(" : "__builtin_fmaf(";
    if (expandedGauss && !leaves.empty()) {
      emitExpandedLeaves(i, leaves, acc, fold);
      return;
    }
    // Offsets of the leaves over missing features, four leaves to a table, while the tables fit; smallest offsets first.
    std::vector<std::string> corrections;
    std::vector<bool> viaTable(leaves.size(), false);
    if (marginalOffsets && !leaves.empty()) {
      std::vector<size_t> order(leaves.size());
      for (size_t k = 0; k < order.size(); ++k) order[k] = k;
      std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) { return std::fabs(offsetOf(g.nodes[leaves[a]])) < std::fabs(offsetOf(g.nodes[leaves[b]])); });
      double together = 0.0;
      std::vector<size_t> chosen;
      for (size_t k : order) {
        const double offset = std::fabs(offsetOf(g.nodes[leaves[k]]));
        if (offset > 8.0 || together + offset > 32.0) break;
        together += offset;
        chosen.push_back(k);
      }
      std::sort(chosen.begin(), chosen.end());
      if ((cTables.size() + 16 * ((chosen.size() + 3) / 4)) * sizeof(float) > size_t(o.marginalTablesKiB) * 1024) chosen.clear();
      for (size_t lo = 0; lo < chosen.size(); lo += 4) {
        std::vector<uint32_t> feats;
        std::vector<double> ks;
        for (size_t j = lo; j < std::min(chosen.size(), lo + 4); ++j) {
          const auto& leaf = g.nodes[leaves[chosen[j]]];
          viaTable[chosen[j]] = true;
          emitFeaturePrep(leaf.feature);
          feats.push_back(leaf.feature);
          ks.push_back(offsetOf(leaf, chosen[j] == 0 ? fold : 0.0));
        }
        auto pattern = patternNames.find(feats);
        if (pattern == patternNames.end()) {
          const std::string name = "pm" + std::to_string(patternNames.size());
          body << "  const unsigned " << name << " = ";
          for (size_t q = 0; q < feats.size(); ++q) body << (q ? " | " : "") << "(gn" << feats[q] << " ? 0u : " << (1u << q) << "u)";
          body << ";\n";
          pattern = patternNames.emplace(feats, name).first;
        }
        const size_t base = cTables.size();
        for (unsigned mask = 0; mask < (1u << feats.size()); ++mask) {   // bit q set: feature q is there
          double sum = 0.0;
          for (size_t q = 0; q < feats.size(); ++q)
            if (!(mask >> q & 1u)) sum -= ks[q];
          cTables.push_back(sum);
        }
        corrections.push_back("SPN_CTAB[" + std::to_string(base) + "u + " + pattern->second + "]");
      }
    }
    for (size_t k = 0; k < leaves.size(); ++k) {
      const auto& leaf = g.nodes[leaves[k]];
      emitFeaturePrep(leaf.feature);
      const bool offsets = viaTable[k];
      const std::string x = (offsets ? "gz" : "g") + std::to_string(leaf.feature);
      const double den = -(1.0 / (2.0 * leaf.stddev * leaf.stddev)) * scale;
      const double coef = (-std::log(leaf.stddev) + -0.5 * std::log(2 * M_PI)) * scale;
      // The weight a parent sum folded into this product rides on the first leaf's constant; with masks it would be
      // cleared along with a missing first feature, so it is added at the end instead.
      const double extra = k == 0 && !nanMasks() ? fold / den : 0.0;
      const std::string d = p + "d" + std::to_string(k), t = p + "t" + std::to_string(k), a = p + "a" + std::to_string(k);
      body << "  const real_t " << d << " = " << x << " - " << lit(leaf.mean) << ";\n";
      if (nanMasks())
        body << "  const real_t " << t << " = " << masked(std::string(fma) + d + ", " + d + ", " + lit(coef / den) + ")", leaf.feature) << ";\n";
      else if (g.supportMarginal && !offsets)
        body << "  const real_t " << t << " = (" << x << " != " << x << ") ? " << lit(extra) << " : " << fma << d << ", " << d << ", "
             << lit(coef / den + extra) << ");\n";
      else
        body << "  const real_t " << t << " = " << fma << d << ", " << d << ", " << lit(coef / den + extra) << ");\n";
      if (acc.empty()) body << "  const real_t " << a << " = " << t << " * " << lit(den) << ";\n";
      else body << "  const real_t " << a << " = " << fma << t << ", " << lit(den) << ", " << acc << ");\n";
      acc = a;
    }
    for (const std::string& c : corrections) acc = "(" + acc + " + " + c + ")";
    if (nanMasks() && fold != 0.0 && !leaves.empty()) body << "  const real_t " << v(i) << " = " << acc << " + " << lit(fold) << ";\n";
    else body << "  const real_t " << v(i) << " = " << acc << ";\n";
  }

  // Emits node i after everything it depends on. Children are emitted lazily, right before
  // their first use, so that a sum over hundreds of children never holds all of them live.
  void emitNode(uint32_t i) {
    if (emitted[i]) return;
    emitted[i] = true;
    const auto& n = g.nodes[i];
    if (n.kind != NodeKind::Product && n.kind != NodeKind::Sum && n.kind != NodeKind::External) emitFeaturePrep(n.feature);
    switch (n.kind) {
      case NodeKind::External:  // computed by an earlier task: row `feature` of the intermediate buffer, this sample's column
        body << "  const real_t " << v(i) << " = spn_in[" << n.feature << "ull * spn_n];\n";
        break;
      case NodeKind::Gaussian: {
        // log: coef + (x-mean)^2 * den with coef = -ln(sd) - ln(2 pi)/2, den = -1/(2 sd^2)
        // (mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:306-374); linear: coef' * exp((x-mean)^2 * den)
        // with coef' = 1/sqrt(2 pi sd^2) (same file :242-304).
        std::string x = "g" + std::to_string(n.feature);
        double den = -(1.0 / (2.0 * n.stddev * n.stddev));
        std::string d = "(" + x + " - " + lit(n.mean) + ")";
        if (logSpace) {
          double coef = -std::log(n.stddev) + -0.5 * std::log(2 * M_PI);
          emitLeafMarginal(i, lit(coef * scale) + " + (" + d + " * " + d + ") * " + lit(den * scale));
        } else {
          double coef = 1.0 / std::sqrt(2.0 * M_PI * n.stddev * n.stddev);
          emitLeafMarginal(i, lit(coef) + " * spn_exp((" + d + " * " + d + ") * " + lit(den) + ")");
        }
        break;
      }
      case NodeKind::Categorical:
      case NodeKind::Histogram:
      {
        const std::string value = tableValue(i);  // may emit the read of the group
        body << "  const real_t " << v(i) << " = " << value << ";\n";
        break;
      }
      case NodeKind::Product: {
        if (logSpace && fusableProduct(i)) {
          emitFusedProduct(i);
          break;
        }
        const char* op = logSpace ? " + " : " * ";
        if (fusedGroupOf[i] >= 0 && !fusedGroups[size_t(fusedGroupOf[i])].emitted) emitFusedGroup(fusedGroups[size_t(fusedGroupOf[i])]);
        std::vector<std::string> ops = productOperands(n.children);
        if (fusedGroupOf[i] >= 0) ops.push_back("pt" + std::to_string(i));
        std::string e = tree(
            0, ops.size(), [&](size_t k) { return ops[k]; },
            [&](const std::string& a, const std::string& b) { return "(" + a + op + b + ")"; });
        body << "  const real_t " << v(i) << " = " << e << ";\n";
        break;
      }
      case NodeKind::Sum:
        emitSum(i);
        break;
    }
  }

  void emitSum(uint32_t i) {
    const auto& n = g.nodes[i];
    const size_t k = n.children.size();
    std::string p = "s" + std::to_string(i) + "_";
    unsigned tmp = 0;
    auto fresh = [&](const std::string& expr) {
      std::string name = p + "t" + std::to_string(tmp++);
      body << "  const real_t " << name << " = " << expr << ";\n";
      return name;
    };
    if (!logSpace) {
      // Linear space: child * weight, then the balanced tree of adds; partial sums are named so
      // that the expression stays flat for sums with hundreds of children.
      std::string e = tree(
          0, k,
          [&](size_t j) {
            emitNode(n.children[j]);
            return fresh(v(n.children[j]) + " * " + lit(n.weights[j]));
          },
          [&](const std::string& a, const std::string& b) { return fresh(a + " + " + b); });
      body << "  const real_t " << v(i) << " = " << e << ";\n";
      return;
    }
    auto term = [&](size_t j) {
      const uint32_t c = n.children[j];
      const double w = logConst(n.weights[j]);
      if (!emitted[c] && g.nodes[c].uses == 1 && fusableProduct(c) && std::isfinite(w)) {
        foldedWeight[c] = w;  // the child adds the log-weight itself
        emitNode(c);
        return v(c);
      }
      emitNode(c);
      return fresh(v(c) + " + " + lit(w));
    };
    if (k == 1) {
      const std::string only = term(0);  // emits the child first
      body << "  const real_t " << v(i) << " = " << only << ";\n";
      return;
    }
    if (o.sumForm == SumForm::Pairwise) {
      // a + log1p(exp(b - a)) with a the larger operand, over the reference's balanced tree
      // (mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:216-240).
      std::string e = tree(0, k, term, [&](const std::string& a, const std::string& b) { return fresh("spn_logadd(" + a + ", " + b + ")"); });
      body << "  const real_t " << v(i) << " = " << e << ";\n";
      return;
    }
    const std::string lowest = f64 ? "(-0x1.fffffffffffffp+1023)" : "(-0x1.fffffep+127f)";
    if (k == 2) {
      // max + log(1 + exp(-|y0 - y1|)): the larger term contributes exp(0) = 1 exactly. Two
      // impossible children give exp(NaN); the max with 0 turns that into log(1 + 0).
      std::string y0 = term(0), y1 = term(1);
      std::string absf = f64 ? "__builtin_fabs" : "__builtin_fabsf";
      body << "  const real_t " << v(i) << " = " << maxOf(y0, y1) << " + "
           << logOf(lit(1.0) + " + " + maxOf(expOf("-" + absf + "(" + y0 + " - " + y1 + ")"), lit(0.0))) << ";\n";
      return;
    }
    // n-ary max-shifted log-sum-exp, m + log(sum_j exp(y_j - m)) with m = max_j y_j, evaluated
    // over chunks of children with a running (m, s): s <- s * exp(m_old - m_new) + sum_chunk exp(y_j - m_new).
    // m is clamped to the lowest finite value so that impossible children (-inf) give exp(-inf) = 0, not NaN.
    const size_t chunk = 16;
    std::string m, sAcc;
    for (size_t lo = 0; lo < k; lo += chunk) {
      const size_t hi = std::min(k, lo + chunk);
      std::vector<std::string> y;
      for (size_t j = lo; j < hi; ++j) y.push_back(term(j));
      std::string cm = tree(
          0, y.size(), [&](size_t j) { return y[j]; }, [&](const std::string& a, const std::string& b) { return maxOf(a, b); });
      // (float64 kernels with marginalisation: their exp2 turns the NaN of -inf - -inf into 0 by itself, so no floor.)
      const bool floorNeeded = !(f64 && log2Dom && g.supportMarginal);
      const std::string mRaw = lo == 0 ? cm : maxOf(m, cm);
      std::string mNew = fresh(floorNeeded ? maxOf(mRaw, lowest) : mRaw);
      std::string part = tree(
          0, y.size(), [&](size_t j) { return expOf(y[j] + " - " + mNew); },
          [&](const std::string& a, const std::string& b) { return "(" + a + " + " + b + ")"; });
      sAcc = lo == 0 ? fresh(part) : fresh(sAcc + " * " + expOf(m + " - " + mNew) + " + " + part);
      m = mNew;
    }
    body << "  const real_t " << v(i) << " = " << m << " + " << logOf(sAcc) << ";\n";
  }
};

unsigned pickVectorBytes(unsigned rowBytes, unsigned elemBytes) {
  for (unsigned vb : {16u, 8u, 4u, 2u, 1u})
    if (vb >= elemBytes && rowBytes % vb == 0) return vb;
  return elemBytes;
}

}  // namespace

// Whether the library's exp/log are inlined at every call: by the size of the graph and its call sites. In linear space
// every Gaussian leaf is a call of the double-precision exp (1326 of them cost 80 s of hipRTC time inlined, 10 s out of line).
bool inlineLibraryMath(const Graph& g, const CompileOptions& o) {
  return g.nodes.size() + g.stats.sumTerms + (o.useLogSpace ? 0 : 3 * size_t(g.stats.gaussians)) <= 4000;
}

JitSource emitHipSource(const Graph& g, const CompileOptions& o, const std::string& entry) {
  Emitter e(g, o);
  // Short rows are fetched with the widest vector loads their size allows, all samples of a
  // lane up front; wide rows are read feature by feature next to the first use.
  e.vectorRows = g.numFeatures * g.ftype.bytes <= 512;
  {
    // Packed rows: wide rows of 32-bit integers that only feed table leaves with short tables, in a complete and
    // decomposable graph (an input outside a one-hot feature's range is reported through a flag, not through a table).
    bool eligible = e.logSpace && e.vectorRows && !g.ftype.isFloat && g.ftype.bytes == 4 && g.numFeatures % 4 == 0 &&
                    g.numFeatures * 4 >= 128 && g.completeDecomposable && !g.supportMarginal && o.samplesPerLane <= 1 && !g.isTask;
    bool anyTable = false;
    for (const auto& n : g.nodes) {
      if (n.kind == NodeKind::Gaussian) eligible = false;
      if (n.kind == NodeKind::Categorical || n.kind == NodeKind::Histogram) {
        anyTable = true;
        if (n.table.size() > 128) eligible = false;  // the range test on packed bytes handles lengths up to 128
      }
    }
    e.packedRows = eligible && anyTable && o.packedRows != 0 && o.waveTranspose != 0;  // packed rows come out of the per-wavefront transposed load
  }
  e.prepare();
  JitSource js;
  js.entry = entry;
  js.blockSize = o.blockSize ? unsigned(o.blockSize) : 256u;
  // Grouped tables with packed indices leave the kernel at about 140 registers and take up to 80 KiB of LDS: one
  // block of 1024 threads per CU then runs four waves per SIMD on one copy of the tables (C3: 1.19 ms with two
  // blocks of 256, 1.18 ms with two of 512, 1.06 ms with one of 1024).
  if (o.blockSize == 0 && e.packedIndices) js.blockSize = 1024;
  js.bytesPerResult = e.f64 ? 8 : 4;
  js.tableEntries = unsigned(e.tablePool.size());
  const unsigned realBytes = e.f64 ? 8 : 4;
  // gfx950 has 160 KiB of LDS per CU, all of it usable by one workgroup.
  js.tablesInLds = js.tableEntries > 0 && size_t(js.tableEntries) * realBytes <= 140 * 1024;

  const unsigned F = g.numFeatures;
  const unsigned eb = g.ftype.bytes;
  const unsigned rowBytes = F * eb;
  // Rows held in registers: the clamped table indices are derived right away, so that a raw feature
  // value and its index are never live together for long.
  auto emitBody = [&] {
    if (e.packedRows) {
      e.emitPackedPrologue();
      e.emitNode(g.root());
      if (e.midpointHook && !e.midpointEmitted) e.body << "  spn_mid();\n";
      return;
    }
    if (e.vectorRows && o.eagerIndices)
      for (uint32_t f = 0; f < F; ++f)
        if (e.featUsed[f] && e.featTableLen[f]) e.emitFeaturePrep(f);
    if (e.packedIndices) e.emitPackedIndices();
    if (g.isTask) {
      for (uint32_t node : g.taskOutputs) e.emitNode(node);
      if (g.taskFinal) e.emitNode(g.root());
      for (size_t k = 0; k < g.taskOutputs.size(); ++k)
        e.body << "  spn_res[" << g.taskOutputSlots[k] << "ull * spn_n] = " << Emitter::v(g.taskOutputs[k]) << ";\n";
      return;
    }
    e.emitNode(g.root());
  };
  const unsigned vb = e.vectorRows ? pickVectorBytes(rowBytes, eb) : eb;
  const unsigned vw = vb / eb;
  js.inputAlign = vb;

  // Samples per lane: two independent samples give the scheduler more to overlap; kernels that
  // are heavy on registers (large LDS tables, NaN selects) stay at one.
  const size_t work = g.nodes.size() + g.stats.sumTerms;
  unsigned U = unsigned(o.samplesPerLane);
  if (U == 0) U = (work <= 4000 && !g.supportMarginal && size_t(js.tableEntries) * realBytes <= 16 * 1024) ? 2 : 1;
  if (!e.vectorRows || e.packedRows || g.isTask) U = 1;  // tasks: one sample per lane, rows fetched by their lane
  js.samplesPerLane = U;
  // Kernels that sit on the HBM bound and stage their input tile through LDS run 2-3 % faster with
  // 512-thread blocks (measured on the six-feature product: 0.82 against 0.80 of the HBM peak).
  if (o.blockSize == 0 && o.gpuSharedMem != 0 && e.vectorRows) {
    const double tHbmAuto = double(rowBytes + realBytes) / 6.4e12, tValuAuto = double(g.stats.issueSlotsMin()) / 6.0e13;
    const size_t bigTile = size_t(512) * U * rowBytes;
    if (tHbmAuto > tValuAuto && bigTile % 16 == 0 && bigTile + size_t(js.tableEntries) * realBytes <= 64 * 1024) js.blockSize = 512;
  }
  // Float kernels without tables: blocks of 512 threads, so that a SIMD always holds an even number of wavefronts. Full
  // rate instructions issue from two wavefronts in turns, and an odd number of wavefronts loses part of that (v_add_f32
  // alone: 1.09 ns per instruction at two wavefronts per SIMD, 1.39 at three, 1.08 at four). Measured: 16 Gaussian
  // features 1.63 -> 1.60 ms, the same with 20 % missing values (95 registers, five wavefronts of 256-thread blocks or
  // four of 512-thread ones) 1.62 -> 1.56 ms. Double kernels are slower that way (4.34 -> 4.89 ms) and stay at 256.
  if (o.blockSize == 0 && !e.f64 && e.logSpace && !g.isTask && js.tableEntries == 0 && e.vectorRows) js.blockSize = 512;
  js.libraryMath = !e.log2Dom;
  js.doubleConstants = e.f64;
  // Wide rows of 32-bit integer features read only by table leaves: a lane that fetches its own row touches 64 cache
  // lines per load instruction of its wavefront, which keeps the memory pipeline at half the bandwidth of a plain copy
  // (measured on 400-byte rows: 1.0 ms for 3.4 GB against 0.53 ms). Instead every wavefront copies the 64 rows of its
  // tile, which are contiguous in memory, with fully coalesced 16-byte loads, packs each loaded vector of four values
  // into four bytes (an index above 255 is out of every table's range anyway), writes the packed tile into its own LDS
  // buffer and lets every lane read its row back: F/4 LDS writes and F/4 reads per sample, and memory at copy speed
  // with as few as two wavefronts per SIMD.
  bool waveTile = false;
  unsigned waveStride = 0;  // dwords per packed row in LDS: odd, so that the 64 lanes' reads fall into distinct banks
  {
    bool eligible = e.vectorRows && !g.ftype.isFloat && eb == 4 && F % 4 == 0 && U == 1 && rowBytes >= 128 && !g.isTask;
    for (uint32_t f = 0; f < F && eligible; ++f)
      if (e.featGauss[f] || e.featTableLen[f] > 255) eligible = false;
    if (eligible && (o.waveTranspose == 1 || (e.packedRows && o.waveTranspose != 0))) {  // beside unpacked indices it gains nothing (0.79 against 0.78 ms on the 100-feature discrete graph): only with packed rows, or on request
      waveStride = (F / 4) | 1u;
      const size_t tables = js.tablesInLds ? size_t(js.tableEntries) * realBytes : 0;
      unsigned block = o.blockSize ? unsigned(o.blockSize) : 512u;
      while (!o.blockSize && block > 64 && tables + size_t(block / 64) * 64 * waveStride * 4 > 150 * 1024) block /= 2;
      // Packed rows address their tables inside LDS: a pool that is too large for LDS leaves the graph to the kernel with
      // one index per feature (built below).
      const bool tablesReachable = !e.packedRows || js.tableEntries == 0 || js.tablesInLds;
      if (tablesReachable && tables + size_t(block / 64) * 64 * waveStride * 4 <= 150 * 1024) {
        waveTile = true;
        js.blockSize = block;
      }
    }
  }
  js.waveTransposedInput = waveTile;
  js.packedRows = e.packedRows && waveTile;
  if (e.packedRows && !waveTile) {  // the row buffers do not fit beside the tables: the same kernel with unpacked rows
    CompileOptions unpacked = o;
    unpacked.packedRows = 0;
    return emitHipSource(g, unpacked, entry);
  }

  std::ostringstream s;
  s << "// generated by spnc-hip for SPN '" << g.name << "': " << g.nodes.size() << " nodes, " << F << " features\n";
  s << "typedef " << (e.f64 ? "double" : "float") << " real_t;\n";
  // Streaming (non-temporal) loads suit rows that one or two instructions per lane fetch whole and
  // the coalesced tile copy; a wider row is fetched by many instructions per lane that revisit the
  // same cache lines, which plain cached loads serve better (measured: +17 % on 400-byte rows).
  const bool streaming = o.nontemporalLoads && g.numFeatures * g.ftype.bytes <= 32;
  s << (streaming ? "#define SPN_LOAD(p) __builtin_nontemporal_load(p)\n" : "#define SPN_LOAD(p) (*(p))\n");
  s << (o.nontemporalLoads ? "#define SPN_LOAD_TILE(p) __builtin_nontemporal_load(p)\n" : "#define SPN_LOAD_TILE(p) (*(p))\n");
  s << "typedef " << g.ftype.hipName << " feat_t;\n";
  if (vw > 1) s << "typedef feat_t rowvec_t __attribute__((ext_vector_type(" << vw << ")));\n";
  s << "#define SPN_F " << F << "\n#define SPN_BLOCK " << js.blockSize << "\n#define SPN_U " << U << "\n";
  if (js.tableEntries) {
    s << "#define SPN_NTAB " << js.tableEntries << "\n";
    s << "typedef real_t spn_r2 __attribute__((ext_vector_type(2)));\ntypedef real_t spn_r4 __attribute__((ext_vector_type(4)));\n";
    s << "__device__ __attribute__((aligned(32))) const real_t spn_tables[SPN_NTAB] = {";
    for (size_t i = 0; i < e.tablePool.size(); ++i) s << (i ? ", " : "") << (i % 8 == 0 ? "\n  " : "") << e.lit(e.tablePool[i]);
    s << "};\n";
  }
  // Out-of-line library math keeps hipRTC times in seconds for large graphs; small graphs inline it.
  const bool inlineMath = o.inlineMath >= 0 ? o.inlineMath == 1 : inlineLibraryMath(g, o);
  const char* mathAttr = inlineMath ? "__forceinline__" : "__attribute__((noinline))";
  if (e.log2Dom && e.f64) {
    // Base-2 exponential and logarithm in double for the arguments this kernel produces (exponents <= 0 up to
    // rounding, logarithms of sums in [1, fan-in] or of exactly 0), by table and short polynomial: about 11 and 11
    // double-rate instructions (plus a few integer ones and one LDS read each) where the general library routines
    // take 40 and 95.
    // exp2: n = rint(64 x), r = x - n/64 (exact), 2^x = 2^(n>>6) * T[n&63] * 2^r, T[j] = 2^(j/64),
    // 2^r - 1 = r (c1 + r (c2 + ... r c5)), c_k = ln(2)^k / k!, |r| <= 1/128 (remainder 4e-17;
    // a table of 256 entries has its reads spread over sixteen times the width of the LDS banks, this one over four).
    // log2: x = 2^e * t, t in [1, 2), j = the top eight bits of t's fraction, u = t * R[j] - 1 in one fma with
    // R[j] = 1/(1 + j/256) rounded, so 0 <= u < 2^-8 up to rounding and R[0] = 1 keeps t - 1 exact near 1;
    // log2 t = G[j] + u (l1 + u (l2 + ... u l7)), G[j] = -log2 R[j] of the rounded R[j], l_k = (-1)^(k+1) / (k ln 2)
    // (remainder 2e-18 relative). Both agree with the library to 1e-15 relative over their ranges (checked on
    // the CPU against exp2/log2 of libm). The tables live in LDS, 4.5 KiB per block.
    s << "#define SPN_DOUBLE_TABLES 1\n";
    const std::vector<double> math = doubleMathTables();
    // Entry j holds 2^(j/64) with j << 14 taken off its upper half, so that adding n << 14 (n = 64 q + j) puts q into the
    // exponent field in one instruction: the j's cancel (modulo 2^32).
    s << "__device__ const unsigned long long spn_exp2_table[64] = {";
    for (int j = 0; j < 64; ++j) {
      uint64_t bits;
      std::memcpy(&bits, &math[j], 8);
      bits = (bits & 0xffffffffull) | (uint64_t(uint32_t(bits >> 32) - (uint32_t(j) << 14)) << 32);
      char hex[32];
      std::snprintf(hex, sizeof(hex), "0x%016llxull", (unsigned long long)bits);
      s << (j ? ", " : "") << (j % 4 == 0 ? "\n  " : "") << hex;
    }
    s << "};\n__device__ const real_t spn_log2_table[512] = {";
    for (int j = 0; j < 512; ++j) s << (j ? ", " : "") << (j % 4 == 0 ? "\n  " : "") << e.lit(math[64 + j]);
    s << "};\n";
    // The polynomial coefficients are read from LDS as well, once per kernel, and stay in registers: as literals
    // every use costs two register moves, since a double constant cannot be an operand of the instruction itself.
    // c5..c1 of exp2, then l7..l1 of log2.
    // Entry 12 is the rounding constant of exp2, 1.5 * 2^52: as a value read from memory it stays in a register pair;
    // as a literal it would be moved into the destination of a multiply-add before every use.
    s << "__device__ const real_t spn_poly[13] = {";
    for (int j = 0; j < 12; ++j) s << (j ? ", " : "") << e.lit(math[576 + j]);
    s << ", 0x1.8p+52};\n";
    s << "#ifndef SPN_EXP2_TABLE\n__shared__ unsigned long long spn_exp2_lds[64];\n__shared__ __attribute__((aligned(16))) real_t spn_log2_lds[512];\n"
         "__shared__ real_t spn_poly_lds[13];\n"
         "#define SPN_EXP2_TABLE spn_exp2_lds\n#define SPN_LOG2_TABLE spn_log2_lds\n#define SPN_POLY spn_poly_lds\n#endif\n";
    // n = rint(64 x) without a rounding or conversion instruction: 64 x + 1.5 * 2^52 has an ulp of 1, so the sum's low
    // mantissa bits are n as an integer and the sum minus the constant is n as a double. 2^(n >> 6) goes into the table
    // value's exponent field by an integer add on its upper half (T[j] lies in [1, 2): field 1023; arguments are cut off
    // at -1023, where the field reaches 0 with T[0] = 1, i.e. exactly 0.0; between -1023 and -1022 the result is
    // some subnormal below 2^-1022, against terms of a sum whose largest is 1). A NaN argument stays NaN through r.
    s << "static __device__ " << mathAttr << " real_t spn_exp2(real_t x) {\n"
      << (g.supportMarginal ? "  x = __builtin_fmax(x, -1023.0);  // missing features are handled at the leaves: no NaN gets here\n"
                            : "  x = x < -1023.0 ? -1023.0 : x;  // keeps NaN\n")
      <<
         "  union { real_t d; unsigned long long u; unsigned w[2]; } s, t;\n"
         "  const real_t magic = SPN_POLY[12];\n"
         "  // s = 64 x + magic with the factor as a scalar operand: written as C the constant is copied into the destination of a v_fmac_f64 every time\n"
         "  asm(\"v_fma_f64 %0, %1, %2, %3\" : \"=v\"(s.d) : \"v\"(x), \"s\"(64.0), \"v\"(magic));\n"
         "  const int ni = (int)s.w[0];\n"
         "  const real_t r = __builtin_fma(s.d - magic, -0x1p-6, x);\n"
         "  t.u = SPN_EXP2_TABLE[ni & 63];\n"
         "  unsigned hi;\n"
         "  asm(\"v_lshl_add_u32 %0, %1, 14, %2\" : \"=v\"(hi) : \"v\"(ni), \"v\"(t.w[1]));\n"
         "  t.w[1] = hi;\n"
         // 2^r - 1 = r (c1 + c2 r + c3 r^2 + c4 r^3) for |r| <= 1/128: the next term, c5 r^5, is below 4e-14 of the
         // result, a thousand times below what the results are held to (1e-10), and one multiply-add per call less.
         "  real_t p = SPN_POLY[1];\n"
         "  p = __builtin_fma(p, r, SPN_POLY[2]);\n"
         "  p = __builtin_fma(p, r, SPN_POLY[3]);\n  p = __builtin_fma(p, r, SPN_POLY[4]);\n"
         "  return __builtin_fma(t.d, p * r, t.d);\n}\n";
    s << "static __device__ " << mathAttr << " real_t spn_log2(real_t x) {\n"
         "  union { real_t d; unsigned long long u; } c;\n  c.d = x;\n"
         "  const unsigned hi = (unsigned)(c.u >> 32);\n"
         "  const int e = (int)(hi >> 20) - 1023;\n"
         "  const unsigned j = (hi >> 12) & 255u;\n"
         "  c.u = (c.u & 0x000fffffffffffffull) | 0x3ff0000000000000ull;\n"
         "  const real_t u = __builtin_fma(c.d, SPN_LOG2_TABLE[2 * j], -1.0);\n"
         // log2(1 + u) = u (l1 + l2 u + ... + l5 u^4) for 0 <= u < 1/256: the next term, l6 u^6, is below 1e-15.
         "  real_t p = SPN_POLY[7];\n"
         "  p = __builtin_fma(p, u, SPN_POLY[8]);\n  p = __builtin_fma(p, u, SPN_POLY[9]);\n"
         "  p = __builtin_fma(p, u, SPN_POLY[10]);\n  p = __builtin_fma(p, u, SPN_POLY[11]);\n"
         "  const real_t r = __builtin_fma(u, p, SPN_LOG2_TABLE[2 * j + 1] + (real_t)e);\n"
      << (g.supportMarginal ? "  return x == 0.0 ? -__builtin_huge_val() : r;  // 0: a sum whose terms are all impossible\n}\n"
                            : "  return x == 0.0 ? -__builtin_huge_val() : (x != x ? x : r);  // 0: a sum whose terms are all impossible\n}\n");
  }
  if (!e.log2Dom) {
    s << "static __device__ " << mathAttr << " real_t spn_exp(real_t x) { return " << (e.f64 ? "exp(x)" : "expf(x)") << "; }\n";
    s << "static __device__ " << mathAttr << " real_t spn_log(real_t x) { return " << (e.f64 ? "log(x)" : "logf(x)") << "; }\n";
  }
  if (e.laneConstants)
    s << "static __device__ __forceinline__ real_t spn_max(real_t a, real_t b) {\n"
         "  real_t r;\n  asm(\"v_max_f64 %0, %1, %2\" : \"=v\"(r) : \"v\"(a), \"v\"(b));\n  return r;\n}\n";
  if (e.nanMasks())
    s << (e.f64 ? "static __device__ __forceinline__ real_t spn_mask(real_t v, unsigned m) {\n"
                  "  union { real_t d; unsigned w[2]; } c;\n  c.d = v;\n  c.w[0] &= m;\n  c.w[1] &= m;\n  return c.d;\n}\n"
                : "static __device__ __forceinline__ real_t spn_mask(real_t v, unsigned m) { return __builtin_bit_cast(float, __builtin_bit_cast(unsigned, v) & m); }\n");
  if (e.logSpace && o.sumForm == SumForm::Pairwise) {
    s << "static __device__ " << (e.log2Dom ? "__forceinline__" : mathAttr) << " real_t spn_logadd(real_t x, real_t y) {\n"
         "  const bool gt = x > y;\n  const real_t a = gt ? x : y;\n  const real_t b = gt ? y : x;\n";
    if (e.f64 && e.log2Dom) s << "  return a + spn_log2(1.0 + spn_exp2(b - a));\n";
    else if (e.f64) s << "  return a + log1p(exp(b - a));\n";
    else if (e.log2Dom) s << "  return a + __builtin_amdgcn_logf(1.0f + __builtin_amdgcn_exp2f(b - a));\n";
    else s << "  return a + log1pf(expf(b - a));\n";
    s << "}\n";
  }

  if (waveTile) {
    // Four values, each saturated (at 255, or with packed rows at the longest table's length: either is outside every
    // table), into the four bytes of a register: a minimum per value and a shift-and-or per further byte, two registers
    // in turns so that no instruction waits for the one before it. The one-instruction form, a minimum that writes one
    // byte of its destination (SDWA), is the slower one on gfx950: a SIMD overlaps nothing with such an instruction.
    const unsigned satValue = e.packedRows ? e.packedSaturation() : 255u;
    const bool satInline = satValue <= 64;
    auto sat = [&](unsigned operand) { return satInline ? std::to_string(satValue) : "%" + std::to_string(operand); };
    const std::string satOperand = satInline ? std::string() : ", \"s\"(" + std::to_string(satValue) + "u)";
    // dst = min(value 3) << 24 | min(value 2) << 16 | min(value 1) << 8 | min(value 0); values are operands first .. first + 3.
    auto step = [&](const char* dst, const char* tmp, unsigned first, unsigned k, unsigned satOp) {
      const std::string m = std::string("v_min_u32 ") + (k == 0 ? dst : tmp) + ", " + sat(satOp) + ", %" + std::to_string(first + 3 - k) + "\\n\\t";
      return k == 0 ? m : m + "v_lshl_or_b32 " + dst + ", " + dst + ", 8, " + tmp + "\\n\\t";
    };
    s << "static __device__ __forceinline__ unsigned spn_pack4(unsigned a, unsigned b, unsigned c, unsigned d) {\n  unsigned q, t;\n  asm(\"";
    for (unsigned k = 0; k < 4; ++k) s << step("%0", "%1", 2, k, 6);
    s << "\"\n      : \"=&v\"(q), \"=&v\"(t) : \"v\"(a), \"v\"(b), \"v\"(c), \"v\"(d)" << satOperand << ");\n  return q;\n}\n";
    s << "static __device__ __forceinline__ void spn_pack8(unsigned& p, unsigned& q, unsigned a0, unsigned a1, unsigned a2, unsigned a3, unsigned b0, unsigned b1, "
         "unsigned b2, unsigned b3) {\n  unsigned t, w;\n  asm(\"";
    for (unsigned k = 0; k < 4; ++k) s << step("%0", "%2", 4, k, 12) << step("%1", "%3", 8, k, 12);
    s << "\"\n      : \"=&v\"(p), \"=&v\"(q), \"=&v\"(t), \"=&v\"(w) : \"v\"(a0), \"v\"(a1), \"v\"(a2), \"v\"(a3), \"v\"(b0), \"v\"(b1), \"v\"(b2), \"v\"(b3)"
      << satOperand << ");\n}\n";
  }
  if (e.vectorRows) {
    s << "static __device__ __forceinline__ void spn_load_row(const feat_t* __restrict__ in, unsigned long long i, feat_t (&x)[SPN_F]) {\n";
    if (vw == 1) {
      s << "  const feat_t* p = in + i * SPN_F;\n";
      for (unsigned f = 0; f < F; ++f)
        if (e.featUsed[f]) s << "  x[" << f << "] = SPN_LOAD(p + " << f << ");\n";
    } else {
      s << "  const rowvec_t* p = reinterpret_cast<const rowvec_t*>(in + i * SPN_F);\n";
    }
    for (unsigned c = 0; vw > 1 && c < F / vw; ++c) {
      bool used = false;
      for (unsigned k = 0; k < vw; ++k) used = used || e.featUsed[c * vw + k];
      if (!used) continue;
      s << "  const rowvec_t r" << c << " = SPN_LOAD(p + " << c << ");\n";
      for (unsigned k = 0; k < vw; ++k)
        if (e.featUsed[c * vw + k]) s << "  x[" << c * vw + k << "] = r" << c << "[" << k << "];\n";
    }
    s << "}\n";
  }

  // Software pipeline of the transposed load: a wavefront fetches its next tile while it evaluates the current one, in
  // two halves that turn round in the middle of the kernel body, so that only half a tile of loaded vectors is in
  // registers at any time. With two wavefronts per SIMD, which is what the tables and registers of such kernels leave
  // room for, nothing else overlaps memory latency with arithmetic.
  const bool prefetch = waveTile && e.packedRows && o.prefetchRows != 0 && F >= 8;
  // A task reads the values of earlier tasks from, and writes its own results to, the column of its sample in the
  // intermediate buffer (spn_in and spn_res point at that column; its rows are spn_n values apart).
  const char* taskParams = g.isTask ? ", const real_t* __restrict__ spn_in, real_t* __restrict__ spn_res, unsigned long long spn_n" : "";
  const char* taskArgs = g.isTask ? ", ext + i, res + i, n" : "";
  e.midpointHook = prefetch;
  emitBody();
  std::string bodyText = e.body.str();
  if (!e.kPool.empty()) {
    e.kPool.resize((e.kPool.size() + 15) / 16 * 16, 0.0);
    s << "__device__ __attribute__((aligned(128))) const real_t spn_kpool[" << e.kPool.size() << "] = {";
    for (size_t i = 0; i < e.kPool.size(); ++i) s << (i ? ", " : "") << (i % 4 == 0 ? "\n  " : "") << e.lit(e.kPool[i]);
    s << "};\n";
    // Vector v is loaded where the marker of vector v - 3 stands (the first three at the top of the body).
    const int vectors = int(e.kPool.size() / 16), ahead = 3;
    auto load = [&](int v) {
      return "  const real_t kv" + std::to_string(v) + " = spn_kpool[" + std::to_string(v * 16) + "u + (threadIdx.x & 15u)];\n";
    };
    std::string top;
    for (int v = 0; v < std::min(ahead, vectors); ++v) top += load(v);
    for (int v = 0; v < vectors; ++v) {
      const std::string marker = "/*KV" + std::to_string(v) + "*/\n";
      const size_t at = bodyText.find(marker);
      bodyText.replace(at, marker.size(), v + ahead < vectors ? load(v + ahead) : std::string());
    }
    bodyText = top + bodyText;
  }
  if (!e.cTables.empty()) {
    s << "#define SPN_NCTAB " << e.cTables.size() << "\n__device__ const real_t spn_ctab[SPN_NCTAB] = {";
    for (size_t i = 0; i < e.cTables.size(); ++i) s << (i ? ", " : "") << (i % 4 == 0 ? "\n  " : "") << e.lit(e.cTables[i]);
    s << "};\n#ifndef SPN_CTAB\n__shared__ real_t spn_ctab_lds[SPN_NCTAB];\n#define SPN_CTAB spn_ctab_lds\n#endif\n";
  }
  if (prefetch)
    s << "template <typename Mid>\nstatic __device__ __forceinline__ real_t spn_eval(const unsigned (&R)[SPN_F / 4], const real_t* __restrict__ tab, unsigned spn_tab_lds, Mid&& spn_mid) {\n";
  else if (e.packedRows)
    s << "static __device__ __forceinline__ real_t spn_eval(const unsigned (&R)[SPN_F / 4], const real_t* __restrict__ tab, unsigned spn_tab_lds) {\n";
  else if (e.vectorRows)
    s << "static __device__ __forceinline__ real_t spn_eval(const feat_t (&x)[SPN_F], const real_t* __restrict__ tab" << taskParams << ") {\n";
  else
    s << "static __device__ __forceinline__ real_t spn_eval(const feat_t* __restrict__ row, const real_t* __restrict__ tab" << taskParams << ") {\n";
  s << bodyText;
  std::string root = Emitter::v(g.root());
  if (e.packedRows) {
    s << "  const real_t spn_root = " << root << (e.log2Dom ? (e.f64 ? " * 0x1.62e42fefa39efp-1" : " * 0x1.62e43p-1f") : "") << ";\n"
      << "  return outside ? " << e.lit(-INFINITY) << " : spn_root;\n";
  } else if (g.isTask && !g.taskFinal) s << "  return " << e.lit(0.0) << ";\n";
  else if (!e.logSpace) s << "  return spn_log(" << root << ");\n";
  else if (e.log2Dom) s << "  return " << root << (e.f64 ? " * 0x1.62e42fefa39efp-1;\n" : " * 0x1.62e43p-1f;\n");  // back to natural log: * ln 2
  else s << "  return " << root << ";\n";
  s << "}\n";

  // Large LDS tables leave room for two blocks per CU at most. The compiler is told to budget
  // registers for two (256 VGPRs) when the indices held per lane leave enough of them for the
  // arithmetic: two waves per SIMD issue VALU work at twice the rate of one and cover each
  // other's LDS waits (C3: 4.6e9 -> 6.6e9 samples/s).
  const size_t ldsTables = js.tablesInLds ? size_t(js.tableEntries) * realBytes : 0;
  unsigned tableFeatures = 0;
  for (uint32_t f = 0; f < F; ++f) tableFeatures += e.featTableLen[f] ? 1 : 0;
  int minBlocks = o.minBlocksPerCU;
  if (minBlocks == 0 && (js.blockSize == 1024 || waveTile)) minBlocks = 1;
  if (minBlocks == 0 && js.tablesInLds && ldsTables > 40 * 1024 && ldsTables <= 80 * 1024 && tableFeatures <= 136) minBlocks = 2;
  s << "extern \"C\" __global__ void __launch_bounds__(SPN_BLOCK" << (minBlocks > 0 ? ", " + std::to_string(minBlocks) : std::string()) << ") " << js.entry
    << "(const feat_t* __restrict__ in, real_t* __restrict__ out, unsigned long long n"
    << (g.isTask ? ", const real_t* __restrict__ ext, real_t* __restrict__ res" : "") << ") {\n";
  if (e.log2Dom && e.f64)
    s << "  for (unsigned t = threadIdx.x; t < 64; t += SPN_BLOCK) spn_exp2_lds[t] = spn_exp2_table[t];\n"
         "  for (unsigned t = threadIdx.x; t < 512; t += SPN_BLOCK) spn_log2_lds[t] = spn_log2_table[t];\n"
         "  if (threadIdx.x < 13) spn_poly_lds[threadIdx.x] = spn_poly[threadIdx.x];\n";
  if (!e.cTables.empty()) s << "  for (unsigned t = threadIdx.x; t < SPN_NCTAB; t += SPN_BLOCK) spn_ctab_lds[t] = spn_ctab[t];\n";
  if ((e.log2Dom && e.f64) || !e.cTables.empty()) s << "  __syncthreads();\n";
  if (js.tableEntries && js.tablesInLds) {
    s << "  __shared__ __attribute__((aligned(32))) real_t tab[SPN_NTAB];\n"
         "  for (unsigned t = threadIdx.x; t < SPN_NTAB; t += SPN_BLOCK) tab[t] = spn_tables[t];\n"
         "  __syncthreads();\n";
    if (e.packedRows)  // the tables' address inside LDS, for reads addressed by plain integers
      s << "  const unsigned spn_tab_lds = (unsigned)(unsigned long long)(__attribute__((address_space(3))) real_t*)tab;\n";
  } else if (js.tableEntries) {
    s << "  const real_t* tab = spn_tables;\n";
  } else {
    s << "  const real_t* tab = nullptr;\n";
  }
  // "gpu-shared-mem": the block copies its tile of rows from HBM into LDS with fully coalesced
  // 16-byte loads, then every lane reads its own rows from LDS. Same role as the reference's
  // shared-memory preload (mlir/lib/Dialect/LoSPN/Passes/LoSPNGPUSharedMemoryInsertion.cpp:99-260)
  // and, like there, skipped when the tile does not fit.
  const size_t tileBytes = size_t(js.blockSize) * U * rowBytes;
  // Without an explicit option the tile is staged when the kernel is closer to the HBM bound
  // than to the VALU bound (about 6.4e12 B/s against 6e13 lane-operations/s on MI355X).
  const double tHbm = double(rowBytes + realBytes) / 6.4e12, tValu = double(g.stats.issueSlotsMin()) / 6.0e13;
  // Static LDS besides the tables: float64 kernels keep their exp2/log2 tables and the leaves' pattern tables there.
  const size_t ldsOther = (e.f64 ? (64 + 512 + 13) * sizeof(double) : 0) + e.cTables.size() * realBytes;
  const bool wantStaged = o.gpuSharedMem < 0 ? tHbm > 0.5 * tValu : o.gpuSharedMem == 1;
  const bool staged = !waveTile && !g.isTask && wantStaged && e.vectorRows && tileBytes % 16 == 0 && tileBytes + ldsTables + ldsOther <= 64 * 1024;
  js.stagedInput = staged;
  // Blocks with next to no set-up take one tile each; blocks that stage tables stay resident.
  js.oneTilePerBlock = js.tableEntries <= 256;
  if (staged || waveTile) js.inputAlign = 16;
  if (waveTile) js.oneTilePerBlock = false;
  if (o.ldsBallastKiB > 0 && !g.isTask)   // claimed, touched once so that it stays, never read for a result
    s << "  __shared__ unsigned spn_ballast[" << o.ldsBallastKiB * 256 << "];\n  if (n == ~0ull) spn_ballast[threadIdx.x] = 1u;\n"
         "  if (n == ~0ull - 1ull) out[0] = (real_t)spn_ballast[threadIdx.x ^ 1u];\n";
  s << "  const unsigned long long tile = (unsigned long long)SPN_BLOCK * SPN_U;\n";
  if (waveTile)
    s << "  typedef unsigned int spn_v4 __attribute__((ext_vector_type(4)));\n"
         "  constexpr unsigned SPN_Q = SPN_F / 4, SPN_S = " << waveStride << ";   // packed dwords per row, and their stride in LDS\n"
         "  __shared__ unsigned spn_rows[SPN_BLOCK / 64][64 * SPN_S];\n"
         "  const unsigned lane = threadIdx.x & 63u;\n"
         "  unsigned* mine = spn_rows[threadIdx.x >> 6];\n";
  if (staged)
    s << "  typedef unsigned int spn_v4 __attribute__((ext_vector_type(4)));\n"
         "  __shared__ __attribute__((aligned(16))) feat_t spn_tile[SPN_BLOCK * SPN_U * SPN_F];\n";
  if (prefetch) {
    // r[0 .. count) = pieces `from` .. of the tile at src; and: those pieces packed into the wavefront's LDS buffer.
    auto issue = [&](unsigned from, unsigned count, const char* indent) {
      for (unsigned j = 0; j < count; ++j) s << indent << "r[" << j << "] = SPN_LOAD_TILE(src + " << (from + j) * 64 << "u + lane);\n";
      s << indent << "asm volatile(\"\" ::: \"memory\");\n" << indent << "__builtin_amdgcn_sched_barrier(0);\n";  // the loads are issued here and nowhere later
    };
    auto stash = [&](unsigned from, unsigned count, const char* indent) {
      s << indent << "{\n" << indent << "  unsigned packed[" << count << "];\n";
      for (unsigned j = 0; j + 1 < count; j += 2)
        s << indent << "  spn_pack8(packed[" << j << "], packed[" << j + 1 << "], r[" << j << "][0], r[" << j << "][1], r[" << j << "][2], r[" << j << "][3], r[" << j + 1
          << "][0], r[" << j + 1 << "][1], r[" << j + 1 << "][2], r[" << j + 1 << "][3]);\n";
      if (count & 1) s << indent << "  packed[" << count - 1 << "] = spn_pack4(r[" << count - 1 << "][0], r[" << count - 1 << "][1], r[" << count - 1 << "][2], r[" << count - 1 << "][3]);\n";
      for (unsigned j = 0; j < count; ++j)
        s << indent << "  { const unsigned p = " << (from + j) * 64 << "u + lane; mine[p + p / SPN_Q * (SPN_S - SPN_Q)] = packed[" << j << "]; }\n";
      s << indent << "}\n";
    };
    const unsigned Q = F / 4, H = (Q + 1) / 2;
    // Piece p = 64 j + lane of a tile (16 bytes, four features of row p / Q) goes to packed dword p of the buffer; row r's
    // packed dwords r Q .. r Q + Q - 1 sit at stride S. A wavefront's LDS operations complete in order and no other
    // wavefront touches its buffer, so no barrier is needed. Where there is no full tile to fetch (the batch's end),
    // the batch's first tile is fetched instead and never used: the loads and their uses then need no branches, which
    // keeps them where they are written.
    s << "  const unsigned long long step = gridDim.x * tile;\n"
         "  const bool big = n >= 64;   // smaller batches have no full tile at all, and nothing is prefetched\n"
         "  const spn_v4* const tile0 = reinterpret_cast<const spn_v4*>(in);\n"
         "  spn_v4 r[" << H << "];   // half a tile as loaded: piece 64 j + lane\n"
         "  if (big) {\n"
         "    const unsigned long long first = blockIdx.x * tile + (threadIdx.x & ~63u);\n"
         "    const spn_v4* src = first + 64 <= n ? reinterpret_cast<const spn_v4*>(in + first * SPN_F) : tile0;\n";
    issue(0, H, "    ");
    stash(0, H, "    ");
    issue(H, Q - H, "    ");
    stash(H, Q - H, "    ");
    s << "  }\n"
         "  for (unsigned long long base = blockIdx.x * tile; base < n; base += step) {\n"
         "    const unsigned long long first = base + (threadIdx.x & ~63u);   // first row of this wavefront's 64\n"
         "    unsigned R[SPN_Q];   // the lane's row, four features to a register, a byte each\n"
         "    const unsigned long long i = first + lane;\n"
         "    if (first + 64 <= n) {\n"
         "#pragma unroll\n"
         "      for (unsigned c = 0; c < SPN_Q; ++c) R[c] = mine[lane * SPN_S + c];\n"
         "    } else {\n"
         "      // the batch's last, partial group of 64 rows: every lane fetches its own row (idle lanes the last one)\n"
         "      feat_t x[SPN_F];\n"
         "      spn_load_row(in, i < n ? i : n - 1, x);\n"
         "#pragma unroll\n"
         "      for (unsigned c = 0; c + 1 < SPN_Q; c += 2) spn_pack8(R[c], R[c + 1], x[4 * c], x[4 * c + 1], x[4 * c + 2], x[4 * c + 3], x[4 * c + 4], x[4 * c + 5], x[4 * c + 6], x[4 * c + 7]);\n"
         "      if (SPN_Q & 1) R[SPN_Q - 1] = spn_pack4(x[SPN_F - 4], x[SPN_F - 3], x[SPN_F - 2], x[SPN_F - 1]);\n"
         "    }\n"
         "    const spn_v4* src = first + step + 64 <= n ? reinterpret_cast<const spn_v4*>(in + (first + step) * SPN_F) : tile0;\n"
         "    if (big) {\n";
    issue(0, H, "      ");
    s << "    }\n"
         "    const real_t value = spn_eval(R, tab, spn_tab_lds, [&] {\n"
         "      if (big) {\n";
    stash(0, H, "        ");
    issue(H, Q - H, "        ");
    s << "      }\n"
         "    });\n"
         "    if (big) {\n";
    stash(H, Q - H, "      ");
    s << "    }\n"
         "    if (i < n) __builtin_nontemporal_store(value, out + i);\n";
  } else {
    s << "  for (unsigned long long base = blockIdx.x * tile; base < n; base += gridDim.x * tile) {\n";
  }
  // Kernels whose multiply-adds read constants from other lanes of their row (lane constants) keep every lane of a
  // wavefront at work: a cross-lane operand taken from a lane that is switched off disables the instruction in the lane
  // that reads it. The lanes past the batch's end evaluate its last row and do not store.
  const bool allLanes = !e.kPool.empty();
  const std::string tailText =
      std::string("      for (int u = 0; u < SPN_U; ++u) {\n"
                  "        const unsigned long long i = base + (unsigned long long)u * SPN_BLOCK + threadIdx.x;\n") +
      (allLanes ? "        {\n"
                  "          feat_t x[SPN_F];\n"
                  "          spn_load_row(in, i < n ? i : n - 1, x);\n"
                  "          const real_t value = spn_eval(x, tab);\n"
                  "          if (i < n) out[i] = value;\n"
                : "        if (i < n) {\n"
                  "          feat_t x[SPN_F];\n"
                  "          spn_load_row(in, i, x);\n"
                  "          out[i] = spn_eval(x, tab);\n") +
      "        }\n"
      "      }\n";
  const char* tail = tailText.c_str();
  if (prefetch) {
    // emitted above
  } else if (waveTile) {
    // Piece p = 64 j + lane of the tile (16 bytes, four features of row p / Q) goes to packed dword p of the tile; row r's
    // packed dwords r Q .. r Q + Q - 1 sit at stride S. A wavefront's LDS operations complete in order and no other
    // wavefront touches its buffer, so no barrier is needed.
    s << "    const unsigned long long first = base + (threadIdx.x & ~63u);   // first row of this wavefront's 64\n"
         "    unsigned R[SPN_Q];   // the lane's row, four features to a register, a byte each\n"
         "    unsigned long long i = first + lane;\n"
         "    if (first + 64 <= n) {\n"
         "      const spn_v4* src = reinterpret_cast<const spn_v4*>(in + first * SPN_F);\n"
         "      spn_v4 r[SPN_Q];\n"
         "#pragma unroll\n"
         "      for (unsigned j = 0; j < SPN_Q; ++j) r[j] = SPN_LOAD_TILE(src + j * 64 + lane);\n"
      << "      unsigned packed[SPN_Q];\n"
         "#pragma unroll\n"
         "      for (unsigned j = 0; j + 1 < SPN_Q; j += 2) spn_pack8(packed[j], packed[j + 1], r[j][0], r[j][1], r[j][2], r[j][3], r[j + 1][0], r[j + 1][1], r[j + 1][2], r[j + 1][3]);\n"
         "      if (SPN_Q & 1) packed[SPN_Q - 1] = spn_pack4(r[SPN_Q - 1][0], r[SPN_Q - 1][1], r[SPN_Q - 1][2], r[SPN_Q - 1][3]);\n"
         "#pragma unroll\n"
         "      for (unsigned j = 0; j < SPN_Q; ++j) {\n"
         "        const unsigned p = j * 64 + lane;\n"
         "        mine[p + p / SPN_Q * (SPN_S - SPN_Q)] = packed[j];\n"
         "      }\n"
         "#pragma unroll\n"
         "      for (unsigned c = 0; c < SPN_Q; ++c) R[c] = mine[lane * SPN_S + c];\n"
         "    } else {\n"
         "      // the batch's last, partial group of 64 rows: every lane fetches its own row (idle lanes the last one)\n"
         "      feat_t x[SPN_F];\n"
         "      spn_load_row(in, i < n ? i : n - 1, x);\n"
         "#pragma unroll\n"
         "      for (unsigned c = 0; c + 1 < SPN_Q; c += 2) spn_pack8(R[c], R[c + 1], x[4 * c], x[4 * c + 1], x[4 * c + 2], x[4 * c + 3], x[4 * c + 4], x[4 * c + 5], x[4 * c + 6], x[4 * c + 7]);\n"
         "      if (SPN_Q & 1) R[SPN_Q - 1] = spn_pack4(x[SPN_F - 4], x[SPN_F - 3], x[SPN_F - 2], x[SPN_F - 1]);\n"
         "    }\n";
    if (e.packedRows) {
      s << "    const real_t value = spn_eval(R, tab, spn_tab_lds);\n";
    } else {
      s << "    feat_t x[SPN_F];\n"
           "#pragma unroll\n"
           "    for (unsigned c = 0; c < SPN_Q; ++c) {\n"
           "      x[4 * c] = R[c] & 255u;\n      x[4 * c + 1] = (R[c] >> 8) & 255u;\n      x[4 * c + 2] = (R[c] >> 16) & 255u;\n      x[4 * c + 3] = R[c] >> 24;\n"
           "    }\n"
           "    const real_t value = spn_eval(x, tab);\n";
    }
    s << "    if (i < n) __builtin_nontemporal_store(value, out + i);\n";
  } else if (staged) {
    s << "    if (base + tile <= n) {\n"
         "      const spn_v4* src = reinterpret_cast<const spn_v4*>(in + base * SPN_F);\n"
         "      spn_v4* dst = reinterpret_cast<spn_v4*>(spn_tile);\n"
         "      constexpr unsigned NV = SPN_BLOCK * SPN_U * SPN_F * sizeof(feat_t) / 16;\n"
         "#pragma unroll\n"
         "      for (unsigned v = threadIdx.x; v < NV; v += SPN_BLOCK) dst[v] = SPN_LOAD_TILE(src + v);\n"
         "      __syncthreads();\n"
         "      feat_t x[SPN_U][SPN_F];\n"
         "#pragma unroll\n"
         "      for (int u = 0; u < SPN_U; ++u)\n"
         "#pragma unroll\n"
         "        for (int f = 0; f < SPN_F; ++f) x[u][f] = spn_tile[(u * SPN_BLOCK + threadIdx.x) * SPN_F + f];\n"
         "      __syncthreads();\n"
         "#pragma unroll\n"
         "      for (int u = 0; u < SPN_U; ++u)\n"
         "        __builtin_nontemporal_store(spn_eval(x[u], tab), out + base + (unsigned long long)u * SPN_BLOCK + threadIdx.x);\n"
         "    } else {\n"
      << tail << "    }\n";
  } else if (U == 1) {
    if (allLanes)
      s << "    const unsigned long long row = base + threadIdx.x;\n"
           "    const unsigned long long i = row < n ? row : n - 1;\n"
           "    {\n";
    else
      s << "    const unsigned long long i = base + threadIdx.x;\n"
           "    if (i < n) {\n";
    if (e.vectorRows)
      s << "      feat_t x[SPN_F];\n"
           "      spn_load_row(in, i, x);\n"
           "      const real_t value = spn_eval(x, tab" << taskArgs << ");\n";
    else
      s << "      const real_t value = spn_eval(in + i * SPN_F, tab" << taskArgs << ");\n";
    if (!g.isTask || g.taskFinal) s << (allLanes ? "      if (row < n) " : "      ") << "__builtin_nontemporal_store(value, out + i);\n";
    else s << "      (void)value;\n";
    s << "    }\n";
  } else {
    s << "    if (base + tile <= n) {\n"
         "      feat_t x[SPN_U][SPN_F];\n"
         "#pragma unroll\n"
         "      for (int u = 0; u < SPN_U; ++u) spn_load_row(in, base + (unsigned long long)u * SPN_BLOCK + threadIdx.x, x[u]);\n"
         "#pragma unroll\n"
         "      for (int u = 0; u < SPN_U; ++u)\n"
         "        __builtin_nontemporal_store(spn_eval(x[u], tab), out + base + (unsigned long long)u * SPN_BLOCK + threadIdx.x);\n"
         "    } else {\n"
      << tail << "    }\n";
  }
  s << "  }\n"
       "}\n";
  js.source = s.str();
  return js;
}

}  // namespace spnc_hip
