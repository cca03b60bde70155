#include "spn_graph.h"

#include <algorithm>
#include <cmath>
#include <map>
#include <stdexcept>
#include <unordered_map>

#include "capnp_reader.h"

namespace spnc_hip {

namespace {

[[noreturn]] void fatal(const std::string& msg) { throw std::runtime_error(msg); }

// Field offsets follow the standard Cap'n Proto layout of the reference's schema
// (xspn/xspn/serialization/binary/capnproto/spflow.capnp:27-102).
RawNode decodeNode(const capnp::StructReader& s) {
  RawNode n;
  n.id = s.get<int32_t>(0);
  n.root = s.getBool(32);
  uint16_t which = s.get<uint16_t>(6);
  capnp::StructReader body = s.getStruct(0);
  switch (which) {
    case 0:
      n.kind = NodeKind::Product;
      n.children = body.getList(0).toVector<int32_t>();
      break;
    case 1:
      n.kind = NodeKind::Sum;
      n.children = body.getList(0).toVector<int32_t>();
      n.weights = body.getList(1).toVector<double>();
      break;
    case 2:
      n.kind = NodeKind::Histogram;
      n.breaks = body.getList(0).toVector<int32_t>();
      n.densities = body.getList(1).toVector<double>();
      n.scope = body.get<int32_t>(4);
      break;
    case 3:
      n.kind = NodeKind::Gaussian;
      n.mean = body.get<double>(0);
      n.stddev = body.get<double>(8);
      n.scope = body.get<int32_t>(16);
      break;
    case 4:
      n.kind = NodeKind::Categorical;
      n.probabilities = body.getList(0).toVector<double>();
      n.scope = body.get<int32_t>(0);
      break;
    default:
      fatal("Unsupported node type " + std::to_string(which));
  }
  return n;
}

RawModel decodeModel(const capnp::StructReader& m) {
  RawModel out;
  out.rootNode = m.get<int32_t>(0);
  out.numFeatures = m.get<int32_t>(4);
  out.name = m.getText(0);
  out.featureType = m.getText(1);
  out.scope = m.getList(2).toVector<int32_t>();
  capnp::ListReader nodes = m.getList(3);
  out.nodes.reserve(nodes.size());
  for (size_t i = 0; i < nodes.size(); ++i) out.nodes.push_back(decodeNode(nodes.getStruct(i)));
  return out;
}

}  // namespace

RawQuery readQueryFile(const std::string& path) {
  capnp::Message msg = capnp::Message::fromFile(path);
  capnp::StructReader header = msg.root();
  uint16_t which = header.get<uint16_t>(0);
  if (which == 0) fatal("Cannot compile raw models");
  if (which != 1) fatal("Unknown header content");
  capnp::StructReader query = header.getStruct(0);
  if (!query.hasPointer(0)) fatal("Can only deserialize joint queries");
  RawQuery q;
  q.batchSize = query.get<int32_t>(0);
  q.errorKind = query.get<uint16_t>(4);
  q.maxError = query.get<double>(8);
  capnp::StructReader joint = query.getStruct(0);
  if (!joint.hasPointer(0)) fatal("No model attached to query");
  q.supportMarginal = joint.getBool(0);  // absent in files written before the field existed
  q.model = decodeModel(joint.getStruct(0));
  return q;
}

FeatureTypeInfo parseFeatureType(const std::string& text) {
  // Accepts the spellings of the reference's translateTypeString
  // (SPFlowToMLIRDeserializer.cpp:226-248): "[u]int<width>" and "float<width>".
  auto digits = [](const std::string& s, size_t from) -> int {
    if (from >= s.size()) return -1;
    int v = 0;
    for (size_t i = from; i < s.size(); ++i) {
      if (s[i] < '1' || s[i] > '9') return -1;
      v = v * 10 + (s[i] - '0');
      if (v > 4096) return -1;
    }
    return v;
  };
  size_t p = 0;
  if (text.rfind("uint", 0) == 0) p = 4;
  else if (text.rfind("int", 0) == 0) p = 3;
  if (p) {
    switch (digits(text, p)) {
      case 8: return {FeatureType::U8, 1, false, "unsigned char"};
      case 16: return {FeatureType::U16, 2, false, "unsigned short"};
      case 32: return {FeatureType::U32, 4, false, "unsigned int"};
      case 64: return {FeatureType::U64, 8, false, "unsigned long long"};
      default: fatal("Unsupported feature data type " + text);
    }
  }
  if (text.rfind("float", 0) == 0) {
    switch (digits(text, 5)) {
      case 32: return {FeatureType::F32, 4, true, "float"};
      case 64: return {FeatureType::F64, 8, true, "double"};
      case -1: break;
      default: fatal("Unsupported floating-point type " + text);
    }
  }
  fatal("Unsupported feature data type " + text);
}

namespace {

void checkNormalized(const std::vector<double>& v, const char* msg) {
  double sum = 0;
  for (double p : v) sum += p;
  if (!(std::fabs(sum - 1.0) <= 1e-6)) fatal(msg);
}

// Flat [0, maxUB) density table with zeros in gaps; the same table the reference builds before
// taking logs (mlir/lib/Conversion/LoSPNtoCPU/NodePatterns.cpp:447-493).
std::vector<double> histogramTable(const RawNode& n) {
  if (n.breaks.size() < 2) fatal("Histogram needs at least two breaks");
  size_t buckets = n.breaks.size() - 1;
  if (n.densities.size() < buckets) fatal("bucketCount must match the actual number of buckets!");
  std::vector<std::pair<int64_t, int64_t>> iv;
  int64_t minLB = INT64_MAX, maxUB = INT64_MIN;
  for (size_t i = 0; i < buckets; ++i) {
    int64_t lb = n.breaks[i], ub = n.breaks[i + 1];
    if (ub < lb) fatal("Lower bound must be less or equal to upper bound!");
    iv.emplace_back(lb, ub);
    minLB = std::min(minLB, lb);
    maxUB = std::max(maxUB, ub);
  }
  std::vector<std::pair<int64_t, int64_t>> sorted = iv;
  std::sort(sorted.begin(), sorted.end());
  for (size_t i = 1; i < sorted.size(); ++i)
    if (sorted[i].first < sorted[i - 1].second) fatal("Overlapping buckets in histogram!");
  if (minLB < 0) fatal("Histogram buckets with negative lower bound are not supported");
  if (maxUB > (int64_t(1) << 24)) fatal("Histogram upper bound too large");
  std::vector<double> tab(size_t(maxUB), 0.0);
  for (size_t i = 0; i < buckets; ++i)
    for (int64_t v = iv[i].first; v < iv[i].second; ++v) tab[size_t(v)] = n.densities[i];
  return tab;
}

void appendBytes(std::string& key, const void* p, size_t n) { key.append(reinterpret_cast<const char*>(p), n); }

std::string structuralKey(const GraphNode& g) {
  std::string key;
  key.push_back(char(g.kind));
  switch (g.kind) {
    case NodeKind::External: break;  // only inside the tasks of a cut graph (partition.cpp), never here
    case NodeKind::Gaussian:
      appendBytes(key, &g.feature, 4);
      appendBytes(key, &g.mean, 8);
      appendBytes(key, &g.stddev, 8);
      break;
    case NodeKind::Categorical:
    case NodeKind::Histogram:
      appendBytes(key, &g.feature, 4);
      appendBytes(key, g.table.data(), g.table.size() * 8);
      break;
    case NodeKind::Sum:
      appendBytes(key, g.weights.data(), g.weights.size() * 8);
      [[fallthrough]];
    case NodeKind::Product:
      appendBytes(key, g.children.data(), g.children.size() * 4);
      break;
  }
  return key;
}

}  // namespace

Graph buildGraph(const RawQuery& q) {
  const RawModel& m = q.model;
  Graph g;
  g.name = m.name.empty() ? std::string("spn_kernel") : m.name;
  g.ftype = parseFeatureType(m.featureType);
  g.supportMarginal = q.supportMarginal;
  g.batchSize = q.batchSize;
  if (m.numFeatures <= 0) fatal("Query has no input features");
  if (size_t(m.numFeatures) != m.scope.size()) fatal("Number of features does not match the size of the scope");
  g.numFeatures = uint32_t(m.numFeatures);
  if (q.supportMarginal && !g.ftype.isFloat) fatal("Feature data type must be floating-point to support marginal");

  // Scope values map to input columns in ascending order.
  std::vector<int32_t> sortedScope = m.scope;
  std::sort(sortedScope.begin(), sortedScope.end());
  std::map<int32_t, uint32_t> column;
  for (size_t i = 0; i < sortedScope.size(); ++i) column[sortedScope[i]] = uint32_t(i);

  // Pass 1: validate every serialized node in file order; children must already be defined.
  std::unordered_map<int32_t, size_t> defined;  // id -> index into m.nodes
  for (size_t i = 0; i < m.nodes.size(); ++i) {
    const RawNode& n = m.nodes[i];
    switch (n.kind) {
      case NodeKind::External: break;  // only inside the tasks of a cut graph (partition.cpp), never here
      case NodeKind::Product:
        if (n.children.empty()) fatal("Number of operands must be at least one");
        break;
      case NodeKind::Sum:
        if (n.weights.size() != n.children.size()) fatal("Number of weights must match the number of addends!");
        if (n.children.empty()) fatal("Number of addends must be greater than zero!");
        checkNormalized(n.weights, "Weights must sum up to 1.0 for normalized SPN");
        break;
      case NodeKind::Categorical:
        checkNormalized(n.probabilities, "Category probabilities should sum to 1.0");
        [[fallthrough]];
      case NodeKind::Histogram:
      case NodeKind::Gaussian:
        if (!column.count(n.scope)) fatal("Leaf node references unknown feature!");
        break;
    }
    for (int32_t c : n.children)
      if (!defined.count(c)) fatal("No definition found for node with ID: " + std::to_string(c));
    defined[n.id] = i;
  }
  if (!defined.count(m.rootNode)) fatal("No definition found for node with ID: " + std::to_string(m.rootNode));
  g.stats.serializedNodes = uint32_t(m.nodes.size());

  // Pass 2: depth-first post-order from the root with structural deduplication.
  std::unordered_map<size_t, uint32_t> placed;         // raw index -> graph index
  std::unordered_map<std::string, uint32_t> interned;  // structural key -> graph index
  struct Frame {
    size_t raw;
    size_t next;
  };
  std::vector<Frame> stack{{defined[m.rootNode], 0}};
  while (!stack.empty()) {
    Frame& f = stack.back();
    const RawNode& n = m.nodes[f.raw];
    if (placed.count(f.raw)) {
      stack.pop_back();
      continue;
    }
    if (f.next < n.children.size()) {
      size_t child = defined[n.children[f.next++]];
      if (!placed.count(child)) stack.push_back({child, 0});
      continue;
    }
    GraphNode gn;
    gn.kind = n.kind;
    switch (n.kind) {
      case NodeKind::External: break;  // only inside the tasks of a cut graph (partition.cpp), never here
      case NodeKind::Product:
      case NodeKind::Sum:
        for (int32_t c : n.children) gn.children.push_back(placed.at(defined[c]));
        gn.weights = n.weights;
        break;
      case NodeKind::Gaussian:
        gn.feature = column[n.scope];
        gn.mean = n.mean;
        gn.stddev = n.stddev;
        if (!(n.stddev > 0) || !std::isfinite(n.stddev) || !std::isfinite(n.mean))
          fatal("Gaussian leaf needs a finite mean and a positive finite standard deviation");
        break;
      case NodeKind::Categorical:
        gn.feature = column[n.scope];
        gn.table = n.probabilities;
        break;
      case NodeKind::Histogram:
        gn.feature = column[n.scope];
        gn.table = histogramTable(n);
        break;
    }
    std::string key = structuralKey(gn);
    auto it = interned.find(key);
    uint32_t idx;
    if (it != interned.end()) {
      idx = it->second;
    } else {
      idx = uint32_t(g.nodes.size());
      g.nodes.push_back(std::move(gn));
      interned.emplace(std::move(key), idx);
    }
    placed[f.raw] = idx;
    stack.pop_back();
  }
  // The root must be the last node; with deduplication it always is, because nothing is
  // appended after the root is placed.
  uint32_t rootIdx = placed.at(defined[m.rootNode]);
  if (rootIdx != g.nodes.size() - 1) fatal("internal error: root is not last in schedule");

  // Scopes, children first: completeness and decomposability.
  {
    const size_t words = (g.numFeatures + 63) / 64;
    std::vector<std::vector<uint64_t>> scope(g.nodes.size(), std::vector<uint64_t>(words, 0));
    bool ok = true;
    for (size_t i = 0; i < g.nodes.size() && ok; ++i) {
      const GraphNode& n = g.nodes[i];
      if (n.kind != NodeKind::Product && n.kind != NodeKind::Sum) {
        scope[i][n.feature / 64] |= uint64_t(1) << (n.feature % 64);
        continue;
      }
      for (size_t k = 0; k < n.children.size() && ok; ++k) {
        const std::vector<uint64_t>& cs = scope[n.children[k]];
        if (n.kind == NodeKind::Sum) {
          if (k == 0) scope[i] = cs;
          else if (scope[i] != cs) ok = false;
        } else {
          for (size_t w = 0; w < words; ++w) {
            if (scope[i][w] & cs[w]) ok = false;
            scope[i][w] |= cs[w];
          }
        }
      }
    }
    g.completeDecomposable = ok;
  }

  // Use counts and statistics.
  for (auto& n : g.nodes)
    for (uint32_t c : n.children) g.nodes[c].uses++;
  g.nodes.back().uses++;
  GraphStats& st = g.stats;
  uint64_t leafSelect = q.supportMarginal ? 1 : 0;
  uint64_t ownSelects = 0, ownCorrections = 0;
  for (const auto& n : g.nodes) {
    uint64_t k = n.children.size();
    st.maxFanIn = std::max<uint32_t>(st.maxFanIn, uint32_t(k));
    switch (n.kind) {
      case NodeKind::External: break;  // only inside the tasks of a cut graph (partition.cpp), never here
      case NodeKind::Gaussian:
        st.gaussians++;
        st.flopsMin += 4 + leafSelect;
        st.flopsPairwise += 4 + leafSelect;
        st.fusedMin += 1;
        break;
      case NodeKind::Categorical:
        st.categoricals++;
        st.flopsMin += leafSelect;
        st.flopsPairwise += leafSelect;
        break;
      case NodeKind::Histogram:
        st.histograms++;
        st.flopsMin += leafSelect;
        st.flopsPairwise += leafSelect;
        break;
      case NodeKind::Product:
        st.products++;
        st.productAdds += k - 1;
        st.flopsMin += k - 1;
        st.flopsPairwise += k - 1;
        {
          uint64_t own = 0;  // Gaussian children read by this product only
          for (uint32_t c : n.children) own += g.nodes[c].kind == NodeKind::Gaussian && g.nodes[c].uses == 1 ? 1 : 0;
          st.fusedMin += std::min<uint64_t>(own, k ? k - 1 : 0);
          // Marginal queries: such leaves need no select of their own. A missing feature is replaced once by a stand-in
          // value, and what the leaves over missing features add to the product is taken off with one table value per
          // four leaves (one add each).
          if (leafSelect && own) ownSelects += own, ownCorrections += (own + 3) / 4;
        }
        break;
      case NodeKind::Sum: {
        st.sums++;
        st.sumTerms += k;
        uint64_t fp = 8 * k - 7, tp = 2 * (k - 1);
        uint64_t fn = 5 * k, tn = k + 1;
        st.flopsPairwise += fp;
        st.transPairwise += tp;
        if (k <= 1) {
          st.flopsMin += 1;  // a single weighted child is one add
        } else if (fp + 3 * tp <= fn + 3 * tn) {
          st.flopsMin += fp;
          st.transMin += tp;
        } else {
          st.flopsMin += fn;
          st.transMin += tn;
        }
        break;
      }
    }
  }
  if (ownSelects) {   // instead of a select per leaf: an add per correction, and per Gaussian feature the stand-in and its bit of the pattern
    std::vector<bool> gaussianFeature(g.numFeatures, false);
    for (const auto& n : g.nodes)
      if (n.kind == NodeKind::Gaussian) gaussianFeature[n.feature] = true;
    uint64_t perFeature = 0;
    for (bool b : gaussianFeature) perFeature += b ? 2 : 0;
    if (ownCorrections + perFeature < ownSelects) st.flopsMin = st.flopsMin - ownSelects + ownCorrections + perFeature;
  }
  // Sums over a complete outer product of two operand vectors: M sums share the ordered child list
  // [prod(a_0,b_0), ..., prod(a_NA-1,b_NB-1)] and nothing else reads those products. Since
  // exp(a_r + b_c - ma - mb) = exp(a_r - ma) * exp(b_c - mb), the group costs NA + NB exponentials, not M*NA*NB.
  // Where that factored form is cheaper than the per-sum accounting above, it is the algorithmic minimum.
  // A group whose sums are read only by the products of one other group, as that group's complete first or
  // second operand vector, can hand them over as acc_t / max(acc) plus one common scale: one logarithm and one
  // reciprocal for the vector instead of a logarithm per sum, and no maximum, shift or exponential for that
  // vector in the consumer.
  struct OuterGroup {
    std::vector<uint32_t> members, a, b;  // the sums (ascending node order) and the two operand vectors
    uint64_t k = 0;
    bool outScaled = false, aScaled = false, bScaled = false;
  };
  std::map<std::vector<uint32_t>, std::vector<uint32_t>> byChildren;
  for (uint32_t i = 0; i < g.nodes.size(); ++i)
    if (g.nodes[i].kind == NodeKind::Sum && g.nodes[i].children.size() >= 4) byChildren[g.nodes[i].children].push_back(i);
  std::vector<OuterGroup> outerGroups;
  std::vector<int> groupOfProduct(g.nodes.size(), -1);
  for (const auto& entry : byChildren) {
    const std::vector<uint32_t>& kids = entry.first;
    const uint64_t members = entry.second.size(), k = kids.size();
    bool ok = true;
    for (uint32_t c : kids) {
      const auto& pn = g.nodes[c];
      if (pn.kind != NodeKind::Product || pn.children.size() != 2 || pn.uses != members) ok = false;
    }
    if (!ok) continue;
    uint64_t nb = 1;
    while (nb < k && g.nodes[kids[nb]].children[0] == g.nodes[kids[0]].children[0]) ++nb;
    if (nb < 2 || k % nb != 0 || k / nb < 2) continue;
    const uint64_t na = k / nb;
    for (uint64_t r = 0; r < na && ok; ++r)
      for (uint64_t c = 0; c < nb && ok; ++c) {
        const auto& pn = g.nodes[kids[r * nb + c]];
        ok = pn.children[0] == g.nodes[kids[r * nb]].children[0] && pn.children[1] == g.nodes[kids[c]].children[1];
      }
    std::vector<uint32_t> sorted = kids;
    std::sort(sorted.begin(), sorted.end());
    if (std::adjacent_find(sorted.begin(), sorted.end()) != sorted.end()) ok = false;
    if (!ok) continue;
    OuterGroup og;
    og.members = entry.second;
    og.k = k;
    for (uint64_t r = 0; r < na; ++r) og.a.push_back(g.nodes[kids[r * nb]].children[0]);
    for (uint64_t c = 0; c < nb; ++c) og.b.push_back(g.nodes[kids[c]].children[1]);
    for (uint32_t c : kids) groupOfProduct[c] = int(outerGroups.size());
    outerGroups.push_back(std::move(og));
  }
  std::vector<std::vector<uint32_t>> parents(g.nodes.size());
  for (uint32_t i = 0; i < g.nodes.size(); ++i)
    for (uint32_t c : g.nodes[i].children) parents[c].push_back(i);
  for (auto& og : outerGroups) {
    int consumer = -1;
    bool ok = true;
    for (uint32_t m : og.members) {
      if (m == g.root() || parents[m].empty()) ok = false;
      for (uint32_t pa : parents[m]) {
        if (groupOfProduct[pa] < 0) ok = false;
        else if (consumer < 0) consumer = groupOfProduct[pa];
        else if (consumer != groupOfProduct[pa]) ok = false;
      }
    }
    if (!ok || consumer < 0) continue;
    OuterGroup& cg = outerGroups[size_t(consumer)];
    if (cg.a == og.members) cg.aScaled = og.outScaled = true;
    else if (cg.b == og.members) cg.bScaled = og.outScaled = true;
  }
  for (const auto& og : outerGroups) {
    const uint64_t members = og.members.size(), k = og.k, na = og.a.size(), nb = og.b.size();
    // Per-sum accounting of the group, products included (k >= 4, so the n-ary form was the one charged).
    const uint64_t naiveFlops = members * 5 * k + k, naiveTrans = members * (k + 1);
    // Factored: per log-valued operand vector a maximum, a shift and an exponential per element (a scaled one
    // costs one add for its scale); NA*NB products; M*NA*NB multiply-adds; then a logarithm and an add per sum,
    // or for a scaled result M-1 maxima, a reciprocal, M multiplies, one logarithm and one add.
    uint64_t factFlops = k + members * k, factTrans = 0;
    factFlops += og.aScaled ? 1 : 2 * na;
    factTrans += og.aScaled ? 0 : na;
    factFlops += og.bScaled ? 1 : 2 * nb;
    factTrans += og.bScaled ? 0 : nb;
    factFlops += og.outScaled ? (members - 1) + members + 1 : 2 * members;
    factTrans += og.outScaled ? 2 : members;
    if (factFlops + 3 * factTrans < naiveFlops + 3 * naiveTrans) {
      st.flopsMin = st.flopsMin - naiveFlops + factFlops;
      st.transMin = st.transMin - naiveTrans + factTrans;
    }
  }
  return g;
}

namespace {

// Depth of operand i below the top operation of a balanced binary tree over k operands with pivot ceil(k/2)
// (mlir/lib/Conversion/HiSPNtoLoSPN/NodePatterns.cpp:17-40,49-88); a tree over one operand is that operand.
int treeDepth(size_t k, size_t i) {
  int d = 0;
  while (k > 2) {
    const size_t pivot = (k + 1) / 2;
    if (i < pivot) {
      k = pivot;
    } else {
      i -= pivot;
      k -= pivot;
    }
    ++d;
  }
  return k == 2 ? d + 1 : d;
}

}  // namespace

LoSpnStats computeLoSpnStats(const RawQuery& q, bool logSpace) {
  const RawModel& m = q.model;
  LoSpnStats st;
  std::unordered_map<int32_t, size_t> byId;
  for (size_t i = 0; i < m.nodes.size(); ++i) {
    const RawNode& n = m.nodes[i];
    byId[n.id] = i;
    const uint64_t k = n.children.size();
    switch (n.kind) {
      case NodeKind::External: break;  // only inside the tasks of a cut graph (partition.cpp), never here
      case NodeKind::Product: st.productCount += k ? k - 1 : 0; break;
      case NodeKind::Sum:
        st.sumCount += k ? k - 1 : 0;
        st.productCount += k;
        st.constantCount += k;
        break;
      case NodeKind::Categorical: st.categoricalCount++; break;
      case NodeKind::Gaussian: st.gaussianCount++; break;
      case NodeKind::Histogram: st.histogramCount++; break;
    }
  }
  // Leaf depths as the reference's SPNNodeLevel takes them (mlir/lib/Dialect/LoSPN/Analysis/SPNNodeLevel.cpp:19-97): a walk
  // from the root along every path, operands in order; an operation met again takes the larger of its old and new
  // level and hands that on, and a leaf is counted once per path that reaches it. Only the top operation of a
  // node's binary tree needs a stored level: the operations inside the tree follow it at fixed offsets.
  auto childDepth = [&](const RawNode& n, size_t i) { return treeDepth(n.children.size(), i) + (n.kind == NodeKind::Sum ? 1 : 0); };
  auto isLeaf = [](const RawNode& n) { return n.kind != NodeKind::Product && n.kind != NodeKind::Sum; };
  const int rootLevel = logSpace ? 0 : 1;
  std::map<int, double> histogram;  // leaf level -> visits
  double visits = 0;
  const auto rootIt = byId.find(m.rootNode);
  if (rootIt == byId.end()) return st;
  {
    std::vector<int> level(m.nodes.size(), -1);
    struct Frame {
      size_t node;
      int level;
      size_t next;
    };
    std::vector<Frame> stack;
    const double budget = 2e7;
    auto enter = [&](size_t node, int incoming) {
      const RawNode& n = m.nodes[node];
      // A product over one operand is that operand: it has no operation of its own.
      int lv = incoming;
      if (level[node] >= 0 && level[node] != incoming) lv = std::max(incoming, level[node]);
      level[node] = lv;
      if (isLeaf(n)) {
        histogram[lv] += 1;
        visits += 1;
      } else {
        stack.push_back({node, lv, 0});
      }
    };
    enter(rootIt->second, rootLevel);
    double steps = 0;
    while (!stack.empty() && steps <= budget) {
      Frame& f = stack.back();
      const RawNode& n = m.nodes[f.node];
      if (f.next >= n.children.size()) {
        stack.pop_back();
        continue;
      }
      const size_t i = f.next++;
      const auto it = byId.find(n.children[i]);
      if (it == byId.end()) continue;
      ++steps;
      enter(it->second, f.level + childDepth(n, i));
    }
    if (!stack.empty()) {
      // Heavily shared graphs (region graphs) have more root-to-leaf paths than anyone can walk. Their leaves are
      // then counted per path by recurrence over the graph, each at its path length, without the
      // larger-level-on-revisit rule of the walk, whose outcome depends on the order of the visits.
      st.depthsExact = false;
      histogram.clear();
      std::vector<std::map<int, double>> below(m.nodes.size());  // node -> (leaf depth below the node's top operation -> paths)
      std::vector<char> done(m.nodes.size(), 0);
      std::vector<std::pair<size_t, size_t>> work{{rootIt->second, 0}};
      while (!work.empty()) {
        auto& [node, next] = work.back();
        const RawNode& n = m.nodes[node];
        if (done[node]) {
          work.pop_back();
          continue;
        }
        if (isLeaf(n)) {
          below[node][0] = 1;
          done[node] = 1;
          work.pop_back();
          continue;
        }
        if (next < n.children.size()) {
          const auto it = byId.find(n.children[next++]);
          if (it != byId.end() && !done[it->second]) work.push_back({it->second, 0});
          continue;
        }
        for (size_t i = 0; i < n.children.size(); ++i) {
          const auto it = byId.find(n.children[i]);
          if (it == byId.end()) continue;
          for (const auto& [d, cnt] : below[it->second]) below[node][d + childDepth(n, i)] += cnt;
        }
        done[node] = 1;
        work.pop_back();
      }
      for (const auto& [d, cnt] : below[rootIt->second]) histogram[d + rootLevel] = cnt;
    }
  }
  if (histogram.empty()) return st;
  st.minDepth = histogram.begin()->first;
  st.maxDepth = histogram.rbegin()->first;
  double total = 0, weighted = 0;
  for (const auto& [d, cnt] : histogram) {
    total += cnt;
    weighted += d * cnt;
  }
  st.averageDepth = weighted / total;
  // The median as the reference finds it (SPNNodeLevel.cpp:43-60): the level whose bucket holds position n/2, and for an
  // even count whose position n/2+1 closes that bucket, the mean of that level and the next one. Where no next level
  // exists the reference reads past its set of levels; with its standard library that read yields the number of
  // distinct levels, which is what its own test expects (two leaves at depth 2: median 1.5) and what is kept here.
  const double pivot = total / 2.0;
  double index = 0;
  for (auto it = histogram.begin(); it != histogram.end(); ++it) {
    index += it->second;
    if (pivot < index && pivot > index - it->second) {
      if (std::fmod(total, 2.0) == 0 && double((long long)(pivot + 1)) == index) {
        auto nextBucket = std::next(it);
        const double nextLevel = nextBucket != histogram.end() ? double(nextBucket->first) : double(histogram.size());
        st.medianDepth = (double(it->first) + nextLevel) / 2.0;
      } else {
        st.medianDepth = it->first;
      }
    }
  }
  return st;
}

}  // namespace spnc_hip
