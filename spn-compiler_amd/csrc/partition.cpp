// Graph partitioning for "maxTaskSize": a large DAG becomes several tasks that run back to back and hand values on
// through a [rows x samples] buffer in device memory.
//
// Follows the reference's partitioner in what it does, on this library's n-ary, deduplicated graph instead of the
// binarised LoSPN operations:
//   - initial partitioning: a topological order built with a stack, so that a node's consumers follow it closely and the
//     cuts run "vertically" through the DAG, chopped into chunks of maxTaskSize operations
//     (mlir/lib/Dialect/LoSPN/Partitioning/GraphPartitioner.cpp:92-157);
//   - refinement: one pass that moves a node to the neighbouring partition when that removes more values crossing a cut
//     than it adds, or balances sizes at equal cost (Partitioning/Heuristic.cpp:50-189), within 1 % slack
//     (GraphPartitioner.cpp:84-88);
//   - one task per partition with the values other partitions need as its results
//     (Passes/LoSPNTaskPartitioner.cpp:150-330); rows of the intermediate buffer are reused once their last reader ran.
#include <algorithm>
#include <cstdint>
#include <map>
#include <stdexcept>

#include "spn_graph.h"

namespace spnc_hip {

uint64_t taskWeight(const GraphNode& n) {
  const uint64_t k = n.children.size();
  switch (n.kind) {
    case NodeKind::External: return 0;
    case NodeKind::Product: return k > 1 ? k - 1 : 1;
    case NodeKind::Sum: return k ? 2 * k - 1 : 1;
    default: return 1;
  }
}

uint64_t taskWeight(const Graph& g) {
  uint64_t w = 0;
  for (const auto& n : g.nodes) w += taskWeight(n);
  return w;
}

namespace {

// Sums and products heavier than `limit` become trees: groups of children under new nodes of the same kind (new sums
// weigh their children with 1), level by level until the top node fits too.
std::vector<GraphNode> splitHeavyNodes(const std::vector<GraphNode>& in, uint64_t limit) {
  std::vector<GraphNode> out;
  std::vector<uint32_t> remap(in.size());
  for (uint32_t i = 0; i < in.size(); ++i) {
    GraphNode n = in[i];
    n.uses = 0;
    for (uint32_t& c : n.children) c = remap[c];
    const bool inner = n.kind == NodeKind::Sum || n.kind == NodeKind::Product;
    const size_t group = n.kind == NodeKind::Sum ? std::max<size_t>(2, size_t((limit + 1) / 2)) : std::max<size_t>(2, size_t(limit + 1));
    while (inner && taskWeight(n) > limit && n.children.size() > group) {
      GraphNode top = n;
      top.children.clear();
      top.weights.clear();
      for (size_t at = 0; at < n.children.size(); at += group) {
        const size_t end = std::min(n.children.size(), at + group);
        if (end - at == 1) {
          top.children.push_back(n.children[at]);
          if (n.kind == NodeKind::Sum) top.weights.push_back(n.weights[at]);
          continue;
        }
        GraphNode part = n;
        part.children.assign(n.children.begin() + at, n.children.begin() + end);
        if (n.kind == NodeKind::Sum) part.weights.assign(n.weights.begin() + at, n.weights.begin() + end);
        out.push_back(std::move(part));
        top.children.push_back(uint32_t(out.size() - 1));
        if (n.kind == NodeKind::Sum) top.weights.push_back(1.0);
      }
      n = std::move(top);
    }
    out.push_back(std::move(n));
    remap[i] = uint32_t(out.size() - 1);
  }
  for (auto& n : out)
    for (uint32_t c : n.children) out[c].uses++;
  out.back().uses++;
  return out;
}

void basicStats(Graph& g) {
  GraphStats st;
  const uint64_t leafSelect = g.supportMarginal ? 1 : 0;
  for (const auto& n : g.nodes) {
    const uint64_t k = n.children.size();
    st.maxFanIn = std::max<uint32_t>(st.maxFanIn, uint32_t(k));
    switch (n.kind) {
      case NodeKind::External: break;
      case NodeKind::Gaussian: st.gaussians++; st.flopsMin += 4 + leafSelect; st.flopsPairwise += 4 + leafSelect; st.fusedMin += 1; break;
      case NodeKind::Categorical: st.categoricals++; st.flopsMin += leafSelect; st.flopsPairwise += leafSelect; break;
      case NodeKind::Histogram: st.histograms++; st.flopsMin += leafSelect; st.flopsPairwise += leafSelect; break;
      case NodeKind::Product: st.products++; st.productAdds += k - 1; st.flopsMin += k - 1; st.flopsPairwise += k - 1; break;
      case NodeKind::Sum: {
        st.sums++;
        st.sumTerms += k;
        const uint64_t fp = 8 * k - 7, tp = 2 * (k - 1), fn = 5 * k, tn = k + 1;
        st.flopsPairwise += fp;
        st.transPairwise += tp;
        if (k <= 1) st.flopsMin += 1;
        else if (fp + 3 * tp <= fn + 3 * tn) st.flopsMin += fp, st.transMin += tp;
        else st.flopsMin += fn, st.transMin += tn;
        break;
      }
    }
  }
  st.serializedNodes = uint32_t(g.nodes.size());
  g.stats = st;
}

}  // namespace

TaskPlan partitionGraph(const Graph& g, int maxTaskSize) {
  TaskPlan plan;
  if (maxTaskSize <= 0) throw std::runtime_error("maxTaskSize must be positive to partition a graph");
  const uint64_t limit = uint64_t(maxTaskSize);
  const uint64_t boundary = limit + std::max<uint64_t>(1, uint64_t(double(limit) * 0.01));  // 1 % slack, at least one operation
  if (taskWeight(g) <= boundary) {
    plan.tasks.push_back(g);
    return plan;
  }
  const std::vector<GraphNode> nodes = splitHeavyNodes(g.nodes, limit);
  const uint32_t N = uint32_t(nodes.size()), root = N - 1;
  std::vector<std::vector<uint32_t>> users(N);
  for (uint32_t i = 0; i < N; ++i)
    for (uint32_t c : nodes[i].children)
      if (users[c].empty() || users[c].back() != i) users[c].push_back(i);

  // ---- initial partitioning: stack-driven topological order, cut into chunks ----
  std::vector<uint32_t> pending(N), order;
  std::vector<uint32_t> stack;
  for (uint32_t i = 0; i < N; ++i) {
    std::vector<uint32_t> distinct = nodes[i].children;
    std::sort(distinct.begin(), distinct.end());
    pending[i] = uint32_t(std::unique(distinct.begin(), distinct.end()) - distinct.begin());
  }
  for (uint32_t i = N; i-- > 0;)
    if (pending[i] == 0) stack.push_back(i);  // leaves, the first one on top
  while (!stack.empty()) {
    const uint32_t cur = stack.back();
    stack.pop_back();
    order.push_back(cur);
    for (uint32_t u : users[cur])
      if (--pending[u] == 0) stack.push_back(u);
  }
  if (order.size() != N) throw std::runtime_error("INTERNAL ERROR: partitioning lost nodes of the graph");
  std::vector<uint32_t> part(N, 0);
  std::vector<uint64_t> size;
  {
    uint64_t filled = 0;
    size.push_back(0);
    for (uint32_t i : order) {
      const uint64_t w = taskWeight(nodes[i]);
      if (filled > 0 && filled + w > limit) {
        size.push_back(0);
        filled = 0;
      }
      part[i] = uint32_t(size.size() - 1);
      size.back() += w;
      filled += w;
    }
  }
  const uint32_t P = uint32_t(size.size());

  // ---- refinement: one pass of single-node moves to a neighbouring partition ----
  for (uint32_t i = 0; i < N && P > 1; ++i) {
    const uint32_t p = part[i];
    const uint64_t w = taskWeight(nodes[i]);
    const int none = INT32_MIN;
    int up = none, down = none;
    if (p + 1 < P && i != root) {
      // Gain of moving to p + 1: the value no longer crosses into p + 1 (+1), every operand defined in p starts to (-1 each).
      int gain = 0;
      bool legal = true;
      for (uint32_t u : users[i]) {
        if (part[u] == p + 1) gain = 1;
        if (part[u] == p) legal = false;
      }
      for (uint32_t c : nodes[i].children)
        if (part[c] == p) --gain;
      if (legal) up = gain;
    }
    if (p > 0) {
      // Gain of moving to p - 1: operands defined there become internal (+1 each); users left behind in p make the value cross (-1).
      int gain = 0;
      bool legal = true;
      for (uint32_t c : nodes[i].children) {
        if (part[c] == p - 1) ++gain;
        if (part[c] == p) legal = false;
      }
      bool usedInSame = false;
      for (uint32_t u : users[i]) usedInSame = usedInSame || part[u] == p;
      if (usedInSame) --gain;
      if (legal) down = gain;
    }
    auto accepts = [&](uint32_t q) { return size[q] + w <= boundary; };
    auto move = [&](uint32_t q) {
      size[p] -= w;
      size[q] += w;
      part[i] = q;
    };
    const long long here = (long long)size[p];
    if (up == down && up >= 0) {
      const long long upDiff = here - (long long)size[p + 1], downDiff = here - (long long)size[p - 1];
      if (upDiff > downDiff && (upDiff > 0 || up > 0) && accepts(p + 1)) move(p + 1);
      else if ((downDiff > 0 || down > 0) && accepts(p - 1)) move(p - 1);
    } else if (up > down && up >= 0) {
      if ((up > 0 || here - (long long)size[p + 1] > 0) && accepts(p + 1)) move(p + 1);
    } else if (down > up && down >= 0) {
      if ((down > 0 || here - (long long)size[p - 1] > 0) && accepts(p - 1)) move(p - 1);
    }
  }

  // ---- tasks ----
  // Rows of the intermediate buffer: a value gets one in the task that computes it and gives it back after the last task
  // that reads it; a task's results only take rows that were free before it started, so a kernel never reads and
  // writes the same row.
  std::vector<uint32_t> lastReader(N, 0), slotOf(N, UINT32_MAX);
  for (uint32_t i = 0; i < N; ++i)
    for (uint32_t u : users[i]) lastReader[i] = std::max(lastReader[i], part[u]);
  std::vector<uint32_t> freeSlots;
  std::vector<std::vector<uint32_t>> releasedAfter(P);
  for (uint32_t p = 0; p < P; ++p) {
    Graph t;
    t.name = g.name;
    t.ftype = g.ftype;
    t.numFeatures = g.numFeatures;
    t.supportMarginal = g.supportMarginal;
    t.batchSize = g.batchSize;
    t.isTask = true;
    std::map<uint32_t, uint32_t> local;  // node of the whole graph -> node of the task
    auto external = [&](uint32_t c) {
      auto it = local.find(c);
      if (it != local.end()) return it->second;
      GraphNode e;
      e.kind = NodeKind::External;
      e.feature = slotOf[c];
      t.nodes.push_back(e);
      return local[c] = uint32_t(t.nodes.size() - 1);
    };
    std::vector<uint32_t> mine;
    for (uint32_t i = 0; i < N; ++i)
      if (part[i] == p) mine.push_back(i);
    if (mine.empty()) continue;
    for (uint32_t i : mine) {
      GraphNode n = nodes[i];
      n.uses = 0;
      for (uint32_t& c : n.children) c = part[c] == p ? local.at(c) : external(c);
      t.nodes.push_back(std::move(n));
      local[i] = uint32_t(t.nodes.size() - 1);
    }
    for (uint32_t i : mine) {
      if (i == root) continue;
      if (lastReader[i] > p) {
        if (freeSlots.empty()) freeSlots.push_back(plan.slots++);
        slotOf[i] = freeSlots.back();
        freeSlots.pop_back();
        releasedAfter[lastReader[i]].push_back(slotOf[i]);
        t.taskOutputs.push_back(local.at(i));
        t.taskOutputSlots.push_back(slotOf[i]);
      }
    }
    for (uint32_t s : releasedAfter[p]) freeSlots.push_back(s);
    if (part[root] == p) {
      t.taskFinal = true;
      if (local.at(root) != t.nodes.size() - 1) throw std::runtime_error("INTERNAL ERROR: the root is not the last node of its task");
    }
    for (auto& n : t.nodes)
      for (uint32_t c : n.children) t.nodes[c].uses++;
    for (uint32_t o : t.taskOutputs) t.nodes[o].uses++;
    if (t.taskFinal) t.nodes.back().uses++;
    basicStats(t);
    plan.tasks.push_back(std::move(t));
  }
  if (plan.tasks.empty() || !plan.tasks.back().taskFinal) throw std::runtime_error("INTERNAL ERROR: the last task does not hold the root");
  return plan;
}

}  // namespace spnc_hip
