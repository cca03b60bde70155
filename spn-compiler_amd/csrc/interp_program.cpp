#include "interp_program.h"

#include "math_tables.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <map>
#include <queue>
#include <set>
#include <sstream>
#include <stdexcept>

namespace spnc_hip {

namespace {

constexpr uint32_t NONE = UINT32_MAX;

struct Builder {
  const Graph& g;
  InterpProgram& p;
  double scale;
  std::ostringstream txt;

  Builder(const Graph& graph, InterpProgram& prog) : g(graph), p(prog) { scale = p.log2Domain ? 1.4426950408889634074 : 1.0; }

  void word(uint32_t w) { p.code.push_back(w); }
  // Every instruction is preceded by one word holding its length, so that the kernel knows where
  // the next instruction starts before it has decoded this one.
  size_t begin() {
    p.code.push_back(0);
    return p.code.size() - 1;
  }
  void end(size_t at) { p.code[at] = uint32_t(p.code.size() - at - 1); }
  void real(double v) {
    if (p.f64) {
      uint64_t b;
      std::memcpy(&b, &v, 8);
      word(uint32_t(b));
      word(uint32_t(b >> 32));
    } else {
      float f = float(v);
      uint32_t b;
      std::memcpy(&b, &f, 4);
      word(b);
    }
  }
  double logConst(double pr) const { return pr > 0 ? std::log(pr) * scale : -INFINITY; }
};

}  // namespace

namespace {
InterpProgram buildWithRange(const Graph& g, const CompileOptions& o, uint32_t longRange, bool stagedLong);

// Operand counts for which the kernel has a matrix-core outer sum (outerSumMatrixAny in interp_kernel.hip).
bool matrixFormShape(uint32_t na, uint32_t nb) {
  return (na == 8 && nb == 8) || (na == 4 && nb == 4) || (na == 4 && nb == 8) || (na == 8 && nb == 4) || (na == 2 && nb == 8) ||
         (na == 8 && nb == 2);
}
}

// Values that stay live for more than `longRange` instructions are numbered after all the others
// ("long pool"), so that the launcher can keep the busy, short-lived slots in LDS and the rarely
// touched long-lived ones in the spill tier; the staged feature values can be moved there too.
// Candidates are tried from "everything short" towards "as little as possible short" until the
// short pool fits the LDS share that lets four blocks reside on a CU, or failing that two.
InterpProgram buildInterpProgram(const Graph& g, const CompileOptions& o) {
  const bool f64 = o.computeType == ComputeType::F64;
  // Short-pool sizes (slots of 256 values) that let five or six, four, or two blocks share the 160 KiB of a CU.
  const uint32_t manyBlocks = o.interpShortSlots > 0 ? uint32_t(o.interpShortSlots) : (f64 ? 13 : 27), fourBlocks = f64 ? 20 : 40,
                 twoBlocks = f64 ? 36 : 72;
  // Candidates differ in which values count as long-lived (and so may leave LDS) and in the tier of
  // the staged features. Preferred: five or six blocks per CU (measured on a RAT-SPN: 8.8 ms with
  // pools of 24 to 27 slots, 9.4 ms with 36 or 40, 9.4 to 10.1 ms with 16 to 20 slots and eight
  // blocks); among equals the candidate that touches the spill tier least.
  InterpProgram best;
  bool have = false;
  auto rank = [&](const InterpProgram& p) { return p.shortSlots <= manyBlocks ? 0 : (p.shortSlots <= fourBlocks ? 1 : (p.shortSlots <= twoBlocks ? 2 : 3)); };
  auto better = [&](const InterpProgram& p) {
    if (!have) return true;
    const int rp = rank(p), rb = rank(best);
    if (rp != rb) return rp < rb;
    if (rp == 3) return p.shortSlots < best.shortSlots;
    return p.spillAccesses < best.spillAccesses;
  };
  for (bool stagedLong : {false, true}) {
    if (o.interpStagedLong >= 0 && stagedLong != (o.interpStagedLong == 1)) continue;
    for (uint32_t range : {0xffffffffu, 256u, 128u, 64u, 32u, 16u, 8u}) {
      if (o.interpLongRange >= 0) {
        if (range != 0xffffffffu) break;  // a fixed range: one candidate per tier choice
        range = uint32_t(o.interpLongRange);
      }
      InterpProgram p = buildWithRange(g, o, range, stagedLong);
      if (better(p)) {
        best = std::move(p);
        have = true;
      }
      if (best.spillAccesses == 0 && rank(best) == 0) break;
    }
    if (have && best.spillAccesses == 0 && rank(best) == 0) break;
  }
  if (best.f64 && best.log2Domain) {
    // The tables of the float64 exp2/log2 routines travel behind the leaf tables (16-byte aligned: the kernel copies
    // them into LDS when it starts).
    if (best.tables.size() % 2) best.tables.push_back(0.0);
    best.mathTables = uint32_t(best.tables.size());
    const std::vector<double> math = doubleMathTables();
    best.tables.insert(best.tables.end(), math.begin(), math.end());
  }
  return best;
}

// Walks a program as the kernel would and throws unless every access the kernel derives from it stays inside the
// slot file, the table pool, the input row and the instruction itself. A program built here passes by
// construction; one read back from a kernel file is only executed after it has passed.
void checkInterpProgram(const InterpProgram& p, uint32_t numFeatures) {
  auto bad = [](const std::string& what, size_t at) -> void {
    throw std::runtime_error("RUNTIME ERROR: malformed interpreter program (" + what + " at word " + std::to_string(at) + ")");
  };
  const std::vector<uint32_t>& c = p.code;
  const size_t RW = p.f64 ? 2 : 1;
  if (p.shortSlots > p.numSlots || p.numSlots > (1u << 20)) bad("slot counts", 0);
  if (p.featureMode != FEAT_STAGED && p.featureMode != FEAT_DIRECT && p.featureMode != FEAT_REGISTER) bad("feature mode", 0);
  const bool inRegisters = p.featureMode == FEAT_REGISTER;
  if (inRegisters && (p.f64 || p.staged.size() > 32)) bad("register features", 0);
  if ((p.f64 && p.log2Domain) != (p.mathTables != 0xFFFFFFFFu)) bad("math tables", 0);
  if (p.mathTables != 0xFFFFFFFFu && (p.mathTables % 2 != 0 || size_t(p.mathTables) + DOUBLE_MATH_TABLE_VALUES > p.tables.size())) bad("math tables", 0);
  std::map<uint32_t, uint32_t> indexBound;  // staged index slot -> largest index it can hold
  std::set<uint32_t> valueSlots;
  for (size_t k = 0; k < p.staged.size(); ++k) {
    const auto& sf = p.staged[k];
    if (sf.column >= numFeatures) bad("staged column", 0);
    if (inRegisters) {
      if (sf.valueSlot != k || sf.indexSlot != NONE) bad("feature register", 0);
      continue;
    }
    if (sf.valueSlot != NONE && sf.valueSlot >= p.numSlots) bad("staged value slot", 0);
    if (sf.indexSlot != NONE && sf.indexSlot >= p.numSlots) bad("staged index slot", 0);
    if (sf.tableLen > (1u << 24)) bad("staged table length", 0);
    if (sf.valueSlot != NONE) valueSlots.insert(sf.valueSlot);
    if (sf.indexSlot != NONE) indexBound[sf.indexSlot] = sf.tableLen + 1;
  }
  const bool staged = p.featureMode == FEAT_STAGED;
  if (!staged && !inRegisters && !p.staged.empty()) bad("staged features in a direct-feature program", 0);
  size_t pc = 0;
  for (;;) {
    if (pc + 1 >= c.size()) bad("stream ends inside an instruction", pc);
    const size_t len = c[pc], first = pc + 1, end = first + len;
    if (len < 2 || end > c.size()) bad("length word", pc);
    const uint32_t w0 = c[first], op = w0 & 0x7fu;
    const bool flagged = (w0 & 0x80u) != 0;
    auto need = [&](size_t words) {
      if (words != len) bad("instruction length", pc);
    };
    auto slot = [&](size_t at) {
      if (at >= end) bad("slot field outside its instruction", pc);
      const uint32_t sl = c[at];
      if (sl >= p.numSlots || (!flagged && sl >= p.shortSlots)) bad("slot number", at);
      return sl;
    };
    // A list of n slots at `at`; tier 0 / 1 promise the short / long pool, `run` that the kernel may take the first
    // number and count on from it.
    auto list = [&](size_t at, size_t n, uint32_t tier, bool run) {
      for (size_t j = 0; j < n; ++j) {
        const uint32_t sl = slot(at + j);
        if (run && sl != c[at] + j) bad("slot run", at + j);
        if ((tier == 0 && sl >= p.shortSlots) || (tier == 1 && sl < p.shortSlots) || tier > 2) bad("slot tier", at + j);
      }
    };
    auto feature = [&](size_t at, uint32_t tier) {
      if (at >= end) bad("feature field outside its instruction", pc);
      if (inRegisters) {
        if (c[at] >= p.staged.size()) bad("feature register", at);
        return;
      }
      if (!staged) {
        if (c[at] >= numFeatures) bad("feature column", at);
        return;
      }
      const uint32_t sl = slot(at);
      if (!valueSlots.count(sl)) bad("feature slot", at);
      if ((tier == 0 && sl >= p.shortSlots) || (tier == 1 && sl < p.shortSlots) || tier > 2) bad("feature tier", at);
    };
    if (op == OP_END) {
      need(2);
      slot(first + 1);
      if (end != c.size()) bad("words after the end instruction", end);
      return;
    }
    if (len < 3) bad("instruction length", pc);
    const uint32_t w1 = c[first + 1];
    switch (op) {
      case OP_PROD: {
        if (first + 5 > end) bad("instruction length", pc);
        const size_t ns = c[first + 2], ng = c[first + 3], nt = c[first + 4];
        if (ns > len || ng > len || nt > len) bad("operand counts", pc);
        need(5 + ns + ng * (1 + 3 * RW) + nt * 3);
        slot(first + 1);
        size_t q = first + 5;
        for (size_t j = 0; j < ns; ++j) slot(q++);
        for (size_t j = 0; j < ng; ++j, q += 1 + 3 * RW) feature(q, 2);
        for (size_t j = 0; j < nt; ++j, q += 3) {
          uint32_t bound;
          if (staged) {
            const auto it = indexBound.find(slot(q));
            if (it == indexBound.end()) bad("table index slot", q);
            bound = it->second;
          } else {
            if (inRegisters || c[q] >= numFeatures) bad("feature column", q);
            bound = c[q + 2] + 1;
          }
          if (size_t(c[q + 1]) + bound >= p.tables.size()) bad("table offset", q + 1);
        }
        break;
      }
      case OP_PRODBATCH: {
        const size_t n = w0 >> 8, G = w1 & 0xffu;
        const uint32_t featTier = (w1 >> 8) & 3u, dstTier = (w1 >> 10) & 3u;
        if (n < 2 || G < 1 || G > 4) bad("product batch shape", pc);
        const size_t rec = 1 + G * (1 + 3 * RW);
        need(2 + n * rec);
        for (size_t i = 0; i < n; ++i) {
          list(first + 2 + i * rec, 1, dstTier, false);
          for (size_t j = 0; j < G; ++j) {
            const size_t at = first + 2 + i * rec + 1 + j * (1 + 3 * RW);
            feature(at, staged ? featTier : 2);
            if (((w1 >> 12) & 1u) && i / 4 * 4 + 4 <= n && c[at] != c[first + 2 + (i / 4 * 4) * rec + 1 + j * (1 + 3 * RW)]) bad("grouped product batch", at);
          }
        }
        break;
      }
      case OP_SUM: {
        const size_t k = w0 >> 8;
        if (k < 1) bad("sum without terms", pc);
        need(2 + k * (1 + RW));
        slot(first + 1);
        for (size_t j = 0; j < k; ++j) slot(first + 2 + j * (1 + RW));
        break;
      }
      case OP_SUMLAYER: {
        const size_t k = w0 >> 8, m = w1;
        if (k < 1 || !(m == 2 || m == 4 || m == 8)) bad("sum layer shape", pc);
        need(2 + m + k + k * m * RW);
        for (size_t j = 0; j < m + k; ++j) slot(first + 2 + j);
        break;
      }
      case OP_OUTERSUM: {
        const size_t na = (w0 >> 8) & 0xffu, nb = (w0 >> 16) & 0xffu, m = w1;
        if (na < 1 || !(nb == 2 || nb == 4 || nb == 8 || nb == 16) || !(m == 2 || m == 4 || m == 8) || (w0 >> 24)) bad("outer sum shape", pc);
        need(2 + m + na + nb + na * nb * m * RW);
        for (size_t j = 0; j < m + na + nb; ++j) slot(first + 2 + j);
        break;
      }
      case OP_OUTERMM: {
        const uint32_t na = (w0 >> 8) & 0xffu, nb = (w0 >> 16) & 0xffu;
        if (p.f64 || !matrixFormShape(na, nb) || (w1 & 0xffu) != 8 || (w1 >> 12)) bad("matrix-form outer sum shape", pc);
        need(2 + 8 + na + nb + 3 + size_t(na) * nb * 8);
        const size_t dst = first + 2, as = dst + 8, bs = as + na, scales = bs + nb;
        list(dst, 8, (w0 >> 28) & 3u, (w1 >> 11) & 1u);
        list(as, na, (w0 >> 24) & 3u, (w1 >> 9) & 1u);
        list(bs, nb, (w0 >> 26) & 3u, (w1 >> 10) & 1u);
        if ((w1 >> 8) & 1u) slot(scales);
        if ((w0 >> 30) & 1u) slot(scales + 1);
        if ((w0 >> 31) & 1u) slot(scales + 2);
        break;
      }
      case OP_LEAFMM:
      case OP_LEAFPAIRMM:
      case OP_LEAFQUADMM: {
        const uint32_t na = (w0 >> 8) & 0xffu, nb = (w0 >> 16) & 0xffu, G = (w1 >> 12) & 0xfu, featTier = (w1 >> 16) & 3u;
        if (p.linear || (w1 & 0xffu) != 8) bad("leaf region shape", pc);
        const size_t rw = p.f64 ? 2 : 1;  // words per constant and per weight
        if (p.f64 && ((w1 >> 8) & 1u)) bad("scaled result in a double program", pc);
        size_t regions, products, weights;
        if (op == OP_LEAFMM) {
          if (!((na == 4 && nb == 4) || (na == 8 && nb == 8)) || !(G == 1 || G == 2 || G == 4)) bad("leaf region shape", pc);
          regions = 1, products = na + nb, weights = size_t(na) * nb * 8;
        } else if (op == OP_LEAFPAIRMM) {
          if (na != 4 || nb != 0 || !(G == 1 || G == 2 || G == 4)) bad("leaf region pair shape", pc);
          regions = 2, products = 16, weights = 2 * 128 + 512;
        } else {
          if (na != 4 || nb != 0 || !(G == 1 || G == 2)) bad("leaf region quad shape", pc);
          regions = 4, products = 32, weights = 2 * (2 * 128 + 512) + 512;
        }
        need(2 + 8 + 1 + 2 * regions * G + (products * G * 3 + weights) * rw);
        list(first + 2, 8, (w0 >> 28) & 3u, (w1 >> 11) & 1u);
        if ((w1 >> 8) & 1u) slot(first + 10);
        for (size_t j = 0; j < 2 * regions * G; ++j) feature(first + 11 + j, staged ? featTier : 2);
        break;
      }
      default:
        bad("opcode", first);
    }
    pc = end;
  }
}

namespace {
InterpProgram buildWithRange(const Graph& g, const CompileOptions& o, uint32_t longRange, bool stagedLong) {
  InterpProgram p;
  // Linear space: probabilities in double, as the reference computes them (computeInLogSpace=False); the same
  // instructions with other constants (linear weights everywhere, linear table values, Gaussian leaves as coefficient
  // and natural-log exponent factor) and no matrix or scaled-vector forms.
  p.linear = !o.useLogSpace;
  p.f64 = p.linear || o.computeType == ComputeType::F64;
  p.log2Domain = !p.linear && o.log2Domain;
  Builder b(g, p);
  const size_t N = g.nodes.size();
  auto isLeaf = [&](uint32_t i) { return g.nodes[i].kind != NodeKind::Product && g.nodes[i].kind != NodeKind::Sum; };
  auto isTable = [&](uint32_t i) { return g.nodes[i].kind == NodeKind::Categorical || g.nodes[i].kind == NodeKind::Histogram; };

  // ---- features: which columns feed Gaussian leaves / table leaves, and the table pool ----
  std::vector<uint32_t> featTableLen(g.numFeatures, 0);
  std::vector<bool> featGauss(g.numFeatures, false);
  for (uint32_t i = 0; i < N; ++i) {
    const auto& n = g.nodes[i];
    if (n.kind == NodeKind::Gaussian) featGauss[n.feature] = true;
    else if (isTable(i)) featTableLen[n.feature] = std::max<uint32_t>(featTableLen[n.feature], uint32_t(n.table.size()));
  }
  // Same pool layout as the straight-line kernel: L_f + 2 entries per table leaf (values,
  // "impossible" up to index L_f, marginal value at L_f + 1).
  std::vector<uint32_t> tableOffset(N, 0);
  for (uint32_t i = 0; i < N; ++i) {
    if (!isTable(i)) continue;
    const auto& n = g.nodes[i];
    uint32_t L = featTableLen[n.feature];
    tableOffset[i] = uint32_t(p.tables.size());
    for (uint32_t j = 0; j <= L; ++j) {
      const double pr = j < n.table.size() ? n.table[j] : 0.0;  // entry L: impossible
      p.tables.push_back(p.linear ? pr : b.logConst(pr));
    }
    p.tables.push_back(p.linear ? 1.0 : 0.0);  // entry L + 1: the marginal value
  }
  uint32_t stagedSlots = 0;
  for (uint32_t f = 0; f < g.numFeatures; ++f) {
    stagedSlots += (featGauss[f] ? 1 : 0) + (featTableLen[f] ? 1 : 0);
  }
  p.featureMode = stagedSlots <= 48 ? FEAT_STAGED : FEAT_DIRECT;
  {
    // Float programs whose features (at most 32) all feed Gaussian leaves keep them in registers for the whole tile:
    // no slot, no memory access per use. (Measured on the RAT-SPN configuration: the staged features, kept in the
    // spill tier, were re-read 320 times per sample, 4 GiB per launch.)
    bool tablesUsed = false;
    uint32_t gaussFeatures = 0;
    for (uint32_t f = 0; f < g.numFeatures; ++f) {
      tablesUsed = tablesUsed || featTableLen[f] != 0;
      gaussFeatures += featGauss[f] ? 1 : 0;
    }
    if (o.interpFeatureRegisters && !p.f64 && !tablesUsed && gaussFeatures > 0 && gaussFeatures <= 32) p.featureMode = FEAT_REGISTER;
  }
  std::vector<uint32_t> valueSlotOf(g.numFeatures, NONE), indexSlotOf(g.numFeatures, NONE);
  constexpr uint32_t LONG_BIT = 0x80000000u;  // marks long-pool slot numbers until they are renumbered
  uint32_t nextSlot = 0, longCount = 0;
  auto stagedSlot = [&]() { return stagedLong ? (LONG_BIT | longCount++) : nextSlot++; };
  if (p.featureMode == FEAT_REGISTER) {
    for (uint32_t f = 0; f < g.numFeatures; ++f) {
      if (!featGauss[f]) continue;
      valueSlotOf[f] = uint32_t(p.staged.size());  // the register number
      p.staged.push_back(StagedFeature{f, valueSlotOf[f], NONE, 0});
    }
  } else if (p.featureMode == FEAT_STAGED) {
    for (uint32_t f = 0; f < g.numFeatures; ++f) {
      if (!featGauss[f] && !featTableLen[f]) continue;
      StagedFeature sf{f, NONE, NONE, featTableLen[f]};
      if (featGauss[f]) sf.valueSlot = valueSlotOf[f] = stagedSlot();
      if (featTableLen[f]) sf.indexSlot = indexSlotOf[f] = stagedSlot();
      p.staged.push_back(sf);
    }
  } else {
    p.directTableLen = featTableLen;
  }
  p.reservedSlots = nextSlot + longCount;

  // ---- instruction selection ----
  // A leaf whose only consumer is a product is evaluated inside that product. Every other leaf
  // becomes a one-term product. Sums with identical ordered child lists form a layer.
  std::vector<uint32_t> soleParent(N, NONE);
  for (uint32_t i = 0; i < N; ++i)
    for (uint32_t c : g.nodes[i].children) soleParent[c] = i;
  std::vector<bool> inlined(N, false);
  for (uint32_t i = 0; i < N; ++i)
    if (isLeaf(i) && g.nodes[i].uses == 1 && soleParent[i] != NONE && g.nodes[soleParent[i]].kind == NodeKind::Product)
      inlined[i] = true;

  // Sums over a complete outer product: the sums of a group share the child list
  // [prod(a_0,b_0), prod(a_0,b_1), ..., prod(a_NA-1,b_NB-1)] and nobody else reads those products.
  // Then exp(a_r + b_c - m) = exp(a_r - ma) * exp(b_c - mb) and the products need not exist.
  struct Outer {
    std::vector<uint32_t> a, b;
  };
  std::map<std::vector<uint32_t>, Outer> outerOf;
  std::vector<bool> absorbed(N, false);
  {
    std::map<std::vector<uint32_t>, uint32_t> groupSize;
    for (uint32_t i = 0; i < N; ++i)
      if (g.nodes[i].kind == NodeKind::Sum && g.nodes[i].children.size() >= 4) groupSize[g.nodes[i].children]++;
    for (const auto& entry : groupSize) {
      const std::vector<uint32_t>& kids = entry.first;
      const uint32_t members = entry.second;
      bool ok = true;
      for (uint32_t c : kids) {
        const auto& pn = g.nodes[c];
        if (pn.kind != NodeKind::Product || pn.children.size() != 2 || pn.uses != members || inlined[pn.children[0]] ||
            inlined[pn.children[1]]) {
          ok = false;
          break;
        }
      }
      if (!ok) continue;
      size_t nb = 1;
      while (nb < kids.size() && g.nodes[kids[nb]].children[0] == g.nodes[kids[0]].children[0]) ++nb;
      if (kids.size() % nb != 0) continue;
      const size_t na = kids.size() / nb;
      if ((nb != 2 && nb != 4 && nb != 8 && nb != 16) || na < 2 || na > 64) continue;
      Outer o;
      for (size_t r = 0; r < na; ++r) o.a.push_back(g.nodes[kids[r * nb]].children[0]);
      for (size_t c = 0; c < nb; ++c) o.b.push_back(g.nodes[kids[c]].children[1]);
      for (size_t r = 0; r < na && ok; ++r)
        for (size_t c = 0; c < nb; ++c) {
          const auto& pn = g.nodes[kids[r * nb + c]];
          if (pn.children[0] != o.a[r] || pn.children[1] != o.b[c]) {
            ok = false;
            break;
          }
        }
      // A child list naming one product twice would make the use counts above meaningless.
      std::vector<uint32_t> sorted = kids;
      std::sort(sorted.begin(), sorted.end());
      if (std::adjacent_find(sorted.begin(), sorted.end()) != sorted.end()) ok = false;
      if (!ok) continue;
      for (uint32_t c : kids) absorbed[c] = true;
      outerOf[kids] = std::move(o);
    }
  }

  struct Instr {
    InterpOp op;
    std::vector<uint32_t> defs;  // graph nodes whose values this instruction writes
    std::vector<uint32_t> srcs;  // graph nodes read from slots
    uint32_t node;               // representative node (PROD / SUM) or first sum of a layer
  };
  std::vector<Instr> instrs;
  std::map<std::vector<uint32_t>, std::vector<uint32_t>> layerOf;  // child list -> sums over it
  for (uint32_t i = 0; i < N; ++i)
    if (g.nodes[i].kind == NodeKind::Sum && g.nodes[i].children.size() >= 2) layerOf[g.nodes[i].children].push_back(i);
  std::vector<bool> emitted(N, false);
  for (uint32_t i = 0; i < N; ++i) {
    if (emitted[i] || inlined[i] || absorbed[i]) continue;
    const auto& n = g.nodes[i];
    if (n.kind == NodeKind::Sum && n.children.size() >= 2) {
      const std::vector<uint32_t>& group = layerOf[n.children];
      auto outer = outerOf.find(n.children);
      if (outer != outerOf.end()) {
        std::vector<uint32_t> srcs = outer->second.a;
        srcs.insert(srcs.end(), outer->second.b.begin(), outer->second.b.end());
        size_t pos = 0;
        while (pos < group.size()) {
          size_t left = group.size() - pos;
          size_t m = left >= 8 ? 8 : (left >= 4 ? 4 : (left >= 2 ? 2 : 1));
          Instr in{OP_OUTERSUM, {}, srcs, group[pos]};
          for (size_t j = 0; j < m; ++j) {
            in.defs.push_back(group[pos + j]);
            emitted[group[pos + j]] = true;
          }
          instrs.push_back(std::move(in));
          pos += m;
        }
        continue;
      }
      // Split the group into layers of 8, 4, 2 sums and single sums.
      size_t pos = 0;
      while (pos < group.size()) {
        size_t left = group.size() - pos;
        size_t m = left >= 8 ? 8 : (left >= 4 ? 4 : (left >= 2 ? 2 : 1));
        Instr in{m == 1 ? OP_SUM : OP_SUMLAYER, {}, n.children, group[pos]};
        for (size_t j = 0; j < m; ++j) {
          in.defs.push_back(group[pos + j]);
          emitted[group[pos + j]] = true;
        }
        instrs.push_back(std::move(in));
        pos += m;
      }
      continue;
    }
    Instr in{n.kind == NodeKind::Sum ? OP_SUM : OP_PROD, {i}, {}, i};
    if (n.kind == NodeKind::Sum) {
      in.srcs = n.children;
    } else if (n.kind == NodeKind::Product) {
      for (uint32_t c : n.children)
        if (!inlined[c]) in.srcs.push_back(c);
    }
    emitted[i] = true;
    instrs.push_back(std::move(in));
  }

  // ---- matrix-form outer sums and the format of the vectors between them ----
  // An outer sum in matrix form whose eight results are read by exactly one other such instruction, as its
  // complete a or b list, hands them over as a scaled linear vector: acc_t / max(acc) in the eight slots and
  // one more slot holding the common log2 scale. The consumer then needs no maximum, subtraction or
  // exponential for that list and the producer one logarithm instead of eight.
  std::vector<bool> matrixInstr(instrs.size(), false);
  std::vector<int> linearConsumer(instrs.size(), -1);  // producer -> consuming instruction
  std::vector<bool> leafRegion(instrs.size(), false), fusedProduct(instrs.size(), false);
  std::vector<std::pair<uint32_t, uint32_t>> leafPair(instrs.size(), {NONE, NONE});  // 8x8 sum -> the two leaf regions it takes in
  std::vector<std::pair<uint32_t, uint32_t>> leafQuad(instrs.size(), {NONE, NONE});  // 8x8 sum -> the two leaf-region pairs it takes in
  {
    for (uint32_t k = 0; k < instrs.size(); ++k) {
      const Instr& in = instrs[k];
      if (in.op != OP_OUTERSUM) continue;
      const Outer& outer = outerOf.at(g.nodes[in.node].children);
      // (double programs: the same instructions qualify, as candidates for the fused leaf forms, whose weights go
      // through lanes; on their own they stay ordinary outer sums and no vector between them is scaled)
      matrixInstr[k] = !p.linear && in.defs.size() == 8 && o.interpMatrixCore &&
                       matrixFormShape(uint32_t(outer.a.size()), uint32_t(outer.b.size()));
    }
    std::vector<std::vector<uint32_t>> readers(N);
    for (uint32_t k = 0; k < instrs.size(); ++k)
      for (uint32_t sidx : instrs[k].srcs)
        if (readers[sidx].empty() || readers[sidx].back() != k) readers[sidx].push_back(k);
    for (uint32_t k = 0; k < instrs.size() && o.interpScaledVectors; ++k) {
      if (!matrixInstr[k]) continue;
      const Instr& in = instrs[k];
      int consumer = -1;
      bool ok = true;
      for (uint32_t d : in.defs) {
        if (d == g.root() || readers[d].size() != 1) ok = false;
        else if (consumer < 0) consumer = int(readers[d][0]);
        else if (consumer != int(readers[d][0])) ok = false;
      }
      if (!ok || consumer < 0 || !matrixInstr[consumer]) continue;
      const Outer& co = outerOf.at(g.nodes[instrs[consumer].node].children);
      if (co.a == in.defs || co.b == in.defs) linearConsumer[k] = consumer;
    }
    // Leaf regions: a matrix-form outer sum over two lists of products of Gaussian leaves only, each product
    // read by nothing else and all products of a list over the same features, computes them itself. The
    // product instructions disappear and with them their slots.
    std::vector<uint32_t> instrOfNode(N, NONE);
    for (uint32_t k = 0; k < instrs.size(); ++k)
      for (uint32_t d : instrs[k].defs) instrOfNode[d] = k;
    auto leafFeatures = [&](uint32_t node, std::vector<uint32_t>& out) {
      const auto& pn = g.nodes[node];
      if (pn.kind != NodeKind::Product || node == g.root() || readers[node].size() != 1) return false;
      for (uint32_t c : pn.children) {
        if (!inlined[c] || g.nodes[c].kind != NodeKind::Gaussian) return false;
        out.push_back(g.nodes[c].feature);
      }
      return true;
    };
    for (uint32_t k = 0; k < instrs.size() && o.interpLeafRegions; ++k) {
      if (!matrixInstr[k]) continue;
      const Outer& outer = outerOf.at(g.nodes[instrs[k].node].children);
      if (!((outer.a.size() == 4 && outer.b.size() == 4) || (outer.a.size() == 8 && outer.b.size() == 8))) continue;
      bool ok = true;
      std::vector<uint32_t> fa, fb;
      for (const std::vector<uint32_t>* list : {&outer.a, &outer.b}) {
        std::vector<uint32_t>& want = list == &outer.a ? fa : fb;
        for (size_t r = 0; r < list->size() && ok; ++r) {
          std::vector<uint32_t> f;
          ok = leafFeatures((*list)[r], f) && (r == 0 || f == want);
          if (r == 0) want = f;
        }
      }
      if (!ok || fa.size() != fb.size() || !(fa.size() == 1 || fa.size() == 2 || fa.size() == 4)) continue;
      leafRegion[k] = true;
      for (uint32_t s : instrs[k].srcs) fusedProduct[instrOfNode[s]] = true;
      instrs[k].srcs.clear();
    }
    // Inside a pair or a quad the result vectors of the inner sums stay in registers as they come out of the matrix
    // chain, linear and not rescaled (a rescaling costs a maximum over eight values, a reciprocal, eight multiplies
    // and a logarithm). That is safe while the vector's largest entry cannot underflow: the operand vectors' largest
    // products are 1 (leaf regions: exp2(value - max)) or at least the product of the operands' floors, and the sum
    // t that weighs this product most gets at least that weight of it. floorLog2 is log2 of this lower bound on
    // max_t(result_t), from the weights alone; a fusion whose bound falls under 2^-90 is not made.
    std::vector<double> floorLog2(instrs.size(), 0.0);
    auto weightFloor = [&](uint32_t k) {
      const std::vector<uint32_t>& sums = instrs[k].defs;
      double low = INFINITY;
      for (size_t q = 0; q < g.nodes[sums[0]].weights.size(); ++q) {
        double best = 0.0;
        for (uint32_t sNode : sums) best = std::max(best, g.nodes[sNode].weights[q]);
        low = std::min(low, best);
      }
      return low > 0.0 ? std::log2(low) : -INFINITY;
    };
    for (uint32_t k = 0; k < instrs.size(); ++k)
      if (leafRegion[k]) floorLog2[k] = weightFloor(k);
    const double lowestFloor = -90.0;
    // Pairs of leaf regions: an 8x8 outer sum whose operand lists are the result vectors of two leaf
    // regions of 4x4 products each, read by nothing else, takes them in: one instruction, the vectors stay in registers.
    for (uint32_t k = 0; k < instrs.size() && o.interpLeafRegions; ++k) {
      if (!matrixInstr[k] || leafRegion[k]) continue;
      const Outer& outer = outerOf.at(g.nodes[instrs[k].node].children);
      if (outer.a.size() != 8 || outer.b.size() != 8) continue;
      const uint32_t i = instrOfNode[outer.a[0]], j = instrOfNode[outer.b[0]];
      if (i == NONE || j == NONE || i == j || !leafRegion[i] || !leafRegion[j] || linearConsumer[i] != int(k) || linearConsumer[j] != int(k) ||
          instrs[i].defs != outer.a || instrs[j].defs != outer.b)
        continue;
      const Outer& oi = outerOf.at(g.nodes[instrs[i].node].children);
      const Outer& oj = outerOf.at(g.nodes[instrs[j].node].children);
      if (oi.a.size() != 4 || oj.a.size() != 4 || g.nodes[oi.a[0]].children.size() != g.nodes[oj.a[0]].children.size()) continue;
      floorLog2[k] = weightFloor(k) + floorLog2[i] + floorLog2[j];
      if (!(floorLog2[k] >= lowestFloor)) continue;
      leafPair[k] = {i, j};
      fusedProduct[i] = fusedProduct[j] = true;
      instrs[k].srcs.clear();
    }
    // And once more: an 8x8 outer sum over the result vectors of two such pairs (one or two leaves per product)
    // takes both pairs in, seven sums over four leaf regions in one instruction.
    for (uint32_t k = 0; k < instrs.size() && o.interpLeafRegions; ++k) {
      if (!matrixInstr[k] || leafRegion[k] || leafPair[k].first != NONE) continue;
      const Outer& outer = outerOf.at(g.nodes[instrs[k].node].children);
      if (outer.a.size() != 8 || outer.b.size() != 8) continue;
      const uint32_t i = instrOfNode[outer.a[0]], j = instrOfNode[outer.b[0]];
      if (i == NONE || j == NONE || i == j || leafPair[i].first == NONE || leafPair[j].first == NONE || linearConsumer[i] != int(k) ||
          linearConsumer[j] != int(k) || instrs[i].defs != outer.a || instrs[j].defs != outer.b)
        continue;
      auto leavesOf = [&](uint32_t pairInstr) {
        const Outer& region = outerOf.at(g.nodes[instrs[leafPair[pairInstr].first].node].children);
        return g.nodes[region.a[0]].children.size();
      };
      if (leavesOf(i) != leavesOf(j) || leavesOf(i) > 2) continue;
      floorLog2[k] = weightFloor(k) + floorLog2[i] + floorLog2[j];
      if (!(floorLog2[k] >= lowestFloor)) continue;
      leafQuad[k] = {i, j};
      fusedProduct[i] = fusedProduct[j] = true;
      instrs[k].srcs.clear();
    }
  }
  std::vector<uint32_t> scaleSlotOfNode(N, NONE);  // first result of a scaled linear vector -> slot of its scale

  // ---- slot allocation by liveness on the instruction order ----
  std::vector<uint32_t> lastUse(N, 0);
  for (uint32_t k = 0; k < instrs.size(); ++k)
    for (uint32_t s : instrs[k].srcs) lastUse[s] = k;
  lastUse[g.root()] = uint32_t(instrs.size());  // read by OP_END
  std::vector<uint32_t> firstDef(N, 0);
  for (uint32_t k = 0; k < instrs.size(); ++k)
    for (uint32_t d : instrs[k].defs) firstDef[d] = k;
  std::vector<uint32_t> slotOf(N, NONE);
  // Each pool (short-lived slots, long-lived slots) hands out single slots and, with vector blocks switched on,
  // blocks of nine consecutive slots: the eight results of a matrix-form outer sum and the scale of a scaled
  // vector, which the kernel then addresses by the first slot alone. Singles are carved out of blocks; a block
  // whose nine slots are free again is whole again, so the slots of a batch of products that has died serve
  // the vector computed from it.
  constexpr uint32_t VECTOR_BLOCK = 9;
  const bool useBlocks = o.interpVectorBlocks;
  struct Pool {
    uint32_t origin = 0;  // number of the pool's first slot (blocks are aligned to it)
    std::set<uint32_t> singles, wholeBlocks;
  };
  Pool shortPool, longPool;
  shortPool.origin = nextSlot;
  longPool.origin = LONG_BIT | longCount;
  uint32_t highWater = nextSlot;
  auto grow = [&](bool isLong, uint32_t count) {
    uint32_t first;
    if (isLong) {
      first = LONG_BIT | longCount;
      longCount += count;
    } else {
      first = highWater;
      highWater += count;
    }
    return first;
  };
  auto takeBlock = [&](bool isLong) {
    Pool& pool = isLong ? longPool : shortPool;
    if (!pool.wholeBlocks.empty()) {
      const uint32_t base = *pool.wholeBlocks.begin();
      pool.wholeBlocks.erase(pool.wholeBlocks.begin());
      return base;
    }
    return grow(isLong, VECTOR_BLOCK);
  };
  auto allocSlot = [&](uint32_t node) {
    const bool isLong = lastUse[node] - firstDef[node] > longRange;
    Pool& pool = isLong ? longPool : shortPool;
    if (pool.singles.empty()) {
      if (!useBlocks) return grow(isLong, 1);
      const uint32_t base = takeBlock(isLong);
      for (uint32_t j = 0; j < VECTOR_BLOCK; ++j) pool.singles.insert(base + j);
    }
    const uint32_t s = *pool.singles.begin();
    pool.singles.erase(pool.singles.begin());
    return s;
  };
  auto releaseSlot = [&](uint32_t s) {
    Pool& pool = (s & LONG_BIT) ? longPool : shortPool;
    pool.singles.insert(s);
    if (!useBlocks) return;
    const uint32_t base = pool.origin + (s - pool.origin) / VECTOR_BLOCK * VECTOR_BLOCK;
    for (uint32_t j = 0; j < VECTOR_BLOCK; ++j)
      if (!pool.singles.count(base + j)) return;
    for (uint32_t j = 0; j < VECTOR_BLOCK; ++j) pool.singles.erase(base + j);
    pool.wholeBlocks.insert(base);
  };
  struct Block {
    uint32_t base, live;
  };
  std::vector<Block> blocks;
  std::vector<int> blockOfNode(N, -1);
  auto allocBlock = [&](uint32_t node) { return takeBlock(lastUse[node] - firstDef[node] > longRange); };
  auto releaseNode = [&](uint32_t node) {
    if (blockOfNode[node] < 0) {
      releaseSlot(slotOf[node]);
      return;
    }
    Block& blk = blocks[size_t(blockOfNode[node])];
    if (--blk.live == 0) ((blk.base & LONG_BIT) ? longPool : shortPool).wholeBlocks.insert(blk.base);
  };
  std::vector<size_t> longWords;  // positions in p.code holding long-pool slot numbers
  auto slotWord = [&](uint32_t s) {
    if (s & LONG_BIT) longWords.push_back(p.code.size());
    b.word(s);
  };
  auto slotName = [&](uint32_t s) { return (s & LONG_BIT) ? "L" + std::to_string(s & ~LONG_BIT) : "s" + std::to_string(s); };

  auto emitInlineLeaf = [&](uint32_t c) {
    const auto& leaf = g.nodes[c];
    if (leaf.kind == NodeKind::Gaussian) {
      double coef = -std::log(leaf.stddev) + -0.5 * std::log(2 * M_PI);
      double den = -(1.0 / (2.0 * leaf.stddev * leaf.stddev));
      if (p.featureMode == FEAT_STAGED) slotWord(valueSlotOf[leaf.feature]);
      else if (p.featureMode == FEAT_REGISTER) b.word(valueSlotOf[leaf.feature]);
      else b.word(leaf.feature);
      b.real(leaf.mean);
      if (p.linear) {
        b.real(std::exp(coef));  // value = coef * exp(d * d * den)
        b.real(den);
      } else {
        b.real(coef / den);  // value = den * (d * d + coef / den): one multiply-add and one multiply, each with one constant
        b.real(den * b.scale);
      }
    } else {
      if (p.featureMode == FEAT_STAGED) slotWord(indexSlotOf[leaf.feature]);
      else b.word(leaf.feature);
      b.word(tableOffset[c]);
      b.word(featTableLen[leaf.feature]);
    }
  };

  auto emitProd = [&](uint32_t node, uint32_t dst, const std::vector<uint32_t>& srcs, const std::vector<uint32_t>& gs,
                      const std::vector<uint32_t>& ts, uint32_t longFlag) {
    const size_t at = b.begin();
    b.word(OP_PROD | longFlag);
    slotWord(dst);
    b.word(uint32_t(srcs.size()));
    b.word(uint32_t(gs.size()));
    b.word(uint32_t(ts.size()));
    for (uint32_t s : srcs) slotWord(slotOf[s]);
    for (uint32_t c : gs) emitInlineLeaf(c);
    for (uint32_t c : ts) emitInlineLeaf(c);
    b.end(at);
    b.txt << "  " << slotName(dst) << " = prod(" << srcs.size() << " slots, " << gs.size() << " gaussians, " << ts.size() << " tables)   ; node "
          << node << "\n";
  };
  struct BatchEntry {
    uint32_t node, dst;
    std::vector<uint32_t> leaves;
  };
  std::vector<BatchEntry> batch;
  uint32_t batchFlag = 0;
  auto flushBatch = [&]() {
    if (batch.empty()) return;
    if (batch.size() == 1) {
      emitProd(batch[0].node, batch[0].dst, {}, batch[0].leaves, {}, batchFlag);
    } else {
      const size_t at = b.begin();
      b.word(OP_PRODBATCH | batchFlag | (uint32_t(batch.size()) << 8));
      // Second word: leaves per product; bits 8-9 / 10-11 the tier of the staged feature slots / of the
      // destinations (0 all in the short pool, 1 all in the long pool, 2 mixed); bit 12: within every full
      // group of four records the j-th leaves all read the same feature (the leaf regions of a region graph
      // are like that), so the kernel reads each feature of a group once.
      // The records do not depend on each other: those that read the same features are put next to each other.
      auto features = [&](const BatchEntry& e) {
        std::vector<uint32_t> f;
        for (uint32_t c : e.leaves) f.push_back(g.nodes[c].feature);
        return f;
      };
      std::stable_sort(batch.begin(), batch.end(), [&](const BatchEntry& x, const BatchEntry& y) { return features(x) < features(y); });
      uint32_t longDsts = 0;
      for (const auto& e : batch) longDsts += (e.dst & LONG_BIT) ? 1 : 0;
      const uint32_t dstTier = longDsts == 0 ? 0u : (longDsts == batch.size() ? 1u : 2u);
      const uint32_t featTier = p.featureMode == FEAT_STAGED && stagedLong ? 1u : 0u;
      bool grouped = batch.size() >= 4;
      for (size_t q = 0; q + 4 <= batch.size() && grouped; q += 4)
        for (size_t r = 1; r < 4; ++r)
          for (size_t j = 0; j < batch[q].leaves.size(); ++j)
            if (g.nodes[batch[q + r].leaves[j]].feature != g.nodes[batch[q].leaves[j]].feature) grouped = false;
      b.word(uint32_t(batch[0].leaves.size()) | (featTier << 8) | (dstTier << 10) | (grouped ? 0x1000u : 0u));
      for (const auto& e : batch) {
        slotWord(e.dst);
        for (uint32_t c : e.leaves) emitInlineLeaf(c);
      }
      b.end(at);
      b.txt << "  " << slotName(batch[0].dst) << ".. = prodbatch(" << batch.size() << " products x " << batch[0].leaves.size()
            << " gaussians)" << (grouped ? " grouped" : "") << "   ; nodes " << batch[0].node << "..\n";
    }
    batch.clear();
  };

  for (uint32_t k = 0; k < instrs.size(); ++k) {
    const Instr& in = instrs[k];
    if (fusedProduct[k]) continue;  // computed inside the outer sum that reads it
    // Sources dying here release their slots before the destinations are chosen: every
    // opcode reads all of its operands before it writes.
    {
      std::vector<uint32_t> uniq = in.srcs;
      std::sort(uniq.begin(), uniq.end());
      uniq.erase(std::unique(uniq.begin(), uniq.end()), uniq.end());
      for (uint32_t s : uniq)
        if (lastUse[s] == k) {
          releaseNode(s);
          if (scaleSlotOfNode[s] != NONE && blockOfNode[s] < 0) releaseSlot(scaleSlotOfNode[s]);  // else part of the block
        }
    }
    if (in.op == OP_OUTERSUM && matrixInstr[k] && !p.f64 && o.interpVectorBlocks) {
      const uint32_t base = allocBlock(in.defs[0]);
      for (uint32_t t = 0; t < in.defs.size(); ++t) {
        slotOf[in.defs[t]] = base + t;
        blockOfNode[in.defs[t]] = int(blocks.size());
      }
      blocks.push_back(Block{base, uint32_t(in.defs.size())});
    } else {
      for (uint32_t d : in.defs) slotOf[d] = allocSlot(d);
    }
    // Bit 7 of the opcode tells the kernel that this instruction touches the long pool.
    uint32_t longFlag = 0;
    for (uint32_t d : in.defs) longFlag |= (slotOf[d] & LONG_BIT) ? 0x80u : 0u;
    for (uint32_t sidx : in.srcs) longFlag |= (slotOf[sidx] & LONG_BIT) ? 0x80u : 0u;
    const auto& n = g.nodes[in.node];
    if (in.op != OP_PROD) flushBatch();
    switch (in.op) {
      case OP_PROD: {
        std::vector<uint32_t> gs, ts;
        if (isLeaf(in.node)) {
          (isTable(in.node) ? ts : gs).push_back(in.node);
        } else {
          for (uint32_t c : n.children)
            if (inlined[c]) (isTable(c) ? ts : gs).push_back(c);
        }
        if (stagedLong && p.featureMode == FEAT_STAGED && !(gs.empty() && ts.empty())) longFlag |= 0x80u;
        // Products of Gaussian leaves only, all of one size, that follow each other become one
        // batch instruction: their records do not depend on each other, so the kernel works on
        // several at a time.
        if (in.srcs.empty() && ts.empty() && !gs.empty() && gs.size() <= 4) {
          if (!batch.empty() && (batch.front().leaves.size() != gs.size() || batchFlag != longFlag)) flushBatch();
          batchFlag = longFlag;
          batch.push_back(BatchEntry{in.node, slotOf[in.node], gs});
          break;
        }
        flushBatch();
        emitProd(in.node, slotOf[in.node], in.srcs, gs, ts, longFlag);
        break;
      }
      case OP_SUM: {
        uint32_t cnt = uint32_t(n.children.size());
        const size_t at = b.begin();
        b.word(OP_SUM | longFlag | (cnt << 8));
        slotWord(slotOf[in.node]);
        for (uint32_t j = 0; j < cnt; ++j) {
          slotWord(slotOf[n.children[j]]);
          if (cnt == 1 && !p.linear) b.real(b.logConst(n.weights[j]));  // single child: value + log weight
          else b.real(n.weights[j]);
        }
        b.end(at);
        b.txt << "  " << slotName(slotOf[in.node]) << " = sum(" << cnt << " terms)   ; node " << in.node << "\n";
        break;
      }
      case OP_SUMLAYER: {
        uint32_t cnt = uint32_t(n.children.size());
        uint32_t m = uint32_t(in.defs.size());
        const size_t at = b.begin();
        b.word(OP_SUMLAYER | longFlag | (cnt << 8));
        b.word(m);
        for (uint32_t d : in.defs) slotWord(slotOf[d]);
        for (uint32_t j = 0; j < cnt; ++j) slotWord(slotOf[n.children[j]]);
        for (uint32_t j = 0; j < cnt; ++j)
          for (uint32_t d : in.defs) b.real(g.nodes[d].weights[j]);
        b.end(at);
        b.txt << "  " << slotName(slotOf[in.defs[0]]) << ".. = sumlayer(" << m << " sums x " << cnt << " terms)   ; nodes " << in.defs[0] << "..\n";
        break;
      }
      case OP_OUTERSUM: {
        const Outer& outer = outerOf.at(n.children);
        const uint32_t na = uint32_t(outer.a.size()), nb = uint32_t(outer.b.size());
        uint32_t m = uint32_t(in.defs.size());
        // A single leftover sum is encoded as a layer of two identical sums writing the same slot.
        std::vector<uint32_t> defs = in.defs;
        if (m == 1) defs.push_back(in.defs[0]);
        const bool matrixForm = matrixInstr[k] && !p.f64;  // double programs: the fused leaf forms below, else an ordinary outer sum
        const size_t at = b.begin();
        // Matrix form: bits 24-29 say where each slot list lives (0 all in the short pool, 1 all in the long pool,
        // 2 mixed), so the kernel picks the access instructions per list, not per slot; bits 30 and 31 say that
        // the a / b list is a scaled linear vector; bit 8 of the second word that the result is one.
        auto tierOf = [&](const std::vector<uint32_t>& nodes) {
          uint32_t longOnes = 0;
          for (uint32_t x : nodes) longOnes += (slotOf[x] & LONG_BIT) ? 1 : 0;
          return longOnes == 0 ? 0u : (longOnes == nodes.size() ? 1u : 2u);
        };
        const uint32_t scaleA = matrixForm ? scaleSlotOfNode[outer.a[0]] : NONE, scaleB = matrixForm ? scaleSlotOfNode[outer.b[0]] : NONE;
        uint32_t scaleDst = NONE;
        if (matrixForm && linearConsumer[k] >= 0) {
          // Lives exactly as long as the vector: the ninth slot of its block, or a slot of its own.
          scaleDst = blockOfNode[in.defs[0]] >= 0 ? slotOf[in.defs[0]] + 8 : allocSlot(in.defs[0]);
          scaleSlotOfNode[in.defs[0]] = scaleDst;
          if (scaleDst & LONG_BIT) longFlag |= 0x80u;
        }
        if (scaleA != NONE && (scaleA & LONG_BIT)) longFlag |= 0x80u;
        if (scaleB != NONE && (scaleB & LONG_BIT)) longFlag |= 0x80u;
        auto consecutive = [&](const std::vector<uint32_t>& nodes) {
          for (size_t j = 1; j < nodes.size(); ++j)
            if (slotOf[nodes[j]] != slotOf[nodes[0]] + j) return false;
          return true;
        };
        // Feature fields: slots of the staged values, or input columns when features are not staged.
        const bool stagedFeatures = p.featureMode == FEAT_STAGED;
        const uint32_t leafFlag = stagedFeatures && stagedLong ? 0x80u : 0u, featTier = stagedFeatures && stagedLong ? 1u << 16 : 0u;
        auto emitLeafFeatures = [&](const Outer& region) {
          for (uint32_t list : {region.a[0], region.b[0]})
            for (uint32_t c : g.nodes[list].children) {
              if (stagedFeatures) slotWord(valueSlotOf[g.nodes[c].feature]);
              else if (p.featureMode == FEAT_REGISTER) b.word(valueSlotOf[g.nodes[c].feature]);
              else b.word(g.nodes[c].feature);
            }
        };
        auto emitLeafConstants = [&](const Outer& region) {
          for (const std::vector<uint32_t>* list : {&region.a, &region.b})
            for (uint32_t prod : *list)
              for (uint32_t c : g.nodes[prod].children) {
                const auto& leaf = g.nodes[c];
                const double coef = -std::log(leaf.stddev) + -0.5 * std::log(2 * M_PI), den = -(1.0 / (2.0 * leaf.stddev * leaf.stddev));
                b.real(leaf.mean);
                b.real(coef / den);
                b.real(den * b.scale);
              }
        };
        auto emitMatrixWeights = [&](const std::vector<uint32_t>& sums, uint32_t products) {
          if (p.f64) {  // product-major, the eight sums of a product side by side: sixteen weights per lane vector
            for (uint32_t q = 0; q < products; ++q)
              for (uint32_t t = 0; t < 8; ++t) b.real(g.nodes[sums[t]].weights[q]);
            return;
          }
          for (uint32_t grp = 0; grp < products / 16; ++grp)
            for (uint32_t half = 0; half < 2; ++half)
              for (uint32_t lane = 0; lane < 64; ++lane) b.real(g.nodes[sums[half * 4 + lane % 4]].weights[grp * 16 + lane / 4]);
        };
        if (leafQuad[k].first != NONE) {
          // Regions in the order 1, 2 (first pair), 3, 4 (second pair); weights: region, region, pair sum, twice, then this sum.
          const uint32_t pairs[2] = {leafQuad[k].first, leafQuad[k].second};
          const Instr* regionInstr[4];
          const Outer* region[4];
          for (int q = 0; q < 2; ++q) {
            regionInstr[2 * q] = &instrs[leafPair[pairs[q]].first];
            regionInstr[2 * q + 1] = &instrs[leafPair[pairs[q]].second];
          }
          for (int r = 0; r < 4; ++r) region[r] = &outerOf.at(g.nodes[regionInstr[r]->node].children);
          const uint32_t G = uint32_t(g.nodes[region[0]->a[0]].children.size());
          longFlag |= leafFlag;
          b.word(OP_LEAFQUADMM | longFlag | (4u << 8) | (tierOf(defs) << 28));
          b.word(8u | (scaleDst != NONE ? 0x100u : 0u) | (consecutive(defs) ? 0x800u : 0u) | (G << 12) | featTier);
          for (uint32_t d : defs) slotWord(slotOf[d]);
          if (scaleDst != NONE) slotWord(scaleDst);
          else b.word(NONE);
          for (int r = 0; r < 4; ++r) emitLeafFeatures(*region[r]);
          for (int r = 0; r < 4; ++r) emitLeafConstants(*region[r]);
          for (int q = 0; q < 2; ++q) {
            emitMatrixWeights(regionInstr[2 * q]->defs, 16);
            emitMatrixWeights(regionInstr[2 * q + 1]->defs, 16);
            emitMatrixWeights(instrs[pairs[q]].defs, 64);
          }
          emitMatrixWeights(defs, 64);
          b.end(at);
          b.txt << "  " << slotName(slotOf[in.defs[0]]) << ".. = leafquad(8 sums x 8x8 products of two pairs of leaf regions: 8 sums x 4x4 products of " << G
                << " gaussians)" << (scaleDst != NONE ? " scaled" : "") << "   ; nodes " << in.defs[0] << "..\n";
          break;
        }
        if (leafPair[k].first != NONE) {
          const Instr& ri = instrs[leafPair[k].first];
          const Instr& rj = instrs[leafPair[k].second];
          const Outer& oi = outerOf.at(g.nodes[ri.node].children);
          const Outer& oj = outerOf.at(g.nodes[rj.node].children);
          const uint32_t N = uint32_t(oi.a.size()), G = uint32_t(g.nodes[oi.a[0]].children.size());
          longFlag |= leafFlag;
          b.word(OP_LEAFPAIRMM | longFlag | (N << 8) | (tierOf(defs) << 28));
          b.word(8u | (scaleDst != NONE ? 0x100u : 0u) | (consecutive(defs) ? 0x800u : 0u) | (G << 12) | featTier);
          for (uint32_t d : defs) slotWord(slotOf[d]);
          if (scaleDst != NONE) slotWord(scaleDst);
          else b.word(NONE);
          emitLeafFeatures(oi);
          emitLeafFeatures(oj);
          emitLeafConstants(oi);
          emitLeafConstants(oj);
          emitMatrixWeights(ri.defs, N * N);
          emitMatrixWeights(rj.defs, N * N);
          emitMatrixWeights(defs, 64);
          b.end(at);
          b.txt << "  " << slotName(slotOf[in.defs[0]]) << ".. = leafpair(8 sums x 8x8 products of two leaf regions: 8 sums x " << N << "x" << N
                << " products of " << G << " gaussians)" << (scaleDst != NONE ? " scaled" : "") << "   ; nodes " << in.defs[0] << "..\n";
          break;
        }
        if (leafRegion[k]) {
          const uint32_t G = uint32_t(g.nodes[outer.a[0]].children.size());
          longFlag |= leafFlag;
          b.word(OP_LEAFMM | longFlag | (na << 8) | (nb << 16) | (tierOf(defs) << 28));
          b.word(8u | (scaleDst != NONE ? 0x100u : 0u) | (consecutive(defs) ? 0x800u : 0u) | (G << 12) | featTier);
          for (uint32_t d : defs) slotWord(slotOf[d]);
          if (scaleDst != NONE) slotWord(scaleDst);
          else b.word(NONE);
          emitLeafFeatures(outer);
          emitLeafConstants(outer);
          emitMatrixWeights(defs, na * nb);
          b.end(at);
          b.txt << "  " << slotName(slotOf[in.defs[0]]) << ".. = leafregion(8 sums x " << na << "x" << nb << " products of " << G << " gaussians)"
                << (scaleDst != NONE ? " scaled" : "") << "   ; nodes " << in.defs[0] << "..\n";
          break;
        }
        const uint32_t tiers = matrixForm ? (tierOf(outer.a) << 24) | (tierOf(outer.b) << 26) | (tierOf(defs) << 28) |
                                                (scaleA != NONE ? 1u << 30 : 0u) | (scaleB != NONE ? 1u << 31 : 0u)
                                          : 0u;
        b.word((matrixForm ? OP_OUTERMM : OP_OUTERSUM) | longFlag | (na << 8) | (nb << 16) | tiers);
        // Bits 9-11 of the second word: the a, b and dst lists are runs of consecutive slots.
        const uint32_t runs = matrixForm ? (consecutive(outer.a) ? 0x200u : 0u) | (consecutive(outer.b) ? 0x400u : 0u) | (consecutive(defs) ? 0x800u : 0u) : 0u;
        b.word(uint32_t(defs.size()) | (scaleDst != NONE ? 0x100u : 0u) | runs);
        for (uint32_t d : defs) slotWord(slotOf[d]);
        for (uint32_t a : outer.a) slotWord(slotOf[a]);
        for (uint32_t c : outer.b) slotWord(slotOf[c]);
        if (matrixForm) {  // the three scale slots, unused ones as NONE
          for (uint32_t sc : {scaleDst, scaleA, scaleB}) {
            if (sc != NONE) slotWord(sc);
            else b.word(NONE);
          }
        }
        if (matrixForm) {
          for (uint32_t grp = 0; grp < na * nb / 16; ++grp)
            for (uint32_t half = 0; half < 2; ++half)
              for (uint32_t lane = 0; lane < 64; ++lane) b.real(g.nodes[defs[half * 4 + lane % 4]].weights[grp * 16 + lane / 4]);
        } else {
          for (uint32_t j = 0; j < na * nb; ++j)
            for (uint32_t d : defs) b.real(g.nodes[d].weights[j]);
        }
        b.end(at);
        b.txt << "  " << slotName(slotOf[in.defs[0]]) << ".. = outersum(" << m << " sums x " << na << "x" << nb << " products)"
              << (scaleDst != NONE ? " scaled" : "") << "   ; nodes " << in.defs[0] << "..\n";
        break;
      }
      default:
        break;
    }
    // A value nobody reads later (cannot happen for reachable nodes, kept for safety).
    for (uint32_t d : in.defs)
      if (d != g.root() && lastUse[d] <= k) releaseNode(d);
  }
  flushBatch();
  {
    const size_t at = b.begin();
    b.word(OP_END | ((slotOf[g.root()] & LONG_BIT) ? 0x80u : 0u));
    slotWord(slotOf[g.root()]);
    b.end(at);
  }
  for (size_t pos : longWords) p.code[pos] = highWater + (p.code[pos] & ~LONG_BIT);
  for (auto& sf : p.staged) {
    if (sf.valueSlot != NONE && (sf.valueSlot & LONG_BIT)) sf.valueSlot = highWater + (sf.valueSlot & ~LONG_BIT);
    if (sf.indexSlot != NONE && (sf.indexSlot & LONG_BIT)) sf.indexSlot = highWater + (sf.indexSlot & ~LONG_BIT);
  }
  p.shortSlots = highWater;
  p.numSlots = highWater + longCount;
  p.numInstructions = uint32_t(instrs.size());
  p.spillAccesses = uint32_t(longWords.size());
  p.ldsSlotLimit = uint32_t(o.interpLdsSlots);
  std::ostringstream hdr;
  hdr << "; interpreter program for SPN '" << g.name << "': " << instrs.size() << " instructions, " << p.code.size() << " words, "
      << p.numSlots << " value slots (" << p.reservedSlots << " staged features, " << (p.numSlots - p.shortSlots) << " long-lived), compute " << (p.f64 ? "f64" : "f32")
      << (p.log2Domain ? " log2-domain" : "") << (p.linear ? " linear space" : "") << ", features " << (p.featureMode == FEAT_STAGED ? "staged" : (p.featureMode == FEAT_REGISTER ? "in registers" : "direct")) << "\n";
  p.listing = hdr.str() + b.txt.str();
  return p;
}
}  // namespace

}  // namespace spnc_hip
