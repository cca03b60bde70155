#include "kernel.h"

#include <hip/hiprtc.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <thread>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <stdexcept>

#include "interp_kernel.h"

namespace spnc_hip {

namespace {

[[noreturn]] void fatal(const std::string& m) { throw std::runtime_error(m); }

void hipCheck(hipError_t e, const char* what) {
  if (e != hipSuccess) fatal(std::string("HIP error in ") + what + ": " + hipGetErrorString(e));
}

std::vector<char> compileWithHipRtc(const JitSource& js, int optLevel, int machineLicm) {
  hiprtcProgram prog;
  if (hiprtcCreateProgram(&prog, js.source.c_str(), "spn_kernel.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS)
    fatal("hiprtcCreateProgram failed");
  std::string opt = "-O" + std::to_string(std::max(0, std::min(3, optLevel)));
  // Packed-FP32 instruction selection is switched off for all device code of this library.
  std::vector<const char*> opts = {"--offload-arch=gfx950", opt.c_str(),       "-std=c++17",       "-ffp-contract=fast",
                                   "-Xclang",               "-target-feature", "-Xclang",          "-packed-fp32-ops"};
  // The kernel body sits in a grid-stride loop. Double constants cannot be instruction literals, and machine LICM
  // moves the thousands of register moves that materialise them out of that loop, where they no longer fit the
  // register file (measured on a 1389-node graph: 512 VGPRs plus 1612 spills with it, 75 VGPRs without).
  // Float kernels with one sample per lane are as fast or a few percent faster without it (16 Gaussian features
  // with NaN selects: +3 %); with two samples per lane it pays (-33 % without).
  if (machineLicm == 0 || (machineLicm < 0 && (js.doubleConstants || js.samplesPerLane == 1))) {
    opts.push_back("-mllvm");
    opts.push_back("-disable-machine-licm");
  }
  hiprtcResult r = hiprtcCompileProgram(prog, int(opts.size()), opts.data());
  if (r != HIPRTC_SUCCESS) {
    size_t ls = 0;
    hiprtcGetProgramLogSize(prog, &ls);
    std::string log(ls, '\0');
    if (ls) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    fatal("COMPILATION ERROR: hipRTC failed: " + log);
  }
  size_t cs = 0;
  hiprtcGetCodeSize(prog, &cs);
  std::vector<char> code(cs);
  hiprtcGetCode(prog, code.data());
  hiprtcDestroyProgram(&prog);
  return code;
}

// Registers the compiler spilled to scratch memory, from the code object's metadata (a msgpack map in an ELF note:
// the key ".vgpr_spill_count" is followed by an unsigned integer). 0 when the key is absent.
uint32_t spilledRegisters(const std::vector<char>& code) {
  static const char key[] = ".vgpr_spill_count";
  const size_t keyLen = sizeof(key) - 1;
  uint32_t most = 0;
  for (size_t at = 0; at + keyLen + 5 <= code.size(); ++at) {
    if (std::memcmp(code.data() + at, key, keyLen) != 0) continue;
    const unsigned char* v = reinterpret_cast<const unsigned char*>(code.data()) + at + keyLen;
    uint32_t n = 0;
    if (v[0] < 0x80) n = v[0];
    else if (v[0] == 0xcc) n = v[1];
    else if (v[0] == 0xcd) n = (uint32_t(v[1]) << 8) | v[2];
    else if (v[0] == 0xce) n = (uint32_t(v[1]) << 24) | (uint32_t(v[2]) << 16) | (uint32_t(v[3]) << 8) | v[4];
    most = std::max(most, n);
  }
  return most;
}

// ---- kernel file: magic, then tagged little-endian fields ----
const char kMagic[8] = {'S', 'P', 'N', 'C', 'H', 'I', 'P', 4};

struct Writer {
  std::vector<char> buf;
  void u32(uint32_t v) { raw(&v, 4); }
  void u64(uint64_t v) { raw(&v, 8); }
  void raw(const void* p, size_t n) { buf.insert(buf.end(), static_cast<const char*>(p), static_cast<const char*>(p) + n); }
  void str(const std::string& s) {
    u64(s.size());
    raw(s.data(), s.size());
  }
  template <typename T>
  void vec(const std::vector<T>& v) {
    u64(v.size());
    raw(v.data(), v.size() * sizeof(T));
  }
};

struct Reader {
  const std::vector<char>& buf;
  size_t pos = 0;
  explicit Reader(const std::vector<char>& b) : buf(b) {}
  void raw(void* p, size_t n) {
    if (n > buf.size() - pos) fatal("RUNTIME ERROR: truncated kernel file");
    std::memcpy(p, buf.data() + pos, n);
    pos += n;
  }
  uint32_t u32() {
    uint32_t v;
    raw(&v, 4);
    return v;
  }
  uint64_t u64() {
    uint64_t v;
    raw(&v, 8);
    return v;
  }
  std::string str() {
    uint64_t n = u64();
    if (n > buf.size() - pos) fatal("RUNTIME ERROR: truncated kernel file");
    std::string s(buf.data() + pos, size_t(n));
    pos += size_t(n);
    return s;
  }
  template <typename T>
  std::vector<T> vec() {
    uint64_t n = u64();
    if (n > (buf.size() - pos) / sizeof(T)) fatal("RUNTIME ERROR: truncated kernel file");
    std::vector<T> v(static_cast<size_t>(n));
    raw(v.data(), size_t(n) * sizeof(T));
    return v;
  }
};

// Shortest decimal form that reads back as the same double, integral values with ".0" (2.0, 4.4).
std::string jsonDouble(double v) {
  char buf[40];
  for (int prec = 1; prec <= 17; ++prec) {
    std::snprintf(buf, sizeof(buf), "%.*g", prec, v);
    if (std::strtod(buf, nullptr) == v) break;
  }
  std::string t(buf);
  if (t.find_first_of(".eEn") == std::string::npos) t += ".0";
  return t;
}

// Copies between pageable host memory and the pinned staging buffers on a few threads: one core moves about
// 10 GB/s, the PCIe link several times that, so a single memcpy is what bounds the host path of small SPNs.
class CopyCrew {
 public:
  static CopyCrew& instance() {
    static CopyCrew* crew = new CopyCrew();  // never destroyed: its parked threads outlive static destruction
    return *crew;
  }
  void copy(void* dst, const void* src, size_t bytes) {
    const size_t parts = workers_.size() + 1;
    // A child process made by fork() inherits this object but not its threads: it copies on its own.
    if (bytes < (size_t(4) << 20) || parts == 1 || getpid() != owner_) {
      std::memcpy(dst, src, bytes);
      return;
    }
    std::lock_guard<std::mutex> serial(callMutex_);  // one copy at a time
    const size_t share = (bytes / parts + 4095) & ~size_t(4095);
    {
      std::lock_guard<std::mutex> lock(mutex_);
      for (size_t w = 0; w < workers_.size(); ++w) {
        const size_t lo = std::min(bytes, (w + 1) * share), hi = std::min(bytes, (w + 2) * share);
        jobs_[w] = Job{static_cast<char*>(dst) + lo, static_cast<const char*>(src) + lo, hi - lo};
      }
      pending_ = workers_.size();
      ++generation_;
    }
    wake_.notify_all();
    std::memcpy(dst, src, std::min(bytes, share));
    std::unique_lock<std::mutex> lock(mutex_);
    done_.wait(lock, [&] { return pending_ == 0; });
  }

 private:
  struct Job {
    char* dst = nullptr;
    const char* src = nullptr;
    size_t bytes = 0;
  };
  CopyCrew() : owner_(getpid()) {
    unsigned n = std::thread::hardware_concurrency();
    n = n >= 8 ? 3 : (n >= 4 ? 1 : 0);  // the calling thread copies a share too
    jobs_.resize(n);
    for (unsigned w = 0; w < n; ++w) workers_.emplace_back([this, w] { run(w); });
    for (auto& t : workers_) t.detach();
  }
  void run(unsigned w) {
    uint64_t seen = 0;
    for (;;) {
      Job job;
      {
        std::unique_lock<std::mutex> lock(mutex_);
        wake_.wait(lock, [&] { return generation_ != seen; });
        seen = generation_;
        job = jobs_[w];
      }
      if (job.bytes) std::memcpy(job.dst, job.src, job.bytes);
      {
        std::lock_guard<std::mutex> lock(mutex_);
        if (--pending_ == 0) done_.notify_one();
      }
    }
  }
  const pid_t owner_;  // the process whose threads these are
  std::vector<std::thread> workers_;
  std::vector<Job> jobs_;
  std::mutex mutex_, callMutex_;
  std::condition_variable wake_, done_;
  size_t pending_ = 0;
  uint64_t generation_ = 0;
};

// True if the `bytes` bytes at `p` are host memory the GPU can copy from directly (hipHostMalloc / pinned), so that no
// staging copy is needed: the first and the last byte must both lie in such an allocation.
bool isPinnedHost(const void* p, size_t bytes) {
  auto pinned = [](const void* q) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, q) != hipSuccess) {
      (void)hipGetLastError();  // ordinary pageable memory is "invalid value" to the runtime
      return false;
    }
    return attr.type == hipMemoryTypeHost;
  };
  return bytes != 0 && pinned(p) && pinned(static_cast<const char*>(p) + bytes - 1);
}

// Launches that share one device buffer take turns on it across streams: every launch records `done`, and a launch on
// another stream than the last one waits for it first. Work on a stream that is being captured into a graph is left
// alone (an event recorded outside the capture cannot be waited for inside it): the graph's own edges order it.
bool capturing(hipStream_t stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status != hipStreamCaptureStatusNone;
}

std::string makeKernelFilePath() {
  const char* dir = std::getenv("TMPDIR");
  std::string tmpl = std::string(dir && *dir ? dir : "/tmp") + "/spnc_hip_XXXXXX.hipk";
  std::vector<char> path(tmpl.begin(), tmpl.end());
  path.push_back('\0');
  int fd = mkstemps(path.data(), 5);
  if (fd < 0) fatal("COMPILATION ERROR: cannot create kernel file " + tmpl);
  close(fd);
  return std::string(path.data());
}

}  // namespace

std::unique_ptr<Kernel> Kernel::compile(const std::string& queryPath, const std::map<std::string, std::string>& options) {
  CompileOptions o = parseOptions(options);
  RawQuery q = readQueryFile(queryPath);
  Graph g = buildGraph(q);
  std::unique_ptr<Kernel> k(new Kernel());
  k->kernelName_ = g.name;
  k->batchSize_ = unsigned(std::max(1, g.batchSize));
  k->numFeatures_ = g.numFeatures;
  k->bytesPerFeature_ = g.ftype.bytes;
  k->featureType_ = unsigned(g.ftype.type);
  k->marginal_ = g.supportMarginal;
  k->stats_ = g.stats;
  k->numNodes_ = unsigned(g.nodes.size());

  // Size estimate that decides between the two kernels under "auto": terms of sums weigh more
  // when the kernel calls the accurate library exp/log (float64 and natural-log float32) than
  // when it uses the hardware exp2/log2 instructions.
  const bool hardwareTranscendentals = o.useLogSpace && o.computeType == ComputeType::F32 && o.log2Domain;
  const uint64_t ops = g.nodes.size() + g.stats.productAdds + g.stats.sumTerms * (hardwareTranscendentals ? 1 : 6);
  // The reference's "maxTaskSize" bounds the operations per compiled task by cutting the graph into several tasks
  // (mlir/lib/Dialect/LoSPN/Passes/LoSPNTaskPartitioner.cpp:36-148); the straight-line kernels are cut the same way
  // (partition.cpp). The interpreter's code does not grow with the graph and ignores the option.
  const uint64_t jitLimit = uint64_t(std::max(0, o.jitMaxOps));
  // In linear space (computed in double, as in the reference) the interpreter takes what is too large for one
  // straight-line kernel as well, unless the caller asked for tasks: its program is there at once, where the kernels
  // of a graph cut into tasks take hipRTC minutes (47 k nodes: 100-125 s).
  bool useInterp = o.kernelMode == KernelMode::Interpreter || (o.kernelMode == KernelMode::Auto && ops > jitLimit && (o.useLogSpace || o.maxTaskSize <= 0));
  if (useInterp) {
    k->kind_ = SPNC_HIP_KERNEL_INTERPRETER;
    k->prog_ = buildInterpProgram(g, o);
    checkInterpProgram(k->prog_, g.numFeatures);  // the builder's invariants, checked before anything runs on a device
    k->bytesPerResult_ = k->prog_.f64 ? 8 : 4;
    k->inputAlign_ = g.ftype.bytes;
    k->text_ = k->prog_.listing;
    k->gridPolicy_ = std::max(0, o.blocksPerCU);  // a limit on the resident blocks; the interpreter is always persistent
  } else {
    k->kind_ = SPNC_HIP_KERNEL_JIT;
    TaskPlan plan;
    int taskSize = o.maxTaskSize;
    if (taskSize > 0) plan = partitionGraph(g, taskSize);
    JitSource js;
    if (plan.tasks.size() > 1) {
      // One translation unit with a kernel per task: each task's source in a namespace of its own, the macros it
      // defines dropped again after it.
      std::string all;
      js.inputAlign = 1;
      // Whether the exp/log routines are inlined is decided by the size of the whole graph, as without the cut: what
      // costs hipRTC time is the sum of all inlined copies, whichever kernel they land in.
      CompileOptions taskOptions = o;
      if (o.inlineMath < 0) taskOptions.inlineMath = inlineLibraryMath(g, o) ? 1 : 0;
      for (size_t t = 0; t < plan.tasks.size(); ++t) {
        const Graph& tg = plan.tasks[t];
        JitSource one = emitHipSource(tg, taskOptions, "spn_task" + std::to_string(t));
        size_t valuesIn = 0;
        for (const auto& n : tg.nodes) valuesIn += n.kind == NodeKind::External ? 1 : 0;
        all += "// task " + std::to_string(t) + " of " + std::to_string(plan.tasks.size()) + ": " + std::to_string(taskWeight(tg)) + " operations, " +
               std::to_string(valuesIn) + " values in, " + std::to_string(tg.taskOutputs.size()) + " values out" + (tg.taskFinal ? ", the result" : "") + "\n";
        all += "namespace spn_task_scope" + std::to_string(t) + " {\n" + one.source + "}  // task " + std::to_string(t) +
               "\n#undef SPN_LOAD\n#undef SPN_LOAD_TILE\n#undef SPN_F\n#undef SPN_BLOCK\n#undef SPN_U\n#undef SPN_NTAB\n#undef SPN_DOUBLE_TABLES\n"
               "#undef SPN_EXP2_TABLE\n#undef SPN_LOG2_TABLE\n#undef SPN_POLY\n#undef SPN_NCTAB\n#undef SPN_CTAB\n";
        Task task;
        task.entry = one.entry;
        task.blockSize = one.blockSize;
        task.gridPolicy = o.blocksPerCU != 0 ? o.blocksPerCU : (one.oneTilePerBlock ? -1 : 0);
        k->tasks_.push_back(task);
        js.inputAlign = std::max(js.inputAlign, one.inputAlign);
        js.libraryMath = js.libraryMath || one.libraryMath;
        js.doubleConstants = js.doubleConstants || one.doubleConstants;
        js.bytesPerResult = one.bytesPerResult;
      }
      js.source = std::move(all);
      js.entry = k->tasks_.back().entry;
      js.blockSize = k->tasks_.back().blockSize;
      js.samplesPerLane = 1;
      k->taskSlots_ = plan.slots;
      k->taskBufferMiB_ = unsigned(o.taskBufferMiB);
    } else {
      js = emitHipSource(g, o);
    }
    // The generated code is already straight-line and CSE'd. Kernels that inline the library
    // exp/log are built at -O1 unless the caller asks otherwise: at -O2 and above the mid-level
    // optimiser stretches live ranges until the float64 kernels spill (512 VGPRs plus scratch,
    // about 7x slower on the 16-feature Gaussian tree).
    const int level = (js.libraryMath && !o.optLevelGiven) ? 1 : o.optLevel;
    k->codeObject_ = compileWithHipRtc(js, level, o.machineLicm);
    if (js.packedRows && o.packedRows < 0 && spilledRegisters(k->codeObject_) > 0) {
      // Packed rows keep one or two values per small-domain feature in registers for the whole kernel; on graphs
      // where that does not fit (measured: 2640 nodes, 537 spilled registers, 6.9 ms against 1.1 ms) the kernel
      // with one index per feature is built instead.
      CompileOptions unpacked = o;
      unpacked.packedRows = 0;
      js = emitHipSource(g, unpacked);
      k->codeObject_ = compileWithHipRtc(js, level, o.machineLicm);
    }
    k->entry_ = js.entry;
    k->blockSize_ = js.blockSize;
    k->samplesPerLane_ = js.samplesPerLane;
    k->inputAlign_ = js.inputAlign;
    k->gridPolicy_ = o.blocksPerCU != 0 ? o.blocksPerCU : (js.oneTilePerBlock ? -1 : 0);
    k->bytesPerResult_ = js.bytesPerResult;
    k->text_ = std::move(js.source);
  }
  if (o.dumpIR) std::cerr << "// *** device code for " << k->kernelName_ << " ***\n" << k->text_ << std::endl;
  if (o.collectGraphStats) {
    // The reference's keys and its compact, key-sorted JSON (LoSPNGraphStatsCollection.cpp:85-102), counted as there
    // on the binarised graph before identical nodes are merged; "hip" holds what this target adds.
    const LoSpnStats ls = computeLoSpnStats(q, o.useLogSpace);
    const GraphStats& s = g.stats;
    std::ofstream st(o.graphStatsFile);
    if (!st) fatal("COMPILATION ERROR: cannot write graph statistics to '" + o.graphStatsFile + "'");
    st << "{\"averageDepth\":" << jsonDouble(ls.averageDepth) << ",\"categoricalCount\":" << ls.categoricalCount
       << ",\"constantCount\":" << ls.constantCount << ",\"featureCount\":" << g.numFeatures << ",\"gaussianCount\":" << ls.gaussianCount
       << ",\"hip\":{\"depthsExact\":" << (ls.depthsExact ? "true" : "false") << ",\"flopsMin\":" << s.flopsMin << ",\"maxFanIn\":" << s.maxFanIn
       << ",\"mergedNodes\":" << g.nodes.size() << ",\"sumTerms\":" << s.sumTerms << ",\"transMin\":" << s.transMin << "}"
       << ",\"histogramCount\":" << ls.histogramCount << ",\"innerCount\":" << ls.innerCount() << ",\"leafCount\":" << ls.leafCount()
       << ",\"maxDepth\":" << ls.maxDepth << ",\"medianDepth\":" << jsonDouble(ls.medianDepth) << ",\"minDepth\":" << ls.minDepth
       << ",\"productCount\":" << ls.productCount << ",\"sumCount\":" << ls.sumCount << "}";
    st.close();
    if (!st) fatal("COMPILATION ERROR: cannot write graph statistics to '" + o.graphStatsFile + "'");
  }
  k->fileName_ = makeKernelFilePath();
  k->save(k->fileName_);
  return k;
}

void Kernel::save(const std::string& path) const {
  Writer w;
  w.raw(kMagic, 8);
  w.str(kernelName_);
  w.u32(batchSize_);
  w.u32(numFeatures_);
  w.u32(bytesPerFeature_);
  w.u32(bytesPerResult_);
  w.u32(featureType_);
  w.u32(marginal_);
  w.u32(kind_);
  w.u32(numNodes_);
  w.raw(&stats_, sizeof(stats_));
  w.str(text_);
  if (kind_ == SPNC_HIP_KERNEL_JIT) {
    w.vec(codeObject_);
    w.str(entry_);
    w.u32(blockSize_);
    w.u32(samplesPerLane_);
    w.u32(inputAlign_);
    w.u32(uint32_t(gridPolicy_));
    w.u32(uint32_t(tasks_.size()));
    for (const Task& t : tasks_) {
      w.str(t.entry);
      w.u32(t.blockSize);
      w.u32(uint32_t(t.gridPolicy));
    }
    w.u32(taskSlots_);
    w.u32(taskBufferMiB_);
  } else {
    w.u32(prog_.f64);
    w.u32(prog_.log2Domain);
    w.u32(prog_.linear);
    w.u32(prog_.featureMode);
    w.vec(prog_.code);
    w.vec(prog_.tables);
    w.vec(prog_.directTableLen);
    w.u64(prog_.staged.size());
    for (const auto& s : prog_.staged) {
      w.u32(s.column);
      w.u32(s.valueSlot);
      w.u32(s.indexSlot);
      w.u32(s.tableLen);
    }
    w.u32(prog_.numSlots);
    w.u32(prog_.shortSlots);
    w.u32(prog_.reservedSlots);
    w.u32(prog_.numInstructions);
    w.u32(prog_.ldsSlotLimit);
    w.u32(prog_.mathTables);
  }
  FILE* f = std::fopen(path.c_str(), "wb");
  if (!f) fatal("COMPILATION ERROR: cannot write kernel file " + path);
  size_t n = std::fwrite(w.buf.data(), 1, w.buf.size(), f);
  std::fclose(f);
  if (n != w.buf.size()) fatal("COMPILATION ERROR: short write to kernel file " + path);
}

std::unique_ptr<Kernel> Kernel::load(const std::string& kernelFile) {
  std::ifstream f(kernelFile, std::ios::binary);
  if (!f) fatal("RUNTIME ERROR: cannot open kernel file " + kernelFile);
  std::vector<char> buf((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
  if (buf.size() < 8 || std::memcmp(buf.data(), kMagic, 8) != 0) fatal("RUNTIME ERROR: " + kernelFile + " is not a spnc-hip kernel file");
  Reader r(buf);
  r.pos = 8;
  std::unique_ptr<Kernel> k(new Kernel());
  k->fileName_ = kernelFile;
  k->kernelName_ = r.str();
  k->batchSize_ = r.u32();
  k->numFeatures_ = r.u32();
  k->bytesPerFeature_ = r.u32();
  k->bytesPerResult_ = r.u32();
  k->featureType_ = r.u32();
  k->marginal_ = r.u32() != 0;
  k->kind_ = r.u32();
  k->numNodes_ = r.u32();
  r.raw(&k->stats_, sizeof(k->stats_));
  k->text_ = r.str();
  if (k->kind_ == SPNC_HIP_KERNEL_JIT) {
    k->codeObject_ = r.vec<char>();
    k->entry_ = r.str();
    k->blockSize_ = r.u32();
    k->samplesPerLane_ = r.u32();
    k->inputAlign_ = r.u32();
    k->gridPolicy_ = int(r.u32());
    const uint32_t numTasks = r.u32();
    if (numTasks > (1u << 20)) fatal("RUNTIME ERROR: kernel file " + kernelFile + " is damaged (task count)");
    for (uint32_t t = 0; t < numTasks; ++t) {
      Task task;
      task.entry = r.str();
      task.blockSize = r.u32();
      task.gridPolicy = int(r.u32());
      k->tasks_.push_back(task);
    }
    k->taskSlots_ = r.u32();
    k->taskBufferMiB_ = r.u32();
  } else if (k->kind_ == SPNC_HIP_KERNEL_INTERPRETER) {
    k->prog_.f64 = r.u32() != 0;
    k->prog_.log2Domain = r.u32() != 0;
    k->prog_.linear = r.u32() != 0;
    k->prog_.featureMode = FeatureMode(r.u32());
    k->prog_.code = r.vec<uint32_t>();
    k->prog_.tables = r.vec<double>();
    k->prog_.directTableLen = r.vec<uint32_t>();
    uint64_t ns = r.u64();
    for (uint64_t i = 0; i < ns; ++i) {
      StagedFeature s;
      s.column = r.u32();
      s.valueSlot = r.u32();
      s.indexSlot = r.u32();
      s.tableLen = r.u32();
      k->prog_.staged.push_back(s);
    }
    k->prog_.numSlots = r.u32();
    k->prog_.shortSlots = r.u32();
    k->prog_.reservedSlots = r.u32();
    k->prog_.numInstructions = r.u32();
    k->prog_.ldsSlotLimit = r.u32();
    k->prog_.mathTables = r.u32();
    k->inputAlign_ = k->bytesPerFeature_;
  } else {
    fatal("RUNTIME ERROR: unknown kernel kind in " + kernelFile);
  }
  // Nothing read from the file reaches a launch unchecked: a truncated, foreign or damaged file is a host error.
  auto reject = [&](const char* what) { fatal("RUNTIME ERROR: kernel file " + kernelFile + " is damaged (" + what + ")"); };
  if (r.pos != buf.size()) reject("trailing bytes");
  if (k->numFeatures_ == 0 || k->numFeatures_ > (1u << 24)) reject("feature count");
  if (k->featureType_ > unsigned(FeatureType::F64)) reject("feature type");
  static const unsigned widths[] = {1, 2, 4, 8, 4, 8};
  if (k->bytesPerFeature_ != widths[k->featureType_]) reject("feature width");
  if (k->bytesPerResult_ != 4 && k->bytesPerResult_ != 8) reject("result width");
  if (k->kind_ == SPNC_HIP_KERNEL_JIT) {
    if (k->blockSize_ < 64 || k->blockSize_ > 1024 || k->blockSize_ % 64 != 0) reject("block size");
    if (k->samplesPerLane_ < 1 || k->samplesPerLane_ > 16) reject("samples per lane");
    if (k->inputAlign_ == 0 || k->inputAlign_ > 16 || (k->inputAlign_ & (k->inputAlign_ - 1)) != 0) reject("input alignment");
    if (k->gridPolicy_ < -1 || k->gridPolicy_ > 64) reject("grid policy");
    if (k->entry_.empty() || k->codeObject_.size() < 64) reject("code object");
    if (k->tasks_.size() == 1 || k->taskSlots_ > (1u << 24) || (k->tasks_.empty() && k->taskSlots_ != 0)) reject("tasks");
    for (const Task& t : k->tasks_) {
      if (t.blockSize < 64 || t.blockSize > 1024 || t.blockSize % 64 != 0) reject("block size of a task");
      if (t.gridPolicy < -1 || t.gridPolicy > 64) reject("grid policy of a task");
      if (t.entry.empty()) reject("entry point of a task");
    }
    if (!k->tasks_.empty() && k->samplesPerLane_ != 1) reject("samples per lane");
    if (k->taskBufferMiB_ < 1 || k->taskBufferMiB_ > 65536) reject("size of the intermediate buffer");
  } else {
    if (k->bytesPerResult_ != (k->prog_.f64 ? 8u : 4u)) reject("result width");
    checkInterpProgram(k->prog_, k->numFeatures_);
  }
  return k;
}

Kernel::~Kernel() { releaseDevice(); }

void Kernel::fillInfo(spnc_hip_info* info) const {
  std::memset(info, 0, sizeof(*info));
  std::snprintf(info->file_name, sizeof(info->file_name), "%s", fileName_.c_str());
  std::snprintf(info->kernel_name, sizeof(info->kernel_name), "%s", kernelName_.c_str());
  info->query_type = SPNC_HIP_QUERY_JOINT;
  info->target = SPNC_HIP_TARGET_HIP;
  info->batch_size = batchSize_;
  info->num_features = numFeatures_;
  info->bytes_per_feature = bytesPerFeature_;
  info->num_results = 1;
  info->bytes_per_result = bytesPerResult_;
  std::snprintf(info->dtype, sizeof(info->dtype), "%s", bytesPerResult_ == 8 ? "float64" : "float32");
  info->kernel_kind = kind_;
  info->input_alignment = inputAlign_;
  info->num_nodes = numNodes_;
  info->num_gaussian = stats_.gaussians;
  info->num_categorical = stats_.categoricals;
  info->num_histogram = stats_.histograms;
  info->num_product = stats_.products;
  info->num_sum = stats_.sums;
  info->max_fan_in = stats_.maxFanIn;
  info->sum_terms = stats_.sumTerms;
  info->product_adds = stats_.productAdds;
  info->flops_min = stats_.flopsMin;
  info->trans_min = stats_.transMin;
  info->flops_pairwise = stats_.flopsPairwise;
  info->trans_pairwise = stats_.transPairwise;
  info->fused_min = stats_.fusedMin;
  info->feature_is_float = featureType_ == unsigned(FeatureType::F32) || featureType_ == unsigned(FeatureType::F64);
  info->support_marginal = marginal_ ? 1u : 0u;
  info->num_tasks = tasks_.empty() ? 1u : unsigned(tasks_.size());
  info->task_rows = taskSlots_;
}

void Kernel::ensureDevice() {
  if (deviceReady_) return;
  try {
    prepareDevice();
  } catch (...) {
    releaseDevice();  // nothing half-built stays behind: the next call starts from scratch
    throw;
  }
  deviceReady_ = true;
}

// What the launcher needs to know about the device and the kernel's footprint on it. Allocates nothing.
void Kernel::queryDevice() {
  if (deviceKnown_) return;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count == 0) fatal("RUNTIME ERROR: no HIP device available");
  hipCheck(hipGetDevice(&device_), "hipGetDevice");
  hipDeviceProp_t prop;
  hipCheck(hipGetDeviceProperties(&prop, device_), "hipGetDeviceProperties");
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    fatal(std::string("RUNTIME ERROR: kernels are built for gfx950, device is ") + prop.gcnArchName);
  numCUs_ = prop.multiProcessorCount;
  if (kind_ == SPNC_HIP_KERNEL_INTERPRETER) {
    const size_t rb = prog_.f64 ? 8 : 4;
    // Value slots in LDS: as many as the program needs, capped so that two blocks fit a CU.
    int ldsPerCU = 0;
    hipCheck(hipDeviceGetAttribute(&ldsPerCU, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, device_), "LDS size query");
    // The kernel's own static LDS (the float64 log2 flavour keeps 4.7 KiB of exp2/log2 tables there) comes out of
    // the same memory: without it in the sum a program of 40 slots would leave room for one block per CU, not two.
    size_t maxBlock = 0, staticLds = 0;
    hipCheck(interpreterMaxLds(prog_.f64, prog_.log2Domain, prog_.linear, prog_.featureMode, &maxBlock, &staticLds), "LDS limit query");
    size_t budget = std::min<size_t>(maxBlock, size_t(ldsPerCU) / 2);
    budget = budget > staticLds ? budget - staticLds : 0;
    uint32_t cap = uint32_t(budget / (INTERP_BLOCK * rb));
    if (prog_.ldsSlotLimit) cap = std::min(cap, prog_.ldsSlotLimit);
    if (prog_.numSlots <= cap) {
      ldsSlots_ = prog_.numSlots;
      interpMode_ = 0;
    } else if (prog_.shortSlots <= cap) {
      ldsSlots_ = prog_.shortSlots;  // long-lived values go to the spill tier, only flagged instructions see them
      interpMode_ = 1;
    } else {
      ldsSlots_ = cap;
      interpMode_ = 2;
    }
    ldsBytes_ = size_t(ldsSlots_) * INTERP_BLOCK * rb;
    int nb = 0;
    hipCheck(interpreterOccupancy(prog_.f64, prog_.log2Domain, prog_.linear, interpMode_, prog_.featureMode, ldsBytes_, &nb), "occupancy query");
    blocksPerCU_ = std::max(1, nb);
    if (gridPolicy_ > 0) blocksPerCU_ = std::min(blocksPerCU_, gridPolicy_);  // "hip-blocks-per-cu": fewer than fit
  }
  deviceKnown_ = true;
}

// The interpreter's constant operands as the device holds them: the instruction stream followed by 512 zero bytes
// (the kernel touches the cache lines that follow an instruction's weights and prefetches one head past the end),
// the table pool in the compute type, and four words per staged feature.
void Kernel::buildImages() {
  if (!codeImage_.empty()) return;
  codeImage_.assign(prog_.code.begin(), prog_.code.end());
  codeImage_.resize(prog_.code.size() + 128, 0u);
  const size_t rb = prog_.f64 ? 8 : 4;
  tableImage_.resize(prog_.tables.size() * rb);
  if (prog_.f64) {
    if (!prog_.tables.empty()) std::memcpy(tableImage_.data(), prog_.tables.data(), tableImage_.size());
  } else {
    for (size_t i = 0; i < prog_.tables.size(); ++i) {
      const float v = float(prog_.tables[i]);
      std::memcpy(tableImage_.data() + 4 * i, &v, 4);
    }
  }
  for (const auto& sf : prog_.staged) {
    stagedImage_.push_back(sf.column);
    stagedImage_.push_back(sf.valueSlot);
    stagedImage_.push_back(sf.indexSlot);
    stagedImage_.push_back(sf.tableLen);
  }
}

void Kernel::prepareDevice() {
  queryDevice();
  if (kind_ == SPNC_HIP_KERNEL_JIT) {
    hipCheck(hipModuleLoadData(&module_, codeObject_.data()), "hipModuleLoadData");
    hipCheck(hipModuleGetFunction(&function_, module_, entry_.c_str()), "hipModuleGetFunction");
    int nb = 0;
    hipCheck(hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&nb, function_, int(blockSize_), 0), "occupancy query");
    blocksPerCU_ = std::max(1, nb);
    for (Task& t : tasks_) {
      hipCheck(hipModuleGetFunction(&t.function, module_, t.entry.c_str()), "hipModuleGetFunction");
      hipCheck(hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&nb, t.function, int(t.blockSize), 0), "occupancy query");
      t.blocksPerCU = std::max(1, nb);
    }
    if (!tasks_.empty()) hipCheck(hipEventCreateWithFlags(&interDone_, hipEventDisableTiming), "hipEventCreate");
  } else {
    const size_t rb = prog_.f64 ? 8 : 4;
    buildImages();
    hipCheck(hipMalloc(&dCode_, codeImage_.size() * 4), "hipMalloc(program)");
    hipCheck(hipMemcpy(dCode_, codeImage_.data(), codeImage_.size() * 4, hipMemcpyHostToDevice), "program upload");
    if (!tableImage_.empty()) {
      hipCheck(hipMalloc(&dTables_, tableImage_.size()), "hipMalloc(tables)");
      hipCheck(hipMemcpy(dTables_, tableImage_.data(), tableImage_.size(), hipMemcpyHostToDevice), "table upload");
    }
    if (!stagedImage_.empty()) {
      hipCheck(hipMalloc(&dStaged_, stagedImage_.size() * 4), "hipMalloc(staged)");
      hipCheck(hipMemcpy(dStaged_, stagedImage_.data(), stagedImage_.size() * 4, hipMemcpyHostToDevice), "staged upload");
    }
    const size_t lanes = size_t(numCUs_) * blocksPerCU_ * INTERP_BLOCK;
    spillBytes_ = size_t(prog_.numSlots - ldsSlots_) * lanes * rb;
    if (spillBytes_) {
      hipCheck(hipMalloc(&dSpill_, spillBytes_), "hipMalloc(spill)");
      hipCheck(hipEventCreateWithFlags(&spillTurn_.done, hipEventDisableTiming), "hipEventCreate");
    }
  }
}

void Kernel::releaseDevice() {
  for (auto& s : stage_) {
    if (s.stream) (void)hipStreamSynchronize(s.stream);
    if (s.hIn) (void)hipHostFree(s.hIn);
    if (s.hOut) (void)hipHostFree(s.hOut);
    if (s.dIn) (void)hipFree(s.dIn);
    if (s.dOut) (void)hipFree(s.dOut);
    if (s.stream) (void)hipStreamDestroy(s.stream);
    s = Stage();
  }
  stageRows_ = 0;
  if (kernelDone_) (void)hipEventDestroy(kernelDone_);
  kernelDone_ = nullptr;
  if (dCode_) (void)hipFree(dCode_);
  if (dTables_) (void)hipFree(dTables_);
  if (dStaged_) (void)hipFree(dStaged_);
  if (dSpill_) (void)hipFree(dSpill_);
  dCode_ = nullptr;
  dTables_ = nullptr;
  dStaged_ = nullptr;
  dSpill_ = nullptr;
  spillTurn_.reset();
  if (dInter_) (void)hipFree(dInter_);
  dInter_ = nullptr;
  interRows_ = 0;
  interUsed_ = false;
  if (interDone_) (void)hipEventDestroy(interDone_);
  interDone_ = nullptr;
  if (module_) (void)hipModuleUnload(module_);
  module_ = nullptr;
  function_ = nullptr;
  for (Task& t : tasks_) t.function = nullptr;
  deviceReady_ = false;
}

void Kernel::launch(size_t n, const void* dIn, void* dOut, hipStream_t stream) {
  if (n == 0) return;
  if (reinterpret_cast<uintptr_t>(dIn) % inputAlign_ != 0)
    fatal("RUNTIME ERROR: input pointer must be aligned to " + std::to_string(inputAlign_) + " bytes");
  if (reinterpret_cast<uintptr_t>(dOut) % bytesPerResult_ != 0) fatal("RUNTIME ERROR: output pointer is misaligned");
  if (kind_ == SPNC_HIP_KERNEL_JIT && !tasks_.empty()) {
    // The tasks one after the other on the caller's stream, over as many rows at a time as the intermediate buffer
    // ("hip-task-buffer-mib", 1 GiB unless asked otherwise) holds: a multiple of 1024 rows, which keeps every chunk's input as aligned as the first.
    const size_t rowBytes = size_t(numFeatures_) * bytesPerFeature_;
    size_t chunk = n;
    if (taskSlots_) {
      const size_t most = std::max<size_t>(1024, (size_t(taskBufferMiB_) << 20) / (size_t(taskSlots_) * bytesPerResult_) / 1024 * 1024);
      chunk = std::min(n, most);
      if (interUsed_) hipCheck(hipStreamWaitEvent(stream, interDone_, 0), "hipStreamWaitEvent");
      if (chunk > interRows_) {
        if (dInter_) hipCheck(hipFree(dInter_), "hipFree(intermediate values)");  // waits for the device to finish with it
        dInter_ = nullptr;
        interRows_ = 0;
        hipCheck(hipMalloc(&dInter_, size_t(taskSlots_) * chunk * bytesPerResult_), "hipMalloc(intermediate values)");
        interRows_ = chunk;
      }
    }
    for (size_t off = 0; off < n; off += chunk) {
      const size_t rows = std::min(chunk, n - off);
      const void* in = static_cast<const char*>(dIn) + off * rowBytes;
      void* out = static_cast<char*>(dOut) + off * bytesPerResult_;
      unsigned long long n64 = rows;
      for (const Task& t : tasks_) {
        const size_t tiles = (rows + t.blockSize - 1) / t.blockSize;
        size_t cap = size_t(numCUs_) * t.blocksPerCU;
        if (t.gridPolicy < 0) cap = tiles;
        else if (t.gridPolicy > 0) cap = size_t(numCUs_) * t.gridPolicy;
        const unsigned grid = unsigned(std::min<size_t>(std::min<size_t>(tiles, cap), 0x7fffffffu));
        void* args[] = {(void*)&in, (void*)&out, (void*)&n64, (void*)&dInter_, (void*)&dInter_};
        hipCheck(hipModuleLaunchKernel(t.function, grid, 1, 1, t.blockSize, 1, 1, 0, stream, args, nullptr), "kernel launch");
      }
    }
    if (taskSlots_) {
      hipCheck(hipEventRecord(interDone_, stream), "hipEventRecord");
      interUsed_ = true;
    }
  } else if (kind_ == SPNC_HIP_KERNEL_JIT) {
    const size_t tile = size_t(blockSize_) * samplesPerLane_;
    const size_t tiles = (n + tile - 1) / tile;
    size_t cap = size_t(numCUs_) * blocksPerCU_;
    if (gridPolicy_ < 0) cap = tiles;
    else if (gridPolicy_ > 0) cap = size_t(numCUs_) * gridPolicy_;
    const unsigned grid = unsigned(std::min<size_t>(std::min<size_t>(tiles, cap), 0x7fffffffu));
    unsigned long long n64 = n;
    void* args[] = {(void*)&dIn, (void*)&dOut, (void*)&n64};
    hipCheck(hipModuleLaunchKernel(function_, grid, 1, 1, blockSize_, 1, 1, 0, stream, args, nullptr), "kernel launch");
  } else {
    // Every launch of this handle uses the one spill buffer: launches on different streams take turns.
    const bool ordered = dSpill_ && !capturing(stream);
    if (ordered) spillTurn_.wait(stream);
    launchProgram(n, dIn, dOut, dCode_, dTables_, dStaged_, dSpill_, size_t(numCUs_) * blocksPerCU_, stream);
    if (ordered) spillTurn_.record(stream);
  }
}

void Turn::wait(hipStream_t stream) {
  if (used && stream != last) hipCheck(hipStreamWaitEvent(stream, done, 0), "hipStreamWaitEvent");
}

void Turn::record(hipStream_t stream) {
  if (!done) hipCheck(hipEventCreateWithFlags(&done, hipEventDisableTiming), "hipEventCreate");
  hipCheck(hipEventRecord(done, stream), "hipEventRecord");
  last = stream;
  used = true;
}

void Turn::reset() {
  if (done) (void)hipEventDestroy(done);
  done = nullptr;
  last = nullptr;
  used = false;
}

void Kernel::launchProgram(size_t n, const void* dIn, void* dOut, const uint32_t* code, const void* tables, const uint32_t* staged,
                           void* spill, size_t maxBlocks, hipStream_t stream) {
  const size_t tiles = (n + INTERP_BLOCK - 1) / INTERP_BLOCK;
  const unsigned grid = unsigned(std::min<size_t>(tiles, maxBlocks));
  InterpLaunch a;
  a.code = code;
  a.in = dIn;
  a.out = dOut;
  a.n = n;
  a.tables = tables;
  a.spill = spill;
  a.staged = staged;
  a.numStaged = uint32_t(prog_.staged.size());
  a.numFeatures = numFeatures_;
  a.featureType = featureType_;
  a.featureMode = prog_.featureMode;
  a.ldsSlots = ldsSlots_;
  a.spillSlots = prog_.numSlots - ldsSlots_;
  a.marginal = marginal_ ? 1u : 0u;
  a.mathTables = prog_.mathTables;
  hipCheck(launchInterpreter(a, prog_.f64, prog_.log2Domain, prog_.linear, interpMode_, grid, ldsBytes_, stream), "interpreter launch");
}

void Kernel::executeDevice(size_t n, const void* dIn, void* dOut, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(mu_);
  ensureDevice();
  launch(n, dIn, dOut, stream);
}

namespace {
std::mutex g_scratchMutex;
uint64_t g_scratchOwner[64] = {};   // per device: id of the kernel whose program the scratch array holds (0 = none)
Turn g_scratchTurn[64];             // per device: calls on different streams take turns on the array
std::atomic<uint64_t> g_nextKernelId{1};
size_t roundUp256(size_t v) { return (v + 255) / 256 * 256; }
}  // namespace

// The launch of executeDevice() for interpreter kernels with every device buffer the kernel needs besides the
// caller's input and output carved out of the library's fixed scratch array: program, tables, staged-feature
// descriptors, then the spill tier, as many blocks' worth as fit (the grid shrinks to that). Calls no allocator.
void Kernel::executeDeviceStatic(size_t n, const void* dIn, void* dOut, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(mu_);
  if (kind_ != SPNC_HIP_KERNEL_INTERPRETER)
    fatal("RUNTIME ERROR: the allocation-free entry point runs interpreter kernels (compile with hip-kernel=interpreter); "
          "a straight-line kernel has no scratch memory, but loading its code object allocates");
  queryDevice();
  if (n == 0) return;
  if (reinterpret_cast<uintptr_t>(dIn) % inputAlign_ != 0)
    fatal("RUNTIME ERROR: input pointer must be aligned to " + std::to_string(inputAlign_) + " bytes");
  if (reinterpret_cast<uintptr_t>(dOut) % bytesPerResult_ != 0) fatal("RUNTIME ERROR: output pointer is misaligned");
  buildImages();
  if (!kernelId_) kernelId_ = g_nextKernelId.fetch_add(1);
  void* base = nullptr;
  size_t capacity = 0;
  int dev = -1;
  hipCheck(interpreterScratch(&base, &capacity, &dev), "hipGetSymbolAddress(scratch)");
  if (dev != device_)
    fatal("RUNTIME ERROR: the kernel was set up on device " + std::to_string(device_) + ", the current device is " + std::to_string(dev));
  const size_t rb = prog_.f64 ? 8 : 4;
  const size_t codeAt = 0, tablesAt = roundUp256(codeImage_.size() * 4), stagedAt = tablesAt + roundUp256(tableImage_.size()),
               spillAt = stagedAt + roundUp256(stagedImage_.size() * 4);
  const size_t spillPerBlock = size_t(prog_.numSlots - ldsSlots_) * INTERP_BLOCK * rb;
  if (spillAt + spillPerBlock > capacity)
    fatal("RUNTIME ERROR: the program needs " + std::to_string(spillAt + spillPerBlock) + " bytes of scratch memory (program, tables and one "
          "block's spilled values), the allocation-free entry point has " + std::to_string(capacity) + "; use spnc_hip_execute_device");
  size_t maxBlocks = size_t(numCUs_) * blocksPerCU_;
  if (spillPerBlock) maxBlocks = std::min(maxBlocks, (capacity - spillAt) / spillPerBlock);
  char* p = static_cast<char*>(base);
  // The array is shared by every kernel handle, thread and stream of the process on this device: the lock covers the
  // whole enqueue, and a call on another stream than the previous one waits for that one's kernel first (its program
  // and spilled values are still in use until then). The event was created when the array's address was resolved.
  std::lock_guard<std::mutex> scratchLock(g_scratchMutex);
  Turn& turn = g_scratchTurn[dev];
  const bool ordered = !capturing(stream);
  if (ordered) turn.wait(stream);
  if (g_scratchOwner[dev] != kernelId_) {
    g_scratchOwner[dev] = 0;  // stays "nobody's" if an upload fails half way
    hipCheck(hipMemcpyAsync(p + codeAt, codeImage_.data(), codeImage_.size() * 4, hipMemcpyHostToDevice, stream), "program upload");
    if (!tableImage_.empty())
      hipCheck(hipMemcpyAsync(p + tablesAt, tableImage_.data(), tableImage_.size(), hipMemcpyHostToDevice, stream), "table upload");
    if (!stagedImage_.empty())
      hipCheck(hipMemcpyAsync(p + stagedAt, stagedImage_.data(), stagedImage_.size() * 4, hipMemcpyHostToDevice, stream), "staged upload");
    g_scratchOwner[dev] = kernelId_;
  }
  launchProgram(n, dIn, dOut, reinterpret_cast<const uint32_t*>(p + codeAt), tableImage_.empty() ? nullptr : p + tablesAt,
                stagedImage_.empty() ? nullptr : reinterpret_cast<const uint32_t*>(p + stagedAt), spillPerBlock ? p + spillAt : nullptr,
                maxBlocks, stream);
  if (ordered) {
    turn.done = static_cast<hipEvent_t>(interpreterScratchEvent(dev));
    turn.record(stream);
  }
}

void Kernel::ensureStaging(size_t rows) {
  if (rows <= stageRows_) return;
  // The old buffers go first and the row count with them, so that a failed allocation below leaves
  // "no staging buffers" behind, never a count that promises more than the pointers hold.
  stageRows_ = 0;
  for (auto& s : stage_) {
    if (s.hIn) (void)hipHostFree(s.hIn);
    if (s.hOut) (void)hipHostFree(s.hOut);
    if (s.dIn) (void)hipFree(s.dIn);
    if (s.dOut) (void)hipFree(s.dOut);
    s.hIn = s.hOut = s.dIn = s.dOut = nullptr;
  }
  const size_t inBytes = rows * numFeatures_ * bytesPerFeature_, outBytes = rows * bytesPerResult_;
  for (auto& s : stage_) {
    hipCheck(hipHostMalloc(&s.hIn, inBytes, hipHostMallocDefault), "hipHostMalloc(input staging)");
    hipCheck(hipHostMalloc(&s.hOut, outBytes, hipHostMallocDefault), "hipHostMalloc(output staging)");
    hipCheck(hipMalloc(&s.dIn, inBytes), "hipMalloc(input)");
    hipCheck(hipMalloc(&s.dOut, outBytes), "hipMalloc(output)");
    if (!s.stream) hipCheck(hipStreamCreate(&s.stream), "hipStreamCreate");
  }
  if (!kernelDone_) hipCheck(hipEventCreateWithFlags(&kernelDone_, hipEventDisableTiming), "hipEventCreate");
  stageRows_ = rows;
}

void Kernel::execute(size_t n, const void* in, void* out) {
  std::lock_guard<std::mutex> lock(mu_);
  ensureDevice();
  if (n == 0) return;
  if (!in || !out) fatal("RUNTIME ERROR: null input or output buffer");
  const size_t rowBytes = size_t(numFeatures_) * bytesPerFeature_;
  // Chunks of about 32 MiB of input, two in flight: copy-in, kernel and copy-out of one
  // chunk overlap the host-side staging of the next.
  size_t chunk = std::max<size_t>(4096, (size_t(32) << 20) / std::max<size_t>(1, rowBytes));
  chunk = std::min(chunk, n);
  ensureStaging(chunk);
  // Buffers the caller has pinned are copied from / to directly; pageable ones go through the pinned staging
  // buffers, filled by a few threads.
  const bool pinnedIn = isPinnedHost(in, n * rowBytes), pinnedOut = isPinnedHost(out, n * bytesPerResult_);
  CopyCrew& crew = CopyCrew::instance();
  auto drain = [&](Stage& s) {
    if (!s.pendingRows) return;
    hipCheck(hipStreamSynchronize(s.stream), "hipStreamSynchronize");
    if (!pinnedOut) std::memcpy(static_cast<char*>(out) + s.pendingOffset * bytesPerResult_, s.hOut, s.pendingRows * bytesPerResult_);
    s.pendingRows = 0;
  };
  size_t done = 0;
  unsigned turn = 0;
  try {
    while (done < n) {
      Stage& s = stage_[turn & 1];
      drain(s);
      const size_t rows = std::min(chunk, n - done);
      const char* src = static_cast<const char*>(in) + done * rowBytes;
      if (!pinnedIn) {
        crew.copy(s.hIn, src, rows * rowBytes);
        src = static_cast<const char*>(s.hIn);
      }
      hipCheck(hipMemcpyAsync(s.dIn, src, rows * rowBytes, hipMemcpyHostToDevice, s.stream), "input copy");
      // Kernels of successive chunks run one after the other (they share the spill buffer);
      // only the copies overlap them.
      if (turn) hipCheck(hipStreamWaitEvent(s.stream, kernelDone_, 0), "hipStreamWaitEvent");
      launch(rows, s.dIn, s.dOut, s.stream);
      hipCheck(hipEventRecord(kernelDone_, s.stream), "hipEventRecord");
      void* dst = pinnedOut ? static_cast<void*>(static_cast<char*>(out) + done * bytesPerResult_) : s.hOut;
      hipCheck(hipMemcpyAsync(dst, s.dOut, rows * bytesPerResult_, hipMemcpyDeviceToHost, s.stream), "output copy");
      s.pendingRows = rows;
      s.pendingOffset = done;
      done += rows;
      ++turn;
    }
    drain(stage_[0]);
    drain(stage_[1]);
  } catch (...) {
    for (auto& s : stage_) {
      if (s.stream) (void)hipStreamSynchronize(s.stream);
      s.pendingRows = 0;
    }
    throw;
  }
}

}  // namespace spnc_hip
