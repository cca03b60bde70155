"""Straight-line C restatement of the reference's vectorised CPU kernel (test infrastructure).

Used only as the timed CPU baseline of ``bench.py`` and in tests; never by the product path.

What it restates: the reference compiles each SPN into one function whose body is the
straight-line log-space arithmetic of the whole graph, evaluated for a vector of samples at a
time (mlir/lib/Conversion/LoSPNtoCPU/Vectorization/VectorizeStructurePatterns.cpp:325-423,
VectorizeNodePatterns.cpp:247-270,372-440,518-610), built with ``clang -O3 -shared``
(compiler/src/pipeline/steps/linker/ClangKernelLinking.cpp:17-32) and driven over chunks of
``batchSize`` samples under ``#pragma omp parallel for`` (runtime/src/Executable.cpp:83-103).
Here the same operation order (balanced product / weighted-sum trees of
mlir/lib/Conversion/HiSPNtoLoSPN/NodePatterns.cpp:17-88, ``a + log1p(exp(b - a))``, constants
rounded once from double) is printed as C, the sample loop is marked ``omp simd`` so that the
host compiler vectorises it with glibc's libmvec, and the chunk loop is the same.
"""
import math
import os
import subprocess
import tempfile

import numpy as np

from . import spn_model as sm
from .evaluate import histogram_table

_CTYPE = {"float32": "float", "float64": "double", "int32": "unsigned int", "uint32": "unsigned int", "uint8": "unsigned char",
          "int8": "unsigned char", "int16": "unsigned short", "uint16": "unsigned short", "int64": "unsigned long long",
          "uint64": "unsigned long long"}


def _lit(v):
    if math.isinf(v):
        return "(-INFINITY)" if v < 0 else "INFINITY"
    return float(np.float32(v)).hex() + "f"


def _balanced(items, combine):
    if len(items) == 1:
        return items[0]
    if len(items) == 2:
        return combine(items[0], items[1])
    pivot = (len(items) + 1) // 2
    return combine(_balanced(items[:pivot], combine), _balanced(items[pivot:], combine))


def generate(model, marginal, batch_size=4096):
    col = model.column_of()
    F = model.num_features
    ctype = _CTYPE[model.feature_type]
    is_float = model.feature_type.startswith("float")
    lines, tables = [], []
    counter = [0]

    def tmp():
        counter[0] += 1
        return "t%d" % counter[0]

    def logadd(a, b):
        r = tmp()
        lines.append(f"      const float {r} = logadd({a}, {b});")
        return r

    def add(a, b):
        r = tmp()
        lines.append(f"      const float {r} = {a} + {b};")
        return r

    for n in sm.reachable_topo(model):
        v = "v%d" % n.id
        x = "x%d" % col[n.scope] if n.kind in (sm.GAUSSIAN, sm.CATEGORICAL, sm.HISTOGRAM) else None
        if n.kind == sm.GAUSSIAN:
            coef = -math.log(n.stddev) + -0.5 * math.log(2 * math.pi)
            den = -(1.0 / (2.0 * n.stddev * n.stddev))
            d = tmp()
            lines.append(f"      const float {d} = (float){x} - {_lit(n.mean)};")
            e = f"{_lit(coef)} + ({d} * {d}) * {_lit(den)}"
            if marginal:
                e = f"({x} != {x}) ? 0.0f : ({e})"
            lines.append(f"      const float {v} = {e};")
        elif n.kind in (sm.CATEGORICAL, sm.HISTOGRAM):
            p = np.asarray(n.probabilities, dtype=np.float64) if n.kind == sm.CATEGORICAL else histogram_table(n)
            with np.errstate(divide="ignore"):
                vals = [float(np.log(q)) if q > 0 else -math.inf for q in p]
            name = "tab%d" % len(tables)
            tables.append(f"static const float {name}[{len(vals) + 1}] = {{{', '.join(_lit(q) for q in vals)}, (-INFINITY)}};")
            L = len(vals)
            if is_float:
                idx = f"(({x} >= 0 && {x} < {L}) ? (unsigned){x} : {L}u)"
            else:
                idx = f"(({x} < {L}u) ? (unsigned){x} : {L}u)"
            e = f"{name}[{idx}]"
            if marginal and is_float:
                e = f"({x} != {x}) ? 0.0f : {e}"
            lines.append(f"      const float {v} = {e};")
        elif n.kind == sm.PRODUCT:
            r = _balanced(["v%d" % c for c in n.children], add)
            lines.append(f"      const float {v} = {r};")
        elif n.kind == sm.SUM:
            terms = []
            for c, w in zip(n.children, n.weights):
                t = tmp()
                lines.append(f"      const float {t} = v{c} + {_lit(math.log(w) if w > 0 else -math.inf)};")
                terms.append(t)
            r = _balanced(terms, logadd)
            lines.append(f"      const float {v} = {r};")
    loads = "\n".join(f"      const {ctype} x{c} = in[i * {F} + {c}];" for c in sorted(set(col.values())))
    src = f"""// generated CPU baseline kernel: reference operation order, f32 log-space
#include <math.h>
#include <stddef.h>
#include <omp.h>
#pragma omp declare simd notinbranch
extern float expf(float);
#pragma omp declare simd notinbranch
extern float log1pf(float);
{chr(10).join(tables)}
#pragma omp declare simd notinbranch
static inline float logadd(float x, float y) {{
  const float a = x > y ? x : y;
  const float b = x > y ? y : x;
  return a + log1pf(expf(b - a));
}}
static void spn_chunk(const {ctype}* restrict in, float* restrict out, size_t n) {{
#pragma omp simd
  for (size_t i = 0; i < n; ++i) {{
{loads}
{chr(10).join(lines)}
      out[i] = v{model.root};
  }}
}}
// Threads the chunk loop runs on (what a caller reports as "cores"), and a way to time one thread.
int spn_cpu_threads(void) {{ return omp_get_max_threads(); }}
void spn_cpu_set_threads(int n) {{ omp_set_num_threads(n); }}
// Chunks of batch_size samples in parallel, like Executable::executeBatch.
void spn_cpu_execute(const {ctype}* in, float* out, size_t n) {{
  const size_t bs = {batch_size};
  const long chunks = (long)((n + bs - 1) / bs);
#pragma omp parallel for schedule(static)
  for (long c = 0; c < chunks; ++c) {{
    const size_t lo = (size_t)c * bs, len = (lo + bs <= n) ? bs : n - lo;
    spn_chunk(in + lo * {F}, out + lo, len);
  }}
}}
"""
    return src


def build(model, marginal, workdir=None, batch_size=4096, opt="-O3"):
    """Compiles the generated kernel with the host compiler; returns (path of the .so, seconds)."""
    import time
    workdir = workdir or tempfile.mkdtemp(prefix="spn_cpu_")
    os.makedirs(workdir, exist_ok=True)
    c_path = os.path.join(workdir, "spn_cpu.c")
    so_path = os.path.join(workdir, "spn_cpu.so")
    with open(c_path, "w") as f:
        f.write(generate(model, marginal, batch_size))
    t0 = time.time()
    subprocess.run(["gcc", opt, "-march=native", "-fopenmp", "-fPIC", "-shared", "-fno-math-errno", "-o", so_path, c_path, "-lm"],
                   check=True)
    return so_path, time.time() - t0


def load(so_path, feature_dtype):
    import ctypes
    lib = ctypes.CDLL(so_path)
    lib.spn_cpu_execute.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    lib.spn_cpu_execute.restype = None

    lib.spn_cpu_threads.restype = ctypes.c_int
    lib.spn_cpu_set_threads.argtypes = [ctypes.c_int]
    lib.spn_cpu_set_threads.restype = None

    def run(X):
        X = np.ascontiguousarray(X, dtype=np.dtype(feature_dtype))
        out = np.empty(X.shape[0], dtype=np.float32)
        lib.spn_cpu_execute(X.ctypes.data, out.ctypes.data, X.shape[0])
        return out

    run.threads = lib.spn_cpu_threads          # OpenMP threads the next call will use
    run.set_threads = lib.spn_cpu_set_threads
    return run
