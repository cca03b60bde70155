"""The kernel body that the generator emits for packed rows, run on the CPU: its text is cut out of a generated kernel,
the assembler statements are rewritten as the C they stand for (bit fields, shift-and-or, 16-bit
multiply-adds), the result is compiled for the host and compared with the oracle. This checks the generator's logic (tables,
offsets, polynomials, range test) without a GPU; what only the hardware can show (LDS behaviour, the order of memory
operations) is left to the GPU tests."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from conftest import compile_spn, oracle_model
from oracle import evaluate as ev

CLANG = "/opt/rocm/llvm/bin/clang++"


def _operand(text, names):
    m = re.fullmatch(r"%(\d+)", text)
    return names[int(m.group(1))] if m else text


def _select(expr, sel):
    if sel is None or sel == "DWORD":
        return f"({expr})"
    return f"((({expr}) >> {8 * int(sel[-1])}) & 255u)"


def _instruction(line, names):
    """One GCN instruction as a C statement over the variables bound to the statement's operands."""
    line = line.strip()
    if not line or line.startswith("s_nop"):
        return ""
    op, rest = line.split(None, 1)
    mods = dict(re.findall(r"(dst_sel|dst_unused|src0_sel|src1_sel|row_newbcast):(\w+)", rest))
    args = [a.strip() for a in re.sub(r"\s+(dst_sel|dst_unused|src0_sel|src1_sel|row_newbcast|row_mask|bank_mask):\w+", "", rest).split(",")]
    v = [_operand(a, names) for a in args]
    if op == "v_fmac_f64_dpp":
        # the first source comes from lane row_newbcast of the register's row: the host build holds such a register
        # (sixteen constants, one per lane of a row) as a pointer to the sixteen values
        return f"{v[0]} = __builtin_fma({v[1]}[{int(mods['row_newbcast'])}], {v[2]}, {v[0]});"
    if op == "v_max_f64":
        return f"{v[0]} = __builtin_fmax({v[1]}, {v[2]});"
    if op == "v_ashrrev_i32":
        return f"{v[0]} = (unsigned)((int)({v[2]}) >> {v[1]});"
    if op == "v_fma_f64":
        return f"{v[0]} = __builtin_fma({v[1]}, {v[2]}, {v[3]});"
    if op == "v_lshl_add_u32":
        return f"{v[0]} = (({v[1]}) << {v[2]}) + ({v[3]});"
    if op == "v_min_u32":
        return f"{v[0]} = ({v[1]}) < ({v[2]}) ? ({v[1]}) : ({v[2]});"
    if op == "v_lshl_or_b32":
        return f"{v[0]} = (({v[1]}) << {v[2]}) | ({v[3]});"
    if op == "v_and_b32":
        return f"{v[0]} = ({v[1]}) & ({v[2]});"
    if op == "v_lshrrev_b32":
        return f"{v[0]} = ({v[2]}) >> {v[1]};"
    if op == "v_mad_u32_u16":   # 16-bit factors, 32-bit sum
        return f"{v[0]} = (({v[1]}) & 0xffffu) * (({v[2]}) & 0xffffu) + ({v[3]});"
    if op == "v_add3_u32":
        return f"{v[0]} = {v[1]} + {v[2]} + {v[3]};"
    if op == "v_add_u32":
        return f"{v[0]} = {v[1]} + {v[2]};"
    if op == "v_bfe_u32":
        return f"{v[0]} = (({v[1]}) >> {v[2]}) & ((1u << {v[3]}) - 1u);"
    m = re.fullmatch(r"v_cvt_f32_ubyte(\d)", op)
    if m:
        return f"{v[0]} = (float)((({v[1]}) >> {8 * int(m.group(1))}) & 255u);"
    raise AssertionError("instruction the host build does not know: " + line)


def _statement(m):
    """asm [volatile] ("text" : outputs : inputs [: clobbers]);  ->  C"""
    text, tail = m.group("text"), m.group("tail")
    text = "".join(re.findall(r'"((?:[^"\\]|\\.)*)"', text)).replace("\\n", "\n").replace("\\t", " ")
    groups = [g.strip() for g in tail.split(":")] if tail else []
    names = []
    for g in groups[:2]:
        names += re.findall(r'"[^"]*"\s*\(((?:[^()]|\([^()]*\))*)\)', g)
    return " ".join(_instruction(line, names) for line in text.split("\n"))


ASM = re.compile(r'asm(?:\s+volatile)?\s*\((?P<text>(?:\s*"(?:[^"\\]|\\.)*")+)\s*(?::(?P<tail>(?:[^;()]|\((?:[^()]|\([^()]*\))*\))*))?\)\s*;')


def lane_constants_on_the_host(body):
    """Registers that hold sixteen constants, one per lane of a row (read through v_fmac_f64_dpp), become pointers to the
    sixteen values in the constant table."""
    return re.sub(r"const real_t (kv\d+) = spn_kpool\[(\d+)u \+ \(threadIdx\.x & 15u\)\];", r"const real_t* \1 = spn_kpool + \2;", body)


def host_library(source, saturation, tmp_path, tag):
    body = source[:source.index('extern "C" __global__')]
    body = ASM.sub(_statement, body)
    body = body.replace("__builtin_amdgcn_sched_barrier(0);", "")
    body = re.sub(r"reinterpret_cast<const __attribute__\(\(address_space\(3\)\)\) (\w+)\*>\(([^;]*)\);",
                  r"reinterpret_cast<const \1*>(reinterpret_cast<const char*>(tab) + (\2));", body)
    body = body.replace("__device__ __attribute__((aligned(32))) const real_t spn_tables", "alignas(32) const real_t spn_tables")
    assert "asm" not in body and "address_space" not in body
    templated = "Mid&& spn_mid" in body
    text = """#include <cmath>
#define __device__
#define __forceinline__ inline
#define __restrict__
#define SPN_EXP2_TABLE spn_exp2_table   // float64 kernels: the routines read their tables where they are, not from LDS
#define SPN_LOG2_TABLE spn_log2_table
#define SPN_POLY spn_poly
static inline float __builtin_amdgcn_exp2f(float x) { return exp2f(x); }
static inline float __builtin_amdgcn_logf(float x) { return log2f(x); }
""" + body + """
extern "C" void eval_rows(const int* in, real_t* out, long n) {
  for (long i = 0; i < n; ++i) {
    unsigned R[SPN_F / 4];
    for (int c = 0; c < SPN_F / 4; ++c)
      R[c] = spn_pack4((unsigned)in[i * SPN_F + 4 * c], (unsigned)in[i * SPN_F + 4 * c + 1], (unsigned)in[i * SPN_F + 4 * c + 2], (unsigned)in[i * SPN_F + 4 * c + 3]);
    out[i] = spn_eval(R, spn_tables, 0u%s);
  }
}
""" % (", [] {}" if templated else "")
    # the value rows are saturated at when they are packed: written into the instruction when it is small enough for that
    assert ("v_min_u32 %%0, %d, %%5" % saturation if saturation <= 64 else "\"s\"(%du)" % saturation) in source
    cpp, so = tmp_path / (tag + ".cpp"), tmp_path / (tag + ".so")
    cpp.write_text(text)
    subprocess.check_call([CLANG, "-O1", "-shared", "-fPIC", "-std=c++17", "-ffp-contract=fast", "-w", "-o", str(so), str(cpp)])
    return ctypes.CDLL(str(so))


def run_host(lib, X, dtype):
    X = np.ascontiguousarray(X, dtype=np.int32)
    out = np.zeros(len(X), dtype)
    lib.eval_rows(X.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(len(X)))
    return out


needs_clang = pytest.mark.skipif(not os.path.isfile(CLANG), reason="host build of the generated code needs the ROCm clang")


@needs_clang
@pytest.mark.parametrize("opts", [{}, {"hip-one-hot-max-domain": 3}, {"hip-one-hot-max-domain": 5, "hip-hoist-feature-values": "false"},
                                  {"hip-one-hot-max-domain": 0, "hip-fused-batch": 0}, {"hip-joint-tables": "false", "hip-prefetch-rows": "false"},
                                  {"hip-table-budget-kib": 24}, {"hip-compute-type": "float64"}, {"hip-table-planes": "false"},
                                  {"hip-table-planes": "false", "hip-compute-type": "float64"}],
                         ids=["default", "quadratic", "one-hot-5", "all-lds", "no-joint", "small-budget", "float64", "side-by-side", "side-by-side-float64"])
@pytest.mark.parametrize("cfg", ["c3", "c3_deep"])
def test_packed_rows_body_on_the_host(native, tmp_path, cfg, opts):
    from spnc import synthetic as syn
    c = syn.CONFIGS[cfg]
    spn, X = c["spn"](), c["inputs"](1500)
    X[5, :] = 77
    X[6, 3] = 9
    X[7, 97] = 2 ** 31 - 1
    X[8, 0] = 255
    X[9, 1] = 256
    X[10, 2] = -1
    k = compile_spn(native, spn, c["dtype"], marginal=False, **dict(opts, **{"hip-packed-rows": "true"}))
    src = k.source()
    os.remove(k.fileName())
    assert "unsigned PK0 = R[0]" in src
    longest = max(d for _, d in syn.c3_domains())
    f64 = opts.get("hip-compute-type") == "float64"
    got = run_host(host_library(src, longest, tmp_path, "c3"), X, np.float64 if f64 else np.float32)
    ref = ev.ll_closed_f64(oracle_model(spn, c["dtype"]), X, marginal=False)
    assert np.array_equal(np.isneginf(got), np.isneginf(ref)) and all(np.isneginf(got[r]) for r in range(5, 11))
    fin = np.isfinite(ref)
    assert np.abs(got[fin] - ref[fin]).max() <= (1e-10 if f64 else 1e-4)


@needs_clang
@pytest.mark.parametrize("planes", [False, True], ids=["side-by-side", "planes"])
def test_packed_rows_body_with_clamped_bytes_on_the_host(native, tmp_path, planes):
    """A feature with 120 categories makes the padding for unclamped bytes too large when the siblings' values lie side
    by side: the bytes are clamped in place. With the siblings' tables in planes the padding stays small and no byte is
    clamped."""
    from spnc.structure import Categorical, Product, Sum
    rng = np.random.default_rng(17)
    domains = [120] + [int(d) for d in rng.integers(2, 7, 31)]
    products = [Product(children=[Categorical(p=[float(v) for v in rng.dirichlet(np.ones(d))], scope=f) for f, d in enumerate(domains)])
                for _ in range(9)]
    spn = Sum([float(v) for v in rng.dirichlet(np.ones(9))], products)
    X = np.column_stack([rng.integers(0, d, 2000) for d in domains]).astype(np.int32)
    X[3, 0], X[4, 0], X[5, 0], X[6, 0], X[7, 0], X[8, 5], X[9, 31] = 120, 127, 128, 255, 256, domains[5], 2 ** 31 - 1
    k = compile_spn(native, spn, "int32", marginal=False, **{"hip-packed-rows": "true", "hip-table-planes": "true" if planes else "false"})
    src = k.source()
    os.remove(k.fileName())
    # the clamp of the long feature's byte, its limit in a register
    assert ("PK0 = spn_q;" not in src) if planes else ("v_min_u32 %1, %3, %1" in src and "PK0 = spn_q;" in src)
    got = run_host(host_library(src, 120, tmp_path, "long"), X, np.float32)
    ref = ev.ll_closed_f64(oracle_model(spn, "int32"), X, marginal=False)
    assert np.array_equal(np.isneginf(got), np.isneginf(ref)) and all(np.isneginf(got[r]) for r in range(3, 10))
    fin = np.isfinite(ref)
    assert np.abs(got[fin] - ref[fin]).max() <= 1e-4
