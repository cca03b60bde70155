"""Host layer through the C-ABI without a GPU: reader, validation, options, code generation, kernel files."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

import rawfile as rf
from conftest import GOLDEN, ROOT, compile_query, compile_spn, model_as_query, oracle_model, quiet

QUERIES = ["categorical-example", "gaussian-example", "mini-example", "categorical6", "gaussian10", "histogram4", "NIPS5", "NIPS10",
           "speaker_FADG0"]
MODELS = ["nltcs", "plants", "fashion_mnist"]


def test_library_exports_every_declared_symbol(native):
    header = open(os.path.join(ROOT, "include", "spnc_hip.h")).read()
    declared = re.findall(r"SPNC_HIP_API[^;(]*?\b(spnc_hip_\w+)\s*\(", header)
    assert len(declared) == 10
    lib = ctypes.CDLL(native.library_path())
    for name in declared:
        assert hasattr(lib, name), name


def test_info_struct_layout_matches_header(native, tmp_path):
    src = tmp_path / "sz.c"
    src.write_text('#include <stdio.h>\n#include "spnc_hip.h"\nint main(){printf("%zu %zu", sizeof(spnc_hip_info), '
                   '__builtin_offsetof(spnc_hip_info, flops_min));return 0;}\n')
    exe = tmp_path / "sz"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), "-o", str(exe), str(src)], check=True)
    size, off = map(int, subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split())
    assert size == ctypes.sizeof(native._Info)
    assert off == native._Info.flops_min.offset


@pytest.mark.parametrize("name", QUERIES)
def test_reference_query_files_compile(native, name):
    from oracle import spn_model as sm
    k = compile_query(native, os.path.join(GOLDEN, name + ".bin"))
    q = sm.load(os.path.join(GOLDEN, name + ".bin"))
    info = k.info()
    assert os.path.isfile(k.fileName())
    assert k.kernelName() == (q.model.name or "spn_kernel")
    assert k.numFeatures() == q.model.num_features and k.batchSize() == q.batch_size
    assert k.bytesPerFeature() == np.dtype(q.model.feature_type).itemsize
    assert (k.numResults(), k.bytesPerResult(), k.dataType(), k.target(), k.queryType()) == (1, 4, "float32", 3, 1)
    assert info["num_nodes"] <= len(q.model.nodes)
    os.remove(k.fileName())


@pytest.mark.parametrize("name", MODELS)
def test_raw_models_are_rejected_then_compile_as_queries(native, name, tmp_path):
    with pytest.raises(RuntimeError, match="Cannot compile raw models"):
        compile_query(native, os.path.join(GOLDEN, name + ".bin"))
    q = model_as_query(os.path.join(GOLDEN, name + ".bin"), "float64", str(tmp_path / "q.bin"))
    k = compile_query(native, q)
    info = k.info()
    assert info["kernel_kind"] == (2 if name == "fashion_mnist" else 1)  # the 47k-node model goes to the interpreter
    assert k.numFeatures() == {"nltcs": 16, "plants": 69, "fashion_mnist": 784}[name]
    os.remove(k.fileName())


def test_dedup_of_identical_leaves(native):
    from spnc.structure import Gaussian, Product, Sum
    a = Product(children=[Gaussian(0.0, 1.0, scope=0), Gaussian(1.0, 2.0, scope=1)])
    b = Product(children=[Gaussian(0.0, 1.0, scope=0), Gaussian(2.0, 2.0, scope=1)])  # same first leaf, other object
    k = compile_spn(native, Sum(weights=[0.5, 0.5], children=[a, b]), "float32")
    assert k.info()["num_nodes"] == 6 and k.info()["num_gaussian"] == 3
    os.remove(k.fileName())


def test_algorithmic_counts(native):
    from spnc import synthetic as syn
    k = compile_spn(native, syn.c1_spn(), "int32")
    i = k.info()
    assert (i["flops_min"], i["trans_min"], i["num_categorical"], i["product_adds"], i["fused_min"]) == (5, 0, 6, 5, 0)
    os.remove(k.fileName())
    k = compile_spn(native, syn.c2_spn(), "float32")
    i = k.info()
    # 1024 Gaussians * 4 + products (36 * 1 + 256 * 3) + 73 sums * 5k (k = 4); transcendentals 73 * (k + 1)
    assert (i["num_gaussian"], i["num_product"], i["num_sum"]) == (1024, 292, 73)
    assert (i["flops_min"], i["trans_min"]) == (4096 + 804 + 73 * 20, 73 * 5)
    assert (i["flops_pairwise"], i["trans_pairwise"]) == (4096 + 804 + 73 * 25, 73 * 6)
    # fused multiply-adds: one inside every Gaussian leaf, and the 256 products of four leaves fold their three adds
    assert i["fused_min"] == 1024 + 256 * 3 and i["fused_min"] < i["flops_min"]
    os.remove(k.fileName())


def test_option_handling(native):
    path = os.path.join(GOLDEN, "NIPS5.bin")
    with pytest.raises(RuntimeError, match="Unknown compile option bogus"):
        compile_query(native, path, bogus=1)
    with quiet(), pytest.raises(RuntimeError, match="Could not verify configuration constraints"):
        native.SPNCompiler().compileQuery(path, {"use-log-space": "true"})  # target is required
    with quiet(), pytest.raises(RuntimeError, match="only supports target 'HIP'"):
        native.SPNCompiler().compileQuery(path, {"target": "CUDA"})
    # options of the reference's CPU pipeline are accepted and ignored
    k = compile_query(native, path, **{"cpu-vectorize": "true", "vector-library": "LIBMVEC", "use-shuffle": "true", "optLevel": 2})
    os.remove(k.fileName())
    with pytest.raises(RuntimeError, match="Could not parse option value"):
        compile_query(native, path, **{"hip-kernel": "magic"})
    # maxTaskSize: a graph above the bound is cut into tasks, one kernel each
    k = compile_query(native, path, maxTaskSize=10)
    assert k.info()["kernel_kind"] == 1 and k.info()["num_tasks"] > 1 and k.info()["task_rows"] >= 1
    os.remove(k.fileName())
    k = compile_query(native, path, maxTaskSize=100000)
    assert k.info()["kernel_kind"] == 1 and k.info()["num_tasks"] == 1 and k.info()["task_rows"] == 0
    os.remove(k.fileName())
    with pytest.raises(RuntimeError, match="hip-interp-staged-features must be lds, spill or auto"):
        compile_query(native, path, **{"hip-kernel": "interpreter", "hip-interp-staged-features": "hbm"})
    with pytest.raises(RuntimeError, match="hip-joint-max-entries must be in"):
        compile_query(native, path, **{"hip-joint-max-entries": -3})


def test_graph_stats_file(native, tmp_path):
    """collect-graph-stats writes the reference's keys, counted on the binarised graph
    (mlir/lib/Dialect/LoSPN/Passes/LoSPNGraphStatsCollection.cpp:85-97)."""
    import json
    from spnc.structure import Histogram, Product
    keys = {"featureCount", "minDepth", "maxDepth", "averageDepth", "medianDepth", "innerCount", "leafCount", "sumCount", "productCount",
            "categoricalCount", "constantCount", "gaussianCount", "histogramCount"}
    out = tmp_path / "stats.json"
    stats_opts = {"collect-graph-stats": "true", "graph-stats-file": str(out)}

    def stats(kernel):
        os.remove(kernel.fileName())
        text = open(out).read()
        st = json.loads(text)
        assert keys <= set(st) and set(st) - keys == {"hip"}
        assert list(st) == sorted(st) and " " not in text      # the reference's JSON writer sorts keys and prints compactly
        return st

    # NIPS5 by hand: one sum over two products of five histograms = 13 nodes. Binarised: 1 add, 2 weight multiplies with 2
    # constants, 2 * 4 product multiplies; leaf depths below a product of five are 3,3,2,2,2 and the product's top
    # multiply sits at level 2 (add, weight multiply, product).
    st = stats(compile_query(native, os.path.join(GOLDEN, "NIPS5.bin"), **stats_opts))
    assert (st["featureCount"], st["sumCount"], st["productCount"], st["constantCount"], st["histogramCount"]) == (5, 1, 10, 2, 10)
    assert (st["innerCount"], st["leafCount"], st["gaussianCount"], st["categoricalCount"]) == (11, 12, 0, 0)
    assert (st["minDepth"], st["maxDepth"], st["averageDepth"], st["medianDepth"]) == (4, 5, 4.4, 4.5)
    assert st["hip"]["depthsExact"] is True and st["hip"]["mergedNodes"] == 13

    # The reference's own expectations: mlir/test/analysis/lospn/lospn-graph-stats-collection-sum.mlir:50-63 (a sum over five
    # categoricals, linear space, so the final log is the root) and ...-mul.mlir:34-48 (a product of two histograms).
    # (that sum mixes scopes, which the serializer of this package refuses, so its file is written field by field)
    probs = [[.35, .55, .1], [.25, .625, .125], [.5, .2, .3], [.6, .15, .25], [.8, .14, .06]]
    path = rf.write(str(tmp_path / "sum.bin"), nodes=[rf.cat(i + 1, i, p=p) for i, p in enumerate(probs)] +
                    [rf.wsum(0, [1, 2, 3, 4, 5], [.1, .1, .1, .4, .3])], scope=[0, 1, 2, 3, 4], feature_type="int32")
    st = stats(compile_query(native, path, **stats_opts, **{"use-log-space": "false"}))
    want = {"averageDepth": 4.4, "categoricalCount": 5, "constantCount": 5, "featureCount": 5, "gaussianCount": 0, "histogramCount": 0,
            "innerCount": 9, "leafCount": 10, "maxDepth": 5, "medianDepth": 4, "minDepth": 4, "productCount": 5, "sumCount": 4}
    assert {k_: st[k_] for k_ in want} == want
    hists = [Histogram([0., 1., 2.], [0.25, 0.75], [1, 1], scope=0), Histogram([0., 1., 2.], [0.45, 0.55], [1, 1], scope=1)]
    st = stats(compile_spn(native, Product(children=hists), "int32", **stats_opts, **{"use-log-space": "false"}))
    want = {"averageDepth": 2.0, "categoricalCount": 0, "constantCount": 0, "featureCount": 2, "gaussianCount": 0, "histogramCount": 2,
            "innerCount": 1, "leafCount": 2, "maxDepth": 2, "medianDepth": 1.5, "minDepth": 2, "productCount": 1, "sumCount": 0}
    assert {k_: st[k_] for k_ in want} == want
    assert '"averageDepth":2.0,' in open(out).read()
    # log space has no final log operation: every depth is one less
    st = stats(compile_spn(native, Product(children=hists), "int32", **stats_opts))
    assert (st["minDepth"], st["maxDepth"], st["averageDepth"]) == (1, 1, 1.0)

    # The region graph shares every node among 8 or 64 parents: 1e10 root-to-leaf paths, counted by recurrence.
    from spnc import synthetic as syn
    st = stats(compile_spn(native, syn.c4_spn(), "float32", **stats_opts))
    # 10 repetitions of: 16 leaf regions of 4 products of two leaves; 8 regions of 8 sums over 4 x 4 products; 7 regions of
    # 8 sums over 8 x 8 products; and the root sum over the 80 root-region sums.
    terms = 10 * (8 * 8 * 16 + 7 * 8 * 64) + 80
    assert st["gaussianCount"] == 10 * 16 * 4 * 2 and st["constantCount"] == terms
    assert st["sumCount"] == 10 * (8 * 8 * 15 + 7 * 8 * 63) + 79
    assert st["productCount"] == terms + 10 * (8 * 16 + 7 * 64) + 10 * 16 * 4
    assert st["hip"]["depthsExact"] is False and st["minDepth"] < st["averageDepth"] < st["maxDepth"]
    with pytest.raises(RuntimeError, match="cannot write graph statistics"):
        compile_query(native, os.path.join(GOLDEN, "NIPS5.bin"), **{"collect-graph-stats": "true", "graph-stats-file": str(tmp_path / "no" / "dir.json")})


def test_table_index_is_compared_in_a_wide_type(native):
    """A table as long as (or longer than) the feature type's range must not wrap the bound of the index clamp."""
    from spnc.structure import Categorical, Product
    for dtype, entries in (("uint8", 256), ("uint8", 300), ("uint16", 65536), ("uint64", 5)):
        p = np.full(entries, 1.0 / entries)
        k = compile_spn(native, Product(children=[Categorical(p=list(p), scope=0), Categorical(p=[0.5, 0.5], scope=1)]), dtype,
                        **{"hip-kernel": "jit"})
        src = k.source()
        os.remove(k.fileName())
        assert "(feat_t)" + str(entries) not in src
        wide = "(unsigned long long)x[0] < %dull" % entries if dtype == "uint64" else "(unsigned)x[0] < %du" % entries
        assert wide in src


def test_damaged_kernel_files_are_rejected(native, tmp_path):
    """Every field of a kernel file is checked on the host before anything could reach a launch."""
    from spnc import synthetic as syn
    import struct
    for opts in ({}, {"hip-kernel": "interpreter"}):
        k = compile_spn(native, syn.c4_spn() if opts else syn.c1_spn(), "float32" if opts else "int32", **opts)
        blob = open(k.fileName(), "rb").read()
        os.remove(k.fileName())
        bad = tmp_path / "bad.hipk"
        bad.write_bytes(blob[: len(blob) // 2])
        with pytest.raises(RuntimeError, match="truncated kernel file|damaged|malformed"):
            native.Kernel(str(bad))
        bad.write_bytes(blob + b"\0\0\0\0")
        with pytest.raises(RuntimeError, match="trailing bytes"):
            native.Kernel(str(bad))
        name_len = struct.unpack_from("<Q", blob, 8)[0]
        fields = 8 + 8 + name_len     # batchSize, numFeatures, bytesPerFeature, bytesPerResult, featureType
        for index, value, what in ((1, 0, "feature count"), (2, 3, "feature width"), (3, 0, "result width"), (4, 77, "feature type")):
            b = bytearray(blob)
            struct.pack_into("<I", b, fields + 4 * index, value)
            bad.write_bytes(bytes(b))
            with pytest.raises(RuntimeError, match=what):
                native.Kernel(str(bad))
    # interpreter programs: a slot number out of range, a broken length word and a bad opcode anywhere in the stream
    words = np.frombuffer(blob, dtype="<u4", offset=len(blob) % 4)
    code_words = k.info()["num_nodes"]  # just a lower bound on the stream length, for the search below
    assert code_words > 1000
    tail = len(blob) - 5 * 4 - 8 - 4 * 4 * 32 - 8   # somewhere inside the weights and slot lists: find the END instruction instead
    # the stream ends with [2][OP_END][slot]; the five u32 trailer fields and the staged list follow it
    b = bytearray(blob)
    hits = [i for i in range(len(b) - 12, 0, -4) if struct.unpack_from("<II", b, i) == (2, 0) or struct.unpack_from("<II", b, i)[0:2] == (2, 0x80)]
    assert hits
    end_at = hits[0]
    struct.pack_into("<I", b, end_at + 8, 1 << 19)
    bad.write_bytes(bytes(b))
    with pytest.raises(RuntimeError, match="malformed interpreter program \\(slot number"):
        native.Kernel(str(bad))
    b = bytearray(blob)
    struct.pack_into("<I", b, end_at + 4, 0x7f)
    bad.write_bytes(bytes(b))
    with pytest.raises(RuntimeError, match="malformed interpreter program"):
        native.Kernel(str(bad))
    b = bytearray(blob)
    struct.pack_into("<I", b, end_at, 3)
    bad.write_bytes(bytes(b))
    with pytest.raises(RuntimeError, match="malformed interpreter program"):
        native.Kernel(str(bad))


def test_execute_checks_the_input_type_not_only_its_width(native):
    from spnc import synthetic as syn
    k = compile_spn(native, syn.c2_spn(), "float32")
    os.remove(k.fileName())
    assert k.info()["feature_is_float"] == 1 and k.info()["support_marginal"] == 0
    with pytest.raises(RuntimeError, match="does not match the kernel's feature type float32"):
        k.execute(4, np.zeros((4, 16), dtype=np.int32))
    with pytest.raises(RuntimeError, match="does not match the kernel's feature type float32"):
        k.execute(4, np.zeros((4, 16), dtype=np.float64))
    k = compile_spn(native, syn.c1_spn(), "int32")
    os.remove(k.fileName())
    assert k.info()["feature_is_float"] == 0
    with pytest.raises(RuntimeError, match="does not match the kernel's feature type int32"):
        k.execute(4, np.zeros((4, 6), dtype=np.float32))


def test_host_feature_queries(native):
    flags = open("/proc/cpuinfo").read()
    C = native.SPNCompiler
    assert C.isFeatureAvailable("AVX2") == (" avx2" in flags) and C.isFeatureAvailable("vectorize") == (C.isFeatureAvailable("AVX") or C.isFeatureAvailable("Neon"))
    assert C.isFeatureAvailable("no-such-feature") is False


def _bad(native, tmp_path, match, **kw):
    path = rf.write(str(tmp_path / "bad.bin"), **kw)
    with pytest.raises(RuntimeError, match=match):
        compile_query(native, path)


def test_validation_errors(native, tmp_path):
    two = [rf.cat(1, 0), rf.cat(2, 1)]
    _bad(native, tmp_path, "Can only deserialize joint queries", nodes=[], scope=[0], with_joint=False)
    _bad(native, tmp_path, "No model attached to query", nodes=[], scope=[0], with_model=False)
    _bad(native, tmp_path, "Cannot compile raw models", nodes=two + [rf.prod(0, [1, 2])], scope=[0, 1], header_kind=0)
    _bad(native, tmp_path, "Leaf node references unknown feature", nodes=[rf.cat(1, 0), rf.cat(2, 7), rf.prod(0, [1, 2])], scope=[0, 1])
    _bad(native, tmp_path, "No definition found for node with ID: 9", nodes=two + [rf.prod(0, [1, 9])], scope=[0, 1])
    _bad(native, tmp_path, "No definition found for node with ID: 2", nodes=[rf.cat(1, 0), rf.prod(0, [1, 2]), rf.cat(2, 1)], scope=[0, 1])
    _bad(native, tmp_path, "No definition found for node with ID: 5", nodes=two + [rf.prod(0, [1, 2])], scope=[0, 1], root=5)
    _bad(native, tmp_path, "Unsupported feature data type complex64", nodes=two + [rf.prod(0, [1, 2])], scope=[0, 1], feature_type="complex64")
    _bad(native, tmp_path, "Unsupported floating-point type float128", nodes=two + [rf.prod(0, [1, 2])], scope=[0, 1], feature_type="float128")
    _bad(native, tmp_path, "Feature data type must be floating-point to support marginal", nodes=two + [rf.prod(0, [1, 2])],
         scope=[0, 1], feature_type="int32", marginal=True)
    _bad(native, tmp_path, "Weights must sum up to 1.0", nodes=[rf.cat(1, 0), rf.cat(2, 0), rf.wsum(0, [1, 2], [0.3, 0.8])], scope=[0])
    _bad(native, tmp_path, "Number of weights must match", nodes=[rf.cat(1, 0), rf.cat(2, 0), rf.wsum(0, [1, 2], [1.0])], scope=[0])
    _bad(native, tmp_path, "Number of addends must be greater than zero", nodes=[rf.wsum(0, [], [])], scope=[0])
    _bad(native, tmp_path, "Number of operands must be at least one", nodes=[rf.prod(0, [])], scope=[0])
    _bad(native, tmp_path, "Category probabilities should sum to 1.0", nodes=[rf.cat(0, 0, p=(0.5, 0.6))], scope=[0])
    _bad(native, tmp_path, "Lower bound must be less or equal", nodes=[rf.hist(0, 0, breaks=(0, 3, 1), densities=(0.5, 0.5))], scope=[0])
    _bad(native, tmp_path, "negative lower bound", nodes=[rf.hist(0, 0, breaks=(-1, 1, 2), densities=(0.5, 0.5))], scope=[0])
    _bad(native, tmp_path, "does not match the size of the scope", nodes=[rf.cat(0, 0)], scope=[0], num_features=3)
    with pytest.raises(RuntimeError, match="cannot open query file"):
        compile_query(native, str(tmp_path / "missing.bin"))
    (tmp_path / "junk.bin").write_bytes(b"\x00\x00\x00\x00\xff\xff\xff\x7f" + b"\x01" * 40)
    with pytest.raises(RuntimeError, match="malformed Cap'n Proto"):
        compile_query(native, str(tmp_path / "junk.bin"))


def test_old_files_without_marginal_field(native, tmp_path):
    """The reference's shipped query files encode JointProbability with an empty data section."""
    path = rf.write(str(tmp_path / "old.bin"), nodes=[rf.cat(0, 0)], scope=[0], feature_type="int32", joint_data_words=0)
    k = compile_query(native, path)  # would fail with 'floating-point to support marginal' if the default were true
    os.remove(k.fileName())


def test_scope_values_map_to_columns_in_ascending_order(native, tmp_path):
    # scope values {5, 2}: column 0 is scope 2, column 1 is scope 5
    path = rf.write(str(tmp_path / "s.bin"), nodes=[rf.cat(1, 5, p=(0.9, 0.1)), rf.cat(2, 2, p=(0.2, 0.8)), rf.prod(0, [1, 2])],
                    scope=[5, 2], feature_type="int32")
    k = compile_query(native, path, **{"hip-joint-tables": "false"})
    src = k.source()
    first = src.index("tab[0u + t1]")   # first table (scope 5) is indexed by column 1
    second = src.index("u + t0]")       # second table (scope 2) by column 0
    assert first < second
    os.remove(k.fileName())
    k = compile_query(native, path)      # default: the two leaves of the product share one joint table, rows of 2 + 1 entries
    assert "tab[0u + t1 * 3u + t0]" in k.source()
    os.remove(k.fileName())


def test_generated_source_variants(native):
    from spnc import synthetic as syn
    k = compile_spn(native, syn.c2_spn(), "float32")
    src = k.source()
    assert "__builtin_amdgcn_exp2f" in src and "spn_logadd" not in src and src.count("__builtin_amdgcn_logf") == 73
    os.remove(k.fileName())
    k = compile_spn(native, syn.c2_spn(), "float32", **{"hip-sum-form": "pairwise", "hip-log2-domain": "false", "hip-inline-math": "false"})
    src = k.source()
    assert src.count("spn_logadd(") == 73 * 3 + 1 and "log1pf(expf(b - a))" in src
    os.remove(k.fileName())
    k = compile_spn(native, syn.c2_spn(), "float32", marginal=True, **{"hip-compute-type": "float64", "hip-inline-math": "false"})
    assert k.dataType() == "float64" and k.bytesPerResult() == 8 and "typedef double real_t;" in k.source()
    os.remove(k.fileName())
    k = compile_spn(native, syn.c2_spn(), "float64", **{"use-log-space": "false", "hip-inline-math": "false"})
    assert k.dataType() == "float64" and "return log(" in k.source()
    os.remove(k.fileName())
    k = compile_spn(native, syn.c2_spn(), "float32", **{"hip-kernel": "interpreter"})
    assert k.info()["kernel_kind"] == 2 and "sumlayer" not in k.source() and "sum(4 terms)" in k.source()
    os.remove(k.fileName())
    k = compile_spn(native, syn.c4_spn(), "float32")
    src = k.source()
    assert k.info()["kernel_kind"] == 2 and "outersum(8 sums x 8x8 products)" in src
    # 32 features, Gaussian leaves only: they live in registers, not in value slots
    assert "(0 staged features," in src and "features in registers" in src
    # the 160 leaf regions are computed inside the outer sums above them, four at a time with the three 8x8 sums over
    # them: no product instructions and no 4x4 outer sums at all; 8x8 sums of their own remain above (10 root regions
    # of two and one more level below them)
    assert src.count("leafquad(8 sums x 8x8 products of two pairs of leaf regions: 8 sums x 4x4 products of 2 gaussians) scaled") == 20
    assert src.count("outersum(8 sums x 8x8 products)") == 10
    assert " = prod(" not in src and "prodbatch" not in src and "leafregion(" not in src and "leafpair(" not in src and "4x4 products)" not in src
    k2 = compile_spn(native, syn.c4_spn(), "float32", **{"hip-interp-leaf-regions": "false"})
    # without that, leaf products come in batches of eight (two leaf regions of four), sorted by feature
    assert k2.source().count("prodbatch(8 products x 2 gaussians) grouped") == 80 and "leafregion" not in k2.source()
    os.remove(k2.fileName())
    # outer-product sums are priced in their factored form: far fewer exponentials than sum terms
    i = k.info()
    assert i["trans_min"] < i["sum_terms"] // 10 and i["flops_min"] < 2 * i["sum_terms"]
    os.remove(k.fileName())
    # the program builder honours the tier and pool-size options
    pools = {"hip-interp-staged-features": "lds", "hip-interp-long-range": 8, "hip-interp-short-slots": 40, "hip-interp-leaf-regions": "false",
             "hip-interp-feature-registers": "false"}
    k = compile_spn(native, syn.c4_spn(), "float32", **pools)
    src = k.source()
    os.remove(k.fileName())
    # region vectors take blocks of nine consecutive slots (eight values and the scale): 32 features + one block
    assert "149 value slots (32 staged features, 108 long-lived)" in src and "prodbatch(8 products x 2 gaussians) grouped" in src
    k = compile_spn(native, syn.c4_spn(), "float32", **pools, **{"hip-interp-vector-blocks": "false"})
    assert "140 value slots (32 staged features, 99 long-lived)" in k.source()   # 41 = 32 features + one vector of 8 and its scale
    assert k.source().count(") scaled ") == 140             # every region vector that only feeds another region
    os.remove(k.fileName())
    k = compile_spn(native, syn.c4_spn(), "float32", **pools, **{"hip-interp-scaled-vectors": "false", "hip-interp-vector-blocks": "false"})
    assert "136 value slots (32 staged features, 96 long-lived)" in k.source() and ") scaled " not in k.source()
    os.remove(k.fileName())


def test_grouped_table_layout(native):
    """Table-heavy graphs: tables read with the same index share blocks of four columns, indices are packed four to a
    register, and the block size goes to 1024; small graphs and the option switch keep plain tables."""
    from spnc import synthetic as syn
    k = compile_spn(native, syn.c3_deep_spn(), "int32", marginal=False)
    src = k.source()
    os.remove(k.fileName())
    reads = src.count("*>(reinterpret_cast<const char*>(tab + ")
    assert 600 < reads < 800 and src.count("const spn_r4 q") > 400 and src.count("v_bfe_u32") >= reads
    assert "const unsigned P24 = " in src and "#define SPN_BLOCK 1024" in src and "__launch_bounds__(SPN_BLOCK, 1)" in src
    pool = int(re.search(r"#define SPN_NTAB (\d+)", src).group(1))
    assert pool % 4 == 0 and pool * 4 <= 80 * 1024
    k = compile_spn(native, syn.c3_deep_spn(), "int32", marginal=False, **{"hip-grouped-tables": "false"})
    src = k.source()
    os.remove(k.fileName())
    assert "spn_r4 q" not in src and "v_bfe_u32" not in src and "#define SPN_BLOCK 256" in src and src.count("= tab[") == 1940
    k = compile_spn(native, syn.c1_spn(), "int32", marginal=False)     # six tables, six indices: nothing to share
    assert "v_bfe_u32" not in k.source()
    os.remove(k.fileName())
    with pytest.raises(RuntimeError, match="hip-table-group-window must not be negative"):
        compile_spn(native, syn.c1_spn(), "int32", marginal=False, **{"hip-table-group-window": -1})
    with pytest.raises(RuntimeError, match="hip-table-pad-kib must be in"):
        compile_spn(native, syn.c1_spn(), "int32", marginal=False, **{"hip-table-pad-kib": 100})


def test_kernel_file_round_trip(native):
    from spnc import synthetic as syn
    for opts in ({}, {"hip-kernel": "interpreter"}):
        k = compile_spn(native, syn.c3_spn(), "int32", **opts)
        k2 = native.Kernel(k.fileName(), k.kernelName(), k.queryType(), k.target(), k.batchSize(), k.numFeatures(), k.bytesPerFeature(),
                           k.numResults(), k.bytesPerResult(), k.dataType())
        assert k2.info() == k.info() and k2.source() == k.source()
        with pytest.raises(RuntimeError, match="holds numFeatures"):
            native.Kernel(k.fileName(), k.kernelName(), 1, 3, k.batchSize(), 7, 4, 1, 4, "float32")
        os.remove(k.fileName())
    with pytest.raises(RuntimeError, match="cannot open kernel file"):
        native.Kernel("/nonexistent/kernel.hipk")
    with pytest.raises(RuntimeError, match="not a spnc-hip kernel file"):
        native.Kernel(os.path.join(GOLDEN, "NIPS5.bin"))


@pytest.mark.parametrize("name,size", [("NIPS5", 3), ("NIPS5", 10), ("nltcs", 1500), ("plants", 40), ("plants", 700)])
def test_max_task_size_cuts_the_graph_into_bounded_tasks(native, tmp_path, name, size):
    """maxTaskSize as in the reference (mlir/lib/Dialect/LoSPN/Partitioning/GraphPartitioner.cpp:84-157): tasks of at
    most that many operations plus 1 % slack (at least one), each a kernel of its own in one code object; every value
    a task hands on has a row of the intermediate buffer, and only the last task writes the result."""
    import re
    if name == "NIPS5":
        path = os.path.join(GOLDEN, "NIPS5.bin")
    else:
        path = model_as_query(os.path.join(GOLDEN, name + ".bin"), "float64", str(tmp_path / "q.bin"))
    k = compile_query(native, path, maxTaskSize=size, **{"hip-kernel": "jit"})
    src, info = k.source(), k.info()
    heads = re.findall(r"// task (\d+) of (\d+): (\d+) operations, (\d+) values in, (\d+) values out(, the result)?", src)
    assert len(heads) == info["num_tasks"] > 1
    slack = max(1, int(size * 0.01))
    # a binary sum is three operations (two weights, one add) and cannot be cut further
    assert all(int(h[2]) <= max(size + slack, 3) for h in heads)
    assert [h[5] != "" for h in heads] == [False] * (len(heads) - 1) + [True]
    assert int(heads[0][3]) == 0 and int(heads[-1][4]) == 0
    assert sum(int(h[4]) for h in heads) >= len(heads) - 1
    for t in range(len(heads)):
        assert 'void __launch_bounds__(SPN_BLOCK) spn_task%d(' % t in src or 'spn_task%d(' % t in src
    rows = [int(r) for r in re.findall(r"spn_res\[(\d+)ull \* spn_n\]", src)] + [int(r) for r in re.findall(r"spn_in\[(\d+)ull \* spn_n\]", src)]
    assert max(rows) + 1 == info["task_rows"]
    # the kernel file keeps the tasks
    k2 = native.Kernel(k.fileName(), k.kernelName(), k.queryType(), k.target(), k.batchSize(), k.numFeatures(), k.bytesPerFeature(), k.numResults(),
                       k.bytesPerResult(), k.dataType())
    assert k2.info()["num_tasks"] == info["num_tasks"] and k2.info()["task_rows"] == info["task_rows"]
    os.remove(k.fileName())


def test_discrete_graph_whose_tables_do_not_fit_lds(native):
    """Packed rows address their tables inside LDS. A graph whose table pool is too large for LDS (10 k nodes over 64
    features here) is built with one index per feature instead, and still compiles."""
    from spnc import synthetic as syn
    spn = syn.c3_spn(64, 33, sum_levels=3, inner_fan_in=(2, 9))
    k = compile_spn(native, spn, "int32", marginal=False)
    src = k.source()
    os.remove(k.fileName())
    assert "unsigned PK0 = R[0]" not in src and "spn_tab_lds" not in src and "const real_t* tab = spn_tables;" in src
