"""The allocation-free entry point, spnc_hip_execute_device_static, against spnc_hip_execute_device.

Both launch the same interpreter kernel over the same program; the static one keeps program, tables and spilled
value slots in the library's fixed scratch array and sizes its grid to what fits there. A sample's arithmetic does not
depend on the grid, so the results must agree bit for bit (the bar for this path is 1e-4 absolute in float32).
"""
import os

import numpy as np
import pytest

from conftest import compile_spn

pytestmark = pytest.mark.gpu


def _device_run(fn, x, n, dtype):
    import torch
    out = torch.full((n,), float("nan"), dtype=dtype, device="cuda")
    fn(n, x.data_ptr(), out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return out


def test_static_entry_point_matches_the_allocating_one(native):
    import torch
    from spnc import synthetic as syn
    c4, c3 = syn.CONFIGS["c4"], syn.CONFIGS["c3_deep"]
    ka = compile_spn(native, c4["spn"](), c4["dtype"])                                       # region graph: spills value slots
    kb = compile_spn(native, c3["spn"](), c3["dtype"], **{"hip-kernel": "interpreter"})      # table leaves, direct features
    assert ka.info()["kernel_kind"] == 2 and kb.info()["kernel_kind"] == 2 and "long-lived" in ka.source()
    n1, n2 = 300_007, 70_001            # the second call is smaller than the first
    xa = torch.from_numpy(c4["inputs"](n1)).cuda()
    xb = torch.from_numpy(c3["inputs"](n2)).cuda()
    want_a1 = _device_run(ka.execute_device, xa, n1, torch.float32)
    want_a2 = _device_run(ka.execute_device, xa, n2, torch.float32)
    want_b = _device_run(kb.execute_device, xb, n2, torch.float32)
    assert bool(torch.isfinite(want_a1).all()) and bool(torch.isfinite(want_b).all())
    # Fresh handles that never took the allocating path: whatever they need must come from the scratch array.
    sa, sb = native.Kernel(ka.fileName()), native.Kernel(kb.fileName())
    # The first use of the library's scratch array makes the runtime load the code object that holds it (64 MiB of
    # device memory, once per process); a third handle takes that first call so that the check below sees only the calls.
    _device_run(native.Kernel(kb.fileName()).execute_device_static, xb, 64, torch.float32)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    got_a1 = _device_run(sa.execute_device_static, xa, n1, torch.float32)
    got_a2 = _device_run(sa.execute_device_static, xa, n2, torch.float32)      # same program: launch only
    got_b = _device_run(sb.execute_device_static, xb, n2, torch.float32)        # another program takes the array over
    got_a3 = _device_run(sa.execute_device_static, xa, n2, torch.float32)      # and the first one takes it back
    assert torch.equal(got_a1, want_a1) and torch.equal(got_a2, want_a2) and torch.equal(got_a3, want_a2)
    assert torch.equal(got_b, want_b)
    # out tensors of this test come from torch's cache after the first round, so the device's free memory must not
    # have gone down by more than what torch took for them
    assert free_before - torch.cuda.mem_get_info()[0] <= 2 * 4 * n1 + (2 << 20)
    # values, not only agreement: the oracle on a slice
    from conftest import oracle_model
    from oracle import evaluate as ev
    ref = ev.ll_closed_f64(oracle_model(c4["spn"](), c4["dtype"]), xa[:500].cpu().numpy(), marginal=False)
    assert np.abs(got_a1[:500].cpu().numpy() - ref).max() <= 1e-4
    for k in (ka, kb):
        os.remove(k.fileName())


def test_static_entry_point_on_two_streams(native):
    """Every call on a GPU shares the one scratch array: calls on different streams, here of two kernels that take the
    array over from each other each time, wait for the call before them."""
    import torch
    from spnc import synthetic as syn
    c4, c2 = syn.CONFIGS["c4"], syn.CONFIGS["c2"]
    ka = compile_spn(native, c4["spn"](), c4["dtype"])
    kb = compile_spn(native, c2["spn"](), c2["dtype"], **{"hip-kernel": "interpreter"})
    n = 150_001
    xa = torch.from_numpy(c4["inputs"](n)).cuda()
    xb = torch.from_numpy(c2["inputs"](n)).cuda()
    want_a = _device_run(ka.execute_device, xa, n, torch.float32)
    want_b = _device_run(kb.execute_device, xb, n, torch.float32)
    outs = [torch.full((n,), float("nan"), dtype=torch.float32, device="cuda") for _ in range(6)]
    streams = [torch.cuda.Stream() for _ in range(2)]
    torch.cuda.synchronize()
    for rep in range(6):
        k, x = (ka, xa) if rep % 2 == 0 else (kb, xb)
        k.execute_device_static(n, x.data_ptr(), outs[rep].data_ptr(), streams[(rep // 2) % 2].cuda_stream if rep < 4 else streams[rep % 2].cuda_stream)
    torch.cuda.synchronize()
    for rep in range(6):
        assert torch.equal(outs[rep], want_a if rep % 2 == 0 else want_b), rep
    for k in (ka, kb):
        os.remove(k.fileName())


def test_static_entry_point_refuses_what_it_cannot_hold(native):
    import torch
    from spnc import synthetic as syn
    k = compile_spn(native, syn.c1_spn(), "int32")
    os.remove(k.fileName())
    x = torch.zeros((64, 6), dtype=torch.int32, device="cuda")
    out = torch.empty(64, dtype=torch.float32, device="cuda")
    with pytest.raises(RuntimeError, match="allocation-free entry point runs interpreter kernels"):
        k.execute_device_static(64, x.data_ptr(), out.data_ptr(), 0)
    # a program whose tables alone outgrow the array: one histogram bucket spanning 2^24 integer values
    from spnc.structure import Categorical, Histogram, Product
    big = 2 ** 24
    k = compile_spn(native, Product(children=[Histogram(breaks=[0, big], densities=[1.0 / big], bin_repr_points=[big / 2], scope=0),
                                              Categorical(p=[0.5, 0.5], scope=1)]), "int32", **{"hip-kernel": "interpreter"})
    os.remove(k.fileName())
    x = torch.zeros((64, 2), dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="bytes of scratch memory"):
        k.execute_device_static(64, x.data_ptr(), out.data_ptr(), 0)
    k.execute_device(64, x.data_ptr(), out.data_ptr(), 0)      # the allocating entry point still takes it
    torch.cuda.synchronize()
    assert abs(float(out[0]) - (np.log(1.0 / big) + np.log(0.5))) <= 1e-4
