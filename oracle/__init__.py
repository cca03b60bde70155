"""CPU oracle for the batched joint log-likelihood path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the shipped
product: only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import it, and only as the checker.  The product path
(``spn-compiler_amd/``) never imports, links or executes anything from here.

Modules
-------
capnp_lite   independent, read-only Cap'n Proto decoder (stream framing, far
             pointers, struct-size evolution) used to decode the reference's
             ``.bin`` fixtures without pycapnp.
spn_model    decodes ``Header{model|query}`` of the reference's schema
             (xspn/xspn/serialization/binary/capnproto/spflow.capnp:27-102)
             into plain Python node records.
evaluate     two evaluators: ``ll_closed_f64`` (textbook closed forms via
             SciPy) and ``ll_reforder`` (the reference's operation order and
             rounding points in f32 or f64).
cgen         emits the straight-line C kernel used as the timed CPU baseline.
spn_oracle.c C restatement of ``ll_reforder`` on the lowered op list.
"""
