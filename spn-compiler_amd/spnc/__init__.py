"""spnc for AMD MI355X: the ``HIPCompiler`` front end of the batched log-likelihood path.

Mirrors the reference's ``spnc`` package (python-interface/spnc/cpu.py, gpu.py): import the
compiler class from its module, ``from spnc.hip import HIPCompiler``; it offers ``compile_ll`` /
``execute`` / ``log_likelihood`` / ``isAvailable``. The native side is ``libspnc_hip.so`` reached
through ``spnc.spncpy`` (ctypes over the C-ABI).
"""
