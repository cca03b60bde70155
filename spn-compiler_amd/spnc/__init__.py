"""spnc for AMD MI355X: the ``HIPCompiler`` front end of the batched log-likelihood path.

Mirrors the reference's ``spnc`` package (python-interface/spnc/__init__.py, cpu.py, gpu.py): a
compiler object with ``compile_ll`` / ``execute`` / ``log_likelihood`` / ``isAvailable``. The
native side is ``libspnc_hip.so`` reached through ``spnc.spncpy`` (ctypes over the C-ABI).
"""
from .hip import HIPCompiler  # noqa: F401
