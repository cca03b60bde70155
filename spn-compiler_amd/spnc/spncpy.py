"""Binding of ``libspnc_hip.so`` with the surface of the reference's native module ``spncpy``
(python-interface/src/python-interface.cpp:19-64): ``SPNCompiler`` and ``Kernel``.

The library is reached through its C-ABI (include/spnc_hip.h) with ctypes; failures of the
native side surface as ``RuntimeError`` like the reference's C++ exceptions do through pybind11.
There is no fallback: without the shared library every call raises.
"""
import ctypes
import os
import platform

import numpy as np

_LIB_NAME = "libspnc_hip.so"
_lib = None


class _Info(ctypes.Structure):
    _fields_ = [
        ("file_name", ctypes.c_char * 1024),
        ("kernel_name", ctypes.c_char * 256),
        ("query_type", ctypes.c_uint),
        ("target", ctypes.c_uint),
        ("batch_size", ctypes.c_uint),
        ("num_features", ctypes.c_uint),
        ("bytes_per_feature", ctypes.c_uint),
        ("num_results", ctypes.c_uint),
        ("bytes_per_result", ctypes.c_uint),
        ("dtype", ctypes.c_char * 16),
        ("kernel_kind", ctypes.c_uint),
        ("input_alignment", ctypes.c_uint),
        ("num_nodes", ctypes.c_uint),
        ("num_gaussian", ctypes.c_uint),
        ("num_categorical", ctypes.c_uint),
        ("num_histogram", ctypes.c_uint),
        ("num_product", ctypes.c_uint),
        ("num_sum", ctypes.c_uint),
        ("max_fan_in", ctypes.c_uint),
        ("sum_terms", ctypes.c_uint64),
        ("product_adds", ctypes.c_uint64),
        ("flops_min", ctypes.c_uint64),
        ("trans_min", ctypes.c_uint64),
        ("flops_pairwise", ctypes.c_uint64),
        ("trans_pairwise", ctypes.c_uint64),
        ("fused_min", ctypes.c_uint64),
        ("feature_is_float", ctypes.c_uint),
        ("support_marginal", ctypes.c_uint),
        ("num_tasks", ctypes.c_uint),
        ("task_rows", ctypes.c_uint),
    ]


def library_path():
    return os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), _LIB_NAME)


def _share_torch_hip_runtime():
    """One process, one HIP runtime. PyTorch ships a copy of libamdhip64 and asks the loader for it by a name that an
    already loaded system copy does not answer to; loaded second, that copy finds no GPU ("No HIP GPUs are
    available"). The other way round works: this library asks for the runtime by its soname, which PyTorch's copy
    carries too. So where PyTorch is installed but not imported yet, its copy is loaded first, by path."""
    import importlib.util
    import sys
    if "torch" in sys.modules:
        return
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    if spec is None or not spec.submodule_search_locations:
        return
    runtime = os.path.join(list(spec.submodule_search_locations)[0], "lib", "libamdhip64.so")
    if os.path.isfile(runtime):
        try:
            ctypes.CDLL(runtime, mode=ctypes.RTLD_GLOBAL)
        except OSError:
            pass  # not loadable on its own: the system's runtime serves this library


def _load():
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.isfile(path):
        raise RuntimeError(f"{_LIB_NAME} not found at {path}; build it with `make -C spn-compiler_amd/csrc`")
    _share_torch_hip_runtime()
    lib = ctypes.CDLL(path)
    vp, cp, sz = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t
    lib.spnc_hip_available.restype = ctypes.c_int
    lib.spnc_hip_compile.argtypes = [cp, ctypes.POINTER(cp), ctypes.POINTER(cp), sz, ctypes.POINTER(vp)]
    lib.spnc_hip_load.argtypes = [cp, ctypes.POINTER(vp)]
    lib.spnc_hip_kernel_info.argtypes = [vp, ctypes.POINTER(_Info)]
    lib.spnc_hip_execute.argtypes = [vp, sz, vp, vp]
    lib.spnc_hip_execute_device.argtypes = [vp, sz, vp, vp, vp]
    lib.spnc_hip_execute_device_static.argtypes = [vp, sz, vp, vp, vp]
    lib.spnc_hip_kernel_source.argtypes = [vp, ctypes.POINTER(cp), ctypes.POINTER(sz)]
    lib.spnc_hip_destroy.argtypes = [vp]
    lib.spnc_hip_destroy.restype = None
    lib.spnc_hip_last_error.restype = cp
    _lib = lib
    return lib


def _check(rc):
    if rc != 0:
        raise RuntimeError(_load().spnc_hip_last_error().decode("utf-8", "replace"))


class Kernel:
    """A compiled kernel: the ten metadata accessors of ``spncpy.Kernel`` plus ``execute``."""

    def __init__(self, fileName, kernelName=None, queryType=1, target=3, batchSize=None, numFeatures=None,
                 bytesPerFeature=None, numResults=1, bytesPerResult=None, dataType=None, _handle=None):
        lib = _load()
        if _handle is None:
            h = ctypes.c_void_p()
            _check(lib.spnc_hip_load(os.fsencode(fileName), ctypes.byref(h)))
            _handle = h
        self._handle = _handle
        self._info = _Info()
        _check(lib.spnc_hip_kernel_info(self._handle, ctypes.byref(self._info)))
        given = dict(kernelName=kernelName, batchSize=batchSize, numFeatures=numFeatures, bytesPerFeature=bytesPerFeature,
                     bytesPerResult=bytesPerResult, dataType=dataType)
        actual = dict(kernelName=self.kernelName(), batchSize=self.batchSize(), numFeatures=self.numFeatures(),
                      bytesPerFeature=self.bytesPerFeature(), bytesPerResult=self.bytesPerResult(), dataType=self.dataType())
        for key, value in given.items():
            if value is not None and value != actual[key]:
                raise RuntimeError(f"Kernel file {fileName} holds {key}={actual[key]!r}, not {value!r}")

    def __del__(self):
        h, self._handle = getattr(self, "_handle", None), None
        if h and _lib is not None:
            _lib.spnc_hip_destroy(h)

    def fileName(self):
        return self._info.file_name.decode()

    def kernelName(self):
        return self._info.kernel_name.decode()

    def queryType(self):
        return self._info.query_type

    def target(self):
        return self._info.target

    def batchSize(self):
        return self._info.batch_size

    def numFeatures(self):
        return self._info.num_features

    def bytesPerFeature(self):
        return self._info.bytes_per_feature

    def numResults(self):
        return self._info.num_results

    def bytesPerResult(self):
        return self._info.bytes_per_result

    def dataType(self):
        return self._info.dtype.decode()

    def info(self):
        """All fields of ``spnc_hip_info`` as a dict (graph statistics, kernel kind, alignment)."""
        out = {}
        for name, _ in _Info._fields_:
            v = getattr(self._info, name)
            out[name] = v.decode() if isinstance(v, bytes) else v
        return out

    def source(self):
        text, n = ctypes.c_char_p(), ctypes.c_size_t()
        _check(_load().spnc_hip_kernel_source(self._handle, ctypes.byref(text), ctypes.byref(n)))
        return ctypes.string_at(text, n.value).decode()

    def execute(self, num_elements, inputs):
        """[num_elements, numFeatures] host array in -> [num_elements] log-likelihoods out."""
        want = ("float" if self._info.feature_is_float else "int") + str(8 * self.bytesPerFeature())
        if inputs.dtype.itemsize != self.bytesPerFeature() or (inputs.dtype.kind == "f") != bool(self._info.feature_is_float) \
                or inputs.dtype.kind not in "fiu":
            raise RuntimeError(f"Input dtype {inputs.dtype} does not match the kernel's feature type {want}")
        if inputs.ndim != 2 or inputs.shape[1] != self.numFeatures() or inputs.shape[0] < num_elements:
            raise RuntimeError(f"Input must have shape [{num_elements}, {self.numFeatures()}], got {inputs.shape}")
        inputs = np.ascontiguousarray(inputs)
        result = np.empty(num_elements, dtype=np.dtype(self.dataType()))
        _check(_load().spnc_hip_execute(self._handle, num_elements, inputs.ctypes.data, result.ctypes.data))
        return result

    def execute_device(self, num_elements, input_ptr, output_ptr, stream=0):
        """Device pointers in/out; enqueues on ``stream`` (a hipStream_t as integer) without waiting."""
        _check(_load().spnc_hip_execute_device(self._handle, num_elements, ctypes.c_void_p(input_ptr),
                                               ctypes.c_void_p(output_ptr), ctypes.c_void_p(stream)))


    def execute_device_static(self, num_elements, input_ptr, output_ptr, stream=0):
        """``execute_device`` for interpreter kernels without any allocation: the kernel's device buffers come out of
        a fixed scratch array inside the library. Calls that overlap on one GPU race on that array."""
        _check(_load().spnc_hip_execute_device_static(self._handle, num_elements, ctypes.c_void_p(input_ptr),
                                                      ctypes.c_void_p(output_ptr), ctypes.c_void_p(stream)))


class SPNCompiler:
    def compileQuery(self, inputFile, options):
        lib = _load()
        keys = [str(k).encode() for k in options.keys()]
        vals = [str(v).encode() for v in options.values()]
        n = len(keys)
        karr = (ctypes.c_char_p * max(1, n))(*keys)
        varr = (ctypes.c_char_p * max(1, n))(*vals)
        h = ctypes.c_void_p()
        _check(lib.spnc_hip_compile(os.fsencode(inputFile), karr, varr, n, ctypes.byref(h)))
        return Kernel(None, _handle=h)

    @staticmethod
    def isTargetSupported(target):
        if target != "HIP":
            return False
        try:
            return bool(_load().spnc_hip_available())
        except (RuntimeError, OSError):
            return False

    @staticmethod
    def isFeatureAvailable(feature):
        """Host CPU features by the reference's names (compiler/src/Driver.cpp:61-82): "vectorize", "AVX", "AVX2",
        "AVX512", "Neon"; anything else is False. Read from the kernel's CPU flags; the HIP kernels do not depend on
        them, the query exists so that callers written against the reference keep working."""
        flags = set()
        try:
            with open("/proc/cpuinfo") as f:
                for line in f:
                    if line.lower().startswith(("flags", "features")):
                        flags.update(line.split(":", 1)[1].split())
                        break
        except OSError:
            return False
        have = {"AVX": "avx" in flags, "AVX2": "avx2" in flags, "AVX512": "avx512f" in flags,
                "Neon": bool(flags & {"neon", "asimd"})}
        have["vectorize"] = any(have.values())
        return bool(have.get(feature, False))

    @staticmethod
    def getHostArchitecture():
        return platform.machine()
