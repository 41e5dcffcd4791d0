"""ctypes binding of the C ABI in include/qgemm.h.

There is no CPU fallback: if libqgemm.so is missing, load_library() raises."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libqgemm.so"

STATUS_OK = 0
STATUS_NAMES = {
    0: "QGEMM_OK", 1: "QGEMM_ERR_INVALID_ARG", 2: "QGEMM_ERR_UNSUPPORTED", 3: "QGEMM_ERR_NO_DEVICE",
    4: "QGEMM_ERR_LAUNCH", 5: "QGEMM_ERR_ALLOC", 6: "QGEMM_ERR_NOT_DIVISIBLE_M", 7: "QGEMM_ERR_NOT_DIVISIBLE_N",
    8: "QGEMM_ERR_NOT_DIVISIBLE_K", 9: "QGEMM_ERR_TOO_LARGE", 10: "QGEMM_ERR_SCRATCH_TOO_SMALL",
}


class QgemmError(RuntimeError):
    """A C-ABI entry returned a non-zero status.  For the divisibility statuses the
    message is the one the reference throws (hip_mix_gemm_kernel.cpp:460,485,503)."""

    def __init__(self, status, message):
        super().__init__(message)
        self.status = status


def library_path():
    """QGEMM_LIBRARY names another build of the library (e.g. the measurement build `make DEBUG=1` leaves as
    libqgemm_dbg.so); default: libqgemm.so beside this file."""
    return os.environ.get("QGEMM_LIBRARY") or os.path.join(_HERE, _LIB_NAME)


# every symbol include/qgemm.h declares: name -> (restype, argtypes)
_sz, _vp, _i = C.c_size_t, C.c_void_p, C.c_int
SIGNATURES = {
    "qgemm_init": (_i, []),
    "qgemm_shutdown": (_i, []),
    "qgemm_device_count": (_i, []),
    "qgemm_status_string": (C.c_char_p, [_i]),
    "qgemm_gemm": (_i, [_i, _i, _i, _vp, _sz, _vp, _sz, _vp, _sz, _sz, _sz, _sz, _vp]),
    "qgemm_scaled_gemm": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _i, _vp]),
    "qgemm_scaled_gemm_static": (_i, [_i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _i, _vp]),
    "qgemm_reserve_workspace": (_i, [_sz]),
    "qgemm_workspace_info": (_i, [C.POINTER(_vp), C.POINTER(_sz)]),
    "qgemm_transpose": (_i, [_i, _vp, _vp, _sz, _sz, _vp]),
    "qgemm_quantize": (_i, [_i, _i, _i, _vp, _sz, _sz, _sz, _vp, _sz, _vp, _sz, _sz, _vp]),
    "qgemm_tile_map": (_i, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.POINTER(C.c_uint32),
                            C.POINTER(C.c_uint32)]),
    "qgemm_set_option": (_i, [C.c_char_p, C.c_long]),
    "qgemm_force_config": (_i, [C.c_char_p]),
    "qgemm_variant_count": (_i, [_i, _i, _i]),
    "qgemm_variant_name": (_i, [_i, _i, _i, _i, C.c_char_p, _sz]),
    "qgemm_last_config": (_i, [C.c_char_p, _sz]),
    "qgemm_plan": (_i, [_i, _i, _i, _sz, _sz, _sz, C.c_char_p, _sz]),
    "qgemm_selftest_layouts": (_i, [C.c_char_p, _sz]),
}

_lib = None


def load_library():
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `make -C qgemm_amd/csrc` (or __graft_entry__.build()). "
            "There is no CPU fallback.")
    lib = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError here = ABI drift, fail loudly
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


_torch_ext = None


def load_torch_extension():
    """The module `qgemm_python` (qgemm_amd/qgemm_python*.so, built by csrc/build_torch_ext.py): the
    torch-facing entry points fp8_mm / int8_mm / bf16_mm the reference's packaging names (setup.py:73).
    Raises ImportError when it has not been built."""
    global _torch_ext
    if _torch_ext is None:
        import glob
        import importlib.util

        import torch  # noqa: F401  (its libraries must be loaded first)

        load_library()
        found = glob.glob(os.path.join(_HERE, "qgemm_python*.so"))
        if not found:
            raise ImportError(f"{_HERE}/qgemm_python*.so is missing: run `python qgemm_amd/csrc/build_torch_ext.py` "
                              "(or __graft_entry__.build())")
        spec = importlib.util.spec_from_file_location("qgemm_python", found[0])
        _torch_ext = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(_torch_ext)
    return _torch_ext


def check(status):
    if status != STATUS_OK:
        lib = load_library()
        msg = lib.qgemm_status_string(status).decode()
        raise QgemmError(status, f"{STATUS_NAMES.get(status, status)}: {msg}")
