"""Loader of the native library.  There is no fallback: every op in this package runs in
libhccl_amd.so (HIP kernels for gfx950 behind a C ABI) or raises."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# HCCL_AMD_LIBRARY names another build of the same library (e.g. one with different tile parameters)
LIB_PATH = os.environ.get("HCCL_AMD_LIBRARY") or os.path.join(_HERE, "lib", "libhccl_amd.so")

MAX_FAN = 16


class Seg(ctypes.Structure):
    """hcclx_seg_t of include/hcclx.h."""
    _fields_ = [
        ("count", ctypes.c_uint64),
        ("nsrc", ctypes.c_uint32),
        ("ndst", ctypes.c_uint32),
        ("src", ctypes.c_void_p * MAX_FAN),
        ("dst", ctypes.c_void_p * MAX_FAN),
        ("prog", ctypes.c_uint8 * (2 * MAX_FAN)),
    ]


MAX_WIDE_FAN = 64


class WideSeg(ctypes.Structure):
    """hcclx_wide_seg_t of include/hcclx.h."""
    _fields_ = [
        ("count", ctypes.c_uint64),
        ("nsrc", ctypes.c_uint32),
        ("ndst", ctypes.c_uint32),
        ("src", ctypes.c_void_p * MAX_WIDE_FAN),
        ("dst", ctypes.c_void_p * MAX_WIDE_FAN),
        ("prog", ctypes.c_uint8 * (2 * MAX_WIDE_FAN)),
    ]


_lib = None


def load():
    """Returns the ctypes handle of libhccl_amd.so, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C hccl_amd/csrc`; there is no CPU fallback")
    lib = ctypes.CDLL(LIB_PATH)
    u64p = ctypes.POINTER(ctypes.c_uint64)
    vpp = ctypes.POINTER(ctypes.c_void_p)
    lib.hcclx_init.restype = ctypes.c_int
    lib.hcclx_last_error.restype = ctypes.c_char_p
    lib.hcclx_dtype_size.restype = ctypes.c_uint32
    lib.hcclx_dtype_size.argtypes = [ctypes.c_int]
    lib.hcclx_fold.restype = ctypes.c_int
    lib.hcclx_fold.argtypes = [ctypes.POINTER(Seg), ctypes.c_uint32, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                               ctypes.c_void_p]
    lib.hcclx_fold_static.restype = ctypes.c_int
    lib.hcclx_fold_static.argtypes = [ctypes.POINTER(Seg), ctypes.c_uint32, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                      ctypes.c_void_p]
    lib.hcclx_plan_create.restype = ctypes.c_int
    lib.hcclx_plan_create.argtypes = [ctypes.POINTER(Seg), ctypes.c_uint32, ctypes.c_int, ctypes.c_int,
                                      ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
    lib.hcclx_fold_wide.restype = ctypes.c_int
    lib.hcclx_fold_wide.argtypes = [ctypes.POINTER(WideSeg), ctypes.c_uint32, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                    ctypes.c_void_p]
    lib.hcclx_plan_create_wide.restype = ctypes.c_int
    lib.hcclx_plan_create_wide.argtypes = [ctypes.POINTER(WideSeg), ctypes.c_uint32, ctypes.c_int, ctypes.c_int,
                                           ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
    lib.hcclx_plan_launch.restype = ctypes.c_int
    lib.hcclx_plan_launch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    lib.hcclx_plan_destroy.restype = ctypes.c_int
    lib.hcclx_plan_destroy.argtypes = [ctypes.c_void_p]
    lib.hcclx_plan_bytes.restype = ctypes.c_uint64
    lib.hcclx_plan_bytes.argtypes = [ctypes.c_void_p]
    lib.hcclx_plan_table_bytes.restype = ctypes.c_uint64
    lib.hcclx_plan_table_bytes.argtypes = [ctypes.c_void_p]
    lib.hcclx_alltoallv.restype = ctypes.c_int
    lib.hcclx_alltoallv.argtypes = [vpp, vpp, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                    ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.hcclx_alltoallv_plan_create.restype = ctypes.c_int
    lib.hcclx_alltoallv_plan_create.argtypes = [vpp, vpp, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                                ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
    lib.hcclx_moe_workspace_bytes.restype = ctypes.c_uint64
    lib.hcclx_moe_workspace_bytes.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
    lib.hcclx_moe_route.restype = ctypes.c_int
    lib.hcclx_moe_route.argtypes = [vpp, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p,
                                    ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, vpp, ctypes.c_void_p,
                                    ctypes.c_void_p]
    lib.hcclx_moe_pack.restype = ctypes.c_int
    lib.hcclx_moe_pack.argtypes = [vpp, vpp, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64, vpp,
                                   ctypes.c_void_p]
    lib.hcclx_moe_combine.restype = ctypes.c_int
    lib.hcclx_moe_combine.argtypes = [vpp, vpp, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64,
                                      ctypes.c_int, vpp, ctypes.c_void_p]
    lib.hcclx_moe_dispatch.restype = ctypes.c_int
    lib.hcclx_moe_dispatch.argtypes = [vpp, vpp, vpp, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64,
                                       ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, vpp, ctypes.c_void_p]
    lib.hcclx_moe_gather_combine.restype = ctypes.c_int
    lib.hcclx_moe_gather_combine.argtypes = [vpp, vpp, vpp, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                             ctypes.c_uint64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, vpp,
                                             ctypes.c_void_p]
    lib.hcclx_displs_from_counts.restype = ctypes.c_int
    lib.hcclx_displs_from_counts.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                                             ctypes.c_void_p, ctypes.c_void_p]
    lib.hcclx_allgatherv.restype = ctypes.c_int
    lib.hcclx_allgatherv.argtypes = [vpp, vpp, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int,
                                     ctypes.c_int, ctypes.c_void_p]
    _lib = lib
    return lib


class HcclError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"HcclResult {code}: {text}")
        self.code = code


def check(rc):
    if rc != 0:
        raise HcclError(rc, load().hcclx_last_error().decode())
