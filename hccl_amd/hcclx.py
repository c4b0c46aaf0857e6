"""Python face of the hcclx C ABI (include/hcclx.h).  Pointers are plain integers (device addresses)."""
import ctypes

from . import _lib
from ._lib import Seg, WideSeg, check

FOLD_CHAIN = 0
FOLD_SELF_FIRST = 1
FOLD_TREE = 2


def make_segs(segs):
    """segs: iterable of (count, [src addresses], [dst addresses][, tree program]) -> ctypes array of
    hcclx_seg_t.  The tree program is a flat list dst0, src0, dst1, src1, ... (FOLD_TREE only)."""
    segs = list(segs)
    arr = (Seg * max(1, len(segs)))()
    for i, seg in enumerate(segs):
        count, srcs, dsts = seg[0], seg[1], seg[2]
        for k, b in enumerate((seg[3] if len(seg) > 3 else [])[:2 * _lib.MAX_FAN]):
            arr[i].prog[k] = b
        arr[i].count = count
        arr[i].nsrc = len(srcs)
        arr[i].ndst = len(dsts)
        for k, p in enumerate(srcs[:_lib.MAX_FAN]):   # the library rejects nsrc/ndst beyond MAX_FAN
            arr[i].src[k] = p
        for k, p in enumerate(dsts[:_lib.MAX_FAN]):
            arr[i].dst[k] = p
    return arr, len(segs)


def make_wide_segs(segs):
    """segs: iterable of (count, [src addresses], [dst addresses][, tree program]) -> ctypes array of
    hcclx_wide_seg_t."""
    segs = list(segs)
    arr = (WideSeg * max(1, len(segs)))()
    for i, seg in enumerate(segs):
        count, srcs, dsts = seg[0], seg[1], seg[2]
        for k, b in enumerate((seg[3] if len(seg) > 3 else [])[:2 * _lib.MAX_WIDE_FAN]):
            arr[i].prog[k] = b
        arr[i].count = count
        arr[i].nsrc = len(srcs)
        arr[i].ndst = len(dsts)
        for k, p in enumerate(srcs[:_lib.MAX_WIDE_FAN]):   # the library rejects nsrc/ndst beyond MAX_WIDE_FAN
            arr[i].src[k] = p
        for k, p in enumerate(dsts[:_lib.MAX_WIDE_FAN]):
            arr[i].dst[k] = p
    return arr, len(segs)


def init():
    check(_lib.load().hcclx_init())


def tune(name, value):
    """Sets a launch-policy knob of the current device (hcclx_tune); plans made before keep their kernels."""
    L = _lib.load()
    L.hcclx_tune.argtypes = [ctypes.c_char_p, ctypes.c_uint64]
    L.hcclx_tune.restype = ctypes.c_int
    check(L.hcclx_tune(name.encode(), int(value)))


def kernels_launched():
    """Kernels the calling thread has launched through the library so far."""
    L = _lib.load()
    L.hcclx_kernels_launched.restype = ctypes.c_uint64
    return int(L.hcclx_kernels_launched())


def fold(segs, dtype, op=0, mode=FOLD_CHAIN, stream=0):
    arr, n = make_segs(segs)
    check(_lib.load().hcclx_fold(arr, n, int(dtype), int(op), int(mode), ctypes.c_void_p(stream)))


STATIC_MAX_SEGS = 128


def fold_static(segs, dtype, op=0, mode=FOLD_CHAIN, stream=0):
    """fold() through the entry point that allocates nothing (hcclx_fold_static): at most STATIC_MAX_SEGS segments,
    launch table in the library's fixed device array."""
    arr, n = make_segs(segs)
    check(_lib.load().hcclx_fold_static(arr, n, int(dtype), int(op), int(mode), ctypes.c_void_p(stream)))


def fold_wide(segs, dtype, op=0, mode=FOLD_CHAIN, stream=0):
    """Fold of segments with up to 64 sources and destinations (chain or tree order)."""
    arr, n = make_wide_segs(segs)
    check(_lib.load().hcclx_fold_wide(arr, n, int(dtype), int(op), int(mode), ctypes.c_void_p(stream)))


class Plan:
    """A fold whose table already sits in device memory: launch() is one kernel launch."""

    def __init__(self, segs, dtype, op=0, mode=FOLD_CHAIN, wide=False):
        h = ctypes.c_void_p()
        if wide:
            arr, n = make_wide_segs(segs)
            check(_lib.load().hcclx_plan_create_wide(arr, n, int(dtype), int(op), int(mode), ctypes.byref(h)))
        else:
            arr, n = make_segs(segs)
            check(_lib.load().hcclx_plan_create(arr, n, int(dtype), int(op), int(mode), ctypes.byref(h)))
        self._h = h

    @property
    def bytes(self):
        return _lib.load().hcclx_plan_bytes(self._h)

    @property
    def table_bytes(self):
        return _lib.load().hcclx_plan_table_bytes(self._h)

    def launch(self, stream=0):
        check(_lib.load().hcclx_plan_launch(self._h, ctypes.c_void_p(stream)))

    def close(self):
        if self._h:
            _lib.load().hcclx_plan_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _ptr_array(ptrs):
    return (ctypes.c_void_p * len(ptrs))(*ptrs)


def _table(t):
    """Host table (sequence of ints / numpy uint64 array) or device address (int)."""
    if isinstance(t, int):
        return ctypes.c_void_p(t), None
    arr = (ctypes.c_uint64 * len(t))(*[int(x) for x in t])
    return ctypes.cast(arr, ctypes.c_void_p), arr


def alltoallv(send, recv, send_counts, sdispls, rdispls, dtype, on_device=False, stream=0):
    n = len(send)
    a, ka = _table(send_counts)
    b, kb = _table(sdispls)
    c, kc = _table(rdispls)
    check(_lib.load().hcclx_alltoallv(_ptr_array(send), _ptr_array(recv), a, b, c, n, int(dtype),
                                      1 if on_device else 0, ctypes.c_void_p(stream)))


class AlltoAllVPlan(Plan):
    """An AlltoAllV with host tables whose block list already sits in device memory: launch() is one kernel
    launch with nothing copied in front of it."""

    def __init__(self, send, recv, send_counts, sdispls, rdispls, dtype):
        a, ka = _table(send_counts)
        b, kb = _table(sdispls)
        c, kc = _table(rdispls)
        h = ctypes.c_void_p()
        check(_lib.load().hcclx_alltoallv_plan_create(_ptr_array(send), _ptr_array(recv), a, b, c, len(send), int(dtype),
                                                      ctypes.byref(h)))
        self._h = h


def allgatherv(send, recv, counts, displs, dtype, on_device=False, stream=0):
    n = len(send)
    a, ka = _table(counts)
    b, kb = _table(displs)
    check(_lib.load().hcclx_allgatherv(_ptr_array(send), _ptr_array(recv), a, b, n, int(dtype),
                                       1 if on_device else 0, ctypes.c_void_p(stream)))


def displs_from_counts(counts, rows, n, displs, totals=0, stream=0):
    """counts, displs, totals: device addresses of uint64 arrays (rows x n, rows x n, rows; totals may be 0)."""
    check(_lib.load().hcclx_displs_from_counts(ctypes.c_void_p(counts), rows, n, ctypes.c_void_p(displs),
                                               ctypes.c_void_p(totals) if totals else None, ctypes.c_void_p(stream)))


def moe_workspace_bytes(n, entries):
    return _lib.load().hcclx_moe_workspace_bytes(n, entries)


def moe_route(dest, entries, row_elems, send_counts, sdispls, recv_counts, rdispls, perm, workspace, stream=0):
    """dest / perm: lists of n device addresses; the tables and the workspace are device addresses."""
    check(_lib.load().hcclx_moe_route(_ptr_array(dest), len(dest), entries, row_elems, ctypes.c_void_p(send_counts),
                                      ctypes.c_void_p(sdispls), ctypes.c_void_p(recv_counts), ctypes.c_void_p(rdispls),
                                      _ptr_array(perm), ctypes.c_void_p(workspace), ctypes.c_void_p(stream)))


def moe_pack(tokens, perm, entries, topk, row_bytes, packed, stream=0):
    check(_lib.load().hcclx_moe_pack(_ptr_array(tokens), _ptr_array(perm), len(tokens), entries, topk, row_bytes,
                                     _ptr_array(packed), ctypes.c_void_p(stream)))


def moe_combine(packed, perm, tokens, topk, row_elems, dtype, out, stream=0):
    check(_lib.load().hcclx_moe_combine(_ptr_array(packed), _ptr_array(perm), len(packed), tokens, topk, row_elems,
                                        int(dtype), _ptr_array(out), ctypes.c_void_p(stream)))


def moe_dispatch(tokens, dest, perm, entries, topk, row_elems, dtype, sdispls, rdispls, recv, stream=0):
    """Pack + AlltoAllV in one pass; sdispls / rdispls are the device tables moe_route wrote."""
    check(_lib.load().hcclx_moe_dispatch(_ptr_array(tokens), _ptr_array(dest), _ptr_array(perm), len(tokens), entries, topk,
                                         row_elems, int(dtype), ctypes.c_void_p(sdispls), ctypes.c_void_p(rdispls),
                                         _ptr_array(recv), ctypes.c_void_p(stream)))


def moe_gather_combine(expert, dest, perm, tokens, topk, row_elems, dtype, sdispls, rdispls, out, stream=0):
    """AlltoAllV back + combine in one pass, reading the rows where moe_dispatch put them."""
    check(_lib.load().hcclx_moe_gather_combine(_ptr_array(expert), _ptr_array(dest), _ptr_array(perm), len(expert), tokens,
                                               topk, row_elems, int(dtype), ctypes.c_void_p(sdispls),
                                               ctypes.c_void_p(rdispls), _ptr_array(out), ctypes.c_void_p(stream)))
