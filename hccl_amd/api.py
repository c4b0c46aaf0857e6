"""Python face of the HCCL entry points (include/hccl.h, include/hccl_comm.h) for virtual ranks.

Buffers are passed as device addresses (ints); count / displacement tables as sequences of ints."""
import ctypes

from . import _lib
from ._lib import HcclError

EXEC_FUSED, EXEC_STEP = 0, 1
CMD_ALLREDUCE, CMD_ALLGATHER, CMD_REDUCE_SCATTER, CMD_ALLTOALLV, CMD_ALLTOALLVC, CMD_ALLTOALL, CMD_ALLGATHER_V = \
    2, 6, 7, 8, 9, 10, 16
CMD_REDUCE_SCATTER_V = 17
SHAPE_CLOS, SHAPE_MESH_1D = 0, 1
LINK_HCCS, LINK_ROCE, LINK_PCIE = 0, 1, 2


class LastOpInfo(ctypes.Structure):
    _fields_ = [("algName", ctypes.c_char * 64), ("levels", ctypes.c_uint32), ("launches", ctypes.c_uint32),
                ("fusedSegments", ctypes.c_uint32), ("fused", ctypes.c_int), ("planCacheHit", ctypes.c_int)]


class CheckReport(ctypes.Structure):
    _fields_ = [("steps", ctypes.c_uint32), ("levels", ctypes.c_uint32), ("copies", ctypes.c_uint32),
                ("reduces", ctypes.c_uint32), ("races", ctypes.c_uint32), ("semanticErrors", ctypes.c_uint32),
                ("exhaustive", ctypes.c_int), ("firstProblem", ctypes.c_char * 256)]


_bound = False


def lib():
    global _bound
    L = _lib.load()
    if not _bound:
        vp, u64, u32, ci = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int
        sig = {
            "hcclxCommInitAll": [u32, u64, ci, ctypes.POINTER(vp)],
            "HcclCommInitAll": [u32, vp, ctypes.POINTER(vp)],
            "HcclCommDestroy": [vp],
            "HcclGetRankSize": [vp, ctypes.POINTER(u32)],
            "HcclGetRankId": [vp, ctypes.POINTER(u32)],
            "hcclxCommSetExecMode": [vp, ci],
            "hcclxCommSetBlocking": [vp, ci],
            "hcclxCommSetAlgorithm": [vp, ci, ctypes.c_char_p],
            "hcclxCommSetTopo": [vp, u32, ci, u32],
            "hcclxCommSetLinkProtocol": [vp, ci],
            "hcclxCommGetLastOpInfo": [vp, ctypes.POINTER(LastOpInfo)],
            "hcclxCommSetTrace": [vp, ci],
            "hcclxCommSetCheck": [vp, ci],
            "hcclxCommSetClosedForm": [vp, ci],
            "hcclxCommGetLastCheck": [vp, ctypes.POINTER(CheckReport)],
            "HcclAllReduce": [vp, vp, u64, ci, ci, vp, vp],
            "HcclReduceScatter": [vp, vp, u64, ci, ci, vp, vp],
            "HcclReduceScatterV": [vp, vp, vp, vp, u64, ci, ci, vp, vp],
            "HcclAllGather": [vp, vp, u64, ci, vp, vp],
            "HcclAllGatherV": [vp, u64, vp, vp, vp, ci, vp, vp],
            "HcclAlltoAllV": [vp, vp, vp, ci, vp, vp, vp, ci, vp, vp],
            "HcclAlltoAll": [vp, u64, ci, vp, u64, ci, vp, vp],
            "HcclAlltoAllVC": [vp, vp, ci, vp, ci, vp, vp],
        }
        for name, args in sig.items():
            fn = getattr(L, name)
            fn.restype = ctypes.c_int
            fn.argtypes = args
        L.hcclxCommGetLastTrace.restype = ctypes.c_uint64
        L.hcclxCommGetLastTrace.argtypes = [vp, ctypes.c_char_p, u64]
        _bound = True
    return L


def check(rc):
    if rc != 0:
        raise HcclError(rc, "collective call failed")


def u64_table(seq):
    """Host count / displacement table as the C entry points take it (uint64 array).  Tables that do not
    change between calls can be converted once and passed again."""
    if isinstance(seq, ctypes.Array):
        return seq
    return (ctypes.c_uint64 * len(seq))(*[int(x) for x in seq])


_u64 = u64_table


class World:
    """N virtual ranks in the current GPU (or none at all when dry=True)."""

    def __init__(self, n, ccl_bytes=200 * 1024 * 1024, dry=False):
        self.n = n
        arr = (ctypes.c_void_p * n)()
        check(lib().hcclxCommInitAll(n, ccl_bytes, 1 if dry else 0, arr))
        self.comms = [arr[i] for i in range(n)]

    def close(self):
        for c in self.comms:
            lib().HcclCommDestroy(c)
        self.comms = []

    def set_mode(self, mode):
        check(lib().hcclxCommSetExecMode(self.comms[0], mode))

    def set_blocking(self, on):
        check(lib().hcclxCommSetBlocking(self.comms[0], 1 if on else 0))

    def set_algorithm(self, cmd, name):
        check(lib().hcclxCommSetAlgorithm(self.comms[0], cmd, (name or "").encode()))

    def set_topo(self, levels=1, shape=SHAPE_MESH_1D, devices_per_server=0):
        check(lib().hcclxCommSetTopo(self.comms[0], levels, shape, devices_per_server))

    def set_link_protocol(self, protocol):
        """LINK_PCIE puts the templates that have a read mode into it (the receiver fetches); the values stay the same."""
        check(lib().hcclxCommSetLinkProtocol(self.comms[0], int(protocol)))

    def set_trace(self, on):
        check(lib().hcclxCommSetTrace(self.comms[0], 1 if on else 0))

    def set_closed_form(self, mode):
        """0 = record every template's steps, 1 = closed forms for plain launches, 2 = also when tracing / dry."""
        check(lib().hcclxCommSetClosedForm(self.comms[0], int(mode)))

    def set_check(self, on):
        check(lib().hcclxCommSetCheck(self.comms[0], 1 if on else 0))

    def last_check(self):
        rep = CheckReport()
        check(lib().hcclxCommGetLastCheck(self.comms[0], ctypes.byref(rep)))
        return rep

    def last_info(self):
        info = LastOpInfo()
        check(lib().hcclxCommGetLastOpInfo(self.comms[0], ctypes.byref(info)))
        return info

    def last_trace(self):
        n = lib().hcclxCommGetLastTrace(self.comms[0], None, 0)
        buf = ctypes.create_string_buffer(n + 1)
        lib().hcclxCommGetLastTrace(self.comms[0], buf, n + 1)
        return buf.value.decode()

    # ---- collectives: one call per rank, in any order; launched by the last one ----
    def all_reduce(self, rank, send, recv, count, dtype, op, stream):
        return lib().HcclAllReduce(send, recv, count, int(dtype), int(op), self.comms[rank], stream)

    def reduce_scatter(self, rank, send, recv, recv_count, dtype, op, stream):
        return lib().HcclReduceScatter(send, recv, recv_count, int(dtype), int(op), self.comms[rank], stream)

    def reduce_scatter_v(self, rank, send, counts, displs, recv, recv_count, dtype, op, stream):
        c, d = _u64(counts), _u64(displs)
        return lib().HcclReduceScatterV(send, ctypes.cast(c, ctypes.c_void_p), ctypes.cast(d, ctypes.c_void_p), recv,
                                        recv_count, int(dtype), int(op), self.comms[rank], stream)

    def all_gather(self, rank, send, recv, send_count, dtype, stream):
        return lib().HcclAllGather(send, recv, send_count, int(dtype), self.comms[rank], stream)

    def all_gather_v(self, rank, send, send_count, recv, counts, displs, dtype, stream):
        c, d = _u64(counts), _u64(displs)
        return lib().HcclAllGatherV(send, send_count, recv, ctypes.cast(c, ctypes.c_void_p),
                                    ctypes.cast(d, ctypes.c_void_p), int(dtype), self.comms[rank], stream)

    def all_to_all_v(self, rank, send, sc, sd, recv, rc, rd, dtype, stream):
        a, b, c, d = _u64(sc), _u64(sd), _u64(rc), _u64(rd)
        cast = lambda x: ctypes.cast(x, ctypes.c_void_p)
        return lib().HcclAlltoAllV(send, cast(a), cast(b), int(dtype), recv, cast(c), cast(d), int(dtype),
                                   self.comms[rank], stream)

    def all_to_all(self, rank, send, count, recv, dtype, stream):
        return lib().HcclAlltoAll(send, count, int(dtype), recv, count, int(dtype), self.comms[rank], stream)

    def all_to_all_vc(self, rank, send, matrix_flat, recv, dtype, stream):
        m = _u64(matrix_flat)
        return lib().HcclAlltoAllVC(send, ctypes.cast(m, ctypes.c_void_p), int(dtype), recv, int(dtype),
                                    self.comms[rank], stream)
