"""GPU parity of the V-collective kernels (hcclx_alltoallv, hcclx_allgatherv) against the API contract."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import hcclx
from hccl_amd._lib import HcclError

from gpu_util import DevBuf

pytestmark = pytest.mark.gpu
GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "st_cases.json")))
NAME2DT = {"int8": T.INT8, "fp16": T.FP16, "bf16": T.BFP16, "int32": T.INT32, "fp32": T.FP32, "fp64": T.FP64}


def run_a2av(m, dtype, rng, on_device=False, send_pad=0):
    n = len(m)
    esz = T.DTYPE_SIZE[dtype]
    npd = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[esz]
    v = [T.alltoallvc_to_v(m, r) for r in range(n)]
    ins = [rng.integers(0, np.iinfo(npd).max, size=sum(m[i]), dtype=npd, endpoint=True) for i in range(n)]
    want = T.run_alltoallv(ins, [x[0] for x in v], [x[1] for x in v], [x[2] for x in v], [x[3] for x in v],
                           [sum(x[2]) for x in v])
    send = [DevBuf(x, offset=send_pad) for x in ins]
    recv = [DevBuf(nbytes=sum(x[2]) * esz) for x in v]
    sc = np.array([x[0] for x in v], dtype=np.uint64).ravel()
    sd = np.array([x[1] for x in v], dtype=np.uint64).ravel()
    rd = np.array([x[3] for x in v], dtype=np.uint64).ravel()
    if on_device:
        tab = torch.from_numpy(np.concatenate([sc, sd, rd]).astype(np.int64)).to("cuda:0")
        p = tab.data_ptr()
        hcclx.alltoallv([s.ptr for s in send], [r.ptr for r in recv], p, p + 8 * n * n, p + 16 * n * n, dtype,
                        on_device=True)
    else:
        hcclx.alltoallv([s.ptr for s in send], [r.ptr for r in recv], sc, sd, rd, dtype)
    torch.cuda.synchronize()
    for j in range(n):
        assert np.array_equal(recv[j].get(npd), want[j]), f"rank {j}"
        assert recv[j].guard_intact()


@pytest.mark.parametrize("case", GOLD["alltoallv"], ids=lambda c: c["name"])
@pytest.mark.parametrize("on_device", [False, True])
def test_alltoallv_reference_matrices(case, on_device):
    # counts of the reference's system tests divided by 2^13 (rounded up): zero cells stay zero
    m = [[-(-c // (1 << 13)) for c in row] for row in case["matrix"]]
    run_a2av(m, NAME2DT[case["dtype"]], np.random.default_rng(len(m)), on_device)


def test_alltoallv_odd_counts_and_misaligned_blocks():
    rng = np.random.default_rng(4)
    for n in (2, 3, 8, 13):
        m = rng.integers(0, 5000, size=(n, n)).tolist()
        m[0][0] = 0
        m[n - 1][0] = 1
        run_a2av(m, T.INT8, rng, send_pad=3)
        run_a2av(m, T.BFP16, rng)


@pytest.mark.parametrize("n", [2, 8, 16, 24, 40, 64])
def test_alltoallv_host_tables_of_any_rank_count_and_as_a_plan(n):
    """Up to 15 ranks the tables ride in the kernel arguments; beyond, the non-empty blocks become a list in device
    memory.  The same exchange as a plan moves new data at every launch, also from a captured graph."""
    rng = np.random.default_rng(n)
    m = rng.integers(0, 3000, size=(n, n))
    m[rng.random((n, n)) < 0.3] = 0                     # empty blocks
    m = m.tolist()
    run_a2av(m, T.BFP16, rng, send_pad=2)
    run_a2av(m, T.INT8, rng, send_pad=1)
    v = [T.alltoallvc_to_v(m, r) for r in range(n)]
    sc = np.array([x[0] for x in v], dtype=np.uint64).ravel()
    sd = np.array([x[1] for x in v], dtype=np.uint64).ravel()
    rd = np.array([x[3] for x in v], dtype=np.uint64).ravel()
    send = [DevBuf(nbytes=max(1, sum(m[i])) * 4) for i in range(n)]
    recv = [DevBuf(nbytes=max(1, sum(x[2])) * 4) for x in v]
    plan = hcclx.AlltoAllVPlan([s.ptr for s in send], [r.ptr for r in recv], sc, sd, rd, T.FP32)
    assert plan.bytes == 2 * 4 * int(sc.sum()) and plan.table_bytes > 0
    stream = torch.cuda.Stream()
    graph = None
    for rep in range(4):
        ins = [rng.integers(0, 2**32 - 1, size=max(1, sum(m[i])), dtype=np.uint32) for i in range(n)]
        for i in range(n):
            send[i].t[:ins[i].nbytes] = torch.from_numpy(ins[i].view(np.uint8).copy()).to("cuda:0")
        for r in recv:
            r.t.fill_(0xA5)
        torch.cuda.synchronize()
        if rep < 2:
            plan.launch(stream.cuda_stream)
        else:
            if graph is None:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.stream(stream):
                    graph.capture_begin()
                    plan.launch(stream.cuda_stream)
                    graph.capture_end()
            graph.replay()
        torch.cuda.synchronize()
        want = T.run_alltoallv([x[:sum(m[i])] for i, x in enumerate(ins)], [x[0] for x in v], [x[1] for x in v],
                               [x[2] for x in v], [x[3] for x in v], [sum(x[2]) for x in v])
        for j in range(n):
            assert np.array_equal(recv[j].get(np.uint32)[:sum(v[j][2])], want[j]), (rep, j)
            assert recv[j].guard_intact()
    del graph
    plan.close()


def test_alltoallv_all_zero_and_single_rank():
    rng = np.random.default_rng(1)
    run_a2av([[0, 0], [0, 0]], T.FP32, rng)
    run_a2av([[777]], T.FP32, rng)


def test_alltoallv_moe_dispatch_shape_small():
    """4 ranks x 96 tokens x hidden 7168 bf16, destinations Zipf(1.2): the MoE dispatch layout."""
    rng = np.random.default_rng(12)
    n, tokens, hidden = 4, 96, 7168
    w = 1.0 / np.arange(1, n + 1) ** 1.2
    w /= w.sum()
    m = [(np.bincount(rng.choice(n, size=tokens, p=w), minlength=n) * hidden).tolist() for _ in range(n)]
    run_a2av(m, T.BFP16, rng, on_device=True)


def run_agv(counts, displs, dtype, rng, on_device=False, total=None):
    n = len(counts)
    esz = T.DTYPE_SIZE[dtype]
    npd = {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[esz]
    total = total if total is not None else max(d + c for d, c in zip(displs, counts))
    ins = [rng.integers(0, np.iinfo(npd).max, size=c, dtype=npd, endpoint=True) for c in counts]
    fill = np.frombuffer(bytes([0xA5]) * (total * esz), dtype=npd)
    want = T.run_allgatherv(ins, counts, displs, total, fill)
    send = [DevBuf(x) for x in ins]
    recv = [DevBuf(nbytes=total * esz) for _ in range(n)]
    c64, d64 = np.array(counts, dtype=np.uint64), np.array(displs, dtype=np.uint64)
    if on_device:
        tab = torch.from_numpy(np.concatenate([c64, d64]).astype(np.int64)).to("cuda:0")
        hcclx.allgatherv([s.ptr for s in send], [r.ptr for r in recv], tab.data_ptr(), tab.data_ptr() + 8 * n, dtype,
                         on_device=True)
    else:
        hcclx.allgatherv([s.ptr for s in send], [r.ptr for r in recv], c64, d64, dtype)
    torch.cuda.synchronize()
    for j in range(n):
        assert np.array_equal(recv[j].get(npd), want[j]), f"rank {j}"
        assert recv[j].guard_intact()


@pytest.mark.parametrize("case", GOLD["allgatherv"], ids=lambda c: c["name"])
def test_allgatherv_reference_lists(case):
    div = 1 << 8 if max(case["counts"]) > 100000 else 1
    counts = [-(-c // div) for c in case["counts"]]
    displs = [sum(counts[:i]) for i in range(len(counts))] if div > 1 else case["displs"]
    run_agv(counts, displs, NAME2DT[case["dtype"]], np.random.default_rng(3))


def test_allgatherv_ragged_with_gaps_and_zero_counts():
    rng = np.random.default_rng(6)
    counts = [0, 1, 4097, 0, 33, 70001, 15, 2]
    displs, off = [], 5
    for c in counts:
        displs.append(off)
        off += c + 3          # holes between blocks must stay untouched
    run_agv(counts, displs, T.FP16, rng, total=off + 9)
    run_agv(counts, displs, T.INT8, rng, on_device=True, total=off + 9)
    run_agv([0, 0, 0], [0, 0, 0], T.FP32, rng, total=4)


def test_allgatherv_16_ranks_random_counts():
    rng = np.random.default_rng(16)
    counts = rng.integers(0, 40000, size=16).tolist()
    displs = [sum(counts[:i]) for i in range(16)]
    run_agv(counts, displs, T.FP16, rng, on_device=True)


@pytest.mark.parametrize("rows,n", [(1, 1), (1, 16), (8, 8), (64, 64), (5, 37)])
def test_displacements_from_counts_on_the_device(rows, n):
    """The exclusive prefix sum per row, by one wavefront: against numpy, with zeros and counts beyond 32 bits."""
    rng = np.random.default_rng(rows * 100 + n)
    counts = rng.integers(0, 1 << 20, size=(rows, n)).astype(np.uint64)
    counts[rng.random((rows, n)) < 0.2] = 0
    counts[0, n // 2] = (1 << 35) + 7
    dc = torch.from_numpy(counts.view(np.int64)).to("cuda:0")
    dd = torch.full((rows, n), -1, dtype=torch.int64, device="cuda:0")
    dt = torch.full((rows,), -1, dtype=torch.int64, device="cuda:0")
    hcclx.displs_from_counts(dc.data_ptr(), rows, n, dd.data_ptr(), dt.data_ptr())
    torch.cuda.synchronize()
    want = np.cumsum(counts, axis=1) - counts
    assert np.array_equal(dd.cpu().numpy().view(np.uint64), want)
    assert np.array_equal(dt.cpu().numpy().view(np.uint64), counts.sum(axis=1))
    dd.fill_(-1)
    hcclx.displs_from_counts(dc.data_ptr(), rows, n, dd.data_ptr())          # totals are optional
    torch.cuda.synchronize()
    assert np.array_equal(dd.cpu().numpy().view(np.uint64), want)


def test_allgatherv_with_counts_and_displacements_that_never_leave_the_device():
    """Config 3 of the baseline in small: 16 ranks, ragged fp16 blocks packed back to back; the displacements come
    from the counts by the device prefix sum and feed hcclx_allgatherv with tables_on_device."""
    rng = np.random.default_rng(3)
    n = 16
    counts = rng.integers(0, 50000, size=n).astype(np.uint64)
    counts[5] = 0
    ins = [rng.integers(0, 65536, size=int(c), dtype=np.uint16) for c in counts]
    total = int(counts.sum())
    send = [DevBuf(x) if x.size else DevBuf(nbytes=2) for x in ins]
    recv = [DevBuf(nbytes=total * 2) for _ in range(n)]
    dc = torch.from_numpy(counts.view(np.int64)).to("cuda:0")
    dd = torch.empty(n, dtype=torch.int64, device="cuda:0")
    hcclx.displs_from_counts(dc.data_ptr(), 1, n, dd.data_ptr())
    hcclx.allgatherv([s.ptr for s in send], [r.ptr for r in recv], dc.data_ptr(), dd.data_ptr(), T.FP16, on_device=True)
    torch.cuda.synchronize()
    displs = (np.cumsum(counts) - counts).astype(np.int64).tolist()
    want = T.run_allgatherv(ins, [int(c) for c in counts], displs, total, 0)
    for j in range(n):
        assert np.array_equal(recv[j].get(np.uint16), want[j]), f"rank {j}"
        assert recv[j].guard_intact()


def test_v_ops_reject_bad_arguments():
    b = DevBuf(nbytes=64)
    with pytest.raises(HcclError) as e:
        hcclx.alltoallv([b.ptr] * 65, [b.ptr] * 65, [0] * 65 * 65, [0] * 65 * 65, [0] * 65 * 65, T.INT8)
    assert e.value.code == 1
    with pytest.raises(HcclError) as e:
        hcclx.allgatherv([b.ptr], [b.ptr], [1], [0], 99)
    assert e.value.code == 5
