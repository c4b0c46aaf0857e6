"""GPU parity of the MoE dispatch entry points (hcclx_moe_route / _pack / _combine) against the oracle, and the
dispatch -> AlltoAllV -> AlltoAllV back -> combine round trip at the size of the baseline's MoE configuration."""
import numpy as np
import pytest
import torch

from oracle import templates as T
from hccl_amd import hcclx
from hccl_amd._lib import HcclError

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev_i32(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).to(DEV)


def route_on_gpu(dests, n, entries, row_elems, skew=0):
    """`skew`: rank i's destination array starts (i * skew) % 4 entries into its allocation, so that some arrays
    are not 16-byte aligned."""
    whole = [dev_i32(np.concatenate([np.zeros((i * skew) % 4, dtype=np.int32), np.asarray(x, dtype=np.int32)]))
             for i, x in enumerate(dests)]
    d = [w[(i * skew) % 4:] for i, w in enumerate(whole)]
    tabs = [torch.full((n * n,), -1, dtype=torch.int64, device=DEV) for _ in range(4)]
    perm = [torch.full((entries,), 12345, dtype=torch.int32, device=DEV) for _ in range(n)]
    ws = torch.empty(hcclx.moe_workspace_bytes(n, entries), dtype=torch.uint8, device=DEV)
    torch.cuda.synchronize()
    hcclx.moe_route([x.data_ptr() for x in d], entries, row_elems, tabs[0].data_ptr(), tabs[1].data_ptr(),
                    tabs[2].data_ptr(), tabs[3].data_ptr(), [p.data_ptr() for p in perm], ws.data_ptr())
    torch.cuda.synchronize()
    return tabs, perm


@pytest.mark.parametrize("n,entries", [(1, 5), (2, 256), (3, 257), (8, 4096), (8, 70001), (16, 1000), (64, 33333),
                                       (64, 3001), (33, 7942), (16, 16384), (16, 16385), (5, 3), (12, 4099)])
@pytest.mark.parametrize("skew", [0, 1])
def test_route_tables_and_stable_permutation(n, entries, skew):
    """Both routing paths (two launches while a rank has at most 64 chunks of 256 entries and the per-chunk histogram at
    most 16384 cells, three beyond), with destination arrays that are and are not 16-byte aligned."""
    rng = np.random.default_rng(n * 1000 + entries)
    p = 1.0 / np.arange(1, n + 1) ** 1.2
    dests = [rng.choice(n, size=entries, p=p / p.sum()) for _ in range(n)]
    dests[0][::7] = -1                      # dropped entries
    if n > 1:
        dests[1][::5] = n
    tabs, perm = route_on_gpu(dests, n, entries, 24, skew)
    sc, sd, rc, rd, perms = T.moe_route(dests, n, 24)
    for got, want in zip(tabs, (sc, sd, rc, rd)):
        assert np.array_equal(got.cpu().numpy().reshape(n, n), np.array(want, dtype=np.int64))
    for i in range(n):
        assert np.array_equal(perm[i].cpu().numpy().view(np.uint32), perms[i]), i


@pytest.mark.parametrize("topk,dtype,width", [(1, T.BFP16, 64), (2, T.BFP16, 40), (4, T.FP32, 12), (3, T.FP16, 8),
                                              (1, T.INT8, 48), (2, T.BFP16, 3000), (1, T.FP32, 1032), (4, T.FP16, 1024)])
def test_pack_and_combine_match_the_oracle(topk, dtype, width):
    rng = np.random.default_rng(topk * 10 + dtype)
    n, tokens = 4, 777
    entries = tokens * topk
    npd = T.NP_STORAGE[dtype]
    esz = T.DTYPE_SIZE[dtype]
    dests = [rng.integers(0, n + 1, size=entries) for _ in range(n)]            # n = dropped
    if dtype == T.FP32:
        toks = [rng.standard_normal((tokens, width)).astype(np.float32) for _ in range(n)]
    elif dtype == T.INT8:
        toks = [rng.integers(-128, 127, size=(tokens, width), dtype=np.int8) for _ in range(n)]
    else:
        toks = [T.narrow16(rng.standard_normal(tokens * width).astype(np.float32), dtype).reshape(tokens, width)
                for _ in range(n)]
    tabs, perm = route_on_gpu(dests, n, entries, width)
    _, _, _, _, perms = T.moe_route(dests, n, width)
    kept = [int(np.count_nonzero(p != T.MOE_DROPPED)) for p in perms]
    d_tok = [torch.from_numpy(t.view(np.uint8).reshape(-1).copy()).to(DEV) for t in toks]
    d_pack = [torch.full((max(1, k) * width * esz + 64,), 0xEE, dtype=torch.uint8, device=DEV) for k in kept]
    torch.cuda.synchronize()
    hcclx.moe_pack([t.data_ptr() for t in d_tok], [p.data_ptr() for p in perm], entries, topk, width * esz,
                   [t.data_ptr() for t in d_pack])
    torch.cuda.synchronize()
    packed = []
    for i in range(n):
        want = T.moe_pack(toks[i], perms[i], topk, max(1, kept[i]))
        got = d_pack[i].cpu().numpy()
        assert np.array_equal(got[:kept[i] * width * esz].view(npd), want[:kept[i]].reshape(-1)), i
        assert (got[max(1, kept[i]) * width * esz:] == 0xEE).all()              # nothing past the last row
        packed.append(want)
    d_out = [torch.full((tokens * width * esz + 64,), 0xEE, dtype=torch.uint8, device=DEV) for _ in range(n)]
    torch.cuda.synchronize()
    hcclx.moe_combine([t.data_ptr() for t in d_pack], [p.data_ptr() for p in perm], tokens, topk, width, dtype,
                      [t.data_ptr() for t in d_out])
    torch.cuda.synchronize()
    for i in range(n):
        want = T.moe_combine(packed[i], perms[i], topk, dtype)
        got = d_out[i].cpu().numpy()
        assert np.array_equal(got[:tokens * width * esz].view(npd).reshape(tokens, width).view(np.uint8),
                              want.view(np.uint8)), i
        assert (got[tokens * width * esz:] == 0xEE).all()


@pytest.mark.parametrize("topk,dtype,width,n,tokens", [(1, T.BFP16, 64, 4, 777), (2, T.BFP16, 40, 5, 300),
                                                        (4, T.FP32, 12, 3, 513), (3, T.FP16, 8, 8, 1000),
                                                        (1, T.INT8, 48, 2, 257), (2, T.FP32, 4, 64, 96),
                                                        # rows of 128 vectors and more: the kernels that move one row per workgroup
                                                        (2, T.BFP16, 3000, 4, 61), (1, T.FP32, 1032, 3, 100),
                                                        (3, T.FP16, 1024, 5, 40), (1, T.INT8, 16 * 129, 2, 33)])
def test_fused_dispatch_and_gather_combine_equal_the_two_pass_pipeline(topk, dtype, width, n, tokens):
    """hcclx_moe_dispatch puts every row where pack + AlltoAllV would; hcclx_moe_gather_combine gives what
    AlltoAllV back + combine would: checked against the oracle's pack -> alltoallv -> alltoallv -> combine."""
    rng = np.random.default_rng(topk * 100 + dtype + n)
    entries = tokens * topk
    npd = T.NP_STORAGE[dtype]
    esz = T.DTYPE_SIZE[dtype]
    dests = [rng.integers(-1, n + 1, size=entries) for _ in range(n)]            # -1 and n are dropped
    if dtype == T.FP32:
        toks = [rng.standard_normal((tokens, width)).astype(np.float32) for _ in range(n)]
    elif dtype == T.INT8:
        toks = [rng.integers(-128, 127, size=(tokens, width), dtype=np.int8) for _ in range(n)]
    else:
        toks = [T.narrow16(rng.standard_normal(tokens * width).astype(np.float32), dtype).reshape(tokens, width)
                for _ in range(n)]
    tabs, perm = route_on_gpu(dests, n, entries, width)
    sc, sd, rc, rd, perms = T.moe_route(dests, n, width)
    kept = [int(np.count_nonzero(p != T.MOE_DROPPED)) for p in perms]
    inbound = [sum(rc[j]) // width for j in range(n)]
    # the oracle's two-pass pipeline, in elements
    packed = [T.moe_pack(toks[i], perms[i], topk, max(1, kept[i])).reshape(-1) for i in range(n)]
    recv_want = T.run_alltoallv(packed, sc, sd, rc, rd, [max(1, r) * width for r in inbound], fill=0)
    d_dest = [dev_i32(x) for x in dests]
    d_tok = [torch.from_numpy(t.view(np.uint8).reshape(-1).copy()).to(DEV) for t in toks]
    d_recv = [torch.full((max(1, r) * width * esz + 64,), 0xEE, dtype=torch.uint8, device=DEV) for r in inbound]
    torch.cuda.synchronize()
    ptrs = lambda ts: [t.data_ptr() for t in ts]
    hcclx.moe_dispatch(ptrs(d_tok), ptrs(d_dest), ptrs(perm), entries, topk, width, dtype, tabs[1].data_ptr(),
                       tabs[3].data_ptr(), ptrs(d_recv))
    torch.cuda.synchronize()
    for j in range(n):
        got = d_recv[j].cpu().numpy()
        assert np.array_equal(got[:inbound[j] * width * esz].view(npd), recv_want[j][:inbound[j] * width]), j
        assert (got[max(1, inbound[j]) * width * esz:] == 0xEE).all()
    # the experts' results: any function of the received rows; here the rows with their bytes reversed per row pair
    expert = [np.ascontiguousarray(r[:inbound[j] * width].reshape(-1, width)[:, ::-1]).reshape(-1) for j, r in enumerate(recv_want)]
    back = T.run_alltoallv([np.concatenate([e, np.zeros(width, dtype=npd)]) for e in expert], rc, rd, sc, sd,
                           [max(1, k) * width for k in kept], fill=0)
    d_exp = [torch.from_numpy(np.concatenate([e, np.zeros(width, dtype=npd)]).view(np.uint8).copy()).to(DEV) for e in expert]
    d_out = [torch.full((tokens * width * esz + 64,), 0xEE, dtype=torch.uint8, device=DEV) for _ in range(n)]
    torch.cuda.synchronize()
    hcclx.moe_gather_combine(ptrs(d_exp), ptrs(d_dest), ptrs(perm), tokens, topk, width, dtype, tabs[1].data_ptr(),
                             tabs[3].data_ptr(), ptrs(d_out))
    torch.cuda.synchronize()
    for i in range(n):
        want = T.moe_combine(back[i].reshape(-1, width), perms[i], topk, dtype)
        got = d_out[i].cpu().numpy()
        assert np.array_equal(got[:tokens * width * esz].view(npd).reshape(tokens, width).view(np.uint8),
                              want.view(np.uint8)), i
        assert (got[tokens * width * esz:] == 0xEE).all()


def test_errors():
    t = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    p = t.data_ptr()
    with pytest.raises(HcclError) as e:
        hcclx.moe_pack([p], [p], 8, 3, 64, [p])              # entries not a multiple of topk
    assert e.value.code == 1
    with pytest.raises(HcclError) as e:
        hcclx.moe_pack([p], [p], 8, 1, 24, [p])              # rows must be multiples of 16 bytes
    assert e.value.code == 1
    with pytest.raises(HcclError) as e:
        hcclx.moe_pack([p + 4], [p], 8, 1, 64, [p])          # 16-byte aligned buffers
    assert e.value.code == 1
    with pytest.raises(HcclError) as e:
        hcclx.moe_combine([p], [p], 8, 2, 16, T.INT32, [p])  # several rows can only be added as floats
    assert e.value.code == 5
    with pytest.raises(HcclError) as e:
        hcclx.moe_pack([p, 0], [p, p], 8, 1, 64, [p, p])
    assert e.value.code == 2


def test_moe_dispatch_round_trip_at_baseline_size():
    """8 ranks x 4096 tokens x hidden 7168 bf16, Zipf(1.2) destinations, routed on the device: pack, AlltoAllV
    with device tables, AlltoAllV back with the transposed tables, combine: every rank gets its tokens back;
    what rank j receives is, rank by rank, the senders' tokens for j in token order."""
    n, tokens, hidden = 8, 4096, 7168
    rng = np.random.default_rng(0)
    p = 1.0 / np.arange(1, n + 1) ** 1.2
    dests = [rng.choice(n, size=tokens, p=p / p.sum()) for _ in range(n)]
    d_dest = [dev_i32(x) for x in dests]
    toks = [torch.randint(-32768, 32767, (tokens, hidden), device=DEV, dtype=torch.int16) for _ in range(n)]
    packed = [torch.empty(tokens * hidden, device=DEV, dtype=torch.int16) for _ in range(n)]
    tabs = [torch.zeros(n * n, dtype=torch.int64, device=DEV) for _ in range(4)]     # send_counts, sdispls, recv_counts, rdispls
    perm = [torch.empty(tokens, dtype=torch.int32, device=DEV) for _ in range(n)]
    ws = torch.empty(hcclx.moe_workspace_bytes(n, tokens), dtype=torch.uint8, device=DEV)
    inbound = np.zeros(n, dtype=np.int64)
    for i in range(n):
        inbound += np.bincount(dests[i], minlength=n)
    recv = [torch.full((max(1, int(inbound[j])) * hidden,), 0x2222, device=DEV, dtype=torch.int16) for j in range(n)]
    back = [torch.full((tokens * hidden,), 0x3333, device=DEV, dtype=torch.int16) for _ in range(n)]
    out = [torch.full((tokens, hidden), 0x4444, device=DEV, dtype=torch.int16) for _ in range(n)]
    s = torch.cuda.Stream()
    torch.cuda.synchronize()
    st = s.cuda_stream
    ptrs = lambda ts: [t.data_ptr() for t in ts]
    hcclx.moe_route(ptrs(d_dest), tokens, hidden, tabs[0].data_ptr(), tabs[1].data_ptr(), tabs[2].data_ptr(),
                    tabs[3].data_ptr(), ptrs(perm), ws.data_ptr(), stream=st)
    hcclx.moe_pack(ptrs(toks), ptrs(perm), tokens, 1, hidden * 2, ptrs(packed), stream=st)
    hcclx.alltoallv(ptrs(packed), ptrs(recv), tabs[0].data_ptr(), tabs[1].data_ptr(), tabs[3].data_ptr(), T.BFP16,
                    on_device=True, stream=st)
    hcclx.alltoallv(ptrs(recv), ptrs(back), tabs[2].data_ptr(), tabs[3].data_ptr(), tabs[1].data_ptr(), T.BFP16,
                    on_device=True, stream=st)
    hcclx.moe_combine(ptrs(back), ptrs(perm), tokens, 1, hidden, T.BFP16, ptrs(out), stream=st)
    s.synchronize()
    for i in range(n):
        assert torch.equal(out[i], toks[i]), i
    for j in range(n):
        pos = 0
        for i in range(n):
            mine = toks[i][torch.from_numpy(dests[i] == j).to(DEV)].reshape(-1)
            assert torch.equal(recv[j][pos:pos + mine.numel()], mine), (i, j)
            pos += mine.numel()
        assert pos == int(inbound[j]) * hidden


def test_one_pass_round_trip_at_baseline_size():
    """The same configuration through the one-pass entry points: route, dispatch straight into the receive buffers,
    gather-combine straight out of them: every rank gets its tokens back, and the receive buffers hold what the
    AlltoAllV delivers."""
    n, tokens, hidden = 8, 4096, 7168
    rng = np.random.default_rng(1)
    p = 1.0 / np.arange(1, n + 1) ** 1.2
    dests = [rng.choice(n, size=tokens, p=p / p.sum()) for _ in range(n)]
    d_dest = [dev_i32(x) for x in dests]
    toks = [torch.randint(-32768, 32767, (tokens, hidden), device=DEV, dtype=torch.int16) for _ in range(n)]
    tabs = [torch.zeros(n * n, dtype=torch.int64, device=DEV) for _ in range(4)]
    perm = [torch.empty(tokens, dtype=torch.int32, device=DEV) for _ in range(n)]
    ws = torch.empty(hcclx.moe_workspace_bytes(n, tokens), dtype=torch.uint8, device=DEV)
    inbound = np.zeros(n, dtype=np.int64)
    for i in range(n):
        inbound += np.bincount(dests[i], minlength=n)
    recv = [torch.full((max(1, int(inbound[j])) * hidden + 32,), 0x2222, device=DEV, dtype=torch.int16) for j in range(n)]
    out = [torch.full((tokens, hidden), 0x4444, device=DEV, dtype=torch.int16) for _ in range(n)]
    s = torch.cuda.Stream()
    torch.cuda.synchronize()
    st = s.cuda_stream
    ptrs = lambda ts: [t.data_ptr() for t in ts]
    hcclx.moe_route(ptrs(d_dest), tokens, hidden, tabs[0].data_ptr(), tabs[1].data_ptr(), tabs[2].data_ptr(),
                    tabs[3].data_ptr(), ptrs(perm), ws.data_ptr(), stream=st)
    hcclx.moe_dispatch(ptrs(toks), ptrs(d_dest), ptrs(perm), tokens, 1, hidden, T.BFP16, tabs[1].data_ptr(),
                       tabs[3].data_ptr(), ptrs(recv), stream=st)
    hcclx.moe_gather_combine(ptrs(recv), ptrs(d_dest), ptrs(perm), tokens, 1, hidden, T.BFP16, tabs[1].data_ptr(),
                             tabs[3].data_ptr(), ptrs(out), stream=st)
    s.synchronize()
    for i in range(n):
        assert torch.equal(out[i], toks[i]), i
    for j in range(n):
        pos = 0
        for i in range(n):
            mine = toks[i][torch.from_numpy(dests[i] == j).to(DEV)].reshape(-1)
            assert torch.equal(recv[j][pos:pos + mine.numel()], mine), (i, j)
            pos += mine.numel()
        assert pos == int(inbound[j]) * hidden
        assert bool((recv[j][pos:] == 0x2222).all())
