"""Host orchestration of the quantized collectives (torchft_amd.collectives)
against the CPU checker, with a process group simulated by threads on one GPU.

Mirrors torchft/collectives_test.py:54-212: every rank holds its own tensors,
`allreduce_quantized` leaves the reduced values in place, and
`reduce_scatter_quantized` fills the tensor from `allocate_reduce_scatter_output`.
The expected bytes come from running the same data flow on the CPU checker; the
reference's own criterion (mean relative error against the unquantized
reduction <= 0.04 / 0.05, :187, :208) is asserted as well.
"""

import threading

import pytest
import torch
from torch.distributed import ReduceOp, ReduceScatterOptions

import sim
from sim_pg import SimGroup

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def coll():
    assert torch.cuda.is_available()
    from torchft_amd import collectives
    return collectives


def run_ranks(ws, fn, group=None):
    """One thread per rank; a failing rank breaks the group's barrier so that the
    other ranks fail too instead of waiting."""
    errors = []

    def body(r):
        try:
            torch.cuda.set_device(0)
            fn(r)
        except BaseException as e:  # noqa: BLE001
            errors.append(e)
            if group is not None:
                group.barrier.abort()

    threads = [threading.Thread(target=body, args=(r,)) for r in range(ws)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
        assert not t.is_alive(), "rank thread hung"
    real = [e for e in errors if not isinstance(e, threading.BrokenBarrierError)]
    if real or errors:
        raise (real or errors)[0]


def make_peers(ws, dtype, shapes, seed, mult):
    g = torch.Generator().manual_seed(seed)
    return [[(torch.rand(s, generator=g) * mult).to(dtype) for s in shapes] for _ in range(ws)]


def mean_rel(actual, expected):
    return ((expected - actual).abs() / (expected.float() + 1e-7)).mean().item()


SHAPES = [(64, 32), (2048,), (3, 700), (17, 128)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("op", [ReduceOp.AVG, ReduceOp.SUM])
@pytest.mark.parametrize("ws,mult", [(2, 1.0), (4, 100.0), (8, 1000.0)])
def test_allreduce_quantized(coll, oracle, dtype, op, ws, mult):
    peers = make_peers(ws, dtype, SHAPES, ws, mult)
    _, _, gathered = sim.allreduce(oracle, [list(t) for t in peers], ws, op)
    expected = [torch.zeros_like(t) for t in peers[0]]
    oracle.fused_dequantize_from_fp8(expected, gathered, ws)

    group = SimGroup(ws)
    on_gpu = [[t.cuda() for t in peers[r]] for r in range(ws)]
    side = [torch.cuda.Stream() for _ in range(ws)]

    def rank_fn(r):
        # explicit stream on even ranks, library-created stream on odd ranks
        stream = side[r] if r % 2 == 0 else None
        work = coll.allreduce_quantized(on_gpu[r], op, group.rank(r), stream)
        work.wait()
        work.get_future().wait()

    run_ranks(ws, rank_fn, group)
    torch.cuda.synchronize()
    exact = torch.cat([sum(p[i].double() for p in peers).reshape(-1) for i in range(len(SHAPES))])
    if op == ReduceOp.AVG:
        exact = exact / ws
    for r in range(ws):
        got = on_gpu[r]
        for i, e in enumerate(expected):
            g = got[i].cpu().reshape(e.shape)
            assert torch.equal(g.view(-1).view(torch.uint8), e.reshape(-1).view(torch.uint8)), (r, i)
        flat = torch.cat([t.cpu().double().reshape(-1) for t in got])
        assert mean_rel(flat, exact) <= 0.04


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("op", [ReduceOp.AVG, ReduceOp.SUM])
@pytest.mark.parametrize("ws", [2, 4])
def test_reduce_scatter_quantized(coll, oracle, dtype, op, ws):
    shapes = [(64, 32), (1030,), (5, 700)]  # 1030 and 5 are not multiples of ws = 4
    peers = make_peers(ws, dtype, shapes, 100 + ws, 10.0)
    qs = sim.quantize_peers(oracle, [list(t) for t in peers], ws)

    group = SimGroup(ws)
    on_gpu = [[t.cuda() for t in peers[r]] for r in range(ws)]
    outputs = [None] * ws

    def rank_fn(r):
        out, padded = coll.allocate_reduce_scatter_output(on_gpu[r], ws)
        assert padded == coll.get_padded_sizes(on_gpu[r], ws)
        opts = ReduceScatterOptions()
        opts.reduceOp = op
        work = coll.reduce_scatter_quantized(out, on_gpu[r], opts, group.rank(r))
        work.get_future().wait()
        outputs[r] = out

    run_ranks(ws, rank_fn, group)
    torch.cuda.synchronize()
    padded = coll.get_padded_sizes(peers[0], ws)
    for r in range(ws):
        recv = sim.recv_buffer(qs, r, ws)
        oracle.fused_reduce_fp8(list(peers[0]), recv, ws, r, op)
        slot = recv.numel() // ws
        shares = [torch.zeros((p[0] // ws,) + tuple(p[1:]), dtype=dtype) for p in padded]
        oracle.fused_dequantize_from_fp8(shares, recv[r * slot:(r + 1) * slot].clone(), 1)
        want = torch.cat([s.reshape(-1) for s in shares])
        got = outputs[r].cpu()
        assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), r
        # against the unquantized reduce-scatter of the row-padded inputs
        parts = []
        for i, p in enumerate(padded):
            tot = sum(pe[i].double().reshape(pe[i].shape[0], -1) for pe in peers)
            pad = torch.zeros(p[0] - tot.shape[0], tot.shape[1], dtype=torch.double)
            tot = torch.cat([tot, pad])
            parts.append(tot[r * (p[0] // ws):(r + 1) * (p[0] // ws)].reshape(-1))
        exact = torch.cat(parts) / (ws if op == ReduceOp.AVG else 1)
        nz = exact != 0
        assert mean_rel(got.double()[nz], exact[nz]) <= 0.05


def test_unsupported_ops_raise(coll):
    group = SimGroup(1)
    t = [torch.ones(4, 4, device="cuda")]
    for op in (ReduceOp.MAX, ReduceOp.MIN, ReduceOp.PRODUCT):
        with pytest.raises(NotImplementedError, match="only AVG and SUM are supported"):
            coll.allreduce_quantized(t, op, group.rank(0))
        out, _ = coll.allocate_reduce_scatter_output(t, 1)
        with pytest.raises(NotImplementedError, match="only AVG and SUM are supported"):
            coll.reduce_scatter_quantized(out, t, op, group.rank(0))


def test_world_size_one_is_quantize_dequantize(coll, oracle):
    """With one rank the collective is quantize -> reduce(self) -> dequantize."""
    x = torch.randn(33, 257).to(torch.bfloat16)
    want = [x.clone()]
    q = oracle.fused_quantize_into_fp8(list(want), 1)
    oracle.fused_reduce_fp8(list(want), q, 1, 0, ReduceOp.SUM)
    oracle.fused_dequantize_from_fp8(want, q, 1)
    got = [x.cuda()]
    work = coll.allreduce_quantized(got, ReduceOp.SUM, SimGroup(1).rank(0))
    work.wait()
    torch.cuda.synchronize()
    assert torch.equal(got[0].cpu().view(torch.int16), want[0].view(torch.int16))


@pytest.fixture(scope="module")
def rccl_group_of_one():
    """A real torch.distributed process group over RCCL (backend "nccl") with this
    process as its only rank: the work objects, futures and callback threads are
    ProcessGroupNCCL's own, only the exchange itself is trivial."""
    import socket

    import torch.distributed as dist

    if not dist.is_nccl_available():
        pytest.skip("torch.distributed has no nccl (RCCL) backend")
    assert not dist.is_initialized()
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
    torch.cuda.set_device(0)
    dist.init_process_group("nccl", init_method=f"tcp://127.0.0.1:{port}", rank=0, world_size=1,
                            device_id=torch.device("cuda:0"))
    try:
        yield dist.distributed_c10d._get_default_group()
    finally:
        dist.destroy_process_group()


@pytest.mark.parametrize("op", [ReduceOp.SUM, ReduceOp.AVG])
def test_collectives_over_rccl_group_of_one(coll, oracle, rccl_group_of_one, op):
    """allreduce_quantized, reduce_scatter_quantized and the managed all-reduce through
    c10d's ProcessGroup API (alltoall_base, allgather_into_tensor_coalesced, Work,
    Future.add_done_callback), bytes against the CPU checker."""
    from torchft_amd.allreduce import allreduce

    pg = rccl_group_of_one
    g = torch.Generator().manual_seed(5)
    cpu = [torch.randn(300, 512, generator=g).to(torch.bfloat16),
           torch.randn(1000, generator=g).to(torch.bfloat16),
           torch.randn(7, 33, generator=g).to(torch.bfloat16)]
    want = [t.clone() for t in cpu]
    packed = oracle.fused_quantize_into_fp8(want, 1)  # 1-D -> [k, 1] in `want`
    oracle.fused_reduce_fp8(want, packed, 1, 0, op)
    oracle.fused_dequantize_from_fp8(want, packed, 1)

    stream = torch.cuda.Stream()
    got = [t.cuda() for t in cpu]
    work = coll.allreduce_quantized(got, op, pg, stream)
    work.wait()
    work.get_future().wait()
    stream.synchronize()
    for a, e in zip(got, want):
        assert torch.equal(a.cpu().reshape(-1).view(torch.int16), e.reshape(-1).view(torch.int16))

    src = [t.cuda() for t in cpu]
    out, _ = coll.allocate_reduce_scatter_output(src, 1)
    work = coll.reduce_scatter_quantized(out, src, op, pg, stream)
    work.wait()
    work.get_future().wait()
    stream.synchronize()
    flat = torch.cat([e.reshape(-1) for e in want])
    assert torch.equal(out.cpu().view(torch.int16), flat.view(torch.int16))

    # the managed all-reduce: AVG becomes SUM for the collective, then / num_participants
    x = cpu[0].cuda()
    w = allreduce(x, pg, num_participants=1, should_quantize=True, reduce_op=op)
    w.wait()
    torch.cuda.synchronize()
    want_sum = [cpu[0].clone()]
    p = oracle.fused_quantize_into_fp8(want_sum, 1)
    oracle.fused_reduce_fp8(want_sum, p, 1, 0, ReduceOp.SUM)
    oracle.fused_dequantize_from_fp8(want_sum, p, 1)
    assert torch.equal(x.cpu().view(torch.int16), want_sum[0].view(torch.int16))
