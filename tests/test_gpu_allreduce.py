"""The managed all-reduce and DiLoCo's bucketised averaging
(torchft_amd.allreduce; manager.py:386-456, local_sgd.py:489-556) on the GPU
with a process group simulated by threads, against the CPU checker.

Expected values: the checker's quantize -> all-to-all -> reduce(SUM) ->
all-gather -> dequantize of the same tensors, then the reference's own
``tensor /= num_participants`` (manager.py:451), executed with torch on the GPU
like the reference does (torch divides a CUDA tensor by a Python scalar by
multiplying with the reciprocal, so the CPU quotient can differ in the last bit).
"""

import pytest
import torch
from torch.distributed import ReduceOp

import sim
from sim_pg import SimGroup
from test_gpu_collectives import run_ranks

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ar():
    assert torch.cuda.is_available()
    from torchft_amd import allreduce
    return allreduce


def checker_sum(oracle, peers, ws):
    """what every rank holds after the quantized SUM all-reduce of peers[r] (lists of tensors)"""
    _, _, gathered = sim.allreduce(oracle, [list(t) for t in peers], ws, ReduceOp.SUM)
    out = [torch.zeros_like(t) for t in peers[0]]
    oracle.fused_dequantize_from_fp8(out, gathered, ws)
    return out


def same_bits(a, b):
    if a.dtype == torch.float16:
        # torch's float16 division by a scalar does not keep the sign of a zero everywhere
        a, b = a + 0.0, b + 0.0  # -0 -> +0 in both
    return torch.equal(a.cpu().reshape(-1).view(torch.uint8), b.cpu().reshape(-1).view(torch.uint8))


@pytest.mark.parametrize("fold", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(5000,), (96, 200)])
@pytest.mark.parametrize("ws,absent", [(2, None), (4, 1), (7, None), (6, 3)])
def test_quantized_average(ar, oracle, dtype, shape, ws, absent, fold):
    g = torch.Generator().manual_seed(ws)
    peers = [[(torch.randn(shape, generator=g) * 0.01).to(dtype)] for _ in range(ws)]
    if absent is not None:
        contributed = [[torch.zeros_like(p[0])] if r == absent else p for r, p in enumerate(peers)]
    else:
        contributed = peers
    participants = ws - (absent is not None)
    want = checker_sum(oracle, contributed, ws)[0].cuda()
    want /= participants

    group = SimGroup(ws)
    on_gpu = [p[0].cuda() for p in peers]
    values = [None] * ws

    def rank_fn(r):
        work = ar.allreduce(on_gpu[r], group.rank(r), participants, is_participating=(r != absent),
                            should_quantize=True, fold_normalization=fold)
        assert work.wait()
        values[r] = work.get_future().value()

    run_ranks(ws, rank_fn, group)
    torch.cuda.synchronize()
    for r in range(ws):
        assert values[r] is on_gpu[r]
        assert on_gpu[r].shape == torch.Size(shape)
        assert same_bits(on_gpu[r], want), r
    exact = sum(p[0].double() for p in contributed) / participants
    rel = (on_gpu[0].cpu().double() - exact).abs().mean() / exact.abs().mean()
    assert rel < 0.05


@pytest.mark.parametrize("op", [ReduceOp.SUM, ReduceOp.AVG])
def test_unquantized_branch(ar, op):
    ws = 4
    g = torch.Generator().manual_seed(1)
    peers = [torch.randn(1000, generator=g) for _ in range(ws)]
    want = torch.zeros(1000).cuda()
    for p in peers:
        want += p.cuda()
    if op == ReduceOp.AVG:
        want /= ws
    group = SimGroup(ws)
    on_gpu = [p.cuda() for p in peers]

    def rank_fn(r):
        ar.allreduce(on_gpu[r], group.rank(r), ws, reduce_op=op).wait()

    run_ranks(ws, rank_fn, group)
    torch.cuda.synchronize()
    for r in range(ws):
        assert same_bits(on_gpu[r], want)


@pytest.mark.parametrize("row_width", [None, 256])
def test_bucketized_quantized_average(ar, oracle, row_width):
    ws = 2
    sizes = [(64, 48), (1000,), (7, 33), (2048,), (300,)]
    g = torch.Generator().manual_seed(5)
    peers = [[(torch.randn(s, generator=g) * 0.1).to(torch.bfloat16) for s in sizes] for _ in range(ws)]
    # 3072 + 1000 + 231 elements fill the first bucket exactly, 2048 + 300 the second
    per_bucket = 4303
    buckets = [[0, 1, 2], [3, 4]]
    caps = [4303, 2348]
    total = sum(torch.Size(s).numel() for s in sizes)
    assert caps == [min(per_bucket, total - k * per_bucket) for k in range(2)]

    want = [None] * len(sizes)
    for members, cap in zip(buckets, caps):
        alloc = cap if row_width is None else -(-cap // row_width) * row_width
        flats = []
        for r in range(ws):
            flat = torch.zeros(alloc, dtype=torch.bfloat16)
            off = 0
            for i in members:
                n = peers[r][i].numel()
                flat[off:off + n] = peers[r][i].reshape(-1)
                off += n
            flats.append([flat if row_width is None else flat.view(-1, row_width)])
        red = checker_sum(oracle, flats, ws)[0].cuda()
        red /= ws
        red = red.reshape(-1)
        off = 0
        for i in members:
            n = peers[0][i].numel()
            want[i] = red[off:off + n]
            off += n

    group = SimGroup(ws)
    on_gpu = [[t.cuda() for t in peers[r]] for r in range(ws)]

    def rank_fn(r):
        pg = group.rank(r)
        works = ar.bucketize_and_allreduce(
            on_gpu[r], per_bucket * 2, lambda t: ar.allreduce(t, pg, ws, should_quantize=True),
            row_width=row_width)
        assert len(works) == 2
        for w in works:
            assert w.wait()

    run_ranks(ws, rank_fn, group)
    torch.cuda.synchronize()
    for r in range(ws):
        for i in range(len(sizes)):
            assert on_gpu[r][i].shape == torch.Size(sizes[i])
            assert same_bits(on_gpu[r][i], want[i]), (r, i)
    if row_width is not None:
        # one scale per 256 elements instead of one per element: 8 packed bytes per element become ~1
        from torchft_amd import quantization as q
        flat = torch.zeros(4608, dtype=torch.bfloat16, device="cuda")
        assert q.fused_quantize_into_fp8([flat.view(-1, 256)], ws).numel() * 7 < \
            q.fused_quantize_into_fp8([flat], ws).numel()
