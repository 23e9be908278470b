"""Parity of the HIP path (through torchft_amd.quantization -> ctypes ->
libtftq.so) with the CPU checker, on a gfx950 GPU.

Bar: every byte of the packed buffer after quantize and after reduce, and every
element after dequantize, equals the checker's.  (The stated tolerance for
reduce / dequantize is one fp8-e4m3 ULP of the row scale, 32 / s; the kernels
reproduce the summation order and use an exact division, so the tests demand
equality and report nothing looser.)
"""

import ctypes
import json
import os

import pytest
import torch
from torch.distributed import ReduceOp

import sim
import workloads

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
NT = min(16, os.cpu_count() or 1)


@pytest.fixture(scope="module")
def q():
    assert torch.cuda.is_available(), "GPU tests need a gfx950 device"
    from torchft_amd import _lib, quantization
    assert _lib.load().tftq_check_device(0) == 0, "device is not gfx950"
    return quantization


def dev(ts):
    """Copies to the GPU that keep the strides (`.cuda()` makes a tensor with gaps contiguous)."""
    out = []
    for t in ts:
        if t.numel() == 0 or t.is_contiguous():
            out.append(t.cuda())
        else:
            d = torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device="cuda")
            d.copy_(t)
            out.append(d)
    return out


def same_bytes(a: torch.Tensor, b: torch.Tensor, what=""):
    a = a.detach().cpu().contiguous().view(-1).view(torch.uint8)
    b = b.detach().cpu().contiguous().view(-1).view(torch.uint8)
    assert a.numel() == b.numel(), what
    if not torch.equal(a, b):
        bad = (a != b).nonzero().flatten()
        raise AssertionError(f"{what}: {bad.numel()} bytes differ, first at {bad[:8].tolist()}: "
                             f"got {a[bad[:8]].tolist()} want {b[bad[:8]].tolist()}")


def full_check(q, oracle, peers_cpu, ws, op, ranks=None):
    """Quantize every peer, reduce on `ranks`, dequantize; all against the checker."""
    peers_gpu = [dev(t) for t in peers_cpu]
    qs_g, red_g, gath_g = sim.allreduce(q, peers_gpu, ws, op, ranks)
    qs_c, red_c, gath_c = sim.allreduce(oracle, [list(t) for t in peers_cpu], ws, op, ranks, nthreads=NT)
    for p, (a, b) in enumerate(zip(qs_g, qs_c)):
        same_bytes(a, b, f"quantize peer {p}")
    for r in red_c:
        same_bytes(red_g[r], red_c[r], f"reduce rank {r}")
    if ranks is None:
        outs_g = [torch.full_like(t, 7.0) for t in peers_gpu[0]]
        outs_c = [torch.full_like(t, 7.0) for t in peers_cpu[0]]
        q.fused_dequantize_from_fp8(outs_g, gath_g, ws)
        oracle.fused_dequantize_from_fp8(outs_c, gath_c, ws, nthreads=NT)
        for i, (a, b) in enumerate(zip(outs_g, outs_c)):
            same_bytes(a, b, f"dequantize tensor {i}")
        return outs_g
    return None


# ---- the fp8 convert instruction against the checker ------------------------
def test_hw_fp8_convert_matches_checker(q, oracle):
    """Rows whose amax is exactly 448 get scale 1.0, so the codes are the raw
    hardware conversion of the inputs: all bf16 patterns up to 464 in magnitude,
    a dense sweep around the overflow boundary, ties and subnormals."""
    allbf = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).to(torch.float32)
    allbf = allbf[allbf.abs() <= 448.0]
    edge = torch.linspace(440.0, 448.0, 20001)
    sub = torch.linspace(0, 2 ** -5, 40001)
    g = torch.Generator().manual_seed(9)
    rnd = (torch.rand(300000, generator=g) * 2 - 1) * 448.0
    ties = torch.tensor([17.0, 19.0, 1.5 * 2 ** -9, 2.5 * 2 ** -9, 2 ** -10, 2 ** -10 * 1.0001,
                         2 ** -6 * 0.9999, 0.0, -0.0, 1e-30, -1e-30, 1e-45])
    x = torch.cat([allbf, edge, -edge, sub, -sub, rnd, ties])
    n = 1023
    rows = -(-x.numel() // n)
    x = torch.cat([x, torch.zeros(rows * n - x.numel())]).view(rows, n)
    x = torch.cat([x, torch.full((rows, 1), 448.0)], dim=1).contiguous()  # amax = 448 -> s = 1
    got = q.fused_quantize_into_fp8([x.cuda()], 1)
    want = oracle.fused_quantize_into_fp8([x], 1)
    same_bytes(got, want, "hw convert")
    assert (want.view(rows, -1)[:, :4].contiguous().view(torch.float32) == 1.0).all()


# ---- golden vectors through the GPU ------------------------------------------
def test_golden_vectors_gpu(q):
    kat = json.load(open(os.path.join(HERE, "golden", "kat.json")))

    def from_hex(h, dtype=torch.uint8):
        return torch.frombuffer(bytearray(bytes.fromhex(h)), dtype=dtype).clone()

    k = kat["kat1_quantize"]
    x = from_hex(k["input_hex"]).view(torch.float32).view(1, 4).cuda()
    assert bytes(q.fused_quantize_into_fp8([x], 1).cpu().tolist()).hex() == k["packed_hex"]
    for name, op in (("sum", ReduceOp.SUM), ("avg", ReduceOp.AVG)):
        k = kat[f"kat2_reduce_{name}"]
        recv = from_hex(k["recv_hex"]).cuda()
        q.fused_reduce_fp8([torch.empty(2, 4, device="cuda")], recv, 2, 0, op)
        assert bytes(recv.cpu().tolist()).hex() == k["reduced_hex"]
        out = torch.zeros(1, 4, device="cuda")
        q.fused_dequantize_from_fp8([out], recv[:8].clone(), 1)
        assert bytes(out.cpu().view(torch.uint8).flatten().tolist()).hex() == k["dequant_slot0_hex"]
    for key in ("kat3_zero_row", "kat3_n1_rows"):
        k = kat[key]
        x = from_hex(k["input_hex"]).view(torch.float32).view(*k["shape"]).cuda()
        assert bytes(q.fused_quantize_into_fp8([x], 1).cpu().tolist()).hex() == k["packed_hex"]
    DT = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}
    for dt in DT:
        k = kat[f"odd_{dt}"]
        ins = [from_hex(h).view(DT[dt]).view(*s).cuda() for h, s in zip(k["inputs_hex"], k["shapes"])]
        buf = q.fused_quantize_into_fp8(list(ins), k["ws"])
        assert bytes(buf.cpu().tolist()).hex() == k["packed_hex"]
        red = buf.clone()
        q.fused_reduce_fp8(list(ins), red, k["ws"], 2, ReduceOp.AVG)
        assert bytes(red.cpu().tolist()).hex() == k["reduced_rank2_avg_hex"]
        outs = [torch.zeros_like(t) for t in ins]
        q.fused_dequantize_from_fp8(list(outs), buf, k["ws"])
        for o, h in zip(outs, k["dequant_hex"]):
            assert bytes(o.cpu().contiguous().view(torch.uint8).flatten().tolist()).hex() == h


# ---- the five benchmark configurations ---------------------------------------------------
def test_cfg1_cpu_plumbing_shapes(q, oracle):
    peers = [workloads.cfg1(s) for s in (0, 1)]
    outs = full_check(q, oracle, peers, 2, ReduceOp.SUM)
    ref = peers[0][0] + peers[1][0]
    rowmax = ref.abs().amax(dim=1, keepdim=True)
    assert ((outs[0].cpu() - ref).abs() / rowmax).max() < 0.13


def test_cfg2_bf16_4096x4096_avg(q, oracle):
    peers = [workloads.cfg2(s) for s in range(8)]
    full_check(q, oracle, peers, 8, ReduceOp.AVG)


@pytest.mark.parametrize("op", [ReduceOp.SUM, ReduceOp.AVG])
def test_cfg3_llama_layer_eighth(q, oracle, op):
    """All nine tensors at full row length, one eighth of the rows."""
    peers = [workloads.cfg3(s, scale_rows=0.125) for s in range(8)]
    full_check(q, oracle, peers, 8, op)


def test_cfg4_diloco_two_layers(q, oracle):
    peers = [workloads.cfg4(s, layers=2, vocab=4000) for s in range(4)]
    assert len(peers[0]) == 21  # more than 16 tensors: descriptor table in device memory
    full_check(q, oracle, peers, 4, ReduceOp.AVG)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_cfg5_edge_case_stress(q, oracle, dtype):
    shapes = workloads.cfg5_shapes(600)
    peers = [workloads.cfg5(s, dtype, shapes) for s in range(16)]
    full_check(q, oracle, peers, 16, ReduceOp.SUM, ranks=[0, 7, 15])
    full_check(q, oracle, peers[:2] * 8, 16, ReduceOp.SUM)


# ---- the reference's own test matrix (quantization_test.py:107-131) ---------------
def _views(size):
    return [(m, size // m) for m in range(1 if size % 2 == 0 else 2, size) if size % m == 0]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("op", [ReduceOp.AVG, ReduceOp.SUM])
@pytest.mark.parametrize("tensor_size,multiplier", [(128, 1.0), (512, 100.0), (4096, 1000.0)])
def test_reference_matrix(q, oracle, dtype, op, tensor_size, multiplier):
    """Shapes and inputs of QuantizationTest.run_test: uniform [0, multiplier),
    three tensors, every 2-D factorisation; world size 2 with identical peers.
    Checked bit for bit against the checker and with the reference's own
    criterion (mean relative error <= 0.05, :96-105)."""
    g = torch.Generator().manual_seed(tensor_size)
    inp = (torch.rand(3 * tensor_size, generator=g) * multiplier).to(dtype)
    views = _views(tensor_size)
    # every view appears in some combination (the full cross product has len(views)^3 entries)
    combos = [(views[i], views[(i * 7 + 3) % len(views)], views[-1 - i]) for i in range(len(views))]
    for split in combos:
        ins = [t.view(*s).clone() for s, t in zip(split, torch.split(inp, tensor_size))]
        outs = full_check(q, oracle, [ins, ins], 2, op)
        out = torch.cat([o.reshape(-1) for o in outs]).cpu().float()
        ref = inp.float() * (2 if op == ReduceOp.SUM else 1)
        assert not torch.isnan(out).any()
        assert ((ref - out).abs() / (ref + 1e-7)).mean() <= 0.05


# ---- layouts the fast paths do not take ----------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_strided_and_misaligned_inputs(q, oracle, dtype):
    g = torch.Generator().manual_seed(11)
    base = (torch.randn(300, 700, generator=g)).to(dtype)
    flat = (torch.randn(5000, generator=g)).to(dtype)
    cpu_views = [base[::2, 1:600:3], base.t()[3:170], base[5:6, :], flat[1:4097].view(64, 64), flat[3:3 + 77]]
    gbase, gflat = base.cuda(), flat.cuda()
    gpu_views = [gbase[::2, 1:600:3], gbase.t()[3:170], gbase[5:6, :], gflat[1:4097].view(64, 64), gflat[3:3 + 77]]
    a = q.fused_quantize_into_fp8(list(gpu_views), 4)
    b = oracle.fused_quantize_into_fp8(list(cpu_views), 4)
    same_bytes(a, b, "strided quantize")
    # dequantize into strided, non-overlapping destinations
    ob, of = torch.zeros(300, 700, dtype=dtype), torch.zeros(5000, dtype=dtype)
    gob, gof = ob.cuda(), of.cuda()
    cpu_out = [ob[::2, 1:600:3], of[1:4097].view(64, 64)]
    gpu_out = [gob[::2, 1:600:3], gof[1:4097].view(64, 64)]
    src_c = [cpu_views[0], cpu_views[3]]
    buf = oracle.fused_quantize_into_fp8(list(src_c), 4)
    oracle.fused_dequantize_from_fp8(list(cpu_out), buf, 4)
    q.fused_dequantize_from_fp8(list(gpu_out), buf.cuda(), 4)
    same_bytes(gob, ob, "strided dequantize base")
    same_bytes(gof, of, "strided dequantize flat")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_unaligned_rows_and_tails(q, oracle, dtype):
    """Contiguous rows whose start or length is not a multiple of 16 bytes take the
    vector kinds with element-aligned 16-byte accesses and a per-element tail."""
    g = torch.Generator().manual_seed(17)
    esz = 4 if dtype == torch.float32 else 2
    cases = []
    for n in (33, 67, 130, 515, 1023, 4092, 4099, 9001):
        flat = torch.randn(6 * n + 7, generator=g).to(dtype)
        for off in (0, 1, 3):
            cases.append((flat, off, 5, n))
    cpu_views = [f[o:o + m * n].view(m, n) for f, o, m, n in cases]
    gpu_flats = {id(f): f.cuda() for f, _, _, _ in cases}
    gpu_views = [gpu_flats[id(f)][o:o + m * n].view(m, n) for f, o, m, n in cases]
    assert any(v.data_ptr() % 16 != 0 for v in gpu_views)
    for ws in (1, 4):
        a = q.fused_quantize_into_fp8(list(gpu_views), ws)
        b = oracle.fused_quantize_into_fp8(list(cpu_views), ws)
        same_bytes(a, b, f"unaligned quantize ws={ws}")
        red_g, red_c = a.clone(), b.clone()
        q.fused_reduce_fp8(list(gpu_views), red_g, ws, ws - 1, ReduceOp.AVG)
        oracle.fused_reduce_fp8(list(cpu_views), red_c, ws, ws - 1, ReduceOp.AVG)
        same_bytes(red_g, red_c, f"unaligned reduce ws={ws}")
        # dequantize into fresh unaligned destinations (distinct storage per case)
        out_c = [torch.full((m * n + 8,), 5.0, dtype=dtype) for _, _, m, n in cases]
        out_g = [t.cuda() for t in out_c]
        dst_c = [t[o:o + m * n].view(m, n) for t, (_, o, m, n) in zip(out_c, cases)]
        dst_g = [t[o:o + m * n].view(m, n) for t, (_, o, m, n) in zip(out_g, cases)]
        oracle.fused_dequantize_from_fp8(list(dst_c), b, ws)
        q.fused_dequantize_from_fp8(list(dst_g), a, ws)
        for i, (x, y) in enumerate(zip(out_g, out_c)):
            same_bytes(x, y, f"unaligned dequantize case {i} ws={ws}")  # guard elements included


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_dequantize_rows_through_lds_spans(q, oracle, dtype):
    """Contiguous rows that do not start and end on 64-byte boundaries are dequantized into
    LDS and written as one span per workgroup: row lengths on both sides of every team limit
    (512 B, 1, 2, 4, 8, 16 KB), row counts that leave the last workgroup partly filled,
    destinations at dword and at odd element offsets inside a 128-byte line, guard elements
    around every destination, and scales outside the range of the fast division in some rows."""
    g = torch.Generator().manual_seed(23)
    esz = 4 if dtype == torch.float32 else 2
    cases = []  # (m, n, element offset of the destination)
    # (70 to 12002: 16-bit rows of an odd number of columns, whose spans start and end at even bytes only)
    for row_bytes in (68, 70, 202, 500, 516, 1000, 1002, 1028, 2000, 2052, 3000, 3002, 4092, 4100, 6000, 6002, 8188,
                      8196, 12000, 12002, 16380, 16388):
        n = row_bytes // esz
        for m, off in ((37, 0), (9, 2 * (4 // esz)), (70, 30 * (4 // esz) + 64), (3, 1)):
            cases.append((m, n, off))
    # rows of 1 to 31 whole vectors: several rows per lane, a workgroup's rows in two halves
    # (22 to 490: rows that are not whole vectors, 16-bit ones of an odd number of columns among them)
    for row_bytes, m in ((16, 5000), (48, 3), (48, 2500), (80, 1500), (144, 700), (272, 300), (400, 333), (496, 130),
                         (22, 3000), (36, 2000), (88, 1500), (120, 1100), (202, 800), (346, 400), (490, 150)):
        for off in (0, 4 // esz, 25 * (4 // esz), 1):
            cases.append((m, row_bytes // esz, off))
    cpu_src = []
    for m, n, _ in cases:
        t = torch.randn(m, n, generator=g) * 0.3
        t[m // 2] *= 1e-30  # a scale beyond the fast division: plain divide in that row
        if dtype == torch.float16:
            t[m // 2] = 0.0
            t[m // 2, 0] = 6e-8
        if n < 16:
            t[0] = 0.0  # an all-zero row
        cpu_src.append(t.to(dtype))
    for ws in (1, 4):
        b = oracle.fused_quantize_into_fp8(list(cpu_src), ws)
        a = q.fused_quantize_into_fp8([t.cuda() for t in cpu_src], ws)
        same_bytes(a, b, f"quantize ws={ws}")
        out_c = [torch.full((m * n + off + 40,), 5.0, dtype=dtype) for m, n, off in cases]
        out_g = [t.cuda() for t in out_c]
        dst_c = [t[off:off + m * n].view(m, n) for t, (m, n, off) in zip(out_c, cases)]
        dst_g = [t[off:off + m * n].view(m, n) for t, (m, n, off) in zip(out_g, cases)]
        oracle.fused_dequantize_from_fp8(list(dst_c), b, ws)
        q.fused_dequantize_from_fp8(list(dst_g), a, ws)
        for i, (x, y) in enumerate(zip(out_g, out_c)):
            same_bytes(x, y, f"dequantize case {cases[i]} ws={ws}")
        if dtype == torch.float16:  # torch's own division does not treat the sign of fp16 zeros uniformly
            continue
        # the same rows as a short list (descriptors in the kernel arguments), with the division folded in
        pick = list(range(5, len(cases), 7))[:12]
        b2 = oracle.fused_quantize_into_fp8([cpu_src[i] for i in pick], ws)
        a2 = q.fused_quantize_into_fp8([cpu_src[i].cuda() for i in pick], ws)
        same_bytes(a2, b2, f"quantize short list ws={ws}")
        o1 = [torch.full_like(dst_g[i], 3.0) for i in pick]
        o2 = [torch.full_like(dst_g[i], 3.0) for i in pick]
        q.fused_dequantize_from_fp8(o1, a2, ws)
        for t in o1:
            t /= 3
        q.fused_dequantize_from_fp8(o2, a2, ws, divide_by=3)
        for i, (x, y) in zip(pick, zip(o2, o1)):
            same_bytes(x, y, f"dequantize with division case {cases[i]} ws={ws}")


@pytest.mark.parametrize("ws,op", [(1, ReduceOp.SUM), (3, ReduceOp.AVG), (5, ReduceOp.SUM),
                                   (6, ReduceOp.AVG), (70, ReduceOp.AVG), (64, ReduceOp.SUM)])
def test_group_sizes(q, oracle, ws, op):
    g = torch.Generator().manual_seed(ws)
    shapes = [(37, 256), (5, 4096), (130,), (3, 14336), (9, 33), (2, 1024)]
    peers = [[(torch.randn(s, generator=g) * (1 + p % 5)).to(torch.bfloat16) for s in shapes]
             for p in range(ws)]
    ranks = None if ws <= 6 else [0, ws // 2, ws - 1]
    full_check(q, oracle, peers, ws, op, ranks)


@pytest.mark.parametrize("ws,op", [(1, ReduceOp.SUM), (2, ReduceOp.AVG), (2, ReduceOp.SUM), (3, ReduceOp.AVG),
                                   (4, ReduceOp.AVG), (4, ReduceOp.SUM)])
def test_small_groups_several_rows_at_once(q, oracle, ws, op):
    """Groups of up to four peers: a team of 64 or 256 lanes reduces two or four rows at
    once.  Row lengths on both sides of every team/vector-count boundary, rows per slot
    that are not multiples of two or four (1, 2, 3, 5, 7, 9), a zero row and a row whose
    scale needs the plain divide in the middle of a set."""
    g = torch.Generator().manual_seed(300 + ws)
    cols = [516, 600, 1024, 1028, 1500, 2048, 2052, 3000, 4096, 4100, 6000, 8192, 8196, 9000]
    slot_rows = [1, 2, 3, 5, 7, 9]
    shapes = [(slot_rows[i % 6] * ws - (i % 2 if ws > 1 else 0), c) for i, c in enumerate(cols)]
    peers = []
    for p in range(ws):
        ts = []
        for r, c in shapes:
            x = torch.randn(r, c, generator=g) * (1 + p)
            if r > 1:
                x[1] *= 1e-30
            if r > 2:
                x[2] = 0.0
            ts.append(x.to(torch.bfloat16))
        peers.append(ts)
    full_check(q, oracle, peers, ws, op)


def test_average_over_a_very_large_group(q, oracle):
    """Group sizes from 1024 on that are not powers of two divide with the plain IEEE
    divide (smaller ones with the three-operation quotient, powers of two with a
    multiplication)."""
    g = torch.Generator().manual_seed(77)
    shapes = [(3, 300), (40,), (2, 5000)]
    base = [[(torch.randn(s, generator=g) * (1 + p)).to(torch.bfloat16) for s in shapes] for p in range(4)]
    for ws in (1030, 1023):
        peers = [base[p % 4] for p in range(ws)]
        full_check(q, oracle, peers, ws, ReduceOp.AVG, ranks=[0, ws // 2, ws - 1])


@pytest.mark.parametrize("ws,op", [(1, ReduceOp.SUM), (2, ReduceOp.AVG), (3, ReduceOp.AVG), (4, ReduceOp.SUM),
                                   (8, ReduceOp.AVG), (16, ReduceOp.SUM), (33, ReduceOp.AVG), (70, ReduceOp.AVG),
                                   (1030, ReduceOp.AVG)])
def test_group_sizes_on_long_lists(q, oracle, ws, op):
    """Lists of more than 16 tensors: reduce numbers its work in quarters of workgroups, one
    wavefront each, so wavefronts of one workgroup work on different tensors.  Every lane
    mapping of reduce, tensors of one row and of many, empty tensors in between, rows that
    take the plain divide, every group-size path (several rows at once for small groups,
    coefficients through lanes, more peers than lanes, the plain-divide average)."""
    g = torch.Generator().manual_seed(1000 + ws)
    shapes = [(1, 40), (3, 12), (130,), (2, 100), (1, 200), (0, 7), (5, 400), (1, 700), (70, 3), (2, 2100),
              (1, 4100), (9, 64), (300, 1), (1, 33), (2, 130), (700, 9), (1, 1030), (3, 260), (40, 40),
              (1, 17000), (6, 520), (1, 5), (2, 2048)]
    if ws > 100:
        shapes = shapes[:19]
    base = [[(torch.randn(s, generator=g) * (1 + p)).to(torch.bfloat16) for s in shapes] for p in range(min(ws, 5))]
    for t in base[0]:
        if t.dim() == 2 and t.shape[0] > 1:
            t[1] *= 1e-30  # a scale beyond the fast division
    peers = [base[p % len(base)] for p in range(ws)]
    ranks = None if ws <= 4 else [0, ws // 2, ws - 1]
    full_check(q, oracle, peers, ws, op, ranks)


@pytest.mark.parametrize("ws,op", [(2, ReduceOp.AVG), (8, ReduceOp.SUM), (16, ReduceOp.AVG), (24, ReduceOp.SUM),
                                   (40, ReduceOp.AVG)])
def test_short_rows_all_team_sizes(q, oracle, ws, op):
    """Rows of 17 ... 600 columns: teams of 8, 16 and 32 lanes in reduce, several rows per
    wavefront, row counts that leave the last workgroup partly empty, group sizes below and
    above the team size, and some rows whose scale needs the plain divide."""
    g = torch.Generator().manual_seed(100 + ws)
    cols = [17, 20, 36, 64, 100, 128, 131, 200, 256, 257, 300, 500, 512, 513, 600]
    rows = [ws * 3 + 5, 45, ws + 1]
    shapes = [(rows[i % 3], c) for i, c in enumerate(cols)]
    peers = []
    for p in range(ws):
        ts = []
        for r, c in shapes:
            x = torch.randn(r, c, generator=g) * (1 + p % 3)
            x[1] *= 1e-30  # row scale beyond 2^64: the exact fallback inside a shared wavefront
            x[min(3, r - 1)] = 0.0
            ts.append(x)
        peers.append(ts)
    ranks = None if ws <= 8 else [0, ws - 1]
    full_check(q, oracle, peers, ws, op, ranks)
    half = [[t.to(torch.bfloat16) for t in ts] for ts in peers]
    full_check(q, oracle, half, ws, op, [ws // 2])


@pytest.mark.parametrize("ws,op", [(1, ReduceOp.SUM), (2, ReduceOp.AVG), (3, ReduceOp.SUM), (4, ReduceOp.AVG),
                                   (5, ReduceOp.AVG), (7, ReduceOp.SUM), (8, ReduceOp.AVG), (9, ReduceOp.SUM),
                                   (12, ReduceOp.AVG), (15, ReduceOp.SUM), (16, ReduceOp.AVG), (17, ReduceOp.AVG)])
def test_rows_of_13_to_64_columns(q, oracle, ws, op):
    """Every row length from 13 to 64 columns (reduce: a lane per row up to 16 columns, pairs of
    lanes up to 32, teams of 4 lanes above, one vector per lane, every peer's vector in flight at
    once in groups of up to 2, 4, 8 and 16 peers; a lane per row with batches of peers in larger
    groups), row counts that leave the last wavefront and the last workgroup partly or wholly
    without rows, rows whose scale needs the plain divide next to rows that do not, rows of
    zeros, and rows in which every peer holds -0."""
    g = torch.Generator().manual_seed(1700 + ws)
    rows = [1, ws, ws * 15 + 1, ws * 16, ws * 33 + 2, ws * 70 + 3, ws * 129]
    shapes = [(rows[c % len(rows)], c) for c in range(13, 65)]
    peers = []
    for p in range(ws):
        ts = []
        for r, c in shapes:
            x = torch.randn(r, c, generator=g) * (1 + p % 3)
            if r > 4:
                x[1] *= 1e-30
                x[2] = 0.0
                x[3] = -0.0
                x[4, ::2] = -0.0
            ts.append(x)
        peers.append(ts)
    full_check(q, oracle, peers, ws, op, None if ws <= 4 else [0, ws // 2, ws - 1])
    half = [[t.to(torch.bfloat16) for t in ts] for ts in peers]
    full_check(q, oracle, half, ws, op, [ws - 1])


@pytest.mark.parametrize("ws,op", [(2, ReduceOp.AVG), (8, ReduceOp.SUM), (8, ReduceOp.AVG), (16, ReduceOp.SUM),
                                   (17, ReduceOp.AVG), (32, ReduceOp.SUM), (33, ReduceOp.AVG), (64, ReduceOp.SUM),
                                   (70, ReduceOp.AVG)])
def test_rows_of_three_vectors_per_lane(q, oracle, ws, op):
    """Rows of 513 ... 3072 columns in tensors of at least 512 rows per rank: reduce gives rows
    that would leave more than a quarter of a team idle to a team a quarter the size, three
    vectors of codes per lane (16 lanes for up to 768 columns, 32 for up to 1536, 64 for up to
    3072), when the group is no larger than the team; group sizes on both sides of 16, 32 and
    64, rows that end inside a vector or a dword, row counts that leave teams of the last
    workgroup without a row, rows whose scale needs the plain divide, and the same lengths
    in tensors of a few rows, which keep the larger teams."""
    g = torch.Generator().manual_seed(300 + ws)
    many = 512 * ws
    shapes = [(5, c) for c in (513, 640, 767, 769, 1025, 1280, 1537, 2049, 2560, 3073)]
    if ws <= 16:
        shapes += [(many + 5, 516), (many + 1, 700), (many, 768)]
    if ws <= 32:
        shapes += [(many + 3, 1028), (many + 2, 1301), (many, 1536)]
    if ws <= 64:
        shapes += [(many + 7, 2052)] + ([(many + 1, 2902), (many, 3072)] if ws <= 17 else [])
    base = []
    for b in range(3):  # three different contributions, dealt to the peers in turn
        ts = []
        for r, c in shapes:
            x = (torch.randn(r, c, generator=g) * (1 + b)).to(torch.bfloat16)
            x[1] *= 1e-30  # row scale beyond 2^64: the exact fallback
            x[min(3, r - 1)] = 0.0
            ts.append(x)
        base.append(ts)
    peers = [base[p % 3] for p in range(ws)]
    ranks = None if ws <= 2 else [0, ws - 1]
    full_check(q, oracle, peers, ws, op, ranks)
    # one tensor per call: the plan with the segment table in the kernel arguments
    for i in (len(shapes) - 1, 10 if ws <= 64 else 3):
        full_check(q, oracle, [[ts[i]] for ts in peers], ws, op, [ws // 2])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("ws", [1, 2, 8, 16])
def test_short_rows_of_whole_vectors(q, oracle, dtype, ws):
    """Contiguous rows of 1 ... 32 whole 16-byte vectors (8 ... 256 16-bit columns, 4 ... 128
    fp32 columns): 1 to 8 lanes per row, several rows per lane; with rows past the end of
    the tensor, padding rows, zero rows, rows that need the plain divide, a row stride larger
    than the row and a base address that is only element-aligned."""
    g = torch.Generator().manual_seed(7 * ws)
    epv = 4 if dtype == torch.float32 else 8
    vecs = [1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 24, 31, 32]
    rows = [1, 7, 300, 1030, 2049]
    peers = []
    for p in range(ws):
        ts = []
        for i, nv in enumerate(vecs):
            r, c = rows[i % len(rows)], nv * epv
            x = torch.randn(r, c, generator=g) * (0.5 + p)
            if r > 4:
                x[1] *= 1e-30
                x[2] = 0.0
                x[3, 0] = -0.0
            ts.append(x.to(dtype))
        # row stride larger than the row, base one element off a 16-byte boundary
        wide = (torch.randn(50 * 40 + 1, generator=g)).to(dtype)[1:].view(50, 40)[:, :2 * epv]
        ts.append(wide)
        peers.append(ts)
    ranks = None if ws <= 2 else [0, ws - 1]
    full_check(q, oracle, peers, ws, ReduceOp.AVG if ws % 2 else ReduceOp.SUM, ranks)


def test_wide_rows(q, oracle):
    """Rows between the regular and the doubled register capacity (16-bit inputs: 16392 to
    32768 columns) run in the kernel variants with more registers, alone and next to short rows."""
    g = torch.Generator().manual_seed(23)
    # 32772 / 32776 / 32780 columns: two passes in chunks of 1024 dwords with 1, 2, 3 dwords left
    # over, whose last vector reaches back into codes that were already replaced in place
    # (reduce: 16392 to 32768 columns are 4 to 8 vectors per lane, fewer in a row's upper wavefronts)
    for dtype, cols in ((torch.bfloat16, [16392, 17410, 22000, 24580, 28672, 31001, 32768, 32772, 32776, 32780]),
                        (torch.float32, [8200, 16384, 20000, 36868])):
        peers = [[torch.randn(3, c, generator=g).to(dtype) * (p + 1) for c in cols] +
                 [torch.randn(70, 512, generator=g).to(dtype)] for p in range(4)]
        for t in peers[1]:
            t[1] *= 1e-30  # the exact fallback
        full_check(q, oracle, peers, 4, ReduceOp.AVG)
        full_check(q, oracle, peers[:3], 3, ReduceOp.AVG, ranks=[2])


def test_rows_parked_in_lds(q, oracle):
    """Rows of 4097 to 7936 input vectors (16-bit: 32776 to 63488 columns, fp32: 16388 to
    31744): the quantize kernel keeps 16 vectors per lane in registers and parks the rest in
    LDS.  Both ends of the range, the first length beyond it (two passes), a tail after the
    last whole vector, a row that does not start on a 16-byte boundary, padding rows."""
    g = torch.Generator().manual_seed(29)
    for dtype, cols in ((torch.bfloat16, [32776, 40001, 53248, 63488, 63493, 63496]),
                        (torch.float16, [53248, 63489]),
                        (torch.float32, [16388, 28672, 31744, 31747, 31748])):
        peers = []
        for p in range(2):
            ts = [torch.randn(3, c, generator=g).to(dtype) * (p + 1) for c in cols]
            flat = torch.randn(2 * 40001 + 1, generator=g).to(dtype)
            ts.append(flat[1:].view(2, 40001))
            ts.append(torch.randn(70, 512, generator=g).to(dtype))
            peers.append(ts)
        peers[1][0][1] *= 1e-30
        peers[0][1][2] = 0.0
        full_check(q, oracle, peers, 2, ReduceOp.AVG)
    # Lists whose longest row parks one or two groups of five vectors per lane: the launch then has
    # 32.9 or 40 KB of LDS instead of 60 (lengths at both ends of either range)
    for dtype, cols in ((torch.bfloat16, [32776, 43008, 36864]), (torch.bfloat16, [43016, 53248, 33000]),
                        (torch.float32, [16388, 21504]), (torch.float32, [21508, 26624, 100]),
                        (torch.float16, [43015]), (torch.float16, [53255])):
        peers = [[torch.randn(3, c, generator=g).to(dtype) * (p + 1) for c in cols] for p in range(2)]
        full_check(q, oracle, peers, 2, ReduceOp.SUM)


@pytest.mark.parametrize("ws,op", [(3, ReduceOp.AVG), (8, ReduceOp.AVG), (9, ReduceOp.SUM), (17, ReduceOp.AVG)])
def test_reduce_rows_beyond_the_registers(q, oracle, ws, op):
    """Reduce on rows of more than 32768 columns: 32768 columns of sums stay in registers, the
    next 16384 are parked in LDS, the rest makes two passes in steps of up to 8 peers whose
    loads are pipelined.  Lengths at both ends of each range, rows that end inside a vector or
    a dword, group sizes of one step and of several, a row whose scale needs the plain divide."""
    g = torch.Generator().manual_seed(4900 + ws)
    cols = [32772, 36867, 49152, 49153, 49156, 49160, 53248, 53250, 57344, 66001, 131072 + 20]
    base = [[torch.randn(2 if c < 60000 else 1, c, generator=g).to(torch.bfloat16) * (1 + p) for c in cols]
            for p in range(3)]
    base[1][2][0] *= 1e-30
    base[2][4][1] = 0.0
    peers = [base[p % 3] for p in range(ws)]
    full_check(q, oracle, peers, ws, op, [0, ws - 1])


def test_long_rows(q, oracle):
    """Rows longer than the register-resident paths hold: 20000 and 70000 columns."""
    g = torch.Generator().manual_seed(21)
    for dtype in (torch.bfloat16, torch.float32):
        peers = [[(torch.randn(5, 20000, generator=g)).to(dtype),
                  (torch.randn(3, 70000, generator=g)).to(dtype),
                  (torch.randn(4, 70003, generator=g)).to(dtype),
                  (torch.randn(40001 * 2 + 1, generator=g)).to(dtype)[1:].view(2, 40001)] for _ in range(2)]
        full_check(q, oracle, peers, 2, ReduceOp.AVG)
        full_check(q, oracle, peers * 2, 4, ReduceOp.SUM, ranks=[3])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_rows_dealt_to_several_workgroups(q, oracle, dtype):
    """Dequantize deals a row of more than 2048 vectors (8192 fp32 or 16384 16-bit columns) to
    several workgroups: 2 to 130 parts, rows that fill
    their 64-byte blocks and rows that do not (through LDS), rows at odd element offsets and
    with gaps between them, columns behind the last whole vector, a row whose scale needs the
    plain divide, guard elements around every destination."""
    g = torch.Generator().manual_seed(77)
    epv = 16 // torch.empty(0, dtype=dtype).element_size()
    cols = [2049 * epv, 2048 * epv + 3, 4096 * epv, 4100 * epv - 1, 6007 * epv + epv // 2, 28672, 53250, 130 * 2044 * epv + 5]
    tensors, guards = [], []
    for i, c in enumerate(cols):
        rows = 3 if c < 200000 else 2
        if i % 3 == 1:  # a view with a gap of 5 elements between the rows, at an odd element offset
            base = torch.full((rows * (c + 5) + 1,), 9.0, dtype=dtype)
            t = base[1:].view(rows, c + 5)[:, :c]
        else:
            base = torch.full((rows * c + 2,), 9.0, dtype=dtype)
            t = base[1:1 + rows * c].view(rows, c)
        t.copy_((torch.randn(rows, c, generator=g) * (i + 1)).to(dtype))
        if i == 2:
            t[1] *= 1e-30
        tensors.append(t)
        guards.append(base)
    ws = 2
    packed_c = oracle.fused_quantize_into_fp8([t.clone() for t in tensors], ws, nthreads=NT)
    bases_g = [b.cuda() for b in guards]
    outs_g = []
    for t, b, bg in zip(tensors, guards, bases_g):
        off = t.storage_offset() - b.storage_offset()
        outs_g.append(torch.as_strided(bg, t.shape, t.stride(), off))
    same_bytes(q.fused_quantize_into_fp8(outs_g, ws), packed_c, "quantize")
    for bg in bases_g:
        bg.fill_(9.0)
    q.fused_dequantize_from_fp8(outs_g, packed_c.cuda(), ws)
    want = [torch.full_like(b, 9.0) for b in guards]
    outs_c = [torch.as_strided(w, t.shape, t.stride(), t.storage_offset() - b.storage_offset())
              for w, t, b in zip(want, tensors, guards)]
    oracle.fused_dequantize_from_fp8(outs_c, packed_c, ws, nthreads=NT)
    for i, (bg, w) in enumerate(zip(bases_g, want)):
        same_bytes(bg, w, f"dequantize tensor {i} with its guard elements")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("ws", [1, 2, 3, 8])
def test_single_column_tensors(q, oracle, dtype, ws):
    """1-D tensors (rows of one column): lengths around the rows a workgroup takes in each
    stage, odd lengths and odd rows per slot (a lane's pair of rows then straddles two
    slots or the end of the tensor), starts that are not 4-byte aligned, a strided 1-D
    view, zeros, negative zeros and a NaN."""
    g = torch.Generator().manual_seed(40 + ws)
    lengths = [1, 2, 3, 5, 511, 1023, 1024, 1025, 2047, 2048, 2049, 4095, 4097, 6145]
    op = ReduceOp.AVG if ws % 2 else ReduceOp.SUM

    def views(bases):
        # odd tensors start one element into their storage, every third one is strided
        return [b[1:1 + 2 * n:2] if i % 3 == 0 else b[i % 2:i % 2 + n]
                for i, (b, n) in enumerate(zip(bases, lengths))]

    peers_cpu, peers_gpu = [], []
    for p in range(ws):
        bases = []
        for n in lengths:
            flat = torch.randn(2 * n + 3, generator=g) * (1 + p)
            flat[::7] = 0.0
            flat[3::11] = -0.0
            bases.append(flat.to(dtype))
        peers_cpu.append(views(bases))
        peers_gpu.append(views([b.cuda() for b in bases]))
    if dtype != torch.float32:
        assert any(t.data_ptr() % 4 for t in peers_gpu[0])
    assert any(t.stride(0) == 2 for t in peers_gpu[0])
    qs_g, red_g, gath_g = sim.allreduce(q, [list(t) for t in peers_gpu], ws, op)
    qs_c, red_c, gath_c = sim.allreduce(oracle, [list(t) for t in peers_cpu], ws, op, nthreads=NT)
    for p, (a, b) in enumerate(zip(qs_g, qs_c)):
        same_bytes(a, b, f"quantize peer {p}")
    for r in red_c:
        same_bytes(red_g[r], red_c[r], f"reduce rank {r}")
    # dequantize into views of guard-filled storage; the storage is compared whole
    out_c = [torch.full((2 * n + 3,), 5.0, dtype=dtype) for n in lengths]
    out_g = [t.cuda() for t in out_c]
    oracle.fused_dequantize_from_fp8(views(out_c), gath_c, ws, nthreads=NT)
    q.fused_dequantize_from_fp8(views(out_g), gath_g, ws)
    for i, (a, b) in enumerate(zip(out_g, out_c)):
        same_bytes(a, b, f"dequantize tensor {i} (length {lengths[i]})")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("divisor", [2, 3, 7, 12, 1000, 2.5])
def test_dequantize_with_division(q, dtype, divisor):
    """divide_by folds the caller's `tensor /= n` (manager.py:450-452) into the store of
    the dequantize kernel.  Expected: the plain dequantize followed by torch's own
    in-place division of each tensor on the GPU, byte for byte; every lane mapping
    (short and long rows, whole vectors and tails, single columns, strided and
    misaligned tensors, more than 16 tensors), rows with scales outside the range of
    the fast division, zero rows and negative zeros."""
    g = torch.Generator().manual_seed(31)
    shapes = [(37, 256), (5, 4096), (130,), (3, 14336), (9, 33), (2, 1024), (64, 16), (40, 48), (11, 520),
              (6, 2100), (3, 9001), (300,), (17, 8), (5, 24), (2, 40000), (1, 1), (4, 100), (8, 64)]
    cpu = []
    for sh in shapes:
        x = torch.randn(sh, generator=g) * 0.3
        if x.dim() == 2 and x.shape[0] > 2:
            x[0] *= 1e-30
            x[1] = 0.0
            x[2, ::2] = -0.0
        cpu.append(x.to(dtype))
    base = torch.randn(50, 300, generator=g).to(dtype)
    flat = torch.randn(5000, generator=g).to(dtype)
    for ws, count in ((1, len(cpu)), (4, 9)):  # 20 tensors: device table; 11: in the kernel arguments
        gbase, gflat = base.cuda(), flat.cuda()
        src = [t.cuda() for t in cpu[:count]] + [gbase[::2, 1:200:3], gflat[3:3 + 77 * 13].view(77, 13)]
        packed = q.fused_quantize_into_fp8(list(src), ws)

        def destinations():  # like the sources: the last two strided and misaligned
            out = [torch.full_like(t, 5.0) for t in src[:count]]
            b, f = torch.full_like(gbase, 5.0), torch.full_like(gflat, 5.0)
            return out + [b[::2, 1:200:3], f[3:3 + 77 * 13].view(77, 13)]

        want = destinations()
        q.fused_dequantize_from_fp8(list(want), packed, ws)
        for t in want:
            t /= divisor
        got = destinations()
        assert got[-2].stride() == (600, 3) and got[-1].data_ptr() % 16 != 0
        q.fused_dequantize_from_fp8(list(got), packed, ws, divide_by=divisor)
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            if dtype == torch.float16:
                # torch's own division of a float16 tensor turns -0 into +0 in the elements
                # its vectorised loop does not cover (short tensors, tails) and keeps -0
                # elsewhere; the kernel keeps -0 (IEEE).  Compare with +0 for both.
                a, b = a.contiguous().clone(), b.contiguous().clone()
                for t in (a, b):
                    bits = t.view(torch.int16)
                    bits[bits == -32768] = 0
            same_bytes(a, b, f"ws={ws} tensor {i} {tuple(a.shape)}")


def test_extreme_scales_and_denormals(q, oracle):
    """Row maxima far outside the range where the fast division applies
    (scale exponent beyond +-64), fp32 denormal inputs, all-zero rows."""
    g = torch.Generator().manual_seed(31)
    mags = torch.tensor([1e-38, 1e-33, 1e-30, 1e-25, 1e-20, 1.0, 1e18, 1e22, 1e25, 1e30, 3e38])
    x = torch.randn(len(mags), 4096, generator=g).clamp(-3, 3) / 3 * mags[:, None]
    x = torch.cat([x, torch.zeros(1, 4096), torch.full((1, 4096), 1e-45)])
    y = torch.randn(len(mags) + 2, 33, generator=g).clamp(-3, 3) / 3 * torch.cat([mags, mags[:2]])[:, None]
    z = (torch.randn(len(mags) + 2, generator=g).clamp(-3, 3) / 3) * torch.cat([mags, mags[:2]])
    peers = [[x * (p + 1) / 4, y * (p + 1) / 4, z * (p + 1) / 4] for p in range(4)]
    full_check(q, oracle, peers, 4, ReduceOp.SUM)
    full_check(q, oracle, peers, 4, ReduceOp.AVG)
    full_check(q, oracle, peers[:1], 1, ReduceOp.SUM)


def test_empty_and_ragged(q, oracle):
    only_empty = [[torch.zeros(0, 64)], [torch.zeros(0, 64)]]  # empty packed buffer, nothing to launch
    full_check(q, oracle, only_empty, 2, ReduceOp.AVG)
    peers = [[torch.zeros(0, 5), torch.ones(3, 0), torch.arange(7.0), torch.ones(1, 1)] for _ in range(2)]
    full_check(q, oracle, peers, 2, ReduceOp.SUM)
    full_check(q, oracle, peers * 2, 4, ReduceOp.AVG)


# ---- properties at full size ---------------------------------------------------
def test_cfg3_full_size(q, oracle):
    """The whole Llama-3-8B layer bucket (218 M elements, ws = 8): peer 0's packed
    buffer and one rank's reduction against the checker, then size-independent
    properties of the full round trip on the GPU."""
    ws = 8
    peers_gpu = []
    q0_cpu = None
    for s in range(ws):
        t = workloads.cfg3(s)
        if s == 0:
            q0_cpu = oracle.fused_quantize_into_fp8(list(t), ws, nthreads=NT)
            peer0_cpu = t
        peers_gpu.append(dev(t))
    qs = sim.quantize_peers(q, peers_gpu, ws)
    assert qs[0].numel() == 218341376
    same_bytes(qs[0], q0_cpu, "cfg3 quantize peer 0")
    del q0_cpu
    rank = 5
    recv = sim.recv_buffer(qs, rank, ws)
    recv_cpu = recv.cpu()
    q.fused_reduce_fp8(list(peers_gpu[0]), recv, ws, rank, ReduceOp.AVG)
    oracle.fused_reduce_fp8(list(peer0_cpu), recv_cpu, ws, rank, ReduceOp.AVG, nthreads=NT)
    same_bytes(recv, recv_cpu, "cfg3 reduce rank 5")
    # the configuration asks for SUM as well as AVG: another rank's slots, summed
    recv_sum = sim.recv_buffer(qs, 2, ws)
    recv_sum_cpu = recv_sum.cpu()
    q.fused_reduce_fp8(list(peers_gpu[0]), recv_sum, ws, 2, ReduceOp.SUM)
    oracle.fused_reduce_fp8(list(peer0_cpu), recv_sum_cpu, ws, 2, ReduceOp.SUM, nthreads=NT)
    same_bytes(recv_sum, recv_sum_cpu, "cfg3 reduce rank 2, SUM")
    del recv_sum, recv_sum_cpu
    # dequantize of that whole buffer (one reduced slot, seven as received), every tensor by bytes
    outs = [torch.empty_like(t) for t in peers_gpu[0]]
    outs_cpu = [torch.empty_like(t) for t in peer0_cpu]
    q.fused_dequantize_from_fp8(outs, recv, ws)
    oracle.fused_dequantize_from_fp8(outs_cpu, recv_cpu, ws, nthreads=NT)
    for i, (a, b) in enumerate(zip(outs, outs_cpu)):
        same_bytes(a, b, f"cfg3 dequantize tensor {i}")
    del outs_cpu, recv_cpu
    # round trip of peer 0 alone: quantize -> dequantize is within half an fp8 ULP per row
    outs = [torch.empty_like(t) for t in peers_gpu[0]]
    q.fused_dequantize_from_fp8(outs, qs[0], ws)
    for x, o in zip(peers_gpu[0], outs):
        xf, of = x.float().view(x.shape[0], -1), o.float().view(x.shape[0], -1)
        amax = xf.abs().amax(dim=1, keepdim=True)
        # fp8 half-ULP (2^-4 relative for normal codes, 2^-10 / s absolute for subnormal
        # ones) plus the bf16 store rounding (half a bf16 ULP of the output, 2^-8 relative)
        tol = torch.maximum(xf.abs() * 2 ** -4, amax * (2 ** -10 / 448.0)) * 1.001 + of.abs() * 2 ** -8
        bad = (xf - of).abs() > tol
        if bad.any():
            r, c = bad.nonzero()[0].tolist()
            raise AssertionError(
                f"round trip out of tolerance in {tuple(x.shape)}: {int(bad.sum())} elements, first at "
                f"({r},{c}): x={xf[r, c].item()!r} out={of[r, c].item()!r} amax={amax[r].item()!r}")
    # idempotence: quantizing the dequantized tensors reproduces the codes (scales may move an ulp)
    q2 = q.fused_quantize_into_fp8(list(outs), ws)
    d2 = [torch.empty_like(t) for t in outs]
    q.fused_dequantize_from_fp8(d2, q2, ws)
    for a, b in zip(outs, d2):
        assert torch.equal(a, b)


def test_cfg4_full_size(q, oracle):
    """The whole 1.1 B-parameter fp32 pseudo-gradient (201 tensors, 4.4 GB per peer,
    ws = 4, AVG), generated on the GPU.  Three tensors of different row classes are
    checked byte for byte against the checker inside the full packed buffers; the
    rest through properties that do not depend on size."""
    ws, rank = 4, 2
    mine = workloads.cfg4(rank, device="cuda")
    assert len(mine) == 201 and sum(t.numel() for t in mine) == 1100048384
    packed = q.fused_quantize_into_fp8(mine, ws)
    assert packed.numel() == 1102526464
    shapes = [tuple(t.shape) for t in mine]
    offs, slot, total = oracle.layout(shapes, ws)
    picks = [3, 7, 9, 199]  # v_proj [256, 2048], down_proj [2048, 5632], a norm [2048, 1], final norm
    for i in picks:
        m, n = shapes[i]
        want = oracle.fused_quantize_into_fp8([mine[i].cpu()], ws, nthreads=NT)
        sr, rb = -(-m // ws), (-(-n // 4) + 1) * 4
        for p in range(ws):
            got = packed[p * slot + offs[i]: p * slot + offs[i] + sr * rb].cpu()
            assert torch.equal(got, want[p * sr * rb:(p + 1) * sr * rb]), (i, p)
    # every scale is 448 / amax (or 1.0), every row's arg-max encodes to +-448
    for i in (0, 5, 200):
        x = mine[i]
        m, n = x.shape
        sr, rb = -(-m // ws), (-(-n // 4) + 1) * 4
        rows = torch.cat([packed[p * slot + offs[i]: p * slot + offs[i] + sr * rb].view(sr, rb)
                          for p in range(ws)])[:m]
        scales = rows[:, :4].contiguous().view(torch.float32).view(m)
        amax = x.abs().amax(dim=1)
        want_s = torch.where(amax > 0, torch.tensor(448.0, device="cuda") / amax, torch.ones_like(amax))
        assert torch.equal(scales, want_s)
        top = rows[torch.arange(m, device="cuda"), 4 + x.abs().argmax(dim=1)] & 0x7F
        assert ((top == 0x7E) | (amax == 0)).all()
    # reduce of 4 identical peers with AVG gives back the same codes (-0 becomes +0); scales
    # within 4 fp32 ulps
    recv = packed[rank * slot:(rank + 1) * slot].repeat(ws)
    before = recv[rank * slot:(rank + 1) * slot].clone()
    q.fused_reduce_fp8(mine, recv, ws, rank, ReduceOp.AVG)
    after = recv[rank * slot:(rank + 1) * slot]
    for i in (0, 7, 200):
        m, n = shapes[i]
        sr, rb = -(-m // ws), (-(-n // 4) + 1) * 4
        a = after[offs[i]: offs[i] + sr * rb].view(sr, rb)
        b = before[offs[i]: offs[i] + sr * rb].view(sr, rb)
        real = min(sr, max(0, m - rank * sr))
        want = b[:real, 4:].clone()
        want[want == 0x80] = 0  # a sum of negative zeros is +0
        assert torch.equal(a[:real, 4:], want)
        da = a[:real, :4].contiguous().view(torch.int32) - b[:real, :4].contiguous().view(torch.int32)
        assert da.abs().max() <= 4
    del recv, before
    # round trip: dequantize(quantize(x)) is within half an fp8 ULP of x, row by row
    outs = [torch.empty_like(t) for t in mine]
    q.fused_dequantize_from_fp8(outs, packed, ws)
    for x, o in zip(mine, outs):
        amax = x.abs().amax(dim=1, keepdim=True)
        tol = torch.maximum(x.abs() * 2 ** -4, amax * (2 ** -10 / 448.0)) * 1.001
        assert ((x - o).abs() <= tol).all()
    del outs

    # One rank's reduction of four different peers and the dequantization of the result, at
    # full size on the GPU; the picked tensors byte for byte against the checker, which works
    # on single-tensor buffers cut out of the full ones (a tensor's rows sit at the same
    # offsets in every slot, so its ws row slices are a packed buffer of that tensor alone).
    recv = torch.empty_like(packed)
    recv[rank * slot:(rank + 1) * slot] = packed[rank * slot:(rank + 1) * slot]
    del packed
    for p in range(ws):
        if p == rank:
            continue
        other = workloads.cfg4(p, device="cuda")
        qp = q.fused_quantize_into_fp8(other, ws)
        recv[p * slot:(p + 1) * slot] = qp[rank * slot:(rank + 1) * slot]
        del other, qp
    received = recv.clone()
    q.fused_reduce_fp8(mine, recv, ws, rank, ReduceOp.AVG)
    outs = [torch.empty_like(t) for t in mine]
    q.fused_dequantize_from_fp8(outs, recv, ws)
    for i in picks:
        m, n = shapes[i]
        sr, rb = -(-m // ws), (-(-n // 4) + 1) * 4

        def cut(buf):
            return torch.cat([buf[p * slot + offs[i]: p * slot + offs[i] + sr * rb] for p in range(ws)]).cpu()

        like = torch.empty(m, n)
        mini = cut(received)
        oracle.fused_reduce_fp8([like], mini, ws, rank, ReduceOp.AVG, nthreads=NT)
        same_bytes(cut(recv), mini, f"cfg4 reduce tensor {i}")
        want = [torch.empty(m, n)]
        oracle.fused_dequantize_from_fp8(want, mini, ws, nthreads=NT)
        same_bytes(outs[i], want[0], f"cfg4 dequantize tensor {i}")


def test_buffers_beyond_four_gib(q, oracle):
    """More than 2^32 elements in a tensor, rows and tensors at more than 2^32 bytes into a
    slot and into the packed buffer (20.8 GB): a bf16 tensor [80000, 60000], a 1-D bf16 tensor
    of 2 * 10^9 elements (8 packed bytes each) and a small tensor behind them, ws = 4.  All
    three stages run at full size on the GPU; sampled rows (the first and last of slots, those
    around element 2^31 and 2^32 and around byte 2^32 of a slot) are compared byte for byte
    with the checker, which works on small buffers cut out of the full ones: a row's packed
    bytes depend on that row alone, a reduced row on the ws rows at its place in the slots."""
    ws, rank = 4, 3
    dev_ = "cuda"
    g = torch.Generator(device=dev_).manual_seed(5)
    A = torch.empty(80000, 60000, dtype=torch.bfloat16, device=dev_)
    for r0 in range(0, 80000, 8000):
        A[r0:r0 + 8000].normal_(generator=g)
        A[r0:r0 + 8000] *= 1 + r0 // 8000
    B = torch.empty(2_000_000_000, dtype=torch.bfloat16, device=dev_)
    for e0 in range(0, B.numel(), 250_000_000):
        B[e0:e0 + 250_000_000].normal_(generator=g)
        B[e0:e0 + 250_000_000] *= 1 + e0 // 250_000_000
    C = torch.randn(5, 7, generator=g, device=dev_).to(torch.bfloat16)
    tensors = [A, B, C]
    shapes = [(80000, 60000), (B.numel(), 1), (5, 7)]
    offs, slot, total = oracle.layout(shapes, ws)
    assert offs[2] > 2 ** 32 and total == 4 * slot and total > 20 * 10 ** 9
    srs = [-(-m // ws) for m, _ in shapes]
    rbs = [(-(-n // 4) + 1) * 4 for _, n in shapes]
    first_b = (2 ** 32 - offs[1]) // 8  # the row of B that starts at byte 2^32 of its slot
    rows_a = sorted({0, 1, 19999, 20000, 20001, 2 ** 31 // 60000, 2 ** 31 // 60000 + 1, 59999, 60000,
                     2 ** 32 // 60000, 2 ** 32 // 60000 + 1, 79998, 79999})
    rows_b = sorted({0, 1, 255, 256, 2047, 2048, 499_999_999, 500_000_000, first_b - 1, first_b, first_b + 1,
                     999_999_999, 1_000_000_000, 1_499_999_999, 1_500_000_000, 1_999_999_998, 1_999_999_999}
                    | set(torch.randint(0, B.numel(), (500,), generator=torch.Generator().manual_seed(6)).tolist()))
    picks = [rows_a, rows_b, list(range(5))]

    def cut(buf, i, rows):
        """The packed rows `rows` of tensor i out of a full packed buffer, as one uint8 tensor."""
        at = torch.tensor([(r // srs[i]) * slot + offs[i] + (r % srs[i]) * rbs[i] for r in rows], device=dev_)
        idx = at[:, None] + torch.arange(rbs[i], device=dev_)[None, :]
        return buf[idx.view(-1)].cpu()

    packed = q.fused_quantize_into_fp8(tensors, ws)
    assert packed.numel() == total
    small = [A[rows_a].cpu(), B[rows_b].cpu(), C.cpu()]
    for i in range(3):
        want = oracle.fused_quantize_into_fp8([small[i]], 1, nthreads=NT)
        same_bytes(cut(packed, i, picks[i]), want[:len(picks[i]) * rbs[i]], f"quantize tensor {i}")

    # Reduce on rank 3 of four different contributions: slot k of the receive buffer is slot
    # (k + 1) % 4 of the packed buffer.  Row j of the slice is checked through a packed buffer
    # of a tensor of ws * len(js) rows: its slot k holds the rows js of slot k.
    recv = torch.cat([packed[((k + 1) % ws) * slot:((k + 1) % ws + 1) * slot] for k in range(ws)])
    js = [sorted({r % srs[i] for r in picks[i]}) for i in range(3)]
    js[2] = [0, 1]
    minis = [torch.cat([cut(recv, i, [k * srs[i] + j for j in js[i]]) for k in range(ws)]) for i in range(3)]
    q.fused_reduce_fp8(tensors, recv, ws, rank, ReduceOp.AVG)
    for i in range(3):
        like = torch.empty(ws * len(js[i]), shapes[i][1], dtype=torch.bfloat16)
        oracle.fused_reduce_fp8([like], minis[i], ws, rank, ReduceOp.AVG, nthreads=NT)
        nb = len(js[i]) * rbs[i]
        same_bytes(cut(recv, i, [rank * srs[i] + j for j in js[i]]), minis[i][rank * nb:(rank + 1) * nb],
                   f"reduce tensor {i}")

    # Dequantize of that buffer (slot 3 reduced, the others as received)
    outs = [torch.full_like(t, 7.0) for t in tensors]
    q.fused_dequantize_from_fp8(outs, recv, ws)
    for i in range(3):
        rows = picks[i]
        want = [torch.full((len(rows), shapes[i][1]), 7.0, dtype=torch.bfloat16)]
        oracle.fused_dequantize_from_fp8(want, cut(recv, i, rows), 1, nthreads=NT)
        got = outs[i][rows] if i != 1 else outs[i][rows].view(-1, 1)
        same_bytes(got, want[0], f"dequantize tensor {i}")
    # and nothing else: every element was written, the two big tensors are finite
    assert not (outs[0] == 7.0).all(dim=1).any()
    assert torch.isfinite(outs[1][::4099].float()).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_cfg5_full_size(q, oracle, dtype):
    """All 10 000 ragged tensors, 16 peers, SUM: every peer's packed buffer, three
    ranks' reductions and the dequantized result against the checker."""
    shapes = workloads.cfg5_shapes(10000)
    peers = [workloads.cfg5(s, dtype, shapes) for s in range(16)]
    full_check(q, oracle, peers, 16, ReduceOp.SUM, ranks=[0, 9, 15])
    outs_g = [torch.empty_like(t).cuda() for t in peers[3]]
    outs_c = [torch.empty_like(t) for t in peers[3]]
    buf = oracle.fused_quantize_into_fp8(list(peers[3]), 16, nthreads=NT)
    q.fused_dequantize_from_fp8(outs_g, buf.cuda(), 16)
    oracle.fused_dequantize_from_fp8(outs_c, buf, 16, nthreads=NT)
    for a, b in zip(outs_g, outs_c):
        assert torch.equal(a.cpu().view(-1).view(torch.uint8), b.view(-1).view(torch.uint8))


# ---- memory safety around the packed buffer ---------------------------------------
def test_no_write_outside_packed_buffer(q):
    """Calls the C ABI with a packed buffer placed between two canary zones."""
    from torchft_amd import _lib
    L = _lib.load()
    g = torch.Generator().manual_seed(41)
    shapes = [(37, 4096), (5, 333), (19,), (64, 64), (3, 14336)]
    ts = [torch.randn(s, generator=g).to(torch.bfloat16).cuda() for s in shapes]
    ts = [t if t.dim() == 2 else t.unsqueeze(1) for t in ts]
    ws, T, guard = 4, len(ts), 4096
    ptrs = (ctypes.c_void_p * T)(*[t.data_ptr() for t in ts])
    sh = (ctypes.c_int64 * (2 * T))(*[v for t in ts for v in t.shape])
    st = (ctypes.c_int64 * (2 * T))(*[v for t in ts for v in t.stride()])
    h = ctypes.c_void_p()
    assert L.tftq_plan_create(2, T, sh, st, ws, ctypes.byref(h)) == 0
    size = L.tftq_plan_output_size(h)
    arena = torch.full((size + 2 * guard,), 0xA5, dtype=torch.uint8, device="cuda")
    packed = arena[guard:guard + size]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    dev = torch.cuda.current_device()
    p = ctypes.c_void_p(packed.data_ptr())
    assert L.tftq_quantize(h, ptrs, None, None, p, size, dev, stream) == 0
    assert L.tftq_reduce(h, None, p, size, 1, 1, dev, stream) == 0
    assert L.tftq_dequantize(h, ptrs, None, None, p, size, -1, stream) == 0  # -1: the current device
    torch.cuda.synchronize()
    assert (arena[:guard] == 0xA5).all() and (arena[guard + size:] == 0xA5).all()
    assert L.tftq_quantize(h, ptrs, None, None, p, size - 4, dev, stream) == -4
    assert L.tftq_reduce(h, None, p, size, 4, 0, dev, stream) == -1
    assert L.tftq_quantize(h, None, None, None, p, size, dev, stream) == -1  # no addresses
    L.tftq_plan_destroy(h)


def test_wrapper_errors_on_gpu(q):
    x = [torch.zeros(8, 8, device="cuda")]
    buf = q.fused_quantize_into_fp8(x, 2)
    with pytest.raises(AssertionError, match="Output size does not match"):
        q.fused_reduce_fp8(x, buf[:-4], 2, 0)
    with pytest.raises(AssertionError, match="Output size does not match"):
        q.fused_dequantize_from_fp8(x, buf[:-4], 2)
    with pytest.raises(RuntimeError):
        q.fused_reduce_fp8(x, buf, 2, 2)
    with pytest.raises(RuntimeError, match="packed buffer is on cpu"):
        q.fused_reduce_fp8(x, buf.cpu(), 2, 0)
    with pytest.raises(RuntimeError, match="packed buffer is on cpu"):
        q.fused_dequantize_from_fp8(x, buf.cpu(), 2)


@pytest.mark.parametrize("n_tensors", [3, 20])
def test_entry_points_under_graph_capture(q, n_tensors):
    """The three entry points only enqueue kernels on the stream they are given, so a HIP
    graph can capture them.  The graph is replayed several times with new inputs and with
    eager work and synchronisations in between; every replay must equal the eager result."""
    from torchft_amd import _lib
    L = _lib.load()
    ws, rank = 4, 2
    g = torch.Generator().manual_seed(77)
    shapes = [(37, 4096), (50, 333), (1900, 1), (64, 64), (9, 1000)]
    ts = [torch.randn(shapes[i % len(shapes)], generator=g).to(torch.bfloat16).cuda() for i in range(n_tensors)]
    outs = [torch.empty_like(t) for t in ts]
    T = len(ts)

    # one plan (shapes only) serves both tensor lists; a list of 20 needs the device copy of
    # the plan's table and a device buffer per list for the addresses
    sh = (ctypes.c_int64 * (2 * T))(*[v for t in ts for v in t.shape])
    st = (ctypes.c_int64 * (2 * T))(*[v for t in ts for v in t.stride()])
    h = ctypes.c_void_p()
    assert L.tftq_plan_create(2, T, sh, st, ws, ctypes.byref(h)) == 0
    assert L.tftq_plan_n_tensors(h) == T
    in_ptrs = (ctypes.c_void_p * T)(*[t.data_ptr() for t in ts])     # quantize reads `ts`
    out_ptrs = (ctypes.c_void_p * T)(*[t.data_ptr() for t in outs])  # dequantize writes `outs`
    table = in_dev = out_dev = None
    nbytes = L.tftq_plan_table_bytes(h)
    assert (nbytes > 0) == (T > 16)
    if nbytes:
        host = (ctypes.c_uint8 * nbytes).from_address(L.tftq_plan_table_host(h))
        table = torch.frombuffer(host, dtype=torch.uint8).cuda()
        in_dev = torch.empty(T, dtype=torch.int64, device="cuda")
        out_dev = torch.empty(T, dtype=torch.int64, device="cuda")
    size = L.tftq_plan_output_size(h)
    packed = torch.empty(size, dtype=torch.uint8, device="cuda")
    dev = torch.cuda.current_device()
    addr = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())  # noqa: E731

    def enqueue(stream):
        s = ctypes.c_void_p(stream.cuda_stream)
        p = ctypes.c_void_p(packed.data_ptr())
        # the addresses are written to the device buffers by small kernels that the capture records too
        assert L.tftq_quantize(h, in_ptrs, addr(table), addr(in_dev), p, size, dev, s) == 0
        assert L.tftq_reduce(h, addr(table), p, size, rank, 1, dev, s) == 0
        assert L.tftq_dequantize(h, out_ptrs, addr(table), addr(out_dev), p, size, dev, s) == 0

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        enqueue(side)  # warm-up outside the capture
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            enqueue(torch.cuda.current_stream())
    torch.cuda.current_stream().wait_stream(side)

    for it in range(4):
        for t in ts:
            t.copy_((torch.randn(t.shape, generator=g) * (it + 1)).to(torch.bfloat16))
        for o in outs:
            o.zero_()
        packed.fill_(0x5A)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        got_packed = packed.clone()
        for o in outs:
            o.zero_()
        packed.fill_(0x5A)
        enqueue(torch.cuda.current_stream())  # eager, same inputs
        torch.cuda.synchronize()
        same_bytes(got_packed, packed, f"replay {it}: packed buffer")
        for i, (a, b) in enumerate(zip(got, outs)):
            same_bytes(a, b, f"replay {it}: tensor {i}")
    L.tftq_plan_destroy(h)


@pytest.mark.parametrize("seed", range(int(os.environ.get("TFTQ_RANDOM_LISTS", "36"))))
def test_random_tensor_lists(q, oracle, seed):
    """Random lists: row lengths on both sides of every kind boundary of the planner, 1-D and
    empty tensors, column-strided and row-strided views, group sizes 1 ... 17, both ops, all
    dtypes; short lists (descriptors in the kernel arguments) and long ones (device table)."""
    import random
    rnd = random.Random(1000 + seed)
    g = torch.Generator().manual_seed(seed)
    dtype = [torch.float32, torch.bfloat16, torch.float16][seed % 3]
    ws = rnd.choice([1, 2, 3, 4, 7, 8, 9, 16, 17])
    op = rnd.choice([ReduceOp.SUM, ReduceOp.AVG])
    n_tensors = rnd.choice([1, 3, 9, 16, 17, 40])
    edges = [1, 2, 3, 4, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 260,
             511, 512, 513, 520, 767, 768, 769, 1023, 1024, 1025, 1536, 1537, 2047, 2048, 2049, 3072, 3073,
             4095, 4096, 4100, 8191, 8192, 8200]
    # rows that dequantize deals to several workgroups, that quantize parks in LDS (one to three
    # groups), that reduce takes in the wide variant
    long_edges = [16383, 16384, 16392, 17001, 20000, 24580, 32768, 32776, 43008, 43016, 53250, 63500]

    def one_tensor():
        kind = rnd.random()
        n = rnd.choice(edges) if rnd.random() < 0.8 else rnd.randint(1, 9000)
        m = rnd.choice([0, 1, 2, 5, 16, 33, 70]) if n > 512 else rnd.choice([0, 1, 7, 64, 300, 1100])
        if rnd.random() < 0.08:
            n, m = rnd.choice(long_edges), rnd.choice([1, 2, 5])
        elif 512 < n <= 3100 and ws <= 8 and rnd.random() < 0.15:
            m = 512 * ws + rnd.randint(0, 9)  # rows enough for reduce's three-vectors-per-lane teams
        if kind < 0.1:
            return torch.randn(rnd.choice([1, 5, 1000, 4097]), generator=g)           # 1-D
        if kind < 0.2:
            return torch.randn(n, max(m, 1), generator=g).t()                           # column-strided
        if kind < 0.3:
            return torch.randn(max(m, 1), n + rnd.randint(1, 9), generator=g)[:, :n]    # row stride > n
        if kind < 0.35:
            return torch.randn(max(m, 1) * n + 1, generator=g)[1:].view(max(m, 1), n)   # element-aligned base
        return torch.randn(m, n, generator=g)

    protos = [one_tensor() for _ in range(n_tensors)]
    peers = []
    for p in range(ws):
        ts = []
        for t in protos:
            x = torch.randn(t.shape, generator=g) * (10.0 ** rnd.randint(-4, 3))
            if x.numel() > 8:
                x.view(-1)[3] = 0.0
            y = torch.empty_strided(t.shape, t.stride(), dtype=dtype) if t.numel() else torch.empty(t.shape, dtype=dtype)
            y.copy_(x)
            ts.append(y)
        peers.append(ts)
    ranks = None if ws <= 4 else sorted({0, rnd.randrange(ws), ws - 1})
    full_check(q, oracle, peers, ws, op, ranks)


def test_plan_cache_eviction(q, oracle, monkeypatch):
    """Plans are dropped from the cache while their kernels may still be queued; results
    stay correct and the cache stays within its limits."""
    monkeypatch.setattr(q, "_PLAN_CACHE_SIZE", 3)
    monkeypatch.setattr(q, "_PLAN_CACHE_TENSORS", 60)
    g = torch.Generator().manual_seed(5)
    ws = 2
    lists = []
    for k in range(8):
        n = 1 if k % 2 else 25  # single tensors and lists long enough for a device table
        lists.append([torch.randn(9 + k, 40 + 3 * j, generator=g) for j in range(n)])
    packed = []
    for _ in range(3):
        packed = [q.fused_quantize_into_fp8(dev(ts), ws) for ts in lists]  # no synchronisation in between
    torch.cuda.synchronize()
    assert len(q._plan_cache) <= 3 and q._plan_cache_tensors <= 60
    for ts, got in zip(lists, packed):
        same_bytes(got, oracle.fused_quantize_into_fp8(list(ts), ws), "quantize after eviction")


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_group_sizes_and_row_lengths(q, oracle, seed):
    """Lists of 1 to 20 tensors with a random group size from 1 to 20, SUM or AVG, any of the
    three dtypes: mostly rows of 1 to 70 columns (a lane, a pair or a team of 4 per row in
    reduce, on both sides of their group sizes 2, 4, 8 and 16), rows of up to 600 columns, rows
    at the limits of what reduce keeps in registers and parks in LDS (32768, 49152 columns and
    their neighbours) and rows of up to 140 000 columns; row counts from one to 200 per rank,
    rows that take the plain divide, rows of -0."""
    import random
    rnd = random.Random(seed)
    for case in range(14):
        ws = rnd.choice([1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 20])
        op = rnd.choice([ReduceOp.AVG, ReduceOp.SUM])
        dtype = rnd.choice([torch.bfloat16, torch.float32, torch.float16])
        shapes = []
        for _ in range(rnd.choice([1, 3, 12, 20])):
            kind = rnd.random()
            if kind < 0.55:
                c = rnd.randint(1, 70)
            elif kind < 0.75:
                c = rnd.randint(65, 600)
            elif kind < 0.85:
                c = rnd.choice([32768, 32769, 32772, 49151, 49152, 49153, 49157, 53248]) + rnd.choice([0, 0, 1, 3, 4])
            else:
                c = rnd.randint(32769, 140000)
            r = rnd.choice([1, 2, ws, ws + 1, 3 * ws + 2, 40 * ws + 7, 200 * ws]) if c < 2000 else rnd.choice([1, 2, ws + 1])
            if r * c * ws > 40_000_000:
                r = 1
            shapes.append((r, c))
        g = torch.Generator().manual_seed(1000 * seed + case)
        base = []
        for p in range(min(ws, 3)):
            ts = []
            for r, c in shapes:
                x = torch.randn(r, c, generator=g) * (1 + p)
                if r > 2 and rnd.random() < 0.3:
                    x[1] *= 1e-30
                if r > 3 and rnd.random() < 0.3:
                    x[2] = -0.0
                ts.append(x.to(dtype))
            base.append(ts)
        peers = [base[p % len(base)] for p in range(ws)]
        ranks = None if ws <= 3 else sorted({0, rnd.randrange(ws), ws - 1})
        print(f"case {case}: ws {ws} {op} {dtype} {shapes}", flush=True)
        full_check(q, oracle, peers, ws, op, ranks)


@pytest.mark.parametrize("seed", range(int(os.environ.get("TFTQ_RANDOM_EXTREMES", "12"))))
def test_random_extremes(q, oracle, seed):
    """Random lists at the far ends: group sizes up to 70, rows of up to 70 003 columns,
    magnitudes from 1e-37 to 1e37 (scales outside the range of the fast division), zero rows."""
    import random
    rnd = random.Random(5000 + seed)
    g = torch.Generator().manual_seed(5000 + seed)
    dtype = [torch.float32, torch.bfloat16, torch.float16][seed % 3]
    ws = rnd.choice([2, 5, 8, 31, 33, 64, 65, 70])
    op = rnd.choice([ReduceOp.SUM, ReduceOp.AVG])
    shapes = []
    for _ in range(rnd.choice([1, 4, 17])):
        n = rnd.choice([1, 5, 40, 130, 500, 1028, 4100, 9000, 16385, 20000, 32768, 32769, 40000, 53248, 63489, 70003])
        shapes.append((rnd.choice([1, 2, ws, ws + 1, 3 * ws - 1]) if n > 2000 else rnd.choice([1, 9, 150]), n))
    top = 4 if dtype == torch.float16 else 37
    peers = []
    for p in range(ws):
        ts = []
        for (m, n) in shapes:
            mags = 10.0 ** torch.randint(-top, top, (m, 1), generator=g).float()
            x = torch.randn(m, n, generator=g).clamp(-3, 3) / 3 * mags
            if m > 1:
                x[rnd.randrange(m)] = 0.0
            ts.append(x.to(dtype))
        peers.append(ts)
    full_check(q, oracle, peers, ws, op, ranks=sorted({0, rnd.randrange(ws), ws - 1}))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_nan_and_inf_rows(q, oracle, dtype):
    """Rows with NaN and Inf (outside what the reference's sources pin down) still follow the
    IEEE restatement: NaN is ignored by the row maximum, an infinite maximum gives scale 0,
    codes of NaN are NaN.  The sign of a NaN result is open in IEEE 754 (x86 and gfx950 differ
    for fp32 inputs), so NaN codes and NaN outputs are compared as NaN, everything else bit for bit."""
    ws = 4
    g = torch.Generator().manual_seed(3)
    shapes = [(16, 4096), (16, 100), (16, 16), (64,), (8, 20000)]
    peers = []
    for p in range(ws):
        ts = []
        for s in shapes:
            x = torch.randn(s, generator=g)
            if x.dim() == 2:
                x[1, 3] = float("nan")
                x[2, 5] = float("inf")
                x[3, 0] = float("-inf")
                x[4, :] = float("nan")
                x[5, 1] = 60000.0 if dtype == torch.float16 else 3e38
                x[5, 2] = float("inf")
            else:
                x[1], x[2], x[3] = float("nan"), float("inf"), float("-inf")
            ts.append(x.to(dtype))
        peers.append(ts)

    def canon(buf):  # 0xFF (NaN with the sign bit) -> 0x7F
        b = buf.cpu().clone()
        b[b == 0xFF] = 0x7F
        return b

    for op in (ReduceOp.SUM, ReduceOp.AVG):
        qg, rg, gg = sim.allreduce(q, [dev(ts) for ts in peers], ws, op)
        qc, rc, gc = sim.allreduce(oracle, [list(ts) for ts in peers], ws, op, nthreads=NT)
        # a scale is never 0xFF-valued in these inputs except as part of a NaN scale, treated alike
        for a, b in zip(qg, qc):
            assert torch.equal(canon(a), canon(b))
        for r in rc:
            assert torch.equal(canon(rg[r]), canon(rc[r]))
        og = [torch.zeros_like(t).cuda() for t in peers[0]]
        oc = [torch.zeros_like(t) for t in peers[0]]
        q.fused_dequantize_from_fp8(og, gg, ws)
        oracle.fused_dequantize_from_fp8(oc, gc, ws, nthreads=NT)
        for a, b in zip(og, oc):
            a = a.cpu()
            assert torch.equal(torch.isnan(a), torch.isnan(b))
            assert torch.equal(torch.nan_to_num(a.float(), nan=0.0), torch.nan_to_num(b.float(), nan=0.0))
            same = ~torch.isnan(a)
            assert torch.equal(torch.signbit(a[same]), torch.signbit(b[same]))


def test_concurrent_threads_and_streams(q, oracle):
    """Eight threads, each on its own stream, hammer the three entry points on shared and on
    private tensor lists at the same time (one plan cache, one library): every result must be
    the checker's."""
    import threading
    ws, rank = 4, 1
    g = torch.Generator().manual_seed(11)
    shared_cpu = [torch.randn(33, 4096, generator=g).to(torch.bfloat16), torch.randn(500, 72, generator=g).to(torch.bfloat16)]
    shared = dev(shared_cpu)
    want_q = oracle.fused_quantize_into_fp8(list(shared_cpu), ws)
    want_r = want_q.clone()
    oracle.fused_reduce_fp8(list(shared_cpu), want_r, ws, rank, ReduceOp.AVG)
    errors = []

    def worker(t):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            gg = torch.Generator().manual_seed(100 + t)
            mine_cpu = [torch.randn(17 + t, 1000 + 8 * t, generator=gg), torch.randn(64 * (t + 1), generator=gg)]
            mine = dev(mine_cpu)
            want_mine = oracle.fused_quantize_into_fp8(list(mine_cpu), ws)
            with torch.cuda.stream(stream):
                for it in range(40):
                    a = q.fused_quantize_into_fp8(shared, ws)
                    b = q.fused_quantize_into_fp8(mine, ws)
                    r = a.clone()
                    q.fused_reduce_fp8(shared, r, ws, rank, ReduceOp.AVG)
                    out = [torch.empty_like(x) for x in mine]
                    q.fused_dequantize_from_fp8(out, b, ws)
                    if it % 13 == 0:
                        stream.synchronize()
                        assert torch.equal(a.cpu(), want_q) and torch.equal(b.cpu(), want_mine)
                        assert torch.equal(r.cpu(), want_r)
                stream.synchronize()
                assert torch.equal(a.cpu(), want_q) and torch.equal(b.cpu(), want_mine) and torch.equal(r.cpu(), want_r)
                ref = [torch.empty_like(x) for x in mine_cpu]
                oracle.fused_dequantize_from_fp8(ref, want_mine, ws)
                for x, y in zip(out, ref):
                    same_bytes(x, y, f"thread {t}")
        except BaseException as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=120)
        assert not th.is_alive()
    if errors:
        raise errors[0]
