"""Pins the CPU checker (oracle/tftq_oracle.c).

What pins what:
  layout      closed-form worked examples; invariants (equal slots, injective
              row addresses, total = ws * slot)
  scale       closed form and special cases (0, tiny, 448, 1)
  e4m3 codec  torch's float8_e4m3fn cast (an independent library routine):
              all 256 codes decoded, all 65536 bf16 patterns and 2M random and
              boundary fp32 values encoded
  f16 / bf16  numpy float16 and torch bfloat16 casts
  Q / R / D   golden vectors in tests/golden/kat.json (hand-checked closed
              forms); byte equality with the independent torch restatement
              (oracle/torch_restatement.py) on random, odd, strided inputs; a
              straight-line numpy-float32 brute force on tiny inputs;
              mathematical special cases (ws = 1 SUM is the identity on codes,
              identical peers with power-of-two ws average back to the input
              codes, arg-max of a row encodes to 0x7E / 0xFE, decode within half
              an fp8 ULP of the input)
"""

import json
import os

import numpy as np
import pytest
import torch
from torch.distributed import ReduceOp

from oracle import torch_restatement as tr
import workloads

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "kat.json")))
DT = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}


def from_hex(h, dtype=torch.uint8):
    return torch.frombuffer(bytearray(bytes.fromhex(h)), dtype=dtype).clone()


# ---- layout -----------------------------------------------------------------
def test_layout_worked_examples(oracle):
    assert oracle.layout([(256, 512), (1024, 1)], 2) == ([0, 66048], 70144, 140288)
    assert oracle.layout([(5, 3), (1, 7)], 4) == ([0, 16], 28, 112)
    # benchmark configurations 2, 3 and 4
    assert oracle.layout([(4096, 4096)], 8)[1:] == (2099200, 16793600)
    shp = [s if len(s) == 2 else (s[0], 1) for _, s in workloads.LLAMA3_8B_LAYER]
    assert oracle.layout(shp, 8)[1:] == (27292672, 218341376)
    shp4 = [s if len(s) == 2 else (s[0], 1) for s in workloads.diloco_1b_shapes()]
    assert len(shp4) == 201
    assert oracle.layout(shp4, 4)[1:] == (275631616, 1102526464)


def test_layout_invariants(oracle):
    g = torch.Generator().manual_seed(0)
    for _ in range(50):
        T = int(torch.randint(1, 6, (1,), generator=g))
        ws = int(torch.randint(1, 9, (1,), generator=g))
        shapes = [(int(torch.randint(0, 40, (1,), generator=g)),
                   int(torch.randint(0, 40, (1,), generator=g))) for _ in range(T)]
        offs, slot, total = oracle.layout(shapes, ws)
        assert total == slot * ws and total % 4 == 0
        assert (offs, slot, total) == tr.layout(shapes, ws)
        seen = set()
        for (m, n), off in zip(shapes, offs):
            sr = -(-m // ws)
            rb = (-(-n // 4) + 1) * 4
            for r in range(sr * ws):
                a = (r // sr) * slot + off + (r % sr) * rb
                assert a % 4 == 0 and a + rb <= total
                assert a // slot == r // sr  # row stays inside its slot
                assert a not in seen
                seen.add(a)


# ---- scalar pieces ----------------------------------------------------------
def test_scale_special_cases(oracle):
    L = oracle.lib()
    assert L.tftq_oracle_scale(0.0) == 1.0
    assert L.tftq_oracle_scale(448.0) == 1.0
    assert L.tftq_oracle_scale(1.0) == 448.0
    assert L.tftq_oracle_scale(4.0) == 112.0
    assert L.tftq_oracle_scale(1e-37) == 1.0          # 448 / 1e-37 overflows
    assert L.tftq_oracle_scale(2e-36) == np.float32(448.0) / np.float32(2e-36)
    assert L.tftq_oracle_scale(float("inf")) == 0.0


def test_e4m3_decode_all_codes(oracle):
    L = oracle.lib()
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32)
    for c in range(256):
        v = L.tftq_oracle_e4m3_to_f32(c)
        if c & 0x7F == 0x7F:
            assert np.isnan(v) and torch.isnan(ref[c])
        else:
            assert np.float32(v).tobytes() == ref[c].numpy().tobytes(), c


def _encode_many(oracle, x: torch.Tensor) -> torch.Tensor:
    """Encodes through the oracle's quantize with scale 1 is not possible, so
    call the scalar routine via a vectorised ctypes loop."""
    L = oracle.lib()
    f = L.tftq_oracle_f32_to_e4m3
    return torch.tensor([f(float(v)) for v in x.tolist()], dtype=torch.uint8)


def test_e4m3_encode_vs_torch_cast(oracle):
    # all bf16 bit patterns (exactly representable in fp32)
    allbf = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).to(torch.float32)
    g = torch.Generator().manual_seed(1)
    rnd = torch.randn(200000, generator=g) * 10 ** (torch.rand(200000, generator=g) * 8 - 5)
    edge = torch.linspace(440.0, 470.0, 30001)
    ties = torch.tensor([17.0, 19.0, 1.5 * 2 ** -9, 2.5 * 2 ** -9, 2 ** -10, 2 ** -10 * 1.0001,
                         464.0, 464.00003, 0.0, -0.0, 2 ** -6 * 0.9999, 448.0, -448.0])
    sub = torch.linspace(0, 2 ** -5, 40001)
    x = torch.cat([allbf, rnd, edge, -edge, ties, sub, -sub])
    x = x[~torch.isnan(x)]
    want = x.to(torch.float8_e4m3fn).view(torch.uint8)
    got = _encode_many(oracle, x)
    bad = (want != got).nonzero()
    assert bad.numel() == 0, (x[bad[:5]], want[bad[:5]], got[bad[:5]])


def test_half_and_bf16_store_casts(oracle):
    L = oracle.lib()
    g = torch.Generator().manual_seed(2)
    x = torch.cat([torch.randn(50000, generator=g) * 10 ** (torch.rand(50000, generator=g) * 12 - 8),
                   torch.tensor([65504.0, 65519.9, 65520.0, 1e6, 2 ** -24, 2 ** -25, 2 ** -25 * 1.001,
                                 2 ** -14, 0.0, -0.0, 1.0009765625, 1.00048828125])])
    want16 = x.numpy().astype(np.float16).view(np.uint16)
    wantbf = x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    for i, v in enumerate(x.tolist()):
        assert L.tftq_oracle_f32_to_f16(v) == want16[i], v
        assert L.tftq_oracle_f32_to_bf16(v) == wantbf[i], v
    for h in range(0, 65536, 7):
        v = np.array([h], dtype=np.uint16).view(np.float16).astype(np.float32)[0]
        o = L.tftq_oracle_f16_to_f32(h)
        assert (np.isnan(v) and np.isnan(o)) or np.float32(o).tobytes() == v.tobytes()


# ---- golden vectors ---------------------------------------------------------
def test_golden_kat1_closed_form(oracle):
    k = KAT["kat1_quantize"]
    assert k["packed_hex"] == "0000e0426ef6667e"  # scale 112.0, codes 112 -224 56 448
    x = from_hex(k["input_hex"]).view(torch.float32).view(1, 4)
    assert bytes(oracle.fused_quantize_into_fp8([x], 1).tolist()).hex() == k["packed_hex"]


@pytest.mark.parametrize("name,op", [("sum", ReduceOp.SUM), ("avg", ReduceOp.AVG)])
def test_golden_kat2_reduce(oracle, name, op):
    k = KAT[f"kat2_reduce_{name}"]
    recv = from_hex(k["recv_hex"])
    shape = [torch.empty(2, 4)]
    oracle.fused_reduce_fp8(shape, recv, 2, 0, op)
    assert bytes(recv.tolist()).hex() == k["reduced_hex"]
    # hand-checked: SUM keeps scale 112 (0x42E00000), AVG doubles it (0x43600000)
    assert k["reduced_hex"][:8] == ("0000e042" if name == "sum" else "00006043")
    assert k["reduced_hex"][8:16] == "7eee5e7b"
    out = torch.zeros(1, 4)
    oracle.fused_dequantize_from_fp8([out], recv[:8].clone(), 1)
    assert bytes(out.view(torch.uint8).flatten().tolist()).hex() == k["dequant_slot0_hex"]


def test_golden_kat3_zero_and_n1(oracle):
    k = KAT["kat3_zero_row"]
    x = from_hex(k["input_hex"]).view(torch.float32).view(1, 3)
    assert bytes(oracle.fused_quantize_into_fp8([x], 1).tolist()).hex() == k["packed_hex"] == "0000803f00800000"
    k = KAT["kat3_n1_rows"]
    x = from_hex(k["input_hex"]).view(torch.float32)
    got = bytes(oracle.fused_quantize_into_fp8([x], 1).tolist()).hex()
    assert got == k["packed_hex"]
    assert got[8:10] == "fe" and got[16:24] == "0000803f" and got[24:26] == "00"


@pytest.mark.parametrize("dt", ["float32", "float16", "bfloat16"])
def test_golden_odd_shapes(oracle, dt):
    k = KAT[f"odd_{dt}"]
    dtype = DT[dt]
    view = {torch.float32: torch.float32, torch.float16: torch.float16, torch.bfloat16: torch.bfloat16}[dtype]
    ins = []
    for h, shp in zip(k["inputs_hex"], k["shapes"]):
        ins.append(from_hex(h).view(view).view(*shp))
    buf = oracle.fused_quantize_into_fp8(list(ins), k["ws"])
    assert bytes(buf.tolist()).hex() == k["packed_hex"]
    red = buf.clone()
    oracle.fused_reduce_fp8(list(ins), red, k["ws"], 2, ReduceOp.AVG)
    assert bytes(red.tolist()).hex() == k["reduced_rank2_avg_hex"]
    outs = [torch.zeros_like(t) for t in ins]
    oracle.fused_dequantize_from_fp8(list(outs), buf, k["ws"])
    for o, h in zip(outs, k["dequant_hex"]):
        assert bytes(o.contiguous().view(torch.uint8).flatten().tolist()).hex() == h


# ---- C checker vs the independent torch restatement -------------------------
def _rand_inputs(g, dtype, shapes, mult=1.0):
    return [(torch.randn(s, generator=g) * mult).to(dtype) for s in shapes]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ws", [1, 2, 3, 4, 8])
def test_c_vs_torch_restatement(oracle, dtype, ws):
    g = torch.Generator().manual_seed(100 + ws)
    shapes = [(7, 5), (16, 64), (3,), (1, 130), (9, 1), (33, 17), (2, 2050)]
    peers = [_rand_inputs(g, dtype, shapes, mult=10.0 ** (p - 4)) for p in range(ws)]  # finite in fp16
    for p in range(ws):  # zero rows, negative zeros
        peers[p][0][2] = 0.0
        peers[p][1][5, ::2] = -0.0
    qs_c = [oracle.fused_quantize_into_fp8(list(t), ws) for t in peers]
    qs_t = [tr.quantize(t, ws) for t in peers]
    for a, b in zip(qs_c, qs_t):
        assert torch.equal(a, b)
    slot = qs_c[0].numel() // ws
    shp2 = [tr._shape2d(t) for t in peers[0]]
    for op, avg in ((ReduceOp.SUM, False), (ReduceOp.AVG, True)):
        gathered = torch.empty_like(qs_c[0])
        for r in range(ws):
            recv = torch.cat([q[r * slot:(r + 1) * slot] for q in qs_c])
            recv_t = recv.clone()
            oracle.fused_reduce_fp8(list(peers[0]), recv, ws, r, op)
            tr.reduce(shp2, recv_t, ws, r, avg)
            assert torch.equal(recv, recv_t), (op, r)
            gathered[r * slot:(r + 1) * slot] = recv[r * slot:(r + 1) * slot]
        out_c = [torch.zeros_like(t) for t in peers[0]]
        out_t = [torch.zeros_like(t) for t in peers[0]]
        oracle.fused_dequantize_from_fp8(list(out_c), gathered, ws)
        tr.dequantize(out_t, gathered, ws)
        for a, b in zip(out_c, out_t):
            assert torch.equal(a.view(-1).view(torch.uint8), b.view(-1).view(torch.uint8))


def test_c_vs_torch_restatement_strided(oracle):
    g = torch.Generator().manual_seed(7)
    base = torch.randn(40, 50, generator=g)
    views = [base[::2, 1:40:3], base.t()[3:17], base[5:6, :]]
    q_c = oracle.fused_quantize_into_fp8(list(views), 4)
    q_t = tr.quantize([v.contiguous() for v in views], 4)
    assert torch.equal(q_c, q_t)
    outb = torch.zeros(40, 50)
    outs = [outb[::2, 1:40:3], outb.t()[3:17]]
    q2 = oracle.fused_quantize_into_fp8(list(views[:2]), 4)
    oracle.fused_dequantize_from_fp8(list(outs), q2, 4)
    ref = [torch.zeros_like(v.contiguous()) for v in views[:2]]
    tr.dequantize(ref, q2, 4)
    # the transposed view overlaps the first one; compare the one written last
    assert torch.equal(outs[1], ref[1])


def test_cfg1_plumbing(oracle):
    """Benchmark configuration 1 (two fp32 tensors, 2 peers, SUM), end to end on the CPU checker."""
    peers = [workloads.cfg1(s) for s in (0, 1)]
    qs = [oracle.fused_quantize_into_fp8(list(t), 2) for t in peers]
    assert qs[0].numel() == 140288
    for q, t in zip(qs, peers):
        assert torch.equal(q, tr.quantize(t, 2))
    slot = 70144
    gathered = torch.empty_like(qs[0])
    for r in range(2):
        recv = torch.cat([q[r * slot:(r + 1) * slot] for q in qs])
        oracle.fused_reduce_fp8(list(peers[0]), recv, 2, r, ReduceOp.SUM)
        gathered[r * slot:(r + 1) * slot] = recv[r * slot:(r + 1) * slot]
    outs = [torch.zeros(256, 512), torch.zeros(1024)]
    oracle.fused_dequantize_from_fp8(outs, gathered, 2)
    for o, a, b in zip(outs, peers[0], peers[1]):
        ref = (a + b).view_as(o)
        # two quantizations, each within 1/16 relative (3 mantissa bits) of the row max
        rowmax = ref.abs().amax(dim=1, keepdim=True).clamp_min(1e-30)
        assert ((o - ref).abs() / rowmax).max() < 0.13


# ---- brute force and mathematical special cases -----------------------------
def test_reduce_brute_force_tiny(oracle):
    """Straight-line numpy float32 restatement of :405-426 and :340-375."""
    g = torch.Generator().manual_seed(3)
    f32 = np.float32
    dec = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    for ws in (1, 2, 3, 4):
        for n in (1, 2, 5, 8):
            peers = [[torch.randn(ws, n, generator=g) * (p + 1)] for p in range(ws)]
            qs = [oracle.fused_quantize_into_fp8(list(t), ws) for t in peers]
            slot = qs[0].numel() // ws
            rb = (-(-n // 4) + 1) * 4
            for rank in range(ws):
                for avg in (False, True):
                    recv = torch.cat([q[rank * slot:(rank + 1) * slot] for q in qs])
                    raw = recv.numpy().copy()
                    oracle.fused_reduce_fp8(list(peers[0]), recv, ws, rank,
                                            ReduceOp.AVG if avg else ReduceOp.SUM)
                    div = f32(ws) if avg else f32(1.0)
                    acc = [f32(0.0)] * n
                    for k in range(ws):
                        p = (rank + k) % ws
                        s = raw[p * slot:p * slot + 4].view(np.float32)[0]
                        s = f32(1.0) if s == 0 else s
                        for c in range(n):
                            acc[c] = f32(acc[c] + f32(dec[raw[p * slot + 4 + c]] / s))
                    amax = max(abs(a) for a in acc)
                    with np.errstate(divide="ignore"):
                        s2 = f32(448.0) / f32(amax / div)
                    s2 = f32(1.0) if np.isinf(s2) else s2
                    y = torch.tensor([float(f32(f32(a * s2) / div)) for a in acc])
                    codes = y.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
                    got = recv.numpy()[rank * slot:rank * slot + rb]
                    assert got[:4].view(np.float32)[0] == s2
                    assert (got[4:4 + n] == codes).all()
                    assert (got[4 + n:] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_quantize_properties(oracle, dtype):
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(64, 96, generator=g) * 10 ** (torch.rand(64, 1, generator=g) * 6 - 4)).to(dtype)
    x[5] = 0
    q = oracle.fused_quantize_into_fp8([x], 1).view(64, 100)
    s = q[:, :4].contiguous().view(torch.float32).view(64)
    codes = q[:, 4:]
    xf = x.to(torch.float32)
    amax = xf.abs().amax(dim=1)
    assert s[5] == 1.0 and (codes[5] == 0).all()
    nz = amax > 0
    assert torch.equal(s[nz], (torch.tensor(448.0) / amax)[nz])  # tensor / tensor: IEEE divide
    arg = xf.abs().argmax(dim=1)
    top = codes[torch.arange(64), arg] & 0x7F
    assert (top[nz] == 0x7E).all()
    dec = codes.view(torch.float8_e4m3fn).to(torch.float32) / s[:, None]
    # half an fp8 ULP: 2^-4 relative for normals, 2^-10 / s absolute for subnormals
    tol = torch.maximum(xf.abs() * 2 ** -4, (2 ** -10 / s)[:, None]) * 1.0001
    assert ((dec - xf).abs() <= tol).all()


def test_reduce_special_cases(oracle):
    g = torch.Generator().manual_seed(5)
    x = [torch.randn(8, 40, generator=g), torch.randn(12, generator=g)]
    # ws = 1, SUM: reduce is dequantize o quantize of codes that are already fp8 -> identity
    q = oracle.fused_quantize_into_fp8(list(x), 1)
    r = q.clone()
    oracle.fused_reduce_fp8(list(x), r, 1, 0, ReduceOp.SUM)
    assert torch.equal(q, r)
    # identical peers, AVG: for ws = 2 acc = 2 * x_hat exactly, so codes and scale return
    # bit for bit; for ws = 4, 8 the running sum 3 * x_hat, ... rounds, which moves the
    # new scale by a few fp32 ulps at most and cannot move a code (acc * s' sits on an fp8
    # value, far from a rounding boundary)
    for ws in (2, 4, 8):
        q = oracle.fused_quantize_into_fp8(list(x), ws)
        slot = q.numel() // ws
        for rank in range(ws):
            own = q[rank * slot:(rank + 1) * slot]
            recv = own.repeat(ws)
            oracle.fused_reduce_fp8(list(x), recv, ws, rank, ReduceOp.AVG)
            got = recv[rank * slot:(rank + 1) * slot]
            want = own.clone()
            # padding rows of the own slot get scale 1.0 after reduce
            for (m, n), off in zip([(8, 40), (12, 1)], oracle.layout([(8, 40), (12, 1)], ws)[0]):
                sr, rb = -(-m // ws), (-(-n // 4) + 1) * 4
                for j in range(sr):
                    if rank * sr + j >= m:
                        want[off + j * rb: off + j * rb + 4] = torch.tensor([0, 0, 0x80, 0x3F], dtype=torch.uint8)
            if ws == 2:
                assert torch.equal(got, want), (ws, rank)
            else:
                for (m, n), off in zip([(8, 40), (12, 1)], oracle.layout([(8, 40), (12, 1)], ws)[0]):
                    sr, rb = -(-m // ws), (-(-n // 4) + 1) * 4
                    g_rows = got[off:off + sr * rb].view(sr, rb)
                    w_rows = want[off:off + sr * rb].view(sr, rb)
                    assert torch.equal(g_rows[:, 4:], w_rows[:, 4:]), (ws, rank)
                    gs = g_rows[:, :4].contiguous().view(torch.int32)
                    wsc = w_rows[:, :4].contiguous().view(torch.int32)
                    assert (gs - wsc).abs().max() <= 4, (ws, rank)
            # other slots untouched
            mask = torch.ones(ws * slot, dtype=torch.bool)
            mask[rank * slot:(rank + 1) * slot] = False
            assert torch.equal(recv[mask], own.repeat(ws)[mask])
