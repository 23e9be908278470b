"""Synthetic workloads of the five benchmark configurations (test and bench
infrastructure; generated on the CPU from seeds so that the CPU checker and the
GPU see identical bits)."""

from __future__ import annotations

import math

import torch

LLAMA3_8B_LAYER = [
    ("q", (4096, 4096)), ("k", (1024, 4096)), ("v", (1024, 4096)), ("o", (4096, 4096)),
    ("gate", (14336, 4096)), ("up", (14336, 4096)), ("down", (4096, 14336)),
    ("norm1", (4096,)), ("norm2", (4096,)),
]


def diloco_1b_shapes(layers: int = 22, hidden: int = 2048, inter: int = 5632,
                     kv: int = 256, vocab: int = 32000):
    shapes = [(vocab, hidden)]
    for _ in range(layers):
        shapes += [(hidden, hidden), (kv, hidden), (kv, hidden), (hidden, hidden),
                   (inter, hidden), (inter, hidden), (hidden, inter), (hidden,), (hidden,)]
    shapes += [(hidden,), (vocab, hidden)]
    return shapes


def cfg1(seed: int, device="cpu"):
    g = torch.Generator(device=device).manual_seed(seed)
    return [torch.randn(256, 512, generator=g, device=device),
            torch.randn(1024, generator=g, device=device)]


def cfg2(seed: int, device="cpu", rows: int = 4096):
    g = torch.Generator(device=device).manual_seed(seed)
    return [(torch.randn(rows, 4096, generator=g, device=device) * 0.02).to(torch.bfloat16)]


def cfg3(seed: int, device="cpu", scale_rows: float = 1.0):
    """Llama-3-8B decoder-layer gradient bucket, bf16; per-row std log-uniform in
    [1e-5, 1e-1].  scale_rows < 1 shrinks the row counts (not the row lengths)."""
    g = torch.Generator(device=device).manual_seed(seed)
    out = []
    for _, shp in LLAMA3_8B_LAYER:
        m = max(1, int(round(shp[0] * scale_rows)))
        full = (m,) + tuple(shp[1:])
        std = 10.0 ** (torch.rand(m, generator=g, device=device) * 4.0 - 5.0)
        x = torch.randn(full, generator=g, device=device)
        x = x * (std[:, None] if len(full) == 2 else std)
        out.append(x.to(torch.bfloat16))
    return out


def cfg4(seed: int, device="cpu", layers: int = 22, vocab: int = 32000):
    """DiLoCo pseudo-gradient of a 1.1B model, fp32, Student-t(df=3) * 1e-4."""
    g = torch.Generator(device=device).manual_seed(seed)
    out = []
    for shp in diloco_1b_shapes(layers=layers, vocab=vocab):
        z = torch.randn(shp, generator=g, device=device)
        chi = (torch.randn((3,) + tuple(shp), generator=g, device=device) ** 2).sum(0) / 3.0
        out.append(z / chi.sqrt() * 1e-4)
    return out


def cfg5_shapes(count: int, seed: int = 5):
    """Shapes for the edge-case stress: element counts uniform in [1, 4096], row
    lengths never a multiple of 16; 1-D tensors (n = 1), n < 4 and n % 4 != 0
    all occur."""
    g = torch.Generator().manual_seed(seed)
    es = torch.randint(1, 4097, (count,), generator=g).tolist()
    kinds = torch.randint(0, 8, (count,), generator=g).tolist()
    ns = torch.randint(1, 4097, (count,), generator=g).tolist()
    shapes = []
    for e, kind, nr in zip(es, kinds, ns):
        if kind == 0:
            shapes.append((e,))  # 1-D -> [e, 1]
            continue
        if kind == 1:
            n = 1 + nr % 3  # 1..3
        elif kind == 2:
            n = e  # a single row
        else:
            n = 1 + nr % max(1, min(e, 600))
        if n % 16 == 0:
            n += 1
        m = max(1, e // n)
        shapes.append((m, n))
    return shapes


def cfg5(seed: int, dtype, shapes, device="cpu"):
    g = torch.Generator(device=device).manual_seed(seed * 7919 + 11)
    out = []
    for shp in shapes:
        x = torch.randn(shp, generator=g, device=device) * 1e-3
        u = torch.rand(shp, generator=g, device=device)
        sign = torch.where(torch.rand(shp, generator=g, device=device) < 0.5, -1.0, 1.0)
        x = torch.where(u < 1e-4, sign * 1e4, x)
        rows = torch.rand(shp[0], generator=g, device=device) < 0.01
        x[rows] = 0.0
        out.append(x.to(dtype))
    return out


def input_bytes(tensors) -> int:
    return sum(t.numel() * t.element_size() for t in tensors)


def packed_bytes(tensors, ws: int) -> int:
    total = 0
    for t in tensors:
        m, n = (t.shape[0], 1) if t.dim() == 1 else t.shape
        total += math.ceil(m / ws) * ws * (math.ceil(n / 4) + 1) * 4
    return total


def algorithmic_bytes(tensors, ws: int) -> dict:
    """Bytes a stage must move: Q and D = tensors + packed buffer; R = packed
    buffer read once + own slot written."""
    inp, out = input_bytes(tensors), packed_bytes(tensors, ws)
    return {"quantize": inp + out, "reduce": out + out // ws, "dequantize": out + inp}
