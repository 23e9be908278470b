"""Second, independent CPU restatement of the FP8 path, vectorised with torch.

Test infrastructure.  It shares no code with ``oracle/tftq_oracle.c``: the
fp32 -> e4m3fn rounding is torch's own ``float8_e4m3fn`` cast, the fp32
arithmetic is torch's CPU kernels (IEEE, denormals kept), the row packing is
done with tensor views.  The two restatements must agree byte for byte; a
mistake in either (a wrong index, a dropped guard, a different rounding) makes
them differ.  Follows torchft/quantization.py:44-50, 108-123, 131-162,
239-257, 318-375, 405-426, 486-503.
"""

from __future__ import annotations

import torch

INF = float("inf")


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def layout(shapes, ws):
    offs, per_rank, total = [], 0, 0
    for m, n in shapes:
        m_pad = cdiv(m, ws) * ws
        padded = m_pad * (cdiv(n, 4) + 1) * 4
        offs.append(per_rank)
        per_rank += padded // ws
        total += padded
    return offs, per_rank, total


def _shape2d(t):
    return (t.shape[0], 1) if t.dim() == 1 else tuple(t.shape)


def _scale(amax: torch.Tensor) -> torch.Tensor:
    s = torch.tensor(448.0, dtype=torch.float32) / amax
    return torch.where(s == INF, torch.ones_like(s), s)


def _region(buf, p, slot_size, off, slice_rows, row_bytes):
    start = p * slot_size + off
    return buf[start:start + slice_rows * row_bytes].view(slice_rows, row_bytes)


def quantize(inputs, ws):
    shapes = [_shape2d(t) for t in inputs]
    offs, slot_size, total = layout(shapes, ws)
    buf = torch.zeros(total, dtype=torch.uint8)
    for t, (m, n), off in zip(inputs, shapes, offs):
        x = t.reshape(m, n)
        slice_rows = cdiv(m, ws)
        row_bytes = (cdiv(n, 4) + 1) * 4
        amax = x.abs().to(torch.float32).amax(dim=1) if n > 0 else torch.zeros(m)
        s = _scale(amax)
        q = (x.to(torch.float32) * s[:, None]).to(torch.float8_e4m3fn).view(torch.uint8)
        sb = s.contiguous().view(torch.uint8).view(m, 4)
        for p in range(ws):
            lo, hi = p * slice_rows, min((p + 1) * slice_rows, m)
            if lo >= hi:
                continue
            reg = _region(buf, p, slot_size, off, slice_rows, row_bytes)
            reg[: hi - lo, 0:4] = sb[lo:hi]
            reg[: hi - lo, 4:4 + n] = q[lo:hi]
    return buf


def reduce(shapes, buf, ws, rank, is_avg):
    offs, slot_size, total = layout(shapes, ws)
    assert buf.numel() == total
    div = torch.tensor(float(ws) if is_avg else 1.0, dtype=torch.float32)
    for (m, n), off in zip(shapes, offs):
        slice_rows = cdiv(m, ws)
        row_bytes = (cdiv(n, 4) + 1) * 4
        acc = torch.zeros(slice_rows, n, dtype=torch.float32)
        for k in range(ws):
            p = (rank + k) % ws
            reg = _region(buf, p, slot_size, off, slice_rows, row_bytes)
            s = reg[:, 0:4].contiguous().view(torch.float32).view(slice_rows)
            s = torch.where(s == 0.0, torch.ones_like(s), s)
            v = reg[:, 4:4 + n].contiguous().view(torch.float8_e4m3fn).to(torch.float32)
            acc = acc + v / s[:, None]
        amax = acc.abs().amax(dim=1) if n > 0 else torch.zeros(slice_rows)
        s2 = _scale(amax / div)
        q = ((acc * s2[:, None]) / div).to(torch.float8_e4m3fn).view(torch.uint8)
        reg = _region(buf, rank, slot_size, off, slice_rows, row_bytes)
        reg[:, 4:4 + n] = q
        reg[:, 0:4] = s2.contiguous().view(torch.uint8).view(slice_rows, 4)


def dequantize(outputs, buf, ws):
    shapes = [_shape2d(t) for t in outputs]
    offs, slot_size, total = layout(shapes, ws)
    assert buf.numel() == total
    for t, (m, n), off in zip(outputs, shapes, offs):
        slice_rows = cdiv(m, ws)
        row_bytes = (cdiv(n, 4) + 1) * 4
        view = t.view(m, n) if t.dim() == 1 else t
        for p in range(ws):
            lo, hi = p * slice_rows, min((p + 1) * slice_rows, m)
            if lo >= hi:
                continue
            reg = _region(buf, p, slot_size, off, slice_rows, row_bytes)[: hi - lo]
            s = reg[:, 0:4].contiguous().view(torch.float32).view(hi - lo)
            v = reg[:, 4:4 + n].contiguous().view(torch.float8_e4m3fn).to(torch.float32)
            view[lo:hi] = (v / s[:, None]).to(t.dtype)
