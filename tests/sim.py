"""One-process simulation of the quantized all-reduce / reduce-scatter data flow
(torchft/collectives.py:364-412 and :240-290) with the two collectives replaced
by slot copies: all-to-all gives rank r slot r of every peer
(process_group_test.py:255-296), all-gather collects slot r of every rank's
reduced buffer (:175-215).  `impl` is any module with the three fused_*
functions (torchft_amd.quantization on the GPU, oracle.oracle on the CPU)."""

from __future__ import annotations

import torch


def quantize_peers(impl, peers, ws, **kw):
    return [impl.fused_quantize_into_fp8(list(t), ws, **kw) for t in peers]


def recv_buffer(qs, rank, ws):
    slot = qs[0].numel() // ws
    return torch.cat([q[rank * slot:(rank + 1) * slot] for q in qs])


def allreduce(impl, peers, ws, op, ranks=None, **kw):
    """Returns (quantized per peer, reduced recv buffer per rank, gathered buffer).
    `ranks` limits the ranks that are reduced (the gathered buffer then only has
    those slots filled; the rest is zero)."""
    qs = quantize_peers(impl, peers, ws, **kw)
    slot = qs[0].numel() // ws
    gathered = torch.zeros_like(qs[0])
    reduced = {}
    for r in (range(ws) if ranks is None else ranks):
        recv = recv_buffer(qs, r, ws)
        impl.fused_reduce_fp8(list(peers[0]), recv, ws, r, op, **kw)
        reduced[r] = recv
        gathered[r * slot:(r + 1) * slot] = recv[r * slot:(r + 1) * slot]
    return qs, reduced, gathered
