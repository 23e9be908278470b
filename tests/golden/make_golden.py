"""Writes tests/golden/kat.json: known-answer vectors for the FP8 path.

The vectors are computed here with torch's CPU float32 arithmetic and torch's
own float8_e4m3fn cast (oracle/torch_restatement.py), i.e. without the C checker
under oracle/ and without the HIP library, and were compared by hand with the
closed forms: amax 4 -> scale 448/4 = 112 (0x42E00000); 1*112 = 112 -> 0x6E;
-2*112 = -224 -> 0xF6; 0.5*112 = 56 -> 0x66; 4*112 = 448 -> 0x7E.
Run:  python tests/golden/make_golden.py
"""

import json
import os
import sys

import torch

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", ".."))
from oracle import torch_restatement as tr  # noqa: E402


def hexs(t: torch.Tensor) -> str:
    return bytes(t.contiguous().view(torch.uint8).flatten().tolist()).hex()


def main() -> None:
    out = {}
    # KAT-1: one fp32 row, ws = 1
    r0 = torch.tensor([[1.0, -2.0, 0.5, 4.0]])
    out["kat1_quantize"] = {"dtype": "float32", "shape": [1, 4], "ws": 1,
                            "input_hex": hexs(r0), "packed_hex": hexs(tr.quantize([r0], 1))}
    # KAT-2: two peers each holding a [2,4] tensor; rank 0 reduces row 0
    r1 = torch.tensor([[3.0, 1.0, -0.25, -1.0]])
    z = torch.zeros(1, 4)
    peer0 = torch.cat([r0, z])
    peer1 = torch.cat([r1, z])
    q0, q1 = tr.quantize([peer0], 2), tr.quantize([peer1], 2)
    slot = q0.numel() // 2
    for name, avg in (("sum", False), ("avg", True)):
        recv = torch.cat([q0[:slot], q1[:slot]]).clone()
        tr.reduce([(2, 4)], recv, 2, 0, avg)
        deq = torch.zeros(1, 4)
        tr.dequantize([deq], recv[:slot].clone(), 1)
        out[f"kat2_reduce_{name}"] = {
            "shape": [2, 4], "ws": 2, "rank": 0,
            "recv_hex": hexs(torch.cat([q0[:slot], q1[:slot]])),
            "reduced_hex": hexs(recv), "dequant_slot0_hex": hexs(deq)}
    # KAT-3: zero row, n = 1 rows, tiny amax
    zr = torch.tensor([[0.0, -0.0, 0.0]])
    out["kat3_zero_row"] = {"dtype": "float32", "shape": [1, 3], "ws": 1,
                            "input_hex": hexs(zr), "packed_hex": hexs(tr.quantize([zr], 1))}
    one = torch.tensor([-0.37, 5e-37, 0.0, 448.0])
    out["kat3_n1_rows"] = {"dtype": "float32", "shape": [4], "ws": 1,
                           "input_hex": hexs(one), "packed_hex": hexs(tr.quantize([one], 1))}
    # odd shapes, three dtypes, ws = 4: full packed buffers
    g = torch.Generator().manual_seed(1234)
    for dt in (torch.float32, torch.float16, torch.bfloat16):
        a = (torch.randn(5, 3, generator=g) * 3).to(dt)
        b = (torch.randn(1, 7, generator=g) * 1e-3).to(dt)
        c = (torch.randn(6, generator=g) * 50).to(dt)
        buf = tr.quantize([a, b, c], 4)
        red = buf.clone()
        tr.reduce([(5, 3), (1, 7), (6, 1)], red, 4, 2, True)
        oa, ob, oc = torch.zeros_like(a), torch.zeros_like(b), torch.zeros_like(c)
        tr.dequantize([oa, ob, oc], buf, 4)
        out[f"odd_{str(dt).split('.')[1]}"] = {
            "dtype": str(dt).split(".")[1], "shapes": [[5, 3], [1, 7], [6]], "ws": 4,
            "inputs_hex": [hexs(a), hexs(b), hexs(c)], "packed_hex": hexs(buf),
            "reduced_rank2_avg_hex": hexs(red),
            "dequant_hex": [hexs(oa), hexs(ob), hexs(oc)]}
    path = os.path.join(os.path.dirname(__file__), "kat.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print("wrote", path)


if __name__ == "__main__":
    main()
