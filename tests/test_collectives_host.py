"""CPU-side checks of torchft_amd.collectives: size helpers and option handling
(no kernel is launched)."""

import torch

from torchft_amd import collectives as coll


def test_get_padded_sizes():
    ts = [torch.zeros(5, 3), torch.zeros(7), torch.zeros(8, 2, 2)]
    assert coll.get_padded_sizes(ts, 4) == [torch.Size((8, 3)), torch.Size((8, 1)), torch.Size((8, 2, 2))]
    assert coll.get_padded_sizes(ts, 1) == [torch.Size((5, 3)), torch.Size((7, 1)), torch.Size((8, 2, 2))]


def test_allocate_reduce_scatter_output():
    ts = [torch.zeros(5, 3, dtype=torch.bfloat16), torch.zeros(7, dtype=torch.bfloat16)]
    out, padded = coll.allocate_reduce_scatter_output(ts, 4)
    assert padded == [torch.Size((8, 3)), torch.Size((8, 1))]
    assert out.shape == (2 * 3 + 2 * 1,) and out.dtype == torch.bfloat16
    try:
        coll.allocate_reduce_scatter_output([torch.zeros(2), torch.zeros(2, dtype=torch.float16)], 2)
    except AssertionError as e:
        assert "same dtype" in str(e)
    else:
        raise AssertionError("dtype mismatch not detected")
