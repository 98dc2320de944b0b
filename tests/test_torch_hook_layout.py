"""Host logic of the PyTorch aggregator that needs no GPU: where the packed stripes sit in the exchange buffers."""
import numpy as np
import pytest
import torch

import oracle
from cntk_amd.torch_hook import stripe_layout


@pytest.mark.parametrize("world_size", [1, 2, 3, 8, 11])
@pytest.mark.parametrize("nbits", [1, 4, 32])
def test_stripe_layout(world_size, nbits):
    shapes = [(300, 96, torch.float32), (144, 40, torch.float32), (96, 1, torch.float32), (2048, 3, torch.float32),
              (130, 24, torch.float64), (7, 0, torch.float32)]
    stripes, rel, slot = stripe_layout(shapes, world_size, nbits)
    assert slot % 8 == 0 and slot >= 8
    for i, (rows, cols, dt) in enumerate(shapes):
        # the workers' stripes partition the columns, in rank order, as the reference's GetStripeForNode cuts them
        nxt = 0
        for s in range(world_size):
            first, n = stripes[s][i]
            assert (first, n) == tuple(oracle.stripe_range(cols, s, world_size))
            assert first == nxt or n == 0
            nxt += n
        assert nxt == cols
    for s in range(world_size):
        # inside a slot the stripes follow each other without overlap, each on an 8-byte boundary, and fit the slot
        end = 0
        for i, (rows, cols, dt) in enumerate(shapes):
            np_dt = np.float64 if dt == torch.float64 else np.float32
            size = stripes[s][i][1] * oracle.qcol_bytes(nbits, rows, np_dt)
            assert rel[s][i] % 8 == 0 and rel[s][i] >= end
            end = rel[s][i] + size
        assert end <= slot
    # the largest worker fills its slot up to the alignment padding
    assert any(slot - 8 * len(shapes) <= rel[s][-1] + stripes[s][-1][1] * oracle.qcol_bytes(nbits, shapes[-1][0], np.float32) <= slot
               for s in range(world_size))
