"""GPU parity: the MI355X engine against the CPU oracle on the same seeded inputs, through the C ABI."""
import numpy as np
import pytest

from genn_amd import configs

pytestmark = pytest.mark.gpu


def test_balanced_lif_bit_exact():
    """C1 shape at full size: one constant weight per projection and one outPost per projection,
    so atomic reordering cannot change a bit — everything must be identical."""
    from parity import run_side_by_side
    net = configs.vogels_abbott(n=4000, steps=1000)
    model, oracle, counts = run_side_by_side(net, check_every=100, exact=True)
    assert counts["E"] > 1000 and counts["I"] > 200
    model.unload()
