"""The numpy-only input generator (tests/gpt2_data.py) draws what the golden fixtures were
made from: checked against the inputs stored in the committed tiny GPT-2 fixtures."""
import numpy as np
import pytest

import fixtures as F
import gpt2_data


@pytest.mark.parametrize("name,bf16", [("gpt2_tiny_bf16", True), ("gpt2_tiny_f32", False)])
def test_named_arrays_reproduce_fixture_inputs(name, bf16):
    fx = F.Fixture(name)
    named = gpt2_data.gpt2_named_arrays(2, 32, 97, 16, 2, seed=3, bf16=bf16)
    seen = 0
    for i in fx.external:
        nm = fx.plan.names[i]
        if nm == "output":
            continue
        assert nm in named, nm
        assert named[nm].dtype == fx.inputs[i].dtype and named[nm].tobytes() == fx.inputs[i].tobytes(), nm
        seen += 1
    assert seen >= 2 * 12 + 6


def test_bf16_round_trip():
    x = np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.14159, -2.5e-3, 65504.0, np.inf], np.float32)
    bits = gpt2_data.f32_to_bf16_bits(x)
    back = gpt2_data.bf16_bits_to_f32(bits)
    assert back[2] == 1.0 and back[3] == 1.0 and back[4] == np.float32(1.015625)    # ties to even, then up
    assert np.all(np.abs(back[:8] - x[:8]) <= np.abs(x[:8]) * 2.0 ** -8) and np.isinf(back[8])
