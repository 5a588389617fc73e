"""What passes between the parts of a block, where it needs no GPU."""
import numpy as np
import pytest
import torch

from nanoinfer_amd.parts.base import pending_for


def test_addends_are_summed_for_a_norm_that_does_not_take_them():
    """A product of a few rows may hand its result on as float32 addends [S, T, d]; a norm that says
    ``takes_addends`` gets them as they are, any other gets their sum in the compute type."""
    class TakesAddends:
        takes_addends = True

    class PlainNorm:
        pass

    addends = torch.arange(24, dtype=torch.float32).view(3, 2, 4)
    assert pending_for(TakesAddends(), addends, torch.bfloat16) is addends
    summed = pending_for(PlainNorm(), addends, torch.bfloat16)
    assert summed.dtype == torch.bfloat16 and torch.equal(summed.float(), addends.sum(0))
    one = torch.zeros(2, 4, dtype=torch.bfloat16)
    assert pending_for(PlainNorm(), one, torch.bfloat16) is one
    assert pending_for(PlainNorm(), None, torch.bfloat16) is None


def test_rotation_frequencies_of_the_engine_as_numbers():
    """The engine's frequencies against the worked numbers of tests/rope_literals.py (the plain
    implementation is held to the same numbers, each by a test of its own)."""
    from nanoinfer_amd.parts.standard import rope_inverse_frequencies
    from rope_literals import CASES
    for hd, theta, scaling, pairs in CASES:
        f = rope_inverse_frequencies(hd, theta, dict(scaling, kind="llama3"))
        assert f.dtype == np.float32 and f.shape == (hd // 2,)
        for p, (band, value) in pairs.items():
            assert float(f[p]) == pytest.approx(value, rel=1e-5), (hd, p, band)
    plain = rope_inverse_frequencies(16, 10000.0, None)
    assert [float(x) for x in plain[:3]] == pytest.approx([1.0, 10000.0 ** -0.125, 10000.0 ** -0.25], rel=1e-6)


def test_another_rotation_scaling_is_a_registered_rule():
    """A scaling rule is looked up by the ``kind`` of the part's ``scaling`` parameter: another one
    (here: every frequency divided by a factor) is registered from outside, and an unknown kind is an error."""
    from nanoinfer_amd.parts.standard import register_rope_scaling, rope_inverse_frequencies

    @register_rope_scaling("test-linear")
    def linear(freqs, params):
        return freqs / np.float32(params["factor"])

    base = rope_inverse_frequencies(32, 10000.0, None)
    got = rope_inverse_frequencies(32, 10000.0, {"kind": "test-linear", "factor": 4.0})
    assert np.allclose(got, base / 4.0, rtol=1e-7)
    with pytest.raises(ValueError, match="not registered"):
        rope_inverse_frequencies(32, 10000.0, {"kind": "no-such-rule"})
    with pytest.raises(ValueError, match="not registered"):
        rope_inverse_frequencies(32, 10000.0, {"factor": 4.0})
