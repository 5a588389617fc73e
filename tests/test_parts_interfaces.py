"""What passes between the parts of a block, where it needs no GPU."""
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
