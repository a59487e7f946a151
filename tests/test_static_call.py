"""Host logic of the recorded-call inputs (``tybok_amd.graph.StaticCall``): no GPU, no recording."""
import pytest
import torch

from tybok_amd.graph import StaticCall


def _call():
    return StaticCall(torch.zeros(1), noise=torch.full((1, 4, 8), 7.0), state=torch.zeros(1, 8), images=[torch.zeros(2), torch.zeros(2)])


def test_store_leading_keeps_the_zero_padding_of_a_padded_store():
    # a value narrower than its static tensor lands in the leading columns; what lies behind it reads as zeros,
    # whatever an earlier request (a wider value, noise drawn in place, a plain store) left there
    call = _call()
    a = torch.arange(12.0).view(1, 4, 3) + 1
    call.store_leading(noise=a)  # the first store clears what recording left behind the value
    want = torch.nn.functional.pad(a, (0, 5))
    assert torch.equal(call.inputs["noise"], want)
    wide = torch.ones(1, 4, 6) * 3
    call.store_leading(noise=wide)
    assert torch.equal(call.inputs["noise"], torch.nn.functional.pad(wide, (0, 2)))
    call.store_leading(noise=a)  # narrower than the last one: columns 3..5 must be cleared again
    assert torch.equal(call.inputs["noise"], want)
    call.inputs["noise"].fill_(9.0)  # (noise drawn in place)
    call.forget_leading("noise")
    call.store_leading(noise=a)
    assert torch.equal(call.inputs["noise"], want)
    call.store(noise=torch.full((1, 4, 8), 5.0))  # a plain store forgets the width as well
    call.store_leading(noise=a)
    assert torch.equal(call.inputs["noise"], want)
    full = torch.randn(1, 4, 8)
    call.store_leading(noise=full)
    assert torch.equal(call.inputs["noise"], full)


def test_store_leading_refuses_what_does_not_fit():
    call = _call()
    with pytest.raises(ValueError):
        call.store_leading(state=torch.zeros(1, 9))
    with pytest.raises(ValueError):
        call.store_leading(state=torch.zeros(2, 4))
    with pytest.raises(ValueError):
        call.store(images=[torch.zeros(2)])


def test_store_owned_copies_only_new_objects():
    call = _call()
    t = torch.ones(1, 8)
    call.store_owned(state=t)
    call.inputs["state"].zero_()
    call.store_owned(state=t)  # the very object stored last time: not copied again
    assert torch.count_nonzero(call.inputs["state"]) == 0
    call.forget_owned("state")
    call.store_owned(state=t)
    assert torch.equal(call.inputs["state"], t)
