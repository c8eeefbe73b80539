"""The parity helper itself: that it fails what it is there to fail."""
import pytest
import torch

from helpers import assert_close_bf16


def _bf16_result(ref):
    return ref.to(torch.bfloat16)


@pytest.mark.parametrize("scale", [1.0, 1e-3, 3e-5])
def test_rounded_reference_passes_at_every_magnitude(scale):
    g = torch.Generator().manual_seed(1)
    ref = torch.randn(4096, 128, generator=g) * scale
    assert_close_bf16(_bf16_result(ref), ref, "rounded")


@pytest.mark.parametrize("scale", [1.0, 1e-3, 3e-5])
def test_five_per_cent_of_entries_doubled_fails(scale):
    """Small-valued tensors (the outputs and gradients of rows that average several hundred thousand keys are 1e-4 to
    1e-2) must be held to their own magnitude: 5 % of the entries off by a factor of two has to fail there as it
    does at N(0,1) scale."""
    g = torch.Generator().manual_seed(2)
    ref = torch.randn(4096, 128, generator=g) * scale
    got = ref.clone()
    bad = torch.rand(ref.shape, generator=g) < 0.05
    got[bad] *= 2
    with pytest.raises(AssertionError):
        assert_close_bf16(_bf16_result(got), ref, "doubled")


@pytest.mark.parametrize("scale", [1.0, 1e-3])
def test_one_entry_off_by_its_own_size_fails(scale):
    g = torch.Generator().manual_seed(3)
    ref = torch.randn(512, 128, generator=g) * scale
    got = ref.clone()
    got[17, 5] = ref[17, 5] + ref.abs().max()
    with pytest.raises(AssertionError):
        assert_close_bf16(_bf16_result(got), ref, "one entry")


def test_everything_ten_times_too_large_fails_for_small_values():
    g = torch.Generator().manual_seed(4)
    ref = torch.randn(1024, 128, generator=g) * 4e-5
    with pytest.raises(AssertionError):
        assert_close_bf16(_bf16_result(ref * 10), ref, "times ten")


def test_zero_reference_needs_a_zero_result():
    ref = torch.randn(64, 128) * 1e-8          # fp32 rounding noise around an exact zero
    assert_close_bf16(torch.zeros(64, 128, dtype=torch.bfloat16), ref, "zero")
    with pytest.raises(AssertionError):
        assert_close_bf16(torch.full((64, 128), 1e-3, dtype=torch.bfloat16), ref, "not zero")
