"""Shared assertions for the test-suite."""

import torch


def bits(t: torch.Tensor) -> torch.Tensor:
    """Integer view of a tensor's raw bits on the CPU (for bit-exact comparisons)."""
    t = t.detach().cpu().contiguous()
    view = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()]
    return t.view(view)


def assert_bits_equal(actual: torch.Tensor, expected: torch.Tensor, what: str = "") -> None:
    a, e = bits(actual), bits(expected)
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    if not torch.equal(a, e):
        bad = (a != e).reshape(-1).nonzero().reshape(-1)
        i = int(bad[0])
        raise AssertionError(
            f"{what}: {bad.numel()} of {a.numel()} elements differ; first at flat index {i}: "
            f"got {actual.detach().cpu().reshape(-1)[i].item()!r}, "
            f"expected {expected.detach().cpu().reshape(-1)[i].item()!r}"
        )


def assert_bits_equal_up_to_nan_payload(actual: torch.Tensor, expected: torch.Tensor, what: str = "") -> None:
    """Bit equality wherever the expected value is a number; where it is a NaN the actual
    value must be a NaN too (which NaN an operation returns is not part of IEEE 754's
    required behaviour and differs between the host's and the GPU's arithmetic)."""
    a, e = actual.detach().cpu().reshape(-1), expected.detach().cpu().reshape(-1)
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    nan = torch.isnan(e.float())
    assert torch.equal(torch.isnan(a.float()), nan), f"{what}: NaNs are not where the checker has them"
    keep = ~nan
    assert_bits_equal(a[keep], e[keep], what)
