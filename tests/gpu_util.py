"""helpers shared by the GPU parity tests"""
import sys

import torch


def announce(*what):
    """name the case before it runs, flushed, so a fault can be attributed"""
    print("[case]", *what, flush=True)
    sys.stdout.flush()


def bits(t: torch.Tensor) -> torch.Tensor:
    """raw bit pattern of a tensor as integers, for bit-exact comparison (NaN-safe, sign-of-zero-safe)"""
    t = t.detach().cpu().contiguous()
    size = t.element_size()
    view = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[size]
    if t.dtype == torch.bool:
        return t.to(torch.uint8)
    return t.view(view)


def assert_bit_equal(got: torch.Tensor, want: torch.Tensor, what=""):
    assert got.dtype == want.dtype, f"{what}: dtype {got.dtype} != {want.dtype}"
    assert tuple(got.shape) == tuple(want.shape), f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    g, w = bits(got), bits(want)
    if not torch.equal(g, w):
        bad = (g != w).nonzero()
        first = tuple(bad[0].tolist())
        raise AssertionError(
            f"{what}: {bad.shape[0]} of {g.numel()} elements differ; first at {first}: "
            f"got {got.detach().cpu()[first]!r} want {want[first]!r}"
        )
