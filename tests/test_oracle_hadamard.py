"""Pin the Hadamard part of the oracle and the product's host-side matrix
construction (no GPU)."""
import json
from pathlib import Path

import pytest
import torch

from oracle import hadamard as oh

GOLDEN = Path(__file__).parent / "golden"
REF_TABLE = Path("/root/reference/src/compressed_tensors/transform/utils/hadamards.safetensors")


def test_seed42_known_answer():
    gold = json.loads((GOLDEN / "hadamard_seed42.json").read_text())
    gen = torch.Generator().manual_seed(gold["seed"])
    one = oh.random_hadamard_matrix(gold["size"], gen=gen)
    two = oh.random_hadamard_matrix(gold["size"], gen=gen)
    assert torch.equal(one[:3, :3].sign().int(), torch.tensor(gold["first_draw_top_left_signs"]).int())
    assert torch.equal(two[:3, :3].sign().int(), torch.tensor(gold["second_draw_top_left_signs"]).int())


@pytest.mark.parametrize("size", [64, 128, 256, 1024, 2048])
def test_orthogonality_and_structure(size):
    gen = torch.Generator().manual_seed(size)
    r = oh.random_hadamard_matrix(size, dtype=torch.float64, gen=gen)
    assert torch.equal(r @ r.T, size * torch.eye(size, dtype=torch.float64))
    assert set(r.unique().tolist()) == {-1.0, 1.0}
    # the butterfly recursion over a Sylvester block gives diag(Q) * Sylvester(size)
    gen = torch.Generator().manual_seed(size)
    q = torch.randint(0, 2, (size,), generator=gen, dtype=torch.float64) * 2 - 1
    assert torch.equal(r, q.unsqueeze(1) * oh.deterministic_hadamard_matrix(size, torch.float64))
    h = oh.deterministic_hadamard_matrix(size, torch.float64)
    assert torch.equal(h @ h.T, size * torch.eye(size, dtype=torch.float64))


def test_sylvester_is_textbook_fwht():
    """H x computed by the textbook in-place fast Walsh-Hadamard butterflies"""
    n = 256
    x = torch.randn(n, dtype=torch.float64)
    y = x.clone()
    h = 1
    while h < n:
        y = y.view(-1, 2, h)
        y = torch.stack((y[:, 0] + y[:, 1], y[:, 0] - y[:, 1]), dim=1).reshape(-1)
        h *= 2
    assert torch.allclose(oh.deterministic_hadamard_matrix(n, torch.float64) @ x, y, atol=1e-9)


@pytest.mark.skipif(not REF_TABLE.exists(), reason="reference tree not present on this machine")
def test_known_blocks_are_sylvester_in_the_reference_table():
    from safetensors import safe_open

    with safe_open(str(REF_TABLE), framework="pt", device="cpu") as f:
        keys = sorted(int(k) for k in f.keys())
        assert {64, 128, 256} <= set(keys)
        for k in (64, 128, 256):
            stored = f.get_tensor(str(k)).to(torch.float64)
            assert torch.equal(stored, oh.deterministic_hadamard_matrix(k, torch.float64)), k
        # and the table lookup picks exactly those for powers of two >= 64
        for n in (64, 128, 256, 512, 1024, 4096, 8192):
            pick = next(k for k in sorted(keys, reverse=True)
                        if n % k == 0 and (n // k) & (n // k - 1) == 0)
            assert pick in (64, 128, 256) and pick == oh.known_block(n, torch.float64).size(0)


def test_transform_algebra():
    """output_tfm(input_tfm(x) @ (U W V)^T) == x W^T  (reference: test_correctness.py:29-57)"""
    torch.manual_seed(0)
    n_in, n_out = 128, 64
    w = torch.randn(n_out, n_in, dtype=torch.float64)
    x = torch.randn(5, n_in, dtype=torch.float64)
    gen = torch.Generator().manual_seed(1)
    v = oh.random_hadamard_matrix(n_in, dtype=torch.float64, gen=gen)
    u = oh.random_hadamard_matrix(n_out, dtype=torch.float64, gen=gen)
    x_t = oh.hadamard_forward(v, x, "input")
    w_t = oh.hadamard_forward(v, w, "weight_input", inverse=True)
    w_t = oh.hadamard_forward(u, w_t, "weight_output")
    y_t = x_t @ w_t.T
    y = oh.hadamard_forward(u, y_t, "output", inverse=True)
    assert torch.allclose(y, x @ w.T, atol=1e-9)


def test_product_host_construction_matches_oracle():
    from compressed_tensors_amd.transform import (
        deterministic_hadamard_matrix, hadamard_factors, random_hadamard_matrix,
    )

    for n in (1, 2, 8, 64, 256):
        assert torch.equal(deterministic_hadamard_matrix(n, torch.float32),
                           oh.deterministic_hadamard_matrix(n, torch.float32))
    for n in (64, 2048):
        g1, g2 = torch.Generator().manual_seed(7), torch.Generator().manual_seed(7)
        assert torch.equal(random_hadamard_matrix(n, torch.float32, gen=g1),
                           oh.random_hadamard_matrix(n, torch.float32, gen=g2))
    with pytest.raises(ValueError):
        deterministic_hadamard_matrix(12)
    for n, (a, b) in {128: (1, 128), 4096: (64, 64), 8192: (64, 128)}.items():
        assert hadamard_factors(n) == (a, b)
        ha = oh.deterministic_hadamard_matrix(a, torch.float32)
        hb = oh.deterministic_hadamard_matrix(b, torch.float32)
        if n <= 4096:
            assert torch.equal(torch.kron(ha, hb), oh.deterministic_hadamard_matrix(n, torch.float32))
