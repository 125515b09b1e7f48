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


# ---------------------------------------------------------------- sizes that are not powers of two


def _table(hadamard_blocks):
    """the golden blocks plus Sylvester's matrices where the reference's table holds them"""
    table = dict(hadamard_blocks)
    for k in (1, 2, 4, 8, 16, 64, 128, 256):
        table[k] = oh.deterministic_hadamard_matrix(k, torch.int8)
    return table


def test_golden_blocks_are_hadamard(hadamard_blocks):
    assert set(hadamard_blocks) == {12, 20, 28, 32, 144, 148, 160, 192, 200, 224, 240}
    for k, h in hadamard_blocks.items():
        hd = h.to(torch.int64)
        assert tuple(h.shape) == (k, k) and bool((hd.abs() == 1).all())
        assert torch.equal(hd @ hd.T, k * torch.eye(k, dtype=torch.int64)), k
    # 32 is the power of two whose entry is not Sylvester's matrix
    assert not torch.equal(hadamard_blocks[32], oh.deterministic_hadamard_matrix(32, torch.int8))


@pytest.mark.skipif(not REF_TABLE.exists(), reason="reference tree not present on this machine")
def test_golden_blocks_equal_the_reference_table(hadamard_blocks):
    from safetensors import safe_open

    with safe_open(str(REF_TABLE), framework="pt", device="cpu") as f:
        for k, h in hadamard_blocks.items():
            assert torch.equal(f.get_tensor(str(k)).to(torch.int8), h), k
        # every power of two but 32 is Sylvester's matrix there
        for k in (1, 2, 4, 8, 16, 64, 128, 256):
            assert torch.equal(f.get_tensor(str(k)).to(torch.int8),
                               oh.deterministic_hadamard_matrix(k, torch.int8)), k
        keys = sorted(int(k) for k in f.keys())
    # the sizes of the reference's own tests end in blocks the fixture holds
    for n, want in {768: 192, 1280: 160, 1600: 200, 3584: 224, 3840: 240, 7168: 224,
                    14336: 224, 18432: 144, 18944: 148}.items():
        pick = next(k for k in sorted(keys, reverse=True) if n % k == 0 and (n // k) & (n // k - 1) == 0)
        assert pick == want, n


@pytest.mark.parametrize("size", [768, 1280, 1600, 3584, 3840])
def test_butterfly_construction_is_orthogonal(size, hadamard_blocks):
    """the reference's own criterion (test_hadamard.py:44-52): H H^T / n == I"""
    gen = torch.Generator().manual_seed(size)
    r = oh.random_hadamard_matrix(size, dtype=torch.float32, gen=gen, table=_table(hadamard_blocks))
    assert set(r.unique().tolist()) == {-1.0, 1.0}
    assert torch.equal(r @ r.T, size * torch.eye(size, dtype=torch.float32))


@pytest.mark.parametrize("size", [24, 40, 56, 32, 96, 448, 768, 1600, 3584])
def test_closed_form_equals_butterflies(size, hadamard_blocks, hadamard_table_path):
    """product: diag(Q) (H_K^T (x) Sylvester(n / K)); oracle: the reference's butterfly
    stages followed by the block - and a brute-force entry formula for three of them"""
    from compressed_tensors_amd.transform import known_hadamard_block, random_hadamard_matrix

    table = _table(hadamard_blocks)
    g1, g2 = torch.Generator().manual_seed(size), torch.Generator().manual_seed(size)
    want = oh.random_hadamard_matrix(size, dtype=torch.float32, gen=g1, table=table)
    got = random_hadamard_matrix(size, torch.float32, gen=g2, table_path=hadamard_table_path)
    assert torch.equal(got, want)
    k, block = known_hadamard_block(size, hadamard_table_path)
    assert k == oh.known_block(size, torch.int8, table).shape[0]
    assert torch.equal(block, oh.known_block(size, torch.int8, table))
    if size <= 96:
        g3 = torch.Generator().manual_seed(size)
        q = torch.randint(0, 2, (size,), generator=g3, dtype=torch.float32) * 2 - 1
        m = size // k
        for i in range(size):
            for j in range(0, size, 7):
                # W[i, j] = Q[i] * H_K[j // m, i // m] * (-1)^popcount((i % m) & (j % m))
                s = -1.0 if bin((i % m) & (j % m)).count("1") & 1 else 1.0
                assert got[i, j] == q[i] * float(block[j // m, i // m]) * s


def test_table_loader_rejects_what_is_not_hadamard(tmp_path, hadamard_table_path):
    from safetensors.torch import save_file

    from compressed_tensors_amd.transform import known_hadamard_block, load_hadamard_table

    table = load_hadamard_table(hadamard_table_path)
    assert table[224].dtype == torch.int8 and 12 in table and 256 in table
    bad = table[12].clone()
    bad[0, 0] = -bad[0, 0]
    path = tmp_path / "bad.safetensors"
    save_file({"12": bad}, str(path))
    with pytest.raises(ValueError):
        load_hadamard_table(str(path))
    with pytest.raises(ValueError):
        known_hadamard_block(14336 + 4, hadamard_table_path)  # 3585 * 4: no entry fits
    assert known_hadamard_block(4096) == (256, None) and known_hadamard_block(16) == (16, None)


def test_power_of_two_entry_of_a_table_is_compared_with_sylvester(tmp_path):
    """a table whose entry for 4 is a Hadamard matrix other than Sylvester's is used as it
    is; one that holds Sylvester's matrix takes the matrix-free route (block None)"""
    from safetensors.torch import save_file

    from compressed_tensors_amd.transform import (
        deterministic_hadamard_matrix, known_hadamard_block, random_hadamard_matrix)

    syl = deterministic_hadamard_matrix(4, torch.int8)
    other = syl[[1, 0, 2, 3]].contiguous()
    other[2] = -other[2]
    plain, odd = tmp_path / "plain.safetensors", tmp_path / "odd.safetensors"
    save_file({"4": syl}, str(plain))
    save_file({"4": other}, str(odd))
    assert known_hadamard_block(16, str(plain)) == (4, None)
    k, block = known_hadamard_block(16, str(odd))
    assert k == 4 and torch.equal(block, other)
    g1, g2 = torch.Generator().manual_seed(5), torch.Generator().manual_seed(5)
    want = oh.random_hadamard_matrix(16, dtype=torch.float32, gen=g1, table={4: other})
    got = random_hadamard_matrix(16, torch.float32, gen=g2, table_path=str(odd))
    assert torch.equal(got, want)
    assert not torch.equal(got, random_hadamard_matrix(
        16, torch.float32, gen=torch.Generator().manual_seed(5), table_path=str(plain)))


def test_matrix_core_split_follows_the_largest_block_rule(ctmi, hadamard_table_path):
    """host logic only (the library's `supported` queries touch no GPU): for the sizes the
    reference builds from its table - the largest block that leaves a power of two,
    hadamard.py:102-129 - HadamardTransform finds a block x Sylvester split the one-product
    kernel takes, and folds a power of two above 128 into the block"""
    from compressed_tensors_amd import _lib
    from compressed_tensors_amd.transform import known_hadamard_block
    from compressed_tensors_amd.transform.hadamard import _matrix_core_split

    code = _lib.dtype_code(torch.bfloat16)
    # with the fixture's table (blocks 12, 20, 28, 144 ... 240 and the powers of two)
    for size, block, inner in ((768, 192, 4), (3072, 192, 16), (3584, 224, 16), (3840, 240, 16),
                               (5120, 160, 32), (7168, 224, 32), (14336, 224, 64), (15360, 240, 64)):
        k, _ = known_hadamard_block(size, hadamard_table_path)
        assert (k, size // k) == (block, inner)
        assert _matrix_core_split(ctmi, k, size // k, code) == (block, inner, True)
    assert _matrix_core_split(ctmi, 224, 128, code) == (224, 128, True)   # 28672
    assert _matrix_core_split(ctmi, 240, 128, code) is None               # 30720: no kernel
    assert _matrix_core_split(ctmi, 20, 256, code) == (40, 128, True)     # a caller's small block: folded
    assert _matrix_core_split(ctmi, 1, 16384, code) == (128, 128, True)   # Sylvester(16384)
    assert _matrix_core_split(ctmi, 1, 32768, code) is None
    assert _matrix_core_split(ctmi, 144, 256, code) is None               # 36864: the folded block has 288 rows
    assert _matrix_core_split(ctmi, 224, 64, _lib.dtype_code(torch.float32)) is None
