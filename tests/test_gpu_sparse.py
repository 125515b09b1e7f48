"""GPU parity: bitmask packing, sparse-bitmask and sparse-24-bitmask vs the oracle."""
import pytest
import torch

from gpu_util import announce, assert_bit_equal
from oracle import quant as oq
from oracle import sparse as osp

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (4, 8), (5, 17), (64, 4096), (2, 3, 20), (33, 4112),
                                   (14336, 4096)])
def test_pack_unpack_bitmasks(shape, gpu):
    from compressed_tensors_amd.utils import pack_bitmasks, unpack_bitmasks

    announce("bitmasks", shape)
    g = torch.Generator().manual_seed(sum(shape))
    mask = torch.rand(shape, generator=g) > 0.5
    packed = pack_bitmasks(mask.to(gpu))
    assert_bit_equal(packed, osp.pack_bitmasks(mask), "pack_bitmasks")
    assert_bit_equal(unpack_bitmasks(packed, list(shape)), mask, "unpack_bitmasks")


@pytest.mark.parametrize("shape", [(6, 40), (5, 17)], ids=["whole-words", "ragged"])
def test_pack_bitmasks_of_bytes_that_are_not_0_or_1(shape, gpu):
    """uint8 / int8 masks count as set wherever they are non-zero (numpy.packbits does the
    same): single high bits, single low bits, 0xff"""
    from compressed_tensors_amd.utils import pack_bitmasks

    announce("bitmasks of arbitrary bytes", shape)
    g = torch.Generator().manual_seed(3)
    picks = torch.tensor([0, 0, 0, 1, 2, 0x40, 0x80, 0xFF, 0x7F, 0x81], dtype=torch.uint8)
    mask = picks[torch.randint(0, len(picks), shape, generator=g)]
    want = osp.pack_bitmasks(mask != 0)
    assert_bit_equal(pack_bitmasks(mask.to(gpu)), want, "uint8")
    assert_bit_equal(pack_bitmasks(mask.view(torch.int8).to(gpu)), want, "int8")


def _sparse_tensor(shape, dtype, sparsity, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g) * 0.02
    x[torch.rand(shape, generator=g) < sparsity] = 0
    if dtype == FP8:
        x = (x * 1000).to(FP8)
    else:
        x = x.to(dtype)
    if x.numel() > 4:
        flat = x.view(torch.uint8 if dtype == FP8 else dtype).view(-1)
        if dtype == FP8:
            flat[1] = 0x80  # -0.0
            flat[2] = 0x7F  # NaN counts as non-zero
        else:
            flat[1] = -0.0
            flat[2] = float("nan")
    return x


BM = [
    ((2, 10), torch.float32, 0.5), ((16, 50), torch.bfloat16, 0.9), ((7, 64), torch.float16, 0.0),
    ((3, 9), torch.bfloat16, 1.0), ((33, 2050), torch.bfloat16, 0.5), ((64, 4096), torch.bfloat16, 0.5),
    ((9, 300), FP8, 0.6), ((5, 100), torch.int8, 0.7), ((300, 24), torch.bfloat16, 0.3),
    # rows of whole 16-column words: the one-wavefront-per-row scatter (several 1024-column
    # steps, a partial last one, row counts that do not fill a workgroup, dense and empty rows)
    ((33, 2064), torch.bfloat16, 0.5), ((6, 16384), FP8, 0.3), ((5, 1040), torch.float32, 0.8),
    ((10, 48), torch.bfloat16, 0.0), ((7, 1024), torch.float16, 1.0), ((3, 16400), torch.bfloat16, 0.5),
]


@pytest.mark.parametrize("shape,dtype,sparsity", BM, ids=[f"bm{i}" for i in range(len(BM))])
def test_bitmask_compress_decompress(shape, dtype, sparsity, gpu):
    from compressed_tensors_amd.compressors import (
        BaseCompressor, BitmaskTensor, bitmask_compress, bitmask_decompress,
    )

    announce("sparse-bitmask", shape, dtype, sparsity)
    if dtype == torch.int8:
        g = torch.Generator().manual_seed(3)
        x = torch.randint(-128, 128, shape, generator=g, dtype=torch.int8)
        x[torch.rand(shape, generator=g) < sparsity] = 0
    else:
        x = _sparse_tensor(shape, dtype, sparsity, seed=shape[1])
    values, bitmask, row_offsets = bitmask_compress(x.to(gpu))
    o_values, o_bitmask, o_offsets = osp.bitmask_compress(x)
    assert_bit_equal(values, o_values, "values")
    assert_bit_equal(bitmask, o_bitmask, "bitmask")
    assert_bit_equal(row_offsets, o_offsets, "row_offsets")
    dense = bitmask_decompress(o_values.to(gpu), o_bitmask.to(gpu), list(shape))
    assert_bit_equal(dense, osp.bitmask_decompress(o_values, o_bitmask, list(shape)), "decompress")
    comp = BaseCompressor.load_from_registry("sparse-bitmask")
    out = comp.compress_weight("layer", x.to(gpu))
    assert set(out) == {"layer.shape", "layer.compressed", "layer.bitmask", "layer.row_offsets"}
    assert out["layer.shape"].tolist() == list(shape) and out["layer.shape"].dtype == torch.int64
    back = comp.decompress_weight({k.split(".", 1)[1]: v for k, v in out.items()})
    want = osp.bitmask_decompress(o_values, o_bitmask, list(shape))
    assert_bit_equal(back, want, "compressor round trip")
    assert BitmaskTensor.from_dense(x.to(gpu)).curr_memory_size_bytes() == (
        o_values.numel() * o_values.element_size() + o_bitmask.numel() + 8 * shape[0])


def test_bitmask_empty_and_state_dict(gpu):
    from compressed_tensors_amd.compressors import BaseCompressor, bitmask_compress

    announce("sparse-bitmask edge")
    z = torch.zeros(4, 16, dtype=torch.bfloat16, device=gpu)
    values, bitmask, row_offsets = bitmask_compress(z)
    assert values.numel() == 0 and int(bitmask.sum()) == 0 and row_offsets.tolist() == [0, 0, 0, 0]
    comp = BaseCompressor.load_from_registry("sparse-bitmask")
    g = torch.Generator().manual_seed(8)
    w = torch.randn(8, 24, generator=g).bfloat16()
    w[w.abs() < 0.7] = 0
    state = {"a.weight": w.to(gpu), "a.bias": torch.ones(8, device=gpu), "b.weight": w.t().contiguous().to(gpu)}
    out = comp.compress(state, compression_targets={"a"})
    assert set(out) == {"a.shape", "a.compressed", "a.bitmask", "a.row_offsets", "a.bias", "b.weight"}
    restored = dict(comp.decompress(out))
    assert_bit_equal(restored["a.weight"], w, "state-dict round trip")
    assert "a.bias" in restored and "b.weight" in restored


def test_bitmask_compress_of_a_state_dict_waits_for_the_gpu_once(gpu, monkeypatch):
    """BitmaskCompressor.compress over several targets (bitmask_compress_many): the oracle's
    values, bitmasks and row offsets for every weight, the key order of the loop over
    compress_weight, other entries passed through, and one read-back of the counts for all"""
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.compressors import sparse_bitmask as sb

    announce("sparse-bitmask state dict")
    state, dense = {}, {}
    for i, (shape, dtype, sparsity) in enumerate(BM[:9] + [((4, 16), torch.bfloat16, 1.0)]):
        x = (_sparse_tensor(shape, dtype, sparsity, seed=50 + i) if dtype != torch.int8
             else (torch.arange(shape[0] * shape[1]).reshape(shape) % 3).to(torch.int8))
        dense[f"m{i}"] = x
        state[f"m{i}.weight"] = x.to(gpu)
        state[f"m{i}.bias"] = torch.full((shape[0],), float(i), device=gpu)
    state["emb.weight"] = torch.ones(3, 5, device=gpu)  # not a target
    state["norm.weight"] = torch.ones(7, device=gpu)    # 1-D and not a target either
    targets = set(dense)
    calls = []
    real = sb.bitmask_compress_many
    monkeypatch.setattr(sb, "bitmask_compress_many", lambda ts: calls.append(len(ts)) or real(ts))
    comp = BaseCompressor.load_from_registry("sparse-bitmask")
    out = comp.compress(state, compression_targets=targets)
    assert calls == [len(dense)]
    want_keys = []
    for name in state:
        prefix = name[: -len(".weight")]
        if name.endswith(".weight") and prefix in targets:
            want_keys += [f"{prefix}.{p}" for p in ("shape", "compressed", "bitmask", "row_offsets")]
        else:
            want_keys.append(name)
    assert list(out) == want_keys
    for name, x in dense.items():
        o_values, o_bitmask, o_offsets = osp.bitmask_compress(x)
        assert_bit_equal(out[f"{name}.compressed"], o_values, f"{name} values")
        assert_bit_equal(out[f"{name}.bitmask"], o_bitmask, f"{name} bitmask")
        assert_bit_equal(out[f"{name}.row_offsets"], o_offsets, f"{name} row_offsets")
        assert out[f"{name}.shape"].tolist() == list(x.shape)
    assert out["emb.weight"] is state["emb.weight"]
    back = dict(comp.decompress(out))
    for name, x in dense.items():
        o_values, o_bitmask, _ = osp.bitmask_compress(x)  # (-0.0 is dropped: comes back as 0.0)
        assert_bit_equal(back[f"{name}.weight"], osp.bitmask_decompress(o_values, o_bitmask, list(x.shape)),
                         f"{name} round trip")


def _prune24(x):
    keep = osp.get_24_bytemasks(x)
    return torch.where(keep, x, torch.zeros_like(x))


S24 = [((8, 16), torch.bfloat16), ((64, 4096), torch.bfloat16), ((33, 40), torch.float16),
       ((16, 64), torch.float32), ((32, 256), FP8), ((12, 32), torch.int8), ((6, 10), torch.bfloat16),
       ((3, 12), torch.bfloat16)]


@pytest.mark.parametrize("shape,dtype", S24, ids=[f"s24-{i}" for i in range(len(S24))])
def test_sparse24(shape, dtype, gpu):
    from compressed_tensors_amd.compressors import (
        BaseCompressor, get_24_bytemasks, sparse24_bitmask_compress, sparse24_bitmask_decompress,
    )

    announce("sparse-24", shape, dtype)
    g = torch.Generator().manual_seed(shape[0] * 7 + shape[1])
    if dtype == FP8:
        base = (torch.randn(shape, generator=g) * 0.02).bfloat16()
        base = _prune24(base)
        scale = (base.float().abs().amax(-1, keepdim=True) / 448).bfloat16()
        args = oq._Args(num_bits=8, type="float", strategy="channel")
        x = oq.quantize(base, scale, None, args, dtype=FP8)  # many groups with < 2 non-zeros, -0.0 codes
    elif dtype == torch.int8:
        x = torch.randint(-128, 128, shape, generator=g, dtype=torch.int8)
        x[torch.rand(shape, generator=g) < 0.5] = 0
    else:
        x = (torch.randn(shape, generator=g) * 0.02).to(dtype)
        x[torch.rand(shape, generator=g) < 0.4] = 0  # ties between zeros
        x.view(-1)[0] = float("nan")
    mask = get_24_bytemasks(x.to(gpu))
    assert_bit_equal(mask, osp.get_24_bytemasks(x), "24 mask")
    if (shape[1] % 2) == 0:
        values, bitmask = sparse24_bitmask_compress(x.to(gpu))
        o_values, o_bitmask = osp.sparse24_bitmask_compress(x)
        assert_bit_equal(values, o_values, "24 values")
        assert_bit_equal(bitmask, o_bitmask, "24 bitmask")
        dense = sparse24_bitmask_decompress(values, bitmask, torch.Size(shape))
        assert_bit_equal(dense, osp.sparse24_bitmask_decompress(o_values, o_bitmask, shape), "24 decompress")
        comp = BaseCompressor.load_from_registry("sparse-24-bitmask")
        out = comp.compress_weight("l.weight", x.to(gpu))
        assert set(out) == {"l.shape", "l.compressed", "l.bitmask"}
        assert tuple(out["l.shape"].shape) == (2, 1)
        back = comp.decompress_weight({k.split(".", 1)[1]: v for k, v in out.items()})
        assert_bit_equal(back, osp.sparse24_bitmask_decompress(o_values, o_bitmask, shape), "24 round trip")


def test_sparse24_errors(gpu):
    from compressed_tensors_amd.compressors import get_24_bytemasks, sparse24_bitmask_compress

    with pytest.raises(ValueError, match="multiple of 4"):
        get_24_bytemasks(torch.zeros(3, 5, dtype=torch.bfloat16, device=gpu))
    with pytest.raises(AssertionError, match="2D"):
        sparse24_bitmask_compress(torch.zeros(2, 2, 4, dtype=torch.bfloat16, device=gpu))
    with pytest.raises(AssertionError, match="2:4"):
        sparse24_bitmask_compress(torch.zeros(4, 8, dtype=torch.bfloat16, device=gpu), "unstructured")


def test_large_bitmask_roundtrip_properties(gpu):
    """full-size (8192 x 8192, 50 % magnitude pruned): sampled parity and a lossless round trip"""
    from compressed_tensors_amd.compressors import bitmask_compress, bitmask_decompress

    announce("large bitmask")
    g = torch.Generator().manual_seed(0)
    w = (torch.randn(8192, 8192, generator=g) * 0.02).bfloat16()
    thr = w.float().abs().flatten().kthvalue(w.numel() // 2).values
    w[w.float().abs() <= thr] = 0
    wg = w.to(gpu)
    values, bitmask, row_offsets = bitmask_compress(wg)
    nnz_rows = (w != 0).sum(-1)
    assert_bit_equal(row_offsets, torch.cumsum(nnz_rows, 0) - nnz_rows, "row offsets")
    assert values.numel() == int(nnz_rows.sum())
    rows = [0, 1, 4097, 8191]
    for r in rows:
        lo = int(row_offsets[r])
        assert_bit_equal(values[lo: lo + int(nnz_rows[r])], w[r][w[r] != 0], f"values row {r}")
    assert_bit_equal(bitmask[:64], osp.pack_bitmasks(w[:64] != 0), "bitmask head")
    assert torch.equal(bitmask_decompress(values, bitmask, list(w.shape)), wg)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e4m3fn, torch.float32])
def test_sparse24_decompress_of_a_bitmask_that_is_not_2_4(dtype, gpu):
    """sparse24_bitmask_decompress is `out[mask] = values` for ANY mask
    (sparse_24_bitmask.py:206-224).  Half of the elements kept, but not 2 per group
    of 4: the streaming 2:4 kernel must notice and the general path take over."""
    from compressed_tensors_amd.compressors import sparse24_bitmask_decompress
    from compressed_tensors_amd.utils.helpers import pack_bitmasks

    announce("sparse24 decompress, malformed mask", dtype)
    g = torch.Generator().manual_seed(7)
    rows, cols = 48, 256
    x = torch.randn(rows, cols, generator=g).clamp(-3, 3)
    x[x == 0] = 1.0
    mask = torch.zeros(rows, cols, dtype=torch.bool)
    mask[:, : cols // 2] = True              # 4 kept in the first groups, none in the last
    mask[5] = torch.arange(cols) % 2 == 0    # one well-formed row in between
    mask[6, :8] = torch.tensor([1, 1, 1, 0, 1, 0, 0, 0], dtype=torch.bool)  # 3 + 1: right total, wrong groups
    mask[6, 8:] = torch.arange(cols - 8) % 2 == 0
    x = torch.where(mask, x, torch.zeros_like(x)).to(dtype)
    raw = x.view(torch.int8) if dtype == torch.float8_e4m3fn else x
    values = raw[mask].reshape(rows, cols // 2)
    if dtype == torch.float8_e4m3fn:
        values = values.view(torch.float8_e4m3fn)
    bitmask = pack_bitmasks(mask.to(gpu))
    dense = sparse24_bitmask_decompress(values.to(gpu), bitmask, torch.Size((rows, cols)))
    assert_bit_equal(dense, x, "general path behind the 2:4 kernel")


def test_random_shapes_sweep(gpu):
    """60 random shapes (row lengths around the 8 / 16 / 1024 / 16384 column boundaries of
    the kernels, 1 to 70 rows, four dtypes, sparsities from 0 to 1): both sparse formats
    against the oracle"""
    from compressed_tensors_amd.compressors import (
        bitmask_compress, bitmask_decompress, get_24_bytemasks, sparse24_bitmask_compress,
        sparse24_bitmask_decompress,
    )

    g = torch.Generator().manual_seed(2024)
    edges = [8, 16, 64, 1024, 2048, 4096, 16384]
    dtypes = [torch.bfloat16, torch.float16, torch.float32, FP8]
    for case in range(60):
        rows = int(torch.randint(1, 71, (1,), generator=g))
        edge = edges[int(torch.randint(0, len(edges), (1,), generator=g))]
        cols = max(1, edge + int(torch.randint(-17, 18, (1,), generator=g)))
        dtype = dtypes[case % 4]
        sparsity = float(torch.rand(1, generator=g)) if case % 7 else float(case % 2)
        announce("sparse sweep", case, (rows, cols), dtype, round(sparsity, 2))
        x = _sparse_tensor((rows, cols), dtype, sparsity, seed=case)
        values, bitmask, offsets = bitmask_compress(x.to(gpu))
        o_values, o_bitmask, o_offsets = osp.bitmask_compress(x)
        assert_bit_equal(values, o_values, f"values {case}")
        assert_bit_equal(bitmask, o_bitmask, f"bitmask {case}")
        assert_bit_equal(offsets, o_offsets, f"offsets {case}")
        assert_bit_equal(bitmask_decompress(values, bitmask, [rows, cols]),
                         osp.bitmask_decompress(o_values, o_bitmask, [rows, cols]), f"decompress {case}")
        cols4 = max(4, cols // 4 * 4)
        y = _sparse_tensor((rows, cols4), dtype, min(sparsity, 0.6), seed=1000 + case)
        assert_bit_equal(get_24_bytemasks(y.to(gpu)), osp.get_24_bytemasks(y), f"24 mask {case}")
        v24, b24 = sparse24_bitmask_compress(y.to(gpu))
        o_v24, o_b24 = osp.sparse24_bitmask_compress(y)
        assert_bit_equal(v24, o_v24, f"24 values {case}")
        assert_bit_equal(b24, o_b24, f"24 bitmask {case}")
        assert_bit_equal(sparse24_bitmask_decompress(v24, b24, torch.Size((rows, cols4))),
                         osp.sparse24_bitmask_decompress(o_v24, o_b24, (rows, cols4)), f"24 decompress {case}")


def test_bitmask_decompress_with_few_values(gpu):
    """set bits beyond the values that exist read as zero, also across tiles of the scatter"""
    from compressed_tensors_amd.compressors import bitmask_decompress

    announce("bitmask decompress, short values")
    x = _sparse_tensor((64, 4096), torch.bfloat16, 0.5, seed=5)
    o_values, o_bitmask, _ = osp.bitmask_compress(x)
    for keep in (o_values.numel() - 1, o_values.numel() // 3, 9, 0):
        short = o_values[:keep]
        padded = torch.cat([short, torch.zeros(o_values.numel() - keep, dtype=o_values.dtype)])
        want = osp.bitmask_decompress(padded, o_bitmask, [64, 4096])
        assert_bit_equal(bitmask_decompress(short.to(gpu), o_bitmask.to(gpu), [64, 4096]), want, f"keep {keep}")


def test_bitmask_many_tiles(gpu):
    """tensors of several hundred scatter tiles (8192 elements each, whatever the row
    length), all element sizes, sparsities from empty to full, a ragged last tile"""
    from compressed_tensors_amd.compressors import bitmask_compress, bitmask_decompress

    cases = [((1024, 4096), torch.bfloat16, 0.5), ((4096, 512), torch.float16, 0.9), ((3, 1048576), torch.bfloat16, 0.1),
             ((2048, 1032), FP8, 0.5), ((512, 2056), torch.float32, 0.7), ((70000, 8), torch.bfloat16, 0.5),
             ((512, 4096), torch.bfloat16, 1.0), ((512, 4096), torch.bfloat16, 0.0), ((1001, 24), torch.bfloat16, 0.4)]
    for shape, dtype, sparsity in cases:
        announce("bitmask, many tiles", shape, dtype, sparsity)
        x = _sparse_tensor(shape, dtype, sparsity, seed=shape[1] + 1)
        o_values, o_bitmask, o_offsets = osp.bitmask_compress(x)
        values, bitmask, offsets = bitmask_compress(x.to(gpu))
        assert_bit_equal(values, o_values, "values")
        assert_bit_equal(bitmask, o_bitmask, "bitmask")
        assert_bit_equal(offsets, o_offsets, "offsets")
        assert_bit_equal(bitmask_decompress(values, bitmask, list(shape)),
                         osp.bitmask_decompress(o_values, o_bitmask, list(shape)), "decompress")


@pytest.mark.parametrize("dtype,shape", [(torch.bfloat16, (8192, 4096)), (FP8, (4096, 8192)),
                                         (torch.float32, (2048, 4096)), (torch.bfloat16, (2048, 4096))],
                         ids=["bf16", "fp8", "f32", "bf16-one-tile-per-workgroup"])
def test_bitmask_decompress_runs_of_tiles(dtype, shape, gpu):
    """tensors of more scatter tiles than workgroups fit the device at once: a workgroup then
    walks a run of neighbouring tiles and takes every tile's place from the one before.
    Row blocks that are empty, full, half and nearly empty; all values, and fewer values
    than set bits (the rest reads as zero).  Expected tensors are built with torch."""
    from compressed_tensors_amd.compressors import bitmask_compress, bitmask_decompress

    announce("bitmask decompress, runs of tiles", dtype, shape)
    rows, cols = shape
    g = torch.Generator(device=gpu).manual_seed(11)
    x = torch.randint(1, 120, (rows, cols), generator=g, device=gpu).to(torch.float32)
    keep_prob = torch.tensor([0.0, 1.0, 0.5, 0.1, 0.97, 0.5, 0.0, 0.5], device=gpu)
    block = keep_prob[(torch.arange(rows, device=gpu) * 8 // rows)].unsqueeze(1)
    x = torch.where(torch.rand((rows, cols), generator=g, device=gpu) < block, x, torch.zeros_like(x))
    x = x.to(dtype)
    values, bitmask, _ = bitmask_compress(x)
    nz = (x.float() != 0).flatten()
    assert values.numel() == int(nz.sum())
    assert_bit_equal(bitmask_decompress(values, bitmask, list(shape)), x, "all values")
    rank = torch.cumsum(nz.to(torch.int64), 0) - 1
    for keep in (values.numel() - 3, values.numel() // 2 + 5, 4097):
        want = torch.where((nz & (rank < keep)).view(shape), x.float(), torch.zeros((), device=gpu)).to(dtype)
        got = bitmask_decompress(values[:keep].clone(), bitmask, list(shape))
        assert_bit_equal(got, want, f"first {keep} values")


def test_bitmask_decompress_on_two_streams_at_once(gpu):
    """decompressions in flight on two streams at the same time (each launch of the count
    pass takes its own ticket counter inside the library): the results of the calls made one
    after the other"""
    from compressed_tensors_amd.compressors import bitmask_compress, bitmask_decompress

    announce("bitmask decompress, two streams")
    tensors = [_sparse_tensor((2048, 4096), torch.bfloat16, sp, seed=60 + i).to(gpu)
               for i, sp in enumerate((0.5, 0.8, 0.2, 0.5))]
    packed = [bitmask_compress(x) for x in tensors]
    alone = [bitmask_decompress(values, bitmask, [2048, 4096]) for values, bitmask, _ in packed]
    for x, back in zip(tensors, alone):
        assert torch.equal(torch.nan_to_num(back.float()), torch.nan_to_num(x.float()))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=gpu), torch.cuda.Stream(device=gpu)]
    results = []
    for rep in range(6):
        for i, (values, bitmask, _) in enumerate(packed):
            with torch.cuda.stream(streams[(rep + i) % 2]):
                results.append((i, bitmask_decompress(values, bitmask, [2048, 4096])))
    torch.cuda.synchronize()
    for i, got in results:
        assert_bit_equal(got, alone[i], f"tensor {i}")


def test_bitmask_decompress_of_a_very_large_tensor(gpu):
    """more tiles than the grouped count handles (> 65536 tiles of 8192 elements): the scatter
    then takes its positions from a scan over all tiles.  Round trip on the GPU, values and
    offsets spot-checked against torch."""
    from compressed_tensors_amd.compressors import bitmask_compress, bitmask_decompress

    announce("bitmask, 537M elements")
    rows, cols = 65600, 8192
    g = torch.Generator(device=gpu).manual_seed(1)
    x = torch.randint(-128, 128, (rows, cols), generator=g, dtype=torch.int8, device=gpu)
    x[torch.rand((rows, cols), generator=g, device=gpu) < 0.5] = 0
    values, bitmask, offsets = bitmask_compress(x)
    nnz_rows = (x != 0).sum(-1)
    assert values.numel() == int(nnz_rows.sum())
    assert torch.equal(offsets, torch.cumsum(nnz_rows, 0) - nnz_rows)
    for r in (0, 1, 40000, rows - 1):
        lo = int(offsets[r])
        assert torch.equal(values[lo: lo + int(nnz_rows[r])], x[r][x[r] != 0])
    back = bitmask_decompress(values, bitmask, [rows, cols])
    assert torch.equal(back, x)


@pytest.mark.parametrize("dtype", [torch.bfloat16, FP8])
@pytest.mark.parametrize("shard_dim,shard_sizes", [(0, [256, 128, 128]), (1, [64, 64, 128]), (1, [128, 128])])
def test_sparse24_shards_recombine(dtype, shard_dim, shard_sizes, gpu):
    """compressed values and bitmask cut into shards along either dimension decompress
    shard by shard into the pieces of the dense tensor
    (reference: tests/test_compressors/sparse_compressors/test_sparse_24_bitmask.py:99-145)"""
    from compressed_tensors_amd.compressors import Sparse24BitMaskTensor
    from compressed_tensors_amd.utils import combine_shards, shard_tensor

    announce("sparse24 shards", dtype, shard_dim, shard_sizes)
    m, k = (512, 256)
    x = _prune24(_sparse_tensor((m, k), torch.bfloat16, 0.0, seed=3).float()).to(torch.bfloat16)
    if dtype == FP8:
        x = (x.float() * 50).to(FP8)
    t = Sparse24BitMaskTensor.from_dense(x.to(gpu))
    v_sizes = [s // 2 for s in shard_sizes] if shard_dim == 1 else shard_sizes
    b_sizes = [s // 8 for s in shard_sizes] if shard_dim == 1 else shard_sizes
    pieces = []
    for values, bitmask in zip(shard_tensor(t.compressed, v_sizes, dim=shard_dim),
                               shard_tensor(t.bitmask, b_sizes, dim=shard_dim)):
        shape = (bitmask.shape[0], bitmask.shape[1] * 8)
        pieces.append(Sparse24BitMaskTensor(shape=shape, compressed=values.contiguous(),
                                            bitmask=bitmask.contiguous()).decompress())
    want = osp.sparse24_bitmask_decompress(*osp.sparse24_bitmask_compress(x), (m, k))
    assert_bit_equal(combine_shards(pieces, dim=shard_dim), want, "recombined")


def test_sparse24_repair_over_many_rows(gpu):
    """a bitmask that is not 2:4 in a tensor of thousands of rows: the kernel behind the
    streaming pass redoes every row, each workgroup counting the set bits before its rows"""
    from compressed_tensors_amd.compressors import sparse24_bitmask_decompress
    from compressed_tensors_amd.utils.helpers import pack_bitmasks

    announce("sparse24 repair, 3000 rows")
    rows, cols = 3000, 512
    g = torch.Generator().manual_seed(12)
    x = torch.randn(rows, cols, generator=g).bfloat16()
    x[x == 0] = 1.0
    # half of the elements kept, row by row, at random places: right total, wrong groups
    keep = torch.zeros(rows, cols, dtype=torch.bool)
    order = torch.rand(rows, cols, generator=g).argsort(dim=1)[:, : cols // 2]
    keep.scatter_(1, order, True)
    x = torch.where(keep, x, torch.zeros_like(x))
    values = x[keep].reshape(rows, cols // 2)
    dense = sparse24_bitmask_decompress(values.to(gpu), pack_bitmasks(keep.to(gpu)), torch.Size((rows, cols)))
    assert_bit_equal(dense, x, "repaired")


QS24 = [
    (dict(num_bits=8, type="float", symmetric=True, strategy="channel"), (64, 512), torch.bfloat16),
    (dict(num_bits=8, type="float", symmetric=True, strategy="channel"), (33, 4112), torch.float16),
    (dict(num_bits=8, type="float", symmetric=True, strategy="tensor"), (16, 64), torch.bfloat16),
    (dict(num_bits=8, type="float", symmetric=True, strategy="channel"), (19, 24), torch.bfloat16),
    (dict(num_bits=8, type="float", symmetric=True, strategy="group", group_size=128), (24, 1024), torch.bfloat16),
    (dict(num_bits=8, type="int", symmetric=True, strategy="channel"), (40, 256), torch.bfloat16),
    (dict(num_bits=8, type="int", symmetric=False, strategy="channel"), (40, 256), torch.float32),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=32), (8, 128), torch.bfloat16),
    (dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[16, 64]), (48, 256), torch.bfloat16),
    (dict(num_bits=8, type="int", symmetric=False, strategy="tensor"), (24, 64), torch.float16),
]


@pytest.mark.parametrize("spec,shape,dtype", QS24, ids=[f"qs24-{i}" for i in range(len(QS24))])
def test_quantization_and_2_4_compression_in_one_pass(spec, shape, dtype, gpu):
    """codes + 2:4 compression of the codes from one kernel == the oracle's quantize followed
    by its sparse24_bitmask_compress, with and without the zero point the observer leaves
    (it decides whether a value that quantizes to -0 keeps its sign bit)"""
    from compressed_tensors_amd.compressors import quantize_sparse24_compress
    from compressed_tensors_amd.quantization import QuantizationArgs

    announce("quantize + 2:4", spec, shape, dtype)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    g = torch.Generator().manual_seed(shape[1])
    w = torch.randn(shape, generator=g) * 0.02
    w[torch.rand(shape, generator=g) < 0.002] *= 30
    w = _prune24(w).to(dtype)
    w.view(-1)[0:4] = torch.tensor([-1e-7, 0.0, 3e-3, 0.0]).to(dtype)   # a code of -0 among the survivors
    scale, zp = oq.observe_weight(w, oargs)
    for zero_point in ((zp,) if not spec["symmetric"] else (zp, None)):
        codes = oq.quantize(w, scale, zero_point, oargs, dtype=args.pytorch_dtype())
        want_values, want_bitmask = osp.sparse24_bitmask_compress(codes)
        got = quantize_sparse24_compress(w.to(gpu), scale.to(gpu), args,
                                         zero_point=None if zero_point is None else zero_point.to(gpu))
        assert got is not None, "expected a fused kernel for this layout"
        assert_bit_equal(got[0], want_values, "values")
        assert_bit_equal(got[1], want_bitmask, "bitmask")


def test_quantization_and_2_4_without_a_fused_kernel(gpu):
    """rows that are not whole 8-element items, an act-order g_idx: None, and the caller takes
    the two steps"""
    from compressed_tensors_amd.compressors import quantize_sparse24_compress
    from compressed_tensors_amd.quantization import QuantizationArgs

    announce("quantize + 2:4, unsupported")
    args = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="channel")
    w = torch.randn(8, 12).bfloat16().to(gpu)
    scale = torch.full((8, 1), 0.01, dtype=torch.bfloat16, device=gpu)
    assert quantize_sparse24_compress(w, scale, args) is None
    w = torch.randn(8, 32).bfloat16().to(gpu)
    assert quantize_sparse24_compress(w, scale, args, g_idx=torch.zeros(32, dtype=torch.int32, device=gpu)) is None
    assert quantize_sparse24_compress(w, scale, args) is not None


@pytest.mark.parametrize("spec,shape,dtype", QS24, ids=[f"s24dq-{i}" for i in range(len(QS24))])
def test_2_4_decompression_and_dequantization_in_one_pass(spec, shape, dtype, gpu):
    """2:4 values + bitmask of a quantized weight -> the dense dequantized weight from one
    kernel == the oracle's sparse24_bitmask_decompress followed by its dequantize (arguments
    inferred from the scale's shape, as the naive compressor's decompress_weight calls it),
    and == this library's own two steps"""
    from compressed_tensors_amd.compressors import (
        sparse24_bitmask_decompress, sparse24_decompress_dequantize,
    )
    from compressed_tensors_amd.quantization import dequantize

    announce("2:4 decompress + dequantize", spec, shape, dtype)
    oargs = oq._Args(**spec)
    code_dtype = torch.float8_e4m3fn if spec["type"] == "float" else torch.int8
    g = torch.Generator().manual_seed(shape[1] + 1)
    w = torch.randn(shape, generator=g) * 0.02
    w[torch.rand(shape, generator=g) < 0.002] *= 30
    w = _prune24(w).to(dtype)
    scale, zp = oq.observe_weight(w, oargs)
    for zero_point in ((zp,) if not spec["symmetric"] else (zp, None)):
        codes = oq.quantize(w, scale, zero_point, oargs, dtype=code_dtype)
        values, bitmask = osp.sparse24_bitmask_compress(codes)
        want = oq.dequantize(osp.sparse24_bitmask_decompress(values, bitmask, shape), scale, zero_point)
        zp_gpu = None if zero_point is None else zero_point.to(gpu)
        got = sparse24_decompress_dequantize(values.to(gpu), bitmask.to(gpu), shape, scale.to(gpu), zp_gpu)
        assert got is not None, "expected a fused kernel for this layout"
        assert got.dtype == dtype and tuple(got.shape) == tuple(shape)
        assert_bit_equal(got, want, "dequantized weight")
        two_steps = dequantize(sparse24_bitmask_decompress(values.to(gpu), bitmask.to(gpu), shape),
                               scale.to(gpu), zp_gpu)
        assert_bit_equal(got, two_steps, "one pass against two steps")


@pytest.mark.parametrize("rows,cols", [(48, 256), (3000, 64)], ids=["48x256", "3000x64"])
def test_2_4_decompression_and_dequantization_of_a_bitmask_that_is_not_2_4(rows, cols, gpu):
    """half of the positions set, but not two in every four: the kernel behind the streaming
    one redoes the tensor as a general scatter, dequantizing as it places the codes"""
    from compressed_tensors_amd.compressors import sparse24_decompress_dequantize

    announce("2:4 decompress + dequantize, bitmask not 2:4", rows, cols)
    g = torch.Generator().manual_seed(rows)
    mask = torch.zeros(rows * cols, dtype=torch.bool)
    mask[torch.randperm(rows * cols, generator=g)[: rows * cols // 2]] = True
    mask = mask.view(rows, cols)
    values = torch.randint(-127, 128, (rows, cols // 2), generator=g, dtype=torch.int8)
    bitmask = osp.pack_bitmasks(mask)
    scale = (torch.rand(rows, 1, generator=g) * 0.01 + 0.001).bfloat16()
    zp = torch.randint(-5, 6, (rows, 1), generator=g, dtype=torch.int8)
    for code_dtype in (torch.int8, torch.float8_e4m3fn):
        vals = values.view(code_dtype)
        zero_point = zp if code_dtype == torch.int8 else None
        if code_dtype == torch.float8_e4m3fn:  # no NaN codes: their payload bits are not part of the contract
            vals = torch.where((values & 0x7F) == 0x7F, torch.zeros_like(values), values).view(code_dtype)
        want = oq.dequantize(osp.bitmask_decompress(vals.flatten(), bitmask, (rows, cols)), scale, zero_point)
        got = sparse24_decompress_dequantize(vals.to(gpu), bitmask.to(gpu), (rows, cols), scale.to(gpu),
                                             None if zero_point is None else zero_point.to(gpu))
        assert got is not None
        assert_bit_equal(got, want, f"dequantized weight ({code_dtype})")


def test_2_4_decompression_and_dequantization_without_a_fused_kernel(gpu):
    """rows that are not whole 8-element items, scales in another dtype than asked for, codes
    that are not 8-bit: None, and the caller takes the two steps"""
    from compressed_tensors_amd.compressors import sparse24_decompress_dequantize

    announce("2:4 decompress + dequantize, unsupported")
    scale = torch.full((8, 1), 0.01, dtype=torch.bfloat16, device=gpu)
    values = torch.zeros(8, 6, dtype=torch.int8, device=gpu)
    bitmask = torch.zeros(8, 2, dtype=torch.uint8, device=gpu)
    assert sparse24_decompress_dequantize(values, bitmask, (8, 12), scale) is None
    values = torch.zeros(8, 16, dtype=torch.int8, device=gpu)
    bitmask = torch.full((8, 4), 0x33, dtype=torch.uint8, device=gpu)
    assert sparse24_decompress_dequantize(values.to(torch.int16), bitmask, (8, 32), scale) is None
    assert sparse24_decompress_dequantize(values, bitmask, (8, 32), scale.double()) is None
    assert sparse24_decompress_dequantize(
        values, bitmask, (8, 32), scale, g_idx=torch.zeros(32, dtype=torch.int32, device=gpu)) is None
    out = sparse24_decompress_dequantize(values, bitmask, (8, 32), scale)
    assert out is not None and out.dtype == torch.bfloat16 and not out.any()


def test_stacked_round_trip_at_full_size(gpu):
    """a 14336 x 4096 bf16 weight (the largest of a Llama-3-8B-shaped model): one-pass
    quantization + 2:4 compression, then one-pass decompression + dequantization, gives what
    quantize -> dequantize gives on the dense weight (the 2:4 zeros quantize to code 0), and
    compressing that result again reproduces values and bitmask (idempotence)"""
    from compressed_tensors_amd.compressors import (
        get_24_bytemasks, quantize_sparse24_compress, sparse24_decompress_dequantize,
    )
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, dequantize, observe_weight_qparams, quantize,
    )

    announce("quantize + 2:4 round trip, 14336 x 4096")
    args = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="channel")
    g = torch.Generator(device=gpu).manual_seed(7)
    w = torch.randn(14336, 4096, generator=g, device=gpu) * 0.02
    # no survivor small enough to quantize to zero: which zero of a group topk then keeps is
    # torch's tie order, and not what this test is about
    w = torch.where(w.abs() < 1e-3, torch.full_like(w, 1e-3), w).bfloat16()
    w = torch.where(get_24_bytemasks(w), w, torch.zeros_like(w))
    scale, _ = observe_weight_qparams(w, args)
    values, bitmask = quantize_sparse24_compress(w, scale, args)
    assert int((values.view(torch.uint8) & 0x7F == 0).sum()) == 0
    assert values.shape == (14336, 2048) and bitmask.shape == (14336, 512)
    back = sparse24_decompress_dequantize(values, bitmask, w.shape, scale)
    want = dequantize(quantize(w, scale, None, args, dtype=torch.float8_e4m3fn), scale)
    assert_bit_equal(back, want, "round trip")
    again = quantize_sparse24_compress(back, scale, args)
    assert_bit_equal(again[1], bitmask, "bitmask of the round trip")
    assert_bit_equal(again[0], values, "values of the round trip")


def test_stacked_2_4_of_fp8_at_full_size_against_the_oracle(gpu):
    """the same 14336 x 4096 weight against the oracle's op chain - quantize (fp8, one scale per
    output channel), then sparse24_bitmask_compress of the codes (sparse_24_bitmask.py:162-224 on
    what quantized_compressors/base.py:91-125 produced) and the way back - on row slices at the
    head, in the middle and at the tail: the one-pass kernels, and the two steps one after the
    other"""
    from compressed_tensors_amd.compressors import (
        get_24_bytemasks, quantize_sparse24_compress, sparse24_bitmask_compress,
        sparse24_bitmask_decompress, sparse24_decompress_dequantize,
    )
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams, quantize

    announce("quantize + 2:4 vs oracle, 14336 x 4096")
    spec = dict(num_bits=8, type="float", symmetric=True, strategy="channel")
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    g = torch.Generator(device=gpu).manual_seed(11)
    w = torch.randn(14336, 4096, generator=g, device=gpu) * 0.02
    # every survivor large enough to keep a non-zero code: which of several zero codes of a
    # group topk keeps is torch's tie order on the CPU, and not what this test is about
    w = torch.where(w.abs() < 1e-3, torch.full_like(w, 1e-3), w).bfloat16()
    w = torch.where(get_24_bytemasks(w), w, torch.zeros_like(w))
    scale, _ = observe_weight_qparams(w, args)
    fused_values, fused_bitmask = quantize_sparse24_compress(w, scale, args)
    codes = quantize(w, scale, None, args, dtype=torch.float8_e4m3fn)
    values, bitmask = sparse24_bitmask_compress(codes)
    dense = sparse24_bitmask_decompress(values, bitmask, codes.shape)
    back = sparse24_decompress_dequantize(fused_values, fused_bitmask, w.shape, scale)
    rows = w.shape[0]
    for sl in (slice(0, 48), slice(rows // 2 - 7, rows // 2 + 41), slice(rows - 48, rows)):
        wc = w[sl].cpu()
        o_scale, _ = oq.observe_weight(wc, oargs)
        assert_bit_equal(scale[sl], o_scale, f"scales {sl}")
        o_codes = oq.quantize(wc, o_scale, None, oargs, dtype=torch.float8_e4m3fn)
        o_values, o_bitmask = osp.sparse24_bitmask_compress(o_codes)
        assert_bit_equal(codes[sl], o_codes, f"codes {sl}")
        assert_bit_equal(values[sl], o_values, f"values, two steps {sl}")
        assert_bit_equal(bitmask[sl], o_bitmask, f"bitmask, two steps {sl}")
        assert_bit_equal(fused_values[sl], o_values, f"values, one pass {sl}")
        assert_bit_equal(fused_bitmask[sl], o_bitmask, f"bitmask, one pass {sl}")
        o_dense = osp.sparse24_bitmask_decompress(o_values, o_bitmask, o_codes.shape)
        assert_bit_equal(dense[sl], o_dense, f"decompressed codes {sl}")
        assert_bit_equal(back[sl], oq.dequantize(o_dense, o_scale), f"decompressed + dequantized {sl}")


# ---------------------------------------------------------------- several 2:4 tensors per call


def _prune24(x):
    """zero the two smallest magnitudes of every group of 4 (ties do not matter here)"""
    g = x.float().abs().reshape(-1, 4)
    keep = torch.zeros_like(g, dtype=torch.bool)
    keep.scatter_(1, g.topk(2, dim=1).indices, True)
    return torch.where(keep.reshape(x.shape), x, torch.zeros_like(x))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float8_e4m3fn, torch.float32, torch.float16])
def test_sparse24_many_tensors_in_one_call(dtype, gpu):
    """sparse24_bitmask_compress_many / _decompress_many == the single-tensor calls, bit for
    bit, and the oracle: more tensors than one launch takes (8), sizes that differ, a shape
    the chained kernels do not take (it gets a call of its own), and among the tensors to
    decompress one whose bitmask is not 2:4 (the last workgroup of the launch redoes it)"""
    from compressed_tensors_amd.compressors import (
        sparse24_bitmask_compress, sparse24_bitmask_compress_many, sparse24_bitmask_decompress,
        sparse24_bitmask_decompress_many,
    )
    from compressed_tensors_amd.utils.helpers import pack_bitmasks

    announce("sparse24 many", dtype)
    g = torch.Generator().manual_seed(31)
    shapes = [(64, 512), (37, 256), (16, 128), (5, 1024), (128, 256), (1, 64), (48, 384), (3, 12), (96, 640),
              (7, 256), (300, 4096)]
    xs = [torch.randn(s, generator=g).clamp(-3, 3).to(dtype) for s in shapes]
    got = sparse24_bitmask_compress_many([x.to(gpu) for x in xs])
    assert len(got) == len(xs)
    for i, (x, (values, bitmask)) in enumerate(zip(xs, got)):
        want_v, want_b = sparse24_bitmask_compress(x.to(gpu))
        assert_bit_equal(values, want_v, f"values {i}")
        assert_bit_equal(bitmask, want_b, f"bitmask {i}")
        o_v, o_b = osp.sparse24_bitmask_compress(x)
        assert_bit_equal(values, o_v, f"values {i} vs oracle")
        assert_bit_equal(bitmask, o_b, f"bitmask {i} vs oracle")
    items = [(v, b, list(s)) for (v, b), s in zip(got, shapes)]
    # a tensor whose bitmask keeps half of the elements but not 2 per group
    rows, cols = 40, 256
    keep = torch.zeros(rows, cols, dtype=torch.bool)
    keep.scatter_(1, torch.rand(rows, cols, generator=g).argsort(dim=1)[:, : cols // 2], True)
    odd = torch.randn(rows, cols, generator=g).clamp(-3, 3)
    odd[odd == 0] = 1.0
    odd = torch.where(keep, odd, torch.zeros_like(odd)).to(dtype)
    raw = odd.view(torch.int8) if dtype == torch.float8_e4m3fn else odd
    odd_values = raw[keep].reshape(rows, cols // 2)
    if dtype == torch.float8_e4m3fn:
        odd_values = odd_values.view(torch.float8_e4m3fn)
    items.insert(4, (odd_values.to(gpu), pack_bitmasks(keep.to(gpu)), [rows, cols]))
    dense = sparse24_bitmask_decompress_many(items)
    assert len(dense) == len(items)
    for i, ((v, b, s), d) in enumerate(zip(items, dense)):
        assert_bit_equal(d, sparse24_bitmask_decompress(v, b, torch.Size(s)), f"dense {i}")
    assert_bit_equal(dense[4], odd, "tensor with a bitmask that is not 2:4")
    for i, x in enumerate(xs):
        k = i if i < 4 else i + 1
        assert_bit_equal(dense[k], osp.sparse24_bitmask_decompress(*osp.sparse24_bitmask_compress(x), shapes[i]),
                         f"dense {k} vs oracle")
    # the calls after a repair find the launch counters back at zero: once more, all 2:4
    again = sparse24_bitmask_decompress_many([it for k, it in enumerate(items) if k != 4])
    for i, d in enumerate(again):
        assert_bit_equal(d, dense[i if i < 4 else i + 1], f"second call {i}")


def test_sparse24_compressor_state_dict_in_few_calls(gpu):
    """Sparse24BitMaskCompressor.compress / decompress on a state dict (one multi-tensor
    call per dtype) against the oracle tensor by tensor"""
    from compressed_tensors_amd.compressors import BaseCompressor

    announce("sparse24 state dict")
    g = torch.Generator().manual_seed(2)
    state = {f"layers.{i}.proj.weight": _prune24(torch.randn(64 + 32 * i, 256, generator=g)).bfloat16().to(gpu)
             for i in range(10)}
    state["layers.0.proj.bias"] = torch.randn(64, generator=g).to(gpu)
    state["norm.weight"] = torch.randn(256, 4, generator=g).to(gpu)  # rows of half a bitmask byte
    comp = BaseCompressor.load_from_registry("sparse-24-bitmask")
    packed = comp.compress(state, compression_targets={n[: -len(".weight")] for n in state if n.endswith("weight")})
    for name, w in state.items():
        if not name.endswith(".weight"):
            assert packed[name] is w
            continue
        prefix = name[: -len(".weight")]
        o_v, o_b = osp.sparse24_bitmask_compress(w.cpu())
        assert_bit_equal(packed[prefix + ".compressed"], o_v, name)
        assert_bit_equal(packed[prefix + ".bitmask"], o_b, name)
        assert packed[prefix + ".shape"].flatten().tolist() == list(w.shape)
    back = dict(comp.decompress(packed))
    assert set(back) == set(state)
    for name, w in state.items():
        want = w if not name.endswith(".weight") else osp.sparse24_bitmask_decompress(
            *osp.sparse24_bitmask_compress(w.cpu()), tuple(w.shape))
        assert_bit_equal(back[name], want, name)


def test_sparse24_decompress_many_launches_back_to_back(gpu):
    """more launches than the library holds verdict words for (256 pairs, one per stream),
    enqueued without a wait in between, on one stream and spread over three: every result
    against the oracle.  Every 50th tensor has a bitmask that is not 2:4, so the repair path
    runs in between and has to leave its words at zero for the launches behind it."""
    from compressed_tensors_amd.compressors import sparse24_bitmask_compress, sparse24_bitmask_decompress
    from compressed_tensors_amd.utils.helpers import pack_bitmasks

    announce("sparse24 decompress x 600")
    g = torch.Generator().manual_seed(77)
    rows, cols = 64, 512
    cases = []
    for k in range(12):
        x = _prune24(torch.randn(rows, cols, generator=g)).bfloat16()
        v, b = osp.sparse24_bitmask_compress(x)
        cases.append((v.to(gpu), b.to(gpu), osp.sparse24_bitmask_decompress(v, b, (rows, cols))))
    keep = torch.zeros(rows, cols, dtype=torch.bool)
    keep.scatter_(1, torch.rand(rows, cols, generator=g).argsort(dim=1)[:, : cols // 2], True)
    odd = torch.randn(rows, cols, generator=g).bfloat16()
    odd[odd == 0] = 1.0
    odd = torch.where(keep, odd, torch.zeros_like(odd))
    malformed = (odd[keep].reshape(rows, cols // 2).to(gpu), pack_bitmasks(keep.to(gpu)), odd)
    streams = [torch.cuda.current_stream(gpu)] + [torch.cuda.Stream(gpu) for _ in range(2)]
    torch.cuda.synchronize()
    for which in ([0] * 600, [i % 3 for i in range(600)]):
        outs = []
        for i, s in enumerate(which):
            v, b, want = malformed if i % 50 == 49 else cases[i % len(cases)]
            with torch.cuda.stream(streams[s]):
                outs.append((sparse24_bitmask_decompress(v, b, torch.Size((rows, cols))), want))
        torch.cuda.synchronize()
        for i, (got, want) in enumerate(outs):
            assert_bit_equal(got, want, f"launch {i} of {len(which)} on {len(set(which))} stream(s)")


def test_stacked_kernels_for_many_weights_in_one_call(gpu):
    """ctmi_quantize_sparse24_compress_many / ctmi_sparse24_decompress_dequantize_many (8 weights
    per launch) against the single-weight entry points: 19 weights of mixed shapes, dtypes,
    strategies (channel, group, tensor), code kinds (fp8, int8) and zero points; one of them with
    a bitmask that is not 2:4 on the way back (the repair pass names it alone)"""
    from compressed_tensors_amd.compressors.sparse_24_bitmask import (
        quantize_sparse24_compress, quantize_sparse24_compress_many,
        sparse24_decompress_dequantize, sparse24_decompress_dequantize_many,
    )
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams

    announce("stacked kernels, many weights")
    g = torch.Generator().manual_seed(31)
    specs = [
        dict(num_bits=8, type="float", symmetric=True, strategy="channel"),
        dict(num_bits=8, type="int", symmetric=True, strategy="group", group_size=64),
        dict(num_bits=8, type="int", symmetric=False, strategy="channel"),
        dict(num_bits=8, type="float", symmetric=True, strategy="tensor"),
    ]
    shapes = [(64, 256), (96, 512), (8, 64), (200, 1024), (33, 128)]
    recs, single = [], []
    for k in range(19):
        args = QuantizationArgs(**specs[k % len(specs)])
        dtype = (torch.bfloat16, torch.float16, torch.float32)[k % 3]
        w = (torch.randn(shapes[k % len(shapes)], generator=g) * 0.05).to(dtype).to(gpu)
        scale, zp = observe_weight_qparams(w, args)
        recs.append((w, scale, zp, args))
        single.append(quantize_sparse24_compress(w, scale, args, zero_point=zp))
    many = quantize_sparse24_compress_many(recs)
    assert all(m is not None for m in many)
    for k, ((values, bitmask), (want_values, want_bitmask)) in enumerate(zip(many, single)):
        assert values.dtype == want_values.dtype
        assert_bit_equal(values, want_values.cpu(), f"weight {k} values")
        assert_bit_equal(bitmask, want_bitmask.cpu(), f"weight {k} bitmask")
    # the way back; weight 11 gets a bitmask with a group of three and one of one
    back = []
    for k, ((w, scale, zp, args), (values, bitmask)) in enumerate(zip(recs, many)):
        zp_back = None if args.symmetric else zp
        if k == 11:
            bitmask = bitmask.clone()
            bitmask[0, 0] = 0b00010111
        back.append((values, bitmask, tuple(w.shape), scale, zp_back))
    want = [sparse24_decompress_dequantize(v, b, shape, s, zero_point=z) for v, b, shape, s, z in back]
    got = sparse24_decompress_dequantize_many(back)
    for k, (a, b) in enumerate(zip(got, want)):
        assert a is not None and a.dtype == b.dtype and a.shape == b.shape
        assert_bit_equal(a, b.cpu(), f"weight {k} restored")
    # what the many-weight helpers do not take comes back as None (the caller goes one by one)
    assert quantize_sparse24_compress_many([(recs[0][0].cpu(), recs[0][1], None, recs[0][3])]) == [None]
    assert sparse24_decompress_dequantize_many([(many[0][0].cpu(), many[0][1], (64, 256), recs[0][1], None)]) == [None]
