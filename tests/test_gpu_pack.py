"""GPU parity: int32 packing, fp4 nibble packing and the quantization
compressors (pack-quantized, naive/int/float-quantized, nvfp4-pack-quantized)
vs the oracle, bit-exact."""
import json
from pathlib import Path

import pytest
import torch

from gpu_util import announce, assert_bit_equal
from oracle import pack as op
from oracle import quant as oq

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).parent / "golden"


def _pair(d):
    from compressed_tensors_amd.quantization import QuantizationArgs

    return QuantizationArgs(**d), oq._Args(**d)


def test_pack_known_answers_on_gpu(gpu):
    from compressed_tensors_amd.compressors import pack_to_int32, unpack_from_int32

    for case in json.loads((GOLDEN / "pack_int32.json").read_text())["cases"]:
        announce("pack golden", case["num_bits"], case["values"])
        values = torch.tensor(case["values"], dtype=torch.int8)
        packed = torch.tensor(case["packed"], dtype=torch.int32)
        assert_bit_equal(pack_to_int32(values.to(gpu), case["num_bits"]), packed, "pack")
        assert_bit_equal(unpack_from_int32(packed.to(gpu), case["num_bits"], values.shape), values, "unpack")


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 7, 8])
@pytest.mark.parametrize("shape", [(1, 1), (5, 37), (16, 64), (3, 1024), (130, 48)])
def test_pack_unpack_random(bits, shape, gpu):
    from compressed_tensors_amd.compressors import pack_to_int32, unpack_from_int32

    announce("pack random", bits, shape)
    g = torch.Generator().manual_seed(bits * 1000 + shape[0])
    v = torch.randint(-(1 << (bits - 1)), 1 << (bits - 1), shape, generator=g, dtype=torch.int8)
    for dim in (1, 0):
        p = pack_to_int32(v.to(gpu), bits, packed_dim=dim)
        want = op.pack_to_int32(v, bits, packed_dim=dim).contiguous()
        assert_bit_equal(p, want, f"pack dim{dim}")
        u = unpack_from_int32(p, bits, v.shape, packed_dim=dim)
        assert_bit_equal(u, v, f"unpack dim{dim}")
    # out-of-range int8 input: the reference adds the shifted terms, carries and all
    wild = torch.randint(-128, 128, shape, generator=g, dtype=torch.int8)
    assert_bit_equal(pack_to_int32(wild.to(gpu), bits), op.pack_to_int32(wild, bits), "wild pack")


def test_pack_errors(gpu):
    from compressed_tensors_amd.compressors import pack_to_int32, unpack_from_int32

    with pytest.raises(ValueError, match="int8"):
        pack_to_int32(torch.zeros(2, 2, dtype=torch.int32, device=gpu), 4)
    with pytest.raises(ValueError, match="less than 8"):
        pack_to_int32(torch.zeros(2, 2, dtype=torch.int8, device=gpu), 9)
    with pytest.raises(ValueError, match="at least 1"):
        pack_to_int32(torch.zeros(2, 2, dtype=torch.int8, device=gpu), 0)
    with pytest.raises(ValueError, match="Expected"):
        unpack_from_int32(torch.zeros(2, 2, dtype=torch.int8, device=gpu), 4, (2, 2))
    e = pack_to_int32(torch.zeros(0, 8, dtype=torch.int8, device=gpu), 4)
    assert e.shape == (0, 1) and e.dtype == torch.int32


PQ = [
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128), (128, 1024), torch.bfloat16),
    (dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=128), (128, 512), torch.bfloat16),
    (dict(num_bits=4, type="int", symmetric=True, strategy="channel"), (64, 520), torch.bfloat16),
    (dict(num_bits=4, type="int", symmetric=False, strategy="channel"), (19, 256), torch.float16),
    (dict(num_bits=8, type="int", symmetric=True, strategy="group", group_size=64), (32, 256), torch.float32),
    (dict(num_bits=8, type="int", symmetric=False, strategy="tensor"), (32, 256), torch.bfloat16),
    (dict(num_bits=4, type="int", symmetric=True, strategy="tensor"), (7, 36), torch.bfloat16),  # ragged: generic kernel
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=12), (10, 36), torch.bfloat16),
    (dict(num_bits=3, type="int", symmetric=True, strategy="channel"), (10, 40), torch.bfloat16),
    (dict(num_bits=4, type="int", symmetric=True, strategy="block", block_structure=[4, 16]), (16, 64), torch.bfloat16),
]


@pytest.mark.parametrize("spec,shape,dtype", PQ, ids=[f"pq{i}-{c[0]['strategy']}" for i, c in enumerate(PQ)])
def test_pack_quantized_compressor(spec, shape, dtype, gpu):
    from compressed_tensors_amd.compressors import BaseCompressor

    announce("pack-quantized", spec, shape, dtype)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(31)
    w = (torch.randn(shape, generator=g) * 0.02).to(dtype)
    w.view(-1)[0] = -0.0
    scale, zp = oq.observe_weight(w, oargs)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    want = op.pack_quantized_compress(w, scale, oargs, zero_point=zp)
    for zero_point in ((zp,) if not spec["symmetric"] else (zp, None)):
        got = comp.compress_weight(
            weight=w.to(gpu), scale=scale.to(gpu), quantization_args=args,
            zero_point=None if zero_point is None else zero_point.to(gpu))
        assert set(got) == set(want)
        assert_bit_equal(got["weight_packed"], want["weight_packed"], "weight_packed")
        assert_bit_equal(got["weight_shape"], want["weight_shape"], "weight_shape")
        if "weight_zero_point" in want:
            assert_bit_equal(got["weight_zero_point"], want["weight_zero_point"], "packed zp")
    data = dict(want, weight_scale=scale)
    if not spec["symmetric"] and spec["strategy"] not in ("group", "channel"):
        data["weight_zero_point"] = zp  # such zero points stay in the state dict unpacked
    dense_want = op.pack_quantized_decompress(dict(data), oargs)
    dense = comp.decompress_weight({k: v.to(gpu) for k, v in data.items()}, quantization_args=args)
    assert_bit_equal(dense, dense_want, "decompress")
    # the reference's own property: compress -> decompress == fake_quantize
    # (by value: fake_quantize keeps the sign of a negative value rounded to zero, int8 cannot)
    assert torch.equal(dense.cpu(), oq.fake_quantize(w, scale, zp, oargs).to(scale.dtype))


ONE_SHOT = [
    # (args, shape, dtype, fused kernel expected)
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128), (128, 1024), torch.bfloat16, True),
    (dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=128), (77, 512), torch.bfloat16, True),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=32), (33, 96), torch.float16, True),
    (dict(num_bits=8, type="int", symmetric=False, strategy="group", group_size=64), (32, 256), torch.float32, True),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=24), (16, 48), torch.bfloat16, False),
    (dict(num_bits=8, type="int", symmetric=True, strategy="group", group_size=512), (9, 2048), torch.float16, True),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=8), (700, 1504), torch.bfloat16, True),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128), (40, 256), torch.float32, True),
    (dict(num_bits=4, type="int", symmetric=True, strategy="channel"), (64, 520), torch.bfloat16, True),
    (dict(num_bits=4, type="int", symmetric=False, strategy="channel"), (19, 4096), torch.float16, True),
    (dict(num_bits=8, type="int", symmetric=True, strategy="channel"), (5, 14336), torch.bfloat16, True),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=12), (10, 36), torch.bfloat16, False),
    (dict(num_bits=4, type="int", symmetric=True, strategy="tensor"), (16, 64), torch.bfloat16, False),
    (dict(num_bits=3, type="int", symmetric=True, strategy="channel"), (10, 40), torch.bfloat16, False),
]


@pytest.mark.parametrize("spec,shape,dtype,fused", ONE_SHOT,
                         ids=[f"os{i}-{c[0]['strategy']}" for i, c in enumerate(ONE_SHOT)])
def test_observe_and_compress_in_one_pass(spec, shape, dtype, fused, gpu):
    """observer + calculate_qparams + quantize + pack from one kernel: the oracle's
    observe_weight followed by its pack_quantized_compress, bit for bit"""
    from compressed_tensors_amd import _lib
    from compressed_tensors_amd.compressors import BaseCompressor

    announce("one-shot pack-quantized", spec, shape, dtype)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(32)
    w = (torch.randn(shape, generator=g) * 0.02).to(dtype)
    w[0, :8] = 0.0
    w[0, 1] = -0.0
    w[-1] = 0.0                     # a row of zeros: the scale floor
    w[1] = w[1].abs()               # one-sided rows: min / max are clamped to include 0
    w[2] = -w[2].abs()
    w[3, 5] = float("nan")
    w[4, 0] = float("inf")
    rows, cols = shape
    blk = {"group": spec.get("group_size", 0), "channel": cols}.get(spec["strategy"], 0)
    assert bool(blk and _lib.load().ctmi_observe_pack_quantized_supported(
        _lib.dtype_code(dtype), rows, cols, blk, spec["num_bits"])) == fused
    comp = BaseCompressor.load_from_registry("pack-quantized")
    table = bool(blk and _lib.load().ctmi_observe_pack_quantized_gidx_supported(
        _lib.dtype_code(dtype), rows, cols, blk, spec["num_bits"]))
    assert comp.one_pass_kernel(w.to(gpu), args) == ("groups" if fused else "table" if table else None)
    scale, zp = oq.observe_weight(w, oargs)
    want = op.pack_quantized_compress(w, scale, oargs, zero_point=zp)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    got = comp.observe_and_compress_weight(w.to(gpu), args)
    assert set(got) == set(want) | {"weight_scale"}
    # a NaN in a cell makes its scale NaN; the codes of such a cell are an int cast of NaN,
    # which is not defined: compare the others
    bad_cells = torch.isnan(scale.float())
    if spec["strategy"] == "tensor":
        ok = torch.full(shape, not bool(bad_cells.any()))
    else:
        ok = ~bad_cells.repeat_interleave(cols // scale.shape[-1], dim=-1)
    nan = torch.full_like(scale, float("nan"))
    assert_bit_equal(torch.where(bad_cells.to(gpu), nan.to(gpu), got["weight_scale"]),
                     torch.where(bad_cells, nan, scale), "scale")
    from oracle.pack import unpack_from_int32 as o_unpack
    got_codes = o_unpack(got["weight_packed"].cpu(), spec["num_bits"], torch.Size(shape))
    want_codes = o_unpack(want["weight_packed"], spec["num_bits"], torch.Size(shape))
    assert torch.equal(got_codes[ok], want_codes[ok]), "codes"
    assert_bit_equal(got["weight_shape"], want["weight_shape"], "weight_shape")
    if "weight_zero_point" in want:
        n_cells = scale.shape[-1]
        gz = o_unpack(got["weight_zero_point"].cpu(), spec["num_bits"], torch.Size((rows, n_cells)), packed_dim=0)
        wz = o_unpack(want["weight_zero_point"], spec["num_bits"], torch.Size((rows, n_cells)), packed_dim=0)
        assert torch.equal(gz[~bad_cells], wz[~bad_cells]), "zero points"


def test_observed_weight_batch_matches_single_calls(gpu):
    """a state dict's worth of weights through one ctmi_observe_pack_quantized_many call
    (mixed schemes and dtypes, more weights of one kind than a launch takes) gives what
    the per-weight calls give"""
    from compressed_tensors_amd.compressors import BaseCompressor, ObservedWeightBatch
    from compressed_tensors_amd.quantization import QuantizationArgs

    announce("observed weight batch")
    g = torch.Generator().manual_seed(8)
    sym = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    asym = QuantizationArgs(num_bits=4, type="int", symmetric=False, strategy="group", group_size=64)
    chan = QuantizationArgs(num_bits=8, type="int", symmetric=True, strategy="channel")
    entries = []
    for i in range(11):
        entries.append(dict(weight=(torch.randn(24 + 8 * i, 1024, generator=g) * 0.02).bfloat16(),
                            quantization_args=sym))
    entries.insert(3, dict(weight=(torch.randn(40, 512, generator=g) * 0.02).half(), quantization_args=asym))
    entries.insert(7, dict(weight=(torch.randn(9, 2056, generator=g) * 0.02).bfloat16(), quantization_args=chan))
    entries.append(dict(weight=(torch.randn(1100, 128, generator=g) * 0.02).bfloat16(), quantization_args=sym))
    for e in entries:
        e["weight"] = e["weight"].to(gpu)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    batch = ObservedWeightBatch(entries)
    for _ in range(2):  # buffers are reused
        got = batch.compress()
    for e, d in zip(entries, got):
        want = comp.observe_and_compress_weight(e["weight"], e["quantization_args"])
        assert set(d) == set(want)
        for k in want:
            assert_bit_equal(d[k], want[k], k)


def test_observed_weight_batch_takes_every_strategy(gpu, monkeypatch):
    """weights that do not share the batch's launches go through it as well: a group size
    that is not a power of two and activation ordering in one pass of their own (the group of
    a column looked up), one scale per tensor and blocks with the observer and the compressor
    one after the other.  Against the oracle's observer (on the columns sorted by g_idx where
    there is one, forward.py:286-303) and compressor."""
    from compressed_tensors_amd.compressors import BaseCompressor, ObservedWeightBatch
    from compressed_tensors_amd.quantization import QuantizationArgs, helpers

    observed = []
    real = helpers.observe_weight_qparams
    monkeypatch.setattr(helpers, "observe_weight_qparams",
                        lambda w, a, *k, **kw: (observed.append(a.strategy), real(w, a, *k, **kw))[1])

    announce("observed weight batch, every strategy")
    g = torch.Generator().manual_seed(18)
    specs = [dict(num_bits=4, type="int", symmetric=True, strategy="tensor"),
             dict(num_bits=4, type="int", symmetric=False, strategy="block", block_structure=[16, 64]),
             dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=24),
             dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128),
             dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=32)]
    shapes = [(32, 128), (48, 192), (16, 48), (64, 512), (24, 256)]
    ws = [(torch.randn(s, generator=g) * 0.02).bfloat16() for s in shapes]
    g_idx = [None, None, None, None, torch.randperm(256, generator=g).to(torch.int32) // 32]
    entries = [dict(weight=w.to(gpu), quantization_args=QuantizationArgs(**spec),
                    **({} if gi is None else {"g_idx": gi.to(gpu)}))
               for w, spec, gi in zip(ws, specs, g_idx)]
    got = ObservedWeightBatch(entries).compress()
    # the separate observer ran for the tensor and the block scheme only
    assert sorted(observed) == ["block", "tensor"]
    comp = BaseCompressor.load_from_registry("pack-quantized")
    assert [comp.one_pass_kernel(e["weight"], e["quantization_args"], e.get("g_idx")) for e in entries] == [
        None, None, "table", "groups", "table"]
    for i, (w, spec, gi, d) in enumerate(zip(ws, specs, g_idx, got)):
        oargs = oq._Args(**spec)
        seen = w if gi is None else w.index_select(1, torch.argsort(gi.long()))
        scale, zp = oq.observe_weight(seen, oargs)
        want = op.pack_quantized_compress(w, scale, oargs, zero_point=zp, g_idx=gi)
        assert_bit_equal(d["weight_scale"], scale, f"scale {i}")
        for k in want:
            assert_bit_equal(d[k], want[k], f"{k} {i}")


ACT_ORDER = [
    # (rows, cols, group_size, dtype, symmetric, num_bits): items per lane 1, 2, 4, 8; rows that do
    # not fill the last block of a workgroup; more row blocks than workgroups
    (37, 1024, 128, torch.bfloat16, True, 4),
    (300, 4096, 128, torch.bfloat16, True, 4),
    (21, 4096, 128, torch.bfloat16, False, 4),
    (19, 8192, 64, torch.float16, True, 8),
    (4100, 512, 32, torch.bfloat16, True, 4),
    (9, 14336, 128, torch.bfloat16, True, 4),
    (5, 14336, 128, torch.float32, False, 8),
    (16, 1536, 24, torch.bfloat16, True, 4),   # no g_idx: groups of 24 by division
]


@pytest.mark.parametrize("rows,cols,group,dtype,symmetric,bits", ACT_ORDER,
                         ids=[f"ao{i}-{c[1]}" for i, c in enumerate(ACT_ORDER)])
def test_one_pass_with_activation_ordering(rows, cols, group, dtype, symmetric, bits, gpu):
    """ctmi_observe_pack_quantized_gidx: min-max observer on the columns as g_idx sorts them,
    calculate_qparams, quantize with g_idx and pack, from one kernel; against the oracle's
    observer on the sorted columns followed by its compressor with g_idx"""
    from compressed_tensors_amd.compressors import BaseCompressor

    announce("one-shot pack-quantized with g_idx", rows, cols, group, dtype, symmetric, bits)
    spec = dict(num_bits=bits, type="int", symmetric=symmetric, strategy="group", group_size=group)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(rows + cols)
    w = (torch.randn(rows, cols, generator=g) * 0.02).to(dtype)
    w[0, :9] = 0.0
    w[-1] = 0.0
    if rows > 4:
        w[1] = w[1].abs()
        w[2] = -w[2].abs()
        w[3, 7] = float("inf")
    gi = None if group == 24 else (torch.randperm(cols, generator=g) // group).to(torch.int32)
    seen = w if gi is None else w.index_select(1, torch.argsort(gi.long(), stable=True))
    scale, zp = oq.observe_weight(seen, oargs)
    want = op.pack_quantized_compress(w, scale, oargs, zero_point=zp, g_idx=gi)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    wg, gg = w.to(gpu), None if gi is None else gi.to(gpu)
    assert comp.one_pass_kernel(wg, args, gg) == "table"
    got = comp.observe_and_compress_weight(wg, args, g_idx=gg)
    assert set(got) == set(want) | {"weight_scale"}
    assert_bit_equal(got["weight_scale"], scale, "scale")
    for k in want:
        assert_bit_equal(got[k], want[k], k)


def test_pack_quantized_state_dict_and_g_idx(gpu):
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.quantization import QuantizationScheme

    announce("pack-quantized state dict")
    spec = dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=32)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(33)
    w = (torch.randn(16, 128, generator=g) * 0.02).bfloat16()
    g_idx = (torch.randperm(128, generator=g) // 32).to(torch.int32)
    scale, zp = oq.observe_weight(w.index_select(-1, torch.argsort(g_idx)), oargs)
    state = {
        "m.weight": w, "m.weight_scale": scale, "m.weight_zero_point": zp, "m.weight_g_idx": g_idx,
        "m.bias": torch.ones(16), "other.weight": torch.ones(4, 4),
    }
    scheme = QuantizationScheme(targets=["Linear"], weights=args)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    out = comp.compress({k: v.to(gpu) for k, v in state.items()}, names_to_scheme={"m": scheme})
    assert set(out) == {"m.weight_packed", "m.weight_shape", "m.weight_scale", "m.weight_zero_point",
                        "m.weight_g_idx", "m.bias", "other.weight"}
    want = op.pack_quantized_compress(w, scale, oargs, zero_point=zp, g_idx=g_idx)
    assert_bit_equal(out["m.weight_packed"], want["weight_packed"], "packed (g_idx)")
    assert_bit_equal(out["m.weight_zero_point"], want["weight_zero_point"], "zp packed")
    assert out["m.weight_zero_point"].dtype == torch.int32 and out["m.weight_shape"].dtype == torch.int64
    (path, data), = list(comp.decompress(out, names_to_scheme={"m": scheme}))
    assert path == "m"
    want_dense = op.pack_quantized_decompress(
        dict(want, weight_scale=scale, weight_g_idx=g_idx), oargs)
    assert_bit_equal(data["weight"], want_dense, "state-dict decompress")
    with pytest.raises(ValueError, match="global_scale"):
        comp.compress_weight(weight=w.to(gpu), scale=scale.to(gpu), quantization_args=args,
                             global_scale=torch.ones(1, device=gpu))


GIDX = [
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128), (64, 1024), torch.bfloat16, None),
    (dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=128), (33, 4096), torch.bfloat16, None),
    (dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=64), (19, 512), torch.float16, None),
    (dict(num_bits=8, type="int", symmetric=True, strategy="group", group_size=8), (13, 2056), torch.bfloat16, None),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=32), (9, 256), torch.float32, None),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128), (16, 512), torch.bfloat16, torch.float32),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=16), (3, 20480), torch.bfloat16, None),
]


@pytest.mark.parametrize("spec,shape,dtype,sdt", GIDX, ids=[f"gidx{i}" for i in range(len(GIDX))])
def test_pack_quantized_with_activation_ordering(spec, shape, dtype, sdt, gpu):
    """weights whose columns were grouped by activation order (a g_idx per column): the
    streaming kernels gather the scales of every element's own group"""
    from compressed_tensors_amd.compressors import BaseCompressor

    announce("pack-quantized g_idx", spec, shape, dtype, sdt)
    args, oargs = _pair(spec)
    rows, cols = shape
    g = torch.Generator().manual_seed(34)
    w = (torch.randn(shape, generator=g) * 0.02).to(dtype)
    w.view(-1)[:3] = torch.tensor([0.0, -0.0, -1e-6]).to(dtype)
    n_groups = cols // spec["group_size"]
    g_idx = (torch.randperm(cols, generator=g) // spec["group_size"]).to(torch.int32)
    scale, zp = oq.observe_weight(w.index_select(-1, torch.argsort(g_idx)), oargs)
    assert scale.shape == (rows, n_groups)
    if sdt is not None:
        scale = scale.to(sdt)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    got = comp.compress_weight(weight=w.to(gpu), scale=scale.to(gpu), quantization_args=args,
                               zero_point=None if spec["symmetric"] else zp.to(gpu), g_idx=g_idx.to(gpu))
    want = op.pack_quantized_compress(w, scale, oargs, zero_point=None if spec["symmetric"] else zp,
                                      g_idx=g_idx)
    assert_bit_equal(got["weight_packed"], want["weight_packed"], "packed")
    data = dict(want, weight_scale=scale, weight_g_idx=g_idx)
    dense_want = op.pack_quantized_decompress(dict(data), oargs)
    dense = comp.decompress_weight({k: v.to(gpu) for k, v in data.items()}, quantization_args=args)
    assert_bit_equal(dense, dense_want, "decompress")


def test_activation_ordered_weights_share_launches(gpu):
    """a batch of activation-ordered weights (more than one launch holds, two scale dtypes,
    with and without zero points, ragged shapes): the shared launches give the bytes of the
    per-weight calls, for compress and for decompress"""
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.compressors.pack_quantized import PackedWeightBatch

    announce("pack-quantized g_idx, many weights per launch")
    sym = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    asym = dict(sym, symmetric=False, group_size=64)
    eight = dict(sym, num_bits=8, group_size=32)
    cases = [(sym, (33, 1024), torch.bfloat16)] * 2 + [(asym, (17, 512), torch.bfloat16),
             (sym, (5, 4096), torch.bfloat16), (eight, (12, 288), torch.bfloat16),
             (sym, (64, 2048), torch.float16), (asym, (40, 2112), torch.bfloat16)]
    cases += [(sym, (r, 1280), torch.bfloat16) for r in (1, 2, 3, 7, 8, 9, 31, 64, 65)]
    g = torch.Generator().manual_seed(35)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    entries, singles = [], []
    for spec, shape, dtype in cases:
        args, oargs = _pair(spec)
        w = (torch.randn(shape, generator=g) * 0.02).to(dtype)
        g_idx = (torch.randperm(shape[1], generator=g) // spec["group_size"]).to(torch.int32)
        scale, zp = oq.observe_weight(w.index_select(-1, torch.argsort(g_idx)), oargs)
        zp = None if spec["symmetric"] else zp
        entry = dict(weight=w.to(gpu), scale=scale.to(gpu), quantization_args=args,
                     g_idx=g_idx.to(gpu), **({} if zp is None else {"zero_point": zp.to(gpu)}))
        entries.append(entry)
        single = comp.compress_weight(**entry)
        dense = comp.decompress_weight(dict(single, weight_scale=entry["scale"], weight_g_idx=entry["g_idx"]),
                                       quantization_args=args)
        singles.append((single["weight_packed"], dense))
    batch = PackedWeightBatch(entries)
    # 12 symmetric bf16 4-bit weights in 2 launches, one launch for each other kind
    assert batch.launches(True) == 5 and batch.launches(False) == 5
    for _ in range(2):
        packed = batch.compress()
        dense = batch.decompress()
        for i, (want_packed, want_dense) in enumerate(singles):
            assert_bit_equal(packed[i], want_packed, f"packed {i}")
            assert_bit_equal(dense[i], want_dense, f"dense {i}")


def test_activation_ordering_with_any_int32_group_labels(gpu):
    """g_idx values are only ever sorted (forward.py:286-289), so labels beyond 32767 and
    negative ones other than -1 must group the columns like small ones; a -1 anywhere
    means the ordering is unset"""
    from compressed_tensors_amd.compressors import BaseCompressor

    spec = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=64)
    args, oargs = _pair(spec)
    announce("pack-quantized g_idx with wide labels")
    g = torch.Generator().manual_seed(35)
    rows, cols = 24, 512
    w = (torch.randn(rows, cols, generator=g) * 0.02).bfloat16()
    small = (torch.randperm(cols, generator=g) // 64).to(torch.int32)
    scale, _ = oq.observe_weight(w.index_select(-1, torch.argsort(small)), oargs)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    want = op.pack_quantized_compress(w, scale, oargs, g_idx=small)["weight_packed"]
    for name, labels in [("wide", small.long() * 70001 - 200000),
                         ("int32 extremes", small.long() * 613566756 - 2147483647)]:
        labels = labels.to(torch.int32)
        assert_bit_equal(op.pack_quantized_compress(w, scale, oargs, g_idx=labels)["weight_packed"], want, name)
        got = comp.compress_weight(weight=w.to(gpu), scale=scale.to(gpu), quantization_args=args,
                                   g_idx=labels.to(gpu))["weight_packed"]
        assert_bit_equal(got, want, name)
    unset = small.clone()
    unset[5] = -1
    got = comp.compress_weight(weight=w.to(gpu), scale=scale.to(gpu), quantization_args=args,
                               g_idx=unset.to(gpu))["weight_packed"]
    assert_bit_equal(got, op.pack_quantized_compress(w, scale, oargs)["weight_packed"], "unset")


NQ = [
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="channel"), (96, 512), torch.bfloat16),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="tensor"), (31, 65), torch.float16),
    ("int-quantized", dict(num_bits=8, type="int", symmetric=True, strategy="channel"), (96, 512), torch.bfloat16),
    ("int-quantized", dict(num_bits=8, type="int", symmetric=False, strategy="group", group_size=128), (16, 256), torch.bfloat16),
    ("naive-quantized", dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=32), (16, 64), torch.float32),
]


@pytest.mark.parametrize("fmt,spec,shape,dtype", NQ, ids=[f"{c[0]}-{i}" for i, c in enumerate(NQ)])
def test_naive_compressors(fmt, spec, shape, dtype, gpu):
    from compressed_tensors_amd.compressors import BaseCompressor

    announce(fmt, spec, shape, dtype)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(41)
    w = torch.randn(shape, generator=g) * 0.02
    w[torch.rand(shape, generator=g) < 0.001] *= 20
    w = w.to(dtype)
    w.view(-1)[1] = -0.0
    scale, zp = oq.observe_weight(w, oargs)
    comp = BaseCompressor.load_from_registry(fmt)
    for zero_point in ((zp,) if not spec["symmetric"] else (zp, None)):
        got = comp.compress_weight(weight=w.to(gpu), scale=scale.to(gpu), quantization_args=args,
                                   zero_point=None if zero_point is None else zero_point.to(gpu))
        want = op.naive_compress(w, scale, oargs, zero_point=zero_point)
        assert list(got) == ["weight"]
        assert_bit_equal(got["weight"], want, "codes")
        data = {"weight": want, "weight_scale": scale}
        if zero_point is not None:
            data["weight_zero_point"] = zero_point
        dense = comp.decompress_weight({k: v.to(gpu) for k, v in data.items()}, quantization_args=args)
        assert_bit_equal(dense, op.naive_decompress(data), "decompress")


def test_fp4_pack_golden_on_gpu(gpu):
    from compressed_tensors_amd.compressors import pack_fp4_to_uint8, unpack_fp4_from_uint8

    announce("fp4 golden")
    gold = json.loads((GOLDEN / "fp4_pack.json").read_text())
    x = torch.tensor(gold["roundtrip"]).to(torch.bfloat16)
    packed = pack_fp4_to_uint8(x.to(gpu))
    assert_bit_equal(packed, op.pack_fp4_to_uint8(x), "fp4 pack")
    back = unpack_fp4_from_uint8(packed, 4, 8, dtype=torch.bfloat16)
    assert_bit_equal(back, x, "fp4 unpack (sign of zero included)")
    with pytest.raises(ValueError, match="even number of columns"):
        pack_fp4_to_uint8(torch.tensor(gold["odd_columns_raise"]).to(gpu))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(3, 6), (16, 64), (5, 1026)])
def test_fp4_pack_off_grid_inputs(dtype, shape, gpu):
    """values off the e2m1 grid go to the nearest entry exactly as the reference's
    argmin over |x - lut| (computed in x's dtype) picks it"""
    from compressed_tensors_amd.compressors import pack_fp4_to_uint8, unpack_fp4_from_uint8

    announce("fp4 off grid", dtype, shape)
    g = torch.Generator().manual_seed(17)
    x = (torch.randn(shape, generator=g) * 3).to(dtype)
    x.view(-1)[:6] = torch.tensor([0.25, 0.75, -1.25, 2.5, 5.0, -7.5]).to(dtype)
    packed = pack_fp4_to_uint8(x.to(gpu))
    want = op.pack_fp4_to_uint8(x)
    assert_bit_equal(packed, want, "fp4 pack off-grid")
    for out_dtype in (torch.bfloat16, torch.float32):
        assert_bit_equal(unpack_fp4_from_uint8(packed, *shape, dtype=out_dtype),
                         op.unpack_fp4_from_uint8(want, *shape, dtype=out_dtype), "fp4 unpack")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_fp4_pack_every_16_bit_pattern_and_mixed_tensors(dtype, gpu):
    """pack_fp4_to_uint8 (fp4_quantized.py:135-178) on all 65 536 patterns of a 16-bit float
    (values of the grid, others, both zeros, infinities, NaNs), and on a large tensor of grid
    values with a few others strewn in: wavefronts with and without a value off the grid"""
    from compressed_tensors_amd.compressors import pack_fp4_to_uint8, unpack_fp4_from_uint8

    announce("fp4 every pattern", dtype)
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype).reshape(256, 256).clone()
    assert_bit_equal(pack_fp4_to_uint8(x.to(gpu)), op.pack_fp4_to_uint8(x), "every pattern")
    g = torch.Generator().manual_seed(5)
    grid = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
    y = (grid[torch.randint(0, 8, (520, 2048), generator=g)]
         * (torch.randint(0, 2, (520, 2048), generator=g) * 2 - 1)).to(dtype)
    flat = y.view(-1)
    where = torch.randint(0, flat.numel(), (40,), generator=g)
    flat[where] = (torch.randn(40, generator=g) * 3).to(dtype)
    flat[where[:4]] = torch.tensor([float("nan"), float("inf"), -float("inf"), 0.75]).to(dtype)
    packed = pack_fp4_to_uint8(y.to(gpu))
    assert_bit_equal(packed, op.pack_fp4_to_uint8(y), "grid values with a few others")
    for out_dtype in (torch.bfloat16, torch.float16, torch.float32):
        assert_bit_equal(unpack_fp4_from_uint8(packed, 520, 2048, dtype=out_dtype),
                         op.unpack_fp4_from_uint8(packed.cpu(), 520, 2048, dtype=out_dtype), "unpack")


@pytest.mark.parametrize("shape,dtype", [((64, 256), torch.bfloat16), ((24, 48), torch.bfloat16),
                                         ((32, 128), torch.float16), ((8, 64), torch.float32)])
def test_nvfp4_compressor(shape, dtype, gpu):
    from compressed_tensors_amd.compressors import BaseCompressor

    announce("nvfp4", shape, dtype)
    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(51)
    w = (torch.randn(shape, generator=g) * 0.02).to(dtype)
    w.view(-1)[:3] = torch.tensor([0.0, -0.0, -1e-6]).to(dtype)
    gs = oq.generate_gparam(*[t.reshape(1) for t in torch.aminmax(w)])
    scale, zp = oq.observe_weight(w, oargs, global_scale=gs)
    assert scale.dtype == torch.float8_e4m3fn and gs.dtype == torch.float32
    comp = BaseCompressor.load_from_registry("nvfp4-pack-quantized")
    for zero_point in (zp, None):
        got = comp.compress_weight(weight=w.to(gpu), scale=scale.to(gpu), global_scale=gs.to(gpu),
                                   quantization_args=args,
                                   zero_point=None if zero_point is None else zero_point.to(gpu))
        want = op.nvfp4_compress(w, scale, gs, oargs, zero_point=zero_point)
        assert list(got) == ["weight_packed"]
        assert_bit_equal(got["weight_packed"], want, f"nvfp4 codes (zp={'yes' if zero_point is not None else 'no'})")
    dense = comp.decompress_weight(
        {"weight_packed": want.to(gpu), "weight_scale": scale.to(gpu),
         "weight_global_scale": gs.to(gpu)}, quantization_args=args)
    assert_bit_equal(dense, op.nvfp4_decompress(want, scale, gs), "nvfp4 decompress")
    assert dense.dtype == torch.bfloat16


@pytest.mark.parametrize("shape,dtype", [((64, 256), torch.bfloat16), ((37, 48), torch.bfloat16),
                                         ((32, 4112), torch.float16), ((8, 64), torch.float32)])
def test_nvfp4_observe_and_compress_in_one_pass(shape, dtype, gpu):
    """global scale, then group scales + codes from one kernel: the oracle's
    generate_gparam, observe_weight and nvfp4_compress, bit for bit"""
    from compressed_tensors_amd.compressors import BaseCompressor

    announce("one-shot nvfp4", shape, dtype)
    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(52)
    w = (torch.randn(shape, generator=g) * 0.02).to(dtype)
    w[0, :16] = 0.0                       # a group of zeros: the 0.125 replacement
    w[0, 17] = -0.0
    w[1, :16] *= 1e-4                     # a scale in the subnormal range of fp8
    w[2, 3] *= 40                         # an outlier that sets the global scale
    gs = oq.generate_gparam(*[t.reshape(1) for t in torch.aminmax(w)])
    scale, zp = oq.observe_weight(w, oargs, global_scale=gs)
    want = op.nvfp4_compress(w, scale, gs, oargs, zero_point=zp)
    comp = BaseCompressor.load_from_registry("nvfp4-pack-quantized")
    got = comp.observe_and_compress_weight(w.to(gpu), args)
    assert set(got) == {"weight_packed", "weight_scale", "weight_global_scale"}
    assert_bit_equal(got["weight_global_scale"], gs, "global scale")
    assert_bit_equal(got["weight_scale"], scale, "group scales")
    assert_bit_equal(got["weight_packed"], want, "codes")
    again = comp.observe_and_compress_weight(w.to(gpu), args, global_scale=gs.to(gpu))
    assert_bit_equal(again["weight_packed"], want, "codes, global scale given")
    with pytest.raises(NotImplementedError):
        comp.observe_and_compress_weight(w.to(gpu)[:, :24].contiguous(), args)


def test_nvfp4_observe_and_compress_many_weights(gpu):
    """nvfp4_observe_and_compress_weights == observe_and_compress_weight weight by weight and
    the oracle: more weights than a launch takes, three dtypes, a chunk that ends ragged"""
    from compressed_tensors_amd.compressors import BaseCompressor, nvfp4_observe_and_compress_weights

    announce("one-shot nvfp4, many weights")
    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    args, oargs = _pair(spec)
    shapes = [(64, 256, torch.bfloat16), (37, 48, torch.bfloat16), (32, 4112, torch.float16), (8, 64, torch.float32),
              (128, 512, torch.bfloat16), (5, 16, torch.bfloat16), (96, 1024, torch.bfloat16), (40, 2048, torch.bfloat16),
              (16, 4096, torch.bfloat16), (300, 64, torch.bfloat16), (24, 768, torch.float16), (12, 3072, torch.bfloat16)]
    g = torch.Generator().manual_seed(66)
    ws = [(torch.randn(r, c, generator=g) * 0.02).to(dt) for r, c, dt in shapes]
    comp = BaseCompressor.load_from_registry("nvfp4-pack-quantized")
    got = nvfp4_observe_and_compress_weights([w.to(gpu) for w in ws], args)
    assert len(got) == len(ws)
    for i, (w, out) in enumerate(zip(ws, got)):
        single = comp.observe_and_compress_weight(w.to(gpu), args)
        assert set(out) == set(single)
        for key in single:
            assert_bit_equal(out[key], single[key], f"weight {i} {key}")
        gs = oq.generate_gparam(*[t.reshape(1) for t in torch.aminmax(w)])
        scale, zp = oq.observe_weight(w, oargs, global_scale=gs)
        assert_bit_equal(out["weight_scale"], scale, f"weight {i} scales vs oracle")
        assert_bit_equal(out["weight_packed"], op.nvfp4_compress(w, scale, gs, oargs, zero_point=zp),
                         f"weight {i} codes vs oracle")
    given = nvfp4_observe_and_compress_weights([w.to(gpu) for w in ws[:3]], args,
                                               global_scales=[o["weight_global_scale"] for o in got[:3]])
    for i in range(3):
        assert_bit_equal(given[i]["weight_packed"], got[i]["weight_packed"], f"global scale given {i}")


@pytest.mark.parametrize("scale_value,global_scale", [(1.0, 1.0), (0.75, 3.0), (448.0, 1234.5),
                                                      (2.0 ** -9, 0.37)])
def test_nvfp4_every_bf16_pattern(scale_value, global_scale, gpu):
    """The no-division fast path and the hardware e2m1 converters against the
    oracle on all 65 536 bf16 inputs (zeros of both signs, subnormals, every
    rounding boundary when the effective scale is 1, infinities, NaNs), for
    compress, decompress and fake-quantize."""
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.quantization import fake_quantize

    announce("nvfp4 all bf16 patterns", scale_value, global_scale)
    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    args, oargs = _pair(spec)
    w = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).reshape(512, 128)
    scale = torch.full((512, 8), scale_value).to(torch.float8_e4m3fn)
    gs = torch.tensor([global_scale], dtype=torch.float32)
    comp = BaseCompressor.load_from_registry("nvfp4-pack-quantized")
    got = comp.compress_weight(weight=w.to(gpu), scale=scale.to(gpu), global_scale=gs.to(gpu),
                               quantization_args=args)["weight_packed"]
    want = op.nvfp4_compress(w, scale, gs, oargs)
    # A NaN input has no defined code: the reference's comes from the sign of a NaN
    # product, which differs between platforms.  Compare the nibbles of all other inputs.
    not_nan = ~torch.isnan(w.float())
    nib = lambda t: torch.stack([t & 15, t >> 4], dim=-1).reshape(512, 128)
    assert_bit_equal(nib(got.cpu())[not_nan], nib(want)[not_nan], "nvfp4 codes")
    dense = comp.decompress_weight({"weight_packed": want.to(gpu), "weight_scale": scale.to(gpu),
                                    "weight_global_scale": gs.to(gpu)}, quantization_args=args)
    assert_bit_equal(dense, op.nvfp4_decompress(want, scale, gs), "nvfp4 decompress")
    finite = ~torch.isnan(w.float())
    fq = fake_quantize(w.to(gpu), scale.to(gpu), None, args, global_scale=gs.to(gpu)).cpu()
    want_fq = oq.fake_quantize(w, scale, None, oargs, global_scale=gs)
    assert_bit_equal(fq[finite], want_fq[finite], "nvfp4 fake-quantize")
    assert bool(torch.isnan(fq[~finite].float()).all() == torch.isnan(want_fq[~finite].float()).all())


@pytest.mark.parametrize("global_scale", [23040.0, 24576.0, 24064.0])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_nvfp4_quotients_on_rounding_boundaries(global_scale, dtype, gpu):
    """Global scales with few significant bits (23040 = 45 * 2^9, 24576 = 3 * 2^13: what
    448 * 6 / amax gives when it is rounded to bfloat16) put a few quotients of nearly every
    wavefront exactly on a rounding boundary of the e2m1 grid, where only the correctly
    rounded division settles the code: every entry point that computes codes, against the
    oracle, plus a tensor where whole rows sit on boundaries (more doubtful vectors than
    the wavefront's queue takes)."""
    from compressed_tensors_amd.compressors import BaseCompressor, nvfp4_observe_and_compress_weights
    from compressed_tensors_amd.quantization import compute_dynamic_scales_and_zp, fake_quantize

    announce("nvfp4 boundaries", global_scale, dtype)
    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(int(global_scale))
    w = (torch.randn(520, 2048, generator=g) * 0.02).to(dtype)
    gs = torch.tensor([global_scale], dtype=torch.float32)
    scale, zp = oq.observe_weight(w, oargs, global_scale=gs)
    # rows 8..15: every element a boundary or a grid value times its group's effective scale
    # (exact in every dtype when the scale has few bits; elsewhere just more inputs)
    eff = (scale[8:16].float() / gs).repeat_interleave(16, dim=1)
    marks = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, -2.5, -0.25])
    w[8:16] = (eff * marks.repeat(8, 2048 // 16)).to(dtype)
    scale, zp = oq.observe_weight(w, oargs, global_scale=gs)
    want = op.nvfp4_compress(w, scale, gs, oargs, zero_point=zp)
    on_boundary = ((w.float() / (scale.float() / gs).repeat_interleave(16, dim=1)).abs().unsqueeze(-1)
                   == marks[:7]).any(-1)
    if dtype == torch.float32:
        assert int(on_boundary[8:16].sum()) > 8000  # the products above are exact
    elif global_scale != 24064.0:
        assert int(on_boundary[16:].sum()) > 100  # here and there in the random rows
    comp = BaseCompressor.load_from_registry("nvfp4-pack-quantized")
    dev = dict(weight=w.to(gpu), scale=scale.to(gpu), global_scale=gs.to(gpu), quantization_args=args)
    assert_bit_equal(comp.compress_weight(**dev)["weight_packed"], want, "compress_weight")
    assert_bit_equal(comp.compress_weight(**dev, zero_point=zp.to(gpu))["weight_packed"], want, "with zero points")
    from compressed_tensors_amd.compressors import Fp4WeightBatch
    batch = Fp4WeightBatch([dev, dict(dev, weight=w.to(gpu).flip(0).contiguous(), scale=scale.to(gpu).flip(0).contiguous())])
    batch.compress()
    assert_bit_equal(batch.packed[0], want, "multi-weight compress")
    assert_bit_equal(batch.packed[1], want.flip(0), "multi-weight compress, second weight")
    one = comp.observe_and_compress_weight(w.to(gpu), args, global_scale=gs.to(gpu))
    assert_bit_equal(one["weight_scale"], scale, "one-shot scales")
    assert_bit_equal(one["weight_packed"], want, "one-shot codes")
    many = nvfp4_observe_and_compress_weights([w.to(gpu), w.to(gpu)[:100].contiguous()], args,
                                              global_scales=[gs.to(gpu), gs.to(gpu)])
    assert_bit_equal(many[0]["weight_packed"], want, "one-shot codes, several weights")
    assert_bit_equal(many[1]["weight_packed"], want[:100], "one-shot codes, several weights (second)")
    fq = fake_quantize(w.to(gpu), scale.to(gpu), None, args, global_scale=gs.to(gpu))
    assert_bit_equal(fq, oq.fake_quantize(w, scale, None, oargs, global_scale=gs), "fake-quantize")
    aspec = dict(spec, dynamic="local")
    aargs, oaargs = _pair(aspec)
    from compressed_tensors_amd.quantization import dynamic_fake_quantize
    dyn = dynamic_fake_quantize(w.to(gpu), aargs, global_scale=gs.to(gpu))
    assert dyn is not None
    s_d, z_d = oq.compute_dynamic_scales_and_zp(w, oaargs, global_scale=gs)
    assert_bit_equal(dyn, oq.fake_quantize(w, s_d, z_d, oaargs, global_scale=gs), "dynamic fake-quantize")


def test_weight_larger_than_4_gib(gpu):
    """a 140 000 x 16 384 bf16 weight (4.6 GB: byte offsets beyond 32 bits, an lm_head of
    a large model): slices at both ends and in the middle against the oracle, and the
    round trip compress(decompress(compress(w))) == compress(w) over the whole tensor"""
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.quantization import observe_weight_qparams

    announce("4.6 GB weight")
    rows, cols = 140_000, 16_384
    spec = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    args, oargs = _pair(spec)
    gen = torch.Generator(device=gpu).manual_seed(99)
    w = torch.empty(rows, cols, dtype=torch.bfloat16, device=gpu)
    for r0 in range(0, rows, 20_000):  # in pieces: the fp32 draw of the whole tensor would be 9 GB
        r1 = min(r0 + 20_000, rows)
        w[r0:r1] = (torch.randn(r1 - r0, cols, generator=gen, device=gpu) * 0.02).bfloat16()
    assert w.numel() * 2 > 1 << 32
    scale, zp = observe_weight_qparams(w, args)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    packed = comp.compress_weight(weight=w, scale=scale, quantization_args=args)["weight_packed"]
    fused = comp.observe_and_compress_weight(w, args)
    assert torch.equal(fused["weight_packed"], packed) and torch.equal(fused["weight_scale"], scale)
    dense = comp.decompress_weight(
        {"weight_packed": packed, "weight_scale": scale, "weight_shape": torch.tensor([rows, cols])},
        quantization_args=args)
    for r0 in (0, 70_001, rows - 48):
        sl = slice(r0, r0 + 48)
        w_cpu = w[sl].cpu()
        o_scale, o_zp = oq.observe_weight(w_cpu, oargs)
        assert_bit_equal(scale[sl], o_scale, f"scale rows {r0}")
        want = op.pack_quantized_compress(w_cpu, o_scale, oargs, zero_point=None)
        assert_bit_equal(packed[sl], want["weight_packed"], f"packed rows {r0}")
        want_dense = op.pack_quantized_decompress(
            dict(want, weight_scale=o_scale, weight_shape=torch.tensor([48, cols])), oargs)
        assert_bit_equal(dense[sl], want_dense, f"dense rows {r0}")
    del w
    again = comp.compress_weight(weight=dense, scale=scale, quantization_args=args)["weight_packed"]
    assert torch.equal(again, packed)


def test_batches_replay_from_a_captured_graph(gpu):
    """the entry points allocate nothing and never synchronise, so a whole pass over a
    state dict can be captured once and replayed: every replay (with eager work and
    synchronisations in between) reproduces the eager result on fresh inputs"""
    from compressed_tensors_amd.compressors import ObservedWeightBatch, PackedWeightBatch
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams

    announce("graph replay")
    args = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    g = torch.Generator(device=gpu).manual_seed(5)
    shapes = [(256, 1024), (64, 512), (512, 256)] * 4  # 12 weights: more than one launch
    weights = [(torch.randn(s, generator=g, device=gpu) * 0.02).bfloat16() for s in shapes]
    entries = []
    for w in weights:
        scale, _ = observe_weight_qparams(w, args)
        entries.append(dict(weight=w, scale=scale, quantization_args=args))
    batch = PackedWeightBatch(entries)
    one_shot = ObservedWeightBatch([dict(weight=w, quantization_args=args) for w in batch.weights])
    lib_stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    batch.compress(), batch.decompress(), one_shot.compress()  # warm up outside the capture
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=lib_stream):
        batch.compress()
        batch.decompress()
        one_shot.compress()
    for replay in range(3):
        for w in batch.weights:  # new data in the captured buffers
            w.copy_((torch.randn(w.shape, generator=g, device=gpu) * 0.02).bfloat16())
        for e, w in zip(entries, batch.weights):  # the scales the captured compress reads
            e["scale"].copy_(observe_weight_qparams(w, args)[0])
        for t in batch.packed + batch.dense + one_shot.packed + one_shot.scales:
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in batch.packed + batch.dense + one_shot.packed + one_shot.scales]
        batch.compress(), batch.decompress(), one_shot.compress()  # eager, same buffers
        torch.cuda.synchronize()
        want = batch.packed + batch.dense + one_shot.packed + one_shot.scales
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f"replay {replay}, tensor {i}"
        assert all(torch.equal(p, q) for p, q in zip(batch.packed, one_shot.packed))


def test_random_shapes_sweep(gpu):
    """random shapes, bit widths and packed dims for pack / unpack; random shapes, group
    sizes, dtypes and symmetry for the pack-quantized compressor (vector, ragged and
    generic kernels alike), against the oracle"""
    from compressed_tensors_amd.compressors import BaseCompressor, pack_to_int32, unpack_from_int32

    g = torch.Generator().manual_seed(77)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    for case in range(40):
        bits, dim = ri(1, 8), ri(0, 1)
        rows, cols = ri(1, 40), ri(1, 300)
        announce("pack sweep", case, bits, dim, (rows, cols))
        lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
        v = torch.randint(lo, hi + 1, (rows, cols), generator=g).to(torch.int8)
        packed = pack_to_int32(v.to(gpu), bits, packed_dim=dim)
        assert_bit_equal(packed, op.pack_to_int32(v, bits, packed_dim=dim), f"pack {case}")
        assert_bit_equal(unpack_from_int32(packed, bits, torch.Size((rows, cols)), packed_dim=dim), v,
                         f"unpack {case}")
    comp = BaseCompressor.load_from_registry("pack-quantized")
    for case in range(40):
        bits = (4, 8, 4, 2, 6)[case % 5]
        group = (8, 16, 32, 64, 128, 24, 4)[case % 7]
        rows, n_groups = ri(1, 70), ri(1, 40)
        cols = group * n_groups
        dtype = (torch.bfloat16, torch.float16, torch.float32)[case % 3]
        symmetric = bool(case % 2)
        strategy = ("group", "channel", "tensor")[ri(0, 2)]
        spec = dict(num_bits=bits, type="int", symmetric=symmetric, strategy=strategy)
        if strategy == "group":
            spec["group_size"] = group
        announce("pack-quantized sweep", case, spec, (rows, cols), dtype)
        args, oargs = _pair(spec)
        w = (torch.randn(rows, cols, generator=g) * 0.02).to(dtype)
        scale, zp = oq.observe_weight(w, oargs)
        zp_arg = None if symmetric else zp
        want = op.pack_quantized_compress(w, scale, oargs, zero_point=zp_arg)
        got = comp.compress_weight(weight=w.to(gpu), scale=scale.to(gpu), quantization_args=args,
                                   zero_point=None if zp_arg is None else zp_arg.to(gpu))
        assert set(got) == set(want)
        for k in want:
            assert_bit_equal(got[k], want[k], f"{k} {case}")
        data = dict(want, weight_scale=scale)
        if not symmetric and strategy == "tensor":
            data["weight_zero_point"] = zp
        dense = comp.decompress_weight({k: v.to(gpu) for k, v in data.items()}, quantization_args=args)
        assert_bit_equal(dense, op.pack_quantized_decompress(dict(data), oargs), f"decompress {case}")


def test_nvfp4_weight_batch_and_state_dict(gpu):
    """Fp4WeightBatch (ctmi_nvfp4_{compress,decompress}_many: 8 weights per launch, more
    than 8 weights, mixed dtypes, a weight whose rows are not whole 16-byte items and so
    falls back to a call of its own) against the per-weight compressor and the oracle; the
    compressor's state-dict compress emits the per-weight loop's keys and values"""
    from compressed_tensors_amd.compressors import BaseCompressor, Fp4WeightBatch
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, QuantizationScheme, generate_gparam, observe_weight_qparams,
    )

    announce("nvfp4 batch")
    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    comp = BaseCompressor.load_from_registry("nvfp4-pack-quantized")
    shapes = [(64, 256, torch.bfloat16), (8, 4096, torch.bfloat16), (33, 48, torch.float16), (128, 512, torch.bfloat16),
              (5, 16, torch.float32), (256, 1024, torch.bfloat16), (16, 32, torch.bfloat16), (40, 80, torch.float16),
              (300, 64, torch.bfloat16), (64, 4112, torch.bfloat16), (7, 16, torch.bfloat16), (96, 160, torch.bfloat16)]
    entries, state, schemes = [], {}, {}
    for i, (r, c, dt) in enumerate(shapes):
        w = (torch.randn((r, c), generator=torch.Generator().manual_seed(40 + i)) * 0.02).to(dt)
        w.view(-1)[:3] = torch.tensor([0.0, -0.0, -1e-6]).to(dt)
        mn, mx = torch.aminmax(w)
        gs = generate_gparam(mn.reshape(1).to(gpu), mx.reshape(1).to(gpu))
        scale, zp = observe_weight_qparams(w.to(gpu), args, global_scale=gs)
        entries.append(dict(weight=w.to(gpu), scale=scale, global_scale=gs, quantization_args=args))
        state[f"m{i}.weight"] = w.to(gpu)
        state[f"m{i}.weight_scale"] = scale
        state[f"m{i}.weight_global_scale"] = gs
        state[f"m{i}.weight_zero_point"] = zp
        schemes[f"m{i}"] = QuantizationScheme(targets=["Linear"], weights=args)
    state["m0.bias"] = torch.ones(64, device=gpu)
    batch = Fp4WeightBatch(entries)
    packed = batch.compress()
    dense = batch.decompress()
    for i, e in enumerate(entries):
        single = comp.compress_weight(weight=e["weight"], scale=e["scale"], global_scale=e["global_scale"],
                                      quantization_args=args)["weight_packed"]
        assert_bit_equal(packed[i], single, f"packed {i} vs single call")
        w, s, g = e["weight"].cpu(), e["scale"].cpu(), e["global_scale"].cpu()
        want = op.nvfp4_compress(w, s, g, oargs)
        assert_bit_equal(packed[i], want, f"packed {i} vs oracle")
        back = comp.decompress_weight({"weight_packed": single, "weight_scale": e["scale"],
                                       "weight_global_scale": e["global_scale"]})
        assert_bit_equal(dense[i], back, f"dense {i} vs single call")
    out = comp.compress(state, names_to_scheme=schemes)
    assert set(out) == ({f"m{i}.weight_packed" for i in range(len(shapes))}
                        | {f"m{i}.weight_scale" for i in range(len(shapes))}
                        | {f"m{i}.weight_global_scale" for i in range(len(shapes))} | {"m0.bias"})
    for i in range(len(shapes)):
        assert_bit_equal(out[f"m{i}.weight_packed"], packed[i], f"state dict {i}")
    restored = dict(comp.decompress_from_state_dict(out, names_to_scheme=schemes))
    for i in range(len(shapes)):
        assert_bit_equal(restored[f"m{i}"]["weight"], dense[i], f"state dict decompress {i}")


OQ = [
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="channel"), (96, 512), torch.bfloat16),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="channel"), (40, 14336), torch.bfloat16),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="channel"), (33, 4104), torch.float16),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="group", group_size=128), (24, 1024), torch.bfloat16),
    ("int-quantized", dict(num_bits=8, type="int", symmetric=True, strategy="channel"), (96, 512), torch.bfloat16),
    ("int-quantized", dict(num_bits=8, type="int", symmetric=False, strategy="channel"), (17, 2048), torch.bfloat16),
    ("int-quantized", dict(num_bits=8, type="int", symmetric=False, strategy="group", group_size=128), (16, 256), torch.float16),
    ("naive-quantized", dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=32), (16, 64), torch.float32),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=False, strategy="channel"), (12, 640), torch.bfloat16),
    # block strategy: one workgroup per block, the block in registers
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[128, 128]), (256, 512), torch.bfloat16),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[128, 128]), (128, 4096), torch.float16),
    ("int-quantized", dict(num_bits=8, type="int", symmetric=False, strategy="block", block_structure=[16, 64]), (48, 192), torch.float32),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=False, strategy="block", block_structure=[3, 8]), (9, 40), torch.bfloat16),
    # no fused kernel: a block of more than 16384 elements, rows longer than 16384, one scale
    # for the whole tensor
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[256, 128]), (256, 256), torch.bfloat16),
    ("float-quantized", dict(num_bits=8, type="float", symmetric=True, strategy="channel"), (3, 16392), torch.bfloat16),
    ("int-quantized", dict(num_bits=8, type="int", symmetric=True, strategy="tensor"), (31, 64), torch.bfloat16),
]


@pytest.mark.parametrize("fmt,spec,shape,dtype", OQ, ids=[f"{c[0]}-{i}" for i, c in enumerate(OQ)])
def test_naive_observe_and_compress_in_one_pass(fmt, spec, shape, dtype, gpu):
    """scales + codes from one kernel: the oracle's observer, calculate_qparams and naive
    compression, bit for bit; shapes without a fused kernel take the two steps"""
    from compressed_tensors_amd.compressors import BaseCompressor

    announce("one-shot", fmt, spec, shape, dtype)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(43)
    w = torch.randn(shape, generator=g) * 0.02
    w[torch.rand(shape, generator=g) < 0.001] *= 20
    w = w.to(dtype)
    w.view(-1)[1] = -0.0
    w[-1] = 0  # an all-zero row: the scale is clamped from below
    scale, zp = oq.observe_weight(w, oargs)
    want = op.naive_compress(w, scale, oargs, zero_point=zp)
    comp = BaseCompressor.load_from_registry(fmt)
    got = comp.observe_and_compress_weight(w.to(gpu), args)
    assert set(got) == ({"weight", "weight_scale"} | (set() if spec["symmetric"] else {"weight_zero_point"}))
    assert_bit_equal(got["weight_scale"], scale, "scale")
    if not spec["symmetric"]:
        assert_bit_equal(got["weight_zero_point"], zp, "zero point")
    assert_bit_equal(got["weight"], want, "codes")
    assert got["weight"].dtype == args.pytorch_dtype()


BLOCKS_MANY = [
    dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[128, 128]),
    dict(num_bits=8, type="int", symmetric=False, strategy="block", block_structure=[16, 64]),
    dict(num_bits=8, type="float", symmetric=False, strategy="block", block_structure=[32, 128]),
]


@pytest.mark.parametrize("spec", BLOCKS_MANY, ids=[f"{s['type']}-{s['block_structure'][0]}x{s['block_structure'][1]}" for s in BLOCKS_MANY])
def test_block_observe_and_compress_many_weights(spec, gpu):
    """block strategy, a list of weights from one call (ctmi_observe_quantize_blocks_many): the
    oracle's observer, calculate_qparams and naive compression bit for bit, and the single
    call; more weights than a launch takes, three dtypes, a weight of a single all-zero block"""
    from compressed_tensors_amd.compressors import BaseCompressor, observe_and_compress_weights

    announce("one-shot blocks, many weights", spec)
    args, oargs = _pair(spec)
    bh, bw = spec["block_structure"]
    mult = [(2, 4), (1, 32), (8, 1), (1, 1), (3, 5), (16, 2), (4, 4), (2, 9), (1, 2), (5, 3), (6, 6)]
    dtypes = [torch.bfloat16, torch.float16, torch.bfloat16, torch.float32]
    g = torch.Generator().manual_seed(17)
    ws = []
    for i, (a, b) in enumerate(mult):
        w = torch.randn(a * bh, b * bw, generator=g) * 0.02
        w[torch.rand(w.shape, generator=g) < 0.002] *= 20
        w = w.to(dtypes[i % len(dtypes)])
        w.view(-1)[1] = -0.0
        if i == 3:
            w[:] = 0  # an all-zero block: the scale is clamped from below
        ws.append(w)
    got = observe_and_compress_weights([w.to(gpu) for w in ws], args)
    comp = BaseCompressor.load_from_registry("naive-quantized")
    assert len(got) == len(ws)
    for i, (w, out) in enumerate(zip(ws, got)):
        scale, zp = oq.observe_weight(w, oargs)
        want = op.naive_compress(w, scale, oargs, zero_point=zp)
        assert set(out) == ({"weight", "weight_scale"} | (set() if spec["symmetric"] else {"weight_zero_point"}))
        assert_bit_equal(out["weight_scale"], scale, f"scale {i}")
        if not spec["symmetric"]:
            assert_bit_equal(out["weight_zero_point"], zp, f"zero point {i}")
        assert_bit_equal(out["weight"], want, f"codes {i}")
        single = comp.observe_and_compress_weight(w.to(gpu), args)
        for key in single:
            assert_bit_equal(out[key], single[key].cpu(), f"single call, weight {i} {key}")
    assert observe_and_compress_weights([], args) == []


def test_naive_observe_and_compress_many_weights(gpu):
    """observe_and_compress_weights == observe_and_compress_weight weight by weight: more
    weights than a launch takes, rows of every length class, two dtypes, a weight whose
    rows have no fused kernel"""
    from compressed_tensors_amd.compressors import BaseCompressor, observe_and_compress_weights
    from compressed_tensors_amd.quantization import QuantizationArgs

    announce("one-shot fp8, many weights")
    shapes = [(64, 512, torch.bfloat16), (8, 4096, torch.bfloat16), (40, 14336, torch.bfloat16), (33, 2048, torch.float16),
              (16, 1032, torch.bfloat16), (5, 8192, torch.bfloat16), (128, 512, torch.bfloat16), (7, 4104, torch.float16),
              (96, 1024, torch.bfloat16), (3, 16392, torch.bfloat16), (24, 768, torch.bfloat16), (12, 3072, torch.bfloat16)]
    g = torch.Generator().manual_seed(91)
    ws = [(torch.randn(r, c, generator=g) * 0.02).to(dt).to(gpu) for r, c, dt in shapes]
    for spec in (dict(num_bits=8, type="float", symmetric=True, strategy="channel"),
                 dict(num_bits=8, type="int", symmetric=False, strategy="channel")):
        args = QuantizationArgs(**spec)
        comp = BaseCompressor.load_from_registry("naive-quantized")
        got = observe_and_compress_weights(ws, args)
        assert len(got) == len(ws)
        for i, (w, out) in enumerate(zip(ws, got)):
            want = comp.observe_and_compress_weight(w, args)
            assert set(out) == set(want)
            for key in want:
                assert_bit_equal(out[key], want[key], f"weight {i} {key}")
