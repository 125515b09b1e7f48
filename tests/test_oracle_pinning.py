"""Pin the oracle: golden vectors held by the reference's own tests, an
independent C restatement of the scalar arithmetic, closed forms and brute
force.  No GPU, no product code."""
import ctypes
import json
import struct
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import pack, quant, sparse

GOLDEN = Path(__file__).parent / "golden"


def _args(d):
    return quant._Args(**d)


# ---------------------------------------------------------------- pack / unpack (A9, A10)
@pytest.mark.parametrize("case", json.loads((GOLDEN / "pack_int32.json").read_text())["cases"])
def test_pack_known_answers(case):
    values = torch.tensor(case["values"], dtype=torch.int8)
    packed = torch.tensor(case["packed"], dtype=torch.int32)
    got = pack.pack_to_int32(values, case["num_bits"])
    assert got.dtype == torch.int32 and torch.equal(got, packed)
    back = pack.unpack_from_int32(packed, case["num_bits"], values.shape)
    assert back.dtype == torch.int8 and torch.equal(back, values)


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_pack_closed_form_every_value_every_slot(bits):
    """element i lands in bits [b*i, b*i+b) as value + 2^(b-1): checked for every
    code value in every slot, against plain Python integers"""
    pf = 32 // bits
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    for slot in range(pf):
        for v in range(lo, hi + 1):
            row = [lo] * pf  # lo encodes as 0 bits
            row[slot] = v
            got = int(pack.pack_to_int32(torch.tensor([row], dtype=torch.int8), bits)[0, 0])
            want = (v - lo) << (bits * slot)
            if want >= 1 << 31:
                want -= 1 << 32
            assert got == want


@pytest.mark.parametrize("bits,shape", [(4, (5, 37)), (8, (3, 10)), (2, (4, 33)), (4, (16, 16))])
def test_pack_roundtrip_and_c(bits, shape, coracle):
    g = torch.Generator().manual_seed(bits * 100 + shape[1])
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1))
    v = torch.randint(lo, hi, shape, generator=g, dtype=torch.int8)
    p = pack.pack_to_int32(v, bits)
    assert torch.equal(pack.unpack_from_int32(p, bits, v.shape), v)
    out = np.zeros(tuple(p.shape), dtype=np.int32)
    vn = v.numpy().copy()
    coracle.oracle_pack_to_int32(vn.ctypes.data, out.ctypes.data, shape[0], shape[1], bits)
    assert np.array_equal(out, p.numpy())
    # packed_dim=0 is the transpose of packing the transposed tensor
    p0 = pack.pack_to_int32(v, bits, packed_dim=0)
    assert torch.equal(p0, pack.pack_to_int32(v.t().contiguous(), bits).t())
    assert torch.equal(pack.unpack_from_int32(p0.contiguous(), bits, v.shape, packed_dim=0), v)


def test_pack_errors():
    with pytest.raises(ValueError):
        pack.pack_to_int32(torch.zeros(2, 2, dtype=torch.int32), 4)
    with pytest.raises(ValueError):
        pack.pack_to_int32(torch.zeros(2, 2, dtype=torch.int8), 9)
    with pytest.raises(ValueError):
        pack.unpack_from_int32(torch.zeros(2, 2, dtype=torch.int8), 4, (2, 2))


# ---------------------------------------------------------------- casts: bf16, fp8
def test_bf16_rounding_matches_c(coracle):
    g = torch.Generator().manual_seed(0)
    bits = torch.randint(0, 2**31 - 1, (200000,), generator=g, dtype=torch.int64)
    bits = (bits | (torch.randint(0, 2, (200000,), generator=g) << 31)).to(torch.int64)
    f = torch.from_numpy(bits.numpy().astype(np.uint32).view(np.float32).copy())
    f = f[~torch.isnan(f)]
    # ties and boundaries
    edge = torch.tensor([1.00390625, 1.01171875, 3.4995, 65504.0, 3.3895e38, 1e-40, -1e-40, 0.0,
                         -0.0, float("inf")])
    f = torch.cat([f, edge])
    want = f.to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16)
    got = np.array([coracle.oracle_f32_to_bf16(float(v)) for v in f[:20000].tolist()]
                   + [coracle.oracle_f32_to_bf16(float(v)) for v in edge.tolist()], dtype=np.uint16)
    assert np.array_equal(got[:20000], want[:20000])
    assert np.array_equal(got[20000:], want[-len(edge):])


def test_fp8_cast_all_bf16_inputs(coracle):
    """torch's float8_e4m3fn cast (used by round_to_quantized_type) against the
    format's definition, on every bf16 bit pattern"""
    allbits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    x = allbits.view(torch.bfloat16)
    got = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    xf = x.float().numpy()
    want = np.array([coracle.oracle_f32_to_f8e4m3(float(v)) for v in xf], dtype=np.uint8)
    nan = np.isnan(xf)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all((got[nan] & 0x7F) == 0x7F)


def test_fp8_cast_fp32_sweep_and_decode(coracle):
    g = torch.Generator().manual_seed(1)
    x = torch.cat([
        (torch.rand(50000, generator=g) - 0.5) * 1000.0,
        (torch.rand(50000, generator=g) - 0.5) * 0.1,
        torch.tensor([448.0, 464.0, 463.99, 479.9, 480.0, 0.001953125, 0.0009765625, 2.0**-10,
                      2.0**-6, 0.0, -0.0]),
    ])
    got = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    want = np.array([coracle.oracle_f32_to_f8e4m3(float(v)) for v in x.tolist()], dtype=np.uint8)
    assert np.array_equal(got, want)
    codes = torch.arange(0, 256, dtype=torch.int32).to(torch.uint8)
    dec = codes.view(torch.float8_e4m3fn).float().numpy()
    for c in range(256):
        v = coracle.oracle_f8e4m3_to_f32(c)
        assert (np.isnan(v) and np.isnan(dec[c])) or v == dec[c]


# ---------------------------------------------------------------- fp4
def test_cast_to_fp4_is_rne_on_e2m1_grid(coracle):
    x = torch.cat([torch.linspace(-7, 7, 5601), torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0,
                                                              -0.25, -0.1, 0.0, -0.0, -5.0])])
    for dt in (torch.float32, torch.bfloat16):
        xd = x.to(dt)
        got = quant.cast_to_fp4(xd.clone()).float()
        want = torch.tensor([coracle.oracle_cast_to_fp4(float(v)) for v in xd.float().tolist()])
        assert torch.equal(got, want)
        assert torch.equal(torch.signbit(got), torch.signbit(want))


def test_fp4_pack_golden():
    gold = json.loads((GOLDEN / "fp4_pack.json").read_text())
    x = torch.tensor(gold["roundtrip"]).to(torch.bfloat16)
    assert torch.equal(torch.signbit(x).int(), torch.tensor(gold["roundtrip_signbits"]).int())
    packed = pack.pack_fp4_to_uint8(x)
    assert packed.dtype == torch.uint8 and packed.shape == (4, 4)
    back = pack.unpack_fp4_from_uint8(packed, 4, 8, dtype=torch.bfloat16)
    assert torch.equal(back, x) and torch.equal(torch.signbit(back), torch.signbit(x))
    with pytest.raises(ValueError):
        pack.pack_fp4_to_uint8(torch.tensor(gold["odd_columns_raise"]))


def test_fp4_code_table(coracle):
    vals = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    x = torch.tensor([vals + [-v for v in vals]], dtype=torch.bfloat16)
    packed = pack.pack_fp4_to_uint8(x).flatten().tolist()
    codes = []
    for b in packed:
        codes += [b & 15, b >> 4]
    assert codes == list(range(16))
    for c in range(16):
        assert coracle.oracle_fp4_code(coracle.oracle_fp4_decode(c)) == c


# ---------------------------------------------------------------- quantize / dequantize (A1, A5-A8)
GOLD_LC = json.loads((GOLDEN / "static_lifecycle.json").read_text())


@pytest.mark.parametrize("case", GOLD_LC["weight_cases"], ids=lambda c: c["args"]["strategy"])
def test_static_weight_golden(case):
    args = _args(case["args"])
    w = torch.arange(24, dtype=torch.bfloat16).reshape(4, 6)
    gs = None
    if args.strategy == "tensor_group":
        gs = quant.generate_gparam(*torch.aminmax(w.reshape(1, 1, -1)))
    # expected observer min / max
    s = args.strategy
    obs = {"tensor": w.reshape(1, 1, -1), "channel": w.unsqueeze(-2).unsqueeze(0)}.get(s)
    if s in ("group", "tensor_group"):
        obs = w.unflatten(-1, (-1, args.group_size)).unsqueeze(0)
    if s == "block":
        bh, bw = args.block_structure
        obs = w.reshape(4 // bh, bh, 6 // bw, bw).transpose(1, 2).flatten(-2, -1).unsqueeze(0)
    assert torch.equal(torch.amin(obs, dim=(0, -1)).float(), torch.tensor(case["min"]).float())
    assert torch.equal(torch.amax(obs, dim=(0, -1)).float(), torch.tensor(case["max"]).float())
    scale, zp = quant.observe_weight(w, args, global_scale=gs)
    out = quant.fake_quantize(w, scale, zp, args, global_scale=gs)
    want = torch.tensor(case["qdq"]).to(out.dtype)
    assert torch.equal(out, want)
    assert torch.nn.functional.mse_loss(out.float(), w.float()) <= case["max_mse"]


@pytest.mark.parametrize("case", GOLD_LC["activation_cases"], ids=lambda c: c["args"]["strategy"])
def test_static_activation_golden(case):
    a = dict(case["args"])
    dynamic = a.pop("dynamic", False)
    args = _args(a)
    x = torch.arange(12, dtype=torch.bfloat16).reshape(1, 2, 6)
    gs = None
    if args.strategy == "tensor_group":
        gs = quant.generate_gparam(*torch.aminmax(x.reshape(1, 1, -1)))
    if dynamic:
        scale, zp = quant.compute_dynamic_scales_and_zp(x, args, global_scale=gs)
    else:
        mn, mx = torch.aminmax(x)
        assert float(mn) == case["min"][0] and float(mx) == case["max"][0]
        scale, zp = quant.calculate_qparams(mn.reshape(1), mx.reshape(1), args)
    out = quant.fake_quantize(x, scale, zp, args, global_scale=gs)
    assert torch.equal(out, torch.tensor(case["qdq"]).to(out.dtype))
    assert torch.nn.functional.mse_loss(out.float(), x.float()) <= case["max_mse"]


def test_w4a16_chain_against_c(coracle):
    """the bf16 chain div -> +zp -> clamp -> round -> int8, and int8 -> bf16 * scale,
    element by element against the C restatement (one fp32 op + one bf16 rounding
    per step)"""
    torch.manual_seed(3)
    R, C, G = 16, 256, 128
    w = (torch.randn(R, C) * 0.02).bfloat16()
    args = _args(dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=G))
    scale, zp = quant.observe_weight(w, args)
    assert scale.dtype == torch.bfloat16 and scale.shape == (R, C // G) and zp.dtype == torch.int8
    # closed form of the symmetric int4 scale: bf16(maxabs / 7.5)
    maxabs = w.float().abs().unflatten(-1, (-1, G)).amax(-1)
    assert torch.equal(scale, (maxabs.bfloat16() / 7.5))
    q = quant.quantize(w, scale, zp, args, dtype=torch.int8)
    wn = w.view(torch.int16).numpy().copy()
    sn = scale.view(torch.int16).numpy().copy()
    zn = zp.numpy().copy()
    out = np.zeros((R, C), dtype=np.int8)
    coracle.oracle_quantize_int_bf16(wn.ctypes.data, sn.ctypes.data, zn.ctypes.data,
                                     out.ctypes.data, R, C, G, 4)
    assert np.array_equal(out, q.numpy())
    dq = quant.dequantize(q, scale, zp)
    assert dq.dtype == torch.bfloat16
    dout = np.zeros((R, C), dtype=np.uint16)
    coracle.oracle_dequantize_int_bf16(out.ctypes.data, sn.ctypes.data, zn.ctypes.data,
                                       dout.ctypes.data, R, C, G)
    assert np.array_equal(dout, dq.view(torch.int16).numpy().astype(np.uint16))
    # and the intermediate bf16 rounding really matters (it is not fp32 math)
    q32 = torch.round(torch.clamp(w.float() / scale.float().repeat_interleave(G, 1), -8, 7))
    assert (q32.to(torch.int8) != q).any()


def test_fp8_channel_chain_against_c(coracle):
    torch.manual_seed(4)
    w = (torch.randn(8, 64) * 0.02).bfloat16()
    w[0, 0] = -0.0
    args = _args(dict(num_bits=8, type="float", symmetric=True, strategy="channel"))
    scale, zp = quant.observe_weight(w, args)
    assert scale.shape == (8, 1) and scale.dtype == torch.bfloat16 and zp.dtype == torch.float8_e4m3fn
    for zero_point in (zp, None):
        q = quant.quantize(w, scale, zero_point, args, dtype=torch.float8_e4m3fn)
        codes = q.view(torch.uint8)
        for r in range(8):
            for c in range(64):
                v = coracle.oracle_quantize(float(w[r, c]), float(scale[r, 0]), 0.0,
                                            int(zero_point is not None), 1, 8, 2)
                assert coracle.oracle_f32_to_f8e4m3(v) == int(codes[r, c])
        # -0.0 survives only when no zero point is added
        assert int(codes[0, 0]) == (0x00 if zero_point is not None else 0x80)


def test_asymmetric_qparams_closed_form():
    args = _args(dict(num_bits=8, type="int", symmetric=False, strategy="channel"))
    mn = torch.tensor([[-1.0], [0.5], [-3.0]])
    mx = torch.tensor([[2.0], [4.0], [-1.0]])
    scale, zp = quant.calculate_qparams(mn, mx, args)
    lo = torch.minimum(mn, torch.zeros(()))
    hi = torch.maximum(mx, torch.zeros(()))
    want_scale = (hi - lo) / 255.0
    assert torch.equal(scale, want_scale)
    assert torch.equal(zp, torch.round(torch.clamp(-128 - lo / want_scale, -128, 127)).to(torch.int8))
    assert zp.dtype == torch.int8


def test_gparam_closed_form():
    mn, mx = torch.tensor([-0.3]), torch.tensor([0.2])
    assert torch.equal(quant.generate_gparam(mn, mx), torch.tensor([448.0 * 6.0 / 0.3]))


def test_range_containment():
    """quantized values stay inside the type's range; fp8 reaches +-448"""
    torch.manual_seed(5)
    x = torch.randn(64, 64) * 3
    for d in (dict(num_bits=4, type="int"), dict(num_bits=8, type="int"),
              dict(num_bits=8, type="float"), dict(num_bits=4, type="float")):
        args = _args(dict(d, symmetric=True, strategy="tensor"))
        mn, mx = torch.aminmax(x)
        scale, zp = quant.calculate_qparams(mn.reshape(1), mx.reshape(1), args)
        q = quant.quantize(x, scale, zp, args)
        lo, hi = quant.calculate_range(args)
        assert q.min() >= lo and q.max() <= hi
        assert q.abs().max() == hi or q.min() == lo


# ---------------------------------------------------------------- bitmasks (A17-A22)
@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (4, 8), (5, 17), (16, 64)])
def test_packbits_matches_c_and_roundtrips(shape, coracle):
    g = torch.Generator().manual_seed(shape[1])
    mask = torch.rand(shape, generator=g) > 0.5
    packed = sparse.pack_bitmasks(mask)
    assert packed.shape == (shape[0], (shape[1] + 7) // 8) and packed.dtype == torch.uint8
    mn = mask.numpy().astype(np.uint8).copy()
    out = np.zeros(tuple(packed.shape), dtype=np.uint8)
    coracle.oracle_packbits_little(mn.ctypes.data, out.ctypes.data, shape[0], shape[1])
    assert np.array_equal(out, packed.numpy())
    assert torch.equal(sparse.unpack_bitmasks(packed, list(shape)), mask)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,sparsity", [((2, 10), 0.5), ((16, 50), 0.9), ((7, 64), 0.0), ((3, 9), 1.0)])
def test_bitmask_lossless_and_row_offsets(dtype, shape, sparsity, coracle):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(shape, generator=g).to(dtype)
    x[torch.rand(shape, generator=g) < sparsity] = 0
    if x.numel() > 3:
        x.view(-1)[1] = -0.0
    values, bitmask, row_offsets = sparse.bitmask_compress(x)
    assert row_offsets.dtype == torch.int64
    nnz_rows = (x != 0).sum(-1)
    assert torch.equal(row_offsets, torch.cumsum(nnz_rows, 0) - nnz_rows)
    assert values.numel() == int(nnz_rows.sum())
    back = sparse.bitmask_decompress(values, bitmask, list(shape))
    assert torch.equal(back, x)
    if dtype == torch.bfloat16:
        xn = x.view(torch.int16).numpy().astype(np.uint16).copy()
        vals = np.zeros(x.numel(), dtype=np.uint16)
        bm = np.zeros(tuple(bitmask.shape), dtype=np.uint8)
        ro = np.zeros(shape[0], dtype=np.int64)
        n = coracle.oracle_bitmask_compress_u16(xn.ctypes.data, shape[0], shape[1],
                                                vals.ctypes.data, bm.ctypes.data, ro.ctypes.data)
        assert n == values.numel()
        assert np.array_equal(vals[:n], values.view(torch.int16).numpy().astype(np.uint16))
        assert np.array_equal(bm, bitmask.numpy()) and np.array_equal(ro, row_offsets.numpy())


def test_24_mask_properties_and_topk_order():
    g = torch.Generator().manual_seed(9)
    x = torch.randn(8, 16, generator=g).bfloat16()
    mask = sparse.get_24_bytemasks(x)
    assert torch.all(mask.reshape(-1, 4).sum(-1) == 2)
    # with distinct magnitudes the survivors are exactly the two largest
    groups = x.float().abs().reshape(-1, 4)
    for grp, m in zip(groups, mask.reshape(-1, 4)):
        if len(set(grp.tolist())) == 4:
            assert grp[m].min() > grp[~m].max()
    # on 2:4-pruned input the mask covers every non-zero
    pruned = torch.where(mask, x, torch.zeros_like(x))
    mask2 = sparse.get_24_bytemasks(pruned)
    assert torch.all(mask2[pruned != 0])
    vals, bm = sparse.sparse24_bitmask_compress(pruned)
    assert vals.shape == (8, 8) and bm.shape == (8, 2)
    assert torch.equal(sparse.sparse24_bitmask_decompress(vals, bm, pruned.shape), pruned)


def test_24_mask_fp8_uses_int8_view():
    codes = torch.tensor([[0x80, 0x01, 0x00, 0x02, 0xFF, 0x7E, 0x81, 0x00]], dtype=torch.uint8)
    x = codes.view(torch.float8_e4m3fn)
    mask = sparse.get_24_bytemasks(x)
    i8 = codes.view(torch.int8)
    want = torch.zeros_like(i8, dtype=torch.bool).reshape(-1, 4)
    want.scatter_(1, i8.reshape(-1, 4).abs().topk(2, dim=1).indices, True)
    assert torch.equal(mask, want.reshape(1, 8))
    # abs(int8(-128)) wraps to -128 and so ranks below zero
    assert not bool(mask[0, 0])


# ---------------------------------------------------------------- MXFP4 scales
def test_mxfp4_round_to_power_2_reference_vector():
    from oracle import mxfp4

    gold = json.loads((GOLDEN / "mxfp4.json").read_text())
    x = torch.tensor(gold["x"]).to(torch.bfloat16)
    want = torch.tensor(gold["rounded"]).to(torch.bfloat16)
    assert torch.equal(mxfp4.round_to_power_2(x), want)


def test_mxfp4_noisy_powers_round_back():
    """the reference's second test (test_mxfp4_utils.py:22-38): a power of two times
    (1 + up to 20 % noise) rounds back to it"""
    from oracle import mxfp4

    g = torch.Generator().manual_seed(0)
    powers = (2.0 ** torch.arange(-10, 2).float()).repeat(50).to(torch.bfloat16)
    noisy = powers * (1 + torch.rand(powers.shape, generator=g).to(torch.bfloat16) * 0.2)
    assert torch.equal(mxfp4.round_to_power_2(noisy), powers)


def test_mxfp4_scales_closed_form():
    """every positive normal bfloat16: the exponent is that of the rounded power of two
    minus 2 (clamped at 0), and 2 ** (e - 127) gives it back (test_mxfp4_utils.py:64-80)"""
    from oracle import mxfp4

    bits = torch.arange(0x0080, 0x7F80, dtype=torch.int32).to(torch.uint16)
    x = bits.view(torch.bfloat16)
    e = mxfp4.generate_mxfp4_scales(x)
    rounded_bits = (bits.to(torch.int32) + 32) & 0xFF80
    biased = rounded_bits >> 7
    want = torch.where(biased == 255, torch.zeros_like(biased), torch.clamp(biased - 2, min=0))
    assert torch.equal(e.to(torch.int32), want)
    ok = (biased >= 2) & (biased < 255)
    back = mxfp4.convert_mxfp4_exp_scale(e)
    assert torch.equal(torch.log2(back.float())[ok], (biased[ok] - 2 - 127).float())
    # all 256 exponents: exact powers of two, subnormal at the bottom, infinite at the top
    every = mxfp4.convert_mxfp4_exp_scale(torch.arange(256, dtype=torch.int32).to(torch.uint8), torch.float32)
    assert every[0].item() == 2.0 ** -127 and every[127].item() == 1.0 and every[254].item() == 2.0 ** 127
    assert torch.isinf(every[255])


# ---------------------------------------------------------------- NVFP4 global scale (A16)
def test_generate_gparam_is_reciprocal_times_constant():
    """`448 * 6 / max_val_pos` (helpers.py:431) has a Python float on the left, so torch
    runs Tensor.__rtruediv__: reciprocal, then the product, each rounded to the tensor's
    dtype.  For max|x| = 1.1953125 in bfloat16 that is bf16(bf16(0.8366) * 2688) = 2240,
    where a single division would give bf16(2248.78) = 2256."""
    m = torch.tensor([1.1953125], dtype=torch.bfloat16)
    got = quant.generate_gparam(-m, m / 2)
    assert got.dtype == torch.float32 and got.shape == (1,)
    assert got.item() == 2240.0
    r = torch.tensor(1.0 / 1.1953125).to(torch.bfloat16)
    assert (r.float() * 2688.0).to(torch.bfloat16).item() == 2240.0
    assert torch.tensor(2688.0 / 1.1953125).to(torch.bfloat16).item() == 2256.0
    # and on every positive normal bfloat16: the two-step closed form
    v = torch.arange(0x0080, 0x7f80, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    closed = ((1.0 / v.float()).to(torch.bfloat16).float() * 2688.0).to(torch.bfloat16).float()
    every = (448.0 * 6.0 / v).float()
    assert torch.equal(every, closed)


@pytest.mark.parametrize("case", GOLD_LC["attention_cases"], ids=lambda c: c["args"]["strategy"])
def test_static_attention_golden(case):
    """keys of shape (batch, heads, seq, head_dim) quantized per tensor and per head
    (test_static_lifecycle.py:278-386); the observer reduces everything but the head"""
    args = _args(case["args"])
    x = torch.arange(24, dtype=torch.bfloat16).reshape(1, 2, 3, 4)
    if args.strategy == "tensor":
        mn, mx = torch.aminmax(x)
        mn, mx = mn.reshape(1), mx.reshape(1)
    else:
        mn = torch.amin(x, dim=(0, 2, 3)).reshape(2, 1, 1)
        mx = torch.amax(x, dim=(0, 2, 3)).reshape(2, 1, 1)
    assert torch.equal(mn.float(), torch.tensor(case["min"]))
    assert torch.equal(mx.float(), torch.tensor(case["max"]))
    scale, zp = quant.calculate_qparams(mn, mx, args)
    out = quant.fake_quantize(x, scale, zp, args)
    assert torch.equal(out, torch.tensor(case["qdq"]).to(out.dtype))
    assert torch.nn.functional.mse_loss(out.float(), x.float()) <= case["max_mse"]
