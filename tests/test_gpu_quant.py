"""GPU parity: quantize / dequantize / fake_quantize and qparams vs the oracle
(bit-exact), called through the Python mirror of the reference API -> C ABI."""
import json
from pathlib import Path

import pytest
import torch

from gpu_util import announce, assert_bit_equal, bits as bits_of
from oracle import pack as op
from oracle import quant as oq

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).parent / "golden"


def _pair(d):
    from compressed_tensors_amd.quantization import QuantizationArgs

    d = dict(d)
    dyn = d.pop("dynamic", False)
    return QuantizationArgs(dynamic=dyn, **d), oq._Args(**d)


def _weights(shape, dtype, seed, std=0.02):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(shape, generator=g) * std).to(dtype)
    flat = w.view(-1)
    flat[0] = 0.0
    if flat.numel() > 8:
        flat[3] = -0.0
        flat[5] = flat[4].abs() * 20
    return w


CASES = [
    # (args, shape, x dtype, scale dtype override)
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128), (64, 512), torch.bfloat16, None),
    (dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=128), (64, 512), torch.bfloat16, None),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=32), (33, 96), torch.float16, None),
    (dict(num_bits=8, type="int", symmetric=True, strategy="channel"), (48, 200), torch.bfloat16, None),
    (dict(num_bits=8, type="int", symmetric=False, strategy="channel"), (48, 200), torch.float32, None),
    (dict(num_bits=8, type="int", symmetric=False, strategy="tensor"), (17, 129), torch.bfloat16, None),
    (dict(num_bits=4, type="int", symmetric=True, strategy="tensor"), (17, 129), torch.float16, None),
    (dict(num_bits=8, type="float", symmetric=True, strategy="channel"), (40, 256), torch.bfloat16, None),
    (dict(num_bits=8, type="float", symmetric=True, strategy="tensor"), (40, 250), torch.float16, None),
    (dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[16, 32]), (64, 128), torch.bfloat16, None),
    (dict(num_bits=4, type="int", symmetric=True, strategy="block", block_structure=[2, 3]), (4, 6), torch.bfloat16, None),
    (dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[128, 128]), (256, 384), torch.bfloat16, None),
    (dict(num_bits=8, type="int", symmetric=False, strategy="block", block_structure=[8, 64]), (64, 256), torch.float16, None),
    (dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[6, 32]), (12, 64), torch.bfloat16, None),
    (dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[1, 16]), (5, 64), torch.float32, None),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128), (32, 256), torch.bfloat16, torch.float32),
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=64), (32, 256), torch.float16, torch.bfloat16),
    (dict(num_bits=2, type="int", symmetric=True, strategy="channel"), (8, 64), torch.bfloat16, None),
]


@pytest.mark.parametrize("spec,shape,dtype,sdt", CASES,
                         ids=[f"{c[0]['type']}{c[0]['num_bits']}-{c[0]['strategy']}-{str(c[2])[6:]}-{i}"
                              for i, c in enumerate(CASES)])
def test_static_qdq_matches_oracle(spec, shape, dtype, sdt, gpu):
    from compressed_tensors_amd.quantization import (
        dequantize, fake_quantize, observe_weight_qparams, quantize,
    )

    announce("static_qdq", spec, shape, dtype, sdt)
    args, oargs = _pair(spec)
    w = _weights(shape, dtype, seed=11)
    o_scale, o_zp = oq.observe_weight(w, oargs)
    # observer + calculate_qparams on the GPU
    scale, zp = observe_weight_qparams(w.to(gpu), args)
    assert_bit_equal(scale, o_scale, "scale")
    assert_bit_equal(zp, o_zp, "zero_point")
    if sdt is not None:
        o_scale = o_scale.to(sdt)
        scale = o_scale.to(gpu)
    qdt = oq.pytorch_dtype(oargs)
    for zero_point, o_zero_point in ((zp, o_zp), (None, None)):
        if zero_point is None and not spec["symmetric"]:
            continue
        q = quantize(w.to(gpu), scale, zero_point, args, dtype=qdt)
        oq_ = oq.quantize(w, o_scale, o_zero_point, oargs, dtype=qdt)
        assert_bit_equal(q, oq_, "quantize")
        qf = quantize(w.to(gpu), scale, zero_point, args)  # no dtype: stays floating
        assert_bit_equal(qf, oq.quantize(w, o_scale, o_zero_point, oargs), "quantize(no dtype)")
        dq = dequantize(q, scale, zero_point, args)
        assert_bit_equal(dq, oq.dequantize(oq_, o_scale, o_zero_point, oargs), "dequantize")
        dq2 = dequantize(q, scale, zero_point)  # strategy inferred from the scale's shape
        assert_bit_equal(dq2, oq.dequantize(oq_, o_scale, o_zero_point), "dequantize(inferred)")
        fq = fake_quantize(w.to(gpu), scale, zero_point, args)
        assert_bit_equal(fq, oq.fake_quantize(w, o_scale, o_zero_point, oargs), "fake_quantize")


def test_reference_golden_qdq_on_gpu(gpu):
    """the reference's own expected QDQ matrices, reproduced by the HIP path"""
    from compressed_tensors_amd.quantization import (
        fake_quantize, generate_gparam, observe_weight_qparams,
    )

    gold = json.loads((GOLDEN / "static_lifecycle.json").read_text())
    w = torch.arange(24, dtype=torch.bfloat16).reshape(4, 6)
    for case in gold["weight_cases"]:
        announce("golden", case["args"])
        args, oargs = _pair(case["args"])
        gs = o_gs = None
        if args.strategy == "tensor_group":
            mn, mx = torch.aminmax(w)
            o_gs = oq.generate_gparam(mn.reshape(1), mx.reshape(1))
            gs = generate_gparam(mn.reshape(1).to(gpu), mx.reshape(1).to(gpu))
            assert_bit_equal(gs, o_gs, "global scale")
        scale, zp = observe_weight_qparams(w.to(gpu), args, global_scale=gs)
        o_scale, o_zp = oq.observe_weight(w, oargs, global_scale=o_gs)
        assert_bit_equal(scale, o_scale, "scale")
        assert_bit_equal(zp, o_zp, "zp")
        out = fake_quantize(w.to(gpu), scale, zp, args, global_scale=gs)
        assert_bit_equal(out, oq.fake_quantize(w, o_scale, o_zp, oargs, global_scale=o_gs), "qdq")
        assert torch.allclose(out.cpu(), torch.tensor(case["qdq"]).to(out.dtype))


def test_act_order_g_idx(gpu):
    from compressed_tensors_amd.quantization import dequantize, quantize

    announce("g_idx")
    spec = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=32)
    args, oargs = _pair(spec)
    w = _weights((24, 128), torch.bfloat16, seed=5)
    g = torch.Generator().manual_seed(6)
    g_idx = (torch.randperm(128, generator=g) // 32).to(torch.int32)
    perm = torch.argsort(g_idx)
    o_scale, o_zp = oq.observe_weight(w.index_select(-1, perm), oargs)
    q = quantize(w.to(gpu), o_scale.to(gpu), o_zp.to(gpu), args, dtype=torch.int8, g_idx=g_idx.to(gpu))
    want = oq.quantize(w, o_scale, o_zp, oargs, dtype=torch.int8, g_idx=g_idx)
    assert_bit_equal(q, want, "quantize g_idx")
    dq = dequantize(q, o_scale.to(gpu), o_zp.to(gpu), g_idx=g_idx.to(gpu))
    assert_bit_equal(dq, oq.dequantize(want, o_scale, o_zp, g_idx=g_idx), "dequantize g_idx")
    # g_idx full of -1 means column order
    unset = torch.full((128,), -1, dtype=torch.int32)
    q2 = quantize(w.to(gpu), o_scale.to(gpu), None, args, dtype=torch.int8, g_idx=unset.to(gpu))
    assert_bit_equal(q2, oq.quantize(w, o_scale, None, oargs, dtype=torch.int8, g_idx=unset), "unset g_idx")


DYN = [
    (dict(num_bits=8, type="float", symmetric=True, strategy="token", dynamic=True), (2, 40, 256), torch.bfloat16),
    (dict(num_bits=8, type="int", symmetric=True, strategy="token", dynamic=True), (1, 33, 100), torch.float16),
    (dict(num_bits=8, type="int", symmetric=False, strategy="token", dynamic=True), (3, 8, 64), torch.bfloat16),
    (dict(num_bits=8, type="int", symmetric=True, strategy="token", dynamic=True), (16, 64), torch.bfloat16),
    (dict(num_bits=8, type="float", symmetric=True, strategy="tensor", dynamic=True), (4, 9, 31), torch.bfloat16),
    (dict(num_bits=8, type="int", symmetric=False, strategy="tensor", dynamic=True), (7, 33), torch.bfloat16),
    (dict(num_bits=8, type="float", symmetric=True, strategy="group", group_size=128, dynamic=True), (1, 16, 512), torch.bfloat16),
    (dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16, dynamic="local"), (1, 32, 256), torch.bfloat16),
]


@pytest.mark.parametrize("spec,shape,dtype", DYN, ids=[f"{c[0]['strategy']}-{i}" for i, c in enumerate(DYN)])
def test_dynamic_activation_quant(spec, shape, dtype, gpu):
    from compressed_tensors_amd.quantization import (
        compute_dynamic_scales_and_zp, fake_quantize, generate_gparam,
    )

    announce("dynamic", spec, shape, dtype)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(21)
    x = torch.randn(shape, generator=g)
    x[..., 3] *= 50
    x = x.to(dtype)
    gs = o_gs = None
    if args.strategy == "tensor_group":
        mn, mx = torch.aminmax(x)
        o_gs = oq.generate_gparam(mn.reshape(1), mx.reshape(1))
        gs = o_gs.to(gpu)
    o_scale, o_zp = oq.compute_dynamic_scales_and_zp(x, oargs, global_scale=o_gs)
    scale, zp = compute_dynamic_scales_and_zp(x.to(gpu), args, None, global_scale=gs)
    assert_bit_equal(scale, o_scale, "dynamic scale")
    assert_bit_equal(zp, o_zp, "dynamic zp")
    out = fake_quantize(x.to(gpu), scale, zp, args, global_scale=gs)
    assert_bit_equal(out, oq.fake_quantize(x, o_scale, o_zp, oargs, global_scale=o_gs), "dynamic qdq")


FUSED = [
    # (args, shape, dtype, fused kernel expected)
    (dict(num_bits=8, type="float", symmetric=True, strategy="token", dynamic=True), (2, 40, 256), torch.bfloat16, True),
    (dict(num_bits=8, type="float", symmetric=True, strategy="token", dynamic=True), (1, 19, 4096), torch.bfloat16, True),
    (dict(num_bits=8, type="float", symmetric=True, strategy="token", dynamic=True), (1, 5, 8192), torch.float16, True),
    (dict(num_bits=8, type="float", symmetric=False, strategy="token", dynamic=True), (2, 7, 1024), torch.bfloat16, True),
    (dict(num_bits=8, type="int", symmetric=True, strategy="token", dynamic=True), (3, 33, 320), torch.bfloat16, True),
    (dict(num_bits=8, type="int", symmetric=False, strategy="token", dynamic=True), (3, 8, 64), torch.bfloat16, True),
    (dict(num_bits=8, type="int", symmetric=False, strategy="token", dynamic=True), (2, 9, 2, 760), torch.float32, True),
    (dict(num_bits=4, type="int", symmetric=False, strategy="token", dynamic=True), (1, 70, 5120), torch.float16, True),
    (dict(num_bits=8, type="int", symmetric=True, strategy="token", dynamic=True), (1, 33, 100), torch.float16, False),
    (dict(num_bits=8, type="int", symmetric=True, strategy="token", dynamic=True), (16, 64), torch.bfloat16, False),
    (dict(num_bits=8, type="float", symmetric=True, strategy="group", group_size=128, dynamic=True), (1, 16, 512), torch.bfloat16, True),
    (dict(num_bits=8, type="int", symmetric=False, strategy="group", group_size=32, dynamic=True), (45, 96), torch.bfloat16, True),
    (dict(num_bits=8, type="int", symmetric=True, strategy="group", group_size=8, dynamic=True), (3, 11, 72), torch.float32, True),
    (dict(num_bits=8, type="int", symmetric=True, strategy="group", group_size=24, dynamic=True), (7, 48), torch.bfloat16, True),
    (dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16, dynamic="local"), (1, 32, 256), torch.bfloat16, True),
    (dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16, dynamic="local"), (77, 48), torch.float16, True),
    (dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16, dynamic="local"), (2, 3, 4112), torch.float32, True),
]


@pytest.mark.parametrize("spec,shape,dtype,fusable", FUSED,
                         ids=[f"{c[0]['type']}{c[0]['num_bits']}-{c[0]['strategy']}-{i}" for i, c in enumerate(FUSED)])
def test_dynamic_quant_in_one_pass(spec, shape, dtype, fusable, gpu):
    """scales + fake-quantization from one kernel: same bits as the oracle's
    compute_dynamic_scales_and_zp followed by fake_quantize, special values included"""
    from compressed_tensors_amd.quantization import forward_quantize
    from compressed_tensors_amd.quantization.helpers import dynamic_fake_quantize

    announce("dynamic one pass", spec, shape, dtype)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(shape, generator=g)
    x[..., 3] *= 50
    x = x.to(dtype)
    flat = x.view(-1, x.shape[-1])
    flat[0, :8] = 0.0                      # a stretch of zeros
    flat[0, 1] = -0.0
    flat[-1] = 0.0                         # a row of zeros: the scale floor
    if flat.shape[0] > 2:
        flat[1, 5] = float("nan")          # poisons its group / token
        flat[2, 0] = float("inf")
    if flat.shape[0] > 6:
        flat[3] *= 1e-5                    # group scales down in the subnormal range of fp8
        flat[4] *= 3e-4
    gs = o_gs = None
    module = torch.nn.Module()
    if args.strategy == "tensor_group":
        finite = torch.nan_to_num(x.float(), nan=0.0, posinf=1.0, neginf=-1.0)
        mn, mx = torch.aminmax(finite)
        o_gs = oq.generate_gparam(mn.reshape(1), mx.reshape(1))
        gs = o_gs.to(gpu)
        module.input_global_scale = gs
    o_scale, o_zp = oq.compute_dynamic_scales_and_zp(x, oargs, global_scale=o_gs)
    want = oq.fake_quantize(x, o_scale, o_zp, oargs, global_scale=o_gs)
    if args.strategy == "tensor_group":
        # the reference's fp4 cast of a NaN is platform dependent: a group that holds one
        # comes out as NaN here, the oracle's choice for the other 15 values is not binding
        bad = torch.isnan(o_scale.float()).repeat_interleave(16, dim=-1)
        want = torch.where(bad, torch.full_like(want, float("nan")), want)

    def canon(t):  # one NaN pattern: which payload a NaN result carries is not part of the contract
        return torch.where(torch.isnan(t.float()).to(t.device), torch.full_like(t, float("nan")), t)

    want, o_scale = canon(want), canon(o_scale)
    res = dynamic_fake_quantize(x.to(gpu), args, gs, return_qparams=True)
    assert (res is not None) == fusable
    if res is not None:
        out, scale, zp = res
        assert_bit_equal(canon(scale), o_scale, "one-pass scale")
        assert_bit_equal(zp, o_zp, "one-pass zp")
        assert_bit_equal(canon(out), want, "one-pass qdq")
        assert_bit_equal(canon(dynamic_fake_quantize(x.to(gpu), args, gs)), want, "one-pass qdq, no qparams")
    routed = forward_quantize(module, x.to(gpu), "input", args)
    if args.strategy == "tensor_group":
        routed = torch.where(bad.to(gpu), torch.full_like(routed, float("nan")), routed)
    assert_bit_equal(canon(routed), want, "forward_quantize")


@pytest.mark.parametrize("spec", [
    dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128),
    dict(num_bits=8, type="int", symmetric=True, strategy="channel"),
    dict(num_bits=8, type="float", symmetric=True, strategy="channel"),
    dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16),
], ids=["int4-group", "int8-channel", "fp8-channel", "nvfp4"])
@pytest.mark.parametrize("with_zp", [False, True], ids=["nozp", "zp"])
def test_float16_results_keep_the_sign_of_zero(spec, with_zp, gpu):
    """small negative values quantize to -0 and must dequantize to -0 in float16 too
    (a multiplication folded into the float16 conversion would give +0)"""
    from compressed_tensors_amd.quantization import dequantize, fake_quantize, quantize

    announce("f16 negative zero", spec, with_zp)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(77)
    w = (torch.randn(64, 512, generator=g) * 0.02).to(torch.float16)
    w[:, ::3] = -w[:, ::3].abs() * 1e-3            # far below half a quantization step
    w[:, 5] = 0.3
    gs = None
    if args.strategy == "tensor_group":
        gs = oq.generate_gparam(*[t.reshape(1) for t in torch.aminmax(w)])
    scale, zp = oq.observe_weight(w, oargs, global_scale=gs)
    if not with_zp:
        zp = None
    dev = lambda t: None if t is None else t.to(gpu)
    want = oq.fake_quantize(w, scale, zp, oargs, global_scale=gs)
    assert (bits_of(want) == -32768).sum() > 100  # the case is there: float16 -0 is 0x8000
    got = fake_quantize(w.to(gpu), dev(scale), dev(zp), args, global_scale=dev(gs))
    assert_bit_equal(got, want, "fake_quantize f16")
    if args.num_bits == 8:
        q = quantize(w.to(gpu), dev(scale), dev(zp), args, dtype=args.pytorch_dtype())
        o_q = oq.quantize(w, scale, zp, oargs, dtype=args.pytorch_dtype())
        assert_bit_equal(q, o_q, "quantize f16")
        assert_bit_equal(dequantize(q, dev(scale), dev(zp), args=args),
                         oq.dequantize(o_q, scale, zp, args=oargs), "dequantize f16")


def test_attn_head_and_errors(gpu):
    from compressed_tensors_amd.quantization import QuantizationArgs, fake_quantize, quantize

    announce("attn_head")
    args = QuantizationArgs(num_bits=8, type="float", strategy="attn_head")
    oargs = oq._Args(num_bits=8, type="float", strategy="attn_head")
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 4, 6, 16, generator=g).bfloat16()
    scale = (x.float().abs().amax(dim=(0, 2, 3), keepdim=False) / 448).bfloat16().reshape(4, 1, 1)
    out = fake_quantize(x.to(gpu), scale.to(gpu), None, args)
    assert_bit_equal(out, oq.fake_quantize(x, scale, None, oargs), "attn_head")
    gargs = QuantizationArgs(num_bits=4, strategy="group", group_size=48)
    with pytest.raises(ValueError, match="divisble"):
        quantize(x.reshape(48, 16).repeat(1, 4).to(gpu), scale.reshape(-1)[:1].to(gpu), None, gargs)
    bargs = QuantizationArgs(num_bits=8, type="float", strategy="block", block_structure=[5, 16])
    with pytest.raises(ValueError, match="block_height"):
        quantize(x.reshape(48, 16).to(gpu), torch.ones(9, 1, dtype=torch.bfloat16, device=gpu), None, bargs)
    with pytest.raises(NotImplementedError):
        quantize(x.to(gpu), scale.to(gpu), None, QuantizationArgs(num_bits=6, type="float", strategy="tensor"))


def test_large_w4a16_properties(gpu):
    """full-size weight (4096 x 4096): sampled-row parity plus size-independent properties"""
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, dequantize, observe_weight_qparams, quantize,
    )

    announce("large w4a16")
    args = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    oargs = oq._Args(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    g = torch.Generator().manual_seed(0)
    w = (torch.randn(4096, 4096, generator=g) * 0.02).bfloat16()
    wg = w.to(gpu)
    scale, zp = observe_weight_qparams(wg, args)
    q = quantize(wg, scale, zp, args, dtype=torch.int8)
    dq = dequantize(q, scale, zp)
    rows = torch.arange(0, 4096, 97)
    o_scale, o_zp = oq.observe_weight(w[rows], oargs)
    assert_bit_equal(scale[rows.to(gpu)], o_scale, "scale rows")
    want_q = oq.quantize(w[rows], o_scale, o_zp, oargs, dtype=torch.int8)
    assert_bit_equal(q[rows.to(gpu)], want_q, "q rows")
    assert_bit_equal(dq[rows.to(gpu)], oq.dequantize(want_q, o_scale, o_zp), "dq rows")
    # idempotence: quantizing the dequantized weight with the same scales gives the same codes
    assert torch.equal(quantize(dq, scale, zp, args, dtype=torch.int8), q)
    assert int(q.min()) >= -8 and int(q.max()) <= 7
    # |w - dq| <= scale/2 plus the bf16 roundings of w/scale and q*scale (each
    # below 2^-8 of 8 code steps) wherever no clamping happened
    err = (wg.float() - dq.float()).abs()
    bound = scale.float().repeat_interleave(128, dim=1) * 0.57 + 1e-12
    assert bool(((err <= bound) | (q == 7) | (q == -8)).all())


def test_fp8_codes_on_every_bf16_pattern(gpu):
    """scale 1: the quantize chain reduces to clamp + cast, so every bf16 bit pattern
    (NaN aside) goes through the fp8 conversion; likewise every fp8 code is decoded"""
    from compressed_tensors_amd.quantization import QuantizationArgs, dequantize, quantize

    announce("fp8 exhaustive")
    args = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="channel")
    oargs = oq._Args(num_bits=8, type="float", symmetric=True, strategy="channel")
    allbits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    x = allbits[~torch.isnan(allbits.float())]
    x = torch.cat([x, x[: (-x.numel()) % 512]]).reshape(-1, 512)
    for s_val in (1.0, 0.5, 3.0, 0.0123):
        scale = torch.full((x.shape[0], 1), s_val, dtype=torch.bfloat16)
        q = quantize(x.to(gpu), scale.to(gpu), None, args, dtype=torch.float8_e4m3fn)
        assert_bit_equal(q, oq.quantize(x, scale, None, oargs, dtype=torch.float8_e4m3fn), f"fp8 codes s={s_val}")
    codes = torch.arange(0, 256, dtype=torch.int32).to(torch.uint8).repeat(16).reshape(8, 512)
    codes = codes[:, [c for c in range(512) if (c % 256) & 0x7F != 0x7F]]  # drop the NaN codes
    codes = codes[:, :504].contiguous().view(torch.float8_e4m3fn)
    scale = torch.full((8, 1), 1.0, dtype=torch.bfloat16)
    dq = dequantize(codes.to(gpu), scale.to(gpu))
    assert_bit_equal(dq, oq.dequantize(codes, scale), "fp8 decode")
    for dt in (torch.float16, torch.float32):
        xs = x.to(dt)
        scale = torch.full((x.shape[0], 1), 0.37, dtype=dt)
        q = quantize(xs.to(gpu), scale.to(gpu), None, args, dtype=torch.float8_e4m3fn)
        assert_bit_equal(q, oq.quantize(xs, scale, None, oargs, dtype=torch.float8_e4m3fn), f"fp8 codes {dt}")


def test_large_fp8_channel_and_token(gpu):
    """full-size fp8 paths: per-channel weight codes and per-token activation QDQ,
    sampled rows against the oracle"""
    from compressed_tensors_amd.quantization import (
        QuantizationArgs, compute_dynamic_scales_and_zp, dequantize, fake_quantize,
        observe_weight_qparams, quantize,
    )

    announce("large fp8")
    g = torch.Generator().manual_seed(1)
    w = torch.randn(14336, 4096, generator=g) * 0.02
    w[torch.rand(w.shape, generator=g) < 0.001] *= 20
    w = w.bfloat16()
    args = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="channel")
    oargs = oq._Args(num_bits=8, type="float", symmetric=True, strategy="channel")
    wg = w.to(gpu)
    scale, zp = observe_weight_qparams(wg, args)
    q = quantize(wg, scale, zp, args, dtype=torch.float8_e4m3fn)
    dq = dequantize(q, scale)
    rows = torch.arange(0, 14336, 211)
    o_scale, o_zp = oq.observe_weight(w[rows], oargs)
    assert_bit_equal(scale[rows.to(gpu)], o_scale, "fp8 scale rows")
    want = oq.quantize(w[rows], o_scale, o_zp, oargs, dtype=torch.float8_e4m3fn)
    assert_bit_equal(q[rows.to(gpu)], want, "fp8 code rows")
    assert_bit_equal(dq[rows.to(gpu)], oq.dequantize(want, o_scale), "fp8 dequant rows")
    assert float(q.float().abs().max()) == 448.0  # every row's extreme value hits the fp8 maximum
    x = torch.randn(1, 8192, 4096, generator=g)
    x[..., torch.rand(4096, generator=g) < 0.005] *= 50
    x = x.bfloat16()
    targs = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="token", dynamic=True)
    toargs = oq._Args(num_bits=8, type="float", symmetric=True, strategy="token")
    xg = x.to(gpu)
    s, z = compute_dynamic_scales_and_zp(xg, targs)
    y = fake_quantize(xg, s, z, targs)
    toks = torch.arange(0, 8192, 301)
    os_, oz_ = oq.compute_dynamic_scales_and_zp(x[:, toks], toargs)
    assert_bit_equal(s[:, toks.to(gpu)], os_, "token scales")
    assert_bit_equal(y[:, toks.to(gpu)], oq.fake_quantize(x[:, toks], os_, oz_, toargs), "token qdq")


def test_quantized_weight_batch_matches_single_calls(gpu):
    """ctmi_qdq_many (chained launches) == one ctmi_qdq per tensor, for a mix of kernel
    instances: fp8 and int8 codes, with and without zero points, channel / group / tensor
    scales, a shape the vectorised kernels do not take, and more than 8 tensors of a kind."""
    from compressed_tensors_amd.compressors import QuantizedWeightBatch
    from compressed_tensors_amd.quantization import (QuantizationArgs, dequantize,
                                                     observe_weight_qparams, quantize)

    announce("qdq_many")
    g = torch.Generator().manual_seed(11)
    specs = [dict(num_bits=8, type="float", symmetric=True, strategy="channel")] * 11 + [
        dict(num_bits=8, type="int", symmetric=False, strategy="group", group_size=32),
        dict(num_bits=8, type="int", symmetric=True, strategy="tensor"),
        dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128),
        dict(num_bits=8, type="int", symmetric=False, strategy="channel"),
    ]
    shapes = [(64, 256), (8, 4096), (33, 128), (1, 8), (128, 1024), (5, 72), (16, 16), (256, 256),
              (3, 4104), (40, 640), (7, 56), (48, 96), (20, 200), (12, 384), (9, 30)]
    entries = []
    for spec, shape in zip(specs, shapes):
        args = QuantizationArgs(**spec)
        w = (torch.randn(shape, generator=g) * 0.05).bfloat16().to(gpu)
        scale, zp = observe_weight_qparams(w, args)
        entries.append(dict(weight=w, scale=scale, zero_point=zp, quantization_args=args))
    batch = QuantizedWeightBatch(entries)
    codes = batch.compress()
    dense = batch.decompress()
    for e, c, d in zip(entries, codes, dense):
        args = e["quantization_args"]
        want = quantize(e["weight"], e["scale"], e["zero_point"], args, dtype=args.pytorch_dtype())
        assert c.dtype == want.dtype and torch.equal(c.view(torch.int8), want.view(torch.int8))
        back = dequantize(want, e["scale"], None if args.symmetric else e["zero_point"])
        assert d.dtype == back.dtype and torch.equal(d.view(torch.int16), back.view(torch.int16))


MANY_OBS = [
    dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128),
    dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=32),
    dict(num_bits=8, type="float", symmetric=True, strategy="channel"),
    dict(num_bits=8, type="int", symmetric=False, strategy="channel"),
    dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16),
    dict(num_bits=8, type="int", symmetric=True, strategy="tensor"),
]


@pytest.mark.parametrize("spec", MANY_OBS, ids=[f"{s['type']}{s['num_bits']}-{s['strategy']}" for s in MANY_OBS])
def test_observer_for_many_weights_in_one_call(spec, gpu):
    """ctmi_observe_qparams_many (8 weights per launch) against the oracle's observer and
    against one call per weight: mixed shapes and dtypes in one list, more than 8 weights of
    a kind, rows longer than one wave covers, shapes no vectorised kernel takes, NaN and
    infinite elements, and (fp4) global scales."""
    from compressed_tensors_amd.quantization import observe_weight_qparams, observe_weights_qparams

    announce("observe_many", spec)
    args, oargs = _pair(spec)
    shapes = [(64, 512), (8, 4096), (33, 128), (16, 14336), (128, 1024), (5, 96), (16, 16), (256, 256),
              (3, 4128), (40, 640), (7, 48), (48, 96), (24, 8192), (12, 384), (9, 32), (4, 1024),
              (2, 4096), (64, 64), (1, 16), (32, 2048)]
    if spec.get("group_size", 16) > 16:
        shapes = [(r, -(-c // spec["group_size"]) * spec["group_size"]) for r, c in shapes]
    dtypes = [torch.bfloat16, torch.bfloat16, torch.float16, torch.bfloat16, torch.float32]
    ws, gss = [], []
    for i, shape in enumerate(shapes):
        w = _weights(shape, dtypes[i % len(dtypes)], seed=100 + i)
        if i == 5:  # (no global scale for this one)
            w[2, 40] = float("inf")
        if i == 7:  # (what a NaN becomes is compared with the single call only)
            w[3, 17] = float("nan")
        ws.append(w)
        gss.append(None)
        if spec["strategy"] == "tensor_group" and i % 3 != 2:
            gss[-1] = oq.generate_gparam(*torch.aminmax(ws[i if i != 7 else 0]))
    wg = [w.to(gpu) for w in ws]
    gg = [None if g is None else g.to(gpu) for g in gss]
    got = observe_weights_qparams(wg, args, global_scales=gg if any(g is not None for g in gg) else None)
    assert len(got) == len(ws)
    for i, (w, gs, (scale, zp)) in enumerate(zip(ws, gss, got)):
        if i != 7:
            o_scale, o_zp = oq.observe_weight(w, oargs, global_scale=gs)
            assert_bit_equal(scale, o_scale, f"scale {i} {tuple(w.shape)} {w.dtype}")
            assert_bit_equal(zp, o_zp, f"zero_point {i} {tuple(w.shape)} {w.dtype}")
        one_s, one_z = observe_weight_qparams(wg[i], args, global_scale=gg[i])
        assert one_s.dtype == scale.dtype and one_s.shape == scale.shape and one_z.dtype == zp.dtype
        assert torch.equal(one_s.view(torch.uint8), scale.view(torch.uint8))
        assert torch.equal(one_z.view(torch.uint8), zp.view(torch.uint8))
    assert observe_weights_qparams([], args) == []


def test_mxfp4_scale_helpers_on_every_input(gpu):
    """round_to_power_2 and generate_mxfp4_scales on all 65 536 bfloat16 patterns,
    convert_mxfp4_exp_scale on all 256 exponents, against the oracle"""
    from compressed_tensors_amd.quantization import (
        convert_mxfp4_exp_scale, generate_mxfp4_scales, round_to_power_2,
    )
    from oracle import mxfp4 as om

    announce("mxfp4 scales")
    x = torch.arange(65536, dtype=torch.int32).to(torch.uint16).view(torch.bfloat16).reshape(256, 256)
    assert_bit_equal(round_to_power_2(x.to(gpu)), om.round_to_power_2(x), "round_to_power_2")
    got = generate_mxfp4_scales(x.to(gpu)).cpu()
    want = om.generate_mxfp4_scales(x)
    # a group maximum is never negative; for negative, infinite and NaN inputs the
    # reference casts a NaN / infinity to int32, which the language leaves undefined
    defined = (x.view(torch.int16) >= 0) & torch.isfinite(x.float()) \
        & torch.isfinite(om.round_to_power_2(x).float())
    assert torch.equal(got[defined], want[defined])
    assert int(defined.sum()) > 32000
    e = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        assert_bit_equal(convert_mxfp4_exp_scale(e.to(gpu), dtype), om.convert_mxfp4_exp_scale(e, dtype),
                         f"convert {dtype}")
    assert convert_mxfp4_exp_scale(e[:0].to(gpu)).shape == (0,)
    with pytest.raises(AssertionError):
        round_to_power_2(torch.zeros(4, device=gpu))


@pytest.mark.parametrize("cols,group_size", [(128, 32), (4096, 128), (1000, 8), (14336, 128), (40, 7)])
def test_column_groups_from_g_idx(cols, group_size, gpu):
    """g_idx -> group of every column: the place of the column in a stable sort by g_idx,
    cut into runs of group_size; also with uneven group populations, and unset (-1)"""
    from compressed_tensors_amd.quantization.forward import _column_groups

    announce("column groups", cols, group_size)
    g = torch.Generator().manual_seed(cols)
    even = (torch.randperm(cols, generator=g) // group_size).to(torch.int32)
    uneven = torch.randint(0, max(cols // group_size, 1), (cols,), generator=g, dtype=torch.int32)
    for g_idx in (even, uneven, torch.arange(cols, dtype=torch.int32) // group_size):
        want = (torch.argsort(torch.argsort(g_idx, stable=True), stable=True) // group_size).to(torch.int32)
        assert_bit_equal(_column_groups(g_idx.to(gpu), group_size), want, "col_group")
        assert_bit_equal(_column_groups(g_idx.to(torch.int64).to(gpu), group_size), want, "int64 g_idx")
    unset = even.clone()
    unset[cols // 2] = -1
    assert_bit_equal(_column_groups(unset.to(gpu), group_size),
                     (torch.arange(cols) // group_size).to(torch.int32), "unset g_idx")
    assert _column_groups(None, group_size) is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_generate_gparam_on_many_values(dtype, gpu):
    """448 * 6 / max|x| as torch evaluates it (reciprocal, then product, each rounded to
    the dtype of min / max): every positive bfloat16 / float16 pattern, a random draw of
    float32 values, on either side of zero"""
    from compressed_tensors_amd import _lib
    from compressed_tensors_amd.quantization import generate_gparam

    announce("generate_gparam", dtype)
    if dtype == torch.float32:
        g = torch.Generator().manual_seed(1)
        v = torch.cat([torch.rand(50000, generator=g) * 4, torch.randn(50000, generator=g).abs() * 1e-3,
                       torch.tensor([0.0, 1e-30, 3e38, float("inf")])])
    else:
        v = torch.arange(0, 0x7c01 if dtype == torch.float16 else 0x7f81, dtype=torch.int32) \
            .to(torch.int16).view(dtype).clone()
    lib = _lib.load()
    for mn, mx in ((torch.zeros_like(v), v), (-v, v / 2), (v / 4, v)):
        # the elementwise arithmetic on all values at once, through the C ABI
        a, b = mn.to(gpu), mx.to(gpu)
        out = torch.empty(v.numel(), dtype=torch.float32, device=gpu)
        _lib.check(lib.ctmi_generate_gparam(a.data_ptr(), b.data_ptr(), _lib.dtype_code(dtype), v.numel(),
                                            out.data_ptr(), _lib.stream_of(gpu)))
        zero = torch.zeros_like(mn)
        m = torch.max(torch.abs(torch.min(mn, zero)), torch.abs(torch.max(mx, zero)))
        assert_bit_equal(out, (448.0 * 6.0 / m).to(torch.float32), "generate_gparam (all values)")
        # and the wrapper against the oracle, one value per call as the reference uses it
        for i in range(1, v.numel(), v.numel() // 7):
            assert_bit_equal(generate_gparam(a[i:i + 1], b[i:i + 1]),
                             oq.generate_gparam(mn[i:i + 1], mx[i:i + 1]), f"generate_gparam [{i}]")


QP_SPECS = [
    dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128),
    dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=128),
    dict(num_bits=8, type="int", symmetric=True, strategy="channel"),
    dict(num_bits=8, type="int", symmetric=False, strategy="channel"),
    dict(num_bits=8, type="float", symmetric=True, strategy="channel"),
    dict(num_bits=8, type="float", symmetric=False, strategy="channel"),
    dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16),
    dict(num_bits=2, type="int", symmetric=False, strategy="channel"),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "f16", "f32"])
@pytest.mark.parametrize("spec", QP_SPECS, ids=[f"{s['type']}{s['num_bits']}-{'sym' if s['symmetric'] else 'asym'}" for s in QP_SPECS])
def test_calculate_qparams_on_many_pairs(spec, dtype, gpu):
    """calculate_qparams on 200 000 (min, max) pairs per scheme and dtype: magnitudes from
    1e-9 to 1e4, one-sided ranges, exact zeros, equal ends, infinities and NaNs"""
    from compressed_tensors_amd.quantization import calculate_qparams

    announce("calculate_qparams many", spec, dtype)
    args, oargs = _pair(spec)
    g = torch.Generator().manual_seed(17)
    n = 200_000
    mag = 10.0 ** (torch.rand(n, generator=g) * 13 - 9)
    lo = -mag * torch.rand(n, generator=g)
    hi = mag * torch.rand(n, generator=g)
    kind = torch.randint(0, 8, (n,), generator=g)
    lo = torch.where(kind == 0, hi * 0.5, lo)          # all positive
    hi = torch.where(kind == 1, lo * 0.5, hi)          # all negative
    lo = torch.where(kind == 2, torch.zeros(n), lo)
    hi = torch.where(kind == 3, lo, hi)                # equal ends
    special = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 1e-45, 65504.0, 3e38])
    lo[:8], hi[:8] = special, special.flip(0)
    lo[8:16], hi[8:16] = -special.abs(), special.abs()
    lo, hi = torch.minimum(lo, hi).to(dtype), torch.maximum(lo, hi).to(dtype)
    lo[4], hi[11] = float("nan"), float("nan")
    gs = o_gs = None
    if spec["strategy"] == "tensor_group":
        o_gs = torch.tensor([37.5], dtype=torch.float32)
        gs = o_gs.to(gpu)
    o_scale, o_zp = oq.calculate_qparams(lo, hi, oargs, global_scale=o_gs)
    scale, zp = calculate_qparams(lo.to(gpu), hi.to(gpu), args, global_scale=gs)
    nan = torch.isnan(o_scale.float())
    assert torch.equal(torch.isnan(scale.float()).cpu(), nan)
    assert_bit_equal(torch.where(nan.to(gpu), torch.zeros_like(scale.float()), scale.float()),
                     torch.where(nan, torch.zeros_like(o_scale.float()), o_scale.float()), "scale")
    assert scale.dtype == o_scale.dtype and zp.dtype == o_zp.dtype
    # where the scale is NaN, or an end is infinite (inf / inf), the zero point is a cast
    # of a NaN to int8 or fp8: not defined / sign and payload not part of the contract
    ok = ~nan & torch.isfinite(lo.float()) & torch.isfinite(hi.float())
    assert torch.equal(zp.cpu().view(torch.uint8 if zp.element_size() == 1 else zp.dtype)[ok],
                       o_zp.view(torch.uint8 if o_zp.element_size() == 1 else o_zp.dtype)[ok]), "zero points"


@pytest.mark.parametrize("xdt,sdt", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                     (torch.bfloat16, torch.float32), (torch.float16, torch.bfloat16)],
                         ids=["bf16", "f16", "bf16-f32scale", "f16-bf16scale"])
@pytest.mark.parametrize("bits,symmetric", [(4, True), (4, False), (8, True), (8, False)])
def test_int_codes_on_every_16_bit_pattern(bits, symmetric, xdt, sdt, gpu):
    """all 65 536 patterns of a 16-bit float as inputs, one row of 128 per scale, 512
    scales from 1e-12 to 1e6 (and the clamp floor, and powers of two), random zero
    points: quantize, fake_quantize, pack-quantized compress and decompress against the
    oracle (NaN inputs have no defined integer code and are left out of the code checks)"""
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.quantization import fake_quantize, quantize

    announce("every 16-bit pattern", bits, symmetric, xdt, sdt)
    spec = dict(num_bits=bits, type="int", symmetric=symmetric, strategy="group", group_size=128)
    args, oargs = _pair(spec)
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(xdt).reshape(512, 128).clone()
    g = torch.Generator().manual_seed(bits * 2 + symmetric)
    scale = (10.0 ** (torch.rand(512, 1, generator=g) * 18 - 12))
    scale[:4, 0] = torch.tensor([1.1920928955078125e-07, 1.0, 0.5, 2.0 ** -20])
    scale = scale.to(sdt)
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    zp = None if symmetric else torch.randint(lo, hi + 1, (512, 1), generator=g).to(torch.int8)
    dev = lambda t: None if t is None else t.to(gpu)
    finite_code = ~torch.isnan(x.float())
    want_q = oq.quantize(x, scale, zp, oargs, dtype=torch.int8)
    got_q = quantize(x.to(gpu), dev(scale), dev(zp), args, dtype=torch.int8).cpu()
    assert torch.equal(got_q[finite_code], want_q[finite_code]), "quantize"
    want_fq = oq.fake_quantize(x, scale, zp, oargs)
    got_fq = fake_quantize(x.to(gpu), dev(scale), dev(zp), args).cpu()
    nan = torch.isnan(want_fq.float())
    assert torch.equal(torch.isnan(got_fq.float()), nan), "fake_quantize NaNs"
    assert torch.equal(bits_of(got_fq)[~nan], bits_of(want_fq)[~nan]), "fake_quantize"
    comp = BaseCompressor.load_from_registry("pack-quantized")
    want_c = op.pack_quantized_compress(x, scale, oargs, zero_point=zp)
    got_c = comp.compress_weight(weight=x.to(gpu), scale=dev(scale), quantization_args=args, zero_point=dev(zp))
    from oracle.pack import unpack_from_int32 as o_unpack
    gc = o_unpack(got_c["weight_packed"].cpu(), bits, torch.Size((512, 128)))
    wc = o_unpack(want_c["weight_packed"], bits, torch.Size((512, 128)))
    assert torch.equal(gc[finite_code], wc[finite_code]), "packed codes"
    data = dict(want_c, weight_scale=scale)
    want_d = op.pack_quantized_decompress(dict(data), oargs)
    got_d = comp.decompress_weight({k: v.to(gpu) for k, v in data.items()}, quantization_args=args)
    assert_bit_equal(got_d, want_d, "decompress")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_scales_computed_in_kernels_for_every_maximum(dtype, gpu):
    """the kernels that derive scales themselves (one-shot compression, dynamic
    quantization) against calculate_qparams for every finite positive 16-bit value as the
    group maximum: max / 7.5, / 127.5, / 448 and / 6 (the bf16 paths multiply by a reciprocal)"""
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.quantization.helpers import dynamic_fake_quantize

    announce("in-kernel scales, every maximum", dtype)
    top = 0x7f80 if dtype == torch.bfloat16 else 0x7c00
    m = torch.arange(1, top, dtype=torch.int32).to(torch.int16).view(dtype)
    rows = m.numel()
    x = torch.zeros(rows, 128, dtype=dtype)
    x[:, 5] = m
    x[::2, 5] = -m[::2]          # the maximum on either side
    x[:, 77] = (m.float() * 0.37).to(dtype)
    xg = x.to(gpu)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    for bits in (4, 8):
        spec = dict(num_bits=bits, type="int", symmetric=True, strategy="group", group_size=128)
        args, oargs = _pair(spec)
        o_scale, _ = oq.observe_weight(x, oargs)
        got = comp.observe_and_compress_weight(xg, args)
        assert_bit_equal(got["weight_scale"], o_scale, f"one-shot int{bits} scales")
        want = op.pack_quantized_compress(x, o_scale, oargs)
        assert_bit_equal(got["weight_packed"], want["weight_packed"], f"one-shot int{bits} codes")
    for spec in (dict(num_bits=8, type="float", symmetric=True, strategy="group", group_size=128, dynamic=True),
                 dict(num_bits=8, type="int", symmetric=True, strategy="group", group_size=128, dynamic=True)):
        args, oargs = _pair(spec)
        o_scale, o_zp = oq.compute_dynamic_scales_and_zp(x, oargs)
        out, scale, zp = dynamic_fake_quantize(xg, args, None, return_qparams=True)
        assert_bit_equal(scale, o_scale, f"dynamic {spec['type']}8 scales")
        assert_bit_equal(out, oq.fake_quantize(x, o_scale, o_zp, oargs), f"dynamic {spec['type']}8 qdq")
    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16, dynamic="local")
    args, oargs = _pair(spec)
    for gs_value in (1.0, 37.5, 2688.0 / 3.0):
        o_gs = torch.tensor([gs_value], dtype=torch.float32)
        o_scale, o_zp = oq.compute_dynamic_scales_and_zp(x, oargs, global_scale=o_gs)
        out, scale, zp = dynamic_fake_quantize(xg, args, o_gs.to(gpu), return_qparams=True)
        assert_bit_equal(scale, o_scale, f"dynamic nvfp4 scales, gs {gs_value}")
        assert_bit_equal(out, oq.fake_quantize(x, o_scale, o_zp, oargs, global_scale=o_gs),
                         f"dynamic nvfp4 qdq, gs {gs_value}")


QG = [
    (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128), (64, 1024), torch.bfloat16),
    (dict(num_bits=8, type="int", symmetric=False, strategy="group", group_size=64), (33, 4096), torch.bfloat16),
    (dict(num_bits=8, type="float", symmetric=True, strategy="group", group_size=32), (19, 512), torch.float16),
    (dict(num_bits=8, type="float", symmetric=False, strategy="group", group_size=128), (9, 2048), torch.bfloat16),
    (dict(num_bits=4, type="int", symmetric=False, strategy="group", group_size=8), (13, 2056), torch.float32),
    (dict(num_bits=8, type="int", symmetric=True, strategy="group", group_size=16), (3, 20480), torch.bfloat16),
]


@pytest.mark.parametrize("spec,shape,dtype", QG, ids=[f"qg{i}" for i in range(len(QG))])
def test_quantize_dequantize_with_activation_ordering(spec, shape, dtype, gpu):
    """quantize, dequantize and fake_quantize with a g_idx per column (the streaming
    kernels gather every element's scale and zero point) against the oracle"""
    from compressed_tensors_amd.quantization import dequantize, fake_quantize, quantize

    announce("qdq g_idx", spec, shape, dtype)
    args, oargs = _pair(spec)
    rows, cols = shape
    g = torch.Generator().manual_seed(rows)
    w = (torch.randn(shape, generator=g) * 0.02).to(dtype)
    w.view(-1)[:3] = torch.tensor([0.0, -0.0, -1e-6]).to(dtype)
    g_idx = (torch.randperm(cols, generator=g) // spec["group_size"]).to(torch.int32)
    scale, zp = oq.observe_weight(w.index_select(-1, torch.argsort(g_idx)), oargs)
    zp_arg = None if spec["symmetric"] else zp
    dev = lambda t: None if t is None else t.to(gpu)
    code_dtype = torch.int8 if spec["type"] == "int" else torch.float8_e4m3fn
    want_q = oq.quantize(w, scale, zp_arg, oargs, dtype=code_dtype, g_idx=g_idx)
    got_q = quantize(w.to(gpu), dev(scale), dev(zp_arg), args, dtype=code_dtype, g_idx=dev(g_idx))
    assert_bit_equal(got_q, want_q, "quantize")
    assert_bit_equal(dequantize(got_q, dev(scale), dev(zp_arg), args=args, g_idx=dev(g_idx)),
                     oq.dequantize(want_q, scale, zp_arg, args=oargs, g_idx=g_idx), "dequantize")
    assert_bit_equal(fake_quantize(w.to(gpu), dev(scale), dev(zp_arg), args, g_idx=dev(g_idx)),
                     oq.fake_quantize(w, scale, zp_arg, oargs, g_idx=g_idx), "fake_quantize")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "f16", "f32"])
@pytest.mark.parametrize("kind,num_bits", [("int", 8), ("float", 8), ("float", 4)])
def test_round_to_quantized_type_on_every_pattern(kind, num_bits, dtype, gpu):
    """A8 on its own (quant_args.py:384-408): all 65 536 patterns of a 16-bit float (for
    float32: those of bfloat16 widened, ties and near-ties of every grid added) through
    round_to_quantized_type, against the oracle, bit for bit; NaNs where the oracle has NaNs"""
    from compressed_tensors_amd.quantization import FP4_E2M1_DATA, round_to_quantized_type

    announce("round_to_quantized_type", kind, num_bits, dtype)
    args, oargs = _pair(dict(num_bits=num_bits, type=kind, symmetric=True, strategy="tensor"))
    if dtype == torch.float32:
        x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()
        ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 0.5, 1.5, 2.5, 3.5, 447.0, 448.0, 464.0,
                             465.0, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -9, 17.0, 18.0, 19.0, 0.0])
        near = torch.cat([ties, torch.nextafter(ties, torch.tensor(1e9)), torch.nextafter(ties, torch.tensor(-1e9))])
        x = torch.cat([x, near, -near, torch.randn(4099, generator=torch.Generator().manual_seed(1)) * 100])
    else:
        x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype).clone()
    x = torch.cat([x, x[:5]])  # a length that is no multiple of the kernel's vector
    want = oq.round_to_quantized_type(x.clone(), oargs)
    got = round_to_quantized_type(x.to(gpu), args)
    assert got.dtype == dtype and got.shape == x.shape and got.is_cuda
    got = got.cpu()
    nan = torch.isnan(want.float())
    assert torch.equal(torch.isnan(got.float()), nan), "NaNs"
    assert torch.equal(bits_of(got)[~nan], bits_of(want)[~nan])
    if kind == "float" and num_bits == 4:
        again = FP4_E2M1_DATA.cast_to_fp4(x.to(gpu)).cpu()
        assert torch.equal(bits_of(again)[~nan], bits_of(want)[~nan])
    # a view that starts in the middle of a buffer
    assert_bit_equal(round_to_quantized_type(x.to(gpu)[3:1000], args).cpu().nan_to_num(0.0),
                     want[3:1000].nan_to_num(0.0), "offset view")
    # a 2-d view that is not contiguous
    m = x[:65536].reshape(256, 256).t()
    assert_bit_equal(round_to_quantized_type(m.to(gpu), args).cpu().nan_to_num(0.0),
                     oq.round_to_quantized_type(m.clone(), oargs).nan_to_num(0.0), "transposed")


def test_round_to_quantized_type_refuses_what_the_reference_refuses(gpu):
    from compressed_tensors_amd.quantization import QuantizationArgs, round_to_quantized_type

    x = torch.zeros(8, device=gpu)
    args = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="tensor")
    args.num_bits = 6
    with pytest.raises(NotImplementedError, match="Only num_bits in"):
        round_to_quantized_type(x, args)
    args.type = "complex"
    with pytest.raises(ValueError, match="Invalid quantization type"):
        round_to_quantized_type(x, args)
