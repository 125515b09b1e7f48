"""GPU parity at the sizes of the benchmark configurations: one Llama-3-8B layer (the
seven real weight shapes) through every multi-weight path, nvfp4 weights and
activations, Hadamard rotations of weights and the fused rotate + quantize + pack.

Rows of a weight are independent in every format here (groups and blocks lie inside a
row), so the oracle runs on row slices: the first rows, rows in the middle, and the last
rows of EVERY tensor (the last chunk of a tensor is the bounds-checked one, and in a
chained launch the first rows of tensor i + 1 follow the last rows of tensor i).  The
multi-weight outputs are also compared, whole, with the single-weight entry points on
the GPU."""
import pytest
import torch

from gpu_util import announce, assert_bit_equal
from oracle import hadamard as oh
from oracle import pack as op
from oracle import quant as oq

pytestmark = pytest.mark.gpu

LLAMA_LAYER = [("q_proj", 4096, 4096), ("k_proj", 1024, 4096), ("v_proj", 1024, 4096),
               ("o_proj", 4096, 4096), ("gate_proj", 14336, 4096), ("up_proj", 14336, 4096),
               ("down_proj", 4096, 14336)]
SLICE = 24


def _slices(rows):
    """row slices the oracle runs on: head, two in the middle (one not aligned to
    anything), tail"""
    mid = rows // 2
    odd = (rows * 5) // 7 + 3
    return [slice(0, SLICE), slice(mid - SLICE // 2, mid + SLICE // 2),
            slice(odd, min(odd + SLICE, rows)), slice(rows - SLICE, rows)]


def _layer(gpu, seed, outliers=False):
    """the seven weights of one layer, N(0, 0.02) bf16, generated on the GPU"""
    g = torch.Generator(device=gpu).manual_seed(seed)
    out = []
    for name, r, c in LLAMA_LAYER:
        w = torch.randn(r, c, generator=g, device=gpu) * 0.02
        if outliers:  # 0.1 % of the entries 20 times larger
            w = torch.where(torch.rand(r, c, generator=g, device=gpu) < 1e-3, w * 20, w)
        out.append((name, w.bfloat16()))
    return out


def test_llama_layer_pack_quantized_batches(gpu):
    """W4A16 g128: PackedWeightBatch (precomputed scales) and ObservedWeightBatch (one
    pass) on the real shapes"""
    from compressed_tensors_amd.compressors import (
        BaseCompressor, ObservedWeightBatch, PackedWeightBatch,
    )
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams

    spec = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    layer = _layer(gpu, 1)
    entries = []
    for name, w in layer:
        scale, zp = observe_weight_qparams(w, args)
        entries.append(dict(name=name, weight=w, scale=scale, zero_point=zp, quantization_args=args))
    batch = PackedWeightBatch(entries)
    assert batch._dense is None  # nothing dense is held until decompress() is asked for
    packed = batch.compress()
    dense = batch.decompress()
    one_shot = ObservedWeightBatch([dict(weight=w, quantization_args=args) for _, w in layer]).compress()
    comp = BaseCompressor.load_from_registry("pack-quantized")
    for i, (name, w) in enumerate(layer):
        announce("llama layer w4a16", name, tuple(w.shape))
        e = entries[i]
        single = comp.compress_weight(weight=w, scale=e["scale"], zero_point=e["zero_point"],
                                      quantization_args=args)["weight_packed"]
        assert torch.equal(packed[i], single), f"{name}: batch vs single call (packed)"
        back = comp.decompress_weight({"weight_packed": single, "weight_scale": e["scale"],
                                       "weight_shape": torch.tensor(w.shape)}, quantization_args=args)
        assert torch.equal(dense[i].view(torch.int16), back.view(torch.int16)), f"{name}: dense"
        assert torch.equal(one_shot[i]["weight_packed"], single), f"{name}: one-pass packed"
        assert torch.equal(one_shot[i]["weight_scale"].view(torch.int16), e["scale"].view(torch.int16))
        for sl in _slices(w.shape[0]):
            wc = w[sl].cpu()
            o_scale, o_zp = oq.observe_weight(wc, oargs)
            assert_bit_equal(e["scale"][sl], o_scale, f"{name} scales {sl}")
            want = op.pack_quantized_compress(wc, o_scale, oargs, zero_point=o_zp)
            assert_bit_equal(packed[i][sl], want["weight_packed"], f"{name} packed {sl}")
            assert_bit_equal(one_shot[i]["weight_packed"][sl], want["weight_packed"], f"{name} one-pass {sl}")
            o_dense = op.pack_quantized_decompress(dict(want, weight_scale=o_scale), oargs)
            assert_bit_equal(dense[i][sl], o_dense, f"{name} dense {sl}")


def test_headline_batch_of_224_weights(gpu):
    """The benchmark's headline configuration as bench.py builds it: the 224 weights of a
    Llama-3-8B-shaped model in one PackedWeightBatch (28 chained launches of 8 per direction;
    compress sees the observer's zero points, decompress does not).  Against the oracle: the
    first and last rows of the tensors on both sides of launch boundaries (entries 7 | 8,
    15 | 16, 111 | 112, the last launch 216 ... 223), and one whole 4096 x 4096 tensor, every
    row, in both directions."""
    from compressed_tensors_amd.compressors import PackedWeightBatch
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams

    announce("headline batch, 224 weights")
    spec = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    g = torch.Generator(device=gpu).manual_seed(0)
    entries = []
    for layer in range(32):
        for name, r, c in LLAMA_LAYER:
            w = (torch.randn(r, c, generator=g, device=gpu) * 0.02).to(torch.bfloat16)
            scale, zp = observe_weight_qparams(w, args)
            entries.append(dict(name=f"layers.{layer}.{name}", weight=w, scale=scale, zero_point=zp,
                                quantization_args=args))
    batch = PackedWeightBatch(entries, decompress_zero_points=False)
    assert batch.launches(compress=True) == 28 and batch.launches(compress=False) == 28
    packed = batch.compress()
    dense = batch.decompress()
    torch.cuda.synchronize()

    def check(t, rows):
        e = entries[t]
        wc, sc, zc = (e[k][rows].cpu() for k in ("weight", "scale", "zero_point"))
        o_scale, o_zp = oq.observe_weight(wc, oargs)
        assert_bit_equal(sc, o_scale, f"{e['name']} scales {rows}")
        want = op.pack_quantized_compress(wc, o_scale, oargs, zero_point=o_zp)
        assert_bit_equal(packed[t][rows], want["weight_packed"], f"{e['name']} packed {rows}")
        o_dense = op.pack_quantized_decompress(dict(want, weight_scale=o_scale), oargs)
        assert_bit_equal(dense[t][rows], o_dense, f"{e['name']} dense {rows}")

    for t in (0, 7, 8, 15, 16, 111, 112, 215, 216, 223):
        n_rows = entries[t]["weight"].shape[0]
        announce("headline batch: entry", t, entries[t]["name"])
        check(t, slice(0, SLICE))
        check(t, slice(n_rows - SLICE, n_rows))
    whole = next(t for t in range(8, 224) if entries[t]["weight"].shape == (4096, 4096))  # not in the first launch
    announce("headline batch: all rows of entry", whole)
    check(whole, slice(0, 4096))


@pytest.mark.parametrize("shape", [(14336, 4096), (4096, 14336)], ids=["14336x4096", "4096x14336"])
def test_one_pass_with_activation_ordering_at_full_size(shape, gpu):
    """W4A16 g128 with a random g_idx on the two largest shapes of the set (every workgroup of
    the one-pass kernel takes several row blocks): scales and packed words against the oracle's
    observer on the columns sorted by g_idx and its compressor, on row slices"""
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.quantization import QuantizationArgs

    announce("one-pass act-order", shape)
    spec = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    g = torch.Generator(device=gpu).manual_seed(5)
    w = (torch.randn(shape, generator=g, device=gpu) * 0.02).bfloat16()
    g_idx = (torch.randperm(shape[1], generator=torch.Generator().manual_seed(6)) // 128).to(torch.int32)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    assert comp.one_pass_kernel(w, args, g_idx.to(gpu)) == "table"
    got = comp.observe_and_compress_weight(w, args, g_idx=g_idx.to(gpu))
    order = torch.argsort(g_idx.long(), stable=True)
    for sl in _slices(shape[0]):
        wc = w[sl].cpu()
        o_scale, o_zp = oq.observe_weight(wc.index_select(1, order), oargs)
        want = op.pack_quantized_compress(wc, o_scale, oargs, zero_point=o_zp, g_idx=g_idx)
        assert_bit_equal(got["weight_scale"][sl], o_scale, f"scales {sl}")
        assert_bit_equal(got["weight_packed"][sl], want["weight_packed"], f"packed {sl}")


def test_llama_layer_fp8_batch(gpu):
    """fp8 e4m3 per-channel (the W8A8 weight set, with outliers): QuantizedWeightBatch and
    the one-pass observer + quantizer on the real shapes"""
    from compressed_tensors_amd.compressors import BaseCompressor, QuantizedWeightBatch
    from compressed_tensors_amd.compressors.naive_quantized import observe_and_compress_weights
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams

    spec = dict(num_bits=8, type="float", symmetric=True, strategy="channel")
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    layer = _layer(gpu, 2, outliers=True)
    entries = []
    for name, w in layer:
        scale, zp = observe_weight_qparams(w, args)
        entries.append(dict(weight=w, scale=scale, zero_point=zp, quantization_args=args))
    batch = QuantizedWeightBatch(entries)
    codes = batch.compress()
    dense = batch.decompress()
    one_shot = observe_and_compress_weights([w for _, w in layer], args)
    comp = BaseCompressor.load_from_registry("float-quantized")
    for i, (name, w) in enumerate(layer):
        announce("llama layer fp8", name, tuple(w.shape))
        e = entries[i]
        single = comp.compress_weight(weight=w, scale=e["scale"], zero_point=e["zero_point"],
                                      quantization_args=args)["weight"]
        assert torch.equal(codes[i].view(torch.uint8), single.view(torch.uint8)), f"{name}: codes"
        assert torch.equal(one_shot[i]["weight"].view(torch.uint8), single.view(torch.uint8))
        assert torch.equal(one_shot[i]["weight_scale"].view(torch.int16), e["scale"].view(torch.int16))
        for sl in _slices(w.shape[0]):
            wc = w[sl].cpu()
            o_scale, o_zp = oq.observe_weight(wc, oargs)
            assert_bit_equal(e["scale"][sl], o_scale, f"{name} scales {sl}")
            want = op.naive_compress(wc, o_scale, oargs, zero_point=o_zp)
            assert_bit_equal(codes[i][sl], want, f"{name} codes {sl}")
            o_dense = op.naive_decompress(dict(weight=want, weight_scale=o_scale))
            assert_bit_equal(dense[i][sl], o_dense, f"{name} dense {sl}")


def _nvfp4_scales(w, args, gpu):
    from compressed_tensors_amd.quantization import generate_gparam, observe_weight_qparams

    mn, mx = torch.aminmax(w)
    gs = generate_gparam(mn.reshape(1), mx.reshape(1))
    scale, zp = observe_weight_qparams(w, args, global_scale=gs)
    return gs, scale, zp


def test_llama_layer_nvfp4_batch(gpu):
    """nvfp4 g16: Fp4WeightBatch on the real shapes, 14336 x 4096 and 4096 x 14336
    included, the single-weight compressor and the one-pass observer + compressor"""
    from compressed_tensors_amd.compressors import BaseCompressor, Fp4WeightBatch
    from compressed_tensors_amd.quantization import QuantizationArgs

    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    layer = _layer(gpu, 3)
    entries = []
    for name, w in layer:
        gs, scale, zp = _nvfp4_scales(w, args, gpu)
        entries.append(dict(weight=w, scale=scale, global_scale=gs, quantization_args=args))
    batch = Fp4WeightBatch(entries)
    packed = batch.compress()
    dense = batch.decompress()
    comp = BaseCompressor.load_from_registry("nvfp4-pack-quantized")
    for i, (name, w) in enumerate(layer):
        announce("llama layer nvfp4", name, tuple(w.shape))
        e = entries[i]
        single = comp.compress_weight(weight=w, scale=e["scale"], global_scale=e["global_scale"],
                                      quantization_args=args)["weight_packed"]
        assert torch.equal(packed[i], single), f"{name}: batch vs single call (packed)"
        back = comp.decompress_weight({"weight_packed": single, "weight_scale": e["scale"],
                                       "weight_global_scale": e["global_scale"]})
        assert torch.equal(dense[i].view(torch.int16), back.view(torch.int16)), f"{name}: dense"
        fused = comp.observe_and_compress_weight(w, args, global_scale=e["global_scale"])
        assert torch.equal(fused["weight_packed"], single), f"{name}: one-pass packed"
        assert torch.equal(fused["weight_scale"].view(torch.uint8), e["scale"].view(torch.uint8))
        mn, mx = torch.aminmax(w)
        o_gs = oq.generate_gparam(mn.cpu().reshape(1), mx.cpu().reshape(1))
        assert_bit_equal(e["global_scale"], o_gs, f"{name} global scale")
        for sl in _slices(w.shape[0]):
            wc = w[sl].cpu()
            o_scale, o_zp = oq.observe_weight(wc, oargs, global_scale=o_gs)
            assert_bit_equal(e["scale"][sl], o_scale, f"{name} scales {sl}")
            want = op.nvfp4_compress(wc, o_scale, o_gs, oargs, zero_point=o_zp)
            assert_bit_equal(packed[i][sl], want, f"{name} packed {sl}")
            assert_bit_equal(dense[i][sl], op.nvfp4_decompress(want, o_scale, o_gs), f"{name} dense {sl}")


def test_dynamic_activation_quant_at_full_size(gpu):
    """dynamic nvfp4 on 4096 x 4096 N(0, 1) activations (static global scale, group-16
    scales per token) and dynamic per-token fp8 on 8192 x 4096 with outlier channels:
    the fused kernels against the oracle's compute_dynamic_scales_and_zp + fake_quantize"""
    from compressed_tensors_amd.quantization import QuantizationArgs, dynamic_fake_quantize, generate_gparam

    g = torch.Generator(device=gpu).manual_seed(4)
    x = torch.randn(1, 4096, 4096, generator=g, device=gpu).bfloat16()
    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16,
                dynamic="local")
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    mn, mx = torch.aminmax(x)
    gs = generate_gparam(mn.reshape(1), mx.reshape(1))
    o_gs = oq.generate_gparam(mn.cpu().reshape(1), mx.cpu().reshape(1))
    assert_bit_equal(gs, o_gs, "activation global scale")
    announce("dynamic nvfp4 activations", tuple(x.shape))
    got = dynamic_fake_quantize(x, args, global_scale=gs)
    for sl in _slices(4096):
        xc = x[:, sl].cpu()
        o_scale, o_zp = oq.compute_dynamic_scales_and_zp(xc, oargs, global_scale=o_gs)
        want = oq.fake_quantize(xc, o_scale, o_zp, oargs, global_scale=o_gs)
        assert_bit_equal(got[:, sl], want, f"nvfp4 tokens {sl}")

    x = torch.randn(1, 8192, 4096, generator=g, device=gpu)
    hot = torch.rand(4096, generator=g, device=gpu) < 5e-3
    x = torch.where(hot, x * 50, x).bfloat16()
    spec = dict(num_bits=8, type="float", symmetric=True, strategy="token", dynamic=True)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    announce("dynamic fp8 activations", tuple(x.shape))
    got = dynamic_fake_quantize(x, args)
    for sl in _slices(8192):
        xc = x[:, sl].cpu()
        o_scale, o_zp = oq.compute_dynamic_scales_and_zp(xc, oargs)
        want = oq.fake_quantize(xc, o_scale, o_zp, oargs)
        assert_bit_equal(got[:, sl], want, f"fp8 tokens {sl}")


def _ulp_bf16(t):
    mag = t.double().abs().clamp_min(2.0 ** -126)
    return torch.exp2(torch.floor(torch.log2(mag)) - 7)


@pytest.mark.parametrize("shape", [(4096, 4096), (14336, 4096)], ids=["4096x4096", "14336x4096"])
@pytest.mark.parametrize("n", [128, 4096])
def test_hadamard_weight_rotation_at_full_size(n, shape, gpu):
    """`weight_input` rotation (W @ R^T / sqrt(n), reference precision fp64) of N(0, 0.02)
    bf16 weights with a random-sign Hadamard of block size n: row slices against the fp64
    product, within 1 bf16 ulp"""
    from compressed_tensors_amd.transform import hadamard_apply

    announce("hadamard weight_input", n, shape)
    g = torch.Generator(device=gpu).manual_seed(n + shape[0])
    w = (torch.randn(shape, generator=g, device=gpu) * 0.02).bfloat16()
    q = (torch.randint(0, 2, (n,), generator=torch.Generator().manual_seed(n)) * 2 - 1).double()
    r64 = q.unsqueeze(1) * oh.deterministic_hadamard_matrix(n, torch.float64)  # R = diag(Q) H
    # W @ R^T = W @ (H^T diag(Q)): no input signs, output signs Q
    got = hadamard_apply(w, n, sign_out=q.float())
    for sl in _slices(shape[0]):
        exact = oh.hadamard_forward(r64, w[sl].cpu(), "weight_input")
        err = (got[sl].cpu().double() - exact.double()).abs()
        tol = _ulp_bf16(exact) + 2.0 ** -21 * exact.double().abs().amax(-1, keepdim=True)
        assert not bool((err > tol).any()), f"rows {sl}: max ratio {(err / tol).max():.2f}"
        # elements that lean on the second term (more than one bf16 ulp off: the fp32 sum fell on
        # the other side of a rounding boundary than the fp64 one): at most 1 in 10000 (none with these seeds)
        leaning = int((err > _ulp_bf16(exact)).sum())
        print(f"[hadamard {n} {shape}] rows {sl.start}..{sl.stop}: {leaning} of {err.numel()} elements more than 1 ulp off", flush=True)
        assert leaning <= 1e-4 * err.numel(), f"rows {sl}: {leaning} elements beyond one ulp"


@pytest.mark.parametrize("n", [128, 4096])
def test_fused_rotation_quantization_packing_at_full_size(n, gpu):
    """hadamard_quantize_pack on a 14336 x 4096 weight (block 128 = group 128, and the full
    4096-wide rotation with groups of 128): the rotated tensor equals hadamard_apply's, and
    scales / packed words equal the oracle's observer and pack-quantized compressor on the
    rotated rows"""
    from compressed_tensors_amd.quantization import QuantizationArgs
    from compressed_tensors_amd.transform import hadamard_apply, hadamard_quantize_pack

    shape = (14336, 4096)
    announce("fused hadamard + int4 + pack", n, shape)
    g = torch.Generator(device=gpu).manual_seed(9)
    w = (torch.randn(shape, generator=g, device=gpu) * 0.02).bfloat16()
    q = (torch.randint(0, 2, (n,), generator=torch.Generator().manual_seed(5)) * 2 - 1).float()
    spec = dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    fused = hadamard_quantize_pack(w, n, args, return_rotated=True, sign_out=q)
    y = hadamard_apply(w, n, sign_out=q)
    unsigned_zero = lambda t: torch.where(t == 0, torch.zeros_like(t), t).view(torch.int16)
    assert torch.equal(unsigned_zero(fused["rotated"]), unsigned_zero(y)), "rotated tensor"
    assert fused["weight_shape"].tolist() == list(shape)
    for sl in _slices(shape[0]):
        yc = y[sl].cpu()
        o_scale, o_zp = oq.observe_weight(yc, oargs)
        want = op.pack_quantized_compress(yc, o_scale, oargs, zero_point=o_zp)["weight_packed"]
        assert_bit_equal(fused["weight_scale"][sl], o_scale, f"scales {sl}")
        assert_bit_equal(fused["weight_packed"][sl], want, f"packed {sl}")


def test_whole_tensors_against_the_oracle(gpu):
    """one whole 4096 x 4096 weight per format against the oracle, every byte (the row slices
    above leave most rows to GPU-vs-GPU comparisons): fp8 per channel with outliers (codes and
    dequantized weight) and nvfp4 g16 (scales, packed codes, dequantized weight)"""
    from compressed_tensors_amd.compressors import BaseCompressor
    from compressed_tensors_amd.quantization import QuantizationArgs, observe_weight_qparams

    g = torch.Generator(device=gpu).manual_seed(21)
    w = torch.randn(4096, 4096, generator=g, device=gpu) * 0.02
    w = torch.where(torch.rand(4096, 4096, generator=g, device=gpu) < 1e-3, w * 20, w).bfloat16()
    wc = w.cpu()

    announce("whole tensor fp8", tuple(w.shape))
    spec = dict(num_bits=8, type="float", symmetric=True, strategy="channel")
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    scale, zp = observe_weight_qparams(w, args)
    o_scale, o_zp = oq.observe_weight(wc, oargs)
    assert_bit_equal(scale, o_scale, "fp8 scales")
    comp = BaseCompressor.load_from_registry("float-quantized")
    codes = comp.compress_weight(weight=w, scale=scale, zero_point=zp, quantization_args=args)["weight"]
    want = op.naive_compress(wc, o_scale, oargs, zero_point=o_zp)
    assert_bit_equal(codes, want, "fp8 codes")
    dense = comp.decompress_weight({"weight": codes, "weight_scale": scale}, quantization_args=args)
    assert_bit_equal(dense, op.naive_decompress(dict(weight=want, weight_scale=o_scale)), "fp8 dense")

    announce("whole tensor nvfp4", tuple(w.shape))
    spec = dict(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    args, oargs = QuantizationArgs(**spec), oq._Args(**spec)
    gs, scale, zp = _nvfp4_scales(w, args, gpu)
    mn, mx = torch.aminmax(wc)
    o_gs = oq.generate_gparam(mn.reshape(1), mx.reshape(1))
    o_scale, o_zp = oq.observe_weight(wc, oargs, global_scale=o_gs)
    assert_bit_equal(gs, o_gs, "nvfp4 global scale")
    assert_bit_equal(scale, o_scale, "nvfp4 scales")
    comp = BaseCompressor.load_from_registry("nvfp4-pack-quantized")
    packed = comp.compress_weight(weight=w, scale=scale, global_scale=gs, quantization_args=args)["weight_packed"]
    want = op.nvfp4_compress(wc, o_scale, o_gs, oargs, zero_point=o_zp)
    assert_bit_equal(packed, want, "nvfp4 packed")
    dense = comp.decompress_weight({"weight_packed": packed, "weight_scale": scale, "weight_global_scale": gs})
    assert_bit_equal(dense, op.nvfp4_decompress(want, o_scale, o_gs), "nvfp4 dense")
