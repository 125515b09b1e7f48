"""GPU: tensors that are views starting inside a buffer, off every vector boundary (a slice of a
flat parameter buffer, a state dict loaded into one allocation).  Every operation gives the
bits it gives for a fresh copy of the same values."""
import pytest
import torch

from gpu_util import announce, assert_bit_equal

pytestmark = pytest.mark.gpu


def _inside(t: torch.Tensor, shift: int = 1) -> torch.Tensor:
    """the same values as t, in a view that starts `shift` elements into a larger buffer"""
    buf = torch.empty(t.numel() + shift + 8, dtype=t.dtype, device=t.device)
    view = buf[shift:shift + t.numel()].view(t.shape)
    view.copy_(t)
    assert view.data_ptr() % 16 != 0 or t.element_size() * shift % 16 == 0
    return view


def _same(got, want, what):
    if isinstance(got, (tuple, list)):
        assert len(got) == len(want), what
        for g, w in zip(got, want):
            _same(g, w, what)
    elif isinstance(got, dict):
        assert set(got) == set(want), what
        for k in got:
            _same(got[k], want[k], f"{what}[{k}]")
    elif isinstance(got, torch.Tensor):
        assert_bit_equal(got, want, what)
    else:
        assert got == want, what


def test_quantization_calls_on_views_inside_a_buffer(gpu):
    from compressed_tensors_amd.compressors import BaseCompressor, pack_to_int32, unpack_from_int32
    from compressed_tensors_amd.compressors.fp4_quantized import pack_fp4_to_uint8, unpack_fp4_from_uint8
    from compressed_tensors_amd.quantization import (QuantizationArgs, compute_dynamic_scales_and_zp,
                                                     dequantize, fake_quantize, generate_gparam,
                                                     observe_weight_qparams, quantize)

    announce("misaligned: quantization")
    g = torch.Generator(device=gpu).manual_seed(1)
    w = (torch.randn(96, 512, generator=g, device=gpu) * 0.02).to(torch.bfloat16)
    wv = _inside(w)
    for spec in (dict(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128),
                 dict(num_bits=8, type="int", symmetric=False, strategy="channel"),
                 dict(num_bits=8, type="float", symmetric=True, strategy="tensor"),
                 dict(num_bits=8, type="float", symmetric=True, strategy="block", block_structure=[32, 128])):
        args = QuantizationArgs(**spec)
        scale, zp = observe_weight_qparams(w, args)
        _same(observe_weight_qparams(wv, args), (scale, zp), f"observer {spec}")
        sv, zv = _inside(scale), (_inside(zp) if zp is not None else None)
        _same(fake_quantize(wv, sv, zv, args), fake_quantize(w, scale, zp, args), f"fake_quantize {spec}")
        q = quantize(w, scale, zp, args, dtype=torch.int8 if spec["type"] == "int" else torch.float8_e4m3fn)
        _same(quantize(wv, sv, zv, args, dtype=q.dtype), q, f"quantize {spec}")
        _same(dequantize(_inside(q, 3), sv, zv, args, dtype=torch.bfloat16),
              dequantize(q, scale, zp, args, dtype=torch.bfloat16), f"dequantize {spec}")
    # pack-quantized weight, both directions
    args = QuantizationArgs(num_bits=4, type="int", symmetric=True, strategy="group", group_size=128)
    scale, zp = observe_weight_qparams(w, args)
    comp = BaseCompressor.load_from_registry("pack-quantized")
    c = comp.compress_weight(weight=w, scale=scale, zero_point=zp, quantization_args=args)
    _same(comp.compress_weight(weight=wv, scale=_inside(scale), zero_point=_inside(zp), quantization_args=args), c,
          "pack-quantized compress")
    data = {"weight_packed": _inside(c["weight_packed"]), "weight_shape": c["weight_shape"],
            "weight_scale": _inside(scale)}
    _same(comp.decompress_weight(data, quantization_args=args),
          comp.decompress_weight(dict(c, weight_scale=scale), quantization_args=args), "pack-quantized decompress")
    q8 = torch.randint(-8, 8, (96, 512), generator=g, device=gpu, dtype=torch.int8)
    packed = pack_to_int32(q8, 4)
    _same(pack_to_int32(_inside(q8, 5), 4), packed, "pack_to_int32")
    _same(unpack_from_int32(_inside(packed), 4, q8.shape), q8, "unpack_from_int32")
    # nvfp4
    fargs = QuantizationArgs(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    gs = generate_gparam(w.min().reshape(1), w.max().reshape(1))
    fs, fz = observe_weight_qparams(w, fargs, global_scale=gs)
    _same(observe_weight_qparams(wv, fargs, global_scale=gs), (fs, fz), "nvfp4 observer")
    fcomp = BaseCompressor.load_from_registry("nvfp4-pack-quantized")
    fc = fcomp.compress_weight(weight=w, scale=fs, global_scale=gs, quantization_args=fargs)
    _same(fcomp.compress_weight(weight=wv, scale=_inside(fs, 3), global_scale=gs, quantization_args=fargs), fc,
          "nvfp4 compress")
    whole = dict(fc, weight_scale=fs, weight_global_scale=gs)
    fd = dict(whole, weight_packed=_inside(fc["weight_packed"], 3), weight_scale=_inside(fs, 3))
    _same(fcomp.decompress_weight(fd, quantization_args=fargs), fcomp.decompress_weight(whole, quantization_args=fargs),
          "nvfp4 decompress")
    grid = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], device=gpu)
    f4 = (grid[torch.randint(0, 8, (64, 64), generator=g, device=gpu)]
          * (torch.randint(0, 2, (64, 64), generator=g, device=gpu) * 2 - 1)).to(torch.bfloat16)
    p4 = pack_fp4_to_uint8(f4)
    _same(pack_fp4_to_uint8(_inside(f4)), p4, "pack_fp4_to_uint8")
    _same(unpack_fp4_from_uint8(_inside(p4, 3), 64, 64, dtype=torch.bfloat16), f4, "unpack_fp4_from_uint8")
    # dynamic activations
    x = _inside(torch.randn(1, 40, 512, generator=g, device=gpu).to(torch.bfloat16))
    targs = QuantizationArgs(num_bits=8, type="float", symmetric=True, strategy="token", dynamic=True)
    _same(compute_dynamic_scales_and_zp(x, targs, None), compute_dynamic_scales_and_zp(x.clone(), targs, None),
          "dynamic per-token scales")


def test_sparse_calls_on_views_inside_a_buffer(gpu):
    from compressed_tensors_amd.compressors.sparse_24_bitmask import (get_24_bytemasks, sparse24_bitmask_compress,
                                                                      sparse24_bitmask_decompress)
    from compressed_tensors_amd.compressors.sparse_bitmask import bitmask_compress, bitmask_decompress
    from compressed_tensors_amd.utils import pack_bitmasks, unpack_bitmasks

    announce("misaligned: sparse")
    g = torch.Generator(device=gpu).manual_seed(2)
    for dtype in (torch.bfloat16, torch.float32, torch.float8_e4m3fn):
        w = torch.randn(64, 256, generator=g, device=gpu)
        w = torch.where(torch.rand(64, 256, generator=g, device=gpu) < 0.5, torch.zeros_like(w), w).to(dtype)
        wv = _inside(w)
        values, masks, offsets = bitmask_compress(w)
        _same(bitmask_compress(wv), (values, masks, offsets), f"bitmask_compress {dtype}")
        _same(bitmask_decompress(_inside(values), _inside(masks), w.shape), w.where(w.float() != 0, torch.zeros_like(w))
              if dtype != torch.float8_e4m3fn else bitmask_decompress(values, masks, w.shape), f"bitmask_decompress {dtype}")
        d = torch.randn(64, 256, generator=g, device=gpu)
        keep = get_24_bytemasks(d.to(torch.bfloat16))
        s = torch.where(keep, d, torch.zeros_like(d)).to(dtype)
        v24, m24 = sparse24_bitmask_compress(s)
        _same(sparse24_bitmask_compress(_inside(s)), (v24, m24), f"sparse24 compress {dtype}")
        _same(sparse24_bitmask_decompress(_inside(v24), _inside(m24), s.shape),
              sparse24_bitmask_decompress(v24, m24, s.shape), f"sparse24 decompress {dtype}")
    bools = torch.rand(64, 256, generator=g, device=gpu) < 0.3
    packed = pack_bitmasks(bools)
    _same(pack_bitmasks(_inside(bools)), packed, "pack_bitmasks")
    _same(unpack_bitmasks(_inside(packed), list(bools.shape)), bools, "unpack_bitmasks")
