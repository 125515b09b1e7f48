"""Oracle: int32 packing, fp4 nibble packing and the per-format weight codecs.

Follows compressors/quantized_compressors/pack_quantized.py:88-309,
naive_quantized.py:73-136 and fp4_quantized.py:84-221 of the reference.
"""
import math

import torch

from . import quant

E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


def pack_to_int32(value, num_bits, packed_dim=1):
    # pack_quantized.py:186-246
    if value.dtype is not torch.int8:
        raise ValueError("Tensor must be quantized to torch.int8 before packing")
    if num_bits > 8:
        raise ValueError("Packing is only supported for less than 8 bits")
    if num_bits < 1:
        raise ValueError(f"num_bits must be at least 1, got {num_bits}")
    offset = 1 << (num_bits - 1)
    value = (value + offset).to(torch.uint8)
    pf = 32 // num_bits
    if packed_dim == 0:
        value = value.transpose(0, 1)
    rows, cols = value.shape
    padded = math.ceil(cols / pf) * pf
    if padded > cols:
        value = torch.nn.functional.pad(value, (0, padded - cols))
    lanes = value.reshape(rows, padded // pf, pf).to(torch.int32)
    shifts = torch.arange(pf, dtype=torch.int32) * num_bits
    packed = (lanes << shifts).sum(dim=2, dtype=torch.int32)
    if packed_dim == 0:
        packed = packed.transpose(0, 1)
    return packed


def unpack_from_int32(value, num_bits, shape, packed_dim=1):
    # pack_quantized.py:249-309
    if value.dtype is not torch.int32:
        raise ValueError(f"Expected {torch.int32} but got {value.dtype}, Aborting unpack.")
    if num_bits > 8:
        raise ValueError("Unpacking is only supported for less than 8 bits")
    pf = 32 // num_bits
    mask = (1 << num_bits) - 1
    if packed_dim == 1:
        out = torch.zeros((value.shape[0], value.shape[1] * pf), dtype=torch.int32)
        for i in range(pf):
            out[:, i::pf] = (value >> (num_bits * i)) & mask
        out = out[:, : int(shape[1])]
    else:
        out = torch.zeros((value.shape[0] * pf, value.shape[1]), dtype=torch.int32)
        for i in range(pf):
            out[i::pf, :] = (value >> (num_bits * i)) & mask
        out = out[: int(shape[0]), :]
    offset = pow(2, num_bits) // 2
    return (out - offset).to(torch.int8)


def _bit_depth(t):
    try:
        return torch.finfo(t.dtype).bits
    except TypeError:
        return torch.iinfo(t.dtype).bits


def pack_quantized_compress(weight, scale, args, zero_point=None, g_idx=None):
    # pack_quantized.py:88-145
    if _bit_depth(weight) > args.num_bits:
        q = quant.quantize(weight, scale, zero_point, args, dtype=torch.int8, g_idx=g_idx)
    else:
        q = weight
    out = {
        "weight_packed": pack_to_int32(q, args.num_bits),
        "weight_shape": torch.tensor(weight.shape),
    }
    if not args.symmetric and args.strategy in ("group", "channel"):
        out["weight_zero_point"] = pack_to_int32(zero_point, args.num_bits, packed_dim=0).contiguous()
    return out


def pack_quantized_decompress(data, args):
    # pack_quantized.py:147-183
    scale = data["weight_scale"]
    zero_point = data.get("weight_zero_point", None)
    shape = torch.Size(data["weight_shape"])
    unpacked = unpack_from_int32(data["weight_packed"], args.num_bits, shape)
    if not args.symmetric and args.strategy in ("group", "channel"):
        assert zero_point is not None, "Asymmetric quantization requires zero-point values"
        zero_point = unpack_from_int32(zero_point, args.num_bits, (shape[0], scale.shape[-1]),
                                       packed_dim=0)
    return quant.dequantize(unpacked, scale, zero_point, g_idx=data.get("weight_g_idx", None))


def naive_compress(weight, scale, args, zero_point=None, g_idx=None):
    # naive_quantized.py:73-114
    if _bit_depth(weight) > args.num_bits:
        return quant.quantize(weight, scale, zero_point, args, dtype=quant.pytorch_dtype(args),
                              g_idx=g_idx)
    return weight


def naive_decompress(data):
    # naive_quantized.py:116-136
    return quant.dequantize(data["weight"], data["weight_scale"],
                            data.get("weight_zero_point", None),
                            g_idx=data.get("weight_g_idx", None))


def pack_fp4_to_uint8(x):
    # fp4_quantized.py:135-178 (eager semantics: the subtraction runs in x.dtype)
    m, n = x.shape
    if n % 2 != 0:
        raise ValueError("tensor must have an even number of columns for nvfp4 compression")
    lut = torch.tensor(E2M1, dtype=x.dtype)
    dist = torch.abs(torch.abs(x).unsqueeze(-1) - lut)
    idx = torch.argmin(dist, dim=-1) + (torch.signbit(x).to(torch.long) << 3)
    pairs = idx.reshape(-1).reshape(-1, 2)
    return (pairs[:, 0] | (pairs[:, 1] << 4)).to(torch.uint8).reshape(m, n // 2)


def unpack_fp4_from_uint8(a, m, n, dtype=torch.bfloat16):
    # fp4_quantized.py:187-221
    assert a.dtype == torch.uint8
    flat = a.flatten()
    hi = (flat & 0xF0) >> 4
    lo = flat & 0x0F
    both = torch.stack((lo, hi), dim=1).flatten()
    neg = (both & 0x08).to(torch.bool)
    mag = (both & 0x07).to(torch.long)
    vals = torch.tensor(E2M1, dtype=torch.float32)[mag] * torch.where(neg, -1.0, 1.0)
    return vals.reshape(m, n).to(dtype=dtype)


def nvfp4_compress(weight, scale, global_scale, args, zero_point=None):
    # fp4_quantized.py:84-106
    q = quant.quantize(weight, scale, zero_point, args, global_scale=global_scale)
    return pack_fp4_to_uint8(q)


def nvfp4_decompress(packed, scale, global_scale):
    # fp4_quantized.py:108-123
    m, n = packed.shape
    unpacked = unpack_fp4_from_uint8(packed, m, n * 2)
    return quant.dequantize(unpacked, scale, global_scale=global_scale, dtype=unpacked.dtype)
