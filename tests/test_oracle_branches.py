"""Pinning of the oracle's composed branches by independent means: hand computation
on tiny cases, Python loops, library routines (torch.block_diag) and the scalar C
restatement.  None of these retypes the oracle's own formula."""
import math

import numpy as np
import torch

from oracle import hadamard as oh
from oracle import pack as op
from oracle import quant as oq


def test_g_idx_branch_against_per_column_arithmetic():
    """act-order (forward.py:286-296, 329-331): sorting the columns by g_idx, cutting runs
    of group_size and unsorting must equal 'column c uses the scale of group g_idx[c]'
    when every group has exactly group_size columns.  2 x 8, groups of 4, computed per
    element with Python floats in bf16 steps."""
    x = torch.tensor([[0.11, -0.52, 0.93, 0.27, -0.78, 0.64, -0.05, 0.36],
                      [-0.41, 0.18, -0.99, 0.73, 0.22, -0.31, 0.57, -0.66]]).bfloat16()
    g_idx = torch.tensor([1, 0, 0, 1, 0, 1, 1, 0], dtype=torch.int32)
    scale = torch.tensor([[0.125, 0.0625], [0.25, 0.09375]]).bfloat16()  # [rows, groups]
    zp = torch.tensor([[1, -2], [0, 3]], dtype=torch.int8)
    args = oq._Args(num_bits=4, type="int", symmetric=False, strategy="group", group_size=4)
    q = oq.quantize(x, scale, zp, args, dtype=torch.int8, g_idx=g_idx)
    dq = oq.dequantize(q, scale, zp, g_idx=g_idx)
    fq = oq.fake_quantize(x, scale, zp, args, g_idx=g_idx)

    def bf(v):  # one rounding to bf16
        return float(torch.tensor(v, dtype=torch.float32).bfloat16())

    for r in range(2):
        for c in range(8):
            g = int(g_idx[c])
            s, z = float(scale[r, g]), float(zp[r, g])
            v = bf(bf(float(x[r, c]) / s) + z)
            v = min(max(v, -8.0), 7.0)
            code = int(np.rint(v))  # half to even, like torch.round
            assert int(q[r, c]) == code, (r, c)
            back = bf(bf(code - z) * s)
            assert float(dq[r, c]) == back, (r, c)
            assert float(fq[r, c]) == back, (r, c)
    # a -1 anywhere in g_idx means "unset": plain column order (forward.py:286)
    unset = oq.quantize(x, scale, zp, args, dtype=torch.int8, g_idx=torch.full((8,), -1, dtype=torch.int32))
    assert torch.equal(unset, oq.quantize(x, scale, zp, args, dtype=torch.int8))
    assert not torch.equal(unset, q)


def test_block_diagonal_matmul_against_block_diag():
    """matrix.py:137-171: a smaller square matrix applies block-diagonally, on either side"""
    g = torch.Generator().manual_seed(5)
    a = torch.randn(6, 12, generator=g, dtype=torch.float64)
    b = torch.randn(4, 4, generator=g, dtype=torch.float64)
    big = torch.block_diag(b, b, b)
    assert torch.allclose(oh.multihead_matmul(a, b), a @ big, rtol=0, atol=1e-12)
    left = torch.randn(3, 3, generator=g, dtype=torch.float64)
    m = torch.randn(12, 5, generator=g, dtype=torch.float64)
    big_left = torch.block_diag(*[left] * 4)
    assert torch.allclose(oh.multihead_matmul(left, m), big_left @ m, rtol=0, atol=1e-12)
    sq = torch.randn(12, 12, generator=g, dtype=torch.float64)
    assert torch.equal(oh.multihead_matmul(a, sq), a @ sq)
    # the three Linear / Embedding orientations of apply_transform_weight (matrix.py:105-131)
    w = torch.randn(12, 12, generator=g, dtype=torch.float64)
    v = torch.randn(7, 12, generator=g, dtype=torch.float64)
    assert torch.equal(oh.apply_transform_weight(w, v, "input", torch.nn.Linear), v @ w)
    assert torch.equal(oh.apply_transform_weight(w, v, "weight_input", torch.nn.Linear), v @ w.T)
    assert torch.equal(oh.apply_transform_weight(w, v.T.contiguous(), "weight_output", torch.nn.Linear),
                       w.T @ v.T.contiguous())
    assert torch.equal(oh.apply_transform_weight(w, v.T.contiguous(), "weight_input", torch.nn.Embedding),
                       w @ v.T.contiguous())
    assert torch.equal(oh.apply_transform_weight(w, v, "weight_output", torch.nn.Embedding), v @ w)


def test_asymmetric_zero_points_pack_along_rows():
    """pack_quantized.py:137-144: int8 zero points [R, G] become int32 [ceil(R / 8), G],
    row r of a group in bits [4 (r % 8), 4 (r % 8) + 4) after the +8 offset; rows beyond R
    pack the offset of 0 (0, not 8: padding happens after the offset, :230-234)"""
    zp = torch.tensor([[-8, 7], [0, -1], [3, 2], [-5, 4], [1, 1], [6, -7], [-2, 0], [7, -8],
                       [5, -3], [-4, 6]], dtype=torch.int8)  # 10 rows, 2 groups
    w = torch.zeros(10, 8).bfloat16()
    scale = torch.ones(10, 2).bfloat16()
    args = oq._Args(num_bits=4, type="int", symmetric=False, strategy="group", group_size=4)
    out = op.pack_quantized_compress(w, scale, args, zero_point=zp)
    got = out["weight_zero_point"]
    assert got.dtype == torch.int32 and tuple(got.shape) == (2, 2)
    for g in range(2):
        for word in range(2):
            want = 0
            for i in range(8):
                r = word * 8 + i
                if r < 10:
                    want |= (int(zp[r, g]) + 8) << (4 * i)
            if want >= 1 << 31:
                want -= 1 << 32
            assert int(got[word, g]) == want, (word, g)
    # and the way back (pack_quantized.py:167-177)
    codes = op.pack_quantized_decompress(dict(out, weight_scale=scale), args)
    assert tuple(codes.shape) == (10, 8)
    # w == 0 quantizes to the zero point itself, dequantizes back to 0
    assert torch.equal(codes, torch.zeros(10, 8).bfloat16())
    # symmetric schemes and the tensor strategy emit no packed zero point
    sym = oq._Args(num_bits=4, type="int", symmetric=True, strategy="group", group_size=4)
    assert "weight_zero_point" not in op.pack_quantized_compress(w, scale, sym, zero_point=zp)


def test_token_reduce_against_a_loop():
    """helpers.py:168-170, 202-203: per-token min / max over everything but dims 0 and 1,
    kept as size-1 dims; a 2-D input has no such dim and reduces over the whole tensor"""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 3, 5, generator=g).bfloat16()
    args = oq._Args(num_bits=8, type="int", symmetric=True, strategy="token")
    scale, zp = oq.compute_dynamic_scales_and_zp(x, args)
    assert tuple(scale.shape) == (2, 3, 1)
    for b in range(2):
        for t in range(3):
            row = [float(v) for v in x[b, t]]
            m = max(abs(min(min(row), 0.0)), abs(max(max(row), 0.0)))
            want = torch.tensor(m, dtype=torch.float32).bfloat16() / 127.5  # bf16 / python float
            want = max(float(want), float(torch.finfo(torch.bfloat16).eps))
            assert float(scale[b, t, 0]) == want, (b, t)
    flat_scale, _ = oq.compute_dynamic_scales_and_zp(x.reshape(6, 5), args)
    assert flat_scale.numel() == 1
    assert float(flat_scale) == float(scale.max())


def test_nvfp4_compress_against_scalar_c(coracle):
    """fp4_quantized.py:84-106 composed: per element fp32(x) / (fp32(scale) / gs), clamp,
    e2m1 rounding, nibble code; two codes a byte, low nibble first"""
    g = torch.Generator().manual_seed(7)
    w = (torch.randn(6, 32, generator=g) * 0.02).bfloat16()
    w[0, 0], w[0, 1], w[0, 2] = 0.0, -0.0, -1e-7
    args = oq._Args(num_bits=4, type="float", symmetric=True, strategy="tensor_group", group_size=16)
    gs = oq.generate_gparam(*[t.reshape(1) for t in torch.aminmax(w)])
    scale, zp = oq.observe_weight(w, args, global_scale=gs)
    packed = op.nvfp4_compress(w, scale, gs, args, zero_point=zp)
    assert packed.dtype == torch.uint8 and tuple(packed.shape) == (6, 16)
    for r in range(6):
        for c in range(32):
            s = np.float32(float(scale[r, c // 16].float())) / np.float32(float(gs))
            v = np.float32(float(w[r, c])) / s
            v = min(max(v, np.float32(-6.0)), np.float32(6.0))
            code = coracle.oracle_fp4_code(coracle.oracle_cast_to_fp4(float(v)))
            byte = int(packed[r, c // 2])
            got = (byte >> 4) if c % 2 else (byte & 0xF)
            assert got == code, (r, c, float(w[r, c]))
    dense = op.nvfp4_decompress(packed, scale, gs)
    assert dense.dtype == torch.bfloat16
    for r in range(6):
        for c in range(32):
            byte = int(packed[r, c // 2])
            code = (byte >> 4) if c % 2 else (byte & 0xF)
            s = np.float32(float(scale[r, c // 16].float())) / np.float32(float(gs))
            want = torch.tensor(float(np.float32(coracle.oracle_fp4_decode(code)) * s)).bfloat16()
            assert dense[r, c].view(torch.int16) == want.view(torch.int16), (r, c)


def test_naive_compress_against_scalar_c(coracle):
    """naive_quantized.py:99-114: quantize with dtype = the scheme's storage type; fp8
    per-channel on bf16 runs every step in bf16 (C restatement: one fp32 op + one bf16
    rounding per step, then the e4m3 cast)"""
    g = torch.Generator().manual_seed(11)
    w = (torch.randn(5, 24, generator=g) * 0.02).bfloat16()
    w[1, 3] *= 30
    args = oq._Args(num_bits=8, type="float", symmetric=True, strategy="channel")
    scale, zp = oq.observe_weight(w, args)
    codes = op.naive_compress(w, scale, args, zero_point=zp)
    assert codes.dtype == torch.float8_e4m3fn
    raw = codes.view(torch.uint8)
    for r in range(5):
        for c in range(24):
            s = float(scale[r, 0])
            v = coracle.oracle_bf16_to_f32(coracle.oracle_f32_to_bf16(float(w[r, c]) / s))
            v = min(max(v, -448.0), 448.0)
            assert int(raw[r, c]) == coracle.oracle_f32_to_f8e4m3(v), (r, c)
    dense = op.naive_decompress(dict(weight=codes, weight_scale=scale))
    for r in range(5):
        for c in range(24):
            v = coracle.oracle_f8e4m3_to_f32(int(raw[r, c]))
            want = coracle.oracle_f32_to_bf16(v * float(scale[r, 0]))
            assert int(dense[r, c].view(torch.int16)) & 0xFFFF == want, (r, c)
