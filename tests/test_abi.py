"""The C-ABI library: it loads, exports every symbol the header declares, and
rejects bad arguments before touching a device (so this runs without a GPU)."""
import ctypes
import re
from pathlib import Path

import pytest

from compressed_tensors_amd import _lib

ROOT = Path(__file__).resolve().parent.parent


def _declared_symbols():
    text = (ROOT / "include" / "ctmi.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ctmi_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(ctmi):
    names = _declared_symbols()
    assert len(names) >= 25
    for name in names:
        assert hasattr(ctmi, name), f"{name} declared in ctmi.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(names)


def test_version_and_struct_layout(ctmi):
    assert ctmi.ctmi_version() == 1
    assert ctypes.sizeof(_lib.QParams) == 4 * 8 + 4 * 8 + 4 * 4


def _err(ctmi):
    return ctmi.ctmi_last_error().decode()


def test_pack_argument_errors(ctmi):
    assert ctmi.ctmi_pack_to_int32(None, None, 4, 4, 9, 1, None) == _lib.CTMI_ERR_VALUE
    assert "less than 8 bits" in _err(ctmi)
    assert ctmi.ctmi_pack_to_int32(None, None, 4, 4, 0, 1, None) == _lib.CTMI_ERR_VALUE
    assert "at least 1" in _err(ctmi)
    assert ctmi.ctmi_pack_to_int32(None, None, 4, 4, 4, 2, None) == _lib.CTMI_ERR_VALUE
    assert ctmi.ctmi_unpack_from_int32(None, None, 4, 4, 16, 1, None) == _lib.CTMI_ERR_VALUE
    # empty tensors are fine and launch nothing
    assert ctmi.ctmi_pack_to_int32(None, None, 0, 8, 4, 1, None) == _lib.CTMI_OK
    # NULL data with a non-empty shape is refused on the host
    assert ctmi.ctmi_pack_to_int32(None, None, 2, 8, 4, 1, None) == _lib.CTMI_ERR_VALUE


def _qp(**kw):
    qp = _lib.QParams()
    qp.scale = 0x1000  # never dereferenced on these paths
    qp.s_rows, qp.s_cols, qp.blk_rows, qp.blk_cols = 1, 1, 4, 8
    qp.scale_dtype = _lib.BF16
    qp.qtype, qp.num_bits = _lib.QTYPE_INT, 4
    for k, v in kw.items():
        setattr(qp, k, v)
    return qp


def test_quant_argument_errors(ctmi):
    qp = _qp(num_bits=6, qtype=_lib.QTYPE_FLOAT)
    rc = ctmi.ctmi_qdq(None, _lib.BF16, None, _lib.BF16, 4, 8, ctypes.byref(qp), 1, 0, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "4 and 8 bits" in _err(ctmi)
    qp = _qp(qtype=7)
    rc = ctmi.ctmi_qdq(None, _lib.BF16, None, _lib.BF16, 4, 8, ctypes.byref(qp), 1, 0, None)
    assert rc == _lib.CTMI_ERR_VALUE and "Invalid quantization type" in _err(ctmi)
    qp = _qp()
    rc = ctmi.ctmi_qdq(None, _lib.I8, None, _lib.I8, 4, 8, ctypes.byref(qp), 1, 0, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED  # cannot quantize an int8 tensor
    qp = _qp(global_scale=0x1000)
    rc = ctmi.ctmi_pack_quantized_compress(None, _lib.BF16, None, 4, 8, ctypes.byref(qp), None)
    assert rc == _lib.CTMI_ERR_VALUE and "global_scale is not supported" in _err(ctmi)
    qp = _qp(num_bits=16)
    rc = ctmi.ctmi_pack_quantized_compress(None, _lib.BF16, None, 4, 8, ctypes.byref(qp), None)
    assert rc == _lib.CTMI_ERR_VALUE and "less than 8 bits" in _err(ctmi)
    qp = _qp(scale_dtype=_lib.F8E4M3)
    rc = ctmi.ctmi_qdq(None, _lib.BF16, None, _lib.BF16, 4, 8, ctypes.byref(qp), 1, 0, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "global_scale" in _err(ctmi)
    qp = _qp(s_cols=1, blk_cols=4)  # grid too small for 8 columns
    rc = ctmi.ctmi_qdq(None, _lib.BF16, None, _lib.BF16, 4, 8, ctypes.byref(qp), 1, 0, None)
    assert rc == _lib.CTMI_ERR_VALUE


def test_fp4_and_sparse_argument_errors(ctmi):
    assert ctmi.ctmi_pack_fp4_to_uint8(None, _lib.BF16, None, 3, 7, None) == _lib.CTMI_ERR_VALUE
    assert "even number of columns" in _err(ctmi)
    assert ctmi.ctmi_pack_fp4_to_uint8(None, _lib.I8, None, 3, 8, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert ctmi.ctmi_get_24_bytemasks(None, _lib.BF16, None, 6, None) == _lib.CTMI_ERR_VALUE
    assert "multiple of 4" in _err(ctmi)
    assert ctmi.ctmi_sparse24_compress(None, _lib.BF16, None, None, 3, 2, None) == _lib.CTMI_ERR_VALUE
    assert ctmi.ctmi_bitmask_count(None, 3, 1, None, None, 0x1000, None, 2, 2, None) == \
        _lib.CTMI_ERR_UNSUPPORTED
    assert ctmi.ctmi_calculate_qparams(None, None, _lib.BF16, 0, 4, _lib.QTYPE_FLOAT, 4, 0, None,
                                       None, _lib.BF16, None, _lib.F8E4M3, None) == \
        _lib.CTMI_ERR_UNSUPPORTED
    assert "Asymmetric Quantization is not supported for FP4" in _err(ctmi)


def test_one_pass_and_many_argument_errors(ctmi):
    """entry points that take lists of tensors or fuse several steps: everything is checked on
    the host, for every job, before anything could be enqueued"""
    # scratch sizes grow with the tensor
    assert ctmi.ctmi_bitmask_tmp_bytes(8192, 8192) > ctmi.ctmi_bitmask_tmp_bytes(8, 8) > 0
    assert ctmi.ctmi_sparse24_tmp_bytes(14336, 4096, 1) >= ctmi.ctmi_bitmask_tmp_bytes(14336, 4096)
    # nvfp4 lists: an odd column count in the second job stops the whole call
    jobs = (_lib.WeightJob * 2)()
    for j, cols in zip(jobs, (32, 31)):
        j.src, j.dst, j.rows, j.cols, j.dense_dtype = 0x1000, 0x2000, 4, cols, _lib.BF16
        j.qp = _qp(scale_dtype=_lib.F8E4M3, global_scale=0x3000, qtype=_lib.QTYPE_FLOAT, num_bits=4,
                   s_rows=4, s_cols=2, blk_rows=1, blk_cols=16)
    assert ctmi.ctmi_nvfp4_compress_many(jobs, 2, None) == _lib.CTMI_ERR_VALUE
    assert ctmi.ctmi_nvfp4_compress_many(None, 0, None) == _lib.CTMI_OK
    assert ctmi.ctmi_nvfp4_decompress_many(None, 3, None) == _lib.CTMI_ERR_VALUE
    # Hadamard lists: sizes must be multiples of the transform size, factorisations built
    hj = (_lib.HadamardJob * 2)()
    hj[0].x, hj[0].out, hj[0].numel = 0x1000, 0x2000, 256
    hj[1].x, hj[1].out, hj[1].numel = 0x1000, 0x2000, 200
    rc = ctmi.ctmi_hadamard_apply_many(hj, 2, _lib.BF16, 1, 128, None, 0x3000, None, None, None)
    assert rc == _lib.CTMI_ERR_VALUE and "not a multiple of the transform size" in _err(ctmi)
    rc = ctmi.ctmi_hadamard_apply_many(hj, 1, _lib.BF16, 3, 5, None, 0x3000, None, None, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED
    assert ctmi.ctmi_hadamard_apply_many(None, 0, _lib.BF16, 1, 128, None, None, None, None, None) == _lib.CTMI_OK
    pj = (_lib.HadamardPackJob * 1)()
    pj[0].x, pj[0].packed, pj[0].scale, pj[0].numel = 0x1000, 0x2000, 0x3000, 256
    rc = ctmi.ctmi_hadamard_quant_pack_many(pj, 1, _lib.F16, 128, 0x4000, None, None, 4, 1, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "bfloat16" in _err(ctmi)
    rc = ctmi.ctmi_hadamard_quant_pack_many(pj, 1, _lib.BF16, 128, 0x4000, None, None, 8, 1, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "4-bit" in _err(ctmi)
    # one-shot codes: layouts without a fused kernel say so
    assert ctmi.ctmi_observe_quantize_supported(_lib.BF16, 64, 4096, 4096, _lib.QTYPE_FLOAT, 8) == 1
    assert ctmi.ctmi_observe_quantize_supported(_lib.BF16, 64, 16392, 16392, _lib.QTYPE_FLOAT, 8) == 0
    assert ctmi.ctmi_observe_quantize_supported(_lib.BF16, 64, 4096, 4096, _lib.QTYPE_FLOAT, 4) == 0
    rc = ctmi.ctmi_observe_quantize(0x1000, _lib.BF16, 0x2000, 4, 100, 100, _lib.QTYPE_INT, 8, 1, 0x3000,
                                    _lib.BF16, None, _lib.I8, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "separately" in _err(ctmi)
    oj = (_lib.ObserveQuantizeJob * 1)()
    oj[0].x, oj[0].codes, oj[0].scale = 0x1000, 0x2000, 0
    oj[0].rows, oj[0].cols, oj[0].blk_cols, oj[0].x_dtype = 4, 4096, 4096, _lib.BF16
    rc = ctmi.ctmi_observe_quantize_many(oj, 1, _lib.QTYPE_FLOAT, 8, 1, -1, _lib.F8E4M3, None)
    assert rc == _lib.CTMI_ERR_VALUE and "NULL tensor pointer" in _err(ctmi)
    # quantization + 2:4: rows of whole bitmask bytes, scales in the tensor's dtype
    qp = _qp(s_rows=4, s_cols=1, blk_rows=1, blk_cols=64, qtype=_lib.QTYPE_FLOAT, num_bits=8)
    assert ctmi.ctmi_quantize_sparse24_compress_supported(_lib.BF16, 4, 64, ctypes.byref(qp)) == 1
    assert ctmi.ctmi_quantize_sparse24_compress_supported(_lib.F16, 4, 64, ctypes.byref(qp)) == 0
    qp = _qp(s_rows=4, s_cols=1, blk_rows=1, blk_cols=12, qtype=_lib.QTYPE_FLOAT, num_bits=8)
    assert ctmi.ctmi_quantize_sparse24_compress_supported(_lib.BF16, 4, 12, ctypes.byref(qp)) == 0
    rc = ctmi.ctmi_quantize_sparse24_compress(0x1000, _lib.BF16, 0x2000, 0x3000, 4, 12, ctypes.byref(qp), None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED
    # ... and the way back: codes are int8 or fp8, as many values as half the elements
    qp = _qp(s_rows=4, s_cols=1, blk_rows=1, blk_cols=64, qtype=_lib.QTYPE_INT, num_bits=8)
    ok = ctmi.ctmi_sparse24_decompress_dequantize_supported
    assert ok(_lib.F8E4M3, _lib.BF16, 4, 64, ctypes.byref(qp)) == 1
    assert ok(_lib.I8, _lib.BF16, 4, 64, ctypes.byref(qp)) == 1
    assert ok(_lib.BF16, _lib.BF16, 4, 64, ctypes.byref(qp)) == 0
    assert ok(_lib.I8, _lib.F32, 4, 64, ctypes.byref(qp)) == 0   # scales are bf16
    assert ctmi.ctmi_sparse24_dequantize_tmp_bytes(14336, 4096) == 0  # the check needs no caller scratch
    # several 2:4 tensors per call: shapes the streaming kernels do not take are refused up front
    sj = (_lib.Sparse24Job * 2)()
    for j, (rows, cols) in zip(sj, ((4, 64), (4, 12))):
        j.dense, j.values, j.bitmask, j.nvalues, j.rows, j.cols = 0x1000, 0x2000, 0x3000, rows * cols // 2, rows, cols
    rc = ctmi.ctmi_sparse24_compress_many(sj, 2, _lib.BF16, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "job 1" in _err(ctmi)
    rc = ctmi.ctmi_sparse24_decompress_many(sj, 2, 2, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "job 1" in _err(ctmi)
    sj[0].nvalues = 5
    rc = ctmi.ctmi_sparse24_decompress_many(sj, 1, 2, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "job 0" in _err(ctmi)
    assert ctmi.ctmi_sparse24_compress_many(sj, 0, _lib.BF16, None) == 0
    assert ctmi.ctmi_sparse24_compress_many(sj, 1, _lib.I32, None) != 0
    rc = ctmi.ctmi_sparse24_decompress_dequantize(0x1000, 100, _lib.I8, 0x2000, 0x3000, _lib.BF16, 0x4000,
                                                  4, 64, ctypes.byref(qp), None)
    assert rc == _lib.CTMI_ERR_VALUE and "128 values" in _err(ctmi)
    rc = ctmi.ctmi_sparse24_decompress_dequantize(0x1000, 128, _lib.I8, 0x2000, None, _lib.BF16, None,
                                                  4, 64, ctypes.byref(qp), None)
    assert rc == _lib.CTMI_ERR_VALUE and "NULL tensor pointer" in _err(ctmi)
    rc = ctmi.ctmi_sparse24_decompress_dequantize(0x1000, 128, _lib.I16, 0x2000, 0x3000, _lib.BF16, 0x4000,
                                                  4, 64, ctypes.byref(qp), None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED


def test_topk24_table_matches_installed_torch(ctmi):
    """the 2:4 keep table compiled into the library against torch.topk on every
    weak ordering of four keys"""
    import itertools

    import torch

    buf = (ctypes.c_uint8 * 4096)()
    ctmi.ctmi_topk24_lut(buf)
    pairs = [(0, 1), (0, 2), (0, 3), (1, 2), (1, 3), (2, 3)]
    seen = 0
    for t in itertools.product(range(4), repeat=4):
        if sorted(set(t)) != list(range(len(set(t)))):
            continue
        idx = 0
        for p, (i, j) in enumerate(pairs):
            idx |= (2 if t[i] > t[j] else (1 if t[i] == t[j] else 0)) << (2 * p)
        for dtype in (torch.float32, torch.bfloat16, torch.int8):
            keep = torch.tensor([t], dtype=dtype).topk(2, dim=1).indices[0].tolist()
            assert buf[idx] == (1 << keep[0]) | (1 << keep[1]), (t, dtype)
        seen += 1
    assert seen == 75


def test_product_refuses_cpu_tensors():
    import torch

    from compressed_tensors_amd.quantization import QuantizationArgs, quantize

    if torch.cuda.is_available():
        pytest.skip("needs a host without GPU")
    x = torch.zeros(4, 8, dtype=torch.bfloat16)
    s = torch.ones(1, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        quantize(x, s, None, QuantizationArgs(num_bits=4))


def test_transform_and_block_entry_point_errors(ctmi):
    """the entry points for explicit transform factors, the fused full-width rotation and the
    block-strategy one-shot: refused on the host, whatever device there is"""
    # ctmi_kron_matmul: what fits, and sizes that do not divide the tensor
    assert ctmi.ctmi_kron_matmul_supported(224, 64, _lib.BF16) == 1
    assert ctmi.ctmi_kron_matmul_supported(1, 512, _lib.F32) == 1
    assert ctmi.ctmi_kron_matmul_supported(12, 3, _lib.BF16) == 0
    assert ctmi.ctmi_kron_matmul_supported(12, 64, _lib.I8) == 0
    rc = ctmi.ctmi_kron_matmul(0x1000, 0x2000, _lib.BF16, 100, 12, 2, 0x3000, None, None, 1, 1.0, None)
    assert rc == _lib.CTMI_ERR_VALUE and "multiple of the transform size" in _err(ctmi)
    rc = ctmi.ctmi_kron_matmul(0x1000, 0x2000, _lib.BF16, 1024, 1, 512, 0x3000, None, None, 0, 1.0, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "Sylvester" in _err(ctmi)
    rc = ctmi.ctmi_kron_matmul(0x1000, 0x2000, _lib.BF16, 24, 12, 2, None, None, None, 1, 1.0, None)
    assert rc == _lib.CTMI_ERR_VALUE and "NULL tensor pointer" in _err(ctmi)
    assert ctmi.ctmi_kron_matmul(None, None, _lib.BF16, 0, 12, 2, None, None, None, 1, 1.0, None) == _lib.CTMI_OK
    rc = ctmi.ctmi_block_matmul(0x1000, 0x2000, _lib.BF16, 400 * 4, 400, 0x3000, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED
    # matrix-core factorisations: 224 x 32 / 64 for 16-bit tensors only
    assert ctmi.ctmi_hadamard_supported(224, 64, _lib.BF16) == 1
    assert ctmi.ctmi_hadamard_supported(224, 32, _lib.F16) == 1
    assert ctmi.ctmi_hadamard_supported(224, 64, _lib.F32) == 0
    assert ctmi.ctmi_hadamard_supported(224, 128, _lib.BF16) == 0
    # fused rotation of 2048 / 4096 + groups of 128
    pj = (_lib.HadamardPackJob * 1)()
    pj[0].x, pj[0].packed, pj[0].scale, pj[0].numel = 0x1000, 0x2000, 0x3000, 4096
    call = ctmi.ctmi_hadamard_kron_quant_pack_many
    assert call(pj, 1, _lib.BF16, 64, 128, 0x4000, 0x5000, None, None, 128, 4, 1, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert call(pj, 1, _lib.BF16, 64, 64, 0x4000, 0x5000, None, None, 64, 4, 1, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert "group size" in _err(ctmi)
    assert call(pj, 1, _lib.F16, 64, 64, 0x4000, 0x5000, None, None, 128, 4, 1, None) == _lib.CTMI_ERR_UNSUPPORTED
    pj[0].numel = 4000
    rc = call(pj, 1, _lib.BF16, 64, 64, 0x4000, 0x5000, None, None, 128, 4, 1, None)
    assert rc == _lib.CTMI_ERR_VALUE and "not a multiple of the transform size" in _err(ctmi)
    pj[0].numel = 4096
    rc = call(pj, 1, _lib.BF16, 64, 64, None, 0x5000, None, None, 128, 4, 1, None)
    assert rc == _lib.CTMI_ERR_VALUE and "matrices" in _err(ctmi)
    assert call(None, 0, _lib.BF16, 64, 64, None, None, None, None, 128, 4, 1, None) == _lib.CTMI_OK
    # one-shot block strategy
    ok = ctmi.ctmi_observe_quantize_blocks_supported
    assert ok(_lib.BF16, 256, 512, 128, 128, _lib.QTYPE_FLOAT, 8) == 1
    assert ok(_lib.BF16, 256, 512, 256, 128, _lib.QTYPE_FLOAT, 8) == 0   # 32768 elements a block
    assert ok(_lib.BF16, 250, 512, 128, 128, _lib.QTYPE_FLOAT, 8) == 0   # blocks must tile the tensor
    assert ok(_lib.BF16, 256, 512, 128, 12, _lib.QTYPE_FLOAT, 8) == 0    # 8 columns at a time
    assert ok(_lib.BF16, 256, 512, 128, 128, _lib.QTYPE_FLOAT, 4) == 0
    rc = ctmi.ctmi_observe_quantize_blocks(0x1000, _lib.BF16, 0x2000, 250, 512, 128, 128, _lib.QTYPE_FLOAT, 8, 1,
                                           0x3000, _lib.BF16, None, _lib.F8E4M3, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "tile the tensor" in _err(ctmi)
    rc = ctmi.ctmi_observe_quantize_blocks(0x1000, _lib.BF16, None, 256, 512, 128, 128, _lib.QTYPE_FLOAT, 8, 1,
                                           0x3000, _lib.BF16, None, _lib.F8E4M3, None)
    assert rc == _lib.CTMI_ERR_VALUE and "NULL tensor pointer" in _err(ctmi)
    # nvfp4 one-shot, several weights: groups of 16 columns, every job checked first
    oj = (_lib.ObserveNvfp4Job * 2)()
    for j, cols in zip(oj, (64, 40)):
        j.x, j.global_scale, j.packed, j.scale = 0x1000, 0x2000, 0x3000, 0x4000
        j.rows, j.cols, j.x_dtype = 4, cols, _lib.BF16
    rc = ctmi.ctmi_observe_nvfp4_compress_many(oj, 2, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "job 1" in _err(ctmi)
    oj[1].cols, oj[1].scale = 64, None
    rc = ctmi.ctmi_observe_nvfp4_compress_many(oj, 2, None)
    assert rc == _lib.CTMI_ERR_VALUE and "job 1" in _err(ctmi)
    assert ctmi.ctmi_observe_nvfp4_compress_many(None, 0, None) == _lib.CTMI_OK


def test_sylvester_entry_point_errors(ctmi):
    """the butterfly kernels' entry points: sizes, dtypes, alignment and job lists, refused on the host"""
    assert ctmi.ctmi_sylvester_supported(4096, _lib.BF16) == 1
    assert ctmi.ctmi_sylvester_supported(8192, _lib.F32) == 1
    assert ctmi.ctmi_sylvester_supported(512, _lib.BF16) == 0
    assert ctmi.ctmi_sylvester_supported(16384, _lib.BF16) == 0
    assert ctmi.ctmi_sylvester_supported(4096, _lib.I8) == 0
    assert ctmi.ctmi_kron_matmul_supported(1, 4096, _lib.F16) == 1
    jobs = (_lib.HadamardJob * 2)()
    jobs[0].x, jobs[0].out, jobs[0].numel = 0x1000, 0x2000, 8192
    jobs[1].x, jobs[1].out, jobs[1].numel = 0x3000, 0x4000, 4096 * 3
    call = ctmi.ctmi_sylvester_apply_many
    assert call(jobs, 2, _lib.BF16, 512, None, None, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert "1024, 2048, 4096 and 8192" in _err(ctmi)
    assert call(jobs, 2, _lib.I8, 4096, None, None, None) == _lib.CTMI_ERR_UNSUPPORTED
    jobs[1].numel = 5000
    assert call(jobs, 2, _lib.BF16, 4096, None, None, None) == _lib.CTMI_ERR_VALUE
    assert "job 1" in _err(ctmi) and "multiple of the transform size" in _err(ctmi)
    jobs[1].numel, jobs[1].out = 4096, None
    assert call(jobs, 2, _lib.BF16, 4096, None, None, None) == _lib.CTMI_ERR_VALUE and "job 1" in _err(ctmi)
    jobs[1].out = 0x4008
    assert call(jobs, 2, _lib.BF16, 4096, None, None, None) == _lib.CTMI_ERR_VALUE and "aligned" in _err(ctmi)
    jobs[1].out = 0x4000
    assert call(jobs, 2, _lib.BF16, 4096, 0x5004, None, None) == _lib.CTMI_ERR_VALUE and "sign vectors" in _err(ctmi)
    assert call(None, 0, _lib.BF16, 4096, None, None, None) == _lib.CTMI_OK
    jobs[0].numel = jobs[1].numel = 0
    assert call(jobs, 2, _lib.BF16, 4096, None, None, None) == _lib.CTMI_OK  # nothing to do, nothing launched
    pj = (_lib.HadamardPackJob * 1)()
    pj[0].x, pj[0].packed, pj[0].scale, pj[0].numel = 0x1000, 0x2000, 0x3000, 8192
    fused = ctmi.ctmi_sylvester_quant_pack_many
    assert fused(pj, 1, _lib.F16, 4096, None, None, 128, 4, 1, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert fused(pj, 1, _lib.BF16, 4096, None, None, 64, 4, 1, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert "group size" in _err(ctmi)
    assert fused(pj, 1, _lib.BF16, 4096, None, None, 128, 8, 1, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert fused(pj, 1, _lib.BF16, 4096, None, None, 128, 4, 0, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert fused(pj, 1, _lib.BF16, 256, None, None, 128, 4, 1, None) == _lib.CTMI_ERR_UNSUPPORTED
    pj[0].scale = None
    assert fused(pj, 1, _lib.BF16, 4096, None, None, 128, 4, 1, None) == _lib.CTMI_ERR_VALUE
    assert fused(None, 0, _lib.BF16, 4096, None, None, 128, 4, 1, None) == _lib.CTMI_OK
    # the same kernel behind ctmi_kron_matmul (h = 1, Sylvester inner factor)
    rc = ctmi.ctmi_kron_matmul(0x1008, 0x2000, _lib.BF16, 4096, 1, 4096, 0x3000, None, None, 1, 1.0, None)
    assert rc == _lib.CTMI_ERR_VALUE and "aligned" in _err(ctmi)


def test_stacked_and_activation_ordered_entry_points_check_their_arguments(ctmi):
    """the many-weight forms of the fp8 / int8 + 2:4 kernels and the one-pass kernel for
    activation-ordered weights: every job is looked at on the host before anything is enqueued"""
    jobs = (_lib.Stacked24Job * 2)()
    for j, cols in zip(jobs, (64, 68)):
        j.dense, j.values, j.bitmask, j.rows, j.cols = 0x1000, 0x2000, 0x3000, 4, cols
        j.dense_dtype, j.values_dtype = _lib.BF16, _lib.F8E4M3
        j.qp = _qp(scale=0x4000, scale_dtype=_lib.BF16, qtype=_lib.QTYPE_FLOAT, num_bits=8,
                   s_rows=4, s_cols=1, blk_rows=1, blk_cols=cols)
    # rows of 68 elements are not whole bitmask bytes: the second job stops the whole call
    assert ctmi.ctmi_quantize_sparse24_compress_many(jobs, 2, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert "job 1" in _err(ctmi)
    assert ctmi.ctmi_sparse24_decompress_dequantize_many(jobs, 2, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert ctmi.ctmi_quantize_sparse24_compress_many(None, 0, None) == _lib.CTMI_OK
    assert ctmi.ctmi_sparse24_decompress_dequantize_many(None, 0, None) == _lib.CTMI_OK
    assert ctmi.ctmi_quantize_sparse24_compress_many(None, 2, None) == _lib.CTMI_ERR_VALUE
    jobs[1].cols = 64
    jobs[1].qp.blk_cols = 64
    jobs[1].values = 0
    assert ctmi.ctmi_quantize_sparse24_compress_many(jobs, 2, None) == _lib.CTMI_ERR_VALUE
    # what the single-weight query says holds for the list
    assert ctmi.ctmi_quantize_sparse24_compress_supported(_lib.BF16, 4, 64, ctypes.byref(jobs[0].qp)) == 1
    assert ctmi.ctmi_quantize_sparse24_compress_supported(_lib.BF16, 4, 68, ctypes.byref(jobs[0].qp)) == 0
    # activation-ordered one pass: rows that fit a workgroup's registers, at most 256 groups a row
    assert ctmi.ctmi_observe_pack_quantized_gidx_supported(_lib.BF16, 64, 4096, 128, 4) == 1
    assert ctmi.ctmi_observe_pack_quantized_gidx_supported(_lib.BF16, 64, 4100, 4, 4) == 0   # cols % 8
    assert ctmi.ctmi_observe_pack_quantized_gidx_supported(_lib.BF16, 64, 16392, 8, 4) == 0  # too wide
    assert ctmi.ctmi_observe_pack_quantized_gidx_supported(_lib.BF16, 64, 4096, 8, 4) == 0   # 512 groups
    assert ctmi.ctmi_observe_pack_quantized_gidx_supported(_lib.BF16, 64, 4096, 128, 3) == 0
    rc = ctmi.ctmi_observe_pack_quantized_gidx(0x1000, _lib.BF16, 64, 4096, 8, 4, 1, None, 0x2000, 0x3000,
                                               None, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED and "separately" in _err(ctmi)
    rc = ctmi.ctmi_observe_pack_quantized_gidx(None, _lib.BF16, 64, 4096, 128, 4, 1, None, 0x2000, 0x3000,
                                               None, None)
    assert rc == _lib.CTMI_ERR_VALUE
    rc = ctmi.ctmi_observe_pack_quantized_gidx(0x1000, _lib.I8, 64, 4096, 128, 4, 1, None, 0x2000, 0x3000,
                                               None, None)
    assert rc == _lib.CTMI_ERR_UNSUPPORTED


def test_many_weight_observer_checks_every_job_first(ctmi):
    """ctmi_observe_qparams_many: the whole list is validated on the host before any launch"""
    jobs = (_lib.ObserveJob * 2)()
    for j in jobs:
        j.x, j.scale, j.zero_point, j.rows, j.cols, j.blk_cols, j.x_dtype = 0x1000, 0x2000, 0x3000, 4, 256, 128, _lib.BF16
    call = ctmi.ctmi_observe_qparams_many
    assert call(None, 0, _lib.QTYPE_INT, 4, 1, -1, _lib.I8, None) == _lib.CTMI_OK
    assert call(None, 2, _lib.QTYPE_INT, 4, 1, -1, _lib.I8, None) == _lib.CTMI_ERR_VALUE
    assert call(jobs, -1, _lib.QTYPE_INT, 4, 1, -1, _lib.I8, None) == _lib.CTMI_ERR_VALUE
    jobs[1].rows = 0
    assert call(jobs, 2, _lib.QTYPE_INT, 4, 1, -1, _lib.I8, None) == _lib.CTMI_ERR_VALUE
    assert "job 1" in _err(ctmi)
    jobs[1].rows, jobs[1].blk_cols = 4, 0
    assert call(jobs, 2, _lib.QTYPE_INT, 4, 1, -1, _lib.I8, None) == _lib.CTMI_ERR_VALUE
    jobs[1].blk_cols, jobs[1].scale = 128, 0
    assert call(jobs, 2, _lib.QTYPE_INT, 4, 1, -1, _lib.I8, None) == _lib.CTMI_ERR_VALUE
    assert "job 1" in _err(ctmi)
    jobs[1].scale, jobs[1].x_dtype = 0x2000, _lib.I8  # an integer tensor has no observer
    assert call(jobs, 2, _lib.QTYPE_INT, 4, 1, -1, _lib.I8, None) != _lib.CTMI_OK
    jobs[1].x_dtype = _lib.BF16
    assert call(jobs, 2, _lib.QTYPE_FLOAT, 4, 0, -1, _lib.F8E4M3, None) != _lib.CTMI_OK  # asymmetric fp4


def test_many_weight_block_one_shot_checks_every_job_first(ctmi):
    """ctmi_observe_quantize_blocks_many: what the single-weight query refuses stops the whole call"""
    jobs = (_lib.ObserveQuantizeBlocksJob * 2)()
    for j in jobs:
        j.x, j.codes, j.scale, j.rows, j.cols, j.blk_rows, j.blk_cols, j.x_dtype = (
            0x1000, 0x2000, 0x3000, 256, 512, 128, 128, _lib.BF16)
    call = ctmi.ctmi_observe_quantize_blocks_many
    fp8 = (_lib.QTYPE_FLOAT, 8, 1, -1, _lib.F8E4M3, None)
    assert call(None, 0, *fp8) == _lib.CTMI_OK
    assert call(None, 2, *fp8) == _lib.CTMI_ERR_VALUE
    jobs[1].blk_rows = 256  # 32768 elements: more than a workgroup's registers hold
    assert call(jobs, 2, *fp8) == _lib.CTMI_ERR_UNSUPPORTED
    assert "job 1" in _err(ctmi)
    assert ctmi.ctmi_observe_quantize_blocks_supported(_lib.BF16, 256, 512, 256, 128, _lib.QTYPE_FLOAT, 8) == 0
    jobs[1].blk_rows, jobs[1].cols = 128, 520  # blocks do not tile the rows
    assert call(jobs, 2, *fp8) == _lib.CTMI_ERR_UNSUPPORTED
    jobs[1].cols, jobs[1].codes = 512, 0
    assert call(jobs, 2, *fp8) == _lib.CTMI_ERR_VALUE
    jobs[1].codes, jobs[1].x = 0x2000, 0x1002  # not aligned to 8 elements
    assert call(jobs, 2, *fp8) == _lib.CTMI_ERR_VALUE
    jobs[1].x, jobs[1].rows = 0x1000, 0
    assert call(jobs, 2, *fp8) == _lib.CTMI_ERR_VALUE


def test_round_to_quantized_type_argument_checks(ctmi):
    """quant_args.py:384-408: FLOAT with other than 4 or 8 bits is not implemented, an unknown
    type is a value error; both are told before any GPU call"""
    f = ctmi.ctmi_round_to_quantized_type
    assert f(None, None, _lib.BF16, 0, 0, 8, None) == 0
    assert f(None, None, _lib.BF16, 16, 1, 6, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert b"Only num_bits in (4, 8)" in ctmi.ctmi_last_error()
    assert f(None, None, _lib.BF16, 16, 2, 8, None) == _lib.CTMI_ERR_VALUE
    assert f(None, None, _lib.I8, 16, 0, 8, None) == _lib.CTMI_ERR_UNSUPPORTED
    assert f(None, None, _lib.F32, 16, 0, 8, None) == _lib.CTMI_ERR_VALUE  # NULL tensors
    assert f(None, None, _lib.F32, -1, 0, 8, None) == _lib.CTMI_ERR_VALUE
