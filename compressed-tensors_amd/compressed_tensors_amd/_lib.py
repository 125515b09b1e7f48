"""ctypes binding of libctmi.so (the C ABI declared in include/ctmi.h).

torch is imported first on purpose: libctmi.so needs the HIP runtime by soname,
and importing torch maps the one torch itself uses, so both share a single
runtime (and therefore streams and allocations).

There is no CPU fallback: every call needs the compiled library, and every
tensor handed to a kernel must live on a GPU.
"""
import ctypes
from ctypes import POINTER, c_char_p, c_float, c_int32, c_int64, c_void_p
from pathlib import Path
from typing import Optional

import torch

import os

# CTMI_LIB points at an alternative build of the library (kernel tuning experiments)
LIB_PATH = Path(os.environ.get("CTMI_LIB") or Path(__file__).resolve().parent / "lib" / "libctmi.so")

CTMI_OK = 0
CTMI_ERR_VALUE = -1
CTMI_ERR_UNSUPPORTED = -2
CTMI_ERR_ASSERT = -3
CTMI_ERR_HIP = -4

F32, F16, BF16, F8E4M3, I8, I16, I32, I64, U8, BOOL = range(10)
QTYPE_INT, QTYPE_FLOAT = 0, 1

_DTYPE_CODE = {
    torch.float32: F32,
    torch.float16: F16,
    torch.bfloat16: BF16,
    torch.float8_e4m3fn: F8E4M3,
    torch.int8: I8,
    torch.int16: I16,
    torch.int32: I32,
    torch.int64: I64,
    torch.uint8: U8,
    torch.bool: BOOL,
}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise NotImplementedError(f"dtype {dtype} is not supported by the HIP kernels")


class QParams(ctypes.Structure):
    """mirror of `struct ctmi_qparams`"""

    _fields_ = [
        ("scale", c_void_p),
        ("zero_point", c_void_p),
        ("global_scale", c_void_p),
        ("col_group", c_void_p),
        ("s_rows", c_int64),
        ("s_cols", c_int64),
        ("blk_rows", c_int64),
        ("blk_cols", c_int64),
        ("scale_dtype", c_int32),
        ("zp_dtype", c_int32),
        ("qtype", c_int32),
        ("num_bits", c_int32),
    ]


_QP = POINTER(QParams)


class WeightJob(ctypes.Structure):
    """mirror of `struct ctmi_weight_job`"""

    _fields_ = [
        ("src", c_void_p),
        ("dst", c_void_p),
        ("rows", c_int64),
        ("cols", c_int64),
        ("dense_dtype", c_int32),
        ("reserved", c_int32),
        ("qp", QParams),
    ]


class HadamardJob(ctypes.Structure):
    """mirror of `struct ctmi_hadamard_job`"""

    _fields_ = [("x", c_void_p), ("out", c_void_p), ("numel", c_int64)]


class HadamardPackJob(ctypes.Structure):
    """mirror of `struct ctmi_hadamard_pack_job`"""

    _fields_ = [("x", c_void_p), ("packed", c_void_p), ("scale", c_void_p), ("rotated", c_void_p),
                ("numel", c_int64)]


class Sparse24Job(ctypes.Structure):
    """mirror of `struct ctmi_sparse24_job`"""

    _fields_ = [("dense", c_void_p), ("values", c_void_p), ("bitmask", c_void_p),
                ("nvalues", c_int64), ("rows", c_int64), ("cols", c_int64)]


class ObserveNvfp4Job(ctypes.Structure):
    """mirror of `struct ctmi_observe_nvfp4_job`"""

    _fields_ = [("x", c_void_p), ("global_scale", c_void_p), ("packed", c_void_p), ("scale", c_void_p),
                ("rows", c_int64), ("cols", c_int64), ("x_dtype", c_int32), ("reserved", c_int32)]


class ObserveQuantizeJob(ctypes.Structure):
    """mirror of `struct ctmi_observe_quantize_job`"""

    _fields_ = [("x", c_void_p), ("codes", c_void_p), ("scale", c_void_p), ("zero_point", c_void_p),
                ("rows", c_int64), ("cols", c_int64), ("blk_cols", c_int64), ("x_dtype", c_int32),
                ("reserved", c_int32)]


class ObserveQuantizeBlocksJob(ctypes.Structure):
    """mirror of `struct ctmi_observe_quantize_blocks_job`"""

    _fields_ = [("x", c_void_p), ("codes", c_void_p), ("scale", c_void_p), ("zero_point", c_void_p),
                ("rows", c_int64), ("cols", c_int64), ("blk_rows", c_int64), ("blk_cols", c_int64),
                ("x_dtype", c_int32), ("reserved", c_int32)]


class ObservePackJob(ctypes.Structure):
    """ctmi_observe_pack_job"""
    _fields_ = [
        ("x", c_void_p), ("packed", c_void_p), ("scale", c_void_p), ("zero_point", c_void_p),
        ("rows", c_int64), ("cols", c_int64), ("blk_cols", c_int64),
        ("x_dtype", c_int32), ("num_bits", c_int32), ("symmetric", c_int32),
    ]


class ObserveJob(ctypes.Structure):
    """ctmi_observe_job"""

    _fields_ = [
        ("x", c_void_p),
        ("scale", c_void_p),
        ("zero_point", c_void_p),
        ("global_scale", c_void_p),
        ("rows", c_int64),
        ("cols", c_int64),
        ("blk_cols", c_int64),
        ("x_dtype", c_int32),
        ("reserved", c_int32),
    ]


class Stacked24Job(ctypes.Structure):
    """ctmi_stacked24_job"""

    _fields_ = [
        ("dense", c_void_p),
        ("values", c_void_p),
        ("bitmask", c_void_p),
        ("rows", c_int64),
        ("cols", c_int64),
        ("dense_dtype", c_int32),
        ("values_dtype", c_int32),
        ("qp", QParams),
    ]


class QdqJob(ctypes.Structure):
    """ctmi_qdq_job"""

    _fields_ = [
        ("x", c_void_p),
        ("out", c_void_p),
        ("rows", c_int64),
        ("cols", c_int64),
        ("x_dtype", c_int32),
        ("out_dtype", c_int32),
        ("qp", QParams),
    ]


# name -> (restype, argtypes); must list every symbol of include/ctmi.h
SIGNATURES = {
    "ctmi_last_error": (c_char_p, []),
    "ctmi_version": (c_int32, []),
    "ctmi_qdq": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int32, c_int64, c_int64, _QP, c_int32, c_int32, c_void_p],
    ),
    "ctmi_round_to_quantized_type": (
        c_int32, [c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32, c_void_p]),
    "ctmi_qdq_many": (c_int32, [POINTER(QdqJob), c_int64, c_int32, c_int32, c_void_p]),
    "ctmi_pack_to_int32": (
        c_int32,
        [c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int32, c_void_p],
    ),
    "ctmi_unpack_from_int32": (
        c_int32,
        [c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int32, c_void_p],
    ),
    "ctmi_pack_quantized_compress": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int64, c_int64, _QP, c_void_p],
    ),
    "ctmi_pack_quantized_decompress": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int64, c_int64, _QP, c_void_p],
    ),
    "ctmi_pack_quantized_compress_many": (c_int32, [POINTER(WeightJob), c_int64, c_void_p]),
    "ctmi_nvfp4_compress_many": (c_int32, [POINTER(WeightJob), c_int64, c_void_p]),
    "ctmi_nvfp4_decompress_many": (c_int32, [POINTER(WeightJob), c_int64, c_void_p]),
    "ctmi_pack_quantized_decompress_many": (c_int32, [POINTER(WeightJob), c_int64, c_void_p]),
    "ctmi_pack_quantized_launches": (c_int64, [POINTER(WeightJob), c_int64, c_int32]),
    "ctmi_pack_fp4_to_uint8": (c_int32, [c_void_p, c_int32, c_void_p, c_int64, c_int64, c_void_p]),
    "ctmi_unpack_fp4_from_uint8": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int64, c_int64, c_void_p],
    ),
    "ctmi_nvfp4_compress": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int64, c_int64, _QP, c_void_p],
    ),
    "ctmi_nvfp4_decompress": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int64, c_int64, _QP, c_void_p],
    ),
    "ctmi_pack_bitmasks": (c_int32, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "ctmi_unpack_bitmasks": (c_int32, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "ctmi_quantize_sparse24_compress_supported": (c_int32, [c_int32, c_int64, c_int64, POINTER(QParams)]),
    "ctmi_quantize_sparse24_compress": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_void_p, c_int64, c_int64, POINTER(QParams), c_void_p],
    ),
    "ctmi_sparse24_decompress_dequantize_supported": (
        c_int32, [c_int32, c_int32, c_int64, c_int64, POINTER(QParams)]),
    "ctmi_sparse24_dequantize_tmp_bytes": (c_int64, [c_int64, c_int64]),
    "ctmi_sparse24_decompress_dequantize": (
        c_int32,
        [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_int32, c_void_p, c_int64, c_int64,
         POINTER(QParams), c_void_p],
    ),
    "ctmi_observe_qparams_many": (
        c_int32, [POINTER(ObserveJob), c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p]),
    "ctmi_quantize_sparse24_compress_many": (c_int32, [POINTER(Stacked24Job), c_int64, c_void_p]),
    "ctmi_sparse24_decompress_dequantize_many": (c_int32, [POINTER(Stacked24Job), c_int64, c_void_p]),
    "ctmi_bitmask_tmp_bytes": (c_int64, [c_int64, c_int64]),
    "ctmi_bitmask_count": (
        c_int32,
        [c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
         c_void_p],
    ),
    "ctmi_bitmask_compact": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p],
    ),
    "ctmi_bitmask_decompress": (
        c_int32,
        [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p],
    ),
    "ctmi_bitmask_decompress_static_max_bytes": (c_int64, []),
    "ctmi_bitmask_decompress_static": (
        c_int32,
        [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_int64, c_int64, c_void_p],
    ),
    "ctmi_hadamard_quant_pack": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
         c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "ctmi_sparse24_decompress": (
        c_int32,
        [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p],
    ),
    "ctmi_get_24_bytemasks": (c_int32, [c_void_p, c_int32, c_void_p, c_int64, c_void_p]),
    "ctmi_sparse24_compress": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_void_p, c_int64, c_int64, c_void_p],
    ),
    "ctmi_topk24_lut": (None, [c_void_p]),
    "ctmi_calib_copy": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p]),
    "ctmi_hadamard_supported": (c_int32, [c_int32, c_int32, c_int32]),
    "ctmi_hadamard_apply_many": (
        c_int32,
        [POINTER(HadamardJob), c_int64, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p],
    ),
    "ctmi_sparse24_compress_many": (c_int32, [POINTER(Sparse24Job), c_int64, c_int32, c_void_p]),
    "ctmi_sparse24_decompress_many": (c_int32, [POINTER(Sparse24Job), c_int64, c_int32, c_void_p]),
    "ctmi_hadamard_quant_pack_many": (
        c_int32,
        [POINTER(HadamardPackJob), c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int32,
         c_int32, c_void_p],
    ),
    "ctmi_sylvester_supported": (c_int32, [c_int32, c_int32]),
    "ctmi_hadamard_sylvester_inner_supported": (c_int32, [c_int32, c_int32, c_int32]),
    "ctmi_sylvester_apply_many": (
        c_int32,
        [POINTER(HadamardJob), c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p],
    ),
    "ctmi_sylvester_quant_pack_many": (
        c_int32,
        [POINTER(HadamardPackJob), c_int64, c_int32, c_int32, c_void_p, c_void_p, c_int32, c_int32,
         c_int32, c_void_p],
    ),
    "ctmi_hadamard_kron_quant_pack_many": (
        c_int32,
        [POINTER(HadamardPackJob), c_int64, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
         c_void_p, c_int32, c_int32, c_int32, c_void_p],
    ),
    "ctmi_hadamard_apply": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p],
    ),
    "ctmi_kron_matmul_supported": (c_int32, [c_int32, c_int32, c_int32]),
    "ctmi_kron_matmul": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
         c_int32, c_float, c_void_p],
    ),
    "ctmi_block_matmul": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p],
    ),
    "ctmi_calculate_qparams": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int32, c_int64, c_int32, c_int32, c_int32, c_void_p,
         c_void_p, c_int32, c_void_p, c_int32, c_void_p],
    ),
    "ctmi_generate_gparam": (c_int32, [c_void_p, c_void_p, c_int32, c_int64, c_void_p, c_void_p]),
    "ctmi_minmax_tmp_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_int32]),
    "ctmi_minmax": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
         c_void_p],
    ),
    "ctmi_observe_pack_quantized_supported": (
        c_int32, [c_int32, c_int64, c_int64, c_int64, c_int32],
    ),
    "ctmi_observe_pack_quantized_many": (c_int32, [c_void_p, c_int64, c_void_p]),
    "ctmi_observe_pack_quantized": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int32, c_int32, c_void_p, c_void_p,
         c_void_p, c_void_p],
    ),
    "ctmi_observe_pack_quantized_gidx_supported": (
        c_int32, [c_int32, c_int64, c_int64, c_int64, c_int32],
    ),
    "ctmi_observe_pack_quantized_gidx": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p],
    ),
    "ctmi_mxfp4_round_to_power_2": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p]),
    "ctmi_mxfp4_generate_scales": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p]),
    "ctmi_mxfp4_convert_exp_scale": (c_int32, [c_void_p, c_void_p, c_int32, c_int64, c_void_p]),
    "ctmi_column_groups": (c_int32, [c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "ctmi_sparse24_tmp_bytes": (c_int64, [c_int64, c_int64, c_int32]),
    "ctmi_observe_nvfp4_compress": (
        c_int32, [c_void_p, c_int32, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "ctmi_dynamic_qdq_supported": (
        c_int32, [c_int32, c_int64, c_int64, c_int64, c_int32, c_int32, c_int32],
    ),
    "ctmi_observe_quantize_supported": (c_int32, [c_int32, c_int64, c_int64, c_int64, c_int32, c_int32]),
    "ctmi_observe_nvfp4_compress_many": (c_int32, [POINTER(ObserveNvfp4Job), c_int64, c_void_p]),
    "ctmi_observe_quantize_blocks_supported": (
        c_int32, [c_int32, c_int64, c_int64, c_int64, c_int64, c_int32, c_int32]),
    "ctmi_observe_quantize_blocks": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int32, c_int32, c_int32,
         c_void_p, c_int32, c_void_p, c_int32, c_void_p],
    ),
    "ctmi_observe_quantize_blocks_many": (
        c_int32,
        [POINTER(ObserveQuantizeBlocksJob), c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p],
    ),
    "ctmi_observe_quantize_many": (
        c_int32,
        [POINTER(ObserveQuantizeJob), c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p],
    ),
    "ctmi_observe_quantize": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int64, c_int64, c_int64, c_int32, c_int32, c_int32, c_void_p,
         c_int32, c_void_p, c_int32, c_void_p],
    ),
    "ctmi_dynamic_qdq": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int64, c_int64, c_int64, c_int32, c_int32, c_int32,
         c_void_p, c_void_p, c_int32, c_void_p, c_int32, c_void_p],
    ),
    "ctmi_observe_qparams": (
        c_int32,
        [c_void_p, c_int32, c_int64, c_int64, c_int64, c_int32, c_int32, c_int32, c_void_p,
         c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_void_p],
    ),
}

_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """Load libctmi.so (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with "
                "`python -m compressed_tensors_amd._build` (there is no CPU fallback)"
            )
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


_EXC = {
    CTMI_ERR_VALUE: ValueError,
    CTMI_ERR_UNSUPPORTED: NotImplementedError,
    CTMI_ERR_ASSERT: AssertionError,
    CTMI_ERR_HIP: RuntimeError,
}


def check(rc: int) -> None:
    if rc != CTMI_OK:
        msg = load().ctmi_last_error().decode("utf-8", "replace")
        raise _EXC.get(rc, RuntimeError)(msg)


def require_gpu(*tensors: Optional[torch.Tensor]) -> torch.device:
    """All given tensors must sit on one GPU; returns that device."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if t.device.type != "cuda":
            raise RuntimeError(
                f"compressed_tensors_amd kernels run on the GPU only, got a tensor on {t.device}"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors live on different devices: {dev} and {t.device}")
    if dev is None:
        raise RuntimeError("no tensor given")
    return dev


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


# torch's own shortcut to the current stream's handle (what its compiled kernels' launchers
# call): a tenth of the cost of building a torch.cuda.Stream object on every library call
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(device: torch.device) -> int:
    """the handle of torch's current stream on `device` (the stream the kernels go to)"""
    if _raw_stream is not None:
        index = device.index
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(device).cuda_stream
