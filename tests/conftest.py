import ctypes
import os
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "compressed-tensors_amd"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _ensure_oracle_lib() -> Path:
    lib = ROOT / "oracle" / "_build" / "libctmi_oracle.so"
    if not lib.exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)
    return lib


@pytest.fixture(scope="session")
def coracle():
    """ctypes handle on the C restatement (oracle/c/ctmi_oracle.c)"""
    lib = ctypes.CDLL(str(_ensure_oracle_lib()))
    f, u8, u16, i32, i64, vp = (ctypes.c_float, ctypes.c_uint8, ctypes.c_uint16, ctypes.c_int32,
                                ctypes.c_int64, ctypes.c_void_p)
    lib.oracle_bf16_to_f32.restype, lib.oracle_bf16_to_f32.argtypes = f, [u16]
    lib.oracle_f32_to_bf16.restype, lib.oracle_f32_to_bf16.argtypes = u16, [f]
    lib.oracle_f8e4m3_to_f32.restype, lib.oracle_f8e4m3_to_f32.argtypes = f, [u8]
    lib.oracle_f32_to_f8e4m3.restype, lib.oracle_f32_to_f8e4m3.argtypes = u8, [f]
    lib.oracle_cast_to_fp4.restype, lib.oracle_cast_to_fp4.argtypes = f, [f]
    lib.oracle_fp4_code.restype, lib.oracle_fp4_code.argtypes = u8, [f]
    lib.oracle_fp4_decode.restype, lib.oracle_fp4_decode.argtypes = f, [u8]
    lib.oracle_quantize.restype = f
    lib.oracle_quantize.argtypes = [f, f, f, i32, i32, i32, i32]
    lib.oracle_dequantize.restype = f
    lib.oracle_dequantize.argtypes = [f, f, f, i32, i32]
    lib.oracle_quantize_int_bf16.restype = None
    lib.oracle_quantize_int_bf16.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32]
    lib.oracle_dequantize_int_bf16.restype = None
    lib.oracle_dequantize_int_bf16.argtypes = [vp, vp, vp, vp, i64, i64, i64]
    lib.oracle_pack_to_int32.restype = None
    lib.oracle_pack_to_int32.argtypes = [vp, vp, i64, i64, i32]
    lib.oracle_unpack_from_int32.restype = None
    lib.oracle_unpack_from_int32.argtypes = [vp, vp, i64, i64, i32]
    lib.oracle_packbits_little.restype = None
    lib.oracle_packbits_little.argtypes = [vp, vp, i64, i64]
    lib.oracle_bitmask_compress_u16.restype = i64
    lib.oracle_bitmask_compress_u16.argtypes = [vp, i64, i64, vp, vp, vp]
    return lib


@pytest.fixture(scope="session")
def ctmi():
    """the product's C ABI, loaded (never built) by the tests"""
    from compressed_tensors_amd import _lib

    if not _lib.LIB_PATH.exists():
        from compressed_tensors_amd._build import build_library

        build_library()
    return _lib.load()


@pytest.fixture(scope="session")
def gpu():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")


def unpack_hadamard_blocks(path=None):
    """{K: int8 K x K} from tests/golden/hadamard_blocks.safetensors (bit-packed rows)"""
    import numpy as np
    import torch
    from safetensors import safe_open

    path = path or ROOT / "tests" / "golden" / "hadamard_blocks.safetensors"
    blocks = {}
    with safe_open(str(path), framework="pt", device="cpu") as f:
        for key in f.keys():
            k = int(key)
            bits = np.unpackbits(f.get_tensor(key).numpy(), axis=1)[:, :k]
            blocks[k] = torch.from_numpy(bits.astype(np.int8) * 2 - 1)
    return blocks


@pytest.fixture(scope="session")
def hadamard_blocks():
    return unpack_hadamard_blocks()


@pytest.fixture(scope="session")
def hadamard_table_path(tmp_path_factory, hadamard_blocks):
    """the golden blocks (and Sylvester's matrices for the powers of two the reference's
    table holds) written out in the layout of the reference's hadamards.safetensors"""
    import torch
    from safetensors.torch import save_file

    table = {str(k): h.clone() for k, h in hadamard_blocks.items()}
    for k in (1, 2, 4, 8, 16, 64, 128, 256):
        h = torch.ones(1, 1, dtype=torch.int8)
        while h.shape[0] < k:
            h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
        table[str(k)] = h.contiguous()
    path = tmp_path_factory.mktemp("hadamard") / "hadamards.safetensors"
    save_file(table, str(path))
    return str(path)
