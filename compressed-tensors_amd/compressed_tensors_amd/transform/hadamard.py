"""Hadamard transforms on the GPU.

Reference surface mirrored here:
  deterministic_hadamard_matrix / random_hadamard_matrix / is_pow2
      transform/utils/hadamard.py:33-99
  apply_transform_weight / _multihead_matmul
      transform/utils/matrix.py:65-171
  HadamardFactory / RandomHadamardFactory / HadamardTransform
      transform/factory/hadamard.py:31-121, transform/factory/random_hadamard.py:21-40
  TransformLocation / TransformArgs / TransformScheme
      transform/transform_args.py:24-85, transform/transform_scheme.py:26-55

A Hadamard transform object remembers how its matrix was built,
    W = diag(signs) * Sylvester(n)                  (signs = 1 for the deterministic kind)
    W = diag(signs) * (H_K^T (x) Sylvester(n / K))  (random kind, n not a power of two)
so `forward` never touches the n x n matrix: the signs are applied on the way
in or out and Sylvester(n) = Sylvester(a) (x) Sylvester(b) runs as two small
products on the matrix cores (ctmi_hadamard_apply); sizes K * 2^m with K from the
table of known Hadamard matrices (12, 20, 28 ... 224: 14336 = 224 * 64) run through
ctmi_kron_matmul.  `weight` materialises the dense matrix on demand for callers that
want to look at it.  Explicit dense matrices go through ctmi_kron_matmul too when a
run fits its LDS tile, else (and for float64) through torch.matmul on the GPU.

The table of known matrices is data, not code: `hadamards.safetensors` as the reference
ships it (keys "12", "20", ...: int8 K x K).  It is looked for at the path given to
`load_hadamard_table`, in $CTMI_HADAMARD_TABLE, and next to an installed
`compressed_tensors` package (found without importing it).
"""
import math
import os
from enum import Enum
from typing import Dict, List, Optional, Tuple

import torch
from torch import Tensor

from compressed_tensors_amd import _lib
from compressed_tensors_amd.compressors.base import to_gpu
from compressed_tensors_amd.registry import RegistryMixin
from compressed_tensors_amd.utils.internal import InternalModule

__all__ = [
    "is_pow2",
    "deterministic_hadamard_matrix",
    "random_hadamard_matrix",
    "random_hadamard_signs",
    "load_hadamard_table",
    "known_hadamard_block",
    "kron_apply",
    "hadamard_factors",
    "hadamard_apply",
    "hadamard_quantize_pack",
    "hadamard_apply_many",
    "hadamard_quantize_pack_many",
    "apply_transform_weight",
    "TransformLocation",
    "TransformArgs",
    "TransformScheme",
    "TransformFactory",
    "HadamardFactory",
    "RandomHadamardFactory",
    "HadamardTransform",
    "TransformBase",
]

_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def is_pow2(n: int) -> bool:
    return n > 0 and (n & (n - 1) == 0)


def deterministic_hadamard_matrix(
    size: int, dtype: torch.dtype = torch.bfloat16, device=torch.device("cpu")
) -> Tensor:
    """Sylvester's construction; entry (i, j) = (-1)^popcount(i & j)."""
    if size <= 0:
        raise ValueError("Cannot construct deterministic hadamard of size <= 0")
    if not is_pow2(size):
        raise ValueError("Cannot construct deterministic hadamard of size != 2^n")
    idx = torch.arange(size, device=device)
    both = idx.unsqueeze(0) & idx.unsqueeze(1)
    parity = torch.zeros_like(both)
    for bit in range(max(size.bit_length() - 1, 1)):
        parity ^= (both >> bit) & 1
    return (1 - 2 * parity).to(dtype)


def random_hadamard_signs(size: int, gen: Optional[torch.Generator] = None) -> Tensor:
    """The +-1 diagonal the reference draws (on the CPU, from `gen`) for a random
    Hadamard matrix: Q = 2 * randint(0, 2, (size,)) - 1  (hadamard.py:85-88)."""
    q = torch.randint(low=0, high=2, size=(size,), generator=gen, dtype=torch.float32)
    return q * 2 - 1


_TABLE_ENV = "CTMI_HADAMARD_TABLE"
_table_cache: Dict[str, Dict[int, Tensor]] = {}


def _default_table_path() -> Optional[str]:
    path = os.environ.get(_TABLE_ENV)
    if path:
        return path
    import importlib.util

    try:
        spec = importlib.util.find_spec("compressed_tensors")
    except (ImportError, ValueError):
        spec = None
    for root in (spec.submodule_search_locations or []) if spec else []:
        candidate = os.path.join(root, "transform", "utils", "hadamards.safetensors")
        if os.path.exists(candidate):
            return candidate
    return None


def load_hadamard_table(path: Optional[str] = None) -> Dict[int, Tensor]:
    """{K: int8 K x K Hadamard matrix} from a safetensors file laid out like the
    reference's hadamards.safetensors (transform/utils/hadamard.py:28, :102-129).  The file
    is read with safetensors (nothing in it is executed) and every matrix is checked:
    entries +-1 and H H^T = K I."""
    path = path or _default_table_path()
    if path is None:
        raise FileNotFoundError(
            "no table of known Hadamard matrices: pass its path, set $" + _TABLE_ENV +
            ", or install compressed_tensors (its transform/utils/hadamards.safetensors is used)")
    path = os.path.abspath(path)
    if path not in _table_cache:
        from safetensors import safe_open

        table = {}
        with safe_open(path, framework="pt", device="cpu") as f:
            for key in f.keys():
                h = f.get_tensor(key)
                k = int(key)
                hd = h.to(torch.float64)
                if tuple(h.shape) != (k, k) or not bool((hd.abs() == 1).all()) or not torch.equal(
                        hd @ hd.T, k * torch.eye(k, dtype=torch.float64)):
                    raise ValueError(f"entry {key!r} of {path} is not a {k} x {k} Hadamard matrix")
                table[k] = h.to(torch.int8)
        _table_cache[path] = table
    return _table_cache[path]


_sylvester_entries: Dict[str, Dict[int, bool]] = {}


def _is_sylvester_entry(path: str, k: int, block: Tensor) -> bool:
    """does entry k of the table at `path` equal Sylvester's matrix?  Compared once per
    (path, k)."""
    seen = _sylvester_entries.setdefault(os.path.abspath(path), {})
    if k not in seen:
        seen[k] = is_pow2(k) and torch.equal(block, deterministic_hadamard_matrix(k, torch.int8))
    return seen[k]


def known_hadamard_block(n: int, table_path: Optional[str] = None) -> Tuple[int, Optional[Tensor]]:
    """(K, H_K) as the reference's _fetch_hadamard_divisor picks it (hadamard.py:102-129):
    the largest K of the table with n / K a power of two.  H_K is None where the block is
    Sylvester's matrix, so that the whole transform is Sylvester(n): an entry of the table
    is compared with Sylvester's matrix before that is said of it.  With no table at hand a
    power of two other than 32 gives (min(n, 256), None), which is what the reference's
    table holds."""
    path = table_path or _default_table_path()
    if path is None and is_pow2(n) and n != 32:
        return min(n, 256), None
    table = load_hadamard_table(path)
    for k in sorted(table, reverse=True):
        if n % k == 0 and is_pow2(n // k):
            return k, (None if _is_sylvester_entry(path, k, table[k]) else table[k])
    raise ValueError(f"Cannot construct random hadamard matrix of size {n}")


def random_hadamard_matrix(
    size: int,
    dtype: torch.dtype = torch.bfloat16,
    device=torch.device("cpu"),
    gen: Optional[torch.Generator] = None,
    table_path: Optional[str] = None,
) -> Tensor:
    """The reference's random Hadamard matrix (hadamard.py:65-89, :132-163): diag(Q)
    pushed through log2(size / K) butterfly stages and the known K x K block, which is
    diag(Q) * (H_K^T (x) Sylvester(size / K)); for a power of two >= 64 that is
    diag(Q) * Sylvester(size)."""
    k, block = known_hadamard_block(size, table_path)
    q = random_hadamard_signs(size, gen).to(device=device)
    if block is None:
        h = deterministic_hadamard_matrix(size, torch.float32, device)
    else:
        s = deterministic_hadamard_matrix(size // k, torch.float32, device)
        h = torch.kron(block.to(device=device, dtype=torch.float32).T.contiguous(), s)
    return (q.unsqueeze(1) * h).to(dtype)


# ------------------------------------------------------------------ kernel plumbing
_KRON = {32: (1, 32), 64: (1, 64), 128: (1, 128), 1024: (32, 32), 2048: (32, 64),
         4096: (64, 64), 8192: (64, 128)}
_factor_cache: Dict[Tuple[int, str], Tensor] = {}


def hadamard_factors(n: int) -> Optional[Tuple[int, int]]:
    """(a, b) with Sylvester(n) = Sylvester(a) (x) Sylvester(b), if an MFMA kernel exists"""
    return _KRON.get(n)


def _sylvester_bf16(size: int, device) -> Tensor:
    key = (size, str(device))
    if key not in _factor_cache:
        _factor_cache[key] = deterministic_hadamard_matrix(size, torch.bfloat16, device).contiguous()
    return _factor_cache[key]


# Sylvester sizes with a butterfly kernel (ctmi_sylvester_*), and those where it is the faster
# one (measured on 14336 x 4096 bf16 weights: 4096: 5.1-5.4 TB/s against 4.4-4.5 on the matrix
# cores, 8192: 4.4 against 0.8; 1024 and 2048 are level)
_BUTTERFLY = (1024, 2048, 4096, 8192)
_BUTTERFLY_FIRST = (4096, 8192)


def _butterfly(n: int, dtype, kernel: Optional[str], matrix_t=None) -> bool:
    """does a Sylvester transform of size n go to the butterfly kernel?  kernel: None (the
    faster one), "butterfly" or "mfma"."""
    if kernel not in (None, "butterfly", "mfma"):
        raise ValueError(f"unknown kernel {kernel!r}")
    if matrix_t is not None or n not in _BUTTERFLY or kernel == "mfma" or dtype not in _FLOATS:
        if kernel == "butterfly":
            raise NotImplementedError(f"no butterfly kernel for size {n}, dtype {dtype} or an explicit matrix")
        return False
    if kernel == "butterfly" or n in _BUTTERFLY_FIRST:
        return True
    fac = _KRON.get(n)
    return fac is None or not _lib.load().ctmi_hadamard_supported(fac[0], fac[1], _lib.dtype_code(dtype))


def hadamard_kernel_exists(n: int, dtype) -> bool:
    """is there a kernel for x -> x Sylvester(n) on tensors of this dtype?"""
    if dtype not in _FLOATS:
        return False
    fac = _KRON.get(n)
    return n in _BUTTERFLY or (fac is not None and bool(
        _lib.load().ctmi_hadamard_supported(fac[0], fac[1], _lib.dtype_code(dtype))))


def _sign(t: Optional[Tensor], dev) -> Optional[Tensor]:
    return None if t is None else t.to(device=dev, dtype=torch.float32).contiguous()


def _aligned(*tensors) -> bool:
    return all(t is None or t.data_ptr() % 16 == 0 for t in tensors)


def _on_16_bytes(x: Tensor) -> Tensor:
    """x, or a copy of it if it starts inside a buffer off a 16-byte boundary (the kernels
    read and write 16 bytes a lane)"""
    return x.clone() if x.data_ptr() % 16 else x


def _matrix_free(n: int, dtype, *tensors) -> bool:
    """does the rotation (alone or fused with the quantization) by Sylvester's matrix of order
    n run without a matrix argument?"""
    return n == 128 and dtype == torch.bfloat16 and _aligned(*tensors)


def hadamard_apply(
    value: Tensor,
    n: int,
    sign_in: Optional[Tensor] = None,
    sign_out: Optional[Tensor] = None,
    matrix_t: Optional[Tensor] = None,
    kernel: Optional[str] = None,
) -> Tensor:
    """every run of n elements x of the last dim becomes
    (x * sign_in) @ M * sign_out / sqrt(n), M = Sylvester(n) or, for n <= 128,
    the explicit matrix whose transpose is `matrix_t` (bf16, entries exact in bf16).
    kernel: "mfma" / "butterfly" to pick between the two implementations of the Sylvester
    sizes 1024 ... 8192 (default: the faster one)."""
    x = _on_16_bytes(to_gpu(value).contiguous())
    if x.dtype not in _FLOATS:
        raise NotImplementedError(f"transforms of dtype {x.dtype} are not supported")
    if x.shape[-1] % n != 0:
        raise ValueError(f"{n} must divide the last dimension {x.shape[-1]}")
    if _butterfly(n, x.dtype, kernel, matrix_t) and (kernel == "butterfly" or _aligned(x)):
        return hadamard_apply_many([x], n, sign_in, sign_out, kernel="butterfly")[0]
    fac = hadamard_factors(n)
    lib = _lib.load()
    code = _lib.dtype_code(x.dtype)
    if fac is None or not lib.ctmi_hadamard_supported(fac[0], fac[1], code):
        raise NotImplementedError(f"no MFMA Hadamard kernel for size {n} and dtype {x.dtype}")
    a, b = fac
    dev = x.device
    if matrix_t is not None:
        if a != 1:
            raise NotImplementedError("explicit matrices are supported for sizes 32, 64 and 128")
        mb_t = matrix_t.to(device=dev, dtype=torch.bfloat16).contiguous()
        ma_t = None
    else:
        mb_t = _sylvester_bf16(b, dev)
        ma_t = _sylvester_bf16(a, dev) if a > 1 else None
    s_in = None if sign_in is None else sign_in.to(device=dev, dtype=torch.float32).contiguous()
    s_out = None if sign_out is None else sign_out.to(device=dev, dtype=torch.float32).contiguous()
    out = torch.empty_like(x)
    if matrix_t is None and _matrix_free(n, x.dtype, x, out, s_in, s_out):
        mb_t = None  # Sylvester's matrix of 128: the kernel that keeps no matrix in memory
    _lib.check(
        lib.ctmi_hadamard_apply(
            x.data_ptr(), out.data_ptr(), code, x.numel(), a, b, _lib.ptr(ma_t), _lib.ptr(mb_t),
            _lib.ptr(s_in), _lib.ptr(s_out), _lib.stream_of(dev),
        )
    )
    return out


def kron_apply(
    value: Tensor,
    w: Tensor,
    inner: int = 1,
    sign_in: Optional[Tensor] = None,
    sign_out: Optional[Tensor] = None,
    sylvester: bool = False,
    scale: Optional[float] = None,
) -> Tensor:
    """every run of h * inner elements x of the last dim, as X[h, inner] after sign_in,
    becomes vec(w^T X S) * sign_out * scale, S = Sylvester(inner) or the identity: the
    product x * diag(sign_in) * (w (x) S) * diag(sign_out) * scale (ctmi_kron_matmul).
    scale defaults to 1 / sqrt(h * inner) with the Sylvester factor, 1 without."""
    x = to_gpu(value).contiguous()
    if x.dtype not in _FLOATS:
        raise NotImplementedError(f"transforms of dtype {x.dtype} are not supported")
    h = int(w.shape[0])
    if w.ndim != 2 or w.shape[1] != h:
        raise ValueError("the explicit factor must be square")
    n = h * inner
    if x.shape[-1] % n != 0:
        raise ValueError(f"{n} must divide the last dimension {x.shape[-1]}")
    lib = _lib.load()
    code = _lib.dtype_code(x.dtype)
    if not lib.ctmi_kron_matmul_supported(h, inner, code):
        raise NotImplementedError(f"no kernel for a {h} x {inner} run of {x.dtype}")
    dev = x.device
    wf = w.to(device=dev, dtype=torch.float32).contiguous()
    s_in = None if sign_in is None else sign_in.to(device=dev, dtype=torch.float32).contiguous()
    s_out = None if sign_out is None else sign_out.to(device=dev, dtype=torch.float32).contiguous()
    for sgn in (s_in, s_out):
        if sgn is not None and sgn.numel() != n:
            raise ValueError(f"sign vectors hold {n} values")
    if scale is None:
        scale = 1.0 / math.sqrt(n) if sylvester else 1.0
    out = torch.empty_like(x)
    _lib.check(
        lib.ctmi_kron_matmul(x.data_ptr(), out.data_ptr(), code, x.numel(), h, inner, wf.data_ptr(),
                             _lib.ptr(s_in), _lib.ptr(s_out), int(bool(sylvester)), float(scale),
                             _lib.stream_of(dev))
    )
    return out


_FUSED_KRON = {2048: (32, 64), 4096: (64, 64)}  # transform sizes fused with group size 128 (MFMA)


def _fused_plan(n: int, args, kernel: Optional[str] = None):
    """None: block size n = group size (32, 64, 128); (a, b): transform size n = a * b with
    groups of 128 on the matrix cores; "butterfly": the same on the butterfly kernel"""
    kind = str(getattr(args.type, "value", args.type))
    strategy = str(getattr(args.strategy, "value", args.strategy))
    if not (args.num_bits == 4 and kind == "int" and args.symmetric and strategy == "group"):
        raise NotImplementedError("the fused path covers symmetric int4 group quantization")
    if n in (32, 64, 128) and args.group_size == n:
        return None
    if args.group_size == 128:
        if n in _BUTTERFLY and kernel != "mfma" and (kernel == "butterfly" or n in _BUTTERFLY_FIRST
                                                      or n not in _FUSED_KRON):
            return "butterfly"
        if n in _FUSED_KRON and kernel != "butterfly":
            return _FUSED_KRON[n]
    raise NotImplementedError(
        "the fused path covers block sizes 32, 64 and 128 with group_size == block size, and "
        "transform sizes 1024, 2048, 4096 and 8192 with group_size 128")


def hadamard_quantize_pack(
    value: Tensor,
    n: int,
    quantization_args,
    sign_in: Optional[Tensor] = None,
    sign_out: Optional[Tensor] = None,
    matrix_t: Optional[Tensor] = None,
    return_rotated: bool = False,
    kernel: Optional[str] = None,
) -> Dict[str, Tensor]:
    """hadamard_apply, the min-max observer and pack-quantized compression in one
    pass over a bf16 [rows, cols] tensor of a symmetric 4-bit integer group scheme:
    block size n (32, 64 or 128) equal to the group size, or a transform of size 1024,
    2048, 4096 or 8192 with groups of 128.  Returns what the three steps return, bit for
    bit (with the same `kernel` in hadamard_apply):
    weight_packed int32 [rows, cols / 8], weight_scale bf16 [rows, cols / group_size],
    weight_shape int64 [2] (and the rotated tensor under "rotated" if asked for)."""
    return _quantize_pack([value], n, quantization_args, sign_in, sign_out, matrix_t,
                          return_rotated, kernel)[0]


def _quantize_pack(values, n, args, sign_in, sign_out, matrix_t, return_rotated, kernel=None):
    xs = [to_gpu(v).contiguous() for v in values]
    plan = _fused_plan(n, args, kernel)
    if plan is not None and matrix_t is not None:
        raise NotImplementedError("explicit matrices are supported for sizes 32, 64 and 128")
    dev = xs[0].device
    for x in xs:
        if x.ndim != 2 or x.dtype != torch.bfloat16 or x.device != dev:
            raise NotImplementedError("the fused path takes 2-D bfloat16 tensors on one device")
        if x.shape[1] % n != 0:
            raise ValueError(f"{n} must divide the last dimension {x.shape[1]}")
    s_in = None if sign_in is None else sign_in.to(device=dev, dtype=torch.float32).contiguous()
    s_out = None if sign_out is None else sign_out.to(device=dev, dtype=torch.float32).contiguous()
    group = args.group_size
    jobs = (_lib.HadamardPackJob * len(xs))()
    results = []
    for job, x in zip(jobs, xs):
        rows, cols = x.shape
        packed = torch.empty((rows, cols // 8), dtype=torch.int32, device=dev)
        scale = torch.empty((rows, cols // group), dtype=torch.bfloat16, device=dev)
        rotated = torch.empty_like(x) if return_rotated else None
        job.x, job.packed, job.scale, job.rotated, job.numel = (
            x.data_ptr(), packed.data_ptr(), scale.data_ptr(), _lib.ptr(rotated), x.numel())
        out = {"weight_packed": packed, "weight_scale": scale, "weight_shape": torch.tensor(x.shape)}
        if return_rotated:
            out["rotated"] = rotated
        results.append(out)
    lib, code, stream = _lib.load(), _lib.dtype_code(torch.bfloat16), _lib.stream_of(dev)
    if plan is None:
        # no matrix argument stands for Sylvester's matrix of 128: that kernel keeps none in memory
        mb_t = None
        if matrix_t is not None:
            mb_t = matrix_t.to(device=dev, dtype=torch.bfloat16).contiguous()
        elif not _matrix_free(n, torch.bfloat16, s_in, s_out):
            mb_t = _sylvester_bf16(n, dev)
        _lib.check(lib.ctmi_hadamard_quant_pack_many(
            jobs, len(xs), code, n, _lib.ptr(mb_t), _lib.ptr(s_in), _lib.ptr(s_out), 4, 1, stream))
    elif plan == "butterfly":
        _lib.check(lib.ctmi_sylvester_quant_pack_many(
            jobs, len(xs), code, n, _lib.ptr(s_in), _lib.ptr(s_out), group, 4, 1, stream))
    else:
        a, b = plan
        _lib.check(lib.ctmi_hadamard_kron_quant_pack_many(
            jobs, len(xs), code, a, b, _sylvester_bf16(a, dev).data_ptr(),
            _sylvester_bf16(b, dev).data_ptr(), _lib.ptr(s_in), _lib.ptr(s_out), group, 4, 1, stream))
    return results


def hadamard_apply_many(
    values: List[Tensor],
    n: int,
    sign_in: Optional[Tensor] = None,
    sign_out: Optional[Tensor] = None,
    matrix_t: Optional[Tensor] = None,
    kernel: Optional[str] = None,
    in_place: bool = False,
) -> List[Tensor]:
    """hadamard_apply on several tensors of one dtype that share the matrix and the
    signs (the weights of a model under one transform scheme), from one call: the
    kernels take 8 tensors per launch.  in_place: the tensors (contiguous, on the GPU)
    are overwritten with their transforms and returned (a workgroup has read all of a
    run of n elements before it writes any of it)."""
    if not values:
        return []
    if in_place and not all(v.is_cuda and v.is_contiguous() and v.data_ptr() % 16 == 0 for v in values):
        raise ValueError("tensors transformed in place are contiguous tensors on the GPU that start on "
                         "16-byte boundaries")
    xs = [_on_16_bytes(to_gpu(v).contiguous()) for v in values]
    dtype, dev = xs[0].dtype, xs[0].device
    if dtype not in _FLOATS:
        raise NotImplementedError(f"transforms of dtype {dtype} are not supported")
    for x in xs:
        if x.dtype != dtype or x.device != dev:
            raise ValueError("tensors of one call share dtype and device")
        if x.shape[-1] % n != 0:
            raise ValueError(f"{n} must divide the last dimension {x.shape[-1]}")
    lib = _lib.load()
    code = _lib.dtype_code(dtype)
    if _butterfly(n, dtype, kernel, matrix_t):
        s_in, s_out = _sign(sign_in, dev), _sign(sign_out, dev)
        if _aligned(s_in, s_out, *xs) or kernel == "butterfly":
            outs = xs if in_place else [torch.empty_like(x) for x in xs]
            jobs = (_lib.HadamardJob * len(xs))()
            for job, x, out in zip(jobs, xs, outs):
                job.x, job.out, job.numel = x.data_ptr(), out.data_ptr(), x.numel()
            _lib.check(lib.ctmi_sylvester_apply_many(jobs, len(xs), code, n, _lib.ptr(s_in), _lib.ptr(s_out),
                                                     _lib.stream_of(dev)))
            return outs
    fac = hadamard_factors(n)
    if fac is None or not lib.ctmi_hadamard_supported(fac[0], fac[1], code):
        raise NotImplementedError(f"no MFMA Hadamard kernel for size {n} and dtype {dtype}")
    a, b = fac
    if matrix_t is not None:
        if a != 1:
            raise NotImplementedError("explicit matrices are supported for sizes 32, 64 and 128")
        mb_t, ma_t = matrix_t.to(device=dev, dtype=torch.bfloat16).contiguous(), None
    else:
        mb_t = _sylvester_bf16(b, dev)
        ma_t = _sylvester_bf16(a, dev) if a > 1 else None
    s_in = None if sign_in is None else sign_in.to(device=dev, dtype=torch.float32).contiguous()
    s_out = None if sign_out is None else sign_out.to(device=dev, dtype=torch.float32).contiguous()
    outs = xs if in_place else [torch.empty_like(x) for x in xs]
    if matrix_t is None and _matrix_free(n, dtype, s_in, s_out, *xs, *outs):
        mb_t = None  # Sylvester's matrix of 128: the kernel that keeps no matrix in memory
    jobs = (_lib.HadamardJob * len(xs))()
    for job, x, out in zip(jobs, xs, outs):
        job.x, job.out, job.numel = x.data_ptr(), out.data_ptr(), x.numel()
    _lib.check(
        lib.ctmi_hadamard_apply_many(jobs, len(xs), code, a, b, _lib.ptr(ma_t), _lib.ptr(mb_t),
                                     _lib.ptr(s_in), _lib.ptr(s_out), _lib.stream_of(dev))
    )
    return outs


def hadamard_quantize_pack_many(
    values: List[Tensor],
    n: int,
    quantization_args,
    sign_in: Optional[Tensor] = None,
    sign_out: Optional[Tensor] = None,
    matrix_t: Optional[Tensor] = None,
    kernel: Optional[str] = None,
) -> List[Dict[str, Tensor]]:
    """hadamard_quantize_pack on several bf16 [rows, cols] tensors from one call (8 per
    launch); one dict per tensor, as hadamard_quantize_pack returns it"""
    if not values:
        return []
    return _quantize_pack(values, n, quantization_args, sign_in, sign_out, matrix_t, False, kernel)


# ------------------------------------------------------------------ vocabulary
class TransformLocation(str, Enum):
    INPUT = "input"
    WEIGHT_INPUT = "weight_input"
    WEIGHT_OUTPUT = "weight_output"
    OUTPUT = "output"
    K_CACHE = "k_cache"
    Q_ATTN = "q_attn"

    def is_online(self) -> bool:
        return self not in (TransformLocation.WEIGHT_INPUT, TransformLocation.WEIGHT_OUTPUT)


def _torch_dtype(value) -> torch.dtype:
    """a torch.dtype, or its name with or without the "torch." in front (utils/type.py:30-40)"""
    if isinstance(value, torch.dtype):
        return value
    found = getattr(torch, str(value).removeprefix("torch."), None) if isinstance(value, str) else None
    if not isinstance(found, torch.dtype):
        raise ValueError(f"No such torch dtype `{value}`")
    return found


def _only_fields(cls, data: Dict, fields) -> None:
    extra = set(data) - set(fields)
    if extra:  # the reference's models forbid extra fields
        raise ValueError(f"{cls.__name__}: unexpected field(s) {sorted(extra)}")


class TransformArgs:
    """how and where a transform is applied (transform/transform_args.py:56-85)"""
    _FIELDS = ("targets", "location", "inverse", "ignore")

    def __init__(self, targets: List[str], location, inverse: bool = False,
                 ignore: Optional[List[str]] = None):
        self.targets = [targets] if isinstance(targets, str) else list(targets)
        self.location = TransformLocation(location)
        self.inverse = bool(inverse)
        self.ignore = [ignore] if isinstance(ignore, str) else list(ignore or [])

    def is_online(self) -> bool:
        return self.location.is_online()

    def model_dump(self) -> Dict:
        return {"targets": list(self.targets), "location": self.location.value,
                "inverse": self.inverse, "ignore": list(self.ignore)}

    @classmethod
    def model_validate(cls, data) -> "TransformArgs":
        if isinstance(data, cls):
            return data
        _only_fields(cls, data, cls._FIELDS)
        return cls(**data)

    def __eq__(self, other) -> bool:
        return isinstance(other, TransformArgs) and self.model_dump() == other.model_dump()

    def __repr__(self) -> str:
        return f"TransformArgs({self.model_dump()})"


class TransformScheme:
    """a transform type and the places of a model it goes to (transform/transform_scheme.py:25-55)"""
    _FIELDS = ("type", "apply", "randomize", "requires_grad", "head_dim", "precision")

    def __init__(self, type: str, apply: Optional[List[TransformArgs]] = None,
                 randomize: bool = False, requires_grad: bool = False,
                 head_dim: Optional[int] = None, precision=torch.float32):
        self.type = type
        self.apply = [TransformArgs.model_validate(a) for a in (apply or [])]
        self.randomize = bool(randomize)
        self.requires_grad = bool(requires_grad)
        self.head_dim = head_dim
        self.precision = _torch_dtype(precision)

    def model_dump(self) -> Dict:
        return {"type": self.type, "apply": [a.model_dump() for a in self.apply],
                "randomize": self.randomize, "requires_grad": self.requires_grad,
                "head_dim": self.head_dim, "precision": str(self.precision)}

    @classmethod
    def model_validate(cls, data) -> "TransformScheme":
        if isinstance(data, cls):
            return data
        _only_fields(cls, data, cls._FIELDS)
        return cls(**data)

    def __eq__(self, other) -> bool:
        return isinstance(other, TransformScheme) and self.model_dump() == other.model_dump()

    def __repr__(self) -> str:
        return f"TransformScheme({self.model_dump()})"


def _kernel_takes(value: Tensor, matrix: Tensor) -> bool:
    if value.dtype != matrix.dtype or value.dtype not in _FLOATS or value.numel() == 0:
        return False
    return bool(_lib.load().ctmi_kron_matmul_supported(int(matrix.shape[0]), 1,
                                                       _lib.dtype_code(value.dtype)))


def _times_blocks(value: Tensor, w: Tensor) -> Tensor:
    """value @ blockdiag(w, w, ...): w acts on every run of w.shape[0] values of the last
    dim (matrix.py:137-171, first branch).  ctmi_kron_matmul where a tile of runs fits in
    LDS and the dtypes agree (float16 / bfloat16 / float32); else a library GEMM."""
    h = w.shape[0]
    if value.shape[-1] % h != 0:
        raise ValueError(f"a {h} x {h} transform does not divide a dimension of {value.shape[-1]}")
    if _kernel_takes(value, w):
        return kron_apply(value, w, scale=1.0)
    if value.shape[-1] == h:
        return value @ w
    return (value.unflatten(-1, (value.shape[-1] // h, h)) @ w).flatten(-2, -1)


def _blocks_times(w: Tensor, value: Tensor) -> Tensor:
    """blockdiag(w, w, ...) @ value (matrix.py:137-171, second branch)
    = (value^T @ blockdiag(w^T, ...))^T"""
    h = w.shape[0]
    if value.shape[-2] % h != 0:
        raise ValueError(f"a {h} x {h} transform does not divide a dimension of {value.shape[-2]}")
    if value.ndim == 2 and _kernel_takes(value, w):
        return kron_apply(value.T.contiguous(), w.T, scale=1.0).T.contiguous()
    if value.shape[-2] == h:
        return w @ value
    return (w @ value.unflatten(-2, (value.shape[-2] // h, h))).flatten(-3, -2)


def apply_transform_weight(
    transform_weight: Tensor, value: Tensor, location, module_type: type
) -> Tensor:
    """Explicit-matrix form (matrix.py:65-134), unscaled: ctmi_kron_matmul on the GPU
    where the matrix fits its tile, a library GEMM otherwise.  The structured, matrix-free
    path is HadamardTransform.forward."""
    assert transform_weight.shape[0] == transform_weight.shape[1]
    w, v = to_gpu(transform_weight), to_gpu(value)
    location = TransformLocation(location)
    if location.is_online():
        return _times_blocks(v, w)
    if module_type == torch.nn.Linear:
        if location == TransformLocation.WEIGHT_INPUT:
            return _times_blocks(v, w.T)
        if location == TransformLocation.WEIGHT_OUTPUT:
            return _blocks_times(w.T, v)
    elif module_type == torch.nn.Embedding:
        if location == TransformLocation.WEIGHT_INPUT:
            return _blocks_times(w, v)
        if location == TransformLocation.WEIGHT_OUTPUT:
            return _times_blocks(v, w)
    raise NotImplementedError(f"Applying transforms to {module_type} {location} is not supported")


def _orientation(location: TransformLocation, module_type: type) -> Tuple[bool, bool]:
    """(left_multiply, transposed): the value is multiplied by W or W^T, from the
    right (along its last dim) or from the left (along its first dim)."""
    if location.is_online():
        return False, False
    if module_type == torch.nn.Linear:
        if location == TransformLocation.WEIGHT_INPUT:
            return False, True
        if location == TransformLocation.WEIGHT_OUTPUT:
            return True, True
    elif module_type == torch.nn.Embedding:
        if location == TransformLocation.WEIGHT_INPUT:
            return True, False
        if location == TransformLocation.WEIGHT_OUTPUT:
            return False, False
    raise NotImplementedError(f"Applying transforms to {module_type} {location} is not supported")


def _kron_plan(n: int, block: Optional[Tensor]) -> Optional[Tuple[int, int]]:
    """(h, b) of the run layout ctmi_kron_matmul gets for a transform of size n: the known
    block times Sylvester(n / K), or for a power of two without an MFMA kernel (256, 512,
    anything below 32) Sylvester(n / b) as the explicit factor beside Sylvester(b)."""
    if block is not None:
        return int(block.shape[0]), n // int(block.shape[0])
    if is_pow2(n):
        b = n if n <= 512 else 64  # up to 512 the butterflies stay inside a wavefront
        return n // b, b
    return None


def _matrix_core_split(lib, k: int, b: int, code: int) -> Optional[Tuple[int, int, bool]]:
    """(a, inner, butterflies) for H = B (x) Sylvester(b) with a k x k block B (k = 1: Sylvester
    alone) on the matrix cores: an a x a block as the explicit factor and Sylvester(inner) as
    butterflies on its product, or both as products.  Where b itself is not an inner size of
    the kernel, the block grows by a Sylvester factor:
    B (x) S(b) = (B (x) S(b / inner)) (x) S(inner), e.g. 5120 = 20 * 256 = 40 * 128."""
    if k > 1 and lib.ctmi_hadamard_sylvester_inner_supported(k, b, code):
        return k, b, True
    for inner in (128, 64, 32):
        if b > inner and b % inner == 0 and lib.ctmi_hadamard_sylvester_inner_supported(
                k * (b // inner), inner, code):
            return k * (b // inner), inner, True
    if k > 1 and lib.ctmi_hadamard_supported(k, b, code):
        return k, b, False
    return None


class TransformBase(InternalModule):
    """A transform as applied at one location of one kind of module
    (transform/factory/base.py:196-213)."""

    args: TransformArgs

    def forward(self, value: Tensor) -> Tensor:
        raise NotImplementedError()

    def forward_many(self, values: List[Tensor], in_place: bool = False) -> List[Tensor]:
        """forward on every tensor of a list (the weights of the modules one TransformArgs
        entry names); kernels that take several tensors per launch override it.  in_place:
        the tensors may be overwritten with their transforms (and returned)"""
        return [self.forward(v) for v in values]

    def same_as(self):
        """a key that two transforms share if forward does the same in both"""
        return id(self)

    def right_inverse(self, value: Tensor) -> Tensor:
        self.args.inverse = not self.args.inverse
        try:
            return self.forward(value)
        finally:
            self.args.inverse = not self.args.inverse

    def __repr__(self) -> str:
        return f"{type(self).__name__}(inverse={self.args.inverse})"


class HadamardTransform(TransformBase):
    """W = diag(signs) * H, optionally row/column permuted by `perm` (W[perm][:, perm]),
    where H = Sylvester(size) or, with `block` = a known K x K Hadamard matrix,
    H = block^T (x) Sylvester(size / K) as the reference builds it for sizes that are not
    powers of two (transform/utils/hadamard.py:65-89, :132-163); forward(value) applies it
    at `args.location`, divides by sqrt(size) and returns value.dtype
    (transform/factory/hadamard.py:85-121)."""

    def __init__(self, size: int, signs: Optional[Tensor], perm: Optional[Tensor],
                 scheme: TransformScheme, args: TransformArgs, module_type: type,
                 precision: torch.dtype = torch.float32, block: Optional[Tensor] = None,
                 dense: Optional[Dict] = None):
        super().__init__()
        if block is None and not is_pow2(size):
            raise ValueError("Cannot construct deterministic hadamard of size != 2^n")
        if block is not None:
            k = int(block.shape[0])
            if block.ndim != 2 or block.shape[1] != k or size % k != 0 or not is_pow2(size // k):
                raise ValueError(f"a {tuple(block.shape)} block does not build a matrix of size {size}")
        self.size = size
        self.signs = signs
        self.perm = perm
        self.block = block
        self.scheme = scheme
        self.args = args
        self.module_type = module_type
        self.precision = precision
        self._scale = torch.tensor(size, dtype=torch.float64).sqrt()
        self._factor: Dict[tuple, Tensor] = {}
        # dense matrices built on demand (state dicts, the library-GEMM path), shared by the
        # transforms a factory makes for one size
        self._dense: Dict[tuple, Tensor] = {} if dense is None else dense

    _dynamic_tied_weights_keys: List[str] = ["weight", "perm"]

    @property
    def weight(self) -> Tensor:
        """the dense matrix the reference would hold (before `perm`); one tensor for all
        transforms that share signs and precision"""
        key = (id(self.signs), self.precision)
        if key not in self._dense:
            self._dense[key] = self._build_weight()
        return self._dense[key]

    def _build_weight(self) -> Tensor:
        if self.block is None:
            h = deterministic_hadamard_matrix(self.size, self.precision, torch.device("cpu"))
        else:
            k = int(self.block.shape[0])
            s = deterministic_hadamard_matrix(self.size // k, self.precision, torch.device("cpu"))
            h = torch.kron(self.block.to(self.precision).cpu().T.contiguous(), s)
        if self.signs is not None:
            h = self.signs.to(self.precision).cpu().unsqueeze(1) * h
        return h

    def _orientation(self) -> Tuple[bool, bool]:
        left, transposed = _orientation(self.args.location, self.module_type)
        if self.args.inverse:
            transposed = not transposed
        if left:
            # M @ V = (V^T @ M^T)^T: the transposed value is multiplied by the other orientation
            transposed = not transposed
        return left, transposed

    def _signs_on(self, device) -> Optional[Tensor]:
        """the sign vector as fp32 on `device`, copied there once (a call per forward pass
        must not pay a host-to-device copy)"""
        if self.signs is None:
            return None
        key = ("signs", id(self.signs), str(device))
        if key not in self._factor:
            self._factor[key] = self.signs.to(device=device, dtype=torch.float32).contiguous()
        return self._factor[key]

    def same_as(self):
        return (self.size, id(self.signs), id(self.perm), id(self.block), self.args.location,
                self.args.inverse, self.module_type, self.precision)

    def forward_many(self, values: List[Tensor], in_place: bool = False) -> List[Tensor]:
        """Sylvester sizes the butterfly or matrix-core kernels take: all tensors in
        launches of 8 (ctmi_hadamard_apply_many); anything else one by one"""
        n = self.size
        if (not values or self.block is not None or self.perm is not None
                or len({v.dtype for v in values}) != 1 or values[0].dtype not in _FLOATS
                or not hadamard_kernel_exists(n, values[0].dtype)):
            return [self.forward(v) for v in values]
        left, transposed = self._orientation()
        xs = [to_gpu(v) for v in values]
        if left:
            xs = [x.transpose(0, -1) for x in xs]
        signs = self._signs_on(xs[0].device)
        s_in, s_out = (None, signs) if transposed else (signs, None)
        in_place = in_place and not left and all(
            x.is_cuda and x.is_contiguous() and x.data_ptr() % 16 == 0 for x in xs)
        ys = hadamard_apply_many(xs, n, sign_in=s_in, sign_out=s_out, in_place=in_place)
        return [y.transpose(0, -1).contiguous() for y in ys] if left else ys

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        """the entries the reference's transform holds as parameters: the dense matrix and
        the permutation (transform/factory/hadamard.py:84-101)"""
        super()._save_to_state_dict(destination, prefix, keep_vars)
        destination[prefix + "weight"] = self.weight
        if self.perm is not None:
            destination[prefix + "perm"] = self.perm

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys,
                              unexpected_keys, error_msgs):
        """a saved dense matrix must be the one this transform stands for; its signs (the
        first column of diag(signs) H) and the permutation are taken over"""
        weight = state_dict.pop(prefix + "weight", None)
        perm = state_dict.pop(prefix + "perm", None)
        if perm is not None:
            self.perm = perm.to(torch.int64).cpu()
        if weight is not None:
            if tuple(weight.shape) != (self.size, self.size):
                error_msgs.append(f"{prefix}weight: {tuple(weight.shape)} is not {self.size} x {self.size}")
            else:
                # row i of diag(signs) H is signs[i] times row i of H, whose first entry is +-1
                had_signs, self.signs = self.signs, None
                self._dense = {}  # its own matrices from here on
                unsigned_first = self.weight[:, 0].to(torch.float64)
                saved = weight.detach().to("cpu", torch.float64)
                self.signs = (saved[:, 0] * unsigned_first).to(torch.float32)
                if not torch.equal(self.weight.to(torch.float64), saved):
                    self.signs = had_signs
                    error_msgs.append(f"{prefix}weight is not a sign-scaled Hadamard matrix of this construction")
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys,
                                      unexpected_keys, error_msgs)

    def _explicit_factor(self, h: int, transposed: bool, device) -> Tensor:
        """fp32 [h, h] factor w of W = diag(q) (w (x) S) for x W, of W^T for x W^T"""
        key = (str(device), transposed)
        if key not in self._factor:
            if self.block is None:
                w = deterministic_hadamard_matrix(h, torch.float32, device)  # symmetric
            else:
                w = self.block.to(device=device, dtype=torch.float32)
                w = w.contiguous() if transposed else w.T.contiguous()
            self._factor[key] = w
        return self._factor[key]

    def forward(self, value: Tensor) -> Tensor:
        left, transposed = self._orientation()
        value = to_gpu(value)
        n = self.size
        lib = _lib.load()
        mfma = self.block is None and hadamard_kernel_exists(n, value.dtype)  # or the butterfly kernel
        big = None  # (a, b): an a x a block times Sylvester(b) on the matrix cores
        inner_butterflies = False  # ... with Sylvester(b) as butterflies on the block product
        if not mfma and value.dtype in _FLOATS:
            k = 1 if self.block is None else int(self.block.shape[0])
            split = _matrix_core_split(lib, k, n // k, _lib.dtype_code(value.dtype))
            if split is not None:
                big, inner_butterflies = split[:2], split[2]
        plan = None if (mfma or big) else _kron_plan(n, self.block)
        if plan is not None and not (value.dtype in _FLOATS and bool(
                lib.ctmi_kron_matmul_supported(plan[0], plan[1], _lib.dtype_code(value.dtype)))):
            plan = None
        if not mfma and big is None and plan is None:
            # float64 values, or a run too long for LDS: the dense matrix and a library GEMM
            w = self.weight.to(value.device)
            if self.perm is not None:
                w = w[self.perm.to(w.device)][:, self.perm.to(w.device)]
            if self.args.inverse:
                w = w.T
            out = apply_transform_weight(w, value.to(w.dtype), self.args.location, self.module_type)
            return (out / self._scale).to(value.dtype)

        x = value.transpose(0, -1) if left else value  # left multiply = right multiply of the transpose
        # W   = diag(q) H  ->  x W   = (x * q) H
        # W^T = H diag(q)  ->  x W^T = (x H) * q
        s_in = s_out = None
        if self.signs is not None:
            if transposed:
                s_out = self._signs_on(x.device)
            else:
                s_in = self._signs_on(x.device)
        if self.perm is not None:
            # W' = W[p][:, p]:  x W' = ((x scattered to p) W) gathered at p
            key = ("perm", id(self.perm), str(x.device))
            if key not in self._factor:  # the permutation and its inverse, on the device once
                on_device = self.perm.to(x.device)
                self._factor[key] = (on_device, torch.argsort(on_device))
            p, p_inverse = self._factor[key]
            blocks = x.unflatten(-1, (x.shape[-1] // n, n))
            x = blocks.index_select(-1, p_inverse).flatten(-2, -1)
        if mfma:
            y = hadamard_apply(x, n, sign_in=s_in, sign_out=s_out)
        elif big is not None:
            # x (Ma (x) S) with Ma = B^T for x W, B for x W^T; the kernel takes Ma^T
            a, b = big
            key = ("bf16", str(x.device), transposed)
            if key not in self._factor:
                k = 1 if self.block is None else int(self.block.shape[0])
                m = (torch.ones(1, 1, dtype=torch.bfloat16, device=x.device) if self.block is None
                     else self.block.to(device=x.device, dtype=torch.bfloat16))
                if a > k:  # the block grown by a Sylvester factor (symmetric: transposes with m)
                    m = torch.kron(m, _sylvester_bf16(a // k, x.device))
                self._factor[key] = (m.T if transposed else m).contiguous()
            x = x.contiguous()
            y = torch.empty_like(x)
            sign = (lambda t: None if t is None else
                    t.to(device=x.device, dtype=torch.float32).contiguous())
            si, so = sign(s_in), sign(s_out)
            mb = None if inner_butterflies else _sylvester_bf16(b, x.device)
            _lib.check(lib.ctmi_hadamard_apply(
                x.data_ptr(), y.data_ptr(), _lib.dtype_code(x.dtype), x.numel(), a, b,
                self._factor[key].data_ptr(), _lib.ptr(mb),
                _lib.ptr(si), _lib.ptr(so), _lib.stream_of(x.device)))
        else:
            # W = diag(q) (B^T (x) S):  x W = (x * q) (B^T (x) S);  x W^T = (x (B (x) S)) * q
            h, b = plan
            y = kron_apply(x.contiguous(), self._explicit_factor(h, transposed, x.device), inner=b,
                           sign_in=s_in, sign_out=s_out, sylvester=True)
        if self.perm is not None:
            y = y.unflatten(-1, (y.shape[-1] // n, n)).index_select(-1, p).flatten(-2, -1)
        return y.transpose(0, -1).contiguous() if left else y


class TransformFactory(RegistryMixin):
    """name -> factory registry with the reference's `from_scheme` entry, and the
    application of a scheme to a model (transform/factory/base.py:53-193)."""

    def __init__(self, name: str, scheme: TransformScheme, seed: Optional[int] = None):
        self.name = name
        self.scheme = scheme
        self.generator = torch.Generator()
        if seed is not None:
            self.generator.manual_seed(seed)

    @classmethod
    def from_scheme(cls, scheme: TransformScheme, **kwargs):
        return cls.get_value_from_registry(scheme.type)(scheme=scheme, **kwargs)

    def create_transform(self, module: torch.nn.Module, args: TransformArgs) -> "TransformBase":
        raise NotImplementedError()

    def apply_to_model(self, model: torch.nn.Module, use_tqdm: bool = True) -> None:
        """create the scheme's transforms and put them into the model
        (transform/factory/base.py:94-110).  The entries of `scheme.apply` are taken in order;
        the weights one entry names are rotated together, several tensors per launch, while
        the walk over the model goes on."""
        from compressed_tensors_amd.utils.match import match_named_modules

        bar = None
        if use_tqdm:
            import tqdm

            bar = tqdm.tqdm(desc=f"Applying {self.name} transforms")
        tick = (lambda k: None) if bar is None else bar.update
        for arg in self.scheme.apply:
            modules = (m for _, m in match_named_modules(model, arg.targets, arg.ignore))
            if arg.location in (TransformLocation.WEIGHT_INPUT, TransformLocation.WEIGHT_OUTPUT):
                self._fuse_into_weights(modules, arg, tick)
            else:
                for module in modules:
                    self._apply_to_module(model, module, arg)
                    tick(1)
        if bar is not None:
            bar.close()

    # modules per call of forward_many when weights are rotated: short calls first, so that
    # the GPU starts while the host still walks the rest of the model
    _FUSE_BATCHES = (8, 24, 64)

    def _transform_key(self, module: torch.nn.Module, args: TransformArgs):
        """modules with equal keys get equal transforms at `args` (one is created for all
        of them); None: one transform per module"""
        return None

    def _fuse_into_weights(self, modules, args: TransformArgs, tick=lambda k: None) -> None:
        """weight <- transform(weight) for every module (transform/factory/base.py:143-160).
        Modules whose transforms are the same (size, signs, permutation) and whose weights
        share dtype and device collect into calls of forward_many, in place where the kernel
        allows it; a call goes out as soon as it is full."""
        if self.scheme.requires_grad:
            raise NotImplementedError(
                "transforms that are trained (requires_grad) are not supported: the kernels "
                "have no backward")
        made: Dict = {}     # _transform_key -> (transform, its same_as())
        pending: Dict = {}  # (same_as, dtype, device) -> [transform, modules, weight addresses, calls made]

        def flush(entry):
            transform, batch = entry[0], entry[1]
            with torch.no_grad():
                outs = transform.forward_many([m.weight.data for m in batch], in_place=True)
                for module, out in zip(batch, outs):
                    w = module.weight
                    if out.data_ptr() != w.data_ptr():
                        w.data = out.to(device=w.device, dtype=w.dtype)
            tick(len(batch))
            entry[1], entry[2], entry[3] = [], set(), entry[3] + 1

        for module in modules:
            assert hasattr(module, "weight")
            key = self._transform_key(module, args)
            if key is None or key not in made:
                transform = self.create_transform(module, args)
                found = (transform, transform.same_as())
                if key is not None:
                    made[key] = found
            else:
                found = made[key]
            w = module.weight
            entry = pending.setdefault((found[1], w.dtype, w.device), [found[0], [], set(), 0])
            # a weight two modules share is transformed once per module, as in the reference's
            # loop over modules: never twice in one call
            if w.data_ptr() in entry[2]:
                flush(entry)
            entry[1].append(module)
            entry[2].add(w.data_ptr())
            if len(entry[1]) >= self._FUSE_BATCHES[min(entry[3], len(self._FUSE_BATCHES) - 1)]:
                flush(entry)
        for entry in pending.values():
            if entry[1]:
                flush(entry)

    def _apply_to_module(self, model: torch.nn.Module, module: torch.nn.Module,
                         args: TransformArgs) -> None:
        """one transform at one module: weights are rotated on the spot, the other locations
        get the transform as a submodule `<name>_<location>` and a hook that calls it
        (transform/factory/base.py:112-193)"""
        location = TransformLocation(args.location)
        if location in (TransformLocation.WEIGHT_INPUT, TransformLocation.WEIGHT_OUTPUT):
            self._fuse_into_weights([module], args)
            return
        transform = self.create_transform(module, args)
        module.register_module(f"{self.name}_{location.value}", transform)
        if location == TransformLocation.INPUT:
            module.register_forward_pre_hook(
                lambda _, inputs: transform(inputs[0]).to(inputs[0].device), prepend=True)
        elif location == TransformLocation.OUTPUT:
            module.register_forward_hook(lambda _, _inputs, output: transform(output).to(output.device))
        elif location in (TransformLocation.Q_ATTN, TransformLocation.K_CACHE):
            from transformers import PreTrainedModel

            from compressed_tensors_amd.modeling import (initialize_hooked_attention,
                                                         initialize_hooked_kv_cache,
                                                         register_key_hook, register_query_hook)

            if not isinstance(model, PreTrainedModel):
                raise ValueError(f"Cannot hook attention of model: {model}")
            if location == TransformLocation.Q_ATTN:
                initialize_hooked_attention(model, module)
                register_query_hook(
                    module, lambda _, query_states: transform(query_states).to(query_states.device))
            else:
                initialize_hooked_kv_cache(model, module)
                register_key_hook(
                    module, lambda _, key_states: transform(key_states).to(key_states.device))
        else:
            raise NotImplementedError()


def _transform_size(module: torch.nn.Module, location: TransformLocation,
                    head_dim: Optional[int]) -> int:
    size = None
    if isinstance(module, torch.nn.Linear):
        size = (module.in_features
                if location in (TransformLocation.INPUT, TransformLocation.WEIGHT_INPUT)
                else module.out_features)
    elif isinstance(module, torch.nn.Embedding):
        size = (module.num_embeddings
                if location in (TransformLocation.INPUT, TransformLocation.WEIGHT_INPUT)
                else module.embedding_dim)
    elif head_dim is None:
        raise NotImplementedError(
            f"Transforms on {type(module)} are not supported without head_dim"
        )
    if head_dim is not None:
        if size is not None and size % head_dim != 0:
            raise ValueError(f"{head_dim} must divide {size} for {type(module)} at {location}")
        size = head_dim
    return size


@TransformFactory.register("hadamard")
class HadamardFactory(TransformFactory):
    def __init__(self, name: str, scheme: TransformScheme, seed: Optional[int] = None):
        super().__init__(name, scheme, seed)
        self._signs: Dict[int, Optional[Tensor]] = {}
        self._blocks: Dict[int, Optional[Tensor]] = {}
        self._perms: Dict[int, Tensor] = {}
        self._dense: Dict[int, Dict] = {}

    def _create_signs(self, size: int) -> Optional[Tensor]:
        return None

    def _create_block(self, size: int) -> Optional[Tensor]:
        return None

    def _transform_key(self, module: torch.nn.Module, args: TransformArgs):
        return (_transform_size(module, args.location, self.scheme.head_dim), type(module))

    def create_transform(self, module: torch.nn.Module, args: TransformArgs) -> HadamardTransform:
        size = _transform_size(module, args.location, self.scheme.head_dim)
        if size not in self._signs:  # one draw per size, as the reference's weight cache
            self._blocks[size] = self._create_block(size)
            self._signs[size] = self._create_signs(size)
        perm = None
        if self.scheme.randomize:
            if size not in self._perms:
                self._perms[size] = torch.randperm(size, generator=self.generator)
            perm = self._perms[size]
        precision = self.scheme.precision if args.is_online() else torch.float64
        return HadamardTransform(size, self._signs[size], perm, self.scheme, args, type(module),
                                 precision=precision, block=self._blocks[size],
                                 dense=self._dense.setdefault(size, {}))


@TransformFactory.register("random-hadamard")
class RandomHadamardFactory(HadamardFactory):
    """`table_path`: the file of known Hadamard matrices that sizes other than powers of two
    (and 32) end in; by default looked up as `load_hadamard_table` describes."""

    def __init__(self, name: str, scheme: TransformScheme, seed: Optional[int] = None,
                 table_path: Optional[str] = None):
        super().__init__(name, scheme, seed)
        self.table_path = table_path

    def _create_block(self, size: int) -> Optional[Tensor]:
        return known_hadamard_block(size, self.table_path)[1]

    def _create_signs(self, size: int) -> Optional[Tensor]:
        return random_hadamard_signs(size, self.generator)
