"""safetensors files on either side of the compress / decompress path.

Reading mirrors the reference's helpers (utils/safetensors_load.py:
get_safetensors_header :79-97, get_weight_mappings :128-178,
get_nested_weight_mappings :181-247, get_quantization_parameter_to_path_mapping
:294-318): a checkpoint is one `.safetensors` file, a directory with
`model.safetensors`, or a directory with `model.safetensors.index.json`;
tensors are read one at a time straight onto the device they are needed on.

Writing: `save_file` takes tensors that live on the GPU (where the compressors
leave them) and streams them into a safetensors file through two pinned staging
buffers, so that the copy of one tensor off the device overlaps the file write of
the one before and no host copy of the whole state dict is ever made.  The result
is an ordinary safetensors file (8-byte little-endian header length, JSON header,
raw little-endian data in header order).
"""
import json
import os
import struct
from typing import Dict, Generator, Iterable, Optional, Tuple, Union

import torch
from torch import Tensor

__all__ = [
    "get_safetensors_header",
    "get_weight_mappings",
    "get_nested_weight_mappings",
    "get_quantization_parameter_to_path_mapping",
    "get_safetensors_folder",
    "match_param_name",
    "is_quantization_param",
    "get_nested_mappings_from_state_dict",
    "iter_tensors",
    "CheckpointReader",
    "save_file",
    "SAFE_WEIGHTS_NAME",
    "SAFE_WEIGHTS_INDEX_NAME",
]

SAFE_WEIGHTS_NAME = "model.safetensors"
SAFE_WEIGHTS_INDEX_NAME = "model.safetensors.index.json"

_DTYPE_NAMES = {
    torch.float64: "F64", torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
    torch.int64: "I64", torch.int32: "I32", torch.int16: "I16", torch.int8: "I8",
    torch.uint8: "U8", torch.bool: "BOOL", torch.float8_e4m3fn: "F8_E4M3",
    torch.float8_e5m2: "F8_E5M2",
}


_DTYPE_RANK = {dt: i for i, dt in enumerate((
    torch.bool, torch.uint8, torch.int8, torch.float8_e5m2, torch.float8_e4m3fn, torch.int16,
    torch.float16, torch.bfloat16, torch.int32, torch.float32, torch.float64, torch.int64))}


def get_safetensors_header(safetensors_path: str) -> Dict[str, dict]:
    """the JSON header of a safetensors file (tensor name -> dtype / shape / offsets)"""
    with open(safetensors_path, "rb") as f:
        (length,) = struct.unpack("<Q", f.read(8))
        return json.loads(f.read(length).decode("utf-8"))


def get_weight_mappings(path_to_model_or_tensors: str) -> Dict[str, str]:
    """tensor name -> file that holds it"""
    path = str(path_to_model_or_tensors)
    if os.path.isfile(path):
        header = get_safetensors_header(path)
        header.pop("__metadata__", None)
        return {key: path for key in header}
    single = os.path.join(path, SAFE_WEIGHTS_NAME)
    index = os.path.join(path, SAFE_WEIGHTS_INDEX_NAME)
    if os.path.exists(single):
        header = get_safetensors_header(single)
        header.pop("__metadata__", None)
        return {key: single for key in header}
    if os.path.exists(index):
        with open(index, "r", encoding="utf-8") as f:
            weight_map = json.load(f)["weight_map"]
        return {key: os.path.join(path, value) for key, value in weight_map.items()}
    raise ValueError(f"Could not find a safetensors weight or index file at {path}")


def _module_of(full_name: str, param_name: str) -> Optional[str]:
    suffix = "." + param_name
    if full_name.endswith(suffix) and len(full_name) > len(suffix):
        return full_name[: -len(suffix)]
    return None


def get_nested_weight_mappings(model_path: str, params_to_nest: Iterable[str],
                               return_unmatched_params: bool = False):
    """module path -> {compression parameter -> file}, optionally with the names that
    matched no compression parameter (needed when compressors are stacked)"""
    params_to_nest = tuple(params_to_nest)
    nested, unmatched = {}, {}
    for key, location in get_weight_mappings(model_path).items():
        matched = False
        for param_name in params_to_nest:
            module_path = _module_of(key, param_name)
            if module_path:
                nested.setdefault(module_path, {})[param_name] = location
                matched = True
        if return_unmatched_params and not matched:
            unmatched[key] = location
    return (nested, unmatched) if return_unmatched_params else nested


def get_safetensors_folder(pretrained_model_name_or_path: str, cache_dir: Optional[str] = None) -> str:
    """the folder that holds a model's safetensors files: a local path as it is, anything else
    through transformers' cache (utils/safetensors_load.py:42-81)"""
    path = str(pretrained_model_name_or_path)
    if os.path.exists(path):
        return os.path.abspath(path)
    from transformers.utils import cached_file

    for name in (SAFE_WEIGHTS_NAME, SAFE_WEIGHTS_INDEX_NAME):
        found = cached_file(path, name, cache_dir=cache_dir, _raise_exceptions_for_missing_entries=False)
        if found is not None:
            return os.path.split(found)[0]
    raise ValueError(f"Could not locate safetensors weight or index file from {path}.")


def match_param_name(full_name: str, param_name: str) -> Optional[str]:
    """the module path of `full_name` if it ends in `.param_name` (utils/safetensors_load.py:99-112)"""
    return _module_of(full_name, param_name)


def is_quantization_param(name: str) -> bool:
    """utils/safetensors_load.py:308-322"""
    return name.endswith(("_scale", "zero_point", "g_idx"))


def get_nested_mappings_from_state_dict(state_dict, params_to_nest: Iterable[str],
                                        return_unmatched_params: bool = False):
    """module path -> {compression parameter -> tensor} for a state dict in memory
    (utils/safetensors_load.py:251-305)"""
    from compressed_tensors_amd.utils.helpers import nest_state_dict

    return nest_state_dict(state_dict, tuple(params_to_nest), return_unmatched_params=return_unmatched_params)


def get_quantization_parameter_to_path_mapping(model_path: str) -> Dict[str, str]:
    """the scale / zero point / g_idx / global scale entries of a checkpoint"""
    suffixes = ("_scale", "_zero_point", "_g_idx", "_global_scale")
    return {k: v for k, v in get_weight_mappings(model_path).items() if k.endswith(suffixes)}


def iter_tensors(path: str, names: Optional[Iterable[str]] = None,
                 device: Union[str, torch.device] = "cpu") -> Generator[Tuple[str, Tensor], None, None]:
    """(name, tensor) for every tensor of a checkpoint (or the named ones), each read
    onto `device` as it is asked for; files are opened once each"""
    from safetensors import safe_open

    mappings = get_weight_mappings(path)
    wanted = list(mappings) if names is None else list(names)
    by_file: Dict[str, list] = {}
    for name in wanted:
        if name not in mappings:
            raise KeyError(f"{name} is not in the checkpoint at {path}")
        by_file.setdefault(mappings[name], []).append(name)
    for file_name, keys in by_file.items():
        with safe_open(file_name, framework="pt", device=str(device)) as f:
            for key in keys:
                yield key, f.get_tensor(key)


class CheckpointReader:
    """random access to the tensors of a checkpoint; every file is opened once and
    tensors are read onto `device` when asked for"""

    def __init__(self, path: str, device: Union[str, torch.device] = "cpu"):
        self.mappings = get_weight_mappings(path)
        self.device = str(device)
        self._open = {}

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def close(self) -> None:
        for handle in self._open.values():
            handle.__exit__(None, None, None)
        self._open = {}

    def names(self):
        return list(self.mappings)

    def get(self, name: str) -> Tensor:
        from safetensors import safe_open

        file_name = self.mappings[name]
        if file_name not in self._open:
            self._open[file_name] = safe_open(file_name, framework="pt", device=self.device).__enter__()
        return self._open[file_name].get_tensor(name)


def save_file(tensors: Dict[str, Tensor], filename: str, metadata: Optional[Dict[str, str]] = None,
              staging_bytes: int = 64 << 20) -> None:
    """write `tensors` (on the GPU or the host) as one safetensors file"""
    if not tensors:
        raise ValueError("No tensors to save")
    items = []
    for name, t in tensors.items():
        if not isinstance(t, Tensor):
            raise ValueError(f"{name} is not a tensor")
        if t.dtype not in _DTYPE_NAMES:
            raise ValueError(f"{name}: dtype {t.dtype} has no safetensors name")
        if t.layout != torch.strided:
            raise ValueError(f"{name}: only dense tensors can be saved")
        items.append((name, t))
    # the order safetensors itself writes: by dtype (its own ranking, wide types
    # first so that every tensor starts aligned), then by name
    items.sort(key=lambda it: (-_DTYPE_RANK[it[1].dtype], it[0]))
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, t in items:
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _DTYPE_NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-len(blob) % 8)

    use_gpu = any(t.is_cuda for _, t in items)
    n_stage = 2
    if use_gpu:
        stage = [torch.empty(staging_bytes, dtype=torch.uint8, pin_memory=True) for _ in range(n_stage)]
        ready = [torch.cuda.Event() for _ in range(n_stage)]
    with open(filename, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        pending = []  # (slot, nbytes) copies in flight, in file order

        def drain(keep: int) -> None:
            while len(pending) > keep:
                slot, nbytes = pending.pop(0)
                ready[slot].synchronize()
                f.write(memoryview(stage[slot].numpy())[:nbytes])

        slot = 0
        for name, t in items:
            flat = t.detach().contiguous().reshape(-1).view(torch.uint8)
            if not flat.is_cuda:
                drain(0)
                f.write(memoryview(flat.numpy()))
                continue
            for start in range(0, flat.numel(), staging_bytes):
                piece = flat[start:start + staging_bytes]
                drain(n_stage - 1)  # the slot about to be reused has been written out
                with torch.cuda.device(piece.device):
                    stage[slot][: piece.numel()].copy_(piece, non_blocking=True)
                    ready[slot].record()
                pending.append((slot, piece.numel()))
                slot = (slot + 1) % n_stage
        if use_gpu:
            drain(0)
