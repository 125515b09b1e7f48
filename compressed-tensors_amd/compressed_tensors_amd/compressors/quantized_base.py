"""State-dict harness shared by the quantization compressors.

Mirrors BaseQuantizationCompressor (reference:
compressors/quantized_compressors/base.py:69-258): a tensor named `*weight`
with a sibling `*weight_scale` is compressed with the scheme registered for
its module; symmetric or packed zero points are dropped; everything else is
passed through.  Results stay on the GPU unless `compression_device` says
otherwise.
"""
from pathlib import Path
from typing import Any, Dict, Generator, Optional, Tuple, Union

import torch
from torch import Tensor

from compressed_tensors_amd.compressors.base import BaseCompressor, to_gpu
from compressed_tensors_amd.quantization.quant_args import QuantizationStrategy
from compressed_tensors_amd.utils.helpers import nest_state_dict
from compressed_tensors_amd.utils.safetensors_io import CheckpointReader, get_nested_weight_mappings

__all__ = ["BaseQuantizationCompressor", "LazyDenseOutputs", "own_parameters", "swap_parameters"]

_PACKABLE = (QuantizationStrategy.GROUP.value, QuantizationStrategy.CHANNEL.value)


def _move(t: Tensor, device) -> Tensor:
    return t if device is None else t.to(device)


def own_parameters(module: torch.nn.Module, prefix: str) -> Dict[str, Tensor]:
    """the module's own parameters under their state-dict names"""
    return {f"{prefix}.{n}": p.data for n, p in module._parameters.items() if p is not None}


def swap_parameters(module: torch.nn.Module, prefix: str, state: Dict[str, Tensor]) -> None:
    """replace the module's own parameters by the entries of `state` (full names).  Slots that
    hold no parameter (the `bias` of a Linear made with bias=False) stay registered as they
    are: forward reads them."""
    params = module._parameters
    for name in [n for n, p in params.items() if p is not None]:
        del params[name]
    cut = len(prefix) + 1
    for name, value in state.items():
        local = name[cut:] if name.startswith(prefix + ".") else name
        params[local] = value if isinstance(value, torch.nn.Parameter) else torch.nn.Parameter(
            value, requires_grad=False)


class LazyDenseOutputs:
    """The dense (decompressed) side of a weight batch, allocated when it is first
    needed: a batch that only ever compresses (the state-dict path) never holds a
    second dense copy of the model.  The batch records one (shape, dtype, device)
    per weight with `_plan_dense`; `dense` / `_ensure_dense` allocate the tensors
    and write their addresses into the decompress job table (`field` names the
    destination member of the job struct)."""

    _dense = None
    _dense_field = "dst"

    def _plan_dense(self, shape, dtype, device):
        if not hasattr(self, "_dense_specs"):
            self._dense_specs = []
        self._dense_specs.append((tuple(shape), dtype, device))

    def _ensure_dense(self):
        if self._dense is None:
            specs = getattr(self, "_dense_specs", [])
            self._dense = [torch.empty(shape, dtype=dtype, device=device)
                           for shape, dtype, device in specs]
            for i, t in enumerate(self._dense):
                self._finish_decompress_job(i)
                setattr(self._djobs[i], self._dense_field, t.data_ptr())
        return self._dense

    def _finish_decompress_job(self, i):
        """hook: whatever else of decompress job i was left for the first decompress()"""

    @property
    def dense(self):
        return self._ensure_dense()


class BaseQuantizationCompressor(BaseCompressor):
    # set by PackedQuantizationCompressor: its group/channel zero points are re-emitted packed
    packs_zero_points = False

    def compress(
        self,
        model_state: Dict[str, Tensor],
        names_to_scheme: Dict[str, Any],
        show_progress: bool = False,
        compression_device: Optional[str] = None,
        **kwargs,
    ) -> Dict[str, Tensor]:
        compressed: Dict[str, Tensor] = {}
        for name in list(model_state.keys()):
            value = model_state[name]
            if name.endswith("weight"):
                prefix = name[: -len("weight")]
                scale = model_state.get(prefix + "weight_scale", None)
                if scale is None:
                    compressed[name] = _move(value, compression_device)
                    continue
                module_path = prefix[:-1] if prefix.endswith(".") else prefix
                quant_args = names_to_scheme[module_path].weights
                out = self.compress_weight(
                    weight=value,
                    scale=scale,
                    zero_point=model_state.get(prefix + "weight_zero_point", None),
                    global_scale=model_state.get(prefix + "weight_global_scale", None),
                    g_idx=model_state.get(prefix + "weight_g_idx", None),
                    quantization_args=quant_args,
                    device=compression_device,
                )
                for key, tensor in out.items():
                    compressed[prefix + key] = _move(tensor, compression_device)
            else:
                if name.endswith("zero_point") and self._skip_zp(name, names_to_scheme):
                    continue
                compressed[name] = _move(value, compression_device)
        return compressed

    def _skip_zp(self, name: str, names_to_scheme: Dict[str, Any]) -> bool:
        module_name, zp_name = name.rsplit(".", 1) if "." in name else ("", name)
        scheme = names_to_scheme[module_name]
        args = {
            "weight_zero_point": getattr(scheme, "weights", None),
            "input_zero_point": getattr(scheme, "input_activations", None),
            "output_zero_point": getattr(scheme, "output_activations", None),
        }[zp_name]
        packed = self.packs_zero_points and args.strategy in _PACKABLE
        return args.symmetric or packed

    def decompress(
        self,
        path_to_model_or_tensors: Union[str, Path, Dict[str, Any]],
        names_to_scheme: Dict[str, Any],
        device: str = "cpu",
    ) -> Generator[Tuple[str, Dict[str, Tensor]], None, None]:
        if not isinstance(path_to_model_or_tensors, (str, Path)):
            yield from self.decompress_from_state_dict(path_to_model_or_tensors, names_to_scheme)
            return
        # one module at a time: only its compression parameters are in memory
        # (quantized_compressors/base.py:186-220)
        path = str(path_to_model_or_tensors)
        nested = get_nested_weight_mappings(path, self.compression_param_names)
        with CheckpointReader(path, device=device) as reader:
            for module_path, params in nested.items():
                if "weight_scale" not in params:
                    continue
                weight_data = {name: reader.get(f"{module_path}.{name}") for name in params}
                quant_args = names_to_scheme[module_path].weights
                weight_data["weight"] = self.decompress_weight(
                    compressed_data=weight_data, quantization_args=quant_args
                )
                yield module_path, weight_data

    def decompress_from_state_dict(
        self, state_dict: Dict[str, Tensor], names_to_scheme: Dict[str, Any]
    ) -> Generator[Tuple[str, Dict[str, Tensor]], None, None]:
        nested = nest_state_dict(state_dict, self.compression_param_names)
        todo = [(module_path, dict(weight_data)) for module_path, weight_data in nested.items()
                if "weight_scale" in weight_data]
        # every weight of the state dict in many-weight calls where the format has them: the
        # kernels are enqueued before the first module is handed back
        dense = self.decompress_weights(
            [(weight_data, names_to_scheme[module_path].weights) for module_path, weight_data in todo])
        for (module_path, weight_data), weight in zip(todo, dense):
            weight_data["weight"] = weight
            yield module_path, weight_data

    def decompress_weights(self, items) -> list:
        """decompress_weight for a list of (compressed_data, quantization_args) pairs;
        formats with a multi-weight entry point in the C ABI override this with one call"""
        return [self.decompress_weight(compressed_data=data, quantization_args=args)
                for data, args in items]

    # ----- module pathways: what ModelCompressor.compress_model / decompress_model call ----- #
    def compress_modules(self, members, names_to_scheme: Dict[str, Any]) -> None:
        """compress_module (compressors/base.py:125-151) for every (prefix, module) pair of
        `members`, the modules' parameters replaced by the compressed ones: all weights go
        through one state-dict call (one many-weight call of the C ABI where the format has one)"""
        state: Dict[str, Tensor] = {}
        for prefix, module in members:
            state.update(own_parameters(module, prefix))
        state = self.compress(state, names_to_scheme=names_to_scheme, show_progress=False)
        per_module: Dict[str, Dict[str, Tensor]] = {prefix: {} for prefix, _ in members}
        for name, value in state.items():
            per_module[name.rpartition(".")[0]][name] = value
        for prefix, module in members:
            swap_parameters(module, prefix, per_module[prefix])

    def decompress_modules(self, members, names_to_scheme: Dict[str, Any]) -> None:
        """decompress_module (compressors/base.py:165-190) for every (prefix, module) pair,
        the dense weight put next to the module's other parameters"""
        local = [{n: p.data for n, p in module._parameters.items() if p is not None}
                 for _, module in members]
        todo = [i for i, data in enumerate(local) if "weight_scale" in data]
        dense = self.decompress_weights(
            [(local[i], names_to_scheme[members[i][0]].weights) for i in todo])
        for i, weight in zip(todo, dense):
            local[i]["weight"] = weight
        for (prefix, module), data in zip(members, local):
            swap_parameters(module, prefix, {f"{prefix}.{k}": v for k, v in data.items()})

    def decompress_module_from_state_dict(
        self, prefix: str, state_dict: Dict[str, Tensor], scheme: Any
    ) -> Dict[str, Tensor]:
        local = {
            (k[len(prefix) + 1 :] if k.startswith(prefix + ".") else k): v
            for k, v in state_dict.items()
        }
        if "weight_scale" in local:
            local["weight"] = self.decompress_weight(
                compressed_data=local, quantization_args=scheme.weights
            )
        return {f"{prefix}.{k}": v for k, v in local.items()}


def gpu_args(*tensors):
    return tuple(to_gpu(t) for t in tensors)
