"""State-dict harness shared by the sparsity compressors.

Mirrors BaseSparseCompressor (reference: compressors/sparse_compressors/base.py:66-202):
only entries named `*.weight` (and, if given, listed in compression_targets)
are compressed; the key prefix of the emitted entries is the name without
`.weight`.
"""
from typing import Dict, Generator, Optional, Set, Tuple

from torch import Tensor

from compressed_tensors_amd.compressors.base import BaseCompressor
from compressed_tensors_amd.utils.helpers import merge_names, nest_state_dict
from compressed_tensors_amd.utils.safetensors_io import CheckpointReader, get_nested_weight_mappings

__all__ = ["BaseSparseCompressor"]


class BaseSparseCompressor(BaseCompressor):
    # device the emitted tensors are moved to; None leaves them on the GPU
    # (the reference always returns host tensors)
    output_device = None

    def compress(
        self,
        model_state: Dict[str, Tensor],
        compression_targets: Optional[Set[str]] = None,
        show_progress: bool = False,
    ) -> Dict[str, Tensor]:
        out: Dict[str, Tensor] = {}
        for name, value in model_state.items():
            if not self.should_compress(name, compression_targets):
                out[name] = value
                continue
            prefix = name[: -len(".weight")] if name.endswith(".weight") else name
            out.update(self.compress_weight(prefix, value))
        return out

    def decompress(
        self,
        path_to_model_or_tensors,
        device: str = "cpu",
        params_to_skip_load: Optional[Tuple] = None,
        **kwargs,
    ) -> Generator[Tuple[str, Tensor], None, None]:
        if isinstance(path_to_model_or_tensors, dict):
            _, ignored = nest_state_dict(
                path_to_model_or_tensors, self.compression_param_names, return_unmatched_params=True
            )
            # through decompress_from_state_dict, which formats with a multi-tensor entry
            # point in the C ABI override
            for name, value in self.decompress_from_state_dict(path_to_model_or_tensors):
                if (name in ignored and params_to_skip_load is not None
                        and any(p in name for p in params_to_skip_load)):
                    continue
                yield name, value
            return
        # one module at a time from the files (sparse_compressors/base.py:114-152)
        path = str(path_to_model_or_tensors)
        nested, ignored = get_nested_weight_mappings(
            path, self.compression_param_names, return_unmatched_params=True
        )
        with CheckpointReader(path, device=device) as reader:
            for module_path, params in nested.items():
                weight_data = {name: reader.get(merge_names(module_path, name)) for name in params}
                yield merge_names(module_path, "weight"), self.decompress_weight(weight_data)
            for name in ignored:
                if params_to_skip_load is not None and any(p in name for p in params_to_skip_load):
                    continue
                yield name, reader.get(name)

    def decompress_from_state_dict(
        self, state_dict: Dict[str, Tensor]
    ) -> Generator[Tuple[str, Tensor], None, None]:
        nested, ignored = nest_state_dict(
            state_dict, self.compression_param_names, return_unmatched_params=True
        )
        for module_path, weight_data in nested.items():
            yield merge_names(module_path, "weight"), self.decompress_weight(dict(weight_data))
        for name, value in ignored.items():
            yield name, value

    @staticmethod
    def should_compress(name: str, expanded_targets: Optional[Set[str]] = None) -> bool:
        if expanded_targets is None:
            return name.endswith(".weight")
        return name.endswith(".weight") and name[: -len(".weight")] in expanded_targets
