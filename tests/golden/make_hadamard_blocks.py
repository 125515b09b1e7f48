"""Writes tests/golden/hadamard_blocks.safetensors: the known Hadamard matrices H_K that the
sizes of the reference's own Hadamard tests end in (tests/test_transform/utils/
test_hadamard.py:26-39: 768 -> K = 192, 1280 -> 160, 1600 -> 200, 3584 / 7168 / 14336 -> 224,
3840 -> 240, 18432 -> 144, 18944 -> 148), plus 12, 20, 28 (small enough for brute-force
checks) and 32 (the one power of two whose entry is not Sylvester's matrix).

The matrices are data of the reference (src/compressed_tensors/transform/utils/
hadamards.safetensors), read here with safetensors, which executes nothing from the file;
no reference code is imported or run.  Each K x K matrix of +-1 is stored bit-packed:
key str(K) -> uint8 [K, ceil(K / 8)], bit 7 of byte 0 = column 0, a set bit = +1
(numpy.packbits order).  tests/conftest.py unpacks them.

    python tests/golden/make_hadamard_blocks.py [path/to/hadamards.safetensors]
"""
import sys
from pathlib import Path

import numpy as np
import torch
from safetensors import safe_open
from safetensors.torch import save_file

KEYS = (12, 20, 28, 32, 144, 148, 160, 192, 200, 224, 240)
DEFAULT = "/root/reference/src/compressed_tensors/transform/utils/hadamards.safetensors"


def main() -> None:
    source = sys.argv[1] if len(sys.argv) > 1 else DEFAULT
    packed = {}
    with safe_open(source, framework="pt", device="cpu") as f:
        for k in KEYS:
            h = f.get_tensor(str(k)).to(torch.int64)
            assert tuple(h.shape) == (k, k) and bool((h.abs() == 1).all()), k
            assert torch.equal(h @ h.T, k * torch.eye(k, dtype=torch.int64)), k
            bits = np.packbits((h > 0).numpy().astype(np.uint8), axis=1)
            packed[str(k)] = torch.from_numpy(bits.copy())
    out = Path(__file__).parent / "hadamard_blocks.safetensors"
    save_file(packed, str(out))
    print(out, out.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
