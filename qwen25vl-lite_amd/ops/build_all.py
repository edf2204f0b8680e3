"""Compile every kernel library the package can ask for."""

from __future__ import annotations

import os
from typing import List

from .library import build_library

__all__ = ["LIBRARIES", "build_everything"]

# (source stem, -D options)
LIBRARIES = [
    ("elementwise", {}),
    ("attention_generic", {}),
    ("gemm_f32", {}),
    ("sample", {}),
    ("gemm_resident", {}),
    ("gemm_resident", {"RK": 4}),
    ("gemm_split", {}),
    ("peaks", {}),
    ("gated", {}),
    ("moe", {}),
    ("rownorm", {}),
    ("short_conv", {}),
    ("latent", {}),
    # the linear-attention kernels are compiled per key size (the sizes the tests and the benchmark
    # use; any other size up to 512 is compiled at its first use)
    *[("linear_attention", {"LA_DIM": d}) for d in (5, 6, 8, 12, 16, 20, 32, 64, 128, 320)],
    # the matrix-core attention is compiled per head size; these are the sizes the tests and the
    # benchmark use, any other multiple of 16 is compiled at its first use
    ("attention_mfma", {"HD": 128}),
    ("attention_mfma", {"HD": 16}),
    ("attention_mfma", {"HD": 48}),
    ("attention_mfma", {"HD": 80}),
    ("attention_mfma", {"HD": 256}),
    ("attention_mfma", {"HD": 32}),
    ("attention_mfma", {"HD": 64}),
    ("attention_mfma", {"HD": 96}),
    ("attention_mfma", {"HD": 112}),
    # the matrix-core attention for windows that keep the first keys is compiled per key and value size
    ("attention_window", {"HD": 128, "VD": 128}),
    ("attention_window", {"HD": 16, "VD": 24}),
    ("attention_window", {"HD": 48, "VD": 16}),
    ("attention_window", {"HD": 16, "VD": 16}),
    ("attention_window", {"HD": 64, "VD": 32}),
    ("attention_window", {"HD": 8, "VD": 8}),
    # one key/value head whose values are the first channels of its keys (attention through a latent)
    ("attention_window", {"HD": 32, "VD": 24}),
    ("attention_window", {"HD": 56, "VD": 40}),
    ("attention_window", {"HD": 32, "VD": 16}),
    ("attention_window", {"HD": 24, "VD": 16}),
    ("attention_window", {"HD": 128, "VD": 64}),
    ("attention_window", {"HD": 40, "VD": 24}),
    ("attention_window", {"HD": 256, "VD": 192}),
    ("attention_window", {"HD": 48, "VD": 40}),
    ("attention_window", {"HD": 24, "VD": 24}),
    ("attention_window", {"HD": 8, "VD": 12}),
    # the kind whose waves carry three column tiles (long prompts)
    ("attention_mfma", {"HD": 128, "BLK_CT": 3}),
    ("attention_mfma", {"HD": 48, "BLK_CT": 3}),
]


def build_everything(force: bool = False, quiet: bool = False) -> List[str]:
    built = [build_library(stem, defines, force=force, quiet=quiet) for stem, defines in LIBRARIES]
    # libraries of sources that have changed since are of no use to anyone
    keep = {os.path.basename(p) for p in built}
    for directory in {os.path.dirname(p) for p in built}:
        for name in os.listdir(directory):
            if name.endswith(".so") and name not in keep:
                os.remove(os.path.join(directory, name))
    return built
