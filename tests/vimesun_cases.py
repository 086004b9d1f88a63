"""Small Vimesun configurations for the tests, their model folders and crafted variants."""

from __future__ import annotations

import functools
import json
import tempfile
from typing import Dict

import torch

from kestrel_amd.weights import InitRecipe, write_random_model


def _layer(heads, kv_heads, dim, vdim, scale, window=None, ff=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _config(vocab, width, max_positions, eps, mult, layers, loop=None):
    out = {"architecture": "Vimesun", "vocab": vocab, "width": width, "max_positions": max_positions,
           "norm": {"eps": eps}, "residual_mult": mult, "layers": layers}
    if loop is not None:
        out["loop"] = dict(zip(("start", "stop", "times"), loop))
    return out


CONFIGS: Dict[str, dict] = {
    # equal layers, the middle one run three times; sizes the matrix-core attention kernel takes
    "P": _config(300, 64, 512, 1e-5, 0.5, [_layer(4, 2, 32, 64, 0.25, 40, 128) for _ in range(3)], (1, 2, 3)),
    # every layer different: as many kv heads as heads and values smaller than keys and a window shorter than a page
    # and no feed-forward; one kv head for eight heads with head sizes only the generic kernel takes; a window of one
    # token with equal sizes; a weight of 1 on the branches; the whole stack as one pass that runs once
    "Q": _config(211, 96, 300, 1e-6, 1.0, [_layer(2, 2, 48, 32, 0.3, 7, None), _layer(8, 1, 16, 20, 0.5, 200, 72),
                                            _layer(3, 1, 64, 64, 0.2, 1, 200)], (0, 3, 1)),
    # no loop at all, a layer without a window, a window longer than any sequence of the tests
    "R": _config(257, 128, 400, 1e-5, 0.8, [_layer(6, 3, 32, 96, 0.2, None, 152), _layer(6, 3, 32, 96, 0.2, 1000, 152)]),
    # the largest head sizes of the matrix-core kernel, a loop that ends with the stack, two passes
    "S": _config(190, 256, 320, 1e-5, 0.6, [_layer(4, 1, 128, 128, 0.09, 50, 264), _layer(2, 2, 96, 112, 0.1, 33, 264)], (1, 2, 2)),
    # sizes that fit none of the fast kernels' alignments: an odd width, head sizes that are no multiple of 8 or of 4, five
    # heads, an odd feed-forward and vocabulary; three passes over the first two layers, the stack ending outside the loop
    "T": _config(77, 100, 260, 1e-5, 0.9, [_layer(5, 5, 24, 10, 0.3, 19, 50), _layer(6, 2, 20, 36, 0.25, 64, None),
                                           _layer(1, 1, 40, 44, 0.2, 33, 90)], (0, 2, 3)),
}
RECIPE = InitRecipe(std=0.08, gain_std=0.1, shift_std=0.05)
SEEDS = {"P": 11, "Q": 12, "R": 13, "S": 14, "T": 15}


@functools.lru_cache(maxsize=None)
def model_dir(name: str) -> str:
    folder = tempfile.mkdtemp(prefix=f"kestrel_amd_vimesun{name}_")
    write_random_model(folder, CONFIGS[name], SEEDS[name], RECIPE, store_dtype="bfloat16")
    return folder


def stored_weights(folder: str) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file

    return load_file(folder + "/model.safetensors")


def config_of(folder: str) -> dict:
    with open(folder + "/config.json") as handle:
        return json.load(handle)


def rewrite(folder: str, edit) -> str:
    """A copy of a model folder whose weights went through ``edit(weights dict)``."""
    from safetensors.torch import save_file

    weights = stored_weights(folder)
    edit(weights)
    out = tempfile.mkdtemp(prefix="kestrel_amd_vimesun_edit_")
    save_file({k: v.contiguous() for k, v in weights.items()}, out + "/model.safetensors")
    with open(out + "/config.json", "w") as handle:
        json.dump(config_of(folder), handle)
    return out
