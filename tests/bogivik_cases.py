"""Small Bogivik configurations for the tests, their model folders and crafted variants."""

from __future__ import annotations

import functools
import json
import tempfile
from typing import Dict

import torch

from kestrel_amd.weights import InitRecipe, write_random_model


def attention(heads, kv_heads, dim, vdim, scale, bias_max, buckets, q_temp=None, v_mix=False, ff=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "bias_max": bias_max,
             "buckets": buckets, "v_mix": v_mix}
    if q_temp is not None:
        mixer["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def parallel(left, right, ff=None):
    heads, kv_heads, dim, vdim, scale, chunk, rot_dims, base, scaling = left
    rot = {"base": base, "dims": rot_dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    r_heads, r_dim, r_vdim, cap = right
    mixer = {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": chunk}, "rot": rot},
             "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "gate_cap": cap}}
    return {"type": "parallel", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def _config(vocab, width, eps, layers):
    return {"architecture": "Bogivik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


CONFIGS: Dict[str, dict] = {
    # sizes the matrix-core kernels take; blending layers around a parallel one; a chunk of one and a half pages
    "P": _config(300, 64, 1e-5, [
        attention(4, 2, 32, 64, 0.2, 40, 16, (0.3, 5), True, 128),
        parallel((4, 2, 32, 32, 0.25, 24, 32, 10000.0, (8.0, 1.0, 4.0, 64)), (2, 16, 32, 10.0), 128),
        attention(4, 2, 32, 64, 0.2, 40, 16, (0.3, 5), True, 128),
        attention(4, 1, 32, 64, 0.15, 25, 10, (0.7, 16), False, None),
    ]),
    # sizes that fit none of the fast kernels' alignments: a parallel layer first, a chunk shorter than a page, fewer rotated
    # channels than a head has, no scaling of frequencies, as many kv heads as heads, a far distance that is no integer, a
    # period of one, a blending layer between layers that do not blend, layers without a feed-forward
    "Q": _config(211, 100, 1e-6, [
        parallel((5, 5, 24, 10, 0.3, 7, 12, 500.0, None), (3, 20, 36, 4.0), None),
        attention(5, 5, 24, 10, 0.3, 9.5, 6, (1.0, 1), True, 50),
        attention(6, 2, 20, 36, 0.25, 30, 7, None, False, 90),
        attention(10, 5, 12, 10, 0.4, 12, 9, (0.1, 3), True, None),
        parallel((3, 1, 40, 44, 0.2, 33, 40, 20.0, (2.0, 2.0, 8.0, 32)), (1, 8, 100, 30.0), 72),
    ]),
    # the largest head sizes of the matrix-core kernels, one kv head, a chunk of whole pages, values larger than keys, a far
    # distance beyond every sequence of the tests, an odd number of buckets, two parallel layers in a row
    "R": _config(190, 256, 1e-3, [
        parallel((2, 1, 128, 128, 0.09, 64, 64, 1e6, (4.0, 1.0, 2.0, 128)), (4, 64, 64, 15.0), 264),
        parallel((4, 2, 64, 96, 0.12, 48, 64, 1e4, (16.0, 0.5, 3.0, 256)), (2, 32, 128, 6.0), 264),
        attention(2, 1, 64, 128, 0.1, 400, 9, (0.5, 32), True, 264),
        attention(2, 1, 64, 128, 0.1, 400, 21, (0.5, 32), True, 264),
    ]),
    # one head everywhere, one bucket pair, one layer of each kind
    "S": _config(77, 48, 1e-5, [
        attention(1, 1, 48, 16, 0.3, 3, 2, (2.0, 7), True, 40),
        parallel((1, 1, 16, 48, 0.5, 1, 2, 3.0, None), (1, 48, 16, 1.0), 40),
    ]),
}
RECIPE = InitRecipe(std=0.08, bias_std=0.5, gain_std=0.2)
SEEDS = {"P": 21, "Q": 22, "R": 23, "S": 24}


@functools.lru_cache(maxsize=None)
def model_dir(name: str) -> str:
    folder = tempfile.mkdtemp(prefix=f"kestrel_amd_bogivik{name}_")
    write_random_model(folder, CONFIGS[name], SEEDS[name], RECIPE, store_dtype="bfloat16")
    return folder


def stored_weights(folder: str) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file

    return load_file(folder + "/model.safetensors")


def config_of(folder: str) -> dict:
    with open(folder + "/config.json") as handle:
        return json.load(handle)


def rewrite(folder: str, edit, edit_config=None) -> str:
    """A copy of a model folder whose weights went through ``edit(weights dict)`` (and its configuration through
    ``edit_config(config dict)``)."""
    from safetensors.torch import save_file

    weights = stored_weights(folder)
    edit(weights)
    config = config_of(folder)
    if edit_config is not None:
        edit_config(config)
    out = tempfile.mkdtemp(prefix="kestrel_amd_bogivik_edit_")
    save_file({k: v.contiguous() for k, v in weights.items()}, out + "/model.safetensors")
    with open(out + "/config.json", "w") as handle:
        json.dump(config, handle)
    return out
