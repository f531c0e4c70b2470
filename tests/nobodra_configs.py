"""Small Nobodra configurations of the tests' own, differing from each other in every size, constant and layer order."""

from __future__ import annotations

import json
from pathlib import Path


def experts(ff, count, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": count, "top": top}}


def attention(heads, kv_heads, dim, scale, window=None, rot=None, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if window is not None:
        mixer["mask"] = {"size": window}
    if rot is not None:
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def delta(heads, kv_heads, dim, vdim, conv, mlp=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def model(vocab, width, eps, layers):
    return {"architecture": "Nobodra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


# routed experts (a few of several), part of a head rotated, windows shorter than the prompts, three heads to a key group
ROUTED = model(211, 64, 1e-5, [
    delta(4, 2, 32, 16, 4, experts(48, 6, 2)),
    attention(6, 2, 32, 0.21, window=24, rot=(10000.0, 16), mlp=experts(48, 6, 2)),
    attention(4, 4, 16, 0.3, window=7, rot=(500.0, 8), mlp=experts(40, 5, 3)),
    delta(2, 1, 24, 40, 2, experts(48, 6, 1)),
])
# every expert runs for every token (no choice to differ in), a layer without feed-forward, whole heads rotated, one without
# rotation and one without window, a convolution of one tap, more experts than a wave has lanes
DENSE = model(157, 96, 3e-6, [
    attention(2, 2, 64, 0.11, window=40, rot=(200000.0, 64), mlp=experts(32, 3, 3)),
    delta(3, 3, 20, 28, 3, None),
    attention(4, 1, 32, 0.2, window=None, rot=None, mlp=experts(24, 70, 70)),
    delta(2, 2, 64, 64, 1, experts(64, 2, 2)),
    attention(8, 2, 16, 0.25, window=1, rot=(100.0, 2), mlp=None),
])
# sizes the matrix-core kernels take: heads of 128 and 64, experts of 64 and 128 columns, a width of 128
CORES = model(300, 128, 1e-6, [
    attention(4, 2, 128, 0.09, window=100, rot=(1e6, 128), mlp=experts(64, 8, 8)),
    delta(2, 1, 128, 128, 4, experts(128, 4, 4)),
    attention(8, 4, 64, 0.125, window=33, rot=(1e4, 32), mlp=experts(64, 8, 8)),
])
# wide enough that prompts go through the products for many rows (the vendor library's, the grouped product with large tiles)
WIDE = model(1000, 512, 1e-6, [
    delta(8, 4, 64, 64, 4, experts(256, 8, 2)),
    attention(8, 2, 64, 0.12, window=150, rot=(1e5, 32), mlp=experts(256, 4, 4)),
    delta(4, 4, 128, 128, 2, None),
])


def write_folder(raw: dict, seed: int, folder, edit=None) -> Path:
    """A model folder with random weights for `raw`; edit(tensors) may change them before they are written."""
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    folder = Path(folder)
    write_model_dir(config_from_dict(raw), seed=seed, model_dir=folder, init="scaled")
    assert json.loads((folder / "config.json").read_text()) == raw
    if edit is not None:
        from safetensors.torch import load_file, save_file

        tensors = load_file(str(folder / "model.safetensors"))
        edit(tensors)
        save_file({name: t.contiguous() for name, t in tensors.items()}, str(folder / "model.safetensors"))
    return folder
