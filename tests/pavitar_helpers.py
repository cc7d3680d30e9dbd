"""Tiny Pavitar configurations for the tests, and model folders made from them."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np


def _attention(heads, kv_heads, dim, vdim, rot_dims, base, size, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size},
            "rot": {"dims": rot_dims, "base": base}, "scale": dim ** -0.5 if scale is None else scale}


def _latent(heads, dim, vdim, q_rank, kv_rank, size, scale=None):
    return {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "mask": {"size": size},
            "scale": dim ** -0.5 if scale is None else scale}


def _moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


# U: attention first, grouped heads, values larger than keys, a partial rotation, tiny chunks and
# windows (so that every prompt crosses many edges), a layer without a feed-forward, a stretch of
# two layers that runs three times.
PAVITAR_U = {
    "architecture": "Pavitar", "vocab": 211, "width": 64, "norm": {"eps": 2e-5}, "logit_softcap": 8.0,
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "attention", "mixer": _attention(4, 2, 16, 24, 8, 1000.0, 7, scale=0.3), "mlp": _moe(5, 2, 24, 40)},
        {"type": "latent_attention", "mixer": _latent(3, 12, 20, 24, 40, 9), "mlp": None},
        {"type": "attention", "mixer": _attention(2, 1, 20, 8, 20, 50.0, 5), "mlp": _moe(4, 4, 16, 8)},
        {"type": "latent_attention", "mixer": _latent(2, 8, 8, 16, 24, 4, scale=0.5), "mlp": _moe(7, 3, 8)},
    ],
}
# V: latent attention first, one key/value head per query head, a rotation of the whole head, one
# expert a token, no shared expert, no loop, no cap; a head size that is no multiple of 8; a
# window of one key (a token sees itself alone).
PAVITAR_V = {
    "architecture": "Pavitar", "vocab": 97, "width": 48, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "latent_attention", "mixer": _latent(1, 20, 12, 8, 16, 13), "mlp": _moe(3, 1, 32)},
        {"type": "attention", "mixer": _attention(3, 3, 12, 12, 12, 10000.0, 16), "mlp": _moe(2, 1, 40, 24)},
        {"type": "latent_attention", "mixer": _latent(5, 4, 6, 12, 8, 1), "mlp": None},
        {"type": "attention", "mixer": _attention(2, 2, 10, 6, 0, 10.0, 1000), "mlp": _moe(6, 2, 8, 16)},
    ],
}
# W: heads and latents of the sizes that the matrix-core attention kernels take, twenty heads over
# one latent (handed to the decode kernel in two groups), contexts of several blocks; the looped
# stretch is the whole model.
PAVITAR_W = {
    "architecture": "Pavitar", "vocab": 160, "width": 128, "norm": {"eps": 3e-6}, "logit_softcap": 30.0,
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        {"type": "attention", "mixer": _attention(4, 2, 64, 64, 32, 10000.0, 70), "mlp": _moe(6, 4, 48, 96)},
        {"type": "latent_attention", "mixer": _latent(20, 32, 32, 64, 64, 100), "mlp": _moe(6, 4, 48, 96)},
    ],
}
# X: a head size and a latent of 128 numbers (with pages of 64 tokens: the prefill kernel that
# loads blocks of a page straight into LDS), a loop of one pass.
PAVITAR_X = {
    "architecture": "Pavitar", "vocab": 131, "width": 96, "norm": {"eps": 1e-5}, "logit_softcap": 12.0,
    "loop": {"start": 1, "stop": 2, "times": 1},
    "layers": [
        {"type": "latent_attention", "mixer": _latent(4, 48, 16, 40, 128, 90), "mlp": _moe(9, 2, 32, 32)},
        {"type": "attention", "mixer": _attention(3, 1, 128, 128, 64, 500000.0, 150), "mlp": None},
    ],
}
CONFIGS = {"U": PAVITAR_U, "V": PAVITAR_V, "W": PAVITAR_W, "X": PAVITAR_X}


def make_folder(tmp: Path, name: str, *, dtype: str = "float32", seed: int = 3, std: float = 0.12,
                router_scale: float = 6.0, config=None) -> Path:
    """A model folder of random weights in which routers are scaled up after drawing (clear
    choices: the tests do not rest on close calls) and norm weights differ from their rest value."""
    from safetensors.torch import load_file, save_file

    from pylon_amd.weights import write_random_model

    folder = write_random_model(Path(tmp) / f"pavitar_{name}_{dtype}_{seed}", config or CONFIGS[name], seed,
                                dtype=dtype, std=std, norm_jitter=0.2)
    path = folder / "model.safetensors"
    tensors = load_file(str(path))
    for key in list(tensors):
        if key.endswith(".mlp.router") or key.endswith(".mlp.router.b"):
            tensors[key] = (tensors[key].float() * router_scale).to(tensors[key].dtype)
    save_file(tensors, str(path))
    return folder


def read_folder(folder: Path):
    import torch
    from safetensors.torch import load_file

    cfg = json.loads((Path(folder) / "config.json").read_text())
    weights = {name: t.to(torch.float64).numpy() for name, t in load_file(str(Path(folder) / "model.safetensors")).items()}
    return cfg, weights


def tokens(vocab: int, count: int, seed: int):
    return np.random.default_rng(seed).integers(0, vocab, count).tolist()
