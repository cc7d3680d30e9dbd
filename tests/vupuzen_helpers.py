"""Tiny Vupuzen configurations for the tests, and model folders made from them."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np


def _attention(heads, kv_heads, dim, vdim, bias_max, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "bias_max": bias_max,
            "scale": dim ** -0.5 if scale is None else scale}


def _retention(heads, dim, vdim, decay, rot_dims, base):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay), "rot": {"dims": rot_dims, "base": base}}


def _mlp(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


# P: attention first, grouped heads, values larger than keys, a partial rotation, one layer
# without a feed-forward, two layers that run an earlier layer's weights again.
_P_ATT = _attention(4, 2, 16, 24, 20)
_P_RET = _retention(2, 24, 8, (0.9, 0.97), 8, 10000.0)
VUPUZEN_P = {
    "architecture": "Vupuzen", "vocab": 211, "width": 64, "canon": {"taps": 4}, "norm": {"eps": 2e-5},
    "logit_scale": 0.7, "bias_rows": [12, None, None, 12, None],
    "layers": [
        {"type": "attention", "mixer": _P_ATT, "mlp": _mlp(96, 1.0)},
        {"type": "retention", "mixer": _P_RET, "mlp": None},
        {"type": "retention", "mixer": _retention(3, 8, 16, (0.5, 0.99, 1.0), 8, 500.0), "mlp": _mlp(80, 2.5)},
        {"type": "attention", "mixer": _P_ATT, "mlp": _mlp(96, 1.0), "weights_of": 0},
        {"type": "retention", "mixer": _P_RET, "mlp": None, "weights_of": 1},
    ],
}
# Q: retention first, one key/value head per query head, a head size that is no multiple of 8,
# two taps, no scaling of the logits, no rotation in one layer.
VUPUZEN_Q = {
    "architecture": "Vupuzen", "vocab": 97, "width": 48, "canon": {"taps": 2}, "norm": {"eps": 1e-6},
    "logit_scale": 1.0, "bias_rows": [None, 6, None, 8],
    "layers": [
        {"type": "retention", "mixer": _retention(1, 16, 16, (0.95,), 16, 100.0), "mlp": _mlp(64, 0.8)},
        {"type": "attention", "mixer": _attention(3, 3, 20, 12, 9.5, scale=0.3), "mlp": _mlp(64, 0.8)},
        {"type": "retention", "mixer": _retention(2, 12, 20, (0.8, 0.9), 0, 100.0), "mlp": _mlp(32, 3.0)},
        {"type": "attention", "mixer": _attention(2, 1, 32, 32, 100), "mlp": None},
    ],
}
# R: heads of the sizes of the matrix-core kernels, long enough contexts for several blocks.
VUPUZEN_R = {
    "architecture": "Vupuzen", "vocab": 160, "width": 128, "canon": {"taps": 5}, "norm": {"eps": 3e-6},
    "logit_scale": 0.25, "bias_rows": [None, 16],
    "layers": [
        {"type": "retention", "mixer": _retention(2, 64, 64, (0.96, 0.999), 32, 10000.0), "mlp": _mlp(192, 2.0)},
        {"type": "attention", "mixer": _attention(4, 2, 64, 64, 300), "mlp": _mlp(192, 2.0)},
    ],
}
CONFIGS = {"P": VUPUZEN_P, "Q": VUPUZEN_Q, "R": VUPUZEN_R}


def make_folder(tmp: Path, name: str, *, dtype: str = "float32", seed: int = 3, std: float = 0.1,
                rel_scale: float = 30.0, conv_scale: float = 4.0) -> Path:
    """A model folder of random weights in which the bias tables and the convolutions are large
    enough that a wrong bucket, a wrong tap or a lost state moves the logits."""
    import torch
    from safetensors.torch import load_file, save_file

    from pylon_amd.weights import write_random_model

    folder = write_random_model(Path(tmp) / f"vupuzen_{name}_{dtype}_{seed}", CONFIGS[name], seed, dtype=dtype,
                                std=std, norm_jitter=0.2)
    path = folder / "model.safetensors"
    tensors = load_file(str(path))
    for key in list(tensors):
        if key.endswith(".mix.rel"):
            tensors[key] = (tensors[key].float() * rel_scale).to(tensors[key].dtype)
        elif key.endswith(".canon1"):
            tensors[key] = (tensors[key].float() * conv_scale).to(tensors[key].dtype)
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
