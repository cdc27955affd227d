"""Small Taluvik configurations for the tests, and model folders with random weights made from them.

The configurations differ from each other in every size and constant, and in what a single model may
happen to make equal: heads and key heads, head sizes of keys and values, rotated channels and head
size, chunks that are and are not multiples of a page, states that one lane or several hold, layers
with and without a feed-forward, layers that use another layer's tensors."""

from __future__ import annotations

from pathlib import Path
from typing import Dict

import torch


def attention(heads, kv_heads, dim, vdim, rot_dims, chunk, scale, softcap, base=10000.0, scaling=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
            "mask": {"size": chunk}, "rot": {"dims": rot_dims, "base": base, "scaling": scaling}}


def layer(kind, mixer, ff=None, weights_of=None):
    d = {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


_ATT_A = attention(4, 2, 32, 16, 16, 24, 0.3, 20.0)
_DELTA_A = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "conv": 4}
_MAMBA_A = {"inner": 96, "state": 16, "dt_rank": 8, "conv": 4}
CONFIG_A = {
    "architecture": "Taluvik", "vocab": 131, "width": 64, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-5},
    "residual_mult": 0.7,
    "layers": [
        layer("attention", _ATT_A, ff=80),
        layer("delta", _DELTA_A, ff=48),
        layer("mamba1", _MAMBA_A, ff=80),
        layer("attention", _ATT_A, ff=80, weights_of=0),
        layer("mamba1", _MAMBA_A, ff=80, weights_of=2),
        layer("delta", {"heads": 2, "kv_heads": 2, "dim": 24, "vdim": 24, "conv": 2}),
    ],
}

_ATT_B = attention(6, 6, 48, 48, 48, 64, 0.2, 50.0, base=500000.0,
                   scaling={"factor": 8.0, "low": 1.0, "high": 4.0, "original": 32})
CONFIG_B = {
    "architecture": "Taluvik", "vocab": 77, "width": 96, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
    "residual_mult": 1.0,
    "layers": [
        layer("mamba1", {"inner": 80, "state": 40, "dt_rank": 5, "conv": 2}),
        layer("delta", {"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 48, "conv": 3}, ff=112),
        layer("attention", _ATT_B),
        layer("delta", {"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 48, "conv": 3}, ff=112, weights_of=1),
    ],
}

CONFIG_C = {
    "architecture": "Taluvik", "vocab": 200, "width": 128, "embedding": {"scale": 11.0}, "norm": {"eps": 1e-5},
    "residual_mult": 0.4,
    "layers": [
        layer("attention", attention(2, 1, 128, 64, 64, 40, 0.09, 8.0, base=1000.0), ff=96),
        layer("mamba1", {"inner": 128, "state": 8, "dt_rank": 16, "conv": 5}, ff=96),
        layer("delta", {"heads": 2, "kv_heads": 2, "dim": 128, "vdim": 128, "conv": 3}, ff=96),
        layer("attention", attention(8, 2, 16, 24, 0, 7, 1.0, 3.0), ff=64),
    ],
}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C}
PAGE_SIZE = {"A": 8, "B": 16, "C": 4}


def single_layer(entry: dict, width: int = 64, vocab: int = 61) -> dict:
    """A model of one layer, for a mechanism alone."""
    return {"architecture": "Taluvik", "vocab": vocab, "width": width, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5},
            "residual_mult": 1.0, "layers": [entry]}


def make_folder(path, cfg_dict: dict, seed: int = 0, dtype=torch.bfloat16) -> Path:
    """A model folder written by the package's random-weights mode, then made harder on faults: the
    sinks get a spread of about one (N(0, 0.02) would make a forgotten sink invisible), the projections
    into queries, keys, values and the recurrences' inputs are scaled up so that mixers weigh as much as
    the feed-forward beside them, and the step sizes and decays get a spread."""
    from safetensors.torch import save_file

    from torchllms_amd.config import TaluvikConfig
    from torchllms_amd.weights import write_model_folder

    folder = write_model_folder(path, TaluvikConfig.from_dict(cfg_dict), seed=seed, dtype=dtype, norm_jitter=0.1)
    _, tensors = read_folder(folder)
    gen = torch.Generator().manual_seed(seed + 1)
    for name in list(tensors):
        t = tensors[name].float()
        leaf = name.split(".", 2)[-1] if name.startswith("l") else name
        if leaf == "mix.sink":
            t = torch.randn(t.shape, generator=gen)
        elif leaf in ("mix.A_log", "mix.dt_bias", "mix.dt.b"):
            t = t + 0.5 * torch.randn(t.shape, generator=gen)
        elif leaf in ("mix.q", "mix.k", "mix.v", "mix.in", "mix.x", "mix.b", "mix.a", "mix.g", "mix.o"):
            t = t * 5.0
        tensors[name] = t.to(dtype)
    save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt"})
    return folder


def read_folder(folder) -> (dict, Dict[str, torch.Tensor]):
    """config.json as a dict and the tensors by their checkpoint names, read with safetensors
    directly (not through the package's loader)."""
    import json

    from safetensors import safe_open

    folder = Path(folder)
    with open(folder / "config.json") as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return cfg, tensors
