"""Small Sebesun configurations for the tests, with sharpened random weights, and helpers around them.

The configurations differ from each other in every size, in the order and number of layers and in which layers have
a feed-forward; between them they cover a rotation over part of the key size and over all of it and none at all, one
kv head per head and one kv head for all, a single head, value sizes below and above the key size, key sizes that are
no power of two, convolutions of 1, 2 and 4 taps, a step-size rank of 1, and a layer kind as first, middle and last.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch

from palm_infra_amd.config import config_from_dict
from palm_infra_amd.weights import random_tensors, write_safetensors


def _ret(heads, dim, vdim, decay, rot):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay, "rot": rot}}


def _att(heads, kv, dim, vdim, scale, diff):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}}


def _scan(inner, state, rank, conv):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": rank, "conv": conv}}


def _with(layer, ff):
    return dict(layer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


CONFIGS = {
    "P": {"architecture": "Sebesun", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "layers": [
        _with(_att(4, 2, 16, 40, 0.5, 0.35), 96),
        _with(_ret(2, 16, 24, [0.9, 0.97], {"dims": 8, "base": 10000.0}), None),
        _with(_scan(96, 8, 5, 4), 80),
        _with(_ret(3, 8, 32, [0.99, 0.5, 0.996], {"dims": 8, "base": 500.0}), 72),
    ]},
    "Q": {"architecture": "Sebesun", "vocab": 130, "width": 48, "norm": {"eps": 2e-6}, "layers": [
        _with(_scan(40, 17, 1, 2), None),
        _with(_att(3, 3, 24, 20, 0.1, 0.8), None),
        _with(_ret(1, 24, 80, [0.995], None), None),
        _with(_att(2, 1, 8, 72, 0.3, 0.2), 56),
        _with(_scan(72, 33, 9, 1), None),
    ]},
    "R": {"architecture": "Sebesun", "vocab": 97, "width": 40, "norm": {"eps": 1e-6}, "layers": [
        _with(_ret(2, 32, 48, [0.999, 0.98], {"dims": 32, "base": 250000.0}), 64),
    ]},
}
SEEDS = {"P": 11, "Q": 12, "R": 13}
# one layer of one kind, for the tests of a mechanism alone
SINGLE = {
    "retention": {"architecture": "Sebesun", "vocab": 90, "width": 32, "norm": {"eps": 1e-6},
                  "layers": [_with(_ret(2, 12, 20, [0.96, 0.9], {"dims": 6, "base": 100.0}), None)]},
    "mamba1": {"architecture": "Sebesun", "vocab": 90, "width": 32, "norm": {"eps": 1e-6},
               "layers": [_with(_scan(48, 6, 3, 3), None)]},
    "attention": {"architecture": "Sebesun", "vocab": 90, "width": 32, "norm": {"eps": 1e-6},
                  "layers": [_with(_att(2, 1, 12, 28, 0.4, 0.5), None)]},
    "feed_forward": {"architecture": "Sebesun", "vocab": 90, "width": 32, "norm": {"eps": 1e-6},
                     "layers": [_with(_scan(16, 2, 2, 2), 100)]},
}


def sharpened_tensors(raw: dict, seed: int, store: str) -> dict:
    """The random-weights mode's numbers, made larger so that faults show: matrices four times (logits and branch
    inputs of order one), the q norm's weight three times (scores of order one and more), the two numbers of the
    activation and the step sizes' bias as they are."""
    tensors = random_tensors(config_from_dict(raw).spec(), seed, "float32")
    out = {}
    for k, t in tensors.items():
        if t.dim() == 2 and not k.endswith(("conv", "A_log")):
            t = t * 4.0
        elif k.endswith("q.norm"):
            t = t * 3.0
        out[k] = t.to({"bfloat16": torch.bfloat16, "float32": torch.float32}[store])
    return out


def write_model(raw: dict, seed: int, path, store: str) -> Path:
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(raw))
    write_safetensors(path / "model.safetensors", sharpened_tensors(raw, seed, store))
    return path


def prompts(raw: dict, lengths, seed: int = 0) -> list:
    g = torch.Generator().manual_seed(2000 + seed)
    return [torch.randint(0, raw["vocab"], (n,), generator=g).tolist() for n in lengths]
