"""Small Pazilorn configurations for the tests, with sharpened random weights, and helpers around them.

The configurations differ from each other in every size, in the order and number of layers, in which layers have a
feed-forward and in which borrow another layer's weights; between them they cover q/k heads shared by several heads and one
each, a single head, key sizes on both sides of a wave's quarter and no power of two, value sizes that are no whole number
of waves, convolutions of 1, 2 and 4 taps, low ranks of 1, latents below and above 64 values, windows below and above a
page and none at all, frequencies stretched and plain, one expert a token, all experts a token, a multiplier and a scale of
1, and no cap on the logits.
"""
from __future__ import annotations

import json
from pathlib import Path

import torch

from palm_infra_amd.config import config_from_dict
from palm_infra_amd.weights import random_tensors, write_safetensors


def _delta(heads, kv, dim, vdim, conv, ra, rg):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv,
                                               "decay_rank": ra, "gate_rank": rg}}


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, window, base, scaling=None):
    return {"type": "latent_attention", "mixer": {
        "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
        "mask": {"size": window} if window else None, "rot": {"dims": rot_dim, "base": base, "scaling": scaling}}}


def _with(layer, ff=None, experts=0, top=0, weights_of=None):
    out = dict(layer, mlp=None if ff is None else {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}})
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


_YARN = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}

CONFIGS = {
    "A": {"architecture": "Pazilorn", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
          "embedding": {"scale": 6.0}, "logit_softcap": 8.0, "layers": [
              _with(_delta(4, 2, 16, 24, 4, 5, 7), 40, 6, 2),
              _with(_latent(3, 24, 8, 20, 40, 48, 0.25, 37, 10000.0, _YARN)),
              _with(_delta(4, 2, 16, 24, 4, 5, 7), 40, 6, 2, weights_of=0),
              _with(_latent(3, 24, 8, 20, 40, 48, 0.25, 37, 10000.0, _YARN), weights_of=1),
          ]},
    "B": {"architecture": "Pazilorn", "vocab": 130, "width": 48, "norm": {"eps": 2e-6}, "residual_mult": 1.0,
          "embedding": {"scale": 1.0}, "logit_softcap": 30.0, "layers": [
              _with(_latent(1, 16, 16, 72, 96, 24, 0.3, 70, 500.0), 24, 3, 3),
              _with(_delta(2, 1, 40, 72, 2, 1, 3)),
              _with(_delta(3, 3, 8, 16, 1, 4, 1), 56, 5, 1),
          ]},
    "C": {"architecture": "Pazilorn", "vocab": 97, "width": 40, "norm": {"eps": 1e-6}, "residual_mult": 0.2,
          "embedding": {"scale": 12.0}, "logit_softcap": None, "layers": [
              _with(_latent(2, 8, 4, 12, 70, 16, 0.5, None, 250000.0, {"factor": 16.0, "original": 32, "fast": 4.0, "slow": 2.0}), 16, 9, 1),
          ]},
    # larger sizes: a key size of two waves' worth of registers, more experts than a wave has lanes, a latent of several
    # values a lane with one head a block, heads that fill no group, a window of several pages, borrowed weights named ahead
    "D": {"architecture": "Pazilorn", "vocab": 150, "width": 96, "norm": {"eps": 1e-5}, "residual_mult": 0.3,
          "embedding": {"scale": 10.0}, "logit_softcap": 12.0, "layers": [
              _with(_latent(5, 32, 16, 48, 136, 72, 0.2, 130, 50000.0, {"factor": 8.0, "original": 128, "fast": 16.0, "slow": 1.0}), 24, 70, 5, weights_of=2),
              _with(_delta(4, 1, 128, 64, 3, 8, 8), 48, 4, 2),
              _with(_latent(5, 32, 16, 48, 136, 72, 0.2, 130, 50000.0, {"factor": 8.0, "original": 128, "fast": 16.0, "slow": 1.0}), 24, 70, 5),
              _with(_latent(2, 16, 2, 8, 600, 40, 0.3, 9, 100.0), None),
          ]},
}
SEEDS = {"A": 31, "B": 32, "C": 33, "D": 34}
# one layer of one kind, for the tests of a mechanism alone
SINGLE = {
    "channel_delta": {"architecture": "Pazilorn", "vocab": 90, "width": 32, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
                      "embedding": {"scale": 4.0}, "logit_softcap": None, "layers": [_with(_delta(2, 1, 12, 20, 3, 3, 2))]},
    "latent_attention": {"architecture": "Pazilorn", "vocab": 90, "width": 32, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
                         "embedding": {"scale": 4.0}, "logit_softcap": None,
                         "layers": [_with(_latent(2, 12, 6, 28, 24, 20, 0.4, 50, 100.0, _YARN))]},
    "feed_forward": {"architecture": "Pazilorn", "vocab": 90, "width": 32, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
                     "embedding": {"scale": 4.0}, "logit_softcap": None, "layers": [_with(_delta(1, 1, 8, 8, 2, 1, 1), 100, 7, 3)]},
}


def sharpened_tensors(raw: dict, seed: int, store: str) -> dict:
    """The random-weights mode's numbers, made larger so that faults show: the projections and the table four times (logits
    and branch inputs of order one and more) and the router likewise (its logits then lie far apart, and the rounding of a
    bfloat16 run seldom changes which experts a token gets); the convolutions, the low-rank pairs' second matrices and the
    experts as the description makes them."""
    tensors = random_tensors(config_from_dict(raw).spec(), seed, "float32")
    out = {}
    for k, t in tensors.items():
        if t.dim() == 2 and not k.endswith((".conv", ".a2", ".g2", ".uq", ".uk", ".uv", ".gate", ".up", ".down")):
            t = t * 4.0
        out[k] = t.to({"bfloat16": torch.bfloat16, "float32": torch.float32}[store])
    return out


def write_model(raw: dict, seed: int, path, store: str, drop_ranks: bool = True) -> Path:
    """A model folder.  ``drop_ranks``: config.json does not give the delta rule's low ranks, as a checkpoint's configuration
    does not (and for some of the configurations not the query latent's either): the tensors' shapes do."""
    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    tensors = sharpened_tensors(raw, seed, store)
    if drop_ranks:
        raw = json.loads(json.dumps(raw))
        for layer in raw["layers"]:
            for key in ("decay_rank", "gate_rank") + (("q_rank",) if raw["width"] % 32 == 0 else ()):      # (q_rank: in some of them)
                layer["mixer"].pop(key, None)
    (path / "config.json").write_text(json.dumps(raw))
    write_safetensors(path / "model.safetensors", tensors)
    return path


def prompts(raw: dict, lengths, seed: int = 0) -> list:
    g = torch.Generator().manual_seed(3000 + seed)
    return [torch.randint(0, raw["vocab"], (n,), generator=g).tolist() for n in lengths]
