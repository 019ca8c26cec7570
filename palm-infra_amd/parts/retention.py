"""Retention: linear attention with one fixed decay per head, without softmax or denominator.

Per head, with q_t, k_t of size ``key_dim`` and v_t of size ``value_dim``:

    S_t = decay_h * S_(t-1) + k_t v_t^T,      o_t = S_t^T q_t

q and k are rotated first if the part has a ``position`` (k is multiplied by ``key_scale`` after the rotation); each
head's o_t is divided by its root mean square (``eps`` inside the root, no weight); the heads are joined, multiplied by
silu of a gate projection and projected back.  One joined product makes q | k | v | gate.  S is float32 and is kept
per sequence (``StateNeed``); rotated values and everything in the recurrence are 32-bit whatever the run's type.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear


@register_part("mixer", "retention")
class Retention:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nh, self.dk, self.dv = int(p["num_heads"]), int(p["key_dim"]), int(p["value_dim"])
        self.key_scale, self.eps = float(p["key_scale"]), float(p["eps"])
        if len(p["decay"]) != self.nh:
            raise ValueError(f"retention: {len(p['decay'])} decays for {self.nh} heads")
        self.decay = torch.tensor([float(d) for d in p["decay"]], dtype=torch.float32).to(builder.device)
        self.qkvg = Linear(builder.tensor(spec, "qkvg"))
        self.out = Linear(builder.tensor(spec, "out"))
        if self.qkvg.weight.shape != (self.nh * 2 * (self.dk + self.dv), self.hidden):
            raise ValueError(f"retention: joined q/k/v/gate weight {tuple(self.qkvg.weight.shape)} does not fit {self.nh} heads "
                             f"of key size {self.dk} and value size {self.dv} over hidden {self.hidden}")
        if self.out.weight.shape != (self.hidden, self.nh * self.dv):
            raise ValueError(f"retention: output weight {tuple(self.out.weight.shape)} does not fit")
        self.position = builder.build(spec.parts["position"]) if "position" in spec.parts else None
        if self.position is not None and (self.position.pairing != "half_split" or self.position.rotary_dim > self.dk):
            raise ValueError("retention: the rotation pairs dimension i with i + rotary_dim/2 within the key size")

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        return [StateNeed("retention", (int(p["num_heads"]), int(p["key_dim"]), int(p["value_dim"])))]

    def forward(self, h, ctx):
        lc = ctx.layer_cache
        if lc is None or not lc.states or "retention" not in lc.states:
            raise RuntimeError("retention needs its state; the step gave it no cache")
        rows = self.qkvg(h)
        tables = self.position.tables(ctx) if self.position is not None else None
        cos, sin = tables if tables is not None else (None, None)
        o = ops.retention(rows, self.nh, self.dk, self.dv, self.decay, self.key_scale, self.eps, lc.states["retention"], ctx,
                          cos=cos, sin=sin, rot=self.position.rotary_dim if tables is not None else 0)
        return self.out(o)
