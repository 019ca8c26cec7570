"""Differential attention: every head has two softmax score maps over one set of values.

    q = W_q h: [heads, 2, key_dim];  k = W_k h: [kv_heads, 2, key_dim];  v = W_v h: [kv_heads, value_dim]
    q, k: RMS norm per head and map over key_dim (one weight vector each, shared by all heads and maps)
    a_m = softmax_j(scale * q_m . k_(m,j)) v_j  over the keys j <= the query's position, m = 1, 2
    lambda = exp(sum(lq1 * lk1)) - exp(sum(lq2 * lk2)) + lambda_init          (one number for the layer)
    o = (a_1 - lambda a_2) / sqrt(mean((a_1 - lambda a_2)^2) + eps) * (1 - lambda_init)      per head

Query head h reads kv head h // (heads / kv_heads).  No position enters the scores.  The cache holds two key rows
and one value row per kv head and position: a ``KVNeed`` with twice the key heads and a value size of its own.
Scores, softmax weights, the combination and the unit norm are 32-bit.
"""
from __future__ import annotations

import math

import torch

from ..cache import KVNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear


@register_part("mixer", "differential_attention")
class DifferentialAttention:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nh, self.nkv, self.dk, self.dv = int(p["num_heads"]), int(p["num_kv_heads"]), int(p["key_dim"]), int(p["value_dim"])
        self.scale, self.lambda_init, self.eps = float(p["scale"]), float(p["lambda_init"]), float(p["eps"])
        if self.nh % self.nkv:
            raise ValueError(f"{self.nh} heads are not a multiple of {self.nkv} kv heads")
        self.qkv = Linear(builder.tensor(spec, "qkv"))
        self.out = Linear(builder.tensor(spec, "out"))
        if self.qkv.weight.shape != (2 * (self.nh + self.nkv) * self.dk + self.nkv * self.dv, self.hidden):
            raise ValueError(f"differential attention: joined q/k/v weight {tuple(self.qkv.weight.shape)} does not fit")
        if self.out.weight.shape != (self.hidden, self.nh * self.dv):
            raise ValueError(f"differential attention: output weight {tuple(self.out.weight.shape)} does not fit")
        self.q_norm_w, self.k_norm_w = builder.tensor(spec, "q_norm"), builder.tensor(spec, "k_norm")
        vec = {n: builder.tensor(spec, n).detach().to("cpu", torch.float64) for n in ("lq1", "lk1", "lq2", "lk2")}
        for n, v in vec.items():
            if v.shape != (self.dk,):
                raise ValueError(f"differential attention: {n} is {tuple(v.shape)}, expected ({self.dk},)")
        self.lam = (math.exp(float((vec["lq1"] * vec["lk1"]).sum())) - math.exp(float((vec["lq2"] * vec["lk2"]).sum()))
                    + self.lambda_init)
        self.dtype = builder.dtype

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        return [KVNeed(2 * int(p["num_kv_heads"]), int(p["key_dim"]), None, value_heads=int(p["num_kv_heads"]),
                       value_dim=int(p["value_dim"]))]

    def forward(self, h, ctx):
        lc = ctx.layer_cache
        if lc is None or lc.kv is None:
            raise RuntimeError("differential attention needs the keys and values of its layer; the step gave it no cache")
        qkv = self.qkv(h)
        q = ops.diff_qkv_store(qkv, self.nh, self.nkv, self.dk, self.dv, self.q_norm_w, self.k_norm_w, self.eps, lc.k, lc.v,
                               lc.kv.table_dev, ctx, write_cache=lc.writes)
        o = ops.attention_diff(q, lc.k, lc.v, lc.kv.table_dev, ctx, self.nh, self.nkv, self.dk, self.dv, self.scale, self.lam,
                               1.0 - self.lambda_init, self.eps)
        return self.out(o)
