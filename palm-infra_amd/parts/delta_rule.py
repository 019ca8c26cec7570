"""The gated delta rule with one decay per key channel.

Per head, with q_t, k_t of size ``key_dim`` (unit vectors, q also times key_dim^-1/2) and v_t of size ``value_dim``:

    S <- diag(g_t) S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t

q, k and v leave one joined projection, a short causal convolution per channel (``taps`` taps, no bias) and silu; head h
reads q/k head h // (heads / qk_heads).  beta_t = sigmoid(W_b h) is one number a head (it rides in the joined
projection, behind the convolution's channels); g_t = exp(-exp(A_log_h) softplus(W_a2 (W_a1 h) + dt_bias)) is one decay
for each row of S; each head's o_t is normed over value_dim (one weight vector for all heads) and multiplied by
sigmoid(W_g2 (W_g1 h)).  The two low-rank pairs are two products: [W_a1; W_g1] h, then a block-diagonal [W_a2, 0; 0, W_g2]
(put together once, when the part is built) whose result is 32-bit.  S is float32 and is kept per sequence beside the
convolution's last inputs (``StateNeed``); unit vectors, decays, gates and everything in the recurrence are 32-bit
whatever the run's type.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear

UNIT_EPS = 1e-6          # inside the root of the unit vectors: x / sqrt(sum(x^2) + UNIT_EPS)


@register_part("mixer", "delta_rule")
class DeltaRule:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nh, self.nqk, self.dk, self.dv = int(p["num_heads"]), int(p["num_qk_heads"]), int(p["key_dim"]), int(p["value_dim"])
        self.taps, self.eps = int(p["taps"]), float(p["eps"])
        self.ra, self.rg = int(p["decay_rank"]), int(p["gate_rank"])
        if self.nh % self.nqk:
            raise ValueError(f"delta rule: {self.nh} heads are not a multiple of {self.nqk} q/k heads")
        t = lambda name: builder.tensor(spec, name)
        self.channels = 2 * self.nqk * self.dk + self.nh * self.dv
        self.qkvb = Linear(t("qkvb"))
        self.low = Linear(t("low"))
        self.out = Linear(t("out"))
        self.conv, self.a_log, self.dt_bias, self.norm_w = t("conv"), t("a_log"), t("dt_bias"), t("norm")
        a2, g2 = t("decay_up"), t("gate_up")
        want = {"qkvb": (self.qkvb.weight, (self.channels + self.nh, self.hidden)), "low": (self.low.weight, (self.ra + self.rg, self.hidden)),
                "out": (self.out.weight, (self.hidden, self.nh * self.dv)), "conv": (self.conv, (self.channels, self.taps)),
                "a_log": (self.a_log, (self.nh,)), "dt_bias": (self.dt_bias, (self.nh * self.dk,)), "norm": (self.norm_w, (self.dv,)),
                "decay_up": (a2, (self.nh * self.dk, self.ra)), "gate_up": (g2, (self.nh * self.dv, self.rg))}
        for name, (tensor, shape) in want.items():
            if tuple(tensor.shape) != shape:
                raise ValueError(f"delta rule: {name} is {tuple(tensor.shape)}, expected {shape}")
        # [W_a2, 0; 0, W_g2]: one product gives the decays' rows and the gate's rows from [W_a1 h | W_g1 h]
        both = torch.zeros((self.nh * (self.dk + self.dv), self.ra + self.rg), dtype=a2.dtype, device=a2.device)
        both[:self.nh * self.dk, :self.ra] = a2
        both[self.nh * self.dk:, self.ra:] = g2
        self.up = Linear(both)

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        H, G, d, dv, taps = (int(p[k]) for k in ("num_heads", "num_qk_heads", "key_dim", "value_dim", "taps"))
        return [StateNeed("delta", (H, d, dv)), StateNeed("delta_conv", (max(taps - 1, 0), 2 * G * d + H * dv))]

    def forward(self, h, ctx):
        lc = ctx.layer_cache
        if lc is None or not lc.states or "delta" not in lc.states:
            raise RuntimeError("the delta rule needs its state; the step gave it no cache")
        rows = self.qkvb(h)                                                # [q | k | v | b]
        u = ops.causal_conv(rows, self.channels, self.conv, None, lc.states["delta_conv"], ctx)
        up = self.up(self.low(h), out_dtype=torch.float32)                # [decay rows | gate rows], 32-bit
        qk = self.nqk * self.dk
        o = ops.delta_rule(u, (0, qk, 2 * qk), rows[:, self.channels:], up[:, :self.nh * self.dk], up[:, self.nh * self.dk:],
                           self.a_log, self.dt_bias, self.norm_w, self.nh, self.nqk, self.dk, self.dv, self.dk ** -0.5, UNIT_EPS,
                           self.eps, lc.states["delta"], ctx)
        return self.out(o)
