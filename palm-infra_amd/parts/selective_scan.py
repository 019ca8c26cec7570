"""The Mamba mixer: a selective scan behind a short causal convolution.

    [x | z] = W_in h;   u = silu(conv(x) + b)            (per channel, ``taps`` taps, the last one the current token's)
    dt = softplus(W_dt (W_x_dt u) + dt_bias);  [B | C] = W_x_bc u;   A = -exp(A_log)
    S_t[c, n] = exp(dt_t[c] A[c, n]) S_(t-1)[c, n] + dt_t[c] u_t[c] B_t[n]
    y_t[c] = sum_n S_t[c, n] C_t[n] + D[c] u_t[c];       out = W_o (y * silu(z))

Per sequence it keeps S (float32 [channels, state]) and the convolution's last ``taps - 1`` inputs.  Step sizes,
decays and the recurrence are 32-bit whatever the run's type: the step-size product gives float32, bias and
softplus are applied where the scan reads them.
"""
from __future__ import annotations

import torch

from ..cache import StateNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear


@register_part("mixer", "selective_scan")
class SelectiveScan:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden, self.C, self.N = int(p["hidden_size"]), int(p["channels"]), int(p["state_size"])
        self.R, self.taps = int(p["dt_rank"]), int(p["taps"])
        t = lambda name: builder.tensor(spec, name)
        self.inp, self.x_dt, self.x_bc, self.dt, self.out = (Linear(t("in")), Linear(t("x_dt")), Linear(t("x_bc")), Linear(t("dt")),
                                                             Linear(t("out")))
        self.conv, self.conv_bias, self.dt_bias, self.a_log, self.skip = t("conv"), t("conv_bias"), t("dt_bias"), t("a_log"), t("skip")
        want = {"in": (self.inp.weight, (2 * self.C, self.hidden)), "x_dt": (self.x_dt.weight, (self.R, self.C)),
                "x_bc": (self.x_bc.weight, (2 * self.N, self.C)), "dt": (self.dt.weight, (self.C, self.R)),
                "out": (self.out.weight, (self.hidden, self.C)), "conv": (self.conv, (self.C, self.taps)),
                "conv_bias": (self.conv_bias, (self.C,)), "dt_bias": (self.dt_bias, (self.C,)), "a_log": (self.a_log, (self.C, self.N)),
                "skip": (self.skip, (self.C,))}
        for name, (tensor, shape) in want.items():
            if tuple(tensor.shape) != shape:
                raise ValueError(f"selective_scan: {name} is {tuple(tensor.shape)}, expected {shape}")

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        C, N, taps = int(p["channels"]), int(p["state_size"]), int(p["taps"])
        return [StateNeed("scan", (C, N)), StateNeed("conv", (max(taps - 1, 0), C))]

    def forward(self, h, ctx):
        lc = ctx.layer_cache
        if lc is None or not lc.states or "scan" not in lc.states:
            raise RuntimeError("the selective scan needs its state; the step gave it no cache")
        xz = self.inp(h)
        u = ops.causal_conv(xz, self.C, self.conv, self.conv_bias, lc.states["conv"], ctx)
        dt_linear = self.dt(self.x_dt(u), out_dtype=torch.float32)
        bc = self.x_bc(u)
        y = ops.selective_scan(u, xz, bc, 0, self.N, dt_linear, self.dt_bias, self.a_log, self.skip, lc.states["scan"], ctx)
        return self.out(y)
