"""Feed-forwards.

``gated_silu``: down( silu(gate(h)) * up(h) ), silu(z) = z / (1 + exp(-z)), with gate and up
joined into one [2I, H] product (models/qwen3.py:276-287; kernels/elementwise.cpp:529-583).

``dense``: down(act(up(h))) with an activation chosen by name.  ``xielu`` has two learned numbers p, q (tensor
``activation``, float32 [2]): for z > 0, softplus(p) z^2 + z/2; for z <= 0, (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
from __future__ import annotations

from ..kernels import ops
from .base import register_part
from .linear import Linear
from .residual import as_tensor


@register_part("feed_forward", "gated_silu")
class GatedSiluFeedForward:
    capturable = True

    def __init__(self, spec, builder):
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        bias = lambda name: builder.tensor(spec, name) if name in spec.tensors else None
        self.gate_up = Linear(builder.tensor(spec, "gate_up"), bias("gate_up_bias"))
        self.down = Linear(builder.tensor(spec, "down"), bias("down_bias"))
        if self.gate_up.weight.shape != (2 * self.inter, self.hidden) or self.down.weight.shape != (self.hidden, self.inter):
            raise ValueError(f"feed-forward: weights {tuple(self.gate_up.weight.shape)}, {tuple(self.down.weight.shape)} "
                             f"do not fit hidden {self.hidden}, intermediate {self.inter}")

    takes_sink = True

    def forward(self, h, ctx, sink=None):
        return self.down(self.gate_up.gated(h), sink=sink)


@register_part("feed_forward", "dense")
class DenseFeedForward:
    capturable = True
    ACTIVATIONS = ("xielu",)

    def __init__(self, spec, builder):
        self.hidden = int(spec.params["hidden_size"])
        self.inter = int(spec.params["intermediate_size"])
        self.activation = str(spec.params.get("activation", "xielu"))
        if self.activation not in self.ACTIVATIONS:
            raise ValueError(f"feed-forward: activation {self.activation!r} is not one of {self.ACTIVATIONS}")
        self.up = Linear(builder.tensor(spec, "up"))
        self.down = Linear(builder.tensor(spec, "down"))
        self.act_params = builder.tensor(spec, "activation")
        if self.up.weight.shape != (self.inter, self.hidden) or self.down.weight.shape != (self.hidden, self.inter):
            raise ValueError(f"feed-forward: weights {tuple(self.up.weight.shape)}, {tuple(self.down.weight.shape)} "
                             f"do not fit hidden {self.hidden}, intermediate {self.inter}")
        if self.act_params.shape != (2,):
            raise ValueError(f"feed-forward: xielu takes two numbers, got {tuple(self.act_params.shape)}")

    takes_sink = True

    def forward(self, h, ctx, sink=None):
        return self.down(ops.xielu(self.up(as_tensor(h)), self.act_params), sink=sink)
