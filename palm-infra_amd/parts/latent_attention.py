"""Attention whose keys and values are made from one compressed row per position.

    [c_q' | c' | r'] = W_down h                 one joined product (the per-head output gates ride in it too)
    c_q = norm(c_q'),  q = W_uq c_q             per head [plain (key_dim) | to rotate (rot_dim)]
    c = norm(c'),      r = rotate(r')           the cache keeps [c | r] for every position: kv_rank + rot_dim values
    head h: key_j = [U_k,h c_j | r_j],  value_j = U_v,h c_j
    score = (q_plain . U_k,h c_j + rotate(q_rot) . r_j) * scale over the visible positions (causal; the last ``window``)
    out = W_o concat_h( sigmoid(gate_h) * sum_j softmax_j(score) value_j )

Keys and values are never expanded: q_plain goes through U_k,h once (a_h = U_k,h^T q_plain, kv_rank values), the scores
are a_h . c_j + q_rot . r_j, the weighted sum is taken over the rows c_j, and U_v,h is applied to the sum.  All heads read
the same rows.  The rotation's angles and the scores, weights and sums are 32-bit.  In the bfloat16 mode the cache keeps the
latents a second time with the positions innermost, which is how the prompt kernel on the matrix cores reads them; single
tokens and the float32 mode go through the exact kernel, which reads the rows alone.
"""
from __future__ import annotations

from ..cache import RowsNeed
from ..kernels import ops
from .base import register_part
from .linear import Linear


@register_part("mixer", "latent_attention")
class LatentAttention:
    capturable = True

    def __init__(self, spec, builder):
        p = spec.params
        self.hidden = int(p["hidden_size"])
        self.nh, self.dk, self.dr, self.dv = int(p["num_heads"]), int(p["key_dim"]), int(p["rot_dim"]), int(p["value_dim"])
        self.q_rank, self.kv_rank = int(p["q_rank"]), int(p["kv_rank"])
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.window = int(p["window"]) if p.get("window") else None
        self.gated = bool(p.get("gated", False))
        t = lambda name: builder.tensor(spec, name)
        self.down = Linear(t("down"))
        self.uq = Linear(t("uq"))
        self.out = Linear(t("out"))
        self.uk, self.uv, self.q_norm_w, self.kv_norm_w = t("uk"), t("uv"), t("q_norm"), t("kv_norm")
        rows = self.q_rank + self.kv_rank + self.dr + (self.nh if self.gated else 0)
        want = {"down": (self.down.weight, (rows, self.hidden)), "uq": (self.uq.weight, (self.nh * (self.dk + self.dr), self.q_rank)),
                "out": (self.out.weight, (self.hidden, self.nh * self.dv)), "uk": (self.uk, (self.nh * self.dk, self.kv_rank)),
                "uv": (self.uv, (self.nh * self.dv, self.kv_rank)), "q_norm": (self.q_norm_w, (self.q_rank,)),
                "kv_norm": (self.kv_norm_w, (self.kv_rank,))}
        for name, (tensor, shape) in want.items():
            if tuple(tensor.shape) != shape:
                raise ValueError(f"latent attention: {name} is {tuple(tensor.shape)}, expected {shape}")
        self.position = builder.build(spec.parts["position"]) if "position" in spec.parts and self.dr else None
        if self.position is not None and (self.position.pairing != "half_split" or self.position.rotary_dim != self.dr):
            raise ValueError("latent attention: the rotation pairs dimension i with i + rot_dim/2 over the whole rotated part")
        self.dtype = builder.dtype

    @staticmethod
    def cache_needs(spec):
        p = spec.params
        window = int(p["window"]) if p.get("window") else None
        # the rows, and the latents once more in bfloat16 for the prompt kernel on the matrix cores (a page of them is read
        # there with the positions innermost: [kv_rank, 64] in the room of [64, kv_rank])
        return [RowsNeed("latent", (int(p["kv_rank"]) + int(p["rot_dim"]),), None, window),
                RowsNeed("latent_t", (int(p["kv_rank"]),), "bfloat16", window)]

    def forward(self, h, ctx):
        lc = ctx.layer_cache
        if lc is None or not lc.rows or "latent" not in lc.rows:
            raise RuntimeError("latent attention needs the rows of its layer; the step gave it no cache")
        view = lc.rows["latent"]
        rows_t = table_t = None
        if "latent_t" in lc.rows and ops.latent_mfma_serves(view.data, self.kv_rank, self.dr):
            turned = lc.rows["latent_t"]
            rows_t, table_t = turned.data.view(turned.data.shape[0], self.kv_rank, turned.data.shape[1]), turned.table_dev
        down = self.down(h)
        tables = self.position.tables(ctx) if self.position is not None else None
        cos, sin = tables if tables is not None else (None, None)
        cq = ops.latent_prep(down, self.q_rank, self.q_rank, self.kv_rank, self.dr, self.q_norm_w, self.kv_norm_w, self.eps, cos, sin,
                             view.data, view.table_dev, ctx, write_cache=lc.writes, rows_t=rows_t, table_t=table_t)
        qa = ops.latent_query(self.uq(cq), self.uk, cos, sin, self.nh, self.dk, self.dr, self.kv_rank)
        gate = down[:, self.q_rank + self.kv_rank + self.dr:] if self.gated else None
        if ops.latent_fused_serves(qa, view.data, rows_t, self.uv, ctx, self.kv_rank, self.dr, self.dv):
            # a prompt on the matrix cores: the value matrices and the gates ride in the attention kernel
            o = ops.latent_attention_fused(qa, view.data, view.table_dev, ctx, self.nh, self.kv_rank, self.dr, self.scale, self.window,
                                           rows_t, table_t, self.uv, gate, self.dv)
            return self.out(o)
        o_lat = ops.latent_attention(qa, view.data, view.table_dev, ctx, self.nh, self.kv_rank, self.dr, self.scale, self.window,
                                     rows_t=rows_t, table_t=table_t)
        return self.out(ops.latent_output(o_lat, self.uv, gate, self.nh, self.kv_rank, self.dv, self.dtype))
