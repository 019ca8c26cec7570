"""A plain, slow implementation of the Pazilorn decoder, used only as the oracle of the tests.

Whole sequences, no cache, no batching, one function for each mechanism, float64 on the CPU.  It shares no code
with the package under test: it reads config.json and the safetensors file with its own few lines.

The design, in this file's notation (t: position from 0, W: model width, m: the residual multiplier):

  embedding        x_t = E[token_t] * s
  layer            x' = x + m N1b(mixer(N1(x)));  x'' = x' + m N2b(ff(N2(x'))) if the layer has a feed-forward.
                   N(y) = y / sqrt(mean(y^2) + eps) * w.  A layer may borrow another layer's weights.
  delta rule       per head, S [key, value]:  S <- diag(g_t) S;  u_t = beta_t (v_t - S^T k_t);  S <- S + k_t u_t^T;
                   o_t = S^T q_t.  q, k, v come out of a short causal convolution and silu; q and k are unit vectors
                   (q also times key^-1/2); g_t is one decay per key channel, beta_t one gate per head.
  latent attention queries through a normed latent; keys and values from one normed latent row per position plus
                   one rotated key part shared by all heads; sliding window; softmax; one output gate per head.
  feed-forward     a router picks `top` of the experts by its logits; their weights are the softmax over the picked
                   logits; every expert is down(silu(gate(h)) * up(h)).
  output           tanh cap of the logits of the final norm against the embedding table.
"""
from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import numpy as np
import torch

F64 = torch.float64


# ---- files ------------------------------------------------------------------------------------------

def read_safetensors(path) -> dict:
    raw = Path(path).read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    base = 8 + hlen
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        a, b = meta["data_offsets"]
        buf = raw[base + a:base + b]
        dt = meta["dtype"]
        if dt == "F32":
            arr = np.frombuffer(buf, dtype="<f4").astype(np.float64)
        elif dt == "BF16":
            arr = (np.frombuffer(buf, dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif dt == "I32":
            arr = np.frombuffer(buf, dtype="<i4").astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {dt}")
        out[name] = torch.from_numpy(arr.reshape(meta["shape"]).copy())
    return out


def read_model(model_dir):
    model_dir = Path(model_dir)
    return json.loads((model_dir / "config.json").read_text()), read_safetensors(model_dir / "model.safetensors")


# ---- small functions --------------------------------------------------------------------------------

def rms_norm(y, w, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def short_conv(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x [T, C], w [C, taps]: y_t[c] = sum_j w[c, j] x_(t - (taps - 1) + j)[c], zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros((taps - 1, C), dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + padded[j:j + T] * w[:, j]
    return y


# ---- the delta rule ---------------------------------------------------------------------------------

def delta_inputs(h, t, p, m):
    """q, k [T, kv_heads, dim] (unit vectors, q scaled), v [T, heads, vdim], beta [T, heads], g [T, heads, dim]."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(short_conv(h @ t[p + "q"].T, t[p + "q.conv"])).reshape(T, G, d)
    k = silu(short_conv(h @ t[p + "k"].T, t[p + "k.conv"])).reshape(T, G, d)
    v = silu(short_conv(h @ t[p + "v"].T, t[p + "v.conv"])).reshape(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ t[p + "b"].T)
    a = (h @ t[p + "a1"].T) @ t[p + "a2"].T + t[p + "dt_bias"]
    g = torch.exp(-torch.exp(t[p + "A_log"]).reshape(1, H, 1) * softplus(a).reshape(T, H, d))
    return q, k, v, beta, g


def delta_recurrence(q, k, v, beta, g, state=None):
    """The recurrence token by token.  Returns o [T, heads, vdim] and the state left behind [heads, dim, vdim]."""
    T, H, dv = v.shape
    G, d = q.shape[1], q.shape[2]
    rep = H // G
    S = torch.zeros((H, d, dv), dtype=F64) if state is None else state.clone()
    o = torch.zeros((T, H, dv), dtype=F64)
    kh, qh = k.repeat_interleave(rep, 1), q.repeat_interleave(rep, 1)          # head h reads q/k head h // rep
    for t in range(T):
        S = g[t].unsqueeze(-1) * S
        u = beta[t].unsqueeze(-1) * (v[t] - torch.einsum("hdv,hd->hv", S, kh[t]))
        S = S + kh[t].unsqueeze(-1) * u.unsqueeze(1)
        o[t] = torch.einsum("hdv,hd->hv", S, qh[t])
    return o, S


def channel_delta(h, t, p, m, eps):
    H, dv = m["heads"], m["vdim"]
    T = h.shape[0]
    q, k, v, beta, g = delta_inputs(h, t, p, m)
    o, _ = delta_recurrence(q, k, v, beta, g)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * t[p + "norm"]
    gate = torch.sigmoid((h @ t[p + "g1"].T) @ t[p + "g2"].T).reshape(T, H, dv)
    return (o * gate).reshape(T, H * dv) @ t[p + "o"].T


# ---- latent attention -------------------------------------------------------------------------------

def rotation_frequencies(rot: dict) -> torch.Tensor:
    """One frequency per rotated pair and the factor on cos and sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, ..., dims]: the pair (i, i + dims/2) turned by position * frequency_i."""
    f, mag = rotation_frequencies(rot)
    dims = int(rot["dims"])
    half = dims // 2
    ang = positions.to(F64).unsqueeze(-1) * f
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = (torch.cos(ang) * mag).reshape(shape), (torch.sin(ang) * mag).reshape(shape)
    u, w = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - w * s, w * c + u * s, x[..., dims:]], -1)


def latent_attention(h, t, p, m, eps):
    H, d, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    pos = torch.arange(T)
    cq = rms_norm(h @ t[p + "dq"].T, t[p + "dq.norm"], eps)
    q = (cq @ t[p + "uq"].T).reshape(T, H, d + dr)
    kv = h @ t[p + "dkv"].T
    c = rms_norm(kv[:, :R], t[p + "dkv.norm"], eps)
    k_rot = rotate(kv[:, R:], pos, m["rot"])                               # [T, dr], one for all heads
    q_rot = rotate(q[..., d:], pos, m["rot"])
    k_plain = (c @ t[p + "uk"].T).reshape(T, H, d)
    v = (c @ t[p + "uv"].T).reshape(T, H, dv)
    scores = (torch.einsum("thd,shd->hts", q[..., :d], k_plain) + torch.einsum("thd,sd->hts", q_rot, k_rot)) * float(m["scale"])
    i, j = pos.unsqueeze(1), pos.unsqueeze(0)
    seen = (j <= i)
    size = (m.get("mask") or {}).get("size")
    if size:
        seen = seen & (i - j < int(size))
    scores = scores.masked_fill(~seen, -math.inf)
    o = torch.einsum("hts,shd->thd", torch.softmax(scores, -1), v)
    gate = torch.sigmoid(h @ t[p + "g"].T)                                  # [T, H]
    return (o * gate.unsqueeze(-1)).reshape(T, H * dv) @ t[p + "o"].T


# ---- feed-forward -----------------------------------------------------------------------------------

def route(h, t, p, top):
    """The chosen experts [T, top] and their weights."""
    z = h @ t[p + "router"].T + t[p + "router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    return idx, torch.softmax(val, -1)


def expert(h, t, p):
    return (silu(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def mixture(h, t, p, f):
    idx, w = route(h, t, p, int(f["router"]["top"]))
    out = torch.zeros_like(h)
    for e in range(int(f["router"]["experts"])):
        for r in range(idx.shape[1]):
            rows = (idx[:, r] == e).nonzero().flatten()
            if rows.numel():
                out[rows] += w[rows, r].unsqueeze(1) * expert(h[rows], t, f"{p}e{e}.")
    return out


# ---- the model --------------------------------------------------------------------------------------

def forward(cfg: dict, t: dict, tokens, layers_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from its first token."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    for i, layer in enumerate(cfg["layers"]):
        src = i
        while cfg["layers"][src].get("weights_of") is not None:
            src = int(cfg["layers"][src]["weights_of"])
        p = f"l{src}."
        h = rms_norm(x, t[p + "norm1"], eps)
        if layer["type"] == "channel_delta":
            y = channel_delta(h, t, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, t, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + mult * rms_norm(y, t[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            y = mixture(rms_norm(x, t[p + "norm2"], eps), t, p + "mlp.", layer["mlp"])
            x = x + mult * rms_norm(y, t[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = rms_norm(x, t["final.norm"], eps) @ t["embed"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy(cfg: dict, t: dict, prompt, n_new: int) -> list:
    """The first maximum of the last position's logits, n_new times."""
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward(cfg, t, ids)[-1])))
    return ids[len(prompt):]
