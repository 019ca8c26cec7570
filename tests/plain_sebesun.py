"""A plain, slow implementation of the Sebesun decoder, used only as the oracle of the tests.

Whole sequences, no cache, no batching, one function for each mechanism, float64 on the CPU (rotation
angles are made in float32, as the product path makes them).  It shares no code with the package under
test: it reads config.json and the safetensors file with its own few lines.

The design, in this file's notation (t: position from 0, W: model width):

  layer            x' = x + N1(mixer(x));  x'' = x' + N2(ff(x')) if the layer has a feed-forward.
                   N(y) = y / sqrt(mean(y^2) + eps) * w: the norm sits on the branch's output, the branches read
                   the stream itself.
  depth average    R_0 = embedding rows, R_(i+1) = x'' of layer i; layer i+1 (or the output) reads
                   sum_j c_i[j] R_j, j = 0 .. i+1.
  retention        S_t = g_h S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t, rotary q and k, k scaled by d^-1/2
  mamba1           S_t = exp(dt_t A) S_(t-1) + dt_t x_t B_t^T,  y_t = S_t C_t + D x_t
  attention        two softmax maps over one set of values, o = a1 - lambda a2, unit-normed per head
  feed-forward     down(xielu(up(h)))
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

def unit_rms(y: torch.Tensor, eps: float) -> torch.Tensor:
    """y / sqrt(mean(y^2) + eps) over the last axis."""
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def rms_norm(y, w, eps):
    return unit_rms(y, eps) * w


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
    sp, sq = softplus(p), softplus(q)
    pos = sp * z * z + 0.5 * z
    neg = (0.5 + sq) * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def rotate_half_split(u: torch.Tensor, dims: int, base: float, first_position: int = 0) -> torch.Tensor:
    """u [T, heads, d]: of each head's first ``dims`` dimensions, i is paired with i + dims/2; the pair (a, b) at
    position p becomes (a cos - b sin, b cos + a sin) with angle p * base^(-2i/dims).  Angles in float32."""
    T = u.shape[0]
    half = dims // 2
    i = np.arange(half, dtype=np.float32)
    freq = np.float32(1.0) / np.power(np.float32(base), np.float32(2.0) * i / np.float32(dims))
    pos = np.arange(first_position, first_position + T, dtype=np.float32)
    ang = (pos[:, None] * freq[None, :]).astype(np.float32)
    cos = torch.from_numpy(np.cos(ang).astype(np.float64))[:, None, :]
    sin = torch.from_numpy(np.sin(ang).astype(np.float64))[:, None, :]
    a, b = u[..., :half], u[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, u[..., dims:]], dim=-1)


# ---- mixers -----------------------------------------------------------------------------------------

def retention(h, w, pre, m, eps):
    """h [T, W].  Per head: S <- decay S + k v^T, o = S^T q; o is unit-normed per head, gated by silu(W_g h)."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(T, H, d)
    k = (h @ w[pre + "k"].T).view(T, H, d)
    v = (h @ w[pre + "v"].T).view(T, H, dv)
    if m.get("rot"):
        q = rotate_half_split(q, m["rot"]["dims"], m["rot"]["base"])
        k = rotate_half_split(k, m["rot"]["dims"], m["rot"]["base"])
    k = k * d ** -0.5
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        g = float(m["decay"][hd])
        for t in range(T):
            S = g * S + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    out = unit_rms(out, eps).reshape(T, H * dv)
    return (out * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def mamba1(h, w, pre, m, eps):
    """Selective scan with a short causal convolution in front."""
    T = h.shape[0]
    inner, n_state, rank, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
    xz = h @ w[pre + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    cw, cb = w[pre + "conv"], w[pre + "conv.b"]
    padded = torch.cat([torch.zeros(taps - 1, inner, dtype=F64), x])
    x = silu(sum(padded[j:j + T] * cw[:, j] for j in range(taps)) + cb)        # the last column is the current token's
    proj = x @ w[pre + "x"].T
    dt, B, C = proj[:, :rank], proj[:, rank:rank + n_state], proj[:, rank + n_state:]
    dt = softplus(dt @ w[pre + "dt"].T + w[pre + "dt.b"])
    A = -torch.exp(w[pre + "A_log"])
    S = torch.zeros(inner, n_state, dtype=F64)
    y = torch.zeros(T, inner, dtype=F64)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + w[pre + "D"] * x[t]
    return (y * silu(z)) @ w[pre + "o"].T


def differential_attention(h, w, pre, m, eps):
    """Two causal softmax maps per head over one set of values; no positions enter the scores."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm((h @ w[pre + "q"].T).view(T, H, 2, d), w[pre + "q.norm"], eps)
    k = rms_norm((h @ w[pre + "k"].T).view(T, G, 2, d), w[pre + "k.norm"], eps)
    v = (h @ w[pre + "v"].T).view(T, G, dv)
    lam = (math.exp(float((w[pre + "lq1"] * w[pre + "lk1"]).sum()))
           - math.exp(float((w[pre + "lq2"] * w[pre + "lk2"]).sum())) + m["diff"])
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        maps = []
        for j in range(2):
            s = (q[:, hd, j] @ k[:, g, j].T) * m["scale"]
            s = s.masked_fill(~causal, -math.inf)
            maps.append(torch.softmax(s, dim=-1) @ v[:, g])
        out[:, hd] = unit_rms(maps[0] - lam * maps[1], eps) * (1.0 - m["diff"])
    return out.reshape(T, H * dv) @ w[pre + "o"].T


MIXERS = {"retention": retention, "mamba1": mamba1, "attention": differential_attention}


def feed_forward(h, w, pre, f):
    if f["kind"] != "dense":
        raise ValueError(f"feed-forward kind {f['kind']!r}")
    act = w[pre + "act"]
    return xielu(h @ w[pre + "up"].T, act[0], act[1]) @ w[pre + "down"].T


# ---- the model --------------------------------------------------------------------------------------

def forward(cfg: dict, w: dict, ids, return_layers: bool = False):
    """Logits [T, vocab] for a whole sequence (and, if asked, the stream after every layer)."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(ids, dtype=torch.long)].to(F64)
    results = [x]
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        x = x + rms_norm(MIXERS[layer["type"]](x, w, pre + "mix.", layer["mixer"], eps), w[pre + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + rms_norm(feed_forward(x, w, pre + "mlp.", layer["mlp"]), w[pre + "norm2"], eps)
        results.append(x)
        c = w[pre + "dwa"]
        x = sum(c[j] * results[j] for j in range(i + 2))
        streams.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(streams)) if return_layers else logits


def greedy(cfg, w, prompt, n_new: int) -> list:
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))
    return ids[len(prompt):]
