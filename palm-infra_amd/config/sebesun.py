"""The typed configuration of the Sebesun decoder and its description as parts.

A Sebesun model is a list of layers, each with a mixer of one of three kinds and an optional dense feed-forward:

  ``retention``   linear attention with one fixed decay per head, rotated q and k, a per-head unit norm and a gate
  ``mamba1``      a selective scan behind a short causal convolution
  ``attention``   differential softmax attention: two score maps per head over one set of values, grouped kv heads

A layer norms the output of each branch, not its input (``x += norm(branch(x))``), and what goes on to the next
layer is a learned weighted sum of the results of all layers so far (and of the embedding rows).

config.json: ``architecture`` "Sebesun", ``vocab``, ``width``, ``norm.eps``, and ``layers``: a list of ``{"type",
"mixer": {sizes and constants}, "mlp": {"kind": "dense", "ff"} or null}``.  Tensor names: ``embed``, ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.{up,down,act}``, ``l<i>.dwa``, ``final.norm``, ``head``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

from .registry import ConfigError, register_architecture
from .spec import LayerCall, ModelSpec, PartSpec, Stored, joined, tensor

_NORM_INIT = ("normal", 1.0, 0.02)
MIXER_TYPES = ("retention", "mamba1", "attention")


def _get(table: dict, key: str, typ, where: str):
    if not isinstance(table, dict) or key not in table or table[key] is None:
        raise ConfigError(f"config.json: {where} lacks {key!r}")
    try:
        return typ(table[key])
    except (TypeError, ValueError):
        raise ConfigError(f"config.json: {where}.{key} = {table[key]!r} is not {typ.__name__}") from None


def _positive(value, what: str):
    if not value > 0:
        raise ConfigError(f"config.json: {what} = {value} must be positive")
    return value


@register_architecture("Sebesun", model_type="sebesun")
@dataclass(frozen=True)
class SebesunConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple          # of dicts as config.json holds them, checked
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, raw: dict) -> "SebesunConfig":
        vocab = _positive(_get(raw, "vocab", int, "the model"), "vocab")
        width = _positive(_get(raw, "width", int, "the model"), "width")
        eps = _positive(_get(raw.get("norm"), "eps", float, "norm"), "norm.eps")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        checked = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            kind = _get(layer, "type", str, where)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}.type = {kind!r} is not one of {', '.join(MIXER_TYPES)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where} lacks its mixer's sizes")
            checked.append({"type": kind, "mixer": cls._check_mixer(kind, m, where + ".mixer"),
                            "mlp": cls._check_mlp(layer.get("mlp"), where + ".mlp")})
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(vocab, width, eps, tuple(checked), eos_ids)

    @staticmethod
    def _check_mixer(kind: str, m: dict, where: str) -> dict:
        if kind == "retention":
            out = {k: _positive(_get(m, k, int, where), f"{where}.{k}") for k in ("heads", "dim", "vdim")}
            decay = m.get("decay")
            if not isinstance(decay, list) or len(decay) != out["heads"]:
                raise ConfigError(f"config.json: {where}.decay must list one decay for each of {out['heads']} heads")
            out["decay"] = [float(d) for d in decay]
            rot = m.get("rot")
            if rot is None:
                out["rot"] = None
            else:
                dims = _get(rot, "dims", int, where + ".rot")
                if dims < 0 or dims % 2 or dims > out["dim"]:
                    raise ConfigError(f"config.json: {where}.rot.dims = {dims} must be even and at most dim = {out['dim']}")
                out["rot"] = {"dims": dims, "base": _positive(_get(rot, "base", float, where + ".rot"), where + ".rot.base")}
            return out
        if kind == "mamba1":
            out = {k: _positive(_get(m, k, int, where), f"{where}.{k}") for k in ("inner", "state", "dt_rank", "conv")}
            if out["conv"] > 16:
                raise ConfigError(f"config.json: {where}.conv = {out['conv']}: the convolution kernel takes at most 16 taps")
            return out
        out = {k: _positive(_get(m, k, int, where), f"{where}.{k}") for k in ("heads", "kv_heads", "dim", "vdim")}
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"config.json: {where}: {out['heads']} heads are not a multiple of {out['kv_heads']} kv heads")
        out["scale"] = _get(m, "scale", float, where)
        out["diff"] = _get(m, "diff", float, where)
        return out

    @staticmethod
    def _check_mlp(f, where: str):
        if f is None:
            return None
        kind = _get(f, "kind", str, where)
        if kind != "dense":
            raise ConfigError(f"config.json: {where}.kind = {kind!r}; this design's feed-forwards are dense")
        return {"kind": kind, "ff": _positive(_get(f, "ff", int, where), where + ".ff")}

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "layers": [dict(layer) for layer in self.layers]}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    # ------------------------------------------------------------------------------------------
    def _mixer(self, i: int, kind: str, m: dict) -> PartSpec:
        W, p = self.width, f"l{i}.mix."
        if kind == "retention":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            parts = {}
            if m["rot"] is not None and m["rot"]["dims"] > 0:
                parts["position"] = PartSpec("position", "rotary", {"rotary_dim": m["rot"]["dims"], "theta": m["rot"]["base"],
                                                                    "pairing": "half_split"})
            return PartSpec(
                "mixer", "retention",
                {"hidden_size": W, "num_heads": H, "key_dim": d, "value_dim": dv, "decay": tuple(m["decay"]),
                 "key_scale": d ** -0.5, "eps": self.eps},
                {"qkvg": joined((p + "q", p + "k", p + "v", p + "g"), ((H * d, W), (H * d, W), (H * dv, W), (H * dv, W))),
                 "out": tensor(p + "o", (W, H * dv))},
                parts)
        if kind == "mamba1":
            C, N, R, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
            return PartSpec(
                "mixer", "selective_scan",
                {"hidden_size": W, "channels": C, "state_size": N, "dt_rank": R, "taps": taps},
                {"in": tensor(p + "in", (2 * C, W)),
                 "conv": tensor(p + "conv", (C, taps), "vector", ("normal", 0.0, 0.3)),
                 "conv_bias": tensor(p + "conv.b", (C,), "vector", ("normal", 0.0, 0.1)),
                 # one stored matrix, two products: the step sizes' low-rank rows, and B | C
                 "x_dt": tensor(p + "x", (R, C), stored=Stored((R + 2 * N, C), rows=(0, R))),
                 "x_bc": tensor(p + "x", (2 * N, C), stored=Stored((R + 2 * N, C), rows=(R, R + 2 * N))),
                 "dt": tensor(p + "dt", (C, R), "matrix", ("normal", 0.0, 0.1)),
                 "dt_bias": tensor(p + "dt.b", (C,), "vector", ("normal", -2.0, 0.5)),
                 "a_log": tensor(p + "A_log", (C, N), "vector", ("normal", 0.0, 0.5)),
                 "skip": tensor(p + "D", (C,), "vector", _NORM_INIT),
                 "out": tensor(p + "o", (W, C))})
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        lam = ("normal", 0.0, 0.1)
        return PartSpec(
            "mixer", "differential_attention",
            {"hidden_size": W, "num_heads": H, "num_kv_heads": G, "key_dim": d, "value_dim": dv, "scale": m["scale"],
             "lambda_init": m["diff"], "eps": self.eps},
            {"qkv": joined((p + "q", p + "k", p + "v"), ((2 * H * d, W), (2 * G * d, W), (G * dv, W))),
             "q_norm": tensor(p + "q.norm", (d,), "vector", _NORM_INIT), "k_norm": tensor(p + "k.norm", (d,), "vector", _NORM_INIT),
             "lq1": tensor(p + "lq1", (d,), "vector", lam), "lk1": tensor(p + "lk1", (d,), "vector", lam),
             "lq2": tensor(p + "lq2", (d,), "vector", lam), "lk2": tensor(p + "lk2", (d,), "vector", lam),
             "out": tensor(p + "o", (W, H * dv))})

    def spec(self, tensor_names=None) -> ModelSpec:
        W, V, eps = self.width, self.vocab, self.eps

        def norm(name: str) -> PartSpec:
            return PartSpec("norm", "rms", {"width": W, "eps": eps}, {"weight": tensor(name, (W,), "vector", _NORM_INIT)})

        layers = []
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            parts = {"mixer": self._mixer(i, layer["type"], layer["mixer"]), "mixer_norm": norm(p + "norm1")}
            if layer["mlp"] is not None:
                F = layer["mlp"]["ff"]
                parts["feed_forward"] = PartSpec(
                    "feed_forward", "dense", {"hidden_size": W, "intermediate_size": F, "activation": "xielu"},
                    {"up": tensor(p + "mlp.up", (F, W)), "down": tensor(p + "mlp.down", (W, F)),
                     "activation": tensor(p + "mlp.act", (2,), "vector", ("normal", 0.0, 0.5))})
                parts["feed_forward_norm"] = norm(p + "norm2")
            # the weights of the average over depth: layer i's result and everything before it, the embedding rows first
            mix = tensor(p + "dwa", (i + 2,), "vector", ("normal", 1.0 / (i + 2), 0.25 / math.sqrt(i + 2)))
            layers.append(PartSpec("block", "post_norm", {"hidden_size": W}, {"depth_weights": mix}, parts))

        return ModelSpec(
            architecture=self.architecture, vocab_size=V, hidden_size=W, max_positions=None,
            embedding=PartSpec("embedding", "token_table", {"vocab_size": V, "hidden_size": W},
                               {"table": tensor("embed", (V, W), "table")}),
            layers=tuple(layers), order=tuple(LayerCall(i) for i in range(len(layers))),
            final_norm=norm("final.norm"),
            head=PartSpec("head", "linear", {"vocab_size": V, "hidden_size": W}, {"weight": tensor("head", (V, W), "matrix")}),
            stop_token_ids=self.eos_token_ids, keeps_results=True,
        )
