"""The typed configuration of the Pazilorn decoder and its description as parts.

A Pazilorn model is a list of layers, each with a mixer of one of two kinds and an optional feed-forward of routed
experts:

  ``channel_delta``      a gated delta rule with one decay per key channel behind short causal convolutions
  ``latent_attention``   softmax attention over one compressed row per position, with a sliding window, a rotated key part
                         shared by all heads (frequencies stretched for long sequences) and one output gate per head

A layer norms each branch on both sides and scales what it adds: ``x += m * norm_b(branch(norm_a(x)))``.  A layer may
borrow another layer's weights (``weights_of``) while keeping a cache and state of its own.  The embedding rows are
multiplied by ``embedding.scale``; the head is the embedding table itself, and the logits are capped by a tanh.

config.json: ``architecture`` "Pazilorn", ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``embedding.scale``,
``logit_softcap``, and ``layers``: a list of ``{"type", "mixer": {sizes and constants}, "mlp": {"kind": "moe", "expert":
{"ff"}, "router": {"experts", "top"}} or null, "weights_of": j (optional)}``.  Tensor names: ``embed``, ``l<i>.norm1``,
``l<i>.norm1b``, ``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.e<k>.{gate,up,down}``, ``l<i>.mlp.router``,
``l<i>.mlp.router.b``, ``final.norm``.  The ranks of the delta rule's two low-rank pairs are the shapes of their tensors;
a configuration that was not read beside a checkpoint takes them from ``mixer.decay_rank`` / ``mixer.gate_rank``.
"""
from __future__ import annotations

from dataclasses import dataclass, replace

from .registry import ConfigError, register_architecture
from .spec import LayerCall, ModelSpec, PartSpec, joined, tensor

_NORM_INIT = ("normal", 1.0, 0.02)
MIXER_TYPES = ("channel_delta", "latent_attention")


def _get(table, key: str, typ, where: str):
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


@register_architecture("Pazilorn", model_type="pazilorn")
@dataclass(frozen=True)
class PazilornConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    embedding_scale: float
    logit_softcap: float | None
    layers: tuple          # of dicts as config.json holds them, checked
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, raw: dict) -> "PazilornConfig":
        vocab = _positive(_get(raw, "vocab", int, "the model"), "vocab")
        width = _positive(_get(raw, "width", int, "the model"), "width")
        eps = _positive(_get(raw.get("norm"), "eps", float, "norm"), "norm.eps")
        mult = float(raw["residual_mult"]) if raw.get("residual_mult") is not None else 1.0
        emb = raw.get("embedding") or {}
        scale = float(emb["scale"]) if emb.get("scale") is not None else 1.0
        cap = raw.get("logit_softcap")
        cap = _positive(float(cap), "logit_softcap") if cap else None
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        checked = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            kind = _get(layer, "type", str, where)
            if kind not in MIXER_TYPES:
                raise ConfigError(f"config.json: {where}.type = {kind!r} is not one of {', '.join(MIXER_TYPES)}")
            if not isinstance(layer.get("mixer"), dict):
                raise ConfigError(f"config.json: {where} lacks its mixer's sizes")
            entry = {"type": kind, "mixer": cls._check_mixer(kind, layer["mixer"], where + ".mixer"),
                     "mlp": cls._check_mlp(layer.get("mlp"), where + ".mlp")}
            if layer.get("weights_of") is not None:
                j = int(layer["weights_of"])
                if not 0 <= j < len(layers) or j == i:
                    raise ConfigError(f"config.json: {where}.weights_of = {j} names no other layer")
                entry["weights_of"] = j
            checked.append(entry)
        for i, entry in enumerate(checked):
            j = cls._source(checked, i)
            if j != i and (checked[j]["type"] != entry["type"] or (checked[j]["mlp"] is None) != (entry["mlp"] is None)):
                raise ConfigError(f"config.json: layers[{i}] borrows the weights of layers[{j}], which is of another kind")
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(vocab, width, eps, mult, scale, cap, tuple(checked), eos_ids)

    @staticmethod
    def _source(layers, i: int) -> int:
        """The layer whose tensors layer i uses (itself, unless it borrows)."""
        seen = set()
        while layers[i].get("weights_of") is not None:
            if i in seen:
                raise ConfigError(f"config.json: layers[{i}].weights_of leads back to itself")
            seen.add(i)
            i = layers[i]["weights_of"]
        return i

    @staticmethod
    def _check_mixer(kind: str, m: dict, where: str) -> dict:
        if kind == "channel_delta":
            out = {k: _positive(_get(m, k, int, where), f"{where}.{k}") for k in ("heads", "kv_heads", "dim", "vdim", "conv")}
            if out["heads"] % out["kv_heads"]:
                raise ConfigError(f"config.json: {where}: {out['heads']} heads are not a multiple of {out['kv_heads']} kv heads")
            if out["conv"] > 16:
                raise ConfigError(f"config.json: {where}.conv = {out['conv']}: the convolution kernel takes at most 16 taps")
            if out["dim"] > 256 or out["vdim"] > 1024:
                raise ConfigError(f"config.json: {where}: the recurrence takes key sizes up to 256 and value sizes up to 1024")
            for k in ("decay_rank", "gate_rank"):
                if m.get(k) is not None:
                    out[k] = _positive(int(m[k]), f"{where}.{k}")
            return out
        out = {k: _positive(_get(m, k, int, where), f"{where}.{k}") for k in ("heads", "dim", "vdim", "kv_rank")}
        if m.get("q_rank") is not None:              # else the rows of the query's down projection give it
            out["q_rank"] = _positive(int(m["q_rank"]), f"{where}.q_rank")
        out["rot_dim"] = _get(m, "rot_dim", int, where)
        out["scale"] = _get(m, "scale", float, where)
        if out["rot_dim"] < 0 or out["rot_dim"] % 2:
            raise ConfigError(f"config.json: {where}.rot_dim = {out['rot_dim']} must be even and not negative")
        if out["kv_rank"] > 1024 or out["kv_rank"] + out["rot_dim"] > 1280 or out["dim"] > 512:
            raise ConfigError(f"config.json: {where}: the attention kernels take latents up to 1024 (with the rotated part 1280) and "
                              "unrotated key sizes up to 512")
        mask = m.get("mask")
        out["mask"] = {"size": _positive(_get(mask, "size", int, where + ".mask"), where + ".mask.size")} if mask else None
        rot = m.get("rot")
        if out["rot_dim"]:
            dims = _get(rot, "dims", int, where + ".rot")
            if dims != out["rot_dim"]:
                raise ConfigError(f"config.json: {where}.rot.dims = {dims}: the whole rotated part of {out['rot_dim']} is rotated")
            r = {"dims": dims, "base": _positive(_get(rot, "base", float, where + ".rot"), where + ".rot.base")}
            sc = rot.get("scaling")
            r["scaling"] = ({k: _positive(_get(sc, k, float, where + ".rot.scaling"), f"{where}.rot.scaling.{k}")
                             for k in ("factor", "original", "fast", "slow")} if sc else None)
            out["rot"] = r
        else:
            out["rot"] = None
        return out

    @staticmethod
    def _check_mlp(f, where: str):
        if f is None:
            return None
        kind = _get(f, "kind", str, where)
        if kind != "moe":
            raise ConfigError(f"config.json: {where}.kind = {kind!r}; this design's feed-forwards are routed experts ('moe')")
        ff = _positive(_get(f.get("expert"), "ff", int, where + ".expert"), where + ".expert.ff")
        experts = _positive(_get(f.get("router"), "experts", int, where + ".router"), where + ".router.experts")
        top = _positive(_get(f.get("router"), "top", int, where + ".router"), where + ".router.top")
        if top > experts or top > 64 or experts > 512:
            raise ConfigError(f"config.json: {where}.router: {top} of {experts} experts (at most 64 of at most 512)")
        return {"kind": kind, "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}

    def with_tensor_shapes(self, shapes: dict) -> "PazilornConfig":
        """The configuration with the sizes that a checkpoint's tensors give: the ranks of the delta rule's low-rank pairs
        (rows of ``l<i>.mix.a1`` and ``l<i>.mix.g1``) and of the attention's query latent (rows of ``l<i>.mix.dq``)."""
        layers = []
        for i, layer in enumerate(self.layers):
            j = self._source(self.layers, i)
            m = dict(layer["mixer"])
            given = (("decay_rank", f"l{j}.mix.a1"), ("gate_rank", f"l{j}.mix.g1")) if layer["type"] == "channel_delta" else (("q_rank", f"l{j}.mix.dq"),)
            for key, name in given:
                if name in shapes and len(shapes[name]) == 2:
                    m[key] = int(shapes[name][0])
            layer = dict(layer, mixer=m)
            layers.append(layer)
        return replace(self, layers=tuple(layers))

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "residual_mult": self.residual_mult, "embedding": {"scale": self.embedding_scale},
             "logit_softcap": self.logit_softcap, "layers": [dict(layer) for layer in self.layers]}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    # ------------------------------------------------------------------------------------------
    def _mixer(self, i: int, kind: str, m: dict) -> PartSpec:
        W, p = self.width, f"l{i}.mix."
        if kind == "channel_delta":
            H, G, d, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            if "decay_rank" not in m or "gate_rank" not in m:
                raise ConfigError(f"layers[{i}].mixer: the ranks of the decay's and the gate's low-rank pairs are given by the shapes of "
                                  f"{p}a1 and {p}g1, or by decay_rank and gate_rank where there is no checkpoint")
            ra, rg = m["decay_rank"], m["gate_rank"]
            conv_init = ("normal", 0.0, 0.4)
            return PartSpec(
                "mixer", "delta_rule",
                {"hidden_size": W, "num_heads": H, "num_qk_heads": G, "key_dim": d, "value_dim": dv, "taps": taps, "eps": self.eps,
                 "decay_rank": ra, "gate_rank": rg},
                {"qkvb": joined((p + "q", p + "k", p + "v", p + "b"), ((G * d, W), (G * d, W), (H * dv, W), (H, W))),
                 "conv": joined((p + "q.conv", p + "k.conv", p + "v.conv"), ((G * d, taps), (G * d, taps), (H * dv, taps)), "vector", conv_init),
                 "low": joined((p + "a1", p + "g1"), ((ra, W), (rg, W))),
                 "decay_up": tensor(p + "a2", (H * d, ra), "matrix", ("normal", 0.0, 0.1)),
                 "gate_up": tensor(p + "g2", (H * dv, rg), "matrix", ("normal", 0.0, 0.1)),
                 "a_log": tensor(p + "A_log", (H,), "vector", ("normal", -1.0, 0.5)),
                 "dt_bias": tensor(p + "dt_bias", (H * d,), "vector", ("normal", -1.0, 1.0)),
                 "norm": tensor(p + "norm", (dv,), "vector", _NORM_INIT),
                 "out": tensor(p + "o", (W, H * dv))})
        if "q_rank" not in m:
            raise ConfigError(f"layers[{i}].mixer: the rank of the query's latent is given by q_rank or by the shape of {p}dq")
        H, d, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        parts = {}
        if m["rot"] is not None:
            parts["position"] = PartSpec("position", "rotary", {"rotary_dim": dr, "theta": m["rot"]["base"], "pairing": "half_split",
                                                                "scaling": m["rot"]["scaling"]})
        return PartSpec(
            "mixer", "latent_attention",
            {"hidden_size": W, "num_heads": H, "key_dim": d, "rot_dim": dr, "value_dim": dv, "kv_rank": R, "q_rank": Q,
             "scale": m["scale"], "window": m["mask"]["size"] if m["mask"] else None, "eps": self.eps, "gated": True},
            {"down": joined((p + "dq", p + "dkv", p + "g"), ((Q, W), (R + dr, W), (H, W))),
             "q_norm": tensor(p + "dq.norm", (Q,), "vector", _NORM_INIT), "kv_norm": tensor(p + "dkv.norm", (R,), "vector", _NORM_INIT),
             "uq": tensor(p + "uq", (H * (d + dr), Q), "matrix", ("normal", 0.0, 0.08)),
             "uk": tensor(p + "uk", (H * d, R), "matrix", ("normal", 0.0, 0.08)),
             "uv": tensor(p + "uv", (H * dv, R), "matrix", ("normal", 0.0, 0.08)),
             "out": tensor(p + "o", (W, H * dv))},
            parts)

    def spec(self, tensor_names=None) -> ModelSpec:
        W, V, eps = self.width, self.vocab, self.eps

        def norm(name: str) -> PartSpec:
            return PartSpec("norm", "rms", {"width": W, "eps": eps}, {"weight": tensor(name, (W,), "vector", _NORM_INIT)})

        layers, index = [], {}                       # layers with tensors of their own; config layer -> its place there
        for i, layer in enumerate(self.layers):
            if layer.get("weights_of") is not None:
                continue
            p = f"l{i}."
            parts = {"mixer_norm": norm(p + "norm1"), "mixer": self._mixer(i, layer["type"], layer["mixer"]),
                     "mixer_out_norm": norm(p + "norm1b")}
            if layer["mlp"] is not None:
                F, E, top = layer["mlp"]["expert"]["ff"], layer["mlp"]["router"]["experts"], layer["mlp"]["router"]["top"]
                gu_names, gu_shapes = [], []
                for e in range(E):
                    gu_names += [f"{p}mlp.e{e}.gate", f"{p}mlp.e{e}.up"]
                    gu_shapes += [(F, W), (F, W)]
                parts["feed_forward_norm"] = norm(p + "norm2")
                parts["feed_forward"] = PartSpec(
                    "feed_forward", "routed_gated_silu", {"hidden_size": W, "intermediate_size": F, "num_experts": E, "top": top},
                    {"router": tensor(p + "mlp.router", (E, W), "matrix", ("normal", 0.0, 0.3)),
                     "router_bias": tensor(p + "mlp.router.b", (E,), "vector", ("normal", 0.0, 0.3)),
                     "gate_up": joined(gu_names, gu_shapes, "matrix", ("normal", 0.0, 0.08)),
                     "down": joined([f"{p}mlp.e{e}.down" for e in range(E)], [(W, F)] * E, "matrix", ("normal", 0.0, 0.08))})
                parts["feed_forward_out_norm"] = norm(p + "norm2b")
            # a checkpoint that holds the second pair of norms for a layer without a feed-forward: bound, and not used
            spare = {}
            if layer["mlp"] is None and tensor_names is not None:
                spare = {f"spare_{n}": tensor(p + n, (W,), "vector", _NORM_INIT) for n in ("norm2", "norm2b") if p + n in set(tensor_names)}
            index[i] = len(layers)
            layers.append(PartSpec("block", "sandwich", {"hidden_size": W, "residual_gain": self.residual_mult}, spare, parts))
        order = tuple(LayerCall(index[self._source(self.layers, i)]) for i in range(len(self.layers)))

        table = tensor("embed", (V, W), "table", ("normal", 0.0, 0.05))
        return ModelSpec(
            architecture=self.architecture, vocab_size=V, hidden_size=W, max_positions=None,
            embedding=PartSpec("embedding", "token_table", {"vocab_size": V, "hidden_size": W, "scale": self.embedding_scale},
                               {"table": table}),
            layers=tuple(layers), order=order, final_norm=norm("final.norm"),
            head=PartSpec("head", "linear", {"vocab_size": V, "hidden_size": W, "softcap": self.logit_softcap}, {"weight": table}),
            stop_token_ids=self.eos_token_ids,
        )
