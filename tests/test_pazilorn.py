"""The Pazilorn design in the engine against the plain implementation (tests/plain_pazilorn.py).

Without a GPU: the configuration, its description as parts, the sizes that only tensors give, and the oracle's own
mechanisms against closed forms.  On the GPU: every mechanism alone (one-layer models, and the kernels called directly with
inputs made so that one far token, one key at a window's or a page's edge, or one tie decides the result), whole prompts,
prompts cut into portions down to two tokens, prefill against token-by-token decoding from the first token, batches of
unequal requests against each alone, slots and pages that are used again, long decoding over several pages and past the
windows, recorded against launched steps, and greedy generation through ``generate`` and the command line.  In float32
and in bfloat16.
"""
import json
import math

import pytest
import torch

import pazilorn_tiny as S
import plain_pazilorn as P
import tiny
from palm_infra_amd.config import ConfigError, config_from_dict

gpu = pytest.mark.gpu
DTYPES = ("float32", "bfloat16")
LENGTHS = {"A": [1, 2, 63, 64, 65, 130, 200, 17], "B": [129, 3, 70, 71, 1, 191], "C": [5, 66, 128, 31], "D": [300, 9, 140]}


# ---- without a GPU ---------------------------------------------------------------------------------------

def test_registry_picks_the_design_by_its_config_key():
    cfg = config_from_dict(S.CONFIGS["A"])
    assert type(cfg).__name__ == "PazilornConfig"
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_spec_names_every_tensor_and_borrowed_layers_have_none():
    spec = config_from_dict(S.CONFIGS["A"]).spec()
    names = spec.expected_tensors()
    assert names["embed"][0] == (211, 64) and names["final.norm"][0] == (64,)
    assert names["l0.mix.q"][0] == (2 * 16, 64) and names["l0.mix.v.conv"][0] == (4 * 24, 4) and names["l0.mix.a1"][0] == (5, 64)
    assert names["l0.mix.g2"][0] == (4 * 24, 7) and names["l0.mix.dt_bias"][0] == (4 * 16,) and names["l0.mix.norm"][0] == (24,)
    assert names["l0.mlp.e5.down"][0] == (64, 40) and names["l0.mlp.router.b"][0] == (6,)
    assert names["l1.mix.dkv"][0] == (40 + 8, 64) and names["l1.mix.uq"][0] == (3 * (24 + 8), 48) and names["l1.mix.g"][0] == (3, 64)
    assert not any(n.startswith(("l2.", "l3.")) for n in names)            # they run layers 0 and 1 again
    assert "l1.norm2" not in names and "l1.norm1b" in names                # no feed-forward, no norms around one
    assert [c.layer for c in spec.order] == [0, 1, 0, 1] and all(c.cache_of is None for c in spec.order)
    assert "head" not in names                                             # the head is the table itself


def test_norms_of_a_feed_forward_that_is_not_there_are_bound_and_not_missed():
    cfg = config_from_dict(S.CONFIGS["A"])
    names = list(cfg.spec().expected_tensors())
    assert "l1.norm2" not in names
    with_spares = cfg.spec(names + ["l1.norm2", "l1.norm2b"]).expected_tensors()
    assert with_spares["l1.norm2"][0] == (64,) and with_spares["l1.norm2b"][0] == (64,) and len(with_spares) == len(names) + 2
    assert set(cfg.spec(names).expected_tensors()) == set(names)


def test_cache_needs_follow_the_run_order():
    from palm_infra_amd.cache import RowsNeed, StateNeed
    from palm_infra_amd.parts import cache_needs
    spec = config_from_dict(S.CONFIGS["A"]).spec()
    needs = [cache_needs(spec.layers[c.layer]) for c in spec.order]
    assert needs[0] == needs[2] == [StateNeed("delta", (4, 16, 24)), StateNeed("delta_conv", (3, 2 * 2 * 16 + 4 * 24))]
    assert needs[1] == needs[3] == [RowsNeed("latent", (48,), None, 37), RowsNeed("latent_t", (40,), "bfloat16", 37)]
    assert cache_needs(config_from_dict(S.CONFIGS["C"]).spec().layers[0]) == [RowsNeed("latent", (74,), None, None),
                                                                              RowsNeed("latent_t", (70,), "bfloat16", None)]


def test_ranks_come_from_the_tensors_where_config_json_has_none(tmp_path):
    from palm_infra_amd.config import config_from_dir
    from palm_infra_amd.weights import ModelFiles
    d = S.write_model(S.CONFIGS["B"], 5, tmp_path, "bfloat16")
    cfg = config_from_dir(d)
    with pytest.raises(ConfigError, match="a1"):
        cfg.spec()
    files = ModelFiles(d)
    cfg = cfg.with_tensor_shapes({n: files.shape(n) for n in files.names()})
    assert (cfg.layers[1]["mixer"]["decay_rank"], cfg.layers[1]["mixer"]["gate_rank"]) == (1, 3)
    assert set(cfg.spec(files.names()).expected_tensors()) == set(files.names())


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="retention"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=4), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=7), "experts"),
    (lambda c: c["layers"][2].update(weights_of=1), "another kind"),
    (lambda c: c["layers"][2].update(weights_of=9), "weights_of"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_bad_configurations_are_refused(change, what):
    raw = json.loads(json.dumps(S.CONFIGS["A"]))
    change(raw)
    with pytest.raises(ConfigError, match=what):
        config_from_dict(raw)


def test_random_model_folder_is_read_by_the_plain_implementation(tmp_path):
    from palm_infra_amd.weights import write_random_model
    write_random_model(S.CONFIGS["B"], 3, tmp_path, "bfloat16")
    cfg, w = P.read_model(tmp_path)
    logits = P.forward(cfg, w, [1, 2, 3, 4, 5])
    assert logits.shape == (5, 130) and torch.isfinite(logits).all() and float(logits.abs().max()) <= 30.0


def test_plain_delta_rule_stores_and_recalls():
    """Orthonormal keys, no decay, full write strength: the state is sum_t k_t v_t^T and a query k_s recalls v_s; a second
    write under the same key replaces the first; with a decay g the recalled value shrinks by g per step."""
    torch.manual_seed(0)
    d, dv, T = 6, 5, 4
    k = torch.linalg.qr(torch.randn(d, d, dtype=P.F64))[0][:T].reshape(T, 1, d)
    v = torch.randn(T, 1, dv, dtype=P.F64)
    ones = torch.ones(T, 1, dtype=P.F64)
    o, state = P.delta_recurrence(k, k, v, ones, torch.ones(T, 1, d, dtype=P.F64))
    assert torch.allclose(o, v) and torch.allclose(state[0], torch.einsum("td,tv->dv", k[:, 0], v[:, 0]))
    k2 = torch.cat([k[:1], k[:1]])
    o2, s2 = P.delta_recurrence(k2, k2, v[:2], ones[:2], torch.ones(2, 1, d, dtype=P.F64))
    assert torch.allclose(s2[0], torch.outer(k[0, 0], v[1, 0]))
    g = torch.full((T, 1, d), 0.5, dtype=P.F64)
    q_last = k[:1].expand(T, 1, d)
    o3, _ = P.delta_recurrence(q_last, k, v, ones, g)
    assert torch.allclose(o3[3, 0], v[0, 0] * 0.5 ** 3)
    # the state is carried: two halves equal the whole
    oa, sa = P.delta_recurrence(q_last[:2], k[:2], v[:2], ones[:2], g[:2])
    ob, sb = P.delta_recurrence(q_last[2:], k[2:], v[2:], ones[2:], g[2:], state=sa)
    assert torch.allclose(torch.cat([oa, ob]), o3)


def test_plain_rotation_frequencies():
    f, mag = P.rotation_frequencies({"dims": 8, "base": 100.0, "scaling": None})
    assert mag == 1.0 and torch.allclose(f, torch.tensor([1.0, 100 ** -0.25, 100 ** -0.5, 100 ** -0.75], dtype=P.F64))
    sc = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    f2, mag2 = P.rotation_frequencies({"dims": 8, "base": 100.0, "scaling": sc})
    assert mag2 == pytest.approx(0.1 * math.log(4.0) + 1.0)
    assert f2[0] == f[0] and f2[-1] == pytest.approx(float(f[-1]) / 4.0)          # the fastest pair turns as before, the slowest 4 times slower
    assert all(float(f[i]) / 4.0 - 1e-15 <= float(f2[i]) <= float(f[i]) + 1e-15 for i in range(4))
    x = torch.randn(3, 2, 8, dtype=P.F64)
    r = P.rotate(x, torch.tensor([0, 5, 9]), {"dims": 8, "base": 100.0, "scaling": None})
    assert torch.allclose(r[0], x[0]) and torch.allclose(r.pow(2).sum(-1), x.pow(2).sum(-1))


def test_plain_latent_attention_equals_its_absorbed_form():
    """Scores through the key matrix applied to the query, values through the value matrix applied to the sum: the same
    numbers as keys and values expanded per head."""
    raw = S.SINGLE["latent_attention"]
    t = {k: v.double() for k, v in S.sharpened_tensors(raw, 3, "float32").items()}
    m, eps = raw["layers"][0]["mixer"], raw["norm"]["eps"]
    torch.manual_seed(1)
    T, H, d, dr, dv, R = 60, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    h = torch.randn(T, 32, dtype=P.F64)
    want = P.latent_attention(h, t, "l0.mix.", m, eps)
    pos = torch.arange(T)
    q = (P.rms_norm(h @ t["l0.mix.dq"].T, t["l0.mix.dq.norm"], eps) @ t["l0.mix.uq"].T).reshape(T, H, d + dr)
    kv = h @ t["l0.mix.dkv"].T
    c, r = P.rms_norm(kv[:, :R], t["l0.mix.dkv.norm"], eps), P.rotate(kv[:, R:], pos, m["rot"])
    a = torch.einsum("thd,hdr->thr", q[..., :d], t["l0.mix.uk"].reshape(H, d, R))
    s = (torch.einsum("thr,sr->hts", a, c) + torch.einsum("thd,sd->hts", P.rotate(q[..., d:], pos, m["rot"]), r)) * m["scale"]
    seen = (pos[None, :] <= pos[:, None]) & (pos[:, None] - pos[None, :] < m["mask"]["size"])
    o_lat = torch.einsum("hts,sr->thr", torch.softmax(s.masked_fill(~seen, -math.inf), -1), c)
    o = torch.einsum("thr,hvr->thv", o_lat, t["l0.mix.uv"].reshape(H, dv, R)) * torch.sigmoid(h @ t["l0.mix.g"].T).unsqueeze(-1)
    assert torch.allclose(o.reshape(T, H * dv) @ t["l0.mix.o"].T, want, atol=1e-10)


def test_plain_router_weights():
    t = {"r.router": torch.tensor([[1.0], [3.0], [2.0], [3.0]], dtype=P.F64), "r.router.b": torch.tensor([0.0, 0.0, 0.5, 0.0], dtype=P.F64)}
    idx, w = P.route(torch.tensor([[1.0]], dtype=P.F64), t, "r.", 2)
    assert sorted(idx[0].tolist()) == [1, 3] and torch.allclose(w, torch.tensor([[0.5, 0.5]], dtype=P.F64))
    idx, w = P.route(torch.tensor([[2.0]], dtype=P.F64), t, "r.", 3)
    assert set(idx[0].tolist()) == {1, 2, 3} and float(w.sum()) == pytest.approx(1.0)
    assert float(w[0][idx[0].tolist().index(2)]) == pytest.approx(math.exp(4.5) / (2 * math.exp(6.0) + math.exp(4.5)))


# ---- engines and references ------------------------------------------------------------------------------

_dirs, _engines, _refs = {}, {}, {}


def raw_of(name):
    return S.CONFIGS.get(name) or S.SINGLE[name]


def model_dir(tmp_path_factory, name: str, store: str):
    key = (name, store)
    if key not in _dirs:
        _dirs[key] = S.write_model(raw_of(name), S.SEEDS.get(name, 41), tmp_path_factory.mktemp(f"pazilorn_{name}_{store}"), store)
    return _dirs[key]


def engine_for(tmp_path_factory, name: str, dtype: str, **options):
    from palm_infra_amd.engine import Engine
    key = (name, dtype, tuple(sorted(options.items())))
    if key not in _engines:
        _engines[key] = Engine.from_dir(model_dir(tmp_path_factory, name, dtype), dtype=dtype, max_tokens=64 * 24, **options)
    return _engines[key]


def reference(tmp_path_factory, name: str, dtype: str, ids):
    key = (name, dtype, tuple(ids))
    if key not in _refs:
        cfg, w = P.read_model(model_dir(tmp_path_factory, name, dtype))
        _refs[key] = P.forward(cfg, w, ids)
    return _refs[key]


def assert_close(got, ref, dtype: str, what: str = "") -> None:
    """float32: 1e-4 of the logits' scale (and no less than 1e-4: some hundred steps of a 32-bit recurrence come to that on
    logits of several units), the gate that shows faults.  bfloat16: a row's root mean square error
    within a fifth of the logits' scale, all rows together within a twentieth, an element within three quarters; one row in
    twenty-five (at least two) may be over the row gate, but never by more than the scale itself: which experts a token gets
    turns on the rounding of the router's input when two logits lie close (with one of five experts a token, as one
    configuration has it, that is a whole other feed-forward, and a rounding of one or two percent of the logits' spread
    does it to some two tokens in a hundred), with float32 twins exact."""
    got = torch.as_tensor(got).double().cpu().reshape(ref.shape)
    assert torch.isfinite(got).all(), f"{what}: logits are not finite"
    err = (got - ref.double()).abs().reshape(-1, ref.shape[-1])
    scale = float(ref.double().pow(2).mean().sqrt())
    if dtype == "float32":
        worst = float(err.max())
        assert worst <= 1e-4 * max(1.0, scale), f"{what}: float32 logits differ by {worst:.3e} (their scale is {scale:.3e})"
        return
    rows = err.pow(2).mean(-1).sqrt()
    over = rows > 0.2 * scale
    assert int(over.sum()) <= max(2, rows.numel() // 25), (f"{what}: bfloat16 rms error over a fifth of {scale:.3e} in "
                                                             f"{int(over.sum())} of {rows.numel()} rows, the worst {float(rows.max()):.3e} in row {int(rows.argmax())}")
    assert float(rows.max()) <= scale, f"{what}: bfloat16 rms error {float(rows.max()):.3e} in row {int(rows.argmax())} vs {scale:.3e}"
    rest = err[~over]
    if rest.shape[0] >= 16:
        assert float(rest.pow(2).mean().sqrt()) <= 0.05 * scale, f"{what}: bfloat16 rms error over all rows vs {scale:.3e}"
    if rest.numel():
        assert float(rest.max()) <= 0.75 * scale, f"{what}: bfloat16 max error {float(rest.max()):.3e} vs {scale:.3e}"


class Pool:
    """Rows checked a few at a time, then all together (the gate over all rows needs many)."""

    def __init__(self, dtype, what):
        self.dtype, self.what, self.got, self.ref = dtype, what, [], []

    def add(self, got, ref):
        got = torch.as_tensor(got).double().cpu().reshape(ref.shape)
        assert_close(got, ref, self.dtype, self.what)
        self.got.append(got.reshape(-1, ref.shape[-1]))
        self.ref.append(ref.double().reshape(-1, ref.shape[-1]))

    def check(self):
        assert_close(torch.cat(self.got), torch.cat(self.ref), self.dtype, self.what + " (all rows together)")


CASES = [(n, d) for n in ("A", "B", "C", "D") for d in DTYPES]


def _step_context(lengths_before, new_counts, slots=None):
    """A cache-less context for kernels that only need the packed layout."""
    from palm_infra_amd.parts import make_context
    slots = list(range(len(new_counts))) if slots is None else list(slots)
    return make_context(slots, list(lengths_before), [[0] * c for c in new_counts], torch.float32, "cuda")


# ---- every mechanism alone -------------------------------------------------------------------------------

@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", sorted(S.SINGLE))
def test_one_layer_of_one_kind(tmp_path_factory, kind, dtype):
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, kind, dtype)
    for ids in S.prompts(raw_of(kind), [1, 7, 64, 150], seed=1):
        slot = eng.open()
        got = eng.step([StepEntry(slot, ids, list(range(len(ids))))])
        eng.close(slot)
        assert_close(got, reference(tmp_path_factory, kind, dtype, ids), dtype, f"{kind} alone, {len(ids)} tokens")


@gpu
@pytest.mark.parametrize("W", [50, 64, 2048, 4100, 5000])      # narrow, no multiple of the block, wide, beyond what a thread holds
def test_scaled_add_of_a_normed_branch_and_the_next_norm(W):
    from palm_infra_amd.kernels import ops
    torch.manual_seed(W)
    n = 5
    x = torch.randn(n, W, device="cuda")
    for dt in (torch.float32, torch.bfloat16):
        y = (torch.randn(n, W, device="cuda") * 3).to(dt)
        w1, w2 = torch.randn(W, device="cuda"), torch.randn(W, device="cuda")
        want_x = x.double() + 0.3 * P.rms_norm(y.double(), w1.double(), 1e-5)
        want_h = P.rms_norm(want_x, w2.double(), 2e-6)
        a, b = x.clone(), x.clone()
        h = ops.add_normed_scaled(a, y, w1, 1e-5, 0.3, w2, 2e-6, torch.float32)
        assert ops.add_normed_scaled(b, y, w1, 1e-5, 0.3) is None
        assert torch.equal(a, b) and torch.allclose(a.double(), want_x, atol=1e-5)
        assert torch.allclose(h.double(), want_h, atol=2e-5)
        hb = ops.add_normed_scaled(x.clone(), y, w1, 1e-5, 0.3, w2, 2e-6, torch.bfloat16)
        assert torch.allclose(hb.double(), want_h, atol=0.02, rtol=0.01)


@gpu
def test_softcap_scaled_table_rows_and_stretched_rotation_tables():
    from palm_infra_amd.kernels import ops
    z = torch.tensor([-100.0, -3.0, 0.0, 0.5, 40.0], device="cuda")
    assert torch.allclose(ops.softcap(z.clone(), 7.0).double().cpu(), 7.0 * torch.tanh(z.double().cpu() / 7.0), atol=1e-6)
    table = torch.randn(9, 6, device="cuda").to(torch.bfloat16)
    ids = torch.tensor([3, 0, 8], dtype=torch.int32, device="cuda")
    assert torch.equal(ops.embed(table, ids, scale=2.5), table.float()[ids.long()] * 2.5)
    assert torch.equal(ops.embed(table, ids), table.float()[ids.long()])
    from palm_infra_amd.config.spec import PartSpec
    from palm_infra_amd.parts import Builder
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}}
    part = Builder(None, torch.float32, "cuda").build(PartSpec("position", "rotary", {"rotary_dim": 8, "theta": 100.0, "scaling": rot["scaling"]}))
    f, mag = P.rotation_frequencies(rot)
    ctx = _step_context([0, 700], [3, 2])
    cos, sin = part.tables(ctx)
    ang = torch.tensor([0, 1, 2, 700, 701], dtype=P.F64).unsqueeze(1) * f
    assert torch.allclose(cos.double().cpu(), torch.cos(ang) * mag, atol=2e-4) and torch.allclose(sin.double().cpu(), torch.sin(ang) * mag, atol=2e-4)


def _delta_case(T, heads, kv, dim, vdim, dtype, seed):
    """Inputs of the recurrence kernel for one sequence in which the first token's write decides the last output: its
    key is a unit vector that no later key touches, decays are close to one, and the last query is that key."""
    g = torch.Generator().manual_seed(seed)
    C = 2 * kv * dim + heads * vdim
    u = torch.randn(T, C, generator=g) * 0.5
    qk = kv * dim
    u[:, qk:2 * qk].view(T, kv, dim)[:, :, 0] = 0.0                 # later keys have no part along the first axis
    u[0, qk:2 * qk] = 0.0
    u[0, qk:2 * qk].view(kv, dim)[:, 0] = 3.0                       # the first key is that axis
    u[T - 1, :qk] = 0.0
    u[T - 1, :qk].view(kv, dim)[:, 0] = 2.0                         # the last query asks for it
    u[0, 2 * qk:] = 4.0 * torch.sign(torch.randn(heads * vdim, generator=g))
    b = torch.randn(T, heads, generator=g)
    b[0] = 9.0                                                      # written in full
    a = torch.randn(T, heads * dim, generator=g) - 6.0              # softplus small: decays close to one
    gate = torch.randn(T, heads * vdim, generator=g)
    a_log = torch.randn(heads, generator=g) * 0.3 - 1.0
    dt_bias = torch.randn(heads * dim, generator=g) * 0.3
    norm_w = 1.0 + 0.1 * torch.randn(vdim, generator=g)
    td = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    return dict(u=u.to(td), b=b.to(td), a=a, gate=gate, a_log=a_log, dt_bias=dt_bias, norm_w=norm_w)


def _delta_plain(c, heads, kv, dim, vdim, eps, drop_first=False):
    T = c["u"].shape[0]
    u, qk = c["u"].double(), kv * dim
    q, k, v = u[:, :qk].reshape(T, kv, dim), u[:, qk:2 * qk].reshape(T, kv, dim), u[:, 2 * qk:].reshape(T, heads, vdim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(c["b"].double())
    g = torch.exp(-torch.exp(c["a_log"].double()).reshape(1, heads, 1) * P.softplus(c["a"].double() + c["dt_bias"].double()).reshape(T, heads, dim))
    if drop_first:
        beta = beta.clone()
        beta[0] = 0.0
    o, state = P.delta_recurrence(q, k, v, beta, g)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * c["norm_w"].double() * torch.sigmoid(c["gate"].double()).reshape(T, heads, vdim)
    return o.reshape(T, heads * vdim), state


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,dim,vdim", [(2, 1, 12, 20), (3, 3, 40, 72), (1, 1, 96, 130), (2, 2, 130, 64), (2, 2, 32, 320)])
def test_delta_rule_kernel_keeps_a_far_write_whole_and_in_portions(dtype, heads, kv, dim, vdim):
    """Whole, in portions down to two tokens and single tokens, and cut by the kernel into chunks that run side by side (of
    a size given here, 0 for none, or of its own choice): the outputs and the state left behind."""
    from palm_infra_amd.kernels import ops
    T, eps = 300, 1e-5
    c = _delta_case(T, heads, kv, dim, vdim, dtype, seed=dim + vdim)
    want, want_state = _delta_plain(c, heads, kv, dim, vdim, eps)
    without, _ = _delta_plain(c, heads, kv, dim, vdim, eps, drop_first=True)
    assert float((want[-1] - without[-1]).abs().max()) > 0.3            # the far write decides the last output
    dev = {k: v.cuda() for k, v in c.items()}
    tol = dict(atol=2e-4, rtol=1e-4) if dtype == "float32" else dict(atol=0.03, rtol=0.03)
    for portions, chunk in (([T], 0), ([150, 64, 5, 2, 79], 0), ([1] * 3 + [T - 3], 0), ([T], 32), ([T], 64), ([T], 104), ([130, 170], 48),
                            ([T], None)):
        state = torch.full((3, heads, dim, vdim), float("nan"), device="cuda")
        state[1] = 0.0                                                   # slot 1 is the sequence's; its neighbours hold rubbish
        got, lo = [], 0
        for n in portions:
            ctx = _step_context([lo], [n], slots=[1])
            sl = slice(lo, lo + n)
            got.append(ops.delta_rule(dev["u"][sl].contiguous(), (0, kv * dim, 2 * kv * dim), dev["b"][sl].contiguous(), dev["a"][sl].contiguous(),
                                      dev["gate"][sl].contiguous(), dev["a_log"], dev["dt_bias"], dev["norm_w"], heads, kv, dim, vdim,
                                      dim ** -0.5, 1e-6, eps, state, ctx, chunk=chunk))
            lo += n
        got = torch.cat(got).double().cpu()
        assert torch.allclose(got, want, **tol), f"portions {portions}, chunks of {chunk}: {float((got - want).abs().max())}"
        assert torch.allclose(state[1].double().cpu(), want_state, atol=1e-4 if dtype == "float32" else 1e-3, rtol=1e-3)
        assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all()


def _latent_plain(qa, rows, starts, counts, heads, R, scale, window):
    """Per sequence b the rows are rows[b] [len, R + dr]; queries are its last counts[b] positions."""
    out, o = [], 0
    for b, (s, n) in enumerate(zip(starts, counts)):
        r = rows[b].double()
        for i in range(n):
            pos = s + i
            lo = max(0, pos - window + 1) if window else 0
            sc = torch.einsum("hd,sd->hs", qa[o + i].double(), r[lo:pos + 1]) * scale
            out.append(torch.softmax(sc, -1) @ r[lo:pos + 1, :R])
        o += n
    return torch.stack(out)


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,R,dr,window", [(3, 40, 8, 37), (1, 96, 16, 70), (5, 70, 4, None), (2, 200, 32, 64), (2, 520, 64, 129),
                                               (7, 256, 32, None), (5, 136, 16, 130)])
def test_latent_attention_kernel_far_keys_page_borders_and_window_edges(dtype, heads, R, dr, window):
    """Two sequences through pages in a scrambled order, one as a prompt portion and one as a single token.  For chosen
    queries one key carries a large score: far back, on either side of a page border, the last key inside the window and
    the first outside it (which must not be seen), and the query's own position; the position after a query holds a
    larger key still, which must stay unseen."""
    from palm_infra_amd.kernels import ops
    td = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    g = torch.Generator().manual_seed(R + dr)
    lens, counts = [330, 200], [70, 1]
    starts = [ln - c for ln, c in zip(lens, counts)]
    dk = R + dr
    rows = [(torch.randn(ln + 1, dk, generator=g) * 0.3).to(td) for ln in lens]        # one row beyond each length: never seen
    n = sum(counts)
    qa = torch.randn(n, heads, dk, generator=g) * 0.3
    marks = []                                                                          # (sequence, query position, key position)
    w = window or 10 ** 9
    for b, (s, c) in enumerate(zip(starts, counts)):
        pos = s + c - 1                                                                 # the sequence's last query
        far = max(0, pos - w + 1)
        marks += [(b, pos, far)]
        if b == 0:
            marks += [(b, s + 3, max(0, s + 3 - w)), (b, s + 10, 63 if w > 300 else (s + 10) // 64 * 64 - 1), (b, s + 20, (s + 20) // 64 * 64),
                      (b, s + 30, s + 30)]
    for b, pos, key in marks:
        qrow = sum(counts[:b]) + pos - starts[b]
        direction = torch.randn(dk, generator=g)
        direction = direction / direction.norm()
        qa[qrow, :, :] = direction * 6.0
        rows[b][key] = (direction * 6.0).to(td)
        rows[b][pos + 1] = (direction * 12.0).to(td)                                    # the next position: larger, and unseen
    # pages in a scrambled order, the rest of the cache NaN
    pages_of = [list(range(7, 1, -1)), [9, 12, 8, 10]]
    cache = torch.full((14, 64, dk), float("nan"), dtype=td, device="cuda")
    table = torch.full((3, 8), 13, dtype=torch.int32)
    for b, pages in enumerate(pages_of):
        table[b + 1, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
        for j in range(lens[b] + 1):
            cache[pages[j // 64], j % 64] = rows[b][j].cuda()
    table = table.cuda()
    ctx = _step_context(starts, counts, slots=[1, 2])
    got = ops.latent_attention(qa.cuda(), cache, table, ctx, heads, R, dr, 0.7, window).double().cpu()
    want = _latent_plain(qa, [r[:-1] for r in rows], starts, counts, heads, R, 0.7, window)
    assert torch.isfinite(got).all()
    assert torch.allclose(got, want, atol=1e-4 if dtype == "float32" else 2e-2, rtol=1e-3 if dtype == "float32" else 2e-2), float((got - want).abs().max())
    if dtype == "bfloat16" and ops.latent_mfma_serves(cache, R, dr):
        # the prompt kernel on the matrix cores: the latents once more with the positions innermost, through pages in another
        # scrambled order, NaN wherever the copy belongs to nobody
        pages_t = [[3, 11, 0, 5, 7, 1], [2, 4, 12, 6]]
        turned = torch.full((14, R, 64), float("nan"), dtype=td, device="cuda")
        table_t = torch.full((3, 8), 13, dtype=torch.int32)
        for b, pages in enumerate(pages_t):
            table_t[b + 1, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
            for j in range(lens[b]):
                turned[pages[j // 64], :, j % 64] = rows[b][j, :R].cuda()
        fast = ops.latent_attention(qa.cuda(), cache, table, ctx, heads, R, dr, 0.7, window, rows_t=turned, table_t=table_t.cuda()).double().cpu()
        assert torch.isfinite(fast).all()
        assert torch.allclose(fast, want, atol=3e-2, rtol=3e-2), float((fast - want).abs().max())
        # and with the value matrices and the heads' gates in the same kernel (value sizes that fill no tile of 16 too)
        for dv in (20, 72):
            uv = (torch.randn(heads * dv, R, generator=g) * 0.2).to(td)
            gate = torch.randn(n, heads + 3, generator=g).to(td)
            fused = ops.latent_attention_fused(qa.cuda(), cache, table, ctx, heads, R, dr, 0.7, window, turned, table_t.cuda(), uv.cuda(),
                                               gate.cuda()[:, 3:], dv).double().cpu()
            rows_out = torch.einsum("thr,hvr->thv", want, uv.double().reshape(heads, dv, R)) * torch.sigmoid(gate.double()[:, 3:]).unsqueeze(-1)
            assert torch.isfinite(fused).all()
            assert torch.allclose(fused, rows_out.reshape(n, heads * dv), atol=4e-2, rtol=4e-2), float((fused - rows_out.reshape(n, heads * dv)).abs().max())
    # the marked keys decide: a window one shorter, or the key outside seen, would change the marked rows by far more
    if window:
        other = _latent_plain(qa, [r[:-1] for r in rows], starts, counts, heads, R, 0.7, window - 1)
        assert float((other - want).abs().max()) > 0.5
        other = _latent_plain(qa, [r[:-1] for r in rows], starts, counts, heads, R, 0.7, window + 1)
        assert float((other - want).abs().max()) > 0.5


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_projections_around_the_attention(dtype):
    """The row written to the cache (normed latent, rotated key part), the normed query latent, the queries through the key
    matrix with their rotated parts, and the sums through the value matrix with the gate."""
    from palm_infra_amd.kernels import ops
    td = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    tol = dict(atol=2e-5, rtol=1e-5) if dtype == "float32" else dict(atol=0.03, rtol=0.02)
    g = torch.Generator().manual_seed(2)
    n, Q, R, dr, H, d, dv = 11, 20, 24, 6, 3, 12, 28
    ctx = _step_context([60, 0], [8, 3], slots=[0, 1])
    down = torch.randn(n, Q + R + dr + H, generator=g).to(td)
    wq, wk = 1 + 0.2 * torch.randn(Q, generator=g), 1 + 0.2 * torch.randn(R, generator=g)
    pos = ctx.positions.cpu()
    rot = {"dims": dr, "base": 50.0, "scaling": None}
    f, _ = P.rotation_frequencies(rot)
    ang = pos.double().unsqueeze(1) * f
    cos, sin = torch.cos(ang).float().cuda(), torch.sin(ang).float().cuda()
    cache = torch.zeros((4, 64, R + dr), dtype=td, device="cuda")
    table = torch.tensor([[2, 1], [0, 3], [3, 3]], dtype=torch.int32, device="cuda")
    turned = torch.zeros((4, R, 64), dtype=torch.bfloat16, device="cuda")
    table_t = torch.tensor([[1, 3], [2, 0], [3, 3]], dtype=torch.int32, device="cuda")
    cq = ops.latent_prep(down.cuda(), Q, Q, R, dr, wq.cuda(), wk.cuda(), 1e-5, cos, sin, cache, table, ctx, rows_t=turned, table_t=table_t)
    dd = down.double()
    assert torch.allclose(cq.double().cpu(), P.rms_norm(dd[:, :Q], wq.double(), 1e-5), **tol)
    want_rows = torch.cat([P.rms_norm(dd[:, Q:Q + R], wk.double(), 1e-5), P.rotate(dd[:, Q + R:Q + R + dr], pos, rot)], 1)
    where = [(1, 60 + i - 64) if 60 + i >= 64 else (2, 60 + i) for i in range(8)] + [(0, i) for i in range(3)]
    got_rows = torch.stack([cache[p, j] for p, j in where]).double().cpu()
    assert torch.allclose(got_rows, want_rows, **tol)
    where_t = [(3, 60 + i - 64) if 60 + i >= 64 else (1, 60 + i) for i in range(8)] + [(2, i) for i in range(3)]
    got_t = torch.stack([turned[p, :, j] for p, j in where_t]).double().cpu()
    assert torch.allclose(got_t, want_rows[:, :R], atol=0.03, rtol=0.02)
    q = torch.randn(n, H * (d + dr), generator=g).to(td)
    uk = (torch.randn(H * d, R, generator=g) * 0.3).to(td)
    qa = ops.latent_query(q.cuda(), uk.cuda(), cos, sin, H, d, dr, R).double().cpu()
    qd = q.double().reshape(n, H, d + dr)
    want_qa = torch.cat([torch.einsum("thd,hdr->thr", qd[..., :d], uk.double().reshape(H, d, R)), P.rotate(qd[..., d:], pos, rot)], -1)
    assert torch.allclose(qa, want_qa, **tol)
    o_lat = torch.randn(n, H, R, generator=g)
    uv = (torch.randn(H * dv, R, generator=g) * 0.3).to(td)
    out = ops.latent_output(o_lat.cuda(), uv.cuda(), down.cuda()[:, Q + R + dr:], H, R, dv, td).double().cpu()
    want = torch.einsum("thr,hvr->thv", o_lat.double(), uv.double().reshape(H, dv, R)) * torch.sigmoid(dd[:, Q + R + dr:]).unsqueeze(-1)
    assert torch.allclose(out, want.reshape(n, H * dv), **tol)


@gpu
def test_router_ties_all_experts_and_more_experts_than_a_wave():
    from palm_infra_amd.kernels import ops
    z = torch.tensor([[1.0, 3.0, 2.5, 3.0], [0.0, 0.0, 0.0, 0.0], [-1.0, 5.0, 4.0, -2.0]], device="cuda")
    chosen, weight = ops.moe_route(z, 2)
    assert chosen.tolist() == [[1, 3], [0, 1], [1, 2]]                              # the lower index wins a tie
    assert torch.allclose(weight.cpu(), torch.tensor([[0.5, 0.5], [0.5, 0.5], [1 / (1 + math.exp(-1)), 1 / (1 + math.e)]]), atol=1e-6)
    chosen, weight = ops.moe_route(z, 4)
    assert sorted(chosen[2].tolist()) == [0, 1, 2, 3] and torch.allclose(weight[2].cpu(), torch.softmax(z[2].cpu()[chosen[2].long().cpu()], 0), atol=1e-6)
    torch.manual_seed(3)
    z = torch.randn(40, 150, device="cuda")
    chosen, weight = ops.moe_route(z, 9)
    val, idx = torch.topk(z.cpu(), 9, dim=-1)
    assert torch.equal(chosen.cpu().long(), idx) and torch.allclose(weight.cpu(), torch.softmax(val, -1), atol=1e-6)


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_experts_few_rows_and_many_rows_agree_with_the_plain_mixture(tmp_path_factory, dtype):
    """The feed-forward part alone: a step of few rows (every row reads its experts itself) and a step of many (rows grouped
    by expert on the host) against the plain mixture, from the one-layer model's weights."""
    from palm_infra_amd.parts import Builder
    from palm_infra_amd.weights import ModelFiles, load_weights
    from palm_infra_amd.config import config_from_dir
    td = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    d = model_dir(tmp_path_factory, "feed_forward", dtype)
    files = ModelFiles(d)
    cfg = config_from_dir(d).with_tensor_shapes({n: files.shape(n) for n in files.names()})
    spec = cfg.spec(files.names())
    part = Builder(load_weights(spec, files, td, "cuda"), td, "cuda").build(spec.layers[0].parts["feed_forward"])
    raw, t = P.read_model(d)
    torch.manual_seed(4)
    for n in (3, 128, 129, 300):
        h = torch.randn(n, 32).to(td)
        want = P.mixture(h.double(), t, "l0.mlp.", raw["layers"][0]["mlp"])
        got = part.forward(h.cuda(), None).double().cpu()
        assert torch.allclose(got, want, atol=1e-4 if dtype == "float32" else 0.05, rtol=1e-4 if dtype == "float32" else 0.03), (n, float((got - want).abs().max()))


# ---- whole models ----------------------------------------------------------------------------------------

@gpu
@pytest.mark.parametrize("name,dtype", CASES)
def test_each_request_alone_and_whole(tmp_path_factory, name, dtype):
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, name, dtype)
    for ids in S.prompts(raw_of(name), LENGTHS[name]):
        slot = eng.open()
        got = eng.step([StepEntry(slot, ids, list(range(len(ids))))])
        eng.close(slot)
        assert_close(got, reference(tmp_path_factory, name, dtype, ids), dtype, f"{name} whole {len(ids)}")
    eng.cache.check()


@gpu
def test_a_checkpoint_with_norms_for_a_feed_forward_that_is_not_there(tmp_path):
    from palm_infra_amd.engine import Engine, StepEntry
    from palm_infra_amd.weights import write_safetensors
    raw = raw_of("A")
    tensors = S.sharpened_tensors(raw, 7, "float32")
    tensors["l1.norm2"] = torch.full((64,), 3.0)
    tensors["l1.norm2b"] = torch.full((64,), -2.0)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    write_safetensors(tmp_path / "model.safetensors", tensors)
    eng = Engine.from_dir(tmp_path, dtype="float32", max_tokens=256)
    ids = S.prompts(raw, [40], seed=12)[0]
    slot = eng.open()
    got = eng.step([StepEntry(slot, ids, list(range(len(ids))))])
    eng.close(slot)
    cfg, w = P.read_model(tmp_path)
    assert_close(got, P.forward(cfg, w, ids), "float32", "spare norms")


@gpu
@pytest.mark.parametrize("name,dtype", CASES)
def test_prompt_then_every_token_alone_from_the_first(tmp_path_factory, name, dtype):
    """Token-by-token decoding from the very first token (every state starts from zero, the convolution from its zero
    padding, the window from an empty page), through recorded steps, across page borders and past the windows; against the
    whole prompt in one step."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, name, dtype)
    ids = S.prompts(raw_of(name), [150], seed=4)[0]
    ref = reference(tmp_path_factory, name, dtype, ids)
    slot = eng.open()
    pool = Pool(dtype, f"{name} one by one")
    for t, tok in enumerate(ids):
        pool.add(eng.step([StepEntry(slot, [tok], [0])]), ref[t:t + 1])
        assert eng.length(slot) == t + 1
    eng.close(slot)
    pool.check()


@gpu
@pytest.mark.parametrize("name,dtype", CASES)
@pytest.mark.parametrize("portion", [2, 3, 7, 64, 65])
def test_prompt_in_portions(tmp_path_factory, name, dtype, portion):
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, name, dtype)
    ids = S.prompts(raw_of(name), [140], seed=5)[0]
    ref = reference(tmp_path_factory, name, dtype, ids)
    slot = eng.open()
    got = []
    for lo in range(0, len(ids), portion):
        piece = ids[lo:lo + portion]
        got.append(eng.step([StepEntry(slot, piece, list(range(len(piece))))]))
    eng.close(slot)
    assert_close(torch.cat(got), ref, dtype, f"{name} in portions of {portion}")


@gpu
@pytest.mark.parametrize("name,dtype", CASES)
def test_batches_of_unequal_requests_and_reused_slots(tmp_path_factory, name, dtype):
    """Two batches through the same slots and pages: prompts of unequal lengths in one step minus their last tokens, which
    come one a step; a request that has no tokens left ends and gives its slot and pages back at once."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, name, dtype)
    for round_no, (seed, tails) in enumerate([(6, [0, 1, 9, 3, 20, 5, 2, 11]), (7, [12, 0, 2, 7, 30, 1, 1, 4])]):
        lengths = LENGTHS[name] if round_no == 0 else LENGTHS[name][::-1]
        reqs = S.prompts(raw_of(name), lengths, seed=seed)
        tails = [min(t, len(r) - 1) for t, r in zip(tails, reqs)]
        slots = [eng.open() for _ in reqs]
        assert sorted(slots) == list(range(len(reqs)))                # the second batch gets the first one's slots
        cuts = [len(r) - t for r, t in zip(reqs, tails)]
        got = {i: [] for i in range(len(reqs))}
        out = eng.step([StepEntry(s, r[:c], list(range(c))) for s, r, c in zip(slots, reqs, cuts)])
        o = 0
        for i, c in enumerate(cuts):
            got[i].append(out[o:o + c])
            o += c
        live, fed = list(range(len(reqs))), list(cuts)
        while True:
            for i in [i for i in live if fed[i] == len(reqs[i])]:
                eng.close(slots[i])
                live.remove(i)
            if not live:
                break
            out = eng.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live])
            for r, i in enumerate(live):
                got[i].append(out[r:r + 1])
                fed[i] += 1
        for i, r in enumerate(reqs):
            assert_close(torch.cat(got[i]), reference(tmp_path_factory, name, dtype, r), dtype,
                         f"{name} batch {round_no} request {i} ({len(r)} tokens, {tails[i]} one by one)")
        eng.cache.check()
        assert all(g.table.pages.held_count == 0 for g in eng.cache.paged_groups)


@gpu
@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("B", "float32"), ("C", "float32")])
def test_long_decoding(tmp_path_factory, name, dtype):
    """A short prompt, then some hundred tokens one by one over several pages and several windows, two sequences side by
    side that started at different lengths; a windowed layer gives pages back on the way."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, name, dtype)
    a, b = S.prompts(raw_of(name), [330, 270], seed=8)
    refs = [reference(tmp_path_factory, name, dtype, a), reference(tmp_path_factory, name, dtype, b)]
    sa, sb = eng.open(), eng.open()
    first = eng.step([StepEntry(sa, a[:70], [69]), StepEntry(sb, b[:10], [9])])
    pool = Pool(dtype, f"{name} long decoding")
    pool.add(first, torch.stack([refs[0][69], refs[1][9]]))
    for i in range(260):
        out = eng.step([StepEntry(sa, [a[70 + i]], [0]), StepEntry(sb, [b[10 + i]], [0])])
        pool.add(out, torch.stack([refs[0][70 + i], refs[1][10 + i]]))
    windowed = [g for g in eng.cache.paged_groups if g.table.window]
    assert all(g.table.pages.held_count <= 2 * (g.table.window // 64 + 2) for g in windowed)      # two sequences' windows, not their lengths
    eng.close(sa)
    eng.close(sb)
    pool.check()


@gpu
@pytest.mark.parametrize("name", ["A", "B"])
def test_recorded_and_launched_steps_agree(tmp_path_factory, name):
    """Decode steps replayed from a HIP graph against the same steps launched kernel by kernel, several replays with other
    work between them."""
    from palm_infra_amd.engine import StepEntry
    ids = S.prompts(raw_of(name), [90], seed=9)[0]
    outs = []
    for graphs in (True, False):
        eng = engine_for(tmp_path_factory, name, "float32", graphs=graphs)
        assert eng.model.capturable
        slot = eng.open()
        got = [eng.step([StepEntry(slot, ids[:50], [49])])]
        for t in range(50, 90):
            got.append(eng.step([StepEntry(slot, [ids[t]], [0])]))
            torch.cuda.synchronize()
        eng.close(slot)
        outs.append(torch.cat(got).cpu())
    assert torch.allclose(outs[0], outs[1], atol=1e-5)
    assert_close(outs[0], reference(tmp_path_factory, name, "float32", ids)[49:], "float32", f"{name} recorded steps")


@gpu
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_greedy_generation_through_generate(tmp_path_factory, name):
    from palm_infra_amd.sampling import GREEDY
    eng = engine_for(tmp_path_factory, name, "float32")
    cfg, w = P.read_model(model_dir(tmp_path_factory, name, "float32"))
    prompts = S.prompts(raw_of(name), [5, 1, 66, 19], seed=10)
    results, metrics = eng.generate(prompts, GREEDY, max_new_tokens=12, ignore_eos=True, max_batch=3)
    for p, r in zip(prompts, results):
        assert r.token_ids == P.greedy(cfg, w, p, 12), f"{name}: prompt of {len(p)} tokens"
    eng.cache.check()
    assert eng.cache.slots.held_count == 0


@gpu
def test_command_line_generates_for_the_design(tmp_path_factory, capsys):
    from palm_infra_amd.engine.cli import chat_main
    d = model_dir(tmp_path_factory, "C", "float32")
    cfg, w = P.read_model(d)
    rc = chat_main(["--package", str(d), "--prompt-ids", "5,6,7", "--max-new-tokens", "6", "--temperature", "0",
                    "--dtype", "float32", "--ignore-eos"])
    assert rc == 0
    assert " ".join(str(t) for t in P.greedy(cfg, w, [5, 6, 7], 6)) in capsys.readouterr().out


@gpu
def test_trace_replay_of_a_batch_then_single_tokens(tmp_path_factory, tmp_path):
    """bin/trace_run as a child process: four requests of unequal lengths in one batch, then one token each while the
    shorter ones end; the files it writes against the plain implementation."""
    import subprocess
    import sys
    from pathlib import Path
    import numpy as np
    d = model_dir(tmp_path_factory, "A", "float32")
    reqs = S.prompts(raw_of("A"), [75, 4, 140, 1], seed=11)
    heads = [70, 2, 130, 1]
    steps = [{"step": 0, "entries": [{"id": f"r{i}", "tokens": r[:h], "want": [0, h - 1]} for i, (r, h) in enumerate(zip(reqs, heads))],
              "end": ["r3"]}]
    fed = list(heads)
    for s in range(1, 11):
        live = [i for i in range(3) if fed[i] < len(reqs[i])]
        steps.append({"step": s, "entries": [{"id": f"r{i}", "tokens": [reqs[i][fed[i]]], "want": [0] if s % 2 else []} for i in live],
                      "end": [f"r{i}" for i in live if fed[i] + 1 == len(reqs[i])]})
        for i in live:
            fed[i] += 1
    root = Path(__file__).resolve().parent.parent
    out = tmp_path / "out"
    run = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(d), "--dtype", "float32", "--out", str(out),
                          "--max-tokens", "320"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [ln for ln in run.stdout.splitlines() if ln.startswith("done")] == [f"done {s}" for s in range(11)]
    refs = [reference(tmp_path_factory, "A", "float32", r) for r in reqs]
    first = np.fromfile(out / "0.f32", dtype="<f4").reshape(8, -1)
    want = torch.stack([refs[i][p] for i, h in enumerate(heads) for p in (0, h - 1)])
    assert_close(torch.from_numpy(first.copy()), want, "float32", "trace step 0")
    fed = list(heads)
    for s in range(1, 11):
        live = [i for i in range(3) if fed[i] < len(reqs[i])]
        if s % 2:
            got = np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(len(live), -1)
            assert_close(torch.from_numpy(got.copy()), torch.stack([refs[i][fed[i]] for i in live]), "float32", f"trace step {s}")
        else:
            assert not (out / f"{s}.f32").exists()
        for i in live:
            fed[i] += 1
