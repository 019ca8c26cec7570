"""The Sebesun design in the engine against the plain implementation (tests/plain_sebesun.py).

Without a GPU: the configuration, its description as parts and the loader's binding.  On the GPU: every mechanism
alone (one-layer models and the kernels called directly with inputs made so that one far token decides the result),
whole prompts, prompts cut into portions down to two tokens, prefill against token-by-token decoding, batches of
unequal requests against each alone, slots and pages that are used again, long decoding over several pages, the
first tokens of a sequence, and greedy generation through ``generate``.  In float32 and in bfloat16.
"""
import math

import pytest
import torch

import plain_sebesun as P
import sebesun_tiny as S
import tiny
from palm_infra_amd.config import ConfigError, config_from_dict

gpu = pytest.mark.gpu
DTYPES = ("float32", "bfloat16")
LENGTHS = {"P": [1, 2, 63, 64, 65, 130, 200, 17], "Q": [129, 3, 70, 64, 1, 191], "R": [5, 66, 128, 31]}


# ---- without a GPU ---------------------------------------------------------------------------------------

def test_registry_picks_the_design_by_its_config_key():
    cfg = config_from_dict(S.CONFIGS["P"])
    assert type(cfg).__name__ == "SebesunConfig" and cfg.architecture == "Sebesun"
    assert config_from_dict(cfg.to_dict()) == cfg


def test_spec_names_every_tensor_with_its_shape():
    spec = config_from_dict(S.CONFIGS["Q"]).spec()
    exp = spec.expected_tensors()
    assert exp["embed"][0] == (130, 48) and exp["head"][0] == (130, 48) and exp["final.norm"][0] == (48,)
    assert exp["l0.mix.x"][0] == (1 + 2 * 17, 40) and exp["l0.mix.conv"][0] == (40, 2) and exp["l0.mix.A_log"][0] == (40, 17)
    assert exp["l1.mix.q"][0] == (3 * 2 * 24, 48) and exp["l1.mix.k"][0] == (3 * 2 * 24, 48) and exp["l1.mix.v"][0] == (3 * 20, 48)
    assert exp["l3.mix.k"][0] == (1 * 2 * 8, 48) and exp["l3.mix.o"][0] == (48, 2 * 72) and exp["l3.mlp.act"][0] == (2,)
    assert exp["l2.mix.g"][0] == (80, 48) and "l2.norm2" not in exp and "l3.norm2" in exp
    assert [exp[f"l{i}.dwa"][0] for i in range(5)] == [(2,), (3,), (4,), (5,), (6,)]
    assert spec.keeps_results


def test_cache_needs_follow_the_layers():
    from palm_infra_amd.cache import KVNeed, StateNeed
    from palm_infra_amd.parts import cache_needs
    spec = config_from_dict(S.CONFIGS["Q"]).spec()
    needs = [cache_needs(layer) for layer in spec.layers]
    assert needs[0] == [StateNeed("scan", (40, 17)), StateNeed("conv", (1, 40))]
    assert needs[1] == [KVNeed(6, 24, None, value_heads=3, value_dim=20)]
    assert needs[2] == [StateNeed("retention", (1, 24, 80))]
    assert needs[4] == [StateNeed("scan", (72, 33)), StateNeed("conv", (0, 72))]


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="lstm"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][1]["mixer"].update(rot={"dims": 7, "base": 10.0}), "rot"),
    (lambda c: c["layers"][2]["mlp"].update(kind="routed"), "dense"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_bad_configurations_are_refused(change, what):
    import copy
    raw = copy.deepcopy(S.CONFIGS["P"])
    change(raw)
    with pytest.raises(ConfigError, match=what):
        config_from_dict(raw)


def test_random_model_folder_is_read_by_the_plain_implementation(tmp_path):
    from palm_infra_amd.weights import write_random_model
    d = write_random_model(S.CONFIGS["R"], 5, tmp_path / "m", "bfloat16")
    cfg, w = P.read_model(d)
    assert cfg["layers"][0]["type"] == "retention" and w["l0.mix.q"].shape == (64, 40) and w["l0.mix.v"].shape == (96, 40)
    logits = P.forward(cfg, w, [1, 2, 3])
    assert logits.shape == (3, 97) and torch.isfinite(logits).all()


def test_plain_retention_equals_its_sum_over_the_past():
    """The oracle's recurrence against the closed form o_t = sum_(s<=t) decay^(t-s) (q_t . k_s) v_s."""
    torch.manual_seed(0)
    m = {"heads": 2, "dim": 6, "vdim": 5, "decay": [0.9, 0.7], "rot": {"dims": 4, "base": 50.0}}
    W, T = 10, 9
    w = {"q": torch.randn(12, W, dtype=P.F64), "k": torch.randn(12, W, dtype=P.F64), "v": torch.randn(10, W, dtype=P.F64),
         "g": torch.randn(10, W, dtype=P.F64), "o": torch.eye(10, dtype=P.F64)}
    h = torch.randn(T, W, dtype=P.F64)
    got = P.retention(h, w, "", m, 1e-6)
    q = P.rotate_half_split((h @ w["q"].T).view(T, 2, 6), 4, 50.0)
    k = P.rotate_half_split((h @ w["k"].T).view(T, 2, 6), 4, 50.0) * 6 ** -0.5
    v = (h @ w["v"].T).view(T, 2, 5)
    o = torch.zeros(T, 2, 5, dtype=P.F64)
    for hd in range(2):
        for t in range(T):
            for s in range(t + 1):
                o[t, hd] += m["decay"][hd] ** (t - s) * (q[t, hd] @ k[s, hd]) * v[s, hd]
    want = P.unit_rms(o, 1e-6).reshape(T, 10) * P.silu(h @ w["g"].T)
    assert torch.allclose(got, want, atol=1e-10)


# ---- engines and references ------------------------------------------------------------------------------

_dirs, _engines, _refs = {}, {}, {}


def model_dir(tmp_path_factory, name: str, store: str):
    key = (name, store)
    if key not in _dirs:
        raw = S.CONFIGS.get(name) or S.SINGLE[name]
        _dirs[key] = S.write_model(raw, S.SEEDS.get(name, 21), tmp_path_factory.mktemp(f"sebesun_{name}_{store}"), store)
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
    """float32: 1e-4 absolute on logits of order one, the gate that shows faults.  bfloat16: a row's root mean square
    error within a fifth of the logits' scale, all rows together within a twentieth, an element within three quarters.
    A row here or there may break these by rounding alone: the q and k norms divide by the root mean square of a
    projection of as few as 8 values, which now and then is small against the rounding of its input (one row in some
    thousand was off by half the scale with float32 twins exact everywhere).  So one row in a hundred (at least one) may
    be over the row gate, but never by more than the scale itself, and the other gates hold for the rest."""
    if dtype == "float32":
        return tiny.assert_logits_close(got, ref, dtype, what)
    got = torch.as_tensor(got).double().cpu().reshape(ref.shape)
    assert torch.isfinite(got).all(), f"{what}: logits are not finite"
    err = (got - ref.double()).abs().reshape(-1, ref.shape[-1])
    scale = float(ref.double().pow(2).mean().sqrt())
    rows = err.pow(2).mean(-1).sqrt()
    over = rows > 0.2 * scale
    assert int(over.sum()) <= max(1, rows.numel() // 100), (f"{what}: bfloat16 rms error over a fifth of {scale:.3e} in "
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


def raw_of(name):
    return S.CONFIGS.get(name) or S.SINGLE[name]


CASES = [(n, d) for n in ("P", "Q", "R") for d in DTYPES]


# ---- every mechanism alone -------------------------------------------------------------------------------

@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", sorted(S.SINGLE))
def test_one_layer_of_one_kind(tmp_path_factory, kind, dtype):
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, kind, dtype)
    for ids in S.prompts(raw_of(kind), [1, 9, 64, 131]):
        slot = eng.open()
        got = eng.step([StepEntry(slot, ids, list(range(len(ids))))])
        eng.close(slot)
        assert_close(got, reference(tmp_path_factory, kind, dtype, ids), dtype, f"{kind} alone, {len(ids)} tokens")


@gpu
@pytest.mark.parametrize("W", [50, 64, 2048, 5000, 20000])      # no multiple of four, narrow, wide, several groups a thread, beyond them
def test_stream_kernel_norms_adds_and_averages_over_depth(W):
    from palm_infra_amd.kernels import ops
    torch.manual_seed(1)
    n, J = 7, 3
    x = torch.randn(n, W, device="cuda")
    y = torch.randn(n, W, device="cuda") * 3
    w = torch.rand(W, device="cuda") + 0.5
    results = torch.randn(J + 2, n, W, device="cuda")
    mix = torch.randn(J + 1, device="cuda")
    for delta in (y, y.bfloat16()):
        d64 = delta.double()
        summed = x.double() + P.rms_norm(d64, w.double(), 1e-5)
        want = sum(mix[j].double() * results[j].double() for j in range(J)) + mix[J].double() * summed
        xs, rs = x.clone(), results.clone()
        h = ops.add_normed(xs, delta, w, 1e-5, torch.bfloat16, results=rs, mix=mix)
        assert torch.allclose(xs.double(), want, atol=1e-5) and torch.allclose(rs[J].double(), summed, atol=1e-5)
        assert torch.equal(rs[J + 1], results[J + 1]) and torch.equal(rs[:J], results[:J])
        assert torch.equal(h, xs.bfloat16())
        xs = x.clone()
        assert ops.add_normed(xs, delta, w, 1e-5, torch.float32) is xs
        assert torch.allclose(xs.double(), summed, atol=1e-5)


@gpu
def test_xielu_on_both_sides_of_zero():
    from palm_infra_amd.kernels import ops
    z = torch.linspace(-12, 12, 1001, device="cuda")
    for p, q in ((0.3, -0.7), (-2.0, 1.5), (25.0, 0.0)):
        pq = torch.tensor([p, q], device="cuda")
        want = P.xielu(z.double().cpu(), torch.tensor(p, dtype=P.F64), torch.tensor(q, dtype=P.F64))
        got = ops.xielu(z, pq).double().cpu()
        assert torch.allclose(got, want, rtol=2e-6, atol=2e-6)
    assert float(ops.xielu(torch.zeros(1, device="cuda"), torch.tensor([0.3, 0.2], device="cuda"))) == 0.0


def _step_context(lengths_before, new_counts, n_slots=None):
    """A cache-less context for kernels that only need the packed layout: slots 0.., given starts."""
    from palm_infra_amd.parts import make_context
    slots = list(range(len(new_counts)))
    return make_context(slots, list(lengths_before), [[0] * c for c in new_counts], torch.float32, "cuda")


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_retention_kernel_keeps_a_far_token_and_forgets_at_its_decay(dtype):
    """One early token has a large key that the last query is aligned with: among some hundred tokens it decides the
    output, scaled by decay^(distance).  The same rows in one step, and cut into portions of 2, 5 and 64 tokens."""
    from palm_infra_amd.kernels import ops
    torch.manual_seed(2)
    H, dk, dv, T, far = 2, 12, 20, 300, 3
    rows = (torch.randn(T, H * (2 * dk + 2 * dv)) * 0.3)
    direction = torch.randn(dk)
    rows[far, H * dk:H * dk + dk] = direction * 150.0            # k of head 0 at the far token
    rows[T - 1, 0:dk] = direction * 5.0                          # q of head 0 at the last token
    rows = rows.to(dtype).cuda()
    decay = torch.tensor([0.99, 0.9], device="cuda")
    r64 = rows.double().cpu()
    q, k = r64[:, :H * dk].view(T, H, dk), r64[:, H * dk:2 * H * dk].view(T, H, dk) * dk ** -0.5
    v, g = r64[:, 2 * H * dk:2 * H * dk + H * dv].view(T, H, dv), r64[:, 2 * H * dk + H * dv:]
    o = torch.zeros(T, H, dv, dtype=P.F64)
    for hd in range(H):
        Sm = torch.zeros(dk, dv, dtype=P.F64)
        for t in range(T):
            Sm = float(decay[hd]) * Sm + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = Sm.T @ q[t, hd]
    want = P.unit_rms(o, 1e-6).reshape(T, H * dv) * P.silu(g)
    # the far token carries the last row of head 0: without it the direction of o changes
    without = o[T - 1, 0] - 0.99 ** (T - 1 - far) * (q[T - 1, 0] @ k[far, 0]) * v[far, 0]
    assert without.norm() < 0.3 * o[T - 1, 0].norm()
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    final = None
    # (tokens a step, tokens a chunk inside the kernel: None = its own choice, 0 = no chunks)
    for portion, chunk in ((T, 0), (T, None), (T, 32), (T, 104), (150, 64), (64, 0), (5, None), (2, None)):
        state = torch.zeros(2, H, dk, dv, device="cuda")
        got = []
        for lo in range(0, T, portion):
            n = min(portion, T - lo)
            ctx = _step_context([lo], [n])
            got.append(ops.retention(rows[lo:lo + n].contiguous(), H, dk, dv, decay, dk ** -0.5, 1e-6, state, ctx, chunk=chunk))
        got = torch.cat(got).double().cpu()
        assert (got - want).abs().max() < tol, f"portion {portion}, chunk {chunk}: {(got - want).abs().max()}"
        assert torch.count_nonzero(state[1]) == 0                 # the other slot's state is not touched
        final = state[0].clone() if final is None else final
        assert torch.allclose(state[0], final, rtol=1e-4, atol=1e-4), f"portion {portion}, chunk {chunk}: the state left behind differs"
    assert ops.retention_chunk(1, 2, 300) > 0 and ops.retention_chunk(1, 2, 300) < 300      # the second case above did cut


@gpu
@pytest.mark.parametrize("dk,dv", [(12, 28), (40, 72)])      # the second pair is one that the matrix-core kernel takes in bfloat16
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_differential_attention_kernel_far_keys_page_borders_and_the_causal_edge(dtype, dk, dv):
    """Keys made so that one decides a query's output: far back, on either side of a page border, at the query's own
    position; and a large aligned key one position after the query, which the query must not see.  Whole, and with
    the last tokens one by one; two sequences of unequal lengths in one batch."""
    from palm_infra_amd.cache import KVNeed, ModelCache
    from palm_infra_amd.kernels import ops
    from palm_infra_amd.parts import make_context
    torch.manual_seed(3)
    H, G = 4, 2
    scale, lam, gain, eps = 0.5, 0.4, 0.6, 1e-6
    assert ops.diff_mfma_serves(torch.empty(0, dtype=dtype), dk, dv) == (dtype == torch.bfloat16 and dk == 40)
    T = [330, 71]
    width = 2 * (H + G) * dk + G * dv
    seqs = [torch.randn(t, width) * 0.5 for t in T]
    direction = torch.randn(dk)
    direction /= direction.norm()

    def aim(rows, query, key, head=1, which=0):
        g = head // (H // G)
        rows[query, (head * 2 + which) * dk:(head * 2 + which + 1) * dk] = direction * 9.0
        rows[key, 2 * H * dk + (g * 2 + which) * dk:2 * H * dk + (g * 2 + which + 1) * dk] = direction * 9.0

    # (query, key): far, page borders, own position; the key after query 200 must stay unseen
    for qy, ky in ((329, 2), (300, 63), (310, 64), (127, 127), (128, 127), (192, 128), (65, 0)):
        aim(seqs[0], qy, ky)
    aim(seqs[0], 200, 201, which=1)
    aim(seqs[1], 70, 64)
    aim(seqs[1], 63, 1, head=2, which=1)
    q_w, k_w = torch.rand(dk) + 0.5, torch.rand(dk) + 0.5
    seqs = [s.to(dtype) for s in seqs]

    def plain(rows):
        r = rows.double()
        n = r.shape[0]
        q = P.rms_norm(r[:, :2 * H * dk].view(n, H, 2, dk), q_w.double(), eps)
        k = P.rms_norm(r[:, 2 * H * dk:2 * (H + G) * dk].view(n, G, 2, dk), k_w.double(), eps)
        if dtype == torch.bfloat16:                                # the kernel keeps normed q and k in the run's type
            q, k = q.bfloat16().double(), k.bfloat16().double()
        v = r[:, 2 * (H + G) * dk:].view(n, G, dv)
        causal = torch.tril(torch.ones(n, n, dtype=torch.bool))
        out = torch.zeros(n, H, dv, dtype=P.F64)
        for hd in range(H):
            g = hd // (H // G)
            a = [torch.softmax(((q[:, hd, j] @ k[:, g, j].T) * scale).masked_fill(~causal, -math.inf), -1) @ v[:, g] for j in range(2)]
            out[:, hd] = P.unit_rms(a[0] - lam * a[1], eps) * gain
        return out.reshape(n, H * dv)

    want = [plain(s) for s in seqs]
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    need = KVNeed(2 * G, dk, None, value_heads=G, value_dim=dv)
    cache = ModelCache([[need]], [None], 64 * 12, 4, None, dtype, torch.device("cuda"))
    lc = cache.layer_caches[0]
    for tail in (0, 9):
        slots = [cache.open() for _ in T]
        got = [[] for _ in T]
        steps = [[(b, 0, t - tail) for b, t in enumerate(T)]] + [[(b, t - tail + i, 1) for b, t in enumerate(T)] for i in range(tail)]
        for step in steps:
            growth = [(slots[b], n) for b, _, n in step]
            cache.reserve(growth)
            ctx = make_context([slots[b] for b, _, _ in step], [lo for _, lo, _ in step], [[0] * n for _, _, n in step], dtype, "cuda")
            rows = torch.cat([seqs[b][lo:lo + n] for b, lo, n in step]).cuda()
            q = ops.diff_qkv_store(rows, H, G, dk, dv, q_w.cuda(), k_w.cuda(), eps, lc.k, lc.v, lc.kv.table_dev, ctx)
            o = ops.attention_diff(q, lc.k, lc.v, lc.kv.table_dev, ctx, H, G, dk, dv, scale, lam, gain, eps).double().cpu()
            cache.commit(growth)
            at = 0
            for b, _, n in step:
                got[b].append(o[at:at + n])
                at += n
        for b in range(len(T)):
            err = (torch.cat(got[b]) - want[b]).abs().max()
            assert err < tol, f"sequence {b}, last {tail} one by one: {err}"
        for s in slots:
            cache.close(s)
    cache.check()


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
@pytest.mark.parametrize("name,dtype", CASES)
def test_prompt_then_every_token_alone_from_the_first(tmp_path_factory, name, dtype):
    """Token-by-token decoding from the very first token (every state starts from zero, the convolution from its
    zero padding), through recorded steps, across page borders; against the whole prompt in one step."""
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
    """Two batches through the same slots and pages: prompts of unequal lengths in one step minus their last tokens,
    which come one a step; a request that has no tokens left ends and gives its slot and pages back at once."""
    from palm_infra_amd.cache import KVNeed
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, name, dtype)
    paged = eng.cache.groups_of(KVNeed)
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
        assert all(g.table.pages.held_count == 0 for g in paged)


@gpu
@pytest.mark.parametrize("name,dtype", [("P", "float32"), ("Q", "bfloat16"), ("Q", "float32")])
def test_long_decoding(tmp_path_factory, name, dtype):
    """A short prompt, then some hundred tokens one by one over several pages, two sequences side by side that
    started at different lengths."""
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
    eng.close(sa)
    eng.close(sb)
    pool.check()


@gpu
@pytest.mark.parametrize("name", ["P", "Q"])
def test_recorded_and_launched_steps_agree(tmp_path_factory, name):
    """Decode steps replayed from a HIP graph against the same steps launched kernel by kernel, several replays with
    other work between them."""
    from palm_infra_amd.engine import StepEntry
    ids = S.prompts(raw_of(name), [90], seed=9)[0]
    outs = []
    for graphs in (True, False):
        eng = engine_for(tmp_path_factory, name, "float32", graphs=graphs)
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
@pytest.mark.parametrize("name", ["P", "Q", "R"])
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
    d = model_dir(tmp_path_factory, "R", "float32")
    cfg, w = P.read_model(d)
    rc = chat_main(["--package", str(d), "--prompt-ids", "5,6,7", "--max-new-tokens", "6", "--temperature", "0",
                    "--dtype", "float32", "--ignore-eos"])
    assert rc == 0
    assert " ".join(str(t) for t in P.greedy(cfg, w, [5, 6, 7], 6)) in capsys.readouterr().out


@gpu
def test_trace_replay_of_many_short_requests_counted_by_their_tokens(tmp_path_factory, tmp_path):
    """bin/trace_run as a child process: six requests of 70 tokens in one batch and then one token each, with
    --max-tokens counting the tokens they hold (426) and not the pages they touch (twelve)."""
    import json
    import subprocess
    import sys
    from pathlib import Path
    import numpy as np
    d = model_dir(tmp_path_factory, "P", "float32")
    reqs = S.prompts(raw_of("P"), [71] * 6, seed=11)
    steps = [{"step": 0, "entries": [{"id": f"r{i}", "tokens": r[:70], "want": [0, 69]} for i, r in enumerate(reqs)], "end": []},
             {"step": 1, "entries": [{"id": f"r{i}", "tokens": r[70:], "want": [0]} for i, r in enumerate(reqs)], "end": [f"r{i}" for i in range(6)]}]
    root = Path(__file__).resolve().parent.parent
    proc = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(d), "--dtype", "float32", "--out", str(tmp_path / "o"),
                           "--max-tokens", "426"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1"]
    V = raw_of("P")["vocab"]
    first = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(-1, V).copy())
    second = torch.from_numpy(np.fromfile(tmp_path / "o" / "1.f32", dtype="<f4").reshape(-1, V).copy())
    for i, r in enumerate(reqs):
        ref = reference(tmp_path_factory, "P", "float32", r)
        assert_close(first[2 * i:2 * i + 2], ref[[0, 69]], "float32", f"request {i}, prompt")
        assert_close(second[i:i + 1], ref[70:71], "float32", f"request {i}, decoded")
