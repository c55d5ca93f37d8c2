"""The Biguzen design in the engine against the plain implementation (tests/plain_biguzen.py).

Without a GPU: the configuration, its description as parts, the run order and cache plan of layers that read another
layer's keys and values, and the oracle's own mechanisms against closed forms.  On the GPU: every mechanism alone (one-layer
models, and the kernels called directly with inputs made so that one far key, one key at a window's or a page's edge, a
sink, a far write into the memory or a group of experts decides the result), whole prompts, prompts cut into portions down
to two tokens, prefill against token-by-token decoding from the first token, batches of unequal requests against each alone,
slots and pages that are used again, long decoding over several pages and past the windows, a prompt longer than a step
takes at once, recorded against launched steps, and greedy generation through ``generate``, the command line and the trace
replay.  In float32 and in bfloat16.
"""
import json
import math

import pytest
import torch

import biguzen_tiny as S
import plain_biguzen as P
from palm_infra_amd.config import ConfigError, config_from_dict

gpu = pytest.mark.gpu
DTYPES = ("float32", "bfloat16")
LENGTHS = {"A": [1, 2, 63, 64, 65, 130, 200, 17], "B": [129, 3, 70, 71, 1, 191], "C": [300, 9, 140], "D": [5, 66, 128, 31]}


# ---- without a GPU ---------------------------------------------------------------------------------------

def test_registry_picks_the_design_by_its_config_key():
    cfg = config_from_dict(S.CONFIGS["A"])
    assert type(cfg).__name__ == "BiguzenConfig"
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    assert config_from_dict(json.loads(json.dumps(cfg.to_dict()))).streams == 3


def test_spec_names_every_tensor():
    spec = config_from_dict(S.CONFIGS["A"]).spec()
    names = spec.expected_tensors()
    assert names["embed"][0] == (211, 64) and names["final.norm"][0] == (64,) and names["final.norm.alpha"][0] == ()
    assert names["l0.mix.q"][0] == (48, 64) and names["l0.mix.v"][0] == (72, 64) and names["l0.mix.i"][0] == (3, 64) and names["l0.mix.f.b"][0] == (3,)
    assert names["l0.mix.norm"][0] == (72,) and names["l0.mix.o"][0] == (64, 72)
    assert names["l0.mlp.e11.up"][0] == (24, 64) and names["l0.mlp.e0.down"][0] == (64, 24) and names["l0.mlp.router"][0] == (12, 64)
    assert names["l0.mlp.correction"][0] == (12,) and names["l0.mlp.shared.sg"][0] == (1, 64) and names["l0.mlp.shared.up"][0] == (40, 64)
    assert names["l1.mix.q"][0] == (96, 64) and names["l1.mix.k"][0] == (48, 64) and names["l1.mix.v"][0] == (80, 64) and names["l1.mix.g"][0] == (4, 64)
    assert names["l1.mix.q.conv"][0] == (96, 4) and names["l1.mix.v.conv"][0] == (80, 4) and names["l1.mix.k.b"][0] == (48,) and names["l1.mix.sink"][0] == (4,)
    assert names["l1.mlp.up"][0] == (40, 64) and names["l1.hc2.mix"][0] == (3, 3) and names["l1.hc1.in"][0] == (3,) and names["l1.norm1.b"][0] == (64,)
    # the layer that reads layer 1's keys and values has none of their tensors; it has no feed-forward either
    assert names["l2.mix.q.conv"][0] == (96, 2) and not any(n.startswith(("l2.mix.k", "l2.mix.v", "l2.mlp", "l2.norm2", "l2.hc2")) for n in names)
    assert "head" not in names                                             # the head is the table itself
    assert "l0.mix.q.conv" not in config_from_dict(S.CONFIGS["B"]).spec().expected_tensors()


def test_second_norm_and_stream_weights_of_a_feed_forward_that_is_not_there_are_bound_if_the_file_has_them():
    cfg = config_from_dict(S.CONFIGS["A"])
    names = list(cfg.spec().expected_tensors())
    with_spares = cfg.spec(names + ["l2.norm2", "l2.norm2.alpha", "l2.hc2.mix"]).expected_tensors()
    assert with_spares["l2.norm2"][0] == (64,) and with_spares["l2.norm2.alpha"][0] == () and with_spares["l2.hc2.mix"][0] == (3, 3)
    assert len(with_spares) == len(names) + 3 and set(cfg.spec(names).expected_tensors()) == set(names)


def test_run_order_and_cache_plan_of_layers_that_read_another_layers_keys():
    from palm_infra_amd.cache import KVNeed, StateNeed
    from palm_infra_amd.parts import cache_needs, cache_needs_beside_shared
    spec = config_from_dict(S.CONFIGS["A"]).spec()
    assert [(c.layer, c.cache_of) for c in spec.order] == [(0, None), (1, None), (2, 1), (3, None)] and spec.streams == 3
    assert cache_needs(spec.layers[0]) == [StateNeed("mlstm", (3, 16, 25)), StateNeed("mlstm_max", (3,))]
    # layer 1's keys are kept by the longer window of its reader; both have a convolution's state over their own channels
    assert cache_needs(spec.layers[1]) == [KVNeed(2, 24, 70, value_dim=40), StateNeed("conv", (3, 96 + 48 + 80))]
    assert cache_needs_beside_shared(spec.layers[2]) == [StateNeed("conv", (1, 96))]
    with pytest.raises(ValueError, match="borrows"):
        cache_needs(spec.layers[2])
    b = config_from_dict(S.CONFIGS["B"]).spec()
    assert cache_needs(b.layers[0]) == [KVNeed(3, 40, None, value_dim=72)]                 # no convolution, no window
    assert cache_needs(b.layers[2])[0] == KVNeed(1, 16, None, value_dim=16)               # its reader has no window: every key is kept
    c = config_from_dict(S.CONFIGS["C"]).spec()
    assert cache_needs(c.layers[0])[0] == KVNeed(2, 64, 200, value_dim=32) and cache_needs(c.layers[4]) == [KVNeed(2, 32, 64, value_dim=96)]


def test_an_entry_that_reads_another_entrys_cache_keeps_a_state_of_its_own():
    from palm_infra_amd.cache import KVNeed, ModelCache, StateNeed
    needs = [[KVNeed(1, 8, 20), StateNeed("conv", (2, 24))], [StateNeed("other", (3,))], [StateNeed("conv", (2, 8))]]
    cache = ModelCache(needs, [None, None, 0], 256, 4, None, torch.float32, "cpu")
    own, reader = cache.layer_caches[0], cache.layer_caches[2]
    assert reader.kv is own.kv and reader.kv_entry == own.kv_entry and not reader.writes and own.writes
    assert own.states["conv"].shape == (5, 2, 24) and reader.states["conv"].shape == (5, 2, 8)
    assert reader.states["conv"].data_ptr() != own.states["conv"].data_ptr() and "other" not in reader.states
    with pytest.raises(ValueError, match="of its own"):
        ModelCache([[KVNeed(1, 8)], [KVNeed(1, 8)]], [None, 0], 256, 4, None, torch.float32, "cpu")


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="retention"), "type"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "kv heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=26), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"].update(conv=40), "conv"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=0), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "kv_from"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=24), "kv_heads, dim or vdim"),
    (lambda c: c["layers"][0]["mixer"].pop("gate_cap"), "gate_cap"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "choices"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=5), "groups"),
    (lambda c: c["layers"][1]["mlp"].pop("ff"), "ff"),
    (lambda c: c.pop("streams"), "streams"),
    (lambda c: c.update(streams=40), "streams"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_bad_configurations_are_refused(change, what):
    raw = json.loads(json.dumps(S.CONFIGS["A"]))
    change(raw)
    with pytest.raises(ConfigError, match=what):
        config_from_dict(raw)


def test_random_model_folder_is_read_by_the_plain_implementation(tmp_path):
    from palm_infra_amd.weights import write_random_model
    write_random_model(S.CONFIGS["D"], 3, tmp_path, "bfloat16")
    cfg, w = P.read_model(tmp_path)
    layers = []
    logits = P.forward(cfg, w, [1, 2, 3, 4, 5], layers)
    assert logits.shape == (5, 97) and torch.isfinite(logits).all() and len(layers) == 2


def test_plain_sink_takes_weight_and_gives_nothing():
    """One key of score s against a sink of score z: the key's weight is e^s / (e^z + e^s), each head with its own z."""
    q = torch.tensor([[[2.0, 0.0], [2.0, 0.0]]], dtype=P.F64)
    k = torch.tensor([[[1.5, 0.0]]], dtype=P.F64)
    v = torch.tensor([[[3.0, -1.0, 2.0]]], dtype=P.F64)
    s = 0.5 * 3.0
    sink = torch.tensor([0.0, 2.0], dtype=P.F64)
    out = P.sink_softmax_heads(q, k, v, 0.5, None, sink)
    assert torch.allclose(out[0, 0], v[0, 0] * math.exp(s) / (1 + math.exp(s)))
    assert torch.allclose(out[0, 1], v[0, 0] * math.exp(s) / (math.exp(2.0) + math.exp(s)))
    assert float(P.sink_softmax_heads(q, -20 * k, v, 0.5, None, sink).abs().max()) < 1e-10


def test_plain_window_sees_itself_and_the_tokens_before_it():
    T, size = 9, 4
    q = torch.zeros(T, 2, 3, dtype=P.F64)
    k = torch.randn(T, 1, 3, dtype=P.F64)
    v = torch.eye(T, dtype=P.F64).reshape(T, 1, T)
    out = P.sink_softmax_heads(q, k, v, 1.0, size, torch.zeros(2, dtype=P.F64))
    for i in range(T):
        seen = [j for j in range(T) if 0 <= i - j < size]
        want = torch.zeros(T, dtype=P.F64)
        want[seen] = 1.0 / (1 + len(seen))
        assert torch.allclose(out[i, 0], want) and torch.allclose(out[i, 1], want)


def test_plain_convolution_and_rotation_of_neighbours():
    u = torch.arange(1.0, 11.0, dtype=P.F64).reshape(5, 2)
    w = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 2.0]], dtype=P.F64)
    y = P.short_convolution(u, w)
    assert y[:, 1].tolist() == [4.0, 8.0, 12.0, 16.0, 20.0]                        # the last tap is the token itself
    assert y[:, 0].tolist() == [100.0, 310.0, 531.0, 753.0, 975.0]                 # zeros before the start
    x = torch.tensor([[[1.0, 0.0, 0.0, 1.0, 5.0, 6.0]]], dtype=P.F64).repeat(3, 1, 1)
    r = P.rotate_neighbours(x, torch.tensor([0, 1, 2]), {"dims": 4, "base": 100.0, "scaling": {"factor": 2.0}})
    assert torch.allclose(r[0], x[0]) and torch.allclose(r[:, :, 4:], x[:, :, 4:])
    f0, f1 = 1.0 / 2.0, 100.0 ** -0.5 / 2.0
    assert torch.allclose(r[2, 0, :4], torch.tensor([math.cos(2 * f0), math.sin(2 * f0), -math.sin(2 * f1), math.cos(2 * f1)], dtype=P.F64))


def test_plain_matrix_memory_is_a_gated_sum_over_its_past():
    torch.manual_seed(0)
    T, d, dv = 9, 3, 4
    q, k, v = (torch.randn(T, n, dtype=P.F64) for n in (d, d, dv))
    li, lf = torch.randn(T, dtype=P.F64), -torch.rand(T, dtype=P.F64)
    out = P.matrix_memory(q, k, v, li, lf)
    m = 0.0
    for t in range(T):
        m = max(float(lf[t]) + m, float(li[t]))
        # the weight of write j at time t: exp(i_j + sum of the forget gates after j), not relative to anything
        wgt = [math.exp(float(li[j]) + float(lf[j + 1:t + 1].sum())) for j in range(t + 1)]
        num = sum(w * float(q[t] @ k[j]) * v[j] for j, w in enumerate(wgt))
        nq = sum(w * float(q[t] @ k[j]) for j, w in enumerate(wgt))
        want = num / (max(abs(nq), 1.0) + 1e-6 * math.exp(m))
        assert torch.allclose(out[t], want, rtol=1e-9, atol=1e-12)


def test_plain_routing_by_groups_with_negative_scores():
    """Four experts in two groups, one group kept.  With a correction that makes every choice score negative, the experts of
    the group that is not kept must not win as if they had scored zero."""
    w = {"r.router": torch.tensor([[1.0], [0.0], [-1.0], [3.0]], dtype=P.F64), "r.correction": torch.tensor([-5.0, -5.0, -5.0, -7.5], dtype=P.F64)}
    r = {"experts": 4, "top": 2, "scale": 2.0, "groups": {"count": 2, "keep": 1}}
    chosen, weights = P.route(torch.tensor([[1.0]], dtype=P.F64), w, "r.", r)
    s = [1 / (1 + math.exp(-z)) for z in (1.0, 0.0, -1.0, 3.0)]
    # group 0: (s0 - 5) + (s1 - 5) = -8.77; group 1: (s2 - 5) + (s3 - 7.5) = -11.28: group 0 is kept
    assert sorted(chosen[0].tolist()) == [0, 1]
    by_expert = dict(zip(chosen[0].tolist(), weights[0].tolist()))
    assert math.isclose(by_expert[0], 2.0 * s[0] / (s[0] + s[1])) and math.isclose(by_expert[1], 2.0 * s[1] / (s[0] + s[1]))
    r1 = {"experts": 4, "top": 2, "scale": 1.0}
    chosen1, _ = P.route(torch.tensor([[1.0]], dtype=P.F64), w, "r.", r1)
    assert sorted(chosen1[0].tolist()) == [0, 1]                    # without groups: the two largest corrected scores
    w["r.correction"] = torch.tensor([0.0, 0.0, 0.0, 0.0], dtype=P.F64)
    assert sorted(P.route(torch.tensor([[1.0]], dtype=P.F64), w, "r.", r1)[0][0].tolist()) == [0, 3]


# ---- on the GPU ------------------------------------------------------------------------------------------

_dirs, _engines, _refs = {}, {}, {}


def raw_of(name: str) -> dict:
    return S.CONFIGS.get(name) or S.SINGLE[name]


def model_dir(tmp_path_factory, name: str, store: str):
    key = (name, store)
    if key not in _dirs:
        _dirs[key] = S.write_model(raw_of(name), S.SEEDS.get(name, 81), tmp_path_factory.mktemp(f"biguzen_{name}_{store}"), store)
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
    """float32: 1e-4 of the logits' scale, the gate that shows faults.  bfloat16: a row's root mean square error within a
    tenth of the logits' scale, all rows together within a twentieth, an element within half of it; but one row in thirty
    (at least one) may lie beyond the row's bound.  The design has places where rounding decides much: a choice between two
    experts of nearly equal scores may fall the other way for a token, and a head of the matrix memory whose query is
    nearly orthogonal to the key just written leaves a small remainder that its unit norm scales up again.  The float32
    runs hold every row; the kernels' own tests below hold every row in bfloat16 with inputs that are not such places."""
    got = torch.as_tensor(got).double().cpu().reshape(ref.shape)
    assert torch.isfinite(got).all(), f"{what}: logits are not finite"
    err = (got - ref.double()).abs().reshape(-1, ref.shape[-1])
    scale = float(ref.double().pow(2).mean().sqrt())
    if dtype == "float32":
        worst = float(err.max())
        assert worst <= 1e-4 * max(1.0, scale), f"{what}: float32 logits differ by {worst:.3e} (their scale is {scale:.3e})"
        return
    rows = err.pow(2).mean(-1).sqrt()
    over = rows > 0.1 * scale
    assert int(over.sum()) <= max(1, rows.numel() // 30), f"{what}: {int(over.sum())} of {rows.numel()} rows beyond the bfloat16 bound"
    err, rows = err[~over], rows[~over]
    if rows.numel() == 0:
        return
    assert float(rows.max()) <= 0.1 * scale, f"{what}: bfloat16 rms error {float(rows.max()):.3e} in row {int(rows.argmax())} vs {scale:.3e}"
    if rows.numel() >= 16:
        assert float(err.pow(2).mean().sqrt()) <= 0.05 * scale, f"{what}: bfloat16 rms error over all rows vs {scale:.3e}"
    assert float(err.max()) <= 0.5 * scale, f"{what}: bfloat16 max error {float(err.max()):.3e} vs {scale:.3e}"


CASES = [(n, d) for n in ("A", "B", "C", "D") for d in DTYPES]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


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
    for ids in S.prompts(raw_of(kind), [1, 7, 64, 131], seed=1):
        slot = eng.open()
        got = eng.step([StepEntry(slot, ids, list(range(len(ids))))])
        eng.close(slot)
        assert_close(got, reference(tmp_path_factory, kind, dtype, ids), dtype, f"{kind} whole {len(ids)}")


@gpu
@pytest.mark.parametrize("W", [50, 64, 2048, 5000])
@pytest.mark.parametrize("norm", [None, "dyt", "rms"])
def test_streams_are_written_and_read_in_one_pass(W, norm):
    """A sublayer's output into S streams with a full mix matrix, and the next reader's weighted sum through its norm; over all
    rows (the streams are left updated) and over a selection (they stay as they were); a read alone; a write alone."""
    from palm_infra_amd.kernels import ops
    torch.manual_seed(W)
    for S_, n in ((1, 5), (3, 70), (5, 9)):
        xs = torch.randn(n, S_, W)
        y = torch.randn(n, W)
        mix, out_w, in_w = torch.randn(S_, S_), torch.randn(S_), torch.randn(S_)
        nw, nb, alpha, eps = torch.randn(W) + 1, torch.randn(W), 0.7, 1e-5
        new = torch.einsum("sr,nsw->nrw", mix.double(), xs.double()) + out_w.double()[None, :, None] * y.double()[:, None, :]

        def normed(u):
            if norm == "dyt":
                return P.dynamic_tanh(u, nw.double(), nb.double(), alpha)
            return P.unit_rows(u, eps) * nw.double() if norm == "rms" else u

        dev = lambda t: t.cuda()
        kw = dict(norm_w=dev(nw) if norm else None, norm_b=dev(nb) if norm == "dyt" else None, alpha=alpha, eps=eps)
        for dt, tol in ((torch.float32, 2e-5), (torch.bfloat16, 2e-2)):
            a = dev(xs.clone())
            got = ops.streams_mix_norm(a, dev(y).to(dt), dev(mix), dev(out_w), dev(in_w), norm, out_dtype=dt, **kw)
            yr = y.to(dt).double()
            new_r = torch.einsum("sr,nsw->nrw", mix.double(), xs.double()) + out_w.double()[None, :, None] * yr[:, None, :]
            want = normed(torch.einsum("s,nsw->nw", in_w.double(), new_r))
            assert torch.allclose(a.cpu().double(), new_r, atol=1e-5, rtol=1e-5)
            assert torch.allclose(got.cpu().double(), want, atol=tol * float(want.abs().max()), rtol=tol), (S_, dt)
        # a selection of rows: the streams stay
        rows = torch.tensor([n - 1, 0, n // 2], dtype=torch.int32)
        a = dev(xs.clone())
        got = ops.streams_mix_norm(a, dev(y), dev(mix), dev(out_w), None, norm, rows=dev(rows), out_dtype=torch.float32, **kw)
        assert torch.equal(a.cpu(), xs)
        want = normed(new.sum(1))[rows.long()]
        assert torch.allclose(got.cpu().double(), want, atol=2e-5 * float(want.abs().max()), rtol=2e-5)
        # a read alone, and a write alone
        got = ops.streams_mix_norm(a, None, None, None, dev(in_w), norm, out_dtype=torch.float32, **kw)
        want = normed(torch.einsum("s,nsw->nw", in_w.double(), xs.double()))
        assert torch.allclose(got.cpu().double(), want, atol=2e-5 * float(want.abs().max()), rtol=2e-5) and torch.equal(a.cpu(), xs)
        assert ops.streams_mix_norm(a, dev(y), dev(mix), dev(out_w), None, None, read=False) is None
        assert torch.allclose(a.cpu().double(), new, atol=1e-5, rtol=1e-5)
    spread = ops.streams_spread(torch.arange(2.0 * W).reshape(2, W).cuda(), 3).cpu()
    assert spread.shape == (2, 3, W) and all(torch.equal(spread[:, s], torch.arange(2.0 * W).reshape(2, W)) for s in range(3))


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps,pairing,own", [(3, "interleaved", True), (4, "interleaved", False), (2, "half_split", True), (0, "interleaved", True),
                                               (1, "interleaved", True)])
def test_q_k_v_pass_bias_convolution_over_portions_rotation_and_pages(dtype, taps, pairing, own):
    """Two sequences of unequal lengths go through the pass in portions of unequal sizes (down to one token, and portions
    shorter than the convolution reaches back), into slots that another sequence used before; q and the pages' contents
    against the plain convolution and rotation over the whole sequences."""
    from palm_infra_amd.kernels import ops
    torch.manual_seed(5 + taps)
    dt = TORCH[dtype]
    H, G, d, dv, rot = 4, 2, 12, 20, 8
    qs, ks, vs = H * d, (G * d if own else 0), (G * dv if own else 0)
    C = qs + ks + vs
    lengths = [150, 67]
    rows = [torch.randn(n, C + 5).to(dt) for n in lengths]            # (five more columns follow: a gate's)
    bias = torch.randn(C)
    conv = torch.randn(C, taps) if taps else None
    rot_cfg = {"dims": rot, "base": 100.0, "scaling": {"factor": 3.0}}
    n_pages, n_slots = 8, 3
    k_cache = torch.full((n_pages + 1, G, 64, d), float("nan"), dtype=dt, device="cuda")
    v_cache = torch.full((n_pages + 1, G, dv, 64), float("nan"), dtype=dt, device="cuda")
    table = torch.tensor([[7, 7, 7], [5, 1, 3], [0, 6, 7]], dtype=torch.int32, device="cuda")        # slots 1 and 2
    state = torch.randn(n_slots, max(taps - 1, 0), C, device="cuda") if taps > 1 else None      # stale from an earlier sequence
    if state is not None:
        state[1:].zero_()                                               # what opening a slot does
    inv = torch.tensor([100.0 ** (-2.0 * i / rot) / 3.0 for i in range(rot // 2)], dtype=torch.float32, device="cuda")
    cuts = [[1, 2, 1, 60, 3, 64, 19], [2, 1, 64]]                       # portions of the two sequences, step by step
    got_q = [[], []]
    fed = [0, 0]
    for step in range(max(len(c) for c in cuts)):
        live = [b for b in range(2) if step < len(cuts[b])]
        counts = [cuts[b][step] for b in live]
        ctx = _step_context([fed[b] for b in live], counts, slots=[b + 1 for b in live])
        packed = torch.cat([rows[b][fed[b]:fed[b] + c] for b, c in zip(live, counts)]).cuda()
        cos, sin = ops.rope_table(ctx.positions, inv)
        q = ops.sink_qkv_store(packed, H, G, d, dv, bias.cuda(), None, None, None, 1e-6, cos, sin, rot, k_cache if own else None,
                               v_cache if own else None, table, ctx, write_cache=own, pairing=pairing, conv=conv.cuda() if taps else None,
                               conv_state=state)
        o = 0
        for b, c in zip(live, counts):
            got_q[b].append(q[o:o + c].cpu())
            o += c
            fed[b] += c
    tol = dict(atol=1e-4, rtol=1e-4) if dtype == "float32" else dict(atol=3e-2, rtol=2e-2)
    for b, n in enumerate([sum(c) for c in cuts]):
        u = rows[b][:n, :C].double() + bias.double()
        y = P.short_convolution(u, conv.double()) if taps else u
        pos = torch.arange(n)

        def turned(x, heads):
            x = x.reshape(n, heads, d)
            if pairing == "interleaved":
                return P.rotate_neighbours(x, pos, rot_cfg)
            half = rot // 2                                                # pairs (i, i + rot/2) with the same angles
            f = torch.tensor([100.0 ** (-2.0 * i / rot) / 3.0 for i in range(half)], dtype=P.F64)
            c, s = torch.cos(pos[:, None] * f)[:, None, :], torch.sin(pos[:, None] * f)[:, None, :]
            a, bb = x[..., :half], x[..., half:rot]
            return torch.cat([a * c - bb * s, bb * c + a * s, x[..., rot:]], dim=-1)

        assert torch.allclose(torch.cat(got_q[b]).double(), turned(y[:, :qs], H), **tol), (b, "q")
        if own:
            want_k, want_v = turned(y[:, qs:qs + ks], G), y[:, qs + ks:].reshape(n, G, dv)
            pages = table[b + 1].tolist()
            for p in range(n):
                assert torch.allclose(k_cache[pages[p // 64], :, p % 64].cpu().double(), want_k[p], **tol), (b, "k", p)
                assert torch.allclose(v_cache[pages[p // 64], :, :, p % 64].cpu().double(), want_v[p], **tol), (b, "v", p)
        if taps > 1:
            assert torch.allclose(state[b + 1].cpu().double(), u[n - taps + 1:], atol=1e-6), (b, "state")


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,window", [(4, 2, 24, 40, 37), (3, 3, 40, 72, 70), (6, 1, 8, 12, None), (16, 2, 64, 32, 130), (6, 2, 32, 96, 64)])
def test_attention_kernel_far_keys_page_borders_window_edges_sinks_and_head_gates(dtype, H, G, d, dv, window):
    """Keys and values straight into the pages.  One key is made to stand out (its score far above the others') at places
    that matter: the first position, far back, a page's last and first key, just inside and just outside the window; a sink
    is made to outweigh every key for one head; every head has a gate value of its own.  Prompts (the matrix cores in
    bfloat16) and single tokens (the exact kernel, in slices)."""
    from palm_infra_amd.kernels import ops
    torch.manual_seed(H * 100 + d)
    dt = TORCH[dtype]
    T, scale = 300, 0.3
    per = H // G
    pages = [3, 0, 5, 2, 4]
    table = torch.tensor([[6] * 5, pages], dtype=torch.int32, device="cuda")
    sinks = torch.randn(H)
    sinks[H - 1] = 30.0                                                   # this head's sink takes nearly all the weight
    targets = [0, 5, 63, 64, 127, 128, 190, 299 - (window or 200) + 1, 299 - (window or 200), 299]
    for target in sorted(set(t for t in targets if 0 <= t < T)):
        k = torch.randn(T, G, d) * 0.3
        v = torch.randn(T, G, dv)
        q = torch.randn(T, H, d) * 0.3
        gate = torch.randn(T, 3 + H)
        # the last query points at the target key with a score of about 40 over the others
        k[target] = torch.nn.functional.normalize(torch.randn(G, d), dim=-1) * 4.0
        for h in range(H):
            q[T - 1, h] = k[target, h // per] / 16.0 * 40.0 / scale
        q, k, v, gate = (t.to(dt) for t in (q, k, v, gate))
        kc = torch.full((7, G, 64, d), float("nan"), dtype=dt)
        vc = torch.full((7, G, dv, 64), float("nan"), dtype=dt)
        for p in range(T):
            kc[pages[p // 64], :, p % 64] = k[p]
            vc[pages[p // 64], :, :, p % 64] = v[p]
        vc[pages[T // 64], :, :, T % 64:] = 0                              # (beyond the sequence: whatever a page held, made finite here)
        kc[pages[T // 64], :, T % 64:] = 0
        want = P.sink_softmax_heads(q.double(), k.double(), v.double(), scale, window, sinks.double())
        want = want * torch.sigmoid(gate.double()[:, 3:, None])
        tol = dict(atol=2e-4, rtol=2e-4) if dtype == "float32" else dict(atol=3e-2, rtol=3e-2)
        # a prompt of all T tokens, and a second one in two portions
        for cuts in ([T], [170, 130]):
            got, at = [], 0
            for c in cuts:
                ctx = _step_context([at], [c], slots=[1])
                got.append(ops.sink_attention(q[at:at + c].cuda(), kc.cuda(), vc.cuda(), table, ctx, H, G, d, dv, scale, window, sinks.cuda(),
                                              gate[at:at + c].cuda(), 3, gate_per_head=True).cpu())
                at += c
            assert torch.allclose(torch.cat(got).double().reshape(T, H, dv), want, **tol), (target, cuts)
        # the last tokens one by one: the exact kernel in slices
        for p in (T - 1, T - 2):
            ctx = _step_context([p], [1], slots=[1])
            for slices in (None, 1, 3):
                got = ops.sink_attention_exact(q[p:p + 1].cuda(), kc.cuda(), vc.cuda(), table, ctx, H, G, d, dv, scale, window, sinks.cuda(),
                                               gate[p:p + 1].cuda(), 3, slices=slices, gate_per_head=True).cpu()
                assert torch.allclose(got.double().reshape(H, dv), want[p], **tol), (target, p, slices)
        # the target decides the last query's output where it is seen, and counts for nothing where it is not
        seen = window is None or T - 1 - target < window
        near_target = (want[T - 1, 0] - v[target, 0].double() * torch.sigmoid(gate.double()[T - 1, 3])).abs().max() < 0.05
        assert bool(near_target) == seen, target
        assert float(want[T - 1, H - 1].abs().max()) < 1e-3 or seen          # the sink's head: nothing but what the target gives


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d,dv", [(3, 16, 24), (1, 40, 130), (2, 128, 64), (4, 32, 16), (2, 24, 70)])
def test_matrix_memory_keeps_a_far_write_whole_in_portions_and_in_chunks(dtype, H, d, dv):
    """The gates are made so that one far token is written with a weight far above the others' and nearly nothing is
    forgotten after it: the last outputs then hold that token's value, whatever lies between.  Whole, in portions down to
    one token, and cut into chunks that run side by side; two sequences of unequal lengths in slots that were used before."""
    from palm_infra_amd.kernels import ops
    torch.manual_seed(d + dv)
    dt = TORCH[dtype]
    T, cap, eps = 260, 12.0, 1e-6
    lengths = [T, 75]
    far = 3
    tol = dict(atol=5e-4, rtol=5e-4) if dtype == "float32" else dict(atol=3e-2, rtol=3e-2)
    rows = [torch.randn(n, H * (2 * d + 2 * dv)) * 0.5 for n in lengths]
    # every query of the long sequence leans towards the far key: a query orthogonal to what the memory holds would leave a
    # remainder of rounding errors for the unit norm to scale up
    rows[0][:, :H * d] += 0.7 * rows[0][far, H * d:2 * H * d]
    rows = [r.to(dt) for r in rows]
    gates = [torch.randn(n, 2 * H) for n in lengths]
    gates[0][:, H:] = 9.0 + torch.rand(T, H)                               # forget gates near one
    gates[0][:, :H] = -4.0 + torch.randn(T, H) * 0.3                       # small input gates ..
    gates[0][far, :H] = 8.0                                                # .. but for one far token
    gate_bias = torch.randn(2 * H) * 0.2
    norm_w = torch.randn(H * dv) + 1.5
    want = []
    for r, g in zip(rows, gates):
        n = r.shape[0]
        r = r.double()
        q = r[:, :H * d].reshape(n, H, d) * d ** -0.5
        k, v = r[:, H * d:2 * H * d].reshape(n, H, d), r[:, 2 * H * d:2 * H * d + H * dv].reshape(n, H, dv)
        z = g.double() + gate_bias.double()
        li, lf = P.capped(z[:, :H], cap), torch.nn.functional.logsigmoid(P.capped(z[:, H:], cap))
        heads = [P.unit_rows(P.matrix_memory(q[:, a], k[:, a], v[:, a], li[:, a], lf[:, a]), eps) for a in range(H)]
        want.append(torch.cat(heads, dim=1) * norm_w.double() * torch.sigmoid(r[:, 2 * H * d + H * dv:]))
    # the far write is what the last output holds, up to the norm: same direction as v[far]
    r0 = rows[0].double()
    v_far = r0[far, 2 * H * d:2 * H * d + dv]
    last = want[0][T - 1, :dv] / (norm_w[:dv].double() * torch.sigmoid(r0[T - 1, 2 * H * d + H * dv:2 * H * d + H * dv + dv]))
    assert float(torch.nn.functional.cosine_similarity(last, v_far, dim=0)) > 0.99
    schedules = {"whole": ([[T], [75]], 0), "chunks of 32": ([[T], [75]], 32), "chunks of 40": ([[200, 60], [75]], 40),
                 "portions": ([[1, 2, 1, 64, 65, 127], [70, 1, 1, 1, 2]], None)}
    for what, (cuts, chunk) in schedules.items():
        state = torch.randn(3, H, d, dv + 1, device="cuda")                 # stale from an earlier sequence
        m_state = torch.randn(3, H, device="cuda")
        state[1:].zero_()
        m_state[1:].zero_()
        got, fed = [[], []], [0, 0]
        for step in range(max(len(c) for c in cuts)):
            live = [b for b in range(2) if step < len(cuts[b])]
            counts = [cuts[b][step] for b in live]
            ctx = _step_context([fed[b] for b in live], counts, slots=[b + 1 for b in live])
            packed = torch.cat([rows[b][fed[b]:fed[b] + c] for b, c in zip(live, counts)]).cuda()
            g = torch.cat([gates[b][fed[b]:fed[b] + c] for b, c in zip(live, counts)]).cuda()
            out = ops.mlstm(packed, g, gate_bias.cuda(), H, d, dv, cap, d ** -0.5, norm_w.cuda(), eps, state, m_state, ctx, chunk=chunk).cpu()
            o = 0
            for b, c in zip(live, counts):
                got[b].append(out[o:o + c])
                o += c
                fed[b] += c
        for b in range(2):
            assert torch.allclose(torch.cat(got[b]).double(), want[b], **tol), (what, b, float((torch.cat(got[b]).double() - want[b]).abs().max()))


@gpu
def test_scored_routing_in_groups_against_the_plain_choice():
    """Random logits and corrections (also corrections that make every choice score negative) for several shapes of groups;
    the kernel's experts and weights against the plain ones, the gate column of a wider row left alone."""
    from palm_infra_amd.kernels import ops
    torch.manual_seed(3)
    for E, top, groups, keep, shift in ((12, 3, 3, 2, 0.0), (16, 4, 4, 2, -6.0), (8, 2, 2, 1, -3.0), (6, 1, 1, 1, 0.0), (5, 5, 1, 1, 0.0), (64, 6, 8, 3, 0.0), (130, 7, 10, 4, 1.0)):
        n = 200
        logits = torch.randn(n, E + 1) * 1.5
        corr = torch.randn(E) * 0.2 + shift
        r = {"experts": E, "top": top, "scale": 2.5}
        if groups > 1:
            r["groups"] = {"count": groups, "keep": keep}
        # the plain router takes h and a matrix: a one-hot h picks a row of logits
        w = {"r.router": logits[:, :E].double().T.contiguous(), "r.correction": corr.double()}
        chosen_ref, weight_ref = P.route(torch.eye(n, dtype=P.F64), w, "r.", r)
        chosen, weight = ops.moe_route_scored(logits.cuda(), E, top, corr.cuda(), groups, keep, 2.5)
        for t in range(n):
            a = dict(zip(chosen[t].tolist(), weight[t].tolist()))
            b = dict(zip(chosen_ref[t].tolist(), weight_ref[t].tolist()))
            assert sorted(a) == sorted(b), (E, t)
            assert all(abs(a[e] - b[e]) < 1e-5 for e in a), (E, t)


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_plain_gelu_experts_for_few_rows_and_many(dtype):
    """The experts alone, with given choices: a decode step's rows (every pair reads its expert itself), a prompt's rows
    (grouped on the device in bfloat16, by the host in float32), and a shared expert behind its gate."""
    from palm_infra_amd.kernels import ops
    torch.manual_seed(11)
    dt = TORCH[dtype]
    E, top, W, F = 6, 2, 48, 24
    up, down = (torch.randn(E * F, W) * W ** -0.5).to(dt), (torch.randn(E * W, F) * F ** -0.5).to(dt)
    tol = dict(atol=1e-4, rtol=1e-4) if dtype == "float32" else dict(atol=4e-2, rtol=4e-2)
    for n in (1, 9, 128, 200):
        h = torch.randn(n, W).to(dt)
        chosen = torch.stack([torch.randperm(E)[:top] for _ in range(n)]).to(torch.int32)
        weight = torch.rand(n, top)
        want = torch.zeros(n, W, dtype=P.F64)
        for t in range(n):
            for c in range(top):
                e = int(chosen[t, c])
                want[t] += weight[t, c].double() * (P.gelu_erf(h[t].double() @ up[e * F:(e + 1) * F].double().T) @ down[e * W:(e + 1) * W].double().T)
        got = ops.moe_experts(h.cuda(), up.cuda(), down.cuda(), chosen.cuda(), weight.cuda(), F, "gelu") if n <= 128 else None
        if got is not None:
            assert torch.allclose(got.cpu().double(), want, **tol), n
        if dtype == "bfloat16":
            got = ops.moe_grouped(h.cuda(), up.cuda(), down.cuda(), chosen.cuda(), weight.cuda(), F, "gelu")
            assert torch.allclose(got.cpu().double(), want, **tol), n
        logits = torch.randn(n, E + 1)
        y = torch.randn(n, W).to(dt)
        out = torch.randn(n, W)
        got = ops.add_gated_rows(out.clone().cuda(), y.cuda(), logits.cuda(), E).cpu()
        assert torch.allclose(got.double(), out.double() + torch.sigmoid(logits[:, E:].double()) * y.double(), atol=1e-5)
    z = (torch.randn(1000) * 3).to(dt)
    for kind, fn in (("relu_squared", P.relu_squared), ("gelu_erf", P.gelu_erf)):
        assert torch.allclose(ops.activation(z.cuda(), kind).cpu().double(), fn(z.double()), **tol)


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
def test_the_streams_sum_after_every_layer(tmp_path_factory):
    """The sum of the streams after each layer, in float32: a hook on the blocks reads it."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, "A", "float32", graphs=False)
    ids = S.prompts(raw_of("A"), [40], seed=2)[0]
    cfg, w = P.read_model(model_dir(tmp_path_factory, "A", "float32"))
    want = []
    P.forward(cfg, w, ids, want)
    seen = []
    originals = {id(b): b.forward for b in eng.model.layers}
    for b in eng.model.layers:
        def hooked(x, h, ctx, sink, _f=b.forward):
            out = _f(x, h, ctx, sink)
            seen.append(x.detach().sum(1))
            return out
        b.forward = hooked
    try:
        slot = eng.open()
        eng.step([StepEntry(slot, ids, list(range(len(ids))))])
        eng.close(slot)
    finally:
        for b in eng.model.layers:
            b.forward = originals[id(b)]
    assert len(seen) == len(want) == 4
    # (the last layer's write is made only for the rows that the final norm reads and is not kept: the logits of the other
    # tests cover it)
    for i, (a, b) in enumerate(zip(seen[:-1], want[:-1])):
        assert torch.allclose(a.cpu().double(), b, atol=2e-4, rtol=1e-4), (i, float((a.cpu().double() - b).abs().max()))


@gpu
def test_a_checkpoint_with_the_second_sublayers_tensors_of_a_layer_without_a_feed_forward(tmp_path):
    from palm_infra_amd.engine import Engine, StepEntry
    from palm_infra_amd.weights import write_safetensors
    raw = raw_of("A")
    tensors = S.tensors_of(raw, 7, "float32")
    tensors.update({"l2.norm2": torch.full((64,), 3.0), "l2.norm2.b": torch.ones(64), "l2.norm2.alpha": torch.tensor(2.0),
                    "l2.hc2.in": torch.ones(3), "l2.hc2.out": torch.ones(3), "l2.hc2.mix": torch.ones(3, 3)})
    (tmp_path / "config.json").write_text(json.dumps(raw))
    write_safetensors(tmp_path / "model.safetensors", tensors)
    eng = Engine.from_dir(tmp_path, dtype="float32", max_tokens=256)
    ids = S.prompts(raw, [40], seed=12)[0]
    slot = eng.open()
    got = eng.step([StepEntry(slot, ids, list(range(len(ids))))])
    eng.close(slot)
    cfg, w = P.read_model(tmp_path)
    assert_close(got, P.forward(cfg, w, ids), "float32", "spare tensors")


@gpu
@pytest.mark.parametrize("name,dtype", CASES)
def test_prompt_then_every_token_alone_from_the_first(tmp_path_factory, name, dtype):
    """Token-by-token decoding from the very first token (every state starts from zero, the convolution from zeros, the window
    from an empty page), through recorded steps, across page borders and past the windows; against the whole prompt in one step."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, name, dtype)
    ids = S.prompts(raw_of(name), [150], seed=4)[0]
    ref = reference(tmp_path_factory, name, dtype, ids)
    slot = eng.open()
    got = []
    for t, tok in enumerate(ids):
        got.append(eng.step([StepEntry(slot, [tok], [0])]))
        assert eng.length(slot) == t + 1
    eng.close(slot)
    assert_close(torch.cat(got), ref, dtype, f"{name} one by one")


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
@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("B", "float32"), ("C", "bfloat16"), ("D", "float32")])
def test_long_decoding(tmp_path_factory, name, dtype):
    """A short prompt, then some hundred tokens one by one over several pages and several windows, two sequences side by
    side that started at different lengths; a windowed layer gives pages back on the way."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, name, dtype)
    a, b = S.prompts(raw_of(name), [330, 270], seed=8)
    refs = [reference(tmp_path_factory, name, dtype, a), reference(tmp_path_factory, name, dtype, b)]
    sa, sb = eng.open(), eng.open()
    got = [eng.step([StepEntry(sa, a[:70], [69]), StepEntry(sb, b[:10], [9])])]
    want = [torch.stack([refs[0][69], refs[1][9]])]
    for i in range(260):
        got.append(eng.step([StepEntry(sa, [a[70 + i]], [0]), StepEntry(sb, [b[10 + i]], [0])]))
        want.append(torch.stack([refs[0][70 + i], refs[1][10 + i]]))
    windowed = [g for g in eng.cache.paged_groups if g.table.window]
    assert all(g.table.pages.held_count <= 2 * (g.table.window // 64 + 2) for g in windowed)      # two sequences' windows, not their lengths
    eng.close(sa)
    eng.close(sb)
    assert_close(torch.cat(got), torch.cat(want), dtype, f"{name} long decoding")


@gpu
@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("C", "bfloat16")])
def test_a_prompt_longer_than_a_step_takes_at_once(tmp_path_factory, name, dtype):
    """A windowed model cuts a long prompt into pieces between which pages go back; the memory's long runs go through in
    chunks; a far token is asked for at the end."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, name, dtype)
    assert eng.step_tokens_per_seq == 1024
    ids = S.prompts(raw_of(name), [1300], seed=13)[0]
    want = [0, 1, 511, 1023, 1024, 1025, 1200, 1299]
    slot = eng.open()
    got = eng.step([StepEntry(slot, ids, want)])
    more = eng.step([StepEntry(slot, [ids[5]], [0])])                       # and a single token after it
    eng.close(slot)
    ref = reference(tmp_path_factory, name, dtype, ids + [ids[5]])
    assert_close(torch.cat([got, more]), ref[want + [1300]], dtype, f"{name} long prompt")


@gpu
@pytest.mark.parametrize("name", ["A", "D"])
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
    d = model_dir(tmp_path_factory, "D", "float32")
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
        if s % 2 and live:
            got = np.fromfile(out / f"{s}.f32", dtype="<f4").reshape(len(live), -1)
            assert_close(torch.from_numpy(got.copy()), torch.stack([refs[i][fed[i]] for i in live]), "float32", f"trace step {s}")
        else:
            assert not (out / f"{s}.f32").exists()
        for i in live:
            fed[i] += 1
