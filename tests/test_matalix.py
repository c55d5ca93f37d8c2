"""The Matalix design in the engine against the plain implementation (tests/plain_matalix.py).

Without a GPU: the configuration, its description as parts, the run order of a range of layers that runs again, and the
oracle's own mechanisms against closed forms.  On the GPU: every mechanism alone (one-layer models, and the kernels called
directly with inputs made so that one far key, one key at a window's or a page's edge, or the sink decides the result),
whole prompts, prompts cut into portions down to two tokens, prefill against token-by-token decoding from the first token,
batches of unequal requests against each alone, slots and pages that are used again, long decoding over several pages and
past the windows, recorded against launched steps, and greedy generation through ``generate``, the command line and the
trace replay.  In float32 and in bfloat16.
"""
import json
import math

import pytest
import torch

import matalix_tiny as S
import plain_matalix as P
from palm_infra_amd.config import ConfigError, config_from_dict

gpu = pytest.mark.gpu
DTYPES = ("float32", "bfloat16")
LENGTHS = {"A": [1, 2, 63, 64, 65, 130, 200, 17], "B": [129, 3, 70, 71, 1, 191], "C": [5, 66, 128, 31], "D": [300, 9, 140]}


# ---- without a GPU ---------------------------------------------------------------------------------------

def test_registry_picks_the_design_by_its_config_key():
    cfg = config_from_dict(S.CONFIGS["A"])
    assert type(cfg).__name__ == "MatalixConfig"
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    assert config_from_dict(json.loads(json.dumps(cfg.to_dict()))).loop == (0, 2, 3)


def test_spec_names_every_tensor():
    spec = config_from_dict(S.CONFIGS["A"]).spec()
    names = spec.expected_tensors()
    assert names["embed"][0] == (211, 64) and names["final.norm"][0] == (64,)
    assert names["l0.mix.left.q"][0] == (4 * 24, 64) and names["l0.mix.left.k"][0] == (2 * 24, 64) and names["l0.mix.left.v"][0] == (2 * 40, 64)
    assert names["l0.mix.left.q.b"][0] == (96,) and names["l0.mix.left.k.norm"][0] == (48,) and names["l0.mix.left.g"][0] == (160, 64)
    assert names["l0.mix.left.o"][0] == (64, 160) and names["l0.mix.right.q"][0] == (48, 64) and names["l0.mix.right.v"][0] == (72, 64)
    assert names["l0.mix.right.norm"][0] == (72,) and names["l0.mix.right.o"][0] == (64, 72)
    assert names["l0.mlp.gate"][0] == (40, 64) and names["l0.mlp.down"][0] == (64, 40) and names["l0.ls2"][0] == (64,)
    assert "l1.mlp.up" not in names and "l1.norm2" not in names and "l1.ls2" not in names and "l1.ls1" in names
    assert "head" not in names                                             # the head is the table itself


def test_norm_and_scale_of_a_feed_forward_that_is_not_there_are_bound_if_the_file_has_them():
    cfg = config_from_dict(S.CONFIGS["A"])
    names = list(cfg.spec().expected_tensors())
    with_spares = cfg.spec(names + ["l1.norm2", "l1.ls2"]).expected_tensors()
    assert with_spares["l1.norm2"][0] == (64,) and len(with_spares) == len(names) + 2
    assert set(cfg.spec(names).expected_tensors()) == set(names)


def test_run_order_of_layers_that_run_again():
    order = lambda name: [(c.layer, c.adds_embedding) for c in config_from_dict(S.CONFIGS[name]).spec().order]
    assert order("A") == [(0, False), (1, False), (0, True), (1, False), (0, True), (1, False), (2, False)]
    assert order("B") == [(0, False), (1, False)]
    assert order("C") == [(0, False), (1, False), (1, True)]
    assert order("D") == [(0, False), (1, False), (0, True), (1, False)]
    for name in S.CONFIGS:
        assert order(name) == P.run_order(S.CONFIGS[name])
        assert all(c.cache_of is None for c in config_from_dict(S.CONFIGS[name]).spec().order)      # every run has a cache of its own


def test_cache_needs_of_both_sides():
    from palm_infra_amd.cache import KVNeed, StateNeed
    from palm_infra_amd.parts import cache_needs
    spec = config_from_dict(S.CONFIGS["A"]).spec()
    assert cache_needs(spec.layers[0]) == [KVNeed(2, 24, 37, value_dim=40), StateNeed("retention", (3, 16, 24))]
    assert cache_needs(spec.layers[2]) == [KVNeed(1, 16, 5, value_dim=16), StateNeed("retention", (1, 8, 8))]
    assert cache_needs(config_from_dict(S.CONFIGS["C"]).spec().layers[0])[0] == KVNeed(1, 8, None, value_dim=12)


@pytest.mark.parametrize("change,what", [
    (lambda c: c["layers"][0].update(type="retention"), "type"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), "kv heads"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=26), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][0]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind"),
    (lambda c: c["layers"][0]["mlp"].pop("limit"), "limit"),
    (lambda c: c["loop"].update(stop=4), "loop"),
    (lambda c: c["loop"].update(times=0), "loop"),
    (lambda c: c["norm"].pop("eps"), "eps"),
])
def test_bad_configurations_are_refused(change, what):
    raw = json.loads(json.dumps(S.CONFIGS["A"]))
    change(raw)
    with pytest.raises(ConfigError, match=what):
        config_from_dict(raw)


def test_random_model_folder_is_read_by_the_plain_implementation(tmp_path):
    from palm_infra_amd.weights import write_random_model
    write_random_model(S.CONFIGS["C"], 3, tmp_path, "bfloat16")
    cfg, w = P.read_model(tmp_path)
    layers = []
    logits = P.forward(cfg, w, [1, 2, 3, 4, 5], layers)
    assert logits.shape == (5, 97) and torch.isfinite(logits).all() and len(layers) == 3


def test_plain_sink_takes_weight_and_gives_nothing():
    """One key of score s: its weight is e^s / (1 + e^s); without the sink it is 1.  Scores far below zero: the output
    vanishes.  A sink of another score shifts the one in the denominator."""
    q = torch.tensor([[[2.0, 0.0]]], dtype=P.F64)
    k = torch.tensor([[[1.5, 0.0]]], dtype=P.F64)
    v = torch.tensor([[[3.0, -1.0, 2.0]]], dtype=P.F64)
    pos = torch.arange(1)
    s = 0.5 * 3.0
    assert torch.allclose(P.sink_softmax_heads(q, k, v, pos, 0.5, None)[0, 0], v[0, 0] * math.exp(s) / (1 + math.exp(s)))
    assert torch.allclose(P.sink_softmax_heads(q, k, v, pos, 0.5, None, sink=None)[0, 0], v[0, 0])
    assert torch.allclose(P.sink_softmax_heads(q, k, v, pos, 0.5, None, sink=2.0)[0, 0], v[0, 0] * math.exp(s) / (math.exp(2.0) + math.exp(s)))
    assert float(P.sink_softmax_heads(q, -20 * k, v, pos, 0.5, None).abs().max()) < 1e-10


def test_plain_window_sees_itself_and_the_tokens_before_it():
    """Zero queries: every seen key has weight 1 / (1 + seen); values are one-hot in the position, so the output says which
    positions were seen."""
    T, size = 9, 4
    q = torch.zeros(T, 2, 3, dtype=P.F64)
    k = torch.randn(T, 1, 3, dtype=P.F64)
    v = torch.eye(T, dtype=P.F64).reshape(T, 1, T)
    out = P.sink_softmax_heads(q, k, v, torch.arange(T), 1.0, size)
    for i in range(T):
        seen = [j for j in range(T) if 0 <= i - j < size]
        want = torch.zeros(T, dtype=P.F64)
        want[seen] = 1.0 / (1 + len(seen))
        assert torch.allclose(out[i, 0], want) and torch.allclose(out[i, 1], want)
    full = P.sink_softmax_heads(q, k, v, torch.arange(T), 1.0, None)
    assert torch.allclose(full[T - 1, 0], torch.full((T,), 1.0 / (1 + T), dtype=P.F64))


def test_plain_rotation_frequencies():
    f, mag = P.rotation_frequencies({"dims": 8, "base": 100.0, "scaling": None})
    assert mag == 1.0 and torch.allclose(f, torch.tensor([1.0, 100 ** -0.25, 100 ** -0.5, 100 ** -0.75], dtype=P.F64))
    sc = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    f2, mag2 = P.rotation_frequencies({"dims": 16, "base": 10000.0, "scaling": sc})
    plain, _ = P.rotation_frequencies({"dims": 16, "base": 10000.0, "scaling": None})
    assert abs(mag2 - (0.1 * math.log(4.0) + 1.0)) < 1e-12
    assert torch.allclose(f2[0], plain[0]) and torch.allclose(f2[-1], plain[-1] / 4.0)          # fast pairs stay, slow ones stretch
    assert all(plain[i] / 4.0 - 1e-15 <= f2[i] <= plain[i] + 1e-15 for i in range(8))
    # a part of the head turns, the rest stays; a turn keeps a pair's length (times the factor on cos and sin)
    x = torch.randn(5, 2, 12, dtype=P.F64)
    y = P.rotate(x, torch.arange(5), {"dims": 8, "base": 100.0, "scaling": None})
    assert torch.equal(y[..., 8:], x[..., 8:]) and torch.equal(y[0], x[0])
    assert torch.allclose(y[..., :4] ** 2 + y[..., 4:8] ** 2, x[..., :4] ** 2 + x[..., 4:8] ** 2)


def test_plain_recurrence_is_a_decayed_sum():
    torch.manual_seed(0)
    T, H, d, dv = 7, 2, 3, 4
    q, k, v = (torch.randn(T, H, n, dtype=P.F64) for n in (d, d, dv))
    decay = [0.5, 0.9]
    o, S = P.decay_recurrence(q, k, v, decay)
    for h in range(H):
        want = sum(decay[h] ** (T - 1 - j) * float(q[T - 1, h] @ k[j, h]) * v[j, h] for j in range(T))
        assert torch.allclose(o[T - 1, h], want)
    o1, S1 = P.decay_recurrence(q[:4], k[:4], v[:4], decay)
    o2, S2 = P.decay_recurrence(q[4:], k[4:], v[4:], decay, S1)
    assert torch.allclose(torch.cat([o1, o2]), o) and torch.allclose(S2, S)


# ---- on the GPU ------------------------------------------------------------------------------------------

_dirs, _engines, _refs = {}, {}, {}


def raw_of(name: str) -> dict:
    return S.CONFIGS.get(name) or S.SINGLE[name]


def model_dir(tmp_path_factory, name: str, store: str):
    key = (name, store)
    if key not in _dirs:
        _dirs[key] = S.write_model(raw_of(name), S.SEEDS.get(name, 61), tmp_path_factory.mktemp(f"matalix_{name}_{store}"), store)
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
    tenth of the logits' scale, all rows together within a twentieth, an element within half of it."""
    got = torch.as_tensor(got).double().cpu().reshape(ref.shape)
    assert torch.isfinite(got).all(), f"{what}: logits are not finite"
    err = (got - ref.double()).abs().reshape(-1, ref.shape[-1])
    scale = float(ref.double().pow(2).mean().sqrt())
    if dtype == "float32":
        worst = float(err.max())
        assert worst <= 1e-4 * max(1.0, scale), f"{what}: float32 logits differ by {worst:.3e} (their scale is {scale:.3e})"
        return
    rows = err.pow(2).mean(-1).sqrt()
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
def test_scaled_add_of_one_and_two_terms_and_the_next_norm(W):
    from palm_infra_amd.kernels import ops
    torch.manual_seed(W)
    n = 9
    x = torch.randn(n, W)
    a, b = torch.randn(n, W), torch.randn(n, W)
    ls, w = torch.randn(W), torch.randn(W)
    eps = 1e-5
    for dt in (torch.float32, torch.bfloat16):
        a_, b_ = a.to(dt), b.to(dt)
        want_x = x.double() + ls.double() * (0.7 * a_.double() + 1.3 * b_.double())
        want_h = want_x / torch.sqrt((want_x ** 2).mean(-1, keepdim=True) + eps) * w.double()
        xd = x.cuda().clone()
        h = ops.add_scaled_normed(xd, [a_.cuda(), b_.cuda()], [0.7, 1.3], ls.cuda(), w.cuda(), eps, torch.float32)
        assert torch.allclose(xd.cpu().double(), want_x, atol=1e-5) and torch.allclose(h.cpu().double(), want_h, atol=1e-4)
        # a selection of rows leaves the stream as it is
        xd = x.cuda().clone()
        rows = torch.tensor([7, 0, 3], dtype=torch.int32).cuda()
        h = ops.add_scaled_normed(xd, [a_.cuda(), b_.cuda()], [0.7, 1.3], ls.cuda(), w.cuda(), eps, torch.float32, rows=rows)
        assert torch.equal(xd.cpu(), x) and torch.allclose(h.cpu().double(), want_h[[7, 0, 3]], atol=1e-4)
        # one term, no norm, no vector
        xd = x.cuda().clone()
        assert ops.add_scaled_normed(xd, [a_.cuda()], [1.0], None, None, 0.0) is None
        assert torch.allclose(xd.cpu().double(), x.double() + a_.double(), atol=1e-5)
        empty = ops.add_scaled_normed(xd, [a_.cuda()], [1.0], ls.cuda(), w.cuda(), eps, torch.float32, rows=torch.empty(0, dtype=torch.int32).cuda())
        assert empty.shape == (0, W)
    # a sum that a part hands back unmade, made by whoever cannot take its terms: three terms, two a pass
    from palm_infra_amd.parts import WeightedSum, as_tensor
    c = torch.randn(n, W)
    total = as_tensor(WeightedSum([a.cuda(), b.cuda(), c.cuda()], [0.5, -1.0, 2.0]))
    assert total.dtype == torch.float32 and torch.allclose(total.cpu().double(), 0.5 * a.double() - b.double() + 2.0 * c.double(), atol=1e-5)


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_capped_gate_at_and_beyond_its_limits(dtype):
    from palm_infra_amd.kernels import ops
    ff, limit = 37, 0.75
    torch.manual_seed(1)
    gu = (torch.randn(11, 2 * ff) * 1.5).to(TORCH[dtype])
    gu[0, :4] = torch.tensor([limit, limit + 1, -limit - 1, -9.0]).to(TORCH[dtype])             # the gate is capped from above only
    gu[0, ff:ff + 4] = torch.tensor([limit + 2, -limit - 2, limit, -limit]).to(TORCH[dtype])    # the up row on both sides
    g = torch.clamp(gu[:, :ff].double(), max=limit)
    u = torch.clamp(gu[:, ff:].double(), -limit, limit)
    want = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    got = ops.capped_gate(gu.cuda(), limit, 1.702, 1.0).cpu().double()
    assert torch.allclose(got, want, atol=1e-6 if dtype == "float32" else 0.02, rtol=1e-5 if dtype == "float32" else 0.01)


def _paged(n_slots, pages_per_slot, G, d, dv, dtype, seed=0):
    """Empty key and value pages and a page table that hands the pages out in a scrambled order."""
    g = torch.Generator().manual_seed(seed)
    n_pages = n_slots * pages_per_slot
    perm = torch.randperm(n_pages, generator=g).to(torch.int32).reshape(n_slots, pages_per_slot)
    table = torch.cat([perm, torch.full((1, pages_per_slot), n_pages, dtype=torch.int32)]).cuda()
    k = torch.zeros((n_pages + 1, G, 64, d), dtype=dtype, device="cuda")
    v = torch.zeros((n_pages + 1, G, dv, 64), dtype=dtype, device="cuda")
    return k, v, table


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("norm", [None, "projection", "head"])
def test_q_k_v_pass_bias_norms_part_rotation_and_pages(dtype, norm):
    """The pass that prepares q, k and v, alone: what it returns and what it leaves in the pages against the plain steps, for
    two sequences of which one starts in the middle of a page."""
    from palm_infra_amd.kernels import ops
    H, G, d, dv, rot = 4, 2, 24, 40, 16
    eps = 1e-5
    torch.manual_seed(3)
    starts, counts = [50, 0], [30, 70]
    n = sum(counts)
    rows = torch.randn(n, H * d + G * d + G * dv + 5).to(TORCH[dtype])
    bias = torch.randn(H * d + G * d + G * dv)
    sizes = (H * d, G * d) if norm == "projection" else (d, d)
    q_w, k_w = torch.rand(sizes[0]) + 0.5, torch.rand(sizes[1]) + 0.5
    rotd = {"dims": rot, "base": 100.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}}
    f, mag = P.rotation_frequencies(rotd)
    positions = torch.cat([torch.arange(s, s + c) for s, c in zip(starts, counts)])
    ang = positions.double()[:, None] * f[None, :]
    cos, sin = (torch.cos(ang) * mag).float().cuda(), (torch.sin(ang) * mag).float().cuda()
    ctx = _step_context(starts, counts)
    kc, vc, table = _paged(2, 3, G, d, dv, TORCH[dtype])
    q = ops.sink_qkv_store(rows.cuda(), H, G, d, dv, bias.cuda(), norm, q_w.cuda() if norm else None, k_w.cuda() if norm else None, eps,
                           cos, sin, rot, kc, vc, table, ctx)
    r = rows.double()
    qq, kk, vv = (r[:, :H * d] + bias[:H * d].double(), r[:, H * d:H * d + G * d] + bias[H * d:H * d + G * d].double(),
                  r[:, H * d + G * d:H * d + G * d + G * dv] + bias[H * d + G * d:].double())
    if norm == "projection":
        qq, kk = P.unit_rows(qq, eps) * q_w.double(), P.unit_rows(kk, eps) * k_w.double()
    qq, kk = qq.reshape(n, H, d), kk.reshape(n, G, d)
    if norm == "head":
        qq, kk = P.unit_rows(qq, eps) * q_w.double(), P.unit_rows(kk, eps) * k_w.double()
    qq, kk = P.rotate(qq, positions, rotd), P.rotate(kk, positions, rotd)
    tol = dict(atol=2e-5, rtol=1e-5) if dtype == "float32" else dict(atol=0.03, rtol=0.02)
    assert torch.allclose(q.cpu().double(), qq, **tol)
    o = 0
    for b, (s, c) in enumerate(zip(starts, counts)):
        for i in range(c):
            p = s + i
            page = int(table[b, p // 64])
            assert torch.allclose(kc[page, :, p % 64].cpu().double(), kk[o + i], **tol), (b, i)
            assert torch.allclose(vc[page, :, :, p % 64].cpu().double(), vv[o + i].reshape(G, dv), **tol), (b, i)
        o += c
    assert float(kc[-1].abs().max()) == 0.0 and float(vc[-1].abs().max()) == 0.0        # the page that pads is not written


def _attend(dtype, H, G, d, dv, window, sink, q, k, v, gate, prompt_cut, slices, exact=True):
    """q, k, v of one sequence through the kernels: the first ``prompt_cut`` tokens in one step (or, a list: in steps of these
    sizes), the others one a step (with ``slices`` slices of their key range); returns [T, H * dv].  ``exact`` False: the
    kernel that the parts would get (the matrix cores for portions in bfloat16)."""
    from palm_infra_amd.kernels import ops
    T = q.shape[0]
    kc, vc, table = _paged(1, -(-T // 64) + 1, G, d, dv, TORCH[dtype], seed=T)
    outs = []
    at = 0
    cuts = list(prompt_cut) if isinstance(prompt_cut, (list, tuple)) else [prompt_cut]
    for count in cuts + [1] * (T - sum(cuts)):
        if count == 0:
            continue
        ctx = _step_context([at], [count])
        rows = torch.cat([q[at:at + count].reshape(count, -1), k[at:at + count].reshape(count, -1), v[at:at + count].reshape(count, -1),
                          gate[at:at + count]], dim=1).to(TORCH[dtype]).cuda()
        qq = ops.sink_qkv_store(rows, H, G, d, dv, None, None, None, None, 0.0, None, None, 0, kc, vc, table, ctx)
        if exact:
            outs.append(ops.sink_attention_exact(qq, kc, vc, table, ctx, H, G, d, dv, 0.3, window, sink, rows, H * d + G * d + G * dv,
                                                 slices=1 if count > 1 else slices))
        else:
            outs.append(ops.sink_attention(qq, kc, vc, table, ctx, H, G, d, dv, 0.3, window, sink, rows, H * d + G * d + G * dv))
        at += count
    return torch.cat(outs).cpu().double()


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,window", [(4, 2, 24, 40, 37), (3, 3, 40, 72, 70), (6, 1, 8, 12, None), (16, 2, 64, 32, 130),
                                             (2, 2, 130, 200, 64), (10, 1, 32, 96, 129), (1, 1, 256, 256, 65)])
def test_attention_kernel_far_keys_page_borders_window_edges_and_the_sink(dtype, H, G, d, dv, window):
    """Queries and keys made so that single keys decide: the last queries point at one key each, one just inside its window
    (or far back, without a window), one just outside it (which must not count: the query then sees little but the sink and
    its output nearly vanishes), one at a page's first place and one at a page's last.  Whole, and with the last tokens one
    a step in one slice and in three."""
    torch.manual_seed(H * 1000 + d)
    T = 200
    q = torch.randn(T, H, d) * 0.3
    k = torch.randn(T, G, d) * 0.3
    v = torch.randn(T, G, dv)
    gate = torch.randn(T, H * dv)
    reach = window if window else T
    targets = {T - 1: T - 1 - (reach - 1), T - 2: T - 2 - reach if window else 0, T - 3: 128, T - 4: 127, T - 5: T - 5}
    for qi, kj in sorted(targets.items()):
        kj = max(kj, 0)
        direction = torch.randn(d)
        direction = direction / direction.norm()
        q[qi] = direction * 6.0
        k[kj] = direction * 6.0 + torch.randn(G, d) * 0.05            # score 0.3 * 36: it outweighs all others and the sink
    if window:                                                        # what query T - 2 does see lies far below the sink
        direction = q[T - 2, 0] / 6.0
        k[T - 2 - reach + 1:T - 1] -= (k[T - 2 - reach + 1:T - 1] @ direction)[..., None] * direction + direction * 4.0
    if dtype == "bfloat16":
        q, k, v, gate = (t.bfloat16().float() for t in (q, k, v, gate))
    pos = torch.arange(T)
    want = P.sink_softmax_heads(q.double(), k.double(), v.double(), pos, 0.3, window).reshape(T, H * dv) * torch.sigmoid(gate.double())
    plain = P.sink_softmax_heads(q.double(), k.double(), v.double(), pos, 0.3, window, sink=None).reshape(T, H * dv) * torch.sigmoid(gate.double())
    assert float((want - plain).abs().max()) > 0.05                       # the sink shows in these inputs
    if window:
        wider = P.sink_softmax_heads(q.double(), k.double(), v.double(), pos, 0.3, window + 1).reshape(T, H * dv) * torch.sigmoid(gate.double())
        assert float((want - wider)[T - 2].abs().max()) > 0.05            # and so does a window that is one token off
        assert float(want[T - 2].abs().max()) < 0.05
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == "float32" else dict(atol=0.02, rtol=0.02)
    for cut, slices in ((T, 1), (T - 20, 1), (T - 20, 3), (1, 2)):
        got = _attend(dtype, H, G, d, dv, window, 0.0, q, k, v, gate, cut, slices)
        assert torch.allclose(got, want, **tol), (cut, slices, float((got - want).abs().max()), int((got - want).abs().max(-1).values.argmax()))
    no_sink = _attend(dtype, H, G, d, dv, window, None, q, k, v, gate, T - 3, 2)
    assert torch.allclose(no_sink, plain, **tol)
    if dtype == "bfloat16":
        # the kernels that the parts get: the matrix cores for the portions (the weights are rounded to bfloat16 there)
        from palm_infra_amd.kernels import ops
        assert ops.sink_mfma_serves(torch.empty(0, dtype=torch.bfloat16), d, dv) == (d % 8 == 0 and dv % 4 == 0)
        for cuts in (T, [T - 2], [50, 33, 17, 98], [2, 3, 64, 65, 7], [129, 70]):
            got = _attend(dtype, H, G, d, dv, window, 0.0, q, k, v, gate, cuts, 1, exact=False)
            assert torch.allclose(got, want, atol=0.03, rtol=0.03), (cuts, float((got - want).abs().max()), int((got - want).abs().max(-1).values.argmax()))
        no_sink = _attend(dtype, H, G, d, dv, window, None, q, k, v, gate, [T - 30, 20], 1, exact=False)
        assert torch.allclose(no_sink, plain, atol=0.03, rtol=0.03)


@gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d,dv", [(3, 16, 24), (1, 40, 72), (2, 8, 130), (2, 128, 64), (4, 32, 16)])
def test_recurrence_options_keep_a_far_write_whole_in_portions_and_in_chunks(dtype, H, d, dv):
    """silu'd inputs, the joined heads normed together with a weight, a sigmoid gate: the kernel against the plain steps.  The
    first token writes a large value under a key that only the last token asks for, through a head that hardly decays; a
    prompt long enough to be cut into chunks that run side by side, the same tokens in portions, and one by one."""
    from palm_infra_amd.kernels import ops
    torch.manual_seed(d * 10 + dv)
    T = 300
    decay = [0.999] + [0.5 + 0.4 * i / max(H - 1, 1) for i in range(H - 1)]
    eps = 1e-5
    rows = torch.randn(T, H * (2 * d + 2 * dv)) * 0.7
    rows[0, H * d:H * d + d] = 4.0                      # head 0's first key
    rows[T - 1, :d] = 4.0                               # head 0's last query
    rows[0, 2 * H * d:2 * H * d + dv] = 5.0             # the value written first
    rows = rows.to(TORCH[dtype])
    w = torch.rand(H * dv) + 0.5
    r = rows.double()
    silu = torch.nn.functional.silu
    q, k = silu(r[:, :H * d]).reshape(T, H, d), silu(r[:, H * d:2 * H * d]).reshape(T, H, d)
    v = silu(r[:, 2 * H * d:2 * H * d + H * dv]).reshape(T, H, dv)
    o, S = P.decay_recurrence(q, k, v, decay)
    want = P.unit_rows(o.reshape(T, H * dv), eps) * w.double() * torch.sigmoid(r[:, 2 * H * d + H * dv:])
    far = P.decay_recurrence(q[1:], k[1:], v[1:], decay)[0]
    assert float((far[-1, 0] - o[-1, 0]).abs().max()) > 1.0          # the first token's write reaches the last token
    dec = torch.tensor(decay, dtype=torch.float32).cuda()
    tol = dict(atol=3e-4, rtol=3e-4) if dtype == "float32" else dict(atol=0.03, rtol=0.03)
    for portions, chunk in (([T], 0), ([T], 40), ([T], None), ([2, 3, 64, 65, 7, T - 141], None), ([40] + [1] * (T - 40), None)):
        state = torch.zeros((3, H, d, dv), dtype=torch.float32, device="cuda")
        state[0] = 7.0                                               # a neighbour's state: not read, not written
        got, at = [], 0
        for count in portions:
            ctx = _step_context([at], [count], slots=[1])
            got.append(ops.retention(rows[at:at + count].cuda(), H, d, dv, dec, 1.0, eps, state, ctx, chunk=chunk, input_silu=True,
                                     joined_norm=w.cuda(), gate_sigmoid=True))
            at += count
        got = torch.cat(got).cpu().double()
        assert torch.allclose(got, want, **tol), (portions[:3], chunk, float((got - want).abs().max()))
        assert torch.allclose(state[1].cpu().double(), S, atol=1e-3, rtol=1e-3) and float((state[0] - 7.0).abs().max()) == 0.0
    # the options off: the per-head unit norm and the silu gate as before
    ctx = _step_context([0], [T], slots=[1])
    state = torch.zeros((3, H, d, dv), dtype=torch.float32, device="cuda")
    got = ops.retention(rows.cuda(), H, d, dv, dec, 1.0, eps, state, ctx).cpu().double()
    o2, _ = P.decay_recurrence(r[:, :H * d].reshape(T, H, d), r[:, H * d:2 * H * d].reshape(T, H, d),
                               r[:, 2 * H * d:2 * H * d + H * dv].reshape(T, H, dv), decay)
    want2 = P.unit_rows(o2, eps).reshape(T, H * dv) * silu(r[:, 2 * H * d + H * dv:])
    assert torch.allclose(got, want2, **tol)


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
def test_the_stream_after_every_layer_run(tmp_path_factory):
    """The residual stream after each entry of the run order, in float32: a hook on the blocks reads it."""
    from palm_infra_amd.engine import StepEntry
    eng = engine_for(tmp_path_factory, "A", "float32", graphs=False)
    ids = S.prompts(raw_of("A"), [40], seed=2)[0]
    cfg, w = P.read_model(model_dir(tmp_path_factory, "A", "float32"))
    want = []
    P.forward(cfg, w, ids, want)
    seen = []
    blocks = {id(b): b for b in eng.model.layers}
    originals = {}
    for b in blocks.values():
        originals[id(b)] = b.forward

        def hooked(x, h, ctx, sink, _f=b.forward):
            out = _f(x, h, ctx, sink)
            seen.append(x.detach().clone())
            return out
        b.forward = hooked
    try:
        slot = eng.open()
        eng.step([StepEntry(slot, ids, list(range(len(ids))))])
        eng.close(slot)
    finally:
        for b in blocks.values():
            b.forward = originals[id(b)]
    assert len(seen) == len(want) == 7
    # (the last run's second sum is made only for the rows that the final norm reads and is not written back: the logits
    # of the other tests cover it)
    for i, (a, b) in enumerate(zip(seen[:-1], want[:-1])):
        assert torch.allclose(a.cpu().double(), b, atol=2e-4, rtol=1e-4), (i, float((a.cpu().double() - b).abs().max()))


@gpu
def test_a_checkpoint_with_a_norm_and_a_scale_for_a_feed_forward_that_is_not_there(tmp_path):
    from palm_infra_amd.engine import Engine, StepEntry
    from palm_infra_amd.weights import write_safetensors
    raw = raw_of("A")
    tensors = S.tensors_of(raw, 7, "float32")
    tensors["l1.norm2"] = torch.full((64,), 3.0)
    tensors["l1.ls2"] = torch.full((64,), -2.0)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    write_safetensors(tmp_path / "model.safetensors", tensors)
    eng = Engine.from_dir(tmp_path, dtype="float32", max_tokens=256)
    ids = S.prompts(raw, [40], seed=12)[0]
    slot = eng.open()
    got = eng.step([StepEntry(slot, ids, list(range(len(ids))))])
    eng.close(slot)
    cfg, w = P.read_model(tmp_path)
    assert_close(got, P.forward(cfg, w, ids), "float32", "spare norm and scale")


@gpu
@pytest.mark.parametrize("name,dtype", CASES)
def test_prompt_then_every_token_alone_from_the_first(tmp_path_factory, name, dtype):
    """Token-by-token decoding from the very first token (every state starts from zero, the window from an empty page),
    through recorded steps, across page borders and past the windows; against the whole prompt in one step."""
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
@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("B", "float32"), ("C", "float32"), ("D", "bfloat16")])
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
@pytest.mark.parametrize("name", ["A", "C"])
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
