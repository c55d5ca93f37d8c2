"""A plain, slow Matalix in float64 on the CPU, written from the design's equations: one function per mechanism, whole
sequences only, no cache, no batching.  It shares no code with the library; the tests compare the library with it.

A model is a raw config.json dict and a dict of tensors by checkpoint name.  Every function takes and returns float64.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rows(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_one(x, w, eps):
    """The layers' norm: the stored weight is the distance from one."""
    return unit_rows(x, eps) * (1.0 + w)


def rotation_frequencies(rot):
    """Pair i's angle per position, and the factor on cos and sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def place(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(place(float(sc["fast"]))), 0)
    hi = min(math.ceil(place(float(sc["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=F64)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, rot):
    """x [T, heads, dim]: the first rot.dims dimensions of every head turn by position * frequency, dimension i with
    i + dims/2; the others stay."""
    dims = int(rot["dims"])
    half = dims // 2
    f, mag = rotation_frequencies(rot)
    ang = positions.to(F64)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def sink_softmax_heads(q, k, v, positions, scale, size, sink=0.0):
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence -> [T, H, dv].  A query at position i sees the keys j with
    0 <= i - j < size (size None: every j <= i); the denominator has one more term, exp(sink), that carries no value
    (sink None: an ordinary softmax)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    i, j = positions[:, None], positions[None, :]
    seen = (i - j >= 0) if size is None else (i - j >= 0) & (i - j < size)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * scale
        e = torch.where(seen, torch.exp(s), torch.zeros_like(s))
        extra = 0.0 if sink is None else math.exp(sink)
        out[:, hd] = (e / (extra + e.sum(-1, keepdim=True))) @ v[:, g]
    return out


def decay_recurrence(q, k, v, decay, state=None):
    """q, k [T, H, d], v [T, H, dv]: S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  Returns (o [T, H, dv], S)."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=F64) if state is None else state.clone()
    o = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for t in range(T):
        for hd in range(H):
            S[hd] = float(decay[hd]) * S[hd] + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S[hd].T @ q[t, hd]
    return o, S


def window_sink_attention(h, w, m, eps, positions):
    """The left side.  h [T, width]; w: the side's tensors by short name ('q', 'q.b', 'q.norm', ..); m: its sizes."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = h @ w["q"].T + w["q.b"]
    k = h @ w["k"].T + w["k.b"]
    v = h @ w["v"].T + w["v.b"]
    q = unit_rows(q, eps) * w["q.norm"]                       # over the whole projection, all heads at once
    k = unit_rows(k, eps) * w["k.norm"]
    q, k, v = q.reshape(T, H, d), k.reshape(T, G, d), v.reshape(T, G, dv)
    if m.get("rot"):
        q, k = rotate(q, positions, m["rot"]), rotate(k, positions, m["rot"])
    size = int(m["mask"]["size"]) if m.get("mask") else None
    out = sink_softmax_heads(q, k, v, positions, float(m["scale"]), size)
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(T, H * dv) * gate) @ w["o"].T


def lightning_attention(h, w, m, eps, state=None):
    """The right side.  Returns (output [T, width], the states after the last token [heads, dim, vdim])."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    silu = torch.nn.functional.silu
    q = silu(h @ w["q"].T).reshape(T, H, d)
    k = silu(h @ w["k"].T).reshape(T, H, d)
    v = silu(h @ w["v"].T).reshape(T, H, dv)
    o, S = decay_recurrence(q, k, v, m["decay"], state)
    o = unit_rows(o.reshape(T, H * dv), eps) * w["norm"]                     # all heads normed together
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T, S


def side_by_side(h, w, m, eps, positions):
    """The 'parallel' mixer: both sides read h."""
    pick = lambda side: {k[len(side) + 1:]: v for k, v in w.items() if k.startswith(side + ".")}
    left = window_sink_attention(h, pick("left"), m["left"], eps, positions)
    right, _ = lightning_attention(h, pick("right"), m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def capped_feed_forward(h, w, f):
    limit = float(f["limit"])
    g = torch.clamp(h @ w["gate"].T, max=limit)
    u = torch.clamp(h @ w["up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def layer(x, i, cfg, tensors, positions):
    eps = float(cfg["norm"]["eps"])
    entry = cfg["layers"][i]
    t = lambda name: tensors[f"l{i}.{name}"].to(F64)
    under = lambda prefix: {k[len(f"l{i}.{prefix}."):]: v.to(F64) for k, v in tensors.items() if k.startswith(f"l{i}.{prefix}.")}
    if entry["type"] != "parallel":
        raise ValueError(f"layer type {entry['type']!r}")
    x = x + t("ls1") * side_by_side(norm_around_one(x, t("norm1"), eps), under("mix"), entry["mixer"], eps, positions)
    if entry.get("mlp") is not None:
        if entry["mlp"]["kind"] != "dense":
            raise ValueError(f"feed-forward kind {entry['mlp']['kind']!r}")
        x = x + t("ls2") * capped_feed_forward(norm_around_one(x, t("norm2"), eps), under("mlp"), entry["mlp"])
    return x


def run_order(cfg):
    """(layer, whether the embedding rows are added before it) for every layer run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    out = [(i, False) for i in range(a)]
    for r in range(times):
        out += [(i, r > 0 and i == a) for i in range(a, b)]
    return out + [(i, False) for i in range(b, n)]


def forward(cfg, tensors, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence.  ``layers_out``: a list that gets the stream after every layer run."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.shape[0])
    table = tensors["embed"].to(F64)
    x0 = table[tokens]
    x = x0.clone()
    for i, add in run_order(cfg):
        if add:
            x = x + x0
        x = layer(x, i, cfg, tensors, positions)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = norm_around_one(x, tensors["final.norm"].to(F64), float(cfg["norm"]["eps"]))
    return x @ table.T


def read_model(path):
    """(raw config, tensors by name) of a model folder."""
    import json
    from pathlib import Path
    from safetensors.torch import load_file
    path = Path(path)
    return json.loads((path / "config.json").read_text()), load_file(str(path / "model.safetensors"))


def greedy(cfg, tensors, prompt, n_new):
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(cfg, tensors, ids)[-1].argmax()))
    return ids[len(prompt):]
