"""A plain, slow Biguzen in float64 on the CPU, written from the design's equations: one function per mechanism, whole
sequences only, no cache, no batching.  It shares no code with the library; the tests compare the library with it.

A model is a raw config.json dict and a dict of tensors by checkpoint name.  Every function takes and returns float64.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def dynamic_tanh(x, w, b, alpha):
    """The design's norm: no statistics, tanh(alpha x) w + b."""
    return torch.tanh(alpha * x) * w + b


def unit_rows(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def relu_squared(z):
    return torch.clamp(z, min=0.0) ** 2


# ---- streams ---------------------------------------------------------------------------------------------------

def streams_read(xs, weights):
    """xs [S, T, W]: what a sublayer reads, sum_s weights[s] xs[s]."""
    return torch.einsum("s,stw->tw", weights, xs)


def streams_write(xs, y, mix, out):
    """All streams at once from the old ones: new[t] = sum_s mix[s, t] xs[s] + out[t] y."""
    return torch.einsum("sr,stw->rtw", mix, xs) + out[:, None, None] * y[None]


# ---- attention ---------------------------------------------------------------------------------------------------

def short_convolution(u, taps_w):
    """u [T, C], taps_w [C, taps]: y_t = sum_j taps_w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    T, C = u.shape
    taps = taps_w.shape[1]
    padded = torch.cat([torch.zeros((taps - 1, C), dtype=F64), u], dim=0)
    y = torch.zeros((T, C), dtype=F64)
    for j in range(taps):
        y = y + taps_w[:, j][None, :] * padded[j:j + T]
    return y


def rotate_neighbours(x, positions, rot):
    """x [T, heads, dim]: of the first rot.dims dimensions of every head, dimension 2i turns with 2i + 1 by
    position * base^(-2i / dims) / factor; the others stay."""
    dims, base = int(rot["dims"]), float(rot["base"])
    factor = float(rot["scaling"]["factor"]) if rot.get("scaling") else 1.0
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=F64)
    ang = positions.to(F64)[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def sink_softmax_heads(q, k, v, scale, size, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence -> [T, H, dv].  Query i sees the keys j with
    0 <= i - j < size (size None: every j <= i); head h's denominator has one more term, exp(sink[h]), with no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    per = H // G
    out = torch.zeros((T, H, v.shape[2]), dtype=F64)
    i = torch.arange(T)
    seen = (i[:, None] >= i[None, :])
    if size is not None:
        seen = seen & (i[:, None] - i[None, :] < size)
    for h in range(H):
        g = h // per
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, -math.inf)
        top = torch.maximum(s.max(dim=1).values, sink[h].expand(T)) if sink is not None else s.max(dim=1).values
        e = torch.exp(s - top[:, None])
        denom = e.sum(dim=1) + (torch.exp(sink[h] - top) if sink is not None else 0.0)
        out[:, h] = (e / denom[:, None]) @ v[:, g]
    return out


def attention_keys_values(h, w, p, m, positions):
    """The keys (convolved, rotated) and values (convolved) that a layer with projections of its own makes."""
    G, d, dv = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = h @ w[p + "v"].T + w[p + "v.b"]
    if m.get("conv"):
        k, v = short_convolution(k, w[p + "k.conv"]), short_convolution(v, w[p + "v.conv"])
    k = k.reshape(T, G, d)
    if m.get("rot"):
        k = rotate_neighbours(k, positions, m["rot"])
    return k, v.reshape(T, G, dv)


def attention_mixer(h, w, p, m, positions, kv):
    """kv: the keys and values to use (this layer's own or another layer's)."""
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = h @ w[p + "q"].T + w[p + "q.b"]
    if m.get("conv"):
        q = short_convolution(q, w[p + "q.conv"])
    q = q.reshape(T, H, d)
    if m.get("rot"):
        q = rotate_neighbours(q, positions, m["rot"])
    k, v = kv
    size = int(m["mask"]["size"]) if m.get("mask") else None
    o = sink_softmax_heads(q, k, v, float(m["scale"]), size, w[p + "sink"])
    gate = torch.sigmoid(h @ w[p + "g"].T)                    # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * dv) @ w[p + "o"].T


# ---- matrix memory ---------------------------------------------------------------------------------------------

def capped(z, cap):
    return cap * torch.tanh(z / cap)


def matrix_memory(q, k, v, log_in, log_forget):
    """q, k [T, d], v [T, dv], the two log gates [T], one head -> [T, dv].  The state is kept relative to a running
    maximum m that starts at zero."""
    T, d = q.shape
    dv = v.shape[1]
    S = torch.zeros((d, dv), dtype=F64)
    n = torch.zeros((d,), dtype=F64)
    m = torch.zeros((), dtype=F64)
    out = torch.zeros((T, dv), dtype=F64)
    for t in range(T):
        m_new = torch.maximum(log_forget[t] + m, log_in[t])
        keep, take = torch.exp(log_forget[t] + m - m_new), torch.exp(log_in[t] - m_new)
        S = keep * S + take * torch.outer(k[t], v[t])
        n = keep * n + take * k[t]
        m = m_new
        out[t] = (S.T @ q[t]) / (torch.maximum(torch.abs(n @ q[t]), torch.exp(-m)) + 1e-6)
    return out


def mlstm_mixer(h, w, p, m, eps):
    H, d, dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    T = h.shape[0]
    q = (h @ w[p + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ w[p + "k"].T).reshape(T, H, d)
    v = (h @ w[p + "v"].T).reshape(T, H, dv)
    log_in = capped(h @ w[p + "i"].T + w[p + "i.b"], cap)                                    # [T, H]
    log_forget = torch.nn.functional.logsigmoid(capped(h @ w[p + "f"].T + w[p + "f.b"], cap))
    heads = [unit_rows(matrix_memory(q[:, a], k[:, a], v[:, a], log_in[:, a], log_forget[:, a]), eps) for a in range(H)]
    o = torch.cat(heads, dim=1) * w[p + "norm"] * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


# ---- feed-forwards -----------------------------------------------------------------------------------------------

def dense_feed_forward(h, w, p):
    return relu_squared(h @ w[p + "up"].T) @ w[p + "down"].T


def expert(h, w, p):
    return gelu_erf(h @ w[p + "up"].T) @ w[p + "down"].T


def route(h, w, p, r):
    """-> chosen [T, top] (expert indices) and weights [T, top]."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(h @ w[p + "router"].T)
    choice = s + w[p + "correction"]
    T = h.shape[0]
    if r.get("groups"):
        count, keep = int(r["groups"]["count"]), int(r["groups"]["keep"])
        size = E // count
        by_group = choice.reshape(T, count, size)
        group_score = by_group.topk(min(2, size), dim=2).values.sum(dim=2)
        best = group_score.topk(keep, dim=1).indices
        allowed = torch.zeros((T, count), dtype=torch.bool)
        allowed.scatter_(1, best, True)
        choice = by_group.masked_fill(~allowed[:, :, None], -math.inf).reshape(T, E)
    chosen = choice.topk(top, dim=1).indices
    picked = s.gather(1, chosen)
    weights = picked / (picked.sum(dim=1, keepdim=True) + 1e-20) * float(r["scale"])
    return chosen, weights


def routed_feed_forward(h, w, p, f):
    chosen, weights = route(h, w, p, f["router"])
    out = torch.zeros((h.shape[0], w[p + "e0.down"].shape[0]), dtype=F64)
    for t in range(h.shape[0]):
        for c in range(chosen.shape[1]):
            e = int(chosen[t, c])
            out[t] += weights[t, c] * expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if f.get("shared"):
        out = out + torch.sigmoid(h @ w[p + "shared.sg"].T) * expert(h, w, p + "shared.")
    return out


# ---- the model -----------------------------------------------------------------------------------------------------

def forward(raw, tensors, ids, layer_results=None):
    """Logits [T, vocab] of one sequence from its first token.  ``layer_results``: a list that gets the sum of the
    streams after every layer."""
    w = {k: t.to(F64) for k, t in tensors.items()}
    eps = float(raw["norm"]["eps"])
    T = len(ids)
    positions = torch.arange(T)
    x = w["embed"][torch.tensor(ids, dtype=torch.long)]
    S = int(raw.get("streams", 1))
    xs = x[None].repeat(S, 1, 1)
    kept = {}                                                    # layer -> its keys and values

    def norm(name, u):
        return dynamic_tanh(u, w[name], w[name + ".b"], w[name + ".alpha"])

    for i, layer in enumerate(raw["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        u = streams_read(xs, w[p + "hc1.in"])
        hn = norm(p + "norm1", u)
        if layer["type"] == "attention":
            if m.get("kv_from") is not None:
                kv = kept[int(m["kv_from"])]
            else:
                kv = kept[i] = attention_keys_values(hn, w, p + "mix.", m, positions)
            y = attention_mixer(hn, w, p + "mix.", m, positions, kv)
        elif layer["type"] == "mlstm":
            y = mlstm_mixer(hn, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        xs = streams_write(xs, y, w[p + "hc1.mix"], w[p + "hc1.out"])
        f = layer.get("mlp")
        if f is not None:
            hn = norm(p + "norm2", streams_read(xs, w[p + "hc2.in"]))
            y = dense_feed_forward(hn, w, p + "mlp.") if f["kind"] == "dense" else routed_feed_forward(hn, w, p + "mlp.", f)
            xs = streams_write(xs, y, w[p + "hc2.mix"], w[p + "hc2.out"])
        if layer_results is not None:
            layer_results.append(xs.sum(0))
    x = xs.sum(0)
    return norm("final.norm", x) @ w["embed"].T


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
