"""The typed configuration of the Biguzen decoder and its description as parts.

A Biguzen model is a list of layers of two kinds around a residual stream that runs in several copies:

  attention   softmax attention with grouped key/value heads of a key size and a value size of their own, biases on q, k
              and v, a short causal convolution over time on every channel of q, k and v right after the projection, a
              rotation of the first ``rot.dims`` dimensions of each head in neighbouring pairs (2i with 2i + 1) with all
              frequencies divided by ``rot.scaling.factor``, a sliding window, a learned sink score per head in the
              softmax's denominator, and one sigmoid gate value per head on the head's output.  A layer with ``kv_from``: j
              has no key and value projections: it reads the keys and values that layer j cached, with its own queries,
              window, sink and gate.
  mlstm       a matrix memory per head with capped input and forget gates, kept relative to a running maximum; each
              head's output is divided by its root mean square, then the joined heads are multiplied by a weight and by
              the sigmoid of a gate projection.

A layer's feed-forward is dense (down(relu(up(h))^2)), or routed: small gelu experts chosen by sigmoid scores plus a
correction, from the best groups of neighbouring experts only, weighted by the scores over their sum times a scale, plus a
shared expert behind a sigmoid gate of one number per token; or the layer has none.  Every norm is a Dynamic Tanh,
tanh(alpha x) w + b.  The residual stream is ``streams`` copies: a sublayer reads sum_s in[s] x_s and its output goes into
every copy, x_t <- sum_s mix[s, t] x_s + out[t] y; the final norm reads the sum of the copies; the head is the embedding table.

config.json: ``architecture`` "Biguzen", ``vocab``, ``width``, ``streams``, ``norm.eps`` and ``layers``, a list of ``{"type":
"attention", "mixer": {heads, kv_heads, dim, vdim, scale, conv, mask: {size}, rot: {dims, base, scaling: {factor}}, kv_from},
"mlp": ..}`` and ``{"type": "mlstm", "mixer": {heads, dim, vdim, gate_cap}, "mlp": ..}`` with ``mlp`` null, ``{"kind": "dense",
"ff"}`` or ``{"kind": "moe", "expert": {ff}, "router": {experts, top, scale, groups: {count, keep}}, "shared": {ff}}``.  A missing
``conv`` is no convolution, a missing ``mask`` no window, a missing ``rot`` no rotation, a missing ``rot.scaling`` plain
frequencies, missing ``groups`` one group, a missing ``shared`` no shared expert.  Tensor names: ``embed``, ``final.norm``,
``l<i>.norm1`` / ``l<i>.norm2`` (each with ``.b`` and ``.alpha``), ``l<i>.hc1.{in,out,mix}`` / ``l<i>.hc2.{in,out,mix}``,
``l<i>.mix.{q,k,v}`` with ``.b`` and ``.conv``, ``l<i>.mix.{sink,g,o}`` (attention), ``l<i>.mix.{q,k,v,g,o,norm,i,f}`` with
``i.b`` and ``f.b`` (mlstm), ``l<i>.mlp.{up,down}`` (dense), ``l<i>.mlp.e<j>.{up,down}``, ``l<i>.mlp.{router,correction}``,
``l<i>.mlp.shared.{up,down,sg}`` (routed).
"""
from __future__ import annotations

from dataclasses import dataclass

from .registry import ConfigError, register_architecture
from .spec import LayerCall, ModelSpec, PartSpec, joined, tensor

LAYER_TYPES = ("attention", "mlstm")
MAX_STREAMS, MAX_TAPS, MAX_EXPERTS, MAX_TOP = 16, 16, 512, 64


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


@register_architecture("Biguzen", model_type="biguzen")
@dataclass(frozen=True)
class BiguzenConfig:
    vocab: int
    width: int
    streams: int
    eps: float
    layers: tuple          # of dicts as config.json holds them, checked
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, raw: dict) -> "BiguzenConfig":
        vocab = _positive(_get(raw, "vocab", int, "the model"), "vocab")
        width = _positive(_get(raw, "width", int, "the model"), "width")
        streams = _positive(_get(raw, "streams", int, "the model"), "streams")
        if streams > MAX_STREAMS:
            raise ConfigError(f"config.json: streams = {streams}; the stream kernels take up to {MAX_STREAMS}")
        eps = _positive(_get(raw.get("norm"), "eps", float, "norm"), "norm.eps")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        checked = []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]"
            kind = _get(layer, "type", str, where)
            if kind not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}.type = {kind!r} is not one of {', '.join(LAYER_TYPES)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where} lacks its mixer's sizes")
            mixer = cls._check_attention(m, where + ".mixer") if kind == "attention" else cls._check_mlstm(m, where + ".mixer")
            checked.append({"type": kind, "mixer": mixer, "mlp": cls._check_mlp(layer.get("mlp"), where + ".mlp")})
        for i, layer in enumerate(checked):
            j = layer["mixer"].get("kv_from")
            if j is None:
                continue
            where = f"layers[{i}].mixer"
            if not 0 <= j < i or checked[j]["type"] != "attention" or checked[j]["mixer"].get("kv_from") is not None:
                raise ConfigError(f"config.json: {where}.kv_from = {j} must name an earlier attention layer with keys and values of its own")
            a, b = layer["mixer"], checked[j]["mixer"]
            if any(a[k] != b[k] for k in ("kv_heads", "dim", "vdim")):
                raise ConfigError(f"config.json: {where} reads layer {j}'s keys and values but has other kv_heads, dim or vdim")
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(vocab, width, streams, eps, tuple(checked), eos_ids)

    @staticmethod
    def _check_attention(m: dict, where: str) -> dict:
        out = {k: _positive(_get(m, k, int, where), f"{where}.{k}") for k in ("heads", "kv_heads", "dim", "vdim")}
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"config.json: {where}: {out['heads']} heads are not a multiple of {out['kv_heads']} kv heads")
        if out["dim"] > 256 or out["vdim"] > 256:
            raise ConfigError(f"config.json: {where}: the attention kernels take key and value sizes up to 256")
        out["scale"] = _get(m, "scale", float, where)
        if m.get("conv") is not None:
            out["conv"] = _positive(_get(m, "conv", int, where), where + ".conv")
            if out["conv"] > MAX_TAPS:
                raise ConfigError(f"config.json: {where}.conv = {out['conv']}; the convolution takes up to {MAX_TAPS} taps")
        mask = m.get("mask")
        if mask:
            out["mask"] = {"size": _positive(_get(mask, "size", int, where + ".mask"), where + ".mask.size")}
        rot = m.get("rot")
        if rot:
            dims = _get(rot, "dims", int, where + ".rot")
            if dims <= 0 or dims % 2 or dims > out["dim"]:
                raise ConfigError(f"config.json: {where}.rot.dims = {dims} must be even, positive and at most the key size {out['dim']}")
            r = {"dims": dims, "base": _positive(_get(rot, "base", float, where + ".rot"), where + ".rot.base")}
            if rot.get("scaling"):
                r["scaling"] = {"factor": _positive(_get(rot["scaling"], "factor", float, where + ".rot.scaling"), where + ".rot.scaling.factor")}
            out["rot"] = r
        if m.get("kv_from") is not None:
            out["kv_from"] = _get(m, "kv_from", int, where)
        return out

    @staticmethod
    def _check_mlstm(m: dict, where: str) -> dict:
        out = {k: _positive(_get(m, k, int, where), f"{where}.{k}") for k in ("heads", "dim", "vdim")}
        out["gate_cap"] = _positive(_get(m, "gate_cap", float, where), where + ".gate_cap")
        if out["dim"] > 256 or out["vdim"] > 1023:
            raise ConfigError(f"config.json: {where}: the matrix memory takes key sizes up to 256 and value sizes up to 1023")
        return out

    @staticmethod
    def _check_mlp(f, where: str):
        if f is None:
            return None
        kind = _get(f, "kind", str, where)
        if kind == "dense":
            return {"kind": kind, "ff": _positive(_get(f, "ff", int, where), where + ".ff")}
        if kind != "moe":
            raise ConfigError(f"config.json: {where}.kind = {kind!r} is neither 'dense' nor 'moe'")
        r = f.get("router")
        out = {"kind": kind, "expert": {"ff": _positive(_get(f.get("expert"), "ff", int, where + ".expert"), where + ".expert.ff")}}
        router = {"experts": _positive(_get(r, "experts", int, where + ".router"), where + ".router.experts"),
                  "top": _positive(_get(r, "top", int, where + ".router"), where + ".router.top"),
                  "scale": _get(r, "scale", float, where + ".router")}
        E, top = router["experts"], router["top"]
        if E > MAX_EXPERTS or top > min(E, MAX_TOP):
            raise ConfigError(f"config.json: {where}.router: {top} of {E} experts (at most {MAX_TOP} of {MAX_EXPERTS})")
        count, keep = 1, 1
        if r.get("groups"):
            count = _positive(_get(r["groups"], "count", int, where + ".router.groups"), where + ".router.groups.count")
            keep = _positive(_get(r["groups"], "keep", int, where + ".router.groups"), where + ".router.groups.keep")
            router["groups"] = {"count": count, "keep": keep}
        if E % count or keep > count or keep * (E // count) < top:
            raise ConfigError(f"config.json: {where}.router: {E} experts in {count} groups of which {keep} are kept cannot give {top} choices")
        out["router"] = router
        if f.get("shared"):
            out["shared"] = {"ff": _positive(_get(f["shared"], "ff", int, where + ".shared"), where + ".shared.ff")}
        return out

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "streams": self.streams,
             "norm": {"eps": self.eps}, "layers": [dict(layer) for layer in self.layers]}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    # ------------------------------------------------------------------------------------------
    def _norm(self, name: str) -> PartSpec:
        W = self.width
        return PartSpec("norm", "dyt", {"width": W, "eps": self.eps},
                        {"weight": tensor(name, (W,), "vector", ("normal", 1.0, 0.1)), "bias": tensor(name + ".b", (W,), "vector", ("normal", 0.0, 0.1)),
                         "alpha": tensor(name + ".alpha", (), "vector", ("normal", 0.6, 0.02))})

    def _reader(self, norm_name: str, in_name: str | None) -> PartSpec:
        S = self.streams
        tensors = {"in": tensor(in_name, (S,), "vector", ("normal", 1.0 / S, 0.2 / S))} if in_name else {}
        return PartSpec("norm", "streams_in", {"streams": S}, tensors, {"norm": self._norm(norm_name)})

    def _storage_window(self, i: int):
        """By which window layer i's keys and values are kept: the longest of its own and its readers' (None: all)."""
        sizes = [layer["mixer"].get("mask") for k, layer in enumerate(self.layers)
                 if k == i or (layer["type"] == "attention" and layer["mixer"].get("kv_from") == i)]
        return None if any(s is None for s in sizes) else max(int(s["size"]) for s in sizes)

    def _attention(self, i: int, p: str, m: dict) -> PartSpec:
        W, H, G, d, dv = self.width, m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        borrows = m.get("kv_from") is not None
        std = W ** -0.5
        names, shapes = [p + "q"], [(H * d, W)]
        if not borrows:
            names += [p + "k", p + "v"]
            shapes += [(G * d, W), (G * dv, W)]
        rows = [s[0] for s in shapes]
        params = {"hidden_size": W, "num_heads": H, "num_kv_heads": G, "key_dim": d, "value_dim": dv, "scale": m["scale"],
                  "window": m["mask"]["size"] if m.get("mask") else None, "eps": self.eps, "qk_norm": None, "sink": "learned",
                  "gate": "head_sigmoid", "kv": "borrowed" if borrows else "own"}
        if not borrows:
            params["storage_window"] = self._storage_window(i)
        tensors = {"qkvg": joined(names + [p + "g"], shapes + [(H, W)], "matrix", ("normal", 0.0, 1.5 * std)),
                   "qkv_bias": joined([n + ".b" for n in names], [(r,) for r in rows], "vector", ("normal", 0.0, 0.3)),
                   "sink_scores": tensor(p + "sink", (H,), "vector", ("normal", 0.0, 1.0)),
                   "out": tensor(p + "o", (W, H * dv), "matrix", ("normal", 0.0, (H * dv) ** -0.5))}
        if m.get("conv"):
            params["conv_taps"] = m["conv"]
            tensors["conv"] = joined([n + ".conv" for n in names], [(r, m["conv"]) for r in rows], "vector", ("normal", 0.4, 0.3))
        parts = {}
        if m.get("rot"):
            sc = m["rot"].get("scaling")
            parts["position"] = PartSpec("position", "rotary", {"rotary_dim": m["rot"]["dims"], "theta": m["rot"]["base"], "pairing": "interleaved",
                                                                "scaling": {"kind": "linear", "factor": sc["factor"]} if sc else None})
        return PartSpec("mixer", "sink_attention", params, tensors, parts)

    def _mlstm(self, p: str, m: dict) -> PartSpec:
        W, H, d, dv = self.width, m["heads"], m["dim"], m["vdim"]
        std = W ** -0.5
        return PartSpec(
            "mixer", "mlstm",
            {"hidden_size": W, "num_heads": H, "key_dim": d, "value_dim": dv, "gate_cap": m["gate_cap"], "eps": self.eps,
             "query_scale": d ** -0.5},
            {"qkvg": joined([p + n for n in "qkvg"], [(H * d, W), (H * d, W), (H * dv, W), (H * dv, W)], "matrix", ("normal", 0.0, 1.5 * std)),
             "gates": joined([p + "i", p + "f"], [(H, W), (H, W)], "matrix", ("normal", 0.0, 2.0 * std)),
             "gate_bias": joined([p + "i.b", p + "f.b"], [(H,), (H,)], "vector", ("normal", 1.0, 1.5)),
             "norm": tensor(p + "norm", (H * dv,), "vector", ("normal", 1.0, 0.1)),
             "out": tensor(p + "o", (W, H * dv), "matrix", ("normal", 0.0, (H * dv) ** -0.5))})

    def _feed_forward(self, p: str, f: dict) -> PartSpec:
        W = self.width
        if f["kind"] == "dense":
            return PartSpec("feed_forward", "dense", {"hidden_size": W, "intermediate_size": f["ff"], "activation": "relu_squared"},
                            {"up": tensor(p + "up", (f["ff"], W), "matrix", ("normal", 0.0, W ** -0.5)),
                             "down": tensor(p + "down", (W, f["ff"]), "matrix", ("normal", 0.0, f["ff"] ** -0.5))})
        r, F = f["router"], f["expert"]["ff"]
        E = r["experts"]
        groups = r.get("groups") or {"count": 1, "keep": 1}
        router_names, router_shapes = [p + "router"], [(E, W)]
        params = {"hidden_size": W, "intermediate_size": F, "num_experts": E, "top": r["top"], "scale": r["scale"],
                  "groups": groups["count"], "keep": groups["keep"]}
        tensors = {"correction": tensor(p + "correction", (E,), "vector", ("normal", 0.0, 0.15)),
                   "up": joined([f"{p}e{e}.up" for e in range(E)], [(F, W)] * E, "matrix", ("normal", 0.0, W ** -0.5)),
                   "down": joined([f"{p}e{e}.down" for e in range(E)], [(W, F)] * E, "matrix", ("normal", 0.0, F ** -0.5))}
        if f.get("shared"):
            SF = f["shared"]["ff"]
            params["shared_size"] = SF
            router_names.append(p + "shared.sg")
            router_shapes.append((1, W))
            tensors["shared_up"] = tensor(p + "shared.up", (SF, W), "matrix", ("normal", 0.0, W ** -0.5))
            tensors["shared_down"] = tensor(p + "shared.down", (W, SF), "matrix", ("normal", 0.0, SF ** -0.5))
        tensors["router"] = joined(router_names, router_shapes, "matrix", ("normal", 0.0, 2.0 * W ** -0.5))
        return PartSpec("feed_forward", "routed_scored", params, tensors)

    def spec(self, tensor_names=None) -> ModelSpec:
        W, V, S = self.width, self.vocab, self.streams
        names = set(tensor_names) if tensor_names is not None else None

        def spread(p: str) -> dict:
            return {"mix": tensor(p + "mix", (S, S), "vector", ("normal", 1.0 / S, 0.3 / S)), "out": tensor(p + "out", (S,), "vector", ("normal", 1.0, 0.3))}

        layers, order = [], []
        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.", layer["mixer"]
            mixer = self._attention(i, p + "mix.", m) if layer["type"] == "attention" else self._mlstm(p + "mix.", m)
            parts = {"mixer_norm": self._reader(p + "norm1", p + "hc1.in"), "mixer": mixer}
            hc1 = spread(p + "hc1.")
            tensors = {"mixer_mix": hc1["mix"], "mixer_out": hc1["out"]}
            if layer["mlp"] is not None:
                hc2 = spread(p + "hc2.")
                parts["feed_forward_norm"] = self._reader(p + "norm2", p + "hc2.in")
                parts["feed_forward"] = self._feed_forward(p + "mlp.", layer["mlp"])
                tensors.update({"feed_forward_mix": hc2["mix"], "feed_forward_out": hc2["out"]})
            elif names is not None:
                # a checkpoint that holds the second sublayer's norm and stream weights of a layer without a feed-forward:
                # bound, and not used
                spare = {p + "norm2": (W,), p + "norm2.b": (W,), p + "norm2.alpha": (), p + "hc2.in": (S,), p + "hc2.out": (S,), p + "hc2.mix": (S, S)}
                tensors.update({f"spare_{n}": tensor(n, shape, "vector") for n, shape in spare.items() if n in names})
            layers.append(PartSpec("block", "hyper_connections", {"streams": S}, tensors, parts))
            order.append(LayerCall(i, cache_of=m.get("kv_from")))

        table = tensor("embed", (V, W), "table", ("normal", 0.0, 1.0))
        return ModelSpec(
            architecture=self.architecture, vocab_size=V, hidden_size=W, max_positions=None,
            embedding=PartSpec("embedding", "token_table", {"vocab_size": V, "hidden_size": W}, {"table": table}),
            layers=tuple(layers), order=tuple(order), final_norm=self._reader("final.norm", None),
            head=PartSpec("head", "linear", {"vocab_size": V, "hidden_size": W}, {"weight": table}),
            stop_token_ids=self.eos_token_ids, streams=S,
        )
