"""The typed configuration of the Matalix decoder and its description as parts.

A Matalix model is a list of pre-norm layers whose mixer is two mixers side by side, both reading the layer's normed
input, their outputs added with one fixed weight each:

  left    softmax attention with grouped key/value heads of a key size and a value size of their own, biases on q, k and
          v, one RMS norm over the whole q projection and one over the whole k projection (before the heads are cut),
          a rotation of the first ``rot.dims`` dimensions of each head (frequencies stretched for long sequences), a
          sliding window, a sink of score zero in the softmax's denominator, and an elementwise sigmoid gate on the
          joined heads
  right   linear attention with one fixed decay per head over silu'd q, k and v, the joined heads normed together
          with a weight and gated by a sigmoid

Every branch's output is multiplied by a learned vector before it is added (``ls1``, ``ls2``); norm weights are stored
as the distance from one; the feed-forward caps its gate and up rows; a range of layers may run several times in a row
with the same weights and a cache of its own each time, the embedding rows added to the stream before every pass but
the first; the head is the embedding table.

config.json: ``architecture`` "Matalix", ``vocab``, ``width``, ``norm.eps``, ``loop`` {start, stop, times} (optional), and
``layers``: a list of ``{"type": "parallel", "mixer": {"left": {heads, kv_heads, dim, vdim, scale, mask: {size}, rot:
{dims, base, scaling: {factor, original, fast, slow}}}, "left_scale", "right": {heads, dim, vdim, decay: [..]},
"right_scale"}, "mlp": {"kind": "dense", "ff", "limit"} or null}``.  Tensor names: ``embed``, ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.ls1``, ``l<i>.ls2``, ``l<i>.mix.left.{q,k,v}`` with ``.b`` and (q, k) ``.norm``,
``l<i>.mix.left.{g,o}``, ``l<i>.mix.right.{q,k,v,g,o,norm}``, ``l<i>.mlp.{gate,up,down}``, ``final.norm``.
"""
from __future__ import annotations

from dataclasses import dataclass

from .registry import ConfigError, register_architecture
from .spec import LayerCall, ModelSpec, PartSpec, joined, tensor

_AROUND_ZERO = ("normal", 0.0, 0.1)          # norm weights are kept as the distance from one
_AROUND_ONE = ("normal", 1.0, 0.1)
LAYER_TYPES = ("parallel",)
# the gate of the feed-forward is g * sigmoid(GATE_SLOPE * g), and the up row is shifted by UP_SHIFT
GATE_SLOPE, UP_SHIFT = 1.702, 1.0


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


@register_architecture("Matalix", model_type="matalix")
@dataclass(frozen=True)
class MatalixConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple          # of dicts as config.json holds them, checked
    loop: tuple | None     # (start, stop, times)
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, raw: dict) -> "MatalixConfig":
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
            if kind not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}.type = {kind!r} is not one of {', '.join(LAYER_TYPES)}")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"config.json: {where} lacks its mixer's sizes")
            checked.append({"type": kind,
                            "mixer": {"left": cls._check_left(m.get("left"), where + ".mixer.left"),
                                      "left_scale": _get(m, "left_scale", float, where + ".mixer"),
                                      "right": cls._check_right(m.get("right"), where + ".mixer.right"),
                                      "right_scale": _get(m, "right_scale", float, where + ".mixer")},
                            "mlp": cls._check_mlp(layer.get("mlp"), where + ".mlp")})
        loop = raw.get("loop")
        if loop:
            a, b, times = (_get(loop, k, int, "loop") for k in ("start", "stop", "times"))
            if not 0 <= a < b <= len(checked) or times < 1:
                raise ConfigError(f"config.json: loop = layers {a} .. {b} - 1, {times} times, over {len(checked)} layers")
            loop = (a, b, times)
        else:
            loop = None
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(vocab, width, eps, tuple(checked), loop, eos_ids)

    @staticmethod
    def _check_left(m, where: str) -> dict:
        out = {k: _positive(_get(m, k, int, where), f"{where}.{k}") for k in ("heads", "kv_heads", "dim", "vdim")}
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"config.json: {where}: {out['heads']} heads are not a multiple of {out['kv_heads']} kv heads")
        if out["dim"] > 256 or out["vdim"] > 256:
            raise ConfigError(f"config.json: {where}: the attention kernels take key and value sizes up to 256")
        out["scale"] = _get(m, "scale", float, where)
        mask = m.get("mask")
        out["mask"] = {"size": _positive(_get(mask, "size", int, where + ".mask"), where + ".mask.size")} if mask else None
        rot = m.get("rot")
        if rot:
            dims = _get(rot, "dims", int, where + ".rot")
            if dims <= 0 or dims % 2 or dims > out["dim"]:
                raise ConfigError(f"config.json: {where}.rot.dims = {dims} must be even, positive and at most the key size {out['dim']}")
            r = {"dims": dims, "base": _positive(_get(rot, "base", float, where + ".rot"), where + ".rot.base")}
            sc = rot.get("scaling")
            r["scaling"] = ({k: _positive(_get(sc, k, float, where + ".rot.scaling"), f"{where}.rot.scaling.{k}")
                             for k in ("factor", "original", "fast", "slow")} if sc else None)
            out["rot"] = r
        else:
            out["rot"] = None
        return out

    @staticmethod
    def _check_right(m, where: str) -> dict:
        out = {k: _positive(_get(m, k, int, where), f"{where}.{k}") for k in ("heads", "dim", "vdim")}
        decay = m.get("decay")
        if not isinstance(decay, (list, tuple)) or len(decay) != out["heads"]:
            raise ConfigError(f"config.json: {where}.decay must list one decay for each of {out['heads']} heads")
        out["decay"] = [float(d) for d in decay]
        if out["dim"] > 256 or out["vdim"] > 1024:
            raise ConfigError(f"config.json: {where}: the recurrence takes key sizes up to 256 and value sizes up to 1024")
        return out

    @staticmethod
    def _check_mlp(f, where: str):
        if f is None:
            return None
        kind = _get(f, "kind", str, where)
        if kind != "dense":
            raise ConfigError(f"config.json: {where}.kind = {kind!r}; this design's feed-forwards are 'dense'")
        return {"kind": kind, "ff": _positive(_get(f, "ff", int, where), where + ".ff"),
                "limit": _positive(_get(f, "limit", float, where), where + ".limit")}

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "layers": [dict(layer) for layer in self.layers]}
        if self.loop:
            d["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d

    # ------------------------------------------------------------------------------------------
    def _left(self, p: str, m: dict) -> PartSpec:
        W, H, G, d, dv = self.width, m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        parts = {}
        if m["rot"] is not None:
            parts["position"] = PartSpec("position", "rotary", {"rotary_dim": m["rot"]["dims"], "theta": m["rot"]["base"],
                                                                "pairing": "half_split", "scaling": m["rot"]["scaling"]})
        return PartSpec(
            "mixer", "sink_attention",
            {"hidden_size": W, "num_heads": H, "num_kv_heads": G, "key_dim": d, "value_dim": dv, "scale": m["scale"],
             "window": m["mask"]["size"] if m["mask"] else None, "eps": self.eps, "qk_norm": "projection", "sink": True,
             "gate": "sigmoid", "input": "shared"},
            {"qkv_bias": joined((p + "q.b", p + "k.b", p + "v.b"), ((H * d,), (G * d,), (G * dv,)), "vector", ("normal", 0.0, 0.3)),
             "q_norm": tensor(p + "q.norm", (H * d,), "vector", ("normal", 1.2, 0.4)),
             "k_norm": tensor(p + "k.norm", (G * d,), "vector", ("normal", 1.2, 0.4)),
             "out": tensor(p + "o", (W, H * dv), "matrix", ("normal", 0.0, 0.06))},
            parts)

    def _shared_input(self, p: str, m: dict):
        """Both sides' input matrices as one: left q | k | v | g, then right q | k | v | g (one product a layer reads the
        normed rows once)."""
        W, a, r = self.width, m["left"], m["right"]
        H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
        names = [p + "left." + n for n in "qkvg"] + [p + "right." + n for n in "qkvg"]
        shapes = [(H * d, W), (G * d, W), (G * dv, W), (H * dv, W),
                  (r["heads"] * r["dim"], W), (r["heads"] * r["dim"], W), (r["heads"] * r["vdim"], W), (r["heads"] * r["vdim"], W)]
        return joined(names, shapes, "matrix", ("normal", 0.0, 0.1))

    def _right(self, p: str, m: dict) -> PartSpec:
        W, H, d, dv = self.width, m["heads"], m["dim"], m["vdim"]
        return PartSpec(
            "mixer", "retention",
            {"hidden_size": W, "num_heads": H, "key_dim": d, "value_dim": dv, "decay": tuple(m["decay"]), "key_scale": 1.0,
             "eps": self.eps, "input_activation": "silu", "norm": "joined", "gate_activation": "sigmoid", "input": "shared"},
            {"norm": tensor(p + "norm", (H * dv,), "vector", _AROUND_ONE),
             "out": tensor(p + "o", (W, H * dv), "matrix", ("normal", 0.0, 0.1))})

    def spec(self, tensor_names=None) -> ModelSpec:
        W, V, eps = self.width, self.vocab, self.eps
        names = set(tensor_names) if tensor_names is not None else None

        def norm(name: str) -> PartSpec:
            return PartSpec("norm", "rms", {"width": W, "eps": eps, "offset": 1.0}, {"weight": tensor(name, (W,), "vector", _AROUND_ZERO)})

        layers = []
        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.", layer["mixer"]
            parts = {"mixer_norm": norm(p + "norm1"),
                     "mixer": PartSpec("mixer", "parallel", {"weights": (m["left_scale"], m["right_scale"])},
                                       {"in": self._shared_input(p + "mix.", m)},
                                       {"left": self._left(p + "mix.left.", m["left"]), "right": self._right(p + "mix.right.", m["right"])})}
            scales = {"mixer_scale": tensor(p + "ls1", (W,), "vector", ("normal", 0.8, 0.2))}
            f = layer["mlp"]
            if f is not None:
                parts["feed_forward_norm"] = norm(p + "norm2")
                parts["feed_forward"] = PartSpec(
                    "feed_forward", "capped_gated", {"hidden_size": W, "intermediate_size": f["ff"], "limit": f["limit"],
                                                     "slope": GATE_SLOPE, "shift": UP_SHIFT},
                    {"gate_up": joined((p + "mlp.gate", p + "mlp.up"), ((f["ff"], W), (f["ff"], W)), "matrix", ("normal", 0.0, 0.08)),
                     "down": tensor(p + "mlp.down", (W, f["ff"]), "matrix", ("normal", 0.0, 0.06))})
                scales["feed_forward_scale"] = tensor(p + "ls2", (W,), "vector", ("normal", 0.8, 0.2))
            elif names is not None:
                # a checkpoint that holds the second norm and scale of a layer without a feed-forward: bound, and not used
                scales.update({f"spare_{n}": tensor(p + n, (W,), "vector", _AROUND_ZERO) for n in ("norm2", "ls2") if p + n in names})
            layers.append(PartSpec("block", "pre_norm_scaled", {"hidden_size": W}, scales, parts))

        n = len(self.layers)
        if self.loop:
            a, b, times = self.loop
            order = [LayerCall(i) for i in range(a)]
            for r in range(times):
                order += [LayerCall(i, adds_embedding=(r > 0 and i == a)) for i in range(a, b)]
            order += [LayerCall(i) for i in range(b, n)]
        else:
            order = [LayerCall(i) for i in range(n)]

        table = tensor("embed", (V, W), "table", ("normal", 0.0, 0.9))
        return ModelSpec(
            architecture=self.architecture, vocab_size=V, hidden_size=W, max_positions=None,
            embedding=PartSpec("embedding", "token_table", {"vocab_size": V, "hidden_size": W}, {"table": table}),
            layers=tuple(layers), order=tuple(order), final_norm=norm("final.norm"),
            head=PartSpec("head", "linear", {"vocab_size": V, "hidden_size": W}, {"weight": table}),
            stop_token_ids=self.eos_token_ids,
        )
