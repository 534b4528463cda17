"""Dotorax: a decoder whose sublayers each stand between two norms (a norm in front, a norm of
their own behind, a gain on what they add) and read their normed rows through a short convolution
over time, with three kinds of mixer in any order: softmax attention with rotated q and k, one
sigmoid gate a head and, optionally, the keys and values of an earlier layer; gated linear
attention with a decay per key channel; and attention over a sliding window with pooled blocks
before it beside a gated linear recurrent unit.  Feed-forwards are gated with clamped branches.
The embedding adds a learned table of positions; the head is a matrix of its own.

This file holds what is specific to the design: the keys of its config.json, their checks, the
tensor names of its checkpoints and the translation into a `ModelSpec` of generic parts.

    config.json
      architecture: "Dotorax"; vocab; width; max_positions; norm.eps; residual_mult; canon.taps
      layers: [{type: "attention", mixer: {heads, kv_heads, dim, vdim, scale, rot: {base, dims}, kv_from?}, mlp}
             | {type: "gla", mixer: {heads, dim, vdim, tau}, mlp}
             | {type: "parallel", mixer: {left: {heads, kv_heads, dim, vdim, scale, rot: {base, dims},
                                                 mask: {size, pool}},
                                          right: {width, blocks, conv}, left_scale, right_scale}, mlp}]
      mlp: null | {kind: "dense", ff, limit}
    tensors
      embed; pos [max_positions, width]; final.norm; head
      l<i>.norm1, norm1b, canon1 [width, taps] and, with a feed-forward, norm2, norm2b, canon2
      attention (l<i>.mix.): q, k, v, g [heads, width], o     (k and v absent with kv_from)
      gla: q, k, v, g, o, norm [vdim], a1 [rank, width], a2, a2.b
      parallel: left.{q, k, v, temp [heads], o}; right.{y, y.b, x, x.b, conv, conv.b, ra, ra.b, ri, ri.b, lam, o}
      l<i>.mlp.{gate, up, down}

Every norm's gain is 1 + the stored weight.  The rank of the decays' low-rank map is the first
size of `a1`; a configuration may state it as `mixer.rank` (random weights need it).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import List

from ..config.registry import ConfigError, register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# every norm's gain is this plus the stored weight
NORM_OFFSET = 1.0
DEFAULT_DECAY_RANK = 16


def _get(d: dict, key: str, where: str, kind=None):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json of Dotorax lacks {where}{key}")
    v = d[key]
    if kind == "int":
        if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
            raise ConfigError(f"{where}{key} must be a positive integer, got {v!r}")
    elif kind == "float":
        if isinstance(v, bool) or not isinstance(v, (int, float)) or not float(v) > 0:
            raise ConfigError(f"{where}{key} must be a positive number, got {v!r}")
    return v


def _check_attention(m: dict, at: str, windowed: bool) -> None:
    for k in ("heads", "kv_heads", "dim", "vdim"):
        _get(m, k, at, "int")
    if m["heads"] % m["kv_heads"]:
        raise ConfigError(f"{at}heads {m['heads']} must be a multiple of kv_heads {m['kv_heads']}")
    _get(m, "scale", at, "float")
    rot = _get(m, "rot", at)
    _get(rot, "base", at + "rot.", "float")
    dims = _get(rot, "dims", at + "rot.", "int")
    if dims % 2 or dims > m["dim"]:
        raise ConfigError(f"{at}rot.dims {dims} must be even and at most dim {m['dim']}")
    if windowed:
        mask = _get(m, "mask", at)
        _get(mask, "size", at + "mask.", "int")
        _get(mask, "pool", at + "mask.", "int")


@register_architecture("Dotorax")
@dataclass
class DotoraxConfig:
    vocab: int
    width: int
    eps: float
    max_positions: int
    residual_mult: float
    taps: int
    layers: List[dict] = field(default_factory=list)
    unused_tensors: List[str] = field(default_factory=list)    # in the folder, without a part to act on

    architecture = "Dotorax"
    cli_type_names = ("dotorax",)

    # ------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: dict) -> "DotoraxConfig":
        layers = _get(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("layers must be a list with at least one layer")
        cfg = cls(vocab=_get(d, "vocab", "", "int"), width=_get(d, "width", "", "int"),
                  eps=float(_get(_get(d, "norm", ""), "eps", "norm.", "float")),
                  max_positions=_get(d, "max_positions", "", "int"),
                  residual_mult=float(_get(d, "residual_mult", "", "float")),
                  taps=_get(_get(d, "canon", ""), "taps", "canon.", "int"),
                  layers=copy.deepcopy(layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.taps > 8:
            raise ConfigError(f"canon.taps {self.taps}: the kernels take up to 8")
        for i, layer in enumerate(self.layers):
            at = f"layers[{i}]."
            kind = _get(layer, "type", at)
            m = _get(layer, "mixer", at)
            at_m = at + "mixer."
            if kind == "attention":
                _check_attention(m, at_m, windowed=False)
                if "kv_from" in m:
                    j = m["kv_from"]
                    if not isinstance(j, int) or isinstance(j, bool) or not 0 <= j < i:
                        raise ConfigError(f"{at_m}kv_from {j!r} must name an earlier layer")
                    src = self.layers[j]
                    if src.get("type") != "attention" or "kv_from" in src["mixer"]:
                        raise ConfigError(f"{at_m}kv_from {j}: that layer has no keys and values of its own")
                    s = src["mixer"]
                    if any(s[k] != m[k] for k in ("kv_heads", "dim", "vdim")) or s["rot"] != m["rot"]:
                        raise ConfigError(f"{at_m}kv_from {j}: kv heads, sizes and rotation must equal that layer's")
            elif kind == "gla":
                for k in ("heads", "dim", "vdim"):
                    _get(m, k, at_m, "int")
                _get(m, "tau", at_m, "float")
                if "rank" in m:
                    _get(m, "rank", at_m, "int")
            elif kind == "parallel":
                _check_attention(_get(m, "left", at_m), at_m + "left.", windowed=True)
                right = _get(m, "right", at_m)
                for k in ("width", "blocks", "conv"):
                    _get(right, k, at_m + "right.", "int")
                if right["width"] % right["blocks"]:
                    raise ConfigError(f"{at_m}right.width {right['width']} must be a multiple of blocks {right['blocks']}")
                if right["conv"] > 8:
                    raise ConfigError(f"{at_m}right.conv {right['conv']}: the kernels take up to 8 taps")
                for k in ("left_scale", "right_scale"):
                    v = _get(m, k, at_m)
                    if isinstance(v, bool) or not isinstance(v, (int, float)):
                        raise ConfigError(f"{at_m}{k} must be a number, got {v!r}")
            else:
                raise ConfigError(f"{at}type {kind!r} is not a mixer of this design (attention, gla, parallel)")
            mlp = layer.get("mlp")
            if mlp is not None:
                if _get(mlp, "kind", at + "mlp.") != "dense":
                    raise ConfigError(f"{at}mlp.kind {mlp['kind']!r} is not a feed-forward of this design (dense)")
                _get(mlp, "ff", at + "mlp.", "int")
                _get(mlp, "limit", at + "mlp.", "float")

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "canon": {"taps": self.taps},
                "layers": copy.deepcopy(self.layers), "max_positions": self.max_positions,
                "norm": {"eps": self.eps}, "residual_mult": self.residual_mult, "vocab": self.vocab,
                "width": self.width}

    def with_tensor_shapes(self, shapes: dict) -> "DotoraxConfig":
        """The configuration with the sizes that only a folder's tensors state (`shapes`: tensor name
        -> shape): the rank of a gla layer's decay map.  What a folder holds of a second sublayer
        that the layer does not have is left in the file."""
        cfg = copy.deepcopy(self)
        for i, layer in enumerate(cfg.layers):
            if layer["type"] == "gla" and f"l{i}.mix.a1" in shapes:
                layer["mixer"]["rank"] = int(shapes[f"l{i}.mix.a1"][0])
            if layer.get("mlp") is None:
                cfg.unused_tensors += [n for n in (f"l{i}.norm2", f"l{i}.norm2b", f"l{i}.canon2") if n in shapes]
        return cfg

    # ------------------------------------------------------------ translation
    def _rotary(self, m: dict, pairing: str) -> PartSpec:
        return PartSpec("rotary", {"head_dim": m["dim"], "rotary_dim": int(m["rot"]["dims"]),
                                   "theta": float(m["rot"]["base"]), "pairing": pairing,
                                   "max_positions": self.max_positions})

    def _attention(self, p: str, m: dict) -> PartSpec:
        own = "kv_from" not in m
        names = {k: p + k for k in (("q", "k", "v", "g", "o") if own else ("q", "g", "o"))}
        return PartSpec("gated_attention",
                        {"hidden_size": self.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
                         "key_dim": m["dim"], "value_dim": m["vdim"], "softmax_scale": float(m["scale"]),
                         "gate": "head", "own_kv": own}, names)

    def _window_attention(self, p: str, m: dict) -> PartSpec:
        names = {k: p + k for k in ("q", "k", "v", "o")}
        names["head_scale"] = p + "temp"
        return PartSpec("gated_attention",
                        {"hidden_size": self.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
                         "key_dim": m["dim"], "value_dim": m["vdim"], "softmax_scale": float(m["scale"]),
                         "window": int(m["mask"]["size"]), "pool": int(m["mask"]["pool"]), "qk_norm": "head",
                         "eps": self.eps, "head_scale": True}, names)

    def _recurrence(self, p: str, m: dict) -> PartSpec:
        names = {k: p + k for k in ("y", "x", "conv", "ra", "ri", "lam", "o")}
        names.update(y_bias=p + "y.b", x_bias=p + "x.b", conv_bias=p + "conv.b", ra_bias=p + "ra.b",
                     ri_bias=p + "ri.b")
        return PartSpec("gated_linear_recurrence",
                        {"hidden_size": self.width, "channels": m["width"], "blocks": m["blocks"],
                         "conv": m["conv"]}, names)

    def _mixer(self, i: int, layer: dict):
        """(mixer, position encoding of the layer or None)."""
        m, p = layer["mixer"], f"l{i}.mix."
        if layer["type"] == "attention":
            return self._attention(p, m), self._rotary(m, "half")
        if layer["type"] == "gla":
            names = {k: p + k for k in ("q", "k", "v", "g", "o", "norm", "a1", "a2")}
            names["a2_bias"] = p + "a2.b"
            return PartSpec("gated_linear_attention",
                            {"hidden_size": self.width, "num_heads": m["heads"], "key_dim": m["dim"],
                             "value_dim": m["vdim"], "decay_rank": int(m.get("rank", DEFAULT_DECAY_RANK)),
                             "tau": float(m["tau"]), "eps": self.eps}, names), None
        left, right = m["left"], m["right"]
        return PartSpec("side_by_side",
                        {"left": self._window_attention(p + "left.", left),
                         "right": self._recurrence(p + "right.", right),
                         "left_scale": float(m["left_scale"]), "right_scale": float(m["right_scale"])}), \
            self._rotary(left, "interleaved")

    def to_spec(self) -> ModelSpec:
        E, V = self.width, self.vocab
        norm = lambda name: PartSpec("rms_norm", {"size": E, "eps": self.eps, "weight_offset": NORM_OFFSET},
                                     {"weight": name})
        layers, schedule = [], []
        for i, layer in enumerate(self.layers):
            mlp = layer.get("mlp")
            ff = PartSpec("none") if mlp is None else PartSpec(
                "clamped_gated", {"hidden_size": E, "intermediate_size": int(mlp["ff"]),
                                  "limit": float(mlp["limit"])},
                {k: f"l{i}.mlp.{k}" for k in ("gate", "up", "down")})
            mixer, position = self._mixer(i, layer)
            own = {"post1": f"l{i}.norm1b", "conv1": f"l{i}.canon1"}
            if mlp is not None:
                own.update(post2=f"l{i}.norm2b", conv2=f"l{i}.canon2")
            layers.append(LayerSpec(
                block="sandwich", mixer=mixer, feed_forward=ff, mixer_norm=norm(f"l{i}.norm1"),
                feed_forward_norm=norm(f"l{i}.norm2") if mlp is not None else None, position=position,
                block_params={"size": E, "eps": self.eps, "gain": self.residual_mult, "taps": self.taps,
                              "weight_offset": NORM_OFFSET},
                block_tensors=own))
            source = layer["mixer"].get("kv_from") if layer["type"] == "attention" else None
            schedule.append(ScheduleEntry(layer=i, cache_line=i if source is None else int(source),
                                          writes_cache=source is None))
        return ModelSpec(
            architecture=self.architecture, vocab_size=V, hidden_size=E, max_positions=self.max_positions,
            embedding=PartSpec("token_pair_embedding",
                               {"vocab_size": V, "hidden_size": E, "scale": 1.0, "positions": self.max_positions},
                               {"weight": "embed", "places": "pos"}),
            layers=layers, schedule=schedule, final_norm=norm("final.norm"),
            head=PartSpec("lm_head", {"hidden_size": E, "vocab_size": V}, {"weight": "head"}),
            bos_token_id=None, eos_token_ids=[], ignored_tensor_suffixes=list(self.unused_tensors))
