"""Sabipel: a decoder whose layers add a mixer's and a feed-forward's output, each computed from an
RMS norm of its own of the same stream, with three kinds of mixer in any order: a state-space mixer,
a matrix memory with exponential gates, and chunked softmax attention with a distance bias, norms
over whole q and k, values mixed with an earlier layer's and an output gate.  The embedding adds a
hashed table of token pairs and a learned table of positions.

This file holds what is specific to the design: the keys of its config.json, their checks, the
tensor names of its checkpoints and the translation into a `ModelSpec` of generic parts.

    config.json
      architecture: "Sabipel"; vocab; width; max_positions; norm.eps
      embedding: {scale, bigram: {buckets, mul_prev, mul_cur}}
      layers: [{type: "mamba2", mixer: {heads, vdim, state, groups, conv, norm_groups}, mlp}
             | {type: "mlstm", mixer: {heads, dim, vdim, gate_cap}, mlp}
             | {type: "attention", mixer: {heads, kv_heads, dim, vdim, scale, mask: {size}?, v_mix?}, mlp}]
      mlp: null | {kind: "dense", ff}
    tensors
      embed; bigram [buckets + 1, width]; pos [max_positions, width]; final.norm;
      l<i>.norm1, l<i>.norm2
      mamba2 (l<i>.mix.): in, conv, conv.b, dt_bias, A_log, D, norm, o
      mlstm: q, k, v, g, o, norm, i, i.b, f, f.b
      attention: q, k, v, q.norm, k.norm, vmix, g, o
      l<i>.mlp.{up, down}

The head is the embedding table itself, without the embedding's scale.  The first attention layer
whose configuration says v_mix hands its values on; every later such layer mixes them into its own
(the first one's stored `vmix` has nothing to act on and is left in the file).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import List, Optional

from ..config.registry import ConfigError, register_architecture
from ..config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# slope_h = 2^(-8 (h + 1) / H): the design fixes the 8
SLOPE_POWER = 8.0


def _get(d: dict, key: str, where: str, kind=None):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError(f"config.json of Sabipel lacks {where}{key}")
    v = d[key]
    if kind == "int":
        if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
            raise ConfigError(f"{where}{key} must be a positive integer, got {v!r}")
    elif kind == "float":
        if isinstance(v, bool) or not isinstance(v, (int, float)) or not float(v) > 0:
            raise ConfigError(f"{where}{key} must be a positive number, got {v!r}")
    return v


@register_architecture("Sabipel")
@dataclass
class SabipelConfig:
    vocab: int
    width: int
    eps: float
    max_positions: int
    embedding_scale: float
    buckets: int
    mul_prev: int
    mul_cur: int
    layers: List[dict] = field(default_factory=list)
    unused_tensors: List[str] = field(default_factory=list)    # in the folder, without a part to act on

    architecture = "Sabipel"
    cli_type_names = ("sabipel",)

    # ------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: dict) -> "SabipelConfig":
        layers = _get(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("layers must be a list with at least one layer")
        emb = _get(d, "embedding", "")
        big = _get(emb, "bigram", "embedding.")
        for k in ("mul_prev", "mul_cur"):
            v = _get(big, k, "embedding.bigram.")
            if not isinstance(v, int) or isinstance(v, bool) or v < 0:
                raise ConfigError(f"embedding.bigram.{k} must be an integer >= 0, got {v!r}")
        cfg = cls(vocab=_get(d, "vocab", "", "int"), width=_get(d, "width", "", "int"),
                  eps=float(_get(_get(d, "norm", ""), "eps", "norm.", "float")),
                  max_positions=_get(d, "max_positions", "", "int"),
                  embedding_scale=float(_get(emb, "scale", "embedding.", "float")),
                  buckets=_get(big, "buckets", "embedding.bigram.", "int"),
                  mul_prev=int(big["mul_prev"]), mul_cur=int(big["mul_cur"]),
                  layers=copy.deepcopy(layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        mixed_width = None
        for i, layer in enumerate(self.layers):
            at = f"layers[{i}]."
            kind = _get(layer, "type", at)
            m = _get(layer, "mixer", at)
            at_m = at + "mixer."
            if kind == "mamba2":
                for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups"):
                    _get(m, k, at_m, "int")
                if m["heads"] % m["groups"]:
                    raise ConfigError(f"{at_m}heads {m['heads']} must be a multiple of groups {m['groups']}")
                if (m["heads"] * m["vdim"]) % m["norm_groups"]:
                    raise ConfigError(f"{at_m}heads * vdim must be a multiple of norm_groups {m['norm_groups']}")
            elif kind == "mlstm":
                for k in ("heads", "dim", "vdim"):
                    _get(m, k, at_m, "int")
                _get(m, "gate_cap", at_m, "float")
            elif kind == "attention":
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    _get(m, k, at_m, "int")
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"{at_m}heads {m['heads']} must be a multiple of kv_heads {m['kv_heads']}")
                _get(m, "scale", at_m, "float")
                mask = m.get("mask")
                if mask is not None:
                    _get(mask, "size", at_m + "mask.", "int")
                if m.get("v_mix"):
                    width = m["kv_heads"] * m["vdim"]
                    if mixed_width is not None and width != mixed_width:
                        raise ConfigError(f"{at_m}v_mix: values {width} wide cannot be mixed with the "
                                          f"first such layer's, {mixed_width} wide")
                    mixed_width = width
            else:
                raise ConfigError(f"{at}type {kind!r} is not a mixer of this design (mamba2, mlstm, attention)")
            mlp = layer.get("mlp")
            if mlp is not None:
                if _get(mlp, "kind", at + "mlp.") != "dense":
                    raise ConfigError(f"{at}mlp.kind {mlp['kind']!r} is not a feed-forward of this design (dense)")
                _get(mlp, "ff", at + "mlp.", "int")

    def to_dict(self) -> dict:
        return {"architecture": self.architecture,
                "embedding": {"bigram": {"buckets": self.buckets, "mul_cur": self.mul_cur,
                                         "mul_prev": self.mul_prev}, "scale": self.embedding_scale},
                "layers": copy.deepcopy(self.layers), "max_positions": self.max_positions,
                "norm": {"eps": self.eps}, "vocab": self.vocab, "width": self.width}

    def first_mixing_layer(self) -> Optional[int]:
        return next((i for i, l in enumerate(self.layers)
                     if l["type"] == "attention" and l["mixer"].get("v_mix")), None)

    def with_tensor_shapes(self, shapes: dict) -> "SabipelConfig":
        """The configuration that leaves in the file what a folder holds without a part to act on:
        the first mixing layer's `vmix`, a second norm of a layer without feed-forward."""
        cfg = copy.deepcopy(self)
        names = [f"l{i}.norm2" for i, l in enumerate(self.layers) if l.get("mlp") is None]
        names += [f"l{i}.mix.vmix" for i, l in enumerate(self.layers)
                  if l["type"] == "attention" and (not l["mixer"].get("v_mix") or i == self.first_mixing_layer())]
        cfg.unused_tensors = [n for n in names if n in shapes]
        return cfg

    # ------------------------------------------------------------ translation
    def _mixer(self, i: int, layer: dict) -> PartSpec:
        m, p, E = layer["mixer"], f"l{i}.mix.", self.width
        if layer["type"] == "mamba2":
            names = {k: p + k for k in ("in", "conv", "dt_bias", "A_log", "D", "norm", "o")}
            names["conv_bias"] = p + "conv.b"
            return PartSpec("state_space_duality",
                            {"hidden_size": E, "num_heads": m["heads"], "groups": m["groups"],
                             "state_size": m["state"], "value_dim": m["vdim"], "conv": m["conv"],
                             "norm_groups": m["norm_groups"], "eps": self.eps}, names)
        if layer["type"] == "mlstm":
            names = {k: p + k for k in ("q", "k", "v", "g", "o", "norm", "i", "f")}
            names.update(i_bias=p + "i.b", f_bias=p + "f.b")
            return PartSpec("matrix_memory",
                            {"hidden_size": E, "num_heads": m["heads"], "key_dim": m["dim"],
                             "value_dim": m["vdim"], "gate_cap": float(m["gate_cap"]), "eps": self.eps}, names)
        names = {k: p + k for k in ("q", "k", "v", "g", "o")}
        names.update(q_norm=p + "q.norm", k_norm=p + "k.norm")
        role = None
        if m.get("v_mix"):
            role = "source" if i == self.first_mixing_layer() else "mixed"
            if role == "mixed":
                names["value_mix"] = p + "vmix"
        return PartSpec("gated_attention",
                        {"hidden_size": E, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
                         "key_dim": m["dim"], "value_dim": m["vdim"], "softmax_scale": float(m["scale"]),
                         "chunk": int((m.get("mask") or {}).get("size", 0)), "slope_power": SLOPE_POWER,
                         "qk_norm": True, "eps": self.eps, "value_mix": role, "gate": True}, names)

    def to_spec(self) -> ModelSpec:
        E, V = self.width, self.vocab
        norm = lambda name: PartSpec("rms_norm", {"size": E, "eps": self.eps}, {"weight": name})
        layers = []
        for i, layer in enumerate(self.layers):
            mlp = layer.get("mlp")
            ff = PartSpec("none") if mlp is None else PartSpec(
                "dense_activation", {"hidden_size": E, "intermediate_size": int(mlp["ff"]),
                                     "activation": "gelu_tanh"},
                {"up": f"l{i}.mlp.up", "down": f"l{i}.mlp.down"})
            layers.append(LayerSpec(block="parallel", mixer=self._mixer(i, layer), feed_forward=ff,
                                    mixer_norm=norm(f"l{i}.norm1"),
                                    feed_forward_norm=norm(f"l{i}.norm2") if mlp is not None else None,
                                    position=None))
        return ModelSpec(
            architecture=self.architecture, vocab_size=V, hidden_size=E, max_positions=self.max_positions,
            embedding=PartSpec("token_pair_embedding",
                               {"vocab_size": V, "hidden_size": E, "scale": self.embedding_scale,
                                "buckets": self.buckets, "mul_prev": self.mul_prev, "mul_cur": self.mul_cur,
                                "positions": self.max_positions},
                               {"weight": "embed", "pairs": "bigram", "places": "pos"}),
            layers=layers,
            schedule=[ScheduleEntry(layer=i, cache_line=i) for i in range(len(layers))],
            final_norm=norm("final.norm"),
            head=PartSpec("lm_head", {"hidden_size": E, "vocab_size": V}, {"weight": "embed"}),
            bos_token_id=None, eos_token_ids=[], ignored_tensor_suffixes=list(self.unused_tensors))
