"""Sabipel's configuration: its keys, their checks, the translation into parts, tensor names."""
import copy

import pytest

import inferllm_amd as I
from inferllm_amd.config.registry import ConfigError
from inferllm_amd.engine.model import expected_tensors
from sabipel_tiny import MIXED, NO_KEYS, ODD


def test_round_trip_and_registry():
    cfg = I.config_from_dict(MIXED)
    assert type(cfg).__name__ == "SabipelConfig" and cfg.to_dict() == MIXED
    assert I.config_from_dict(cfg.to_dict()).to_dict() == MIXED
    assert "Sabipel" in I.registered_architectures() if hasattr(I, "registered_architectures") else True


def test_parts_and_constants_come_from_the_configuration():
    spec = I.config_from_dict(MIXED).to_spec()
    kinds = [l.mixer.kind for l in spec.layers]
    assert kinds == ["gated_attention", "matrix_memory", "state_space_duality", "gated_attention",
                     "gated_attention", "state_space_duality"]
    a0, a3, a4 = (spec.layers[i].mixer.params for i in (0, 3, 4))
    assert (a0["chunk"], a3["chunk"], a4["chunk"]) == (37, 50, 0)
    assert (a0["value_mix"], a3["value_mix"], a4["value_mix"]) == ("source", "mixed", None)
    assert a0["softmax_scale"] == 0.2 and a0["num_kv_heads"] == 2 and a0["value_dim"] == 12
    assert spec.layers[1].mixer.params["gate_cap"] == 9.0
    assert spec.layers[2].feed_forward.kind == "none" and spec.layers[2].feed_forward_norm is None
    assert spec.layers[0].feed_forward.params == {"hidden_size": 80, "intermediate_size": 112,
                                                  "activation": "gelu_tanh"}
    assert all(l.block == "parallel" for l in spec.layers)
    e = spec.embedding.params
    assert (e["scale"], e["buckets"], e["mul_prev"], e["mul_cur"], e["positions"]) == (5.5, 97, 13, 5, 512)
    assert spec.head.tensors["weight"] == "embed" and spec.max_positions == 512


def test_tensor_names_and_shapes():
    t = expected_tensors(I.config_from_dict(MIXED).to_spec())
    shape = lambda n: tuple(t[n].shape)
    assert shape("embed") == (310, 80) and shape("bigram") == (98, 80) and shape("pos") == (512, 80)
    assert shape("l0.mix.q") == (120, 80) and shape("l0.mix.k") == (40, 80) and shape("l0.mix.v") == (24, 80)
    assert shape("l0.mix.q.norm") == (120,) and shape("l0.mix.k.norm") == (40,) and shape("l0.mix.g") == (72, 80)
    assert "l0.mix.vmix" not in t and shape("l3.mix.vmix") == () and "l4.mix.vmix" not in t
    assert shape("l1.mix.i") == (3, 80) and shape("l1.mix.f.b") == (3,) and shape("l1.mix.norm") == (84,)
    assert shape("l2.mix.in") == (2 * 96 + 2 * 20 + 4, 80) and shape("l2.mix.conv") == (136, 4)
    assert shape("l2.mix.conv.b") == (136,) and shape("l2.mix.norm") == (96,) and "l2.norm2" not in t
    assert shape("l5.mix.in") == (2 * 60 + 2 * 72 + 6, 80) and shape("l5.mlp.up") == (64, 80)


def test_cache_needs():
    from inferllm_amd.engine import DecoderModel
    m = DecoderModel(I.config_from_dict(NO_KEYS).to_spec())
    assert m.kv_lines() == {} and set(m.state_lines()) == {"embedding", 0, 1, 2}
    m = DecoderModel(I.config_from_dict(ODD).to_spec())
    assert set(m.kv_lines()) == {1, 3, 4} and set(m.state_lines()) == {"embedding", 0, 2}
    assert m.state_lines()[0]["S"].shape == (2, 40, 13) and m.state_lines()[2]["tail"].shape == (4, 42 + 2 * 108)
    assert not m.one_token_mixers


@pytest.mark.parametrize("path, value, needle", [
    (("layers", 0, "type"), "conv", "not a mixer"),
    (("layers", 0, "mixer", "kv_heads"), 4, "multiple"),
    (("layers", 2, "mixer", "norm_groups"), 5, "norm_groups"),
    (("layers", 2, "mixer", "groups"), 3, "multiple"),
    (("layers", 3, "mixer", "vdim"), 7, "v_mix"),
    (("layers", 1, "mixer", "gate_cap"), 0, "gate_cap"),
    (("layers", 0, "mlp", "kind"), "moe", "feed-forward"),
    (("embedding", "bigram", "buckets"), 0, "buckets"),
    (("norm", "eps"), -1.0, "eps"),
])
def test_bad_values_are_refused(path, value, needle):
    d = copy.deepcopy(MIXED)
    at = d
    for k in path[:-1]:
        at = at[k]
    at[path[-1]] = value
    with pytest.raises(ConfigError, match=needle):
        I.config_from_dict(d)


@pytest.mark.parametrize("key", ["vocab", "width", "max_positions", "norm", "embedding", "layers"])
def test_missing_keys_are_named(key):
    d = copy.deepcopy(ODD)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        I.config_from_dict(d)
