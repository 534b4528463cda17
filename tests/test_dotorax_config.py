"""Dotorax's configuration: keys, checks, the translation into parts, the schedule with shared
cache lines, sizes taken from a folder's tensors, and the round trip through config.json."""
import copy

import pytest

import inferllm_amd as I
from inferllm_amd.config.registry import ConfigError
from inferllm_amd.engine import DecoderModel
from dotorax_tiny import CONFIGS, MIXED, ODD


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_round_trip_and_spec(name):
    cfg = I.config_from_dict(CONFIGS[name])
    assert type(cfg).__name__ == "DotoraxConfig"
    assert I.config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    spec = cfg.to_spec()
    assert len(spec.layers) == len(CONFIGS[name]["layers"])
    assert all(l.block == "sandwich" for l in spec.layers)
    DecoderModel(spec)


def test_layers_that_read_an_earlier_layers_keys_share_its_cache_line():
    spec = I.config_from_dict(ODD).to_spec()
    lines = [(e.layer, e.cache_line, e.writes_cache) for e in spec.schedule]
    assert lines == [(0, 0, True), (1, 1, True), (2, 2, True), (3, 1, False), (4, 1, False)]
    model = DecoderModel(spec)
    wants = model.wants()
    assert "l1.mix.k" in wants and "l3.mix.k" not in wants and "l4.mix.v" not in wants
    assert wants["l3.mix.g"].shape == (10, ODD["width"])                 # one gate a head
    assert "l1.norm2" not in wants and "l1.canon2" not in wants          # no feed-forward there
    assert sorted(model.kv_lines()) == [1, 2]
    # the arrangement's own state (what its input convolutions still need) is kept per run, so
    # the runs that share line 1 do not share it
    states = model.state_lines()
    assert {("block", i) for i in range(5)} <= set(states) and 0 in states and 2 in states


def test_pooled_window_keeps_pooled_rows_beside_the_tokens():
    model = DecoderModel(I.config_from_dict(MIXED).to_spec())
    spec = model.kv_lines()[2]
    assert [t.name for t in spec.tensors] == ["k", "v", "kp", "vp"] and spec.kind == "full"


def test_rank_comes_from_the_folders_tensors():
    d = copy.deepcopy(MIXED)
    del d["layers"][1]["mixer"]["rank"]
    cfg = I.config_from_dict(d).with_tensor_shapes({"l1.mix.a1": (7, 80), "l2.norm2": (80,)})
    assert cfg.layers[1]["mixer"]["rank"] == 7
    assert cfg.unused_tensors == ["l2.norm2"]
    assert DecoderModel(cfg.to_spec()).wants()["l1.mix.a2"].shape == (3 * 16, 7)


@pytest.mark.parametrize("edit, message", [
    (lambda d: d["layers"][3]["mixer"].update(kv_from=3), "earlier layer"),
    (lambda d: d["layers"][3]["mixer"].update(kv_from=1), "no keys and values"),
    (lambda d: d["layers"][3]["mixer"].update(dim=24), "must equal"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=22), "even and at most"),
    (lambda d: d["layers"][2]["mixer"]["right"].update(blocks=5), "multiple of blocks"),
    (lambda d: d["layers"][2]["mixer"]["left"].pop("mask"), "lacks"),
    (lambda d: d["layers"][1].update(type="rnn"), "not a mixer"),
    (lambda d: d.pop("residual_mult"), "lacks"),
    (lambda d: d["canon"].update(taps=9), "up to 8"),
])
def test_bad_configurations_are_refused(edit, message):
    d = copy.deepcopy(MIXED)
    edit(d)
    with pytest.raises(ConfigError, match=message):
        I.config_from_dict(d)
