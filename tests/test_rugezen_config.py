"""The Rugezen configuration, its run order, its ModelSpec and the oracle's own consistency (CPU)."""

from __future__ import annotations

import json

import pytest
import torch

from tests.helpers import prompt, rugezen_configs
from tests.plain import rugezen as plain
from tinyserve_llm_amd.config.llama import ConfigError
from tinyserve_llm_amd.config.rugezen import RugezenConfig
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.models.registry import read_config, resolve
from tinyserve_llm_amd.weights.random_init import write_random_model


def test_round_trip_and_registry(tmp_path):
    for name, (config, seed) in rugezen_configs().items():
        folder = write_random_model(str(tmp_path / name), config, seed, torch.bfloat16)
        arch, back = read_config(folder)
        assert arch.name == "Rugezen" and back == config
        raw = json.load(open(f"{folder}/config.json"))
        assert raw["architecture"] == "Rugezen" and resolve(raw) is arch
        assert RugezenConfig.from_dict(raw).to_dict() == {k: v for k, v in raw.items() if k not in ("architectures", "model_type")}


def test_run_order_and_plans():
    P, Q = (rugezen_configs()[k][0] for k in "PQ")
    assert P.run_order() == [0, 1, 0, 1, 0, 1, 2] and Q.run_order() == [0, 1, 2, 3]
    model = DecoderModel(__import__("tinyserve_llm_amd.models.rugezen", fromlist=["x"]).rugezen_spec(P))
    # every pass of the looped stretch has a cache or a state of its own
    assert [e.owner for e in model.cache_plan()] == [1, 3, 5, 6]
    assert [e.run for e in model.state_plan()] == [0, 2, 4]
    assert model.cache_plan()[0].kv.v_dim == 48 and model.cache_plan()[0].kv.head_dim == 32
    assert model.cache_plan()[-1].kv.v_dim == 8
    assert model.spec.max_position is None and model.spec.residual_dtype == "float32"
    # a layer without feed-forward declares no second norm and no feed-forward tensors
    names = set(model.spec.checkpoint)
    assert "l2.norm1" in names and "l2.norm2" not in names and not any(n.startswith("l2.mlp") for n in names)
    assert {"l0.mix.z", "l0.mix.z.b", "l0.mix.x", "l0.mix.x.b", "l0.mix.g", "l0.mix.o", "l1.mix.q", "l1.mix.k", "l1.mix.v",
            "l1.mix.o", "l1.mlp.up", "l1.mlp.up.b", "l1.mlp.down", "l1.mlp.down.b", "embed", "head", "final.norm"} <= names


def test_loop_absent_or_single_pass():
    P = rugezen_configs()["P"][0]
    raw = P.to_dict()
    raw["loop"] = None
    assert RugezenConfig.from_dict(raw).run_order() == [0, 1, 2]
    raw["loop"] = {"start": 1, "stop": 3, "times": 1}
    assert RugezenConfig.from_dict(raw).run_order() == [0, 1, 2]
    raw["loop"] = {"start": 2, "stop": 3, "times": 2}
    assert RugezenConfig.from_dict(raw).run_order() == [0, 1, 2, 2]


@pytest.mark.parametrize("spoil, key", [
    (lambda r: r["layers"][1]["mixer"].pop("vdim"), "vdim"),
    (lambda r: r["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda r: r["layers"][0].update(type="lstm"), "type"),
    (lambda r: r.update(loop={"start": 2, "stop": 1, "times": 2}), "loop"),
    (lambda r: r.pop("residual_mult"), "residual_mult"),
])
def test_bad_configurations_name_the_key(spoil, key):
    raw = rugezen_configs()["P"][0].to_dict()
    spoil(raw)
    with pytest.raises(ConfigError, match=key.replace(".", r"\.")):
        RugezenConfig.from_dict(raw)


def test_oracle_prefix_property(tmp_path):
    """The oracle itself: logits at a position do not depend on what follows it, and the recurrence
    carried by hand over two portions equals the whole."""
    config, seed = rugezen_configs()["P"]
    folder = write_random_model(str(tmp_path / "m"), config, seed, torch.bfloat16)
    m = plain.PlainRugezen(folder)
    ids = prompt(5, 40, config.vocab)
    whole = m.logits(ids)
    assert torch.allclose(m.logits(ids[:17]), whole[:17], atol=1e-12)
    z, x, g = (torch.randn(30, 9, dtype=torch.float64) for _ in range(3))
    rows, last = plain.mingru_walk(z, x, g, torch.zeros(9, dtype=torch.float64))
    r1, s1 = plain.mingru_walk(z[:11], x[:11], g[:11], torch.zeros(9, dtype=torch.float64))
    r2, s2 = plain.mingru_walk(z[11:], x[11:], g[11:], s1)
    assert torch.allclose(torch.cat([r1, r2]), rows, atol=1e-14) and torch.allclose(s2, last, atol=1e-14)


def test_oracle_mechanisms_by_hand():
    # one pair turned by a quarter turn: position 1, frequency pi/2 is not reachable through base, so take base 1 (a = p)
    x = torch.tensor([[[1.0, 0.0, 5.0, 7.0]]], dtype=torch.float64)
    out = plain.turn_pairs(x, torch.tensor([2]), 2, 1.0)
    c, s = torch.cos(torch.tensor(2.0, dtype=torch.float64)), torch.sin(torch.tensor(2.0, dtype=torch.float64))
    assert torch.allclose(out[0, 0], torch.stack([c, s, torch.tensor(5.0, dtype=torch.float64), torch.tensor(7.0, dtype=torch.float64)]))
    # a single key of score 0: the sink halves its weight
    q = torch.zeros(1, 1, 4, dtype=torch.float64)
    k = torch.ones(1, 1, 4, dtype=torch.float64)
    v = torch.full((1, 1, 3), 6.0, dtype=torch.float64)
    assert torch.allclose(plain.sink_attention(q, k, v, torch.tensor([0]), 1.0), torch.full((1, 1, 3), 3.0, dtype=torch.float64))
    assert torch.allclose(plain.sink_attention(q, k, v, torch.tensor([0]), 1.0, sink=False), v)
    # the cap bounds a large score: two keys with raw scores 100 and 0, cap 1 -> weights e / (1 + e + 1), 1 / (2 + e)
    q = torch.tensor([[[10.0]]], dtype=torch.float64)
    k = torch.tensor([[[10.0]], [[0.0]]], dtype=torch.float64)
    v = torch.tensor([[[1.0]], [[0.0]]], dtype=torch.float64)
    e = torch.exp(torch.tanh(torch.tensor(100.0, dtype=torch.float64)))
    assert torch.allclose(plain.sink_attention(q, k, v, torch.tensor([1]), 1.0, softcap=1.0)[0, 0, 0], e / (2 + e))
    # the candidate's two branches meet neither in value nor in slope at 0: 1/2 on both sides
    rows, S = plain.mingru_walk(torch.tensor([[100.0]], dtype=torch.float64), torch.tensor([[0.0]], dtype=torch.float64),
                                torch.tensor([[100.0]], dtype=torch.float64), torch.zeros(1, dtype=torch.float64))
    assert abs(float(S) - 0.5) < 1e-12 and abs(float(rows) - 50.0) < 1e-9
