"""The Fanotar configuration and model description on the CPU: config.json round trip, errors that name
the key, run order and cache and state plans with shared caches, the checkpoint table against the
tensors a model folder holds, and the plain implementation's own mechanisms worked out by hand."""

from __future__ import annotations

import json
import math

import pytest
import torch

from tests.helpers import fanotar_configs, prompt
from tests.plain import fanotar as plain
from tinyserve_llm_amd.config.fanotar import FanotarConfig
from tinyserve_llm_amd.config.llama import ConfigError
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.models.registry import architecture_of, read_config, resolve
from tinyserve_llm_amd.weights.random_init import write_random_model

F64 = torch.float64


@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_round_trip_through_config_json(name, tmp_path):
    config, seed = fanotar_configs()[name]
    raw = json.loads(json.dumps(architecture_of(config).to_dict(config)))
    assert raw["architecture"] == "Fanotar" and resolve(raw).name == "Fanotar"
    assert FanotarConfig.from_dict(raw) == config
    write_random_model(str(tmp_path), config, seed, torch.bfloat16)
    arch, again = read_config(str(tmp_path))
    assert arch.name == "Fanotar" and again == config


def test_errors_name_the_key():
    config, _ = fanotar_configs()["P"]
    raw = architecture_of(config).to_dict(config)
    def broken(edit):
        r = json.loads(json.dumps(raw))
        edit(r)
        return r
    for edit, word in ((lambda r: r.pop("vocab"), "vocab"), (lambda r: r["layers"][0]["mixer"].pop("conv"), "conv"),
                       (lambda r: r["layers"][0]["mixer"].update(kv_heads=3), "kv_heads"),
                       (lambda r: r["layers"][1]["mixer"].update(kv_from=1), "kv_from"),
                       (lambda r: r["layers"][1]["mixer"].update(kv_from=0, vdim=8), "kv_from"),
                       (lambda r: r["layers"][1]["mlp"]["router"].update(top=9), "top"),
                       (lambda r: r["layers"][0]["mlp"].update(kind="other"), "kind"),
                       (lambda r: r["layers"][0].update(type="mingru"), "type"),
                       (lambda r: r["layers"][0]["mixer"]["mask"].update(size=0), "mask")):
        with pytest.raises(ConfigError, match=word):
            FanotarConfig.from_dict(broken(edit))


def test_plans_of_layers_that_share_a_cache():
    config, _ = fanotar_configs()["P"]
    model = DecoderModel(architecture_of(config).build_spec(config))
    order = model.spec.order
    assert [(r.layer, r.cache, r.store) for r in order] == [(0, None, True), (1, 0, False), (2, None, True)]
    plan = model.cache_plan()
    # layer 0 keeps its keys for the wider window of the layer that reads them; layer 2 keeps every key
    assert [(e.owner, e.kv.window, e.kv.num_kv_heads, e.kv.head_dim, e.kv.v_dim) for e in plan] == [(0, 50, 2, 32, 48), (2, 0, 1, 24, 8)]
    # state: the last taps - 1 projected rows of q | k | v (q alone for the reader); none for a single tap
    assert [(e.run, tuple(e.state.shape)) for e in model.state_plan()] == [(0, (2, 4 * 32 + 2 * 32 + 2 * 48)), (1, (1, 4 * 32))]
    assert model.graph_safe()
    config_q, _ = fanotar_configs()["Q"]
    model_q = DecoderModel(architecture_of(config_q).build_spec(config_q))
    assert [(e.owner, e.kv.window) for e in model_q.cache_plan()] == [(0, 1), (1, 70)]


def test_checkpoint_names_and_shapes(tmp_path):
    from safetensors import safe_open
    config, seed = fanotar_configs()["P"]
    write_random_model(str(tmp_path), config, seed, torch.bfloat16)
    with safe_open(str(tmp_path / "model.safetensors"), "pt", "cpu") as f:
        shapes = {k: tuple(f.get_slice(k).get_shape()) for k in f.keys()}
    assert shapes["embed"] == (200, 80) and shapes["embed.norm.alpha"] == () and shapes["final.norm.b"] == (80,)
    assert shapes["l0.mix.q"] == (128, 80) and shapes["l0.mix.v.conv"] == (96, 3) and shapes["l0.mix.k.norm"] == (32,)
    assert shapes["l0.mix.g"] == (192, 80) and shapes["l0.mix.o"] == (80, 192) and shapes["l0.mix.sink"] == (4,)
    assert "l1.mix.k" not in shapes and "l1.mix.k.norm" not in shapes and shapes["l1.mix.q.conv"] == (128, 2)
    assert shapes["l1.mlp.e5.gate"] == (40, 80) and shapes["l1.mlp.e0.down"] == (80, 40) and shapes["l1.mlp.router"] == (6, 80)
    assert shapes["l1.mlp.correction"] == (6,) and shapes["l1.mlp.shared.up"] == (24, 80)
    assert shapes["l0.mlp.gate"] == (96, 80) and "l2.norm2" not in shapes and "l2.mlp.gate" not in shapes
    # the loader puts every tensor back where the writer took it from
    from tinyserve_llm_amd.weights.loader import load_params
    model = DecoderModel(architecture_of(config).build_spec(config))
    params = load_params(model, str(tmp_path), torch.bfloat16, "cpu")
    with safe_open(str(tmp_path / "model.safetensors"), "pt", "cpu") as f:
        assert torch.equal(params["layers.1.ff.gate_up"][4, 40:], f.get_tensor("l1.mlp.e4.up"))
        assert torch.equal(params["layers.0.mixer.proj"][128:192], f.get_tensor("l0.mix.k"))
        assert torch.equal(params["layers.0.mixer.conv"][192:], f.get_tensor("l0.mix.v.conv").float())
        assert torch.equal(params["embed.norm_alpha"], f.get_tensor("embed.norm.alpha"))


# ---- the plain implementation's mechanisms by hand ------------------------------------------------

def test_short_convolution_by_hand():
    u = torch.tensor([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0]], dtype=F64)
    w = torch.tensor([[0.5, 0.25, 1.0], [0.0, 1.0, -1.0]], dtype=F64)       # taps: two back, one back, now
    y = plain.short_convolution(u, w)
    assert y.tolist() == [[1.0, -10.0], [2.25, -10.0], [4.0, -10.0]]
    # a portion that starts where another ended gives the same rows
    tail = plain.short_convolution(u[1:], w, before=torch.stack([torch.zeros(2, dtype=F64), u[0]]))
    assert torch.equal(tail, y[1:])


def test_query_multiplier_steps_at_multiples_of_its_period():
    m = plain.query_multiplier(torch.tensor([0, 6, 7, 14, 15], dtype=F64), 0.5, 8)
    assert m.tolist() == pytest.approx([1.0, 1.0, 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(3)])


def test_sink_window_and_slopes_by_hand():
    # one head, keys that all score 0, values 1, 2, 3, ...: the weights are exp(-slope * distance) over the window and the sink
    n, window = 6, 3
    q = torch.zeros(n, 1, 2, dtype=F64)
    k = torch.zeros(n, 1, 2, dtype=F64)
    v = torch.arange(1, n + 1, dtype=F64).view(n, 1, 1)
    sink = torch.tensor([math.log(2.0)], dtype=F64)
    out = plain.sloped_sink_attention(q, k, v, torch.arange(n), 1.0, [math.log(2.0)], sink, window)
    # position 5 sees 3, 4, 5 with weights 1/4, 1/2, 1 over 2 + 1.75
    assert float(out[5, 0, 0]) == pytest.approx((4 * 0.25 + 5 * 0.5 + 6) / 3.75)
    assert float(out[0, 0, 0]) == pytest.approx(1 / 3.0)                      # the first token: itself and the sink
    assert plain.distance_slopes(4) == [0.25, 0.0625, 0.015625, 0.00390625]


def test_router_and_capped_unit_by_hand():
    z = torch.tensor([[0.0, 2.0, 1.0, -1.0]], dtype=F64)
    corr = torch.tensor([0.0, -10.0, 0.0, 0.6], dtype=F64)                  # pushes the best expert out and the worst in
    chosen, w = plain.route(z, corr, 2, 3.0)
    s = torch.sigmoid(z[0])
    assert sorted(chosen[0].tolist()) == [2, 3]
    by = dict(zip(chosen[0].tolist(), w[0].tolist()))
    assert by[2] == pytest.approx(3.0 * float(s[2] / (s[2] + s[3]))) and by[3] == pytest.approx(3.0 * float(s[3] / (s[2] + s[3])))
    y = plain.capped_gated_unit(torch.tensor([5.0, -5.0, 1.0], dtype=F64), torch.tensor([9.0, -9.0, 0.5], dtype=F64), 2.0)
    sg = lambda g: g / (1 + math.exp(-1.702 * g))
    assert y.tolist() == pytest.approx([sg(2.0) * 3.0, sg(-5.0) * -1.0, sg(1.0) * 1.5])


def test_prefix_property_of_the_plain_model(tmp_path):
    config, seed = fanotar_configs()["Q"]
    write_random_model(str(tmp_path), config, seed, torch.bfloat16)
    oracle = plain.PlainFanotar(str(tmp_path))
    p = prompt(5, 40, config.vocab)
    torch.testing.assert_close(oracle.logits(p)[:25], oracle.logits(p[:25]), atol=1e-10, rtol=0)
