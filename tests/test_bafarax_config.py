"""The Bafarax configuration and model description on the CPU: config.json round trip, errors that name
the key, the run order, cache and state plans of layers that run with another layer's weights, the
checkpoint table against the tensors a model folder holds, and the plain implementation's own
mechanisms worked out by hand."""

from __future__ import annotations

import json
import math

import pytest
import torch

from tests.helpers import bafarax_configs, prompt
from tests.plain import bafarax as plain
from tinyserve_llm_amd.config.bafarax import BafaraxConfig
from tinyserve_llm_amd.config.llama import ConfigError
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.models.registry import architecture_of, read_config, resolve
from tinyserve_llm_amd.weights.random_init import write_random_model

F64 = torch.float64


@pytest.mark.parametrize("name", ["P", "Q", "R", "S"])
def test_round_trip_through_config_json(name, tmp_path):
    config, seed = bafarax_configs()[name]
    raw = json.loads(json.dumps(architecture_of(config).to_dict(config)))
    assert raw["architecture"] == "Bafarax" and resolve(raw).name == "Bafarax"
    assert BafaraxConfig.from_dict(raw) == config
    write_random_model(str(tmp_path), config, seed, torch.bfloat16)
    arch, again = read_config(str(tmp_path))
    assert arch.name == "Bafarax" and again == config


def test_errors_name_the_key():
    config, _ = bafarax_configs()["P"]
    raw = architecture_of(config).to_dict(config)

    def broken(edit):
        r = json.loads(json.dumps(raw))
        edit(r)
        return r
    for edit, word in ((lambda r: r.pop("vocab"), "vocab"), (lambda r: r["norm"].pop("eps"), "eps"),
                       (lambda r: r["layers"][0]["mixer"].pop("gate_cap"), "gate_cap"),
                       (lambda r: r["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
                       (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=34), "rot"),
                       (lambda r: r["layers"][1]["mixer"]["mask"].update(size=0), "mask"),
                       (lambda r: r["layers"][2]["mixer"].pop("kv_rank"), "kv_rank"),
                       (lambda r: r["layers"][2]["mixer"]["rot"].update(dims=4), "rot.dims"),
                       (lambda r: r["layers"][2]["mixer"]["rot"]["scaling"].pop("slow"), "slow"),
                       (lambda r: r["layers"][1]["mlp"]["router"].update(top=7), "top"),
                       (lambda r: r["layers"][0]["mlp"].update(kind="other"), "kind"),
                       (lambda r: r["layers"][0].update(type="mingru"), "type"),
                       (lambda r: r["layers"][3].update(weights_of=3), "weights_of"),
                       (lambda r: r["layers"][3].update(weights_of=2), "weights_of"),
                       (lambda r: r["layers"][3]["mixer"].update(scale=0.5), "weights_of")):
        with pytest.raises(ConfigError, match=word):
            BafaraxConfig.from_dict(broken(edit))


def test_optional_keys_have_their_defaults():
    config, _ = bafarax_configs()["Q"]
    raw = architecture_of(config).to_dict(config)
    raw.pop("embedding")
    assert BafaraxConfig.from_dict(raw).embedding_scale == 1.0
    last = raw["layers"][-1]["mixer"]
    assert "mask" not in last and "rot" not in last, "attention over everything before, nothing turns"
    assert BafaraxConfig.from_dict(raw).layers[-1].mixer.chunk == 0


def test_plans_of_layers_that_run_with_another_layers_weights():
    config, _ = bafarax_configs()["Q"]
    model = DecoderModel(architecture_of(config).build_spec(config))
    # six runs over four sets of weights: the mLSTM twice in a row, then the latent layer again
    assert [r.layer for r in model.spec.order] == [0, 1, 2, 2, 1, 3] and len(model.layers) == 4
    assert all(r.cache is None and r.store for r in model.spec.order), "every run keeps a cache or state of its own"
    plan = model.cache_plan()
    # chunks of one position; the latent's rows (latent and shared key part; the latent once more as the values) for its
    # window, once per run; and a layer that sees everything
    assert [(e.owner, e.kv.window, e.kv.num_kv_heads, e.kv.head_dim, e.kv.v_dim) for e in plan] == \
        [(0, 1, 2, 16, 16), (1, 70, 1, 32, 16), (4, 70, 1, 32, 16), (5, 0, 1, 8, 24)]
    # per head S [dim, vdim], n [dim] and m, for each of the two runs
    assert [(e.run, tuple(e.state.shape)) for e in model.state_plan()] == [(2, (16 * 16 + 16 + 1,)), (3, (16 * 16 + 16 + 1,))]
    assert model.graph_safe()
    config_p, _ = bafarax_configs()["P"]
    model_p = DecoderModel(architecture_of(config_p).build_spec(config_p))
    assert [(e.owner, e.kv.window) for e in model_p.cache_plan()] == [(1, 24), (2, 50), (3, 24)]
    assert [(e.run, tuple(e.state.shape)) for e in model_p.state_plan()] == [(0, (3 * (20 * 28 + 20 + 1),))]


def test_checkpoint_names_and_shapes(tmp_path):
    from safetensors import safe_open
    config, seed = bafarax_configs()["P"]
    write_random_model(str(tmp_path), config, seed, torch.bfloat16)
    with safe_open(str(tmp_path / "model.safetensors"), "pt", "cpu") as f:
        shapes = {k: tuple(f.get_slice(k).get_shape()) for k in f.keys()}
    assert shapes["embed"] == (200, 80) and shapes["head"] == (200, 80) and shapes["final.norm"] == (80,)
    assert shapes["l0.mix.q"] == (60, 80) and shapes["l0.mix.v"] == (84, 80) and shapes["l0.mix.i"] == (3, 80)
    assert shapes["l0.mix.f.b"] == (3,) and shapes["l0.mix.g"] == (84, 80) and shapes["l0.mix.norm"] == (84,)
    assert shapes["l0.mix.o"] == (80, 84) and shapes["l0.mlp.gate"] == (96, 80) and shapes["l0.mlp.down"] == (80, 96)
    assert shapes["l1.mix.q"] == (128, 80) and shapes["l1.mix.k"] == (64, 80) and shapes["l1.mix.v"] == (96, 80)
    assert shapes["l1.mix.q.norm"] == (128,) and shapes["l1.mix.k.norm"] == (64,) and shapes["l1.mix.sink"] == (4,)
    assert shapes["l1.mlp.router"] == (6, 80) and shapes["l1.mlp.e5.up"] == (40, 80) and shapes["l1.mlp.e0.down"] == (80, 40)
    assert shapes["l2.mix.dq"] == (36, 80) and shapes["l2.mix.dq.norm"] == (36,) and shapes["l2.mix.uq"] == (3 * 32, 36)
    assert shapes["l2.mix.dkv"] == (48, 80) and shapes["l2.mix.dkv.norm"] == (40,) and shapes["l2.mix.uk"] == (72, 40)
    assert shapes["l2.mix.uv"] == (60, 40) and shapes["l2.mix.g"] == (60, 80) and shapes["l2.mix.o"] == (80, 60)
    assert "l2.norm2" not in shapes and not any(k.startswith("l3.") for k in shapes), "no feed-forward; no weights of its own"
    # the loader puts every tensor back where the writer took it from
    from tinyserve_llm_amd.weights.loader import load_params
    model = DecoderModel(architecture_of(config).build_spec(config))
    params = load_params(model, str(tmp_path), torch.bfloat16, "cpu")
    with safe_open(str(tmp_path / "model.safetensors"), "pt", "cpu") as f:
        assert torch.equal(params["layers.1.ff.up"][4], f.get_tensor("l1.mlp.e4.up"))
        assert torch.equal(params["layers.1.mixer.qkv"][128:192], f.get_tensor("l1.mix.k"))
        assert torch.equal(params["layers.2.mixer.down"][36:84], f.get_tensor("l2.mix.dkv"))
        assert torch.equal(params["layers.2.mixer.down"][84:], f.get_tensor("l2.mix.g"))
        assert torch.equal(params["layers.0.mixer.proj"][60:120], f.get_tensor("l0.mix.k"))
        assert torch.equal(params["layers.0.mixer.proj"][204:207], f.get_tensor("l0.mix.i"))
        assert torch.equal(params["layers.0.mixer.gate_bias"][3:], f.get_tensor("l0.mix.f.b").float())
        assert torch.equal(params["layers.1.mixer.sinks"], f.get_tensor("l1.mix.sink").float())


def test_the_engines_frequencies_are_the_plain_ones():
    from tinyserve_llm_amd.parts.rope import RotaryFrequencies
    for dims, base, ramp in ((8, 5000.0, dict(factor=3.0, original=64.0, fast=16.0, slow=2.0)), (16, 300.0, None),
                             (6, 2000.0, dict(factor=8.0, original=32.0, fast=4.0, slow=1.0)),
                             (64, 10000.0, dict(factor=40.0, original=4096.0, fast=32.0, slow=1.0))):
        enc = RotaryFrequencies(dims, base, True, ramp)
        f, amp = plain.rotary_frequencies(dims, base, ramp)
        torch.testing.assert_close(enc.host_frequencies(), f, atol=0, rtol=1e-14)
        assert enc.amplitude == pytest.approx(amp, rel=1e-14)


# ---- the plain implementation's mechanisms by hand ------------------------------------------------

def test_frequency_ramp_by_hand():
    # dims 8, base 16: f = 1, 1/2, 1/4, 1/8. original 2 pi 16: d(t) = 8 ln(16 / t) / (2 ln 16) = 4 - log2(t) ... in pairs
    L = 2 * math.pi * 16
    f, amp = plain.rotary_frequencies(8, 16.0, dict(factor=2.0, original=L, fast=8.0, slow=2.0))
    # d(8) = 8 ln 2 / (2 ln 16) = 1, d(2) = 8 ln 8 / (2 ln 16) = 3: pair 0, 1 keep their frequency, pair 2 is half way, pair 3 slowed
    assert f.tolist() == pytest.approx([1.0, 0.5, 0.25 * 0.75, 0.125 / 2])
    assert amp == pytest.approx(0.1 * math.log(2.0) + 1)
    assert plain.rotary_frequencies(8, 16.0, None)[0].tolist() == pytest.approx([1.0, 0.5, 0.25, 0.125])


def test_the_two_pairings_of_a_rotation():
    x = torch.tensor([[[1.0, 0.0, 0.0, 1.0, 5.0]]], dtype=F64)
    f = torch.tensor([math.pi / 2, math.pi], dtype=F64)
    pos = torch.tensor([1])
    # pairs (0, 1) and (2, 3): (1, 0) a quarter turn -> (0, 1); (0, 1) half a turn -> (0, -1); the rest passes; times 2
    assert plain.rotate(x, pos, f, 2.0, True)[0, 0].tolist() == pytest.approx([0.0, 2.0, 0.0, -2.0, 5.0])
    # pairs (0, 2) and (1, 3): (1, 0) a quarter turn -> (0, 1); (0, 1) half a turn -> (0, -1)
    assert plain.rotate(x, pos, f, 1.0, False)[0, 0].tolist() == pytest.approx([0.0, 0.0, 1.0, -1.0, 5.0])


def test_chunks_windows_and_the_sink_by_hand():
    see = plain.visibility(torch.tensor([0, 2, 3, 5]), 6, "chunk", 3)
    assert see.int().tolist() == [[1, 0, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0], [0, 0, 0, 1, 0, 0], [0, 0, 0, 1, 1, 1]]
    see = plain.visibility(torch.tensor([1, 4]), 6, "window", 3)
    assert see.int().tolist() == [[1, 1, 0, 0, 0, 0], [0, 0, 1, 1, 1, 0]]
    # keys that all score 0, values 1, 2, ...: equal weights over what is seen, and the sink counts as ln 2 -> 2 more
    n = 6
    q, k = torch.zeros(n, 1, 2, dtype=F64), torch.zeros(n, 1, 2, dtype=F64)
    v = torch.arange(1, n + 1, dtype=F64).view(n, 1, 1)
    sink = torch.tensor([math.log(2.0)], dtype=F64)
    out = plain.masked_attention(q, k, v, torch.arange(n), 1.0, "chunk", 4, sink)
    assert out[:, 0, 0].tolist() == pytest.approx([1 / 3, 3 / 4, 6 / 5, 10 / 6, 5 / 3, 11 / 4])
    out = plain.masked_attention(q, k, v, torch.arange(n), 1.0, "window", 2, None)
    assert out[:, 0, 0].tolist() == pytest.approx([1.0, 1.5, 2.5, 3.5, 4.5, 5.5])


def test_matrix_memory_by_hand():
    # one head, dim 1, vdim 2, every projection picks a coordinate of the input: q = x0 (dim 1: no scaling), k = x1,
    # v = (x2, x3), gates' sums x4 and x5, no output gate to speak of (g = 40 -> sigmoid 1), W_o = identity
    W = {n: torch.zeros(r, 8, dtype=F64) for n, r in (("q", 1), ("k", 1), ("v", 2), ("i", 1), ("f", 1), ("g", 2))}
    W["q"][0, 0] = W["k"][0, 1] = W["v"][0, 2] = W["v"][1, 3] = W["i"][0, 4] = W["f"][0, 5] = 1.0
    W["g"][:, 6] = 40.0
    W.update({"i.b": torch.zeros(1, dtype=F64), "f.b": torch.zeros(1, dtype=F64), "norm": torch.ones(2, dtype=F64), "o": torch.eye(2, dtype=F64)})
    m = dict(heads=1, dim=1, vdim=2, gate_cap=1e6)
    x = torch.tensor([[1.0, 2.0, 3.0, 1.0, math.log(4.0), 0.0, 1.0, 0.0],
                      [1.0, 1.0, 1.0, -5.0, 0.0, 50.0, 1.0, 0.0]], dtype=F64)
    state = {}
    out = plain.mlstm(x, W, m, 0.0, state)
    # token 0: i = ln 4, f = logsigmoid(0) = -ln 2; m = max(-ln 2 + 0, ln 4) = ln 4; S = k v = (6, 2), n = 2
    assert float(state["m"][0]) == pytest.approx(math.log(4.0))
    # (before token 1 is folded in; checked through the first row: o = S q / max(|n q|, 1/4) = (3, 1), then unit rms)
    rms = math.sqrt((9 + 1) / 2)
    assert out[0].tolist() == pytest.approx([3 / rms, 1 / rms], rel=1e-6)
    # token 1: i = 0, f = logsigmoid(50) = 0: m stays ln 4; S = S + (1/4) k v = (6.25, 0.75), n = 2.25
    assert state["S"][0, 0].tolist() == pytest.approx([6.25, 0.75]) and float(state["n"][0, 0]) == pytest.approx(2.25)
    # the cap: a sum far beyond it gives the cap itself
    capped = plain.mlstm(torch.tensor([[1.0, 1.0, 1.0, 1.0, 100.0, 0.0, 1.0, 0.0]], dtype=F64), W, dict(m, gate_cap=3.0), 0.0, s2 := {})
    assert float(s2["m"][0]) == pytest.approx(3.0, abs=1e-9) and capped.shape == (1, 2)
    # a state that starts at m = 0, not at minus infinity: a very negative first input gate keeps m at f + 0
    plain.mlstm(torch.tensor([[1.0, 1.0, 1.0, 1.0, -30.0, 0.0, 1.0, 0.0]], dtype=F64), W, m, 0.0, s3 := {})
    assert float(s3["m"][0]) == pytest.approx(-math.log(2.0))


def test_softmax_over_the_chosen_experts_only():
    z = torch.tensor([[0.0, 2.0, 1.0, -1.0], [5.0, 5.0, -9.0, 4.0]], dtype=F64)
    idx, w = plain.chosen_experts(z, 2)
    assert sorted(idx[0].tolist()) == [1, 2]
    by = dict(zip(idx[0].tolist(), w[0].tolist()))
    assert by[1] == pytest.approx(math.e / (1 + math.e)) and by[2] == pytest.approx(1 / (1 + math.e))
    assert w[1].tolist() == pytest.approx([0.5, 0.5])
    idx, w = plain.chosen_experts(z, 1)
    assert idx[:, 0].tolist()[0] == 1 and w[:, 0].tolist() == [1.0, 1.0]


@pytest.mark.parametrize("name", ["P", "Q"])
def test_prefix_and_portions_of_the_plain_model(name, tmp_path):
    config, seed = bafarax_configs()[name]
    write_random_model(str(tmp_path), config, seed, torch.bfloat16)
    oracle = plain.PlainBafarax.from_folder(str(tmp_path))
    p = prompt(5, 60, config.vocab)
    whole = oracle.logits(p)
    torch.testing.assert_close(whole[:25], oracle.logits(p[:25]), atol=1e-10, rtol=0)
    oracle.reset()
    parts = torch.cat([oracle.forward(p[:7]), oracle.forward(p[7:9]), oracle.forward(p[9:58]), oracle.forward(p[58:59]), oracle.forward(p[59:])])
    torch.testing.assert_close(parts, whole, atol=1e-9, rtol=0)
    # a layer that runs with another's weights keeps a memory of its own: its run sees other rows than the first
    assert len(oracle.after_layers) == len(config.layers)
