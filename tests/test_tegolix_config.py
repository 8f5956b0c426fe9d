"""Tegolix on the CPU: the typed configuration (round trip, optional keys, errors that name the key, sizes that only
the checkpoint's tensors give), the model as data (parts, cache and state plans, the checkpoint table against a folder's
tensors and the loader), and the plain implementation's mechanisms worked out by hand, with its prefix and portion
properties."""

from __future__ import annotations

import json
import math
import os

import pytest
import torch

from tests.helpers import prompt, tegolix_configs
from tests.plain import tegolix as plain
from tinyserve_llm_amd.config import ConfigError
from tinyserve_llm_amd.config.tegolix import TegolixConfig
from tinyserve_llm_amd.models import read_config, resolve
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.models.registry import checkpoint_shapes
from tinyserve_llm_amd.weights.loader import load_params
from tinyserve_llm_amd.weights.random_init import write_random_model

F64 = torch.float64


@pytest.mark.parametrize("name", ["P", "Q", "R", "S", "T"])
def test_configuration_round_trip_and_folder(name, tmp_path):
    config, seed = tegolix_configs()[name]
    raw = config.to_dict()
    assert TegolixConfig.from_dict(json.loads(json.dumps(raw))) == config
    assert resolve(raw).name == "Tegolix"
    folder = write_random_model(str(tmp_path), config, seed, torch.bfloat16)
    arch, back = read_config(folder)
    assert arch.name == "Tegolix" and back == config
    model = DecoderModel(arch.build_spec(back))
    shapes = checkpoint_shapes(folder)
    assert set(shapes) == set(model.spec.checkpoint), "the table names the folder's tensors, all of them and no others"
    params = load_params(model, folder, torch.float32, "cpu")
    assert set(params) == set(model.param_specs())
    # without the ranks in config.json they come from the tensors' shapes
    for layer in raw["layers"]:
        m = layer["mixer"]
        (m.get("right") or m).pop("decay_rank")
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f)
    assert read_config(folder)[1] == config
    # plans: a cache per attention side (with its window), a state per layer
    caches, states = model.cache_plan(), model.state_plan()
    parallel = [i for i, l in enumerate(config.layers) if l.type == "parallel"]
    assert [c.owner for c in caches] == parallel
    for c in caches:
        a = config.layers[c.owner].mixer.left
        assert (c.kv.num_kv_heads, c.kv.head_dim, c.kv.v_dim, c.kv.window) == (a.kv_heads, a.dim, a.vdim, a.window)
    assert [s.run for s in states] == list(range(len(config.layers)))
    for s in states:
        m = config.layers[s.run].mixer
        want = m.heads * m.dim * m.vdim if config.layers[s.run].type == "gla" else m.right.heads * m.right.dim ** 2 + config.width
        assert s.state.shape == (want,) and s.state.dtype == torch.float32
    assert model.graph_safe()


def test_errors_name_the_key_and_optional_keys_may_be_absent():
    config, _ = tegolix_configs()["P"]
    raw = config.to_dict()
    for path, key in ((("layers", 0, "mixer"), "tau"), (("layers", 1, "mixer", "left"), "rot"), (("layers", 1, "mixer"), "left_scale"),
                      (("layers", 1, "mlp", "router"), "top"), ((), "vocab"), (("norm",), "eps")):
        broken = json.loads(json.dumps(raw))
        at = broken
        for step in path:
            at = at[step]
        del at[key]
        with pytest.raises(ConfigError, match=key):
            TegolixConfig.from_dict(broken)
    bad = json.loads(json.dumps(raw))
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ConfigError, match="type"):
        TegolixConfig.from_dict(bad)
    bad = json.loads(json.dumps(raw))
    bad["layers"][1]["mlp"]["router"]["top"] = 9
    with pytest.raises(ConfigError, match="top"):
        TegolixConfig.from_dict(bad)
    lean = json.loads(json.dumps(raw))
    del lean["token_side"], lean["layers"][1]["mixer"]["left"]["mask"], lean["layers"][1]["mixer"]["left"]["softcap"]
    del lean["layers"][1]["mlp"]["shared"], lean["layers"][1]["mlp"]["router"]["identity"], lean["layers"][1]["mixer"]["left"]["rot"]["scaling"]
    c = TegolixConfig.from_dict(lean)
    left, mlp = c.layers[1].mixer.left, c.layers[1].mlp
    assert (c.side_dim, left.window, left.softcap, left.rot.ramp, mlp.shared_ff, mlp.identity) == (0, 0, 0.0, None, 0, 0)
    spec = resolve(lean).build_spec(c)
    assert not spec.layers[1].token_inputs and "side.embed" not in spec.checkpoint


def test_engine_frequencies_equal_the_plain_ones():
    from tinyserve_llm_amd.parts.rope import RotaryFrequencies
    for dims, base, ramp in ((16, 10000.0, dict(factor=3.0, original=64.0, fast=16.0, slow=2.0)), (48, 700.0, None),
                             (10, 50000.0, dict(factor=8.0, original=32.0, fast=4.0, slow=1.0))):
        enc = RotaryFrequencies(dims, base, interleaved=False, ramp=ramp)
        f, amp = plain.rotary_frequencies(dims, base, ramp)
        torch.testing.assert_close(enc.host_frequencies(), f, atol=0, rtol=1e-14)
        assert enc.amplitude == pytest.approx(amp)


def test_plain_mechanisms_by_hand():
    # the window: position 5 with a window of 3 sees 3, 4, 5; equal scores give the mean of their values
    v = torch.arange(8, dtype=F64).reshape(8, 1, 1)
    out = plain.window_attention(torch.zeros(1, 1, 2, dtype=F64), torch.ones(8, 1, 2, dtype=F64), v, torch.tensor([5]), 1.0, 0.0, 3)
    assert float(out) == pytest.approx(4.0)
    # the cap: a score of 100 under a cap of 2 counts as 2 tanh(50) = 2
    k = torch.tensor([[[100.0]], [[0.0]]], dtype=F64)
    out = plain.window_attention(torch.ones(1, 1, 1, dtype=F64), k, torch.tensor([[[1.0]], [[0.0]]], dtype=F64), torch.tensor([1]), 1.0, 2.0, 0)
    assert float(out) == pytest.approx(math.exp(2.0) / (math.exp(2.0) + 1.0))
    # a value turned by its position and the sum turned back: a query that sees only itself gets its value back
    f, _ = plain.rotary_frequencies(4, 100.0, None)
    x = torch.randn(3, 1, 4, dtype=F64)
    pos = torch.tensor([0, 7, 1000])
    torch.testing.assert_close(plain.rotate_halves(plain.rotate_halves(x, pos, f), pos, f, back=True), x)
    assert not torch.allclose(plain.rotate_halves(x, pos, f)[1:], x[1:])
    # identity experts: with every router weight zero the scores are uniform, the correction picks, the input comes back
    h = torch.randn(2, 6, dtype=F64)
    W = {"router": torch.zeros(4, 6, dtype=F64), "correction": torch.tensor([0.0, 0.0, 0.5, 0.4], dtype=F64)}
    for e in range(2):
        W[f"e{e}.gate"], W[f"e{e}.up"], W[f"e{e}.down"] = (torch.randn(3, 6, dtype=F64), torch.randn(3, 6, dtype=F64), torch.randn(6, 3, dtype=F64))
    out = plain.expert_mixture(h, W, {"router": {"experts": 2, "identity": 2, "top": 2}})
    torch.testing.assert_close(out, 0.5 * h)                                   # two identity experts at a quarter each
    idx, w = plain.chosen_experts(torch.tensor([[0.0, 1.0, 2.0]], dtype=F64), torch.tensor([0.0, 0.0, -1.0], dtype=F64), 1)
    s = torch.softmax(torch.tensor([0.0, 1.0, 2.0], dtype=F64), -1)
    assert idx.tolist() == [[1]] and float(w) == pytest.approx(float(s[1])), "the correction chooses, the weight is the score without it"


def test_recurrences_by_hand():
    eps = 0.0
    # gated linear attention, one head of one channel: alpha = sigmoid(b)^(1/tau)
    W = {n: torch.ones(1, 1, dtype=F64) for n in ("q", "k", "v", "g", "o", "a1", "a2")}
    W["a2"] = torch.zeros(1, 1, dtype=F64)
    W["a2.b"], W["norm"] = torch.zeros(1, dtype=F64), torch.ones(1, dtype=F64)
    m = {"heads": 1, "dim": 1, "vdim": 1, "tau": 2.0}
    state = {}
    plain.gated_linear_attention(torch.tensor([[2.0], [3.0]], dtype=F64), W, m, eps, state)
    assert float(state["S"]) == pytest.approx(4.0 * math.sqrt(0.5) + 9.0)
    # the shifted recurrence: the first token's mixes read zeros before it, the bonus is the current token's alone
    W = {n: torch.ones(1, 1, dtype=F64) for n in ("r", "k", "v", "g", "o", "w1")}
    W.update({f"mu.{s}": torch.full((1,), 0.25, dtype=F64) for s in ("r", "k", "v", "g", "w")})
    W["w2"], W["w0"], W["u"], W["norm"] = torch.zeros(1, 1, dtype=F64), torch.zeros(1, dtype=F64), torch.full((1, 1), 0.5, dtype=F64), torch.ones(1, dtype=F64)
    state = {}
    plain.right_recurrence(torch.tensor([[4.0], [8.0]], dtype=F64), W, {"heads": 1, "dim": 1}, eps, state)
    first, second = 4.0 * 0.75, 8.0 + (4.0 - 8.0) * 0.25
    assert float(state["S"]) == pytest.approx(first * first * math.exp(-1.0) + second * second)
    assert float(state["prev"]) == 8.0


@pytest.mark.parametrize("name", ["P", "Q"])
def test_plain_model_in_portions_equals_whole(name, tmp_path):
    config, seed = tegolix_configs()[name]
    folder = write_random_model(str(tmp_path), config, seed, torch.bfloat16)
    oracle = plain.PlainTegolix.from_folder(folder)
    p = prompt(3, 60, config.vocab)
    whole = oracle.logits(p)
    oracle.reset()
    parts = torch.cat([oracle.forward(p[:25]), oracle.forward(p[25:27]), oracle.forward(p[27:28]), oracle.forward(p[28:])])
    torch.testing.assert_close(parts, whole, atol=1e-12, rtol=1e-10)
    assert len(oracle.streams(p)) == len(config.layers)
