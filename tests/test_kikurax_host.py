"""Kikurax on the CPU: properties of the oracle's mechanisms in closed form or in limiting cases (the oracle is what the
GPU tests compare with, so it is checked against arithmetic that does not share its code), the configuration reader, the
registry, the pool shapes and the merges of load_weights.  No kernel runs."""
import json
import math

import torch

from oracle import kikurax as ko
from tests import kikurax_util as U


def test_oracle_is_causal_and_every_mixer_reaches_the_logits():
    cfg = U.full_config()
    w = ko.random_weights(cfg, 3)
    toks = U.tokens(40, cfg["vocab"], 4)
    full = ko.forward(toks, w, cfg)
    assert torch.allclose(ko.forward(toks[:25], w, cfg), full[:25], atol=1e-9)
    other = list(toks)
    other[3] = (other[3] + 1) % cfg["vocab"]
    moved = ko.forward(other, w, cfg)
    assert torch.allclose(moved[:3], full[:3], atol=1e-9) and (moved[39] - full[39]).abs().max() > 1e-6


def test_group_norm_parts_have_unit_mean_square():
    x = torch.randn(5, 24, dtype=torch.float64) * torch.tensor([1.0] * 8 + [30.0] * 8 + [0.01] * 8, dtype=torch.float64)
    y = ko.group_norm(x, torch.ones(24, dtype=torch.float64), 3, 0.0).reshape(5, 3, 8)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, 3, dtype=torch.float64))
    one = ko.group_norm(x, torch.ones(24, dtype=torch.float64), 1, 0.0)
    assert not torch.allclose(one, y.reshape(5, 24))


def test_sink_of_score_zero_in_closed_form():
    """one token: the only key's weight is e^s / (1 + e^s), so the output is sigmoid(s) v"""
    m = U.attention(1, 1, 4, 3, dims=0, softcap=None, scale=0.5)["mixer"]
    W = 4
    w = {"a.q": torch.eye(4, dtype=torch.float64), "a.k": torch.eye(4, dtype=torch.float64),
         "a.v": torch.eye(3, 4, dtype=torch.float64), "a.q.b": torch.zeros(4, dtype=torch.float64),
         "a.k.b": torch.zeros(4, dtype=torch.float64), "a.v.b": torch.zeros(3, dtype=torch.float64),
         "a.temp": torch.tensor([2.0], dtype=torch.float64), "a.o": torch.eye(W, 3, dtype=torch.float64)}
    h = torch.tensor([[1.0, 2.0, -1.0, 0.5]], dtype=torch.float64)
    out, handed = ko.softmax_attention(h, w, "a", m, 0.0, None, True)
    s = 4.0 * 0.5 * 2.0                                   # normed q . normed k = dim; times scale and the head's number
    assert torch.allclose(out[0, :3], torch.sigmoid(torch.tensor(s, dtype=torch.float64)) * h[0, :3])
    assert torch.equal(handed[0, 0], h[0, :3])
    m["softcap"] = 1.5
    out, _ = ko.softmax_attention(h, w, "a", m, 0.0, None, True)
    assert torch.allclose(out[0, :3], torch.sigmoid(torch.tensor(1.5 * math.tanh(s / 1.5), dtype=torch.float64)) * h[0, :3])


def test_sigmoid_attention_weights_are_not_normalised_and_grow_with_the_position():
    m = U.parallel(1, 1, 2, 2, 1, 1, 2, 2, coef=1.0, every=2)["mixer"]["left"]
    z = torch.zeros
    w = {"a.q": torch.eye(2, dtype=torch.float64), "a.k": torch.eye(2, dtype=torch.float64), "a.v": torch.eye(2, dtype=torch.float64),
         "a.g": z(2, 2, dtype=torch.float64), "a.pb": torch.tensor([0.25], dtype=torch.float64), "a.o": torch.eye(2, dtype=torch.float64)}
    h = torch.tensor([[1.0, 1.0]] * 4, dtype=torch.float64)
    out = ko.sigmoid_attention(h, w, "a", m, 0.0)
    # normed q . normed k = 2, scale 2^-1/2; position p multiplies q by 1 + ln(floor((p + 1) / 2) + 1); the gate is 1/2
    for p in range(4):
        mult = 1 + math.log((p + 1) // 2 + 1)
        want = 0.5 * (p + 1) / (1 + math.exp(-(2 * 2 ** -0.5 * mult + 0.25)))
        assert abs(float(out[p, 0]) - want) < 1e-12


def test_delta_rule_returns_a_stored_value_and_forgets_by_channel():
    """with beta = 1 and no decay a key reads back its value exactly; a decayed channel returns less"""
    D, Dv = 4, 3
    S = torch.zeros(D, Dv, dtype=torch.float64)
    k = torch.tensor([1.0, 0.0, 0.0, 0.0], dtype=torch.float64)
    v = torch.tensor([2.0, -1.0, 0.5], dtype=torch.float64)
    u = 1.0 * (v - S.T @ k)
    S = S + torch.outer(k, u)
    assert torch.allclose(S.T @ k, v)
    u = 1.0 * (v - S.T @ k)                               # writing the same pair again changes nothing
    assert torch.allclose(S + torch.outer(k, u), S)
    g = torch.tensor([0.5, 1.0, 1.0, 1.0], dtype=torch.float64)
    assert torch.allclose((g[:, None] * S).T @ k, 0.5 * v)


def test_router_weights_are_the_softmax_over_the_chosen_logits():
    w = {"r.router": torch.tensor([[1.0], [3.0], [2.0], [-1.0]], dtype=torch.float64),
         "r.router.b": torch.tensor([0.0, 0.0, 2.0, 0.0], dtype=torch.float64)}
    ids, wt = ko.route(torch.tensor([[1.0]], dtype=torch.float64), w, "r", 2)
    assert ids.tolist() == [[2, 1]]
    assert torch.allclose(wt, torch.tensor([[math.e / (1 + math.e), 1 / (1 + math.e)]], dtype=torch.float64))


def test_frequency_rule_matches_the_products():
    from scratchpad_amd.layers import wavelength_blend
    for rot in ({"dims": 16, "base": 500.0, "scaling": {"factor": 3.0, "low": 1.0, "high": 3.0, "original": 40}},
                {"dims": 24, "base": 10000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}):
        sc = rot["scaling"]
        got = wavelength_blend(rot["dims"], rot["base"], sc["factor"], sc["original"], sc["low"], sc["high"])
        assert torch.allclose(got, ko.rotary_frequencies(rot), rtol=1e-12)


def test_configuration_registry_and_pool_shapes(tmp_path):
    from scratchpad_amd import registry
    raw = U.full_config()
    folder, _ = U.make_model(tmp_path, raw, seed=1, rank_a=5, rank_g=7)
    cfg = registry.load_config(folder, context_len=128)
    assert type(cfg).__name__ == "KikuraxConfig" and registry.model_class_for(cfg).__name__ == "KikuraxForCausalLM"
    assert cfg.norm_groups == 3 and cfg.embedding_scale == 3.0 and cfg.v_first_layer == 1
    assert cfg.window_cache() == {1: (2, 24, 40, False), 2: (2, 24, 16, False), 3: (2, 32, 40, False), 4: (1, 16, 24, False),
                                  5: (2, 16, 40, False)}
    st = cfg.named_state()
    assert st[0] == {"ssm": (3, 16, 24), "conv": (3, 3 * 24 + 2 * 3 * 16)}
    assert st[2] == {"S": (4, 16, 40), "conv": (3, 2 * 2 * 16 + 4 * 40)} and st[4]["conv"] == (1, 2 * 2 * 40 + 2 * 24)
    assert cfg.rank(2, "a1") == 5 and cfg.rank(4, "g1") == 7 and cfg.shift_layers() == []


def test_model_loads_a_checkpoint_on_cpu(tmp_path):
    """names and merges of load_weights (no kernel runs): merged projections hold the checkpoint's rows in order"""
    from scratchpad_amd import distributed, registry
    from scratchpad_amd.kikurax import KikuraxForCausalLM
    if not distributed.model_parallel_is_initialized():
        distributed.initialize_model_parallel(1)
    raw = U.full_config()
    folder, w = U.make_model(tmp_path, raw, seed=2, rank_a=5, rank_g=7)
    cfg = registry.load_config(folder, context_len=64)
    model = KikuraxForCausalLM(cfg, dtype=torch.float32)
    registry.load_weights(model, folder)
    a = model.layers[1].mix
    assert a.v_first is None and a.attn.v_mix is None and model.layers[3].mix.v_first == 1 and model.layers[5].mix.v_first == 1
    assert torch.equal(a.qkv[6 * 24:6 * 24 + 2 * 24].double(), w["l1.mix.k"]) and torch.equal(a.attn.head_scale.double(), w["l1.mix.temp"])
    assert float(model.layers[3].mix.attn.v_mix) == float(w["l3.mix.vmix"]) and float(a.attn.sinks.abs().max()) == 0.0
    p = model.layers[2].mix
    assert p.left_rows == 4 * 24 + 2 * 24 + 2 * 16 + 4 * 16 and p.right.in_rows == 2 * 2 * 16 + 4 * 40 + 4 + 5 + 7
    assert torch.equal(p.in_proj[4 * 24 + 2 * 24 + 2 * 16:p.left_rows].double(), w["l2.mix.left.g"])
    r0 = p.left_rows + p.right.conv_rows
    assert torch.equal(p.in_proj[r0:r0 + 4].double(), w["l2.mix.right.b"]) and torch.equal(p.in_proj[-7:].double(), w["l2.mix.right.g1"])
    assert torch.equal(p.right.a2t.double(), w["l2.mix.right.a2"].T) and torch.equal(p.right.conv[2 * 16:4 * 16].double(), w["l2.mix.right.k.conv"])
    assert torch.equal(p.branch_weight[1].double(), w["l2.mix.right.out"]) and torch.equal(p.attn.head_bias.double(), w["l2.mix.left.pb"])
    m = model.layers[0].mix
    assert torch.equal(m.dt_proj.double(), w["l0.mix.in"][-3:]) and model.layers[2].mlp is None
    e = model.layers[1].mlp
    assert torch.equal(e.experts.gate_up[4, 24:].double(), w["l1.mlp.e4.up"]) and torch.equal(e.router.bias.double(), w["l1.mlp.router.b"])
    assert torch.equal(model.lm_head.weight[:cfg.vocab_size].double(), w["embed"])
    assert json.load(open(folder + "/config.json"))["architecture"] == "Kikurax"
