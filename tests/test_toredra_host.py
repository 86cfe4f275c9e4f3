"""CPU tests around the Toredra design: the oracle against itself (causality, recurrences carried in pieces, the sink, the
frequency rule), the configuration reader and its layer runs, the registry, and the shapes the pools are built from."""
import json
import math

import pytest
import torch

from oracle import toredra as to
from tests import toredra_util as U


def test_oracle_is_causal_and_deterministic():
    cfg = U.full_config()
    w = to.random_weights(cfg, 3)
    toks = U.tokens(40, cfg["vocab"], 1)
    a = to.forward(toks, w, cfg)
    b = to.forward(toks[:25], w, cfg)
    assert torch.allclose(a[:25], b, atol=1e-9)
    assert torch.isfinite(a).all()
    assert float(a.abs().max()) <= cfg["logit_softcap"]


def test_layer_runs_of_a_loop():
    cfg = U.full_config()
    assert to.layer_runs(cfg) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert to.layer_runs({**cfg, "loop": {"start": 0, "stop": 5, "times": 2}}) == [0, 1, 2, 3, 4] * 2
    assert to.layer_runs({k: v for k, v in cfg.items() if k != "loop"}) == [0, 1, 2, 3, 4]
    cap = []
    to.forward(U.tokens(5, cfg["vocab"], 0), to.random_weights(cfg, 0), cfg, cap)
    assert len(cap) == 9


def test_oracle_recurrences_do_what_their_names_say():
    g = torch.Generator().manual_seed(0)
    T, H, D = 12, 2, 6
    r, k, v = (torch.randn(T, H, D, generator=g, dtype=torch.float64) for _ in range(3))
    one, zero = torch.ones(T, H, D, dtype=torch.float64), torch.zeros(T, H, D, dtype=torch.float64)
    # no decay, nothing removed: plain linear attention
    o = to.delta_recurrence(r, k, v, one, zero)
    mask = torch.tril(torch.ones(T, T, dtype=torch.float64))
    want = torch.einsum("ts,thd,shd,she->the", mask, r, k, v)
    assert torch.allclose(o, want, atol=1e-9)
    # everything removed along a repeated unit key: what the key wrote before is gone, the new value stays
    k2 = k.clone()
    k2[1] = k2[0]
    o2 = to.delta_recurrence(k2, k2, v, one, one)                     # read with the key itself
    n2 = (k2[1] ** 2).sum(-1)
    assert torch.allclose(o2[1], v[1] * n2[:, None] + v[0] * (n2 * 1e-6 / (n2 + 1e-6))[:, None], atol=1e-6)
    # forget gate 1 writes nothing, forget gate 0 replaces the row by the value
    q = torch.randn(T, H, D, generator=g, dtype=torch.float64)
    assert float(to.forget_write_recurrence(q, one, v).abs().max()) == 0.0
    assert torch.allclose(to.forget_write_recurrence(q, zero, v), q.sum(-1, keepdim=True) * v, atol=1e-9)


def test_sink_only_shrinks_the_output():
    g = torch.Generator().manual_seed(1)
    T, H, G, D, Dv = 9, 4, 2, 8, 5
    q, k, v = (torch.randn(T, n, d, generator=g, dtype=torch.float64) for n, d in ((H, D), (G, D), (G, Dv)))
    gone = to.sink_attention(q, k, v, torch.full((H,), -1e9, dtype=torch.float64), 0.3)
    plain = torch.stack([torch.stack([torch.softmax((k[:i + 1, h // 2] @ q[i, h]) * 0.3, 0) @ v[:i + 1, h // 2] for h in range(H)])
                         for i in range(T)])
    assert torch.allclose(gone, plain, atol=1e-9)
    sink = torch.tensor([0.0, 1.0, -2.0, 3.0], dtype=torch.float64)
    got = to.sink_attention(q, k, v, sink, 0.3)
    den = torch.stack([torch.stack([torch.exp((k[:i + 1, h // 2] @ q[i, h]) * 0.3).sum() for h in range(H)]) for i in range(T)])
    assert torch.allclose(got, plain * (den / (den + torch.exp(sink)))[..., None], atol=1e-9)
    # the first token sees itself and the sink only
    assert torch.allclose(got[0], v[0].repeat_interleave(2, 0) * (den[0] / (den[0] + torch.exp(sink)))[:, None], atol=1e-9)


def test_frequency_rule_of_oracle_and_product_agree():
    from scratchpad_amd.layers import AngleRotary, wavelength_blend
    for rot in ({"dims": 40, "base": 30000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 3.0, "original": 512}},
                {"dims": 16, "base": 100.0, "scaling": {"factor": 3.0, "low": 2.0, "high": 2.0, "original": 40}},
                {"dims": 8, "base": 10000.0}):
        f = to.rotary_frequencies(rot)
        sc = rot.get("scaling")
        if sc:
            g = wavelength_blend(rot["dims"], rot["base"], sc["factor"], sc["original"], sc["low"], sc["high"])
            assert torch.allclose(f, g, rtol=1e-14)
            plain = torch.tensor([rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)], dtype=torch.float64)
            wl = 2 * math.pi / plain
            assert torch.equal(f[wl < sc["original"] / sc["high"]], plain[wl < sc["original"] / sc["high"]])
            assert torch.allclose(f[wl > sc["original"] / sc["low"]], plain[wl > sc["original"] / sc["low"]] / sc["factor"])
            assert (f <= plain).all() and (f >= plain / sc["factor"] * (1 - 1e-12)).all()
        mod = AngleRotary(rot["dims"], rot["base"], sc)
        assert mod.adjacent_pairs and mod.magnitude == 1.0
        assert torch.allclose(mod.freq.double(), f, rtol=1e-6)


def test_config_reader_registry_and_pool_shapes():
    from scratchpad_amd import registry
    from scratchpad_amd.toredra import ToredraConfig, ToredraForCausalLM
    raw = U.full_config()
    assert registry.architecture_of(raw) == "Toredra"
    cfg = registry.MODELS["Toredra"][0](raw, context_len=256, tensor_shapes={"l0.mix.w1": (5, 96), "l2.mix.w1": (11, 96)})
    assert isinstance(cfg, ToredraConfig) and registry.model_class_for(cfg) is ToredraForCausalLM
    assert [i for i, _ in cfg.runs] == to.layer_runs(raw)
    assert [again for _, again in cfg.runs] == [False, False, False, True, False, True, False, False, False]
    # one cache per RUN of an attention layer, one state per run of every layer
    assert cfg.window_cache() == {1: (2, 24, 40, False), 3: (2, 24, 40, False), 5: (2, 24, 40, False), 7: (1, 32, 16, False)}
    named = cfg.named_state()
    assert sorted(named) == list(range(9))
    assert named[0] == {"S": (3, 24, 24)} and named[1] == {"S": (3, 16, 24)} and named[4] == {"S": (2, 40, 40)}
    assert named[7] == {"S": (1, 40, 72)} and named[8] == {"S": (1, 72, 72)}
    assert cfg.shift_layers() == []
    assert cfg.cache_bytes_per_token(torch.bfloat16) == 2 * (3 * 2 * (24 + 40) + (32 + 16))
    assert cfg.decay_rank(0) == 5 and cfg.decay_rank(2) == 11 and cfg.decay_rank(4) == cfg.default_decay_rank
    assert cfg.logit_scale == 0.5 and cfg.final_logit_softcapping == 20.0
    plain = ToredraConfig({k: v for k, v in raw.items() if k not in ("loop", "logit_scale", "logit_softcap")})
    assert [i for i, _ in plain.runs] == list(range(5)) and not any(a for _, a in plain.runs)
    assert plain.logit_scale == 1.0 and plain.final_logit_softcapping == 0.0
    once = ToredraConfig({**raw, "loop": {"start": 0, "stop": 5, "times": 1}})
    assert [i for i, _ in once.runs] == list(range(5)) and not any(a for _, a in once.runs)
    with pytest.raises(ValueError):
        ToredraConfig({**raw, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]})
    with pytest.raises(ValueError):
        ToredraConfig({**raw, "loop": {"start": 3, "stop": 9, "times": 2}})


def test_model_loads_a_checkpoint_on_cpu(tmp_path):
    """names and merges of load_weights (no kernel runs): merged projections hold the checkpoint's rows in order"""
    from scratchpad_amd import distributed, registry
    from scratchpad_amd.toredra import ToredraForCausalLM
    if not distributed.model_parallel_is_initialized():
        distributed.initialize_model_parallel(1)
    raw = U.full_config()
    folder, w = U.make_model(tmp_path, raw, seed=2, rank=5)
    cfg = registry.load_config(folder, context_len=64)
    model = ToredraForCausalLM(cfg, dtype=torch.float32)
    registry.load_weights(model, folder)
    d = model.layers[0].mix
    n = 3 * 24
    assert d.rank == 5 and d.in_proj.shape[0] == 5 * n + 5 + 96
    assert torch.equal(d.in_proj[n:2 * n].double(), w["l0.mix.k"]) and torch.equal(d.in_proj[4 * n:5 * n].double(), w["l0.mix.a"])
    assert torch.equal(d.in_proj[5 * n:5 * n + 5].double(), w["l0.mix.w1"]) and torch.equal(d.in_proj[-96:].double(), w["l0.rg1"])
    assert torch.equal(d.w2t.double(), w["l0.mix.w2"].T) and abs(d.rate - math.exp(-0.5)) < 1e-12
    p = model.layers[1].mix
    assert p.left_rows == 6 * 24 + 2 * 24 + 2 * 40 and p.right.in_rows == 2 * 3 * 16 + 3 * 24
    assert torch.equal(p.in_proj[:6 * 24].double(), w["l1.mix.left.q"])
    assert torch.equal(p.in_proj[p.left_rows + 3 * 16:p.left_rows + 2 * 3 * 16].double(), w["l1.mix.right.f"])
    assert torch.equal(p.in_proj[-96:].double(), w["l1.rg1"]) and torch.equal(p.attn.sinks.double(), w["l1.mix.left.sink"])
    assert torch.equal(model.layers[1].tail1.branch_weight[1].double(), w["l1.mix.right.out"])
    assert model.layers[2].mlp is None and torch.equal(model.layers[0].mlp.up[-96:].double(), w["l0.rg2"])
    assert torch.equal(model.lm_head.weight[:cfg.vocab_size].double(), w["embed"])
    assert json.load(open(folder + "/config.json"))["architecture"] == "Toredra"
