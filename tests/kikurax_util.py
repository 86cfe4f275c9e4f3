"""Helpers of the Kikurax tests: small configurations whose sizes differ from one another (key width unlike value width,
query heads unlike key/value heads, a rotation narrower than the head, widths that are no power of two), a checkpoint
folder written from the oracle's random weights, and the comparison used throughout."""
import torch

from oracle import kikurax as ko
from tests.tizalorn_util import rel, tokens, write_checkpoint  # noqa: F401  (the checkpoint writer is format-only)


def attention(heads, kv_heads, dim, vdim, dims=None, scaling=True, base=500.0, scale=None, softcap=8.0, v_mix=True):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or 2.0 * dim ** -0.5, "v_mix": v_mix}
    if softcap:
        m["softcap"] = softcap
    if dims != 0:
        m["rot"] = {"base": base, "dims": dims or dim}
        if scaling:
            m["rot"]["scaling"] = {"factor": 3.0, "low": 1.0, "high": 3.0, "original": 40}
    return {"type": "attention", "mixer": m}


def mamba(heads, vdim, state, groups=1, conv=3, norm_groups=1):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}}


def parallel(heads, kv_heads, dim, vdim, rheads, rkv, rdim, rvdim, conv=3, coef=0.7, every=5, scale=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5}
    if every:
        left["q_temp"] = {"coef": coef, "every": every}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": rheads, "kv_heads": rkv, "dim": rdim, "vdim": rvdim,
                                                                  "conv": conv}}}


def moe(experts, top, ff, limit=1.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def config(layers, width=80, vocab=173, eps=1e-5, groups=2, scale=3.0):
    return {"architecture": "Kikurax", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups},
            "embedding": {"scale": scale}, "layers": [{**spec, "mlp": mlp} for spec, mlp in layers]}


def full_config():
    """all three mixers in an order of their own, sizes unlike each other, three attention layers that blend values (the
    first is not the model's first layer), one layer without a feed-forward"""
    return config([
        (mamba(3, 24, 16, groups=3, conv=4, norm_groups=3), moe(5, 2, 40)),
        (attention(6, 2, 24, 40, dims=16), moe(7, 3, 24)),
        (parallel(4, 2, 24, 16, 4, 2, 16, 40, conv=4), None),
        (attention(2, 2, 32, 40, scaling=False, softcap=3.0), moe(4, 1, 56)),
        (parallel(3, 1, 16, 24, 2, 2, 40, 24, conv=2, every=3), moe(6, 6, 16, limit=0.4)),
        (attention(4, 2, 16, 40, dims=8, softcap=None), moe(3, 2, 32)),
    ], width=96, groups=3)


def make_model(tmp_path, cfg, seed=0, name="m", rank_a=6, rank_g=10):
    w = ko.random_weights(cfg, seed, rank_a=rank_a, rank_g=rank_g)
    return write_checkpoint(str(tmp_path / name), cfg, w), w


def greedy(prompt, w, cfg, n):
    """n tokens of greedy generation by the oracle (the whole sequence again for every token)"""
    seq, out = list(prompt), []
    for _ in range(n):
        t = int(torch.argmax(ko.forward(seq, w, cfg)[-1]))
        out.append(t)
        seq.append(t)
    return out


def random_config(seed: int):
    """a design drawn at random: layer order, every size and constant"""
    import random
    r = random.Random(seed)
    layers, vm = [], None
    for _ in range(r.randint(2, 5)):
        kind = r.choice(["attention", "mamba2", "parallel"])
        if kind == "attention":
            heads = r.choice([1, 2, 3, 4, 6])
            kv = r.choice([d for d in range(1, heads + 1) if heads % d == 0])
            dim = r.choice([8, 16, 24, 32, 64])
            mix = r.random() < 0.7
            vdim = r.choice([8, 16, 40, 64])
            if mix:                                   # layers that blend values agree on their value rows
                if vm is None:
                    vm = (kv, vdim)
                elif heads % vm[0] == 0:
                    kv, vdim = vm
                else:
                    mix = False
            spec = attention(heads, kv, dim, vdim, dims=r.choice([0, dim, dim // 2 // 2 * 2 or 2]), scaling=r.random() < 0.6,
                             base=r.choice([100.0, 10000.0]), scale=r.choice([None, 0.3, 0.11]),
                             softcap=r.choice([None, 2.0, 30.0]), v_mix=mix)
        elif kind == "mamba2":
            heads = r.choice([1, 2, 4, 6])
            groups = r.choice([d for d in range(1, heads + 1) if heads % d == 0])
            vdim = r.choice([8, 16, 24])
            spec = mamba(heads, vdim, r.choice([8, 16, 40]), groups, r.choice([1, 2, 4]),
                         r.choice([d for d in (1, 2, heads) if (heads * vdim) % d == 0]))
        else:
            heads = r.choice([1, 2, 4, 6])
            kv = r.choice([d for d in range(1, heads + 1) if heads % d == 0])
            rheads = r.choice([1, 2, 4])
            spec = parallel(heads, kv, r.choice([8, 16, 40]), r.choice([8, 24, 64]), rheads,
                            r.choice([d for d in range(1, rheads + 1) if rheads % d == 0]), r.choice([8, 16, 40]),
                            r.choice([8, 24, 64]), conv=r.choice([1, 2, 4]), coef=r.choice([0.2, 1.0]), every=r.choice([0, 1, 4, 16]),
                            scale=r.choice([None, 0.2]))
        e = r.choice([2, 4, 9])
        layers.append((spec, None if r.random() < 0.25 else moe(e, r.randint(1, e), r.choice([8, 24, 40]), r.choice([0.5, 2.0]))))
    width = r.choice([48, 64, 96, 120])
    return config(layers, width=width, vocab=r.choice([61, 130, 257]), eps=r.choice([1e-6, 1e-5]),
                  groups=r.choice([1, 2, 4]), scale=r.choice([1.0, 7.5]))
