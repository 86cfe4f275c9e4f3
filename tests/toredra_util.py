"""Helpers of the Toredra tests: small configurations whose sizes differ from one another (key width unlike value width,
query heads unlike key/value heads, a rotation narrower than the head, head widths that are no power of two), loops over
parts of the layer list, a checkpoint folder written from the oracle's random weights, and the comparison used throughout."""
import torch

from oracle import toredra as to
from tests.tizalorn_util import rel, tokens, write_checkpoint  # noqa: F401  (the checkpoint writer is format-only)


def delta(heads, dim):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim}}


def parallel(heads, kv_heads, dim, vdim, rheads, rdim, rvdim, dims=None, scaling=True, base=500.0, scale=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5}
    if dims != 0:
        left["rot"] = {"base": base, "dims": dims or dim}
        if scaling:
            left["rot"]["scaling"] = {"factor": 3.0, "low": 1.0, "high": 3.0, "original": 40}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": rheads, "dim": rdim, "vdim": rvdim}}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def config(layers, width=80, vocab=173, eps=1e-5, loop=None, logit_scale=0.5, softcap=20.0):
    cfg = {"architecture": "Toredra", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "layers": [{**spec, "mlp": mlp} for spec, mlp in layers]}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if logit_scale is not None:
        cfg["logit_scale"] = logit_scale
    if softcap is not None:
        cfg["logit_softcap"] = softcap
    return cfg


def full_config():
    """both mixers in an order of their own, sizes unlike each other, one layer without a feed-forward, a loop that
    starts behind the first layer, holds an attention layer (one cache per pass) and ends before the last layer"""
    return config([
        (delta(3, 24), dense(120)),
        (parallel(6, 2, 24, 40, 3, 16, 24, dims=16), dense(56)),
        (delta(2, 40), None),
        (parallel(2, 1, 32, 16, 1, 40, 72, scaling=False), dense(96)),
        (delta(1, 72), dense(64)),
    ], width=96, loop=(1, 3, 3))


def make_model(tmp_path, cfg, seed=0, name="m", rank=8):
    w = to.random_weights(cfg, seed, rank=rank)
    return write_checkpoint(str(tmp_path / name), cfg, w), w


def greedy(prompt, w, cfg, n):
    """n tokens of greedy generation by the oracle (the whole sequence again for every token)"""
    seq, out = list(prompt), []
    for _ in range(n):
        t = int(torch.argmax(to.forward(seq, w, cfg)[-1]))
        out.append(t)
        seq.append(t)
    return out


def random_config(seed: int):
    """a design drawn at random: layer order, loop, every size and constant (small enough for the oracle, odd enough to
    miss every power of two now and then)"""
    import random
    r = random.Random(seed)
    layers = []
    for _ in range(r.randint(2, 5)):
        if r.random() < 0.5:
            spec = delta(r.choice([1, 2, 3, 5]), r.choice([8, 16, 24, 40, 64]))
        else:
            heads = r.choice([1, 2, 3, 4, 6])
            kv = r.choice([d for d in range(1, heads + 1) if heads % d == 0])
            dim = r.choice([8, 16, 24, 32, 64])
            spec = parallel(heads, kv, dim, r.choice([8, 16, 40, 64]), r.choice([1, 2, 3]), r.choice([8, 16, 40]),
                            r.choice([8, 24, 64]), dims=r.choice([0, dim, dim // 2 // 2 * 2 or 2]), scaling=r.random() < 0.6,
                            base=r.choice([100.0, 10000.0]), scale=r.choice([None, 0.3, 0.11]))
        layers.append((spec, None if r.random() < 0.25 else dense(r.choice([24, 56, 100]))))
    n = len(layers)
    loop = None
    if r.random() < 0.7:
        a = r.randint(0, n - 1)
        loop = (a, r.randint(a + 1, n), r.choice([1, 2, 3]))
    return config(layers, width=r.choice([48, 64, 96, 128]), vocab=r.choice([61, 130, 257]), eps=r.choice([1e-6, 1e-5]),
                  loop=loop, logit_scale=r.choice([None, 0.3, 2.0]), softcap=r.choice([None, 5.0, 25.0]))
