"""CPU oracle of the Toredra design: one plain, slow function per mechanism, written from the design's equations.

TEST INFRASTRUCTURE ONLY: nothing under scratchpad_amd/ imports this, and this imports nothing from there.  Every
function works on ONE whole sequence in float64 (or the dtype it is given) and keeps no cache and no state: a sequence
is recomputed from its first token, which is what makes it a reference for caches, states, portions and batches.

Notation: T tokens, W model width, x the residual stream [T, W].  A layer is
    h = N(x) w1;    x <- x + N(mixer(h) * sigmoid(R1 h + b1)) w1b
    h = N(x) w2;    x <- x + N(ff(h)    * sigmoid(R2 h + b2)) w2b
with N(z) = z / sqrt(mean(z^2) + eps).  The layers ``start .. stop - 1`` of the list run ``times`` times in a row on
the same weights; every pass after the first begins with x <- x + x0, x0 being the embedding rows.
"""
import math
from typing import Dict, List, Optional

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


# ----------------------------------------------------------------------------------------------- rotary
def rotary_frequencies(rot: dict) -> torch.Tensor:
    """frequency per pair [dims/2]: base^(-2i/dims), bent by the wavelength rule of ``scaling`` = {factor, low, high,
    original}: wavelengths below original/high keep their frequency, those above original/low have it divided by factor,
    between the two the frequencies are blended linearly in original/wavelength"""
    dims, base = int(rot["dims"]), float(rot["base"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            wl = 2 * math.pi / f
            if wl < orig / high:
                pass
            elif wl > orig / low:
                f = f / factor
            else:
                s = (orig / wl - low) / (high - low)
                f = (1 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def rotate_adjacent_pairs(x: torch.Tensor, rot: Optional[dict], first: int = 0) -> torch.Tensor:
    """x [T, heads, n]: coordinates (2i, 2i + 1), i < dims/2, turn by position * f_i; the rest of n passes.  ``first``:
    position of the sequence's row 0"""
    if not rot or int(rot["dims"]) == 0:
        return x
    dims = int(rot["dims"])
    f = rotary_frequencies(rot)
    pos = torch.arange(first, first + x.shape[0], dtype=torch.float64)
    ang = pos[:, None] * f[None, :]
    c, s = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ----------------------------------------------------------------------------------------------- attention with a sink
def sink_attention(q, k, v, sink, scale: float) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, Dv], sink [H] -> [T, H, Dv].  Causal; per head the softmax's denominator holds
    one more term exp(sink_h) that has no key and no value and is not scaled."""
    T, H, D = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for i in range(T):
        for h in range(H):
            g = h // (H // G)
            s = (k[:i + 1, g] @ q[i, h]) * scale
            m = torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            out[i, h] = (e @ v[:i + 1, g]) / (e.sum() + torch.exp(sink[h] - m))
    return out


def attention_branch(h, w, p: str, m: dict, kv_round=None) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[f"{p}.q"].T + w[f"{p}.q.b"]).view(T, H, D)
    k = (h @ w[f"{p}.k"].T + w[f"{p}.k.b"]).view(T, G, D)
    v = (h @ w[f"{p}.v"].T + w[f"{p}.v.b"]).view(T, G, Dv)
    q, k = rotate_adjacent_pairs(q, m.get("rot")), rotate_adjacent_pairs(k, m.get("rot"))
    if kv_round is not None:           # what a cache of lower precision holds
        k, v = kv_round(k), kv_round(v)
    o = sink_attention(q, k, v, w[f"{p}.sink"], float(m["scale"]))
    return o.reshape(T, H * Dv) @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------------------------- gated linear attention whose forget gate also writes
def forget_write_recurrence(q, f, v) -> torch.Tensor:
    """q, f [T, H, D], v [T, H, Dv] -> [T, H, Dv]:  S <- diag(f) S + (1 - f) v^T,  o = S^T q  (S [D, Dv] from zero)"""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[-1], dtype=q.dtype)
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for t in range(T):
        for hd in range(H):
            S[hd] = f[t, hd][:, None] * S[hd] + torch.outer(1 - f[t, hd], v[t, hd])
            out[t, hd] = S[hd].T @ q[t, hd]
    return out


def hgrn2_branch(h, w, p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ w[f"{p}.q"].T).view(T, H, D)
    v = (h @ w[f"{p}.v"].T).view(T, H, Dv)
    low = w[f"{p}.lower"]
    f = (low + (1 - low) * torch.sigmoid(h @ w[f"{p}.f"].T + w[f"{p}.f.b"])).view(T, H, D)
    o = rms(forget_write_recurrence(q, f, v), eps) * w[f"{p}.norm"]
    return o.reshape(T, H * Dv) @ w[f"{p}.o"].T


def parallel_mixer(h, w, p: str, m: dict, eps: float, kv_round=None) -> torch.Tensor:
    left = attention_branch(h, w, f"{p}.left", m["left"], kv_round)
    right = hgrn2_branch(h, w, f"{p}.right", m["right"], eps)
    return 0.5 * (rms(left, eps) * w[f"{p}.left.out"] + rms(right, eps) * w[f"{p}.right.out"])


# ----------------------------------------------------------------------------------------------- generalized delta rule
DECAY_RATE = math.exp(-0.5)


def delta_recurrence(r, k, v, decay, remove) -> torch.Tensor:
    """r, k, v, decay, remove [T, H, D] -> [T, H, D].  With u = k / sqrt(|k|^2 + 1e-6):
    S <- diag(decay) S - (remove * u) (u^T S) + k v^T  (both first terms read the state of the previous token),
    o = S^T r"""
    T, H, D = r.shape
    S = torch.zeros(H, D, D, dtype=r.dtype)
    out = torch.zeros(T, H, D, dtype=r.dtype)
    for t in range(T):
        for hd in range(H):
            u = k[t, hd] / torch.sqrt((k[t, hd] ** 2).sum() + 1e-6)
            S[hd] = decay[t, hd][:, None] * S[hd] - torch.outer(remove[t, hd] * u, u @ S[hd]) + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S[hd].T @ r[t, hd]
    return out


def delta_mixer(h, w, p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D = int(m["heads"]), int(m["dim"])
    r, k, v = ((h @ w[f"{p}.{s}"].T).view(T, H, D) for s in "rkv")
    decay = torch.exp(-DECAY_RATE * torch.sigmoid(torch.tanh(h @ w[f"{p}.w1"].T) @ w[f"{p}.w2"].T + w[f"{p}.w0"])).view(T, H, D)
    remove = torch.sigmoid(h @ w[f"{p}.a"].T + w[f"{p}.a.b"]).view(T, H, D)
    o = rms(delta_recurrence(r, k, v, decay, remove), eps).reshape(T, H * D)
    return (o * w[f"{p}.norm"] * torch.sigmoid(h @ w[f"{p}.g"].T)) @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------------------------- feed-forward
def relu2_ff(h, w, p: str) -> torch.Tensor:
    return (torch.relu(h @ w[f"{p}.up"].T) ** 2) @ w[f"{p}.down"].T


# ----------------------------------------------------------------------------------------------- the model
def layer_runs(cfg: dict) -> List[int]:
    """index of the layer (its weights) of every layer run, in order"""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(tokens, w: Dict[str, torch.Tensor], cfg: dict, capture: Optional[list] = None, kv_round=None) -> torch.Tensor:
    """logits [T, vocab] of one sequence; ``capture`` collects the stream after every layer run"""
    eps = float(cfg["norm"]["eps"])
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    seen_first = False
    for li in layer_runs(cfg):
        if li == int(loop["start"]) and int(loop["stop"]) > int(loop["start"]):
            if seen_first:
                x = x + x0
            seen_first = True
        spec, p = cfg["layers"][li], f"l{li}"
        h = rms(x, eps) * w[f"{p}.norm1"]
        if spec["type"] == "parallel":
            y = parallel_mixer(h, w, f"{p}.mix", spec["mixer"], eps, kv_round)
        elif spec["type"] == "general_delta":
            y = delta_mixer(h, w, f"{p}.mix", spec["mixer"], eps)
        else:
            raise ValueError(spec["type"])
        y = y * torch.sigmoid(h @ w[f"{p}.rg1"].T + w[f"{p}.rg1.b"])
        x = x + rms(y, eps) * w[f"{p}.norm1b"]
        if spec.get("mlp") is not None:
            h = rms(x, eps) * w[f"{p}.norm2"]
            y = relu2_ff(h, w, f"{p}.mlp") * torch.sigmoid(h @ w[f"{p}.rg2"].T + w[f"{p}.rg2.b"])
            x = x + rms(y, eps) * w[f"{p}.norm2b"]
        if capture is not None:
            capture.append(x.clone())
    z = (rms(x, eps) * w["final.norm"]) @ w["embed"].T * float(cfg.get("logit_scale", 1.0))
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


# ----------------------------------------------------------------------------------------------- random weights
def tensor_shapes(cfg: dict, rank: int = 8) -> Dict[str, tuple]:
    """name -> shape of a checkpoint of the design; ``rank``: rows of the decay's first projection (a checkpoint's tensor
    shape gives it, no configuration key does)"""
    W, V = int(cfg["width"]), int(cfg["vocab"])
    s = {"embed": (V, W), "final.norm": (W,)}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}", spec["mixer"]
        for n in ("norm1", "norm1b", "rg1.b"):
            s[f"{p}.{n}"] = (W,)
        s[f"{p}.rg1"] = (W, W)
        if spec["type"] == "parallel":
            a, b = m["left"], m["right"]
            H, G, D, Dv = (int(a[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                s[f"{p}.mix.left.{n}"] = (rows, W)
                s[f"{p}.mix.left.{n}.b"] = (rows,)
            s[f"{p}.mix.left.sink"] = (H,)
            s[f"{p}.mix.left.o"] = (W, H * Dv)
            H, D, Dv = (int(b[k]) for k in ("heads", "dim", "vdim"))
            s[f"{p}.mix.right.q"] = s[f"{p}.mix.right.f"] = (H * D, W)
            s[f"{p}.mix.right.f.b"] = s[f"{p}.mix.right.lower"] = (H * D,)
            s[f"{p}.mix.right.v"] = (H * Dv, W)
            s[f"{p}.mix.right.norm"] = (Dv,)
            s[f"{p}.mix.right.o"] = (W, H * Dv)
            s[f"{p}.mix.left.out"] = s[f"{p}.mix.right.out"] = (W,)
        else:
            n = int(m["heads"]) * int(m["dim"])
            for name in "rkvga":
                s[f"{p}.mix.{name}"] = (n, W)
            s[f"{p}.mix.a.b"] = s[f"{p}.mix.w0"] = s[f"{p}.mix.norm"] = (n,)
            s[f"{p}.mix.w1"], s[f"{p}.mix.w2"] = (rank, W), (n, rank)
            s[f"{p}.mix.o"] = (W, n)
        if spec.get("mlp") is not None:
            ff = int(spec["mlp"]["ff"])
            for n in ("norm2", "norm2b", "rg2.b"):
                s[f"{p}.{n}"] = (W,)
            s[f"{p}.rg2"] = (W, W)
            s[f"{p}.mlp.up"], s[f"{p}.mlp.down"] = (ff, W), (W, ff)
    return s


def random_weights(cfg: dict, seed: int = 0, dtype=torch.float64, rank: int = 8) -> Dict[str, torch.Tensor]:
    """weights that keep every mechanism visible in the logits; values are exactly representable in bfloat16"""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg, rank).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        if len(shape) == 2:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[1]))
            if name == "embed":
                t = torch.randn(shape, generator=g)
        elif leaf.endswith("norm") or leaf.endswith("norm1") or leaf.endswith("norm2") or leaf.endswith("norm1b") \
                or leaf.endswith("norm2b") or leaf.endswith(".out"):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf.endswith("lower"):
            t = torch.rand(shape, generator=g) * 0.9
        elif leaf.endswith("sink"):
            t = torch.randn(shape, generator=g) * 1.5
        elif leaf.endswith("w0"):
            t = torch.randn(shape, generator=g) * 1.5 - 1.0
        else:
            t = torch.randn(shape, generator=g) * 0.5
        w[name] = t.to(torch.bfloat16).to(dtype)
    return w
