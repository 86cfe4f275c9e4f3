"""CPU oracle of the Kikurax design: one plain, slow function per mechanism, written from the design's equations.

TEST INFRASTRUCTURE ONLY: nothing under scratchpad_amd/ imports this, and this imports nothing from there.  Every
function works on ONE whole sequence in float64 (or the dtype it is given) and keeps no cache and no state: a sequence
is recomputed from its first token, which is what makes it a reference for caches, states, portions and batches.

Notation: T tokens, W model width, x the residual stream [T, W].  A layer is
    x <- x + mixer(GN(x) w1);    x <- x + ff(GN(x) w2)
with GN the root-mean-square norm taken separately over ``norm.groups`` equal consecutive parts of the row.  The mixer
is, layer by layer, softmax attention with a zero-score sink, a Mamba-2 state-space mixer, or a sigmoid-weighted
attention beside a channel-gated delta rule (each normed over the width, averaged).  The feed-forward is a mixture of
clamped gated experts; the head is the embedding table.
"""
import math
from typing import Dict, List, Optional

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """every one of ``groups`` equal consecutive parts of a row divided by its own root mean square, the row times w"""
    T, n = x.shape
    return (rms(x.reshape(T, groups, n // groups), eps).reshape(T, n)) * w


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


# ----------------------------------------------------------------------------------------------- rotary
def rotary_frequencies(rot: dict) -> torch.Tensor:
    """frequency per pair [dims/2]: base^(-2i/dims), bent by the wavelength rule of ``scaling`` = {factor, low, high,
    original}"""
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


def rotate_half_pairs(x: torch.Tensor, rot: Optional[dict]) -> torch.Tensor:
    """x [T, heads, n]: coordinate i < dims/2 pairs with i + dims/2 and the pair turns by position * f_i; the rest passes"""
    if not rot or int(rot["dims"]) == 0:
        return x
    dims = int(rot["dims"])
    half = dims // 2
    f = rotary_frequencies(rot)
    ang = torch.arange(x.shape[0], dtype=torch.float64)[:, None] * f[None, :]
    c, s = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


# ----------------------------------------------------------------------------------------------- attention (softmax with a sink)
def softmax_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                      v_first: Optional[torch.Tensor], is_first: bool):
    """returns (output [T, W], the values this layer hands on as v_first or None)"""
    T = h.shape[0]
    H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    q = (h @ w[f"{p}.q"].T + w[f"{p}.q.b"]).reshape(T, H, D)
    k = (h @ w[f"{p}.k"].T + w[f"{p}.k.b"]).reshape(T, G, D)
    v = (h @ w[f"{p}.v"].T + w[f"{p}.v.b"]).reshape(T, G, Dv)
    q, k = rotate_half_pairs(q, m.get("rot")), rotate_half_pairs(k, m.get("rot"))
    q, k = rms(q, eps), rms(k, eps)
    handed = None
    if m.get("v_mix"):
        if is_first:
            handed = v
        else:
            lam = w[f"{p}.vmix"]
            v = (1 - lam) * v + lam * v_first
    cap = float(m["softcap"]) if m.get("softcap") else 0.0
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * float(m["scale"]) * w[f"{p}.temp"][hh]
        if cap:
            s = cap * torch.tanh(s / cap)
        for i in range(T):
            e = torch.exp(s[i, :i + 1] - s[i, :i + 1].max())
            den = e.sum() + torch.exp(-s[i, :i + 1].max())            # the sink: score 0, no value
            out[i, hh] = (e / den) @ v[:i + 1, g]
    return out.reshape(T, H * Dv) @ w[f"{p}.o"].T, handed


# ----------------------------------------------------------------------------------------------- sigmoid attention
def sigmoid_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    q = rms((h @ w[f"{p}.q"].T).reshape(T, H, D), eps)
    k = rms((h @ w[f"{p}.k"].T).reshape(T, G, D), eps)
    v = (h @ w[f"{p}.v"].T).reshape(T, G, Dv)
    qt = m.get("q_temp")
    if qt:
        pos = torch.arange(T, dtype=torch.float64)
        mult = 1 + float(qt["coef"]) * torch.log(torch.floor((pos + 1) / int(qt["every"])) + 1)
        q = q * mult.to(h.dtype)[:, None, None]
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].T) * float(m["scale"]) + w[f"{p}.pb"][hh]
        wt = torch.tril(torch.sigmoid(s))
        out[:, hh] = wt @ v[:, g]
    out = out.reshape(T, H * Dv) * torch.sigmoid(h @ w[f"{p}.g"].T)
    return out @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------------------------- short convolution
def causal_conv(u: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u [T, C], taps [C, K]: out[t, c] = sum_j taps[c, j] u[t - (K - 1 - j), c], zeros before the start"""
    T, C = u.shape
    K = taps.shape[1]
    pad = torch.cat([torch.zeros(K - 1, C, dtype=u.dtype), u], 0)
    out = torch.zeros_like(u)
    for j in range(K):
        out = out + pad[j:j + T] * taps[:, j]
    return out if bias is None else out + bias


# ----------------------------------------------------------------------------------------------- channel-gated delta rule
def gated_delta(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    q = silu(causal_conv(h @ w[f"{p}.q"].T, w[f"{p}.q.conv"])).reshape(T, G, D)
    k = silu(causal_conv(h @ w[f"{p}.k"].T, w[f"{p}.k.conv"])).reshape(T, G, D)
    v = silu(causal_conv(h @ w[f"{p}.v"].T, w[f"{p}.v.conv"])).reshape(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[f"{p}.b"].T)                                              # [T, H]
    step = softplus((h @ w[f"{p}.a1"].T) @ w[f"{p}.a2"].T + w[f"{p}.dt_bias"]).reshape(T, H, D)
    decay = torch.exp(-torch.exp(w[f"{p}.A_log"])[None, :, None] * step)                 # [T, H, D]
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for t in range(T):
            S = decay[t, hh][:, None] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, hh] = S.T @ q[t, g]
    gate = torch.sigmoid((h @ w[f"{p}.g1"].T) @ w[f"{p}.g2"].T).reshape(T, H, Dv)
    out = rms(out, eps) * w[f"{p}.norm"] * gate
    return out.reshape(T, H * Dv) @ w[f"{p}.o"].T


def parallel_mixer(h, w, p, m, eps):
    a = sigmoid_attention(h, w, f"{p}.left", m["left"], eps)
    b = gated_delta(h, w, f"{p}.right", m["right"], eps)
    return 0.5 * (rms(a, eps) * w[f"{p}.left.out"] + rms(b, eps) * w[f"{p}.right.out"])


# ----------------------------------------------------------------------------------------------- Mamba-2
def mamba2(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, Dv, N, G = (int(m[k]) for k in ("heads", "vdim", "state", "groups"))
    inner = H * Dv
    a = h @ w[f"{p}.in"].T
    z, xbc, dt = a[:, :inner], a[:, inner:2 * inner + 2 * G * N], a[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[f"{p}.conv"], w[f"{p}.conv.b"]))
    x = xbc[:, :inner].reshape(T, H, Dv)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[f"{p}.dt_bias"])                                                # [T, H]
    A = torch.exp(w[f"{p}.A_log"])
    y = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(N, Dv, dtype=h.dtype)
        for t in range(T):
            S = torch.exp(-A[hh] * dt[t, hh]) * S + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S.T @ C[t, g] + w[f"{p}.D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    y = group_norm(y, w[f"{p}.norm"], int(m["norm_groups"]), eps)
    return y @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------------------------- experts
def route(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, top: int):
    """(ids [T, top], weights [T, top]): the largest router logits, softmax over the chosen ones only"""
    z = h @ w[f"{p}.router"].T + w[f"{p}.router.b"]
    val, ids = torch.topk(z, top, dim=-1)
    return ids, torch.softmax(val, -1)


def expert(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, limit: float) -> torch.Tensor:
    g = torch.clamp(h @ w[f"{p}.gate"].T, max=limit)
    u = torch.clamp(h @ w[f"{p}.up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[f"{p}.down"].T


def moe(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    top, limit = int(mlp["router"]["top"]), float(mlp["expert"]["limit"])
    ids, wt = route(h, w, p, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            out[t] += wt[t, j] * expert(h[t:t + 1], w, f"{p}.e{int(ids[t, j])}", limit)[0]
    return out


# ----------------------------------------------------------------------------------------------- the model
def forward(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict, layers_out: Optional[list] = None) -> torch.Tensor:
    """logits [T, vocab] of one sequence; ``layers_out`` collects the stream after every layer"""
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups", 1))
    x = w["embed"][torch.tensor(tokens)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    v_first = None
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}", spec["mixer"]
        h = group_norm(x, w[f"{p}.norm1"], groups, eps)
        if spec["type"] == "attention":
            y, handed = softmax_attention(h, w, f"{p}.mix", m, eps, v_first, v_first is None)
            if handed is not None:
                v_first = handed
        elif spec["type"] == "mamba2":
            y = mamba2(h, w, f"{p}.mix", m, eps)
        elif spec["type"] == "parallel":
            y = parallel_mixer(h, w, f"{p}.mix", m, eps)
        else:
            raise ValueError(spec["type"])
        x = x + y
        if spec.get("mlp") is not None:
            x = x + moe(group_norm(x, w[f"{p}.norm2"], groups, eps), w, f"{p}.mlp", spec["mlp"])
        if layers_out is not None:
            layers_out.append(x.clone())
    return group_norm(x, w["final.norm"], groups, eps) @ w["embed"].T


# ----------------------------------------------------------------------------------------------- random weights
def tensor_shapes(cfg: dict, rank_a: int = 6, rank_g: int = 10) -> Dict[str, tuple]:
    """name -> shape of a checkpoint of the design; the ranks of the right mixer's low-rank projections are given by a
    checkpoint's tensor shapes only"""
    W, V = int(cfg["width"]), int(cfg["vocab"])
    s = {"embed": (V, W), "final.norm": (W,)}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}", spec["mixer"]
        s[f"{p}.norm1"] = (W,)
        if spec["type"] == "attention":
            H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                s[f"{p}.mix.{n}"] = (rows, W)
                s[f"{p}.mix.{n}.b"] = (rows,)
            s[f"{p}.mix.temp"] = (H,)
            if m.get("v_mix"):
                s[f"{p}.mix.vmix"] = ()
            s[f"{p}.mix.o"] = (W, H * Dv)
        elif spec["type"] == "mamba2":
            H, Dv, N, G, K = (int(m[k]) for k in ("heads", "vdim", "state", "groups", "conv"))
            inner, ch = H * Dv, H * Dv + 2 * G * N
            s[f"{p}.mix.in"] = (inner + ch + H, W)
            s[f"{p}.mix.conv"], s[f"{p}.mix.conv.b"] = (ch, K), (ch,)
            s[f"{p}.mix.dt_bias"] = s[f"{p}.mix.A_log"] = s[f"{p}.mix.D"] = (H,)
            s[f"{p}.mix.norm"] = (inner,)
            s[f"{p}.mix.o"] = (W, inner)
        else:
            a, b = m["left"], m["right"]
            H, G, D, Dv = (int(a[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
            L, R = f"{p}.mix.left", f"{p}.mix.right"
            s[f"{L}.q"], s[f"{L}.k"], s[f"{L}.v"], s[f"{L}.g"] = (H * D, W), (G * D, W), (G * Dv, W), (H * Dv, W)
            s[f"{L}.pb"] = (H,)
            s[f"{L}.o"] = (W, H * Dv)
            H, G, D, Dv, K = (int(b[k]) for k in ("heads", "kv_heads", "dim", "vdim", "conv"))
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                s[f"{R}.{n}"] = (rows, W)
                s[f"{R}.{n}.conv"] = (rows, K)
            s[f"{R}.b"] = (H, W)
            s[f"{R}.A_log"] = (H,)
            s[f"{R}.norm"] = (Dv,)
            s[f"{R}.a1"], s[f"{R}.a2"], s[f"{R}.dt_bias"] = (rank_a, W), (H * D, rank_a), (H * D,)
            s[f"{R}.g1"], s[f"{R}.g2"] = (rank_g, W), (H * Dv, rank_g)
            s[f"{R}.o"] = (W, H * Dv)
            s[f"{L}.out"] = s[f"{R}.out"] = (W,)
        mlp = spec.get("mlp")
        if mlp is not None:
            s[f"{p}.norm2"] = (W,)
            ff, E = int(mlp["expert"]["ff"]), int(mlp["router"]["experts"])
            for e in range(E):
                s[f"{p}.mlp.e{e}.gate"] = s[f"{p}.mlp.e{e}.up"] = (ff, W)
                s[f"{p}.mlp.e{e}.down"] = (W, ff)
            s[f"{p}.mlp.router"], s[f"{p}.mlp.router.b"] = (E, W), (E,)
    return s


def random_weights(cfg: dict, seed: int = 0, dtype=torch.float64, rank_a: int = 6, rank_g: int = 10) -> Dict[str, torch.Tensor]:
    """weights that keep every mechanism visible in the logits; values are exactly representable in bfloat16"""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg, rank_a, rank_g).items():
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        if name == "embed":
            t = torch.randn(shape, generator=g) * 0.5
        elif leaf.endswith(".conv"):
            t = torch.randn(shape, generator=g) * 0.6
        elif leaf.endswith("router"):
            t = torch.randn(shape, generator=g) * (4.0 / math.sqrt(shape[1]))          # clear choices
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[1]))
        elif leaf.endswith("norm") or leaf.endswith("norm1") or leaf.endswith("norm2") or leaf.endswith(".out"):
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif leaf.endswith("temp"):
            t = 0.5 + torch.rand(shape, generator=g) * 3.0
        elif leaf.endswith("vmix"):
            t = torch.rand(shape, generator=g) * 0.8 + 0.1
        elif leaf.endswith("A_log"):
            t = torch.randn(shape, generator=g) * 0.7 - 1.0
        elif leaf.endswith("dt_bias"):
            t = torch.randn(shape, generator=g) - 1.0
        elif leaf.endswith(".D"):
            t = 1.0 + 0.5 * torch.randn(shape, generator=g)
        elif leaf.endswith("pb"):
            t = torch.randn(shape, generator=g) - 1.0
        else:
            t = torch.randn(shape, generator=g) * 0.5
        w[name] = t.to(torch.bfloat16).to(dtype)
    return w
