"""Recurrent token mixers over per-request state in the RecurrentStatePool: WKVMixer (RWKV-style time mixing, csrc/wkv.hip),
Mamba2Mixer (state-space duality form, csrc/ssm.hip), MLSTMMixer (matrix memory with exponential gating, csrc/mlstm.hip),
GeneralDeltaMixer (generalized delta rule, csrc/delta_rule.hip), HGRN2Mixer (linear attention whose forget gate also
writes, csrc/hgrn.hip) and GatedDeltaMixer (delta rule with a decay per key channel, csrc/gated_delta.hip).

WKVMixer:

Per token t with layer input h[t] (the fp32 residual stream) and h[t-1] (zeros at a sequence's first token):
  m_s = h[t] + (h[t-1] - h[t]) * mu_s                      one mix per projection s in (r, k, v, g, w)
  r, k, v = W_r m_r, W_k m_k, W_v m_v   gate = silu(W_g m_g)   decay = exp(-exp(W_w2 tanh(W_w1 m_w) + w0))
  o = (S + diag(u) k v^T)^T r ;  S <- diag(decay) S + k v^T     per head, S in fp32 in the RecurrentStatePool
  out = W_o ((o / rms_head(o)) * norm * gate)
The four projections that feed the recurrence run as ONE batched matrix product over their stacked weights."""
import math
from typing import Optional

import torch
from torch import nn

from . import _native
from .forward_info import ForwardBatch


class WKVMixer(nn.Module):
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, width: int, heads: int, dim: int, decay_rank: int, layer_id: int, eps: float, dtype=None):
        super().__init__()
        self.width, self.heads, self.dim, self.layer_id, self.eps = width, heads, dim, layer_id, eps
        n = heads * dim
        f32 = dict(dtype=torch.float32)
        self.mu = nn.Parameter(torch.zeros(len(self.MIXES), width, **f32), requires_grad=False)
        self.rkvg = nn.Parameter(torch.empty(4, n, width, dtype=dtype), requires_grad=False)
        self.w1 = nn.Parameter(torch.empty(decay_rank, width, dtype=dtype), requires_grad=False)
        self.w2t = nn.Parameter(torch.zeros(decay_rank, n, **f32), requires_grad=False)      # W_w2 transposed, fp32
        self.w0 = nn.Parameter(torch.zeros(n, **f32), requires_grad=False)
        self.u = nn.Parameter(torch.zeros(heads, dim, **f32), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(n, **f32), requires_grad=False)
        self.o = nn.Parameter(torch.empty(width, n, dtype=dtype), requires_grad=False)

    def forward(self, x: torch.Tensor, forward_batch: ForwardBatch) -> torch.Tensor:
        """x: the fp32 stream [T, W] -> the mixer's output [T, W] in the projections' dtype"""
        seq = forward_batch.attn_backend.seq
        states = forward_batch.state_pool
        dtype = self.o.dtype
        shift = states.shift_state(self.layer_id)
        mixes = _native.token_shift(x, self.mu.data, shift, seq, dtype)               # [5, T, W]
        _native.save_last_rows(shift, x, seq)                                         # after its only reader this step
        rkvg = torch.bmm(mixes[:4], self.rkvg.transpose(1, 2))                        # [4, T, H * D]
        decay = _native.wkv_decay(_native.linear(mixes[4], self.w1), self.w2t.data, self.w0.data)
        o = _native.wkv_recurrence(rkvg[0], rkvg[1], rkvg[2], rkvg[3], decay, self.u.data, self.norm.data,
                                   states.matrix_state(self.layer_id), seq, self.heads, self.dim, self.eps)
        return _native.linear(o, self.o)


class Mamba2Mixer(nn.Module):
    """State-space mixer.  With inner = heads * vdim, N = state, G = groups, the input projection's rows are
    [z: inner | x: inner | B: G N | C: G N | dt: heads]; x, B, C pass a causal per-channel convolution (its latest
    taps - 1 inputs are request state) and silu; per head h (group h // (heads / G)), in fp32:
      dt = softplus(dt + dt_bias)    S <- exp(-exp(A_log) dt) S + dt B x^T    y = S^T C + D x        (S [N, vdim])
    then out = W_o (groupnorm(y * silu(z)) * norm): the gate before the norm, ``norm_groups`` equal parts.
    The dt rows of the projection are kept apart in fp32 (a step size is never rounded to 16 bits)."""

    def __init__(self, width: int, heads: int, vdim: int, state: int, groups: int, taps: int, norm_groups: int,
                 layer_id: int, eps: float, dtype=None):
        super().__init__()
        if heads % groups or (heads * vdim) % norm_groups:
            raise ValueError("heads must divide into groups, heads * vdim into norm_groups")
        self.heads, self.vdim, self.state, self.groups, self.taps = heads, vdim, state, groups, taps
        self.norm_groups, self.layer_id, self.eps = norm_groups, layer_id, eps
        inner, ch = heads * vdim, heads * vdim + 2 * groups * state
        f32 = dict(dtype=torch.float32)
        self.in_proj = nn.Parameter(torch.empty(inner + ch, width, dtype=dtype), requires_grad=False)     # [z | x | B | C]
        self.dt_proj = nn.Parameter(torch.zeros(heads, width, **f32), requires_grad=False)
        self.conv = nn.Parameter(torch.zeros(ch, taps, **f32), requires_grad=False)
        self.conv_bias = nn.Parameter(torch.zeros(ch, **f32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(heads, **f32), requires_grad=False)
        self.A_log = nn.Parameter(torch.zeros(heads, **f32), requires_grad=False)
        self.D = nn.Parameter(torch.ones(heads, **f32), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(inner, **f32), requires_grad=False)
        self.o = nn.Parameter(torch.empty(width, inner, dtype=dtype), requires_grad=False)

    @staticmethod
    def state_shapes(heads: int, vdim: int, state: int, groups: int, taps: int):
        return {"ssm": (heads, state, vdim), "conv": (max(taps - 1, 0), heads * vdim + 2 * groups * state)}

    def forward(self, h: torch.Tensor, forward_batch: ForwardBatch) -> torch.Tensor:
        seq, states = forward_batch.attn_backend.seq, forward_batch.state_pool
        inner = self.heads * self.vdim
        zxbc = _native.linear(h, self.in_proj)
        dt = _native.small_linear_f32(h, self.dt_proj.data)
        xbc = _native.causal_conv_silu(zxbc[:, inner:], self.conv.data, self.conv_bias.data,
                                       states.state(self.layer_id, "conv"), seq)
        y = _native.mamba2_scan(xbc, dt, self.dt_bias.data, self.A_log.data, self.D.data, states.state(self.layer_id, "ssm"),
                                seq, self.heads, self.groups, self.state, self.vdim)
        return _native.linear(_native.gated_group_norm(y, zxbc[:, :inner], self.norm.data, self.norm_groups, self.eps), self.o)


class MLSTMMixer(nn.Module):
    """Matrix-memory mixer with exponential gating.  q, k [heads, dim], v [heads, vdim], an output gate g and, per head, a
    log input gate i = cap tanh((W_i h + b_i) / cap) and a log forget gate f = logsigmoid(cap tanh((W_f h + b_f) / cap));
    with a running maximum m (0 for a new sequence):  m' = max(f + m, i),  S <- exp(f + m - m') S + exp(i - m') k v^T,
    n likewise with k,  o = S^T q / (max(|n . q|, exp(-m')) + 1e-6) with q scaled by dim^(-1/2);
    out = W_o (o / rms_head(o) * norm * sigmoid(g)).  q, k, v, g come from ONE product; the gate rows are a separate fp32
    product (a gate is never rounded to 16 bits)."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, gate_cap: float, layer_id: int, eps: float, dtype=None):
        super().__init__()
        self.heads, self.dim, self.vdim, self.cap, self.layer_id, self.eps = heads, dim, vdim, gate_cap, layer_id, eps
        f32 = dict(dtype=torch.float32)
        self.qkvg = nn.Parameter(torch.empty(2 * heads * dim + 2 * heads * vdim, width, dtype=dtype), requires_grad=False)
        self.gates = nn.Parameter(torch.zeros(2 * heads, width, **f32), requires_grad=False)       # [i rows | f rows]
        self.gates_bias = nn.Parameter(torch.zeros(2 * heads, **f32), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(heads * vdim, **f32), requires_grad=False)
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype), requires_grad=False)

    @staticmethod
    def state_shapes(heads: int, dim: int, vdim: int):
        return {"S": (heads, dim, vdim), "n": (heads, dim), "m": (heads,)}

    def forward(self, h: torch.Tensor, forward_batch: ForwardBatch) -> torch.Tensor:
        seq, states = forward_batch.attn_backend.seq, forward_batch.state_pool
        nk, nv, H = self.heads * self.dim, self.heads * self.vdim, self.heads
        a = _native.linear(h, self.qkvg)
        gates = _native.small_linear_f32(h, self.gates.data, self.gates_bias.data)
        ipre, fpre = gates[:, :H].contiguous(), gates[:, H:].contiguous()
        L = self.layer_id
        o = _native.mlstm_scan(a[:, :nk], a[:, nk:2 * nk], a[:, 2 * nk:2 * nk + nv], a[:, 2 * nk + nv:], ipre, fpre,
                               self.norm.data, states.state(L, "S"), states.state(L, "n"), states.state(L, "m"), seq,
                               self.heads, self.dim, self.vdim, self.cap, self.eps)
        return _native.linear(o, self.o)


class GeneralDeltaMixer(nn.Module):
    """Generalized delta rule.  r, k, v [heads, dim] and an output gate g are projections of h; per head and key channel a
    decay w = exp(-rate sigmoid(W_w2 tanh(W_w1 h) + w0)) and a removal rate a = sigmoid(W_a h + a_bias); with the unit key
    u = k / sqrt(|k|^2 + 1e-6), in fp32:
        S <- diag(w) S - (a * u)(u^T S) + k v^T   (both first terms read the previous S),   o = S^T r,
    out = W_o (o / rms_head(o) * norm * sigmoid(g)).  r, k, v, g, the removal rate's and the decay's first projection
    come from ONE product (rows [r | k | v | g | a | w1 | extra]); ``extra_rows`` further rows of that product are handed
    back untouched (a layer's gate on this sublayer reads the same h).  The decay's second projection is fp32."""

    def __init__(self, width: int, heads: int, dim: int, decay_rank: int, eps: float, rate: float = math.exp(-0.5),
                 layer_id: Optional[int] = None, extra_rows: int = 0, dtype=None):
        super().__init__()
        self.width, self.heads, self.dim, self.rank, self.eps, self.rate = width, heads, dim, decay_rank, eps, rate
        self.layer_id, self.extra_rows = layer_id, extra_rows
        n = heads * dim
        f32 = dict(dtype=torch.float32)
        self.in_proj = nn.Parameter(torch.empty(5 * n + decay_rank + extra_rows, width, dtype=dtype), requires_grad=False)
        self.w2t = nn.Parameter(torch.zeros(decay_rank, n, **f32), requires_grad=False)      # W_w2 transposed, fp32
        self.w0 = nn.Parameter(torch.zeros(n, **f32), requires_grad=False)
        self.a_bias = nn.Parameter(torch.zeros(n, **f32), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(n, **f32), requires_grad=False)
        self.o = nn.Parameter(torch.empty(width, n, dtype=dtype), requires_grad=False)

    @staticmethod
    def state_shapes(heads: int, dim: int):
        return {"S": (heads, dim, dim)}

    def forward(self, h: torch.Tensor, forward_batch: ForwardBatch, state_id: Optional[int] = None):
        """h [T, W] in the projections' dtype -> the mixer's output [T, W] (and the extra rows' outputs [T, extra_rows]).
        ``state_id``: the state to use instead of ``layer_id`` (a layer that runs several times on the same weights keeps one
        state per run)."""
        seq, states = forward_batch.attn_backend.seq, forward_batch.state_pool
        n = self.heads * self.dim
        a = _native.linear(h, self.in_proj)
        decay, remove = _native.delta_gates(a[:, 5 * n:5 * n + self.rank], self.w2t.data, self.w0.data, a[:, 4 * n:5 * n],
                                            self.a_bias.data, self.rate)
        S = states.state(self.layer_id if state_id is None else state_id, "S")
        o = _native.delta_recurrence(a[:, :n], a[:, n:2 * n], a[:, 2 * n:3 * n], a[:, 3 * n:4 * n], decay, remove,
                                     self.norm.data, S, seq, self.heads, self.dim, self.eps)
        y = _native.linear(o, self.o)
        return (y, a[:, 5 * n + self.rank:]) if self.extra_rows else y


class HGRN2Mixer(nn.Module):
    """Linear attention in which the forget gate also decides what is written.  q = silu(W_q h) [heads, dim], v = W_v h
    [heads, vdim], f = lower + (1 - lower) sigmoid(W_f h + f_bias) per head and query channel; in fp32
        S <- diag(f) S + (1 - f) v^T,   o = S^T q          (S [dim, vdim]; no key, no other scale)
    out = W_o (o / rms_head(o) * norm), norm [vdim] shared by the heads.  The rows [q | f | v] of the input projection may
    be part of a larger product of the caller (``scan`` takes the three views); ``forward`` runs the mixer's own."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, eps: float, layer_id: Optional[int] = None,
                 own_input: bool = True, dtype=None):
        super().__init__()
        self.heads, self.dim, self.vdim, self.eps, self.layer_id = heads, dim, vdim, eps, layer_id
        f32 = dict(dtype=torch.float32)
        self.in_rows = 2 * heads * dim + heads * vdim
        self.in_proj = nn.Parameter(torch.empty(self.in_rows, width, dtype=dtype), requires_grad=False) if own_input else None
        self.f_bias = nn.Parameter(torch.zeros(heads * dim, **f32), requires_grad=False)
        self.lower = nn.Parameter(torch.zeros(heads * dim, **f32), requires_grad=False)
        self.norm = nn.Parameter(torch.ones(vdim, **f32), requires_grad=False)
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype), requires_grad=False)

    @staticmethod
    def state_shapes(heads: int, dim: int, vdim: int):
        return {"S": (heads, dim, vdim)}

    def scan(self, a: torch.Tensor, forward_batch: ForwardBatch, state_id: Optional[int] = None) -> torch.Tensor:
        """a [T, >= in_rows]: the outputs of the rows [q | f | v] -> the mixer's output [T, W]"""
        seq, states = forward_batch.attn_backend.seq, forward_batch.state_pool
        nk = self.heads * self.dim
        S = states.state(self.layer_id if state_id is None else state_id, "S")
        o = _native.hgrn2_scan(a[:, :nk], a[:, nk:2 * nk], a[:, 2 * nk:self.in_rows], self.f_bias.data, self.lower.data,
                               self.norm.data, S, seq, self.heads, self.dim, self.vdim, self.eps)
        return _native.linear(o, self.o)

    def forward(self, h: torch.Tensor, forward_batch: ForwardBatch, state_id: Optional[int] = None) -> torch.Tensor:
        return self.scan(_native.linear(h, self.in_proj), forward_batch, state_id)


class GatedDeltaMixer(nn.Module):
    """Delta rule with a decay per head and key channel.  q, k [kv_heads, dim] and v [heads, vdim] are projections of h that
    pass a causal per-channel convolution of ``taps`` taps (no bias; its latest taps - 1 inputs are request state) and silu;
    value head h reads query/key head h // (heads / kv_heads).  In fp32, per head:
        qn = q / sqrt(|q|^2 + 1e-6) dim^(-1/2),   kn = k / sqrt(|k|^2 + 1e-6),   beta = sigmoid(W_b h)
        w  = exp(-exp(A_log) softplus(W_a2 (W_a1 h) + dt_bias))                    [dim] per head
        S <- diag(w) S;   u = beta (v - S^T kn);   S <- S + kn u^T;   o = S^T qn   (S [dim, vdim])
    out = W_o (o / rms_head(o) * norm * sigmoid(W_g2 (W_g1 h))), norm [vdim] shared by the heads.  The rows
    [q | k | v | b | a1 | g1] of the input projection may be part of a larger product of the caller (``scan`` takes the
    views); ``forward`` runs the mixer's own.  The second projections of decay and gate are fp32."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, taps: int, decay_rank: int, gate_rank: int,
                 eps: float, layer_id: Optional[int] = None, own_input: bool = True, dtype=None):
        super().__init__()
        if heads % kv_heads:
            raise ValueError("value heads must be a multiple of query/key heads")
        self.heads, self.kv_heads, self.dim, self.vdim, self.taps, self.eps = heads, kv_heads, dim, vdim, taps, eps
        self.decay_rank, self.gate_rank, self.layer_id = decay_rank, gate_rank, layer_id
        self.conv_rows = 2 * kv_heads * dim + heads * vdim
        self.in_rows = self.conv_rows + heads + decay_rank + gate_rank
        f32 = dict(dtype=torch.float32)
        self.in_proj = nn.Parameter(torch.empty(self.in_rows, width, dtype=dtype), requires_grad=False) if own_input else None
        self.conv = nn.Parameter(torch.zeros(self.conv_rows, taps, **f32), requires_grad=False)
        self.a2t = nn.Parameter(torch.zeros(decay_rank, heads * dim, **f32), requires_grad=False)      # W_a2 transposed
        self.dt_bias = nn.Parameter(torch.zeros(heads * dim, **f32), requires_grad=False)
        self.A_log = nn.Parameter(torch.zeros(heads, **f32), requires_grad=False)
        self.g2t = nn.Parameter(torch.zeros(gate_rank, heads * vdim, **f32), requires_grad=False)      # W_g2 transposed
        self.norm = nn.Parameter(torch.ones(vdim, **f32), requires_grad=False)
        self.o = nn.Parameter(torch.empty(width, heads * vdim, dtype=dtype), requires_grad=False)

    @staticmethod
    def state_shapes(heads: int, kv_heads: int, dim: int, vdim: int, taps: int):
        return {"S": (heads, dim, vdim), "conv": (max(taps - 1, 0), 2 * kv_heads * dim + heads * vdim)}

    def scan(self, a: torch.Tensor, forward_batch: ForwardBatch, state_id: Optional[int] = None) -> torch.Tensor:
        """a [T, >= in_rows]: the outputs of the rows [q | k | v | b | a1 | g1] -> the mixer's output [T, W]"""
        seq, states = forward_batch.attn_backend.seq, forward_batch.state_pool
        sid = self.layer_id if state_id is None else state_id
        nk, H, c = self.kv_heads * self.dim, self.heads, self.conv_rows
        qkv = _native.causal_conv_silu(a[:, :c], self.conv.data, None, states.state(sid, "conv"), seq)
        decay = _native.lowrank_gate(a[:, c + H:c + H + self.decay_rank], self.a2t.data, self.dt_bias.data, "decay",
                                     self.A_log.data)
        gate = _native.lowrank_gate(a[:, c + H + self.decay_rank:self.in_rows], self.g2t.data, None, "sigmoid")
        o = _native.gated_delta_scan(qkv[:, :nk], qkv[:, nk:2 * nk], qkv[:, 2 * nk:], a[:, c:c + H], decay, gate,
                                     self.norm.data, states.state(sid, "S"), seq, H, self.kv_heads, self.dim, self.vdim,
                                     self.eps)
        return _native.linear(o, self.o)

    def forward(self, h: torch.Tensor, forward_batch: ForwardBatch, state_id: Optional[int] = None) -> torch.Tensor:
        return self.scan(_native.linear(h, self.in_proj), forward_batch, state_id)
