"""RMSNorm / SiluAndMul / rotary embedding modules over the HIP kernels.

Mirrors nn/layers/layernorm.py:12-32, nn/layers/activation.py:21-31 and
nn/layers/rotary_embedding.py:52-170, 677-720, 918-1088 (same class names, constructor
arguments, return conventions and in-place contracts)."""
import math
from typing import Any, Dict, Optional, Tuple, Union

import torch
import torch.nn as nn

from . import _native
from .custom_op import CustomOp


class RMSNorm(CustomOp):
    """layernorm.py:12-32.  With ``residual``: both tensors are updated IN PLACE and returned
    (flashinfer fused_add_rmsnorm contract); without: a new tensor is returned."""

    def __init__(self, hidden_size: int, eps: float = 1e-6) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size))
        self.variance_epsilon = eps

    def forward_hip(self, x: torch.Tensor, residual: Optional[torch.Tensor] = None
                    ) -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
        if residual is not None:
            _native.fused_add_rmsnorm(x, residual, self.weight.data, self.variance_epsilon)
            return x, residual
        return _native.rmsnorm(x, self.weight.data, self.variance_epsilon)


class ReluSquare(CustomOp):
    """max(x, 0)^2, element by element"""

    def forward_hip(self, x: torch.Tensor) -> torch.Tensor:
        return _native.relu_square(x)


class SiluAndMul(CustomOp):
    """activation.py:21-31: silu(x[..., :d]) * x[..., d:]."""

    def forward_hip(self, x: torch.Tensor) -> torch.Tensor:
        return _native.silu_and_mul(x)


class RotaryEmbedding(CustomOp):
    """rotary_embedding.py:52-170.  ``forward`` rotates query and key IN PLACE and returns them."""

    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: int,
                 is_neox_style: bool, dtype: torch.dtype) -> None:
        super().__init__()
        self.head_size = head_size
        self.rotary_dim = rotary_dim
        self.max_position_embeddings = max_position_embeddings
        self.base = base
        self.is_neox_style = is_neox_style
        self.dtype = dtype
        cache = self._compute_cos_sin_cache().to(dtype)
        self.cos_sin_cache: torch.Tensor
        self.register_buffer("cos_sin_cache", cache, persistent=False)

    def _compute_inv_freq(self, base: Union[int, float]) -> torch.Tensor:
        # rotary_embedding.py:77-90
        return 1.0 / (base ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float) / self.rotary_dim))

    def _compute_cos_sin_cache(self) -> torch.Tensor:
        # rotary_embedding.py:92-101 (fp32 on the host, once at init)
        inv_freq = self._compute_inv_freq(self.base)
        t = torch.arange(self.max_position_embeddings, dtype=torch.float)
        freqs = torch.einsum("i,j -> ij", t, inv_freq)
        return torch.cat((freqs.cos(), freqs.sin()), dim=-1)

    def forward_hip(self, positions: torch.Tensor, query: torch.Tensor, key: torch.Tensor,
                    offsets: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        if self.cos_sin_cache.device != query.device or self.cos_sin_cache.dtype != query.dtype:
            # rotary_embedding.py:141: the cache follows the activations' device and dtype
            self.cos_sin_cache = self.cos_sin_cache.to(query.device, dtype=query.dtype)
        if offsets is not None:
            positions = positions + offsets
        _native.rotary_embedding(positions, query, key, self.head_size, self.cos_sin_cache,
                                 self.is_neox_style)
        return query, key

    def extra_repr(self) -> str:
        return (f"head_size={self.head_size}, rotary_dim={self.rotary_dim}, "
                f"max_position_embeddings={self.max_position_embeddings}, base={self.base}, "
                f"is_neox_style={self.is_neox_style}")


class Llama3RotaryEmbedding(RotaryEmbedding):
    """rotary_embedding.py:677-720: wavelength-dependent rescale of inv_freq.

    Provenance: this is the public Llama-3.1 RoPE rescaling (Meta's reference implementation; the same formula in HF
    transformers `_compute_llama3_parameters` and in vLLM, from which the reference's class descends).  The cos/sin
    table has to equal the reference's bit for bit (tests/test_host_logic.py against rotary.npz), which fixes the order
    of the fp32 operations below; it runs once at init on the host and no kernel depends on it."""

    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: int,
                 is_neox_style: bool, dtype: torch.dtype, scaling_factor: float,
                 low_freq_factor: float, high_freq_factor: float, orig_max_position: int) -> None:
        self.scaling_factor = scaling_factor
        self.low_freq_factor = low_freq_factor
        self.high_freq_factor = high_freq_factor
        self.orig_max_position = orig_max_position
        super().__init__(head_size, rotary_dim, max_position_embeddings, base, is_neox_style, dtype)

    def _compute_inv_freq(self, base: Union[int, float]) -> torch.Tensor:
        inv_freqs = super()._compute_inv_freq(base)
        low_freq_wavelen = self.orig_max_position / self.low_freq_factor
        high_freq_wavelen = self.orig_max_position / self.high_freq_factor
        wave_len = 2 * math.pi / inv_freqs
        if self.low_freq_factor != self.high_freq_factor:
            smooth = (self.orig_max_position / wave_len - self.low_freq_factor) / (
                self.high_freq_factor - self.low_freq_factor)
        else:
            smooth = 0
        return torch.where(
            wave_len < high_freq_wavelen, inv_freqs,
            torch.where(wave_len > low_freq_wavelen, inv_freqs / self.scaling_factor,
                        (1 - smooth) * inv_freqs / self.scaling_factor + smooth * inv_freqs))


class ScaledRotaryEmbedding(RotaryEmbedding):
    """The context-extension variants get_rope hands out besides llama3 (rotary_embedding.py:173-414, 996-1036), as
    ONE table builder: a variant is (how the inverse frequencies are bent, what the positions are divided by, how long
    the table is, what cos / sin are multiplied by); the rotation kernel only ever sees the finished cos | sin table.

      "linear"  (position interpolation): positions / factor, table for max_pos * factor positions;
      "dynamic" (dynamic NTK): base * ((factor * len / max_pos) - (factor - 1)) ** (rot / (rot - 2)) with len =
                max_pos * factor - the reference evaluates the NTK base once, at the longest length;
      "yarn"    (Peng et al.): per-frequency blend of interpolated (1 / (factor * f)) and original (1 / f) inverse
                frequencies along a linear ramp between the dimensions that complete beta_fast and beta_slow
                rotations inside the ORIGINAL context, and cos / sin scaled by (0.1 ln(factor) + 1) * attn_factor.

    Public formulas (kaiokendev's interpolation; bloc97 / emozilla's NTK scaling; the YaRN paper and repository); the
    tables equal the reference classes' bit for bit (rotary.npz cases 6-10), which fixes the order of the fp32
    operations.  A LIST of linear factors (one table per LoRA adapter, rotary_embedding.py:173-258) is not built."""

    def __init__(self, head_size: int, rotary_dim: int, max_position_embeddings: int, base: int,
                 is_neox_style: bool, dtype: torch.dtype, kind: str, factor: float,
                 extrapolation_factor: float = 1, attn_factor: float = 1, beta_fast: int = 32,
                 beta_slow: int = 1) -> None:
        if kind not in ("linear", "dynamic", "yarn"):
            raise ValueError(f"Unknown RoPE scaling type {kind}")
        if isinstance(factor, (list, tuple)):
            raise NotImplementedError("several linear scaling factors in one table (per-LoRA tables) are not built")
        self.kind, self.scaling_factor = kind, factor
        self.yarn = (extrapolation_factor, attn_factor, beta_fast, beta_slow)
        self.mscale = float((0.1 * math.log(factor) + 1.0 if factor > 1 else 1.0) * attn_factor) if kind == "yarn" else 1.0
        super().__init__(head_size, rotary_dim, max_position_embeddings, base, is_neox_style, dtype)

    def _yarn_inv_freq(self) -> torch.Tensor:
        extrapolation_factor, _, beta_fast, beta_slow = self.yarn
        rot, base, ctx = self.rotary_dim, self.base, self.max_position_embeddings
        freq = base ** (torch.arange(0, rot, 2, dtype=torch.float) / rot)
        # the (fractional) dimension whose wavelength makes `turns` full rotations over the original context
        turn_dim = lambda turns: (rot * math.log(ctx / (turns * 2 * math.pi))) / (2 * math.log(base))
        lo = max(math.floor(turn_dim(beta_fast)), 0)
        hi = min(math.ceil(turn_dim(beta_slow)), rot - 1)
        if lo == hi:
            hi += 0.001
        ramp = torch.clamp((torch.arange(rot // 2, dtype=torch.float) - lo) / (hi - lo), 0, 1)
        keep = (1 - ramp) * extrapolation_factor                  # 1: the original frequency, 0: the interpolated one
        return (1.0 / (self.scaling_factor * freq)) * (1 - keep) + (1.0 / freq) * keep

    def _compute_cos_sin_cache(self) -> torch.Tensor:
        f, ctx = self.scaling_factor, self.max_position_embeddings
        length = ctx * f
        t = torch.arange(length, dtype=torch.float)
        if self.kind == "linear":
            inv_freq, t = self._compute_inv_freq(self.base), t / f
        elif self.kind == "dynamic":
            inv_freq = self._compute_inv_freq(
                self.base * ((f * length / ctx) - (f - 1)) ** (self.rotary_dim / (self.rotary_dim - 2)))
        else:
            inv_freq = self._yarn_inv_freq()
        freqs = torch.einsum("i,j -> ij", t, inv_freq)
        if self.kind == "yarn":
            return torch.cat((freqs.cos() * self.mscale, freqs.sin() * self.mscale), dim=-1)
        return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


_ROPE_DICT: Dict[Tuple, RotaryEmbedding] = {}


def get_rope(head_size: int, rotary_dim: int, max_position: int, base: int,
             is_neox_style: bool = True, rope_scaling: Optional[Dict[str, Any]] = None,
             dtype: Optional[torch.dtype] = None,
             partial_rotary_factor: float = 1.0) -> RotaryEmbedding:
    """rotary_embedding.py:918-1088: "default", "llama3" (the hot-path configs), "linear", "dynamic" and "yarn"
    (ScaledRotaryEmbedding); "deepseek_yarn", "longrope" and mrope raise (MLA / Phi-3 / Qwen2-VL: model families out
    of scope)."""
    if dtype is None:
        dtype = torch.get_default_dtype()
    if rope_scaling is not None:
        rope_scaling_args = tuple(
            (k, tuple(v) if isinstance(v, list) else v) for k, v in rope_scaling.items())
    else:
        rope_scaling_args = None
    if partial_rotary_factor < 1.0:
        rotary_dim = int(rotary_dim * partial_rotary_factor)
    key = (head_size, rotary_dim, max_position, base, is_neox_style, rope_scaling_args, dtype)
    if key in _ROPE_DICT:
        return _ROPE_DICT[key]
    scaling_type = None if rope_scaling is None else rope_scaling.get(
        "rope_type", rope_scaling.get("type"))
    if scaling_type in (None, "default"):
        rope = RotaryEmbedding(head_size, rotary_dim, max_position, base, is_neox_style, dtype)
    elif scaling_type == "llama3":
        rope = Llama3RotaryEmbedding(
            head_size, rotary_dim, max_position, base, is_neox_style, dtype,
            rope_scaling["factor"], rope_scaling["low_freq_factor"],
            rope_scaling["high_freq_factor"], rope_scaling["original_max_position_embeddings"])
    elif scaling_type in ("linear", "dynamic"):
        rope = ScaledRotaryEmbedding(head_size, rotary_dim, max_position, base, is_neox_style, dtype,
                                     scaling_type, rope_scaling["factor"])
    elif scaling_type == "yarn":
        # (the table is built over the ORIGINAL context times the factor: rotary_embedding.py:1018-1036)
        extra = {k: rope_scaling[k] for k in ("extrapolation_factor", "attn_factor", "beta_fast", "beta_slow")
                 if k in rope_scaling}
        rope = ScaledRotaryEmbedding(head_size, rotary_dim, rope_scaling["original_max_position_embeddings"], base,
                                     is_neox_style, dtype, "yarn", rope_scaling["factor"], **extra)
    else:
        raise ValueError(f"Unknown RoPE scaling type {scaling_type}")
    _ROPE_DICT[key] = rope
    return rope


# --------------------------------------------------------------------------- fp32-stream norms, PolyNorm, table-free rotary
class ScalarRMSNorm(nn.Module):
    """RMS norm with ONE gain for all coordinates, applied to a sublayer's OUTPUT before it joins an fp32 residual
    stream: ``add_into(x, y)`` is x += y / rms(y) * g in place and returns the new x in y's dtype (what the next
    projection reads); ``forward(x, dtype)`` is the plain norm of the stream (a model's final norm)."""

    def __init__(self, eps: float = 1e-6) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(1, dtype=torch.float32), requires_grad=False)
        self.variance_epsilon = eps

    def add_into(self, x: torch.Tensor, y: torch.Tensor, want_lo: bool = True) -> torch.Tensor:
        return _native.add_scalar_norm(x, y, self.weight.data, self.variance_epsilon, want_lo)

    def forward(self, x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        return _native.scalar_norm(x, self.weight.data, self.variance_epsilon, dtype)


class PolyNorm(nn.Module):
    """a N(z) + b N(z^2) + c N(z^3) + e with N = division by the root mean square over the row; weight = (a, b, c, e)"""

    def __init__(self, eps: float = 1e-6) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.tensor([1.0, 0.0, 0.0, 0.0], dtype=torch.float32), requires_grad=False)
        self.variance_epsilon = eps

    def forward(self, z: torch.Tensor) -> torch.Tensor:
        return _native.polynorm(z, self.weight.data, self.variance_epsilon)


def yarn_blend(dims: int, base: float, factor: float, original: float, fast: float, slow: float) -> torch.Tensor:
    """Rotary frequencies f_i = base^(-2i/dims), i < dims/2, blended with f_i / factor along a linear ramp between the
    (fractional) dimensions that complete `fast` and `slow` turns inside `original` positions: below the ramp the
    frequency stays, above it is divided by the factor.  float64."""
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)

    def dim_of(turns: float) -> float:
        return dims * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(dim_of(fast)), 0)
    hi = min(math.ceil(dim_of(slow)), dims - 1)
    ramp = torch.clamp((torch.arange(dims // 2, dtype=torch.float64) - lo) / max(hi - lo, 0.001), 0, 1)
    return f / factor * ramp + f * (1 - ramp)


def wavelength_blend(dims: int, base: float, factor: float, original: float, low: float, high: float) -> torch.Tensor:
    """Rotary frequencies f_i = base^(-2i/dims), i < dims/2, rescaled by their wavelength 2 pi / f (the rule of Llama 3.1's
    context extension): a wavelength below original / high keeps its frequency, one above original / low has it divided by
    ``factor``, and between the two the frequency is (1 - s) f / factor + s f with s = (original / wavelength - low) /
    (high - low).  float64."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        wavelength = 2 * math.pi / f
        if wavelength > original / low:
            f = f / factor
        elif wavelength >= original / high and high != low:
            s = (original / wavelength - low) / (high - low)
            f = (1 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


class AngleRotary(nn.Module):
    """Rotary embedding without a table: fp32 frequencies, the angle position * f_i formed in fp32 inside the kernel,
    interleaved pairs (2i, 2i+1) of the first ``dims`` coordinates, cos and sin scaled by ``magnitude``.  ``scaling`` =
    {factor, original, fast, slow} blends the frequencies (yarn_blend) and sets magnitude = 0.1 ln(factor) + 1;
    ``scaling`` = {factor, original, low, high} rescales them by wavelength (wavelength_blend), magnitude 1."""
    adjacent_pairs = True

    def __init__(self, dims: int, base: float, scaling: Optional[Dict[str, Any]] = None) -> None:
        super().__init__()
        if dims % 2:
            raise ValueError("rotary dims must be even")
        if scaling and "low" in scaling:
            freq = wavelength_blend(dims, base, float(scaling["factor"]), float(scaling["original"]), float(scaling["low"]),
                                    float(scaling["high"]))
            self.magnitude = 1.0
        elif scaling:
            freq = yarn_blend(dims, base, scaling["factor"], scaling["original"], scaling["fast"], scaling["slow"])
            self.magnitude = 0.1 * math.log(scaling["factor"]) + 1.0
        else:
            freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
            self.magnitude = 1.0
        self.dims = dims
        self.register_buffer("freq", freq.to(torch.float32), persistent=False)

    def forward(self, positions: torch.Tensor, x: torch.Tensor, offset: int = 0) -> None:
        """in place on x [T, H, n]: coordinates offset .. offset + dims of every head"""
        _native.rotary_interleaved(x, positions, self.freq, self.magnitude, offset)


class HalfAngleRotary(AngleRotary):
    """The same fp32 frequencies and magnitude, for the "rotate half" pairing: coordinate i < dims / 2 pairs with
    i + dims / 2.  Applied by the fused rotation + cache store (_native.qkv_rotary_store), not by a call of its own."""
    adjacent_pairs = False

    def forward(self, positions: torch.Tensor, x: torch.Tensor, offset: int = 0) -> None:
        raise NotImplementedError("the half-pair rotation runs inside _native.qkv_rotary_store")


class ShiftedRMSNorm(nn.Module):
    """Weighted RMS norm of an fp32 residual stream followed by a token shift: h = x / rms(x) * weight is what a layer's
    feed-forward reads, hs = h + (h[t-1] - h) * mu what its mixer reads; h[t-1] before a step's first row is the request's
    saved h (RecurrentStatePool.shift_state; zeros for a sequence's first token).  Both come out in the projections'
    dtype; the arithmetic and the saved row are fp32.  Without ``shift`` it is a plain weighted norm (a model's last)."""

    def __init__(self, width: int, eps: float = 1e-6, shift: bool = True, layer_id: Optional[int] = None) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(width, dtype=torch.float32), requires_grad=False)
        self.mu = nn.Parameter(torch.zeros(width, dtype=torch.float32), requires_grad=False) if shift else None
        self.variance_epsilon, self.layer_id = eps, layer_id

    def forward(self, x: torch.Tensor, dtype: torch.dtype, forward_batch=None, want_h: bool = True):
        if self.mu is None:
            return _native.norm_shift(x, self.weight.data, self.variance_epsilon, dtype)[0]
        return _native.norm_shift(x, self.weight.data, self.variance_epsilon, dtype, self.mu.data,
                                  forward_batch.state_pool.shift_state(self.layer_id), forward_batch.attn_backend.seq, want_h)


class GluFF(nn.Module):
    """Gated feed-forward with the gate and up projections as ONE product: act = "silu": W_down (silu(g) * u);
    act = "clamped": g' = min(g, limit), u' = clamp(u, -limit, limit), W_down (g' * sigmoid(alpha g') * (u' + 1))."""

    def __init__(self, width: int, ff: int, act: str = "silu", limit: float = 0.0, alpha: float = 1.702, dtype=None):
        super().__init__()
        if act not in ("silu", "clamped"):
            raise ValueError(f"unknown activation {act!r}")
        self.ff, self.act, self.limit, self.alpha = ff, act, limit, alpha
        self.gate_up = nn.Parameter(torch.empty(2 * ff, width, dtype=dtype), requires_grad=False)
        self.down = nn.Parameter(torch.empty(width, ff, dtype=dtype), requires_grad=False)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        gu = _native.linear(h, self.gate_up)
        y = _native.silu_and_mul(gu) if self.act == "silu" else _native.moe_glu(gu.contiguous(), self.limit, self.alpha)
        return _native.linear(y, self.down)


class GatedAddNorm(nn.Module):
    """How a sublayer's result y joins an fp32 residual stream when it is gated and normed first:
    x += N(y * sigmoid(gate + bias)) * weight, N = division by the row's root mean square.  The gate's pre-activation is a
    product of the sublayer's own input, so its rows ride in the sublayer's input projection and arrive here as ``gate``.
    ``y`` may be two branches (a, b), each normed over the row with its own weight and averaged: y = (N(a) wa + N(b) wb) / 2.
    ``extra`` (fp32) is added to the stream afterwards; with ``next_weight`` the call also returns N(x) * next_weight in the
    projections' dtype - the next sublayer's input - from the same pass over the row."""

    def __init__(self, width: int, eps: float = 1e-6, gated: bool = True, branches: int = 1) -> None:
        super().__init__()
        f32 = dict(dtype=torch.float32)
        self.weight = nn.Parameter(torch.ones(width, **f32), requires_grad=False)
        self.gate_bias = nn.Parameter(torch.zeros(width, **f32), requires_grad=False) if gated else None
        self.branch_weight = nn.Parameter(torch.ones(2, width, **f32), requires_grad=False) if branches == 2 else None
        self.variance_epsilon = eps

    def forward(self, x: torch.Tensor, y, gate: Optional[torch.Tensor] = None, extra: Optional[torch.Tensor] = None,
                next_weight: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        a, b = y if isinstance(y, (tuple, list)) else (y, None)
        if (b is not None) != (self.branch_weight is not None):
            raise RuntimeError("GatedAddNorm: built for another number of branches")
        wa, wb = (self.branch_weight.data[0], self.branch_weight.data[1]) if b is not None else (None, None)
        return _native.gated_add_norm(x, a, self.weight.data, self.variance_epsilon, gate=gate,
                                      gate_bias=None if self.gate_bias is None else self.gate_bias.data, b=b, wa=wa, wb=wb,
                                      extra=extra, next_weight=next_weight)


class GroupRMSNorm(nn.Module):
    """Weighted RMS norm of an fp32 residual stream taken in ``groups`` equal consecutive parts of the row, each divided by
    its own root mean square; fused with the sum that precedes it in a pre-norm layer: ``forward(x, dtype, y)`` adds a
    sublayer's result y to the stream in place first (two branches (a, b) with ``branch_weights`` (wa, wb): each normed
    over the whole row with its weight, then averaged) and returns GN(x) * weight in the projections' dtype."""

    def __init__(self, width: int, groups: int = 1, eps: float = 1e-6) -> None:
        super().__init__()
        if width % groups:
            raise ValueError("the width must divide into the norm's groups")
        self.weight = nn.Parameter(torch.ones(width, dtype=torch.float32), requires_grad=False)
        self.groups, self.variance_epsilon = groups, eps

    def forward(self, x: torch.Tensor, dtype: torch.dtype, y=None, branch_weights=None) -> torch.Tensor:
        return add_join(x, y, branch_weights, self.groups, self.variance_epsilon, dtype, self.weight.data)


def add_join(x: torch.Tensor, y, branch_weights, groups: int, eps: float, dtype: torch.dtype,
             next_weight: Optional[torch.Tensor] = None):
    """x += y in place (y one tensor, or two branches each normed over the row with its weight and averaged), then,
    with ``next_weight``, the group norm of the new x times that weight"""
    a, b = y if isinstance(y, (tuple, list)) else (y, None)
    wa, wb = branch_weights if b is not None else (None, None)
    return _native.add_group_norm(x, a, groups, eps, dtype, b=b, wa=wa, wb=wb, next_weight=next_weight)


class ReluSquareFF(nn.Module):
    """Feed-forward W_down relu(W_up h)^2.  ``extra_rows`` further rows of the up projection are not activated: their
    outputs come back beside the result (a layer's gate on this sublayer reads the same h, so it rides in this product)."""

    def __init__(self, width: int, ff: int, extra_rows: int = 0, dtype=None):
        super().__init__()
        self.ff, self.extra_rows = ff, extra_rows
        self.up = nn.Parameter(torch.empty(ff + extra_rows, width, dtype=dtype), requires_grad=False)
        self.down = nn.Parameter(torch.empty(width, ff, dtype=dtype), requires_grad=False)
        self.act = ReluSquare()

    def forward(self, h: torch.Tensor):
        a = _native.linear(h, self.up)
        y = _native.linear(self.act(a[:, :self.ff]), self.down)
        return (y, a[:, self.ff:]) if self.extra_rows else y
