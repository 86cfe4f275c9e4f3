"""Mixture-of-experts feed-forward over the HIP kernels of csrc/moe.hip: an fp32 router (sigmoid scores, a choice
correction, optional group-limited choice), the step's (token, expert) pairs ordered by expert on the device, two grouped
matrix products around the clamped gated activation, and the weighted sum of each token's experts in a fixed order."""
import torch
from torch import nn

from . import _native


class GroupLimitedRouter(nn.Module):
    """ids, weights = top-`top` experts by sigmoid(W x) + correction (weights: the sigmoid without it, not renormalised);
    with `groups` > 1 only experts of the `keep` groups with the largest sum of their two best choices compete."""

    def __init__(self, width: int, experts: int, top: int, groups: int = 1, keep: int = 1):
        super().__init__()
        self.experts, self.top, self.groups, self.keep = experts, top, groups, keep
        self.weight = nn.Parameter(torch.zeros(experts, width, dtype=torch.float32), requires_grad=False)
        self.correction = nn.Parameter(torch.zeros(experts, dtype=torch.float32), requires_grad=False)

    def forward(self, x: torch.Tensor):
        return _native.moe_route(x, self.weight.data, self.correction.data, self.top, self.groups, self.keep)


class ClampedGluExperts(nn.Module):
    """Experts y = W_down (g * sigmoid(alpha g) * (u + 1)), g = min(W_gate x, limit), u = clamp(W_up x, +-limit);
    gate_up [E, 2 ff, W] holds each expert's gate rows, then its up rows."""

    def __init__(self, width: int, experts: int, ff: int, limit: float, alpha: float = 1.702, dtype=None):
        super().__init__()
        self.experts, self.ff, self.limit, self.alpha = experts, ff, limit, alpha
        self.gate_up = nn.Parameter(torch.empty(experts, 2 * ff, width, dtype=dtype), requires_grad=False)
        self.down = nn.Parameter(torch.empty(experts, width, ff, dtype=dtype), requires_grad=False)

    def activation(self, gu: torch.Tensor) -> torch.Tensor:
        return _native.moe_glu(gu, self.limit, self.alpha)

    def forward(self, x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
        top = ids.shape[1]
        pairs = ids.numel()
        offsets, order, place = _native.moe_align(ids, self.experts)
        gu = _native.moe_grouped_gemm(x, self.gate_up.data, offsets, pairs, order, top)
        y = self.activation(gu)
        z = _native.moe_grouped_gemm(y, self.down.data, offsets, pairs)
        return _native.moe_combine(z, place, weights)


class SparseMoE(nn.Module):
    def __init__(self, width: int, experts: int, top: int, ff: int, limit: float, groups: int = 1, keep: int = 1,
                 dtype=None):
        super().__init__()
        self.router = GroupLimitedRouter(width, experts, top, groups, keep)
        self.experts = ClampedGluExperts(width, experts, ff, limit, dtype=dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        ids, weights = self.router(x)
        return self.experts(x, ids, weights)


class SoftmaxRouter(nn.Module):
    """ids, weights = the `top` experts with the largest softmax(W x) over ALL experts (fp32 logits); the weights are
    those scores times `scale`, not renormalised over the chosen ones.  ``bias``: the logits are W x + b.  ``renorm``:
    the weights are the softmax over the CHOSEN logits only (they sum to `scale`)."""

    def __init__(self, width: int, experts: int, top: int, scale: float = 1.0, bias: bool = False, renorm: bool = False):
        super().__init__()
        self.experts, self.top, self.scale, self.renorm = experts, top, scale, renorm
        self.weight = nn.Parameter(torch.zeros(experts, width, dtype=torch.float32), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(experts, dtype=torch.float32), requires_grad=False) if bias else None

    def forward(self, x: torch.Tensor):
        return _native.moe_route_softmax(x, self.weight.data, self.top, self.scale,
                                         None if self.bias is None else self.bias.data, self.renorm)


class SiluGluExperts(ClampedGluExperts):
    """Experts y = W_down (silu(W_gate x) * (W_up x)): the same stacked layout and grouped products, no clamps."""

    def __init__(self, width: int, experts: int, ff: int, dtype=None):
        super().__init__(width, experts, ff, 0.0, dtype=dtype)

    def activation(self, gu: torch.Tensor) -> torch.Tensor:
        return _native.silu_and_mul(gu)


class SoftmaxMoE(nn.Module):
    """SoftmaxRouter + SiluGluExperts; `forward` returns the routed experts' weighted sum (a shared expert, if the model
    has one, is a dense feed-forward of its own beside this)."""

    def __init__(self, width: int, experts: int, top: int, ff: int, scale: float = 1.0, dtype=None):
        super().__init__()
        self.router = SoftmaxRouter(width, experts, top, scale)
        self.experts = SiluGluExperts(width, experts, ff, dtype=dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        ids, weights = self.router(x)
        return self.experts(x, ids, weights)


class ChosenSoftmaxMoE(nn.Module):
    """Experts chosen by the largest router logits W x + b and weighted by the softmax over the chosen logits only, each a
    clamped gated unit (ClampedGluExperts); `forward` returns their weighted sum."""

    def __init__(self, width: int, experts: int, top: int, ff: int, limit: float, dtype=None):
        super().__init__()
        self.router = SoftmaxRouter(width, experts, top, bias=True, renorm=True)
        self.experts = ClampedGluExperts(width, experts, ff, limit, dtype=dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        ids, weights = self.router(x)
        return self.experts(x, ids, weights)
