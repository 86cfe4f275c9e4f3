"""The Kikurax kernels at the layer sizes of real models (bf16 and fp32), each against a plain fp32 torch expression of
the same operation evaluated on the GPU: several requests of unequal length in one launch, a second launch that goes on from
the states the first one left.  Every case prints its name before it launches."""
import pytest
import torch

from tests.test_gpu_toredra_kernels import DEV, announce, close, rms, seq_extend

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,bar", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,G,D,Dv", [(16, 8, 128, 128), (8, 8, 64, 256), (32, 4, 64, 64)])
def test_gated_delta_scan_at_model_size(dtype, bar, H, G, D, Dv):
    from scratchpad_amd import _native
    lens, slots = [500, 1, 223], [3, 1, 4]
    T = sum(lens)
    announce("gated_delta_scan", dtype, "heads", H, "kv heads", G, "dim", D, "vdim", Dv, "tokens", lens)
    g = torch.Generator(device=DEV).manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV)
    state = torch.full((6, H, D, Dv), float("nan"), device=DEV)
    S = {s: torch.zeros(H, D, Dv, device=DEV) for s in slots}
    rep = H // G
    for launch, prefixes in enumerate(([0, 0, 0], lens)):                      # the second launch goes on from the first's states
        q, k = (rn(T, G * D).mul_(0.5).to(dtype) for _ in range(2))
        v, bpre = rn(T, H * Dv).mul_(0.5).to(dtype), rn(T, H).to(dtype)
        decay = torch.rand(T, H * D, generator=g, device=DEV) * 0.3 + 0.7
        gate = torch.rand(T, H * Dv, generator=g, device=DEV)
        nw = torch.rand(Dv, generator=g, device=DEV) + 0.5
        got = _native.gated_delta_scan(q, k, v, bpre, decay, gate, nw, state, seq_extend(lens, prefixes, slots), H, G, D, Dv, 1e-5)
        want = torch.empty(T, H, Dv, device=DEV)
        at = 0
        for m, slot in zip(lens, slots):
            qq, kk = (t[at:at + m].float().view(m, G, D).repeat_interleave(rep, 1) for t in (q, k))
            vv, ww, bb = v[at:at + m].float().view(m, H, Dv), decay[at:at + m].view(m, H, D), torch.sigmoid(bpre[at:at + m].float())
            qq = qq / torch.sqrt((qq * qq).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
            kk = kk / torch.sqrt((kk * kk).sum(-1, keepdim=True) + 1e-6)
            for t in range(m):
                Sd = ww[t].unsqueeze(-1) * S[slot]
                u = bb[t].unsqueeze(-1) * (vv[t] - torch.einsum("hij,hi->hj", Sd, kk[t]))
                S[slot] = Sd + kk[t].unsqueeze(-1) * u.unsqueeze(-2)
                want[at + t] = torch.einsum("hij,hi->hj", S[slot], qq[t])
            close(state[slot], S[slot], 1e-3 if dtype == torch.float32 else bar)
            at += m
        close(got, (rms(want, 1e-5) * nw).reshape(T, H * Dv) * gate, bar)
    assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all()          # no other slot was touched


@pytest.mark.parametrize("dtype,bar", [(torch.float32, 2e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("T", [8, 4096])
def test_joins_and_gates_at_model_size(dtype, bar, T):
    from scratchpad_amd import _native
    W, groups = 4096, 8
    announce("add_group_norm / lowrank_gate", dtype, "rows", T)
    g = torch.Generator(device=DEV).manual_seed(1)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV)
    x, prod = rn(T, W), rn(T, 2 * W + 64).to(dtype)
    a, b, p = prod[:, :W], prod[:, W:2 * W], prod[:, 2 * W:]                   # views of one product
    wa, wb, nw = (rn(W) * 0.2 + 1 for _ in range(3))
    want = x + 0.5 * (rms(a.float(), 1e-5) * wa + rms(b.float(), 1e-5) * wb)
    xs = x.clone()
    out = _native.add_group_norm(xs, a, groups, 1e-5, dtype, b=b, wa=wa, wb=wb, next_weight=nw)
    close(xs, want, 2e-6)
    close(out, rms(want.view(T, groups, W // groups), 1e-5).view(T, W) * nw, bar)
    w2t, bias, A = rn(64, 2048) * 0.2, rn(2048), rn(16) * 0.5
    z = p.float() @ w2t + bias
    close(_native.lowrank_gate(p, w2t, bias, "decay", A),
          torch.exp(-torch.exp(A).repeat_interleave(128) * torch.nn.functional.softplus(z)), 2e-5)
    close(_native.lowrank_gate(p, w2t, None, "sigmoid"), torch.sigmoid(p.float() @ w2t), 2e-5)
