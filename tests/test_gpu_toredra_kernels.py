"""The Toredra kernels at the layer sizes of real models (bf16 and fp32), each against a plain fp32 torch expression of
the same operation evaluated on the GPU: several requests of unequal length in one launch, a second launch that goes on from
the states the first one left.  Every case prints its name before it launches."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def announce(*what):
    print("[case]", *what, flush=True)


def i32(xs):
    return torch.tensor(xs, dtype=torch.int32, device=DEV)


def seq_extend(lens, prefixes, slots):
    from scratchpad_amd import _native
    starts = [sum(lens[:i]) for i in range(len(lens))]
    token_req = torch.repeat_interleave(torch.arange(len(lens), dtype=torch.int32, device=DEV), torch.tensor(lens, device=DEV))
    return _native.SeqParams(torch.tensor(slots, device=DEV), torch.tensor([p + n for p, n in zip(prefixes, lens)], device=DEV),
                             i32(lens), i32(prefixes), i32(starts), token_req)


def close(got, want, bar):
    err = float((got.float() - want.float()).abs().max() / want.float().abs().max())
    assert err < bar, err


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


@pytest.mark.parametrize("dtype,bar", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,K", [(32, 64), (16, 128)])
def test_delta_recurrence_at_model_size(dtype, bar, H, K):
    from scratchpad_amd import _native
    lens, slots = [700, 1, 323], [3, 1, 4]
    T, n = sum(lens), H * K
    announce("delta_recurrence", dtype, "heads", H, "dim", K, "tokens", lens)
    g = torch.Generator(device=DEV).manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV)
    state = torch.full((6, H, K, K), float("nan"), device=DEV)
    S = {s: torch.zeros(H, K, K, device=DEV) for s in slots}
    for launch, prefixes in enumerate(([0, 0, 0], lens)):                      # the second launch goes on from the first's states
        r, k, v, gt = (rn(T, n).mul_(0.5).to(dtype) for _ in range(4))
        decay = torch.rand(T, n, generator=g, device=DEV) * 0.3 + 0.7
        remove = torch.rand(T, n, generator=g, device=DEV) * 0.8
        nw = torch.rand(n, generator=g, device=DEV) + 0.5
        got = _native.delta_recurrence(r, k, v, gt, decay, remove, nw, state, seq_extend(lens, prefixes, slots), H, K, 1e-5)
        want = torch.empty(T, H, K, device=DEV)
        at = 0
        for m, slot in zip(lens, slots):
            rr, kk, vv, ww, aa = (t[at:at + m].float().view(m, H, K) for t in (r, k, v, decay, remove))
            uu = kk / torch.sqrt((kk * kk).sum(-1, keepdim=True) + 1e-6)
            for t in range(m):
                proj = torch.einsum("hi,hij->hj", uu[t], S[slot])
                S[slot] = ww[t].unsqueeze(-1) * S[slot] - (aa[t] * uu[t]).unsqueeze(-1) * proj.unsqueeze(-2) \
                    + kk[t].unsqueeze(-1) * vv[t].unsqueeze(-2)
                want[at + t] = torch.einsum("hij,hi->hj", S[slot], rr[t])
            close(state[slot], S[slot], 1e-3 if dtype == torch.float32 else bar)
            at += m
        close(got, (rms(want, 1e-5).reshape(T, n) * nw * torch.sigmoid(gt.float())), bar)
    assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all()          # no other slot was touched


@pytest.mark.parametrize("dtype,bar", [(torch.float32, 1e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,D,Dv", [(8, 128, 128), (16, 64, 256)])
def test_forget_write_scan_at_model_size(dtype, bar, H, D, Dv):
    from scratchpad_amd import _native
    lens, slots = [700, 1, 323], [3, 1, 4]
    T = sum(lens)
    announce("hgrn2_scan", dtype, "heads", H, "dim", D, "vdim", Dv, "tokens", lens)
    g = torch.Generator(device=DEV).manual_seed(1)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV)
    state = torch.full((6, H, D, Dv), float("nan"), device=DEV)
    S = {s: torch.zeros(H, D, Dv, device=DEV) for s in slots}
    fb, nw = rn(H * D) * 0.5, torch.rand(Dv, generator=g, device=DEV) + 0.5
    lower = torch.rand(H * D, generator=g, device=DEV) * 0.9
    for launch, prefixes in enumerate(([0, 0, 0], lens)):
        qpre, fpre, v = rn(T, H * D).to(dtype), (rn(T, H * D) + 1.0).to(dtype), rn(T, H * Dv).to(dtype)
        got = _native.hgrn2_scan(qpre, fpre, v, fb, lower, nw, state, seq_extend(lens, prefixes, slots), H, D, Dv, 1e-5)
        q = torch.nn.functional.silu(qpre.float()).view(T, H, D)
        f = (lower + (1 - lower) * torch.sigmoid(fpre.float() + fb)).view(T, H, D)
        vv = v.float().view(T, H, Dv)
        want = torch.empty(T, H, Dv, device=DEV)
        at = 0
        for m, slot in zip(lens, slots):
            for t in range(at, at + m):
                S[slot] = f[t].unsqueeze(-1) * S[slot] + (1 - f[t]).unsqueeze(-1) * vv[t].unsqueeze(-2)
                want[t] = torch.einsum("hij,hi->hj", S[slot], q[t])
            close(state[slot], S[slot], 1e-3 if dtype == torch.float32 else bar)
            at += m
        close(got, (rms(want, 1e-5) * nw).reshape(T, H * Dv), bar)
    assert torch.isnan(state[0]).all() and torch.isnan(state[5]).all()


@pytest.mark.parametrize("dtype,bar", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
def test_row_kernels_at_model_size(dtype, bar):
    from scratchpad_amd import _native
    T, W, n, rank, ff = 4096, 4096, 2048, 64, 8192
    announce("gated_add_norm / delta_gates / relu_square / scale_softcap", dtype, "rows", T, "width", W)
    g = torch.Generator(device=DEV).manual_seed(2)
    rn = lambda *s: torch.randn(*s, generator=g, device=DEV)
    x, extra = rn(T, W), rn(T, W)
    prod = rn(T, 3 * W).to(dtype)                         # [a | b | gate]: views of one product, as the model hands them over
    a, b, gate = prod[:, :W], prod[:, W:2 * W], prod[:, 2 * W:]
    w, wa, wb, gb, nxt = (1 + 0.3 * rn(W) for _ in range(5))
    y = 0.5 * (rms(a.float(), 1e-5) * wa + rms(b.float(), 1e-5) * wb) * torch.sigmoid(gate.float() + gb)
    want = x + rms(y, 1e-5) * w + extra
    xs = x.clone()
    out = _native.gated_add_norm(xs, a, w, 1e-5, gate=gate, gate_bias=gb, b=b, wa=wa, wb=wb, extra=extra, next_weight=nxt)
    close(xs, want, 1e-5)
    close(out, rms(want, 1e-5) * nxt, bar)
    for rows in (T, 8):                                   # a prompt's portion (8 tokens per workgroup) and a decode step
        p, apre = rn(rows, rank).to(dtype), rn(rows, n).to(dtype)
        w2t, w0, ab = rn(rank, n) * 0.2, rn(n), rn(n)
        dec, rem = _native.delta_gates(p, w2t, w0, apre, ab, 0.6)
        close(dec, torch.exp(-0.6 * torch.sigmoid(torch.tanh(p.float()) @ w2t + w0)), 1e-5)
        close(rem, torch.sigmoid(apre.float() + ab), 1e-5)
    up = rn(T, ff + W).to(dtype)
    assert torch.equal(_native.relu_square(up[:, :ff]), (torch.relu(up[:, :ff].float()) ** 2).to(dtype))
    z = rn(64, 128256).mul_(20).to(dtype)
    close(_native.scale_softcap(z, 0.5, 30.0), 30.0 * torch.tanh(z.float() * 0.5 / 30.0), 1e-5)
