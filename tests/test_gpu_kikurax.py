"""Kikurax through the engine on the GPU against the CPU oracle (float64, one sequence at a time, no cache or state):
single mechanisms, kernels on crafted inputs (a far key among hundreds, a tempting key one position ahead, a sink that
takes most of the weight, decays that keep the first token audible), whole prompts with the stream after every layer,
decoding through cache and state, portions down to two tokens, unequal batches, reused rows and slots, graph replay,
other sizes, and generation through the engine's scheduler.

Sharp comparisons run the engine in fp32 (the oracle's weights are bf16-representable, so both see the same numbers); a
bf16 pass checks the serving precision against a looser bar."""
import math

import pytest
import torch

from oracle import kikurax as ko
from tests import kikurax_util as U
from tests.test_gpu_toredra import engine, entry, portions, run_portions, run_whole, seq_params

pytestmark = pytest.mark.gpu
F32_BAR = 2e-4


# ------------------------------------------------------------------------------------------------ mechanisms alone
LAYERS = [
    (U.attention(4, 2, 16, 24, dims=8), None),
    (U.attention(3, 3, 24, 8, scaling=False, softcap=None), None),          # kv heads = heads, no cap
    (U.attention(5, 1, 8, 72, dims=0, softcap=1.5, v_mix=False), None),      # no rotation, one kv head, a tight cap
    (U.attention(2, 1, 136, 200, dims=72, scale=0.05), None),               # heads above 128
    (U.mamba(3, 24, 16, groups=3, conv=4, norm_groups=3), None),
    (U.mamba(4, 8, 40, groups=1, conv=1, norm_groups=1), None),             # one tap: no convolution state
    (U.mamba(2, 72, 136, groups=2, conv=2, norm_groups=4), None),
    (U.parallel(4, 2, 16, 24, 4, 2, 8, 40, conv=4), None),
    (U.parallel(3, 3, 24, 8, 1, 1, 72, 8, conv=2, every=1), None),
    (U.parallel(5, 1, 8, 72, 6, 3, 16, 16, conv=1, every=0), None),          # no query temperature, one tap
    (U.parallel(2, 1, 40, 16, 2, 1, 136, 136, conv=3, every=7), None),       # state above 128
    (U.parallel(2, 2, 136, 200, 2, 2, 24, 200, scale=0.02), None),
    (U.attention(2, 2, 16, 16), U.moe(6, 2, 40)), (U.mamba(2, 16, 8), U.moe(4, 1, 24, limit=0.3)),
    (U.parallel(2, 1, 16, 16, 2, 2, 16, 16), U.moe(5, 5, 16)),
]


@pytest.mark.parametrize("layer", LAYERS, ids=lambda l: f"{l[0]['type']}-{'none' if l[1] is None else l[1]['kind']}")
@pytest.mark.parametrize("groups", [1, 4])
def test_single_layer_models_match_oracle(tmp_path, layer, groups):
    cfg = U.config([layer], width=80, groups=groups)
    folder, w = U.make_model(tmp_path, cfg, seed=5)
    toks = U.tokens(70, cfg["vocab"], 6)
    eng = engine(folder)
    eng.runner.model.capture_layers = []
    got = run_whole(eng, toks)
    lay = []
    want = ko.forward(toks, w, cfg, lay)
    assert U.rel(eng.runner.model.capture_layers[0], lay[0]) < F32_BAR
    assert U.rel(got, want) < F32_BAR


# ------------------------------------------------------------------------------------------------ row kernels
@pytest.mark.parametrize("W,groups", [(200, 1), (120, 3), (77, 7), (3072, 4)])
def test_add_group_norm_kernel_in_every_form(W, groups):
    from scratchpad_amd import _native
    g = torch.Generator().manual_seed(0)
    T, eps = 37, 1e-5
    rn = lambda *s: torch.randn(*s, generator=g)
    x, a, b = rn(T, W) * torch.linspace(0.1, 9.0, W), rn(T, 2 * W) * 3, rn(T, W) * 0.2
    wa, wb, nw = (1 + 0.3 * rn(W) for _ in range(3))
    N = lambda z: z / torch.sqrt((z * z).mean(-1, keepdim=True) + eps)
    for dtype, bar in ((torch.float32, 2e-6), (torch.bfloat16, 1e-2)):
        r = lambda t: t.to(dtype).double()
        for form in ("norm", "add", "add+norm", "two", "two+norm"):
            av = a.to(dtype).cuda()[:, W:]                                     # a view: its stride is taken
            want = x.double()
            if form.startswith("add"):
                want = want + r(a[:, W:])
            if form.startswith("two"):
                want = want + 0.5 * (N(r(a[:, W:])) * wa.double() + N(r(b)) * wb.double())
            xs = x.clone().cuda()
            two = form.startswith("two")
            out = _native.add_group_norm(xs, None if form == "norm" else av, groups, eps, dtype, b=b.to(dtype).cuda() if two else None,
                                         wa=wa.cuda() if two else None, wb=wb.cuda() if two else None,
                                         next_weight=nw.cuda() if form.endswith("norm") else None)
            assert U.rel(xs, want) < 2e-6, (dtype, form)
            if form.endswith("norm"):
                assert out.dtype == dtype and U.rel(out, ko.group_norm(want, nw.double(), groups, eps)) < bar, (dtype, form)
            else:
                assert out is None


def test_router_chooses_by_logit_and_weights_over_the_chosen():
    from scratchpad_amd import _native
    g = torch.Generator().manual_seed(1)
    for E, top in ((12, 3), (5, 5), (70, 1), (9, 4)):
        x, W, b = torch.randn(50, 24, generator=g), torch.randn(E, 24, generator=g) * 3, torch.randn(E, generator=g) * 4
        ids, wt = _native.moe_route_softmax(x.cuda(), W.cuda(), top, 1.0, b.cuda(), renorm=True)
        wi, ww = ko.route(x.double(), {"r.router": W.double(), "r.router.b": b.double()}, "r", top)
        assert torch.equal(ids.cpu().long(), wi) and U.rel(wt, ww) < 1e-5


# ------------------------------------------------------------------------------------------------ the delta rule's kernels
def delta_oracle(q, k, v, bpre, decay, gate, norm_w, H, G, D, Dv, eps):
    T = q.shape[0]
    q, k, v = q.double().view(T, G, D), k.double().view(T, G, D), v.double().view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta, decay = torch.sigmoid(bpre.double()), decay.double().view(T, H, D)
    out = torch.zeros(T, H, Dv, dtype=torch.float64)
    for h in range(H):
        S = torch.zeros(D, Dv, dtype=torch.float64)
        for t in range(T):
            S = decay[t, h][:, None] * S
            S = S + torch.outer(k[t, h // (H // G)], beta[t, h] * (v[t, h] - S.T @ k[t, h // (H // G)]))
            out[t, h] = S.T @ q[t, h // (H // G)]
    return (ko.rms(out, eps) * norm_w.double() * gate.double().view(T, H, Dv)).reshape(T, H * Dv)


@pytest.mark.parametrize("sizes", [[300], [1], [7, 2, 40, 1, 1, 1, 3, 64, 1], [2]], ids=["whole", "decode", "mixed", "pairs"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 24), (2, 2, 32, 64), (3, 1, 8, 200), (2, 1, 136, 40), (1, 1, 64, 136), (6, 3, 72, 16)],
                         ids=lambda s: "x".join(map(str, s)))
def test_gated_delta_scan_keeps_the_first_token_audible(shape, sizes):
    """300 tokens with decays of 0.99 and more: what token 0 wrote is still read at the end, so a state that is lost,
    started late or decayed by the wrong channel shows at every later position; the state starts from NaN-filled slots"""
    from scratchpad_amd import _native
    H, G, D, Dv = shape
    g = torch.Generator().manual_seed(4)
    T, eps = 300, 1e-5
    q, k, v = (torch.randn(T, n, generator=g) for n in (G * D, G * D, H * Dv))
    bpre, decay = torch.randn(T, H, generator=g) - 4.0, 0.997 + 0.003 * torch.rand(T, H * D, generator=g)
    bpre[0] = 4.0                                                         # token 0 is written in full, later ones lightly
    decay[:, ::3] = 0.6                                                   # some channels forget fast: rows are not alike
    gate, nw = torch.rand(T, H * Dv, generator=g), 1 + 0.3 * torch.randn(Dv, generator=g)
    want = delta_oracle(q, k, v, bpre, decay, gate, nw, H, G, D, Dv, eps)
    late = delta_oracle(q[1:], k[1:], v[1:], bpre[1:], decay[1:], gate[1:], nw, H, G, D, Dv, eps)
    assert U.rel(late[-1], want[-1]) > 1e-3                               # token 0 is audible at the end
    state = torch.full((4, H, D, Dv), float("nan"), device="cuda")
    c = lambda t: t.cuda()
    outs, held = [], 0
    for at, n in portions(T, sizes):
        s = slice(at, at + n)
        outs.append(_native.gated_delta_scan(c(q[s]), c(k[s]), c(v[s]), c(bpre[s]), c(decay[s]).contiguous(), c(gate[s]).contiguous(),
                                             c(nw), state, seq_params(2, held, n), H, G, D, Dv, eps).cpu())
        held += n
    assert U.rel(torch.cat(outs), want) < 2e-5
    assert torch.isnan(state[1]).all() and torch.isnan(state[3]).all()     # neighbouring slots untouched


def test_lowrank_gates_against_torch():
    from scratchpad_amd import _native
    g = torch.Generator().manual_seed(2)
    for T in (5, 200):
        for dtype in (torch.float32, torch.bfloat16):
            p = torch.randn(T, 40, generator=g).to(dtype)
            w2t, bias, A = torch.randn(7, 6 * 24, generator=g), torch.randn(6 * 24, generator=g), torch.randn(6, generator=g)
            z = p[:, 3:10].double() @ w2t.double()
            got = _native.lowrank_gate(p.cuda()[:, 3:10], w2t.cuda(), bias.cuda(), "decay", A.cuda())
            want = torch.exp(-torch.exp(A.double()).repeat_interleave(24) * torch.nn.functional.softplus(z + bias.double()))
            assert U.rel(got, want) < 2e-6
            assert U.rel(_native.lowrank_gate(p.cuda()[:, 3:10], w2t.cuda(), None, "sigmoid"), torch.sigmoid(z)) < 2e-6


# ------------------------------------------------------------------------------------------------ the attention kernels
class AttnBench:
    """the store + attention kernels as the model drives them, on shuffled slots of a NaN-filled pool"""

    def __init__(self, H, G, D, Dv, rot=None, dtype=torch.float32, matrix=True, scale=0.25, **kw):
        from scratchpad_amd.layers import HalfAngleRotary
        self.H, self.G, self.D, self.Dv, self.dtype, self.matrix, self.scale, self.kw = H, G, D, Dv, dtype, matrix, scale, kw
        self.rotary = HalfAngleRotary(rot["dims"], rot["base"], rot.get("scaling")).cuda() if rot else None
        P = 700
        self.k = torch.full((P + 1, G * D), float("nan"), dtype=dtype, device="cuda")
        self.v = torch.full((P + 1, G * Dv), float("nan"), dtype=dtype, device="cuda")
        self.first = torch.full((P + 1, G * Dv), float("nan"), dtype=dtype, device="cuda")
        self.slots = (torch.randperm(P, generator=torch.Generator().manual_seed(9)) + 1).to(torch.int32).cuda()
        self.table = torch.zeros((4, P), dtype=torch.int32, device="cuda")
        self.table[2] = self.slots
        self.held = 0

    def step(self, q, k, v, vf, gate):
        from scratchpad_amd import _native as n_
        n = q.shape[0]
        loc = self.slots[self.held:self.held + n].long()
        pos = torch.arange(self.held, self.held + n, device="cuda")
        seq = seq_params(2, self.held, n)
        c = lambda t: None if t is None else t.cuda()
        q = q.to(self.dtype).cuda().clone()
        freq, mag = (self.rotary.freq, self.rotary.magnitude) if self.rotary else (None, 1.0)
        kw = self.kw
        if vf is not None:
            self.first[loc] = vf.to(self.dtype).cuda()
        n_.qkv_rotary_store(q, k.to(self.dtype).cuda(), v.to(self.dtype).cuda(), self.k, self.v, pos, loc, freq, mag, self.H, self.G,
                            self.D, self.Dv, 1e-6, norm_values=False, q_bias=c(kw.get("qb")), k_bias=c(kw.get("kb")),
                            v_bias=c(kw.get("vb")), qk_norm=True, q_head_scale=c(kw.get("temp")), q_temp=kw.get("q_temp"),
                            v_first=self.first if vf is not None else None, v_mix=c(kw.get("lam")) if vf is not None else None)
        out = n_.window_attention(q, self.k, self.v, None, None, self.table, seq, self.H, self.G, self.D, self.Dv, 0, 0,
                                  self.scale, self.matrix, sinks=c(kw.get("sinks")), softcap=kw.get("softcap", 0.0),
                                  sigmoid_weights=kw.get("sigmoid", False), head_bias=c(kw.get("pb")),
                                  gate=None if gate is None else gate.to(self.dtype).cuda())
        self.held += n
        return out.float().cpu()

    def run(self, q, k, v, sizes, vf=None, gate=None):
        cut = lambda t, at, m: None if t is None else t[at:at + m]
        return torch.cat([self.step(q[at:at + m], k[at:at + m], v[at:at + m], cut(vf, at, m), cut(gate, at, m))
                          for at, m in portions(q.shape[0], sizes)])


def attn_oracle(q, k, v, H, G, D, Dv, scale=0.25, rot=None, qb=0, kb=0, vb=0, temp=None, softcap=0.0, lam=None, vf=None, sigmoid=False,
                pb=None, q_temp=None, gate=None, eps=1e-6, **_):
    T = q.shape[0]
    q, k, v = (q.double() + (qb.double() if torch.is_tensor(qb) else 0)).view(T, H, D), \
        (k.double() + (kb.double() if torch.is_tensor(kb) else 0)).view(T, G, D), \
        (v.double() + (vb.double() if torch.is_tensor(vb) else 0)).view(T, G, Dv)
    q, k = ko.rms(ko.rotate_half_pairs(q, rot), eps), ko.rms(ko.rotate_half_pairs(k, rot), eps)
    if vf is not None:
        v = (1 - lam.double()) * v + lam.double() * vf.double().view(T, G, Dv)
    if q_temp:
        pos = torch.arange(T, dtype=torch.float64)
        q = q * (1 + q_temp[0] * torch.log(torch.floor((pos + 1) / q_temp[1]) + 1))[:, None, None]
    out = torch.zeros(T, H, Dv, dtype=torch.float64)
    for h in range(H):
        s = (q[:, h] @ k[:, h // (H // G)].T) * scale * (float(temp[h]) if temp is not None else 1.0)
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        vv = v[:, h // (H // G)]
        if sigmoid:
            out[:, h] = torch.tril(torch.sigmoid(s + (float(pb[h]) if pb is not None else 0.0))) @ vv
        else:
            e = torch.tril(torch.exp(s - 60.0))
            out[:, h] = (e / (e.sum(-1, keepdim=True) + math.exp(-60.0))) @ vv         # the sink: exp(0 - 60)
    out = out.reshape(T, H * Dv)
    return out * torch.sigmoid(gate.double()) if gate is not None else out


@pytest.mark.parametrize("sizes", [[150], [1], [7, 2, 40, 1, 1, 1, 3, 64, 1], [2]], ids=["whole", "decode", "mixed", "pairs"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 24, 8), (2, 2, 8, 8, 8), (3, 1, 24, 72, 10), (6, 3, 40, 16, 0), (2, 1, 136, 200, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_softmax_attention_with_normed_heads_a_cap_a_sink_and_blended_values(shape, sizes):
    """scores of several units after the per-head numbers, a cap that bites, the zero sink holding a visible share, values
    blended with another pool's rows: a key wrongly seen or missed, a norm taken before the rotation's bias, a head's number
    or the cap left out each move the output by far more than the bar; every position of 150 is compared"""
    H, G, D, Dv, dims = shape
    g = torch.Generator().manual_seed(3)
    T = 150
    q, k, v, vf = (torch.randn(T, n, generator=g) for n in (H * D, G * D, G * Dv, G * Dv))
    kw = dict(qb=torch.randn(H * D, generator=g), kb=torch.randn(G * D, generator=g), vb=torch.randn(G * Dv, generator=g),
              temp=torch.linspace(0.5, 3.0, H), softcap=4.0, lam=torch.tensor([0.3]), sinks=torch.zeros(H))
    rot = {"dims": dims, "base": 100.0, "scaling": {"factor": 2.0, "low": 1.0, "high": 4.0, "original": 32}} if dims else None
    scale = 6.0 / D
    got = AttnBench(H, G, D, Dv, rot, scale=scale, **kw).run(q, k, v, sizes, vf=vf)
    want = attn_oracle(q, k, v, H, G, D, Dv, scale, rot, vf=vf, **kw)
    assert U.rel(got, want) < 2e-5
    for drop in ("temp", "softcap", "qb", "lam"):                             # the oracle moves when a piece is left out
        less = {**kw, drop: None if drop != "lam" else torch.tensor([0.0])}
        assert U.rel(attn_oracle(q, k, v, H, G, D, Dv, scale, rot, vf=vf, **less), want) > 1e-2, drop


@pytest.mark.parametrize("sizes", [[150], [1], [7, 2, 40, 1, 1, 1, 3, 64, 1], [2]], ids=["whole", "decode", "mixed", "pairs"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 24), (2, 2, 8, 8), (3, 1, 24, 72), (6, 3, 40, 16), (2, 1, 136, 200)],
                         ids=lambda s: "x".join(map(str, s)))
def test_sigmoid_attention_with_query_temperature_bias_and_gate(shape, sizes):
    H, G, D, Dv = shape
    g = torch.Generator().manual_seed(5)
    T = 150
    q, k, v, gate = (torch.randn(T, n, generator=g) for n in (H * D, G * D, G * Dv, H * Dv))
    kw = dict(sigmoid=True, pb=torch.linspace(-3.0, 0.5, H), q_temp=(0.8, 7))
    scale = 3.0 / D
    got = AttnBench(H, G, D, Dv, scale=scale, **kw).run(q, k, v, sizes, gate=gate)
    want = attn_oracle(q, k, v, H, G, D, Dv, scale, gate=gate, **kw)
    assert U.rel(got, want) < 2e-5
    assert U.rel(attn_oracle(q, k, v, H, G, D, Dv, scale, gate=gate, sigmoid=True, pb=kw["pb"]), want) > 1e-2
    assert U.rel(attn_oracle(q, k, v, H, G, D, Dv, scale, gate=gate, sigmoid=True, q_temp=(0.8, 7)), want) > 1e-2


@pytest.mark.parametrize("sigmoid", [False, True], ids=["softmax", "sigmoid"])
def test_far_key_and_a_tempting_future_key(sigmoid):
    """one loud key at position 3 among 600 quiet ones: every later query hears it, in a prompt of 600 and decoded token by
    token behind a prompt; a louder key at position p + 1 must never reach query p; the temperature's step at a multiple of
    `every` falls on the right position"""
    H = G = 1
    D, Dv, T = 16, 64, 600
    g = torch.Generator().manual_seed(1)
    q, k, v = torch.randn(T, D, generator=g) * 0.1, torch.randn(T, D, generator=g) * 0.1, torch.randn(T, Dv, generator=g) * 0.01
    q[:, 0], k[3, 0] = 6.0, 8.0                               # after the norms: q . k = 16 for the pair, about 0 otherwise
    k[:, 1] = 1.0
    k[3, 1] = 0.0
    v[3] = torch.arange(Dv) - 31.5
    k[400] = 0.0
    k[400, 0], v[400] = 30.0, 1000.0                          # position 399 must not see it; 400 and later do
    kw = dict(sigmoid=True, pb=torch.tensor([-12.0]), q_temp=(1.0, 64)) if sigmoid else dict(sinks=torch.zeros(1), softcap=20.0)
    scale = 0.7
    want = attn_oracle(q, k, v, H, G, D, Dv, scale, **kw)
    loud = v[3].double()
    cos = lambda a: float(torch.dot(a.double(), loud) / a.double().norm() / loud.norm())
    assert cos(want[399]) > 0.99 and abs(cos(want[2])) < 0.5 and float(want[400].min()) > 400
    if sigmoid:                                               # position 62 -> 63: the multiplier steps from 1 to 1 + ln 2
        assert float(want[63].norm() / want[62].norm()) > 2.5
    for sizes in ([T], [390, 1], [64], [63, 2, 1]):
        got = AttnBench(H, G, D, Dv, scale=scale, **kw).run(q, k, v, sizes)
        assert cos(got[399]) > 0.99 and cos(got[150]) > 0.99 and float(got[399].max()) < 100
        assert U.rel(got, want) < 2e-5


@pytest.mark.parametrize("sizes", [[200], [17, 2, 64, 1, 1, 33, 16, 5], [3]], ids=["whole", "mixed", "threes"])
@pytest.mark.parametrize("shape", [(8, 2, 128, 128), (4, 4, 64, 128), (6, 1, 128, 64)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("sigmoid", [False, True], ids=["softmax", "sigmoid"])
def test_matrix_core_attention_in_both_forms_against_the_vector_kernel(shape, sizes, sigmoid):
    """portions of prompts in bf16 with heads of 64 / 128 run on the matrix cores: the cap, the per-key sigmoid and the gate
    there against the fp32-arithmetic vector kernel that the tests above pin (same cache, same portions)"""
    H, G, D, Dv = shape
    g = torch.Generator().manual_seed(7)
    T = 200
    q, k, v, gate = (torch.randn(T, n, generator=g) for n in (H * D, G * D, G * Dv, H * Dv))
    kw = dict(sigmoid=True, pb=torch.linspace(-4.0, -1.0, H), q_temp=(0.5, 16)) if sigmoid else \
        dict(sinks=torch.zeros(H), softcap=5.0, temp=torch.linspace(0.5, 2.0, H))
    outs = [AttnBench(H, G, D, Dv, dtype=torch.bfloat16, matrix=m, scale=4.0 / D, **kw).run(q, k, v, sizes, gate=gate if sigmoid else None)
            for m in (True, False)]
    assert torch.isfinite(outs[0]).all()
    assert U.rel(outs[0], outs[1]) < 1.5e-2


# ------------------------------------------------------------------------------------------------ the whole model
@pytest.fixture(scope="module")
def full(tmp_path_factory):
    cfg = U.full_config()
    folder, w = U.make_model(tmp_path_factory.mktemp("full"), cfg, seed=11)
    toks = U.tokens(130, cfg["vocab"], 12)
    lay = []
    want = ko.forward(toks, w, cfg, lay)
    return cfg, folder, w, toks, want, lay


def test_whole_prompt_with_the_stream_after_every_layer(full):
    cfg, folder, w, toks, want, lay = full
    eng = engine(folder)
    eng.runner.model.capture_layers = []
    got = run_whole(eng, toks)
    for i, (a, b) in enumerate(zip(eng.runner.model.capture_layers, lay)):
        assert U.rel(a, b) < F32_BAR, i
    assert U.rel(got, want) < F32_BAR
    eng.runner.model.capture_layers = None
    assert U.rel(run_whole(eng, toks, "again"), want) < F32_BAR            # the fused joins, on rows and slots used before


def test_serving_precision(full):
    cfg, folder, w, toks, want, _ = full
    got = run_whole(engine(folder, dtype=torch.bfloat16), toks)
    err = (got.double().cpu() - want).abs().amax(-1) / want.abs().max()
    # (a router's close call that falls the other way in 16 bits moves single positions by more: the bulk is the bar)
    assert float(err.median()) < 5e-2 and float(err.quantile(0.9)) < 0.15


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_decoding_from_the_first_token(full, graphs):
    """130 single-token steps: the first is a first token on a fresh slot, every later one a decode step through cache,
    convolution state and matrix states"""
    cfg, folder, w, toks, want, _ = full
    assert U.rel(run_portions(engine(folder, graphs=graphs), toks, [1]), want) < F32_BAR


def test_long_decoding_behind_a_prompt(tmp_path):
    cfg = U.config([(U.parallel(2, 1, 16, 24, 2, 1, 16, 24, every=64), U.moe(4, 2, 24)), (U.attention(2, 1, 16, 24), None),
                    (U.mamba(2, 16, 16), U.moe(3, 1, 16))], width=48, vocab=61)
    folder, w = U.make_model(tmp_path, cfg, seed=8)
    toks = U.tokens(400, 61, 9)
    want = ko.forward(toks, w, cfg)
    assert U.rel(run_portions(engine(folder, graphs=True), toks, [40, 1]), want) < F32_BAR


@pytest.mark.parametrize("sizes", [[2], [3, 2, 17, 1, 1, 64, 5, 1], [64, 2, 1], [15, 16, 17, 1]],
                         ids=["pairs", "mixed", "big-then-small", "near-16"])
def test_portions_of_prompts(full, sizes):
    cfg, folder, w, toks, want, _ = full
    assert U.rel(run_portions(engine(folder), toks, sizes), want) < F32_BAR


def test_garbage_in_reused_rows_and_slots_is_never_read(full):
    cfg, folder, w, toks, want, _ = full
    eng = engine(folder)
    sp, kv = eng.runner.state_pool, eng.runner.token_to_kv_pool
    for spec in sp.named.values():
        for t in spec.values():
            t.fill_(float("nan"))
    for b in kv._all():
        b.fill_(float("nan"))
    assert U.rel(run_portions(eng, toks[:60], [7, 1]), want[:60]) < F32_BAR


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_unequal_batches_with_rows_and_slots_reused(full, graphs):
    """seven requests of unequal length through three rows and a pool that holds far fewer tokens than their sum: portions
    of some beside single tokens of others, pauses, rows and slots handed on; every request's logits must be what it gets
    alone"""
    cfg, folder, w, _, _, _ = full
    reqs = {f"r{i}": U.tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate([45, 3, 70, 1, 26, 58, 12])}
    want = {r: ko.forward(t, w, cfg) for r, t in reqs.items()}
    eng = engine(folder, tokens=200, slots=3, graphs=graphs)
    plan = {"r0": [5, 1, 1, 30, 1, 7], "r1": [2, 1], "r2": [33, 2, 1, 1, 1, 1, 1, 30], "r3": [1], "r4": [1, 1, 24],
            "r5": [2, 50, 1, 1, 1, 1, 1, 1], "r6": [6, 1, 1, 1, 1, 1, 1]}
    fed, got, waiting, live, step = {r: 0 for r in reqs}, {r: [] for r in reqs}, list(reqs), [], 0
    while waiting or live:
        while waiting and len(live) < 3 and sum(len(reqs[r]) for r in live) + len(reqs[waiting[0]]) <= 200:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            if (step + int(r[1:])) % 5 == 4 and len(live) > 1:
                continue                                           # left out of this step, goes on later
            n = plan[r].pop(0) if plan[r] else 1
            n = min(n, len(reqs[r]) - fed[r])
            entries.append(entry(r, reqs[r][fed[r]:fed[r] + n]))
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        if entries:
            out = eng.step(entries, end)
            at = 0
            for e in entries:
                got[e.rid].append(out[at:at + len(e.tokens)])
                at += len(e.tokens)
        live = [r for r in live if r not in end]
        step += 1
    for r in reqs:
        assert U.rel(torch.cat(got[r]), want[r]) < F32_BAR, r


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_graph_replay_of_larger_decode_steps(full, dtype):
    """40 requests decoding together; every replay (six, with eager steps of the other engine and synchronisations between)
    is compared with the same step run eagerly"""
    cfg, folder, w, _, _, _ = full
    reqs = {f"q{i}": U.tokens(3 + i % 9, cfg["vocab"], 300 + i) + U.tokens(6, cfg["vocab"], 900 + i) for i in range(40)}
    outs = []
    for graphs in (True, False):
        eng = engine(folder, dtype=dtype, tokens=900, slots=40, graphs=graphs)
        eng.step([entry(r, t[:-6], []) for r, t in reqs.items()])                     # the prompts, one extend batch
        steps = []
        for k in range(6):
            steps.append(eng.step([entry(r, [t[len(t) - 6 + k]]) for r, t in reqs.items()], list(reqs) if k == 5 else []))
            torch.cuda.synchronize()
        outs.append(torch.stack(steps))
    bar = 1e-5 if dtype == torch.float32 else 3e-2
    for k in range(6):
        assert U.rel(outs[0][k], outs[1][k]) < bar, k
    if dtype == torch.float32:
        want = torch.stack([ko.forward(t, w, cfg)[-6:] for t in reqs.values()], 1)    # [step, request, vocab]
        assert U.rel(outs[0], want) < F32_BAR


def test_generation_through_the_scheduler(full):
    """greedy generation of three prompts through Engine.generate (admission, chunked prefill of 16 tokens beside decoding
    requests, release) equals the oracle's greedy continuation; sampled generation runs and stays in the vocabulary"""
    from scratchpad_amd.sampler import SamplingParams
    cfg, folder, w, _, _, _ = full
    prompts = [U.tokens(n, cfg["vocab"], 40 + n) for n in (37, 5, 21)]
    eng = engine(folder, tokens=300, slots=2, graphs=True, chunk=16)
    got = eng.generate(prompts, max_new_tokens=12)
    for p, out in zip(prompts, got):
        ref = U.greedy(p, w, cfg, 12)
        agree = next((i for i, (a, b) in enumerate(zip(out, ref)) if a != b), 12)
        if agree < 12:      # a near-tie in fp32 against float64 may flip one choice: the logits there must be that close
            lg = ko.forward(p + ref[:agree], w, cfg)[-1]
            assert float(lg[ref[agree]] - lg[out[agree]]) < 1e-3 * float(lg.abs().max()), (agree, out, ref)
        else:
            assert out == ref
    sampled = eng.generate(prompts[:2], SamplingParams(max_new_tokens=6, temperature=0.8, top_p=0.9, top_k=20))
    assert all(len(o) == 6 and all(0 <= t < cfg["vocab"] for t in o) for o in sampled)


@pytest.mark.parametrize("seed", range(10))
def test_designs_drawn_at_random(tmp_path, seed):
    """layer order, sizes and constants drawn at random: whole prompt, then portions of random sizes with single tokens
    between them, both against the oracle"""
    import random
    cfg = U.random_config(100 + seed)
    folder, w = U.make_model(tmp_path, cfg, seed=seed, rank_a=2 + seed, rank_g=12 - seed)
    toks = U.tokens(90, cfg["vocab"], seed)
    want = ko.forward(toks, w, cfg)
    assert U.rel(run_whole(engine(folder), toks), want) < F32_BAR, cfg
    r = random.Random(seed)
    sizes = [r.choice([1, 1, 2, 3, 7, 16, 29]) for _ in range(40)]
    assert U.rel(run_portions(engine(folder), toks, sizes), want) < F32_BAR, (sizes, cfg)


def test_sizes_that_are_one_or_equal(tmp_path):
    """a model whose sizes are 1 or equal where the others' differ: one head everywhere, key width = value width = model
    width, rotation over the whole head, one norm group, one expert, embedding scale 1, attention layers that do not blend"""
    cfg = U.config([
        (U.attention(1, 1, 16, 16, dims=16, scale=1.0, v_mix=False), U.moe(1, 1, 16)),
        (U.parallel(1, 1, 16, 16, 1, 1, 16, 16, conv=1, every=1, scale=1.0), U.moe(1, 1, 16)),
        (U.mamba(1, 16, 16, conv=1), None),
        (U.attention(1, 1, 16, 16, dims=16, scale=1.0, v_mix=False), None),
    ], width=16, vocab=17, groups=1, scale=1.0)
    folder, w = U.make_model(tmp_path, cfg, seed=4, rank_a=1, rank_g=1)
    toks = U.tokens(50, 17, 3)
    want = ko.forward(toks, w, cfg)
    assert U.rel(run_whole(engine(folder), toks), want) < F32_BAR
    assert U.rel(run_portions(engine(folder), toks, [3, 1]), want) < F32_BAR
