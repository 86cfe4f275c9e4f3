"""Toredra through the engine on the GPU against the CPU oracle (float64, one sequence at a time, no cache or state):
single mechanisms, kernels on crafted inputs (a far key among hundreds, a tempting key one position ahead, a sink that
takes most of the weight, decays that keep the first token visible), whole prompts with the stream after every layer run,
loops, decoding through cache and state, portions down to two tokens, unequal batches, reused rows and slots, graph replay,
other sizes, and generation through the engine's scheduler.

Sharp comparisons run the engine in fp32 (the oracle's weights are bf16-representable, so both see the same numbers); a
bf16 pass checks the serving precision against a looser bar."""
import math

import pytest
import torch

from oracle import toredra as to
from tests import toredra_util as U

pytestmark = pytest.mark.gpu
F32_BAR = 2e-4


def engine(folder, dtype=torch.float32, tokens=512, slots=4, graphs=False, chunk=2048):
    from scratchpad_amd.engine import Engine
    return Engine(folder, dtype=dtype, max_total_tokens=tokens, max_running_requests=slots, use_graphs=graphs, chunk_size=chunk)


def entry(rid, toks, want=None):
    from scratchpad_amd.engine import StepEntry
    return StepEntry(rid, list(toks), list(range(len(toks))) if want is None else want)


def run_whole(eng, toks, rid="w"):
    return eng.step([entry(rid, toks)], [rid])


def run_portions(eng, toks, sizes, rid="p"):
    """feed toks in portions of the given sizes (the last size repeats), logits of every position"""
    outs, at, i = [], 0, 0
    while at < len(toks):
        n = min(sizes[min(i, len(sizes) - 1)], len(toks) - at)
        outs.append(eng.step([entry(rid, toks[at:at + n])], [rid] if at + n == len(toks) else []))
        at, i = at + n, i + 1
    return torch.cat(outs)


def seq_params(row, held, n):
    """the kernels' description of a step that brings n tokens of one request that holds `held`"""
    from scratchpad_amd import _native
    dev = "cuda"
    rows, lens = torch.tensor([row], device=dev), torch.tensor([held + n], device=dev)
    if n == 1 and held > 0:
        return _native.SeqParams(rows, lens)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    return _native.SeqParams(rows, lens, i32([n]), i32([held]), i32([0]), torch.zeros(n, dtype=torch.int32, device=dev))


def portions(T, sizes):
    at, i = 0, 0
    while at < T:
        n = min(sizes[min(i, len(sizes) - 1)], T - at)
        yield at, n
        at, i = at + n, i + 1


# ------------------------------------------------------------------------------------------------ mechanisms alone
LAYERS = [
    (U.delta(3, 16), None), (U.delta(1, 40), None), (U.delta(2, 72), None), (U.delta(2, 136), None), (U.delta(5, 8), None),
    (U.parallel(4, 2, 16, 24, 2, 8, 40, dims=8), None),
    (U.parallel(3, 3, 24, 8, 1, 72, 8, scaling=False), None),              # kv heads = heads
    (U.parallel(5, 1, 8, 72, 3, 16, 16, dims=0), None),                    # no rotation, one kv head
    (U.parallel(2, 1, 40, 16, 2, 136, 136, dims=20), None),                # head width no multiple of 16; state above 128
    (U.parallel(2, 1, 136, 200, 4, 24, 200, dims=72, scale=0.05), None),
    (U.delta(2, 16), U.dense(100)), (U.parallel(2, 2, 16, 16, 2, 16, 16), U.dense(40)),
]


@pytest.mark.parametrize("layer", LAYERS, ids=lambda l: f"{l[0]['type']}-{'none' if l[1] is None else l[1]['kind']}")
def test_single_layer_models_match_oracle(tmp_path, layer):
    cfg = U.config([layer], width=80)
    folder, w = U.make_model(tmp_path, cfg, seed=5)
    toks = U.tokens(70, cfg["vocab"], 6)
    eng = engine(folder)
    eng.runner.model.capture_layers = []
    got = run_whole(eng, toks)
    lay = []
    want = to.forward(toks, w, cfg, lay)
    assert U.rel(eng.runner.model.capture_layers[0], lay[0]) < F32_BAR
    assert U.rel(got, want) < F32_BAR


# ------------------------------------------------------------------------------------------------ row kernels
@pytest.mark.parametrize("W", [200, 77, 3000], ids=["vectors", "scalars", "several-vectors-per-thread"])
def test_gated_add_norm_kernel_in_every_form(W):
    """rows of whole 16-byte vectors stay in registers; other widths take the scalar kernel"""
    from scratchpad_amd import _native
    g = torch.Generator().manual_seed(0)
    T, eps = 37, 1e-5
    rn = lambda *s: torch.randn(*s, generator=g)
    x, a, b, gate, extra = rn(T, W), rn(T, W) * 3, rn(T, W) * 0.2, rn(T, 2 * W), rn(T, W)
    w, wa, wb, gb, nw = (1 + 0.3 * rn(W) for _ in range(5))
    N = lambda z: z / torch.sqrt((z * z).mean(-1, keepdim=True) + eps)
    for dtype, bar in ((torch.float32, 2e-6), (torch.bfloat16, 1e-2)):
        r = lambda t: t.to(dtype).double()
        for two, gated, ex, nxt in ((0, 0, 0, 0), (0, 1, 0, 1), (1, 1, 1, 1), (1, 0, 0, 0), (0, 1, 1, 0)):
            y = r(a) if not two else 0.5 * (N(r(a)) * wa.double() + N(r(b)) * wb.double())
            if gated:
                y = y * torch.sigmoid(r(gate[:, W:]) + gb.double())
            want = x.double() + N(y) * w.double() + (extra.double() if ex else 0)
            xs = x.clone().cuda()
            out = _native.gated_add_norm(xs, a.to(dtype).cuda(), w.cuda(), eps,
                                         gate=gate.to(dtype).cuda()[:, W:] if gated else None,      # a view: its stride is taken
                                         gate_bias=gb.cuda() if gated else None, b=b.to(dtype).cuda() if two else None,
                                         wa=wa.cuda() if two else None, wb=wb.cuda() if two else None,
                                         extra=extra.cuda() if ex else None, next_weight=nw.cuda() if nxt else None)
            assert U.rel(xs, want) < 2e-6, (dtype, two, gated, ex)
            assert (out is not None) == bool(nxt)
            if nxt:
                assert out.dtype == dtype and U.rel(out, N(want) * nw.double()) < bar


def test_relu_square_and_scaled_soft_cap_kernels():
    from scratchpad_amd import _native
    g = torch.Generator().manual_seed(1)
    for dtype in (torch.float32, torch.bfloat16):
        for cols in (96, 77):                                   # 16-byte rows and rows that are not
            x = (torch.randn(33, 2 * cols, generator=g) * 3).to(dtype).cuda()
            got = _native.relu_square(x[:, cols:])
            assert torch.equal(got, (torch.relu(x[:, cols:].float()) ** 2).to(dtype))
            z = x[:, :cols]
            assert U.rel(_native.scale_softcap(z, 0.25, 7.0), 7.0 * torch.tanh(z.double() * 0.25 / 7.0)) < 2e-6
            assert U.rel(_native.scale_softcap(z, 3.0, 0.0), z.double() * 3.0) < 1e-6


# ------------------------------------------------------------------------------------------------ the recurrences
@pytest.mark.parametrize("sizes", [[300], [1], [7, 2, 40, 1, 1, 1, 3, 64, 1], [2]], ids=["whole", "decode", "mixed", "pairs"])
@pytest.mark.parametrize("shape", [(3, 16), (2, 40), (1, 128), (2, 200)], ids=lambda s: "x".join(map(str, s)))
def test_delta_recurrence_carries_its_state(shape, sizes):
    """decays of 0.995 and more keep what token 0 wrote visible at token 299, so a state lost or mixed up between portions
    shows; garbage in the slot before the first token must not"""
    from scratchpad_amd import _native
    H, D = shape
    T, n, rank = 300, H * D, 4
    g = torch.Generator().manual_seed(2)
    rn = lambda *s: torch.randn(*s, generator=g)
    r, k, v, gt, apre, p = rn(T, n), rn(T, n), rn(T, n), rn(T, n), rn(T, n) - 4.0, rn(T, rank)
    v[0] = 25.0                                                       # a loud first token
    w2t, w0, ab, nw = rn(rank, n) * 0.3, rn(n) * 0.3 - 7.0, rn(n) * 0.3, 1 + 0.2 * rn(n)
    rate = 0.7
    decay = torch.exp(-rate * torch.sigmoid(torch.tanh(p.double()) @ w2t.double() + w0.double()))
    remove = torch.sigmoid(apre.double() + ab.double())
    assert float(decay.min()) > 0.99
    o = to.delta_recurrence(*(t.double().view(T, H, D) for t in (r, k, v)), decay.view(T, H, D), remove.view(T, H, D))
    quiet = to.delta_recurrence(*(t.double().view(T, H, D) for t in (r, k, torch.cat([v[:1] * 0, v[1:]]))), decay.view(T, H, D),
                                remove.view(T, H, D))
    assert float((o[-1] - quiet[-1]).abs().max()) > 0.05 * float(o[-1].abs().max())      # token 0 is still heard at the end
    want = (to.rms(o, 1e-5).reshape(T, n) * nw.double() * torch.sigmoid(gt.double()))
    state = torch.full((4, H, D, D), float("nan"), device="cuda")
    outs = []
    for at, m in portions(T, sizes):
        cu = lambda t: t[at:at + m].cuda()
        dec, rem = _native.delta_gates(cu(p), w2t.cuda(), w0.cuda(), cu(apre), ab.cuda(), rate)
        assert U.rel(dec, decay[at:at + m]) < 1e-6 and U.rel(rem, remove[at:at + m]) < 1e-6
        outs.append(_native.delta_recurrence(cu(r), cu(k), cu(v), cu(gt), dec, rem, nw.cuda(), state, seq_params(2, at, m),
                                             H, D, 1e-5).cpu())
    assert U.rel(torch.cat(outs), want) < 5e-5
    assert torch.isnan(state[1]).all() and torch.isfinite(state[2]).all()


@pytest.mark.parametrize("sizes", [[300], [1], [7, 2, 40, 1, 1, 1, 3, 64, 1], [2]], ids=["whole", "decode", "mixed", "pairs"])
@pytest.mark.parametrize("shape", [(3, 16, 24), (2, 40, 8), (1, 128, 64), (2, 24, 256), (1, 200, 72)], ids=lambda s: "x".join(map(str, s)))
def test_forget_write_scan_carries_its_state(shape, sizes):
    """a third of the channels take token 0 in whole (forget gate 0 there) and keep it (gates of 0.999 afterwards), so it is
    still in the state at the end"""
    from scratchpad_amd import _native
    H, D, Dv = shape
    T = 300
    g = torch.Generator().manual_seed(3)
    rn = lambda *s: torch.randn(*s, generator=g)
    qpre, fpre, v = rn(T, H * D), rn(T, H * D), rn(T, H * Dv)
    v[0] = 25.0
    fb, nw = rn(H * D) * 0.5, 1 + 0.2 * rn(Dv)
    lower = torch.rand(H * D, generator=g) * 0.5
    lower[::3], fb[::3], fpre[0, ::3] = 0.0, 0.0, -20.0
    fpre[1:, ::3] = 7.0 + 0.3 * fpre[1:, ::3]
    q = to.silu(qpre.double()).view(T, H, D)
    f = (lower.double() + (1 - lower.double()) * torch.sigmoid(fpre.double() + fb.double())).view(T, H, D)
    o = to.forget_write_recurrence(q, f, v.double().view(T, H, Dv))
    quiet = to.forget_write_recurrence(q, f, torch.cat([v[:1] * 0, v[1:]]).double().view(T, H, Dv))
    assert float((o[-1] - quiet[-1]).abs().max()) > 0.05 * float(o[-1].abs().max())
    want = (to.rms(o, 1e-5) * nw.double()).reshape(T, H * Dv)
    state = torch.full((4, H, D, Dv), float("nan"), device="cuda")
    outs = []
    for at, m in portions(T, sizes):
        cu = lambda t: t[at:at + m].cuda()
        outs.append(_native.hgrn2_scan(cu(qpre), cu(fpre), cu(v), fb.cuda(), lower.cuda(), nw.cuda(), state, seq_params(2, at, m),
                                       H, D, Dv, 1e-5).cpu())
    assert U.rel(torch.cat(outs), want) < 5e-5
    assert torch.isnan(state[3]).all() and torch.isfinite(state[2]).all()


# ------------------------------------------------------------------------------------------------ attention with a sink
class SinkBench:
    """one request on row 2 of a request table whose slots are a shuffled part of a NaN-filled pool: biases, rotation, store
    and attention driven the way the model drives them, in portions"""

    def __init__(self, H, G, D, Dv, rot=None, dtype=torch.float32, slots=700, seed=0, matrix=True, sinks=None, biases=None,
                 scale=0.25):
        from scratchpad_amd import _native
        from scratchpad_amd.layers import AngleRotary
        self.n, self.H, self.G, self.D, self.Dv, self.dtype, self.scale = _native, H, G, D, Dv, dtype, scale
        g = torch.Generator().manual_seed(seed)
        self.perm = (torch.randperm(slots, generator=g) + 1).cuda()
        mk = lambda w: torch.full((slots + 1, w), float("nan"), dtype=dtype, device="cuda")       # reading a stale slot shows
        self.k, self.v = mk(G * D), mk(G * Dv)
        self.table = torch.zeros((4, slots + 8), dtype=torch.int32, device="cuda")
        self.rotary = AngleRotary(rot["dims"], rot["base"], rot.get("scaling")).cuda() if rot else None
        self.sinks = None if sinks is None else sinks.float().cuda()
        self.biases = [None if b is None else b.float().cuda() for b in (biases or (None, None, None))]
        self.held, self.matrix = 0, matrix

    def step(self, q, k, v):
        n_ = self.n
        n = q.shape[0]
        loc = self.perm[self.held:self.held + n].long()
        self.table[2, self.held:self.held + n] = loc.int()
        pos = torch.arange(self.held, self.held + n, device="cuda")
        seq = seq_params(2, self.held, n)
        q = q.to(self.dtype).cuda().clone()
        freq, mag = (self.rotary.freq, self.rotary.magnitude) if self.rotary else (None, 1.0)
        n_.qkv_rotary_store(q, k.to(self.dtype).cuda(), v.to(self.dtype).cuda(), self.k, self.v, pos, loc, freq, mag,
                            self.H, self.G, self.D, self.Dv, 1e-6, adjacent=True, norm_values=False, q_bias=self.biases[0],
                            k_bias=self.biases[1], v_bias=self.biases[2])
        out = n_.window_attention(q, self.k, self.v, None, None, self.table, seq, self.H, self.G, self.D, self.Dv, 0, 0,
                                  self.scale, self.matrix, sinks=self.sinks)
        self.held += n
        return out.float().cpu()

    def run(self, q, k, v, sizes):
        return torch.cat([self.step(q[at:at + m], k[at:at + m], v[at:at + m]) for at, m in portions(q.shape[0], sizes)])


def sink_oracle(q, k, v, H, G, D, Dv, sinks, rot=None, biases=(0, 0, 0), scale=0.25):
    T = q.shape[0]
    q, k, v = (t.double() + (b.double() if torch.is_tensor(b) else 0) for t, b in zip((q, k, v), biases))
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, Dv)
    q, k = to.rotate_adjacent_pairs(q, rot), to.rotate_adjacent_pairs(k, rot)
    return to.sink_attention(q, k, v, sinks.double(), scale).reshape(T, H * Dv)


@pytest.mark.parametrize("sizes", [[150], [1], [7, 2, 40, 1, 1, 1, 3, 64, 1], [2]], ids=["whole", "decode", "mixed", "pairs"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 24, 8), (2, 2, 8, 8, 8), (3, 1, 24, 72, 10), (6, 3, 40, 16, 0), (2, 1, 136, 200, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_sink_attention_with_biases_and_partial_rotation(shape, sizes):
    """peaked softmaxes (scores of a few units), sinks between -2 and 4: a key that is wrongly seen or missed, a sink that is
    left out or scaled, a bias that is left out or a pair that is rotated with the wrong partner moves the output by far
    more than the bar; every position of 150 is compared"""
    H, G, D, Dv, dims = shape
    g = torch.Generator().manual_seed(3)
    T = 150
    q, k, v = torch.randn(T, H * D, generator=g) * 2, torch.randn(T, G * D, generator=g) * 2, torch.randn(T, G * Dv, generator=g)
    biases = [torch.randn(n, generator=g) for n in (H * D, G * D, G * Dv)]
    sinks = torch.linspace(-2.0, 4.0, H)
    rot = {"dims": dims, "base": 100.0, "scaling": {"factor": 2.0, "low": 1.0, "high": 4.0, "original": 32}} if dims else None
    got = SinkBench(H, G, D, Dv, rot, sinks=sinks, biases=biases).run(q, k, v, sizes)
    want = sink_oracle(q, k, v, H, G, D, Dv, sinks, rot, biases)
    assert U.rel(got, want) < 2e-5
    # the oracle itself moves when a piece is left out: the comparison above can tell
    assert U.rel(sink_oracle(q, k, v, H, G, D, Dv, sinks - 50.0, rot, biases), want) > 1e-2
    assert U.rel(sink_oracle(q, k, v, H, G, D, Dv, sinks, rot), want) > 1e-2


def test_far_key_and_a_tempting_future_key():
    """one loud key at position 3 among 600 quiet ones: every later query hears it, in a prompt of 600 and decoded token by
    token behind a prompt; a louder key at position p + 1 must never reach query p; the first query sees itself and the
    sink only"""
    H = G = 1
    D, Dv, T = 16, 64, 600
    g = torch.Generator().manual_seed(1)
    q, k, v = torch.randn(T, D, generator=g) * 0.1, torch.randn(T, D, generator=g) * 0.1, torch.randn(T, Dv, generator=g)
    q[:, 0], k[3, 0] = 6.0, 8.0
    v[3] = torch.arange(Dv) - 31.5
    k[400, 0], v[400] = 30.0, 1000.0                     # position 399 must not see it; 400 and later do
    sinks = torch.tensor([2.0])
    want = sink_oracle(q, k, v, H, G, D, Dv, sinks)
    loud = v[3].double()
    cos = lambda a: float(torch.dot(a.double(), loud) / a.double().norm() / loud.norm())
    assert cos(want[399]) > 0.99 and abs(cos(want[2])) < 0.5 and float(want[400].min()) > 900
    # the first token: weight exp(s) / (exp(s) + exp(sink)) on its own value
    s0 = float(q[0].double() @ k[0].double()) * 0.25
    assert torch.allclose(want[0], v[0].double() * (math.exp(s0) / (math.exp(s0) + math.exp(2.0))), atol=1e-12)
    for sizes in ([T], [390, 1], [64]):
        got = SinkBench(H, G, D, Dv, sinks=sinks).run(q, k, v, sizes)
        assert cos(got[399]) > 0.99 and cos(got[150]) > 0.99 and float(got[399].max()) < 100
        assert U.rel(got, want) < 2e-5


def test_sink_attention_kernels_in_bf16():
    H, G, D, Dv, T = 4, 2, 32, 32, 120
    g = torch.Generator().manual_seed(2)
    q, k, v = torch.randn(T, H * D, generator=g), torch.randn(T, G * D, generator=g), torch.randn(T, G * Dv, generator=g)
    sinks = torch.tensor([0.0, 1.0, 2.0, -1.0])
    got = SinkBench(H, G, D, Dv, dtype=torch.bfloat16, sinks=sinks).run(q, k, v, [50, 1])
    r = lambda x: x.bfloat16().float()
    assert U.rel(got, sink_oracle(r(q), r(k), r(v), H, G, D, Dv, sinks)) < 3e-2


@pytest.mark.parametrize("sizes", [[200], [17, 2, 64, 1, 1, 33, 16, 5], [3]], ids=["whole", "mixed", "threes"])
@pytest.mark.parametrize("shape", [(8, 2, 128, 128), (4, 4, 64, 128), (6, 1, 128, 64)], ids=lambda s: "x".join(map(str, s)))
def test_matrix_core_attention_with_sinks_against_the_vector_kernel(shape, sizes):
    """portions of prompts in bf16 with heads of 64 / 128 run on the matrix cores; the sink joins the denominator after the
    last key tile.  Same cache, same portions, against the fp32-arithmetic vector kernel that the tests above pin."""
    H, G, D, Dv = shape
    g = torch.Generator().manual_seed(7)
    T = 200
    q, k, v = torch.randn(T, H * D, generator=g) * 0.7, torch.randn(T, G * D, generator=g) * 0.7, torch.randn(T, G * Dv, generator=g)
    sinks = torch.linspace(-1.0, 6.0, H)
    rot = {"dims": D // 2, "base": 100.0}
    outs = [SinkBench(H, G, D, Dv, rot, dtype=torch.bfloat16, matrix=m, sinks=sinks, scale=D ** -0.5).run(q, k, v, sizes)
            for m in (True, False)]
    assert torch.isfinite(outs[0]).all()
    assert U.rel(outs[0], outs[1]) < 1.2e-2
    off = SinkBench(H, G, D, Dv, rot, dtype=torch.bfloat16, matrix=True, sinks=sinks - 60.0, scale=D ** -0.5).run(q, k, v, sizes)
    assert U.rel(off, outs[0]) > 5e-2                                   # the sink carries weight in this test


# ------------------------------------------------------------------------------------------------ the whole model
@pytest.fixture(scope="module")
def full(tmp_path_factory):
    cfg = U.full_config()
    folder, w = U.make_model(tmp_path_factory.mktemp("full"), cfg, seed=11, rank=6)
    toks = U.tokens(130, cfg["vocab"], 12)
    lay = []
    want = to.forward(toks, w, cfg, lay)
    return cfg, folder, w, toks, want, lay


def test_whole_prompt_and_every_layer_run(full):
    cfg, folder, w, toks, want, lay = full
    eng = engine(folder)
    eng.runner.model.capture_layers = []
    got = run_whole(eng, toks)
    runs = to.layer_runs(cfg)
    assert len(eng.runner.model.capture_layers) == len(lay) == len(runs)
    for i, (a, b) in enumerate(zip(eng.runner.model.capture_layers, lay)):
        assert U.rel(a, b) < F32_BAR, f"run {i} (layer {runs[i]}, {cfg['layers'][runs[i]]['type']})"
    assert U.rel(got, want) < F32_BAR
    eng.runner.model.capture_layers = None                  # the fused tails (next norm and the pass's added rows inside)
    assert U.rel(run_whole(eng, toks), want) < F32_BAR


@pytest.mark.parametrize("loop", [None, (0, 5, 2), (0, 1, 3), (4, 5, 2), (2, 4, 1), (3, 3, 4)], ids=str)
def test_loops_over_other_parts_of_the_layer_list(full, tmp_path, loop):
    cfg, _, w, toks, _, _ = full
    cfg = {k: v for k, v in cfg.items() if k != "loop"}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    folder = U.write_checkpoint(str(tmp_path / "m"), cfg, w)
    want = to.forward(toks[:60], w, cfg)
    assert U.rel(run_whole(engine(folder), toks[:60]), want) < F32_BAR
    assert U.rel(run_portions(engine(folder), toks[:60], [9, 1, 1, 2]), want) < F32_BAR


def test_bf16_serving_precision(full):
    cfg, folder, w, toks, want, _ = full
    got = run_portions(engine(folder, dtype=torch.bfloat16), toks, [40, 1]).double().cpu()
    err = ((got - want) ** 2).mean(-1).sqrt() / (want ** 2).mean(-1).sqrt()
    assert float(err.median()) < 0.03 and float(err.max()) < 0.15, err


def test_bf16_model_whose_prompts_take_the_matrix_core_attention(tmp_path):
    cfg = U.config([(U.parallel(4, 2, 64, 128, 2, 32, 64, dims=32), U.dense(96)),
                    (U.parallel(2, 1, 128, 64, 1, 64, 64), None)], width=128)
    folder, w = U.make_model(tmp_path, cfg, seed=9)
    toks = U.tokens(150, cfg["vocab"], 2)
    want = to.forward(toks, w, cfg)
    outs = [run_portions(engine(folder, dtype=torch.bfloat16), toks, sizes).double().cpu() for sizes in ([150], [33, 1], [1])]
    for got in outs:
        err = ((got - want) ** 2).mean(-1).sqrt() / (want ** 2).mean(-1).sqrt()
        assert float(err.median()) < 0.03 and float(err.max()) < 0.15, err
    assert U.rel(outs[0], outs[2]) < 0.1 and U.rel(outs[1], outs[2]) < 0.1


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_decoding_token_by_token_from_the_first_token(full, graphs):
    """130 single-token steps from an empty cache and state"""
    cfg, folder, w, toks, want, _ = full
    assert U.rel(run_portions(engine(folder, graphs=graphs), toks, [1]), want) < F32_BAR


def test_long_decoding_behind_a_prompt(full):
    cfg, folder, w, _, _, _ = full
    toks = U.tokens(420, cfg["vocab"], 77)
    want = to.forward(toks, w, cfg)
    assert U.rel(run_portions(engine(folder, graphs=True), toks, [60, 1]), want) < F32_BAR


@pytest.mark.parametrize("sizes", [[2], [3, 2, 17, 1, 1, 64, 5, 1], [64, 2, 1], [15, 16, 17, 1]],
                         ids=["pairs", "mixed", "big-then-small", "near-16"])
def test_portions_of_prompts(full, sizes):
    cfg, folder, w, toks, want, _ = full
    assert U.rel(run_portions(engine(folder), toks, sizes), want) < F32_BAR


def test_garbage_in_reused_rows_and_slots_is_never_read(full):
    """every state tensor and cache buffer poisoned before a request starts: a first token must start from the initial
    state and see only its own keys"""
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
    """seven requests of unequal length through three rows and a pool that holds far fewer tokens than their sum:
    portions of some beside single tokens of others, pauses, rows and slots handed on; every request's logits must be
    what it gets alone"""
    cfg, folder, w, _, _, _ = full
    reqs = {f"r{i}": U.tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate([45, 3, 70, 1, 26, 58, 12])}
    want = {r: to.forward(t, w, cfg) for r, t in reqs.items()}
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
    """40 requests decoding together: steps above 16 rows take the library's products inside the captured graph.  Every
    replay (six of them, with the eager prompt steps of the other engine and synchronisations between) is compared with
    the same step run eagerly."""
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
        want = torch.stack([to.forward(t, w, cfg)[-6:] for t in reqs.values()], 1)    # [step, request, vocab]
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
            lg = to.forward(p + ref[:agree], w, cfg)[-1]
            assert float(lg[ref[agree]] - lg[out[agree]]) < 1e-3 * float(lg.abs().max()), (agree, out, ref)
        else:
            assert out == ref
    sampled = eng.generate(prompts[:2], SamplingParams(max_new_tokens=6, temperature=0.8, top_p=0.9, top_k=20))
    assert all(len(o) == 6 and all(0 <= t < cfg["vocab"] for t in o) for o in sampled)


@pytest.mark.parametrize("seed", range(10))
def test_designs_drawn_at_random(tmp_path, seed):
    """layer order, loop, sizes and constants drawn at random (toredra_util.random_config): whole prompt, then portions of
    random sizes with single tokens between them, both against the oracle"""
    import random
    cfg = U.random_config(100 + seed)
    folder, w = U.make_model(tmp_path, cfg, seed=seed, rank=3 + seed)
    toks = U.tokens(90, cfg["vocab"], seed)
    want = to.forward(toks, w, cfg)
    assert U.rel(run_whole(engine(folder), toks), want) < F32_BAR, cfg
    r = random.Random(seed)
    sizes = [r.choice([1, 1, 2, 3, 7, 16, 29]) for _ in range(40)]
    assert U.rel(run_portions(engine(folder), toks, sizes), want) < F32_BAR, (sizes, cfg)


def test_sizes_that_are_one_or_equal(tmp_path):
    """a second model whose sizes are 1 or equal where the first one's differ: one head everywhere, key width = value
    width = model width, rotation over the whole head, a loop of one layer run once, scale 1 and no cap on the logits"""
    cfg = U.config([
        (U.parallel(1, 1, 16, 16, 1, 16, 16, dims=16, scale=1.0), U.dense(16)),
        (U.delta(1, 16), U.dense(16)),
    ], width=16, vocab=17, loop=(0, 1, 1), logit_scale=1.0, softcap=None)
    folder, w = U.make_model(tmp_path, cfg, seed=4, rank=1)
    toks = U.tokens(50, 17, 3)
    want = to.forward(toks, w, cfg)
    assert U.rel(run_whole(engine(folder), toks), want) < F32_BAR
    assert U.rel(run_portions(engine(folder), toks, [3, 1]), want) < F32_BAR
