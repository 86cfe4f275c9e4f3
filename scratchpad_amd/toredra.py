"""Toredra: a decoder-only design of sequential sublayers over an fp32 residual stream whose results are gated and normed
before they join it,
    h = N(x) w1;   x <- x + N(mixer(h) * sigmoid(R1 h + b1)) w1b;      h = N(x) w2;   x <- x + N(ff(h) * sigmoid(R2 h + b2)) w2b,
with N = division by the row's root mean square.  The mixer is, layer by layer, a generalized delta rule (a per-head
matrix state with per-channel decay and removal along the unit key) or two mixers side by side on the same input -
grouped-query attention with biases, adjacent-pair rotary on part of each head (frequencies rescaled by wavelength), a
constant attention scale and a learned sink per head in the softmax's denominator, beside a linear attention whose forget
gate also writes - each normed over the model width and averaged.  The feed-forward is W_down relu(W_up h)^2.  A stretch
of the layer list can run several times in a row on the same weights, every run with a cache and a state of its own; each
pass after the first starts from x + (the embedding rows).  The head is the embedding table; logits are scaled and
soft-capped.

Everything that differs between models of the design comes from config.json (``ToredraConfig``) or a tensor's shape; the
model is assembled from the framework's mechanisms - ShiftedRMSNorm / AngleRotary / GatedAddNorm / ReluSquareFF
(layers.py), PooledWindowAttention + SequenceBackend (attention.py), GeneralDeltaMixer / HGRN2Mixer (recurrent.py),
WindowKVPool + RecurrentStatePool (pool.py), LogitsProcessor (llama.py) - and served by the ModelRunner like the other
model classes.  A cache layer / state id is the index of a layer RUN, not of a layer."""
from typing import Dict, Iterable, List, Optional, Tuple

import torch
from torch import nn

from . import _native
from .attention import PooledWindowAttention
from .forward_info import ForwardBatch
from .layers import AngleRotary, GatedAddNorm, ReluSquareFF, ShiftedRMSNorm
from .llama import LogitsProcessor, LogitsProcessorOutput, ParallelLMHead
from .recurrent import GeneralDeltaMixer, HGRN2Mixer

MIXERS = ("general_delta", "parallel")


class ToredraConfig:
    """config.json of the design, plus what the runner asks of any model configuration (vocab_size, context_len,
    num_hidden_layers, is_encoder_decoder) and what it builds the pools from."""
    architecture = "Toredra"
    is_encoder_decoder = False
    vision_config = None

    def __init__(self, raw: dict, context_len: int = 8192, tensor_shapes: Optional[Dict[str, Tuple[int, ...]]] = None,
                 decay_rank: int = 64):
        self.raw = raw
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.layers: List[dict] = raw["layers"]
        self.num_hidden_layers = len(self.layers)
        self.rms_norm_eps = float(raw["norm"]["eps"])
        self.logit_scale = float(raw.get("logit_scale", 1.0))
        self.final_logit_softcapping = float(raw.get("logit_softcap") or 0.0)
        self.context_len = context_len
        self.tie_word_embeddings = True
        self.tensor_shapes = tensor_shapes or {}
        self.default_decay_rank = decay_rank          # models without a checkpoint (random weights)
        for layer in self.layers:
            if layer["type"] not in MIXERS:
                raise ValueError(f"unknown layer type {layer['type']!r}")
            if layer.get("mlp") is not None and layer["mlp"]["kind"] != "dense":
                raise ValueError(f"unknown feed-forward kind {layer['mlp']['kind']!r}")
        loop = raw.get("loop") or {}
        n = len(self.layers)
        start, stop, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
        if not (0 <= start <= stop <= n) or times < 1:
            raise ValueError(f"loop {loop!r} does not fit {n} layers")
        if stop == start:
            times = 1
        # the layer runs in order: (layer index, whether the embedding rows join the stream right before this run)
        self.runs: List[Tuple[int, bool]] = [(i, False) for i in range(start)]
        for p in range(times):
            self.runs += [(i, p > 0 and i == start) for i in range(start, stop)]
        self.runs += [(i, False) for i in range(stop, n)]

    def decay_rank(self, layer: int) -> int:
        """rows of the decay's first projection: a checkpoint's tensor shape gives it"""
        shape = self.tensor_shapes.get(f"l{layer}.mix.w1")
        return int(shape[0]) if shape else self.default_decay_rank

    # ---- what the runner builds its pools from (keys: the index of a layer run)
    def window_cache(self):
        """{run: (kv_heads, dim, vdim, pooled)} of the runs that keep a key/value row per token"""
        out = {}
        for r, (i, _) in enumerate(self.runs):
            if self.layers[i]["type"] == "parallel":
                m = self.layers[i]["mixer"]["left"]
                out[r] = (int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), False)
        return out

    def shift_layers(self):
        return []                                     # no mixer reads the previous token's input

    def named_state(self):
        """{run: {name: shape}} of the fp32 state the recurrent mixers carry per request"""
        out = {}
        for r, (i, _) in enumerate(self.runs):
            m = self.layers[i]["mixer"]
            if self.layers[i]["type"] == "general_delta":
                out[r] = GeneralDeltaMixer.state_shapes(int(m["heads"]), int(m["dim"]))
            else:
                m = m["right"]
                out[r] = HGRN2Mixer.state_shapes(int(m["heads"]), int(m["dim"]), int(m["vdim"]))
        return out

    def cache_bytes_per_token(self, kv_dtype: torch.dtype) -> int:
        per = sum(g * (d + dv) for g, d, dv, _ in self.window_cache().values())
        return max(1, per * torch.finfo(kv_dtype).bits // 8)


class ToredraParallel(nn.Module):
    """Two mixers on the same input: attention with a sink (left) and a forget-write linear attention (right).  ONE
    product makes the rows [q | k | v (left) | q | f | v (right) | extra]; the two results go back separately (the layer
    norms each over the model width and averages them)."""

    def __init__(self, width: int, m: dict, eps: float, extra_rows: int = 0, dtype=None):
        super().__init__()
        a, b = m["left"], m["right"]
        H, G, D, Dv = (int(a[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        self.heads, self.kv_heads, self.dim, self.vdim, self.eps, self.extra_rows = H, G, D, Dv, eps, extra_rows
        self.left_rows = H * D + G * D + G * Dv
        self.right = HGRN2Mixer(width, int(b["heads"]), int(b["dim"]), int(b["vdim"]), eps, own_input=False, dtype=dtype)
        self.in_proj = nn.Parameter(torch.empty(self.left_rows + self.right.in_rows + extra_rows, width, dtype=dtype),
                                    requires_grad=False)
        f32 = dict(dtype=torch.float32)
        self.q_bias = nn.Parameter(torch.zeros(H * D, **f32), requires_grad=False)
        self.k_bias = nn.Parameter(torch.zeros(G * D, **f32), requires_grad=False)
        self.v_bias = nn.Parameter(torch.zeros(G * Dv, **f32), requires_grad=False)
        self.left_o = nn.Parameter(torch.empty(width, H * Dv, dtype=dtype), requires_grad=False)
        rot = a.get("rot")
        self.rotary = None
        if rot and int(rot["dims"]) > 0:
            if int(rot["dims"]) > D:
                raise ValueError("rot.dims exceeds the head size")
            self.rotary = AngleRotary(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        self.attn = PooledWindowAttention(H, G, D, Dv, float(a["scale"]), None, sinks=True, norm_values=False)

    def forward(self, positions, h: torch.Tensor, forward_batch: ForwardBatch, run: int):
        nq, nk, nv = self.heads * self.dim, self.kv_heads * self.dim, self.kv_heads * self.vdim
        a = _native.linear(h, self.in_proj)
        q = a[:, :nq]
        self.attn.store(q, a[:, nq:nq + nk], a[:, nq + nk:self.left_rows], self.rotary, positions, self.eps, forward_batch,
                        cache_id=run, biases=(self.q_bias.data, self.k_bias.data, self.v_bias.data))
        left = _native.linear(self.attn(q, forward_batch, cache_id=run), self.left_o)
        right = self.right.scan(a[:, self.left_rows:], forward_batch, state_id=run)
        return (left, right), (a[:, self.left_rows + self.right.in_rows:] if self.extra_rows else None)


class ToredraLayer(nn.Module):
    def __init__(self, config: ToredraConfig, layer_id: int, dtype=None):
        super().__init__()
        spec, W, eps = config.layers[layer_id], config.hidden_size, config.rms_norm_eps
        self.kind = spec["type"]
        m = spec["mixer"]
        self.norm1 = ShiftedRMSNorm(W, eps, shift=False)
        if self.kind == "parallel":
            self.mix = ToredraParallel(W, m, eps, extra_rows=W, dtype=dtype)
            self.tail1 = GatedAddNorm(W, eps, branches=2)
        else:
            self.mix = GeneralDeltaMixer(W, int(m["heads"]), int(m["dim"]), config.decay_rank(layer_id), eps, extra_rows=W,
                                         dtype=dtype)
            self.tail1 = GatedAddNorm(W, eps)
        self.mlp = None
        if spec.get("mlp") is not None:
            self.norm2 = ShiftedRMSNorm(W, eps, shift=False)
            self.mlp = ReluSquareFF(W, int(spec["mlp"]["ff"]), extra_rows=W, dtype=dtype)
            self.tail2 = GatedAddNorm(W, eps)

    def forward(self, positions, x: torch.Tensor, h: torch.Tensor, forward_batch: ForwardBatch, run: int,
                next_weight: Optional[torch.Tensor], extra: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """x: the fp32 stream, updated in place; h = N(x) * norm1 in the projections' dtype.  Returns N(x') * next_weight of
        the stream as this run leaves it (x' includes ``extra``, the rows a further pass adds before its first layer)."""
        y, gate = self.mix(positions, h, forward_batch, run) if self.kind == "parallel" else self.mix(h, forward_batch, run)
        if self.mlp is None:
            return self.tail1(x, y, gate, extra=extra, next_weight=next_weight)
        h = self.tail1(x, y, gate, next_weight=self.norm2.weight.data)
        y, gate = self.mlp(h)
        return self.tail2(x, y, gate, extra=extra, next_weight=next_weight)


class ToredraForCausalLM(nn.Module):
    # parameters keep the dtypes they are declared with (fp32 norms, biases of gates, decays) whatever the runner's dtype
    keeps_parameter_dtypes = True
    supports_tensor_parallel = False
    # Largest decode step that is captured into a HIP graph (the step has no host synchronisation and no data-dependent
    # shape); larger steps run eagerly.
    max_graph_batch = 64
    # sources of the HIP library this model's path needs beyond the core (scratchpad_amd.build.build_native(only=...))
    NATIVE_SOURCES = ["stream_norm.hip", "window_attention.hip", "delta_rule.hip", "hgrn.hip"]

    def __init__(self, config: ToredraConfig, dtype=None):
        super().__init__()
        self.config = config
        self.dtype = dtype or torch.get_default_dtype()
        self.layers = nn.ModuleList([ToredraLayer(config, i, dtype) for i in range(config.num_hidden_layers)])
        self.norm = ShiftedRMSNorm(config.hidden_size, config.rms_norm_eps, shift=False)
        self.lm_head = ParallelLMHead(config.vocab_size, config.hidden_size, dtype)      # also the embedding table
        self.logits_processor = LogitsProcessor(config)
        self.capture_layers: Optional[list] = None     # set to a list to collect the stream after every layer run

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch: ForwardBatch, input_embeds=None) -> LogitsProcessorOutput:
        runs, table = self.config.runs, self.lm_head.weight
        x = _native.embed_scale(table.data, input_ids, 1.0)
        x0 = x.clone() if any(again for _, again in runs) else None
        dtype = table.dtype
        h = self.layers[runs[0][0]].norm1(x, dtype) if runs else None
        for r, (i, _) in enumerate(runs):
            nxt = runs[r + 1] if r + 1 < len(runs) else None
            next_weight = (self.layers[nxt[0]].norm1 if nxt else self.norm).weight.data
            extra = x0 if nxt and nxt[1] else None
            if self.capture_layers is None:
                h = self.layers[i](positions, x, h, forward_batch, r, next_weight, extra)
            else:                                      # the stream as the run leaves it, before a next pass adds to it
                self.layers[i](positions, x, h, forward_batch, r, None, None)
                self.capture_layers.append(x.clone())
                if extra is not None:
                    _native.stream_add(x, extra)
                h = (self.layers[nxt[0]].norm1 if nxt else self.norm)(x, dtype)
        if h is None:
            h = self.norm(x, dtype)
        return self.logits_processor(input_ids, h, self.lm_head, forward_batch)

    # ---- weights --------------------------------------------------------------------------------------------------
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> None:
        """Checkpoint names of the design ('embed', 'l<i>.norm1|norm1b|norm2|norm2b', 'l<i>.rg1|rg2' with '.b',
        'l<i>.mix.*', 'l<i>.mlp.up|down', 'final.norm') -> this module's (partly merged) parameters."""
        w = dict(weights)
        used = set()

        def take(name):
            used.add(name)
            return w[name]

        def put(param: nn.Parameter, value: torch.Tensor):
            value = value.reshape(param.shape) if value.numel() == param.numel() and value.dim() != param.dim() else value
            if value.shape != param.shape:
                raise RuntimeError(f"shape {tuple(value.shape)} does not fit parameter {tuple(param.shape)}")
            param.data.copy_(value.to(param.dtype))

        put(self.lm_head.weight, self.lm_head.shard_from_full(take("embed")))
        put(self.norm.weight, take("final.norm"))
        for i, layer in enumerate(self.layers):
            p, mix = f"l{i}", layer.mix
            put(layer.norm1.weight, take(f"{p}.norm1"))
            put(layer.tail1.weight, take(f"{p}.norm1b"))
            put(layer.tail1.gate_bias, take(f"{p}.rg1.b"))
            gate = take(f"{p}.rg1")
            if layer.kind == "parallel":
                L, R = f"{p}.mix.left", f"{p}.mix.right"
                put(mix.in_proj, torch.cat([take(f"{L}.q"), take(f"{L}.k"), take(f"{L}.v"), take(f"{R}.q"), take(f"{R}.f"),
                                            take(f"{R}.v"), gate], 0))
                put(mix.q_bias, take(f"{L}.q.b"))
                put(mix.k_bias, take(f"{L}.k.b"))
                put(mix.v_bias, take(f"{L}.v.b"))
                put(mix.attn.sinks, take(f"{L}.sink"))
                put(mix.left_o, take(f"{L}.o"))
                put(mix.right.f_bias, take(f"{R}.f.b"))
                put(mix.right.lower, take(f"{R}.lower"))
                put(mix.right.norm, take(f"{R}.norm"))
                put(mix.right.o, take(f"{R}.o"))
                put(layer.tail1.branch_weight, torch.stack([take(f"{L}.out"), take(f"{R}.out")]))
            else:
                M = f"{p}.mix"
                put(mix.in_proj, torch.cat([take(f"{M}.{s}") for s in ("r", "k", "v", "g", "a", "w1")] + [gate], 0))
                put(mix.w2t, take(f"{M}.w2").t().contiguous())
                put(mix.w0, take(f"{M}.w0"))
                put(mix.a_bias, take(f"{M}.a.b"))
                put(mix.norm, take(f"{M}.norm"))
                put(mix.o, take(f"{M}.o"))
            if layer.mlp is not None:
                put(layer.norm2.weight, take(f"{p}.norm2"))
                put(layer.tail2.weight, take(f"{p}.norm2b"))
                put(layer.tail2.gate_bias, take(f"{p}.rg2.b"))
                put(layer.mlp.up, torch.cat([take(f"{p}.mlp.up"), take(f"{p}.rg2")], 0))
                put(layer.mlp.down, take(f"{p}.mlp.down"))
        extra = set(w) - used
        if extra:
            import warnings
            warnings.warn(f"checkpoint tensors no part of the configured model reads: {sorted(extra)[:8]}")

    def init_random(self, generator: torch.Generator) -> None:
        """random weights of a plausible scale (benchmarks and tests of the host path: no checkpoint)"""
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("weight", "norm", "branch_weight") and p.dim() <= 2 and "lm_head" not in name:
                p.data.fill_(1.0)
            elif leaf == "lower":
                p.data.uniform_(0.0, 0.9, generator=generator)
            elif leaf == "w0":
                p.data.normal_(-1.0, 1.0, generator=generator)
            elif p.dim() >= 2:
                p.data.normal_(0.0, 1.0 / (p.shape[-1] ** 0.5), generator=generator)
            else:
                p.data.normal_(0.0, 0.1, generator=generator)
