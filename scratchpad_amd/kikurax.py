"""Kikurax: a decoder-only design of sequential pre-norm sublayers over an fp32 residual stream,
    x <- x + mixer(GN(x) w1);    x <- x + ff(GN(x) w2),
GN being the root-mean-square norm taken separately over ``norm.groups`` equal parts of the row.  The mixer is, layer by
layer, one of three: grouped-query softmax attention (biases, rotate-half rotary on part of each head with frequencies
rescaled by wavelength, q and k normed per head after the rotation, a learned score multiplier per head, capped scores,
a sink of score zero in the denominator, values blended with the first such layer's values of the same token); a
Mamba-2 state-space mixer; or two mixers side by side on the same input, each normed over the model width and averaged -
a sigmoid-weighted attention (no softmax, a learned bias per head, queries that grow with the logarithm of the position,
an output gate) beside a delta rule with a decay per key channel (short convolutions, unit keys, low-rank decay and
gate).  The feed-forward is a mixture of clamped gated experts chosen by the largest router logits and weighted by the
softmax over the chosen ones.  The embedding is scaled by a constant; the head is the embedding table.

Everything that differs between models of the design comes from config.json (``KikuraxConfig``) or a tensor's shape; the
model is assembled from the framework's mechanisms - GroupRMSNorm / HalfAngleRotary (layers.py), PooledWindowAttention +
SequenceBackend (attention.py), Mamba2Mixer / GatedDeltaMixer (recurrent.py), ChosenSoftmaxMoE (moe.py), WindowKVPool +
RecurrentStatePool (pool.py), LogitsProcessor (llama.py) - and served by the ModelRunner like the other model classes."""
from typing import Dict, Iterable, List, Optional, Tuple

import torch
from torch import nn

from . import _native
from .attention import PooledWindowAttention
from .forward_info import ForwardBatch
from .layers import GroupRMSNorm, HalfAngleRotary, add_join
from .llama import LogitsProcessor, LogitsProcessorOutput, ParallelLMHead
from .moe import ChosenSoftmaxMoE
from .recurrent import GatedDeltaMixer, Mamba2Mixer

MIXERS = ("attention", "mamba2", "parallel")


class KikuraxConfig:
    """config.json of the design, plus what the runner asks of any model configuration (vocab_size, context_len,
    num_hidden_layers, is_encoder_decoder) and what it builds the pools from."""
    architecture = "Kikurax"
    is_encoder_decoder = False
    vision_config = None

    def __init__(self, raw: dict, context_len: int = 8192, tensor_shapes: Optional[Dict[str, Tuple[int, ...]]] = None,
                 low_rank: int = 32):
        self.raw = raw
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.layers: List[dict] = raw["layers"]
        self.num_hidden_layers = len(self.layers)
        self.rms_norm_eps = float(raw["norm"]["eps"])
        self.norm_groups = int(raw["norm"].get("groups", 1))
        self.embedding_scale = float((raw.get("embedding") or {}).get("scale", 1.0))
        self.context_len = context_len
        self.tie_word_embeddings = True
        self.tensor_shapes = tensor_shapes or {}
        self.default_low_rank = low_rank              # models without a checkpoint (random weights)
        if self.hidden_size % self.norm_groups:
            raise ValueError("the width does not divide into norm.groups")
        self.v_first_layer: Optional[int] = None      # the first attention layer whose values the later ones blend in
        for i, layer in enumerate(self.layers):
            if layer["type"] not in MIXERS:
                raise ValueError(f"unknown layer type {layer['type']!r}")
            if layer.get("mlp") is not None and layer["mlp"]["kind"] != "moe":
                raise ValueError(f"unknown feed-forward kind {layer['mlp']['kind']!r}")
            if layer["type"] == "attention" and layer["mixer"].get("v_mix"):
                m = layer["mixer"]
                if self.v_first_layer is None:
                    self.v_first_layer = i
                else:
                    f = self.layers[self.v_first_layer]["mixer"]
                    if (int(m["kv_heads"]), int(m["vdim"])) != (int(f["kv_heads"]), int(f["vdim"])):
                        raise ValueError("layers that blend values must agree on kv_heads and vdim")

    def rank(self, layer: int, name: str) -> int:
        """rows of a low-rank first projection ('a1', 'g1') of a parallel layer's right mixer: a checkpoint's tensor shape
        gives it"""
        shape = self.tensor_shapes.get(f"l{layer}.mix.right.{name}")
        return int(shape[0]) if shape else self.default_low_rank

    # ---- what the runner builds its pools from
    def window_cache(self):
        """{layer id: (kv_heads, dim, vdim, pooled)} of the layers that keep a key/value row per token"""
        out = {}
        for i, l in enumerate(self.layers):
            m = l["mixer"] if l["type"] == "attention" else (l["mixer"]["left"] if l["type"] == "parallel" else None)
            if m is not None:
                out[i] = (int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), False)
        return out

    def shift_layers(self):
        return []                                     # no mixer reads the previous token's input

    def named_state(self):
        """{layer id: {name: shape}} of the fp32 state the recurrent mixers carry per request"""
        out = {}
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            if l["type"] == "mamba2":
                out[i] = Mamba2Mixer.state_shapes(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]))
            elif l["type"] == "parallel":
                r = m["right"]
                out[i] = GatedDeltaMixer.state_shapes(int(r["heads"]), int(r["kv_heads"]), int(r["dim"]), int(r["vdim"]),
                                                      int(r["conv"]))
        return out

    def cache_bytes_per_token(self, kv_dtype: torch.dtype) -> int:
        per = sum(g * (d + dv) for g, d, dv, _ in self.window_cache().values())
        return max(1, per * torch.finfo(kv_dtype).bits // 8)


class KikuraxAttention(nn.Module):
    """softmax attention with a zero-score sink; ``v_first``: the cache layer whose values this layer blends in (None for
    the first such layer, and for layers that do not blend)"""

    def __init__(self, width: int, m: dict, layer_id: int, eps: float, v_first: Optional[int], dtype=None):
        super().__init__()
        H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        self.heads, self.kv_heads, self.dim, self.vdim, self.eps, self.v_first = H, G, D, Dv, eps, v_first
        self.qkv = nn.Parameter(torch.empty(H * D + G * D + G * Dv, width, dtype=dtype), requires_grad=False)
        f32 = dict(dtype=torch.float32)
        self.q_bias = nn.Parameter(torch.zeros(H * D, **f32), requires_grad=False)
        self.k_bias = nn.Parameter(torch.zeros(G * D, **f32), requires_grad=False)
        self.v_bias = nn.Parameter(torch.zeros(G * Dv, **f32), requires_grad=False)
        self.o = nn.Parameter(torch.empty(width, H * Dv, dtype=dtype), requires_grad=False)
        rot = m.get("rot")
        self.rotary = None
        if rot and int(rot["dims"]) > 0:
            if int(rot["dims"]) > D:
                raise ValueError("rot.dims exceeds the head size")
            self.rotary = HalfAngleRotary(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        # the sink's score is zero by design: the layer's `sinks` stay the zeros they are made with
        self.attn = PooledWindowAttention(H, G, D, Dv, float(m["scale"]), layer_id, sinks=True, norm_values=False, qk_norm=True,
                                          head_scale=True, softcap=float(m.get("softcap") or 0.0), v_mix=v_first is not None)

    def forward(self, positions, h: torch.Tensor, forward_batch: ForwardBatch) -> torch.Tensor:
        nq, nk = self.heads * self.dim, self.kv_heads * self.dim
        qkv = _native.linear(h, self.qkv)
        q = qkv[:, :nq]
        self.attn.store(q, qkv[:, nq:nq + nk], qkv[:, nq + nk:], self.rotary, positions, self.eps, forward_batch,
                        biases=(self.q_bias.data, self.k_bias.data, self.v_bias.data), v_first_cache=self.v_first)
        return _native.linear(self.attn(q, forward_batch), self.o)


class KikuraxParallel(nn.Module):
    """Two mixers on the same input: sigmoid-weighted attention with an output gate (left) and a channel-gated delta rule
    (right).  ONE product makes the rows [q | k | v | gate (left) | q | k | v | b | a1 | g1 (right)]; the two results go back
    separately (the layer norms each over the model width and averages them)."""

    def __init__(self, width: int, m: dict, layer_id: int, eps: float, decay_rank: int, gate_rank: int, dtype=None):
        super().__init__()
        a, b = m["left"], m["right"]
        H, G, D, Dv = (int(a[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        self.heads, self.kv_heads, self.dim, self.vdim, self.eps = H, G, D, Dv, eps
        self.left_rows = H * D + G * D + G * Dv + H * Dv
        self.right = GatedDeltaMixer(width, int(b["heads"]), int(b["kv_heads"]), int(b["dim"]), int(b["vdim"]), int(b["conv"]),
                                     decay_rank, gate_rank, eps, layer_id=layer_id, own_input=False, dtype=dtype)
        self.in_proj = nn.Parameter(torch.empty(self.left_rows + self.right.in_rows, width, dtype=dtype), requires_grad=False)
        self.left_o = nn.Parameter(torch.empty(width, H * Dv, dtype=dtype), requires_grad=False)
        self.branch_weight = nn.Parameter(torch.ones(2, width, dtype=torch.float32), requires_grad=False)
        qt = a.get("q_temp")
        self.attn = PooledWindowAttention(H, G, D, Dv, float(a["scale"]), layer_id, norm_values=False, qk_norm=True,
                                          q_temp=(float(qt["coef"]), int(qt["every"])) if qt else None, weights="sigmoid")

    def forward(self, positions, h: torch.Tensor, forward_batch: ForwardBatch):
        nq, nk, nv = self.heads * self.dim, self.kv_heads * self.dim, self.kv_heads * self.vdim
        a = _native.linear(h, self.in_proj)
        q = a[:, :nq]
        self.attn.store(q, a[:, nq:nq + nk], a[:, nq + nk:nq + nk + nv], None, positions, self.eps, forward_batch)
        left = _native.linear(self.attn(q, forward_batch, gate=a[:, nq + nk + nv:self.left_rows]), self.left_o)
        right = self.right.scan(a[:, self.left_rows:], forward_batch)
        return left, right


class KikuraxLayer(nn.Module):
    def __init__(self, config: KikuraxConfig, layer_id: int, dtype=None):
        super().__init__()
        spec, W, eps = config.layers[layer_id], config.hidden_size, config.rms_norm_eps
        self.kind = spec["type"]
        m = spec["mixer"]
        self.norm1 = GroupRMSNorm(W, config.norm_groups, eps)
        if self.kind == "attention":
            first = config.v_first_layer
            self.mix = KikuraxAttention(W, m, layer_id, eps, first if (m.get("v_mix") and first != layer_id) else None, dtype)
        elif self.kind == "mamba2":
            self.mix = Mamba2Mixer(W, int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]),
                                   int(m["norm_groups"]), layer_id, eps, dtype)
        else:
            self.mix = KikuraxParallel(W, m, layer_id, eps, config.rank(layer_id, "a1"), config.rank(layer_id, "g1"), dtype)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            self.norm2 = GroupRMSNorm(W, config.norm_groups, eps)
            r = mlp["router"]
            self.mlp = ChosenSoftmaxMoE(W, int(r["experts"]), int(r["top"]), int(mlp["expert"]["ff"]),
                                        float(mlp["expert"]["limit"]), dtype)

    def forward(self, positions, x: torch.Tensor, h: torch.Tensor, forward_batch: ForwardBatch, dtype,
                next_norm: Optional[GroupRMSNorm]) -> Optional[torch.Tensor]:
        """x: the fp32 stream, updated in place; h = GN(x) * norm1 in the projections' dtype.  Returns the next layer's (or
        the model's last) norm of the stream as this layer leaves it; without ``next_norm`` only the stream moves on."""
        if self.kind == "parallel":
            y, bw = self.mix(positions, h, forward_batch), (self.mix.branch_weight.data[0], self.mix.branch_weight.data[1])
        else:
            y, bw = (self.mix(positions, h, forward_batch) if self.kind == "attention" else self.mix(h, forward_batch)), None
        if self.mlp is not None:
            y, bw = self.mlp(self.norm2(x, dtype, y, bw)), None
        if next_norm is None:
            add_join(x, y, bw, 1, self.norm1.variance_epsilon, dtype)
            return None
        return next_norm(x, dtype, y, bw)


class KikuraxForCausalLM(nn.Module):
    # parameters keep the dtypes they are declared with (fp32 norms, biases, decays, router) whatever the runner's dtype
    keeps_parameter_dtypes = True
    supports_tensor_parallel = False
    # Largest decode step that is captured into a HIP graph (the step has no host synchronisation and no data-dependent
    # shape); larger steps run eagerly.
    max_graph_batch = 64
    # sources of the HIP library this model's path needs beyond the core (scratchpad_amd.build.build_native(only=...))
    NATIVE_SOURCES = ["stream_norm.hip", "window_attention.hip", "ssm.hip", "gated_delta.hip", "moe.hip"]

    def __init__(self, config: KikuraxConfig, dtype=None):
        super().__init__()
        self.config = config
        self.dtype = dtype or torch.get_default_dtype()
        self.layers = nn.ModuleList([KikuraxLayer(config, i, dtype) for i in range(config.num_hidden_layers)])
        self.norm = GroupRMSNorm(config.hidden_size, config.norm_groups, config.rms_norm_eps)
        self.lm_head = ParallelLMHead(config.vocab_size, config.hidden_size, dtype)      # also the embedding table
        self.logits_processor = LogitsProcessor(config)
        self.capture_layers: Optional[list] = None     # set to a list to collect the stream after every layer

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch: ForwardBatch, input_embeds=None) -> LogitsProcessorOutput:
        table = self.lm_head.weight
        dtype = table.dtype
        x = _native.embed_scale(table.data, input_ids, self.config.embedding_scale)
        n = len(self.layers)
        h = (self.layers[0].norm1 if n else self.norm)(x, dtype)
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.norm
            if self.capture_layers is None:
                h = layer(positions, x, h, forward_batch, dtype, nxt)
            else:
                layer(positions, x, h, forward_batch, dtype, None)
                self.capture_layers.append(x.clone())
                h = nxt(x, dtype)
        return self.logits_processor(input_ids, h, self.lm_head, forward_batch)

    # ---- weights --------------------------------------------------------------------------------------------------
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> None:
        """Checkpoint names of the design ('embed', 'l<i>.norm1|norm2', 'l<i>.mix.*', 'l<i>.mlp.e<j>.gate|up|down',
        'l<i>.mlp.router' with '.b', 'final.norm') -> this module's (partly merged) parameters."""
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
            M = f"{p}.mix"
            if layer.kind == "attention":
                put(mix.qkv, torch.cat([take(f"{M}.q"), take(f"{M}.k"), take(f"{M}.v")], 0))
                put(mix.q_bias, take(f"{M}.q.b"))
                put(mix.k_bias, take(f"{M}.k.b"))
                put(mix.v_bias, take(f"{M}.v.b"))
                put(mix.attn.head_scale, take(f"{M}.temp"))
                if f"{M}.vmix" in w:
                    lam = take(f"{M}.vmix")
                    if mix.attn.v_mix is not None:
                        put(mix.attn.v_mix, lam.reshape(1))
                put(mix.o, take(f"{M}.o"))
            elif layer.kind == "mamba2":
                full = take(f"{M}.in")
                put(mix.in_proj, full[:mix.in_proj.shape[0]])
                put(mix.dt_proj, full[mix.in_proj.shape[0]:])
                put(mix.conv, take(f"{M}.conv"))
                put(mix.conv_bias, take(f"{M}.conv.b"))
                for name in ("dt_bias", "A_log", "D", "norm", "o"):
                    put(getattr(mix, name), take(f"{M}.{name}"))
            else:
                L, R, right = f"{M}.left", f"{M}.right", mix.right
                put(mix.in_proj, torch.cat([take(f"{L}.{s}") for s in ("q", "k", "v", "g")] +
                                           [take(f"{R}.{s}") for s in ("q", "k", "v", "b", "a1", "g1")], 0))
                put(mix.attn.head_bias, take(f"{L}.pb"))
                put(mix.left_o, take(f"{L}.o"))
                put(right.conv, torch.cat([take(f"{R}.q.conv"), take(f"{R}.k.conv"), take(f"{R}.v.conv")], 0))
                put(right.a2t, take(f"{R}.a2").t().contiguous())
                put(right.g2t, take(f"{R}.g2").t().contiguous())
                for name in ("dt_bias", "A_log", "norm", "o"):
                    put(getattr(right, name), take(f"{R}.{name}"))
                put(mix.branch_weight, torch.stack([take(f"{L}.out"), take(f"{R}.out")]))
            if layer.mlp is None:
                continue
            put(layer.norm2.weight, take(f"{p}.norm2"))
            ex = layer.mlp.experts
            put(ex.gate_up, torch.stack([torch.cat([take(f"{p}.mlp.e{e}.gate"), take(f"{p}.mlp.e{e}.up")], 0)
                                         for e in range(ex.experts)]))
            put(ex.down, torch.stack([take(f"{p}.mlp.e{e}.down") for e in range(ex.experts)]))
            put(layer.mlp.router.weight, take(f"{p}.mlp.router"))
            put(layer.mlp.router.bias, take(f"{p}.mlp.router.b"))
        extra = set(w) - used
        if extra:
            import warnings
            warnings.warn(f"checkpoint tensors no part of the configured model reads: {sorted(extra)[:8]}")

    def init_random(self, generator: torch.Generator) -> None:
        """random weights of a plausible scale (benchmarks and tests of the host path: no checkpoint)"""
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("weight", "norm", "branch_weight", "head_scale", "D") and "lm_head" not in name and "router" not in name:
                p.data.fill_(1.0)
            elif leaf in ("A_log", "dt_bias"):
                p.data.normal_(-1.0, 0.5, generator=generator)
            elif leaf == "sinks":
                p.data.zero_()
            elif leaf == "v_mix":
                p.data.fill_(0.25)
            elif leaf == "conv":
                p.data.normal_(0.0, 0.5, generator=generator)
            elif p.dim() >= 2:
                p.data.normal_(0.0, 1.0 / (p.shape[-1] ** 0.5), generator=generator)
            else:
                p.data.normal_(0.0, 0.1, generator=generator)
