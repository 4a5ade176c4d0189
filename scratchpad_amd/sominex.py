"""Sominex: a decoder-only design of parallel layers over an fp32 residual stream,
    h = rms(x) * w;   x <- x + mixer(shift(h)) + ff(h),   shift(h)[t] = h[t] + (h[t-1] - h[t]) * mu,
whose mixer is, layer by layer, grouped-query attention over a sliding window with pooled blocks behind it (rotate-half
rotary on part of each head, blended frequencies, values normed per head), a Mamba-2 state-space mixer, or an mLSTM
matrix memory; the feed-forward is a clamped gated unit or a softmax-routed mixture of silu experts with a shared expert.
The embedding is scaled by a constant; a weighted norm and the head end the model.

Everything that differs between models of the design comes from config.json (``SominexConfig``) or a tensor's shape; the
model is assembled from the framework's mechanisms - ShiftedRMSNorm / HalfAngleRotary / GluFF (layers.py),
PooledWindowAttention + SequenceBackend (attention.py), Mamba2Mixer / MLSTMMixer (recurrent.py), SoftmaxMoE (moe.py),
WindowKVPool + RecurrentStatePool (pool.py) - and served by the ModelRunner like the other model classes."""
from typing import Dict, Iterable, List, Optional, Tuple

import torch
from torch import nn

from . import _native
from .attention import PooledWindowAttention
from .forward_info import ForwardBatch
from .layers import GluFF, HalfAngleRotary, ShiftedRMSNorm
from .llama import LogitsProcessor, LogitsProcessorOutput, ParallelLMHead
from .moe import SoftmaxMoE
from .recurrent import Mamba2Mixer, MLSTMMixer

MIXERS = ("attention", "mamba2", "mlstm")


class SominexConfig:
    """config.json of the design, plus what the runner asks of any model configuration (vocab_size, context_len,
    num_hidden_layers, is_encoder_decoder) and what it builds the pools from."""
    architecture = "Sominex"
    is_encoder_decoder = False
    vision_config = None

    def __init__(self, raw: dict, context_len: int = 8192, tensor_shapes: Optional[Dict[str, Tuple[int, ...]]] = None):
        self.raw = raw
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.layers: List[dict] = raw["layers"]
        self.num_hidden_layers = len(self.layers)
        self.rms_norm_eps = float(raw["norm"]["eps"])
        self.embedding_scale = float((raw.get("embedding") or {}).get("scale", 1.0))
        self.context_len = context_len
        self.tie_word_embeddings = False
        self.tensor_shapes = tensor_shapes or {}
        for layer in self.layers:
            if layer["type"] not in MIXERS:
                raise ValueError(f"unknown layer type {layer['type']!r}")
            if layer.get("mlp") is not None and layer["mlp"]["kind"] not in ("dense", "moe"):
                raise ValueError(f"unknown feed-forward kind {layer['mlp']['kind']!r}")

    # ---- what the runner builds its pools from
    def window_cache(self):
        """{layer id: (kv_heads, dim, vdim, pooled)} of the layers that keep a key/value row per token"""
        out = {}
        for i, l in enumerate(self.layers):
            if l["type"] == "attention":
                m, mask = l["mixer"], l["mixer"].get("mask") or {}
                out[i] = (int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), bool(mask.get("size") and mask.get("pool")))
        return out

    def shift_layers(self):
        return list(range(self.num_hidden_layers))          # every layer's mixer reads the shifted input

    def named_state(self):
        """{layer id: {name: shape}} of the fp32 state the recurrent layers carry per request"""
        out = {}
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            if l["type"] == "mamba2":
                out[i] = Mamba2Mixer.state_shapes(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]))
            elif l["type"] == "mlstm":
                out[i] = MLSTMMixer.state_shapes(int(m["heads"]), int(m["dim"]), int(m["vdim"]))
        return out

    def cache_bytes_per_token(self, kv_dtype: torch.dtype) -> int:
        per = sum(g * (d + dv) * (2 if p else 1) for g, d, dv, p in self.window_cache().values())
        return max(1, per * torch.finfo(kv_dtype).bits // 8)


class SominexAttention(nn.Module):
    def __init__(self, width: int, m: dict, layer_id: int, eps: float, dtype=None):
        super().__init__()
        H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        self.heads, self.kv_heads, self.dim, self.vdim, self.eps = H, G, D, Dv, eps
        self.qkv = nn.Parameter(torch.empty(H * D + G * D + G * Dv, width, dtype=dtype), requires_grad=False)
        self.o = nn.Parameter(torch.empty(width, H * Dv, dtype=dtype), requires_grad=False)
        rot = m.get("rot")
        self.rotary = None
        if rot and int(rot["dims"]) > 0:
            if int(rot["dims"]) > D:
                raise ValueError("rot.dims exceeds the head size")
            self.rotary = HalfAngleRotary(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        mask = m.get("mask") or {}
        self.attn = PooledWindowAttention(H, G, D, Dv, float(m["scale"]), layer_id, mask.get("size"), mask.get("pool"))

    def forward(self, positions, h: torch.Tensor, forward_batch: ForwardBatch) -> torch.Tensor:
        nq, nk = self.heads * self.dim, self.kv_heads * self.dim
        qkv = _native.linear(h, self.qkv)
        q = qkv[:, :nq]
        self.attn.store(q, qkv[:, nq:nq + nk], qkv[:, nq + nk:], self.rotary, positions, self.eps, forward_batch)
        return _native.linear(self.attn(q, forward_batch), self.o)


class SominexMoE(nn.Module):
    """routed experts + the shared expert (both read h; the layer adds both to the stream)"""

    def __init__(self, width: int, mlp: dict, dtype=None):
        super().__init__()
        r = mlp["router"]
        self.routed = SoftmaxMoE(width, int(r["experts"]), int(r["top"]), int(mlp["expert"]["ff"]), float(r.get("scale", 1.0)), dtype)
        self.shared = GluFF(width, int(mlp["shared"]["ff"]), "silu", dtype=dtype) if mlp.get("shared") else None


class SominexLayer(nn.Module):
    def __init__(self, config: SominexConfig, layer_id: int, dtype=None):
        super().__init__()
        spec, W, eps = config.layers[layer_id], config.hidden_size, config.rms_norm_eps
        self.kind = spec["type"]
        m = spec["mixer"]
        self.norm1 = ShiftedRMSNorm(W, eps, shift=True, layer_id=layer_id)
        if self.kind == "attention":
            self.mix = SominexAttention(W, m, layer_id, eps, dtype)
        elif self.kind == "mamba2":
            self.mix = Mamba2Mixer(W, int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]),
                                   int(m["norm_groups"]), layer_id, eps, dtype)
        else:
            self.mix = MLSTMMixer(W, int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"]), layer_id, eps, dtype)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            self.mlp = GluFF(W, int(mlp["ff"]), "clamped", float(mlp["limit"]), dtype=dtype) if mlp["kind"] == "dense" \
                else SominexMoE(W, mlp, dtype)

    def forward(self, positions, x: torch.Tensor, forward_batch: ForwardBatch, dtype: torch.dtype) -> None:
        """x: the fp32 stream, updated in place"""
        h, hs = self.norm1(x, dtype, forward_batch, want_h=self.mlp is not None)
        y = self.mix(positions, hs, forward_batch) if self.kind == "attention" else self.mix(hs, forward_batch)
        if self.mlp is None:
            _native.stream_add(x, y)
        elif isinstance(self.mlp, GluFF):
            _native.stream_add(x, y, self.mlp(h))
        else:
            _native.stream_add(x, y, self.mlp.routed(h), None if self.mlp.shared is None else self.mlp.shared(h))


class SominexForCausalLM(nn.Module):
    # parameters keep the dtypes they are declared with (fp32 norms, gates, decays, router) whatever the runner's dtype
    keeps_parameter_dtypes = True
    supports_tensor_parallel = False
    # Largest decode step that is captured into a HIP graph.  Up to 16 rows the 16-bit projections of a step run on the
    # framework's own weight-streaming kernel, above that on the library's (as Llama's captured steps do); up to 64 rows
    # the fp32 gate projections stay on the own kernel.  Replays of 40-row steps are tested against eager steps; larger
    # steps run eagerly.
    max_graph_batch = 64
    # sources of the HIP library this model's path needs beyond the core (scratchpad_amd.build.build_native(only=...))
    NATIVE_SOURCES = ["stream_norm.hip", "window_attention.hip", "ssm.hip", "mlstm.hip", "moe.hip"]

    def __init__(self, config: SominexConfig, dtype=None):
        super().__init__()
        self.config = config
        self.dtype = dtype or torch.get_default_dtype()
        self.embed = nn.Parameter(torch.empty(config.vocab_size, config.hidden_size, dtype=dtype), requires_grad=False)
        self.layers = nn.ModuleList([SominexLayer(config, i, dtype) for i in range(config.num_hidden_layers)])
        self.norm = ShiftedRMSNorm(config.hidden_size, config.rms_norm_eps, shift=False)
        self.lm_head = ParallelLMHead(config.vocab_size, config.hidden_size, dtype)
        self.logits_processor = LogitsProcessor(config)
        self.capture_layers: Optional[list] = None     # set to a list to collect the stream after every layer

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch: ForwardBatch, input_embeds=None) -> LogitsProcessorOutput:
        x = _native.embed_scale(self.embed.data, input_ids, self.config.embedding_scale)
        dtype = self.lm_head.weight.dtype
        for layer in self.layers:
            layer(positions, x, forward_batch, dtype)
            if self.capture_layers is not None:
                self.capture_layers.append(x.clone())
        return self.logits_processor(input_ids, self.norm(x, dtype), self.lm_head, forward_batch)

    # ---- weights --------------------------------------------------------------------------------------------------
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> None:
        """Checkpoint names of the design ('embed', 'l<i>.norm1', 'l<i>.shift', 'l<i>.mix.*', 'l<i>.mlp.*', 'final.norm',
        'head') -> this module's (partly merged) parameters."""
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

        def put_glu(ff: GluFF, p: str):
            put(ff.gate_up, torch.cat([take(f"{p}.gate"), take(f"{p}.up")], 0))
            put(ff.down, take(f"{p}.down"))

        put(self.embed, take("embed"))
        put(self.norm.weight, take("final.norm"))
        put(self.lm_head.weight, self.lm_head.shard_from_full(take("head")))
        for i, layer in enumerate(self.layers):
            p, mix = f"l{i}", layer.mix
            put(layer.norm1.weight, take(f"{p}.norm1"))
            put(layer.norm1.mu, take(f"{p}.shift"))
            if layer.kind == "attention":
                put(mix.qkv, torch.cat([take(f"{p}.mix.q"), take(f"{p}.mix.k"), take(f"{p}.mix.v")], 0))
                put(mix.o, take(f"{p}.mix.o"))
            elif layer.kind == "mamba2":
                full = take(f"{p}.mix.in")
                put(mix.in_proj, full[:mix.in_proj.shape[0]])
                put(mix.dt_proj, full[mix.in_proj.shape[0]:])
                put(mix.conv, take(f"{p}.mix.conv"))
                put(mix.conv_bias, take(f"{p}.mix.conv.b"))
                for name in ("dt_bias", "A_log", "D", "norm", "o"):
                    put(getattr(mix, name), take(f"{p}.mix.{name}"))
            else:
                put(mix.qkvg, torch.cat([take(f"{p}.mix.{s}") for s in "qkvg"], 0))
                put(mix.gates, torch.cat([take(f"{p}.mix.i"), take(f"{p}.mix.f")], 0))
                put(mix.gates_bias, torch.cat([take(f"{p}.mix.i.b"), take(f"{p}.mix.f.b")], 0))
                put(mix.norm, take(f"{p}.mix.norm"))
                put(mix.o, take(f"{p}.mix.o"))
            if layer.mlp is None:
                continue
            if isinstance(layer.mlp, GluFF):
                put_glu(layer.mlp, f"{p}.mlp")
            else:
                ex = layer.mlp.routed.experts
                put(ex.gate_up, torch.stack([torch.cat([take(f"{p}.mlp.e{e}.gate"), take(f"{p}.mlp.e{e}.up")], 0)
                                             for e in range(ex.experts)]))
                put(ex.down, torch.stack([take(f"{p}.mlp.e{e}.down") for e in range(ex.experts)]))
                put(layer.mlp.routed.router.weight, take(f"{p}.mlp.router"))
                if layer.mlp.shared is not None:
                    put_glu(layer.mlp.shared, f"{p}.mlp.shared")
        extra = set(w) - used
        if extra:
            import warnings
            warnings.warn(f"checkpoint tensors no part of the configured model reads: {sorted(extra)[:8]}")

    def init_random(self, generator: torch.Generator) -> None:
        """random weights of a plausible scale (benchmarks and tests of the host path: no checkpoint)"""
        for name, p in self.named_parameters():
            if name.endswith("norm.weight") or name.endswith(".norm") or name.endswith("norm1.weight"):
                p.data.fill_(1.0)
            elif name.endswith(".mu"):
                p.data.uniform_(0.0, 1.0, generator=generator)
            elif name.endswith("A_log") or name.endswith("dt_bias"):
                p.data.normal_(-1.0, 0.5, generator=generator)
            elif name.endswith(".D"):
                p.data.fill_(1.0)
            elif name.endswith("gates_bias"):
                p.data.normal_(1.0, 1.0, generator=generator)
            elif name.endswith(".conv"):
                p.data.normal_(0.0, 0.5, generator=generator)
            elif p.dim() >= 2:
                p.data.normal_(0.0, 1.0 / (p.shape[-1] ** 0.5), generator=generator)
            else:
                p.data.normal_(0.0, 0.1, generator=generator)
