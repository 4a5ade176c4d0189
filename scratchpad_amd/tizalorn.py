"""Tizalorn: a decoder-only design that mixes recurrent (matrix-state) layers with latent-attention layers, dense
PolyNorm and mixture-of-experts feed-forwards, a hashed bigram embedding, and an fp32 residual stream that takes every
sublayer's output through a single-gain RMS norm (x <- x + g * f(x) / rms(f(x)); the sublayers read x itself).

Everything that differs between models of the design comes from its config.json (``TizalornConfig.from_dict``) or from
a tensor's shape; the model is assembled from the framework's mechanisms - ScalarRMSNorm / PolyNorm / AngleRotary
(layers.py), WKVMixer (recurrent.py), LatentAttention + SequenceBackend (attention.py), SparseMoE (moe.py),
LatentTokenToKVPool + RecurrentStatePool (pool.py) - and served by the ModelRunner like the other model classes."""
import json
import os
from typing import Dict, Iterable, List, Optional, Tuple

import torch
from torch import nn

from . import _native
from .attention import LatentAttention
from .forward_info import ForwardBatch
from .layers import AngleRotary, PolyNorm, ScalarRMSNorm
from .llama import LogitsProcessor, LogitsProcessorOutput, ParallelLMHead
from .moe import SparseMoE
from .recurrent import WKVMixer


class TizalornConfig:
    """config.json of the design, plus what the runner asks of any model configuration (vocab_size, context_len,
    num_hidden_layers, is_encoder_decoder).  Sizes a tensor's shape gives (the decay projection's rank) are read from
    the checkpoint's shapes when there is one (``tensor_shapes``), else from ``decay_rank`` in the layer's mixer."""
    architecture = "Tizalorn"
    is_encoder_decoder = False
    vision_config = None

    def __init__(self, raw: dict, context_len: int = 8192, tensor_shapes: Optional[Dict[str, Tuple[int, ...]]] = None):
        self.raw = raw
        self.vocab_size = int(raw["vocab"])
        self.hidden_size = int(raw["width"])
        self.layers: List[dict] = raw["layers"]
        self.num_hidden_layers = len(self.layers)
        self.rms_norm_eps = float(raw["norm"]["eps"])
        self.bigram = raw["embedding"]["bigram"]
        self.context_len = context_len
        self.tie_word_embeddings = False
        self.tensor_shapes = tensor_shapes or {}
        for layer in self.layers:
            if layer["type"] not in ("wkv", "latent_attention"):
                raise ValueError(f"unknown layer type {layer['type']!r}")
            if layer.get("mlp") is not None and layer["mlp"]["kind"] not in ("dense", "moe"):
                raise ValueError(f"unknown feed-forward kind {layer['mlp']['kind']!r}")
    @classmethod
    def from_dict(cls, raw: dict, **kw) -> "TizalornConfig":
        return cls(raw, **kw)

    def decay_rank(self, layer_id: int) -> int:
        shape = self.tensor_shapes.get(f"l{layer_id}.mix.w1")
        return int(shape[0]) if shape else int(self.layers[layer_id]["mixer"].get("decay_rank", 16))

    # ---- what the runner builds its pools from
    def latent_cache(self):
        """{layer id: (rank, rot_dim)} of the layers that keep a latent key/value row per token"""
        return {i: (int(l["mixer"]["kv_rank"]), int(l["mixer"]["rot_dim"])) for i, l in enumerate(self.layers)
                if l["type"] == "latent_attention"}

    def recurrent_layers(self):
        """{layer id: (heads, dim)} of the layers with a matrix state"""
        return {i: (int(l["mixer"]["heads"]), int(l["mixer"]["dim"])) for i, l in enumerate(self.layers)
                if l["type"] == "wkv"}

    def cache_bytes_per_token(self, kv_dtype: torch.dtype) -> int:
        return max(1, sum(r + d for r, d in self.latent_cache().values()) * torch.finfo(kv_dtype).bits // 8)


class BigramEmbedding(nn.Module):
    """x = ScalarRMS(embed[token] + bigram[(previous * mul_prev + token * mul_cur) mod buckets]); a sequence's first token
    takes the bigram table's last row.  The previous token of a step's first row is the request's state."""

    def __init__(self, vocab: int, width: int, buckets: int, mul_prev: int, mul_cur: int, eps: float, dtype=None):
        super().__init__()
        self.buckets, self.mul_prev, self.mul_cur = buckets, mul_prev, mul_cur
        self.weight = nn.Parameter(torch.empty(vocab, width, dtype=dtype), requires_grad=False)
        self.bigram = nn.Parameter(torch.empty(buckets + 1, width, dtype=dtype), requires_grad=False)
        self.norm = ScalarRMSNorm(eps)

    def forward(self, input_ids: torch.Tensor, forward_batch: ForwardBatch):
        seq, states = forward_batch.attn_backend.seq, forward_batch.state_pool
        rows = _native.bigram_rows(input_ids, states.last_token, seq, self.buckets, self.mul_prev, self.mul_cur)
        _native.save_last_token(states.last_token, input_ids, seq)
        return _native.embed_bigram_norm(self.weight.data, self.bigram.data, input_ids, rows, self.norm.weight.data,
                                         self.norm.variance_epsilon)


class TizalornLatentAttention(nn.Module):
    def __init__(self, width: int, m: dict, layer_id: int, eps: float, dtype=None):
        super().__init__()
        H, D, R, Dv, C, Q = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
        self.heads, self.dim, self.rot_dim, self.vdim, self.rank, self.eps = H, D, R, Dv, C, eps
        f32 = dict(dtype=torch.float32)
        self.dq = nn.Parameter(torch.empty(Q, width, dtype=dtype), requires_grad=False)
        self.dq_norm = nn.Parameter(torch.ones(Q, dtype=dtype), requires_grad=False)
        self.uq = nn.Parameter(torch.empty(H * (D + R), Q, dtype=dtype), requires_grad=False)
        # the latent down-projection and the per-head output gate read the same input: one product
        self.dkv_g = nn.Parameter(torch.empty(C + R + H, width, dtype=dtype), requires_grad=False)
        self.dkv_norm = nn.Parameter(torch.ones(C, **f32), requires_grad=False)
        self.uk = nn.Parameter(torch.empty(H, D, C, dtype=dtype), requires_grad=False)       # per head [dim, rank]
        self.uv_t = nn.Parameter(torch.empty(H, C, Dv, dtype=dtype), requires_grad=False)    # per head [rank, vdim]
        self.o = nn.Parameter(torch.empty(width, H * Dv, dtype=dtype), requires_grad=False)
        rot = m["rot"]
        if int(rot["dims"]) > R:
            raise ValueError("rot.dims exceeds rot_dim")
        self.rotary = AngleRotary(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        self.attn = LatentAttention(H, C, R, float(m["scale"]), layer_id)

    def forward(self, positions, h: torch.Tensor, forward_batch: ForwardBatch) -> torch.Tensor:
        H, D, R, C = self.heads, self.dim, self.rot_dim, self.rank
        T = h.shape[0]
        cq = _native.rmsnorm(_native.linear(h, self.dq), self.dq_norm.data, self.eps)
        q = _native.linear(cq, self.uq).view(T, H, D + R)
        dkv_g = _native.linear(h, self.dkv_g)
        pool = forward_batch.token_to_kv_pool.get_key_buffer(self.attn.layer_id)
        _native.latent_kv_store(pool, dkv_g[:, :C + R], self.dkv_norm.data, positions, self.rotary.freq,
                                self.rotary.magnitude, forward_batch.out_cache_loc, C, self.eps)
        self.rotary(positions, q, offset=D)
        q_lat = torch.bmm(q[:, :, :D].transpose(0, 1), self.uk)                    # [H, T, C]
        o_lat = self.attn(q_lat, q[:, :, D:], forward_batch)                       # [H, T, C]
        o = torch.bmm(o_lat, self.uv_t)                                            # [H, T, Dv]
        return _native.linear(_native.gate_heads(o, dkv_g[:, C + R:]), self.o)


class DenseFF(nn.Module):
    def __init__(self, width: int, ff: int, eps: float, dtype=None):
        super().__init__()
        self.up = nn.Parameter(torch.empty(ff, width, dtype=dtype), requires_grad=False)
        self.down = nn.Parameter(torch.empty(width, ff, dtype=dtype), requires_grad=False)
        self.act = PolyNorm(eps)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return _native.linear(self.act(_native.linear(h, self.up)), self.down)


class TizalornLayer(nn.Module):
    def __init__(self, config: TizalornConfig, layer_id: int, dtype=None):
        super().__init__()
        spec, W, eps = config.layers[layer_id], config.hidden_size, config.rms_norm_eps
        self.kind = spec["type"]
        m = spec["mixer"]
        if self.kind == "wkv":
            self.mix = WKVMixer(W, int(m["heads"]), int(m["dim"]), config.decay_rank(layer_id), layer_id, eps, dtype)
        else:
            self.mix = TizalornLatentAttention(W, m, layer_id, eps, dtype)
        self.norm1 = ScalarRMSNorm(eps)
        mlp = spec.get("mlp")
        self.mlp, self.norm2 = None, None
        if mlp is not None:
            if mlp["kind"] == "dense":
                self.mlp = DenseFF(W, int(mlp["ff"]), eps, dtype)
            else:
                r = mlp["router"]
                groups = r.get("groups") or {"count": 1, "keep": 1}
                self.mlp = SparseMoE(W, int(r["experts"]), int(r["top"]), int(mlp["expert"]["ff"]),
                                     float(mlp["expert"]["limit"]), int(groups["count"]), int(groups["keep"]), dtype)
            self.norm2 = ScalarRMSNorm(eps)

    def forward(self, positions, x: torch.Tensor, lo: torch.Tensor, forward_batch: ForwardBatch, last: bool):
        """x: the fp32 stream (updated in place); lo: x in the projections' dtype; returns the new lo"""
        y = self.mix(x, forward_batch) if self.kind == "wkv" else self.mix(positions, lo, forward_batch)
        lo = self.norm1.add_into(x, y, want_lo=self.mlp is not None or not last)
        if self.mlp is not None:
            lo = self.norm2.add_into(x, self.mlp(lo), want_lo=not last)
        return lo


class TizalornForCausalLM(nn.Module):
    # parameters keep the dtypes they are declared with (fp32 gains, decays, router) whatever the runner's dtype
    keeps_parameter_dtypes = True
    supports_tensor_parallel = False
    # Largest decode step that is captured into a HIP graph.  Up to 16 rows the 16-bit projections of a step run on the
    # framework's own weight-streaming kernel; above that they are library products, whose captured form (they may record
    # workspace clears) has not been replay-tested for this design's shapes, so larger steps run eagerly.
    max_graph_batch = 16
    # sources of the HIP library this model's path needs beyond the core (scratchpad_amd.build.build_native(only=...))
    NATIVE_SOURCES = ["scalar_norm.hip", "wkv.hip", "latent_attention.hip", "moe.hip"]

    def __init__(self, config: TizalornConfig, dtype=None):
        super().__init__()
        self.config = config
        b = config.bigram
        self.embed = BigramEmbedding(config.vocab_size, config.hidden_size, int(b["buckets"]), int(b["mul_prev"]),
                                     int(b["mul_cur"]), config.rms_norm_eps, dtype)
        self.layers = nn.ModuleList([TizalornLayer(config, i, dtype) for i in range(config.num_hidden_layers)])
        self.norm = ScalarRMSNorm(config.rms_norm_eps)
        self.lm_head = ParallelLMHead(config.vocab_size, config.hidden_size, dtype)
        self.logits_processor = LogitsProcessor(config)
        self.capture_layers: Optional[list] = None     # set to a list to collect the stream after every layer

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch: ForwardBatch, input_embeds=None) -> LogitsProcessorOutput:
        x, lo = self.embed(input_ids, forward_batch)
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            lo = layer(positions, x, lo, forward_batch, last=i == n - 1)
            if self.capture_layers is not None:
                self.capture_layers.append(x.clone())
        hidden = self.norm(x, self.lm_head.weight.dtype)
        return self.logits_processor(input_ids, hidden, self.lm_head, forward_batch)

    # ---- weights --------------------------------------------------------------------------------------------------
    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> None:
        """Checkpoint names of the design ('embed', 'bigram', 'l<i>.mix.*', 'l<i>.mlp.*', 'final.norm', 'head') -> this
        module's (partly merged, partly transposed) parameters."""
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

        put(self.embed.weight, take("embed"))
        put(self.embed.bigram, take("bigram"))
        put(self.embed.norm.weight, take("embed.norm"))
        put(self.norm.weight, take("final.norm"))
        put(self.lm_head.weight, self.lm_head.shard_from_full(take("head")))
        for i, layer in enumerate(self.layers):
            p, mix = f"l{i}", layer.mix
            put(layer.norm1.weight, take(f"{p}.norm1"))
            if layer.kind == "wkv":
                put(mix.mu, torch.stack([take(f"{p}.mix.mu.{s}") for s in WKVMixer.MIXES]))
                put(mix.rkvg, torch.stack([take(f"{p}.mix.{s}") for s in "rkvg"]))
                put(mix.w1, take(f"{p}.mix.w1"))
                put(mix.w2t, take(f"{p}.mix.w2").t())
                for name in ("w0", "u", "norm", "o"):
                    put(getattr(mix, name), take(f"{p}.mix.{name}"))
            else:
                H, D, Dv, C = mix.heads, mix.dim, mix.vdim, mix.rank
                put(mix.dq, take(f"{p}.mix.dq"))
                put(mix.dq_norm, take(f"{p}.mix.dq.norm"))
                put(mix.uq, take(f"{p}.mix.uq"))
                put(mix.dkv_g, torch.cat([take(f"{p}.mix.dkv"), take(f"{p}.mix.g")], 0))
                put(mix.dkv_norm, take(f"{p}.mix.dkv.norm"))
                put(mix.uk, take(f"{p}.mix.uk").view(H, D, C))
                put(mix.uv_t, take(f"{p}.mix.uv").view(H, Dv, C).transpose(1, 2))
                put(mix.o, take(f"{p}.mix.o"))
            if layer.mlp is None:
                continue
            put(layer.norm2.weight, take(f"{p}.norm2"))
            if isinstance(layer.mlp, DenseFF):
                put(layer.mlp.up, take(f"{p}.mlp.up"))
                put(layer.mlp.down, take(f"{p}.mlp.down"))
                put(layer.mlp.act.weight, take(f"{p}.mlp.act"))
            else:
                ex = layer.mlp.experts
                put(ex.gate_up, torch.stack([torch.cat([take(f"{p}.mlp.e{e}.gate"), take(f"{p}.mlp.e{e}.up")], 0)
                                             for e in range(ex.experts)]))
                put(ex.down, torch.stack([take(f"{p}.mlp.e{e}.down") for e in range(ex.experts)]))
                put(layer.mlp.router.weight, take(f"{p}.mlp.router"))
                put(layer.mlp.router.correction, take(f"{p}.mlp.correction"))
        extra = set(w) - used
        if extra:       # (e.g. the second norm of a layer without a feed-forward: nothing reads it)
            import warnings
            warnings.warn(f"checkpoint tensors no part of the configured model reads: {sorted(extra)[:8]}")

    def init_random(self, generator: torch.Generator) -> None:
        """random weights of a plausible scale (benchmarks and tests of the host path: no checkpoint)"""
        for name, p in self.named_parameters():
            if name.endswith("norm.weight") or name.endswith(".norm") or name.endswith("dq_norm") or name.endswith("dkv_norm"):
                p.data.fill_(1.0)
            elif name.endswith(".mu"):
                p.data.uniform_(0.0, 1.0, generator=generator)
            elif name.endswith(".w0"):
                p.data.normal_(-1.0, 0.5, generator=generator)
            elif name.endswith("act.weight"):
                p.data.copy_(torch.tensor([0.9, 0.4, -0.3, 0.05]))
            elif name.endswith("correction"):
                p.data.normal_(0.0, 0.1, generator=generator)
            elif p.dim() >= 2:
                p.data.normal_(0.0, 1.0 / (p.shape[-1] ** 0.5), generator=generator)
            else:
                p.data.normal_(0.0, 0.5, generator=generator)


def read_config(model_dir: str, **kw) -> TizalornConfig:
    with open(os.path.join(model_dir, "config.json")) as f:
        return TizalornConfig(json.load(f), **kw)
