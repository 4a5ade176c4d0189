"""CPU oracle of the Tizalorn design: one plain, slow function per mechanism, written from the design's equations.

TEST INFRASTRUCTURE ONLY: nothing under scratchpad_amd/ imports this, and this imports nothing from there.  Every
function works on ONE sequence in float64 (or the dtype of what it is given) and keeps no cache: a whole sequence is
recomputed from its first token, which is what makes it a reference for caches, states, portions and batches.

Notation: T tokens, W model width, x the residual stream [T, W].
"""
import math
from typing import Dict, List, Optional

import torch


def scalar_rms(x: torch.Tensor, g, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * g with ONE gain g for all coordinates"""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * g


def weighted_rms(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


# ----------------------------------------------------------------------------------------------- embedding
def embed(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict) -> torch.Tensor:
    """token row + hashed (previous token, token) row; the first token of a sequence takes the table's last row"""
    b = cfg["embedding"]["bigram"]
    rows = []
    for i, t in enumerate(tokens):
        row = b["buckets"] if i == 0 else (tokens[i - 1] * b["mul_prev"] + t * b["mul_cur"]) % b["buckets"]
        rows.append(w["embed"][t] + w["bigram"][row])
    return scalar_rms(torch.stack(rows), w["embed.norm"], cfg["norm"]["eps"])


# ----------------------------------------------------------------------------------------------- wkv mixer
def wkv_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Token-shifted projections, data-dependent decay, and the per-head matrix state
    o_t = (S + diag(u) k_t v_t^T)^T r_t ;  S <- diag(w_t) S + k_t v_t^T   (S: key channel x value channel)."""
    T, W = h.shape
    H, D = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, W, dtype=h.dtype), h[:-1]])
    mix = {s: h + (prev - h) * w[f"{p}.mu.{s}"] for s in "rkvgw"}
    r = (mix["r"] @ w[f"{p}.r"].T).view(T, H, D)
    k = (mix["k"] @ w[f"{p}.k"].T).view(T, H, D)
    v = (mix["v"] @ w[f"{p}.v"].T).view(T, H, D)
    g = mix["g"] @ w[f"{p}.g"].T
    gate = g * torch.sigmoid(g)
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w[f"{p}.w1"].T) @ w[f"{p}.w2"].T + w[f"{p}.w0"])).view(T, H, D)
    u = w[f"{p}.u"]                                          # [H, D]
    S = torch.zeros(H, D, D, dtype=h.dtype)
    out = torch.zeros(T, H, D, dtype=h.dtype)
    for t in range(T):
        kv = k[t].unsqueeze(-1) * v[t].unsqueeze(-2)         # [H, D(key), D(value)]
        out[t] = torch.einsum("hij,hi->hj", S + u.unsqueeze(-1) * kv, r[t])
        S = decay[t].unsqueeze(-1) * S + kv
    out = out / torch.sqrt((out * out).mean(-1, keepdim=True) + eps)      # per head
    return (out.reshape(T, H * D) * w[f"{p}.norm"] * gate) @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------------------------- rotary
def yarn_frequencies(rot: dict) -> torch.Tensor:
    dims, base = rot["dims"], rot["base"]
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    sc = rot.get("scaling")
    if not sc:
        return f

    def dim_of(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(dim_of(sc["fast"])), 0)
    hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)],
                        dtype=torch.float64)
    return f / sc["factor"] * ramp + f * (1 - ramp)


def rotate_interleaved(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, ..., n >= dims]: pairs (2i, 2i+1) of the first dims coordinates turned by position * f_i"""
    dims = rot["dims"]
    f = yarn_frequencies(rot)
    mag = 0.1 * math.log(rot["scaling"]["factor"]) + 1.0 if rot.get("scaling") else 1.0
    a = positions.to(torch.float64).unsqueeze(-1) * f                      # [T, dims / 2]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    cos, sin = (torch.cos(a) * mag).to(x.dtype).view(shape), (torch.sin(a) * mag).to(x.dtype).view(shape)
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


# ----------------------------------------------------------------------------------------------- latent attention
def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    T, W = h.shape
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = weighted_rms(h @ w[f"{p}.dq"].T, w[f"{p}.dq.norm"], eps)
    q = (cq @ w[f"{p}.uq"].T).view(T, H, D + R)
    dkv = h @ w[f"{p}.dkv"].T
    c = weighted_rms(dkv[:, :C], w[f"{p}.dkv.norm"], eps)
    k_rot = rotate_interleaved(dkv[:, C:], pos, m["rot"])                  # [T, R], shared by the heads
    q_rot = rotate_interleaved(q[..., D:], pos, m["rot"])                  # [T, H, R]
    k_plain = (c @ w[f"{p}.uk"].T).view(T, H, D)
    val = (c @ w[f"{p}.uv"].T).view(T, H, Dv)
    score = (torch.einsum("thd,shd->hts", q[..., :D], k_plain) + torch.einsum("thr,sr->hts", q_rot, k_rot)) * m["scale"]
    causal = torch.ones(T, T, dtype=torch.bool).tril()
    score = score.masked_fill(~causal, float("-inf"))
    out = torch.einsum("hts,shd->thd", torch.softmax(score, -1), val)
    gate = torch.sigmoid(h @ w[f"{p}.g"].T)                                # [T, H]
    return (out * gate.unsqueeze(-1)).reshape(T, H * Dv) @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------------------------- feed-forward
def polynorm_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, eps: float) -> torch.Tensor:
    z = h @ w[f"{p}.up"].T
    a, b, c, e = w[f"{p}.act"].tolist()

    def unit(y):
        return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)
    return (a * unit(z) + b * unit(z ** 2) + c * unit(z ** 3) + e) @ w[f"{p}.down"].T


def route(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, router: dict):
    """chosen experts [T, top] and their weights: sigmoid scores; the choice adds a correction, the weights do not;
    only experts of the best groups (by the sum of a group's two largest choice scores) can be chosen"""
    E, top = router["experts"], router["top"]
    s = torch.sigmoid(h @ w[f"{p}.router"].T)
    choice = s + w[f"{p}.correction"]
    groups = router.get("groups")
    if groups:
        G, keep = groups["count"], groups["keep"]
        per = choice.view(-1, G, E // G)
        gscore = per.topk(min(2, E // G), dim=-1).values.sum(-1)           # [T, G]
        kept = gscore.topk(keep, dim=-1).indices
        mask = torch.zeros_like(gscore, dtype=torch.bool).scatter(1, kept, True)
        choice = per.masked_fill(~mask.unsqueeze(-1), float("-inf")).view(-1, E)
    idx = choice.topk(top, dim=-1).indices
    return idx, s.gather(1, idx)


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    idx, wt = route(h, w, p, mlp["router"])
    limit = mlp["expert"]["limit"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j, e in enumerate(idx[t].tolist()):
            g = torch.clamp(h[t] @ w[f"{p}.e{e}.gate"].T, max=limit)
            u = torch.clamp(h[t] @ w[f"{p}.e{e}.up"].T, -limit, limit)
            y = g * torch.sigmoid(1.702 * g) * (u + 1)
            out[t] += wt[t, j] * (y @ w[f"{p}.e{e}.down"].T)
    return out


# ----------------------------------------------------------------------------------------------- the model
def forward(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict, layers_out: Optional[list] = None) -> torch.Tensor:
    """logits [T, vocab] of one sequence; ``layers_out`` collects the residual stream after every layer"""
    eps = cfg["norm"]["eps"]
    x = embed(tokens, w, cfg)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        if layer["type"] == "wkv":
            y = wkv_mixer(x, w, p + ".mix", layer["mixer"], eps)
        elif layer["type"] == "latent_attention":
            y = latent_attention(x, w, p + ".mix", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + scalar_rms(y, w[f"{p}.norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            y = polynorm_ff(x, w, p + ".mlp", eps) if mlp["kind"] == "dense" else moe_ff(x, w, p + ".mlp", mlp)
            x = x + scalar_rms(y, w[f"{p}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return scalar_rms(x, w["final.norm"], eps) @ w["head"].T


def random_weights(cfg: dict, seed: int = 0, dtype=torch.float64) -> Dict[str, torch.Tensor]:
    """weights of the design's tensor names for a configuration, values rounded to bfloat16"""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(o, i, s=1.0):
        return torch.randn(o, i, generator=g) * (s / math.sqrt(i))

    w = {"embed": torch.randn(V, W, generator=g), "embed.norm": torch.tensor(1.0 + 0.1 * torch.randn((), generator=g).item()),
         "bigram": torch.randn(cfg["embedding"]["bigram"]["buckets"] + 1, W, generator=g) * 0.5,
         "final.norm": torch.tensor(1.1), "head": mat(V, W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}", layer["mixer"]
        w[f"{p}.norm1"] = torch.tensor(0.5 + 0.2 * torch.rand((), generator=g).item())
        if layer.get("mlp") is not None:
            w[f"{p}.norm2"] = torch.tensor(0.5 + 0.2 * torch.rand((), generator=g).item())
        if layer["type"] == "wkv":
            HD = m["heads"] * m["dim"]
            lora = m.get("decay_rank", 8)
            for s in "rkvgw":
                w[f"{p}.mix.mu.{s}"] = torch.rand(W, generator=g)
            for s in "rkvg":
                w[f"{p}.mix.{s}"] = mat(HD, W)
            w[f"{p}.mix.w1"] = mat(lora, W)
            w[f"{p}.mix.w2"] = mat(HD, lora)
            w[f"{p}.mix.w0"] = torch.randn(HD, generator=g) * 0.5 - 1.0
            w[f"{p}.mix.u"] = torch.randn(m["heads"], m["dim"], generator=g) * 0.5
            w[f"{p}.mix.norm"] = 1.0 + 0.1 * torch.randn(HD, generator=g)
            w[f"{p}.mix.o"] = mat(W, HD)
        else:
            H, D, R, Dv, C, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            w[f"{p}.mix.dq"] = mat(Q, W)
            w[f"{p}.mix.dq.norm"] = 1.0 + 0.1 * torch.randn(Q, generator=g)
            w[f"{p}.mix.uq"] = mat(H * (D + R), Q, 2.0)
            w[f"{p}.mix.dkv"] = mat(C + R, W)
            w[f"{p}.mix.dkv.norm"] = 1.0 + 0.1 * torch.randn(C, generator=g)
            w[f"{p}.mix.uk"] = mat(H * D, C, 2.0)
            w[f"{p}.mix.uv"] = mat(H * Dv, C)
            w[f"{p}.mix.g"] = mat(H, W)
            w[f"{p}.mix.o"] = mat(W, H * Dv)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            w[f"{p}.mlp.up"] = mat(mlp["ff"], W)
            w[f"{p}.mlp.down"] = mat(W, mlp["ff"])
            w[f"{p}.mlp.act"] = torch.tensor([0.9, 0.4, -0.3, 0.05])
        else:
            E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
            for e in range(E):
                w[f"{p}.mlp.e{e}.gate"] = mat(F, W, 2.0)
                w[f"{p}.mlp.e{e}.up"] = mat(F, W, 2.0)
                w[f"{p}.mlp.e{e}.down"] = mat(W, F)
            w[f"{p}.mlp.router"] = mat(E, W, 2.0)
            w[f"{p}.mlp.correction"] = torch.randn(E, generator=g) * 0.3
    return {k: v.to(torch.bfloat16).to(dtype) for k, v in w.items()}
