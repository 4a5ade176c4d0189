"""CPU oracle of the Sominex design: one plain, slow function per mechanism, written from the design's equations.

TEST INFRASTRUCTURE ONLY: nothing under scratchpad_amd/ imports this, and this imports nothing from there.  Every
function works on ONE whole sequence in float64 (or the dtype it is given) and keeps no cache and no state: a sequence
is recomputed from its first token, which is what makes it a reference for caches, states, portions and batches.

Notation: T tokens, W model width, x the residual stream [T, W], h = the layer's normed input.
A layer is  x <- x + mixer(shift(h)) + ff(h)  with h = rms(x) * w1 and shift(h)[t] = h[t] + (h[t-1] - h[t]) * mu.
"""
import math
from typing import Dict, List, Optional

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (prev - h) * mu


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def logsigmoid(z):
    return -softplus(-z)


# ----------------------------------------------------------------------------------------------- rotary
def rotary_frequencies(rot: dict) -> (torch.Tensor, float):
    """(frequency per pair [dims/2], magnitude of cos and sin)"""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor = float(sc["factor"])

    def at(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(at(sc["fast"])), 0)
    hi = min(math.ceil(at(sc["slow"])), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)], dtype=torch.float64)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half_pairs(x: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, heads, n]: coordinate i < dims/2 is paired with i + dims/2; the rest of n passes"""
    dims = int(rot["dims"])
    if dims == 0:
        return x
    f, mag = rotary_frequencies(rot)
    half = dims // 2
    pos = torch.arange(x.shape[0], dtype=torch.float64)
    ang = pos[:, None] * f[None, :]
    c, s = (torch.cos(ang) * mag).to(x.dtype)[:, None, :], (torch.sin(ang) * mag).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


# ----------------------------------------------------------------------------------------------- attention
def visible(i: int, size: int, pool: int):
    """(pooled blocks, tokens) that position i sees: tokens j with 0 <= i - j < size, and block b (positions b*pool ..
    b*pool + pool - 1) once its last position is at most i - size"""
    tokens = list(range(max(0, i - size + 1), i + 1))
    blocks = []
    if pool:
        b = 0
        while b * pool + pool - 1 <= i - size:
            blocks.append(b)
            b += 1
    return blocks, tokens


def pooled_window_attention(q, k, v, size: int, pool: int, scale: float) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, Dv] as the cache holds them -> [T, H, Dv]; one softmax over a query's window
    tokens and the means of the blocks wholly behind the window"""
    T, H, D = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for i in range(T):
        blocks, tokens = visible(i, size, pool)
        ks = [k[b * pool:(b + 1) * pool].mean(0) for b in blocks] + [k[j] for j in tokens]
        vs = [v[b * pool:(b + 1) * pool].mean(0) for b in blocks] + [v[j] for j in tokens]
        K, V = torch.stack(ks), torch.stack(vs)              # [n, G, *]
        for h in range(H):
            g = h // (H // G)
            p = torch.softmax((K[:, g] @ q[i, h]) * scale, 0)
            out[i, h] = p @ V[:, g]
    return out


def attention_mixer(h, w, p: str, m: dict, eps: float, kv_round=None) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[f"{p}.q"].T).view(T, H, D)
    k = (h @ w[f"{p}.k"].T).view(T, G, D)
    v = (h @ w[f"{p}.v"].T).view(T, G, Dv)
    rot = m.get("rot") or {"dims": 0}
    q, k = rotate_half_pairs(q, rot), rotate_half_pairs(k, rot)
    v = rms(v, eps)
    if kv_round is not None:           # what a cache of lower precision holds
        k, v = kv_round(k), kv_round(v)
    mask = m.get("mask") or {}
    o = pooled_window_attention(q, k, v, int(mask.get("size", T + 1)), int(mask.get("pool", 0)), float(m["scale"]))
    return o.reshape(T, H * Dv) @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------------------------- mamba2
def causal_conv(u: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """u [T, C], weight [C, taps] (last column = the current token's), zeros before the start"""
    T, C = u.shape
    taps = weight.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=u.dtype), u])
    out = bias.expand(T, C).clone()
    for j in range(taps):
        out = out + pad[j:j + T] * weight[:, j]
    return out


def mamba2_mixer(h, w, p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, Dv, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = H * Dv
    a = h @ w[f"{p}.in"].T
    z, xbc, dt = a[:, :inner], a[:, inner:2 * inner + 2 * G * N], a[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[f"{p}.conv"], w[f"{p}.conv.b"]))
    xs = xbc[:, :inner].view(T, H, Dv)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[f"{p}.dt_bias"])                    # [T, H]
    decay = torch.exp(-torch.exp(w[f"{p}.A_log"]) * dt)      # [T, H]
    S = torch.zeros(H, N, Dv, dtype=h.dtype)
    y = torch.zeros(T, H, Dv, dtype=h.dtype)
    for t in range(T):
        for hd in range(H):
            g = hd // (H // G)
            S[hd] = decay[t, hd] * S[hd] + dt[t, hd] * torch.outer(B[t, g], xs[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + w[f"{p}.D"][hd] * xs[t, hd]
    y = y.reshape(T, inner) * silu(z)
    parts = int(m["norm_groups"])
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[f"{p}.norm"]
    return y @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------------------------- mlstm
def mlstm_mixer(h, w, p: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, Dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    q = (h @ w[f"{p}.q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[f"{p}.k"].T).view(T, H, D)
    v = (h @ w[f"{p}.v"].T).view(T, H, Dv)
    ig = cap * torch.tanh((h @ w[f"{p}.i"].T + w[f"{p}.i.b"]) / cap)                   # log input gate [T, H]
    fg = logsigmoid(cap * torch.tanh((h @ w[f"{p}.f"].T + w[f"{p}.f.b"]) / cap))       # log forget gate
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    n = torch.zeros(H, D, dtype=h.dtype)
    mx = torch.zeros(H, dtype=h.dtype)
    o = torch.zeros(T, H, Dv, dtype=h.dtype)
    for t in range(T):
        m_new = torch.maximum(fg[t] + mx, ig[t])
        keep, take = torch.exp(fg[t] + mx - m_new), torch.exp(ig[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        o[t] = num / den[:, None]
    o = rms(o, eps).reshape(T, H * Dv) * w[f"{p}.norm"] * torch.sigmoid(h @ w[f"{p}.g"].T)
    return o @ w[f"{p}.o"].T


# ----------------------------------------------------------------------------------------------- feed-forwards
def dense_ff(h, w, p: str, mlp: dict) -> torch.Tensor:
    limit = float(mlp["limit"])
    g = torch.clamp(h @ w[f"{p}.gate"].T, max=limit)
    u = torch.clamp(h @ w[f"{p}.up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[f"{p}.down"].T


def plain_expert(h, w, p: str) -> torch.Tensor:
    return (silu(h @ w[f"{p}.gate"].T) * (h @ w[f"{p}.up"].T)) @ w[f"{p}.down"].T


def route(h, router: torch.Tensor, top: int, scale: float):
    """(ids [T, top], weights [T, top]): the `top` largest of softmax(router h), times scale, not renormalised"""
    s = torch.softmax(h @ router.T, -1)
    val, ids = torch.topk(s, top, dim=-1)
    return ids, val * scale


def moe_ff(h, w, p: str, mlp: dict) -> torch.Tensor:
    r = mlp["router"]
    ids, wts = route(h, w[f"{p}.router"], int(r["top"]), float(r["scale"]))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(ids[t].tolist(), wts[t]):
            out[t] = out[t] + a * plain_expert(h[t:t + 1], w, f"{p}.e{e}")[0]
    if mlp.get("shared"):
        out = out + plain_expert(h, w, f"{p}.shared")
    return out


# ----------------------------------------------------------------------------------------------- the model
MIXERS = {"attention": attention_mixer, "mamba2": mamba2_mixer, "mlstm": mlstm_mixer}


def layer(x, w, i: int, spec: dict, eps: float) -> torch.Tensor:
    p = f"l{i}"
    h = rms(x, eps) * w[f"{p}.norm1"]
    y = MIXERS[spec["type"]](token_shift(h, w[f"{p}.shift"]), w, f"{p}.mix", spec["mixer"], eps)
    mlp = spec.get("mlp")
    if mlp is not None:
        y = y + (dense_ff(h, w, f"{p}.mlp", mlp) if mlp["kind"] == "dense" else moe_ff(h, w, f"{p}.mlp", mlp))
    return x + y


def forward(tokens: List[int], w: Dict[str, torch.Tensor], cfg: dict, streams: Optional[list] = None) -> torch.Tensor:
    """logits [T, vocab] of one whole sequence; `streams` (a list) receives the residual stream after every layer"""
    eps = float(cfg["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)] * float(cfg["embedding"]["scale"])
    for i, spec in enumerate(cfg["layers"]):
        x = layer(x, w, i, spec, eps)
        if streams is not None:
            streams.append(x.clone())
    return (rms(x, eps) * w["final.norm"]) @ w["head"].T


def random_weights(cfg: dict, seed: int = 0, dtype=torch.float64) -> Dict[str, torch.Tensor]:
    """a checkpoint's tensors (names and shapes of the design) with random values of a scale that keeps every branch
    busy; values are rounded to bfloat16, as a checkpoint stores them"""
    g = torch.Generator().manual_seed(seed)
    W, w = int(cfg["width"]), {}

    def mat(o, i, s=1.0):
        return torch.randn(o, i, generator=g) * s / math.sqrt(i)

    def vec(n, mean=0.0, s=1.0):
        return mean + torch.randn(n, generator=g) * s

    def glu(p, ff):
        w[f"{p}.gate"], w[f"{p}.up"], w[f"{p}.down"] = mat(ff, W, 1.5), mat(ff, W, 1.5), mat(W, ff)
    w["embed"] = torch.randn(int(cfg["vocab"]), W, generator=g)
    w["head"] = mat(int(cfg["vocab"]), W)
    w["final.norm"] = vec(W, 1.0, 0.1)
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}", spec["mixer"]
        w[f"{p}.norm1"], w[f"{p}.shift"] = vec(W, 1.0, 0.1), torch.rand(W, generator=g)
        if spec["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[f"{p}.mix.q"], w[f"{p}.mix.k"], w[f"{p}.mix.v"] = mat(H * D, W, 2.0), mat(G * D, W, 2.0), mat(G * Dv, W)
            w[f"{p}.mix.o"] = mat(W, H * Dv)
        elif spec["type"] == "mamba2":
            H, Dv, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            inner, ch = H * Dv, H * Dv + 2 * G * N
            w[f"{p}.mix.in"] = mat(2 * inner + 2 * G * N + H, W)
            w[f"{p}.mix.conv"], w[f"{p}.mix.conv.b"] = torch.randn(ch, taps, generator=g) * 0.5, vec(ch, 0.0, 0.1)
            w[f"{p}.mix.dt_bias"], w[f"{p}.mix.A_log"], w[f"{p}.mix.D"] = vec(H, -1.0, 1.0), vec(H, -1.0, 1.0), vec(H, 1.0, 0.3)
            w[f"{p}.mix.norm"], w[f"{p}.mix.o"] = vec(inner, 1.0, 0.1), mat(W, inner)
        elif spec["type"] == "mlstm":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            w[f"{p}.mix.q"], w[f"{p}.mix.k"], w[f"{p}.mix.v"] = mat(H * D, W), mat(H * D, W), mat(H * Dv, W)
            w[f"{p}.mix.g"], w[f"{p}.mix.o"], w[f"{p}.mix.norm"] = mat(H * Dv, W), mat(W, H * Dv), vec(H * Dv, 1.0, 0.1)
            w[f"{p}.mix.i"], w[f"{p}.mix.i.b"] = mat(H, W, 3.0), vec(H, 0.0, 1.0)
            w[f"{p}.mix.f"], w[f"{p}.mix.f.b"] = mat(H, W, 3.0), vec(H, 3.0, 1.0)
        else:
            raise ValueError(spec["type"])
        mlp = spec.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            glu(f"{p}.mlp", mlp["ff"])
        else:
            for e in range(mlp["router"]["experts"]):
                glu(f"{p}.mlp.e{e}", mlp["expert"]["ff"])
            w[f"{p}.mlp.router"] = mat(mlp["router"]["experts"], W, 2.0)
            if mlp.get("shared"):
                glu(f"{p}.mlp.shared", mlp["shared"]["ff"])
    return {k: v.to(torch.bfloat16).to(dtype) for k, v in w.items()}
