"""Helpers of the Tizalorn tests: small configurations (sizes chosen to differ from one another: head sizes that are no
power of two, a rotation narrower than the rotated part, value width unlike key width, groups with and without pruning),
a checkpoint folder written from the oracle's random weights, and the comparison used throughout."""
import json
import os
import struct

import torch

from oracle import tizalorn as tz


def wkv(heads, dim, rank=6):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim, "decay_rank": rank}}


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, dims=None, scaling=True, base=10000.0):
    rot = {"base": base, "dims": dims or rot_dim}
    if scaling:
        rot["scaling"] = {"factor": 3.0, "original": 64, "fast": 16.0, "slow": 2.0}
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "rot": rot, "scale": (dim + rot_dim) ** -0.5}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, groups=None, keep=None, limit=1.5):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}


def config(layers, width=96, vocab=211, eps=1e-5, buckets=97, mul_prev=31, mul_cur=7):
    out = []
    for spec, mlp in layers:
        out.append({**spec, "mlp": mlp})
    return {"architecture": "Tizalorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": out,
            "embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}}


def full_config():
    """every mechanism, sizes unlike each other: two recurrent layers of different head shapes, two latent layers of
    different cache widths, a layer without a feed-forward, experts with pruned groups / without groups / top 1"""
    return config([
        (wkv(3, 32, rank=5), dense(160)),
        (latent(3, 24, 12, 40, 72, 56, dims=8), moe(12, 3, 48, groups=3, keep=2)),
        (wkv(2, 48), None),
        (latent(2, 16, 8, 16, 40, 64, scaling=False), moe(6, 1, 40)),
        (wkv(1, 96), moe(8, 2, 56, groups=2, keep=2)),
    ])


_ST = {torch.bfloat16: "BF16", torch.float32: "F32", torch.int32: "I32"}


def write_checkpoint(folder, cfg, weights, dtype=torch.bfloat16):
    """config.json + model.safetensors (8-byte header length, JSON header, raw little-endian data)"""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, t in weights.items():
        t = t.to(dtype).contiguous()
        raw = t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes()
        header[name] = {"dtype": _ST[dtype], "shape": list(t.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    head = json.dumps(header).encode()
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(head)) + head + b"".join(blobs))
    return folder


def make_model(tmp_path, cfg, seed=0, name="m"):
    w = tz.random_weights(cfg, seed)
    return write_checkpoint(str(tmp_path / name), cfg, w), w


def rel(got: torch.Tensor, want: torch.Tensor) -> float:
    """largest deviation relative to the reference's largest magnitude"""
    want = want.detach().cpu().to(torch.float64)
    return float((got.detach().cpu().to(torch.float64) - want).abs().max() / want.abs().max())


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
