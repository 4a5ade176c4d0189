"""Helpers of the Sominex tests: small configurations whose sizes differ from one another (key width unlike value width,
state size unlike head width, a rotation narrower than the head, windows and blocks of a few tokens), a checkpoint folder
written from the oracle's random weights, and the comparison used throughout."""
import torch

from oracle import sominex as so
from tests.tizalorn_util import rel, tokens, write_checkpoint  # noqa: F401  (the checkpoint writer is format-only)


def attention(heads, kv_heads, dim, vdim, size=12, pool=4, dims=None, scaling=True, base=500.0, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5}
    if dims != 0:
        m["rot"] = {"base": base, "dims": dims or dim}
        if scaling:
            m["rot"]["scaling"] = {"factor": 3.0, "original": 48, "fast": 16.0, "slow": 2.0}
    if size:
        m["mask"] = {"size": size, "pool": pool}
    return {"type": "attention", "mixer": m}


def mamba2(heads, vdim, state, groups=1, conv=4, norm_groups=1):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                         "norm_groups": norm_groups}}


def mlstm(heads, dim, vdim, cap=9.0):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def dense(ff, limit=1.5):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff, scale=1.5, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def config(layers, width=80, vocab=173, eps=1e-5, scale=0.7):
    return {"architecture": "Sominex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": [{**spec, "mlp": mlp} for spec, mlp in layers]}


def full_config():
    """every mechanism in an order of its own, sizes unlike each other, one layer without a feed-forward"""
    return config([
        (mlstm(3, 24, 40), moe(6, 2, 32, shared=48)),
        (attention(6, 2, 24, 40, size=10, pool=3, dims=16), dense(120)),
        (mamba2(4, 24, 40, groups=2, conv=3, norm_groups=2), None),
        (attention(2, 1, 32, 16, size=7, pool=2, scaling=False), moe(5, 1, 40, scale=0.8)),
        (mamba2(2, 72, 16, groups=2, conv=4, norm_groups=1), dense(96, limit=0.8)),
        (mlstm(1, 80, 16, cap=4.0), None),
    ], width=96)


def make_model(tmp_path, cfg, seed=0, name="m"):
    w = so.random_weights(cfg, seed)
    return write_checkpoint(str(tmp_path / name), cfg, w), w


def greedy(prompt, w, cfg, n):
    """n tokens of greedy generation by the oracle (the whole sequence again for every token)"""
    seq, out = list(prompt), []
    for _ in range(n):
        t = int(torch.argmax(so.forward(seq, w, cfg)[-1]))
        out.append(t)
        seq.append(t)
    return out
