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


def random_config(seed: int):
    """a design drawn at random: layer order, every size and constant (small enough for the oracle, odd enough to miss
    every power of two now and then)"""
    import random
    r = random.Random(seed)
    layers = []
    for _ in range(r.randint(3, 6)):
        kind = r.choice(["attention", "mamba2", "mlstm"])
        if kind == "attention":
            heads = r.choice([1, 2, 3, 4, 6])
            kv = r.choice([d for d in range(1, heads + 1) if heads % d == 0])
            dim = r.choice([8, 16, 24, 32, 64])
            size = r.choice([None, 1, 2, 5, 11, 17, 32])
            spec = attention(heads, kv, dim, r.choice([8, 16, 40, 64]), size=size, pool=r.choice([1, 2, 3, 5, 8, 0]) if size else 0,
                             dims=r.choice([0, dim, dim // 2 // 2 * 2 or 2]), scaling=r.random() < 0.6,
                             base=r.choice([100.0, 10000.0]), scale=r.choice([None, 0.3, 0.11]))
            if size and not spec["mixer"]["mask"]["pool"]:
                del spec["mixer"]["mask"]["pool"]
        elif kind == "mamba2":
            heads = r.choice([1, 2, 3, 4])
            spec = mamba2(heads, r.choice([8, 16, 24]), r.choice([8, 16, 40]), groups=r.choice([d for d in range(1, heads + 1) if heads % d == 0]),
                          conv=r.choice([1, 2, 3, 4]), norm_groups=r.choice([d for d in range(1, heads + 1) if heads % d == 0]))
        else:
            spec = mlstm(r.choice([1, 2, 3]), r.choice([8, 16, 40]), r.choice([8, 24, 64]), cap=r.choice([2.0, 7.5, 15.0]))
        pick = r.random()
        if pick < 0.2:
            mlp = None
        elif pick < 0.55:
            mlp = dense(r.choice([24, 56, 100]), limit=r.choice([0.5, 2.0, 6.0]))
        else:
            experts = r.randint(2, 9)
            mlp = moe(experts, r.randint(1, min(experts, 4)), r.choice([8, 24, 40]), scale=r.choice([0.5, 1.0, 2.5]),
                      shared=r.choice([None, 16, 48]))
        layers.append((spec, mlp))
    return config(layers, width=r.choice([48, 64, 96, 128]), vocab=r.choice([61, 130, 257]), eps=r.choice([1e-6, 1e-5]),
                  scale=r.choice([0.25, 1.0, 3.0]))
