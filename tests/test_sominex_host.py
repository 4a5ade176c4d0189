"""CPU tests around the Sominex design: the oracle against itself (visibility rule, recurrences carried in pieces), the
configuration reader, the registry, and the shapes the pools are built from."""
import json

import pytest
import torch

from oracle import sominex as so
from tests import sominex_util as U


def test_visibility_rule_counts():
    # window 4, blocks of 3: position 9 sees tokens 6..9 and blocks 0 (0..2) and 1 (3..5); position 8 sees 5..8 and only
    # block 0: token 3 and 4 have left the window and their block is not complete behind it
    assert so.visible(9, 4, 3) == ([0, 1], [6, 7, 8, 9])
    assert so.visible(8, 4, 3) == ([0], [5, 6, 7, 8])
    assert so.visible(3, 4, 3) == ([], [0, 1, 2, 3])
    assert so.visible(6, 4, 3) == ([0], [3, 4, 5, 6])
    assert so.visible(5, 4, 0) == ([], [2, 3, 4, 5])


def test_oracle_is_causal_and_deterministic():
    cfg = U.full_config()
    w = so.random_weights(cfg, 3)
    toks = U.tokens(40, cfg["vocab"], 1)
    a = so.forward(toks, w, cfg)
    b = so.forward(toks[:25], w, cfg)
    assert torch.allclose(a[:25], b, atol=1e-9)
    assert torch.isfinite(a).all()


def test_oracle_softmax_router_weights_are_not_renormalised():
    g = torch.Generator().manual_seed(0)
    h = torch.randn(9, 16, generator=g, dtype=torch.float64)
    r = torch.randn(7, 16, generator=g, dtype=torch.float64)
    ids, wts = so.route(h, r, 3, 2.5)
    s = torch.softmax(h @ r.T, -1)
    assert torch.allclose(wts, s.gather(1, ids) * 2.5)
    assert (wts.sum(-1) < 2.5).all()


def test_config_reader_registry_and_pool_shapes():
    from scratchpad_amd import registry
    from scratchpad_amd.sominex import SominexConfig, SominexForCausalLM
    raw = U.full_config()
    assert registry.architecture_of(raw) == "Sominex"
    cfg = registry.MODELS["Sominex"][0](raw, context_len=256)
    assert isinstance(cfg, SominexConfig) and registry.model_class_for(cfg) is SominexForCausalLM
    assert cfg.window_cache() == {1: (2, 24, 40, True), 3: (1, 32, 16, True)}
    named = cfg.named_state()
    assert named[0] == {"S": (3, 24, 40), "n": (3, 24), "m": (3,)}
    assert named[2] == {"ssm": (4, 40, 24), "conv": (2, 4 * 24 + 2 * 2 * 40)}
    assert cfg.shift_layers() == list(range(6))
    assert cfg.cache_bytes_per_token(torch.bfloat16) == 2 * 2 * (2 * (24 + 40) + 1 * (32 + 16))
    no_pool = U.config([(U.attention(2, 2, 8, 8, size=None), None)])
    assert registry.MODELS["Sominex"][0](no_pool).window_cache() == {0: (2, 8, 8, False)}
    with pytest.raises(ValueError):
        SominexConfig({**raw, "layers": [{"type": "conv", "mixer": {}, "mlp": None}]})


def test_model_loads_a_checkpoint_on_cpu(tmp_path):
    """names and merges of load_weights (no kernel runs): merged projections hold the checkpoint's rows in order"""
    from scratchpad_amd import distributed, registry
    from scratchpad_amd.sominex import SominexForCausalLM
    if not distributed.model_parallel_is_initialized():
        distributed.initialize_model_parallel(1)
    raw = U.full_config()
    folder, w = U.make_model(tmp_path, raw, seed=2)
    cfg = registry.load_config(folder, context_len=64)
    model = SominexForCausalLM(cfg, dtype=torch.float32)
    registry.load_weights(model, folder)
    att = model.layers[1].mix
    assert torch.equal(att.qkv[:6 * 24].double(), w["l1.mix.q"]) and torch.equal(att.qkv[-2 * 40:].double(), w["l1.mix.v"])
    mam = model.layers[2].mix
    assert torch.equal(mam.dt_proj.double(), w["l2.mix.in"][-4:]) and mam.in_proj.shape[0] == 2 * 96 + 2 * 2 * 40
    ml = model.layers[0].mix
    assert torch.equal(ml.gates[3:].double(), w["l0.mix.f"]) and torch.equal(ml.gates_bias[:3].double(), w["l0.mix.i.b"])
    ex = model.layers[0].mlp.routed.experts
    assert torch.equal(ex.gate_up[4, 32:].double(), w["l0.mlp.e4.up"]) and model.layers[2].mlp is None
    assert json.load(open(folder + "/config.json"))["architecture"] == "Sominex"
