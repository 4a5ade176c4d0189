"""CPU tests of the Tizalorn path: the oracle's own consistency (a recurrence continued from a state equals the whole
run; a rotation is position-relative), the product's frequency blend against the oracle's, the checkpoint reader and
registry, the request table's reserved rows, and the partial-build bookkeeping."""
import math

import pytest
import torch

from oracle import tizalorn as tz
from tests import tizalorn_util as U


def test_oracle_wkv_is_causal_and_prefix_consistent():
    cfg = U.config([(U.wkv(2, 16), None)], width=32)
    w = tz.random_weights(cfg, 1)
    toks = U.tokens(40, cfg["vocab"], 2)
    full = tz.forward(toks, w, cfg)
    part = tz.forward(toks[:25], w, cfg)
    assert torch.allclose(full[:25], part, atol=1e-12)
    assert not torch.allclose(full[30], tz.forward(toks[:5] + [toks[5] ^ 1] + toks[6:], w, cfg)[30])   # an early token reaches far


def test_oracle_rotation_depends_on_relative_position_only():
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 2.0, "original": 32, "fast": 8.0, "slow": 1.0}}
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 12, generator=g, dtype=torch.float64), torch.randn(1, 12, generator=g, dtype=torch.float64)
    def score(pq, pk):
        return float((tz.rotate_interleaved(q, torch.tensor([pq]), rot)[0, :8] * tz.rotate_interleaved(k, torch.tensor([pk]), rot)[0, :8]).sum())
    assert abs(score(7, 3) - score(104, 100)) < 1e-9
    assert torch.equal(tz.rotate_interleaved(q, torch.tensor([5]), rot)[0, 8:], q[0, 8:])          # beyond dims: unchanged
    mag = 0.1 * math.log(2.0) + 1
    assert abs(float(tz.rotate_interleaved(q, torch.tensor([0]), rot)[0, 0]) - float(q[0, 0]) * mag) < 1e-12


@pytest.mark.parametrize("scaling", [None, {"factor": 2.5, "original": 1000, "fast": 24.0, "slow": 0.5},
                                     {"factor": 3.0, "original": 64, "fast": 16.0, "slow": 2.0},
                                     {"factor": 8.0, "original": 4096, "fast": 1.0, "slow": 1.0}])
def test_frequency_blend_matches_oracle(scaling):
    from scratchpad_amd.layers import AngleRotary
    for dims, base in ((16, 10000.0), (8, 100.0), (64, 500000.0)):
        rot = {"dims": dims, "base": base}
        if scaling:
            rot["scaling"] = scaling
        mod = AngleRotary(dims, base, scaling)
        want = tz.yarn_frequencies(rot)
        assert torch.allclose(mod.freq.double(), want, rtol=1e-6, atol=0)
        assert abs(mod.magnitude - (0.1 * math.log(scaling["factor"]) + 1 if scaling else 1.0)) < 1e-12


def test_oracle_router_masks_groups_with_minus_infinity():
    # all choice scores negative: a pruned group must not win by counting as 0
    w = {"p.router": torch.zeros(8, 4, dtype=torch.float64),
         "p.correction": torch.tensor([-5, -6, -7, -8, -1.0, -9, -9, -9], dtype=torch.float64)}
    idx, wt = tz.route(torch.ones(1, 4, dtype=torch.float64), w, "p", {"experts": 8, "top": 2, "groups": {"count": 2, "keep": 1}})
    # group 0: -4.5 + -5.5 = -10; group 1: -0.5 + -8.5 = -9 -> group 1 stays: experts 4 and one of 5..7
    assert idx[0, 0].item() == 4 and idx[0, 1].item() in (5, 6, 7)
    assert torch.allclose(wt, torch.full_like(wt, 0.5))


def test_registry_reads_config_and_weights(tmp_path):
    from scratchpad_amd import registry
    cfg = U.full_config()
    folder, w = U.make_model(tmp_path, cfg, seed=3)
    c = registry.load_config(folder, context_len=128)
    assert type(c).__name__ == "TizalornConfig" and c.vocab_size == cfg["vocab"] and c.num_hidden_layers == 5
    assert c.decay_rank(0) == 5 and c.decay_rank(2) == 6          # from the tensors' shapes
    assert c.latent_cache() == {1: (72, 12), 3: (40, 8)} and c.recurrent_layers() == {0: (3, 32), 2: (2, 48), 4: (1, 96)}
    got = dict(registry.iter_safetensors(folder))
    assert set(got) == set(w)
    for k in w:
        assert got[k].dtype == torch.bfloat16 and torch.equal(got[k].double(), w[k]), k
    assert registry.model_class_for(c).__name__ == "TizalornForCausalLM"
    with pytest.raises(ValueError):
        registry.architecture_of({"architecture": "NoSuchDesign"})


def test_request_table_reserved_rows():
    from scratchpad_amd.pool import ReqToTokenPool
    pool = ReqToTokenPool(5, 8, "cpu", reserved_rows=1)
    assert pool.available_size() == 4 and pool.alloc(4) == [1, 2, 3, 4] and pool.alloc(1) is None
    pool.free([3, 1])
    assert pool.alloc(2) == [3, 1]
    pool.clear()
    assert 0 not in pool.free_slots


def test_model_names_its_native_sources():
    import os
    from scratchpad_amd import build
    from scratchpad_amd.tizalorn import TizalornForCausalLM
    for src in TizalornForCausalLM.NATIVE_SOURCES + build.CORE_SOURCES:
        assert os.path.exists(os.path.join(build.CSRC, src)), src
    have = build.built_sources()
    assert have is None or set(build.CORE_SOURCES) <= set(have)
