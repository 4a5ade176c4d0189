"""Sominex through the engine on the GPU against the CPU oracle (float64, one sequence at a time, no cache or state):
single mechanisms, kernels on crafted inputs (window and block edges, a far key that only a pooled block carries), whole
prompts, decoding through cache and state, portions down to two tokens, unequal batches, reused rows and slots, graph
replay, other sizes, and generation through the engine's scheduler.

Sharp comparisons run the engine in fp32 (the oracle's weights are bf16-representable, so both see the same numbers); a
bf16 pass checks the serving precision against a looser bar."""
import pytest
import torch

from oracle import sominex as so
from tests import sominex_util as U

pytestmark = pytest.mark.gpu
F32_BAR = 2e-4


def engine(folder, dtype=torch.float32, tokens=512, slots=4, graphs=False, chunk=2048):
    from scratchpad_amd.engine import Engine
    return Engine(folder, dtype=dtype, max_total_tokens=tokens, max_running_requests=slots, use_graphs=graphs, chunk_size=chunk)


def entry(rid, toks, want=None):
    from scratchpad_amd.engine import StepEntry
    return StepEntry(rid, list(toks), list(range(len(toks))) if want is None else want)


def run_whole(eng, toks, rid="w"):
    return eng.step([entry(rid, toks)], [rid])


def run_portions(eng, toks, sizes, rid="p"):
    """feed toks in portions of the given sizes (the last size repeats), logits of every position"""
    outs, at, i = [], 0, 0
    while at < len(toks):
        n = min(sizes[min(i, len(sizes) - 1)], len(toks) - at)
        outs.append(eng.step([entry(rid, toks[at:at + n])], [rid] if at + n == len(toks) else []))
        at, i = at + n, i + 1
    return torch.cat(outs)


# ------------------------------------------------------------------------------------------------ mechanisms alone
LAYERS = [
    (U.attention(4, 2, 16, 24, size=9, pool=3, dims=8), None),
    (U.attention(3, 3, 24, 8, size=5, pool=1, scaling=False), None),          # blocks of one token, kv heads = heads
    (U.attention(5, 1, 8, 72, size=1, pool=4), None),                         # a window of the token itself
    (U.attention(2, 2, 16, 16, size=None, dims=0), None),                     # no window, no rotation
    (U.attention(2, 1, 40, 16, size=30, pool=7, dims=20), None),              # head width no multiple of 16
    (U.mamba2(4, 16, 24, groups=2, conv=4, norm_groups=2), None),
    (U.mamba2(3, 40, 8, groups=3, conv=2, norm_groups=1), None),              # a group per head
    (U.mamba2(1, 80, 72, groups=1, conv=5, norm_groups=5), None),
    (U.mamba2(2, 136, 136, groups=2, conv=3, norm_groups=4), None),          # state and head width above 128
    (U.mlstm(3, 16, 24), None), (U.mlstm(1, 72, 8, cap=3.0), None), (U.mlstm(4, 8, 80), None),
    (U.mlstm(2, 136, 136, cap=20.0), None), (U.attention(2, 1, 136, 200, size=33, pool=5, dims=72), None),
    (U.mlstm(2, 16, 16), U.dense(100)), (U.mlstm(2, 16, 16), U.dense(40, limit=0.3)),
    (U.mlstm(2, 16, 16), U.moe(12, 3, 24, scale=2.0, shared=56)), (U.mlstm(2, 16, 16), U.moe(5, 1, 40, scale=1.0)),
    (U.mlstm(2, 16, 16), U.moe(4, 4, 16, shared=8)),
]


@pytest.mark.parametrize("layer", LAYERS, ids=lambda l: f"{l[0]['type']}-{'none' if l[1] is None else l[1]['kind']}")
def test_single_layer_models_match_oracle(tmp_path, layer):
    cfg = U.config([layer], width=80)
    folder, w = U.make_model(tmp_path, cfg, seed=5)
    toks = U.tokens(70, cfg["vocab"], 6)
    eng = engine(folder)
    eng.runner.model.capture_layers = []
    got = run_whole(eng, toks)
    lay = []
    want = so.forward(toks, w, cfg, lay)
    assert U.rel(eng.runner.model.capture_layers[0], lay[0]) < F32_BAR
    assert U.rel(got, want) < F32_BAR


def test_softmax_router_kernel_against_oracle():
    from scratchpad_amd import _native
    g = torch.Generator().manual_seed(0)
    for E, top, scale in ((12, 3, 2.0), (5, 1, 1.0), (64, 8, 0.5), (70, 70, 1.0), (3, 2, 4.0)):
        x = torch.randn(50, 40, generator=g)
        router = torch.randn(E, 40, generator=g) * 0.6
        ids, wt = _native.moe_route_softmax(x.cuda(), router.cuda(), top, scale)
        want_ids, want_wt = so.route(x.double(), router.double(), top, scale)
        assert torch.equal(ids.cpu().long().sort(-1).values, want_ids.sort(-1).values), (E, top)
        order = ids.cpu().long().argsort(-1)
        assert torch.allclose(wt.cpu().gather(1, order).double(), want_wt.gather(1, want_ids.argsort(-1)), atol=1e-6)


# ------------------------------------------------------------------------------------------------ the attention kernels
class AttnBench:
    """one request on row 2 of a request table whose slots are a shuffled part of a pool: the store, the block means and
    the attention kernel driven the way the model drives them, in portions"""

    def __init__(self, H, G, D, Dv, size, P, rot=None, dtype=torch.float32, slots=400, seed=0, matrix=True):
        from scratchpad_amd import _native
        from scratchpad_amd.layers import HalfAngleRotary
        self.n, self.H, self.G, self.D, self.Dv, self.size, self.P, self.dtype = _native, H, G, D, Dv, size, P, dtype
        g = torch.Generator().manual_seed(seed)
        self.perm = (torch.randperm(slots, generator=g) + 1).cuda()
        mk = lambda w: torch.full((slots + 1, w), float("nan"), dtype=dtype, device="cuda")       # reading a stale slot shows
        self.k, self.v, self.kp, self.vp = mk(G * D), mk(G * Dv), mk(G * D), mk(G * Dv)
        self.table = torch.zeros((4, slots + 8), dtype=torch.int32, device="cuda")
        self.rotary = HalfAngleRotary(rot["dims"], rot["base"], rot.get("scaling")).cuda() if rot else None
        self.held, self.matrix = 0, matrix

    def step(self, q, k, v):
        """q [n, H*D], k [n, G*D], v [n, G*Dv] of the next n positions -> [n, H*Dv]"""
        n_, dev = self.n, "cuda"
        n = q.shape[0]
        loc = self.perm[self.held:self.held + n].long()
        self.table[2, self.held:self.held + n] = loc.int()
        pos = torch.arange(self.held, self.held + n, device=dev)
        rows, lens = torch.tensor([2], device=dev), torch.tensor([self.held + n], device=dev)
        if n == 1 and self.held > 0:
            seq = n_.SeqParams(rows, lens)
        else:
            i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
            seq = n_.SeqParams(rows, lens, i32([n]), i32([self.held]), i32([0]), torch.zeros(n, dtype=torch.int32, device=dev))
        q = q.to(self.dtype).cuda().clone()
        freq, mag = (self.rotary.freq, self.rotary.magnitude) if self.rotary else (None, 1.0)
        n_.qkv_rotary_store(q, k.to(self.dtype).cuda(), v.to(self.dtype).cuda(), self.k, self.v, pos, loc, freq, mag,
                            self.H, self.G, self.D, self.Dv, 1e-6)
        if self.P:
            n_.pool_blocks(self.kp, self.vp, self.k, self.v, self.table, seq, self.P)
        out = n_.window_attention(q, self.k, self.v, self.kp if self.P else None, self.vp if self.P else None, self.table, seq,
                                  self.H, self.G, self.D, self.Dv, self.size, self.P, 0.25, self.matrix)
        self.held += n
        return out.float().cpu()


def attn_oracle(q, k, v, H, G, D, Dv, size, P, rot=None):
    T = q.shape[0]
    q, k, v = q.double().view(T, H, D), k.double().view(T, G, D), v.double().view(T, G, Dv)
    if rot:
        q, k = so.rotate_half_pairs(q, rot), so.rotate_half_pairs(k, rot)
    return so.pooled_window_attention(q, k, so.rms(v, 1e-6), size or T + 1, P, 0.25).reshape(T, H * Dv)


@pytest.mark.parametrize("sizes", [[150], [1], [7, 2, 40, 1, 1, 1, 3, 64, 1], [2]], ids=["whole", "decode", "mixed", "pairs"])
@pytest.mark.parametrize("shape", [(4, 2, 16, 24, 12, 4), (2, 2, 8, 8, 1, 1), (3, 1, 24, 72, 20, 16), (2, 1, 16, 16, 0, 0),
                                   (2, 2, 16, 8, 64, 3)], ids=lambda s: "x".join(map(str, s)))
def test_window_attention_edges_in_prompts_and_decoding(shape, sizes):
    """peaked softmaxes (scores of a few units): a key that is wrongly seen, missed, or taken from a block one step early
    or late moves the output by far more than the bar; every position of 150 is compared, so every window and block edge
    is crossed by a portion's start, its end and single tokens"""
    H, G, D, Dv, size, P = shape
    g = torch.Generator().manual_seed(3)
    T = 150
    q, k, v = torch.randn(T, H * D, generator=g) * 2, torch.randn(T, G * D, generator=g) * 2, torch.randn(T, G * Dv, generator=g)
    rot = {"dims": D // 2, "base": 100.0, "scaling": {"factor": 2.0, "original": 32, "fast": 8.0, "slow": 1.0}}
    bench = AttnBench(H, G, D, Dv, size, P, rot)
    outs, at, i = [], 0, 0
    while at < T:
        n = min(sizes[min(i, len(sizes) - 1)], T - at)
        outs.append(bench.step(q[at:at + n], k[at:at + n], v[at:at + n]))
        at, i = at + n, i + 1
    assert U.rel(torch.cat(outs), attn_oracle(q, k, v, H, G, D, Dv, size, P, rot)) < 2e-5


def test_far_key_reaches_a_query_only_through_its_block():
    """one loud key at position 5 among 300 quiet ones (positions 0..5 share one value pattern), window 32, blocks of 8:
    queries see it as a token up to position 36, not at all at 37 and 38 (its block 0..7 is seen once 7 <= p - 32), and
    from 39 on through the block's mean"""
    H = G = 1
    D, Dv, size, P, T = 16, 64, 32, 8, 300
    g = torch.Generator().manual_seed(1)
    q, k, v = torch.randn(T, D, generator=g) * 0.1, torch.randn(T, D, generator=g) * 0.1, torch.randn(T, Dv, generator=g)
    q[:, 0], k[5, 0] = 6.0, 40.0
    v[:6] = torch.arange(Dv) - 31.5
    for sizes in ([T], [33, 1]):
        bench = AttnBench(H, G, D, Dv, size, P)
        outs, at, i = [], 0, 0
        while at < T:
            n = min(sizes[min(i, len(sizes) - 1)], T - at)
            outs.append(bench.step(q[at:at + n], k[at:at + n], v[at:at + n]))
            at, i = at + n, i + 1
        got, want = torch.cat(outs), attn_oracle(q, k, v, H, G, D, Dv, size, P)
        loud = so.rms(v[5:6].double(), 1e-6)[0]
        cos = lambda a: float(torch.dot(a.double(), loud) / a.double().norm() / loud.norm())
        assert cos(want[36]) > 0.99 and abs(cos(want[37])) < 0.3 and abs(cos(want[38])) < 0.3
        assert cos(want[39]) > 0.9 and cos(want[299]) > 0.9 and cos(got[39]) > 0.9 and abs(cos(got[38])) < 0.3
        assert U.rel(got, want) < 2e-5


def test_attention_kernels_in_bf16():
    H, G, D, Dv, size, P, T = 4, 2, 32, 32, 20, 4, 120
    g = torch.Generator().manual_seed(2)
    q, k, v = torch.randn(T, H * D, generator=g), torch.randn(T, G * D, generator=g), torch.randn(T, G * Dv, generator=g)
    bench = AttnBench(H, G, D, Dv, size, P, dtype=torch.bfloat16)
    got = torch.cat([bench.step(q[:50], k[:50], v[:50])] + [bench.step(q[t:t + 1], k[t:t + 1], v[t:t + 1]) for t in range(50, T)])
    r = lambda x: x.bfloat16().float()
    assert U.rel(got, attn_oracle(r(q), r(k), r(v), H, G, D, Dv, size, P)) < 3e-2


@pytest.mark.parametrize("sizes", [[200], [17, 2, 64, 1, 1, 33, 16, 5], [3]], ids=["whole", "mixed", "threes"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("shape", [(8, 2, 128, 128, 48, 8), (4, 4, 64, 128, 20, 1), (6, 1, 128, 64, 0, 0), (2, 1, 64, 64, 70, 16),
                                   (5, 5, 128, 128, 1, 3)], ids=lambda s: "x".join(map(str, s)))
def test_matrix_core_attention_against_the_vector_kernel(shape, dtype, sizes):
    """portions of prompts in 16-bit types run on the matrix cores (16 tokens x one key/value head per workgroup, masks per
    key and query over the tile's union of keys): same cache, same portions, against the fp32 vector kernel, which the
    tests above pin to the oracle.  Peaked softmaxes, so a wrong mask shows; the bar is a few roundings of the output."""
    H, G, D, Dv, size, P = shape
    g = torch.Generator().manual_seed(7)
    T = 200
    q, k, v = torch.randn(T, H * D, generator=g) * 0.7, torch.randn(T, G * D, generator=g) * 0.7, torch.randn(T, G * Dv, generator=g)
    rot = {"dims": D // 2, "base": 100.0}
    outs = []
    for matrix in (True, False):
        bench = AttnBench(H, G, D, Dv, size, P, rot, dtype=dtype, matrix=matrix)
        got, at, i = [], 0, 0
        while at < T:
            n = min(sizes[min(i, len(sizes) - 1)], T - at)
            got.append(bench.step(q[at:at + n], k[at:at + n], v[at:at + n]))
            at, i = at + n, i + 1
        outs.append(torch.cat(got))
    assert torch.isfinite(outs[0]).all()
    assert U.rel(outs[0], outs[1]) < (1.2e-2 if dtype == torch.bfloat16 else 2e-3)


# ------------------------------------------------------------------------------------------------ the whole model
@pytest.fixture(scope="module")
def full(tmp_path_factory):
    cfg = U.full_config()
    folder, w = U.make_model(tmp_path_factory.mktemp("full"), cfg, seed=11)
    toks = U.tokens(130, cfg["vocab"], 12)
    lay = []
    want = so.forward(toks, w, cfg, lay)
    return cfg, folder, w, toks, want, lay


def test_whole_prompt_and_every_layer(full):
    cfg, folder, w, toks, want, lay = full
    eng = engine(folder)
    eng.runner.model.capture_layers = []
    got = run_whole(eng, toks)
    for i, (a, b) in enumerate(zip(eng.runner.model.capture_layers, lay)):
        assert U.rel(a, b) < F32_BAR, f"layer {i} ({cfg['layers'][i]['type']})"
    assert U.rel(got, want) < F32_BAR


def test_bf16_serving_precision(full):
    cfg, folder, w, toks, want, _ = full
    got = run_portions(engine(folder, dtype=torch.bfloat16), toks, [40, 1]).double().cpu()
    # per position: rms of the deviation over the vocabulary against the rms of the logits.  16-bit rounding may flip a
    # close expert choice at a position, so the bar is on the bulk of the positions, with a cap on the rest.
    err = ((got - want) ** 2).mean(-1).sqrt() / (want ** 2).mean(-1).sqrt()
    assert float(err.median()) < 0.03 and float((err > 0.15).double().mean()) <= 0.05 and float(err.max()) < 0.6, err


def test_bf16_model_whose_prompts_take_the_matrix_core_attention(tmp_path):
    """heads of 64 and 128 in bf16: portions of prompts run the matrix-core kernel, single tokens the vector kernel; both
    against the oracle, and the two ways of feeding the same prompt against each other"""
    cfg = U.config([(U.attention(4, 2, 64, 128, size=24, pool=8, dims=32), U.dense(96)),
                    (U.attention(2, 1, 128, 64, size=40, pool=5), None)], width=128)
    folder, w = U.make_model(tmp_path, cfg, seed=9)
    toks = U.tokens(150, cfg["vocab"], 2)
    want = so.forward(toks, w, cfg)
    outs = [run_portions(engine(folder, dtype=torch.bfloat16), toks, sizes).double().cpu() for sizes in ([150], [33, 1], [1])]
    for got in outs:
        err = ((got - want) ** 2).mean(-1).sqrt() / (want ** 2).mean(-1).sqrt()
        assert float(err.median()) < 0.03 and float(err.max()) < 0.15, err
    assert U.rel(outs[0], outs[2]) < 0.1 and U.rel(outs[1], outs[2]) < 0.1


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_decoding_token_by_token_from_the_first_token(full, graphs):
    """130 single-token steps: every window (7 and 10 tokens) and block passes over decoded tokens many times"""
    cfg, folder, w, toks, want, _ = full
    assert U.rel(run_portions(engine(folder, graphs=graphs), toks, [1]), want) < F32_BAR


@pytest.mark.parametrize("sizes", [[2], [3, 2, 17, 1, 1, 64, 5, 1], [64, 2, 1], [9, 10, 11, 12, 13]],
                         ids=["pairs", "mixed", "big-then-small", "near-window"])
def test_portions_of_prompts(full, sizes):
    cfg, folder, w, toks, want, _ = full
    assert U.rel(run_portions(engine(folder), toks, sizes), want) < F32_BAR


def test_garbage_in_reused_rows_and_slots_is_never_read(full):
    """every state tensor and cache buffer poisoned before a request starts: a first token must start from the initial
    state and see only its own keys"""
    cfg, folder, w, toks, want, _ = full
    eng = engine(folder)
    sp, kv = eng.runner.state_pool, eng.runner.token_to_kv_pool
    sp.shift.fill_(float("nan"))
    for spec in sp.named.values():
        for t in spec.values():
            t.fill_(float("nan"))
    for b in kv._all():
        b.fill_(float("nan"))
    assert U.rel(run_portions(eng, toks[:60], [7, 1]), want[:60]) < F32_BAR


@pytest.mark.parametrize("graphs", [False, True], ids=["eager", "graphs"])
def test_unequal_batches_with_rows_and_slots_reused(full, graphs):
    """seven requests of unequal length through three rows and a pool that holds far fewer tokens than their sum:
    portions of some beside single tokens of others, pauses, rows and slots handed on; every request's logits must be
    what it gets alone"""
    cfg, folder, w, _, _, _ = full
    reqs = {f"r{i}": U.tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate([45, 3, 70, 1, 26, 58, 12])}
    want = {r: so.forward(t, w, cfg) for r, t in reqs.items()}
    eng = engine(folder, tokens=200, slots=3, graphs=graphs)
    plan = {"r0": [5, 1, 1, 30, 1, 7], "r1": [2, 1], "r2": [33, 2, 1, 1, 1, 1, 1, 30], "r3": [1], "r4": [1, 1, 24],
            "r5": [2, 50, 1, 1, 1, 1, 1, 1], "r6": [6, 1, 1, 1, 1, 1, 1]}
    fed, got, waiting, live, step = {r: 0 for r in reqs}, {r: [] for r in reqs}, list(reqs), [], 0
    while waiting or live:
        while waiting and len(live) < 3 and sum(len(reqs[r]) for r in live) + len(reqs[waiting[0]]) <= 200:
            live.append(waiting.pop(0))
        entries, end = [], []
        for r in live:
            if (step + int(r[1:])) % 5 == 4 and len(live) > 1:
                continue                                           # left out of this step, goes on later
            n = plan[r].pop(0) if plan[r] else 1
            n = min(n, len(reqs[r]) - fed[r])
            entries.append(entry(r, reqs[r][fed[r]:fed[r] + n]))
            fed[r] += n
            if fed[r] == len(reqs[r]):
                end.append(r)
        if entries:
            out = eng.step(entries, end)
            at = 0
            for e in entries:
                got[e.rid].append(out[at:at + len(e.tokens)])
                at += len(e.tokens)
        live = [r for r in live if r not in end]
        step += 1
    for r in reqs:
        assert U.rel(torch.cat(got[r]), want[r]) < F32_BAR, r


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_graph_replay_of_larger_decode_steps(full, dtype):
    """40 requests decoding together: steps above 16 rows take the library's products inside the captured graph.  Every
    replay (six of them, with the eager prompt steps of the other engine and synchronisations between) is compared with
    the same step run eagerly."""
    cfg, folder, w, _, _, _ = full
    reqs = {f"q{i}": U.tokens(3 + i % 9, cfg["vocab"], 300 + i) + U.tokens(6, cfg["vocab"], 900 + i) for i in range(40)}
    outs = []
    for graphs in (True, False):
        eng = engine(folder, dtype=dtype, tokens=900, slots=40, graphs=graphs)
        eng.step([entry(r, t[:-6], []) for r, t in reqs.items()])                     # the prompts, one extend batch
        steps = []
        for k in range(6):
            steps.append(eng.step([entry(r, [t[len(t) - 6 + k]]) for r, t in reqs.items()], list(reqs) if k == 5 else []))
            torch.cuda.synchronize()
        outs.append(torch.stack(steps))
    bar = 1e-5 if dtype == torch.float32 else 3e-2
    for k in range(6):
        assert U.rel(outs[0][k], outs[1][k]) < bar, k
    if dtype == torch.float32:
        want = torch.stack([so.forward(t, w, cfg)[-6:] for t in reqs.values()], 1)    # [step, request, vocab]
        assert U.rel(outs[0], want) < F32_BAR


def test_generation_through_the_scheduler(full):
    """greedy generation of three prompts through Engine.generate (admission, chunked prefill of 16 tokens beside decoding
    requests, release) equals the oracle's greedy continuation; sampled generation runs and stays in the vocabulary"""
    from scratchpad_amd.sampler import SamplingParams
    cfg, folder, w, _, _, _ = full
    prompts = [U.tokens(n, cfg["vocab"], 40 + n) for n in (37, 5, 21)]
    eng = engine(folder, tokens=300, slots=2, graphs=True, chunk=16)
    got = eng.generate(prompts, max_new_tokens=12)
    for p, out in zip(prompts, got):
        ref = U.greedy(p, w, cfg, 12)
        agree = next((i for i, (a, b) in enumerate(zip(out, ref)) if a != b), 12)
        if agree < 12:      # a near-tie in fp32 against float64 may flip one choice: the logits there must be that close
            lg = so.forward(p + ref[:agree], w, cfg)[-1]
            assert float(lg[ref[agree]] - lg[out[agree]]) < 1e-3 * float(lg.abs().max()), (agree, out, ref)
        else:
            assert out == ref
    sampled = eng.generate(prompts[:2], SamplingParams(max_new_tokens=6, temperature=0.8, top_p=0.9, top_k=20))
    assert all(len(o) == 6 and all(0 <= t < cfg["vocab"] for t in o) for o in sampled)


@pytest.mark.parametrize("seed", range(10))
def test_designs_drawn_at_random(tmp_path, seed):
    """layer order, sizes and constants drawn at random (sominex_util.random_config): whole prompt, then portions of
    random sizes with single tokens between them, both against the oracle"""
    import random
    cfg = U.random_config(100 + seed)
    folder, w = U.make_model(tmp_path, cfg, seed=seed)
    toks = U.tokens(90, cfg["vocab"], seed)
    want = so.forward(toks, w, cfg)
    assert U.rel(run_whole(engine(folder), toks), want) < F32_BAR, cfg
    r = random.Random(seed)
    sizes = [r.choice([1, 1, 2, 3, 7, 16, 29]) for _ in range(40)]
    assert U.rel(run_portions(engine(folder), toks, sizes), want) < F32_BAR, (sizes, cfg)


def test_sizes_that_are_one_or_equal(tmp_path):
    """a second model whose sizes are 1 or equal where the first one's differ: one head everywhere, key width = value
    width = state size, one expert of which one is chosen, one norm group, a block as long as the window"""
    cfg = U.config([
        (U.attention(1, 1, 16, 16, size=4, pool=4, dims=16), U.moe(1, 1, 16, scale=1.0)),
        (U.mamba2(1, 16, 16, groups=1, conv=1, norm_groups=1), U.dense(16, limit=5.0)),
        (U.mlstm(1, 16, 16, cap=1.0), U.moe(2, 2, 8, scale=1.0, shared=8)),
    ], width=16, vocab=17, scale=1.0)
    folder, w = U.make_model(tmp_path, cfg, seed=4)
    toks = U.tokens(50, 17, 3)
    want = so.forward(toks, w, cfg)
    assert U.rel(run_whole(engine(folder), toks), want) < F32_BAR
    assert U.rel(run_portions(engine(folder), toks, [3, 1]), want) < F32_BAR
