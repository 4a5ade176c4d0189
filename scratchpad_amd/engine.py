"""Engine: a model from a checkpoint folder behind the framework's own runner, pools, scheduler batches and sampler.

Two ways in, one step function (``run_step``):
* ``generate(prompts, sampling_params)`` - continuous batching with chunked prefill: waiting requests are admitted while
  request rows and cache slots last, their prompts are cut into portions of at most ``chunk_size`` tokens, and running
  requests decode one token per step beside them;
* ``step(entries)`` - an explicit schedule (trace replay, prompt scoring): the caller says which request gets which next
  tokens in this step and of which rows it wants the logits.

A step whose rows are all single tokens of running requests is a DECODE batch (``ScheduleBatch.prepare_for_decode``, the
HIP-graph path when graphs are on); any other step is an extend batch in which every request brings its next tokens on
top of what it already holds in the cache (``prepare_for_extend`` with the request's own slots as its prefix).  Requests
keep their row of the request table - and with it their state slot - until they finish; a finished request's row and
cache slots go back to the pools at once."""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

from . import registry
from .forward_info import ForwardMode
from .model_runner import ModelRunner, ServerArgs, TpModelWorker
from .radix_cache import ChunkCache
from .sampler import SamplingBatchInfo, SamplingParams
from .schedule_batch import Req, ScheduleBatch


@dataclass
class StepEntry:
    rid: str
    tokens: List[int]
    want: List[int] = field(default_factory=list)     # indices into `tokens` whose logits are returned


class Engine:
    def __init__(self, model_dir: str, dtype: torch.dtype = torch.bfloat16, max_total_tokens: Optional[int] = None,
                 max_running_requests: int = 64, context_len: Optional[int] = None, chunk_size: int = 2048,
                 use_graphs: bool = True, gpu_id: int = 0, kv_cache_dtype: str = "auto"):
        if dtype == torch.float32:
            torch.backends.cuda.matmul.allow_tf32 = False          # true 32-bit products
            torch.backends.cudnn.allow_tf32 = False
        if context_len is None:
            context_len = max_total_tokens or 8192
        self.config = registry.load_config(model_dir, context_len=context_len)
        args = ServerArgs(max_total_tokens=max_total_tokens, max_running_requests=max_running_requests,
                          disable_cuda_graph=not use_graphs, cuda_graph_max_bs=min(max_running_requests, 256),
                          kv_cache_dtype=kv_cache_dtype)
        self.runner = ModelRunner(self.config, args, dtype=dtype, gpu_id=gpu_id, init_weights=False)
        registry.load_weights(self.runner.model, model_dir)
        self.worker = TpModelWorker(self.runner)
        self.device = self.runner.device
        self.chunk_size = chunk_size
        self.req_pool, self.kv_alloc = self.worker.get_memory_pool()
        self.cache = ChunkCache(self.req_pool, token_to_kv_pool_allocator=self.kv_alloc)
        self.live: Dict[str, Req] = {}
        if use_graphs:
            self.runner.init_cuda_graphs()

    # ------------------------------------------------------------------------------------------------ one step
    def run_step(self, parts: Sequence, logit_rows: Optional[List[int]] = None):
        """parts: (Req, next tokens) per request of the step.  Returns (LogitsProcessorOutput, ScheduleBatch): one
        logits row per request (its last token), or exactly ``logit_rows`` (indices into the step's token rows)."""
        reqs = [r for r, _ in parts]
        decode = all(len(t) == 1 and r.seqlen > 0 and r.req_pool_idx is not None for r, t in parts)
        for r, toks in parts:
            r.step_prefix = r.seqlen                       # tokens held before this step
            r.origin_input_ids = list(r.origin_input_ids) + [int(t) for t in toks]
        batch = ScheduleBatch(reqs, self.req_pool, self.kv_alloc, tree_cache=self.cache, model_config=self.config,
                              device=self.device)
        if any(r.sampling_params is not None for r in reqs):          # (None = every request greedy)
            batch.sampling_info = SamplingBatchInfo.from_schedule_batch(batch, self.config.vocab_size)
        if decode:
            batch.req_pool_indices = torch.tensor([r.req_pool_idx for r in reqs], dtype=torch.int64).to(self.device)
            lens = [r.step_prefix for r in reqs]
            batch.seq_lens = torch.tensor(lens, dtype=torch.int64).to(self.device)
            batch.seq_lens_sum = sum(lens)
            batch.output_ids = torch.tensor([t[0] for _, t in parts], dtype=torch.int64).to(self.device)
            batch.prepare_for_decode()
        else:
            for r in reqs:
                r.fill_ids = list(r.origin_input_ids)
            batch.prepare_for_extend()
            if any(r.step_prefix > 0 and len(t) == 1 for r, t in parts) and any(len(t) > 1 for _, t in parts):
                batch.forward_mode = ForwardMode.MIXED
        mwb = batch.get_model_worker_batch()
        if logit_rows is not None and not decode:
            mwb.logit_rows = torch.tensor(logit_rows, dtype=torch.int64)
        out, _ = self.worker.forward_batch_generation(mwb, skip_sample=True)
        if logit_rows is not None and decode and logit_rows != list(range(len(reqs))):
            full = out.next_token_logits
            out = type(out)(next_token_logits=full[torch.tensor(logit_rows, dtype=torch.int64, device=full.device)],
                            vocab_size=out.vocab_size)
        for r in reqs:
            r.keeps_pool_row = True
            self.cache.cache_unfinished_req(r, token_ids=r.origin_input_ids)       # its own slots = next step's prefix
        return out, batch

    def release(self, req: Req) -> None:
        """give the request's table row (its state slot) and cache slots back"""
        self.cache.cache_finished_req(req, token_ids=req.origin_input_ids)
        req.keeps_pool_row, req.req_pool_idx = False, None
        self.live.pop(req.rid, None)

    # ------------------------------------------------------------------------------------------------ explicit schedule
    def step(self, entries: Sequence[StepEntry], end: Sequence[str] = ()) -> Optional[torch.Tensor]:
        """Run the entries as ONE batch; returns the logits [wanted rows, vocab] fp32 in entry / want order (None if no
        row is wanted).  A request is admitted at its first entry; ``end`` names those that finish with this step."""
        parts, rows, at = [], [], 0
        for e in entries:
            req = self.live.get(e.rid)
            if req is None:
                req = self.live[e.rid] = Req(e.rid, "", [], None)
            parts.append((req, list(e.tokens)))
            rows += [at + i for i in e.want]
            at += len(e.tokens)
        logits = None
        if parts:
            out, _ = self.run_step(parts, logit_rows=rows if rows else [0])
            if rows:
                logits = out.next_token_logits.clone()      # (a graph replay's output lives in the graph's own buffer)
        for rid in end:
            if rid in self.live:
                self.release(self.live[rid])
        return logits

    # ------------------------------------------------------------------------------------------------ generation
    def generate(self, prompts: Sequence[Sequence[int]], sampling_params=None, max_new_tokens: int = 16) -> List[List[int]]:
        """token ids generated for every prompt (greedy unless sampling_params - one, or one per prompt - say otherwise)"""
        if sampling_params is None or isinstance(sampling_params, SamplingParams):
            sampling_params = [sampling_params] * len(prompts)
        waiting = []
        for i, (p, sp) in enumerate(zip(prompts, sampling_params)):
            req = Req(f"g{i}", "", [], sp)
            req.prompt, req.fed, req.limit = [int(t) for t in p], 0, (sp.max_new_tokens if sp is not None else max_new_tokens)
            if not req.prompt:
                raise ValueError("empty prompt")
            waiting.append(req)
        order = list(waiting)
        running: List[Req] = []
        while waiting or running:
            # admit while a table row is free and the prompt plus its generation fits the cache beside the running ones
            reserved = sum(len(r.prompt) + r.limit for r in running)
            rows_free = self.req_pool.available_size() - sum(r.req_pool_idx is None for r in running)
            while waiting and rows_free > 0 and len(running) < self.runner.max_running_requests \
                    and reserved + len(waiting[0].prompt) + waiting[0].limit <= self.kv_alloc.size:
                rows_free -= 1
                req = waiting.pop(0)
                reserved += len(req.prompt) + req.limit
                self.live[req.rid] = req
                running.append(req)
            if not running:
                raise RuntimeError("a prompt does not fit the cache pool")
            parts, budget = [], self.chunk_size
            for r in running:
                if r.fed < len(r.prompt):                      # a portion of its prompt
                    n = min(len(r.prompt) - r.fed, max(budget, 1))
                    parts.append((r, r.prompt[r.fed:r.fed + n]))
                    r.fed += n
                    budget -= n
                else:
                    parts.append((r, [r.output_ids_pending]))
            # only requests whose prompt is complete after this step sample a token
            out, batch = self.run_step(parts)
            next_ids = self._sample(out, batch).tolist()
            for (r, _), tok in zip(parts, next_ids):
                if r.fed < len(r.prompt):
                    continue
                r.output_ids_pending = tok
                r.generated = getattr(r, "generated", []) + [tok]
                stop = set(getattr(r.sampling_params, "stop_token_ids", None) or ())
                if len(r.generated) >= r.limit or tok in stop:
                    running.remove(r)
                    self.release(r)
        return [getattr(r, "generated", []) for r in order]

    def _sample(self, out, batch: ScheduleBatch) -> torch.Tensor:
        if batch.sampling_info is None:
            return out.greedy_token_ids()
        return self.runner.sampler(out, batch.sampling_info, False, None, None)


def main(argv=None) -> int:
    """python -m scratchpad_amd.engine --model DIR --prompt 5,17,3 [--prompt ...] [--max-new-tokens N] [--temperature T ...]"""
    import argparse
    ap = argparse.ArgumentParser(description="generate token ids from prompts of token ids")
    ap.add_argument("--model", required=True, help="folder with config.json and *.safetensors")
    ap.add_argument("--prompt", action="append", required=True, help="comma-separated token ids (repeatable)")
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--max-new-tokens", type=int, default=16)
    ap.add_argument("--max-tokens", type=int, default=8192, help="cache slots for all live requests together")
    ap.add_argument("--slots", type=int, default=8, help="requests live at the same time")
    ap.add_argument("--chunk", type=int, default=2048, help="prompt tokens per step")
    ap.add_argument("--temperature", type=float, default=0.0)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--no-graphs", action="store_true")
    a = ap.parse_args(argv)
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in a.prompt]
    eng = Engine(a.model, dtype=getattr(torch, a.dtype), max_total_tokens=a.max_tokens, max_running_requests=a.slots,
                 chunk_size=a.chunk, use_graphs=not a.no_graphs)
    params = None
    if a.temperature > 0:
        params = SamplingParams(max_new_tokens=a.max_new_tokens, temperature=a.temperature, top_p=a.top_p, top_k=a.top_k)
    for p, out in zip(prompts, eng.generate(prompts, params, max_new_tokens=a.max_new_tokens)):
        print(",".join(map(str, p)), "->", ",".join(map(str, out)), flush=True)
    return 0


if __name__ == "__main__":
    import sys
    sys.exit(main())
