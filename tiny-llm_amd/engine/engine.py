"""The Python entry point: a model, its cache, the scheduler and the sampler behind
`generate(prompt_token_ids, SamplingParams) -> token ids`.

It stands where the reference's `Pipeline` stands (tiny_llm/pipeline/pipeline.hpp:14-29:
constructor from a model folder and a config, `apply(prompts, max_new_tokens, do_sample,
temperature, top_k, top_p)`), with token ids instead of text on both sides; text is the
command line's business.
"""
from __future__ import annotations

import itertools
from typing import Callable, Dict, Hashable, Iterator, List, Mapping, Optional, Sequence, Tuple, Union

from ..config import EngineConfig
from ..sampling import SamplingParams
from .loading import build_runner, load_model, random_model
from .scheduler import Request, Scheduler
from .step import SampleSpec, StepEntry


class Engine:
    # Finished requests stay in `requests` (their tokens, their finish reason) until their caller
    # has had them: `generate` and `stream` let go of theirs at the end, `release` does it for the
    # caller of `add_request`; beyond this many the oldest finished ones go by themselves.
    FINISHED_KEPT = 4096

    def __init__(self, model_path: Optional[str] = None, *, config: Optional[Mapping] = None,
                 engine_config: Optional[EngineConfig] = None, weights_seed: int = 0,
                 init_std: Optional[float] = None, norm_std: float = 0.0, **engine_kwargs):
        """Either `model_path` (a folder with config.json and safetensors) or `config`
        (config.json keys as a dict: seeded random weights are made on the device)."""
        self.engine_config = engine_config or EngineConfig(**engine_kwargs)
        if (model_path is None) == (config is None):
            raise ValueError("give exactly one of model_path and config")
        if model_path is not None:
            self.model_config, self.decoder = load_model(model_path, self.engine_config)
        else:
            self.model_config, self.decoder = random_model(config, self.engine_config, weights_seed, init_std, norm_std)
        self.runner = build_runner(self.decoder, self.engine_config)
        self.eos_token_ids = tuple(self.decoder.spec.eos_token_ids)
        self.scheduler = Scheduler(self.runner.cache, self.engine_config.max_num_seqs,
                                   self.engine_config.max_num_batched_tokens, self.runner.max_model_len,
                                   self.eos_token_ids)
        self._ids = itertools.count()
        self.requests: Dict[Hashable, Request] = {}
        self.steps_run = 0

    # ---------------------------------------------------------------- requests
    def add_request(self, prompt_token_ids: Sequence[int], params: Optional[SamplingParams] = None,
                    req_id: Optional[Hashable] = None) -> Hashable:
        n = next(self._ids)
        req_id = n if req_id is None else req_id
        if req_id in self.requests and self.requests[req_id].status != "finished":
            raise ValueError(f"request {req_id!r} is already live")
        params = params or SamplingParams()
        vocab = self.decoder.spec.vocab_size
        prompt = [int(t) for t in prompt_token_ids]
        for t in prompt:
            if not (0 <= t < vocab):
                raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        seed = params.seed if params.seed is not None else (self.engine_config.seed * 1000003 + n)
        req = Request(req_id, prompt, params, seed=seed)
        if params.max_new_tokens == 0:
            req.status, req.finish_reason = "finished", "length"
            self.requests[req_id] = req
            return req_id
        self.scheduler.add(req)
        self.requests[req_id] = req
        if len(self.requests) > self.FINISHED_KEPT:
            for old in [k for k, r in self.requests.items() if r.status == "finished"][:len(self.requests) - self.FINISHED_KEPT]:
                del self.requests[old]
        return req_id

    def release(self, req_id: Hashable) -> Optional[Request]:
        """Forgets a finished request (the caller has its tokens) and returns it; a live one stays."""
        r = self.requests.get(req_id)
        if r is None or r.status != "finished":
            return None
        return self.requests.pop(req_id)

    def abort(self, req_id: Hashable) -> None:
        self.scheduler.abort(req_id)

    def has_unfinished(self) -> bool:
        return self.scheduler.has_work()

    # -------------------------------------------------------------------- step
    def step(self, max_decode_steps: Optional[int] = None) -> List[Request]:
        """One scheduler decision and one forward pass with the sampler at its end, or, where every
        request decodes and nothing has to be decided for a while, a run of up to `decode_burst`
        such steps that the device chains by itself (`max_decode_steps` bounds the run for this
        call).  Returns the requests that finished."""
        plan = self.scheduler.schedule()
        done = list(plan.finished)
        if not plan.entries:
            return done
        entries, rows, samples = [], [], []
        for e in plan.entries:
            r = e.request
            entries.append(StepEntry(r.req_id, r.token_slice(e.start, e.count), [e.count - 1] if e.samples else []))
            if e.samples:
                p = r.params
                rows.append(r)
                samples.append(SampleSpec(p.temperature if p.do_sample else 0.0, p.top_k, p.top_p, r.seed, r.num_tokens))
        if self.engine_config.use_graphs and self.engine_config.decode_burst > 1:
            # a run of decode steps without the host in between, where nothing has to be decided
            most = self.engine_config.decode_burst
            if max_decode_steps is not None:
                most = max(1, min(most, max_decode_steps))
            k = self.scheduler.burst_length(plan, most)
            by_step = self.runner.run_burst(entries, samples, k) if k > 1 else None
            if by_step is not None:
                done += self.scheduler.update_burst(plan, by_step)
                self.steps_run += k
                return done
        toks = self.runner.run(entries, samples, use_graph=self.engine_config.use_graphs)
        done += self.scheduler.update(plan, {r.req_id: t for r, t in zip(rows, toks)})
        self.steps_run += 1
        return done

    # ---------------------------------------------------------------- generate
    def stream(self, prompt_token_ids: Sequence[Sequence[int]],
               params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
               max_decode_steps: Optional[int] = None) -> Iterator[Tuple[int, List[int], Optional[str]]]:
        """Generates for every prompt and yields `(index of the prompt, its new token ids, finish
        reason or None)` after each step that gave that prompt tokens, in the order of the prompts.
        A run of chained decode steps hands over all its tokens at once; `max_decode_steps` bounds
        such a run (1: a token at a time).  A request preempted for want of pages yields nothing
        twice: what it had generated is kept and recomputed, not sampled again."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompt_token_ids)
        ids = [self.add_request(p, sp) for p, sp in zip(prompt_token_ids, params)]
        told = [0] * len(ids)
        closed = [False] * len(ids)
        while True:
            for i, rid in enumerate(ids):
                r = self.requests[rid]
                fresh = list(r.output[told[i]:])
                ended = r.status == "finished" and not closed[i]
                if fresh or ended:
                    told[i] += len(fresh)
                    closed[i] = closed[i] or ended
                    yield i, fresh, (r.finish_reason if ended else None)
            if not self.scheduler.has_work():
                for rid in ids:
                    self.release(rid)
                return
            self.step(max_decode_steps)

    def generate(self, prompt_token_ids: Sequence[Sequence[int]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 on_tokens: Optional[Callable[[int, List[int], Optional[str]], None]] = None) -> List[List[int]]:
        """Generated token ids of every prompt (eos, when it ends a request, is part of them,
        as in tiny_llm/pipeline/pipeline.cpp:216-223).  `on_tokens(index, new ids, finish reason
        or None)` is called as tokens arrive (what `stream` yields)."""
        out: List[List[int]] = [[] for _ in prompt_token_ids]
        for i, fresh, reason in self.stream(prompt_token_ids, params):
            out[i] += fresh
            if on_tokens is not None:
                on_tokens(i, fresh, reason)
        return out
