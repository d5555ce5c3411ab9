"""The generation loop above the step function (tools/infer.cpp:267-324, widened from
one sequence to batches): prompts of unequal length in one step, then one token for
each live sequence; a sequence ends at a stop token (which is not kept), at its
token budget, or at the model's last position; as many batches one after another as
the requests need."""
from __future__ import annotations

import time
from dataclasses import dataclass, field

import torch

from ..cache import PAGE
from ..sampling import Sampler


class RequestError(ValueError):
    pass


def per_request(value, n: int, what: str = "max_new_tokens") -> list:
    """One number for every request, or a list with one for each."""
    if isinstance(value, (list, tuple)):
        if len(value) != n:
            raise RequestError(f"{what}: {len(value)} values for {n} requests")
        return [int(v) for v in value]
    return [int(value)] * n


def plan_batches(prompt_lens, max_new_tokens, max_batch: int, capacity_tokens: int, max_positions: int):
    """Cuts the requests, in their order, into batches that fit the slots and the cache.
    A request holds room for its prompt and all it may generate (``max_new_tokens``: one number, or one for
    each request), rounded up to whole pages."""
    batches, cur, used = [], [], 0
    budget = per_request(max_new_tokens, len(prompt_lens))
    for i, n in enumerate(prompt_lens):
        if n <= 0:
            raise RequestError(f"request {i} has an empty prompt")
        if n >= max_positions:
            # tools/infer.cpp:262-265
            raise RequestError(f"Prompt too long: {n} tokens (max: {max_positions})")
        need = -(-min(n + budget[i], max_positions) // PAGE) * PAGE
        if need > capacity_tokens:
            raise RequestError(f"request {i} needs room for {need} tokens, the cache holds {capacity_tokens}")
        if cur and (len(cur) >= max_batch or used + need > capacity_tokens):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


class BatchTracker:
    """The loop's decisions for one batch, free of any device work.

    ``accept(live, sampled)`` takes the tokens sampled for the live requests and returns the
    requests that go on, i.e. whose new token is to be run (tools/infer.cpp:289-324: sample,
    stop check before the token is kept, append, forward unless it was the last).
    """

    def __init__(self, prompt_lens, max_new_tokens, stop_token_ids, max_positions):
        self.prompt_lens = list(prompt_lens)
        self.max_new = per_request(max_new_tokens, len(self.prompt_lens))     # a budget for each request
        self.stop, self.max_positions = set(stop_token_ids or ()), max_positions
        self.outputs = [[] for _ in prompt_lens]
        self.finished = [m <= 0 for m in self.max_new]
        self.reason = ["length" if f else None for f in self.finished]

    def live(self):
        return [i for i, f in enumerate(self.finished) if not f]

    def will_go_on(self, live) -> bool:
        """True if every live request goes on after its next token unless that is a stop token."""
        return all(len(self.outputs[i]) + 1 < self.max_new[i] and
                   self.prompt_lens[i] + len(self.outputs[i]) + 1 <= self.max_positions for i in live)

    def accept(self, live, sampled):
        go_on = []
        for i, t in zip(live, sampled):
            if self.finished[i]:
                raise RuntimeError(f"request {i} had finished")
            if t in self.stop:
                self.finished[i], self.reason[i] = True, "stop"
                continue
            self.outputs[i].append(int(t))
            if len(self.outputs[i]) >= self.max_new[i]:
                self.finished[i], self.reason[i] = True, "length"
            elif self.prompt_lens[i] + len(self.outputs[i]) > self.max_positions:
                self.finished[i], self.reason[i] = True, "context"
            else:
                go_on.append(i)
        return go_on


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    generated_tokens: int = 0
    prefill_s: float = 0.0
    decode_s: float = 0.0
    batches: int = 0
    finish_reasons: list = field(default_factory=list)


def generate(engine, prompts, max_new_tokens=256, temperature: float = 1.0, seed: int = 0,
             stop_token_ids=None, max_batch: int | None = None, return_stats: bool = False,
             use_graph: bool = True):
    """Generates for every prompt (a list of token ids); returns the new tokens of each, in order.
    ``max_new_tokens``: one budget for all requests, or a list with one for each."""
    if stop_token_ids is None:
        stop_token_ids = engine.model.spec.stop_token_ids
    cache = engine.cache
    max_batch = min(max_batch or cache.n_slots, cache.n_slots)
    for i, p in enumerate(prompts):
        if len(p) and (min(p) < 0 or max(p) >= engine.vocab_size):
            raise RequestError(f"request {i}: token id outside [0, {engine.vocab_size})")
    capacity = (cache.n_pages - 1) * PAGE
    max_new_tokens = per_request(max_new_tokens, len(prompts))
    batches = plan_batches([len(p) for p in prompts], max_new_tokens, max_batch, capacity, engine.max_positions)
    sampler = Sampler(temperature, seed)
    outputs = [None] * len(prompts)
    stats = GenerationStats(finish_reasons=[None] * len(prompts))
    for batch in batches:
        slots = []
        try:
            for _ in batch:                      # inside the try: a slot that cannot be had leaks none of the others
                slots.append(engine.alloc_slot())
            tracker = BatchTracker([len(prompts[r]) for r in batch], [max_new_tokens[r] for r in batch],
                                   stop_token_ids, engine.max_positions)
            sampler.start(cache, slots, batch)
            live = tracker.live()
            if live:
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                logits = engine.step(slots, [list(prompts[r]) for r in batch])
                slot_dev = torch.tensor(slots, dtype=torch.int32, device=engine.device)
                sampled = sampler.sample(logits, slot_dev, cache).tolist()
                stats.prefill_s += time.perf_counter() - t0
                stats.prompt_tokens += sum(len(prompts[r]) for r in batch)
                t0 = time.perf_counter()
                live = tracker.accept(live, sampled)
                runner = engine.decode_runner(sampler, use_graph)
                while live:
                    new = [tracker.outputs[i][-1] for i in live]
                    sampled = runner.run([slots[i] for i in live], new, may_follow=tracker.will_go_on(live))
                    live = tracker.accept(live, sampled)
                runner.drain()
                torch.cuda.synchronize()
                stats.decode_s += time.perf_counter() - t0
            for j, r in enumerate(batch):
                outputs[r] = tracker.outputs[j]
                stats.finish_reasons[r] = tracker.reason[j]
                stats.generated_tokens += len(tracker.outputs[j])
        finally:
            for s in slots:
                engine.free_slot(s)
        stats.batches += 1
    return (outputs, stats) if return_stats else outputs
