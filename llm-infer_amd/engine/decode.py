"""Decoding one token for each live sequence, step after step.

The plain runner calls the engine's step function.  The graph runner records the
same work (bookkeeping kernel, the model's forward pass, sampling) once for each
batch size into a HIP graph and replays it, so that a step costs one launch
instead of some hundred; positions and context lengths are advanced on the device,
and the sampled tokens are fed back without leaving it.  The reference replays a
CUDA graph per token in the same spirit (src/model/model.cu:11-22).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .step import decode_splits


class PlainDecodeRunner:
    def __init__(self, engine, sampler):
        self.engine, self.sampler = engine, sampler

    def run(self, slots, tokens):
        logits = self.engine.step(slots, [[t] for t in tokens])
        slot_dev = torch.tensor(slots, dtype=torch.int32, device=self.engine.device)
        return self.sampler.sample(logits, slot_dev, self.engine.cache).tolist()


class _GraphContext:
    """The step description of a recorded decode step: fixed device buffers."""
    is_decode = True

    def __init__(self, bufs, n, splits):
        self.n_seqs = self.n_tokens = self.n_want = n
        self.token_ids, self.pos, self.seq_ctx = bufs["tokens"][:n], bufs["pos"][:n], bufs["ctx"][:n]
        self.tok_slot = self.seq_slot = bufs["slots"][:n]
        self.want_rows = bufs["rows"][:n]
        self._splits = splits

    def decode_splits(self, n_kv_heads, n_heads):
        return self._splits

    def prefill_meta(self):
        raise RuntimeError("a recorded decode step has no prompt")


class GraphDecodeRunner:
    """Replays a recorded step while the set of live sequences stays the same; when it
    changes, the slots and tokens are uploaded anew and the graph of the new size is used.
    A step is run eagerly the first time its (batch size, split) is seen and recorded the
    second time."""

    def __init__(self, engine, sampler):
        self.engine, self.sampler = engine, sampler
        cache = engine.cache
        n = cache.n_slots
        dev = engine.device
        self.bufs = engine._graph_bufs
        if self.bufs is None:
            self.bufs = {k: torch.zeros((n,), dtype=torch.int32, device=dev)
                         for k in ("tokens", "slots", "pos", "ctx", "next")}
            self.bufs["rows"] = torch.arange(n, dtype=torch.int32, device=dev)
            engine._graph_bufs = self.bufs
        self.current = None            # the slots now in the buffers

    def _splits(self, n, max_ctx):
        spec = None
        for s in self.engine.model.cache_specs():
            if s is not None and hasattr(s, "n_kv_heads"):
                spec = s
                break
        if spec is None:
            return 1
        mixer = self.engine.model.layers[0].mixer
        n_heads = getattr(mixer, "n_heads", spec.n_kv_heads)
        return decode_splits(n, spec.n_kv_heads, n_heads, max_ctx)

    def _body(self, n, splits):
        eng, b = self.engine, self.bufs
        ops.decode_prepare(b["slots"], eng.cache.lens_dev, b["pos"], b["ctx"], n)
        ctx = _GraphContext(b, n, splits)
        logits = eng.model.forward(ctx, eng.cache)
        self.sampler.sample(logits, b["slots"][:n], eng.cache, out=b["next"])
        b["tokens"][:n].copy_(b["next"][:n])

    def run(self, slots, tokens):
        eng, cache, b = self.engine, self.engine.cache, self.bufs
        n = len(slots)
        new_lens = [cache.lens[s] + 1 for s in slots]
        cache.grow(slots, new_lens, sync_lens=False)
        if self.current != list(slots):
            b["slots"][:n].copy_(torch.tensor(slots, dtype=torch.int32))
            b["tokens"][:n].copy_(torch.tensor(tokens, dtype=torch.int32))
            self.current = list(slots)
        splits = self._splits(n, max(new_lens))
        key = (n, splits, self.sampler.temperature > 0.0, self.sampler.temperature)
        entry = eng._graphs.get(key)
        if entry is None:
            self._body(n, splits)
            eng._graphs[key] = "seen"
        else:
            if entry == "seen":
                g = torch.cuda.CUDAGraph()
                torch.cuda.synchronize()
                with torch.cuda.graph(g):
                    self._body(n, splits)
                eng._graphs[key] = entry = g
            entry.replay()
        out = b["next"][:n].tolist()
        cache.trim_windows(slots)
        return out
