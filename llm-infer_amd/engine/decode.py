"""Decoding one token for each live sequence, step after step.

The plain runner calls the engine's step function.  The graph runner records the
same work (bookkeeping kernel, the model's forward pass, sampling) once for each
batch size into a HIP graph and replays it, so that a step costs one launch
instead of some hundred; positions and context lengths are advanced on the device,
and the sampled tokens are fed back without leaving it.  The reference replays a
CUDA graph per token in the same spirit (src/model/model.cu:11-22).
"""
from __future__ import annotations

import contextlib
import gc

import torch

from ..kernels import ops
from ..tensor import Tensor
from .step import StepShared, decode_splits, split_bucket


@contextlib.contextmanager
def recording(graph):
    """What runs inside is recorded into ``graph`` (a HIP graph) instead of being run.  The garbage collector
    is kept off meanwhile: an object that it frees in the middle of a recording (the recorded steps of an engine
    that is no longer used, say) calls into the runtime, which refuses such calls while a stream is being
    recorded, and the process ends.  (It is not run beforehand either: a full collection takes 25 to 60 ms with
    this many objects alive, several times the recording itself.)"""
    torch.cuda.synchronize()
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            yield
    finally:
        if was_enabled:
            gc.enable()


class PlainDecodeRunner:
    def __init__(self, engine, sampler):
        self.engine, self.sampler = engine, sampler

    def run(self, slots, tokens, may_follow: bool = False):
        logits = self.engine.step(slots, [[t] for t in tokens])
        slot_dev = torch.tensor(slots, dtype=torch.int32, device=self.engine.device)
        return self.sampler.sample(logits, slot_dev, self.engine.cache).tolist()

    def drain(self):
        pass


class _GraphContext(StepShared):
    """The step description of a recorded decode step: fixed device buffers.  The lengths of the
    sequences are known to it only as a bucket (``split_bucket``), which is what the split count of a
    decode attention depends on."""
    is_decode = True

    def __init__(self, bufs, n, bucket):
        self.n_seqs = self.n_tokens = self.n_want = n
        self.token_ids, self.pos, self.seq_ctx = bufs["tokens"][:n], bufs["pos"][:n], bufs["ctx"][:n]
        self.tok_slot = self.seq_slot = bufs["slots"][:n]
        self.want_rows = bufs["rows"][:n]
        self.device = self.token_ids.device
        self._bucket = bucket

    def decode_splits(self, n_kv_heads, n_heads):
        return decode_splits(self.n_seqs, n_kv_heads, n_heads, self._bucket)


MAX_RECORDED_STEPS = 48        # recorded steps an engine keeps; the least recently used goes first


def batch_bucket(n: int, limit: int) -> int:
    """The number of rows a recorded step runs for ``n`` live sequences: the next of 1, 2, 4, 8, 12, 16, 24,
    32, 48, 64, 96, ... (powers of two and the sizes half-way between them), at most ``limit``; the rows beyond
    ``n`` are idle rows on the cache's scratch slot.  A batch that shrinks from 64 sequences to 1 so meets ten
    sizes instead of 64, each of them often enough to be worth recording."""
    b = 1
    while b < n:
        b = b * 2 if b < 8 else (b // 2 * 3 if b & (b - 1) == 0 else b // 3 * 4)
    return max(n, min(b, limit))


class GraphDecodeRunner:
    """Replays a recorded step while the set of live sequences stays the same; when it
    changes, the slots and tokens are uploaded anew and the graph of the new size is used.
    A step is keyed by (rows, bucket of context lengths, sampling mode): the rows are the number of live
    sequences rounded up to a ``batch_bucket`` (idle rows run on the cache's scratch slot and their tokens
    are dropped); the temperature is read from the device, so it is no part of the key.  The first step of an
    engine is run eagerly (whatever is built or loaded at first use must not happen while a graph is being
    recorded) and recorded when its key comes again; every later key is recorded when it is first seen.  An
    engine keeps at most MAX_RECORDED_STEPS recorded steps and counts what it did in ``engine.decode_counts``
    (steps run eagerly, steps recorded, steps replayed)."""

    def __init__(self, engine, sampler):
        self.engine, self.sampler = engine, sampler
        cache = engine.cache
        n = cache.n_slots
        dev = engine.device
        self.bufs = engine._graph_bufs
        if self.bufs is None:
            self.bufs = {k: torch.zeros((n,), dtype=torch.int32, device=dev) for k in ("tokens", "slots", "pos", "ctx")}
            self.bufs["rows"] = torch.arange(n, dtype=torch.int32, device=dev)
            self.bufs["temperature"] = torch.ones((1,), dtype=torch.float32, device=dev)
            # where the tokens of the steps in flight arrive on the host
            self.bufs["host"] = [Tensor.pinned((n,), torch.int32) for _ in range(3)]
            self.bufs["done"] = [torch.cuda.Event() for _ in range(3)]
            engine._graph_bufs = self.bufs
        self.current = None            # the rows' slots now in the buffers
        self._ahead = None             # a step enqueued before its predecessor's tokens were read
        self._fed = None               # slot -> the token that step was fed on the device
        self._host, self._done = self.bufs["host"], self.bufs["done"]
        self._turn = 0
        # one table of rotation angles for the whole model: the bookkeeping kernel fills it
        wanted = [p.step_table() for p in engine.model.positions.values() if hasattr(p, "step_table")]
        wanted = [w for w in wanted if w is not None]
        self._table = wanted[0] if len(wanted) == 1 else None

    def _body(self, n, bucket):
        eng, b = self.engine, self.bufs
        ctx = _GraphContext(b, n, bucket)
        table = ops.decode_prepare(b["slots"], eng.cache.lens_dev, b["pos"], b["ctx"], n, eng.cache.scratch_slot,
                                   self._table[1] if self._table else None)
        if table is not None:
            ctx.shared(self._table[0], lambda: table)
        logits = eng.model.forward(ctx, eng.cache)
        # the sampled tokens go where the next step reads its tokens (the copy to the host is enqueued
        # between the two steps)
        self.sampler.sample(logits, b["slots"][:n], eng.cache, out=b["tokens"], temperature_dev=b["temperature"])

    def _launch(self, slots, tokens):
        """Enqueues one step for ``slots`` and the copy of its tokens to pinned host memory.
        ``tokens`` None: the tokens the step before left on the device are fed."""
        eng, cache, b = self.engine, self.engine.cache, self.bufs
        n = len(slots)
        rows = batch_bucket(n, cache.n_slots)
        new_lens = [cache.lens[s] + 1 for s in slots]
        cache.grow(slots, new_lens, sync_lens=False)
        padded = list(slots) + [cache.scratch_slot] * (rows - n)
        if self.current != padded:
            if tokens is None:
                raise RuntimeError("a new set of sequences needs its tokens")
            b["slots"][:rows].copy_(torch.tensor(padded, dtype=torch.int32))
            b["tokens"][:rows].copy_(torch.tensor(list(tokens) + [0] * (rows - n), dtype=torch.int32))
            self.current = padded
        bucket = split_bucket(max(new_lens))
        hot = self.sampler.temperature > 0.0
        if hot and b.get("temperature_value") != self.sampler.temperature:
            b["temperature"].fill_(self.sampler.temperature)
            b["temperature_value"] = self.sampler.temperature
        key = (rows, bucket, hot)
        graphs, counts = eng._graphs, eng.decode_counts
        entry = graphs.pop(key, None)            # taken out and put back: the dict is in order of last use
        if entry is None and not graphs:
            self._body(rows, bucket)             # the engine's first decode step
            entry = "seen"
            counts["eager"] += 1
        else:
            if entry is None or entry == "seen":
                g = torch.cuda.CUDAGraph()
                with recording(g):
                    self._body(rows, bucket)
                entry = g
                counts["recorded"] += 1
            else:
                counts["replayed"] += 1
            entry.replay()
        graphs[key] = entry
        while len(graphs) > MAX_RECORDED_STEPS:
            old = next(iter(graphs))
            if graphs[old] != "seen":
                torch.cuda.synchronize()         # a recorded step may still be running: let it finish first
            del graphs[old]
        self._turn = (self._turn + 1) % len(self._host)
        host, done = self._host[self._turn], self._done[self._turn]
        host[:n].copy_(b["tokens"][:n], non_blocking=True)
        done.record()
        return list(slots), host, done

    @staticmethod
    def _collect(step):
        slots, host, done = step
        done.synchronize()
        return host[:len(slots)].tolist()

    def run(self, slots, tokens, may_follow: bool = False):
        """One token for each of ``slots``.  ``may_follow``: the caller will ask for the same
        sequences again with the tokens returned here unless one of them ends; then the next
        step is enqueued before this one's tokens are read, so the device does not wait for
        the host.  If sequences do end, the step already enqueued still serves those that go
        on (a sequence's step does not depend on the rest of the batch); what it computed for
        the others is dropped with their slots."""
        slots = list(slots)
        if self._ahead is not None:
            step, self._ahead = self._ahead, None
            if list(tokens) != [self._fed[s] for s in slots] or any(s not in step[0] for s in slots):
                raise RuntimeError("a step was enqueued ahead for other sequences or tokens than those asked for now")
            if slots == step[0] and may_follow:
                self._ahead = self._launch(slots, None)
            every = self._collect(step)
            out = [every[step[0].index(s)] for s in slots]
        else:
            step = self._launch(slots, tokens)
            if may_follow:
                self._ahead = self._launch(slots, None)
            out = self._collect(step)
        self._fed = dict(zip(slots, out)) if self._ahead is not None else None
        self.engine.cache.trim_windows(slots)
        return out

    def drain(self):
        """Waits for a step enqueued ahead and drops its tokens.  Its sequences have moved on by
        that step all the same: they can be freed, not continued with other tokens."""
        if self._ahead is not None:
            self._collect(self._ahead)
            self._ahead = self._fed = None
