"""Short prompts as recorded steps.

A step of a few tokens on a model of many layers is bound by the host: some three hundred kernel
launches take longer to enqueue than the device needs to run them.  Such a step (at most
``MAX_TOKENS`` tokens in at most ``MAX_SEQS`` sequences) is therefore recorded into a HIP graph, keyed by
the numbers of rows it runs, and replayed.  The rows are the step's tokens, sequences and wanted places, each
rounded up to a bucket (``decode.batch_bucket``); what a step does not fill is padding that changes no
result: padded tokens sit on the cache's scratch slot (they write the null page and belong to no sequence,
so no attention tile covers them), padded sequences have no tokens, padded wanted places repeat row 0 and
are cut off the result.  Everything a recorded step reads of the step lies in one device buffer of index
arrays that is refilled with one copy before each replay; page tables and lengths are updated outside the
graph, as for decoding.  The reference replays a recorded graph per token in the same spirit
(src/model/model.cu:11-22).

Only parts that say so are recorded (``prefill_recordable``): a part that plans on the host from the step's
lengths (``ctx.host_qlens``) would have its plan frozen into the graph.
"""
from __future__ import annotations

import numpy as np
import torch

from ..kernels import ops
from .decode import batch_bucket, recording
from .step import StepShared

MAX_TOKENS = 512          # a longer step keeps the device busy longer than the host needs to enqueue it
MAX_SEQS = 16
MAX_RECORDED = 32         # recorded prefill steps an engine keeps; the least recently used goes first


class _RecordedContext(StepShared):
    """The step description of a recorded prefill step: slices of the one device buffer."""
    is_decode = False

    def __init__(self, fields, n_tokens, n_seqs, n_want, device):
        self.n_tokens, self.n_seqs, self.n_want, self.device = n_tokens, n_seqs, n_want, device
        for name, t in fields.items():
            setattr(self, name, t)


class PrefillRecorder:
    """The recorded prefill steps of one engine (which is handed in with every call: the engine holds this
    object, and a reference back would keep both alive until the garbage collector finds the cycle)."""

    def __init__(self):
        self.graphs = {}                   # key -> "seen" | (graph, logits)
        self.counts = {"eager": 0, "recorded": 0, "replayed": 0}
        self._buffers = {}                 # key -> (device buffer, layout)

    # -- which steps ---------------------------------------------------------------
    def takes(self, eng, ctx) -> bool:
        """A step of whole prompts (or chunks of them) that is small enough, on a model whose parts can all
        be recorded."""
        if ctx.is_decode or ctx.n_want == 0 or ctx.n_tokens > MAX_TOKENS or ctx.n_seqs > MAX_SEQS:
            return False
        if getattr(self, "_model_ok", None) is None:
            model = eng.model
            mixers = [m for ms in model.layer_mixers for m in ms]
            self._model_ok = model.recordable() and all(getattr(m, "prefill_recordable", False) for m in mixers)
        return self._model_ok

    # -- the buffer of index arrays ------------------------------------------------
    @staticmethod
    def _layout(rows, seqs, wants):
        tiles = -(-rows // ops.Q_TILE) + seqs            # at most this many attention tiles
        sizes = [("token_ids", rows), ("pos", rows), ("tok_slot", rows), ("seq_slot", seqs), ("seq_qstart", seqs),
                 ("seq_qlen", seqs), ("seq_ctx", seqs), ("want_rows", wants), ("tile_seq", tiles), ("tile_q0", tiles)]
        layout, at = {}, 0
        for name, n in sizes:
            layout[name] = (at, n)
            at += (n + 3) // 4 * 4
        return layout, at

    @staticmethod
    def _fill(ctx, layout, total, scratch):
        """The step's index arrays with their padding, as one int32 array."""
        packed = np.zeros(total, dtype=np.int32)

        def put(name, values, pad):
            at, n = layout[name]
            packed[at:at + n] = pad
            packed[at:at + len(values)] = values
        qlens, before = ctx.host_qlens, ctx.host_lens_before
        qstart = np.concatenate([[0], np.cumsum(qlens)])[:-1]
        put("token_ids", ctx.host_tokens, 0)
        put("pos", [b + j for b, q in zip(before, qlens) for j in range(q)], 0)
        put("tok_slot", [s for s, q in zip(ctx.host_slots, qlens) for _ in range(q)], scratch)
        put("seq_slot", ctx.host_slots, scratch)
        put("seq_qstart", qstart, 0)
        put("seq_qlen", qlens, 0)
        put("seq_ctx", [b + q for b, q in zip(before, qlens)], 0)
        put("want_rows", ctx.host_want_rows, 0)
        tile_seq, tile_q0 = ops.prefill_tiles(qlens)
        put("tile_seq", tile_seq, 0)
        put("tile_q0", tile_q0, 1 << 30)                  # a tile that begins beyond its sequence does nothing
        return packed

    # -- the step --------------------------------------------------------------------
    def run(self, eng, ctx):
        """The logits of the step [n_want, vocab], or None if this step is to be run eagerly (the first time
        its key is seen)."""
        rows = batch_bucket(ctx.n_tokens, MAX_TOKENS)
        seqs = batch_bucket(ctx.n_seqs, MAX_SEQS)
        wants = batch_bucket(ctx.n_want, rows)
        key = (rows, seqs, wants)
        entry = self.graphs.pop(key, None)
        if entry is None:
            self.graphs[key] = "seen"
            self.counts["eager"] += 1
            self._trim()
            return None
        layout, total = self._layout(rows, seqs, wants)
        if key not in self._buffers:
            self._buffers[key] = torch.zeros((total,), dtype=torch.int32, device=eng.device)
        buf = self._buffers[key]
        buf.copy_(torch.from_numpy(self._fill(ctx, layout, total, eng.cache.scratch_slot)))
        if entry == "seen":
            fields = {name: buf[at:at + n] for name, (at, n) in layout.items()}
            tiles = {"tile_seq": fields.pop("tile_seq"), "tile_q0": fields.pop("tile_q0"), "n_tiles": layout["tile_seq"][1]}
            graph = torch.cuda.CUDAGraph()
            with recording(graph):
                rec = _RecordedContext(fields, rows, seqs, wants, eng.device)
                rec.shared(ops.PREFILL_TILES_KEY, lambda: tiles)
                logits = eng.model.forward(rec, eng.cache)
            entry = (graph, logits)
            self.counts["recorded"] += 1
        else:
            self.counts["replayed"] += 1
        entry[0].replay()
        self.graphs[key] = entry
        self._trim()
        return entry[1][:ctx.n_want].clone()

    def _trim(self):
        while len(self.graphs) > MAX_RECORDED:
            old = next(iter(self.graphs))
            if self.graphs[old] != "seen":
                torch.cuda.synchronize()             # it may still be running
            del self.graphs[old]
            self._buffers.pop(old, None)
