"""The description of one step on the device: which tokens run, where they stand in
their sequences, and where their sequences live in the cache."""
from __future__ import annotations

import numpy as np
import torch

PAGE = 64
Q_TILE = 128            # tokens of one workgroup of the prefill attention kernel


class StepContext:
    """All index arrays are int32 on the device, uploaded with one copy.

    per token   : token_ids, pos (position in its sequence), tok_slot (its sequence's slot)
    per sequence: seq_slot, seq_qstart (first token of the sequence in this step),
                  seq_qlen (tokens in this step), seq_ctx (context length after the step)
    want_rows   : rows of the step whose logits are asked for
    """

    def __init__(self, device, slots, tokens, lens_before, want):
        self.n_seqs = len(slots)
        qlens = [len(t) for t in tokens]
        self.n_tokens = sum(qlens)
        self.is_decode = all(q == 1 for q in qlens) and all(l >= 1 for l in lens_before)
        self.max_ctx = max((l + q for l, q in zip(lens_before, qlens)), default=0)
        self.host_slots, self.host_qlens, self.host_lens_before = list(slots), qlens, list(lens_before)
        qstart = np.concatenate([[0], np.cumsum(qlens)])[:-1] if qlens else np.zeros(0)
        flat = [t for seq in tokens for t in seq]
        pos = [l + j for l, q in zip(lens_before, qlens) for j in range(q)]
        tok_slot = [s for s, q in zip(slots, qlens) for _ in range(q)]
        want_rows = [int(qstart[i]) + w for i, ws in enumerate(want) for w in ws]
        self.n_want = len(want_rows)
        tile_seq, tile_q0 = [], []
        for i, q in enumerate(qlens):
            for q0 in range(0, q, Q_TILE):
                tile_seq.append(i)
                tile_q0.append(q0)
        self.n_tiles = len(tile_seq)
        fields = [("token_ids", flat), ("pos", pos), ("tok_slot", tok_slot), ("seq_slot", slots),
                  ("seq_qstart", qstart), ("seq_qlen", qlens),
                  ("seq_ctx", [l + q for l, q in zip(lens_before, qlens)]),
                  ("want_rows", want_rows), ("tile_seq", tile_seq), ("tile_q0", tile_q0)]
        sizes = [len(v) for _, v in fields]
        offs = np.concatenate([[0], np.cumsum([(s + 3) // 4 * 4 for s in sizes])])
        packed = np.zeros(int(offs[-1]) + 4, dtype=np.int32)
        for (_, v), o, s in zip(fields, offs, sizes):
            packed[int(o):int(o) + s] = np.asarray(v, dtype=np.int32)
        dev = torch.from_numpy(packed).to(device)
        for (name, _), o, s in zip(fields, offs, sizes):
            setattr(self, name, dev[int(o):int(o) + s])
        self._packed = dev

    def prefill_meta(self) -> dict:
        return {"tile_seq": self.tile_seq, "tile_q0": self.tile_q0, "n_tiles": self.n_tiles,
                "seq_slot": self.seq_slot, "seq_qstart": self.seq_qstart, "seq_qlen": self.seq_qlen,
                "seq_ctx": self.seq_ctx}

    def decode_splits(self, n_kv_heads: int, n_heads: int) -> int:
        """How many ways the decode attention cuts each sequence's context so that the chip is filled."""
        return decode_splits(self.n_seqs, n_kv_heads, n_heads, self.max_ctx)


def decode_splits(n_seqs: int, n_kv_heads: int, n_heads: int, max_ctx: int) -> int:
    waves = n_seqs * n_kv_heads * ((n_heads // n_kv_heads + 31) // 32)
    pages = (max_ctx + PAGE - 1) // PAGE
    # measured on MI355X: 1,024 waves fill the chip best, but from 512 waves on one pass without the
    # merge kernel is faster than two halves with it
    want = 1 if waves >= 512 else max(1, 1024 // max(1, waves))
    s = max(1, min(want, pages // 2, 64))
    p = 1
    while p * 2 <= s:                 # powers of two, so that a captured step is reused for many lengths
        p *= 2
    return p
