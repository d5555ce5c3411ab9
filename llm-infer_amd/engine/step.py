"""The description of one step on the device: which tokens run, where they stand in
their sequences, and where their sequences live in the cache."""
from __future__ import annotations

import numpy as np
import torch

PAGE = 64


class StepShared:
    """What the parts of a step share: a value that depends on the step alone (a table of angles, the
    index arrays of a kernel's grid) is made by the first part that asks for it under its key and
    found by the others."""

    def shared(self, key, make):
        store = self.__dict__.setdefault("_shared", {})
        if key not in store:
            store[key] = make()
        return store[key]


class StepContext(StepShared):
    """All index arrays are int32 on the device, uploaded with one copy.

    per token   : token_ids, pos (position in its sequence), tok_slot (its sequence's slot)
    per sequence: seq_slot, seq_qstart (first token of the sequence in this step),
                  seq_qlen (tokens in this step), seq_ctx (context length after the step)
    want_rows   : rows of the step whose logits are asked for
    The host keeps ``host_slots``, ``host_qlens`` and ``host_lens_before`` for parts that plan on the host.
    ``upload=False`` leaves the device arrays out until ``upload()`` is called (a step that is replayed from a
    recording reads them from the recording's own buffer).
    """

    def __init__(self, device, slots, tokens, lens_before, want, upload: bool = True):
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
        self.device = device
        self.host_tokens, self.host_want_rows = flat, want_rows
        self._fields = [("token_ids", flat), ("pos", pos), ("tok_slot", tok_slot), ("seq_slot", slots),
                        ("seq_qstart", qstart), ("seq_qlen", qlens),
                        ("seq_ctx", [l + q for l, q in zip(lens_before, qlens)]),
                        ("want_rows", want_rows)]
        if upload:
            self.upload()

    def upload(self) -> None:
        """The index arrays onto the device, with one copy."""
        fields, device = self._fields, self.device
        sizes = [len(v) for _, v in fields]
        offs = np.concatenate([[0], np.cumsum([(s + 3) // 4 * 4 for s in sizes])])
        packed = np.zeros(int(offs[-1]) + 4, dtype=np.int32)
        for (_, v), o, s in zip(fields, offs, sizes):
            packed[int(o):int(o) + s] = np.asarray(v, dtype=np.int32)
        dev = torch.from_numpy(packed).to(device)
        for (name, _), o, s in zip(fields, offs, sizes):
            setattr(self, name, dev[int(o):int(o) + s])
        self._packed = dev

    def decode_splits(self, n_kv_heads: int, n_heads: int) -> int:
        """How many ways the decode attention of a mixer with these heads cuts each sequence's context."""
        return decode_splits(self.n_seqs, n_kv_heads, n_heads, split_bucket(self.max_ctx))


def split_bucket(max_ctx: int) -> int:
    """The most splits that a context of this length is worth (a power of two up to 64): at least two
    pages a split.  It is all that the split count needs to know of the lengths, so a recorded step
    serves every length of one bucket."""
    pages = (max_ctx + PAGE - 1) // PAGE
    s = max(1, min(pages // 2, 64))
    return 1 << (s.bit_length() - 1)


def decode_splits(n_seqs: int, n_kv_heads: int, n_heads: int, bucket: int) -> int:
    """Splits of the context for a decode attention of ``n_seqs`` sequences (a power of two, at most
    ``bucket``), so that the chip is filled."""
    waves = n_seqs * n_kv_heads * ((n_heads // n_kv_heads + 31) // 32)
    # measured on MI355X: 1,024 waves (one a SIMD) fill the chip best; two or four splits are merged inside
    # a workgroup and cost no second kernel
    want = max(1, 1024 // max(1, waves))
    s = max(1, min(want, bucket))
    return 1 << (s.bit_length() - 1)
