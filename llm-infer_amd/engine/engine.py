"""The engine: a model, its cache, and the one step function."""
from __future__ import annotations

import math
import sys

import torch

from ..cache import Cache, CacheError
from ..registry import config_from_folder
from ..weights import (OnDemand, choose_dtype, load_into, place_tensor, random_tensors, read_checkpoint,
                       stored_matrix_dtype)
from .model import DecoderModel
from .step import StepContext

_DTYPES = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32,
           "bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


# up to this many parameters an engine with random weights draws them as a folder's writer would
SAME_AS_FOLDER_LIMIT = 1 << 29


def as_dtype(d):
    if isinstance(d, torch.dtype):
        return d
    if d not in _DTYPES:
        raise ValueError(f"dtype {d!r}: one of bfloat16, float16, float32")
    return _DTYPES[d]


def _say(msg: str) -> None:
    print(f"[llm_infer_amd] {msg}", file=sys.stderr, flush=True)


def _require_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("llm_infer_amd runs on an MI355X through its HIP kernels; no GPU is visible "
                           "and there is no CPU implementation")


class Engine:
    """``step`` runs a batch of sequences that started together: their prompts in one step, then
    one token each.  It runs only the tokens it is given, against what earlier steps left in
    the cache, and returns the logits at the wanted places."""

    def __init__(self, config, model: DecoderModel, max_tokens: int, n_slots: int | None = None, kv_round=None):
        self.config, self.model = config, model
        self.dtype, self.device = model.dtype, model.device
        self.max_positions = model.spec.max_positions
        self.vocab_size = model.spec.vocab_size
        # kv_round="float16" with dtype float32 is the reference's own mix: float32 activations, keys and
        # values rounded to float16 on their way into the cache (src/model/block.cpp:145-148)
        self.cache = Cache(model.cache_specs(), max_tokens, self.max_positions, model.dtype, model.device, n_slots,
                           as_dtype(kv_round) if kv_round else None)
        self._graphs = {}
        self._graph_bufs = None
        self.decode_counts = {"eager": 0, "recorded": 0, "replayed": 0}      # what the recorded-step runner did
        # short prompts are recorded too (engine/prefill.py); False runs every prefill step eagerly
        self.record_prefill = True
        self._prefill = None

    # -- construction ----------------------------------------------------------
    @classmethod
    def from_folder(cls, folder: str, dtype=None, max_tokens: int = 8192, n_slots=None, device="cuda",
                    kv_round=None):
        """``dtype`` None: the model's own (``torch_dtype`` of config.json, else the type its matrices are
        stored in); a dtype that narrows what is stored, or swaps the 16-bit type, is said in one line."""
        _require_gpu()
        config = config_from_folder(folder)
        spec = config.model_spec()
        table = DecoderModel(spec, torch.float32, device, allocate=False).params()
        ckpt = read_checkpoint(folder, table, config)
        dt = choose_dtype(dtype, getattr(config, "torch_dtype", None), stored_matrix_dtype(table, ckpt), _say)
        model = DecoderModel(spec, dt, device)
        load_into(model, folder, config, ckpt)
        return cls(config, model, max_tokens, n_slots, kv_round)

    @classmethod
    def from_random(cls, config, seed: int = 0, dtype=None, max_tokens: int = 8192, n_slots=None,
                    device="cuda", stored_dtype=None, kv_round=None, same_as_folder=None):
        """Random weights without a folder: matrices as ``stored_dtype`` would store them.
        ``dtype`` None: the configuration's ``torch_dtype``, else bfloat16.
        ``same_as_folder``: the tensors are drawn by the CPU's generator and are those that
        ``write_random_model`` writes for this seed and stored dtype, so that what follows a folder (a plain
        implementation, another run) follows this engine too.  False draws them with the device's generator:
        other values for the same seed, and seconds instead of minutes for billions of parameters.  None (the
        default) means True up to ``SAME_AS_FOLDER_LIMIT`` parameters."""
        _require_gpu()
        dt = choose_dtype(dtype, getattr(config, "torch_dtype", None), None)
        model = DecoderModel(config.model_spec(), dt, device)
        stored = as_dtype(stored_dtype) if stored_dtype else (dt if dt != torch.float32 else torch.bfloat16)
        params = model.params()
        if same_as_folder is None:
            same_as_folder = sum(math.prod(spec.shape) for spec in params.values()) <= SAME_AS_FOLDER_LIMIT
        drawn_on = "cpu" if same_as_folder else device
        model.bind(OnDemand(lambda name: place_tensor(random_tensors({name: params[name]}, seed, stored, drawn_on)[name],
                                                      params[name].kind, dt, device)))
        return cls(config, model, max_tokens, n_slots, kv_round)

    # -- sequences -----------------------------------------------------------------
    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def length(self, slot: int) -> int:
        return self.cache.lens[slot]

    def decode_runner(self, sampler, use_graph: bool = True):
        from .decode import GraphDecodeRunner, PlainDecodeRunner
        if use_graph and self.model.recordable():
            return GraphDecodeRunner(self, sampler)
        return PlainDecodeRunner(self, sampler)

    def generate(self, prompts, **kw):
        from .generate import generate
        return generate(self, prompts, **kw)

    # -- the step ----------------------------------------------------------------------
    def step(self, slots, tokens, want=None) -> torch.Tensor:
        """slots[i]: a held slot; tokens[i]: that sequence's next tokens (at least one);
        want[i]: places among these tokens whose logits are returned (default: the last).
        Returns float32 [sum(len(want[i])), vocab] in the order of the sequences and of want."""
        ctx = self.prepare(slots, tokens, want, upload=False)
        try:
            logits = None
            if self.record_prefill:
                if self._prefill is None:
                    from .prefill import PrefillRecorder
                    self._prefill = PrefillRecorder()
                if self._prefill.takes(self, ctx):
                    logits = self._prefill.run(self, ctx)    # None the first time a size is seen
            if logits is None:
                ctx.upload()
                logits = self.model.forward(ctx, self.cache)
        except Exception:
            # a kernel refused its operands: the sequences are as long as before the step, and the pages
            # the step took are given back
            self.cache.truncate(slots, ctx.host_lens_before)
            raise
        self.cache.trim_windows(slots)
        return logits

    def prepare(self, slots, tokens, want=None, upload: bool = True) -> StepContext:
        if len(slots) != len(tokens) or len(set(slots)) != len(slots):
            raise ValueError("step: one token list for each slot, each slot once")
        if want is None:
            want = [[len(t) - 1] for t in tokens]
        for s, t, w in zip(slots, tokens, want):
            if len(t) == 0:
                raise ValueError(f"step: sequence in slot {s} brings no token")
            if min(t) < 0 or max(t) >= self.vocab_size:
                raise ValueError(f"step: token id outside [0, {self.vocab_size}) in slot {s}")
            if any(not 0 <= i < len(t) for i in w):
                raise ValueError(f"step: wanted place outside the {len(t)} tokens of slot {s}")
        before = [self.cache.lens[s] for s in slots]
        # every mixer writes all of the step's tokens into its cache before anything reads it
        self.cache.grow(slots, [b + len(t) for b, t in zip(before, tokens)], filled=True)
        return StepContext(self.device, slots, tokens, before, want, upload)
