"""The engine: a model with its weights on the GPU, its cache, and one step function.

`step` is the only way tokens reach the model. It takes a batch of sequences,
each with the next tokens of that sequence (a whole prompt, or one token), runs
exactly these tokens as one batch against what the cache holds, appends them to
the cache and returns float32 logits at the wanted places. The reference has
three entry points for one sequence each (crates/xrt-models/src/llama.rs:388-394
forward_token, :617-622 forward_batch, :830-835 forward_batch_all_logits);
positions are implied here by each sequence's length in the cache, where the
reference checks the caller's position against it (llama.rs:434-439).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache import BLOCK_TOKENS, CacheError, CacheFull, SequenceCache
from ..config import architecture, load_config
from ..host import last_error, load_host
from ..models import DecoderModel, ModelSpec
from ..parts.base import Runtime
from ..weights import CheckpointSource, RandomSource
from ..staging import staging_for
from .batch import build_batch, flatten

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32}


def compute_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype must be bfloat16 or float32, found {name}")
        return name
    if name not in _DTYPES:
        raise ValueError(f"dtype must be one of {sorted(_DTYPES)}, found {name!r}")
    return _DTYPES[name]


MOST_SLOTS_BY_DEFAULT = 1024     # slots of a cache whose maker names no number: a block each, up to this many


class StepError(ValueError):
    """A step that cannot run; nothing was computed and the cache is unchanged."""


class Engine:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], dtype="bfloat16",
                 max_tokens: int = 4096, max_slots: Optional[int] = None,
                 max_context: Optional[int] = None, device="cuda:0", ops=None, graphs: bool = True,
                 pack_weights="auto"):
        self.dtype = compute_dtype(dtype)
        self.device = torch.device(device)
        if ops is None:
            from ..ops import load_ops
            ops = load_ops()            # raises if the HIP library cannot be loaded: there is no other path
        self.ops = ops
        self.runtime = Runtime(ops, self.dtype, self.device, pack_weights)
        self.config = spec.config
        # by checkpoint name: a dict, or a source that reads or makes a tensor when a part asks for it and
        # keeps none, so that the device holds every weight once, in the form the parts bound it
        self.tensors = tensors
        self.model = DecoderModel(spec, tensors, self.runtime)
        if hasattr(tensors, "release"):
            tensors.release()           # every part has bound what it needs: a checkpoint's files are closed (get_tensor opens them again)
        model_context = getattr(spec.config, "max_position_embeddings", None)
        limit = max_context if max_context is not None else model_context
        if limit is None:
            limit = max_tokens
        if model_context is not None:
            limit = min(limit, model_context)
        if max_slots is None:
            max_slots = max(1, min((max_tokens + BLOCK_TOKENS - 1) // BLOCK_TOKENS, MOST_SLOTS_BY_DEFAULT))
        schedule = spec.schedule
        reads_from = [i if call.reads_cache_of is None else call.reads_cache_of
                      for i, call in enumerate(schedule)]
        self.cache = SequenceCache(spec.cache_needs(), reads_from, max_tokens, max_slots, limit,
                                   self.dtype, self.device)
        self.vocab_size = spec.head.vocab
        # decode steps are replayed as HIP graphs where the model allows it
        self.graphs = None
        if graphs and self.device.type == "cuda" and spec.capturable():
            from .graphs import DecodeGraphs
            self.graphs = DecodeGraphs(self.model, self.cache, self.device)

    # -- construction ----------------------------------------------------------
    @classmethod
    def load(cls, folder: str, dtype="bfloat16", **options) -> "Engine":
        """From a folder with config.json and model.safetensors (or shards with an index)."""
        config = load_config(folder)
        spec = architecture(config.architecture).build(config)
        tensors = CheckpointSource(folder, spec.weight_specs(), spec.ignored_names())
        return cls(spec, tensors, dtype=dtype, **options)

    @classmethod
    def random(cls, config, seed: int = 0, dtype="bfloat16", std: float = 0.02, gain_std: float = 0.0,
               **options) -> "Engine":
        """With random weights made on the device; no file is written. The values are those of the folder
        that `write_random_model` writes for the same configuration, seed and deviations, in the compute
        dtype (`get_tensor` makes them again on the host)."""
        spec = architecture(config.architecture).build(config)
        device = options.get("device", "cuda:0")
        ops = options.get("ops")
        if ops is None:
            from ..ops import load_ops
            ops = options["ops"] = load_ops()
        tensors = RandomSource(spec.weight_specs(), seed, std, compute_dtype(dtype), device, ops, gain_std)
        return cls(spec, tensors, dtype=dtype, **options)

    # -- slots -------------------------------------------------------------------
    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    @property
    def max_context(self) -> int:
        return self.cache.max_context

    # -- conveniences ------------------------------------------------------------
    def generate(self, prompts: Sequence[Sequence[int]], max_tokens: int = 128, temperature: float = 0.0,
                 top_k: int = 0, top_p: float = 1.0, repetition_penalty: float = 1.0, seed: Optional[int] = 0,
                 stop_ids: Optional[Sequence[int]] = None, batch_size: Optional[int] = None) -> List[List[int]]:
        """The generated token ids of every prompt, with one set of sampling options for all
        (greedy unless told otherwise). Every prompt draws from a stream of its own, made from `seed`
        and the prompt's index (seed=None: from the system's randomness). `generate()` of this package
        takes a request per prompt with options of its own and returns finish reasons and timings as well."""
        from ..sampling import request_seed
        from .generate import GenerateRequest, generate
        requests = [GenerateRequest(list(ids), max_tokens=max_tokens, temperature=temperature, top_k=top_k,
                                    top_p=top_p, repetition_penalty=repetition_penalty,
                                    seed=None if seed is None else request_seed(seed, index),
                                    stop_ids=None if stop_ids is None else tuple(stop_ids))
                    for index, ids in enumerate(prompts)]
        return [list(result.tokens) for result in generate(self, requests, batch_size=batch_size)]

    def get_tensor(self, name: str) -> torch.Tensor:
        """A weight by its checkpoint name, as the file (or the random-weights mode) gives it,
        on the host: what a reference computation outside this library needs."""
        if name not in self.tensors:
            raise KeyError(f"no tensor named '{name}'")
        if hasattr(self.tensors, "host"):
            return self.tensors.host(name)
        return self.tensors[name].detach().to("cpu")

    # -- the step ----------------------------------------------------------------
    def step(self, entries: Sequence[Tuple[int, Sequence[int], Sequence[int]]]) -> torch.Tensor:
        """Run the next tokens of some sequences; return logits [wanted, vocab] (float32, on the device).

        entries: (slot, tokens, want) per sequence; `want` are indices into `tokens`, in the order
        in which their logits are returned (entries first, then want). The sequences of a step may
        start (length 0) or continue, with any token counts, in any mixture.
        """
        slots, tokens, wants, starts = self.prepare(entries)
        try:
            if self.graphs is not None and all(len(ids) == 1 for ids in tokens) and all(w == [0] for w in wants):
                logits = self.graphs.step(slots, [ids[0] for ids in tokens], starts)
            else:
                with self.runtime.step_memory():                # the step's tensors come from memory kept for steps
                    batch = build_batch(slots, tokens, starts, wants, self.device, allocate=self._step_integers)
                    logits = self.model.forward(batch, self.cache)
        except Exception:
            for slot in slots:
                self.cache.cancel(slot)
            raise
        for slot, start, ids in zip(slots, starts, tokens):
            self.cache.commit(slot, start + len(ids))
        return logits

    def step_from(self, tokens: torch.Tensor, entries: Sequence[Tuple[int, int]]) -> torch.Tensor:
        """One more token for some sequences, taken from the device: entries are (slot, row), and the
        sequence in `slot` goes on with tokens[row] (int32, ids below the vocabulary's size: what the
        sampler wrote). Returns logits [len(entries), vocab] like `step`. Nothing here waits for the
        device, so a caller can start the next step before it has seen the tokens of the last one."""
        slots, _, _, starts = self.prepare([(slot, [0], [0]) for slot, _ in entries])
        rows = [int(row) for _, row in entries]
        try:
            if min(rows) < 0 or max(rows) >= tokens.numel():
                raise StepError(f"rows {rows} are outside the {tokens.numel()} tokens given")
            if self.graphs is not None:
                logits = self.graphs.step(slots, [0] * len(slots), starts, source=(tokens, rows))
            else:
                with self.runtime.step_memory():
                    batch = build_batch(slots, [[0]] * len(slots), starts, [[0]] * len(slots), self.device, allocate=self._step_integers)
                    batch.token_ids.copy_(tokens.index_select(0, staging_for(self.device).upload(rows)))
                    logits = self.model.forward(batch, self.cache)
        except Exception:
            for slot in slots:
                self.cache.cancel(slot)
            raise
        for slot, start in zip(slots, starts):
            self.cache.commit(slot, start + 1)
        return logits

    def _step_integers(self, count: int) -> torch.Tensor:
        return self.runtime.empty((count,), torch.int32)

    def prepare(self, entries):
        """Check a step and reserve its cache blocks; returns (slots, tokens, wants, starts) per sequence.
        Raises StepError before anything changes."""
        if len(entries) == 0:
            raise StepError("a step needs at least one sequence")
        slots, tokens, wants, starts = [], [], [], []
        for slot, ids, want in entries:
            if not self.cache.slots.is_held(slot):
                raise StepError(f"slot {slot} is not allocated")
            slots.append(int(slot))
            tokens.append(list(ids))
            wants.append(list(want))
            starts.append(self.cache.length(slot))
        # the rest of the checks are the host library's (no slot twice, a token at least, ids below the embedding's
        # rows, wanted places inside the tokens given, the context limit): one call for the whole step
        try:
            counts, flat_tokens = flatten(tokens)
            want_counts, flat_wants = flatten(wants)
        except (OverflowError, ValueError, TypeError):
            raise StepError("token ids and wanted places must be integers that fit 32 bits") from None
        host = load_host()
        as_array = lambda values: np.ascontiguousarray(values, dtype=np.int32)
        slot_array, start_array = as_array(slots), as_array(starts)
        if host.xrt_step_check(len(slots), slot_array.ctypes.data, counts.ctypes.data, start_array.ctypes.data,
                               flat_tokens.ctypes.data, want_counts.ctypes.data, flat_wants.ctypes.data,
                               int(self.vocab_size), int(self.cache.max_context)) != 0:
            raise StepError(last_error())
        reserved = []
        try:
            for slot, ids, start in zip(slots, tokens, starts):
                self.cache.reserve(slot, start + len(ids))
                reserved.append(slot)
        except (CacheFull, CacheError) as error:
            for slot in reserved:
                self.cache.cancel(slot)
            raise StepError(f"the cache cannot hold this step: {error}") from None
        self.cache.sync()
        return slots, tokens, wants, starts
