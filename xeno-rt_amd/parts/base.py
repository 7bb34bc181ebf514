"""What every part of a model is: the interfaces, and the registry of part kinds.

A model is put together from parts: a mixer (attention here), a feed-forward,
norms, a position encoding, and a block that arranges them. A part is built with
its sizes and constants as arguments and with the prefix of its tensors in the
checkpoint; it does not know which model it is in. It says which tensors it
binds (`weight_specs`), what it needs from the cache (`cache_needs`, mixers
only), takes its tensors at load (`bind`) and runs on the tokens of one step
(`forward`).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Optional, Tuple

import torch


# ----------------------------------------------------------------------------
# declarations a part makes
# ----------------------------------------------------------------------------

@dataclass(frozen=True)
class WeightSpec:
    """One tensor of the checkpoint that a part binds.

    init: how the random-weights mode fills it ("normal": N(0, std), "ones", "zeros").
    kind: "matrix" is converted to the engine's compute dtype when bound;
          "vector" keeps 32-bit storage if the file stores it so;
          "table" is an integer table, kept as int32.
    """
    shape: Tuple[int, ...]
    init: str = "normal"
    kind: str = "matrix"


@dataclass(frozen=True)
class KVSpec:
    """Keys and values for every token: n_kv_heads rows of head_dim (keys) and of value_dim (values;
    as wide as the keys unless given).

    window = None keeps all tokens; window = W keeps what a query can still see
    when it looks at the W most recent tokens (itself included).
    """
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class StateSpec:
    """State of fixed size for each sequence, zero when the sequence starts."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass(frozen=True)
class CacheNeeds:
    kv: Optional[KVSpec] = None
    state: Optional[StateSpec] = None


class StepArena:
    """One stretch of device memory that the tensors of a step are cut from, one after another; the next step
    starts at its beginning again. It is as large as the largest step so far needed (the reference grows its
    scratch on demand and keeps it, crates/xrt-models/src/llama.rs:240-268): a step that needs more than there is
    takes what does not fit from torch, and the stretch is made longer before the step after it. So a step of a size
    that has been seen before allocates nothing. What a step hands to its caller (the logits) never lies here."""

    ALIGN = 256

    def __init__(self, device):
        self.device = torch.device(device)
        self.buffer: Optional[torch.Tensor] = None
        self.at = 0                 # bytes handed out in this step, those that did not fit included
        self.wanted = 0             # the most a step has needed
        self.active = False

    def begin(self) -> None:
        capacity = 0 if self.buffer is None else self.buffer.numel()
        if self.wanted > capacity:
            self.buffer = None                                   # (given back before the longer one is taken)
            self.buffer = torch.empty(self.wanted + self.wanted // 8, dtype=torch.uint8, device=self.device)
        self.at = 0
        self.active = True

    def end(self) -> None:
        self.wanted = max(self.wanted, self.at)
        self.active = False

    def take(self, shape, dtype: torch.dtype) -> Optional[torch.Tensor]:
        """A tensor of this shape from the stretch, or None if it does not fit (the caller takes it from torch)."""
        count = 1
        for size in (shape if isinstance(shape, (tuple, list, torch.Size)) else (shape,)):
            count *= int(size)
        size = count * torch.empty(0, dtype=dtype).element_size()
        start = (self.at + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        self.at = start + size
        if self.buffer is None or self.at > self.buffer.numel():
            return None
        return self.buffer[start:start + size].view(dtype).view(shape)


class Runtime:
    """What a part needs to run: the kernels, the compute dtype and the device."""

    def __init__(self, ops, dtype: torch.dtype, device, pack_weights="auto"):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, found {dtype}")
        if pack_weights not in ("auto", "always", False):
            raise ValueError(f"pack_weights must be 'auto', 'always' or False, found {pack_weights!r}")
        self.ops = ops
        self.dtype = dtype
        self.device = torch.device(device)
        self.pack_weights = pack_weights        # "auto": where the kernels say it pays; "always": wherever it can be done
        self.arena = StepArena(self.device)     # what `empty` cuts a step's tensors from, while a step is under way

    def matrix(self, tensor: torch.Tensor) -> torch.Tensor:
        """A weight matrix in the compute dtype, contiguous, on the device. A tensor that comes from the
        host in another type is converted there, so that the device never holds it twice."""
        if tensor.device != self.device and tensor.dtype != self.dtype:
            tensor = tensor.to(self.dtype)
        return tensor.to(device=self.device, dtype=self.dtype).contiguous()

    def stacked(self, tensors) -> torch.Tensor:
        """Matrices of equal width one below the other, as one matrix in the compute dtype on the device:
        allocated once, each piece copied into its rows."""
        tensors = list(tensors)
        width = tensors[0].shape[1]
        if any(t.dim() != 2 or t.shape[1] != width for t in tensors):
            raise ValueError(f"stacked matrices need one width, found {[tuple(t.shape) for t in tensors]}")
        out = torch.empty((sum(t.shape[0] for t in tensors), width), dtype=self.dtype, device=self.device)
        at = 0
        for tensor in tensors:
            if tensor.device != self.device and tensor.dtype != self.dtype:
                tensor = tensor.to(self.dtype)
            out[at:at + tensor.shape[0]].copy_(tensor)
            at += tensor.shape[0]
        return out

    def weight(self, tensors, kind: str = "tiles", **details):
        """What `ops.linear` (or `linear_glu`, `linear_qkv`, `embed`) takes as its w: the matrix (or the matrices
        of equal width, one below the other) in the compute dtype on the device, and, where the kernels have a
        faster layout for matrices of its sizes, in that layout. kind and details name what the product's
        epilogue combines: "tiles" nothing, "gated" gate rows and up rows (gated_n of each), "rotary" the
        pairs of a rotation over whole heads (head_dim, rotated_heads). Only products read the result."""
        matrix = self.stacked(tensors) if isinstance(tensors, (list, tuple)) else self.matrix(tensors)
        pack = getattr(self.ops, "pack", None)
        if (pack is None or not self.pack_weights or self.dtype != torch.bfloat16 or matrix.device.type != "cuda"
                or matrix.shape[1] % 32 != 0 or (matrix.shape[0] + 15) * matrix.shape[1] >= 2 ** 31):
            return matrix
        if kind == "gated" and details.get("gated_n", 0) % 8 != 0:
            return matrix
        if kind == "rotary" and details.get("head_dim", 0) % 16 != 0:
            return matrix
        if self.pack_weights != "always" and not self.ops.packing_suits(matrix.shape[0], matrix.shape[1]):
            return matrix
        return pack(matrix, kind, **details)

    def vector(self, tensor: torch.Tensor) -> torch.Tensor:
        """A small float vector: bfloat16 if the file stores it so and the model computes in bfloat16,
        float32 otherwise (a float16 vector widens exactly)."""
        if self.dtype == torch.bfloat16 and tensor.dtype == torch.bfloat16:
            return tensor.to(device=self.device).contiguous()
        return tensor.to(device=self.device, dtype=torch.float32).contiguous()

    def empty(self, shape, dtype: Optional[torch.dtype] = None, outlives_the_step: bool = False) -> torch.Tensor:
        """An uninitialised tensor on the device for the step under way. It is gone when the next step begins, unless
        the part says that it outlives the step (what a model returns to its caller)."""
        if self.arena.active and not outlives_the_step:
            taken = self.arena.take(shape, dtype or self.dtype)
            if taken is not None:
                return taken
        return torch.empty(shape, dtype=dtype or self.dtype, device=self.device)

    def step_memory(self):
        """A context in which `empty`, and the kernels' workspaces, come from the step arena."""
        return _StepMemory(self)


class _StepMemory:
    def __init__(self, runtime: Runtime):
        self.runtime = runtime

    def __enter__(self):
        runtime = self.runtime
        runtime.arena.begin()
        if hasattr(runtime.ops, "allocate"):                   # the kernels' own workspaces and handed-on rows
            self.before = runtime.ops.allocate
            runtime.ops.allocate = lambda shape, dtype, device: runtime.empty(shape, dtype)
        return runtime.arena

    def __exit__(self, *exc):
        runtime = self.runtime
        if hasattr(runtime.ops, "allocate"):
            runtime.ops.allocate = self.before
        runtime.arena.end()


# ----------------------------------------------------------------------------
# interfaces
# ----------------------------------------------------------------------------

class Part:
    """Base of all parts."""

    # True if `forward` only launches kernels on the current stream with arguments that do not
    # depend on the step's contents, so that a decode step can be recorded once and replayed.
    # Parts that look at the batch on the host (loops over sequences, Python arithmetic on
    # lengths) leave it False; a model with such a part runs every step directly.
    capturable = False

    def weight_specs(self) -> Dict[str, WeightSpec]:
        """Full checkpoint name -> WeightSpec of every tensor this part binds."""
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor], runtime: Runtime) -> None:
        """Take the tensors named in `weight_specs` (stored dtype, any device)."""
        self.runtime = runtime


class Norm(Part):
    def forward(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Normalise the float32 rows of x (only `rows`, if given); result in the compute dtype."""
        raise NotImplementedError

    def row_scale(self) -> Optional[Tuple[torch.Tensor, float]]:
        """(gain, eps) if the norm is y = x / sqrt(mean(x^2) + eps) * gain over whole rows, None otherwise.

        Such a norm between two matrix products can be done by the two of them (`then` below), which
        saves a kernel where a step is short of work.
        """
        return None


@dataclass(frozen=True)
class HalfSplitRotation:
    """What a position encoding says of itself when it rotates the pairs (i, i + rope_dim / 2) of every head of q and k by
    the angle position * scale / theta[i]: theta is float32 [rope_dim / 2] on the device (None until the encoding is bound)."""
    rope_dim: int
    scale: float
    theta: Optional[torch.Tensor]
    table: Optional[torch.Tensor] = None       # float32 [positions, rope_dim / 2, 2]: cosine and sine of the first positions' angles,
                                               # made by `ops.rope_table`, for kernels that would rather read than work them out


class PositionEncoding(Part):
    def rotation(self) -> Optional[HalfSplitRotation]:
        """An encoding that is such a rotation returns it; the mixer then lets the kernel that follows its q/k/v projection
        rotate (fused into the projection where a step is short) and, when the rotation spans the whole head, keeps the two
        rows of a pair side by side in the projection's packed weight. None: the mixer calls `apply`."""
        return None

    def apply(self, qkv: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, batch) -> None:
        """Encode the positions of the step's tokens into q and k, in place.

        qkv is [tokens, (n_heads + 2*n_kv_heads) * head_dim]: queries, then keys, then values.
        """
        raise NotImplementedError

    def score_slopes(self) -> Optional[torch.Tensor]:
        """For an encoding that acts on the attention scores: float32 [n_heads] on the device; a key at position j
        then adds slope * (j - P) to the scaled score of the query at position P. None: the scores stay as they are."""
        return None


# A mixer, a feed-forward or a block may set `passes_norms = True`. It then promises two things.
# Its `forward` takes a keyword `then`: the norm that follows it on the residual stream, or None. If
# it can have its last product do that norm's work (`ops.linear(..., then_norm=then.row_scale())`),
# it returns what that product returns, else None, and the caller runs the norm. And what it is
# given as `h` may be such a returned object instead of a tensor: it hands `h` to `ops.linear` or
# `ops.linear_glu` and reads nothing of it but `h.shape`. Parts without the attribute are called
# as their interface below says and always get tensors.


class Mixer(Part):
    """Mixes information along the sequence; owns what it keeps in the cache."""

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds()

    def forward(self, h: torch.Tensor, batch, cache, residual: torch.Tensor) -> None:
        """Add the mixer's output for h [tokens, hidden] to the float32 `residual`, in place.

        `batch` is the step's StepBatch; `cache` the LayerCache of this call
        (`.kv` a KVView or None, `.state` a tensor [slots, *shape] or None,
        `.writable` False when the call reads another call's cache).
        """
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, batch, residual: torch.Tensor) -> None:
        """Add the feed-forward's output for h [tokens, hidden] to `residual`, in place."""
        raise NotImplementedError


class Block(Part):
    """The arrangement of a mixer, a feed-forward and their norms around the residual stream."""

    def cache_needs(self) -> CacheNeeds:
        return CacheNeeds()

    def forward(self, x: torch.Tensor, batch, cache) -> None:
        """Update the float32 residual stream x [tokens, hidden] in place.

        A block with `passes_norms` also takes `h`, the result of its first norm if the block before it
        has already made it, and `then`, the first norm of the block after it, and returns that norm's
        result or None.
        """
        raise NotImplementedError

    def first_norm(self) -> Optional[Norm]:
        """The norm this block applies to the residual stream before anything else, if it starts with one."""
        return None


# ----------------------------------------------------------------------------
# registry of part kinds, by name
# ----------------------------------------------------------------------------

_KINDS = ("mixer", "feed_forward", "norm", "position", "block")
_PARTS: Dict[str, Dict[str, Callable]] = {kind: {} for kind in _KINDS}


def register_part(kind: str, name: str, factory: Callable) -> None:
    """Make `factory(**arguments)` available to model builders as (kind, name)."""
    if kind not in _PARTS:
        raise KeyError(f"unknown part kind '{kind}'; kinds: {_KINDS}")
    _PARTS[kind][name] = factory


def create_part(kind: str, name: str, **arguments):
    if kind not in _PARTS:
        raise KeyError(f"unknown part kind '{kind}'; kinds: {_KINDS}")
    if name not in _PARTS[kind]:
        raise KeyError(f"no {kind} named '{name}'; registered: {sorted(_PARTS[kind])}")
    return _PARTS[kind][name](**arguments)


def registered_parts(kind: str):
    return sorted(_PARTS[kind])
