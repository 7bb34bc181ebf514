"""Python face of the HIP kernel library: checks tensors, passes raw pointers.

Every operation works on the current torch stream of the tensors' device. A
tensor of the wrong dtype, shape, layout or device is refused here, before a
kernel could read outside of it.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import build as _build

_CODES = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    """The kernel library refused an operation, or could not be loaded."""


def _code(tensor: torch.Tensor) -> int:
    if tensor.dtype not in _CODES:
        raise KernelError(f"unsupported element type {tensor.dtype}")
    return _CODES[tensor.dtype]


def _ptr(tensor: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if tensor is None else tensor.data_ptr())


ACTIVATIONS = {"silu": 0}   # gate activations of the gated product: name -> XRT_ACT_* code of the library
SQUARES_STRIDE = 64         # rows of a table of sums of squares (XRT_SQUARES_STRIDE of the library)


@dataclass
class Prescaled:
    """Rows of the residual stream on their way through an RMSNorm whose division is still to do:
    values[m, k] = bfloat16(x[m, k] * gain[k]) and squares[t, m] = the sum of x[m, k]^2 over the
    columns k of tile t (16 or fewer a tile, as the product that wrote them cut its columns). `linear`
    and `linear_glu` take it in place of the normed rows and divide the rows of their result by the
    rms; nothing else can read it."""
    values: torch.Tensor
    squares: torch.Tensor
    eps: float

    @property
    def shape(self):
        return self.values.shape


class _Packing(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int), ("gated_n", ctypes.c_int), ("head_dim", ctypes.c_int),
                ("rotated_heads", ctypes.c_int)]


PACK_TILES, PACK_GATED, PACK_ROTARY = 1, 2, 3


class PackedMatrix:
    """A bfloat16 weight matrix [rows, k] kept in tiles of 16 rows x 32 columns in the order in which the matrix
    cores take them (XRT_PACK_* of the library's header), so that products of few rows stream it faster.
    `linear`, `linear_glu`, `linear_qkv` and `embed` take it in place of the plain matrix; nothing else reads it."""

    def __init__(self, data: torch.Tensor, rows: int, cols: int, packing: _Packing):
        self.data, self.packing = data, packing
        self.shape = (rows, cols)
        self.dtype, self.device = data.dtype, data.device

    def dim(self) -> int:
        return 2

    def unpacked(self) -> torch.Tensor:
        """The matrix [rows, k] with rows contiguous along k again (for inspection and tests; products never need it)."""
        rows, cols = self.shape
        groups = (rows + 15) // 16
        by_packed_row = self.data.view(groups, cols // 32, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(groups * 16, cols)
        logical = torch.arange(rows, device=self.data.device)
        p = self.packing
        if p.kind == PACK_GATED:
            up = logical >= p.gated_n
            j = torch.where(up, logical - p.gated_n, logical)
            packed = j // 8 * 16 + up.long() * 8 + j % 8
        elif p.kind == PACK_ROTARY:
            head, d = logical // p.head_dim, logical % p.head_dim
            half, within = d // (p.head_dim // 2), d % (p.head_dim // 2)
            paired = head * p.head_dim + within // 8 * 16 + half * 8 + within % 8
            packed = torch.where(head < p.rotated_heads, paired, logical)
        else:
            packed = logical
        return by_packed_row[packed]


def _matrix(w):
    """(tensor that holds the data, packing argument) of a weight in either form."""
    if isinstance(w, PackedMatrix):
        return w.data, ctypes.byref(w.packing)
    return w, None


class _QkvFinish(ctypes.Structure):
    _fields_ = [("q_norm", ctypes.c_void_p), ("k_norm", ctypes.c_void_p), ("norm_dtype", ctypes.c_int),
                ("norm_eps", ctypes.c_float), ("rope_dim", ctypes.c_int), ("rope_table", ctypes.c_void_p),
                ("table_positions", ctypes.c_int)]


@dataclass
class QkvFinish:
    """What `attention` is to do to q, k and v before it uses them, in place of `qkv_prepare`: the head norms (weights
    [head_dim] each, or None), the rotation over the whole head (rope_table: what `rope_table` made of the rotation's
    theta and scale, [positions, head_dim / 2, 2], for at least the step's positions; None: no rotation), and the write
    of the step's keys and values into the cache."""
    q_norm: Optional[torch.Tensor] = None
    k_norm: Optional[torch.Tensor] = None
    norm_eps: float = 0.0
    rope_table: Optional[torch.Tensor] = None


class _LinearNorm(ctypes.Structure):
    _fields_ = [("squares_in", ctypes.c_void_p), ("tiles_in", ctypes.c_int), ("width_in", ctypes.c_int),
                ("eps", ctypes.c_float), ("scaled_out", ctypes.c_void_p), ("gain", ctypes.c_void_p),
                ("gain_dtype", ctypes.c_int), ("squares_out", ctypes.c_void_p)]


class HipOps:
    name = "hip"
    _instance = None
    QkvFinish = QkvFinish                       # (so that a part that holds the operations needs no import of this module)

    @classmethod
    def instance(cls) -> "HipOps":
        if cls._instance is None:
            cls._instance = cls()
        return cls._instance

    # Where the workspaces of kernels and the rows that one product hands to the next come from: None is torch; a
    # runtime that keeps a stretch of memory for the tensors of a step puts its own function here while a step runs.
    allocate = None

    def _empty(self, shape, dtype, device) -> torch.Tensor:
        if self.allocate is not None:
            return self.allocate(shape, dtype, device)
        return torch.empty(shape, dtype=dtype, device=device)

    def __init__(self):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the kernels of this library run on an MI355X only")
        path = _build.find_library()
        if path is None:
            try:
                path = _build.build()
            except _build.BuildError as error:
                raise KernelError(f"the HIP kernel library is missing and cannot be built: {error}") from None
        try:
            self.lib = ctypes.CDLL(path)
        except OSError as error:
            raise KernelError(f"cannot load {path}: {error}") from None
        self.path = path
        self.lib.xrt_last_error.restype = ctypes.c_char_p
        for name in ("xrt_embed", "xrt_add", "xrt_rmsnorm", "xrt_linear", "xrt_qkv_prepare",
                     "xrt_attention", "xrt_sample", "xrt_linear_takes_norm", "xrt_linear_norm_tiles", "xrt_linear_normed", "xrt_linear_qkv", "xrt_random_normal",
                     "xrt_linear_with", "xrt_pack_weight", "xrt_packing_suits", "xrt_block_tokens",
                     "xrt_attention_finishes_qkv", "xrt_attention_finishing", "xrt_rope_table"):
            getattr(self.lib, name).restype = ctypes.c_int
        from ..cache.allocator import BLOCK_TOKENS
        if int(self.lib.xrt_block_tokens()) != BLOCK_TOKENS:
            raise KernelError(f"{path} keeps {int(self.lib.xrt_block_tokens())} tokens in a cache block, "
                              f"the cache's bookkeeping {BLOCK_TOKENS}: library and package do not belong together")
        self.lib.xrt_linear_workspace.restype = ctypes.c_long
        self.lib.xrt_linear_whole_norm_workspace.restype = ctypes.c_long
        self.lib.xrt_attention_workspace.restype = ctypes.c_long
        self.lib.xrt_probe_read_bytes.restype = ctypes.c_long
        self.lib.xrt_sample_workspace.restype = ctypes.c_long

    # -- helpers -------------------------------------------------------------
    def _check(self, status: int) -> None:
        if status != 0:
            raise KernelError(self.lib.xrt_last_error().decode())

    @staticmethod
    def _stream(tensor: torch.Tensor):
        return ctypes.c_void_p(torch.cuda.current_stream(tensor.device).cuda_stream)

    @staticmethod
    def _require(tensor: torch.Tensor, what: str, dtype=None, shape=None, like=None) -> None:
        if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda:
            raise KernelError(f"{what}: expected a tensor on the GPU")
        if like is not None and tensor.device != like.device:
            raise KernelError(f"{what}: on {tensor.device}, expected {like.device}")
        if not tensor.is_contiguous():
            raise KernelError(f"{what}: must be contiguous")
        if dtype is not None and tensor.dtype != dtype:
            raise KernelError(f"{what}: dtype {tensor.dtype}, expected {dtype}")
        if shape is not None and tuple(tensor.shape) != tuple(shape):
            raise KernelError(f"{what}: shape {tuple(tensor.shape)}, expected {tuple(shape)}")

    # -- operations ----------------------------------------------------------
    def embed(self, table, ids, out):
        vocab, hidden = table.shape
        tokens = ids.shape[0]
        data, packing = _matrix(table)
        self._require(data, "embed table")
        self._require(ids, "embed ids", torch.int32, (tokens,), data)
        self._require(out, "embed out", torch.float32, (tokens, hidden), data)
        self._check(self.lib.xrt_embed(_ptr(data), _code(data), packing, _ptr(ids), _ptr(out), tokens, hidden, vocab,
                                       self._stream(out)))

    def packing_suits(self, rows: int, cols: int) -> bool:
        """Whether a bfloat16 matrix of these sizes is better kept packed."""
        return bool(self.lib.xrt_packing_suits(int(rows), int(cols)))

    def pack(self, w: torch.Tensor, kind: str = "tiles", gated_n: int = 0, head_dim: int = 0, rotated_heads: int = 0):
        """w [rows, k] (bfloat16, on the GPU) in the packed layout `kind`: "tiles", "gated" (w is gate rows then
        up rows, gated_n each) or "rotary" (w is heads x head_dim rows, the first rotated_heads heads rotated over
        the whole head)."""
        self._require(w, "pack w", torch.bfloat16)
        if w.dim() != 2:
            raise KernelError("pack: w must be [rows, k]")
        rows, cols = w.shape
        code = {"tiles": PACK_TILES, "gated": PACK_GATED, "rotary": PACK_ROTARY}.get(kind)
        if code is None:
            raise KernelError(f"pack: unknown kind {kind!r}")
        packing = _Packing(code, int(gated_n), int(head_dim), int(rotated_heads))
        data = torch.empty(((rows + 15) // 16 * 16) * cols, dtype=torch.bfloat16, device=w.device)
        self._check(self.lib.xrt_pack_weight(_ptr(w), _ptr(data), rows, cols, ctypes.byref(packing), self._stream(w)))
        return PackedMatrix(data, rows, cols, packing)

    def random_normal(self, out, key: int, scale: float, offset: float = 0.0):
        """out[i] = element i of the random-weights stream `key` (weights/random_init.py), times scale, plus offset."""
        self._require(out, "random_normal out")
        self._check(self.lib.xrt_random_normal(_ptr(out), _code(out), ctypes.c_long(out.numel()),
                                               ctypes.c_ulonglong(key & ((1 << 64) - 1)), ctypes.c_float(scale),
                                               ctypes.c_float(offset), self._stream(out)))

    def probe_read(self, buffer, nontemporal: bool = False) -> int:
        """Read `buffer` once and write nothing; returns the bytes read (a little under the buffer's size)."""
        self._require(buffer, "probe buffer")
        sink = torch.zeros(1, dtype=torch.int32, device=buffer.device)
        size = buffer.numel() * buffer.element_size()
        self._check(self.lib.xrt_probe_read(_ptr(buffer), ctypes.c_long(size), int(nontemporal), _ptr(sink),
                                            self._stream(buffer)))
        return int(self.lib.xrt_probe_read_bytes(ctypes.c_long(size)))

    def probe_mfma(self, iterations: int, device, random_operands: bool = False) -> int:
        """Matrix-core products on tiles held in registers; returns the flops done."""
        sink = torch.zeros(1, dtype=torch.float32, device=device)
        self._check(self.lib.xrt_probe_mfma(ctypes.c_long(iterations), int(random_operands), _ptr(sink), self._stream(sink)))
        return 512 * 4 * iterations * 4 * 2 * 32 * 32 * 16

    def add(self, residual, delta):
        self._require(residual, "add residual", torch.float32)
        self._require(delta, "add delta", None, residual.shape, residual)
        self._check(self.lib.xrt_add(_ptr(residual), _ptr(delta), _code(delta),
                                     ctypes.c_long(residual.numel()), self._stream(residual)))

    def rmsnorm(self, x, weight, eps, out, rows=None):
        hidden = x.shape[-1]
        self._require(x, "rmsnorm x", torch.float32)
        if x.dim() != 2:
            raise KernelError("rmsnorm x: expected [rows, hidden]")
        n_rows = x.shape[0] if rows is None else rows.shape[0]
        self._require(weight, "rmsnorm weight", None, (hidden,), x)
        self._require(out, "rmsnorm out", None, (n_rows, hidden), x)
        if rows is not None:
            self._require(rows, "rmsnorm rows", torch.int32, (n_rows,), x)
        self._check(self.lib.xrt_rmsnorm(_ptr(x), _ptr(weight), _code(weight), ctypes.c_float(eps), _ptr(out),
                                         _code(out), _ptr(rows), n_rows, hidden, self._stream(x)))

    def _linear(self, a, w, out, coded_mode, n, then_norm=None):
        mode = coded_mode & 255                 # what rides above is a gated product's activation
        scaled = a if isinstance(a, Prescaled) else None
        if scaled is not None:
            a = scaled.values
        if a.dim() != 2 or w.dim() != 2:
            raise KernelError("linear: operands must be [rows, k]")
        m, k = a.shape
        data, packing = _matrix(w)
        self._require(a, "linear a")
        self._require(data, "linear w", a.dtype, None, a)
        if w.shape[1] != k:
            raise KernelError(f"linear: a has {k} columns, w has {w.shape[1]}")
        if w.shape[0] != (2 * n if mode == 2 else n):
            raise KernelError(f"linear: w has {w.shape[0]} rows for {n} outputs")
        self._require(out, "linear out", None, (m, n), a)
        sizes = (_ptr(a), _ptr(data), _code(a))
        packed = (_ptr(a), _ptr(data), packing, _code(a))
        # the norm after an accumulating product: only if that product, and one of the same rows
        # over the n columns it writes, can take it
        emit = None
        takes = int(self.lib.xrt_linear_takes_norm(*packed, m, n, k, mode)) if then_norm is not None and mode == 1 and n % 8 == 0 else 0
        if takes == 2 and scaled is None and out.dtype == torch.float32:
            # many rows: the product's second kernel adds its parts and writes the rows' norm outright
            gain, eps = then_norm
            self._require(gain, "norm gain", None, (n,), a)
            normed = self._empty((m, n), torch.bfloat16, a.device)
            norm = _LinearNorm()
            norm.eps = float(eps)
            norm.scaled_out, norm.gain, norm.gain_dtype = normed.data_ptr(), gain.data_ptr(), _code(gain)
            need = int(self.lib.xrt_linear_whole_norm_workspace(*sizes, m, n, k, mode))
            workspace = self._empty(need, torch.float32, a.device)
            self._check(self.lib.xrt_linear_normed(*packed, _ptr(out), _code(out), m, n, k, coded_mode, ctypes.byref(norm),
                                                   _ptr(workspace), ctypes.c_long(need), self._stream(a)))
            return normed
        if takes == 1:
            gain, eps = then_norm
            self._require(gain, "norm gain", None, (n,), a)
            emit = Prescaled(self._empty((m, n), torch.bfloat16, a.device),
                             self._empty((int(self.lib.xrt_linear_norm_tiles(*packed, m, n, k)), SQUARES_STRIDE), torch.float32, a.device),
                             float(eps))
        if scaled is not None or emit is not None:
            norm = _LinearNorm()
            if scaled is not None:
                tiles = scaled.squares.shape[0]         # as many as the product that wrote them had tiles of columns
                self._require(scaled.squares, "sums of squares", torch.float32, (tiles, SQUARES_STRIDE), a)
                norm.squares_in, norm.tiles_in, norm.width_in, norm.eps = scaled.squares.data_ptr(), tiles, k, scaled.eps
            if emit is not None:
                norm.scaled_out, norm.squares_out = emit.values.data_ptr(), emit.squares.data_ptr()
                norm.gain, norm.gain_dtype = then_norm[0].data_ptr(), _code(then_norm[0])
            need = int(self.lib.xrt_linear_workspace(*sizes, m, n, k, mode))
            workspace = self._empty(need, torch.float32, a.device) if need > 0 else None
            self._check(self.lib.xrt_linear_normed(*packed, _ptr(out), _code(out), m, n, k, coded_mode, ctypes.byref(norm),
                                                   _ptr(workspace), ctypes.c_long(need), self._stream(a)))
            return emit
        need = int(self.lib.xrt_linear_workspace(*sizes, m, n, k, mode))
        workspace = self._empty(need, torch.float32, a.device) if need > 0 else None
        self._check(self.lib.xrt_linear_with(*packed, _ptr(out), _code(out), m, n, k, coded_mode,
                                             _ptr(workspace), ctypes.c_long(need), self._stream(a)))
        return None

    def linear(self, a, w, out, accumulate=False, then_norm: Optional[Tuple[torch.Tensor, float]] = None):
        """out (+)= a w^T. `a` may be a Prescaled. then_norm = (gain, eps) of an RMSNorm that follows an
        accumulating product: if this product can, it returns the normed rows of the updated `out` for the
        product after the norm (a Prescaled, whose division that product does; with many rows the normed
        rows themselves); None means that the caller runs the norm."""
        return self._linear(a, w, out, 1 if accumulate else 0, w.shape[0], then_norm)

    def linear_glu(self, a, w_gate_up, out, activation: str = "silu"):
        """out = act(a w_gate^T) * (a w_up^T) with w_gate_up = [gate rows | up rows]."""
        if w_gate_up.shape[0] % 2 != 0:
            raise KernelError("linear_glu: the weight needs gate rows followed by as many up rows")
        if activation not in ACTIVATIONS:
            raise KernelError(f"linear_glu: activation must be one of {sorted(ACTIVATIONS)}, found {activation!r}")
        self._linear(a, w_gate_up, out, 2 | (ACTIVATIONS[activation] << 8), w_gate_up.shape[0] // 2)

    def _prepare_arguments(self, qkv, n_heads, n_kv_heads, head_dim, positions, slots, q_norm, k_norm, norm_eps,
                           rope_theta, rope_dim, rope_scale, kv, longest_run):
        """Checks the operands of qkv_prepare; returns the C arguments from n_heads to longest_run."""
        tokens = qkv.shape[0]
        width = (n_heads + 2 * n_kv_heads) * head_dim
        self._require(qkv, "qkv", None, (tokens, width))
        self._require(positions, "positions", torch.int32, (tokens,), qkv)
        self._require(slots, "slots", torch.int32, (tokens,), qkv)
        if (q_norm is None) != (k_norm is None):
            raise KernelError("qkv_prepare: q_norm and k_norm come together")
        norm_code = 0
        if q_norm is not None:
            self._require(q_norm, "q_norm", None, (head_dim,), qkv)
            self._require(k_norm, "k_norm", q_norm.dtype, (head_dim,), qkv)
            norm_code = _code(q_norm)
        if rope_theta is not None:
            self._require(rope_theta, "rope_theta", torch.float32, (rope_dim // 2,), qkv)
        k_cache = v_cache = table = None
        stride = n_blocks = 0
        if kv is not None:
            k_cache, v_cache, table, stride, n_blocks = self._kv(kv, qkv, n_kv_heads, head_dim)
        return (n_heads, n_kv_heads, head_dim, _ptr(positions), _ptr(slots),
                _ptr(q_norm), _ptr(k_norm), norm_code, ctypes.c_float(norm_eps), _ptr(rope_theta), int(rope_dim),
                ctypes.c_float(rope_scale), _ptr(k_cache), _ptr(v_cache), _ptr(table), stride, n_blocks,
                int(longest_run))

    def qkv_prepare(self, qkv, n_heads, n_kv_heads, head_dim, positions, slots, q_norm=None, k_norm=None,
                    norm_eps=0.0, rope_theta=None, rope_dim=0, rope_scale=1.0, kv=None, longest_run=0):
        prepare = self._prepare_arguments(qkv, n_heads, n_kv_heads, head_dim, positions, slots, q_norm, k_norm,
                                          norm_eps, rope_theta, rope_dim, rope_scale, kv, longest_run)
        self._check(self.lib.xrt_qkv_prepare(_ptr(qkv), _code(qkv), qkv.shape[0], *prepare, self._stream(qkv)))

    def linear_qkv(self, a, w, qkv, n_heads, n_kv_heads, head_dim, positions, slots, q_norm=None, k_norm=None,
                   norm_eps=0.0, rope_theta=None, rope_dim=0, rope_scale=1.0, kv=None, longest_run=0):
        """qkv = a w^T, then qkv_prepare of it: one kernel where a step is short enough. `a` may be a Prescaled."""
        scaled = a if isinstance(a, Prescaled) else None
        if scaled is not None:
            a = scaled.values
        if a.dim() != 2 or w.dim() != 2:
            raise KernelError("linear_qkv: operands must be [rows, k]")
        m, k = a.shape
        data, packing = _matrix(w)
        self._require(a, "linear_qkv a")
        self._require(data, "linear_qkv w", a.dtype, None, a)
        if tuple(w.shape) != ((n_heads + 2 * n_kv_heads) * head_dim, k):
            raise KernelError(f"linear_qkv w: shape {tuple(w.shape)}, expected {((n_heads + 2 * n_kv_heads) * head_dim, k)}")
        self._require(qkv, "qkv", a.dtype, (m, w.shape[0]), a)
        prepare = self._prepare_arguments(qkv, n_heads, n_kv_heads, head_dim, positions, slots, q_norm, k_norm,
                                          norm_eps, rope_theta, rope_dim, rope_scale, kv, longest_run)
        norm = None
        if scaled is not None:
            tiles = scaled.squares.shape[0]
            self._require(scaled.squares, "sums of squares", torch.float32, (tiles, SQUARES_STRIDE), a)
            norm = _LinearNorm()
            norm.squares_in, norm.tiles_in, norm.width_in, norm.eps = scaled.squares.data_ptr(), tiles, k, scaled.eps
        need = int(self.lib.xrt_linear_workspace(_ptr(a), _ptr(data), _code(a), m, w.shape[0], k, 0))
        workspace = self._empty(need, torch.float32, a.device) if need > 0 else None
        self._check(self.lib.xrt_linear_qkv(_ptr(a), _ptr(data), packing, _code(a), _ptr(qkv), m, k,
                                            None if norm is None else ctypes.byref(norm), *prepare,
                                            _ptr(workspace), ctypes.c_long(need), self._stream(a)))

    def _kv(self, kv, like, n_kv_heads, head_dim):
        from ..cache import BLOCK_TOKENS
        n_blocks = kv.k.shape[0]
        self._require(kv.k, "key cache", like.dtype, (n_blocks, n_kv_heads, BLOCK_TOKENS, head_dim), like)
        if kv.v.dim() == 4 and kv.v.shape[2] != head_dim:
            raise KernelError(f"value cache: values of width {kv.v.shape[2]} beside keys of width {head_dim}: the attention "
                              "kernels of this library take values as wide as the keys (a mixer whose values differ "
                              "brings its own kernel and reads the cache's tensors itself)")
        self._require(kv.v, "value cache", like.dtype, (n_blocks, n_kv_heads, head_dim, BLOCK_TOKENS), like)
        self._require(kv.block_table, "block table", torch.int32, None, like)
        if kv.block_table.dim() != 2:
            raise KernelError("block table: expected [slots, blocks]")
        return kv.k, kv.v, kv.block_table, kv.block_table.shape[1], n_blocks

    def rope_table(self, theta: torch.Tensor, rope_dim: int, scale: float, positions: int) -> torch.Tensor:
        """float32 [positions, rope_dim / 2, 2]: cosine and sine of the angles position * scale / theta[i], as the kernels
        that rotate work them out; `attention(finish=...)` reads them instead of working them out again."""
        self._require(theta, "rope_theta", torch.float32, (rope_dim // 2,))
        table = torch.empty((positions, rope_dim // 2, 2), dtype=torch.float32, device=theta.device)
        self._check(self.lib.xrt_rope_table(_ptr(theta), int(rope_dim), ctypes.c_float(scale), int(positions), _ptr(table),
                                            self._stream(theta)))
        return table

    def attention_finishes_qkv(self, dtype, n_heads, n_kv_heads, head_dim, batch, window=None, rope_dim=0, rope_table=None) -> bool:
        """Whether `attention` can take this step's q, k and v as the projection left them (finish=...): a bfloat16 decode
        step with heads of 64 or 128 dims that are not rotated, or rotated whole with a table that covers the step's positions."""
        if dtype != torch.bfloat16 or getattr(batch, "sequence_offsets", None) is None:
            return False
        return bool(self.lib.xrt_attention_finishes_qkv(_CODES[dtype], n_heads, n_kv_heads, head_dim, int(window or 0),
                                                        int(batch.max_count), int(rope_dim),
                                                        0 if rope_table is None else int(rope_table.shape[0]), int(batch.max_context)))

    def attention(self, qkv, n_heads, n_kv_heads, head_dim, kv, batch, out, scale, window=None, distance_slopes=None,
                  finish: Optional[QkvFinish] = None):
        """Causal attention of the step's tokens over the cache. distance_slopes: float32 [n_heads], or None; a key at
        position j adds slope * (j - P) to the scaled score of the query at position P. finish: what is still to do to
        q, k and v (only where `attention_finishes_qkv` says so); the cache must be writable then."""
        from ..cache import BLOCK_TOKENS
        if finish is not None:
            return self._attention_finishing(qkv, n_heads, n_kv_heads, head_dim, kv, batch, out, scale, finish)
        tokens = qkv.shape[0]
        width = (n_heads + 2 * n_kv_heads) * head_dim
        self._require(qkv, "qkv", None, (tokens, width))
        self._require(out, "attention out", qkv.dtype, (tokens, n_heads * head_dim), qkv)
        self._require(batch.positions, "positions", torch.int32, (tokens,), qkv)
        self._require(batch.slots, "slots", torch.int32, (tokens,), qkv)
        k_cache, v_cache, table, stride, n_blocks = self._kv(kv, qkv, n_kv_heads, head_dim)
        if distance_slopes is not None:
            self._require(distance_slopes, "attention distance_slopes", torch.float32, (n_heads,), qkv)
        # the step's sequences, if the batch describes them: lets the matrix-core kernels run
        offsets = getattr(batch, "sequence_offsets", None)
        seq_slots = getattr(batch, "sequence_slots", None)
        starts = getattr(batch, "sequence_starts", None)
        n_seqs = max_count = max_context = 0
        workspace, workspace_floats = None, 0
        if offsets is not None and seq_slots is not None and starts is not None:
            n_seqs = int(batch.n_sequences)
            max_count, max_context = int(batch.max_count), int(batch.max_context)
            self._require(offsets, "sequence offsets", torch.int32, (n_seqs + 1,), qkv)
            self._require(seq_slots, "sequence slots", torch.int32, (n_seqs,), qkv)
            self._require(starts, "sequence starts", torch.int32, (n_seqs,), qkv)
            if max_context > stride * BLOCK_TOKENS:
                raise KernelError(f"attention: a sequence of {max_context} tokens exceeds the block table")
            workspace_floats = int(self.lib.xrt_attention_workspace(_code(qkv), tokens, n_heads, n_kv_heads, head_dim,
                                                                    int(window or 0), max_count, max_context))
            if workspace_floats > 0:
                workspace = self._empty(workspace_floats, torch.float32, qkv.device)
        self._check(self.lib.xrt_attention(
            _ptr(qkv), _code(qkv), tokens, n_heads, n_kv_heads, head_dim, _ptr(k_cache), _ptr(v_cache),
            _ptr(table), stride, n_blocks, _ptr(batch.positions), _ptr(batch.slots), _ptr(out),
            ctypes.c_float(scale), int(window or 0), _ptr(distance_slopes), _ptr(offsets), _ptr(seq_slots), _ptr(starts), n_seqs,
            max_count, max_context, _ptr(workspace), ctypes.c_long(workspace_floats), self._stream(qkv)))

    def _attention_finishing(self, qkv, n_heads, n_kv_heads, head_dim, kv, batch, out, scale, finish: QkvFinish):
        from ..cache import BLOCK_TOKENS
        tokens = qkv.shape[0]
        width = (n_heads + 2 * n_kv_heads) * head_dim
        self._require(qkv, "qkv", torch.bfloat16, (tokens, width))
        self._require(out, "attention out", qkv.dtype, (tokens, n_heads * head_dim), qkv)
        self._require(batch.positions, "positions", torch.int32, (tokens,), qkv)
        self._require(batch.slots, "slots", torch.int32, (tokens,), qkv)
        k_cache, v_cache, table, stride, n_blocks = self._kv(kv, qkv, n_kv_heads, head_dim)
        if int(batch.max_count) != 1 or int(batch.max_context) > stride * BLOCK_TOKENS:
            raise KernelError("attention (finishing q/k/v): a decode step whose sequences fit the block table")
        record = _QkvFinish()
        if (finish.q_norm is None) != (finish.k_norm is None):
            raise KernelError("attention (finishing q/k/v): q_norm and k_norm come together")
        if finish.q_norm is not None:
            self._require(finish.q_norm, "q_norm", None, (head_dim,), qkv)
            self._require(finish.k_norm, "k_norm", finish.q_norm.dtype, (head_dim,), qkv)
            record.q_norm, record.k_norm = finish.q_norm.data_ptr(), finish.k_norm.data_ptr()
            record.norm_dtype, record.norm_eps = _code(finish.q_norm), float(finish.norm_eps)
        if finish.rope_table is not None:
            positions = finish.rope_table.shape[0]
            self._require(finish.rope_table, "rope_table", torch.float32, (positions, head_dim // 2, 2), qkv)
            record.rope_dim, record.rope_table, record.table_positions = head_dim, finish.rope_table.data_ptr(), positions
        need = int(self.lib.xrt_attention_workspace(_code(qkv), tokens, n_heads, n_kv_heads, head_dim, 0, 1, int(batch.max_context)))
        workspace = self._empty(need, torch.float32, qkv.device) if need > 0 else None
        self._check(self.lib.xrt_attention_finishing(
            _ptr(qkv), _code(qkv), tokens, n_heads, n_kv_heads, head_dim, _ptr(k_cache), _ptr(v_cache), _ptr(table), stride,
            n_blocks, _ptr(batch.positions), _ptr(batch.slots), _ptr(out), ctypes.c_float(scale), ctypes.byref(record),
            int(batch.max_context), _ptr(workspace), ctypes.c_long(need), self._stream(qkv)))

    def sample(self, logits, out, temperature, top_k, top_p, penalty, history, history_spans, uniforms,
               small_top_k=False, append_at=None):
        """Row r's penalty reads history[history_spans[2r]:history_spans[2r + 1]]; with append_at, row r's
        token is also written to history[append_at[r]] (nowhere if negative).
        small_top_k: some row has a temperature and a top-k of 1 to 64, or a top-p without top-k: worth the
        kernels that look for candidates slice by slice."""
        if logits.dim() != 2:
            raise KernelError("sample: logits must be [rows, vocab]")
        rows, vocab = logits.shape
        self._require(logits, "logits", torch.float32)
        self._require(out, "sample out", torch.int32, (rows,), logits)
        for what, tensor, dtype, shape in (
                ("temperature", temperature, torch.float32, (rows,)), ("top_k", top_k, torch.int32, (rows,)),
                ("top_p", top_p, torch.float32, (rows,)), ("penalty", penalty, torch.float32, (rows,)),
                ("history_spans", history_spans, torch.int32, (2 * rows,)),
                ("uniforms", uniforms, torch.float32, (rows,)), ("history", history, torch.int32, None)):
            self._require(tensor, f"sample {what}", dtype, shape, logits)
        if append_at is not None:
            self._require(append_at, "sample append_at", torch.int32, (rows,), logits)
        need = int(self.lib.xrt_sample_workspace(rows, vocab)) if small_top_k else 0
        workspace = torch.empty(need, dtype=torch.uint8, device=logits.device) if need > 0 else None
        self._check(self.lib.xrt_sample(_ptr(logits), rows, vocab, _ptr(out), _ptr(temperature), _ptr(top_k),
                                        _ptr(top_p), _ptr(penalty), _ptr(history), _ptr(history_spans),
                                        _ptr(append_at), _ptr(uniforms), _ptr(workspace), ctypes.c_long(need), self._stream(logits)))
