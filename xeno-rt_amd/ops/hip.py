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


class _Recurrence(ctypes.Structure):
    _fields_ = [("q", ctypes.c_void_p), ("k", ctypes.c_void_p), ("v", ctypes.c_void_p),
                ("q_stride", ctypes.c_long), ("k_stride", ctypes.c_long), ("v_stride", ctypes.c_long),
                ("heads", ctypes.c_int), ("dim", ctypes.c_int), ("vdim", ctypes.c_int),
                ("q_scale", ctypes.c_float), ("k_scale", ctypes.c_float), ("decay_mode", ctypes.c_int),
                ("decay", ctypes.c_void_p), ("decay_bias", ctypes.c_void_p), ("decay_bias_dtype", ctypes.c_int),
                ("decay_power", ctypes.c_float), ("bonus", ctypes.c_void_p), ("bonus_dtype", ctypes.c_int),
                ("state", ctypes.c_void_p), ("norm", ctypes.c_int), ("eps", ctypes.c_float),
                ("norm_weight", ctypes.c_void_p), ("norm_weight_dtype", ctypes.c_int), ("norm_weight_per_head", ctypes.c_int),
                ("gate", ctypes.c_void_p), ("gate_stride", ctypes.c_long), ("gate_act", ctypes.c_int), ("out", ctypes.c_void_p),
                ("decay_stride", ctypes.c_long), ("decay_rate", ctypes.c_void_p), ("decay_rate_dtype", ctypes.c_int),
                ("qk_heads", ctypes.c_int), ("skip", ctypes.c_void_p), ("skip_dtype", ctypes.c_int),
                ("norm_groups", ctypes.c_int), ("gate_is_float32", ctypes.c_int), ("input_silu", ctypes.c_int),
                ("gate_after_norm", ctypes.c_int)]


class _SelectiveScan(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("x_stride", ctypes.c_long), ("dtype", ctypes.c_int),
                ("step", ctypes.c_void_p), ("step_stride", ctypes.c_long), ("step_bias", ctypes.c_void_p),
                ("b", ctypes.c_void_p), ("b_stride", ctypes.c_long), ("c", ctypes.c_void_p), ("c_stride", ctypes.c_long),
                ("a_log", ctypes.c_void_p), ("skip", ctypes.c_void_p), ("small_dtype", ctypes.c_int),
                ("gate", ctypes.c_void_p), ("gate_stride", ctypes.c_long), ("gate_dtype", ctypes.c_int),
                ("state", ctypes.c_void_p), ("out", ctypes.c_void_p), ("channels", ctypes.c_int), ("n", ctypes.c_int)]


CONV_MODES = {"plain": 0, "plus_input": 1, "towards_last": 2}          # XRT_CONV_* of the library
DECAY_MODES = {"per_head": 0, "given": 1, "exp_neg_exp": 2, "sigmoid_power": 3, "step": 4}      # XRT_DECAY_*
CONV_ACTIVATIONS = {None: 0, "silu": 1}                                # XRT_CONV_ACT_*
MOST_EXPERTS = 256                                                     # XRT_MOST_EXPERTS
UNARY = {"tanh": 0, "silu": 1, "xielu": 2}                             # XRT_UNARY_*


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
                     "xrt_attention_finishes_qkv", "xrt_attention_finishing", "xrt_rope_table", "xrt_short_conv",
                     "xrt_linear_recurrence", "xrt_add_normed", "xrt_activation", "xrt_rows_add", "xrt_kv_store",
                     "xrt_attention_general", "xrt_rmsnorm_conv_step", "xrt_attention_sigmoid", "xrt_qkv_complete",
                     "xrt_layernorm", "xrt_layernorm_shift", "xrt_add_layernormed", "xrt_short_conv_with", "xrt_selective_scan",
                     "xrt_bigram_add", "xrt_gated_rows", "xrt_add_weighted", "xrt_glu_clamped", "xrt_softcap", "xrt_cast",
                     "xrt_route_experts", "xrt_scale_blocks", "xrt_attention_stretches", "xrt_attention_stretches_accepts",
                     "xrt_experts_sort", "xrt_gather_rows", "xrt_linear_groups", "xrt_linear_groups_accepts", "xrt_experts_combine",
                     "xrt_linear_groups_tile_rows", "xrt_linear_groups_parts", "xrt_streams_open", "xrt_streams_read", "xrt_streams_write",
                     "xrt_latent_complete", "xrt_latent_queries", "xrt_linear_heads", "xrt_causal_softmax", "xrt_transpose", "xrt_attention_latent",
                     "xrt_attention_latent_accepts"):
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
        self.lib.xrt_linear_recurrence_workspace.restype = ctypes.c_long
        self.lib.xrt_attention_sigmoid_workspace.restype = ctypes.c_long
        self.lib.xrt_selective_scan_workspace.restype = ctypes.c_long
        self.lib.xrt_experts_sort_room.restype = ctypes.c_long
        self.lib.xrt_attention_latent_workspace.restype = ctypes.c_long

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

    def _kv(self, kv, like, n_kv_heads, head_dim, value_dim=None):
        from ..cache import BLOCK_TOKENS
        n_blocks = kv.k.shape[0]
        self._require(kv.k, "key cache", like.dtype, (n_blocks, n_kv_heads, BLOCK_TOKENS, head_dim), like)
        if value_dim is not None:
            self._require(kv.v, "value cache", like.dtype, (n_blocks, n_kv_heads, value_dim, BLOCK_TOKENS), like)
            self._require(kv.block_table, "block table", torch.int32, None, like)
            if kv.block_table.dim() != 2:
                raise KernelError("block table: expected [slots, blocks]")
            return kv.k, kv.v, kv.block_table, kv.block_table.shape[1], n_blocks
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
                  finish: Optional[QkvFinish] = None, value_dim: Optional[int] = None, sink=False,
                  distance_bias: Optional[torch.Tensor] = None, queries_alone: bool = False, chunk: Optional[int] = None):
        """Causal attention of the step's tokens over the cache. chunk: positions are cut into stretches of this many from a
        sequence's first token on, and a query sees the keys of its own stretch only. distance_slopes: float32 [n_heads], or None; a key at
        position j adds slope * (j - P) to the scaled score of the query at position P. distance_bias: float32
        [n_heads, span], or None; a key d tokens behind the query adds distance_bias[h, min(d, span - 1)]. queries_alone: the
        rows of `qkv` hold the queries only (keys and values are in the cache already). sink: True, or float32 [n_heads]: the softmax's
        denominator has one more term, exp(0) or exp of the head's number. finish: what is still to do to
        q, k and v (only where `attention_finishes_qkv` says so); the cache must be writable then."""
        from ..cache import BLOCK_TOKENS
        if finish is not None:
            return self._attention_finishing(qkv, n_heads, n_kv_heads, head_dim, kv, batch, out, scale, finish)
        if (queries_alone and sink is not True and distance_slopes is None and not window
                and self._attention_stretches(qkv, n_heads, n_kv_heads, head_dim, value_dim or head_dim, kv, batch, out, scale, chunk,
                                              distance_bias, sink if isinstance(sink, torch.Tensor) else None)):
            return None
        if (queries_alone and n_kv_heads == 1 and sink is not True and distance_bias is None and distance_slopes is None and not window and not chunk
                and self._attention_one_kv_head(qkv, n_heads, head_dim, value_dim or head_dim, kv, batch, out, scale,
                                                sink if isinstance(sink, torch.Tensor) else None)):
            return None
        if sink is not False or (value_dim is not None and value_dim != head_dim) or distance_bias is not None or queries_alone or chunk:
            return self._attention_general(qkv, n_heads, n_kv_heads, head_dim, value_dim or head_dim, kv, batch, out, scale, window,
                                           distance_slopes, sink, distance_bias, queries_alone, chunk)
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

    def _attention_one_kv_head(self, q, n_heads, head_dim, value_dim, kv, batch, out, scale, sink_scores) -> bool:
        """The matrix-core kernel for many query heads on one key/value head (the queries alone in `q`; bfloat16, key and value
        sizes that are multiples of 32 up to 512). False: not served here, and nothing was done."""
        tokens = q.shape[0]
        max_context = int(getattr(batch, "max_context", 0) or 0)
        if tokens > 65535 or max_context <= 0 or not self.lib.xrt_attention_latent_accepts(_code(q), 1, head_dim, value_dim):
            return False
        q_stride = self._rows(q, "attention q", n_heads * head_dim)
        if q_stride % 8 != 0 or q.data_ptr() % 16 != 0:
            return False
        self._require(out, "attention out", q.dtype, (tokens, n_heads * value_dim), q)
        self._require(batch.positions, "positions", torch.int32, (tokens,), q)
        self._require(batch.slots, "slots", torch.int32, (tokens,), q)
        k_cache, v_cache, table, stride, n_blocks = self._kv(kv, q, 1, head_dim, value_dim)
        if sink_scores is not None:
            self._require(sink_scores, "attention sink", torch.float32, (n_heads,), q)
        need = int(self.lib.xrt_attention_latent_workspace(ctypes.c_long(tokens), n_heads, value_dim, max_context))
        workspace = self._empty(need, torch.float32, q.device)
        self._check(self.lib.xrt_attention_latent(
            _ptr(q), ctypes.c_long(q_stride), ctypes.c_long(tokens), n_heads, head_dim, value_dim, _ptr(k_cache), _ptr(v_cache), _ptr(table), stride,
            n_blocks, _ptr(batch.positions), _ptr(batch.slots), _ptr(out), ctypes.c_float(scale), _ptr(sink_scores), max_context, _ptr(workspace),
            ctypes.c_long(need), self._stream(q)))
        return True

    def _attention_stretches(self, q, n_heads, n_kv_heads, head_dim, value_dim, kv, batch, out, scale, chunk, distance_bias=None,
                             sink_scores=None) -> bool:
        """The matrix-core kernel for a step that brings some sequence several tokens, the queries alone in `q`, every query
        seeing its own stretch of `chunk` positions (or, chunk None, all keys before it). False: not served here (another
        element type or head size, stretches that are not whole cache blocks, a step that is not described by sequences, or
        one token a sequence), and nothing was done."""
        offsets = getattr(batch, "sequence_offsets", None)
        seq_slots = getattr(batch, "sequence_slots", None)
        starts = getattr(batch, "sequence_starts", None)
        if offsets is None or seq_slots is None or starts is None or int(getattr(batch, "max_count", 0) or 0) <= 1:
            return False
        if not self.lib.xrt_attention_stretches_accepts(_code(q), head_dim, value_dim, int(chunk or 0)):
            return False
        tokens, n_seqs = q.shape[0], int(batch.n_sequences)
        if n_seqs <= 0 or n_seqs > tokens:
            return False
        q_stride = self._rows(q, "attention q", n_heads * head_dim)
        self._require(out, "attention out", q.dtype, (tokens, n_heads * head_dim), q)
        self._require(offsets, "sequence offsets", torch.int32, (n_seqs + 1,), q)
        self._require(seq_slots, "sequence slots", torch.int32, (n_seqs,), q)
        self._require(starts, "sequence starts", torch.int32, (n_seqs,), q)
        k_cache, v_cache, table, stride, n_blocks = self._kv(kv, q, n_kv_heads, head_dim, value_dim)
        from ..cache import BLOCK_TOKENS
        if int(batch.max_context) > stride * BLOCK_TOKENS:
            raise KernelError(f"attention: a sequence of {int(batch.max_context)} tokens exceeds the block table")
        counts = getattr(batch, "host_counts", None)
        if counts is None or sum(counts) < tokens:
            out.zero_()                       # padding rows: written by no one, read by the product that follows
        span = 0
        if distance_bias is not None:
            span = distance_bias.shape[-1]
            self._require(distance_bias, "attention distance_bias", torch.float32, (n_heads, span), q)
        if sink_scores is not None:
            self._require(sink_scores, "attention sink", torch.float32, (n_heads,), q)
        self._check(self.lib.xrt_attention_stretches(
            _ptr(q), ctypes.c_long(q_stride), _code(q), tokens, n_heads, n_kv_heads, head_dim, _ptr(k_cache), _ptr(v_cache), _ptr(table),
            stride, n_blocks, _ptr(offsets), _ptr(seq_slots), _ptr(starts), n_seqs, _ptr(out), ctypes.c_float(scale), int(chunk or 0),
            _ptr(distance_bias), int(span), _ptr(sink_scores), self._stream(q)))
        return True

    def _attention_general(self, qkv, n_heads, n_kv_heads, head_dim, value_dim, kv, batch, out, scale, window, distance_slopes, sink,
                           distance_bias=None, queries_alone=False, chunk=None):
        """Rows of qkv are [n_heads x head_dim | n_kv_heads x head_dim | n_kv_heads x value_dim] (or the queries alone), rows of
        out n_heads x value_dim. sink: the softmax's denominator has one more (a key without a value whose score is 0 or, if sink is
        a tensor float32 [n_heads], the head's number there)."""
        tokens = qkv.shape[0]
        q_stride = 0
        if queries_alone:
            q_stride = self._rows(qkv, "attention q", n_heads * head_dim)
        else:
            self._require(qkv, "qkv", None, (tokens, (n_heads + n_kv_heads) * head_dim + n_kv_heads * value_dim))
        span = 0
        if distance_bias is not None:
            span = distance_bias.shape[-1]
            self._require(distance_bias, "attention distance_bias", torch.float32, (n_heads, span), qkv)
        self._require(out, "attention out", qkv.dtype, (tokens, n_heads * value_dim), qkv)
        self._require(batch.positions, "positions", torch.int32, (tokens,), qkv)
        self._require(batch.slots, "slots", torch.int32, (tokens,), qkv)
        k_cache, v_cache, table, stride, n_blocks = self._kv(kv, qkv, n_kv_heads, head_dim, value_dim)
        if distance_slopes is not None:
            self._require(distance_slopes, "attention distance_slopes", torch.float32, (n_heads,), qkv)
        sink_scores = sink if isinstance(sink, torch.Tensor) else None
        if sink_scores is not None:
            self._require(sink_scores, "attention sink", torch.float32, (n_heads,), qkv)
        self._check(self.lib.xrt_attention_general(
            _ptr(qkv), _code(qkv), tokens, n_heads, n_kv_heads, head_dim, value_dim, _ptr(k_cache), _ptr(v_cache), _ptr(table), stride,
            n_blocks, _ptr(batch.positions), _ptr(batch.slots), _ptr(out), ctypes.c_float(scale), int(window or 0),
            _ptr(distance_slopes), int(sink is not False and sink is not None), _ptr(sink_scores), ctypes.c_long(q_stride), _ptr(distance_bias), int(span), int(chunk or 0),
            self._stream(qkv)))

    def attention_sigmoid(self, q, n_heads, n_kv_heads, head_dim, value_dim, kv, batch, out, scale, window=None, head_mix=None,
                          head_bias=None, gate=None):
        """Attention whose weights are sigmoid(score + head_bias[h]) of every visible key, not normalised over the keys. q: rows
        of n_heads x head_dim (they may be columns of a wider matrix); the keys and values of the step are in the cache already.
        head_mix: float32 [n_heads, n_heads], the heads' scaled scores of a (query, key) pair are multiplied by it before the
        sigmoid; head_bias: float32 [n_heads]; gate: float32 rows with one number per head (columns of a wider matrix, if
        need be): a head's output is multiplied by sigmoid(gate)."""
        from ..cache import BLOCK_TOKENS
        tokens = q.shape[0]
        q_stride = self._rows(q, "attention q", n_heads * head_dim)
        self._require(out, "attention out", q.dtype, (tokens, n_heads * value_dim), q)
        self._require(batch.positions, "positions", torch.int32, (tokens,), q)
        self._require(batch.slots, "slots", torch.int32, (tokens,), q)
        k_cache, v_cache, table, stride, n_blocks = self._kv(kv, q, n_kv_heads, head_dim, value_dim)
        if head_mix is not None:
            self._require(head_mix, "attention head_mix", torch.float32, (n_heads, n_heads), q)
        if head_bias is not None:
            self._require(head_bias, "attention head_bias", torch.float32, (n_heads,), q)
        gate_stride = 0 if gate is None else self._rows(gate, "attention gate", n_heads, torch.float32, q)
        # a step of few tokens is shared out among more workgroups, if the batch says how long its sequences are
        max_context = int(getattr(batch, "max_context", 0) or 0)
        if max_context > stride * BLOCK_TOKENS:
            raise KernelError(f"attention: a sequence of {max_context} tokens exceeds the block table")
        need = int(self.lib.xrt_attention_sigmoid_workspace(ctypes.c_long(tokens), n_heads, head_dim, value_dim, int(window or 0), max_context))
        workspace = self._empty(need, torch.float32, q.device) if need > 0 else None
        self._check(self.lib.xrt_attention_sigmoid(
            _ptr(q), ctypes.c_long(q_stride), _code(q), ctypes.c_long(tokens), n_heads, n_kv_heads, head_dim, value_dim, _ptr(k_cache),
            _ptr(v_cache), _ptr(table), stride, n_blocks, _ptr(batch.positions), _ptr(batch.slots), _ptr(out), ctypes.c_float(scale),
            int(window or 0), _ptr(head_mix), _ptr(head_bias), _ptr(gate), ctypes.c_long(gate_stride), max_context, _ptr(workspace),
            ctypes.c_long(need), self._stream(q)))

    def qkv_complete(self, proj, n_heads, n_kv_heads, head_dim, value_dim, batch, q_out, kv=None, biases=None, norms=None,
                     norm_eps=0.0, frequencies=None, rot_dims=0, neighbours=True, magnitude=1.0, values_in=None, values_out=None,
                     blend=None, plain_norm=False, query_temperature=None, queries_only=False):
        """What lies between an attention's projection and its scores. proj: float32 rows [q | k | v | ...] (the leading columns
        of the projection's output). biases: (q, k, v) vectors or None; norms: (q, k) weights [head_dim] of an RMS norm of every
        head, or None; frequencies: float32 [rot_dims / 2], the first rot_dims dims of every head of q and k turn by
        position * frequency in pairs of neighbours (or of halves), cosines and sines times magnitude; values_out: float32
        [tokens, n_kv_heads * value_dim] takes the values as projected; values_in (same shape) with blend (one number on the
        device): v <- (1 - blend) v + blend values_in. q goes to q_out (compute dtype), k and v into the cache `kv` (if given).
        plain_norm: every head of q and k is divided by its root mean square (no weights). query_temperature = (coef, every): the
        queries at position p times 1 + coef * ln(floor((p + 1) / every) + 1). queries_only: proj holds [q | ...] and only q_out
        is written (biases = (q's, None, None))."""
        tokens = proj.shape[0]
        width = n_heads * head_dim if queries_only else (n_heads + n_kv_heads) * head_dim + n_kv_heads * value_dim
        if proj.dim() != 2 or proj.shape[1] < width:
            raise KernelError(f"qkv_complete proj: {tuple(proj.shape)}, expected at least {width} columns")
        proj_stride = self._rows(proj, "qkv_complete proj", None, torch.float32)
        q_stride = self._rows(q_out, "qkv_complete q_out", n_heads * head_dim, None, proj)
        self._require(batch.positions, "positions", torch.int32, (tokens,), proj)
        self._require(batch.slots, "slots", torch.int32, (tokens,), proj)
        small = [t for t in (*(biases or ()), *(norms or ()), blend) if t is not None]
        small_dtype = small[0].dtype if small else torch.float32
        b_q = b_k = b_v = n_q = n_k = None
        if biases is not None:
            b_q, b_k, b_v = biases
            self._require(b_q, "qkv_complete bias of q", small_dtype, (n_heads * head_dim,), proj)
            if not queries_only:
                self._require(b_k, "qkv_complete bias of k", small_dtype, (n_kv_heads * head_dim,), proj)
                self._require(b_v, "qkv_complete bias of v", small_dtype, (n_kv_heads * value_dim,), proj)
        if norms is not None:
            n_q, n_k = norms
            self._require(n_q, "qkv_complete norm of q", small_dtype, (head_dim,), proj)
            self._require(n_k, "qkv_complete norm of k", small_dtype, (head_dim,), proj)
        if frequencies is not None:
            self._require(frequencies, "qkv_complete frequencies", torch.float32, (rot_dims // 2,), proj)
        for what, tensor in (("values_in", values_in), ("values_out", values_out)):
            if tensor is not None:
                self._require(tensor, f"qkv_complete {what}", torch.float32, (tokens, n_kv_heads * value_dim), proj)
        if values_in is not None:
            if blend is None or blend.numel() != 1:
                raise KernelError("qkv_complete: values to blend in need their share, one number on the device")
            self._require(blend, "qkv_complete blend", small_dtype, None, proj)
        k_cache = v_cache = table = None
        stride = n_blocks = 0
        if kv is not None:
            k_cache, v_cache, table, stride, n_blocks = self._kv(kv, q_out, n_kv_heads, head_dim, value_dim)
        temp_coef, temp_every = (0.0, 0) if query_temperature is None else (float(query_temperature[0]), int(query_temperature[1]))
        self._check(self.lib.xrt_qkv_complete(
            _ptr(proj), ctypes.c_long(proj_stride), _code(q_out), ctypes.c_long(tokens), n_heads, n_kv_heads, head_dim, value_dim,
            _ptr(b_q), _ptr(b_k), _ptr(b_v), _ptr(n_q), _ptr(n_k), ctypes.c_float(norm_eps), _CODES[small_dtype], _ptr(frequencies),
            int(rot_dims), int(bool(neighbours)), ctypes.c_float(magnitude), _ptr(values_in), _ptr(values_out), _ptr(blend),
            _ptr(batch.positions), _ptr(batch.slots), _ptr(q_out), ctypes.c_long(q_stride), _ptr(k_cache), _ptr(v_cache), _ptr(table),
            stride, n_blocks, int(bool(plain_norm)), ctypes.c_float(temp_coef), temp_every, int(bool(queries_only)), self._stream(proj)))

    # -- layer norm ---------------------------------------------------------------------------------
    def layernorm(self, x, weight, bias, eps, out, rows=None):
        """out = (x - mean) / sqrt(var + eps) * weight + bias over whole rows (only `rows` of x, if given); x float32."""
        hidden = x.shape[-1]
        self._require(x, "layernorm x", torch.float32)
        if x.dim() != 2:
            raise KernelError("layernorm x: expected [rows, hidden]")
        n_rows = x.shape[0] if rows is None else rows.shape[0]
        self._require(weight, "layernorm weight", None, (hidden,), x)
        self._require(bias, "layernorm bias", weight.dtype, (hidden,), x)
        self._require(out, "layernorm out", None, (n_rows, hidden), x)
        if rows is not None:
            self._require(rows, "layernorm rows", torch.int32, (n_rows,), x)
        self._check(self.lib.xrt_layernorm(_ptr(x), _ptr(weight), _ptr(bias), _code(weight), ctypes.c_float(eps), _ptr(out), _code(out),
                                           _ptr(rows), n_rows, hidden, self._stream(x)))

    def layernorm_shift(self, x, weight, bias, eps, mix, state, batch, out):
        """The layer norm h of every row, then out = h + (h of the token before - h) * mix along each sequence; state
        [slots, hidden] float32 holds the last h of every sequence (zeros when it starts) and is brought up to date."""
        tokens, hidden = x.shape
        self._require(x, "layernorm_shift x", torch.float32)
        self._require(weight, "layernorm_shift weight", None, (hidden,), x)
        self._require(bias, "layernorm_shift bias", weight.dtype, (hidden,), x)
        self._require(mix, "layernorm_shift mix", weight.dtype, (hidden,), x)
        self._require(state, "layernorm_shift state", torch.float32, (state.shape[0], hidden), x)
        self._require(out, "layernorm_shift out", None, (tokens, hidden), x)
        self._require(batch.slots, "slots", torch.int32, (tokens,), x)
        offsets, slots, n = self._sequences(batch, tokens, x)
        self._check(self.lib.xrt_layernorm_shift(_ptr(x), _ptr(weight), _ptr(bias), _ptr(mix), _code(weight), ctypes.c_float(eps),
                                                 _ptr(state), _ptr(batch.slots), offsets, slots, n, int(batch.max_count), _ptr(out),
                                                 _code(out), tokens, hidden, self._stream(x)))

    def add_layernormed(self, residual, y, weight, bias, eps, scale=1.0, pre_bias=None, then=None, then_out=None):
        """residual += scale * layer_norm(y + pre_bias); y float32 like residual. then = (weight, bias, eps) of a layer norm of
        the updated residual, written to then_out in the same pass."""
        self._require(residual, "add_layernormed residual", torch.float32)
        if residual.dim() != 2:
            raise KernelError("add_layernormed: a residual [rows, width]")
        rows, width = residual.shape
        self._require(y, "add_layernormed y", torch.float32, (rows, width), residual)
        self._require(weight, "add_layernormed weight", None, (width,), residual)
        self._require(bias, "add_layernormed bias", weight.dtype, (width,), residual)
        if pre_bias is not None:
            self._require(pre_bias, "add_layernormed pre_bias", weight.dtype, (width,), residual)
        next_w = next_b = None
        next_eps, out_code = 0.0, 0
        if then is not None:
            next_w, next_b, next_eps = then
            self._require(next_w, "add_layernormed next weight", weight.dtype, (width,), residual)
            self._require(next_b, "add_layernormed next bias", weight.dtype, (width,), residual)
            self._require(then_out, "add_layernormed then_out", None, (rows, width), residual)
            out_code = _code(then_out)
        self._check(self.lib.xrt_add_layernormed(_ptr(residual), _ptr(y), _ptr(pre_bias), _ptr(weight), _ptr(bias), _code(weight),
                                                 ctypes.c_float(eps), ctypes.c_float(scale), _ptr(next_w), _ptr(next_b),
                                                 ctypes.c_float(next_eps), _ptr(then_out if then is not None else None), out_code,
                                                 ctypes.c_long(rows), width, self._stream(residual)))

    # -- mixing along the sequence with state of fixed size ----------------------------
    def _rows(self, tensor, what, width=None, dtype=None, like=None):
        """A matrix whose rows are contiguous (it may be some columns of a wider one); returns its row stride."""
        if not isinstance(tensor, torch.Tensor) or not tensor.is_cuda or tensor.dim() != 2 or (tensor.shape[1] > 1 and tensor.stride(1) != 1):
            raise KernelError(f"{what}: expected a matrix on the GPU with contiguous rows")
        if like is not None and (tensor.device != like.device or tensor.shape[0] != like.shape[0]):
            raise KernelError(f"{what}: {tuple(tensor.shape)} on {tensor.device} does not go with {tuple(like.shape)} on {like.device}")
        if width is not None and tensor.shape[1] != width:
            raise KernelError(f"{what}: {tensor.shape[1]} columns, expected {width}")
        if dtype is not None and tensor.dtype != dtype:
            raise KernelError(f"{what}: dtype {tensor.dtype}, expected {dtype}")
        return int(tensor.stride(0)) if tensor.shape[0] > 1 else int(tensor.shape[1])

    def _sequences(self, batch, tokens, like):
        n = int(batch.n_sequences)
        self._require(batch.sequence_offsets, "sequence offsets", torch.int32, (n + 1,), like)
        self._require(batch.sequence_slots, "sequence slots", torch.int32, (n,), like)
        if int(batch.n_tokens) != tokens:
            raise KernelError(f"the step has {batch.n_tokens} tokens, the operand {tokens} rows")
        return _ptr(batch.sequence_offsets), _ptr(batch.sequence_slots), n

    def short_conv(self, x, w, state, batch, out, mode="plain", bias=None, activation=None):
        """out[o, t, c] = sum_j w[o, c, j] x[t - taps + 1 + j, c] along each sequence; state [slots, taps - 1, channels] (float32)
        holds what came before the step and is brought up to date. w is [channels, taps] or [n_out, channels, taps]; mode
        "plus_input" adds x, "towards_last" (w [n_out, channels], two taps) gives x + (x[t - 1] - x) * w."""
        if mode not in CONV_MODES:
            raise KernelError(f"short_conv: mode must be one of {sorted(CONV_MODES)}")
        tokens, channels = x.shape
        stride = self._rows(x, "short_conv x")
        if mode == "towards_last":
            taps, n_out = 2, (1 if w.dim() == 1 else w.shape[0])
            self._require(w, "short_conv w", None, (channels,) if w.dim() == 1 else (n_out, channels), x)
        else:
            taps, n_out = w.shape[-1], (1 if w.dim() == 2 else w.shape[0])
            self._require(w, "short_conv w", None, (channels, taps) if w.dim() == 2 else (n_out, channels, taps), x)
        self._require(state, "short_conv state", torch.float32, (state.shape[0], taps - 1, channels), x)
        self._require(out, "short_conv out", None, (tokens, channels) if out.dim() == 2 and n_out == 1 else (n_out, tokens, channels), x)
        if bias is not None:
            self._require(bias, "short_conv bias", w.dtype, (channels,) if n_out == 1 and bias.dim() == 1 else (n_out, channels), x)
        offsets, slots, n = self._sequences(batch, tokens, x)
        self._check(self.lib.xrt_short_conv_with(_ptr(x), _code(x), ctypes.c_long(tokens), ctypes.c_long(stride), channels, _ptr(w), _code(w),
                                                 taps, n_out, CONV_MODES[mode], _ptr(state), offsets, slots, n, int(batch.max_count),
                                                 _ptr(out), _code(out), _ptr(bias), CONV_ACTIVATIONS[activation], self._stream(x)))

    def rmsnorm_conv_step(self, x, weight, eps, conv_w, state, batch, out, plus_input=False):
        """`rmsnorm` of the rows of x, then `short_conv` of the normed rows (plain or plus the input), in one kernel and to the
        same bits: for a step in which every sequence brings exactly one token."""
        tokens, hidden = x.shape
        taps = conv_w.shape[-1]
        if int(batch.max_count) != 1 or int(batch.n_tokens) != tokens:
            raise KernelError("rmsnorm_conv_step: a step in which every sequence brings one token")
        self._require(x, "rmsnorm_conv_step x", torch.float32)
        self._require(weight, "rmsnorm_conv_step weight", None, (hidden,), x)
        self._require(conv_w, "rmsnorm_conv_step conv_w", None, (hidden, taps), x)
        self._require(state, "rmsnorm_conv_step state", torch.float32, (state.shape[0], taps - 1, hidden), x)
        self._require(out, "rmsnorm_conv_step out", None, (tokens, hidden), x)
        self._require(batch.slots, "slots", torch.int32, (tokens,), x)
        self._check(self.lib.xrt_rmsnorm_conv_step(_ptr(x), _ptr(weight), _code(weight), ctypes.c_float(eps), _ptr(out), _code(out), tokens,
                                                   hidden, _ptr(conv_w), _code(conv_w), taps, int(bool(plus_input)), _ptr(state),
                                                   _ptr(batch.slots), self._stream(x)))

    def linear_recurrence(self, q, k, v, state, batch, out, heads, dim, vdim, decay, decay_mode="per_head", decay_bias=None,
                          decay_power=1.0, q_scale=1.0, k_scale=1.0, bonus=None, norm_eps=None, norm_weight=None, gate=None,
                          gate_activation="silu", decay_rate=None, qk_heads=None, skip=None, norm_groups=None, input_activation=None,
                          gate_after_norm=False):
        """Per sequence and head S <- diag(decay) S + k v^T, o = S^T q (with `bonus` [heads, dim]: o = (S + diag(bonus) k v^T)^T q
        before the update); state [slots, heads, dim, vdim] float32. decay: float32 [heads] ("per_head") or [tokens, heads * dim]
        ("given": the decay itself; "exp_neg_exp": exp(-exp(z + bias)); "sigmoid_power": sigmoid(z + bias)^decay_power). Then per head
        o / sqrt(mean(o^2) + norm_eps) (if norm_eps is given), times norm_weight ([vdim] or [heads * vdim]), times gate
        (through silu, or "plain"; the gate's rows may be float32 beside bfloat16 operands).
        decay_mode "step": decay is float32 [tokens, heads] (columns of a wider matrix will do), a step size softplus(z + bias)
        per token and head with decay_bias [heads]; the head's channels all decay by exp(-exp(decay_rate[head]) * step) and v
        enters the state times the step. qk_heads: q and k have this many heads, shared by neighbouring heads in equal groups.
        skip [heads]: o += skip * v. norm_groups: the gate comes before the norm, which then spans each of that many equal
        parts of the token's whole row, with norm_weight [heads * vdim]; gate_after_norm: such a norm and its weight come first and
        the gate after them. gate_activation: "silu", "sigmoid" or "plain". input_activation "silu": q, k and v are silu of the rows given."""
        tokens = q.shape[0]
        record = _Recurrence()
        if input_activation not in (None, "silu"):
            raise KernelError(f"linear_recurrence: input_activation must be None or 'silu', found {input_activation!r}")
        record.input_silu, record.gate_after_norm = int(input_activation == "silu"), int(bool(gate_after_norm))
        if gate_after_norm and norm_groups is None:
            raise KernelError("linear_recurrence: a gate after the norm is served for a norm over parts of the whole row")
        qk = heads if qk_heads is None else int(qk_heads)
        record.qk_heads = qk
        record.q_stride = self._rows(q, "recurrence q", qk * dim)
        record.k_stride = self._rows(k, "recurrence k", qk * dim, q.dtype, q)
        record.v_stride = self._rows(v, "recurrence v", heads * vdim, q.dtype, q)
        record.q, record.k, record.v = q.data_ptr(), k.data_ptr(), v.data_ptr()
        record.heads, record.dim, record.vdim = heads, dim, vdim
        record.q_scale, record.k_scale = float(q_scale), float(k_scale)
        if decay_mode not in DECAY_MODES:
            raise KernelError(f"linear_recurrence: decay_mode must be one of {sorted(DECAY_MODES)}")
        record.decay_mode = DECAY_MODES[decay_mode]
        if decay_mode == "step":
            record.decay_stride = self._rows(decay, "recurrence steps", heads, torch.float32, q)
            if decay_rate is None:
                raise KernelError("linear_recurrence: decays from step sizes need a rate per head")
            self._require(decay_rate, "recurrence decay_rate", None, (heads,), q)
            record.decay_rate, record.decay_rate_dtype = decay_rate.data_ptr(), _code(decay_rate)
        else:
            self._require(decay, "recurrence decay", torch.float32, (heads,) if decay_mode == "per_head" else (tokens, heads * dim), q)
        record.decay = decay.data_ptr()
        if skip is not None:
            self._require(skip, "recurrence skip", None, (heads,), q)
            record.skip, record.skip_dtype = skip.data_ptr(), _code(skip)
        if norm_groups is not None:
            record.norm_groups = int(norm_groups)
        if decay_bias is not None:
            self._require(decay_bias, "recurrence decay_bias", None, (heads,) if decay_mode == "step" else (heads * dim,), q)
            record.decay_bias, record.decay_bias_dtype = decay_bias.data_ptr(), _code(decay_bias)
        record.decay_power = float(decay_power)
        if bonus is not None:
            self._require(bonus, "recurrence bonus", None, (heads, dim), q)
            record.bonus, record.bonus_dtype = bonus.data_ptr(), _code(bonus)
        self._require(state, "recurrence state", torch.float32, (state.shape[0], heads, dim, vdim), q)
        record.state = state.data_ptr()
        record.norm, record.eps = int(norm_eps is not None), float(norm_eps or 0.0)
        if norm_weight is not None:
            if tuple(norm_weight.shape) not in ((vdim,), (heads * vdim,)):
                raise KernelError(f"recurrence norm_weight: shape {tuple(norm_weight.shape)}, expected ({vdim},) or ({heads * vdim},)")
            self._require(norm_weight, "recurrence norm_weight", None, None, q)
            record.norm_weight, record.norm_weight_dtype = norm_weight.data_ptr(), _code(norm_weight)
            record.norm_weight_per_head = int(tuple(norm_weight.shape) == (heads * vdim,) and heads > 1)
        if gate is not None:
            record.gate_stride = self._rows(gate, "recurrence gate", heads * vdim, None, q)
            if gate.dtype not in (q.dtype, torch.float32):
                raise KernelError(f"recurrence gate: dtype {gate.dtype}, expected {q.dtype} or float32")
            record.gate_is_float32 = int(gate.dtype == torch.float32)
            record.gate, record.gate_act = gate.data_ptr(), {"plain": 0, "silu": 1, "sigmoid": 2}[gate_activation]
        self._require(out, "recurrence out", q.dtype, (tokens, heads * vdim), q)
        record.out = out.data_ptr()
        offsets, slots, n = self._sequences(batch, tokens, q)
        self._require(batch.slots, "slots", torch.int32, (tokens,), q)
        need = int(self.lib.xrt_linear_recurrence_workspace(n, int(batch.max_count), ctypes.c_long(tokens), heads, dim, vdim))
        workspace = self._empty(need, torch.float32, q.device)
        self._check(self.lib.xrt_linear_recurrence(ctypes.byref(record), _code(q), offsets, slots, n, int(batch.max_count),
                                                   _ptr(batch.slots), ctypes.c_long(tokens), _ptr(workspace), ctypes.c_long(need),
                                                   self._stream(q)))

    def selective_scan(self, x, step, b, c, state, batch, out, a_log, step_bias=None, skip=None, gate=None):
        """Per sequence and channel S[c, :] <- exp(dt A[c, :]) S[c, :] + dt x[t, c] b[t, :], y = S[c, :] . c[t, :] + skip[c] x[t, c],
        with dt = softplus(step[t, c] + step_bias[c]) and A = -exp(a_log) [channels, n]; out = y * silu(gate). x and out have
        the compute dtype; step [tokens, channels], b and c [tokens, n] are float32 (columns of wider matrices will do); state
        [slots, channels, n] float32; gate compute dtype or float32."""
        tokens, channels = x.shape
        n = a_log.shape[1]
        record = _SelectiveScan()
        record.x_stride, record.dtype, record.x = self._rows(x, "selective_scan x"), _code(x), x.data_ptr()
        record.step_stride, record.step = self._rows(step, "selective_scan step", channels, torch.float32, x), step.data_ptr()
        record.b_stride, record.b = self._rows(b, "selective_scan b", n, torch.float32, x), b.data_ptr()
        record.c_stride, record.c = self._rows(c, "selective_scan c", n, torch.float32, x), c.data_ptr()
        self._require(a_log, "selective_scan a_log", None, (channels, n), x)
        record.a_log, record.small_dtype = a_log.data_ptr(), _code(a_log)
        for what, tensor in (("step_bias", step_bias), ("skip", skip)):
            if tensor is not None:
                self._require(tensor, f"selective_scan {what}", a_log.dtype, (channels,), x)
                setattr(record, what, tensor.data_ptr())
        if gate is not None:
            record.gate_stride, record.gate_dtype, record.gate = self._rows(gate, "selective_scan gate", channels, None, x), _code(gate), gate.data_ptr()
        self._require(state, "selective_scan state", torch.float32, (state.shape[0], channels, n), x)
        self._require(out, "selective_scan out", x.dtype, (tokens, channels), x)
        record.state, record.out, record.channels, record.n = state.data_ptr(), out.data_ptr(), channels, n
        offsets, slots, n_seqs = self._sequences(batch, tokens, x)
        self._require(batch.slots, "slots", torch.int32, (tokens,), x)
        need = int(self.lib.xrt_selective_scan_workspace(n_seqs, int(batch.max_count), ctypes.c_long(tokens), channels, n))
        workspace = self._empty(need, torch.float32, x.device) if need > 0 else None
        self._check(self.lib.xrt_selective_scan(ctypes.byref(record), offsets, slots, n_seqs, int(batch.max_count), _ptr(batch.slots),
                                                ctypes.c_long(tokens), _ptr(workspace), ctypes.c_long(need), self._stream(x)))

    def bigram_add(self, x, scale, batch, table=None, before=None, buckets=0, mul_prev=0, mul_cur=0):
        """x <- x * scale + table[row]: row (token before * mul_prev + token * mul_cur) mod buckets, row `buckets` for a sequence's
        first token; before [slots] (int32) holds every sequence's last token of the step before and is brought up to date."""
        tokens, width = x.shape
        self._require(x, "bigram_add x", torch.float32)
        n_seqs = 0
        offsets = seq_slots = None
        if table is not None:
            self._require(table, "bigram_add table", None, (buckets + 1, width), x)
            self._require(before, "bigram_add before", torch.int32, None, x)
            self._require(batch.token_ids, "token ids", torch.int32, (tokens,), x)
            self._require(batch.positions, "positions", torch.int32, (tokens,), x)
            self._require(batch.slots, "slots", torch.int32, (tokens,), x)
            offsets, seq_slots, n_seqs = self._sequences(batch, tokens, x)
        self._check(self.lib.xrt_bigram_add(_ptr(x), ctypes.c_long(tokens), width, ctypes.c_float(scale), _ptr(table),
                                            0 if table is None else _code(table), int(buckets), int(mul_prev), int(mul_cur),
                                            _ptr(batch.token_ids), _ptr(batch.positions), _ptr(batch.slots), offsets, seq_slots, n_seqs,
                                            _ptr(before), self._stream(x)))

    def gated_rows(self, s, table, ids, offset, out):
        """out[t, c] = gelu_tanh(s[t, c]) * table[ids[t], offset + c]; s float32 [tokens, width]."""
        tokens, width = s.shape
        stride = self._rows(s, "gated_rows s", None, torch.float32)
        self._require(table, "gated_rows table", None, None, s)
        self._require(ids, "gated_rows ids", torch.int32, (tokens,), s)
        self._require(out, "gated_rows out", None, (tokens, width), s)
        if table.dim() != 2 or offset < 0 or offset + width > table.shape[1]:
            raise KernelError(f"gated_rows: columns {offset} to {offset + width} of a table {tuple(table.shape)}")
        self._check(self.lib.xrt_gated_rows(_ptr(s), ctypes.c_long(stride), _ptr(table), _code(table), ctypes.c_long(table.shape[1]),
                                            ctypes.c_long(offset), table.shape[0], _ptr(ids), _ptr(out), _code(out), ctypes.c_long(tokens),
                                            width, self._stream(s)))

    def add_weighted(self, residual, terms, copy=None):
        """residual += sum over (y, gain, scale) in terms of scale * gain * y; y float32 like residual, gain [width] or None; one to
        four terms. copy: a tensor shaped like residual that takes the updated rows in its own element type."""
        self._require(residual, "add_weighted residual", torch.float32)
        if residual.dim() != 2 or not 1 <= len(terms) <= 4:
            raise KernelError("add_weighted: a residual [rows, width] and one to four terms")
        rows, width = residual.shape
        gains = [gain for _, gain, _ in terms if gain is not None]
        for y, gain, _ in terms:
            self._require(y, "add_weighted y", torch.float32, (rows, width), residual)
            if gain is not None:
                self._require(gain, "add_weighted gain", gains[0].dtype, (width,), residual)
        count = len(terms)
        ys = (ctypes.c_void_p * count)(*[y.data_ptr() for y, _, _ in terms])
        gs = (ctypes.c_void_p * count)(*[0 if gain is None else gain.data_ptr() for _, gain, _ in terms])
        scales = (ctypes.c_float * count)(*[float(scale) for _, _, scale in terms])
        if copy is not None:
            self._require(copy, "add_weighted copy", None, (rows, width), residual)
        self._check(self.lib.xrt_add_weighted(_ptr(residual), count, ys, gs, scales, _code(gains[0]) if gains else 0, ctypes.c_long(rows),
                                              width, _ptr(copy), 0 if copy is None else _code(copy), self._stream(residual)))

    def glu_clamped(self, sums, out, limit, alpha, row_weights=None):
        """out = g * sigmoid(alpha g) * (u + 1) with g = min(sums[:, :n], limit), u = clamp(sums[:, n:], -limit, limit); every row
        times its entry of row_weights (float32, one number a row in any shape), if given."""
        rows, n = out.shape
        self._require(sums, "glu_clamped sums", torch.float32, (rows, 2 * n))
        self._require(out, "glu_clamped out", None, (rows, n), sums)
        if row_weights is not None:
            self._require(row_weights, "glu_clamped row_weights", torch.float32, None, sums)
            if row_weights.numel() != rows:
                raise KernelError(f"glu_clamped row_weights: {row_weights.numel()} numbers for {rows} rows")
        self._check(self.lib.xrt_glu_clamped(_ptr(sums), _ptr(out), _code(out), ctypes.c_long(rows), n, ctypes.c_float(limit),
                                             ctypes.c_float(alpha), _ptr(row_weights), self._stream(sums)))

    def softcap(self, x, cap):
        """x <- cap * tanh(x / cap), in place; x float32."""
        self._require(x, "softcap x", torch.float32)
        self._check(self.lib.xrt_softcap(_ptr(x), ctypes.c_long(x.numel()), ctypes.c_float(cap), self._stream(x)))

    def cast(self, x, out):
        """out = x in out's element type."""
        self._require(x, "cast x")
        self._require(out, "cast out", None, x.shape, x)
        self._check(self.lib.xrt_cast(_ptr(x), _code(x), _ptr(out), _code(out), ctypes.c_long(x.numel()), self._stream(x)))

    def route_experts(self, logits, weights, top, groups=1, keep=1, group_top=2, floor=1e-20, chosen=None, scores="sigmoid", scale=1.0):
        """From router logits [tokens, experts] (float32) the weights [tokens, experts] (float32; zero for experts not chosen):
        scores sigmoid(z) or, scores="softmax", softmax(z) over all experts; the chosen weights times `scale` in the end; experts in `groups` equal groups of neighbours, a group's score the sum of its group_top largest,
        experts of the `keep` best groups stay open; the `top` largest open scores are chosen and divided by their sum + floor.
        chosen (int32 [tokens, top], or None) takes the chosen experts in the order of their scores."""
        tokens, experts = logits.shape
        self._require(logits, "route_experts logits", torch.float32)
        self._require(weights, "route_experts weights", torch.float32, (tokens, experts), logits)
        if chosen is not None:
            self._require(chosen, "route_experts chosen", torch.int32, (tokens, top), logits)
        if scores not in ("sigmoid", "softmax"):
            raise KernelError(f"route_experts: scores are 'sigmoid' or 'softmax', found {scores!r}")
        self._check(self.lib.xrt_route_experts(_ptr(logits), ctypes.c_long(tokens), experts, int(top), int(groups), int(keep), int(group_top),
                                               ctypes.c_float(floor), _ptr(weights), _ptr(chosen), int(scores == "softmax"),
                                               ctypes.c_float(scale), self._stream(logits)))

    # -- a residual stream in several copies -----------------------------------------------------------
    def streams_open(self, x, streams):
        """streams [tokens, copies, width] (float32): every copy is the token's row of x [tokens, width] (float32)."""
        tokens, copies, width = streams.shape
        self._require(x, "streams_open x", torch.float32, (tokens, width))
        self._require(streams, "streams_open streams", torch.float32, None, x)
        self._check(self.lib.xrt_streams_open(_ptr(x), _ptr(streams), ctypes.c_long(tokens), width, copies, self._stream(x)))

    def streams_read(self, streams, weights, gain, eps, out, rows=None):
        """out[r] = norm(sum over the copies s of weights[s] * streams[rows[r] or r, s]): the norm is u / sqrt(mean(u^2) + eps) * gain,
        or, gain None, u itself. streams float32 [tokens, copies, width], weights float32 [copies]."""
        tokens, copies, width = streams.shape
        n_rows = tokens if rows is None else rows.shape[0]
        self._require(streams, "streams_read streams", torch.float32)
        self._require(weights, "streams_read weights", torch.float32, (copies,), streams)
        self._require(out, "streams_read out", None, (n_rows, width), streams)
        if gain is not None:
            self._require(gain, "streams_read gain", None, (width,), streams)
        if rows is not None:
            self._require(rows, "streams_read rows", torch.int32, (n_rows,), streams)
        self._check(self.lib.xrt_streams_read(_ptr(streams), copies, _ptr(weights), _ptr(gain), 0 if gain is None else _code(gain),
                                              ctypes.c_float(eps), _ptr(out), _code(out), _ptr(rows), ctypes.c_long(n_rows), width,
                                              self._stream(streams)))

    def streams_write(self, streams, mix, out_weights, y, then=None):
        """All copies at once from the old ones: copy t <- sum over s of mix[s, t] * copy s + out_weights[t] * y (y float32
        [tokens, width]). then = (weights, gain, eps, out): the read of the new copies (as `streams_read`) in the same pass."""
        tokens, copies, width = streams.shape
        self._require(streams, "streams_write streams", torch.float32)
        self._require(mix, "streams_write mix", torch.float32, (copies, copies), streams)
        self._require(out_weights, "streams_write out_weights", torch.float32, (copies,), streams)
        self._require(y, "streams_write y", torch.float32, (tokens, width), streams)
        weights = gain = out = None
        eps = 0.0
        if then is not None:
            weights, gain, eps, out = then
            self._require(weights, "streams_write next weights", torch.float32, (copies,), streams)
            self._require(out, "streams_write next out", None, (tokens, width), streams)
            if gain is not None:
                self._require(gain, "streams_write gain", None, (width,), streams)
        self._check(self.lib.xrt_streams_write(_ptr(streams), copies, _ptr(mix), _ptr(out_weights), _ptr(y), ctypes.c_long(tokens), width,
                                               _ptr(weights), _ptr(gain), 0 if gain is None else _code(gain), ctypes.c_float(eps), _ptr(out),
                                               0 if out is None else _code(out), self._stream(streams)))

    # -- attention through a latent -----------------------------------------------------------------------
    def latent_complete(self, down, rank, rot_dim, gain, eps, frequencies, rot_dims, kv, batch, like, rows_out=None):
        """From the float32 rows `down` [latent (rank) | key part (rot_dim)] (columns of a wider matrix will do): the latent divided
        by its root mean square, times gain, and the key part with its first rot_dims turned in pairs of neighbours by
        position * frequencies[pair], into the cache `kv` of one key/value head (keys rank + rot_dim wide, values rank wide), whose
        element type is that of `like`. rows_out ([tokens, rank + rot_dim] of that type, or None) takes the same rows once more."""
        tokens = down.shape[0]
        stride = self._rows(down, "latent_complete down", rank + rot_dim, torch.float32)
        if rows_out is not None:
            self._require(rows_out, "latent_complete rows_out", like.dtype, (tokens, rank + rot_dim), down)
        self._require(gain, "latent_complete gain", None, (rank,), down)
        if rot_dims:
            self._require(frequencies, "latent_complete frequencies", torch.float32, (rot_dims // 2,), down)
        self._require(batch.positions, "positions", torch.int32, (tokens,), down)
        self._require(batch.slots, "slots", torch.int32, (tokens,), down)
        k_cache, v_cache, table, table_stride, n_blocks = self._kv(kv, like, 1, rank + rot_dim, rank)
        self._check(self.lib.xrt_latent_complete(_ptr(down), ctypes.c_long(stride), _code(like), ctypes.c_long(tokens), rank, rot_dim, int(rot_dims),
                                                 _ptr(gain), _code(gain), ctypes.c_float(eps), _ptr(frequencies), _ptr(batch.positions),
                                                 _ptr(batch.slots), _ptr(k_cache), _ptr(v_cache), _ptr(table), table_stride, n_blocks,
                                                 _ptr(rows_out), self._stream(down)))

    def causal_softmax(self, scores, heads, first_position, scale, sinks, rounded, rest):
        """scores float32 [queries * heads, keys], row m the query at position first_position + m // heads of head m % heads:
        the softmax's weights over the keys at or before the query (score * scale; sinks float32 [heads] or None joins the
        denominator as exp(sinks[head])), zero behind it, into `rounded` and `rest` (bfloat16, same shape): the rounded weight and
        what the rounding left."""
        rows, keys = scores.shape
        self._require(scores, "causal_softmax scores", torch.float32)
        self._require(rounded, "causal_softmax rounded", torch.bfloat16, (rows, keys), scores)
        self._require(rest, "causal_softmax rest", torch.bfloat16, (rows, keys), scores)
        if sinks is not None:
            self._require(sinks, "causal_softmax sinks", torch.float32, (heads,), scores)
        self._check(self.lib.xrt_causal_softmax(_ptr(scores), ctypes.c_long(rows), ctypes.c_long(keys), int(heads), int(first_position),
                                                ctypes.c_float(scale), _ptr(sinks), _ptr(rounded), _ptr(rest), self._stream(scores)))

    def transpose(self, src, out):
        """out[c, r] = src[r, c]; the rows of src may be columns of a wider matrix."""
        rows, cols = src.shape
        stride = self._rows(src, "transpose src")
        self._require(out, "transpose out", src.dtype, (cols, rows), src)
        self._check(self.lib.xrt_transpose(_ptr(src), ctypes.c_long(stride), _code(src), ctypes.c_long(rows), cols, _ptr(out), self._stream(src)))

    def latent_queries(self, q, heads, dim, rot_dim, frequencies, rot_dims, batch, plain, full, rank):
        """From the float32 rows q of heads x [plain (dim) | part to turn (rot_dim)]: the plain parts to `plain` [tokens, heads * dim],
        the turned parts to the last rot_dim columns of every head of `full` [tokens, heads * (rank + rot_dim)]."""
        tokens = q.shape[0]
        stride = self._rows(q, "latent_queries q", heads * (dim + rot_dim), torch.float32)
        self._require(plain, "latent_queries plain", None, (tokens, heads * dim), q)
        self._require(full, "latent_queries full", plain.dtype, (tokens, heads * (rank + rot_dim)), q)
        if rot_dims:
            self._require(frequencies, "latent_queries frequencies", torch.float32, (rot_dims // 2,), q)
        self._require(batch.positions, "positions", torch.int32, (tokens,), q)
        self._check(self.lib.xrt_latent_queries(_ptr(q), ctypes.c_long(stride), _code(plain), ctypes.c_long(tokens), heads, dim, rot_dim,
                                                int(rot_dims), _ptr(frequencies), _ptr(batch.positions), _ptr(plain), _ptr(full),
                                                ctypes.c_long(heads * (rank + rot_dim)), rank, self._stream(q)))

    def linear_heads(self, a, w, out, out_head=None):
        """out[t, h, :n] = w[h] a[t, h]: a [tokens, heads * k], w [heads, n, k], out [tokens, heads * out_head] with the head's
        n outputs at the beginning of its out_head columns (out_head None: n). One element type, float32 sums in the order of k."""
        heads, n, k = w.shape
        tokens = a.shape[0]
        out_head = n if out_head is None else int(out_head)
        self._require(a, "linear_heads a", None, (tokens, heads * k))
        self._require(w, "linear_heads w", a.dtype, None, a)
        self._require(out, "linear_heads out", a.dtype, (tokens, heads * out_head), a)
        self._check(self.lib.xrt_linear_heads(_ptr(a), ctypes.c_long(heads * k), ctypes.c_long(k), _ptr(w), _code(a), _ptr(out),
                                              ctypes.c_long(heads * out_head), ctypes.c_long(out_head), ctypes.c_long(tokens), heads, n, k,
                                              self._stream(a)))

    # -- experts that multiply only the tokens that chose them
    def _expert_matrices(self, w_gate_up, w_down, experts, width, stacked=False):
        """(data, packing, elements between two experts' matrices, row distance) of the gate/up matrix and of the down matrix, as
        `xrt_linear_groups` wants them, or None: [all gates | all ups] packed for a gated epilogue lies expert after expert
        already (a group of sixteen packed rows holds eight outputs' gate and up rows); an expert's down matrix is `width`
        columns of the wide one. stacked: the gate/up matrix is a plain one that holds every expert's [gate rows | up rows] one
        below the other (for experts whose activation reads float32 sums of both)."""
        if width % 64 != 0:
            return None
        hidden = w_gate_up.shape[1]
        if stacked:
            if tuple(w_gate_up.shape) != (2 * experts * width, hidden) or tuple(w_down.shape) != (hidden, experts * width):
                return None
            if isinstance(w_gate_up, PackedMatrix):            # in tiles of 16 rows, an expert's rows (a multiple of 128) begin where they would unpacked
                if w_gate_up.packing.kind != PACK_TILES:
                    return None
                up = (w_gate_up.data, w_gate_up.packing, 2 * width * hidden, hidden)
            else:
                up = (w_gate_up, None, 2 * width * hidden, hidden)
        else:
            if not isinstance(w_gate_up, PackedMatrix) or w_gate_up.packing.kind != PACK_GATED:
                return None
            if w_gate_up.packing.gated_n != experts * width or tuple(w_down.shape) != (hidden, experts * width):
                return None
            up = (w_gate_up.data, _Packing(PACK_GATED, width, 0, 0), 2 * width * hidden, hidden)
        if isinstance(w_down, PackedMatrix):
            if w_down.packing.kind != PACK_TILES:
                return None
            down = (w_down.data, w_down.packing, width * 16, experts * width)
        else:
            down = (w_down, None, width, experts * width)
        return up, down

    def experts_sorted_takes(self, h, w_gate_up, w_down, experts, width, top, stacked=False) -> bool:
        """Whether `experts_sorted` serves these operands, and pays: it multiplies every pick once, in tiles that are filled up
        per expert, where the plain way multiplies every token with every expert. stacked: see `_expert_matrices`."""
        matrices = self._expert_matrices(w_gate_up, w_down, experts, width, stacked)
        if matrices is None or h.dtype != torch.bfloat16 or h.dim() != 2 or h.shape[1] % 64 != 0 or experts > 256:
            return False
        tokens, hidden = h.shape
        room = int(self.lib.xrt_experts_sort_room(ctypes.c_long(tokens), top, experts))
        if tokens < 64 or 4 * tokens * experts < 5 * room or room // 128 > 65535:
            return False
        (up, up_packing, _, up_rows), (down, down_packing, _, down_rows) = matrices
        takes_up = (self.lib.xrt_linear_groups_accepts(_ptr(h), hidden, _ptr(up), up_rows, 2 * width, hidden, 0,
                                                       None if up_packing is None else ctypes.byref(up_packing)) if stacked else
                    self.lib.xrt_linear_groups_accepts(_ptr(h), hidden, _ptr(up), up_rows, width, hidden, 2, ctypes.byref(up_packing)))
        return bool(takes_up and self.lib.xrt_linear_groups_accepts(_ptr(h), width, _ptr(down), down_rows, hidden, width, 0,
                                                           None if down_packing is None else ctypes.byref(down_packing)))

    def group_tile(self, tokens: int, top: int, experts: int) -> int:
        """Rows of a tile of sorted picks for a step of that many tokens."""
        return int(self.lib.xrt_linear_groups_tile_rows(ctypes.c_long(tokens), int(top), int(experts)))

    def experts_sorted(self, h, w_gate_up, w_down, weights, chosen, width, out, activation: str = "silu", clamp=None):
        """out[t] (float32) = sum over the experts e that token t chose, in the order of `chosen`, of weights[t, e] *
        W_down_e (act(W_gate_e h_t) * (W_up_e h_t)): the picks are sorted by expert, every expert multiplies its own rows, and
        the outputs go back to their tokens. A token's result does not depend on what else the step holds.
        clamp = (limit, alpha): the experts are clamped ones (`glu_clamped`) whose gate and up rows lie stacked expert after
        expert in a plain matrix; their product keeps float32 sums, and the clamps and the activation are a pass of their own."""
        tokens, hidden = h.shape
        experts, top = weights.shape[1], chosen.shape[1]
        matrices = self._expert_matrices(w_gate_up, w_down, experts, width, stacked=clamp is not None)
        if matrices is None:
            raise KernelError("experts_sorted: the experts' matrices do not lie expert after expert")
        (up, up_packing, up_stride, up_rows), (down, down_packing, down_stride, down_rows) = matrices
        self._require(h, "experts_sorted h", torch.bfloat16)
        self._require(weights, "experts_sorted weights", torch.float32, (tokens, experts), h)
        self._require(chosen, "experts_sorted chosen", torch.int32, (tokens, top), h)
        self._require(out, "experts_sorted out", torch.float32, (tokens, hidden), h)
        h_stride = self._rows(h, "experts_sorted h", hidden)
        stream, tile = self._stream(h), self.group_tile(tokens, top, experts)
        room = int(self.lib.xrt_experts_sort_room(ctypes.c_long(tokens), top, experts))
        index = self._empty(room + tokens * top + room // tile, torch.int32, h.device)
        rows, places, tile_group = index[:room], index[room:room + tokens * top], index[room + tokens * top:]
        self._check(self.lib.xrt_experts_sort(_ptr(chosen), ctypes.c_long(tokens), top, experts, _ptr(rows), ctypes.c_long(room), _ptr(places),
                                              _ptr(tile_group), stream))
        gathered = self._empty((room, hidden), torch.bfloat16, h.device)
        self._check(self.lib.xrt_gather_rows(_ptr(h), ctypes.c_long(h_stride), _ptr(rows), ctypes.c_long(room), hidden, _ptr(gathered), stream))
        act = self._empty((room, width), torch.bfloat16, h.device)
        if clamp is not None:
            sums = self._empty((room, 2 * width), torch.float32, h.device)
            self._check(self.lib.xrt_linear_groups(_ptr(gathered), hidden, _ptr(up), ctypes.c_long(up_stride), up_rows,
                                                   None if up_packing is None else ctypes.byref(up_packing), _ptr(sums), _code(sums),
                                                   tile, ctypes.c_long(room // tile), 2 * width, hidden, 0, _ptr(tile_group), 1, stream))
            self.glu_clamped(sums, act, float(clamp[0]), float(clamp[1]))
        else:
            self._check(self.lib.xrt_linear_groups(_ptr(gathered), hidden, _ptr(up), ctypes.c_long(up_stride), up_rows, ctypes.byref(up_packing),
                                                   _ptr(act), _code(act), tile, ctypes.c_long(room // tile), width, hidden,
                                                   2 | (ACTIVATIONS[activation] << 8), _ptr(tile_group), 1, stream))
        # (few tiles: the sum over an expert's width in two halves, which the last kernel adds)
        parts = int(self.lib.xrt_linear_groups_parts(ctypes.c_long(room // tile), hidden, width, 0))
        sorted_out = self._empty((room * parts, hidden), torch.float32, h.device)
        self._check(self.lib.xrt_linear_groups(_ptr(act), width, _ptr(down), ctypes.c_long(down_stride), down_rows,
                                               None if down_packing is None else ctypes.byref(down_packing), _ptr(sorted_out),
                                               _code(sorted_out), tile, ctypes.c_long(room // tile), hidden, width, 0, _ptr(tile_group), parts, stream))
        self._check(self.lib.xrt_experts_combine(_ptr(sorted_out), _ptr(places), _ptr(chosen), _ptr(weights), ctypes.c_long(tokens), top, experts,
                                                 hidden, tile, parts, _ptr(out), stream))

    def scale_blocks(self, act, weights, width):
        """act[t, e * width + c] *= weights[t, e], in place."""
        tokens, experts = weights.shape
        self._require(weights, "scale_blocks weights", torch.float32)
        self._require(act, "scale_blocks act", None, (tokens, experts * width), weights)
        self._check(self.lib.xrt_scale_blocks(_ptr(act), _code(act), _ptr(weights), ctypes.c_long(tokens), experts, int(width),
                                              self._stream(act)))

    def add_normed(self, residual, parts, eps, scale=1.0):
        """residual += scale * sum over (x, gain) in parts of x / sqrt(mean(x^2) + eps) * gain; x float32 like residual; one or two parts."""
        self._require(residual, "add_normed residual", torch.float32)
        if residual.dim() != 2 or not 1 <= len(parts) <= 2:
            raise KernelError("add_normed: a residual [rows, width] and one or two parts")
        rows, width = residual.shape
        for x, gain in parts:
            self._require(x, "add_normed x", torch.float32, (rows, width), residual)
            self._require(gain, "add_normed gain", parts[0][1].dtype, (width,), residual)
        (x0, g0), (x1, g1) = parts[0], (parts[1] if len(parts) == 2 else (None, None))
        self._check(self.lib.xrt_add_normed(_ptr(residual), _ptr(x0), _ptr(g0), _ptr(x1), _ptr(g1), _code(g0), ctypes.c_long(rows), width,
                                            ctypes.c_float(eps), ctypes.c_float(scale), self._stream(residual)))

    def activation(self, x, out, kind, params=None):
        """out = f(x) elementwise in float32: "tanh", "silu", or "xielu" with params = (p, q) on the device."""
        if kind not in UNARY:
            raise KernelError(f"activation: kind must be one of {sorted(UNARY)}")
        self._require(x, "activation x")
        self._require(out, "activation out", None, x.shape, x)
        if kind == "xielu":
            self._require(params, "activation params", None, (2,), x)
        self._check(self.lib.xrt_activation(_ptr(x), _code(x), _ptr(out), _code(out), ctypes.c_long(x.numel()), UNARY[kind],
                                            _ptr(params), 0 if params is None else _code(params), self._stream(x)))

    def rows_add(self, table, ids, out):
        """out[t] += table[ids[t]]; out float32 [tokens, width]."""
        rows, width = table.shape
        tokens = ids.shape[0]
        self._require(table, "rows_add table")
        self._require(ids, "rows_add ids", torch.int32, (tokens,), table)
        self._require(out, "rows_add out", torch.float32, (tokens, width), table)
        self._check(self.lib.xrt_rows_add(_ptr(table), _code(table), _ptr(ids), _ptr(out), ctypes.c_long(tokens), width, rows,
                                          self._stream(out)))

    def kv_store(self, k, v, n_kv_heads, head_dim, value_dim, kv, batch):
        """The step's keys k [tokens, n_kv_heads * head_dim] and values v [tokens, n_kv_heads * value_dim] into the cache."""
        tokens = k.shape[0]
        k_stride = self._rows(k, "kv_store k", n_kv_heads * head_dim)
        v_stride = self._rows(v, "kv_store v", n_kv_heads * value_dim, k.dtype, k)
        k_cache, v_cache, table, stride, n_blocks = self._kv(kv, k, n_kv_heads, head_dim, value_dim)
        self._require(batch.positions, "positions", torch.int32, (tokens,), k)
        self._require(batch.slots, "slots", torch.int32, (tokens,), k)
        self._check(self.lib.xrt_kv_store(_ptr(k), ctypes.c_long(k_stride), _ptr(v), ctypes.c_long(v_stride), _code(k), ctypes.c_long(tokens),
                                          n_kv_heads, head_dim, value_dim, _ptr(batch.positions), _ptr(batch.slots), _ptr(k_cache),
                                          _ptr(v_cache), _ptr(table), stride, n_blocks, self._stream(k)))

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
