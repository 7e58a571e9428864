"""The kernels as Python calls on torch tensors.

``load_ops()`` loads the compiled library (building it first if no up-to-date one
exists) and fails loudly when that is impossible: there is no fallback.  Each
method checks what only the Python side can know (device, dtype, contiguity), hands
raw pointers and the current HIP stream to the entry point, and raises
``KernelError`` with the library's message when it refuses its operands.
"""
from __future__ import annotations

import ctypes as C
import threading
from dataclasses import dataclass
from typing import Dict, Optional

import torch

from . import build as _build

XR_F32, XR_BF16 = 0, 1
_CODE = {torch.float32: XR_F32, torch.bfloat16: XR_BF16}
# activations of a gated feed-forward, by the code the kernels know them under (XR_ACT_* of common.h)
GATE_ACTIVATIONS = {"silu": 0, "clamped_swish": 1, "gelu_tanh": 2}
# gates that take a number of their own (``param``) and shape both branches (``gate_value`` of common.h)
SHAPED_GATES = {"clamped_swish"}
NORM_GATES = {"silu": 0, "sigmoid": 1}                  # XR_GATE_SILU / XR_GATE_SIGMOID of sequence_kernels.hip


class KernelError(RuntimeError):
    pass


@dataclass(frozen=True)
class Chunked:
    """In place of a window's length, where a step's attention work is planned: a position reads the keys of its own
    chunk of ``size`` positions, chunks counted from position 0 of its request."""
    size: int


def activation_code(name: str) -> int:
    try:
        return GATE_ACTIVATIONS[name]
    except KeyError:
        raise KernelError(f"gate activation {name!r} is not built into the kernels (known: {sorted(GATE_ACTIVATIONS)})") from None


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _CODE[dt]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dt}") from None


_p, _i, _f, _sz, _u32 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint32

_PROTOS = {
    "xr_embedding": [_p, _p, _p, _i, _i, _i, _f, _i, _i, _p],
    "xr_rmsnorm": [_p, _p, _p, _p, _i, _i, _i, _f, _i, _i, _p],
    "xr_rope_kv_write": [_p, _p, _p, _i, _p, _p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _p],
    "xr_gate_mul": [_p, _p, _i, _i, _i, _i, _i, _i, _f, _p],
    "xr_add": [_p, _p, _sz, _i, _f, _p],
    "xr_fill_rows": [_p, _p, _i, _sz, _u32, _p],
    "xr_fill_rows_many": [_p, _p, _i, _sz, _p, _i, _u32, _p],
    "xr_convert": [_p, _p, _sz, _i, _i, _p],
    "xr_stream_read": [_p, _sz, _p, _i, _p],
    "xr_gemm_ref": [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "xr_gemm_bf16": [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _p, _sz, _p, _p, _p],
    "xr_pack_weight": [_p, _p, _i, _i, _p],
    "xr_rope_table": [_p, _p, _p, _i, _i, _f, _p],
    "xr_attention_ref": [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _i, _p, _p, _p],
    "xr_attn_extra_partial": [_p, _p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _f, _i, _i, _i, _p, _p, _i, _p],
    "xr_decay_prepare": [_p, _i, _i, _i, _i, _i, _f, _p, _p, _p],
    "xr_head_gate": [_p, _p, _i, _i, _i, _i, _i, _p],
    "xr_pair_combine": [_p, _p, _p, _p, _p, _f, _f, _f, _i, _i, _i, _i, _p, _p, _f, _i, _p],
    "xr_add_rows": [_p, _p, _p, _f, _i, _i, _p],
    "xr_dyt_step": [_p, _p, _p, _p, _f, _f, _p, _p, _p, _f, _p, _i, _i, _i, _i, _i, _p],
    "xr_token_shift": [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _p],
    "xr_head_rmsnorm": [_p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _f, _f, _i, _p],
    "xr_moe_table_route": [_p, _p, _p, _p, _i, _i, _i, _i, _f, _p],
    "xr_sample": [_p, _p, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i, _p, _p],
    "xr_layernorm": [_p, _p, _p, _p, _i, _i, _i, _f, _i, _p],
    "xr_layernorm_conv": [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _f, _i, _p],
    "xr_causal_conv": [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "xr_polynorm": [_p, _p, _p, _i, _i, _i, _f, _i, _i, _p],
    "xr_rotate_rows": [_p, _p, _p, _i, _i, _i, _i, _i, _f, _p],
    "xr_gated_rmsnorm": [_p, _p, _p, _p, _i, _i, _i, _i, _f, _i, _i, _i, _p],
    "xr_act_rows": [_p, _i, _i, _i, _i, _p, _i, _p],
    "xr_embedding_pairs": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f, _i, _p],
    "xr_streams_expand": [_p, _p, _i, _i, _i, _p],
    "xr_streams_sum": [_p, _p, _i, _i, _i, _p],
    "xr_streams_step": [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _f, _i, _p],
    "xr_latent_prepare": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _f, _i, _p],
    "xr_moe_route": [_p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _f, _p],
    "xr_moe_experts_grouped": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p, _p],
    "xr_heads_gemm_bf16": [_p, _p, _p, _i, _i, _i, _i, _i, C.c_longlong, _i, C.c_longlong, _i, _p],
    "xr_moe_experts": [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "xr_delta_prepare": [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _f, _f, _p],
    "xr_linear_recurrence": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p, _p, _i, _f, _f, _p],
    "xr_qkv_store": [_p, _p, _p, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "xr_pool_blocks": [_p, _p, _p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p],
    "xr_attention_pool_partial": [_p, _p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _p],
    "xr_attention_pooled": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i, _p],
}

CONV_ACTIVATIONS = {None: 0, "none": 0, "silu": 1}      # XR_CONV_* of sequence_kernels.hip
RECURRENCES = {"retention": 0, "delta": 1, "wkv": 2, "gla": 3, "delta_channel": 4}    # XR_REC_* of recurrent_kernels.hip
ROW_ACTIVATIONS = {"silu": 1, "tanh": 2}                # what act_rows_ applies in place
EXPERT_ACTIVATIONS = {"relu2": 0, "swiglu": 1}          # MOE_ACT_* of moe_kernels.hip


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


class PackedWeight:
    """A bfloat16 weight matrix ``[rows, cols]`` in the order the MFMA kernels read it: blocks of
    16 rows x 32 columns, 1 KB each (``data[row group, column block, row, column]``), rows and
    columns padded with zeros.  Made by
    ``Ops.pack_weight``; ``Ops.linear`` and ``Ops.linear_gated`` take it in place of the matrix."""

    def __init__(self, data: torch.Tensor, rows: int, cols: int):
        self.data, self.rows, self.cols = data, rows, cols

    @property
    def shape(self):
        return (self.rows, self.cols)

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device


class UnscaledRows:
    """The rows of an RMSNorm that still lack their division by the root mean square:
    ``data [M, E]`` (bfloat16) holds ``x * weight``, ``sumsq [P, 16]`` partial sums of ``x^2`` per
    row (row t's sum is ``sumsq[:, t].sum()``), so the norm's row t is
    ``data[t] * rsqrt(sumsq[:, t].sum() / E + eps)``.  As that factor is one number a row, a
    product ``rows @ w^T`` may apply it to its result instead: ``Ops.linear`` and
    ``Ops.linear_gated`` take this in place of the rows.  Made by ``Ops.linear_add_rmsnorm``."""

    MAX_ROWS = 16

    def __init__(self, data: torch.Tensor, sumsq: torch.Tensor, eps: float):
        self.data, self.sumsq, self.eps = data, sumsq, eps

    @property
    def shape(self):
        return self.data.shape

    @property
    def dtype(self):
        return self.data.dtype

    @property
    def device(self):
        return self.data.device


class _GemmNorm(C.Structure):
    """XrGemmNorm of the library."""
    _fields_ = [("ss_in", _p), ("n_ss", _i), ("ss_inv_width", _f), ("ss_eps", _f), ("norm_w", _p),
                ("norm_w_bf16", _i), ("xg", _p), ("ss_out", _p), ("ss_out_rows", _i)]


class _GemmRope(C.Structure):
    """XrGemmRope of the library."""
    _fields_ = [("positions", _p), ("req_of_token", _p), ("block_table", _p), ("table_stride", _i),
                ("inv_freq", _p), ("H", _i), ("Hk", _i), ("D", _i), ("rot", _i), ("interleaved", _i),
                ("mscale", _f), ("page_size", _i), ("q_out", _p), ("k_cache", _p), ("v_cache", _p), ("cs_table", _p)]


def paired_order(D: int, rot: int) -> list:
    """``order[c]`` = the channel of a head that stands at column ``c`` in "paired order": a
    rotation's pairs ``(j, j + rot/2)`` side by side in groups of 16 columns (8 first halves, then
    their 8 partners), channels from ``rot`` on in place.  ``rot`` must be a multiple of 16."""
    if rot % 16 or rot > D:
        raise ValueError(f"paired order needs a rotary width that is a multiple of 16 and at most {D}, got {rot}")
    order = list(range(D))
    half = rot // 2
    for d in range(rot):
        hi, j = (1, d - half) if d >= half else (0, d)
        order[(j // 8) * 16 + hi * 8 + j % 8] = d
    return order


class _Lib:
    def __init__(self, path: str, protos: Dict[str, list]):
        self.path = path
        self.dll = C.CDLL(path)
        self.dll.xr_last_error.restype = C.c_char_p
        self.dll.xr_last_error.argtypes = []
        for name, args in protos.items():
            fn = getattr(self.dll, name)
            fn.argtypes = args
            fn.restype = C.c_int
            setattr(self, name, fn)

    def check(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self.dll.xr_last_error().decode("utf-8", "replace"))


class Ops:
    """All kernels of the forward pass and of sampling."""

    def __init__(self, lib: _Lib):
        self.lib = lib
        self._attn_libs: Dict[int, object] = {}
        self.use_mfma = True
        self.fold_norms = True      # False: linear_add_rmsnorm always runs the norm's own kernel
        self.fuse_rope = True       # False: project_rope_kv_write always runs two kernels
        self.ROPE_TILE_ROWS = int(lib.dll.xr_rope_tile_rows())
        self.FINISH_ROWS = self.ROPE_TILE_ROWS - 1

    # -- checks -----------------------------------------------------------------
    @staticmethod
    def _dev(*ts: Optional[torch.Tensor]) -> None:
        for t in ts:
            if t is not None and not t.is_cuda:
                raise KernelError("kernel operand is not on the GPU (there is no CPU path)")

    @staticmethod
    def _contig(t: torch.Tensor, what: str) -> None:
        if not t.is_contiguous():
            raise KernelError(f"{what} must be contiguous")

    # -- element-wise and row-wise ----------------------------------------------
    def embedding(self, table, ids: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        """``out[t] = table[ids[t]] * scale`` as 32-bit rows; ``table`` is a matrix or a ``PackedWeight``."""
        packed = isinstance(table, PackedWeight)
        data = table.data if packed else table
        self._dev(data, ids)
        self._contig(data, "embedding table")
        T, (V, E) = ids.numel(), table.shape
        out = torch.empty((T, E), dtype=torch.float32, device=data.device)
        self.lib.check(self.lib.xr_embedding(out.data_ptr(), data.data_ptr(), ids.data_ptr(), T, E, V,
                                             float(scale), dtype_code(data.dtype), 1 if packed else 0, _stream()))
        return out

    def rmsnorm(self, x: torch.Tensor, w: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """RMSNorm of the rows of 32-bit ``x`` (or of the rows ``rows`` selects)."""
        self._dev(x, w, rows)
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
            raise KernelError("rmsnorm input must be float32 [rows, width] with unit column stride")
        E = x.shape[1]
        if w is not None and (w.numel() != E or not w.is_contiguous()):
            raise KernelError(f"rmsnorm weight has {w.numel()} elements, the row has {E}")
        R = x.shape[0] if rows is None else rows.numel()
        out = torch.empty((R, E), dtype=out_dtype, device=x.device)
        self.lib.check(self.lib.xr_rmsnorm(out.data_ptr(), x.data_ptr(), _ptr(w), _ptr(rows), R, E, x.stride(0),
                                           float(eps), dtype_code(out_dtype),
                                           dtype_code(w.dtype) if w is not None else XR_F32, _stream()))
        return out

    def gate_mul(self, gu: torch.Tensor, activation: str = "silu", param: float = 0.0,
                 out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        """``act(gu[:, :F]) * gu[:, F:]`` for a gate of ``GATE_ACTIVATIONS``; for one of ``SHAPED_GATES`` the
        value the gate makes of both branches with its number ``param`` ("clamped_swish" with limit L:
        ``g' = min(g, L)``, ``u' = clamp(u, -L, L)``, ``g' sigmoid(1.702 g') (u' + 1)``).  32-bit branches may
        leave in ``out_dtype``."""
        self._dev(gu)
        T, F2 = gu.shape
        F = F2 // 2
        if gu.stride(1) != 1 or F2 % 2:
            raise KernelError("gate_mul input must be [rows, 2F] with unit column stride")
        code = activation_code(activation)
        out = torch.empty((T, F), dtype=out_dtype or gu.dtype, device=gu.device)
        self.lib.check(self.lib.xr_gate_mul(out.data_ptr(), gu.data_ptr(), T, F, gu.stride(0), dtype_code(gu.dtype),
                                            dtype_code(out.dtype), code, float(param), _stream()))
        return out

    def silu_mul(self, gu: torch.Tensor) -> torch.Tensor:
        """``silu(gu[:, :F]) * gu[:, F:]``."""
        return self.gate_mul(gu, "silu")

    def add_(self, x: torch.Tensor, y: torch.Tensor, scale: float = 1.0) -> None:
        """``x += scale * y`` with 32-bit ``x``."""
        self._dev(x, y)
        if x.dtype != torch.float32 or x.shape != y.shape:
            raise KernelError(f"add_: x must be float32 and shapes equal, got {x.dtype} {tuple(x.shape)} {tuple(y.shape)}")
        self._contig(x, "add_ x")
        self._contig(y, "add_ y")
        self.lib.check(self.lib.xr_add(x.data_ptr(), y.data_ptr(), x.numel(), dtype_code(y.dtype), float(scale), _stream()))

    def fill_rows_(self, base: torch.Tensor, rows: Optional[torch.Tensor], n_rows: int, value_bits: int = 0) -> None:
        """Set whole rows of ``base`` (first axis) to a 32-bit pattern."""
        self._dev(base, rows)
        self._contig(base, "fill_rows_ base")
        row_bytes = base[0].numel() * base.element_size()
        if row_bytes % 4:
            raise KernelError("fill_rows_: a row must be a multiple of 4 bytes")
        self.lib.check(self.lib.xr_fill_rows(base.data_ptr(), _ptr(rows), int(n_rows), row_bytes // 4,
                                             value_bits & 0xFFFFFFFF, _stream()))

    def row_filler(self, arrays):
        """A callable ``fill(rows, n_rows, value_bits=0)`` that sets the rows ``rows`` (device int32) of
        every array of ``arrays`` (first axis) to a 32-bit pattern in one launch; None if there are none."""
        arrays = list(arrays)
        if not arrays:
            return None
        self._dev(*arrays)
        words = []
        for t in arrays:
            self._contig(t, "row_filler array")
            row_bytes = t[0].numel() * t.element_size()
            if row_bytes % 4:
                raise KernelError("row_filler: a row must be a multiple of 4 bytes")
            words.append(row_bytes // 4)
        device = arrays[0].device
        bases = torch.tensor([t.data_ptr() for t in arrays], dtype=torch.int64, device=device)
        sizes = torch.tensor(words, dtype=torch.int64, device=device)

        def fill(rows: torch.Tensor, n_rows: int, value_bits: int = 0, _keep=(arrays, bases, sizes)) -> None:
            self.lib.check(self.lib.xr_fill_rows_many(bases.data_ptr(), sizes.data_ptr(), len(arrays), max(words),
                                                      rows.data_ptr(), int(n_rows), value_bits & 0xFFFFFFFF, _stream()))
        return fill

    def convert(self, x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
        self._dev(x)
        self._contig(x, "convert input")
        out = torch.empty(x.shape, dtype=dtype, device=x.device)
        self.lib.check(self.lib.xr_convert(out.data_ptr(), x.data_ptr(), x.numel(), dtype_code(x.dtype),
                                           dtype_code(dtype), _stream()))
        return out

    def stream_read(self, buf: torch.Tensor, blocks: int = 2048) -> torch.Tensor:
        """Read ``buf`` once, every workgroup a range of its own (the yardstick for what a kernel
        that only reads gets from memory); returns ``[blocks]`` int32 whose XOR is the XOR of the
        buffer's 32-bit words."""
        self._dev(buf)
        self._contig(buf, "stream_read buffer")
        sink = torch.empty((blocks,), dtype=torch.int32, device=buf.device)
        self.lib.check(self.lib.xr_stream_read(buf.data_ptr(), buf.numel() * buf.element_size(), sink.data_ptr(),
                                               blocks, _stream()))
        return sink

    # -- matrix product ---------------------------------------------------------
    GEMM_WORKSPACE_BYTES = 96 << 20
    ROPE_TILE_ROWS = 512    # from here the q/k/v product has tiles enough with K whole, and its tile kernel rotates and caches
    FINISH_ROWS = 511       # up to here the kernel that adds a product's K ranges up rotates and caches (the library's own number)

    def _gemm_workspace(self, device):
        """Room for the sums of K ranges when a product with few rows is split (one buffer per process;
        products on one stream use it one after another)."""
        ws = getattr(self, "_gemm_ws", None)
        if ws is None or ws.device != device:
            ws = torch.empty((self.GEMM_WORKSPACE_BYTES // 4,), dtype=torch.float32, device=device)
            self._gemm_ws = ws
        return ws.data_ptr(), self.GEMM_WORKSPACE_BYTES

    def _mfma_ok(self, a: torch.Tensor, w: torch.Tensor) -> bool:
        return (self.use_mfma and a.dtype == torch.bfloat16 and a.shape[1] % 8 == 0 and a.stride(0) % 8 == 0
                and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)

    def pack_weight(self, w: torch.Tensor, gated: bool = False):
        """``w`` for use as the weight of ``linear`` (``gated``: of ``linear_gated``): packed for
        the MFMA kernels where they will serve it (bfloat16, a width that is a multiple of 8, for
        gate and up rows a height that is a multiple of 32), else ``w`` itself."""
        if not (self.use_mfma and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % 8 == 0):
            return w
        N, K = w.shape
        if gated and N % 32:
            return w
        self._dev(w)
        self._contig(w, "pack_weight input")
        data = torch.empty((-(-N // 16), -(-K // 32), 16, 32), dtype=torch.bfloat16, device=w.device)
        self.lib.check(self.lib.xr_pack_weight(data.data_ptr(), w.data_ptr(), N, K, _stream()))
        return PackedWeight(data, N, K)

    def linear(self, a: torch.Tensor, w, bias: Optional[torch.Tensor] = None,
               out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None,
               accumulate: bool = False, variant: int = 0, _then: Optional[_GemmNorm] = None) -> torch.Tensor:
        """``a [M, K] @ w [N, K]^T (+ bias)``; with ``accumulate`` added into 32-bit ``out``.

        bfloat16 operands run on the matrix cores (32-bit accumulation); float32 operands, and
        shapes the MFMA kernels do not take, run the plain 32-bit FMA kernel.  ``w`` is a matrix
        or a ``PackedWeight``.
        """
        packed = isinstance(w, PackedWeight)
        wt = w.data if packed else w
        norm, a = self._norm_before(a, _then)
        self._dev(a, wt, bias, out)
        if a.dim() != 2 or len(w.shape) != 2 or a.shape[1] != w.shape[1]:
            raise KernelError(f"linear: shapes {tuple(a.shape)} x {tuple(w.shape)}^T do not fit")
        if a.dtype != w.dtype:
            raise KernelError(f"linear: input is {a.dtype}, weight is {w.dtype}")
        if a.stride(1) != 1:
            raise KernelError("linear: input must have unit column stride")
        self._contig(wt, "linear weight")
        M, K = a.shape
        N = w.shape[0]
        if out is None:
            if accumulate:
                raise KernelError("linear: accumulate needs an output")
            out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
        elif out.shape != (M, N) or out.stride(1) != 1:
            raise KernelError(f"linear: output is {tuple(out.shape)}, product is {(M, N)}")
        if bias is not None and (bias.dtype != torch.float32 or bias.numel() != N):
            raise KernelError("linear: bias must be float32 [N]")
        if self._mfma_ok(a, wt):
            self.lib.check(self.lib.xr_gemm_bf16(out.data_ptr(), a.data_ptr(), wt.data_ptr(), _ptr(bias), M, N, K,
                                                 a.stride(0), out.stride(0), dtype_code(out.dtype),
                                                 1 if accumulate else 0, 0, 0.0, variant, 1 if packed else 0,
                                                 *self._gemm_workspace(a.device),
                                                 C.addressof(norm) if norm is not None else None, None, _stream()))
            return out
        if norm is not None:
            raise KernelError("linear: rows that still lack their norm's scale need the MFMA kernels")
        if packed:
            raise KernelError("linear: a packed weight needs bfloat16 rows that are 16-byte aligned")
        self.lib.check(self.lib.xr_gemm_ref(out.data_ptr(), a.data_ptr(), w.data_ptr(), _ptr(bias), M, N, K,
                                            a.stride(0), out.stride(0), dtype_code(a.dtype),
                                            dtype_code(out.dtype), 1 if accumulate else 0, _stream()))
        return out

    @staticmethod
    def _norm_before(a, then: Optional[_GemmNorm]):
        """(what the library needs to know about a norm folded into this product, the rows)"""
        if not isinstance(a, UnscaledRows):
            return then, a
        if a.data.shape[0] > UnscaledRows.MAX_ROWS:
            raise KernelError(f"a product takes at most {UnscaledRows.MAX_ROWS} rows that still lack their norm's scale")
        norm = then if then is not None else _GemmNorm()
        norm.ss_in, norm.n_ss = a.sumsq.data_ptr(), a.sumsq.shape[0]
        norm.ss_inv_width, norm.ss_eps = 1.0 / a.data.shape[1], float(a.eps)
        return norm, a.data

    def linear_add_rmsnorm(self, a, w, residual: torch.Tensor, norm_weight: Optional[torch.Tensor], eps: float,
                           out_dtype: torch.dtype, bias: Optional[torch.Tensor] = None, defer: bool = False):
        """``residual += a @ w^T (+ bias)``, then the RMSNorm of the updated rows.

        With ``defer`` the caller says that what reads the result is a ``linear`` or
        ``linear_gated``: for at most 16 bfloat16 rows the product's kernel then also writes the
        weighted rows and their partial sums of squares, and an ``UnscaledRows`` comes back, whose
        scale the next product applies.  With more rows, where the product is split over K (always
        from 17 to 64 rows, above that when its tiles are too few for the chip), the kernel that adds up
        the K ranges takes whole rows and writes the finished norm.  In every other case the norm's own
        kernel runs.  A tensor comes back in both."""
        wt = w.data if isinstance(w, PackedWeight) else w
        rows = a.data if isinstance(a, UnscaledRows) else a
        M, N = rows.shape[0], w.shape[0]
        fits = (self.fold_norms and out_dtype == torch.bfloat16 and norm_weight is not None
                and N % 8 == 0 and norm_weight.numel() == N and norm_weight.is_contiguous()
                and residual.dtype == torch.float32 and self._mfma_ok(rows, wt))
        deferred = fits and defer and M <= UnscaledRows.MAX_ROWS
        # More rows: where the product is split over K (always from 17 to 64 rows, above that when
        # its tiles are too few for the chip), the kernel that adds the parts up takes whole rows and
        # writes the finished norm; the library says whether it did.
        whole = fits and M > UnscaledRows.MAX_ROWS and N % 4 == 0 and residual.stride(0) % 4 == 0
        if deferred or whole:
            self._dev(norm_weight)
            then = _GemmNorm()
            xg = torch.empty((M, N), dtype=torch.bfloat16, device=rows.device)
            parts = -(-N // 16)
            sumsq = torch.empty((parts, 16), dtype=torch.float32, device=rows.device) if deferred else None
            then.norm_w, then.norm_w_bf16 = norm_weight.data_ptr(), dtype_code(norm_weight.dtype)
            then.xg, then.ss_out, then.ss_out_rows = xg.data_ptr(), _ptr(sumsq), parts
            then.ss_inv_width, then.ss_eps = 1.0 / N, float(eps)
            self.linear(a, w, bias=bias, out=residual, accumulate=True, _then=then)
            if then.ss_out_rows < 0:
                return xg                                   # the finished norm
            if deferred:
                return UnscaledRows(xg, sumsq[:then.ss_out_rows], eps)
            return self.rmsnorm(residual, norm_weight, eps, out_dtype)      # the library declined
        self.linear(a, w, bias=bias, out=residual, accumulate=True)
        return self.rmsnorm(residual, norm_weight, eps, out_dtype)

    def linear_gated(self, a: torch.Tensor, w, bias: Optional[torch.Tensor] = None, activation: str = "silu",
                     variant: int = 0, param: float = 0.0) -> torch.Tensor:
        """``act(a @ w[:F]^T) * (a @ w[F:]^T)`` for ``w [2F, K]`` = gate rows then up rows
        (a matrix, or a ``PackedWeight`` made with ``gated=True``); ``activation`` is one of
        ``GATE_ACTIVATIONS``, with its number ``param`` for one of ``SHAPED_GATES``.  The matrix-core kernels
        apply the gate in their epilogue; where they do not serve (float32, sizes they do not take) the
        product leaves both branches in 32 bits and ``gate_mul`` makes the value of them."""
        act = activation_code(activation)
        packed = isinstance(w, PackedWeight)
        wt = w.data if packed else w
        norm, a = self._norm_before(a, None)
        F = w.shape[0] // 2
        if w.shape[0] % 2:
            raise KernelError("linear_gated: the weight must have an even number of rows")
        if self._mfma_ok(a, wt):
            self._dev(a, wt, bias)
            self._contig(wt, "linear_gated weight")
            M, K = a.shape
            if K != w.shape[1] or a.stride(1) != 1:
                raise KernelError(f"linear_gated: shapes {tuple(a.shape)} x {tuple(w.shape)}^T do not fit")
            if bias is not None and (bias.dtype != torch.float32 or bias.numel() != 2 * F):
                raise KernelError("linear_gated: bias must be float32 [2F]")
            out = torch.empty((M, F), dtype=a.dtype, device=a.device)
            self.lib.check(self.lib.xr_gemm_bf16(out.data_ptr(), a.data_ptr(), wt.data_ptr(), _ptr(bias), M, F, K,
                                                 a.stride(0), F, dtype_code(out.dtype), 2, act, float(param), variant,
                                                 1 if packed else 0, *self._gemm_workspace(a.device),
                                                 C.addressof(norm) if norm is not None else None, None, _stream()))
            return out
        if norm is not None:
            raise KernelError("linear_gated: rows that still lack their norm's scale need the MFMA kernels")
        if packed:
            raise KernelError("linear_gated: a packed weight needs bfloat16 rows that are 16-byte aligned")
        return self.gate_mul(self.linear(a, w, bias=bias, out_dtype=torch.float32), activation, param, out_dtype=a.dtype)

    def linear_swiglu(self, a: torch.Tensor, w, bias: Optional[torch.Tensor] = None, variant: int = 0) -> torch.Tensor:
        """``linear_gated`` with the SiLU gate."""
        return self.linear_gated(a, w, bias=bias, activation="silu", variant=variant)

    # -- attention --------------------------------------------------------------
    def rope_kv_write(self, q_in, k_in, v_in, q_out, k_cache, v_cache, positions, req_of_token,
                      block_table, inv_freq, H: int, Hk: int, D: int, rot: int, interleaved: bool,
                      mscale: float, page_size: int, paired: bool = False) -> None:
        """Rotate queries (into ``q_out``) and keys, and write keys and values to their pages.

        ``q_in``/``k_in``/``v_in`` are 32-bit views with one common row stride.  ``paired``: the
        channels of every query and key head come in ``paired_order``.
        """
        self._dev(q_in, k_in, v_in, q_out, k_cache, v_cache, positions, req_of_token, block_table, inv_freq)
        T = positions.numel()
        ins = [t for t in (q_in, k_in, v_in) if t is not None]
        if any(t.dtype != torch.float32 or t.stride(-1) != 1 for t in ins):
            raise KernelError("rope_kv_write: inputs must be float32 with unit column stride")
        strides = {t.stride(0) for t in ins}
        if len(strides) > 1:
            raise KernelError("rope_kv_write: q, k and v inputs must share a row stride")
        stride = strides.pop() if strides else 0
        store = q_out if q_out is not None else k_cache
        if k_cache is not None and q_out is not None and k_cache.dtype != q_out.dtype:
            raise KernelError("rope_kv_write: query output and cache differ in dtype")
        self.lib.check(self.lib.xr_rope_kv_write(
            _ptr(q_in), _ptr(k_in), _ptr(v_in), stride, _ptr(q_out), _ptr(k_cache), _ptr(v_cache),
            positions.data_ptr(), _ptr(req_of_token), _ptr(block_table),
            block_table.stride(0) if block_table is not None else 0, _ptr(inv_freq), T, H, Hk, D, rot,
            1 if interleaved else 0, float(mscale), page_size, dtype_code(store.dtype), 1 if paired else 0,
            _stream()))

    def rope_table(self, positions: torch.Tensor, inv_freq: torch.Tensor, mscale: float = 1.0) -> torch.Tensor:
        """``[T, rot/2, 2]`` float32: cosine and sine (times ``mscale``) of every row's angles, as
        ``project_rope_kv_write`` takes them for a product of many rows (``cs_table``); the same for
        every layer that rotates by ``inv_freq``, so a step needs it once."""
        self._dev(positions, inv_freq)
        T, half = positions.numel(), inv_freq.numel()
        out = torch.empty((T, half, 2), dtype=torch.float32, device=positions.device)
        self.lib.check(self.lib.xr_rope_table(out.data_ptr(), positions.data_ptr(), inv_freq.data_ptr(), T, half,
                                              float(mscale), _stream()))
        return out

    def project_rope_kv_write(self, h, w, bias, k_cache, v_cache, positions, req_of_token, block_table,
                              inv_freq, H: int, Hk: int, D: int, rot: int, interleaved: bool, mscale: float,
                              page_size: int, paired: bool = False, cs_table=None, variant: int = 0) -> torch.Tensor:
        """``[q | k | v] = h @ w^T (+ bias)``, queries and keys rotated, keys and values written
        to their pages; returns the rotated queries ``[T, H*D]`` in the compute dtype.

        ``w`` holds ``H`` query heads, then ``Hk`` key heads and ``Hk`` value heads (``Hk`` = 0 and
        no caches: queries alone); with ``paired`` its query and key rows are in ``paired_order``.
        Up to 16 bfloat16 rows (``h`` may be an ``UnscaledRows``) the product's kernel rotates and
        stores its own result, up to 511 the kernel that adds the product's K ranges up does, from
        512 the tile kernel (with the rows' cosines and sines from a table made first), which
        saves a kernel; in float32, and where the kernels' conditions on sizes do not hold, the
        product and ``rope_kv_write`` run one after the other.  ``cs_table``: a callable that returns the
        step's ``rope_table`` (asked for only where the tile kernel rotates).  ``variant``: a tile kernel
        by number instead of the library's choice (tests; from 512 rows on)."""
        rows = h.data if isinstance(h, UnscaledRows) else h
        wt = w.data if isinstance(w, PackedWeight) else w
        T, Q, KV = rows.shape[0], H * D, Hk * D
        if w.shape[0] != Q + 2 * KV:
            raise KernelError(f"projection has {w.shape[0]} rows, {H} query and 2 x {Hk} key/value heads of {D} need {Q + 2 * KV}")
        q = torch.empty((T, Q), dtype=rows.dtype, device=rows.device)
        if (self.fuse_rope and (T <= self.FINISH_ROWS or T >= self.ROPE_TILE_ROWS) and self._mfma_ok(rows, wt) and D % 16 == 0
                and (T * w.shape[0] * 4 if T <= self.FINISH_ROWS else T * (rot // 2 + 1) * 8) <= self.GEMM_WORKSPACE_BYTES
                and (Hk == 0 or (k_cache.dtype == torch.bfloat16 and v_cache.dtype == torch.bfloat16))
                and (rot == 0 or interleaved or (paired and rot % 16 == 0))):
            self._dev(rows, wt, bias, k_cache, v_cache, positions, req_of_token, block_table, inv_freq)
            self._contig(wt, "projection weight")
            if rows.shape[1] != w.shape[1] or rows.stride(1) != 1:
                raise KernelError(f"projection: shapes {tuple(rows.shape)} x {tuple(w.shape)}^T do not fit")
            if bias is not None and (bias.dtype != torch.float32 or bias.numel() != w.shape[0]):
                raise KernelError("projection: bias must be float32 [N]")
            norm, rows = self._norm_before(h, None)
            rp = _GemmRope()
            rp.positions, rp.req_of_token, rp.block_table = positions.data_ptr(), _ptr(req_of_token), _ptr(block_table)
            rp.table_stride = block_table.stride(0) if block_table is not None else 0
            rp.inv_freq, rp.H, rp.Hk, rp.D, rp.rot = _ptr(inv_freq), H, Hk, D, rot
            rp.interleaved, rp.mscale, rp.page_size = 1 if interleaved else 0, float(mscale), page_size
            rp.q_out, rp.k_cache, rp.v_cache = q.data_ptr(), _ptr(k_cache) if Hk else None, _ptr(v_cache) if Hk else None
            table = cs_table() if (cs_table is not None and T >= self.ROPE_TILE_ROWS and rot > 0) else None
            rp.cs_table = _ptr(table)
            self.lib.check(self.lib.xr_gemm_bf16(None, rows.data_ptr(), wt.data_ptr(), _ptr(bias), T, w.shape[0],
                                                 rows.shape[1], rows.stride(0), w.shape[0], XR_F32, 0, 0, 0.0, variant,
                                                 1 if isinstance(w, PackedWeight) else 0,
                                                 *self._gemm_workspace(rows.device),
                                                 C.addressof(norm) if norm is not None else None,
                                                 C.addressof(rp), _stream()))
            return q
        proj = self.linear(h, w, bias=bias, out_dtype=torch.float32)
        k_in = proj[:, Q:Q + KV] if Hk else None
        v_in = proj[:, Q + KV:Q + 2 * KV] if Hk else None
        self.rope_kv_write(proj[:, :Q], k_in, v_in, q, k_cache if Hk else None, v_cache if Hk else None, positions,
                           req_of_token, block_table, inv_freq, H, Hk, D, rot, interleaved, mscale, page_size,
                           paired=paired)
        return q

    def attention(self, q, k_cache, v_cache, ctx, group: int, H: int, Hk: int, D: int, page_size: int,
                  scale: float, window: Optional[int] = None, slopes: Optional[torch.Tensor] = None,
                  chunk: Optional[int] = None, keep_first: int = 0, sinks: Optional[torch.Tensor] = None,
                  v_head_dim: Optional[int] = None) -> torch.Tensor:
        """Causal attention of every token of the step over its request's cached keys and values.
        ``slopes`` (32-bit ``[H]``): ``slopes[h] * (i - j)`` is taken off the score of query i and key j.
        ``window``: a position reads the last ``window`` keys; ``chunk``: it reads the keys of its own chunk of
        ``chunk`` positions, counted from 0; ``keep_first``: the first so many keys are read whatever the window.
        ``sinks`` (32-bit ``[H]``): the softmax's denominator also holds ``exp(sinks[h])``, an entry without key
        or value.  ``v_head_dim``: the size of a value where it is not the keys' (``[T, H * v_head_dim]`` comes back).

        bfloat16 runs on the matrix cores (head sizes in steps of 16 up to 256, pages of at least
        16 positions); float32, and what the MFMA kernel does not take, runs the 32-bit kernel.
        """
        positions, req_of_token, block_table = ctx.positions, ctx.req_of_token, ctx.block_table(group)
        self._dev(q, k_cache, v_cache, positions, req_of_token, block_table)
        T = positions.numel()
        self._contig(q, "attention queries")
        if q.dtype != k_cache.dtype or q.dtype != v_cache.dtype:
            raise KernelError("attention: queries and cache differ in dtype")
        if H % Hk:
            raise KernelError(f"attention: {H} query heads are not a multiple of {Hk} key/value heads")
        Dv = int(v_head_dim) if v_head_dim is not None else D
        out = torch.empty((T, H * Dv), dtype=q.dtype, device=q.device)
        for name, t in (("slopes", slopes), ("sinks", sinks)):
            if t is not None:
                self._dev(t)
                if t.dtype != torch.float32 or t.numel() != H or not t.is_contiguous():
                    raise KernelError(f"attention: the {name} must be float32 [{H}]")
        if chunk and window:
            raise KernelError("attention: a layer reads a window or its chunk, not both")
        if (self.use_mfma and q.dtype == torch.bfloat16 and D == Dv and D % 16 == 0 and 16 <= D <= 256 and page_size >= 16):
            # The first keys that a window has passed enter the same softmax as a partial result of its own, which
            # the kernels' merge adds to the key ranges' (with the sink, if there is one); a sink alone is added by
            # the kernels themselves where they finish a row.
            extra = keep_first > 0
            lib = self.attention_lib(D)
            mask = Chunked(int(chunk)) if chunk else window
            plan = (ctx.attention_plan(group, H // Hk, mask, Hk, page_size, extra_slot=True) if extra
                    else ctx.attention_plan(group, H // Hk, mask, Hk, page_size))
            part_o = part_ml = None
            if plan.n_slots:
                part_o = torch.empty((plan.n_slots, Hk, 32, D), dtype=torch.float32, device=q.device)
                part_ml = torch.empty((plan.n_slots, Hk, 32, 2), dtype=torch.float32, device=q.device)
            if extra:
                self.lib.check(self.lib.xr_attn_extra_partial(
                    part_o.data_ptr(), part_ml.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                    plan.extras.data_ptr(), plan.n_extras, block_table.data_ptr(), block_table.stride(0), H, Hk, D, page_size,
                    float(scale), int(window or 0), int(chunk or 0), int(keep_first), _ptr(sinks), _ptr(slopes),
                    dtype_code(q.dtype), _stream()))
            lib.check(lib.xr_attention_mfma(
                out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), plan.items.data_ptr(),
                plan.n_items, plan.n_cta_items, _ptr(plan.jobs), plan.n_jobs, ctx.cu_q.data_ptr(),
                ctx.starts_dev.data_ptr(), block_table.data_ptr(), block_table.stride(0), _ptr(part_o), _ptr(part_ml), H, Hk, D, page_size,
                float(scale), int(window or 0), int(chunk or 0), _ptr(slopes), None if extra else _ptr(sinks), _stream()))
            return out
        self.lib.check(self.lib.xr_attention_ref(
            out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), positions.data_ptr(),
            req_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0), T, H, Hk, D, Dv, page_size,
            float(scale), int(window or 0), int(chunk or 0), int(keep_first), dtype_code(q.dtype), _ptr(slopes),
            _ptr(sinks), _stream()))
        return out

    def head_gate_(self, o: torch.Tensor, g: torch.Tensor, H: int, Dv: int) -> None:
        """``o[t, h, :] *= sigmoid(g[t, h])`` in place: ``o [T, H * Dv]`` contiguous, ``g`` a 32-bit view ``[T, H]``."""
        self._dev(o, g)
        self._contig(o, "head_gate_ rows")
        T = o.shape[0]
        if tuple(o.shape) != (T, H * Dv) or g.dtype != torch.float32 or tuple(g.shape) != (T, H) or g.stride(1) != 1:
            raise KernelError(f"head_gate_: rows [{T}, {H * Dv}] and a float32 gate view [{T}, {H}] are needed")
        self.lib.check(self.lib.xr_head_gate(o.data_ptr(), g.data_ptr(), T, H, Dv, g.stride(0), dtype_code(o.dtype), _stream()))

    def decay_prepare_(self, x: torch.Tensor, H: int, D: int, form: str, tau: float = 1.0,
                       a_log: Optional[torch.Tensor] = None, dt_bias: Optional[torch.Tensor] = None) -> None:
        """In place on a 32-bit view ``x [T, H * D]``: the decays a token, head and key channel of a recurrence.
        ``form`` "sigmoid_root": ``sigmoid(x)^(1 / tau)``; "exp_softplus": ``exp(-exp(a_log[h]) * softplus(x + dt_bias[h, c]))``."""
        self._dev(x, a_log, dt_bias)
        forms = {"sigmoid_root": 0, "exp_softplus": 1}
        if form not in forms:
            raise KernelError(f"decay_prepare_: form {form!r} (known: {sorted(forms)})")
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1 or x.shape[1] != H * D:
            raise KernelError(f"decay_prepare_: x must be a float32 view [rows, {H * D}] with unit column stride")
        if form == "exp_softplus" and (a_log is None or dt_bias is None or a_log.dtype != torch.float32 or dt_bias.dtype != torch.float32
                                       or a_log.numel() != H or dt_bias.numel() != H * D):
            raise KernelError(f"decay_prepare_: float32 A_log [{H}] and dt_bias [{H * D}] are needed")
        self.lib.check(self.lib.xr_decay_prepare(x.data_ptr(), x.shape[0], H, D, x.stride(0), forms[form], float(tau),
                                                 _ptr(a_log), _ptr(dt_bias), _stream()))

    def pair_combine_(self, x: torch.Tensor, y_left: torch.Tensor, y_right: torch.Tensor, a_left: float, a_right: float,
                      w_left: Optional[torch.Tensor] = None, w_right: Optional[torch.Tensor] = None, eps: float = 0.0,
                      then_norm=None, out_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
        """``x += a_left f(y_left) + a_right f(y_right)`` for 32-bit rows ``[T, E]``; with the weights, ``f`` is a row
        over its root mean square (eps inside the root) times the side's weight ``[E]``, else the identity.
        ``then_norm`` = (32-bit weight ``[E]``, eps): the RMS norm of the updated rows comes back in ``out_dtype``."""
        self._dev(x, y_left, y_right, w_left, w_right)
        T, E = y_left.shape
        if (x.dtype != torch.float32 or x.stride(1) != 1 or tuple(x.shape) != (T, E)
                or any(t.dtype != torch.float32 or tuple(t.shape) != (T, E) or not t.is_contiguous() for t in (y_left, y_right))):
            raise KernelError(f"pair_combine_: x and both results must be float32 [{T}, {E}]")
        normed = w_left is not None
        if normed and any(w is None or w.dtype != torch.float32 or w.numel() != E or not w.is_contiguous() for w in (w_left, w_right)):
            raise KernelError(f"pair_combine_: the sides' norm weights must be float32 [{E}]")
        h = None
        if then_norm is not None:
            w_h, eps_h = then_norm
            self._dev(w_h)
            if w_h.dtype != torch.float32 or w_h.numel() != E or not w_h.is_contiguous():
                raise KernelError(f"pair_combine_: the following norm's weight must be float32 [{E}]")
            h = torch.empty((T, E), dtype=out_dtype or torch.float32, device=x.device)
        self.lib.check(self.lib.xr_pair_combine(x.data_ptr(), y_left.data_ptr(), y_right.data_ptr(), _ptr(w_left), _ptr(w_right),
                                                float(a_left), float(a_right), float(eps), T, E, x.stride(0), 1 if normed else 0,
                                                _ptr(h), _ptr(then_norm[0]) if then_norm is not None else None,
                                                float(then_norm[1]) if then_norm is not None else 0.0,
                                                dtype_code(h.dtype) if h is not None else XR_F32, _stream()))
        return h

    def add_rows_(self, x: torch.Tensor, v: torch.Tensor, y: Optional[torch.Tensor] = None, scale: float = 1.0) -> None:
        """``x[t] += scale * y[t] + v`` for 32-bit contiguous rows ``[T, E]`` and a 32-bit vector ``v [E]`` (``y`` absent:
        the vector alone)."""
        self._dev(x, v, y)
        self._contig(x, "add_rows_ x")
        T, E = x.shape
        if x.dtype != torch.float32 or v.dtype != torch.float32 or v.numel() != E or not v.is_contiguous():
            raise KernelError(f"add_rows_: x must be float32 rows and v float32 [{E}]")
        if y is not None and (y.dtype != torch.float32 or tuple(y.shape) != (T, E) or not y.is_contiguous()):
            raise KernelError(f"add_rows_: y must be contiguous float32 [{T}, {E}]")
        self.lib.check(self.lib.xr_add_rows(x.data_ptr(), _ptr(y), v.data_ptr(), float(scale), T, E, _stream()))

    def attention_lib(self, D: int) -> "_Lib":
        """The MFMA attention library for head size ``D`` (compiled at first use)."""
        lib = self._attn_libs.get(D)
        if lib is None:
            unit = f"attn_d{D}"
            path = _build.find_built(unit) or _build.build_unit(unit)
            lib = _Lib(path, {"xr_attention_mfma": [_p, _p, _p, _p, _p, _i, _i, _p, _i, _p, _p, _p, _i, _p, _p,
                                                    _i, _i, _i, _i, _f, _i, _i, _p, _p, _p]})
            self._attn_libs[D] = lib
        return lib

    # -- row-wise and time-wise operations around the sequence mixers ----------
    def layernorm(self, x: torch.Tensor, w: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype,
                  rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``(x - mean) / sqrt(var + eps) * w`` of the rows of 32-bit ``x`` (or of the rows ``rows``
        selects); ``w`` 32-bit or absent, no bias."""
        self._dev(x, w, rows)
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
            raise KernelError("layernorm input must be float32 [rows, width] with unit column stride")
        E = x.shape[1]
        if w is not None and (w.dtype != torch.float32 or w.numel() != E or not w.is_contiguous()):
            raise KernelError(f"layernorm weight must be float32 [{E}]")
        R = x.shape[0] if rows is None else rows.numel()
        out = torch.empty((R, E), dtype=out_dtype, device=x.device)
        self.lib.check(self.lib.xr_layernorm(out.data_ptr(), x.data_ptr(), _ptr(w), _ptr(rows), R, E, x.stride(0),
                                             float(eps), dtype_code(out_dtype), _stream()))
        return out

    def dyt(self, x: torch.Tensor, alpha: float, w: torch.Tensor, b: torch.Tensor, out_dtype: torch.dtype,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Dynamic tanh of the rows of 32-bit ``x`` (or of the rows ``rows`` selects): ``tanh(alpha x) * w + b``,
        a norm that takes no statistic of the row; ``w`` and ``b`` 32-bit ``[E]``."""
        return self.dyt_step(x, norm=(alpha, w, b), out_dtype=out_dtype, rows=rows)

    def dyt_step(self, x: torch.Tensor, y: Optional[torch.Tensor] = None, post=None, mult: float = 1.0, norm=None,
                 out_dtype: Optional[torch.dtype] = None, rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """What lies between two sublayers that are normed before and after, in one pass over the 32-bit
        residual rows ``x [T, E]``: with ``y [T, E]`` (a sublayer's result, 32-bit or the compute dtype) and
        ``post`` = (alpha, w, b): ``x += mult * (tanh(alpha y) w + b)`` in place; with ``norm`` = (alpha, w, b):
        ``tanh(alpha x) w + b`` of the rows (updated or not) comes back in ``out_dtype``.  Either half alone too."""
        self._dev(x, y, rows)
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
            raise KernelError("dyt: x must be float32 [rows, width] with unit column stride")
        E = x.shape[1]
        for part in (post, norm):
            if part is not None:
                _, w, b = part
                self._dev(w, b)
                if any(t.dtype != torch.float32 or t.numel() != E or not t.is_contiguous() for t in (w, b)):
                    raise KernelError(f"dyt: weight and bias must be float32 [{E}]")
        if (y is None) != (post is None):
            raise KernelError("dyt: a sublayer's result and its norm come together")
        if y is not None and (tuple(y.shape) != tuple(x.shape) or not y.is_contiguous() or rows is not None):
            raise KernelError(f"dyt: y must be contiguous {tuple(x.shape)} and the rows all")
        R = x.shape[0] if rows is None else rows.numel()
        h = torch.empty((R, E), dtype=out_dtype or torch.float32, device=x.device) if norm is not None else None
        self.lib.check(self.lib.xr_dyt_step(
            x.data_ptr(), _ptr(y), _ptr(post[1]) if post else None, _ptr(post[2]) if post else None,
            float(post[0]) if post else 0.0, float(mult), _ptr(h), _ptr(norm[1]) if norm else None,
            _ptr(norm[2]) if norm else None, float(norm[0]) if norm else 0.0, _ptr(rows), R, E, x.stride(0),
            dtype_code(y.dtype) if y is not None else XR_F32, dtype_code(h.dtype) if h is not None else XR_F32, _stream()))
        return h

    def token_shift(self, h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, ctx, out_dtype: torch.dtype) -> torch.Tensor:
        """``out[t, s] = h[t] + (h[t - 1] - h[t]) * mu[s]`` for the ``n`` mixes ``mu [n, E]`` (32-bit) of the 32-bit rows
        ``h [T, E]``, as ``[T, n * E]`` in ``out_dtype``.  The row before a request's first row of the step is its row
        of ``state [slots + 1, E]`` (zero for a request that begins), which is brought up to date."""
        self._dev(h, mu, state)
        if h.dtype != torch.float32 or h.dim() != 2 or h.stride(1) != 1:
            raise KernelError("token_shift: h must be float32 [rows, width] with unit column stride")
        T, E = h.shape
        if mu.dtype != torch.float32 or mu.dim() != 2 or mu.shape[1] != E or not mu.is_contiguous():
            raise KernelError(f"token_shift: the mixes must be float32 [n, {E}]")
        if state.dtype != torch.float32 or tuple(state.shape[1:]) != (E,) or not state.is_contiguous():
            raise KernelError(f"token_shift: state must be float32 [slots, {E}]")
        n = mu.shape[0]
        out = torch.empty((T, n * E), dtype=out_dtype, device=h.device)
        self.lib.check(self.lib.xr_token_shift(out.data_ptr(), h.data_ptr(), mu.data_ptr(), state.data_ptr(), ctx.cu_q.data_ptr(),
                                               ctx.slots.data_ptr(), ctx.req_of_token.data_ptr(), T, ctx.B, E, n, h.stride(0),
                                               dtype_code(out_dtype), 1 if (ctx.max_q_len == 1 and T == ctx.B) else 0, _stream()))
        return out

    def head_rmsnorm_(self, q: Optional[torch.Tensor], k: Optional[torch.Tensor], wq: Optional[torch.Tensor],
                      wk: Optional[torch.Tensor], eps: float, positions: Optional[torch.Tensor] = None,
                      temp_coef: float = 0.0, temp_every: int = 0) -> None:
        """In place on the 32-bit views ``q [T, H, D]`` and ``k [T, Hk, D]`` (one row stride): every head over its
        root mean square times a weight ``[D]`` that the heads share (``wq`` / ``wk``; absent: that side stays);
        with ``temp_every`` > 0 the queries at position p also times ``1 + temp_coef ln(floor((p + 1) / temp_every) + 1)``."""
        self._dev(q, k, wq, wk, positions)
        views = [t for t in (q, k) if t is not None]
        if not views:
            return
        if any(t.dtype != torch.float32 or t.dim() != 3 or t.stride(2) != 1 or t.stride(1) != t.shape[2] for t in views):
            raise KernelError("head_rmsnorm_: q and k must be float32 views [rows, heads, size] with the heads side by side")
        one_row = views[0].shape[0] <= 1        # (a single row has no stride to speak of)
        if (not one_row and len({t.stride(0) for t in views}) != 1) or len({t.shape[2] for t in views}) != 1:
            raise KernelError("head_rmsnorm_: q and k must share a row stride and a head size")
        D = views[0].shape[2]
        for w in (wq, wk):
            if w is not None and (w.dtype != torch.float32 or w.numel() != D or not w.is_contiguous()):
                raise KernelError(f"head_rmsnorm_: a weight must be float32 [{D}]")
        self.lib.check(self.lib.xr_head_rmsnorm(_ptr(q), _ptr(k), views[0].stride(0), _ptr(wq), _ptr(wk), _ptr(positions),
                                                views[0].shape[0], q.shape[1] if q is not None else 0,
                                                k.shape[1] if k is not None else 0, D, float(eps), float(temp_coef),
                                                int(temp_every), _stream()))

    def causal_conv(self, u: torch.Tensor, w: torch.Tensor, state: Optional[torch.Tensor], ctx, out_dtype: torch.dtype,
                    residual: bool = False, activation: Optional[str] = None) -> torch.Tensor:
        """A convolution over time on every channel of ``u [T, C]``: ``y_t = sum_j w[:, j] u_(t-taps+1+j)``
        (plus ``u_t`` with ``residual``), then the activation.  ``state [slots + 1, taps - 1, C]`` (the
        dtype of ``u``) holds every request's last ``taps - 1`` inputs and is brought up to date;
        ``ctx`` gives the step's rows (``cu_q``, ``slots``, ``req_of_token``)."""
        self._dev(u, w, state)
        if u.dim() != 2 or u.stride(1) != 1:
            raise KernelError("causal_conv input must be [rows, channels] with unit column stride")
        T, Cn = u.shape
        if w.dtype != torch.float32 or w.dim() != 2 or w.shape[0] != Cn or not w.is_contiguous():
            raise KernelError(f"causal_conv weight must be float32 [{Cn}, taps]")
        taps = w.shape[1]
        if taps > 1:
            if state is None or state.dtype != u.dtype or tuple(state.shape[1:]) != (taps - 1, Cn) or not state.is_contiguous():
                raise KernelError(f"causal_conv state must be {u.dtype} [slots, {taps - 1}, {Cn}]")
        if activation not in CONV_ACTIVATIONS:
            raise KernelError(f"causal_conv: activation {activation!r} is not built (known: none, silu)")
        out = torch.empty((T, Cn), dtype=out_dtype, device=u.device)
        self.lib.check(self.lib.xr_causal_conv(out.data_ptr(), u.data_ptr(), w.data_ptr(), _ptr(state), ctx.cu_q.data_ptr(),
                                               ctx.slots.data_ptr(), ctx.req_of_token.data_ptr(), T, ctx.B, Cn, taps,
                                               u.stride(0), Cn, dtype_code(u.dtype), dtype_code(out_dtype),
                                               1 if residual else 0, CONV_ACTIVATIONS[activation],
                                               1 if (ctx.max_q_len == 1 and T == ctx.B) else 0, _stream()))
        return out

    def layernorm_conv(self, x: torch.Tensor, w: Optional[torch.Tensor], eps: float, conv_w: torch.Tensor,
                       state: Optional[torch.Tensor], ctx, out_dtype: torch.dtype) -> torch.Tensor:
        """``h + conv(h)`` with ``h = layernorm(x)`` in one kernel, for a step in which every request
        brings one row (row b of ``x`` is request b's): the same result as ``layernorm`` in 32 bits
        followed by ``causal_conv`` with ``residual``, and the same update of ``state``."""
        self._dev(x, w, conv_w, state)
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
            raise KernelError("layernorm_conv input must be float32 [rows, width] with unit column stride")
        R, E = x.shape
        if ctx.max_q_len != 1 or R != ctx.B:
            raise KernelError("layernorm_conv is for steps of one row a request")
        if w is not None and (w.dtype != torch.float32 or w.numel() != E or not w.is_contiguous()):
            raise KernelError(f"layernorm_conv: the norm's weight must be float32 [{E}]")
        if conv_w.dtype != torch.float32 or conv_w.dim() != 2 or conv_w.shape[0] != E or not conv_w.is_contiguous():
            raise KernelError(f"layernorm_conv: the convolution's weight must be float32 [{E}, taps]")
        taps = conv_w.shape[1]
        if taps > 1 and (state is None or state.dtype != torch.float32 or tuple(state.shape[1:]) != (taps - 1, E)
                         or not state.is_contiguous()):
            raise KernelError(f"layernorm_conv state must be float32 [slots, {taps - 1}, {E}]")
        out = torch.empty((R, E), dtype=out_dtype, device=x.device)
        self.lib.check(self.lib.xr_layernorm_conv(out.data_ptr(), x.data_ptr(), _ptr(w), conv_w.data_ptr(), _ptr(state),
                                                  ctx.slots.data_ptr(), R, E, x.stride(0), taps, float(eps),
                                                  dtype_code(out_dtype), _stream()))
        return out

    def polynorm(self, z: torch.Tensor, coef: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
        """``a N(z) + b N(z^2) + c N(z^3) + e`` per row, ``N(v) = v / sqrt(mean(v^2) + eps)``,
        ``coef`` = (a, b, c, e) as 32-bit floats on the device."""
        self._dev(z, coef)
        if z.dim() != 2 or z.stride(1) != 1:
            raise KernelError("polynorm input must be [rows, width] with unit column stride")
        if coef.dtype != torch.float32 or coef.numel() != 4:
            raise KernelError("polynorm takes four 32-bit coefficients")
        T, F = z.shape
        out = torch.empty((T, F), dtype=out_dtype, device=z.device)
        self.lib.check(self.lib.xr_polynorm(out.data_ptr(), z.data_ptr(), coef.data_ptr(), T, F, z.stride(0), float(eps),
                                            dtype_code(z.dtype), dtype_code(out_dtype), _stream()))
        return out

    def rotate_rows_(self, x: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor], heads: int, D: int,
                     rot: int, scale: float = 1.0) -> None:
        """Rotate the first ``rot`` channels of every head of the 32-bit view ``x [T, heads * D]`` in
        place (channel j pairs with j + rot/2, angle = position x ``inv_freq[j]``), then scale."""
        self._dev(x, positions, inv_freq)
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1 or x.shape[1] != heads * D:
            raise KernelError(f"rotate_rows_: x must be a float32 view [rows, {heads * D}] with unit column stride")
        if rot and (inv_freq is None or inv_freq.numel() != rot // 2 or inv_freq.dtype != torch.float32):
            raise KernelError(f"rotate_rows_: {rot // 2} 32-bit frequencies are needed")
        self.lib.check(self.lib.xr_rotate_rows(x.data_ptr(), positions.data_ptr(), _ptr(inv_freq), x.shape[0], heads, D,
                                               rot, x.stride(0), float(scale), _stream()))

    def gated_rmsnorm(self, o: torch.Tensor, gate: torch.Tensor, w: Optional[torch.Tensor], H: int, Dv: int, eps: float,
                      out_dtype: torch.dtype, gate_activation: str = "silu") -> torch.Tensor:
        """``o / rms(o) * w * act(gate)`` per head: ``o [T, H * Dv]`` 32-bit and contiguous, ``gate`` a
        32-bit view of the same shape; ``w`` 32-bit: ``[Dv]`` (the heads share it), ``[H * Dv]`` (one a
        channel of the row) or absent; ``act`` "silu" or "sigmoid".  A norm over all heads together is
        ``H = 1`` with ``Dv`` the whole row."""
        self._dev(o, gate, w)
        T = o.shape[0]
        if o.dtype != torch.float32 or not o.is_contiguous() or o.shape[1] != H * Dv:
            raise KernelError(f"gated_rmsnorm: o must be contiguous float32 [rows, {H * Dv}]")
        if gate.dtype != torch.float32 or gate.stride(1) != 1 or tuple(gate.shape) != (T, H * Dv):
            raise KernelError("gated_rmsnorm: the gate must be a float32 view of o's shape")
        if w is not None and (w.dtype != torch.float32 or w.numel() not in (Dv, H * Dv) or not w.is_contiguous()):
            raise KernelError(f"gated_rmsnorm: the weight must be float32 [{Dv}] or [{H * Dv}]")
        if gate_activation not in NORM_GATES:
            raise KernelError(f"gated_rmsnorm: gate activation {gate_activation!r} (known: {sorted(NORM_GATES)})")
        out = torch.empty((T, H * Dv), dtype=out_dtype, device=o.device)
        self.lib.check(self.lib.xr_gated_rmsnorm(out.data_ptr(), o.data_ptr(), gate.data_ptr(), _ptr(w), T, H, Dv,
                                                 gate.stride(0), float(eps), dtype_code(out_dtype),
                                                 1 if (w is not None and H > 1 and w.numel() == H * Dv) else 0,
                                                 NORM_GATES[gate_activation], _stream()))
        return out

    def act_rows_(self, x: torch.Tensor, activation: str = "silu") -> None:
        """``x <- act(x)`` in place on a 32-bit view ``[rows, width]`` with unit column stride."""
        self._act_rows(x, activation, None)

    def act_rows(self, x: torch.Tensor, activation: str, out_dtype: torch.dtype) -> torch.Tensor:
        """``act(x)`` of a 32-bit view ``[rows, width]`` as contiguous rows in ``out_dtype`` (what a product reads next)."""
        out = torch.empty(tuple(x.shape), dtype=out_dtype, device=x.device)
        self._act_rows(x, activation, out)
        return out

    def _act_rows(self, x, activation, out) -> None:
        self._dev(x)
        if x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
            raise KernelError("act_rows: x must be a float32 view [rows, width] with unit column stride")
        if activation not in ROW_ACTIVATIONS:
            raise KernelError(f"act_rows: activation {activation!r} is not built ({', '.join(sorted(ROW_ACTIVATIONS))})")
        self.lib.check(self.lib.xr_act_rows(x.data_ptr(), x.shape[0], x.shape[1], x.stride(0), ROW_ACTIVATIONS[activation],
                                            _ptr(out), dtype_code(out.dtype) if out is not None else XR_F32, _stream()))

    # -- an embedding with a hashed table of token pairs --------------------------
    def embedding_pairs(self, table: torch.Tensor, pairs: Optional[torch.Tensor], norm_w: Optional[torch.Tensor], ids, ctx,
                        last_token: Optional[torch.Tensor], buckets: int, mul_prev: int, mul_cur: int, eps: float) -> torch.Tensor:
        """``rmsnorm(table[id] + pairs[(prev * mul_prev + id * mul_cur) % buckets]) * norm_w`` as 32-bit rows
        (``pairs`` absent: the token's row alone; ``norm_w`` absent: no norm).  The token at position 0 reads
        row ``buckets`` of ``pairs [buckets + 1, E]``.  ``last_token [slots + 1]`` (int32) holds every request's
        last token of the step before and is brought up to date; ``ctx`` gives the step's rows."""
        self._dev(table, pairs, norm_w, ids, last_token)
        self._contig(table, "embedding table")
        V, E = table.shape
        if pairs is not None:
            self._contig(pairs, "pair table")
            if pairs.dtype != table.dtype or tuple(pairs.shape) != (buckets + 1, E):
                raise KernelError(f"embedding_pairs: the pair table must be {table.dtype} [{buckets + 1}, {E}]")
            if last_token is None or last_token.dtype != torch.int32 or not last_token.is_contiguous():
                raise KernelError("embedding_pairs: the requests' last tokens must be int32 [slots]")
        if norm_w is not None and (norm_w.dtype != torch.float32 or norm_w.numel() != E or not norm_w.is_contiguous()):
            raise KernelError(f"embedding_pairs: the norm's weight must be float32 [{E}]")
        if buckets:     # (a b) mod n = ((a mod n)(b mod n)) mod n: the kernel's 64-bit products then hold any multiplier
            mul_prev, mul_cur = int(mul_prev) % int(buckets), int(mul_cur) % int(buckets)
        T = ids.numel()
        out = torch.empty((T, E), dtype=torch.float32, device=table.device)
        self.lib.check(self.lib.xr_embedding_pairs(out.data_ptr(), table.data_ptr(), _ptr(pairs), _ptr(norm_w), ids.data_ptr(),
                                                   ctx.positions.data_ptr(), ctx.req_of_token.data_ptr(), ctx.cu_q.data_ptr(),
                                                   ctx.slots.data_ptr(), _ptr(last_token), T, E, V, int(buckets), int(mul_prev),
                                                   int(mul_cur), float(eps), dtype_code(table.dtype), _stream()))
        return out

    # -- several copies of the residual stream -------------------------------------
    MAX_STREAMS = 8

    def streams_expand(self, x: torch.Tensor, S: int) -> torch.Tensor:
        """``[S, T, E]``: ``S`` copies of the 32-bit rows ``x [T, E]``."""
        self._dev(x)
        if x.dtype != torch.float32 or x.dim() != 2 or not x.is_contiguous():
            raise KernelError("streams_expand: x must be contiguous float32 [rows, width]")
        xs = torch.empty((S,) + tuple(x.shape), dtype=torch.float32, device=x.device)
        self.lib.check(self.lib.xr_streams_expand(xs.data_ptr(), x.data_ptr(), x.shape[0], x.shape[1], int(S), _stream()))
        return xs

    def streams_sum(self, xs: torch.Tensor) -> torch.Tensor:
        """The sum ``[T, E]`` of the copies ``xs [S, T, E]``."""
        self._dev(xs)
        if xs.dtype != torch.float32 or xs.dim() != 3 or not xs.is_contiguous():
            raise KernelError("streams_sum: xs must be contiguous float32 [streams, rows, width]")
        x = torch.empty(tuple(xs.shape[1:]), dtype=torch.float32, device=xs.device)
        self.lib.check(self.lib.xr_streams_sum(x.data_ptr(), xs.data_ptr(), xs.shape[1], xs.shape[2], xs.shape[0], _stream()))
        return x

    def streams_step(self, xs: torch.Tensor, y: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None,
                     out_w: Optional[torch.Tensor] = None, in_w: Optional[torch.Tensor] = None,
                     norm_w: Optional[torch.Tensor] = None, eps: float = 0.0,
                     h_dtype: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
        """One pass over the copies ``xs [S, T, E]`` around a sublayer.  With ``y [T, E]`` (32-bit), all
        copies at once from the old ones: ``xs_t <- sum_s mix[s, t] xs_s + out_w[t] y``.  With ``in_w``, then:
        ``u = sum_s in_w[s] xs_s`` and its RMSNorm times ``norm_w`` comes back in ``h_dtype`` (``norm_w``
        absent: ``u`` itself).  Weights are 32-bit."""
        self._dev(xs, y, mix, out_w, in_w, norm_w)
        if xs.dtype != torch.float32 or xs.dim() != 3 or not xs.is_contiguous():
            raise KernelError("streams_step: xs must be contiguous float32 [streams, rows, width]")
        S, T, E = xs.shape
        if S > self.MAX_STREAMS:
            raise KernelError(f"streams_step: {S} streams (the kernel takes up to {self.MAX_STREAMS})")
        if y is not None:
            if y.dtype != torch.float32 or tuple(y.shape) != (T, E) or not y.is_contiguous():
                raise KernelError(f"streams_step: y must be contiguous float32 [{T}, {E}]")
            if (mix is None or out_w is None or mix.dtype != torch.float32 or out_w.dtype != torch.float32
                    or tuple(mix.shape) != (S, S) or out_w.numel() != S or not mix.is_contiguous()):
                raise KernelError(f"streams_step: the write needs float32 mix [{S}, {S}] and out [{S}]")
        h = None
        if in_w is not None:
            if in_w.dtype != torch.float32 or in_w.numel() != S:
                raise KernelError(f"streams_step: the read needs float32 in [{S}]")
            if norm_w is not None and (norm_w.dtype != torch.float32 or norm_w.numel() != E or not norm_w.is_contiguous()):
                raise KernelError(f"streams_step: the norm's weight must be float32 [{E}]")
            h = torch.empty((T, E), dtype=h_dtype or torch.float32, device=xs.device)
        self.lib.check(self.lib.xr_streams_step(xs.data_ptr(), _ptr(y), _ptr(mix), _ptr(out_w), _ptr(in_w), _ptr(norm_w), _ptr(h),
                                                T, E, S, float(eps), dtype_code(h.dtype) if h is not None else XR_F32, _stream()))
        return h

    # -- latent attention ------------------------------------------------------------
    def latent_prepare(self, q_in: torch.Tensor, kv_in: torch.Tensor, c_w: torch.Tensor, eps: float, q_out: torch.Tensor,
                       k_cache: torch.Tensor, v_cache: torch.Tensor, ctx, group: int, inv_freq: Optional[torch.Tensor],
                       H: int, D: int, R: int, C: int, dims: int, page_size: int) -> torch.Tensor:
        """Between a latent attention's down projections and its attention.  ``q_in [T, H * (D + R)]`` and
        ``kv_in [T, C + R]`` are 32-bit views.  The first ``C`` channels of ``kv_in`` are normed (RMS, weight
        ``c_w``) into the latent; the last ``R`` are the shared key part, whose first ``dims`` channels are
        rotated in pairs ``(2i, 2i + 1)`` by position x ``inv_freq[i]``, as are the last ``R`` channels of every
        query head.  The row ``[latent | key part]`` goes to the key pages ``[pages, 1, page, C + R]`` and,
        transposed, to the value pages ``[pages, 1, C or C + R, page]``; the rotated query channels go to
        ``q_out[:, h, C:]`` (``q_out [T, H * (C + R)]``); the unrotated ones come back ``[T, H * D]`` in
        ``q_out``'s dtype."""
        self._dev(q_in, kv_in, c_w, q_out, k_cache, v_cache, inv_freq)
        T = q_in.shape[0]
        if any(t.dtype != torch.float32 or t.stride(1) != 1 for t in (q_in, kv_in)):
            raise KernelError("latent_prepare: q and kv inputs must be float32 views with unit column stride")
        if tuple(q_in.shape) != (T, H * (D + R)) or tuple(kv_in.shape) != (T, C + R):
            raise KernelError("latent_prepare: input widths do not fit the heads")
        if c_w.dtype != torch.float32 or c_w.numel() != C or not c_w.is_contiguous():
            raise KernelError(f"latent_prepare: the latent norm's weight must be float32 [{C}]")
        dt = q_out.dtype
        if tuple(q_out.shape) != (T, H * (C + R)) or not q_out.is_contiguous():
            raise KernelError(f"latent_prepare: the query output must be contiguous [{T}, {H * (C + R)}]")
        Dvc = v_cache.shape[2]
        if (k_cache.dtype != dt or v_cache.dtype != dt or tuple(k_cache.shape[1:]) != (1, page_size, C + R)
                or tuple(v_cache.shape[1:]) != (1, Dvc, page_size) or Dvc not in (C, C + R)):
            raise KernelError("latent_prepare: the cache does not fit one key/value head of the latent's row")
        if dims and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != dims // 2):
            raise KernelError(f"latent_prepare: {dims // 2} 32-bit frequencies are needed")
        table = ctx.block_table(group)
        qn = torch.empty((T, H * D), dtype=dt, device=q_in.device)
        self.lib.check(self.lib.xr_latent_prepare(qn.data_ptr(), q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                                  q_in.data_ptr(), kv_in.data_ptr(), c_w.data_ptr(), ctx.positions.data_ptr(),
                                                  ctx.req_of_token.data_ptr(), table.data_ptr(), table.stride(0), _ptr(inv_freq),
                                                  T, H, D, R, C, Dvc, int(dims), q_in.stride(0), kv_in.stride(0), page_size,
                                                  float(eps), dtype_code(dt), _stream()))
        return qn

    def heads_linear(self, a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, G: int, a_width: int, out_width: int) -> None:
        """``out[:, g * out_width : g * out_width + N] = a[:, g * a_width : g * a_width + K] @ w[g]^T`` for the ``G``
        groups (heads) of ``w [G, N, K]``: every head's column range of the rows ``a`` through a matrix of the
        head's own, into the head's column range of ``out``.  bfloat16 with sizes the matrix cores take
        (``K`` and the ranges' starts multiples of 8) runs as one launch; everything else head by head."""
        self._dev(a, w, out)
        T = a.shape[0]
        Gw, N, K = w.shape
        if Gw != G or a.stride(1) != 1 or out.stride(1) != 1 or a.shape[1] < (G - 1) * a_width + K or out.shape[1] < (G - 1) * out_width + N:
            raise KernelError("heads_linear: the heads' column ranges do not fit the rows")
        if a.dtype != w.dtype:
            raise KernelError(f"heads_linear: rows are {a.dtype}, weights {w.dtype}")
        self._contig(w, "heads_linear weights")
        if (self.use_mfma and a.dtype == torch.bfloat16 and K % 8 == 0 and a_width % 8 == 0 and a.stride(0) % 8 == 0
                and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and (N * K) % 8 == 0):
            self.lib.check(self.lib.xr_heads_gemm_bf16(out.data_ptr(), a.data_ptr(), w.data_ptr(), T, G, N, K, a.stride(0),
                                                       a_width, out.stride(0), out_width, dtype_code(out.dtype), _stream()))
            return
        for g in range(G):
            self.linear(a[:, g * a_width:g * a_width + K], w[g], out=out[:, g * out_width:g * out_width + N])

    # -- mixture of experts ------------------------------------------------------------
    def moe_route(self, h: torch.Tensor, router, correction: torch.Tensor, top: int, **how):
        """``(experts [T, top] int32, weights [T, top] float32)``: 32-bit logits ``h @ router [n, E]^T`` (a matrix
        product with 32-bit accumulation and a 32-bit result; ``router`` in ``h``'s dtype, a matrix or a
        ``PackedWeight``), a softmax over all experts, the ``top`` largest of score + ``correction`` (the lower
        index on a tie), weights = the chosen scores over their sum + 1e-20."""
        logits = self.linear(h, router, out_dtype=torch.float32)
        return self.route_logits(logits, correction, top, **how)

    def route_logits(self, logits: torch.Tensor, correction: torch.Tensor, top: int, scores: str = "softmax",
                     groups: int = 1, keep_groups: int = 1, weight_scale: Optional[float] = None):
        """``moe_route`` from the 32-bit logits ``[T, n]``.  ``scores`` "sigmoid": every expert's score is the sigmoid
        of its logit.  ``groups`` > 1: the experts form that many equal groups of neighbours, a group scores the
        sum of its two largest score + correction, and only the ``keep_groups`` best groups' experts can be chosen.
        ``weight_scale``: the weights are the chosen scores times it instead of their shares of their sum."""
        if scores not in ("softmax", "sigmoid"):
            raise KernelError(f"route_logits: scores {scores!r} (softmax or sigmoid)")
        if weight_scale is not None and not weight_scale > 0:
            raise KernelError(f"route_logits: weight scale {weight_scale} must be positive")
        self._dev(logits, correction)
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
            raise KernelError("route_logits: logits must be float32 [rows, experts] with unit column stride")
        T, n = logits.shape
        if correction.dtype != torch.float32 or correction.numel() != n:
            raise KernelError(f"route_logits: the correction must be float32 [{n}]")
        idx = torch.empty((T, top), dtype=torch.int32, device=logits.device)
        wts = torch.empty((T, top), dtype=torch.float32, device=logits.device)
        self.lib.check(self.lib.xr_moe_route(idx.data_ptr(), wts.data_ptr(), logits.data_ptr(), correction.data_ptr(), T,
                                             logits.stride(0), n, int(top), 1 if scores == "sigmoid" else 0, int(groups),
                                             int(keep_groups), float(weight_scale or 0.0), _stream()))
        return idx, wts

    def table_route(self, table: torch.Tensor, ids: torch.Tensor, n_experts: int):
        """``(experts [T, top] int32, weights [T, top] float32)`` without a router: row ``ids[t]`` of ``table
        [vocab, top]`` (int32), every chosen expert with the weight ``1 / top``."""
        self._dev(table, ids)
        if table.dtype != torch.int32 or table.dim() != 2 or not table.is_contiguous():
            raise KernelError("table_route: the table must be contiguous int32 [vocab, top]")
        V, top = table.shape
        T = ids.numel()
        idx = torch.empty((T, top), dtype=torch.int32, device=table.device)
        wts = torch.empty((T, top), dtype=torch.float32, device=table.device)
        self.lib.check(self.lib.xr_moe_table_route(idx.data_ptr(), wts.data_ptr(), table.data_ptr(), ids.data_ptr(), T, V, top,
                                                   int(n_experts), 1.0 / top, _stream()))
        return idx, wts

    GROUPED_EXPERTS_FROM = 32       # choices (rows x top) from which the experts' rows are sorted and run on the matrix cores

    def moe_experts(self, h: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, idx: torch.Tensor, wts: torch.Tensor,
                    out: Optional[torch.Tensor] = None, accumulate: bool = False, activation: str = "relu2") -> torch.Tensor:
        """``out[t] (+)= sum_j wts[t, j] * w_down[e] @ relu(w_up[e] @ h[t])^2`` with ``e = idx[t, j]``, as 32-bit
        rows; ``w_up [n, F, E]`` and ``w_down [n, E, F]`` in ``h``'s dtype.  ``activation`` "swiglu": gated experts,
        ``w_down[e] @ (silu(g) * u)`` with ``[g; u] = w_up[e] @ h[t]`` for ``w_up [n, 2F, E]`` (an expert's gate rows
        before its up rows).  A few choices stream the chosen
        experts' weights, a wave an output column; from ``GROUPED_EXPERTS_FROM`` choices on (bfloat16, widths
        that are multiples of 8) the rows are sorted by expert on the device, both products run on the matrix
        cores and a last kernel adds a token's experts up in the order of its choice."""
        self._dev(h, w_up, w_down, idx, wts, out)
        T, E = h.shape
        if activation not in EXPERT_ACTIVATIONS:
            raise KernelError(f"moe_experts: activation {activation!r} (known: {sorted(EXPERT_ACTIVATIONS)})")
        gated = activation == "swiglu"
        n, Fu, _ = w_up.shape
        F = Fu // 2 if gated else Fu
        top = idx.shape[1]
        if h.stride(1) != 1 or w_up.dtype != h.dtype or w_down.dtype != h.dtype:
            raise KernelError("moe_experts: h must have unit column stride and the experts its dtype")
        if tuple(w_up.shape) != (n, 2 * F if gated else F, E) or tuple(w_down.shape) != (n, E, F) or not w_up.is_contiguous() or not w_down.is_contiguous():
            raise KernelError("moe_experts: the experts' weights must be contiguous [n, F, E] and [n, E, F]")
        if idx.dtype != torch.int32 or wts.dtype != torch.float32 or tuple(idx.shape) != (T, top) or tuple(wts.shape) != (T, top):
            raise KernelError("moe_experts: the choice must be int32 [T, top] with float32 weights")
        if out is None:
            if accumulate:
                raise KernelError("moe_experts: accumulate needs an output")
            out = torch.empty((T, E), dtype=torch.float32, device=h.device)
        elif out.dtype != torch.float32 or tuple(out.shape) != (T, E) or out.stride(1) != 1:
            raise KernelError(f"moe_experts: the output must be float32 [{T}, {E}]")
        z = torch.empty((T * top, F), dtype=h.dtype, device=h.device)
        if (self.use_mfma and h.dtype == torch.bfloat16 and T * top >= self.GROUPED_EXPERTS_FROM and E % 8 == 0 and F % 8 == 0
                and h.stride(0) % 8 == 0 and h.data_ptr() % 16 == 0 and n <= 1024 and T * top <= (1 << 24)):
            # many rows: sorted by expert, both products on the matrix cores, then the weighted sum
            A = T * top
            yz = torch.empty((A, E), dtype=torch.float32, device=h.device)
            scratch = torch.empty((A + 3 * (-(-A // 16) + n) + 1,), dtype=torch.int32, device=h.device)
            gu = torch.empty((A, 2 * F), dtype=torch.float32, device=h.device) if gated else None
            self.lib.check(self.lib.xr_moe_experts_grouped(out.data_ptr(), z.data_ptr(), yz.data_ptr(), scratch.data_ptr(),
                                                           h.data_ptr(), w_up.data_ptr(), w_down.data_ptr(), idx.data_ptr(),
                                                           wts.data_ptr(), T, E, F, h.stride(0), out.stride(0), n, top,
                                                           1 if accumulate else 0, _ptr(gu), _stream()))
            return out
        self.lib.check(self.lib.xr_moe_experts(out.data_ptr(), z.data_ptr(), h.data_ptr(), w_up.data_ptr(), w_down.data_ptr(),
                                               idx.data_ptr(), wts.data_ptr(), T, E, F, h.stride(0), out.stride(0), n, top,
                                               1 if accumulate else 0, dtype_code(h.dtype), EXPERT_ACTIVATIONS[activation],
                                               _stream()))
        return out

    def delta_prepare_(self, q, k, b, a, a_log, dt_bias, G: int, H: int, D: int, q_scale: float, unit_eps: float) -> None:
        """In place on 32-bit views (``q`` and ``k`` with one row stride, ``b`` and ``a`` with one):
        query and key heads become unit vectors (queries times ``q_scale``), ``b`` becomes
        ``sigmoid(b)``, ``a`` becomes ``exp(-exp(a_log) * softplus(a + dt_bias))`` (``a`` absent: the decays are
        made elsewhere, by ``decay_prepare_`` for one a key channel)."""
        self._dev(q, k, b, a, a_log, dt_bias)
        views = [t for t in (q, k, b, a) if t is not None]
        if (any(v.dtype != torch.float32 or v.stride(1) != 1 for v in views) or q.stride(0) != k.stride(0)
                or (a is not None and b.stride(0) != a.stride(0))):
            raise KernelError("delta_prepare_: q and k, and b and a, must be float32 views with one row stride each")
        if tuple(q.shape[1:]) != (G * D,) or tuple(k.shape[1:]) != (G * D,) or b.shape[1] != H or (a is not None and a.shape[1] != H):
            raise KernelError("delta_prepare_: view widths do not fit the heads")
        if a is not None and (a_log.dtype != torch.float32 or dt_bias.dtype != torch.float32 or a_log.numel() != H or dt_bias.numel() != H):
            raise KernelError(f"delta_prepare_: A_log and dt_bias must be float32 [{H}]")
        self.lib.check(self.lib.xr_delta_prepare(q.data_ptr(), k.data_ptr(), b.data_ptr(), _ptr(a), _ptr(a_log) if a is not None else None,
                                                 _ptr(dt_bias) if a is not None else None, q.shape[0], G, H, D, q.stride(0), b.stride(0),
                                                 float(q_scale), float(unit_eps), _stream()))

    @staticmethod
    def recurrence_state_shape(H: int, D: int, Dv: int):
        """The per-request state of ``linear_recurrence``: S[R j + r][c] of head h at ``[h, j, c, r]``,
        R = the lanes that share a column in the kernel (16 for key sizes above 32, else 4; the
        library is asked for the same numbers before every call)."""
        R = 16 if D > 32 else 4
        return (H, (D + R - 1) // R, Dv, R)

    def linear_recurrence(self, kind: str, q, k, v, state: torch.Tensor, ctx, H: int, G: int, D: int, Dv: int,
                          beta=None, gate=None, decay=None, activation: Optional[str] = None, q_scale: float = 1.0,
                          k_scale: float = 1.0) -> torch.Tensor:
        """The read-outs ``[T, H * Dv]`` (32-bit) of a linear recurrence over every request's rows,
        from and into ``state [slots + 1, *recurrence_state_shape]``.  ``kind`` "retention":
        ``S <- decay_h S + k v^T`` with ``decay [H]``; "delta": ``S <- g S; u = beta (v - S^T k);
        S <- S + k u^T`` with ``beta``/``gate [T, H]``; ``o = S^T q`` after the update in both.  "wkv":
        ``o = (S + diag(u) k v^T)^T q`` before the update ``S <- diag(w) S + k v^T``, with ``w = exp(-exp(x))``
        a token, head and key channel from ``gate`` = x ``[T, H * D]`` and the bonus ``decay`` = u ``[H, D]``.
        "gla": ``S <- diag(w) S + k v^T`` with the decays ``gate`` = w ``[T, H * D]`` as they are, read out after the
        update; "delta_channel": the delta rule with a decay a key channel, ``gate`` = w ``[T, H * D]``, ``beta [T, H]``.
        ``q, k [T, G * D]``, ``v [T, H * Dv]``: 32-bit views that share a row stride.  ``activation`` "silu":
        q, k and v pass SiLU on their way into the kernel (the views themselves stay as they are).  ``q_scale`` / ``k_scale``:
        factors on the queries and on the keys, applied on the way in as well (behind the activation)."""
        if activation not in (None, "silu"):
            raise KernelError(f"linear_recurrence: activation {activation!r} is not built (none, silu)")
        if kind not in RECURRENCES:
            raise KernelError(f"linear_recurrence: kind {kind!r} (known: {sorted(RECURRENCES)})")
        self._dev(q, k, v, state, beta, gate, decay)
        views, gates = (q, k, v), [t for t in (beta, gate) if t is not None]
        if (any(t.dtype != torch.float32 or t.stride(1) != 1 for t in list(views) + gates)
                or len({t.stride(0) for t in views}) != 1 or (kind == "delta" and len({t.stride(0) for t in gates}) > 1)):
            raise KernelError("linear_recurrence: q, k and v, and the gates, must be float32 views with one row stride each")
        T = q.shape[0]
        if tuple(q.shape) != (T, G * D) or tuple(k.shape) != (T, G * D) or tuple(v.shape) != (T, H * Dv):
            raise KernelError("linear_recurrence: view widths do not fit the heads")
        rows, lanes = C.c_int(), C.c_int()
        self.lib.dll.xr_recurrence_state_dims(int(D), C.byref(rows), C.byref(lanes))
        if (H, rows.value, Dv, lanes.value) != self.recurrence_state_shape(H, D, Dv):
            raise KernelError("linear_recurrence: the library lays its state out differently from recurrence_state_shape")
        if state.dtype != torch.float32 or tuple(state.shape[1:]) != self.recurrence_state_shape(H, D, Dv) or not state.is_contiguous():
            raise KernelError(f"linear_recurrence: state must be float32 [slots, {self.recurrence_state_shape(H, D, Dv)}]")
        if kind == "delta":
            if beta is None or gate is None or tuple(beta.shape) != (T, H) or tuple(gate.shape) != (T, H):
                raise KernelError("linear_recurrence: the delta rule needs beta and gate [T, H]")
        elif kind == "delta_channel":
            if beta is None or gate is None or tuple(beta.shape) != (T, H) or tuple(gate.shape) != (T, H * D) or activation is not None:
                raise KernelError(f"linear_recurrence: the delta rule with channel decays needs beta [T, {H}] and decays [T, {H * D}]")
        elif kind == "gla":
            if G != H or beta is not None or activation is not None or gate is None or tuple(gate.shape) != (T, H * D):
                raise KernelError(f"linear_recurrence: gla needs a key head a head and decays [T, {H * D}]")
        elif kind == "wkv":
            if (G != H or beta is not None or activation is not None or gate is None or tuple(gate.shape) != (T, H * D)
                    or decay is None or decay.dtype != torch.float32 or decay.numel() != H * D or not decay.is_contiguous()):
                raise KernelError(f"linear_recurrence: wkv needs a key head a head, decays [T, {H * D}] and float32 bonus [{H}, {D}]")
        elif decay is None or decay.dtype != torch.float32 or decay.numel() != H:
            raise KernelError(f"linear_recurrence: retention needs float32 decay [{H}]")
        out = torch.empty((T, H * Dv), dtype=torch.float32, device=q.device)
        # Retention and wkv over long portions run in chunks side by side (the state before a chunk enters the
        # chunk's last state through the chunk's decays alone: one number a head, or their product channel by
        # channel; a chunk's sum from zero and that add up); the delta rule's chain cannot be cut.
        chunk_len, n_chunks, scratch, prod = 0, 0, None, None
        if kind in ("retention", "wkv", "gla") and ctx.max_q_len >= self.RETENTION_CHUNKED_FROM:
            n = -(-ctx.max_q_len // self.RETENTION_CHUNK)
            if ctx.B * n <= 4096:
                chunk_len, n_chunks = self.RETENTION_CHUNK, n
                scratch = torch.empty((ctx.B * n,) + tuple(state.shape[1:]), dtype=torch.float32, device=q.device)
                if kind in ("wkv", "gla"):
                    prod = torch.empty((ctx.B * n, H, rows.value * lanes.value), dtype=torch.float32, device=q.device)
        self.lib.check(self.lib.xr_linear_recurrence(out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), _ptr(beta),
                                                     _ptr(gate), _ptr(decay), state.data_ptr(), ctx.cu_q.data_ptr(),
                                                     ctx.slots.data_ptr(), ctx.B, H, G, D, Dv, q.stride(0),
                                                     gate.stride(0) if gate is not None else 0,
                                                     beta.stride(0) if beta is not None else 0, RECURRENCES[kind],
                                                     chunk_len, n_chunks, _ptr(scratch), _ptr(prod), 1 if activation else 0,
                                                     float(q_scale), float(k_scale), _stream()))
        return out

    RETENTION_CHUNK = 256            # rows a chunk; a multiple of the kernel's 16 staged tokens
    RETENTION_CHUNKED_FROM = 1024    # the longest portion of a step from which chunks pay

    # -- windowed attention with pooled blocks ----------------------------------
    def qkv_store(self, q, k, v, k_cache, v_cache, ctx, group: int, H: int, Hk: int, D: int, Dv: int, page_size: int,
                  out_dtype: torch.dtype) -> torch.Tensor:
        """Queries ``[T, H * D]`` in ``out_dtype``; keys ``[T, Hk * D]`` and values ``[T, Hk * Dv]`` to
        their pages (``k``/``v`` None: this layer stores none).  Inputs are 32-bit views with one row stride."""
        self._dev(q, k, v, k_cache, v_cache)
        views = [t for t in (q, k, v) if t is not None]
        if any(t.dtype != torch.float32 or t.stride(1) != 1 for t in views) or len({t.stride(0) for t in views}) != 1:
            raise KernelError("qkv_store: q, k and v must be float32 views with one row stride")
        T = q.shape[0]
        writes = k is not None
        if writes and (k_cache.dtype != out_dtype or tuple(k_cache.shape[1:]) != (Hk, page_size, D)
                       or tuple(v_cache.shape[1:]) != (Hk, Dv, page_size)):
            raise KernelError("qkv_store: the cache does not fit the heads")
        table = ctx.block_table(group)
        q_out = torch.empty((T, H * D), dtype=out_dtype, device=q.device)
        self.lib.check(self.lib.xr_qkv_store(q_out.data_ptr(), _ptr(k_cache) if writes else None,
                                             _ptr(v_cache) if writes else None, q.data_ptr(), _ptr(k), _ptr(v), q.stride(0),
                                             ctx.positions.data_ptr(), ctx.req_of_token.data_ptr(), table.data_ptr(),
                                             table.stride(0), T, H, Hk if writes else 0, D, Dv, page_size,
                                             dtype_code(out_dtype), _stream()))
        return q_out

    def pool_blocks(self, pk, pv, k_cache, v_cache, ctx, group: int, pool_group: int, Hk: int, D: int, Dv: int, P: int,
                    page_size: int) -> None:
        """Write the mean key and mean value of every block of ``P`` positions that this step
        completes into the blocks' cache (entry b of a request at place b of its table in ``pool_group``)."""
        self._dev(pk, pv, k_cache, v_cache)
        table, ptable = ctx.block_table(group), ctx.block_table(pool_group)
        most = ctx.max_q_len // P + 1           # no request completes more blocks than this in one step
        self.lib.check(self.lib.xr_pool_blocks(pk.data_ptr(), pv.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                               ctx.starts_dev.data_ptr(), ctx.cu_q.data_ptr(), table.data_ptr(),
                                               table.stride(0), ptable.data_ptr(), ptable.stride(0), ctx.B, most, Hk, D, Dv,
                                               P, page_size, dtype_code(k_cache.dtype), _stream()))

    def attention_pooled(self, q, k_cache, v_cache, pk, pv, ctx, group: int, pool_group: Optional[int], H: int, Hk: int,
                         D: int, Dv: int, page_size: int, scale: float, size: int, P: int,
                         matrix_cores: bool = True) -> torch.Tensor:
        """Attention of every token of the step over the last ``size`` keys of its request and the
        means of the blocks of ``P`` positions that end at least ``size`` positions back (``P`` = 0: none); ``[T, H * Dv]``."""
        self._dev(q, k_cache, v_cache, pk, pv)
        self._contig(q, "attention queries")
        if q.dtype != k_cache.dtype or q.dtype != v_cache.dtype:
            raise KernelError("attention: queries and cache differ in dtype")
        T = q.shape[0]
        table = ctx.block_table(group)
        ptable = ctx.block_table(pool_group) if P else None
        out = torch.empty((T, H * Dv), dtype=q.dtype, device=q.device)
        if (matrix_cores and self.use_mfma and q.dtype == torch.bfloat16 and D == Dv and D % 16 == 0 and 16 <= D <= 256
                and page_size >= 16 and H % Hk == 0):
            # The window's keys go to the matrix-core kernels, every row block leaving a partial
            # result; the block means leave theirs in a slot of their own; the kernels' merge adds them.
            lib = self.attention_lib(D)
            plan = ctx.attention_plan(group, H // Hk, size, Hk, page_size, extra_slot=bool(P))
            part_o = part_ml = None
            if plan.n_slots:
                part_o = torch.empty((plan.n_slots, Hk, 32, D), dtype=torch.float32, device=q.device)
                part_ml = torch.empty((plan.n_slots, Hk, 32, 2), dtype=torch.float32, device=q.device)
            if P:
                self.lib.check(self.lib.xr_attention_pool_partial(
                    part_o.data_ptr(), part_ml.data_ptr(), q.data_ptr(), pk.data_ptr(), pv.data_ptr(), plan.extras.data_ptr(),
                    plan.n_extras, ptable.data_ptr(), ptable.stride(0), H, Hk, D, Dv, page_size, float(scale), int(size),
                    int(P), dtype_code(q.dtype), _stream()))
            lib.check(lib.xr_attention_mfma(
                out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), plan.items.data_ptr(),
                plan.n_items, plan.n_cta_items, _ptr(plan.jobs), plan.n_jobs, ctx.cu_q.data_ptr(),
                ctx.starts_dev.data_ptr(), table.data_ptr(), table.stride(0), _ptr(part_o), _ptr(part_ml), H, Hk, D, page_size,
                float(scale), int(size), 0, None, None, _stream()))
            return out
        self.lib.check(self.lib.xr_attention_pooled(
            out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), _ptr(pk) if P else None,
            _ptr(pv) if P else None, ctx.positions.data_ptr(), ctx.req_of_token.data_ptr(), table.data_ptr(),
            table.stride(0), _ptr(ptable), ptable.stride(0) if P else 0, T, H, Hk, D, Dv, page_size, float(scale),
            int(size), int(P), dtype_code(q.dtype), _stream()))
        return out

    # -- sampling ---------------------------------------------------------------
    def sample(self, logits, temp, draw, top_k=None, top_p=None, min_p=None, repeat_penalty=None,
               recent=None, n_recent=None, exempt=None) -> torch.Tensor:
        """One token id per row of 32-bit ``logits`` (rows with a penalty are changed in place)."""
        self._dev(logits, temp, draw, top_k, top_p, min_p, repeat_penalty, recent, n_recent, exempt)
        if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1:
            raise KernelError("sample: logits must be float32 [rows, vocab]")
        W, V = logits.shape
        out = torch.empty((W,), dtype=torch.int32, device=logits.device)
        # room for the greedy rows' first pass (32 ranges a row) when a row is long enough to need one
        greedy_ws = torch.empty((W, 32, 2), dtype=torch.float32, device=logits.device) if V >= 8192 else None
        self.lib.check(self.lib.xr_sample(
            out.data_ptr(), logits.data_ptr(), W, V, logits.stride(0), temp.data_ptr(), _ptr(top_k),
            _ptr(top_p), _ptr(min_p), _ptr(repeat_penalty), draw.data_ptr(), _ptr(recent), _ptr(n_recent),
            recent.shape[1] if recent is not None else 0, _ptr(exempt),
            exempt.numel() if exempt is not None else 0, _ptr(greedy_ws), _stream()))
        return out


_LOCK = threading.Lock()
_OPS: Optional[Ops] = None


def load_ops() -> Ops:
    """The kernel library, loaded once per process (compiled first if it must be)."""
    global _OPS
    with _LOCK:
        if _OPS is None:
            path = _build.find_built("kernels") or _build.build_unit("kernels")
            _OPS = Ops(_Lib(path, _PROTOS))
        return _OPS
