"""The engine's operations, as checked calls into the HIP kernel library.

Every function checks on the host that shapes, dtypes, devices and contiguity
are what its kernel and grid assume before anything is launched, and raises
otherwise.  There is no CPU implementation here: on a machine without the
library or without a GPU every call raises.  Kernels run on torch's current
HIP stream, so they order with torch's own work and can be captured in graphs.

dtype rules: activations are float32 or bfloat16; the residual stream and
logits are always float32; a weight may be float32 or bfloat16 independently of
the activations (a tensor stored in 32-bit stays so).
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import build as _build
from . import key_pieces

F32, BF16, I32 = 0, 1, 2
_CODES = {torch.float32: F32, torch.bfloat16: BF16}

_hip = None


class KernelError(RuntimeError):
    pass


def _code(t: torch.Tensor, what: str) -> int:
    if t.dtype not in _CODES:
        raise KernelError("%s has dtype %s; float32 or bfloat16 expected" % (what, t.dtype))
    return _CODES[t.dtype]


def _check(cond: bool, msg: str, *args) -> None:
    """``msg % args`` is made only when the check fails."""
    if not cond:
        raise KernelError(msg % args if args else msg)


def _dev(*tensors) -> None:
    # (messages are made only when a check fails: a step has thousands of these)
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("a kernel operand lies on %s; the kernels run on the GPU only" % t.device)
        if not t.is_contiguous():
            raise KernelError("a kernel operand is not contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError("kernel operands lie on different devices")


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


class _Hip:
    """ctypes view of the library; one instance per process."""

    def __init__(self):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: spyinfer_amd runs on an AMD GPU (gfx950) only")
        self.lib = _build.load()
        self.lib.spy_last_error.restype = ctypes.c_char_p
        for name in ("spy_embedding", "spy_add_rmsnorm", "spy_rmsnorm", "spy_gemm", "spy_qknorm_rope_store",
                     "spy_attention_generic", "spy_attention_mfma", "spy_attention_mfma_workspace", "spy_attention_mfma_part_workspace", "spy_attention_prefill",
                     "spy_attention_prefill_workspace", "spy_swiglu", "spy_untile_weight",
                     "spy_sample", "spy_sample_workspace", "spy_gemm_skinny", "spy_gemm_skinny_swiglu",
                     "spy_gemm_decode", "spy_gemm_decode_workspace", "spy_embedding_sumsq", "spy_sample_static", "spy_measure_read"):
            if not hasattr(self.lib, name):
                raise KernelError("the kernel library %s lacks %s: it is older than its sources; build it again "
                                  "(spyinfer_amd.kernels.build.build())" % (self.lib._name, name))
            getattr(self.lib, name).restype = ctypes.c_int64 if name.endswith("_workspace") else ctypes.c_int
        # the entry point that a step calls most: with its argument types declared, plain numbers go in as they are (no
        # ctypes object per argument: 3 us of the host's 14 per call)
        P, I = ctypes.c_void_p, ctypes.c_int
        self.lib.spy_gemm_decode.argtypes = [P, I, P, I, ctypes.c_float, P, I, P, I, P, P, P, P, I, I, I, I, I, P, ctypes.c_int64, P]

    def call(self, name, *args):
        rc = getattr(self.lib, name)(*args)
        if rc != 0:
            message = self.lib.spy_last_error().decode()
            # a call that failed may have left counters of the device's workspace away from zero (a launch that went out
            # in part); with such a counter no block of a later call would ever count itself last, and that call would
            # write nothing and report nothing.  So the workspaces start from zero again.
            if not torch.cuda.is_current_stream_capturing():
                for ws in _decode_workspaces.values():
                    try:
                        ws.zero_()
                    except RuntimeError:
                        pass                      # the device itself is in trouble: the first error is the one to report
            raise KernelError("%s: %s" % (name, message))

    @staticmethod
    def stream():
        # torch's current HIP stream of the current device, by the two calls that do no more than read it (the Stream
        # object of torch.cuda.current_stream() costs 3 us to build, and a step has hundreds of launches)
        return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice()))


def hip() -> _Hip:
    global _hip
    if _hip is None:
        _hip = _Hip()
    return _hip


def library_path() -> str:
    return hip().lib._name


# --------------------------------------------------------------------------
def embedding(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] widened to float32 (the start of the residual stream)."""
    _dev(ids, table)
    _check(ids.dtype == torch.int32 and ids.dim() == 1, "embedding: ids must be int32 [T]")
    _check(table.dim() == 2, "embedding: table must be [V, H]")
    T, (V, H) = ids.shape[0], table.shape
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    if T:
        hip().call("spy_embedding", _ptr(out), _ptr(table), _code(table, "embedding table"), _ptr(ids),
                   ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(V), _Hip.stream())
    return out


def add_rms_norm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                 out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """resid += delta (float32, in place; skipped if delta is None), then RMS-normalise.

    Without ``rows``: every row is updated and normalised -> [T, H].  With ``rows``
    (int32 [R]): only those rows are summed and normalised -> [R, H]; resid is left as it is."""
    _dev(resid, delta, weight, rows)
    _check(resid.dtype == torch.float32 and resid.dim() == 2, "add_rms_norm: the residual stream must be float32 [T, H]")
    T, H = resid.shape
    _check(weight.shape == (H,), "add_rms_norm: weight must be [H]")
    if delta is not None:
        _check(delta.shape == (T, H) and delta.dtype == out_dtype, "add_rms_norm: delta must be [T, H] of the activation dtype")
    if rows is not None:
        _check(rows.dtype == torch.int32 and rows.dim() == 1, "add_rms_norm: rows must be int32 [R]")
    n_out = T if rows is None else rows.shape[0]
    out = torch.empty((n_out, H), dtype=out_dtype, device=resid.device)
    if n_out:
        hip().call("spy_add_rmsnorm", _ptr(resid), _ptr(delta), _ptr(weight), _code(weight, "norm weight"),
                   ctypes.c_float(eps), _ptr(out), _code(out, "norm output"), _ptr(rows), ctypes.c_int(n_out),
                   ctypes.c_int(T), ctypes.c_int(H), _Hip.stream())
    return out


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm over the last dimension, same dtype out as in."""
    _dev(x, weight)
    n = x.shape[-1]
    _check(weight.shape == (n,), "rms_norm: weight must match the last dimension")
    out = torch.empty_like(x)
    rows = x.numel() // n if n else 0
    if rows:
        hip().call("spy_rmsnorm", _ptr(x), _code(x, "rms_norm input"), _ptr(weight), _code(weight, "norm weight"),
                   ctypes.c_float(eps), _ptr(out), ctypes.c_int64(rows), ctypes.c_int(n), _Hip.stream())
    return out


#: A bfloat16 product with at most this many rows runs on the hand-written streaming MFMA kernel
#: (decode); above, the library product (hipBLASLt via torch) stands, as the reference sends
#: m >= 8 to cuBLAS (src/backends/cuda/cuda_operator.cpp).  float32 results of bfloat16 operands
#: (logits) always come from the hand-written kernels, which keep the float32 sums.
SKINNY_MAX_ROWS = 16
SKINNY_MAX_ROWS_F32_OUT = 64
_LIBRARY_F32_OUT = True      # torch.mm(..., out_dtype=float32) exists in this torch (float32 sums kept in the result)


#: Most rows that the decode products (``decode_linear`` and its kin) take.
FUSED_DECODE_MAX_ROWS = 128


def default_fold_rows(weight_elements: int) -> int:
    """Most rows of a step for which a part with ``weight_elements`` matrix elements should run its products with the
    norms and residual sums folded in (above: the library product with norm kernels of their own), where the part's
    builder names no limit.  Measured on MI355X at the Qwen3-8B shape: a step of 32 / 64 requests takes 4.4 / 5.8 ms with
    them against 5.9 / 7.4 with the library's products, one of 65 / 96 / 128 requests 7.0 / 7.9 / 9.5 against 7.9 / 9.0
    / 10.3.  So: as many rows as the decode products take, whatever the size."""
    return FUSED_DECODE_MAX_ROWS


def tile_weight(w: torch.Tensor) -> Optional[torch.Tensor]:
    """``w [N, K]`` in the order the decode kernel reads it: [K/128 chunks][N/16 tiles][4 steps][g = 4][r = 16][8], the
    values of lane 16 g + r being w[16 tile + r][128 chunk + 32 step + 8 g ..].  None if the shape or dtype
    does not allow it (then the kernel for row-major matrices stands)."""
    if not w.is_cuda or w.dtype != torch.bfloat16 or w.dim() != 2:
        return None
    N, K = w.shape
    if N % 16 or K % 128 or N * 256 + 8192 >= (1 << 32):
        return None
    return w.view(N // 16, 16, K // 128, 4, 4, 8).permute(2, 0, 3, 4, 1, 5).contiguous().view(N, K)


#: False while a model's weights are bound: a bfloat16 matrix that has a tiled copy is kept in that form only
#: (``weight_forms``), which halves the weights' device memory; a product of many rows then restores the rows into a
#: scratch tensor first (``TiledOnly.rows``), which costs a sixth more time in a prompt portion of 2048 tokens.
ROW_MAJOR_WEIGHTS = True
#: most rows that a product takes straight from the tiled copy when the rows of the matrix are not kept
TILED_ONLY_DIRECT_ROWS = 64
_untile_scratch = {}          # device -> the newest tensor that restored rows go to


def untile_weight(tiled: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The matrix [N, K] whose ``tile_weight`` is ``tiled``, into ``out`` if one is brought."""
    _dev(tiled, out)
    _check(tiled.dtype == torch.bfloat16 and tiled.dim() == 2, "untile_weight: a bfloat16 matrix from tile_weight expected")
    N, K = tiled.shape
    out = _result(out, N, K, torch.bfloat16, tiled.device)
    hip().call("spy_untile_weight", _ptr(out), _ptr(tiled), ctypes.c_int(N), ctypes.c_int(K), _Hip.stream())
    return out


class TiledOnly:
    """Stands where a product expects the matrix [N, K] of which only the tiled copy is kept: it has the matrix's
    shape, dtype and device, and ``rows()`` restores the matrix for the library's product into a scratch tensor of the
    device, which the matrices use in turn and which holds the rows until the next call (the steps run on one stream).
    A matrix keeps the scratch tensor it was made with: if a larger matrix makes a larger one later, the older matrices
    go on with theirs, so that the address a captured step has recorded for a matrix's rows stays good as long as the
    matrix lives, and a captured step holds no restored rows of its own."""
    __slots__ = ("tiled", "_buf")

    shape = property(lambda self: self.tiled.shape)
    dtype = property(lambda self: self.tiled.dtype)
    device = property(lambda self: self.tiled.device)
    is_cuda = property(lambda self: self.tiled.is_cuda)

    def dim(self) -> int:
        return 2

    def is_contiguous(self) -> bool:
        return True

    def __init__(self, tiled: torch.Tensor):
        self.tiled = tiled
        # The device's scratch tensor is made large enough now, while the weights are bound, so that the memory left for
        # the cache counts it; the matrix takes hold of it at its first use, when all matrices of its model exist and
        # the tensor has the size of the largest.
        buf = _untile_scratch.get(tiled.device)
        if buf is None or buf.numel() < tiled.numel():
            _untile_scratch[tiled.device] = torch.empty((tiled.numel(),), dtype=torch.bfloat16, device=tiled.device)
        self._buf = None

    def rows(self) -> torch.Tensor:
        t = self.tiled
        if self._buf is None:
            self._buf = _untile_scratch[t.device]
        return untile_weight(t, self._buf[:t.numel()].view(t.shape))


def weight_forms(w: torch.Tensor, keep_rows: bool = False):
    """(matrix, tiled copy or None) as a part keeps them for ``linear``: both forms, or, with ROW_MAJOR_WEIGHTS off and
    a tiled copy at hand, the tiled copy alone (the first member is then a TiledOnly).  ``keep_rows``: the rows are
    needed for something else than products (an embedding table) and stay."""
    tiled = tile_weight(w)
    if tiled is not None and not ROW_MAJOR_WEIGHTS and not keep_rows:
        return TiledOnly(tiled), tiled
    return w, tiled


def _result(out: Optional[torch.Tensor], M: int, N: int, dtype: torch.dtype, device) -> torch.Tensor:
    """The [M, N] result tensor of a product: ``out`` if the caller brought one (checked), else a new one."""
    if out is None:
        return torch.empty((M, N), dtype=dtype, device=device)
    _check(tuple(out.shape) == (M, N) and out.dtype == dtype and out.device == device and out.is_contiguous(),
           "the result tensor brought by the caller must be contiguous %s [%d, %d] on %s", dtype, M, N, device)
    return out


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           tiled: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x . w^T with w stored [N, K] (out_features, in_features), float32 accumulation.
    ``tiled``: the same matrix from ``tile_weight``, used when few bfloat16 rows stream it.
    ``out``: the result is written there (a tensor of the result's shape and dtype) instead of into a new tensor.

    float32 anywhere among x and w -> the hand-written true-fp32 kernel.  All bfloat16: the streaming
    MFMA kernel for few rows, the library product for many."""
    _dev(x, w)
    _check(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], "linear: x [M, K] and w [N, K] expected, got %s and %s"
           % (tuple(x.shape), tuple(w.shape)))
    M, K = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or x.dtype
    _check(out_dtype in _CODES, "linear: output dtype must be float32 or bfloat16")
    out = _result(out, M, N, out_dtype, x.device)
    if M == 0:
        return out
    all_bf16 = x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
    if isinstance(w, TiledOnly):
        _check(x.dtype == torch.bfloat16, "linear: a matrix kept in tiles only takes bfloat16 rows")
        tiled = w.tiled
    if all_bf16 and tiled is not None and M <= (TILED_ONLY_DIRECT_ROWS if isinstance(w, TiledOnly) else SKINNY_MAX_ROWS):
        _check(tiled.shape == w.shape, "linear: the tiled copy does not fit the matrix")
        return decode_linear(x, tiled, out_dtype, out)
    if isinstance(w, TiledOnly):
        w = w.rows()
    global _LIBRARY_F32_OUT
    if all_bf16 and out_dtype == torch.float32 and M > SKINNY_MAX_ROWS and _LIBRARY_F32_OUT:
        try:
            return torch.mm(x, w.t(), out_dtype=torch.float32, out=out)      # logits of many rows: the library, float32 result
        except TypeError:
            _LIBRARY_F32_OUT = False
    if all_bf16 and K % 8 == 0 and M <= (SKINNY_MAX_ROWS_F32_OUT if out_dtype == torch.float32 else SKINNY_MAX_ROWS):
        hip().call("spy_gemm_skinny", _ptr(x), _ptr(w), _ptr(out), _code(out, "out"), ctypes.c_int(M), ctypes.c_int(N),
                   ctypes.c_int(K), _Hip.stream())
        return out
    if all_bf16 and out_dtype == torch.bfloat16 and M > SKINNY_MAX_ROWS:
        return torch.matmul(x, w.t(), out=out)
    hip().call("spy_gemm", _ptr(x), _code(x, "x"), _ptr(w), _code(w, "w"), _ptr(out), _code(out, "out"),
               ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(K), _Hip.stream())
    return out


def linear_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor, tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(x . Wgate^T) * (x . Wup^T) with ``w_gate_up [2 I, K]`` = [Wgate | Wup] -> [M, I].  For few bfloat16 rows
    (decode) one kernel does both products and the SwiGLU; otherwise it is linear() followed by swiglu()."""
    _dev(x, w_gate_up)
    _check(x.dim() == 2 and w_gate_up.dim() == 2 and x.shape[1] == w_gate_up.shape[1] and w_gate_up.shape[0] % 2 == 0,
           "linear_swiglu: x [M, K] and w [2 I, K] expected")
    M, K = x.shape
    I = w_gate_up.shape[0] // 2
    if x.dtype == torch.bfloat16 and tiled is not None and 0 < M <= SKINNY_MAX_ROWS and I % 16 == 0:
        _check(tiled.shape == w_gate_up.shape, "linear_swiglu: the tiled copy does not fit")
        return decode_linear_swiglu(x, tiled)
    if x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16 and 0 < M <= SKINNY_MAX_ROWS and K % 8 == 0 \
            and (I + 16) * K * 2 < (1 << 32):
        out = torch.empty((M, I), dtype=x.dtype, device=x.device)
        hip().call("spy_gemm_skinny_swiglu", _ptr(x), _ptr(w_gate_up), _ptr(out), _code(out, "out"), ctypes.c_int(M),
                   ctypes.c_int(I), ctypes.c_int(K), _Hip.stream())
        return out
    return swiglu(linear(x, w_gate_up))


# --------------------------------------------------------------------------
# Decode-time products with the norm and the residual sum folded in
def row_tiles(rows: int) -> int:
    """Row tiles of 16 that the decode products are built with for ``rows`` rows: as many as the rows need up to four
    (64 rows); beyond, six (65 to 96 rows) or eight (97 to 128)."""
    return -(-rows // 16) if rows <= 64 else (6 if rows <= 96 else 8)


class OperandRows:
    """Rows of bfloat16 [M, K], M <= 128, in the order the MFMA operand wants them: ``data`` is [K/32 steps, MT row
    tiles, 64 lanes, 8] with lane 16 g + r of row tile t and step s holding x[16 t + r][32 s + 8 g ..]; MT = row_tiles(M);
    rows from M on hold anything.  The decode products write their outputs for each other this way (an
    operand is then one load of 1 KiB in one piece)."""
    __slots__ = ("data", "rows", "width")

    def __init__(self, data: torch.Tensor, rows: int, width: int):
        self.data, self.rows, self.width = data, rows, width

    @property
    def tiles(self) -> int:
        return row_tiles(self.rows)

    @staticmethod
    def empty(rows: int, width: int, device) -> "OperandRows":
        _check(0 < rows <= FUSED_DECODE_MAX_ROWS and width % 32 == 0,
               "operand order takes 1..%d rows of a width that is a multiple of 32", FUSED_DECODE_MAX_ROWS)
        return OperandRows(torch.empty((width // 32, row_tiles(rows), 64, 8), dtype=torch.bfloat16, device=device), rows, width)

    def to_rows(self) -> torch.Tensor:
        """The same values as an ordinary [M, K] tensor (for tests; not used by the engine)."""
        mt = self.tiles
        return self.data.view(self.width // 32, mt, 4, 16, 8).permute(1, 3, 0, 2, 4).reshape(16 * mt, self.width)[:self.rows].contiguous()


class ScaledInput:
    """The input of a product as 'the RMS norm of the residual stream' with the scale still to come:
    ``xw`` = bfloat16(h * w_norm), as [M, K] or as OperandRows, and the parts ``ss_parts [n, MP]`` of every row's sum
    of squares (row r of the stream in column r; their sum over n is sum(h[r]^2); MP = M rounded up to 16).  ``decode_linear`` and
    ``decode_linear_swiglu`` multiply their result by rsqrt(sum / K + eps), which equals the product with the
    normed rows.  ``norm`` is the norm part this was prepared for."""
    __slots__ = ("xw", "ss_parts", "eps", "norm")

    def __init__(self, xw, ss_parts: torch.Tensor, eps: float, norm=None):
        self.xw, self.ss_parts, self.eps, self.norm = xw, ss_parts, float(eps), norm


# Two switches that the tests flip, to hold the folded decode steps against the same steps with norm kernels of their own,
# and the hand-over in operand order against the row-major one; nothing in the engine sets them.
#: False switches the folded decode products off (every norm then runs as a kernel of its own).
FUSED_DECODE = True
#: False: the decode products hand their outputs to each other row-major
OPERAND_ORDER = True


def fused_decode_ok(rows: int, act_dtype, *tiled_weights, max_rows: Optional[int] = None) -> bool:
    """True if products of ``rows`` rows with these tiled matrices can run with the norm's scale and the residual
    sum folded in: bfloat16 activations, at most ``max_rows`` rows (default: ``default_fold_rows`` of the matrices),
    tiled bfloat16 weights."""
    if not FUSED_DECODE or act_dtype != torch.bfloat16 or not 0 < rows <= FUSED_DECODE_MAX_ROWS:
        return False
    if max_rows is None:
        max_rows = default_fold_rows(sum(t.numel() for t in tiled_weights if t is not None))
    if rows > max_rows:
        return False
    if rows > 64 and not (OPERAND_ORDER and all(t is not None and t.shape[0] % 32 == 0 for t in tiled_weights)):
        return False                 # beyond 64 rows the products are built for hand-over in operand order only
    return all(t is not None and t.dtype == torch.bfloat16 and t.shape[0] % 16 == 0 and t.shape[1] % 128 == 0
               for t in tiled_weights)


def folded_products_take(prepared, rows: int) -> bool:
    """Whether the folded decode products can start from what a block has at hand for ``rows`` rows: ``prepared`` is the
    ``ScaledInput`` that the part before made for the block's first norm, or None (a norm kernel then makes ordinary
    [M, K] rows).  Up to 64 rows they take either; beyond, only the operand order that they write for each other."""
    return rows <= 64 or (isinstance(prepared, ScaledInput) and isinstance(prepared.xw, OperandRows))


_decode_workspaces = {}
ATTENTION_COUNTERS = 4096          # counters at the start of the device's workspace (16 KB)


def decode_workspace(device) -> Optional[torch.Tensor]:
    """The device's workspace of the kernels whose blocks meet through memory: the decode products that split K over
    blocks (counters that every call leaves at zero, and the blocks' partial sums) and the attention whose key parts are
    merged by a tile's last block (the same counters).  Made once per device, outside any stream capture, and shared by all calls on the
    device, which therefore must not overlap (the engine runs them on one stream).  None while a capture is under way
    and the device has none yet: those products are then not taken."""
    device = torch.device(device)
    index = device.index if device.index is not None else torch.cuda.current_device()
    ws = _decode_workspaces.get(index)
    if ws is None and not torch.cuda.is_current_stream_capturing():
        ws = torch.zeros((hip().lib.spy_gemm_decode_workspace(),), dtype=torch.uint8, device=torch.device("cuda", index))
        _decode_workspaces[index] = ws
    return ws


def workspace_counters_clean(device) -> bool:
    """True if every counter of the device's workspace is at zero, as each call leaves them (a check for tests and for
    debugging; it waits for the device)."""
    ws = decode_workspace(device)
    return ws is None or not bool(ws[:4 * ATTENTION_COUNTERS].any())


def _gemm_decode(x, tiled: torch.Tensor, epi: int, n_out: int, out, resid, xw_out, w_next, ss_out) -> None:
    _check(tiled.dtype == torch.bfloat16 and tiled.dim() == 2, "decode product: the tiled matrix must be bfloat16 [N, K]")
    K = tiled.shape[1]
    if isinstance(x, ScaledInput):
        xs, ss, eps = x.xw, x.ss_parts, x.eps
        _check(ss.dtype == torch.float32 and ss.dim() == 2 and ss.shape[0] > 0,
               "decode product: the parts of the sums of squares must be float32 [n, rows rounded up to 16]")
    else:
        xs, ss, eps = x, None, 0.0
    x_tiled = isinstance(xs, OperandRows)
    if x_tiled:
        _check(xs.width == K and tuple(xs.data.shape) == (K // 32, xs.tiles, 64, 8) and xs.data.dtype == torch.bfloat16,
               "decode product: x in operand order must be bfloat16 [%d / 32, row tiles, 64, 8]", K)
        M, xs = xs.rows, xs.data
    else:
        _check(xs.dtype == torch.bfloat16 and xs.dim() == 2 and xs.shape[1] == K, "decode product: x must be bfloat16 [M, %d]", K)
        M = xs.shape[0]
    out_tiled = isinstance(out, OperandRows) or isinstance(xw_out, OperandRows)
    mp = 16 * row_tiles(M)
    _check(ss is None or ss.shape[1] == mp, "decode product: the parts of the sums of squares must have %d columns", mp)
    _check(ss_out is None or tuple(ss_out.shape) == (n_out // 16, mp), "decode product: the new parts must be [N / 16, %d]", mp)
    for o in (out, xw_out):
        if isinstance(o, OperandRows):
            _check(o.rows == M and o.width == n_out and tuple(o.data.shape) == (n_out // 32, o.tiles, 64, 8),
                   "decode product: the output in operand order does not fit")
    out_t = out.data if isinstance(out, OperandRows) else out
    xw_t = xw_out.data if isinstance(xw_out, OperandRows) else xw_out
    _dev(xs, ss, tiled, out_t, resid, xw_t, w_next, ss_out)
    _check(0 < M <= FUSED_DECODE_MAX_ROWS, "decode product: %d rows (1..%d allowed)", M, FUSED_DECODE_MAX_ROWS)
    ws = decode_workspace(xs.device)
    at = lambda t: None if t is None else t.data_ptr()              # (argument types are declared: see _Hip)
    hip().call("spy_gemm_decode", at(xs), 0 if ss is None else 1, at(ss), 0 if ss is None else ss.shape[0], eps, at(tiled), epi,
               at(out_t), 0 if out_t is None else _code(out_t, "out"), at(resid), at(xw_t), at(w_next), at(ss_out), M, n_out, K,
               1 if x_tiled else 0, 1 if out_tiled else 0, at(ws), 0 if ws is None else ws.numel(), _Hip.stream())


def _rows_of(x) -> int:
    x = x.xw if isinstance(x, ScaledInput) else x
    return x.rows if isinstance(x, OperandRows) else x.shape[0]


def _operand_order_ok(width: int) -> bool:
    return OPERAND_ORDER and width % 32 == 0


def decode_linear(x, tiled: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x . w^T for few rows; ``x`` bfloat16 [M, K], OperandRows or a ScaledInput, ``tiled`` from tile_weight; the
    result goes into ``out`` if one is brought."""
    N = tiled.shape[0]
    out = _result(out, _rows_of(x), N, out_dtype, tiled.device)
    _gemm_decode(x, tiled, 0, N, out, None, None, None, None)
    return out


def decode_linear_swiglu(x, tiled_gate_up: torch.Tensor, for_product: bool = False):
    """silu(x . Wgate^T) * (x . Wup^T) for at most 128 rows (beyond 64: a normed input in operand order only); ``tiled_gate_up [2 I, K]`` = tiles of [Wgate | Wup].
    ``for_product``: the result goes into another decode product only, and may come as OperandRows."""
    _check(tiled_gate_up.shape[0] % 32 == 0, "decode_linear_swiglu: [2 I, K] with I a multiple of 16 expected")
    I = tiled_gate_up.shape[0] // 2
    if for_product and _operand_order_ok(I):
        out = OperandRows.empty(_rows_of(x), I, tiled_gate_up.device)
    else:
        out = torch.empty((_rows_of(x), I), dtype=torch.bfloat16, device=tiled_gate_up.device)
    _gemm_decode(x, tiled_gate_up, 1, I, out, None, None, None, None)
    return out


def decode_linear_residual(x, tiled: torch.Tensor, resid: torch.Tensor, next_norm_weight: torch.Tensor,
                           eps: float, norm=None) -> ScaledInput:
    """resid += x . w^T (float32, in place) for at most 128 rows (beyond 64: x in operand order only) -> the ScaledInput of the norm that reads the
    stream next: bfloat16(resid * next_norm_weight) and the parts [N / 16, 16] of the new rows' sums of squares."""
    N = tiled.shape[0]
    M = _rows_of(x)
    _check(resid.dtype == torch.float32 and resid.dim() == 2 and resid.shape == (M, N),
           "decode_linear_residual: the stream must be float32 [M, %d]", N)
    _check(next_norm_weight.dtype == torch.bfloat16 and next_norm_weight.shape == (N,),
           "decode_linear_residual: the next norm's weight must be bfloat16 [%d]", N)
    ss = torch.empty((N // 16, 16 * row_tiles(M)), dtype=torch.float32, device=resid.device)
    if _operand_order_ok(N):
        xw = OperandRows.empty(M, N, resid.device)
    else:
        xw = torch.empty((M, N), dtype=torch.bfloat16, device=resid.device)
    _gemm_decode(x, tiled, 2, N, None, resid, xw, next_norm_weight, ss)
    return ScaledInput(xw, ss, eps, norm)


def embedding_scaled(ids: torch.Tensor, table: torch.Tensor, norm_weight: torch.Tensor, eps: float, norm=None):
    """embedding() for few tokens -> (stream, ScaledInput of the first norm)."""
    _dev(ids, table, norm_weight)
    _check(ids.dtype == torch.int32 and ids.dim() == 1 and 0 < ids.shape[0] <= FUSED_DECODE_MAX_ROWS,
           "embedding_scaled: ids must be int32 [1..%d]", FUSED_DECODE_MAX_ROWS)
    _check(table.dim() == 2, "embedding: table must be [V, H]")
    T, (V, H) = ids.shape[0], table.shape
    _check(norm_weight.dtype == torch.bfloat16 and norm_weight.shape == (H,), "embedding_scaled: the norm weight must be bfloat16 [H]")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    tiled = _operand_order_ok(H)
    xw = OperandRows.empty(T, H, table.device) if tiled else torch.empty((T, H), dtype=torch.bfloat16, device=table.device)
    ss = torch.empty((1, 16 * row_tiles(T)), dtype=torch.float32, device=table.device)
    hip().call("spy_embedding_sumsq", _ptr(out), _ptr(xw.data if tiled else xw), _ptr(ss), _ptr(table), _code(table, "embedding table"),
               _ptr(norm_weight), _ptr(ids), ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(V), ctypes.c_int(1 if tiled else 0),
               ctypes.c_int(row_tiles(T)), _Hip.stream())
    return out, ScaledInput(xw, ss, eps, norm)


def qk_norm_rope_store(qkv: torch.Tensor, n_q: int, n_kv: int, d: int, q_norm_w, k_norm_w, eps: float,
                       cos, sin, rotary_dim: int, positions: torch.Tensor, k_cache, v_cache, page_size: int,
                       slots: Optional[torch.Tensor]) -> torch.Tensor:
    """From the fused projection ``qkv [T, (n_q + 2 n_kv) d]``: per-head RMS norm of q and k (if
    weights are given), half-split rotation of the first ``rotary_dim`` dims by the tables
    ``cos/sin [positions, rotary_dim/2]`` (if given), q written to the result ``[T, n_q d]``;
    k and v written into the cache pages at ``slots[t] = page * page_size + offset``
    (skipped for slot -1 or when ``slots`` is None)."""
    _dev(qkv, q_norm_w, k_norm_w, cos, sin, positions, k_cache, v_cache, slots)
    T = qkv.shape[0]
    _check(qkv.dim() == 2 and qkv.shape[1] == (n_q + 2 * n_kv) * d, "qk_norm_rope_store: qkv must be [T, (n_q + 2 n_kv) d]")
    _check(positions.dtype == torch.int32 and positions.shape == (T,), "qk_norm_rope_store: positions must be int32 [T]")
    _check((q_norm_w is None) == (k_norm_w is None), "qk_norm_rope_store: q and k norm weights come together")
    if q_norm_w is not None:
        _check(q_norm_w.shape == (d,) and k_norm_w.shape == (d,) and q_norm_w.dtype == k_norm_w.dtype,
               "qk_norm_rope_store: norm weights must be [head_dim] of one dtype")
    max_pos = 0
    if cos is not None:
        _check(rotary_dim % 2 == 0 and 0 < rotary_dim <= d, "qk_norm_rope_store: rotary_dim must be even and <= head_dim")
        _check(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.dim() == 2 and cos.shape == sin.shape
               and cos.shape[1] == rotary_dim // 2, "qk_norm_rope_store: cos/sin must be float32 [positions, rotary_dim/2]")
        max_pos = cos.shape[0]
    else:
        rotary_dim = 0
    num_pages = 0
    if slots is not None:
        _check(slots.dtype == torch.int32 and slots.shape == (T,), "qk_norm_rope_store: slots must be int32 [T]")
        _check(k_cache is not None and k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype,
               "qk_norm_rope_store: the cache must have the activation dtype")
        num_pages = k_cache.shape[0]
        _check(tuple(k_cache.shape) == (num_pages, n_kv, page_size, d) and tuple(v_cache.shape) == (num_pages, n_kv, d, page_size),
               "qk_norm_rope_store: cache pages must be K [pages, n_kv, page, d] and V [pages, n_kv, d, page]")
    q = torch.empty((T, n_q * d), dtype=qkv.dtype, device=qkv.device)
    if T:
        hip().call("spy_qknorm_rope_store", _ptr(qkv), _code(qkv, "qkv"), _ptr(q), ctypes.c_int(T), ctypes.c_int(n_q),
                   ctypes.c_int(n_kv), ctypes.c_int(d), _ptr(q_norm_w), _ptr(k_norm_w),
                   ctypes.c_int(-1 if q_norm_w is None else _code(q_norm_w, "q norm weight")), ctypes.c_float(eps),
                   _ptr(cos), _ptr(sin), ctypes.c_int(rotary_dim), ctypes.c_int(max_pos), _ptr(positions),
                   _ptr(k_cache if slots is not None else None), _ptr(v_cache if slots is not None else None),
                   ctypes.c_int(page_size), ctypes.c_int(num_pages), _ptr(slots), _Hip.stream())
    return q


class AttentionMeta:
    """Batch description that the attention kernels read (all int32, on the device).

    cu_q [S+1]: first query token of each entry;  pos0 [S]: position of that token in its request;
    kv_len [S]: keys the request has after this step (pos0 + tokens of the entry);
    block_table [S, max_blocks]: logical page -> physical page (-1 = none);
    token_entry [T], positions [T]: per query token.
    tiles: {"small": (tile_entry [N], tile_row0 [N], N), "big": (...)}: 16-row tiles of (token,
    head-in-group) rows for entries with few rows and 128-row tiles for entries with many, built
    for one group size ``tiles_group``; None if not built.
    ``big_rows``: rows of a "big" tile (128 or 256, see ``prefill_tile_rows``).
    Host-side: S, T, max_blocks, max_kv_len, max_q_len.
    What the arrays say must be true: the kernels read entries, pages and pieces as they are given."""

    def __init__(self, cu_q, pos0, kv_len, block_table, token_entry, positions, S, T, max_blocks, max_kv_len, max_q_len,
                 tiles=None, tiles_group=0, fixed_shape=False, big_rows=128, pieces=None):
        self.cu_q, self.pos0, self.kv_len, self.block_table = cu_q, pos0, kv_len, block_table
        self.token_entry, self.positions = token_entry, positions
        self.S, self.T, self.max_blocks, self.max_kv_len, self.max_q_len = S, T, max_blocks, max_kv_len, max_q_len
        self.tiles, self.tiles_group, self.big_rows = tiles, tiles_group, big_rows
        #: True: the step is captured in a graph (block tables have a fixed width; what a launch's shape takes from the
        #: requests' lengths, the number of key parts, is part of the graph's key)
        self.fixed_shape = fixed_shape
        #: {(n_kv, window, head_dim): int32 [records, 8] on the device}: the keys of a step of single tokens cut into pieces by
        #: ``decode_pieces``, for the attention that takes the raw product; empty if not built
        self.pieces = pieces or {}


MFMA_ATTENTION = True      # False forces the plain kernel for bfloat16 too (the kernel tests flip it; nothing else does)
DECODE_MAX_SPLITS = 16      # most key parts of a tile where the grid cuts them (the merge's time grows with them)
DECODE_KEYS_PER_SPLIT = 256  # a part wants this many keys at least (measured at 1100 keys, 1 to 4 requests: 4-8 parts best)


def key_parts_for(max_kv_len: int) -> int:
    """The most parts into which the keys of 16-row tiles are split when the longest request has ``max_kv_len`` keys.
    A step captured in a graph keeps the number it was captured with, so this number belongs to the graph's key."""
    return max(1, min(DECODE_MAX_SPLITS, -(-int(max_kv_len) // DECODE_KEYS_PER_SPLIT)))
DECODE_SPLIT_TARGET = 256   # blocks (of 4 waves) wanted in flight when all entries are single tokens (measured: B=8 best at 4 parts)


# ---- the keys of a step of single tokens, cut into even shares on the host (key_pieces.py) ----------------------------
DECODE_PIECES = True        # False: every entry's keys in one number of parts (for comparison: tests and the benchmark's --even-key-parts flip it)


def decode_pieces_ok(entries: int, tokens: int, act_dtype, n_kv: int, d: int) -> bool:
    """Whether a step's keys are cut on the host: single tokens only, bfloat16, a head size whose parts the attention
    kernel merges by itself, a counter for every (entry, kv head)."""
    return (DECODE_PIECES and MFMA_ATTENTION and entries == tokens and entries > 0 and act_dtype == torch.bfloat16
            and d in (64, 128) and entries * n_kv <= ATTENTION_COUNTERS)


PREFILL_ATTENTION_MAX_HEAD_DIM = 128
PREFILL_SPLIT_BELOW = 256   # fewer (128-row tile, kv head) pairs than this: split the keys to fill the chip


def prefill_attention_ok(d: int, page_size: int) -> bool:
    """Whether entries with many rows may be cut into 128-row tiles: the LDS-sharing kernel takes head
    sizes up to 128 and pages of a power of two; other shapes run wholly through the general kernel."""
    return d <= PREFILL_ATTENTION_MAX_HEAD_DIM and page_size >= 8 and page_size & (page_size - 1) == 0


#: blocks (pairs of 256-row tiles times kv heads) from which the prefill kernel's tiles have 256 rows instead of 128:
#: three quarters of the 256 compute units (measured: 7 % faster at 192 blocks, 15 % at 256, 26 % slower at 128)
PREFILL_WIDE_TILES_MIN_BLOCKS = 192


def prefill_tile_rows(d: int, rows_of_entries, n_kv: int) -> int:
    """Rows of the tiles that entries with many rows are cut into: 256 for head sizes 64 and 128 when that still gives
    enough blocks to fill the chip (a block takes two tiles of one kv head), else 128.  ``rows_of_entries``: the rows
    (tokens times heads of a group) of every entry that goes to the prefill kernel."""
    if d not in (64, 128):
        return 128
    tiles = sum(-(-int(r) // 256) for r in rows_of_entries)
    return 256 if (tiles + 1) // 2 * n_kv >= PREFILL_WIDE_TILES_MIN_BLOCKS else 128


def mfma_attention_ok(dtype, d: int, page_size: int) -> bool:
    return MFMA_ATTENTION and dtype == torch.bfloat16 and d % 16 == 0 and 16 <= d <= 256 and page_size % 8 == 0


def attention_hands_over_operand_rows(dtype, n_q: int, d: int, page_size: int) -> bool:
    """Whether ``paged_attention(..., for_product=True)`` gives a step of at most 128 tokens, single or in portions, as
    OperandRows: what the folded decode products need of their input beyond 64 rows."""
    return _operand_order_ok(n_q * d) and mfma_attention_ok(dtype, d, page_size)


class RawQKV:
    """The step's raw product [q | k | v] with what turns it into queries, keys and values: the per-head norm weights
    (or None), eps, the rotation tables (or None) and whether this call stores its keys and values.  Handed to
    ``paged_attention`` in place of q when ``fused_attention_ok`` allows it: the attention kernel then does the norm,
    the rotation and the store itself (no kernel of their own in a decode step)."""
    __slots__ = ("qkv", "q_norm_w", "k_norm_w", "eps", "cos", "sin", "store")

    def __init__(self, qkv, q_norm_w, k_norm_w, eps, cos, sin, store):
        self.qkv, self.q_norm_w, self.k_norm_w, self.eps, self.cos, self.sin, self.store = qkv, q_norm_w, k_norm_w, eps, cos, sin, store



def fused_attention_ok(dtype, meta: AttentionMeta, n_q: int, n_kv: int, d: int, page_size: int, rotary_dim: int, q_norm_w, k_norm_w) -> bool:
    """True if this step's attention may take the raw product (``RawQKV``): every entry a single token, bfloat16,
    head_dim 64, 128 or 256 rotated whole or not at all, 16-row tiles built for this group size."""
    if not mfma_attention_ok(dtype, d, page_size):
        return False
    if meta.T != meta.S or meta.max_q_len != 1 or meta.tiles is None or meta.tiles_group != n_q // n_kv or n_q // n_kv > 16:
        return False
    if meta.tiles["small"][2] != meta.S or meta.tiles["big"][2] != 0:
        return False
    if d not in (64, 128, 256) or rotary_dim not in (0, d) or (q_norm_w is None) != (k_norm_w is None):
        return False
    return q_norm_w is None or (q_norm_w.dtype == k_norm_w.dtype and q_norm_w.dtype in _CODES)


def paged_attention(q: Optional[torch.Tensor], k_cache: torch.Tensor, v_cache: torch.Tensor, page_size: int, meta: AttentionMeta,
                    n_q: int, n_kv: int, d: int, scale: float, window: Optional[int], raw: Optional[RawQKV] = None,
                    for_product: bool = False):
    """Causal grouped-query attention of the step's query tokens over the paged cache
    (which already holds this step's keys and values, or gets them from ``raw`` in this call).  Query at position p
    reads keys max(0, p - window + 1) .. p.  Scores, softmax and the weighted sum are float32.
    ``for_product``: the result goes into a decode product only and may come as OperandRows (it does for steps of at
    most 128 tokens, ``attention_hands_over_operand_rows``)."""
    T, S = meta.T, meta.S
    if raw is not None:
        _dev(raw.qkv, raw.q_norm_w, raw.k_norm_w, raw.cos, raw.sin)
        _check(raw.qkv.dtype == torch.bfloat16 and raw.qkv.shape == (T, (n_q + 2 * n_kv) * d), "paged_attention: raw qkv must be bfloat16 [T, (n_q + 2 n_kv) d]")
        rot = 0 if raw.cos is None else d
        _check(fused_attention_ok(raw.qkv.dtype, meta, n_q, n_kv, d, page_size, rot, raw.q_norm_w, raw.k_norm_w),
               "paged_attention: this step cannot take the raw product (ops.fused_attention_ok)")
        if raw.cos is not None:
            _check(raw.cos.dtype == torch.float32 and raw.sin.dtype == torch.float32 and raw.cos.dim() == 2 and raw.cos.shape[1] == d // 2
                   and raw.sin.shape == raw.cos.shape, "paged_attention: rotation tables must be float32 [positions, d / 2]")
        if raw.q_norm_w is not None:
            _check(raw.q_norm_w.shape == (d,) and raw.k_norm_w.shape == (d,), "paged_attention: head norm weights must be [d]")
        for t in (raw.qkv, raw.q_norm_w, raw.k_norm_w, raw.cos, raw.sin):
            _check(t is None or t.data_ptr() % 16 == 0, "paged_attention: operands of the raw product must be 16-byte aligned")
        q = torch.empty((T, n_q * d), dtype=raw.qkv.dtype, device=raw.qkv.device)     # shape and dtype of the result only
    _dev(q, k_cache, v_cache, meta.cu_q, meta.pos0, meta.kv_len, meta.block_table, meta.token_entry, meta.positions)
    _check(q.shape == (T, n_q * d), "paged_attention: q must be [T, n_q d]")
    _check(n_q % n_kv == 0, "paged_attention: n_q must be a multiple of n_kv")
    num_pages = k_cache.shape[0]
    _check(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype, "paged_attention: cache and q must have one dtype")
    _check(tuple(k_cache.shape) == (num_pages, n_kv, page_size, d) and tuple(v_cache.shape) == (num_pages, n_kv, d, page_size),
           "paged_attention: cache pages must be K [pages, n_kv, page, d] and V [pages, n_kv, d, page]")
    for name, t, shape in (("cu_q", meta.cu_q, (S + 1,)), ("pos0", meta.pos0, (S,)), ("kv_len", meta.kv_len, (S,)),
                           ("block_table", meta.block_table, (S, meta.max_blocks)), ("token_entry", meta.token_entry, (T,)),
                           ("positions", meta.positions, (T,))):
        _check(t.dtype == torch.int32 and tuple(t.shape) == shape, "paged_attention: %s must be int32 %s", name, shape)
    _check(meta.max_kv_len <= meta.max_blocks * page_size, "paged_attention: block tables are shorter than the longest request")
    win = 0 if window is None else int(window)
    _check(win >= 0, "paged_attention: window must be positive")
    out = q if raw is not None else torch.empty_like(q)
    if T == 0:
        return out
    group = n_q // n_kv
    operand = None
    if for_product and T <= FUSED_DECODE_MAX_ROWS and meta.tiles is not None and meta.tiles_group == group \
            and attention_hands_over_operand_rows(q.dtype, n_q, d, page_size):
        operand = OperandRows.empty(T, n_q * d, q.device)
        out = operand.data
    if mfma_attention_ok(q.dtype, d, page_size) and meta.tiles is not None and meta.tiles_group == group:
        small_entry, small_row0, n_small = meta.tiles["small"]
        big_entry, big_row0, n_big = meta.tiles["big"]
        for name, t, n in (("small tile entries", small_entry, n_small), ("small tile rows", small_row0, n_small),
                           ("big tile entries", big_entry, n_big), ("big tile rows", big_row0, n_big)):
            _check(t.dtype == torch.int32 and tuple(t.shape) == (n,), "paged_attention: %s must be int32 [%d]", name, n)
        common = (ctypes.c_int(page_size), ctypes.c_int(num_pages), _ptr(meta.cu_q), _ptr(meta.pos0), _ptr(meta.kv_len),
                  _ptr(meta.block_table), ctypes.c_int(meta.max_blocks))
        sizes = (ctypes.c_int(S), ctypes.c_int(T), ctypes.c_int(n_q), ctypes.c_int(n_kv), ctypes.c_int(d), ctypes.c_float(scale),
                 ctypes.c_int(win))
        if n_big and not prefill_attention_ok(d, page_size):
            raise KernelError("paged_attention: 128-row tiles were built for head_dim %d and pages of %d, which the prefill "
                              "kernel refuses; build 16-row tiles only (ops.prefill_attention_ok)" % (d, page_size))
        if n_big:
            # few tiles with many keys (a late portion of a long prompt): their keys are split into parts as well
            bsplits = 1
            if n_big * n_kv < PREFILL_SPLIT_BELOW:
                bsplits = max(1, min(PREFILL_SPLIT_BELOW * 2 // (n_big * n_kv), meta.max_kv_len // 256, 16))
            _check(meta.big_rows in (128, 256), "paged_attention: tiles of 128 or 256 rows expected")
            bws_floats = hip().lib.spy_attention_prefill_workspace(ctypes.c_int(n_big), ctypes.c_int(meta.big_rows), ctypes.c_int(n_kv),
                                                                   ctypes.c_int(d), ctypes.c_int(bsplits))
            bws = torch.empty((max(1, bws_floats),), dtype=torch.float32, device=q.device)
            hip().call("spy_attention_prefill", _ptr(out), _ptr(q), _ptr(k_cache), _ptr(v_cache), *common, _ptr(big_entry),
                       _ptr(big_row0), ctypes.c_int(n_big), ctypes.c_int(meta.big_rows), *sizes, ctypes.c_int(bsplits), _ptr(bws),
                       ctypes.c_int(operand.tiles if operand is not None else 0), _Hip.stream())
        if n_small:
            # Few 16-row tiles cannot fill the chip by themselves (decoding requests, short portions): their keys are
            # split into parts, each part a block of 4 waves that wants 128 keys at least, and a second kernel merges.
            want = max(1, DECODE_SPLIT_TARGET // max(1, n_small * n_kv))
            splits = max(1, min(want, key_parts_for(meta.max_kv_len)))
            # a step of single tokens whose keys the host has cut into pieces (decode_pieces): one block per record
            pieces = meta.pieces.get((n_kv, win, d)) if raw is not None and d <= 128 and n_small * n_kv <= ATTENTION_COUNTERS else None
            counters = decode_workspace(q.device) if splits > 1 or pieces is not None else None
            if counters is None:
                pieces = None
            if pieces is not None:
                _dev(pieces)
                _check(pieces.dtype == torch.int32 and pieces.dim() == 2 and pieces.shape[1] == key_pieces.PIECE_RECORD and pieces.shape[0] > 0
                       and pieces.data_ptr() % 16 == 0, "paged_attention: pieces must be int32 [records, 8], 16-byte aligned")
                ws_floats = pieces.shape[0] * hip().lib.spy_attention_mfma_part_workspace(ctypes.c_int(d))
                splits = 1
            else:
                ws_floats = hip().lib.spy_attention_mfma_workspace(ctypes.c_int(n_small), ctypes.c_int(n_kv), ctypes.c_int(d),
                                                                   ctypes.c_int(splits))
            ws = torch.empty((max(1, ws_floats),), dtype=torch.float32, device=q.device)
            # with counters the last block of a (tile, kv head) merges its parts; without, a second kernel does
            if raw is not None:
                wcode = _code(raw.q_norm_w, "head norm weight") if raw.q_norm_w is not None else F32
                fused = (_ptr(raw.qkv), _ptr(raw.q_norm_w), _ptr(raw.k_norm_w), ctypes.c_int(wcode), ctypes.c_float(raw.eps),
                         _ptr(raw.cos), _ptr(raw.sin), ctypes.c_int(0 if raw.cos is None else raw.cos.shape[0]),
                         ctypes.c_int(1 if raw.store else 0))
            else:
                fused = (_ptr(None), _ptr(None), _ptr(None), ctypes.c_int(0), ctypes.c_float(0.0), _ptr(None), _ptr(None),
                         ctypes.c_int(0), ctypes.c_int(0))
            hip().call("spy_attention_mfma", _ptr(out), _ptr(None if raw is not None else q), _ptr(k_cache), _ptr(v_cache), *common,
                       _ptr(small_entry), _ptr(small_row0), ctypes.c_int(n_small), *sizes, ctypes.c_int(splits), _ptr(ws), *fused,
                       ctypes.c_int(operand.tiles if operand is not None else 0), _ptr(counters),
                       ctypes.c_int(0 if counters is None else ATTENTION_COUNTERS), _ptr(pieces),
                       ctypes.c_int(0 if pieces is None else pieces.shape[0]), _Hip.stream())
        return operand if operand is not None else out
    hip().call("spy_attention_generic", _ptr(out), _ptr(q), _code(q, "q"), _ptr(k_cache), _ptr(v_cache),
               ctypes.c_int(page_size), ctypes.c_int(num_pages), _ptr(meta.kv_len), _ptr(meta.block_table),
               ctypes.c_int(meta.max_blocks), _ptr(meta.token_entry), _ptr(meta.positions), ctypes.c_int(S), ctypes.c_int(T),
               ctypes.c_int(n_q), ctypes.c_int(n_kv), ctypes.c_int(d), ctypes.c_float(scale), ctypes.c_int(win), _Hip.stream())
    return out


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    """``gate_up [T, 2 I]`` = [gate | up]  ->  silu(gate) * up  [T, I], float32 arithmetic."""
    _dev(gate_up)
    _check(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0, "swiglu: [T, 2 I] expected")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    if T * I:
        hip().call("spy_swiglu", _ptr(gate_up), _ptr(out), _code(gate_up, "gate_up"), ctypes.c_int(T), ctypes.c_int(I),
                   _Hip.stream())
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    """Row r: temperature[r] == 0 -> first maximum of logits[r]; else the token whose cumulative
    probability of softmax(logits[r] / temperature[r]), over ascending token ids, first exceeds
    u[r] in [0, 1).  int32 [R]."""
    _dev(logits, temperature, u)
    _check(logits.dtype == torch.float32 and logits.dim() == 2, "sample: logits must be float32 [R, V]")
    R, V = logits.shape
    _check(temperature.dtype == torch.float32 and temperature.shape == (R,) and u.dtype == torch.float32 and u.shape == (R,),
           "sample: temperature and u must be float32 [R]")
    _check(V > 0, "sample: empty vocabulary")
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    if R:
        ws = torch.empty((hip().lib.spy_sample_workspace(ctypes.c_int(R)),), dtype=torch.float32, device=logits.device)
        hip().call("spy_sample", _ptr(logits), _ptr(temperature), _ptr(u), _ptr(out), ctypes.c_int(R), ctypes.c_int(V),
                   _ptr(ws), _Hip.stream())
    return out


# --------------------------------------------------------------------------
def measure_read_rate(device, num_bytes: int = 2 << 30, repeats: int = 5) -> float:
    """Bytes per second that a kernel which only reads gets from this device's memory: ``num_bytes`` (far more than the
    caches hold) read once per launch, the best of ``repeats`` launches.  For measurements (bench.py quotes the decode
    step against it); the engine does not call it."""
    device = torch.device(device)
    num_bytes = max(1 << 20, num_bytes // 16 * 16)
    buf = torch.empty((num_bytes,), dtype=torch.uint8, device=device)
    buf.random_(0, 256)
    blocks = 8 * torch.cuda.get_device_properties(device).multi_processor_count
    sink = torch.zeros((blocks * 256,), dtype=torch.int32, device=device)
    best = None
    for _ in range(repeats + 1):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        hip().call("spy_measure_read", _ptr(buf), ctypes.c_int64(num_bytes), ctypes.c_int(blocks), _ptr(sink), _Hip.stream())
        end.record()
        end.synchronize()
        ms = start.elapsed_time(end)
        best = ms if best is None else min(best, ms)
    return num_bytes / (best * 1e-3)
