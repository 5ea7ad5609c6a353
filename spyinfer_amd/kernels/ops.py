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
                     "spy_gemm_decode", "spy_gemm_decode_workspace", "spy_embedding_sumsq", "spy_sample_static", "spy_measure_read",
                     "spy_pair_embedding", "spy_norm_residual", "spy_depth_mix", "spy_xielu", "spy_mingru", "spy_latent_prepare",
                     "spy_gemm_strided", "spy_latent_attention", "spy_latent_attention_mfma", "spy_latent_attention_mfma_workspace", "spy_head_products",
                     "spy_bias_rope_store", "spy_sigmoid_gate", "spy_mlstm", "spy_causal_conv_silu", "spy_delta_rule", "spy_moe_route",
                     "spy_moe_align", "spy_moe_gemm", "spy_moe_combine", "spy_moe_tile_rows", "spy_token_shift", "spy_tanh", "spy_time_mix",
                     "spy_norm_pair_mean", "spy_scale_cap"):
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
def embedding(ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[t, :] = table[ids[t], :] * scale widened to float32 (the start of the residual stream)."""
    _dev(ids, table)
    _check(ids.dtype == torch.int32 and ids.dim() == 1, "embedding: ids must be int32 [T]")
    _check(table.dim() == 2, "embedding: table must be [V, H]")
    T, (V, H) = ids.shape[0], table.shape
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    if T:
        hip().call("spy_embedding", _ptr(out), _ptr(table), _code(table, "embedding table"), _ptr(ids),
                   ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(V), ctypes.c_float(scale), _Hip.stream())
    return out


def add_rms_norm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                 out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None, delta2: Optional[torch.Tensor] = None, groups: int = 1,
                 gate=None, base: Optional[torch.Tensor] = None, vec: Optional[torch.Tensor] = None,
                 weight2: Optional[torch.Tensor] = None):
    """resid += delta (float32, in place; skipped if delta is None), then RMS-normalise.  ``delta2``: a second addend
    (two sublayers that read one norm): resid += delta + delta2, the two summed in float32 first.  ``groups``: the row is
    cut into that many equal consecutive parts, each over its own root mean square.  ``gate`` = (rows [T, H] of the activation
    dtype, bias [H] of the weight's dtype, constant): the addend is delta * constant * sigmoid(rows + bias), formed in float32.
    ``base``: a float32 addend [T, H] (an earlier state of the stream); ``vec``: a float32 vector [H] added to every row.
    ``weight2``: a second norm of the same sum with this weight: the result is then the pair of both outputs.

    Without ``rows``: every row is updated and normalised -> [T, H].  With ``rows``
    (int32 [R]): only those rows are summed and normalised -> [R, H]; resid is left as it is."""
    _dev(resid, delta, weight, rows, delta2)
    _check(resid.dtype == torch.float32 and resid.dim() == 2, "add_rms_norm: the residual stream must be float32 [T, H]")
    if delta2 is not None:
        _check(delta is not None and delta2.shape == delta.shape and delta2.dtype == delta.dtype, "add_rms_norm: the second addend must be like the first")
    T, H = resid.shape
    _check(weight.shape == (H,), "add_rms_norm: weight must be [H]")
    _check(groups >= 1 and H % groups == 0, "add_rms_norm: %d groups do not divide rows of %d", groups, H)
    if delta is not None:
        _check(delta.shape == (T, H) and delta.dtype == out_dtype, "add_rms_norm: delta must be [T, H] of the activation dtype")
    if rows is not None:
        _check(rows.dtype == torch.int32 and rows.dim() == 1, "add_rms_norm: rows must be int32 [R]")
    g_rows, g_bias, g_mult = gate if gate is not None else (None, None, 1.0)
    if gate is not None:
        _dev(g_rows, g_bias)
        _check(delta is not None and g_rows.shape == (T, H) and g_rows.dtype == out_dtype and g_bias.shape == (H,) and g_bias.dtype == weight.dtype,
               "add_rms_norm: the gate's rows must be like the addend and its bias like the norm's weight")
    _dev(base, vec, weight2)
    _check(base is None or (base.shape == (T, H) and base.dtype == torch.float32 and base.is_contiguous()),
           "add_rms_norm: the float32 addend must be [T, H]")
    _check(vec is None or (vec.shape == (H,) and vec.dtype == torch.float32 and vec.is_contiguous()), "add_rms_norm: the row vector must be float32 [H]")
    _check(weight2 is None or (weight2.shape == (H,) and weight2.dtype == weight.dtype), "add_rms_norm: the second weight must be like the first")
    n_out = T if rows is None else rows.shape[0]
    out = torch.empty((n_out, H), dtype=out_dtype, device=resid.device)
    out2 = torch.empty_like(out) if weight2 is not None else None
    if n_out:
        hip().call("spy_add_rmsnorm", _ptr(resid), _ptr(delta), _ptr(delta2), _ptr(weight), _code(weight, "norm weight"),
                   ctypes.c_float(eps), _ptr(out), _code(out, "norm output"), _ptr(rows), ctypes.c_int(n_out),
                   ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(groups), _ptr(g_rows), _ptr(g_bias), ctypes.c_float(g_mult),
                   _ptr(base), _ptr(vec), _ptr(weight2), _ptr(out2), _Hip.stream())
    return out if weight2 is None else (out, out2)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm over the last dimension, same dtype out as in.  A two-dimensional ``x`` may be a view into the rows of a
    wider product (its row stride is taken); the result is dense."""
    _dev(weight)
    _check(x.is_cuda and x.device == weight.device and x.dtype in _CODES, "rms_norm: float32 or bfloat16 rows on the weight's device expected")
    n = x.shape[-1]
    _check(weight.shape == (n,), "rms_norm: weight must match the last dimension")
    ldx = n
    if x.dim() == 2 and x.stride(1) == 1 and x.stride(0) >= n:
        ldx = x.stride(0)
    else:
        _check(x.is_contiguous(), "rms_norm: dense input, or rows of a wider product, expected")
    out = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
    rows = x.numel() // n if n else 0
    if rows:
        hip().call("spy_rmsnorm", ctypes.c_void_p(x.data_ptr()), ctypes.c_longlong(ldx), _code(x, "rms_norm input"), _ptr(weight),
                   _code(weight, "norm weight"), ctypes.c_float(eps), _ptr(out), ctypes.c_int64(rows), ctypes.c_int(n), _Hip.stream())
    return out


def scale_cap(x: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """In place over float32 values: x = cap tanh(x scale / cap) (``cap`` 0: x * scale): logits behind their head."""
    _dev(x)
    _check(x.dtype == torch.float32 and x.is_contiguous() and cap >= 0.0, "scale_cap: dense float32 values and a cap >= 0 expected")
    if x.numel() and (scale != 1.0 or cap > 0.0):
        hip().call("spy_scale_cap", _ptr(x), ctypes.c_int64(x.numel()), ctypes.c_float(scale), ctypes.c_float(cap), _Hip.stream())
    return x


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


#: most rows of ordinary [M, K] bfloat16 rows that the decode products take (beyond: inputs in operand order only)
DECODE_ROWS_PLAIN = 64


def linear_few(x: torch.Tensor, w: torch.Tensor, tiled: Optional[torch.Tensor] = None, out_dtype: Optional[torch.dtype] = None,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``linear`` for parts that do not fold norms into their products: up to DECODE_ROWS_PLAIN bfloat16 rows go to the
    decode products (which stream the tiled matrix once and beat the library there: 18.7 against 20.3 us for 6144 x 4096 at
    32 rows, 10.5 against 20.6 for 4096 x 4096), everything else to ``linear``."""
    if tiled is not None and x.dtype == torch.bfloat16 and x.dim() == 2 and 0 < x.shape[0] <= DECODE_ROWS_PLAIN and x.is_contiguous():
        return decode_linear(x, tiled, out_dtype or torch.bfloat16, out)
    return linear(x, w, out_dtype, tiled=tiled, out=out)


def linear_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor, tiled: Optional[torch.Tensor] = None, few_rows: int = 0) -> torch.Tensor:
    """silu(x . Wgate^T) * (x . Wup^T) with ``w_gate_up [2 I, K]`` = [Wgate | Wup] -> [M, I].  For few bfloat16 rows
    (decode) one kernel does both products and the SwiGLU; otherwise it is linear() followed by swiglu().  ``few_rows``:
    most rows that the tiled kernel takes here (0: SKINNY_MAX_ROWS)."""
    _dev(x, w_gate_up)
    _check(x.dim() == 2 and w_gate_up.dim() == 2 and x.shape[1] == w_gate_up.shape[1] and w_gate_up.shape[0] % 2 == 0,
           "linear_swiglu: x [M, K] and w [2 I, K] expected")
    M, K = x.shape
    I = w_gate_up.shape[0] // 2
    if x.dtype == torch.bfloat16 and tiled is not None and 0 < M <= max(SKINNY_MAX_ROWS, few_rows) and I % 16 == 0 and x.is_contiguous():
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


class GatedAddend:
    """A sublayer's result that meets the stream behind a gate: the addend is ``y * mult * sigmoid(gate + bias)``.  The
    norm that sums it into the stream forms it in the same pass (``add_rms_norm(gate=)``); whoever cannot calls ``resolve``."""
    __slots__ = ("y", "gate", "bias", "mult")

    def __init__(self, y, gate, bias, mult):
        self.y, self.gate, self.bias, self.mult = y, gate, bias, mult

    def resolve(self):
        return sigmoid_gate(self.y, self.gate, self.bias, self.mult)


class EntryAddends:
    """What meets the stream where a walk over a run of layers begins: whatever the block before left pending (None, an
    addend, a pair of addends), an earlier state of the stream (``base``, float32 [T, H], or None) and a vector that
    every row gets (``vec``, float32 [H]).  The norm that reads the stream next sums all of it in its kernel's pass."""

    __slots__ = ("pending", "base", "vec")

    def __init__(self, pending, base, vec):
        self.pending, self.base, self.vec = pending, base, vec

    def resolve(self, resid: torch.Tensor) -> None:
        """Sums everything into the stream with plain tensor operations (for a reader that has no kernel for it)."""
        pend = None if isinstance(self.pending, ScaledInput) else self.pending
        for addend in (pend if isinstance(pend, (tuple, list)) else (pend,)):
            if addend is not None:
                resid.add_((addend.resolve() if isinstance(addend, GatedAddend) else addend).float())
        if self.base is not None:
            resid.add_(self.base)
        if self.vec is not None:
            resid.add_(self.vec)


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


def decode_linear(x, tiled: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, out: Optional[torch.Tensor] = None,
                  xielu_pq: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x . w^T for few rows; ``x`` bfloat16 [M, K], OperandRows or a ScaledInput, ``tiled`` from tile_weight; the
    result goes into ``out`` if one is brought.  ``xielu_pq``: two bfloat16 numbers (p, q) on the device; the store
    epilogue then applies the xIELU to the result (up to DECODE_ROWS_PLAIN rows)."""
    N = tiled.shape[0]
    out = _result(out, _rows_of(x), N, out_dtype, tiled.device)
    if xielu_pq is not None:
        _check(xielu_pq.dtype == torch.bfloat16 and xielu_pq.numel() == 2 and _rows_of(x) <= DECODE_ROWS_PLAIN,
               "decode_linear: the activation's two numbers must be bfloat16, and the rows at most %d", DECODE_ROWS_PLAIN)
    _gemm_decode(x, tiled, 0, N, out, None, None, xielu_pq, None)
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
                    for_product: bool = False, softcap: float = 0.0, distance: Optional[torch.Tensor] = None, zero_sink: bool = False):
    """Causal grouped-query attention of the step's query tokens over the paged cache
    (which already holds this step's keys and values, or gets them from ``raw`` in this call).  Query at position p
    reads keys max(0, p - window + 1) .. p.  Scores, softmax and the weighted sum are float32.  ``softcap`` > 0: a
    score is softcap tanh(q . k scale / softcap).  ``distance``: float32 [2, n_q]: head h's (capped) score of a key that lies
    x positions back is lowered by distance[0, h] ln(1 + distance[1, h] x).  ``zero_sink``: the softmax's denominator
    holds one more term, e^0, that has no value: p_j = e^(s_j) / (1 + sum e^(s_j)).
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
    softcap = float(softcap or 0.0)
    _check(softcap >= 0.0 and (raw is None or softcap == 0.0), "paged_attention: the scores' cap must not be negative (and the raw product takes none)")
    _dev(distance)
    _check(distance is None or (distance.dtype == torch.float32 and tuple(distance.shape) == (2, n_q) and distance.is_contiguous()),
           "paged_attention: the distance penalty's numbers must be float32 [2, n_q]")
    _check(raw is None or (distance is None and not zero_sink), "paged_attention: the raw product takes neither a distance penalty nor a sink")
    extras = (_ptr(distance), ctypes.c_int(1 if zero_sink else 0))
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
                 ctypes.c_int(win), ctypes.c_float(softcap))
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
                       ctypes.c_int(operand.tiles if operand is not None else 0), *extras, _Hip.stream())
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
                       ctypes.c_int(0 if pieces is None else pieces.shape[0]), *extras, _Hip.stream())
        return operand if operand is not None else out
    hip().call("spy_attention_generic", _ptr(out), _ptr(q), _code(q, "q"), _ptr(k_cache), _ptr(v_cache),
               ctypes.c_int(page_size), ctypes.c_int(num_pages), _ptr(meta.kv_len), _ptr(meta.block_table),
               ctypes.c_int(meta.max_blocks), _ptr(meta.token_entry), _ptr(meta.positions), ctypes.c_int(S), ctypes.c_int(T),
               ctypes.c_int(n_q), ctypes.c_int(n_kv), ctypes.c_int(d), ctypes.c_float(scale), ctypes.c_int(win), ctypes.c_float(softcap),
               *extras, _Hip.stream())
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
# The stream of layers that norm a sublayer's output, kept layer results, and their activation
def _copy_of(like: torch.Tensor, copy_dtype: Optional[torch.dtype]):
    """The activation-dtype copy that a stream kernel writes beside its float32 result (None where the activations are
    float32 themselves: the result serves)."""
    if copy_dtype is None or copy_dtype == torch.float32:
        return None
    _check(copy_dtype == torch.bfloat16, "a copy of the stream is bfloat16 or float32")
    return torch.empty(like.shape, dtype=copy_dtype, device=like.device)


def pair_embedding(ids: torch.Tensor, table: torch.Tensor, pair: Optional[torch.Tensor], buckets: int, mul_prev: int, mul_cur: int,
                   positions: torch.Tensor, token_entry: torch.Tensor, cu_q: torch.Tensor, slot_ids: torch.Tensor,
                   last_token: Optional[torch.Tensor], copy_dtype: Optional[torch.dtype] = None):
    """out[t] = table[ids[t]] + pair[(prev * mul_prev + ids[t] * mul_cur) mod buckets] in float32, row ``buckets`` of
    ``pair`` for a request's first token; prev is the token before, inside the step or, for an entry's first token, in
    ``last_token[slot]`` (int32 [slots]), where every entry's last token is left afterwards.  Returns (out [T, H]
    float32, copy in ``copy_dtype`` or None)."""
    _dev(ids, table, pair, positions, token_entry, cu_q, slot_ids, last_token)
    _check(ids.dtype == torch.int32 and ids.dim() == 1, "pair_embedding: ids must be int32 [T]")
    _check(table.dim() == 2, "pair_embedding: table must be [V, H]")
    T, (V, H), S = ids.shape[0], table.shape, slot_ids.shape[0]
    for name, arr, n in (("positions", positions, T), ("token_entry", token_entry, T), ("cu_q", cu_q, S + 1), ("slot_ids", slot_ids, S)):
        _check(arr.dtype == torch.int32 and tuple(arr.shape) == (n,), "pair_embedding: %s must be int32 [%d]", name, n)
    if pair is not None:
        _check(pair.dtype == table.dtype and tuple(pair.shape) == (buckets + 1, H) and buckets > 0,
               "pair_embedding: the pair table must be [buckets + 1, H] of the table's dtype")
        _check(last_token is not None and last_token.dtype == torch.int32 and last_token.dim() == 1,
               "pair_embedding: the slots' last tokens must be int32 [slots]")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    copy = _copy_of(out, copy_dtype)
    if T:
        hip().call("spy_pair_embedding", _ptr(out), _ptr(copy), BF16 if copy is not None else F32, _ptr(table), _ptr(pair),
                   _code(table, "embedding table"), _ptr(ids), _ptr(positions), _ptr(token_entry), _ptr(cu_q), _ptr(slot_ids),
                   _ptr(last_token), ctypes.c_int(0 if last_token is None else last_token.shape[0]), ctypes.c_int(S),
                   ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(V), ctypes.c_int(buckets), ctypes.c_longlong(mul_prev),
                   ctypes.c_longlong(mul_cur), _Hip.stream())
    return out, copy


def norm_residual(base: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None,
                  copy_dtype: Optional[torch.dtype] = None, mix=None):
    """out = base + y / sqrt(mean(y^2) + eps) * weight, float32 (``out`` may be ``base``; a new tensor if None).
    Returns (out, copy of out in ``copy_dtype`` or None).

    ``mix`` = (kept [layers, T, H] float32, n, a [n]): ``out`` must be ``kept[n - 1]``; the kernel also forms
    sum_j a[j] * kept[j] over j < n (``depth_mix`` in the same pass) and returns (that sum, its copy) instead."""
    _dev(base, y, weight, out)
    _check(base.dtype == torch.float32 and base.dim() == 2, "norm_residual: the stream must be float32 [T, H]")
    T, H = base.shape
    _check(tuple(y.shape) == (T, H) and weight.shape == (H,), "norm_residual: y [T, H] and weight [H] expected")
    if out is None:
        out = torch.empty_like(base)
    _check(out.dtype == torch.float32 and tuple(out.shape) == (T, H), "norm_residual: out must be float32 [T, H]")
    mixed = kept = a = None
    n = 0
    if mix is not None:
        kept, n, a = mix
        _dev(kept, a)
        _check(kept.dtype == torch.float32 and kept.dim() == 3 and tuple(kept.shape[1:]) == (T, H) and 0 < n <= kept.shape[0]
               and out.data_ptr() == kept[n - 1].data_ptr(), "norm_residual: the result must be the last of the n kept results [layers, T, H]")
        _check(a.shape == (n,) and a.dtype == weight.dtype, "norm_residual: one mix weight per kept result, of the norm weight's dtype")
        mixed = torch.empty_like(base)
    copy = _copy_of(out, copy_dtype)
    if T:
        hip().call("spy_norm_residual", _ptr(out), _ptr(copy), BF16 if copy is not None else F32, _ptr(base), _ptr(y), _code(y, "y"),
                   _ptr(weight), _code(weight, "norm weight"), ctypes.c_float(eps), ctypes.c_int(T), ctypes.c_int(H), _ptr(mixed),
                   _ptr(kept), ctypes.c_longlong(T * H), _ptr(a), ctypes.c_int(n), _Hip.stream())
    return (out if mixed is None else mixed), copy


def depth_mix(kept: torch.Tensor, n: int, a: torch.Tensor, copy_dtype: Optional[torch.dtype] = None):
    """sum over j < n of a[j] * kept[j] for ``kept [layers, T, H]`` float32, added in ascending j.  Returns (float32
    [T, H], copy in ``copy_dtype`` or None)."""
    _dev(kept, a)
    _check(kept.dtype == torch.float32 and kept.dim() == 3 and 0 < n <= kept.shape[0], "depth_mix: kept must be float32 [layers >= n, T, H]")
    _check(a.dim() == 1 and a.shape[0] == n, "depth_mix: one weight per kept layer expected")
    out = torch.empty(kept.shape[1:], dtype=torch.float32, device=kept.device)
    copy = _copy_of(out, copy_dtype)
    if out.numel():
        hip().call("spy_depth_mix", _ptr(out), _ptr(copy), BF16 if copy is not None else F32, _ptr(kept), ctypes.c_longlong(out.numel()),
                   _ptr(a), _code(a, "depth weights"), ctypes.c_int(n), ctypes.c_longlong(out.numel()), _Hip.stream())
    return out, copy


def xielu(x: torch.Tensor, pq: torch.Tensor) -> torch.Tensor:
    """In place: x > 0: softplus(p) x^2 + x/2; x <= 0: (1/2 + softplus(q)) (e^x - 1 - x) + x/2, with pq = (p, q) on the device."""
    _dev(x, pq)
    _check(pq.numel() == 2, "xielu: two numbers (p, q) expected")
    if x.numel():
        hip().call("spy_xielu", _ptr(x), _ptr(x), _code(x, "x"), _ptr(pq), _code(pq, "xielu numbers"), ctypes.c_longlong(x.numel()),
                   _Hip.stream())
    return x


def linear_xielu(x: torch.Tensor, w: torch.Tensor, pq: torch.Tensor, tiled: Optional[torch.Tensor] = None) -> torch.Tensor:
    """xielu(x . w^T)."""
    if (tiled is not None and x.dtype == torch.bfloat16 and pq.dtype == torch.bfloat16 and x.dim() == 2 and 0 < x.shape[0] <= DECODE_ROWS_PLAIN
            and x.is_contiguous()):
        return decode_linear(x, tiled, torch.bfloat16, None, pq)           # the activation in the product's store epilogue
    return xielu(linear_few(x, w, tiled), pq)


# --------------------------------------------------------------------------
def mingru(zxg: torch.Tensor, bz: torch.Tensor, bx: torch.Tensor, state: torch.Tensor, pieces: torch.Tensor, n_pieces: int,
           multi: bool, slot_ids: torch.Tensor) -> torch.Tensor:
    """The minGRU recurrence over the step's tokens.  ``zxg [T, 3 W]`` = the projections [z | x | g] of every token;
    S = (1 - z) S + z c with z = sigmoid(. + bz), c from x + bx; ``state [slots, W]`` float32 is read at an entry's
    start and left at its end.  ``pieces`` int32 [4 n]: entry, first row, end row and the entry's first piece, for
    every piece of tokens (an entry in several pieces is walked by several blocks; ``multi`` says there is one).
    Returns S_t * silu(g_t), [T, W] in the dtype of ``zxg``."""
    _dev(zxg, bz, bx, state, pieces, slot_ids)
    _check(zxg.dim() == 2 and zxg.shape[1] % 3 == 0, "mingru: projections [T, 3 W] expected")
    T, W = zxg.shape[0], zxg.shape[1] // 3
    _check(bz.shape == (W,) and bx.shape == (W,) and bz.dtype == bx.dtype, "mingru: two biases [W] of one dtype expected")
    _check(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == W, "mingru: state must be float32 [slots, W]")
    _check(pieces.dtype == torch.int32 and pieces.shape == (4 * n_pieces,) and slot_ids.dtype == torch.int32,
           "mingru: pieces must be int32 [4 n] and slot_ids int32")
    out = torch.empty((T, W), dtype=zxg.dtype, device=zxg.device)
    if T:
        ab = torch.empty((n_pieces, 2, W), dtype=torch.float32, device=zxg.device) if multi else None
        hip().call("spy_mingru", _ptr(out), _ptr(state), _ptr(ab), _ptr(zxg), _code(zxg, "projections"), _ptr(bz), _ptr(bx),
                   _code(bz, "biases"), _ptr(pieces), ctypes.c_int(n_pieces), ctypes.c_int(1 if multi else 0), _ptr(slot_ids),
                   ctypes.c_int(state.shape[0]), ctypes.c_int(T), ctypes.c_int(W), _Hip.stream())
    return out


# --------------------------------------------------------------------------
def gemm_strided(a: torch.Tensor, a_strides, b: torch.Tensor, b_strides, c: torch.Tensor, c_strides, batch: int, M: int, N: int,
                 K: int) -> torch.Tensor:
    """c[i][m][n] = sum_k a[i][m][k] * b[i][n][k] with element strides (batch, row, inner) for each operand, taken from
    the tensors' first elements; float32 products and sums.  The caller answers for the strides staying inside the
    tensors (checked here against their sizes)."""
    _dev(a, b, c)
    for t, (sb, sr, si), (nr, ni), name in ((a, a_strides, (M, K), "a"), (b, b_strides, (N, K), "b"), (c, c_strides, (M, N), "c")):
        last = (batch - 1) * sb + (nr - 1) * sr + (ni - 1) * si
        _check(min(sb, sr, si) >= 0 and last < t.numel(), "gemm_strided: the strides of %s reach beyond the tensor", name)
    if batch * M * N:
        hip().call("spy_gemm_strided", _ptr(a), _code(a, "a"), *(ctypes.c_longlong(s) for s in a_strides), _ptr(b), _code(b, "b"),
                   *(ctypes.c_longlong(s) for s in b_strides), _ptr(c), _code(c, "c"), *(ctypes.c_longlong(s) for s in c_strides),
                   ctypes.c_int(batch), ctypes.c_int(M), ctypes.c_int(N), ctypes.c_int(K), _Hip.stream())
    return c


def latent_prepare(q: torch.Tensor, dkv: Optional[torch.Tensor], cache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor],
                   w_norm: Optional[torch.Tensor], eps: float, freq: Optional[torch.Tensor], mag: float, dims: int,
                   positions: torch.Tensor, H: int, DN: int, DR: int, R: int, qa_dtype: torch.dtype = torch.float32,
                   interleaved: bool = False) -> torch.Tensor:
    """Queries ``q [T, >= H (DN + DR)]`` (a row may be a view into a wider product: its stride is taken) and, if given,
    ``dkv [T, >= R + DR]``: the latent rmsnorm(dkv[:R]) * w_norm and the rotated dkv[R:] go to ``cache [pages, P, R + DR]``
    at the tokens' slots; returns the absorbed query rows [T, H, R + DR] in ``qa_dtype`` with the rotated part filled in
    (the first R values of a row are for the caller's product with the keys' expansion matrix).  ``interleaved``: pair j of
    the rotated dims is (2 j, 2 j + 1) instead of (j, j + dims / 2)."""
    _check(q.dim() == 2 and q.stride(1) == 1 and q.is_cuda, "latent_prepare: q must be rows on the GPU")
    T = q.shape[0]
    _check(q.shape[1] >= H * (DN + DR), "latent_prepare: q rows hold %d values, %d heads of %d needed", q.shape[1], H, DN + DR)
    _dev(cache, slot_mapping, w_norm, freq, positions)
    _check(positions.dtype == torch.int32 and positions.shape == (T,), "latent_prepare: positions must be int32 [T]")
    _check(dims == 0 or (freq is not None and freq.dtype == torch.float32 and freq.shape == (dims // 2,)),
           "latent_prepare: one float32 frequency per rotated pair expected")
    rows = 0
    if dkv is not None:
        _check(dkv.dim() == 2 and dkv.stride(1) == 1 and dkv.shape == (T, R + DR) and dkv.dtype == q.dtype and dkv.device == q.device,
               "latent_prepare: dkv must be [T, R + DR] like q")
        _check(cache is not None and cache.dtype == q.dtype and cache.dim() == 3 and cache.shape[2] == R + DR,
               "latent_prepare: the cache must be [pages, P, R + DR] of the activation dtype")
        _check(slot_mapping is not None and slot_mapping.dtype == torch.int32 and slot_mapping.shape == (T,) and w_norm is not None
               and w_norm.shape == (R,), "latent_prepare: slot_mapping int32 [T] and a norm weight [R] expected")
        rows = cache.shape[0] * cache.shape[1]
    qa = torch.empty((T, H, R + DR), dtype=qa_dtype, device=q.device)
    if T:
        hip().call("spy_latent_prepare", _ptr(qa), _code(qa, "qa"), ctypes.c_void_p(q.data_ptr()), ctypes.c_int(q.stride(0)),
                   ctypes.c_void_p(0 if dkv is None else dkv.data_ptr()), ctypes.c_int(0 if dkv is None else dkv.stride(0)),
                   _code(q, "q"), _ptr(cache if dkv is not None else None), _ptr(slot_mapping if dkv is not None else None),
                   ctypes.c_longlong(rows), _ptr(w_norm if dkv is not None else None),
                   _code(w_norm, "norm weight") if dkv is not None else F32, ctypes.c_float(eps), _ptr(freq), ctypes.c_float(mag),
                   ctypes.c_int(dims), _ptr(positions), ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(DN), ctypes.c_int(DR),
                   ctypes.c_int(R), ctypes.c_int(1 if interleaved else 0), _Hip.stream())
    return qa


def head_products_ok(x: torch.Tensor, xt: int, xh: int, K: int) -> bool:
    """Whether ``head_products`` takes these operands."""
    return x.dtype == torch.bfloat16 and K % 8 == 0 and 0 < K <= 512 and xt % 8 == 0 and xh % 8 == 0 and x.data_ptr() % 16 == 0


def head_products(x: torch.Tensor, xt: int, xh: int, w: torch.Tensor, out: torch.Tensor, ct: int, ch: int, T: int) -> torch.Tensor:
    """out[t, h, n] = sum_k x[t, h, k] * w[h, n, k] on MFMA: ``w [H, N, K]`` bfloat16 in one piece, ``x`` bfloat16 with
    element strides (xt between tokens, xh between heads, k innermost), ``out`` float32 or bfloat16 with strides (ct, ch).
    Built for few rows (a wave keeps its part of ``w`` in registers and walks the tokens)."""
    _check(x.is_cuda and out.is_cuda and x.device == out.device, "head_products: operands on one GPU expected")
    _dev(w)
    _check(w.dim() == 3 and w.dtype == torch.bfloat16, "head_products: w must be bfloat16 [H, N, K]")
    H, N, K = w.shape
    _check(head_products_ok(x, xt, xh, K), "head_products: x must be bfloat16 in 16-byte pieces, K a multiple of 8 up to 512")
    _check((T - 1) * xt + (H - 1) * xh + K <= x.untyped_storage().nbytes() // 2 - x.storage_offset(), "head_products: x's strides reach beyond it")
    _check((T - 1) * ct + (H - 1) * ch + N <= out.untyped_storage().nbytes() // out.element_size() - out.storage_offset(),
           "head_products: out's strides reach beyond it")
    if T:
        hip().call("spy_head_products", ctypes.c_void_p(out.data_ptr()), _code(out, "out"), ctypes.c_longlong(ct), ctypes.c_longlong(ch),
                   ctypes.c_void_p(x.data_ptr()), ctypes.c_longlong(xt), ctypes.c_longlong(xh), _ptr(w), ctypes.c_int(T), ctypes.c_int(H),
                   ctypes.c_int(N), ctypes.c_int(K), _Hip.stream())
    return out


#: most rows of a step for which the per-head products of the latent attention run on ``head_products``; more rows take
#: the library's batched product
HEAD_PRODUCTS_MAX_ROWS = 128
LATENT_TILE_ROWS = 64       # query rows, (token, head) pairs, of one block of the MFMA latent attention (4 waves)
LATENT_TILE_ROWS_MANY = 128  # the same for steps with rows for every compute unit twice over (8 waves: a staged chunk of keys serves twice the rows)


def latent_tile_rows(total_rows: int) -> int:
    return LATENT_TILE_ROWS_MANY if total_rows >= LATENT_TILE_ROWS_MANY * 512 else LATENT_TILE_ROWS
LATENT_MFMA = True          # False forces the plain kernel for bfloat16 too (tests flip it; nothing else does)


def latent_attention_mfma_ok(dtype, R: int, D: int) -> bool:
    """Whether the MFMA kernel takes latent rows of D values of which R are the values: bfloat16, 16-byte pieces, and
    sums of a row tile that fit a wave's registers."""
    return LATENT_MFMA and dtype == torch.bfloat16 and D % 8 == 0 and R % 8 == 0 and D <= 576 and R <= 512


def latent_key_parts(num_tiles: int, max_keys: int) -> int:
    """Parts into which the MFMA latent attention cuts every tile's keys so that a step of few tiles (single tokens)
    still has blocks for the whole device; a part wants 64 keys at least."""
    return max(1, min(512 // max(1, num_tiles), 16, -(-max_keys // 64)))


def latent_attention(qa: torch.Tensor, cache: torch.Tensor, page_size: int, meta: "AttentionMeta", sink: Optional[torch.Tensor],
                     R: int, scale: float, window: Optional[int], out_dtype: torch.dtype, tiles=None, key_parts: int = 1) -> torch.Tensor:
    """Attention of ``qa [T, H, R + DR]`` (absorbed queries: float32 for the plain kernel, bfloat16 with ``tiles`` for the
    MFMA kernel) over the latent rows ``cache [pages, P, R + DR]``:
    score = qa . row * scale, softmax with exp(sink[h]) added to the denominator, causal with ``window``; the result is
    sum_j p_j row_j[:R], [T, H, R] in ``out_dtype``."""
    _dev(qa, cache, sink, meta.kv_len, meta.block_table, meta.token_entry, meta.positions)
    _check(qa.dim() == 3, "latent_attention: qa must be [T, H, D]")
    T, H, D = qa.shape
    mfma = tiles is not None and out_dtype == torch.bfloat16 and latent_attention_mfma_ok(cache.dtype, R, D)
    _check(qa.dtype == (torch.bfloat16 if mfma else torch.float32), "latent_attention: query rows are bfloat16 for the MFMA kernel, float32 for the plain one")
    _check(T == meta.T and cache.dim() == 3 and cache.shape[1] == page_size and cache.shape[2] == D and 0 < R <= D,
           "latent_attention: cache [pages, P, %d] expected for %d tokens", D, meta.T)
    _check(sink is None or sink.shape == (H,), "latent_attention: one sink per head expected")
    _check(meta.block_table.shape == (meta.S, meta.max_blocks), "latent_attention: block table must be [S, max_blocks]")
    out = torch.empty((T, H, R), dtype=out_dtype, device=qa.device)
    if T and mfma:
        # tiles: (entry [n], first row [n], n, rows of a tile) planned on the host
        tile_entry, tile_row0, n = tiles[:3]
        tile_rows = tiles[3] if len(tiles) > 3 else LATENT_TILE_ROWS
        _dev(tile_entry, tile_row0, meta.cu_q, meta.pos0)
        _check(n > 0 and tile_entry.shape == (n,) and tile_row0.shape == (n,), "latent_attention: the tiles' arrays do not fit their number")
        ws = None
        if key_parts > 1:
            ws = torch.empty((hip().lib.spy_latent_attention_mfma_workspace(ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(R),
                                                                            ctypes.c_int(key_parts)),), dtype=torch.float32, device=qa.device)
        hip().call("spy_latent_attention_mfma", _ptr(out), _ptr(ws), _ptr(qa), _ptr(cache), ctypes.c_int(page_size),
                   ctypes.c_int(cache.shape[0]), _ptr(meta.cu_q), _ptr(meta.pos0), _ptr(meta.kv_len), _ptr(meta.block_table),
                   ctypes.c_int(meta.max_blocks), _ptr(tile_entry), _ptr(tile_row0), ctypes.c_int(n), _ptr(sink),
                   _code(sink, "sink") if sink is not None else F32, ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(R),
                   ctypes.c_int(D - R), ctypes.c_float(scale), ctypes.c_int(int(window or 0)), ctypes.c_int(key_parts), ctypes.c_int(tile_rows),
                   _Hip.stream())
        return out
    if T:
        hip().call("spy_latent_attention", _ptr(out), _code(out, "out"), _ptr(qa), _ptr(cache), _code(cache, "cache"),
                   ctypes.c_int(page_size), ctypes.c_int(cache.shape[0]), _ptr(meta.kv_len), _ptr(meta.block_table),
                   ctypes.c_int(meta.max_blocks), _ptr(meta.token_entry), _ptr(meta.positions), _ptr(sink),
                   _code(sink, "sink") if sink is not None else F32, ctypes.c_int(meta.S), ctypes.c_int(T), ctypes.c_int(H),
                   ctypes.c_int(R), ctypes.c_int(D - R), ctypes.c_float(scale), ctypes.c_int(int(window or 0)), _Hip.stream())
    return out


# --------------------------------------------------------------------------
# Attention layers with projection biases, heads rotated in part by angles formed in the kernel, and an output gate
def _row_view(x: torch.Tensor, what: str) -> int:
    """Rows of a wider product: a 2-D view on the GPU whose values lie side by side; returns the row stride."""
    _check(x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and x.dtype in _CODES, "%s: rows of float32 or bfloat16 on the GPU expected", what)
    return x.stride(0)


def bias_rope_store(x: torch.Tensor, n_q: int, n_kv: int, d: int, bias: Optional[torch.Tensor], freq: Optional[torch.Tensor],
                    rotary_dim: int, positions: torch.Tensor, k_cache, v_cache, page_size: int, slots: Optional[torch.Tensor],
                    mag: float = 1.0, value_norm=None, query_temperature=None) -> torch.Tensor:
    """From rows ``x [T, >= (n_q + 2 n_kv) d]`` = [q heads | k heads | v heads] (a view into a wider product may be
    given): the biases ``bias [(n_q + 2 n_kv) d]`` added, the first ``rotary_dim`` dims of every q and k head rotated
    (pair (j, j + rotary_dim/2), angle float32(position) * freq[j]), q written to the result [T, n_q d], k and v into
    the cache pages at ``slots`` (skipped when None).  ``mag``: factor on cos and sin.  ``value_norm`` = (eps, n): every
    value head is divided by sqrt(mean of its first n values squared + eps) before it is stored.  ``query_temperature`` =
    (coef, every): the query at position p is multiplied by 1 + coef ln(floor((p + 1) / every) + 1), in float32."""
    xs = _row_view(x, "bias_rope_store")
    qt_coef, qt_every = (float(query_temperature[0]), int(query_temperature[1])) if query_temperature is not None else (0.0, 0)
    _check(query_temperature is None or qt_every > 0, "bias_rope_store: the query temperature's step must be positive")
    v_eps, v_n = (float(value_norm[0]), int(value_norm[1])) if value_norm is not None else (0.0, 0)
    _check(0 <= v_n <= d, "bias_rope_store: a value norm over %d of %d values", v_n, d)
    T = x.shape[0]
    _dev(bias, freq, positions, k_cache, v_cache, slots)
    _check(x.shape[1] >= (n_q + 2 * n_kv) * d, "bias_rope_store: rows of %d values hold no %d heads of %d", x.shape[1], n_q + 2 * n_kv, d)
    _check(bias is None or bias.shape == ((n_q + 2 * n_kv) * d,), "bias_rope_store: one bias per projected value expected")
    _check(positions.dtype == torch.int32 and positions.shape == (T,), "bias_rope_store: positions must be int32 [T]")
    _check(rotary_dim == 0 or (freq is not None and freq.dtype == torch.float32 and freq.shape == (rotary_dim // 2,) and rotary_dim % 2 == 0
                               and rotary_dim <= d), "bias_rope_store: one float32 frequency per rotated pair expected")
    num_pages = 0
    if slots is not None:
        _check(slots.dtype == torch.int32 and slots.shape == (T,), "bias_rope_store: slots must be int32 [T]")
        num_pages = k_cache.shape[0]
        _check(k_cache.dtype == x.dtype and v_cache.dtype == x.dtype and tuple(k_cache.shape) == (num_pages, n_kv, page_size, d)
               and tuple(v_cache.shape) == (num_pages, n_kv, d, page_size),
               "bias_rope_store: cache pages must be K [pages, n_kv, page, d] and V [pages, n_kv, d, page] of the activation dtype")
    q = torch.empty((T, n_q * d), dtype=x.dtype, device=x.device)
    if T:
        hip().call("spy_bias_rope_store", ctypes.c_void_p(x.data_ptr()), ctypes.c_longlong(xs), _code(x, "x"), _ptr(q), ctypes.c_int(T),
                   ctypes.c_int(n_q), ctypes.c_int(n_kv), ctypes.c_int(d), _ptr(bias), _code(bias, "bias") if bias is not None else F32,
                   _ptr(freq), ctypes.c_int(rotary_dim), _ptr(positions), _ptr(k_cache if slots is not None else None),
                   _ptr(v_cache if slots is not None else None), ctypes.c_int(page_size), ctypes.c_int(num_pages), _ptr(slots),
                   ctypes.c_float(mag), ctypes.c_float(v_eps), ctypes.c_int(v_n), ctypes.c_float(qt_coef), ctypes.c_int(qt_every), _Hip.stream())
    return q


def sigmoid_gate(y: torch.Tensor, gate: torch.Tensor, bias: Optional[torch.Tensor] = None, mult: float = 1.0, per: int = 1) -> torch.Tensor:
    """In place: y[t, j] *= mult * sigmoid(gate[t, j / per] + bias[j / per]); ``gate`` may be a view into a wider product.
    ``per``: columns of y that share one gate value (a head's size: one number per head)."""
    _dev(y, bias)
    _check(per >= 1 and y.dim() == 2 and y.shape[1] % per == 0, "sigmoid_gate: %d columns per gate value do not divide the rows", per)
    _check(bias is None or bias.shape == (y.shape[1] // per,), "sigmoid_gate: one bias per gate value expected")
    gs = _row_view(gate, "sigmoid_gate")
    _check(y.is_contiguous() and tuple(gate.shape) == (y.shape[0], y.shape[1] // per) and gate.dtype == y.dtype and gate.device == y.device,
           "sigmoid_gate: gate rows like y expected")
    if y.numel():
        hip().call("spy_sigmoid_gate", _ptr(y), ctypes.c_void_p(gate.data_ptr()), ctypes.c_longlong(gs), _code(y, "y"), _ptr(bias),
                   _code(bias, "bias") if bias is not None else F32, ctypes.c_float(mult), ctypes.c_int(y.shape[0]), ctypes.c_int(y.shape[1]),
                   ctypes.c_int(per), _Hip.stream())
    return y


# --------------------------------------------------------------------------
# Recurrent mixers with a matrix state per head
MATRIX_MEMORY_MAX_DIM, MATRIX_MEMORY_MAX_VDIM = 256, 1024
MATRIX_MEMORY_SLICE = 16          # value channels that one wave of the recurrences owns (four lanes a channel)


def mlstm_state_size(H: int, d: int, dv: int) -> int:
    """float32 values of one request's mLSTM state: per head S [d, dv], then n [d] and the running maximum once for every
    slice of value channels (the slices' waves each keep their own copy)."""
    return H * (d * dv + -(-dv // MATRIX_MEMORY_SLICE) * (d + 1))


def _entries(cu_q: torch.Tensor, slot_ids: torch.Tensor, what: str) -> int:
    S = slot_ids.shape[0]
    _check(cu_q.dtype == torch.int32 and cu_q.shape == (S + 1,) and slot_ids.dtype == torch.int32, "%s: cu_q int32 [S + 1] and slot_ids int32 [S] expected", what)
    return S


def mlstm(x: torch.Tensor, q_off: int, k_off: int, v_off: int, g_off: int, gates: torch.Tensor, bi: torch.Tensor, bf: torch.Tensor,
          cap: float, norm_w: torch.Tensor, eps: float, state: torch.Tensor, cu_q: torch.Tensor, slot_ids: torch.Tensor, H: int, d: int,
          dv: int, pieces=None) -> torch.Tensor:
    """The mLSTM recurrence over the step's tokens.  ``x``: rows of the fused projection with q (H heads of d) at column
    ``q_off``, k at ``k_off``, v (H heads of dv) at ``v_off`` and the output gate's rows at ``g_off``; ``gates [T, 2 H]``
    float32: the raw products of the input and forget gates, overwritten with the log gates (their biases ``bi``, ``bf [H]``; both capped by
    cap tanh(. / cap)); ``state [slots, mlstm_state_size(H, d, dv)]`` float32 holds S, n and the running maximum of every
    head, read at an entry's start and left at its end.  ``pieces`` = (int32 [4 n]: entry, first row, end row and the
    entry's first piece for every piece of tokens; n; whether an entry has several): entries in several pieces are walked
    by several waves, whose effects on the state are composed.  Returns [T, H dv]: each head's read-out over its root
    mean square, times ``norm_w``, times sigmoid(gate)."""
    xs = _row_view(x, "mlstm")
    T = x.shape[0]
    _dev(gates, bi, bf, norm_w, state, cu_q, slot_ids)
    S = _entries(cu_q, slot_ids, "mlstm")
    _check(0 < d <= MATRIX_MEMORY_MAX_DIM and 0 < dv <= MATRIX_MEMORY_MAX_VDIM, "mlstm: heads of %d x %d (up to %d x %d)", d, dv,
           MATRIX_MEMORY_MAX_DIM, MATRIX_MEMORY_MAX_VDIM)
    _check(max(q_off, k_off) + H * d <= x.shape[1] and max(v_off, g_off) + H * dv <= x.shape[1] and min(q_off, k_off, v_off, g_off) >= 0,
           "mlstm: the projections' columns reach beyond the rows")
    _check(gates.dtype == torch.float32 and gates.shape == (T, 2 * H), "mlstm: the gates' products must be float32 [T, 2 H]")
    _check(bi.shape == (H,) and bf.shape == (H,) and norm_w.shape == (H * dv,) and bi.dtype == bf.dtype == norm_w.dtype,
           "mlstm: gate biases [H] and a norm weight [H dv] of one dtype expected")
    _check(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == mlstm_state_size(H, d, dv),
           "mlstm: state must be float32 [slots, mlstm_state_size(H, d, dv)]")
    out = torch.empty((T, H * dv), dtype=x.dtype, device=x.device)
    if T:
        tmp = torch.empty((T, H * dv), dtype=torch.float32, device=x.device)        # the read-outs before the heads' norm
        parr, n_pieces, multi, work, abe, mfin = None, 0, False, None, None, None
        if pieces is not None and pieces[2]:
            parr, n_pieces, multi = pieces
            _dev(parr)
            _check(parr.dtype == torch.int32 and parr.shape == (4 * n_pieces,) and n_pieces > 0, "mlstm: pieces must be int32 [4 n]")
            work = torch.empty((n_pieces, state.shape[1]), dtype=torch.float32, device=x.device)
            abe = torch.empty((T, 3 * H), dtype=torch.float32, device=x.device)
            mfin = torch.empty((S, H), dtype=torch.float32, device=x.device)
        hip().call("spy_mlstm", _ptr(out), _ptr(tmp), _ptr(state), ctypes.c_void_p(x.data_ptr()), ctypes.c_longlong(xs), _code(x, "x"), ctypes.c_int(q_off),
                   ctypes.c_int(k_off), ctypes.c_int(v_off), ctypes.c_int(g_off), _ptr(gates), _ptr(bi), _ptr(bf), _code(bi, "gate biases"),
                   ctypes.c_float(cap), _ptr(norm_w), ctypes.c_float(eps), _ptr(cu_q), _ptr(slot_ids), ctypes.c_int(state.shape[0]),
                   ctypes.c_int(S), ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(d), ctypes.c_int(dv), _ptr(parr), ctypes.c_int(n_pieces),
                   ctypes.c_int(1 if multi else 0), _ptr(work), _ptr(abe), _ptr(mfin), _Hip.stream())
    return out


def causal_conv_silu(x: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, keep_off: int, token_entry: torch.Tensor,
                     cu_q: torch.Tensor, slot_ids: torch.Tensor) -> torch.Tensor:
    """y[t, c] = silu(sum_j taps[c, j] x[t - (n - 1) + j, c]) per request (``x [T, C]`` may be a view into a wider
    product); inputs before an entry's first token are the request's kept inputs ``state[slot, keep_off + i C + c]``
    (i = 0 .. n - 2, the newest last; float32), which afterwards hold the entry's last n - 1 inputs."""
    xs = _row_view(x, "causal_conv_silu")
    T, C = x.shape
    _dev(taps, state, token_entry, cu_q, slot_ids)
    S = _entries(cu_q, slot_ids, "causal_conv_silu")
    _check(taps.dim() == 2 and taps.shape[0] == C and 1 <= taps.shape[1] <= 8, "causal_conv_silu: taps [C, 1..8] expected")
    n = taps.shape[1]
    _check(token_entry.dtype == torch.int32 and token_entry.shape == (T,), "causal_conv_silu: token_entry must be int32 [T]")
    _check(state.dtype == torch.float32 and state.dim() == 2 and 0 <= keep_off and keep_off + (n - 1) * C <= state.shape[1],
           "causal_conv_silu: the kept inputs reach beyond the float32 state")
    y = torch.empty((T, C), dtype=x.dtype, device=x.device)
    if T:
        hip().call("spy_causal_conv_silu", _ptr(y), ctypes.c_void_p(x.data_ptr()), ctypes.c_longlong(xs), _code(x, "x"), _ptr(taps),
                   _code(taps, "taps"), ctypes.c_void_p(state.data_ptr() + 4 * keep_off), ctypes.c_longlong(state.shape[1]), _ptr(token_entry),
                   _ptr(cu_q), _ptr(slot_ids), ctypes.c_int(state.shape[0]), ctypes.c_int(S), ctypes.c_int(T), ctypes.c_int(C), ctypes.c_int(n),
                   _Hip.stream())
    return y


def delta_rule(qkv: torch.Tensor, beta_pre: torch.Tensor, dec_pre: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
               gate: torch.Tensor, norm_w: torch.Tensor, eps: float, state: torch.Tensor, cu_q: torch.Tensor, slot_ids: torch.Tensor,
               H: int, G: int, d: int, dv: int, gate_act: str = "sigmoid") -> torch.Tensor:
    """The gated delta rule over the step's tokens.  ``qkv [T, 2 G d + H dv]``: q and k (G heads of d; made unit vectors
    here, q also times d^-1/2) and v (H heads of dv); ``beta_pre [T, H]`` and ``dec_pre [T, H d]`` float32: the raw products
    (overwritten with what they turn into) behind beta = sigmoid(.) and the decay exp(-exp(a_log[h]) softplus(. + dt_bias)) per head and key channel; per head
    S = diag(decay) S, u = beta (v - S^T k), S += k u^T, o = S^T q with ``state[slot, h d dv ..]`` float32.  Returns
    [T, H dv]: o over its root mean square, times ``norm_w [dv]``, times sigmoid(``gate``) (rows of H dv values, a view
    into a wider product allowed; ``gate_act`` "silu": times silu(gate)).  One decay per head instead of one per key
    channel: ``dec_pre [T, H]`` and ``dt_bias [H]``."""
    _dev(qkv, a_log, dt_bias, norm_w, state, cu_q, slot_ids)
    gs = _row_view(gate, "delta_rule")
    bs, zs = _row_view(beta_pre, "delta_rule"), _row_view(dec_pre, "delta_rule")       # (both may be columns of one wider product)
    T = qkv.shape[0]
    S = _entries(cu_q, slot_ids, "delta_rule")
    _check(qkv.dim() == 2 and qkv.shape[1] == 2 * G * d + H * dv and qkv.dtype in _CODES and gate.dtype == qkv.dtype and gate.shape == (T, H * dv),
           "delta_rule: qkv [T, 2 G d + H dv] and gate rows [T, H dv] of one dtype expected")
    _check(H % G == 0 and 0 < d <= MATRIX_MEMORY_MAX_DIM and 0 < dv <= MATRIX_MEMORY_MAX_VDIM, "delta_rule: heads of %d x %d (up to %d x %d)",
           d, dv, MATRIX_MEMORY_MAX_DIM, MATRIX_MEMORY_MAX_VDIM)
    dd = 1 if dec_pre.dim() == 2 and dec_pre.shape[1] == H and dt_bias.shape == (H,) else d        # decays per head: one, or one per key channel
    _check(gate_act in ("sigmoid", "silu"), "delta_rule: the gate's activation is sigmoid or silu")
    _check(beta_pre.dtype == torch.float32 and beta_pre.shape == (T, H) and dec_pre.dtype == torch.float32 and dec_pre.shape == (T, H * dd),
           "delta_rule: the products behind beta [T, H] and the decay [T, H d] (or [T, H]) must be float32")
    _check(a_log.shape == (H,) and dt_bias.shape == (H * dd,) and norm_w.shape == (dv,) and a_log.dtype == dt_bias.dtype == norm_w.dtype,
           "delta_rule: a_log [H], dt_bias [H d] (or [H]) and a norm weight [dv] of one dtype expected")
    _check(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] >= H * d * dv, "delta_rule: state must be float32 [slots, >= H d dv]")
    out = torch.empty((T, H * dv), dtype=qkv.dtype, device=qkv.device)
    if T:
        tmp = torch.empty((T, H * dv), dtype=torch.float32, device=qkv.device)      # the read-outs before the heads' norm
        unit = torch.empty((T, 2 * G * d), dtype=torch.float32, device=qkv.device)  # q and k as unit vectors
        hip().call("spy_delta_rule", _ptr(out), _ptr(tmp), _ptr(unit), _ptr(state), ctypes.c_longlong(state.shape[1]), _ptr(qkv), _code(qkv, "qkv"),
                   ctypes.c_void_p(beta_pre.data_ptr()), ctypes.c_void_p(dec_pre.data_ptr()), _ptr(a_log), _ptr(dt_bias), _code(a_log, "decay numbers"), ctypes.c_void_p(gate.data_ptr()), ctypes.c_longlong(gs),
                   _ptr(norm_w), ctypes.c_float(eps), _ptr(cu_q), _ptr(slot_ids), ctypes.c_int(state.shape[0]), ctypes.c_int(S), ctypes.c_int(T),
                   ctypes.c_int(H), ctypes.c_int(G), ctypes.c_int(d), ctypes.c_int(dv), ctypes.c_int(dd), ctypes.c_int(1 if gate_act == "silu" else 0),
                   ctypes.c_longlong(bs), ctypes.c_longlong(zs), _Hip.stream())
    return out


def token_shift(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, keep_off: int, token_entry: torch.Tensor, cu_q: torch.Tensor,
                slot_ids: torch.Tensor) -> torch.Tensor:
    """out[s, t, c] = x[t, c] + (x'[t, c] - x[t, c]) mu[s, c], x' the row of the token before t in its request: the
    entry's row before, or, for an entry's first token, the request's kept row ``state[slot, keep_off + c]`` (float32;
    zeros for a request's first token), which afterwards holds the entry's last row.  ``mu [n, W]`` -> [n, T, W]."""
    _dev(x, mu, state, token_entry, cu_q, slot_ids)
    _check(x.dim() == 2 and x.dtype in _CODES and mu.dim() == 2 and mu.shape[1] == x.shape[1], "token_shift: rows [T, W] and blends [n, W] expected")
    T, W = x.shape
    S = _entries(cu_q, slot_ids, "token_shift")
    _check(token_entry.dtype == torch.int32 and token_entry.shape == (T,), "token_shift: token_entry must be int32 [T]")
    _check(state.dtype == torch.float32 and state.dim() == 2 and 0 <= keep_off and keep_off + W <= state.shape[1],
           "token_shift: the kept row reaches beyond the float32 state")
    out = torch.empty((mu.shape[0], T, W), dtype=x.dtype, device=x.device)
    if T:
        hip().call("spy_token_shift", _ptr(out), _ptr(x), _code(x, "x"), _ptr(mu), _code(mu, "blends"), ctypes.c_int(mu.shape[0]),
                   ctypes.c_void_p(state.data_ptr() + 4 * keep_off), ctypes.c_longlong(state.shape[1]), _ptr(token_entry), _ptr(cu_q),
                   _ptr(slot_ids), ctypes.c_int(state.shape[0]), ctypes.c_int(S), ctypes.c_int(T), ctypes.c_int(W), _Hip.stream())
    return out


def tanh_cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """tanh of a float32 tensor, rounded once to ``dtype`` (what the next product reads)."""
    _dev(x)
    _check(x.dtype == torch.float32 and dtype in _CODES, "tanh_cast: float32 in, float32 or bfloat16 out")
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    if x.numel():
        hip().call("spy_tanh", _ptr(out), _code(out, "out"), _ptr(x), ctypes.c_longlong(x.numel()), _Hip.stream())
    return out


def time_mix(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, dec_pre: torch.Tensor, w0: torch.Tensor, u: torch.Tensor, gate: torch.Tensor,
             norm_w: torch.Tensor, eps: float, state: torch.Tensor, cu_q: torch.Tensor, slot_ids: torch.Tensor, H: int, d: int) -> torch.Tensor:
    """Per head a state S [d, d] (``state[slot, h d d ..]`` float32, row = key channel): o = (S + diag(u) k v^T)^T r, then
    S = diag(w) S + k v^T with w = exp(-exp(dec_pre + w0)) per key channel.  ``r``, ``k``, ``v``, ``gate [T, H d]``;
    ``dec_pre [T, H d]`` float32 (overwritten with the decays); ``w0``, ``u``, ``norm_w [H d]``.  Returns [T, H d]: each head's
    o over its root mean square, times ``norm_w``, times silu(gate)."""
    _dev(r, k, v, dec_pre, w0, u, gate, norm_w, state, cu_q, slot_ids)
    T, N = r.shape
    S = _entries(cu_q, slot_ids, "time_mix")
    _check(N == H * d and 0 < d <= MATRIX_MEMORY_MAX_DIM, "time_mix: %d heads of %d (up to %d)", H, d, MATRIX_MEMORY_MAX_DIM)
    _check(r.dtype in _CODES and all(t.shape == (T, N) and t.dtype == r.dtype for t in (k, v, gate)), "time_mix: r, k, v and gate [T, H d] of one dtype expected")
    _check(dec_pre.dtype == torch.float32 and dec_pre.shape == (T, N), "time_mix: the decay's products must be float32 [T, H d]")
    _check(all(t.shape == (N,) for t in (w0, u, norm_w)) and w0.dtype == u.dtype == norm_w.dtype, "time_mix: w0, u and a norm weight [H d] of one dtype expected")
    _check(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] >= H * d * d, "time_mix: state must be float32 [slots, >= H d d]")
    out = torch.empty((T, N), dtype=r.dtype, device=r.device)
    if T:
        tmp = torch.empty((T, N), dtype=torch.float32, device=r.device)           # the read-outs before the heads' norm
        bonus = torch.empty((T, H), dtype=torch.float32, device=r.device)         # sum_i r u k per token and head
        hip().call("spy_time_mix", _ptr(out), _ptr(tmp), _ptr(bonus), _ptr(state), ctypes.c_longlong(state.shape[1]), _ptr(r), _ptr(k), _ptr(v),
                   _ptr(gate), _code(r, "r"), _ptr(dec_pre), _ptr(w0), _ptr(u), _ptr(norm_w), _code(w0, "decay numbers"), ctypes.c_float(eps),
                   _ptr(cu_q), _ptr(slot_ids), ctypes.c_int(state.shape[0]), ctypes.c_int(S), ctypes.c_int(T), ctypes.c_int(H), ctypes.c_int(d),
                   _Hip.stream())
    return out


def norm_pair_mean(a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, eps: float) -> torch.Tensor:
    """(a / rms(a) * wa + b / rms(b) * wb) / 2 per row, float32 inside; the result has the rows' dtype."""
    _dev(a, b, wa, wb)
    _check(a.dim() == 2 and a.shape == b.shape and a.dtype == b.dtype and a.dtype in _CODES, "norm_pair_mean: two sets of rows of one shape and dtype expected")
    T, W = a.shape
    _check(wa.shape == (W,) and wb.shape == (W,) and wa.dtype == wb.dtype, "norm_pair_mean: weights [W] of one dtype expected")
    out = torch.empty_like(a)
    if T:
        hip().call("spy_norm_pair_mean", _ptr(out), _ptr(a), _ptr(b), _code(a, "rows"), _ptr(wa), _ptr(wb), _code(wa, "norm weight"),
                   ctypes.c_float(eps), ctypes.c_int(T), ctypes.c_int(W), _Hip.stream())
    return out


# --------------------------------------------------------------------------
# Mixture of experts
def moe_route(z: torch.Tensor, correction: Optional[torch.Tensor], top: int, groups: int, keep: int, scale: float, score: str = "softmax",
              renormalize: bool = True, logit_bias: Optional[torch.Tensor] = None):
    """Router logits ``z [T, E]`` float32 -> (experts int32 [T, top], weights float32 [T, top]): s = softmax(z) (``score``
    "sigmoid": sigmoid of each logit); the choice goes by s + ``correction`` (None: by s) among the experts of the ``keep``
    best of ``groups`` equal groups of neighbours (a group's score: its largest choice score); the weights are the chosen s
    over their sum (+ 1e-20; ``renormalize`` False: as they are), times ``scale``.  ``logit_bias``: float32 [E], added to the
    logits before anything else (softmax scores over their chosen sum are then the softmax over the chosen biased logits)."""
    _dev(z, correction, logit_bias)
    _check(logit_bias is None or (logit_bias.dtype == torch.float32 and logit_bias.shape == (z.shape[1],) and logit_bias.is_contiguous()),
           "moe_route: a float32 bias [E] expected")
    _check(score in ("softmax", "sigmoid"), "moe_route: scores are softmax or sigmoid")
    _check(z.dtype == torch.float32 and z.dim() == 2 and (correction is None or (correction.dtype == torch.float32 and correction.shape == (z.shape[1],))),
           "moe_route: logits float32 [T, E] and a float32 correction [E] expected")
    T, E = z.shape
    _check(0 < groups and E % groups == 0 and 0 < keep <= groups and 0 < top <= keep * (E // groups) and E <= 1024,
           "moe_route: %d choices among %d of %d groups of %d experts" % (top, keep, groups, E))
    ids = torch.empty((T, top), dtype=torch.int32, device=z.device)
    w = torch.empty((T, top), dtype=torch.float32, device=z.device)
    if T:
        hip().call("spy_moe_route", _ptr(ids), _ptr(w), _ptr(z), _ptr(correction), ctypes.c_int(T), ctypes.c_int(E), ctypes.c_int(top),
                   ctypes.c_int(groups), ctypes.c_int(keep), ctypes.c_float(scale), ctypes.c_int(1 if score == "sigmoid" else 0),
                   ctypes.c_int(1 if renormalize else 0), _ptr(logit_bias), _Hip.stream())
    return ids, w


MOE_MFMA = True            # False forces the plain float32 kernel for bfloat16 too (tests flip it; nothing else does)


def moe_experts(x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, w_gate_up: torch.Tensor, w_down: torch.Tensor,
                activation: str = "silu", limit: float = 0.0, weight_input: bool = False, add: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = sum_k weights[t, k] * down_e( silu(gate_e x[t]) * up_e x[t] ), e = ids[t, k]; ``w_gate_up [E, 2 F, K]`` =
    every expert's [gate rows | up rows], ``w_down [E, K, F]``.  The (token, choice) pairs are sorted by expert on the
    device and the experts' products run over the sorted rows; no size here depends on the choice.  ``activation``
    "clamped": g = min(gate, limit), u = clamp(up, -limit, limit), g sigmoid(1.702 g) (u + 1) in place of silu(gate) up.
    ``weight_input``: the weight multiplies the expert's input, out[t] = sum_k expert_e(weights[t, k] x[t]) (the two
    products being linear, it is multiplied into their sums, ahead of the activation).  ``add [T, K]``: added to the result
    in the pass that sums the choices (the result of a layer that every token uses)."""
    _dev(add)
    _check(add is None or (add.shape == x.shape and add.dtype == x.dtype and add.is_contiguous()), "moe_experts: the addend must be like x")
    _check(activation in ("silu", "clamped") and (activation == "silu" or limit > 0.0), "moe_experts: activation silu, or clamped with a positive limit")
    act_kind = 1 if activation == "clamped" else 0
    _dev(x, ids, weights, w_gate_up, w_down)
    T, K = x.shape
    top = ids.shape[1]
    E, F2, _ = w_gate_up.shape
    F = F2 // 2
    _check(x.dim() == 2 and ids.dtype == torch.int32 and ids.shape == (T, top) and weights.dtype == torch.float32 and weights.shape == (T, top),
           "moe_experts: experts int32 [T, top] and weights float32 [T, top] expected")
    _check(w_gate_up.dim() == 3 and w_gate_up.shape == (E, 2 * F, K) and tuple(w_down.shape) == (E, K, F) and w_down.dtype == w_gate_up.dtype,
           "moe_experts: expert matrices [E, 2 F, K] and [E, K, F] of one dtype expected")
    out = torch.empty((T, K), dtype=x.dtype, device=x.device)
    if not T:
        return out
    tm = hip().lib.spy_moe_tile_rows()
    P = T * top
    max_tiles = P // tm + min(E, P)
    dev = x.device
    sorted_pair = torch.empty((max_tiles * tm,), dtype=torch.int32, device=dev)
    pair_row = torch.empty((P,), dtype=torch.int32, device=dev)
    tile_expert = torch.empty((max_tiles,), dtype=torch.int32, device=dev)
    hip().call("spy_moe_align", _ptr(sorted_pair), _ptr(pair_row), _ptr(tile_expert), _ptr(ids), ctypes.c_int(P), ctypes.c_int(E),
               ctypes.c_int(max_tiles), _Hip.stream())
    # bfloat16: the matrix cores, a block taking one row tile of an expert when the experts have few rows (decoding:
    # blocks for the whole device), up to eight when they have many (an expert's matrices are read once per 128 rows)
    per_block = 0 if not MOE_MFMA or x.dtype != torch.bfloat16 or w_gate_up.dtype != torch.bfloat16 else (8 if P >= 16 * E else 1)
    act = torch.empty((max_tiles * tm, F), dtype=x.dtype, device=dev)
    hip().call("spy_moe_gemm", _ptr(act), _code(act, "act"), _ptr(x), _code(x, "x"), _ptr(w_gate_up), _code(w_gate_up, "expert matrices"),
               _ptr(tile_expert), _ptr(sorted_pair), ctypes.c_int(top), ctypes.c_int(1), ctypes.c_int(max_tiles), ctypes.c_int(E), ctypes.c_int(F),
               ctypes.c_int(K), ctypes.c_int(per_block), ctypes.c_int(act_kind), ctypes.c_float(limit), _ptr(weights if weight_input else None), _Hip.stream())
    y = torch.empty((max_tiles * tm, K), dtype=torch.float32, device=dev)
    hip().call("spy_moe_gemm", _ptr(y), F32, _ptr(act), _code(act, "act"), _ptr(w_down), _code(w_down, "expert matrices"), _ptr(tile_expert),
               _ptr(sorted_pair), ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(max_tiles), ctypes.c_int(E), ctypes.c_int(K), ctypes.c_int(F),
               ctypes.c_int(per_block), ctypes.c_int(0), ctypes.c_float(0.0), _ptr(None), _Hip.stream())
    hip().call("spy_moe_combine", _ptr(out), _code(out, "out"), _ptr(y), _ptr(None if weight_input else weights), _ptr(pair_row), ctypes.c_int(T), ctypes.c_int(top),
               ctypes.c_int(K), _ptr(add), _Hip.stream())
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
