"""Python face of the HIP kernels. Every function checks on the host that the
operands' shapes, dtypes, strides and device fit what its kernel assumes, and
only then launches on torch's current stream. There is no CPU or library
fallback: a tensor that is not on the GPU, or a missing library, is an error."""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from .csrc.build import load
from .errors import AlofaError

F32, BF16 = 0, 1
STORE, ADD_TO_RESIDUAL = 0, 1
MAX_HEAD_DIM = 256

_P = ctypes.c_void_p
_I = ctypes.c_int
_L = ctypes.c_int64
_F = ctypes.c_float


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype is torch.float32:
        return F32
    if t.dtype is torch.bfloat16:
        return BF16
    raise AlofaError("unsupported", "kernels take float32 or bfloat16 tensors", f"dtype={t.dtype}")


def _gpu(name: str, t: torch.Tensor, dtype=None, dims: Optional[int] = None) -> torch.Tensor:
    # (the checks in the order that a good operand passes fastest: these run some thousand times a step)
    try:
        if t.is_cuda and (dtype is None or t.dtype is dtype) and (dims is None or t.dim() == dims):
            return t
    except AttributeError:
        pass
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise AlofaError("invalid_argument", "kernel operand must be a GPU tensor", f"operand={name}")
    if dtype is not None and t.dtype is not dtype:
        raise AlofaError("invalid_argument", "kernel operand has the wrong dtype", f"operand={name} has={t.dtype} wants={dtype}")
    raise AlofaError("shape_mismatch", "kernel operand has the wrong rank", f"operand={name} shape={tuple(t.shape)} wants_rank={dims}")


def _rows(name: str, t: torch.Tensor) -> int:
    """Leading dimension of a 2-d tensor whose rows are contiguous."""
    strides = t.stride()
    if len(strides) == 2:
        rows, columns = t.shape
        if strides[1] == 1 or columns <= 1:
            return strides[0] if rows > 1 else max(strides[0], columns)
    raise AlofaError("shape_mismatch", "kernel operand must be 2-d with contiguous rows", f"operand={name} shape={tuple(t.shape)} strides={t.stride()}")


def _contig(name: str, t: torch.Tensor) -> torch.Tensor:
    if not t.is_contiguous():
        raise AlofaError("shape_mismatch", "kernel operand must be contiguous", f"operand={name} shape={tuple(t.shape)} strides={t.stride()}")
    return t


_scoped_stream: Optional[ctypes.c_void_p] = None


def _stream() -> ctypes.c_void_p:
    if _scoped_stream is not None:
        return _scoped_stream
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class stream_scope:
    """Within the scope every kernel goes to the stream that is torch's current
    one at entry; asking torch once per step instead of once per kernel saves
    about three microseconds of host time per launch. Scopes nest (a graph
    capture inside a step opens its own on the capture stream)."""

    def __enter__(self):
        global _scoped_stream
        self._outer = _scoped_stream
        _scoped_stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        return self

    def __exit__(self, *exc):
        global _scoped_stream
        _scoped_stream = self._outer
        return False


_entries: dict = {}      # the library's entry points by name (looked up once: a step makes some two hundred calls)


def _call(fn_name: str, *args) -> None:
    fn = _entries.get(fn_name)
    if fn is None:
        fn = _entries[fn_name] = getattr(load(), fn_name)
    if fn(*args) != 0:
        raise AlofaError("invalid_argument", "kernel refused its arguments", load().alofa_last_error().decode())


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return _P(t.data_ptr() if t is not None else None)


# ----------------------------------------------------------------- embedding

def embed_gather(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, store: Optional[torch.Tensor] = None) -> None:
    """out[t] = table[ids[t]] widened to float32. ``ids`` must already be
    checked against the vocabulary on the host. With ``store`` (int32) an id
    below zero, -(s + 1), stands for the token store[s] that an earlier choice
    left on the device (``argmax`` and ``sample`` with ``store=``); the caller has
    checked such s against the store's length."""
    _gpu("out", out, torch.float32, 2), _gpu("table", table, None, 2), _gpu("ids", ids, torch.int32, 1)
    _contig("out", out), _contig("table", table), _contig("ids", ids)
    T, h = out.shape
    if table.shape[1] != h or ids.shape[0] != T:
        raise AlofaError("shape_mismatch", "embedding width or token count does not fit", f"out={tuple(out.shape)} table={tuple(table.shape)} ids={tuple(ids.shape)}")
    if store is not None:
        _gpu("store", store, torch.int32, 1), _contig("store", store)
    _call("alofa_embed_gather", _ptr(out), _ptr(table), _I(dtype_code(table)), _ptr(ids), _I(T), _I(h), _ptr(store), _I(table.shape[0]), _stream())


# ---------------------------------------------------------------------- norm

def rmsnorm(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, eps: float, exact: bool,
            rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = rmsnorm(x[rows[r]] if rows is given else x[r]) * w."""
    _gpu("out", out, None, 2), _gpu("x", x, torch.float32, 2), _gpu("w", w, torch.float32, 1)
    _contig("out", out), _contig("x", x), _contig("w", w)
    n, h = out.shape
    if x.shape[1] != h or w.shape[0] != h:
        raise AlofaError("shape_mismatch", "norm width does not fit", f"out={tuple(out.shape)} x={tuple(x.shape)} w={tuple(w.shape)}")
    if rows is not None:
        _gpu("rows", rows, torch.int32, 1), _contig("rows", rows)
        if rows.shape[0] != n:
            raise AlofaError("shape_mismatch", "one row index per output row", f"rows={tuple(rows.shape)} out={tuple(out.shape)}")
    elif x.shape[0] != n:
        raise AlofaError("shape_mismatch", "norm row count does not fit", f"out={tuple(out.shape)} x={tuple(x.shape)}")
    if exact and out.dtype is not torch.float32:
        raise AlofaError("invalid_argument", "the exact path is float32 throughout", f"out={out.dtype}")
    _call("alofa_rmsnorm", _ptr(out), _I(dtype_code(out)), _ptr(x), _ptr(w), _ptr(rows), _I(n), _I(h), _F(eps), _I(int(exact)), _stream())


# ------------------------------------------------------------ matrix product

SKINNY_MAX_ROWS = 64
SWIGLU = 2


ROWS_MAX_M, ROWS_MAX_K = 8, 6144      # what the vector-unit kernel for very few rows takes (longer rows: plain products only)
ROWS_MAX_M_PLAIN = 16                 # ... and up to so many rows for plain products of rows up to ROWS_MAX_K


def rows_kernel_takes(M: int, K: int, swiglu: bool = False, normed: bool = False) -> bool:
    """Sizes the vector-unit kernel takes: at most eight rows, K a multiple of 8; K beyond 6,144 only for a plain
    product (bfloat16 rows, store or residual epilogue), which a second kernel loops over; nine to sixteen rows
    only for a plain product with K up to 6,144."""
    if ROWS_MAX_M < M <= ROWS_MAX_M_PLAIN:
        return K % 8 == 0 and K <= ROWS_MAX_K and not (swiglu or normed)
    return 1 <= M <= ROWS_MAX_M and K % 8 == 0 and (K <= ROWS_MAX_K or not (swiglu or normed))
USE_ROWS_KERNEL = os.environ.get("ALOFA_ROWS_KERNEL", "1") != "0"


def few_rows_kernel(M: int, w_rows: int, K: int, swiglu: bool = False, normed: bool = False) -> str:
    """``few_rows_rule``, remembered per shape (every layer of every step asks)."""
    key = (M, w_rows, K, swiglu, normed, USE_ROWS_KERNEL)
    chosen = _few_rows_known.get(key)
    if chosen is None:
        if len(_few_rows_known) > 1 << 16:
            _few_rows_known.clear()
        chosen = _few_rows_known[key] = few_rows_rule(M, w_rows, K, swiglu, normed)
    return chosen


_few_rows_known: dict = {}


def few_rows_rule(M: int, w_rows: int, K: int, swiglu: bool = False, normed: bool = False) -> str:
    """Which bfloat16 product takes ``M`` rows against ``w_rows`` rows of weights
    (gate and up together for the fused feed-forward entry): ``"rows"``, the
    vector-unit kernel for at most eight rows, whose blocks own four or eight
    columns each and read every row of ``a`` (float32 rows that take a norm on
    their way if ``normed``); ``"stream"``, every wave reading its own operands
    straight from memory into matrix-core tiles (M <= 64 only); or ``"tiled"``,
    blocks that share both operands through LDS.

    The vector-unit kernel has the most and the smallest blocks and no hand-over
    between them, which is what a small matrix's time is made of; but it reads the
    rows once per four columns and its arithmetic grows with M. Measured at the
    projection sizes of 0.5B, 7B and 32B models against the streaming kernel
    (w_rows * K in elements): it wins at one and two rows everywhere (0.5B down
    projection 3.6 against 8.3 us, 7B gate/up 47 against 59); at three and four
    rows except with float32 rows against 24 M elements or more (32B QKV: 28.9
    against 26.8) and gate and up of 256 M or more (32B: 129 against 105 for the
    tiled kernel with its wide tiles); at five to eight rows for plain rows up to 32 M (0.5B down 5.2
    against 8.6, 32B output projection 18.3 against 23.2), for float32 rows only up
    to 4 M (0.5B QKV 4.8 against 5.5, 7B QKV 20.5 against 17.1), and never for gate
    and up together (0.5B: 10.8 against 9.9); at nine to sixteen rows for plain rows
    up to 8 M (0.5B down 6.6 against 8.8, 7B output projection 13.4 against 12.0).

    The streaming kernel reads the rows of ``a`` once per 16 or 32 weight rows, so
    its time grows with M; the tiled kernel's hardly does, but it needs more work
    per block to get going. Measured on one MI355X at the projection sizes of
    0.5B, 7B and 32B models, the tiled kernel wins from these weight sizes on
    (w_rows * K, in elements): 64 M at 5..8 rows, 14 M at 9..16 rows (12 M where the rows
    are longer than the vector-unit kernel takes in one go), 8 M at 17..32 rows
    (the gate and up matrices of the 0.5B sizes, 8.7 M: 12.0 against 13.5 us at 32
    rows, 12.2 against 15.0 at 64; its down matrix, 4.4 M: 18.4 against 13.1), 5 M above;
    the sizes between those three models (1.5B, 3B, 14B) were measured later and moved
    the thresholds where the comments below say so;
    and against a matrix as long as a vocabulary (256 column tiles of 128 or more)
    from the first row on."""
    if M > SKINNY_MAX_ROWS:
        return "tiled"
    if not swiglu and (w_rows + 127) // 128 >= 256:
        return "tiled"
    elements = w_rows * K
    if USE_ROWS_KERNEL and rows_kernel_takes(M, K, swiglu, normed):
        # (gate and up with the norm at three and four rows against small matrices: the streaming kernel since its blocks
        # are dealt out evenly over the compute units, 0.5B sizes 7.0 and 7.1 against 7.3 us; at two rows 6.8 against 6.4)
        small_gate_up = swiglu and normed and M >= 3 and elements <= 16 << 20
        # (three and four rows against a large matrix of long rows whose blocks of four columns leave the last round
        # of an MI355X's 256 compute units half empty: 3,584 x 18,944, 896 blocks, 35.4-36.3 us against the tiled
        # kernel's 31.5; with 5,120 x 13,824, 1,280 blocks, five full rounds, it stays ahead: 34.9-35.8 against 37.4)
        blocks = (w_rows + 3) // 4
        ragged_rounds = K > ROWS_MAX_K and elements >= 64 << 20 and M >= 3 and blocks * 10 < -(-blocks // 256) * 256 * 9
        if M <= 2 or (M <= 4 and not small_gate_up and not ragged_rounds and ((swiglu and elements < 256 << 20) or (not swiglu and (not normed or elements < 24 << 20)))):
            return "rows"
        # (five to eight rows of more than ROWS_MAX_K values: its looping form loses, a 1,536 x 8,960 matrix 14.1-14.7 us
        # against 11.5-12.1 for the streaming kernel, 2,048 x 11,008 19.1-19.4 against 15.9-16.5)
        if 4 < M <= 8 and not swiglu and K <= ROWS_MAX_K and elements <= ((4 << 20) if normed else (32 << 20)):
            return "rows"
        if M > 8 and elements <= 8 << 20:
            return "rows"
    if M <= 4:
        if swiglu:
            return "tiled" if elements >= 256 << 20 else "stream"
        return "tiled" if K > ROWS_MAX_K and elements >= 64 << 20 else "stream"
    if M <= 8:
        return "tiled" if elements >= 64 << 20 else "stream"
    if M <= 16:
        # (4,608 x 3,584: 16.0 against 16.9-17.4 us. Long rows against few columns, a down projection: the tiled kernel
        # shares K out over more blocks, 2,048 x 11,008 15.9-16.1 us against 17.7-18.6, 1,536 x 8,960 13.4 against 13.4-14.4)
        return "tiled" if elements >= 14 << 20 or (K > ROWS_MAX_K and elements >= 12 << 20) else "stream"
    if M <= 32:
        return "tiled" if elements >= 8 << 20 else "stream"
    # (2,560 x 2,048 against 48 and 64 rows: 12.5 and 13.3 us against 14.0 and 15.9; 2,048 x 2,048 against 64: the same either way)
    return "tiled" if elements >= 5 << 20 else "stream"


RIDE_ON_SHARES = os.environ.get("ALOFA_RIDE_ON_SHARES", "1") != "0"


def norm_rides_on_shares(M: int, N: int, K: int) -> bool:
    """Whether a product of 17 to 64 rows that adds to the residual stream and has a norm behind it should go to the
    tiled kernel although the streaming kernel alone would be as fast or a little faster: with K long and the columns
    few the tiled kernel shares K out and adds the shares in a second launch, which has whole rows in hand and takes
    the norm with it, and the norm's own launch (some 4.5 us) is saved."""
    return RIDE_ON_SHARES and 16 < M <= SKINNY_MAX_ROWS and K % 64 == 0 and K >= 3072 and N % 4 == 0 and N <= 4608 and few_rows_kernel(M, N, K) == "stream"


def _product_entry(kernel: Optional[str], M: int, w_rows: int, K: int, swiglu: bool = False, normed: bool = False) -> str:
    kernel = kernel or few_rows_kernel(M, w_rows, K, swiglu, normed)
    if kernel == "stream" and M <= SKINNY_MAX_ROWS:
        return "alofa_gemm_skinny"
    if kernel == "rows" and rows_kernel_takes(M, K, swiglu, normed):
        return "alofa_gemm_rows"
    if kernel == "tiled":
        return "alofa_gemm_mfma"
    if kernel == "wide" and not normed and K % 32 == 0:      # (the tiled kernel's form for many rows, whatever the sizes: for tests and measurements)
        return "alofa_gemm_wide"
    raise AlofaError("invalid_argument", "no such product kernel for these rows", f"kernel={kernel} M={M}")


_workspace_ready = False


def _ensure_workspace(device) -> None:
    """Once per process: the library allocates its workspace (partial results that
    blocks hand to one another). It is never moved, so captured graphs keep valid
    pointers. One stream at a time may run the kernels that use it."""
    global _workspace_ready
    if not _workspace_ready:
        _call("alofa_workspace_init")
        _workspace_ready = True


def _mfma_operands(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the bfloat16 MFMA kernels can take these operands: 16-byte loads
    along K need K and the leading dimensions in multiples of 8 and aligned bases."""
    if a.dtype is not torch.bfloat16 or w.dtype is not torch.bfloat16:
        return False
    K = a.shape[1]
    return (K % 8 == 0 and _rows("a", a) % 8 == 0 and _rows("w", w) % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def norm_goes_apart(M: int, N: int, K: int) -> bool:
    """Whether a norm in front of a plain product of at most eight rows should run as a kernel of its own although
    a product could take it along: the vector-unit kernel reads every row once per four columns, float32 rows
    with the norm on it, so against a large matrix the rows' traffic (N / 4 x M x K x 4 bytes) outgrows what the
    norm's own launch costs (some 3 us): from N x M x K of 63 M on the norm kernel and the product of bfloat16
    rows win. Measured: 4,608 x 3,584 against 6 and 8 rows 13.6 and 14.1 us (norm kernel + product) where the
    product with the norm takes 20.5 and 20.9 and the streaming kernel with the norm 15.2 and 15.6; 7,168 x 5,120
    against 2, 3 and 4 rows 17.7, 18.8 and 19.2 against 19.6, 25.8 and 25.9 (streaming 23.0-24.1); smaller
    products are faster with the norm on them (2,560 x 2,048 against 8 rows 7.3 against 8.0)."""
    return (USE_ROWS_KERNEL and M <= ROWS_MAX_M and N * M * K > 63 << 20 and rows_kernel_takes(M, K)
            and few_rows_kernel(M, N, K) == "rows")


NORM_MAX_ROWS, NORM_MAX_COLUMNS = 16, 8192     # what the streaming kernel's norm form takes (one tile of rows; the norm's weights lie in LDS)
FUSE_NORMS = os.environ.get("ALOFA_FUSE_NORMS", "1") != "0"   # 0: every norm runs as a kernel of its own


def can_fuse_norm(M: int, w: torch.Tensor, out_dtype, swiglu: bool = False, kernel: Optional[str] = None) -> bool:
    """Whether the product of ``M`` float32 rows with the bfloat16 matrix ``w`` can take an RMSNorm
    of those rows on its way (``gemm(..., norm=)``, ``gemm_swiglu(..., norm=)``): the vector-unit
    kernel for very few rows does, and the streaming kernel where it does not share K out over
    blocks; whichever is the kernel of choice (or ``kernel``)."""
    N, K = w.shape
    if not FUSE_NORMS:
        return False
    if w.dtype is not torch.bfloat16 or out_dtype is not torch.bfloat16 or K % 8 or w.stride(0) % 8 or w.data_ptr() % 16:
        return False
    if kernel is None and not swiglu and norm_goes_apart(M, N, K):
        return False
    chosen = kernel or few_rows_kernel(M, 2 * N if swiglu else N, K, swiglu, normed=True)
    if chosen == "rows":
        return rows_kernel_takes(M, K, swiglu, True)
    if M > NORM_MAX_ROWS or K > NORM_MAX_COLUMNS or chosen != "stream":
        return False
    if swiglu:
        return True
    _ensure_workspace(w.device)
    return load().alofa_gemm_skinny_splits(_I(BF16), _I(M), _I(N), _I(K), _I(STORE)) == 1


def _norm_operands(a: torch.Tensor, norm: tuple, K: int):
    weight, eps = norm
    _gpu("a", a, torch.float32, 2), _gpu("norm weight", weight, torch.float32, 1), _contig("norm weight", weight)
    if weight.shape[0] != K or _rows("a", a) % 4 or a.data_ptr() % 16 or weight.data_ptr() % 16 or not eps > 0:
        raise AlofaError("shape_mismatch", "the fused norm needs float32 rows, 16-byte aligned, one weight per column and a positive eps",
                         f"a={tuple(a.shape)} weight={tuple(weight.shape)} eps={eps}")
    return _ptr(weight), _F(eps)


def gemm(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
         add_to_out: bool = False, exact: bool = False, kernel: Optional[str] = None, norm: Optional[tuple] = None,
         then_norm: Optional[tuple] = None) -> None:
    """out = a @ w.T (+ bias), or out += a @ w.T when ``add_to_out`` (out is then
    the float32 residual stream). w is [out_features, in_features]. ``kernel``
    names the bfloat16 kernel ("rows", "stream" or "tiled") instead of ``few_rows_kernel``.
    ``norm`` = (weight, eps): ``a`` holds float32 rows that take an RMSNorm on their way
    into the product (only where ``can_fuse_norm`` says so).
    ``then_norm`` = (weight, eps, rows) with ``add_to_out``: afterwards ``rows`` (out's shape, the
    activation dtype) holds the RMSNorm of out's new rows. Where the product's last launch has whole
    rows in hand (the tiled kernel with K shared out and a launch that adds the shares) the norm rides
    on it; everywhere else it is the norm kernel, run here: the values are the same either way."""
    _gpu("out", out, None, 2), _gpu("a", a, None, 2), _gpu("w", w, None, 2)
    M, K = a.shape
    N = w.shape[0]
    then_w = then_rows = None
    then_eps = 0.0
    if then_norm is not None:
        then_w, then_eps, then_rows = then_norm
        if not add_to_out or norm is not None:
            raise AlofaError("invalid_argument", "a norm behind a product goes with a product that adds to the residual stream")
        _gpu("norm weight", then_w, torch.float32, 1), _contig("norm weight", then_w), _gpu("normed rows", then_rows, None, 2), _contig("normed rows", then_rows)
        if then_w.shape[0] != N or tuple(then_rows.shape) != (M, N) or not then_eps > 0:
            raise AlofaError("shape_mismatch", "the norm behind the product does not fit its output", f"weight={tuple(then_w.shape)} rows={tuple(then_rows.shape)} out={tuple(out.shape)}")
    if norm is not None:
        if add_to_out or exact or not can_fuse_norm(M, w, out.dtype, kernel=kernel) or tuple(out.shape) != (M, N) or w.shape[1] != K:
            raise AlofaError("unsupported", "no kernel takes a norm with this product", f"a={tuple(a.shape)} w={tuple(w.shape)} out={out.dtype}")
        if bias is not None:
            _gpu("bias", bias, torch.float32, 1), _contig("bias", bias)
            if bias.shape[0] != N:
                raise AlofaError("shape_mismatch", "bias length does not fit", f"bias={tuple(bias.shape)} N={N}")
        _call(_product_entry(kernel, M, N, K, normed=True), _ptr(out), _I(BF16), _L(_rows("out", out)), _ptr(a), _L(_rows("a", a)), _ptr(w), _ptr(None), _L(_rows("w", w)),
              _ptr(bias), _I(M), _I(N), _I(K), _I(STORE), *_norm_operands(a, norm, K), _stream())
        return
    if w.shape[1] != K or tuple(out.shape) != (M, N):
        raise AlofaError("shape_mismatch", "matrix product shapes do not fit", f"a={tuple(a.shape)} w={tuple(w.shape)} out={tuple(out.shape)}")
    if bias is not None:
        _gpu("bias", bias, torch.float32, 1), _contig("bias", bias)
        if bias.shape[0] != N:
            raise AlofaError("shape_mismatch", "bias length does not fit", f"bias={tuple(bias.shape)} N={N}")
    if add_to_out and out.dtype is not torch.float32:
        raise AlofaError("invalid_argument", "the residual stream is float32", f"out={out.dtype}")
    if add_to_out and bias is not None:
        # no kernel's residual epilogue adds a bias: the same call would otherwise give different results by dtype
        raise AlofaError("unsupported", "a product that adds to the residual stream takes no bias; add the bias in a buffer of its own")
    if not exact and _mfma_operands(a, w):
        _ensure_workspace(a.device)
        if kernel is None and then_rows is not None and then_rows.dtype is torch.bfloat16 and FUSE_NORMS and norm_rides_on_shares(M, N, K):
            kernel = "tiled"
        entry = _product_entry(kernel, M, N, K)
        done = _I(0)
        if entry == "alofa_gemm_mfma":
            ride = then_rows is not None and then_rows.dtype is torch.bfloat16 and FUSE_NORMS
            more = (_ptr(then_w if ride else None), _F(then_eps), _ptr(then_rows if ride else None), _L(N), ctypes.byref(done))
        else:
            more = (_ptr(None), _F(0.0))
        _call(entry, _ptr(out), _I(dtype_code(out)), _L(_rows("out", out)),
              _ptr(a), _L(_rows("a", a)), _ptr(w), _ptr(None), _L(_rows("w", w)), _ptr(bias), _I(M), _I(N), _I(K),
              _I(ADD_TO_RESIDUAL if add_to_out else STORE), *more, _stream())
        if then_rows is not None and not done.value:
            rmsnorm(then_rows, out, then_w, then_eps, False)
        return
    _call("alofa_gemm_simple", _ptr(out), _I(dtype_code(out)), _L(_rows("out", out)), _ptr(a), _I(dtype_code(a)), _L(_rows("a", a)),
          _ptr(w), _I(dtype_code(w)), _L(_rows("w", w)), _ptr(bias), _I(M), _I(N), _I(K),
          _I(ADD_TO_RESIDUAL if add_to_out else STORE), _I(int(exact)), _stream())
    if then_rows is not None:
        rmsnorm(then_rows, out, then_w, then_eps, exact)


def gemm_swiglu(out: torch.Tensor, a: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, exact: bool = False,
                kernel: Optional[str] = None, norm: Optional[tuple] = None) -> None:
    """out = silu(a @ w_gate.T) * (a @ w_up.T). ``kernel`` and ``norm`` as for ``gemm``."""
    _gpu("out", out, None, 2), _gpu("a", a, None, 2), _gpu("w_gate", w_gate, None, 2), _gpu("w_up", w_up, None, 2)
    M, K = a.shape
    N = w_gate.shape[0]
    if tuple(w_gate.shape) != (N, K) or tuple(w_up.shape) != (N, K) or tuple(out.shape) != (M, N):
        raise AlofaError("shape_mismatch", "gate/up product shapes do not fit", f"a={tuple(a.shape)} gate={tuple(w_gate.shape)} up={tuple(w_up.shape)} out={tuple(out.shape)}")
    if w_gate.dtype is not w_up.dtype or _rows("w_gate", w_gate) != _rows("w_up", w_up):
        raise AlofaError("invalid_argument", "gate and up matrices must share dtype and layout")
    if norm is not None:
        if exact or not can_fuse_norm(M, w_gate, out.dtype, swiglu=True, kernel=kernel) or w_up.data_ptr() % 16:
            raise AlofaError("unsupported", "no kernel takes a norm with this product", f"a={tuple(a.shape)} gate={tuple(w_gate.shape)} out={out.dtype}")
        _call(_product_entry(kernel, M, 2 * N, K, True, normed=True), _ptr(out), _I(BF16), _L(_rows("out", out)), _ptr(a), _L(_rows("a", a)), _ptr(w_gate), _ptr(w_up),
              _L(_rows("w_gate", w_gate)), _ptr(None), _I(M), _I(N), _I(K), _I(SWIGLU), *_norm_operands(a, norm, K), _stream())
        return
    if not exact and out.dtype is torch.bfloat16 and _mfma_operands(a, w_gate) and _mfma_operands(a, w_up):
        _ensure_workspace(a.device)
        entry = _product_entry(kernel, M, 2 * N, K, True)
        more = (_ptr(None), _F(0.0)) if entry != "alofa_gemm_mfma" else (_ptr(None), _F(0.0), _ptr(None), _L(0), _ptr(None))
        _call(entry, _ptr(out), _I(BF16), _L(_rows("out", out)), _ptr(a), _L(_rows("a", a)), _ptr(w_gate), _ptr(w_up),
              _L(_rows("w_gate", w_gate)), _ptr(None), _I(M), _I(N), _I(K), _I(SWIGLU), *more, _stream())
        return
    _call("alofa_gemm_swiglu_simple", _ptr(out), _I(dtype_code(out)), _L(_rows("out", out)), _ptr(a), _I(dtype_code(a)), _L(_rows("a", a)),
          _ptr(w_gate), _ptr(w_up), _I(dtype_code(w_gate)), _L(_rows("w_gate", w_gate)), _I(M), _I(N), _I(K), _I(int(exact)), _stream())


def swiglu(out: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, exact: bool = False) -> None:
    for n, t in (("out", out), ("gate", gate), ("up", up)):
        _gpu(n, t), _contig(n, t)
    if out.shape != gate.shape or up.shape != gate.shape or out.dtype is not gate.dtype or up.dtype is not gate.dtype:
        raise AlofaError("shape_mismatch", "swiglu operands must agree in shape and dtype")
    _call("alofa_swiglu", _ptr(out), _ptr(gate), _ptr(up), _I(dtype_code(out)), _L(out.numel()), _I(int(exact)), _stream())


# ----------------------------------------------------- positions + cache write

def check_cache(name: str, cache: torch.Tensor, kv_heads: int, d: int, transposed: bool = False) -> int:
    """A key cache is [blocks, kv_heads, block_size, d]; a value cache is transposed,
    [blocks, kv_heads, d, block_size]. Contiguous. Returns block_size."""
    _gpu(name, cache, None, 4), _contig(name, cache)
    want_d, bs = (cache.shape[2], cache.shape[3]) if transposed else (cache.shape[3], cache.shape[2])
    if cache.shape[1] != kv_heads or want_d != d:
        raise AlofaError("shape_mismatch", "cache does not fit the heads", f"{name}={tuple(cache.shape)} kv_heads={kv_heads} d={d}")
    return bs


_checked_caches: dict = {}      # id(key cache) -> (key cache, value cache, kv_heads, d, block size): what has been checked already


def check_caches(k_cache: torch.Tensor, v_cache: torch.Tensor, kv_heads: int, d: int) -> int:
    """Key cache and (transposed) value cache of one layer; returns block_size. (A layer's caches are the same
    two tensors step after step, and three kernels a layer ask: what has been checked is remembered by object.)"""
    known = _checked_caches.get(id(k_cache))
    if known is not None and known[0] is k_cache and known[1] is v_cache and known[2] == kv_heads and known[3] == d:
        return known[4]
    bs = _check_caches(k_cache, v_cache, kv_heads, d)
    if len(_checked_caches) > 4096:
        _checked_caches.clear()
    _checked_caches[id(k_cache)] = (k_cache, v_cache, kv_heads, d, bs)
    return bs


def _check_caches(k_cache: torch.Tensor, v_cache: torch.Tensor, kv_heads: int, d: int) -> int:
    bs = check_cache("k_cache", k_cache, kv_heads, d)
    if check_cache("v_cache", v_cache, kv_heads, d, transposed=True) != bs or k_cache.shape[0] != v_cache.shape[0] or k_cache.dtype is not v_cache.dtype:
        raise AlofaError("shape_mismatch", "key and value caches must agree in blocks, block size and dtype",
                         f"k_cache={tuple(k_cache.shape)} v_cache={tuple(v_cache.shape)}")
    return bs


def rope_kv_write(qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                  heads: int, kv_heads: int, d: int, slots: Optional[torch.Tensor] = None,
                  k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None) -> None:
    """Rotate the query and key heads of qkv [T, (heads + 2 kv_heads) d] in place
    by each token's position (half-split pairing); when caches are given, write
    the rotated keys and the values to each token's slot. ``cos``/``sin`` are
    float32 [positions, d/2]. Positions and slots are checked by the caller
    against the table and the cache."""
    _gpu("qkv", qkv, None, 2)
    T = qkv.shape[0]
    write = k_cache is not None
    width = (heads + 2 * kv_heads) * d if write else qkv.shape[1]
    if qkv.shape[1] != width or (not write and (heads + kv_heads) * d > width):
        raise AlofaError("shape_mismatch", "qkv width does not fit the heads", f"qkv={tuple(qkv.shape)} heads={heads} kv_heads={kv_heads} d={d}")
    _gpu("cos", cos, torch.float32, 2), _gpu("sin", sin, torch.float32, 2), _contig("cos", cos), _contig("sin", sin)
    if cos.shape != sin.shape or cos.shape[1] != d // 2 or d % 2:
        raise AlofaError("shape_mismatch", "rotary table must be [positions, d/2]", f"cos={tuple(cos.shape)} d={d}")
    _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
    if positions.shape[0] != T:
        raise AlofaError("shape_mismatch", "one position per token", f"positions={tuple(positions.shape)} T={T}")
    bs = 0
    if write:
        bs = check_caches(k_cache, v_cache, kv_heads, d)
        if k_cache.dtype is not qkv.dtype:
            raise AlofaError("shape_mismatch", "the caches must have qkv's dtype")
        _gpu("slots", slots, torch.int64, 1), _contig("slots", slots)
        if slots.shape[0] != T:
            raise AlofaError("shape_mismatch", "one cache slot per token", f"slots={tuple(slots.shape)} T={T}")
    _call("alofa_rope_kv_write", _ptr(qkv), _I(dtype_code(qkv)), _L(_rows("qkv", qkv)), _ptr(cos), _ptr(sin), _ptr(positions),
          _ptr(slots if write else None), _ptr(k_cache), _ptr(v_cache), _I(T), _I(heads), _I(kv_heads), _I(d), _I(bs), _I(int(write)), _stream())


# ----------------------------------------------------------------- attention

DECODE_MAX_Q = 4          # requests with at most this many query tokens use the decode kernel
MIN_FAST_PAGE = 8         # the bfloat16 attention kernels load eight keys of a value channel at once


def decode_waves(d: int) -> int:
    """Waves of a decode attention block; each takes a share of the keys (the kernel's own rule)."""
    return 8 if d < 128 else 4


FORCED_DECODE_PARTS = int(os.environ.get("ALOFA_DECODE_PARTS", "0"))     # for measurements: so many parts whatever the sizes (0: the rule below)


def decode_splits(tokens: int, heads: int, kv_heads: int, d: int, max_context: int) -> int:
    """Parts the keys of a (token, key head) are cut into beyond the waves of a block. A block reads
    its keys at the rate of one compute unit, so while the blocks are far fewer than the compute
    units more of them are faster: none up to two steps of 32 keys a wave; up to four steps four
    parts, which the last block to arrive combines (``decode_hand_over``: up to eight parts), if the chip has room for
    four (batch 32 at 600 keys: 1.26 against 1.30 ms a step); then a part per step of all the waves, at most eight (the merge grows with them), and
    from there on a part per two steps, combined by a second kernel; never more parts than fill
    the chip, and up to eight steps a wave none where the chip has room for two or three only (two
    parts gain at the long end of such a context bound what they lose at its short end). (Measured at 14:2 heads of 64 and 28:4 of 128, batches of 1 to 64, contexts of 200
    to 4,000: at 2,000 keys and batch 8, 9.6 us with eight parts against 17.6 with one; at 1,000
    keys 9.2 with four against 11.9.)"""
    if FORCED_DECODE_PARTS:
        return FORCED_DECODE_PARTS
    key = (tokens, heads, kv_heads, d, max_context, compute_units())
    known = _decode_splits_known.get(key)
    if known is None:
        if len(_decode_splits_known) > 1 << 16:
            _decode_splits_known.clear()
        known = _decode_splits_known[key] = _decode_splits_rule(tokens, heads, kv_heads, d, max_context)
    return known


_decode_splits_known: dict = {}
_hand_over_known: dict = {}


def _decode_splits_rule(tokens: int, heads: int, kv_heads: int, d: int, max_context: int) -> int:
    waves = decode_waves(d)
    step = 32 * waves
    if max_context <= 2 * step:
        return 1
    blocks = tokens * kv_heads * -(-(heads // kv_heads) // 16)
    by_chip = max(1, compute_units() // max(1, blocks))
    if max_context <= 4 * step:
        return 4 if by_chip >= 4 else 1
    if max_context <= 8 * step and by_chip < 4:
        return 1
    by_length = -(-max_context // step)
    if by_length > 8:
        by_length = max(8, -(-max_context // (2 * step)))
    return max(1, min(64, by_length, by_chip))


HAND_OVER_MAX_PARTS = 8    # up to so many parts the last block combines them; a second kernel combines more


def decode_hand_over(tokens: int, heads: int, kv_heads: int, d: int, n_splits: int) -> bool:
    """Whether ``n_splits`` parts of a (token, key head) hand their states over in the library's workspace, where
    the block that arrives last combines them (few parts that fit it); else they go to the caller's scratch and a
    second kernel."""
    if n_splits <= 1 or n_splits > HAND_OVER_MAX_PARTS:
        return False
    key = (tokens, heads, kv_heads, d, n_splits)
    known = _hand_over_known.get(key)
    if known is None:      # (what fits the workspace does not change once it is there)
        _ensure_workspace(None)
        if len(_hand_over_known) > 1 << 16:
            _hand_over_known.clear()
        known = _hand_over_known[key] = bool(load().alofa_attention_decode_can_hand_over(_I(tokens), _I(heads), _I(kv_heads), _I(d), _I(n_splits)))
    return known


def decode_scratch_floats(tokens: int, heads: int, kv_heads: int, d: int, max_context: int, window: Optional[int]) -> int:
    """Floats of scratch the decode kernel needs for these sizes (0: none)."""
    n = decode_splits(tokens, heads, kv_heads, d, min(max_context, window or max_context))
    return tokens * heads * n * (d + 2) if n > 1 and not decode_hand_over(tokens, heads, kv_heads, d, n) else 0


def paged_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, req_of_token: torch.Tensor, positions: torch.Tensor,
                    heads: int, kv_heads: int, d: int, window: Optional[int], scale: float, exact: bool,
                    max_q_len: Optional[int] = None, max_context: Optional[int] = None,
                    scratch: Optional[torch.Tensor] = None) -> None:
    """out[t] = attention of query token t (q [T, >= heads*d] rows, heads packed)
    over the keys lo..positions[t] of its request's pages. ``max_q_len`` (most
    query tokens of one request in this step) and ``max_context`` (longest
    context) only choose the kernel and its launch shape; with them the caller
    passes ``scratch`` (float32, ``decode_scratch_floats`` long) when that is not 0."""
    _gpu("out", out, None, 2), _gpu("q", q, None, 2)
    T = q.shape[0]
    if out.shape[0] != T or out.shape[1] < heads * d or q.shape[1] < heads * d or out.dtype is not q.dtype:
        raise AlofaError("shape_mismatch", "attention rows do not fit", f"out={tuple(out.shape)} q={tuple(q.shape)} heads={heads} d={d}")
    if d % 2 or d > MAX_HEAD_DIM or d <= 0:
        raise AlofaError("unsupported", f"head size must be even and at most {MAX_HEAD_DIM}", f"head_dim={d}")
    bs = check_caches(k_cache, v_cache, kv_heads, d)
    if k_cache.dtype is not q.dtype:
        raise AlofaError("shape_mismatch", "the caches must have q's dtype")
    _gpu("block_table", block_table, torch.int32, 2), _contig("block_table", block_table)
    _gpu("req_of_token", req_of_token, torch.int32, 1), _contig("req_of_token", req_of_token)
    _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
    if req_of_token.shape[0] != T or positions.shape[0] != T:
        raise AlofaError("shape_mismatch", "one request index and one position per token")
    if (not exact and q.dtype is torch.bfloat16 and max_q_len is not None and max_q_len <= DECODE_MAX_Q and d % 16 == 0
            and _rows("q", q) % 8 == 0 and q.data_ptr() % 16 == 0 and bs >= MIN_FAST_PAGE and bs & (bs - 1) == 0):
        attention_decode(out, q, k_cache, v_cache, block_table, req_of_token, positions, heads, kv_heads, d, window, scale,
                         max_context or 1 << 30, scratch)
        return
    _call("alofa_attention_simple", _ptr(out), _L(_rows("out", out)), _ptr(q), _L(_rows("q", q)), _ptr(k_cache), _ptr(v_cache),
          _I(dtype_code(q)), _ptr(block_table), _I(block_table.shape[1]), _ptr(req_of_token), _ptr(positions), _I(T),
          _I(heads), _I(kv_heads), _I(d), _I(bs), _I(int(window or 0)), _F(scale), _I(int(exact)), _stream())


def _attention_operands(out, q, k_cache, v_cache, block_table, heads, kv_heads, d):
    _gpu("out", out, torch.bfloat16, 2), _gpu("q", q, torch.bfloat16, 2)
    T = q.shape[0]
    if out.shape[0] != T or out.shape[1] < heads * d or q.shape[1] < heads * d:
        raise AlofaError("shape_mismatch", "attention rows do not fit", f"out={tuple(out.shape)} q={tuple(q.shape)} heads={heads} d={d}")
    if d % 16 or not 16 <= d <= MAX_HEAD_DIM or kv_heads <= 0 or heads % kv_heads:
        raise AlofaError("unsupported", "head size 16..256 in steps of 16, kv_heads dividing heads", f"head_dim={d} heads={heads} kv_heads={kv_heads}")
    bs = check_caches(k_cache, v_cache, kv_heads, d)
    if k_cache.dtype is not torch.bfloat16:
        raise AlofaError("shape_mismatch", "the caches must be bfloat16")
    if bs < MIN_FAST_PAGE or bs & (bs - 1):
        raise AlofaError("unsupported", f"the bfloat16 attention kernels take pages of a power of two of tokens, at least {MIN_FAST_PAGE}", f"block_size={bs}")
    _gpu("block_table", block_table, torch.int32, 2), _contig("block_table", block_table)
    if _rows("q", q) % 8 or q.data_ptr() % 16 or _rows("out", out) % 4 or out.data_ptr() % 8:
        raise AlofaError("alignment", "attention rows must be 16-byte aligned", f"q_stride={_rows('q', q)} out_stride={_rows('out', out)}")
    return T, bs


def attention_decode(out, q, k_cache, v_cache, block_table, req_of_token, positions, heads, kv_heads, d, window, scale,
                     max_context: int, scratch: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None,
                     rope: Optional[tuple] = None, n_splits: Optional[int] = None, hand_over: Optional[bool] = None) -> None:
    """bfloat16 attention for tokens of requests that bring few tokens: every
    token of the batch, or the tokens ``rows`` (int32 indices into the batch).
    ``req_of_token`` None: every request brings one token and token i is request
    i (the kernel then starts on the block table without waiting for an index).
    With ``rope`` = (cos, sin, slots) the rows of ``q`` are the fused projection's
    [queries | keys | values] of ONE new token per request, not yet rotated: the
    kernel rotates queries and the new key itself, uses the new key and value from
    registers and writes them to the token's cache slot (``can_fuse_rope_into_decode``).
    ``n_splits`` (default ``decode_splits``): blocks that share the keys of a (token, key head);
    ``hand_over`` (default ``decode_hand_over``): the last of them to arrive combines their states,
    else the states go to ``scratch`` and a second kernel combines them."""
    T, bs = _attention_operands(out, q, k_cache, v_cache, block_table, heads, kv_heads, d)
    for n, t in (("req_of_token", req_of_token), ("positions", positions)):
        if t is None and n == "req_of_token":
            continue
        _gpu(n, t, torch.int32, 1), _contig(n, t)
        if t.shape[0] != T:
            raise AlofaError("shape_mismatch", "one request index and one position per token")
    if req_of_token is None and (rows is not None or block_table.shape[0] < T):
        # no request indices: token i is the one token of request i
        raise AlofaError("invalid_argument", "without request indices every request brings one token, in table order",
                         f"tokens={T} table_rows={block_table.shape[0]} rows={'given' if rows is not None else 'none'}")
    n_tok = T
    if rows is not None:
        _gpu("rows", rows, torch.int32, 1), _contig("rows", rows)
        n_tok = rows.shape[0]
    cos = sin = slots = None
    if rope is not None:
        cos, sin, slots = rope
        if not can_fuse_rope_into_decode(d) or q.shape[1] < (heads + 2 * kv_heads) * d:
            raise AlofaError("unsupported", "the rotary decode kernel needs head sizes in steps of 64 and rows of queries, keys and values",
                             f"head_dim={d} q={tuple(q.shape)}")
        _gpu("cos", cos, torch.float32, 2), _gpu("sin", sin, torch.float32, 2), _contig("cos", cos), _contig("sin", sin)
        if cos.shape != sin.shape or cos.shape[1] != d // 2:
            raise AlofaError("shape_mismatch", "rotary table must be [positions, d/2]", f"cos={tuple(cos.shape)} d={d}")
        _gpu("slots", slots, torch.int64, 1), _contig("slots", slots)
        if slots.shape[0] != T:
            raise AlofaError("shape_mismatch", "one cache slot per token", f"slots={tuple(slots.shape)} T={T}")
    if n_splits is None:
        n_splits = decode_splits(n_tok, heads, kv_heads, d, min(max_context, window or max_context))
    if hand_over is None:
        hand_over = decode_hand_over(n_tok, heads, kv_heads, d, n_splits)
    elif hand_over and not (n_splits > 1 and _ensure_workspace(None) is None
                            and load().alofa_attention_decode_can_hand_over(_I(n_tok), _I(heads), _I(kv_heads), _I(d), _I(n_splits))):
        raise AlofaError("out_of_range", "the parts' states do not fit the library's workspace (or there is one part only)", f"tokens={n_tok} heads={heads} d={d} n_splits={n_splits}")
    floats = n_tok * heads * n_splits * (d + 2) if n_splits > 1 and not hand_over else 0
    if floats and (scratch is None or scratch.dtype is not torch.float32 or not scratch.is_cuda or scratch.numel() < floats or not scratch.is_contiguous()):
        raise AlofaError("invalid_argument", "decode attention needs a float32 scratch buffer", f"floats={floats}")
    _call("alofa_attention_decode", _ptr(out), _L(_rows("out", out)), _ptr(scratch if floats else None), _ptr(q), _L(_rows("q", q)),
          _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _I(block_table.shape[1]), _ptr(req_of_token), _ptr(positions), _ptr(rows),
          _I(n_tok), _I(heads), _I(kv_heads), _I(d), _I(bs), _I(int(window or 0)), _F(scale), _I(n_splits),
          _ptr(cos), _ptr(sin), _ptr(slots), _I(int(hand_over)), _stream())


def can_fuse_rope_into_decode(d: int) -> bool:
    """Head sizes for which the decode attention kernel can rotate and write the new token itself."""
    return d % 64 == 0


PREFILL_HEAD_DIMS = (16, 32, 48, 64, 96, 128, 256)


_compute_units: Optional[int] = None


def compute_units() -> int:
    global _compute_units
    if _compute_units is None:
        _compute_units = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    return _compute_units


def prefill_share(heads: int, kv_heads: int, d: int, runs: int) -> int:
    """How many query heads of a group share their key and value tiles in one block of the prefill
    attention kernel when it serves ``runs`` runs of up to 64 rows (the kernel's own rule: six to
    eight heads, when the launch has blocks enough to fill the chip twice): 0 when every head has
    blocks of its own."""
    return int(load().alofa_attention_prefill_share(_I(heads), _I(kv_heads), _I(d), _I(runs), _I(compute_units())))


PREFILL_ROWS_16_ONLY = os.environ.get("ALOFA_PREFILL_ROWS") == "16"   # the prefill kernel's 16-row form everywhere


def prefill_rows(heads: int, kv_heads: int, d: int, share: int, runs: int) -> int:
    """Query rows a wave of the prefill attention kernel owns when it serves ``runs`` runs: 32 where
    ``share`` heads share their tiles, the head size is 32, 64 or 96 and the blocks of 32 rows are
    at least one and a half per compute unit, or where no heads share, the head size is 128 and
    the blocks are at least two per compute unit (the kernel's own rule), else 16."""
    if PREFILL_ROWS_16_ONLY:
        return 16
    return int(load().alofa_attention_prefill_rows(_I(heads), _I(kv_heads), _I(d), _I(share), _I(runs), _I(compute_units())))


def prefill_blocks_per_run(heads: int, kv_heads: int, share: int, rows: int = 16) -> int:
    """Blocks of the prefill attention kernel that serve one run of up to 64 rows: one per query
    head, or, where ``share`` heads of a group share their tiles, per chunk of that many heads
    four blocks of 16 rows or two of 32 (``rows`` from ``prefill_rows``)."""
    if not share:
        return heads
    return kv_heads * -(-(heads // kv_heads) // share) * (64 // rows)


def pair_tiles(runs: list, window: Optional[int] = None, heads: Optional[int] = None) -> list:
    """``runs``: (request index, first row, rows <= 64, position of the first
    row) per run of rows. Returns per block two runs (the second may be empty).
    When there are more blocks (runs x ``heads``, the blocks that serve one run)
    than compute units, the run
    that walks the most key tiles shares a block with the one that walks the
    fewest, and so on, so that blocks carry about the same work; with fewer,
    every run has a block of its own (a portion deep in a long context would
    otherwise leave most of the chip idle)."""
    if heads is not None and len(runs) * heads <= compute_units():
        return [[list(r), [0, 0, 0, 0]] for r in runs]

    def key_tiles(r):
        first = max(0, r[3] - window + 1) if window else 0
        return (r[3] + r[2] - 1) // 64 - first // 64 + 1
    order = sorted(runs, key=key_tiles, reverse=True)
    out, i, j = [], 0, len(order) - 1
    while i <= j:
        out.append([list(order[i]), list(order[j]) if j > i else [0, 0, 0, 0]])
        i, j = i + 1, j - 1
    return out


def attention_prefill(out, q, k_cache, v_cache, block_table, tiles, heads, kv_heads, d, window, scale, share: int = 0,
                      rows: int = 16) -> None:
    """bfloat16 attention for portions of prompts. ``tiles`` is int32 [n, 2, 4]
    from ``pair_tiles``: per block up to two runs of rows, each (request index,
    first row, rows <= 64 or 0 for none, position of the first row). ``share``
    (from ``prefill_share``; the tiles were paired for its count of blocks):
    that many heads of a group are served from one staged tile. ``rows``: query rows a wave owns
    (from ``prefill_rows``; the tiles were paired for it too)."""
    T, bs = _attention_operands(out, q, k_cache, v_cache, block_table, heads, kv_heads, d)
    if d not in PREFILL_HEAD_DIMS:
        raise AlofaError("unsupported", "the prefill attention kernel is not built for this head size", f"head_dim={d} built={PREFILL_HEAD_DIMS}")
    _gpu("tiles", tiles, torch.int32, 3), _contig("tiles", tiles)
    if tuple(tiles.shape[1:]) != (2, 4) or tiles.shape[0] == 0:
        raise AlofaError("shape_mismatch", "tiles must be [n, 2, 4]", f"tiles={tuple(tiles.shape)}")
    _call("alofa_attention_prefill", _ptr(out), _L(_rows("out", out)), _ptr(q), _L(_rows("q", q)), _ptr(k_cache), _ptr(v_cache),
          _ptr(block_table), _I(block_table.shape[1]), _ptr(tiles), _I(tiles.shape[0]), _I(heads), _I(kv_heads), _I(d), _I(bs),
          _I(int(window or 0)), _F(scale), _I(share), _I(rows), _stream())


# ------------------------------------------------------------------ sampling

_argmax_scratch: dict = {}
_argmax_retired: list = []       # outgrown scratch buffers: a captured step may still address them


def _store_operands(store, store_index, n: int):
    if (store is None) != (store_index is None):
        raise AlofaError("invalid_argument", "a token store goes with the index of every row's place in it")
    if store is not None:
        _gpu("store", store, torch.int32, 1), _contig("store", store), _gpu("store_index", store_index, torch.int32, 1), _contig("store_index", store_index)
        if store_index.shape[0] != n:
            raise AlofaError("shape_mismatch", "one place in the store per row", f"store_index={tuple(store_index.shape)} rows={n}")


def argmax(out: torch.Tensor, logits: torch.Tensor, store: Optional[torch.Tensor] = None,
           store_index: Optional[torch.Tensor] = None) -> None:
    """out[r] = first index of the maximum of logits[r] (lowest index on ties); with ``store``
    also store[store_index[r]] = out[r] (indices the caller has checked against the store)."""
    _gpu("out", out, torch.int32, 1), _gpu("logits", logits, torch.float32, 2), _contig("out", out)
    n = logits.shape[0]
    if out.shape[0] != n:
        raise AlofaError("shape_mismatch", "one choice per row")
    _store_operands(store, store_index, n)
    # long rows are searched by 64 blocks each, through a small scratch (values, then indices) that is kept
    scratch = None
    if logits.shape[1] >= 8192:
        key = logits.device
        scratch = _argmax_scratch.get(key)
        if scratch is None or scratch.numel() < 2 * 64 * n:
            if scratch is not None:
                _argmax_retired.append(scratch)
            # (room for twice the rows asked for: batches that grow one by one do not pile up retired buffers)
            scratch = _argmax_scratch[key] = torch.empty(2 * 64 * max(2 * n, 64), dtype=torch.float32, device=logits.device)
    if store is None:
        _call("alofa_argmax", _ptr(out), _ptr(logits), _L(_rows("logits", logits)), _I(n), _I(logits.shape[1]), _ptr(scratch), _stream())
    else:
        _call("alofa_argmax_to_store", _ptr(out), _ptr(logits), _L(_rows("logits", logits)), _I(n), _I(logits.shape[1]), _ptr(scratch),
              _ptr(store), _ptr(store_index), _stream())


def can_gemm_argmax(M: int, w: torch.Tensor) -> bool:
    """Whether ``gemm_argmax`` takes M rows against ``w``: the few-rows form of the tiled product
    against a matrix as long as a vocabulary (bfloat16; what ``few_rows_kernel`` sends there)."""
    return (w.dtype is torch.bfloat16 and w.dim() == 2 and 0 < M <= SKINNY_MAX_ROWS and (w.shape[0] + 127) // 128 >= 256
            and w.shape[1] % 8 == 0 and os.environ.get("ALOFA_FUSE_ARGMAX", "1") != "0")


_gemm_argmax_scratch: dict = {}
_argmax_retired: list = []       # outgrown scratch buffers: a captured step may still address them
_gemm_argmax_retired: list = []


def gemm_argmax(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, store: Optional[torch.Tensor] = None,
                store_index: Optional[torch.Tensor] = None) -> None:
    """out[m] = the first index of the maximum of a[m] @ w.T (lowest index on ties) without the
    products ever being written: the blocks of the vocabulary product leave the best of their
    columns per row, and the argmax's last stage takes the best of those. ``store`` as for ``argmax``."""
    _gpu("out", out, torch.int32, 1), _contig("out", out)
    _gpu("a", a, torch.bfloat16, 2), _gpu("w", w, torch.bfloat16, 2)
    M, K = a.shape
    if not can_gemm_argmax(M, w) or w.shape[1] != K or out.shape[0] != M:
        raise AlofaError("unsupported", "the product with the argmax on it takes at most 64 bfloat16 rows against a long bfloat16 matrix",
                         f"a={tuple(a.shape)} w={tuple(w.shape)} out={tuple(out.shape)}")
    _store_operands(store, store_index, M)
    need = 4 * SKINNY_MAX_ROWS * ((w.shape[0] + 127) // 128)
    scratch = _gemm_argmax_scratch.get(a.device)
    if scratch is None or scratch.numel() < need:      # (kept: a captured step addresses it)
        if scratch is not None:
            _gemm_argmax_retired.append(scratch)
        scratch = _gemm_argmax_scratch[a.device] = torch.empty(need, dtype=torch.float32, device=a.device)
    _call("alofa_gemm_argmax", _ptr(out), _ptr(store), _ptr(store_index), _ptr(scratch), _L(scratch.numel()), _ptr(a), _L(_rows("a", a)),
          _ptr(w), _L(_rows("w", w)), _I(M), _I(w.shape[0]), _I(K), _stream())


def sample(out: torch.Tensor, logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor,
           store: Optional[torch.Tensor] = None, store_index: Optional[torch.Tensor] = None) -> None:
    """out[r] = inverse-CDF draw from softmax(logits[r] / temperature[r]) at uniform[r] in [0, 1); ``store`` as for ``argmax``."""
    _gpu("out", out, torch.int32, 1), _gpu("logits", logits, torch.float32, 2), _contig("out", out)
    _gpu("temperature", temperature, torch.float64, 1), _gpu("uniform", uniform, torch.float64, 1)
    _contig("temperature", temperature), _contig("uniform", uniform)
    n = logits.shape[0]
    if out.shape[0] != n or temperature.shape[0] != n or uniform.shape[0] != n:
        raise AlofaError("shape_mismatch", "one choice, temperature and uniform number per row")
    _store_operands(store, store_index, n)
    _call("alofa_sample", _ptr(out), _ptr(logits), _L(_rows("logits", logits)), _I(n), _I(logits.shape[1]), _ptr(temperature), _ptr(uniform),
          _ptr(store), _ptr(store_index), _stream())
