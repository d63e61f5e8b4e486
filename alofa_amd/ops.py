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
    # (float32 ``out``: the kernels leave their results unrounded there)
    _gpu("out", out, torch.float32 if out.dtype is torch.float32 else torch.bfloat16, 2), _gpu("q", q, torch.bfloat16, 2)
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
    if _rows("q", q) % 8 or q.data_ptr() % 16 or _rows("out", out) % 4 or out.data_ptr() % (16 if out.dtype is torch.float32 else 8):
        raise AlofaError("alignment", "attention rows must be 16-byte aligned", f"q_stride={_rows('q', q)} out_stride={_rows('out', out)}")
    return T, bs


def _value_planes(out, all_value_heads: bool, v_head, kv_heads: int) -> int:
    """How many planes ``out`` has, one per value head (0: rows of one attention result)."""
    if not all_value_heads:
        return 0
    if v_head is not None or out.dtype is not torch.float32 or out.dim() != 3 or out.shape[0] != kv_heads or not out.is_contiguous():
        raise AlofaError("invalid_argument", "all value heads in one launch: float32 [kv_heads, T, heads * d], and no value head named",
                         f"out={tuple(out.shape)} dtype={out.dtype} v_head={v_head} kv_heads={kv_heads}")
    return kv_heads


def attention_decode(out, q, k_cache, v_cache, block_table, req_of_token, positions, heads, kv_heads, d, window, scale,
                     max_context: int, scratch: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None,
                     rope: Optional[tuple] = None, n_splits: Optional[int] = None, hand_over: Optional[bool] = None,
                     v_head: Optional[int] = None, fine_weights: bool = False, all_value_heads: bool = False) -> None:
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
    else the states go to ``scratch`` and a second kernel combines them.
    ``v_head``: every query head's weights meet the values of this one value head (the keys stay its own key head's).
    ``all_value_heads``: one launch serves every value head in turn as ``v_head``; ``out`` is then float32 [kv_heads, T, heads * d], a
    plane per value head, and a scratch buffer is sized with tokens x kv_heads for ``tokens``.
    ``out`` may be float32: the results are then stored unrounded. ``fine_weights``: every softmax weight meets the values as two bfloat16
    numbers, its rounding and what the rounding took away, so that sixteen bits of it count (twice the second product's instructions)."""
    planes = _value_planes(out, all_value_heads, v_head, kv_heads)
    T, bs = _attention_operands(out[0] if planes else out, q, k_cache, v_cache, block_table, heads, kv_heads, d)
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
    served = n_tok      # (the grid's first dimension: tokens, or (token, value head) pairs)
    n_tok *= max(planes, 1)
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
    if v_head is not None and (rope is not None or not 0 <= v_head < kv_heads):
        raise AlofaError("invalid_argument", "a value head of its own: one of the value heads, and not with the rotary variant", f"v_head={v_head} kv_heads={kv_heads}")
    as32 = out.dtype is torch.float32
    _call("alofa_attention_decode_v", _ptr(None if as32 else out), _L(_rows("out", out[0] if planes else out)), _ptr(scratch if floats else None), _ptr(q), _L(_rows("q", q)),
          _ptr(k_cache), _ptr(v_cache), _ptr(block_table), _I(block_table.shape[1]), _ptr(req_of_token), _ptr(positions), _ptr(rows),
          _I(served), _I(heads), _I(kv_heads), _I(d), _I(bs), _I(int(window or 0)), _F(scale), _I(n_splits),
          _ptr(cos), _ptr(sin), _ptr(slots), _I(int(hand_over)), _I(-1 if v_head is None else v_head), _ptr(out if as32 else None), _I(int(fine_weights)),
          _I(planes), _L(out.stride(0) if planes else 0), _stream())


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
                      rows: int = 16, v_head: Optional[int] = None, fine_weights: bool = False, all_value_heads: bool = False) -> None:
    """bfloat16 attention for portions of prompts. ``tiles`` is int32 [n, 2, 4]
    from ``pair_tiles``: per block up to two runs of rows, each (request index,
    first row, rows <= 64 or 0 for none, position of the first row). ``share``
    (from ``prefill_share``; the tiles were paired for its count of blocks):
    that many heads of a group are served from one staged tile. ``rows``: query rows a wave owns
    (from ``prefill_rows``; the tiles were paired for it too). ``v_head``: every query head's weights meet the values of this one
    value head; ``all_value_heads``: one launch serves every value head in turn so, ``out`` float32 [kv_heads, T, heads * d]. ``out`` may be float32: the results are then stored unrounded. ``fine_weights`` (with ``share`` 0 and 16 ``rows``): every softmax
    weight meets the values as two bfloat16 numbers, so that sixteen bits of it count."""
    planes = _value_planes(out, all_value_heads, v_head, kv_heads)
    T, bs = _attention_operands(out[0] if planes else out, q, k_cache, v_cache, block_table, heads, kv_heads, d)
    if d not in PREFILL_HEAD_DIMS:
        raise AlofaError("unsupported", "the prefill attention kernel is not built for this head size", f"head_dim={d} built={PREFILL_HEAD_DIMS}")
    _gpu("tiles", tiles, torch.int32, 3), _contig("tiles", tiles)
    if tuple(tiles.shape[1:]) != (2, 4) or tiles.shape[0] == 0:
        raise AlofaError("shape_mismatch", "tiles must be [n, 2, 4]", f"tiles={tuple(tiles.shape)}")
    if v_head is not None and not 0 <= v_head < kv_heads:
        raise AlofaError("invalid_argument", "a value head of its own: one of the value heads", f"v_head={v_head} kv_heads={kv_heads}")
    as32 = out.dtype is torch.float32
    _call("alofa_attention_prefill_v", _ptr(None if as32 else out), _L(_rows("out", out[0] if planes else out)), _ptr(q), _L(_rows("q", q)), _ptr(k_cache), _ptr(v_cache),
          _ptr(block_table), _I(block_table.shape[1]), _ptr(tiles), _I(tiles.shape[0]), _I(heads), _I(kv_heads), _I(d), _I(bs),
          _I(int(window or 0)), _F(scale), _I(share), _I(rows), _I(-1 if v_head is None else v_head), _ptr(out if as32 else None), _I(int(fine_weights)),
          _I(planes), _L(out.stride(0) if planes else 0), _stream())


# ------------------------------------------------------------------ sampling

_argmax_scratch: dict = {}
_argmax_retired: list = []       # outgrown scratch buffers: a captured step may still address them


def turn_norm_write(qkv: torch.Tensor, positions: torch.Tensor, qk_table: tuple, v_table: Optional[tuple], heads: int, kv_heads: int, d: int, dv: int,
                    eps: float, unit_norm: bool, exact: bool, slots: Optional[torch.Tensor] = None, k_cache: Optional[torch.Tensor] = None,
                    v_cache: Optional[torch.Tensor] = None) -> None:
    """What a step's projections become before attention with turned values. ``qkv`` [T, heads * d + kv_heads * (d + dv)]: query heads, key
    heads, value heads side by side (``kv_heads`` 0: queries only). Queries and keys are turned on their first channels by ``qk_table``
    (cos, sin float32 [n, pairs]: channel i with i + pairs) and, with ``unit_norm``, divided by their root mean square over d; values are
    turned on all channels by ``v_table`` [n, dv / 2]. Queries are left in place; keys go to ``k_cache`` [pages, kv_heads, page, d] and
    values, transposed, to ``v_cache`` [pages, kv_heads, dv, page] at ``slots`` int64 [T]."""
    _gpu("qkv", qkv, None, 2), _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
    T = qkv.shape[0]
    cos, sin = qk_table
    _gpu("cos", cos, torch.float32, 2), _gpu("sin", sin, torch.float32, 2), _contig("cos", cos), _contig("sin", sin)
    half = cos.shape[1]
    if qkv.shape[1] != heads * d + kv_heads * (d + dv) or positions.shape[0] != T or cos.shape != sin.shape or 2 * half > d:
        raise AlofaError("shape_mismatch", "rows, positions or tables do not fit", f"qkv={tuple(qkv.shape)} heads={heads} kv_heads={kv_heads} d={d} dv={dv} table={tuple(cos.shape)}")
    cv = sv = None
    block = 0
    if kv_heads:
        cv, sv = v_table
        _gpu("cos_v", cv, torch.float32, 2), _gpu("sin_v", sv, torch.float32, 2), _contig("cos_v", cv), _contig("sin_v", sv)
        _gpu("slots", slots, torch.int64, 1), _contig("slots", slots), _gpu("k_cache", k_cache, qkv.dtype, 4), _gpu("v_cache", v_cache, qkv.dtype, 4)
        _contig("k_cache", k_cache), _contig("v_cache", v_cache)
        block = k_cache.shape[2]
        if (cv.shape[1] != dv // 2 or cv.shape != sv.shape or cv.shape[0] < cos.shape[0] or slots.shape[0] != T or tuple(k_cache.shape[1:]) != (kv_heads, block, d)
                or tuple(v_cache.shape) != (k_cache.shape[0], kv_heads, dv, block)):
            raise AlofaError("shape_mismatch", "caches, slots or the values' table do not fit", f"k={tuple(k_cache.shape)} v={tuple(v_cache.shape)} table={tuple(cv.shape)} slots={tuple(slots.shape)}")
    _call("alofa_turn_norm_write", _ptr(qkv), _L(_rows("qkv", qkv)), _I(dtype_code(qkv)), _ptr(positions), _ptr(cos), _ptr(sin), _I(half), _ptr(cv), _ptr(sv),
          _ptr(slots), _ptr(k_cache), _ptr(v_cache), _I(block), _I(T), _I(heads), _I(kv_heads), _I(d), _I(dv), _F(eps), _I(int(unit_norm)), _I(int(exact)), _stream())


def talking_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      req_of_token: Optional[torch.Tensor], positions: torch.Tensor, heads: int, kv_heads: int, d: int, dv: int, window: Optional[int],
                      scale: float, talk: Optional[torch.Tensor], v_table: Optional[tuple], gate: Optional[torch.Tensor], exact: bool = False) -> None:
    """out[t, h] = turn_back(sum_j (sum_g talk[h, g] softmax_g(t, j)) v[j, h // group]) * sigmoid(gate[t, h]): softmax per query head g over
    the keys row t may see (its request's, up to its position; the last ``window`` of them), weights mixed over heads by ``talk`` [heads,
    heads] (None: not mixed), values [pages, kv_heads, dv, page] that were turned by their positions (``v_table``: the result is turned back
    by the row's; None: nothing is turned). ``q`` [T, heads * d] and ``out``, ``gate`` [T, heads * dv] rows (row strides allowed)."""
    _gpu("out", out, None, 2), _gpu("q", q, out.dtype, 2), _gpu("k_cache", k_cache, out.dtype, 4), _gpu("v_cache", v_cache, out.dtype, 4)
    _contig("k_cache", k_cache), _contig("v_cache", v_cache), _gpu("block_table", block_table, torch.int32, 2), _contig("block_table", block_table)
    _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
    T, block = q.shape[0], k_cache.shape[2]
    if (tuple(q.shape) != (T, heads * d) or tuple(out.shape) != (T, heads * dv) or tuple(k_cache.shape[1:]) != (kv_heads, block, d)
            or tuple(v_cache.shape) != (k_cache.shape[0], kv_heads, dv, block) or positions.shape[0] != T):
        raise AlofaError("shape_mismatch", "attention operands do not fit", f"out={tuple(out.shape)} q={tuple(q.shape)} k={tuple(k_cache.shape)} v={tuple(v_cache.shape)} heads={heads} kv_heads={kv_heads} d={d} dv={dv}")
    if req_of_token is not None:
        _gpu("req_of_token", req_of_token, torch.int32, 1), _contig("req_of_token", req_of_token)
    elif block_table.shape[0] < T:
        raise AlofaError("shape_mismatch", "without a request per row every row is a request of its own", f"rows={T} tables={block_table.shape[0]}")
    if talk is not None:
        _gpu("talk", talk, torch.float32, 2), _contig("talk", talk)
        if tuple(talk.shape) != (heads, heads):
            raise AlofaError("shape_mismatch", "the heads' mixing matrix is [heads, heads]", f"talk={tuple(talk.shape)}")
    cv = sv = None
    if v_table is not None:
        cv, sv = v_table
        _gpu("cos_v", cv, torch.float32, 2), _gpu("sin_v", sv, torch.float32, 2), _contig("cos_v", cv), _contig("sin_v", sv)
        if cv.shape[1] != dv // 2 or cv.shape != sv.shape:
            raise AlofaError("shape_mismatch", "the values' table does not fit", f"table={tuple(cv.shape)} dv={dv}")
    if gate is not None:
        _gpu("gate", gate, out.dtype, 2)
        if gate.shape != out.shape:
            raise AlofaError("shape_mismatch", "one gate per output", f"gate={tuple(gate.shape)} out={tuple(out.shape)}")
    _call("alofa_talking_attention", _ptr(out), _L(_rows("out", out)), _ptr(q), _L(_rows("q", q)), _ptr(k_cache), _ptr(v_cache), _I(dtype_code(out)),
          _ptr(block_table), _I(block_table.shape[1]), _ptr(req_of_token), _ptr(positions), _I(T), _I(heads), _I(kv_heads), _I(d), _I(dv), _I(block),
          _I(int(window or 0)), _F(scale), _ptr(talk), _ptr(cv), _ptr(sv), _ptr(gate), _L(_rows("gate", gate) if gate is not None else 0), _I(int(exact)), _stream())


def talk_mix(out: torch.Tensor, applied: torch.Tensor, positions: torch.Tensor, heads: int, kv_heads: int, dv: int, talk: Optional[torch.Tensor],
             v_table: Optional[tuple], gate: Optional[torch.Tensor]) -> None:
    """The heads' talk after the fact: ``applied`` float32 [kv_heads, T, heads * dv] holds, per value head c, every query head's unmixed
    softmax weights applied to the values of c; out[t, h] = turn_back(sum_g talk[h, g] applied[h // group, t, g]) * sigmoid(gate[t, h])
    (``talk`` None: head h alone; ``v_table`` None: nothing is turned; ``gate`` None: no gate)."""
    _gpu("out", out, None, 2), _gpu("applied", applied, torch.float32, 3), _contig("applied", applied)
    _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
    T = out.shape[0]
    if tuple(applied.shape) != (kv_heads, T, heads * dv) or out.shape[1] != heads * dv or positions.shape[0] != T or heads % kv_heads or dv % 2:
        raise AlofaError("shape_mismatch", "the applied weights do not fit", f"applied={tuple(applied.shape)} out={tuple(out.shape)} heads={heads} kv_heads={kv_heads} dv={dv}")
    if talk is not None:
        _gpu("talk", talk, torch.float32, 2), _contig("talk", talk)
        if tuple(talk.shape) != (heads, heads):
            raise AlofaError("shape_mismatch", "the heads' mixing matrix is [heads, heads]", f"talk={tuple(talk.shape)}")
    cv = sv = None
    if v_table is not None:
        cv, sv = v_table
        _gpu("cos_v", cv, torch.float32, 2), _gpu("sin_v", sv, torch.float32, 2), _contig("cos_v", cv), _contig("sin_v", sv)
        if cv.shape[1] != dv // 2 or cv.shape != sv.shape:
            raise AlofaError("shape_mismatch", "the values' table does not fit", f"table={tuple(cv.shape)} dv={dv}")
    if gate is not None:
        _gpu("gate", gate, out.dtype, 2)
        if gate.shape != out.shape:
            raise AlofaError("shape_mismatch", "one gate per output", f"gate={tuple(gate.shape)} out={tuple(out.shape)}")
    _call("alofa_talk_mix", _ptr(out), _L(_rows("out", out)), _I(dtype_code(out)), _ptr(applied), _ptr(positions), _I(T), _I(heads), _I(kv_heads), _I(dv),
          _ptr(talk), _ptr(cv), _ptr(sv), _ptr(gate), _L(_rows("gate", gate) if gate is not None else 0), _stream())


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


# ------------------------------------------------- layer norm, head norm, activations, sums over depth and branches

def layernorm(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, exact: bool,
              rows: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> None:
    """out[r] = (x[r'] - mean) / sqrt(var + eps) * w + b (times ``out_scale``), r' = rows[r] if given else r; var is the
    mean of the squared deviations. ``out`` may be ``x`` itself."""
    _gpu("out", out, None, 2), _gpu("x", x, torch.float32, 2), _gpu("w", w, torch.float32, 1), _gpu("b", b, torch.float32, 1)
    _contig("out", out), _contig("x", x), _contig("w", w), _contig("b", b)
    n, h = out.shape
    if x.shape[1] != h or w.shape[0] != h or b.shape[0] != h:
        raise AlofaError("shape_mismatch", "norm width does not fit", f"out={tuple(out.shape)} x={tuple(x.shape)} w={tuple(w.shape)} b={tuple(b.shape)}")
    if rows is not None:
        _gpu("rows", rows, torch.int32, 1), _contig("rows", rows)
        if rows.shape[0] != n:
            raise AlofaError("shape_mismatch", "one row index per output row", f"rows={tuple(rows.shape)} out={tuple(out.shape)}")
        if out.data_ptr() == x.data_ptr():
            raise AlofaError("invalid_argument", "a norm of gathered rows cannot write over its input")
    elif x.shape[0] != n:
        raise AlofaError("shape_mismatch", "norm row count does not fit", f"out={tuple(out.shape)} x={tuple(x.shape)}")
    if exact and out.dtype is not torch.float32:
        raise AlofaError("invalid_argument", "the exact path is float32 throughout", f"out={out.dtype}")
    _call("alofa_layernorm", _ptr(out), _I(dtype_code(out)), _ptr(x), _ptr(w), _ptr(b), _ptr(rows), _I(n), _I(h), _F(eps), _F(out_scale),
          _I(int(exact)), _stream())


def layernorm_add(residual: torch.Tensor, x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, exact: bool = False) -> None:
    """residual[r] += (x[r] - mean) / sqrt(var + eps) * w + b: the norm behind a sub-layer on its way into the stream (all float32)."""
    _gpu("residual", residual, torch.float32, 2), _gpu("x", x, torch.float32, 2), _gpu("w", w, torch.float32, 1), _gpu("b", b, torch.float32, 1)
    _contig("residual", residual), _contig("x", x), _contig("w", w), _contig("b", b)
    n, h = residual.shape
    if tuple(x.shape) != (n, h) or w.shape[0] != h or b.shape[0] != h:
        raise AlofaError("shape_mismatch", "norm width does not fit", f"residual={tuple(residual.shape)} x={tuple(x.shape)} w={tuple(w.shape)} b={tuple(b.shape)}")
    _call("alofa_layernorm_add", _ptr(residual), _ptr(x), _ptr(w), _ptr(b), _I(n), _I(h), _F(eps), _I(int(exact)), _stream())


def layernorm_add_norm(residual: torch.Tensor, x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float, out: torch.Tensor, w2: torch.Tensor,
                       b2: torch.Tensor, eps2: float, exact: bool = False) -> None:
    """``layernorm_add`` and then ``out[r]`` = the layer norm (w2, b2, eps2) of the row as it now stands, in one launch: the norm behind one
    sub-layer and the one in front of the next. ``out`` [n, h] contiguous in the activation dtype."""
    for n_, t in (("residual", residual), ("x", x)):
        _gpu(n_, t, torch.float32, 2), _contig(n_, t)
    for n_, t in (("w", w), ("b", b), ("w2", w2), ("b2", b2)):
        _gpu(n_, t, torch.float32, 1), _contig(n_, t)
    _gpu("out", out, None, 2), _contig("out", out)
    n, h = residual.shape
    if tuple(x.shape) != (n, h) or tuple(out.shape) != (n, h) or any(t.shape[0] != h for t in (w, b, w2, b2)):
        raise AlofaError("shape_mismatch", "norm width does not fit", f"residual={tuple(residual.shape)} x={tuple(x.shape)} out={tuple(out.shape)} w={tuple(w.shape)}")
    if exact and out.dtype is not torch.float32:
        raise AlofaError("invalid_argument", "the exact path is float32")
    _call("alofa_layernorm_add_norm", _ptr(residual), _ptr(x), _ptr(w), _ptr(b), _F(eps), _ptr(out), _I(dtype_code(out)), _ptr(w2), _ptr(b2), _F(eps2),
          _I(n), _I(h), _I(int(exact)), _stream())


def add_row_scaled(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, exact: bool = False) -> None:
    """out[t] += w[t] * x[t]: ``out`` float32 [T, h] contiguous, ``x`` [T, h] rows of any type (row strides allowed), ``w`` float32 [T]."""
    _gpu("out", out, torch.float32, 2), _gpu("x", x, None, 2), _gpu("w", w, torch.float32, 1), _contig("out", out), _contig("w", w)
    if x.shape != out.shape or w.shape[0] != out.shape[0]:
        raise AlofaError("shape_mismatch", "one weight per row; rows of one shape", f"out={tuple(out.shape)} x={tuple(x.shape)} w={tuple(w.shape)}")
    _call("alofa_add_row_scaled", _ptr(out), _ptr(x), _L(_rows("x", x)), _I(dtype_code(x)), _ptr(w), _L(out.shape[0]), _I(out.shape[1]), _I(int(exact)), _stream())


def headnorm_gate(out: torch.Tensor, o: torch.Tensor, gate: torch.Tensor, weight: Optional[torch.Tensor], heads: int, dv: int,
                  eps: float, exact: bool, out_scale: float = 1.0, parts: int = 1, gate_kind: str = "silu", extra: int = 0,
                  floor: Optional[torch.Tensor] = None) -> None:
    """out[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * weight[h, :] * silu(gate[t, h, :]); ``o`` float32
    [T, heads * dv] contiguous, or [P, T, heads * dv] whose first ``parts`` are added first (read-outs that
    ``linear_recurrence`` left in parts); ``gate`` and ``out`` rows of heads * dv in the activation dtype (row strides
    allowed), ``weight`` float32 [heads * dv] or None. ``gate_kind`` "sigmoid": the gate is sigmoid(gate) instead. ``extra``: a head
    of ``o`` holds so many channels more than its dv (o is [.., T, heads * (dv + extra)]); with ``floor`` float32 [T, heads] the first of
    them is a normaliser: the head's values are divided by max(|it|, floor) + 1e-6 before the norm."""
    _gpu("out", out, None, 2), _gpu("o", o, torch.float32), _gpu("gate", gate, out.dtype, 2), _contig("o", o)
    if gate_kind not in ("silu", "sigmoid") or extra < 0 or (floor is not None and extra < 1):
        raise AlofaError("invalid_argument", "the gate is silu or sigmoid; a normaliser needs a channel of its own", f"gate_kind={gate_kind} extra={extra}")
    if floor is not None:
        _gpu("floor", floor, torch.float32, 2), _contig("floor", floor)
        if tuple(floor.shape) != (o.shape[-2], heads):
            raise AlofaError("shape_mismatch", "one floor per row and head", f"floor={tuple(floor.shape)}")
    part_stride = 0
    if o.dim() == 3:
        if not 1 <= parts <= o.shape[0]:
            raise AlofaError("shape_mismatch", "more parts than the read-outs have room for", f"o={tuple(o.shape)} parts={parts}")
        part_stride, o = o.stride(0), o[0]
    elif o.dim() != 2 or parts != 1:
        raise AlofaError("shape_mismatch", "read-outs are [T, heads * dv] or parts of that", f"o={tuple(o.shape)} parts={parts}")
    T = o.shape[0]
    if o.shape[1] != heads * (dv + extra) or tuple(out.shape) != (T, heads * dv) or tuple(gate.shape) != (T, heads * dv):
        raise AlofaError("shape_mismatch", "head norm operands do not fit", f"out={tuple(out.shape)} o={tuple(o.shape)} gate={tuple(gate.shape)} heads={heads} dv={dv}")
    if weight is not None:
        _gpu("weight", weight, torch.float32, 1), _contig("weight", weight)
        if weight.shape[0] != heads * dv:
            raise AlofaError("shape_mismatch", "one weight per head and channel", f"weight={tuple(weight.shape)} heads={heads} dv={dv}")
    if exact and out.dtype is not torch.float32:
        raise AlofaError("invalid_argument", "the exact path is float32 throughout", f"out={out.dtype}")
    _call("alofa_headnorm_gate", _ptr(out), _L(_rows("out", out)), _ptr(o), _ptr(gate), _L(_rows("gate", gate)), _I(dtype_code(out)), _ptr(weight),
          _I(T), _I(heads), _I(dv), _F(eps), _F(out_scale), _I(parts), _L(part_stride), _I(int(exact)),
          _I(int(gate_kind == "sigmoid")), _I(extra), _ptr(floor), _stream())


XIELU, TANH, SILU, GELU_TANH = 0, 1, 2, 3


def activation(out: torch.Tensor, x: torch.Tensor, kind: int, a: float = 0.0, b: float = 0.0, exact: bool = False) -> None:
    """out = act(x) element by element on rows ([T, n], row strides allowed; out may be x). ``XIELU`` with a = softplus(p),
    b = 1/2 + softplus(q): z > 0: a z^2 + z/2, else b (exp(z) - 1 - z) + z/2. ``TANH``. ``SILU``: z sigmoid(z). ``GELU_TANH``:
    z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))."""
    _gpu("out", out, None, 2), _gpu("x", x, out.dtype, 2)
    if out.shape != x.shape or kind not in (XIELU, TANH, SILU, GELU_TANH):
        raise AlofaError("shape_mismatch", "activation operands do not fit", f"out={tuple(out.shape)} x={tuple(x.shape)} kind={kind}")
    if exact and out.dtype is not torch.float32:
        raise AlofaError("invalid_argument", "the exact path is float32 throughout", f"out={out.dtype}")
    _call("alofa_activation", _ptr(out), _L(_rows("out", out)), _ptr(x), _L(_rows("x", x)), _I(dtype_code(out)), _L(x.shape[0]), _I(x.shape[1]),
          _I(kind), _F(a), _F(b), _I(int(exact)), _stream())


def depth_average(x: torch.Tensor, stack: torch.Tensor, weights: Optional[torch.Tensor], n: int, exact: bool = False) -> None:
    """stack[n - 1] = x, then x = sum_{j < n} weights[j] * stack[j] (j ascending); without weights only the copy.
    ``stack`` float32 [levels, *x.shape] contiguous."""
    _gpu("x", x, torch.float32), _gpu("stack", stack, torch.float32), _contig("x", x), _contig("stack", stack)
    if tuple(stack.shape[1:]) != tuple(x.shape) or not 1 <= n <= stack.shape[0]:
        raise AlofaError("shape_mismatch", "the stack of levels does not fit", f"x={tuple(x.shape)} stack={tuple(stack.shape)} n={n}")
    if weights is not None:
        _gpu("weights", weights, torch.float32, 1), _contig("weights", weights)
        if weights.shape[0] != n:
            raise AlofaError("shape_mismatch", "one weight per level", f"weights={tuple(weights.shape)} n={n}")
    _call("alofa_depth_average", _ptr(x), _ptr(stack), _L(x.numel()), _ptr(weights), _I(n), _L(x.numel()), _I(int(exact)), _stream())


def add_scaled(residual: torch.Tensor, x: torch.Tensor, a: float, y: Optional[torch.Tensor] = None, b: float = 0.0, exact: bool = False) -> None:
    """residual += a * x (+ b * y), all float32 of one shape."""
    _gpu("residual", residual, torch.float32), _gpu("x", x, torch.float32), _contig("residual", residual), _contig("x", x)
    if y is not None:
        _gpu("y", y, torch.float32), _contig("y", y)
    if x.shape != residual.shape or (y is not None and y.shape != residual.shape):
        raise AlofaError("shape_mismatch", "the branches must have the residual stream's shape", f"residual={tuple(residual.shape)} x={tuple(x.shape)}")
    _call("alofa_add_scaled", _ptr(residual), _ptr(x), _F(a), _ptr(y), _F(b), _L(residual.numel()), _I(int(exact)), _stream())


def scale_(x: torch.Tensor, s: float) -> None:
    """x *= s (float32, contiguous)."""
    _gpu("x", x, torch.float32), _contig("x", x)
    _call("alofa_scale", _ptr(x), _F(s), _L(x.numel()), _stream())


# ------------------------------------------------------------- state of fixed size per request: rows, convolution, recurrence

class RowsOfRequests:
    """How a step's rows belong to requests, as the kernels of stateful parts read it from the device: ``slots`` int32
    [R] (the state slot of request r of the step), ``offsets`` int32 [R + 1] (request r owns rows offsets[r] ..
    offsets[r+1] - 1) or None when every request brings one row, ``req_of_row`` int32 [T] or None likewise."""

    def __init__(self, slots: torch.Tensor, offsets: Optional[torch.Tensor], req_of_row: Optional[torch.Tensor], requests: int, rows: int, n_slots: int):
        _gpu("slots", slots, torch.int32, 1), _contig("slots", slots)
        if slots.shape[0] != requests or requests > rows:
            raise AlofaError("shape_mismatch", "one state slot per request of the step", f"slots={tuple(slots.shape)} requests={requests} rows={rows}")
        if offsets is None:
            if requests != rows or req_of_row is not None:
                raise AlofaError("shape_mismatch", "without offsets every request brings one row", f"requests={requests} rows={rows}")
        else:
            _gpu("offsets", offsets, torch.int32, 1), _contig("offsets", offsets), _gpu("req_of_row", req_of_row, torch.int32, 1), _contig("req_of_row", req_of_row)
            if offsets.shape[0] != requests + 1 or req_of_row.shape[0] != rows:
                raise AlofaError("shape_mismatch", "offsets hold one more than the requests, and every row names its request",
                                 f"offsets={tuple(offsets.shape)} req_of_row={tuple(req_of_row.shape)} requests={requests} rows={rows}")
        self.slots, self.offsets, self.req_of_row, self.requests, self.rows, self.n_slots = slots, offsets, req_of_row, requests, rows, n_slots

    def fits(self, name: str, state: torch.Tensor) -> None:
        if state.shape[0] < self.n_slots:
            raise AlofaError("shape_mismatch", "the state has fewer slots than the step's requests may name", f"operand={name} state={tuple(state.shape)} slots={self.n_slots}")


CONV_MAX_TAPS = 16


def short_conv(out: torch.Tensor, h: torch.Tensor, w: torch.Tensor, state: torch.Tensor, rows: RowsOfRequests, exact: bool = False) -> None:
    """out[t] = h[t] + sum_j w[:, j] * h[t - taps + 1 + j] per channel, within each request; the rows before a request's
    first row of this step come from ``state`` [slots, taps - 1, width] (h's dtype; the newest last), which is not
    written (``keep_last_rows`` does that afterwards). ``w`` float32 [width, taps]."""
    _gpu("out", out, None, 2), _gpu("h", h, None, 2), _gpu("w", w, torch.float32, 2), _gpu("state", state, h.dtype, 3)
    _contig("out", out), _contig("h", h), _contig("w", w), _contig("state", state)
    T, width = h.shape
    taps = w.shape[1]
    if tuple(out.shape) != (T, width) or w.shape[0] != width or tuple(state.shape[1:]) != (taps - 1, width) or T != rows.rows or not 1 <= taps <= CONV_MAX_TAPS:
        raise AlofaError("shape_mismatch", "convolution operands do not fit", f"out={tuple(out.shape)} h={tuple(h.shape)} w={tuple(w.shape)} state={tuple(state.shape)} rows={rows.rows}")
    rows.fits("state", state)
    if exact and (out.dtype is not torch.float32 or h.dtype is not torch.float32):
        raise AlofaError("invalid_argument", "the exact path is float32 throughout")
    _call("alofa_short_conv", _ptr(out), _I(dtype_code(out)), _ptr(h), _I(dtype_code(h)), _ptr(w), _ptr(state), _ptr(rows.slots), _ptr(rows.offsets),
          _ptr(rows.req_of_row), _I(T), _I(width), _I(taps), _I(int(exact)), _stream())


def norm_conv_step(out: torch.Tensor, x: torch.Tensor, norm_w: torch.Tensor, norm_b: torch.Tensor, eps: float, w: torch.Tensor,
                   state: torch.Tensor, rows: RowsOfRequests, exact: bool = False) -> None:
    """``layernorm``, ``short_conv`` and ``keep_last_rows`` in one launch for a step in which every request brings one row:
    out[r] = n + conv(n), n the layer norm of x[r]; the state (float32 [slots, taps - 1, width]) moves on by n."""
    _gpu("out", out, None, 2), _gpu("x", x, torch.float32, 2), _gpu("w", w, torch.float32, 2), _gpu("state", state, torch.float32, 3)
    _gpu("norm_w", norm_w, torch.float32, 1), _gpu("norm_b", norm_b, torch.float32, 1)
    for n, t in (("out", out), ("x", x), ("w", w), ("state", state), ("norm_w", norm_w), ("norm_b", norm_b)):
        _contig(n, t)
    T, width = x.shape
    taps = w.shape[1]
    if (tuple(out.shape) != (T, width) or w.shape[0] != width or tuple(state.shape[1:]) != (taps - 1, width) or norm_w.shape[0] != width or norm_b.shape[0] != width
            or rows.offsets is not None or rows.rows != T or not 1 <= taps <= CONV_MAX_TAPS):
        raise AlofaError("shape_mismatch", "norm and convolution operands do not fit (one row per request)", f"out={tuple(out.shape)} x={tuple(x.shape)} w={tuple(w.shape)} state={tuple(state.shape)}")
    rows.fits("state", state)
    if exact and out.dtype is not torch.float32:
        raise AlofaError("invalid_argument", "the exact path is float32 throughout", f"out={out.dtype}")
    _call("alofa_norm_conv_step", _ptr(out), _I(dtype_code(out)), _ptr(x), _ptr(norm_w), _ptr(norm_b), _F(eps), _ptr(w), _ptr(state), _ptr(rows.slots),
          _I(T), _I(width), _I(taps), _I(int(exact)), _stream())


def keep_last_rows(state: torch.Tensor, h: torch.Tensor, rows: RowsOfRequests) -> None:
    """state[slot] [keep, width] = the last ``keep`` rows its request has seen once this step's rows ``h`` are in (older
    ones from the state itself where the step brought fewer)."""
    _gpu("state", state, h.dtype, 3), _gpu("h", h, None, 2), _contig("state", state), _contig("h", h)
    if state.shape[2] != h.shape[1] or h.shape[0] != rows.rows or state.shape[1] > CONV_MAX_TAPS - 1:
        raise AlofaError("shape_mismatch", "the kept rows do not fit", f"state={tuple(state.shape)} h={tuple(h.shape)} rows={rows.rows}")
    rows.fits("state", state)
    _call("alofa_keep_last_rows", _ptr(state), _ptr(h), _I(dtype_code(h)), _ptr(rows.slots), _ptr(rows.offsets), _I(rows.requests), _I(h.shape[1]),
          _I(state.shape[1]), _stream())


def shift_mix(out: torch.Tensor, x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, rows: RowsOfRequests, keep: bool = False) -> None:
    """out[s, t] = x[t] + (x[t - 1] - x[t]) * mu[s], the row before a request's first row of this step taken from
    ``state`` [slots, 1, width] (x's dtype). ``mu`` float32 [n, width]; out [n, T, width] in x's dtype. The state is not
    written (``keep_last_rows`` does that), unless ``keep`` is set in a step of single rows: then it moves on in the same launch."""
    _gpu("out", out, x.dtype, 3), _gpu("x", x, None, 2), _gpu("mu", mu, torch.float32, 2), _gpu("state", state, x.dtype, 3)
    _contig("out", out), _contig("x", x), _contig("mu", mu), _contig("state", state)
    T, width = x.shape
    if tuple(out.shape) != (mu.shape[0], T, width) or mu.shape[1] != width or tuple(state.shape[1:]) != (1, width) or T != rows.rows:
        raise AlofaError("shape_mismatch", "token mix operands do not fit", f"out={tuple(out.shape)} x={tuple(x.shape)} mu={tuple(mu.shape)} state={tuple(state.shape)}")
    rows.fits("state", state)
    if keep and rows.offsets is not None:
        raise AlofaError("invalid_argument", "the token mix keeps its state itself only in steps of single rows")
    _call("alofa_shift_mix", _ptr(out), _ptr(x), _I(dtype_code(x)), _ptr(mu), _ptr(state), _ptr(rows.slots), _ptr(rows.offsets), _ptr(rows.req_of_row),
          _I(T), _I(width), _I(mu.shape[0]), _I(int(keep)), _stream())


DECAY_PER_HEAD, DECAY_SIGMOID_ROOT, DECAY_EXP_NEG_EXP, DECAY_GIVEN = 0, 1, 2, 3
RECURRENCE_MAX_KEYS = 512


def recurrence_max_parts(dk: int) -> int:
    """In how many parts ``linear_recurrence`` may leave its read-outs when it is given room for them (``out`` [P, T, heads * dv])."""
    return int(load().alofa_linear_recurrence_max_parts(_I(dk)))


def linear_recurrence(out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, rows: RowsOfRequests,
                      heads: int, dk: int, dv: int, decay_kind: int, decay: torch.Tensor, tau: float = 1.0, bonus: Optional[torch.Tensor] = None,
                      q_scale: float = 1.0, k_scale: float = 1.0, before_update: bool = False) -> int:
    """Per request (in its rows' order) and head: S = diag(w_t) S + k_t v_t^T and out_t = S^T q_t, or with
    ``before_update`` out_t = (S + diag(bonus) k_t v_t^T)^T q_t first and the update after it. S float32
    [slots, heads, dk, dv] is read and left in ``state``. q, k [T, heads * dk] and v [T, heads * dv] are rows in one
    dtype (row strides allowed); ``out`` float32 [T, heads * dv], or [P, T, heads * dv]: then a step of many rows may deal a
    head's key channels out over blocks, each of which leaves its part of the read-outs; the number of parts used is returned
    (1 otherwise), and ``headnorm_gate(parts=)`` adds them. The decay w_t: ``DECAY_PER_HEAD`` with ``decay``
    float32 [heads]; ``DECAY_SIGMOID_ROOT`` sigmoid(z)^(1/tau) or ``DECAY_EXP_NEG_EXP`` exp(-exp(z)) with ``decay`` = z
    float32 [T, heads * dk] rows, which a step of many rows overwrites with the decays made of them; ``DECAY_GIVEN``:
    ``decay`` holds the w_t themselves."""
    _gpu("out", out, torch.float32), _contig("out", out), _gpu("q", q, None, 2), _gpu("k", k, q.dtype, 2), _gpu("v", v, q.dtype, 2)
    _gpu("state", state, torch.float32, 4), _contig("state", state)
    T = q.shape[0]
    max_parts, part_stride = 1, 0
    if out.dim() == 3:
        max_parts, part_stride, out = out.shape[0], out.stride(0), out[0]
    if (tuple(q.shape) != (T, heads * dk) or tuple(k.shape) != (T, heads * dk) or tuple(v.shape) != (T, heads * dv) or tuple(out.shape) != (T, heads * dv)
            or tuple(state.shape[1:]) != (heads, dk, dv) or T != rows.rows or not 0 < dk <= RECURRENCE_MAX_KEYS):
        raise AlofaError("shape_mismatch", "recurrence operands do not fit", f"q={tuple(q.shape)} k={tuple(k.shape)} v={tuple(v.shape)} out={tuple(out.shape)} "
                         f"state={tuple(state.shape)} heads={heads} dk={dk} dv={dv} rows={rows.rows}")
    rows.fits("state", state)
    per_head = decay_kind == DECAY_PER_HEAD
    _gpu("decay", decay, torch.float32, 1 if per_head else 2)
    if per_head:
        _contig("decay", decay)
    if (tuple(decay.shape) != (heads,)) if per_head else (tuple(decay.shape) != (T, heads * dk)) or decay_kind not in (DECAY_PER_HEAD, DECAY_SIGMOID_ROOT, DECAY_EXP_NEG_EXP, DECAY_GIVEN):
        raise AlofaError("shape_mismatch", "the decay does not fit its kind", f"decay={tuple(decay.shape)} kind={decay_kind} heads={heads} dk={dk}")
    if bonus is not None:
        _gpu("bonus", bonus, torch.float32, 2), _contig("bonus", bonus)
        if tuple(bonus.shape) != (heads, dk) or not before_update:
            raise AlofaError("shape_mismatch", "the bonus is [heads, dk] and goes with the read-out before the update", f"bonus={tuple(bonus.shape)}")
    used = _I(1)
    _call("alofa_linear_recurrence", _ptr(out), _I(max_parts), _L(part_stride), ctypes.byref(used), _ptr(q), _L(_rows("q", q)), _ptr(k), _L(_rows("k", k)), _ptr(v), _L(_rows("v", v)), _I(dtype_code(q)),
          _ptr(None if per_head else decay), _L(0 if per_head else _rows("decay", decay)), _ptr(decay if per_head else None), _ptr(bonus), _ptr(state),
          _ptr(rows.slots), _ptr(rows.offsets), _I(rows.requests), _I(T), _I(heads), _I(dk), _I(dv), _I(decay_kind), _F(tau), _F(q_scale), _F(k_scale),
          _I(int(before_update)), _stream())
    return used.value


def gate_scan(gates: torch.Tensor, z: torch.Tensor, state: torch.Tensor, rows: RowsOfRequests, heads: int, cap: float) -> None:
    """Exponential gates kept in range by a running maximum m (``state`` float32 [slots, heads], read and left there), per request over
    its rows in order: with z [T, 2 * heads] float32 (input gates' then forget gates' products), i = cap tanh(zi / cap),
    f = log sigmoid(cap tanh(zf / cap)), m' = max(f + m, i): gates[0], [1], [2] = exp(f + m - m'), exp(i - m'), exp(-m'), each float32 [T, heads] (``gates`` [3, T, heads])."""
    _gpu("gates", gates, torch.float32, 3), _contig("gates", gates), _gpu("z", z, torch.float32, 2), _gpu("state", state, torch.float32, 2), _contig("state", state)
    T = z.shape[0]
    if tuple(gates.shape) != (3, T, heads) or z.shape[1] != 2 * heads or state.shape[1] != heads or T != rows.rows or not cap > 0:
        raise AlofaError("shape_mismatch", "gate operands do not fit", f"gates={tuple(gates.shape)} z={tuple(z.shape)} state={tuple(state.shape)} heads={heads} rows={rows.rows}")
    rows.fits("state", state)
    _call("alofa_gate_scan", _ptr(gates), _ptr(z), _L(_rows("z", z)), _ptr(state), _ptr(rows.slots), _ptr(rows.offsets), _I(rows.requests), _L(T), _I(heads), _F(cap), _stream())


def gated_operands(qf: torch.Tensor, kf: torch.Tensor, vf: torch.Tensor, decay: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                   gates: torch.Tensor, heads: int, dk: int, dv: int) -> None:
    """What ``linear_recurrence`` takes for a memory with gates per row and head (``gate_scan``), as float32 rows: qf = q, kf = take * k,
    decay = keep for every key channel of the head, vf [T, heads * (dv + 1)] = the head's values and a one (whose read-out is the normaliser)."""
    T = q.shape[0]
    for n, t, w in (("qf", qf, heads * dk), ("kf", kf, heads * dk), ("decay", decay, heads * dk), ("vf", vf, heads * (dv + 1))):
        _gpu(n, t, torch.float32, 2), _contig(n, t)
        if tuple(t.shape) != (T, w):
            raise AlofaError("shape_mismatch", "the float operands do not fit", f"operand={n} shape={tuple(t.shape)} rows={T} width={w}")
    _gpu("q", q, None, 2), _gpu("k", k, q.dtype, 2), _gpu("v", v, q.dtype, 2), _gpu("gates", gates, torch.float32, 3), _contig("gates", gates)
    if tuple(q.shape) != (T, heads * dk) or tuple(k.shape) != (T, heads * dk) or tuple(v.shape) != (T, heads * dv) or tuple(gates.shape) != (3, T, heads):
        raise AlofaError("shape_mismatch", "the rows do not fit", f"q={tuple(q.shape)} k={tuple(k.shape)} v={tuple(v.shape)} gates={tuple(gates.shape)}")
    _call("alofa_gated_operands", _ptr(qf), _ptr(kf), _ptr(vf), _ptr(decay), _ptr(q), _L(_rows("q", q)), _ptr(k), _L(_rows("k", k)), _ptr(v), _L(_rows("v", v)),
          _I(dtype_code(q)), _ptr(gates), _L(T), _I(heads), _I(dk), _I(dv), _stream())


# ------------------------------------------------------------- scaled sub-layers, pair embedding, stream joins, choices among experts

def pair_embed(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0, store: Optional[torch.Tensor] = None,
               pairs: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None, state: Optional[torch.Tensor] = None,
               rows: Optional[RowsOfRequests] = None, buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0) -> None:
    """out[t] = table[ids[t]] * scale, plus, with ``pairs`` [buckets + 1, width], its row (before * mul_prev + id * mul_cur) mod
    buckets, ``before`` being the request's token one place earlier: the row above in the step, or, for a request's first
    row of the step, ``state[slot]`` (int32 [slots, 1]); a token at position 0 takes the row ``buckets``. The request's last
    token of the step is left in ``state``. Ids below zero name tokens in ``store``, as for ``embed_gather``."""
    _gpu("out", out, torch.float32, 2), _gpu("table", table, None, 2), _gpu("ids", ids, torch.int32, 1)
    _contig("out", out), _contig("table", table), _contig("ids", ids)
    T, h = out.shape
    if table.shape[1] != h or ids.shape[0] != T:
        raise AlofaError("shape_mismatch", "embedding width or token count does not fit", f"out={tuple(out.shape)} table={tuple(table.shape)} ids={tuple(ids.shape)}")
    if store is not None:
        _gpu("store", store, torch.int32, 1), _contig("store", store)
    slots = offsets = req_of_row = None
    if pairs is not None:
        _gpu("pairs", pairs, table.dtype, 2), _contig("pairs", pairs), _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
        _gpu("state", state, torch.int32), _contig("state", state)
        if rows is None or tuple(pairs.shape) != (buckets + 1, h) or positions.shape[0] != T or rows.rows != T or buckets <= 0 or state.numel() < rows.n_slots:
            raise AlofaError("shape_mismatch", "the pair table, positions, rows or state do not fit", f"pairs={tuple(pairs.shape)} buckets={buckets} tokens={T}")
        slots, offsets, req_of_row = rows.slots, rows.offsets, rows.req_of_row
    _call("alofa_pair_embed", _ptr(out), _ptr(table), _ptr(pairs), _I(dtype_code(table)), _ptr(ids), _ptr(positions), _ptr(state), _ptr(slots), _ptr(offsets),
          _ptr(req_of_row), _I(T), _I(h), _ptr(store), _I(table.shape[0]), _F(scale), _L(buckets), _L(mul_prev), _L(mul_cur), _stream())


def concat_rows(out: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> None:
    """out[t] = [a[t] | b[t]]: two float32 streams side by side in out's dtype."""
    _gpu("out", out, None, 2), _gpu("a", a, torch.float32, 2), _gpu("b", b, torch.float32, 2), _contig("out", out), _contig("a", a), _contig("b", b)
    if a.shape != b.shape or tuple(out.shape) != (a.shape[0], 2 * a.shape[1]):
        raise AlofaError("shape_mismatch", "two streams of one shape, and an output twice as wide", f"out={tuple(out.shape)} a={tuple(a.shape)} b={tuple(b.shape)}")
    _call("alofa_concat_rows", _ptr(out), _I(dtype_code(out)), _ptr(a), _ptr(b), _L(a.shape[0]), _I(a.shape[1]), _stream())


def rmsnorm_spread(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, eps: float, pad: int, copies: int, exact: bool = False) -> None:
    """out[t, k * pad + j] = rmsnorm(x[t])[j] * w[j] for k < copies (zeros for j from x's width up to pad). x float32 rows (or
    bfloat16 ones for a bfloat16 result), out rows of at least copies * pad values; row strides allowed."""
    _gpu("out", out, None, 2), _gpu("x", x, None, 2), _gpu("w", w, torch.float32, 1), _contig("w", w)
    if x.dtype is not torch.float32 and (x.dtype is not out.dtype or exact):
        raise AlofaError("invalid_argument", "the rows to norm are float32, or bfloat16 for a bfloat16 result", f"x={x.dtype} out={out.dtype}")
    n, r = x.shape
    if out.shape[0] != n or out.shape[1] != copies * pad or w.shape[0] != r or pad < r:
        raise AlofaError("shape_mismatch", "the copies of the normed rows do not fit", f"out={tuple(out.shape)} x={tuple(x.shape)} pad={pad} copies={copies}")
    _call("alofa_rmsnorm_spread", _ptr(out), _I(dtype_code(out)), _L(_rows("out", out)), _ptr(x), _I(dtype_code(x)), _L(_rows("x", x)), _ptr(w), _I(n), _I(r), _I(pad), _I(copies),
          _F(eps), _I(int(exact)), _stream())


def sigmoid_gate(x: torch.Tensor, g: torch.Tensor, exact: bool = False) -> None:
    """x *= sigmoid(g), element by element on rows (row strides allowed)."""
    _gpu("x", x, None, 2), _gpu("g", g, x.dtype, 2)
    if x.shape != g.shape:
        raise AlofaError("shape_mismatch", "gate and rows must agree", f"x={tuple(x.shape)} g={tuple(g.shape)}")
    _call("alofa_sigmoid_gate", _ptr(x), _L(_rows("x", x)), _ptr(g), _L(_rows("g", g)), _I(dtype_code(x)), _L(x.shape[0]), _I(x.shape[1]), _I(int(exact)), _stream())


def add_channel_scaled(residual: torch.Tensor, x: torch.Tensor, scale: torch.Tensor, exact: bool = False) -> None:
    """residual[t, c] += scale[c] * x[t, c], all float32."""
    _gpu("residual", residual, torch.float32, 2), _gpu("x", x, torch.float32, 2), _gpu("scale", scale, torch.float32, 1)
    _contig("residual", residual), _contig("x", x), _contig("scale", scale)
    if x.shape != residual.shape or scale.shape[0] != residual.shape[1]:
        raise AlofaError("shape_mismatch", "one factor per channel of the stream", f"residual={tuple(residual.shape)} x={tuple(x.shape)} scale={tuple(scale.shape)}")
    _call("alofa_add_channel_scaled", _ptr(residual), _ptr(x), _ptr(scale), _L(residual.shape[0]), _I(residual.shape[1]), _I(int(exact)), _stream())


def softcap_(x: torch.Tensor, cap: float, exact: bool = False) -> None:
    """x = cap * tanh(x / cap) (float32, contiguous)."""
    _gpu("x", x, torch.float32), _contig("x", x)
    _call("alofa_softcap", _ptr(x), _F(cap), _L(x.numel()), _I(int(exact)), _stream())


def relu_squared(out: torch.Tensor, x: torch.Tensor) -> None:
    """out = max(x, 0)^2 on rows (row strides allowed; out may be x)."""
    _gpu("out", out, None, 2), _gpu("x", x, out.dtype, 2)
    if out.shape != x.shape:
        raise AlofaError("shape_mismatch", "activation operands do not fit", f"out={tuple(out.shape)} x={tuple(x.shape)}")
    _call("alofa_relu_squared", _ptr(out), _L(_rows("out", out)), _ptr(x), _L(_rows("x", x)), _I(dtype_code(out)), _L(x.shape[0]), _I(x.shape[1]), _stream())


MAX_EXPERTS = 512


def route_top(z: torch.Tensor, dense: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor, top: int, scale: float = 1.0,
              renormalize: bool = False, exact: bool = False) -> None:
    """Per row of the router products z [T, E] (float32) the ``top`` largest (the lower index among equals):
    ``chosen`` int32 [T, top] and ``weights`` float32 [T, top] = sigmoid(z) * scale (made to sum to one first with
    ``renormalize``), in order of falling score; ``dense`` float32 [T, E] holds the same weights at the chosen places and 0 elsewhere."""
    _gpu("z", z, torch.float32, 2), _gpu("dense", dense, torch.float32, 2), _gpu("chosen", chosen, torch.int32, 2), _gpu("weights", weights, torch.float32, 2)
    for n, t in (("z", z), ("dense", dense), ("chosen", chosen), ("weights", weights)):
        _contig(n, t)
    T, E = z.shape
    if tuple(dense.shape) != (T, E) or tuple(chosen.shape) != (T, top) or tuple(weights.shape) != (T, top) or not 0 < top <= E <= MAX_EXPERTS:
        raise AlofaError("shape_mismatch", "the choice's outputs do not fit", f"z={tuple(z.shape)} dense={tuple(dense.shape)} chosen={tuple(chosen.shape)} top={top}")
    _call("alofa_route_top", _ptr(z), _ptr(dense), _ptr(chosen), _ptr(weights), _I(T), _I(E), _I(top), _F(scale), _I(int(renormalize)), _I(int(exact)), _stream())


def route_groups(z: torch.Tensor, correction: Optional[torch.Tensor], dense: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor,
                 pass_weight: torch.Tensor, top: int, passing: int = 0, groups: int = 1, keep: int = 1, scale: float = 1.0, renormalize: bool = False,
                 exact: bool = False) -> None:
    """The choice by softmax scores: s = softmax(z) over all E columns of z [T, E]; the choice goes by s + correction; the experts form
    ``groups`` equal groups of neighbours, of which the ``keep`` with the largest member stay in the choice; the ``top`` largest of those are
    taken (``chosen`` int32 [T, top]), weighted by their s (``weights``). The last ``passing`` experts have no matrices: ``dense`` float32
    [T, E - passing] holds the weights of the others, ``pass_weight`` float32 [T] the summed weights of taken experts without matrices."""
    _gpu("z", z, torch.float32, 2), _gpu("dense", dense, torch.float32, 2), _gpu("chosen", chosen, torch.int32, 2), _gpu("weights", weights, torch.float32, 2)
    _gpu("pass_weight", pass_weight, torch.float32, 1)
    for n, t in (("z", z), ("dense", dense), ("chosen", chosen), ("weights", weights), ("pass_weight", pass_weight)):
        _contig(n, t)
    T, E = z.shape
    if correction is not None:
        _gpu("correction", correction, torch.float32, 1), _contig("correction", correction)
    if (tuple(dense.shape) != (T, E - passing) or tuple(chosen.shape) != (T, top) or tuple(weights.shape) != (T, top) or pass_weight.shape[0] != T
            or not 0 < top <= E <= MAX_EXPERTS or not 0 <= passing < E or (correction is not None and correction.shape[0] != E)
            or groups < 1 or E % groups or not 1 <= keep <= groups or top > keep * (E // groups)):
        raise AlofaError("shape_mismatch", "the choice's operands do not fit", f"z={tuple(z.shape)} dense={tuple(dense.shape)} chosen={tuple(chosen.shape)} top={top} passing={passing} groups={groups} keep={keep}")
    _call("alofa_route_groups", _ptr(z), _ptr(correction), _ptr(dense), _ptr(chosen), _ptr(weights), _ptr(pass_weight), _I(T), _I(E), _I(passing), _I(top),
          _I(groups), _I(keep), _F(scale), _I(int(renormalize)), _I(int(exact)), _stream())


def clamped_glu(act: torch.Tensor, g: torch.Tensor, u: torch.Tensor, dense: Optional[torch.Tensor], experts: int, ff: int, shared_ff: int,
                limit: float, shared_limit: float, slope: float, exact: bool = False, offset: float = 1.0) -> None:
    """act[t, c] = w a sigmoid(slope a) (b + offset), a = min(g, limit), b = clamp(u, -limit, limit), for the channels of ``experts``
    experts of ``ff`` channels side by side (w = dense[t, expert]) and then ``shared_ff`` channels with w = 1 and a limit of their own."""
    for n, t in (("act", act), ("g", g), ("u", u)):
        _gpu(n, t, act.dtype, 2), _contig(n, t)
    F = experts * ff + shared_ff
    T = act.shape[0]
    if tuple(g.shape) != (T, F) or tuple(u.shape) != (T, F) or act.shape[1] != F:
        raise AlofaError("shape_mismatch", "gate, up and output are [rows, all experts' channels]", f"act={tuple(act.shape)} g={tuple(g.shape)} u={tuple(u.shape)} F={F}")
    if experts:
        _gpu("dense", dense, torch.float32, 2), _contig("dense", dense)
        if tuple(dense.shape) != (T, experts):
            raise AlofaError("shape_mismatch", "one weight per row and expert", f"dense={tuple(dense.shape)}")
    _call("alofa_clamped_glu", _ptr(act), _ptr(g), _ptr(u), _I(dtype_code(act)), _ptr(dense if experts else None), _L(T), _I(experts), _I(ff), _I(shared_ff),
          _F(limit), _F(shared_limit), _F(slope), _F(offset), _I(int(exact)), _stream())


def gemm_channel_scaled(residual: torch.Tensor, a: torch.Tensor, w: torch.Tensor, scale: torch.Tensor, tmp: torch.Tensor, exact: bool = False,
                        then_norm: Optional[tuple] = None, bias: Optional[torch.Tensor] = None) -> None:
    """residual[t, c] += scale[c] * ((a @ w.T)[t, c] + bias[c]); ``tmp`` float32 of the residual's shape takes the product on its way.
    ``then_norm`` = (weight, eps, rows): afterwards ``rows`` holds the RMSNorm of the residual's new rows (the same launch adds and norms)."""
    gemm(tmp, a, w, bias, exact=exact)
    if then_norm is None:
        add_channel_scaled(residual, tmp, scale, exact)
    else:
        add_channel_scaled_norm(residual, tmp, scale, *then_norm, exact=exact)


def add_channel_scaled_norm(residual: torch.Tensor, x: torch.Tensor, scale: torch.Tensor, weight: torch.Tensor, eps: float, normed: torch.Tensor,
                            exact: bool = False) -> None:
    """residual[t, c] += scale[c] * x[t, c]; normed[t] = rmsnorm(residual[t]) * weight."""
    _gpu("residual", residual, torch.float32, 2), _gpu("x", x, torch.float32, 2), _gpu("scale", scale, torch.float32, 1), _gpu("weight", weight, torch.float32, 1)
    _gpu("normed", normed, None, 2)
    for n, t in (("residual", residual), ("x", x), ("scale", scale), ("weight", weight), ("normed", normed)):
        _contig(n, t)
    T, h = residual.shape
    if x.shape != residual.shape or normed.shape != residual.shape or scale.shape[0] != h or weight.shape[0] != h:
        raise AlofaError("shape_mismatch", "one factor and one norm weight per channel; rows of the stream's shape", f"residual={tuple(residual.shape)} x={tuple(x.shape)} normed={tuple(normed.shape)}")
    _call("alofa_add_channel_scaled_norm", _ptr(residual), _ptr(x), _ptr(scale), _ptr(normed), _I(dtype_code(normed)), _ptr(weight), _L(T), _I(h), _F(eps),
          _I(int(exact)), _stream())


GR_STORE, GR_SIGMOID_GATE, GR_CLAMPED_GLU = 0, 1, 2
GROUPED_BIG_TILES = 256     # rows of a step from which the many-small-products kernel takes tiles of 64 rows instead of 16


def _grouped(out, out_step, x, x_step, w, w2, w_stride, w_step, n_out, K, last, rows, x_by_slot, tiles, tiles_per_batch, tile_batch, row_in,
             gate, slot_weight, limit, limit_last, slope, epilogue, tile_rows=16, offset=1.0) -> None:
    last_batch, n_out_last, K_last = last if last is not None else (-1, n_out, K)
    _call("alofa_grouped_product", _ptr(out), _I(dtype_code(out)), _L(_rows("out", out)), _L(out_step), _ptr(x), _L(_rows("x", x)), _L(x_step),
          _ptr(w), _ptr(w2), _L(w_stride), _L(w_step), _I(n_out), _I(K), _I(last_batch), _I(n_out_last), _I(K_last), _I(rows), _I(int(x_by_slot)), _I(tiles),
          _I(tiles_per_batch), _I(tile_rows), _ptr(tile_batch), _ptr(row_in), _ptr(gate), _L(_rows("gate", gate) if gate is not None else 0), _ptr(slot_weight),
          _F(limit), _F(limit_last), _F(slope), _F(offset), _I(epilogue), _stream())


def _aligned_rows(t: torch.Tensor) -> bool:
    return t.dtype is torch.bfloat16 and t.stride(-1) == 1 and t.stride(0) % 8 == 0 and t.data_ptr() % 16 == 0


def head_project(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, exact: bool = False, gate: Optional[torch.Tensor] = None) -> None:
    """out[t, a, :] = w[a] @ x[t, a, :] for every head a: x [T, H * din] and out [T, H * dout] hold the heads side by side (row
    strides allowed), w is [H, dout, din]. With ``gate`` (out's shape): out *= sigmoid(gate). bfloat16 rows whose heads start at
    16-byte borders run as one launch on the matrix cores; everything else head by head through ``gemm``."""
    _gpu("out", out, None, 2), _gpu("x", x, out.dtype, 2), _gpu("w", w, None, 3), _contig("w", w)
    H, dout, din = w.shape
    if x.shape[0] != out.shape[0] or x.shape[1] != H * din or out.shape[1] != H * dout:
        raise AlofaError("shape_mismatch", "the heads' rows do not fit their matrices", f"out={tuple(out.shape)} x={tuple(x.shape)} w={tuple(w.shape)}")
    if gate is not None:
        _gpu("gate", gate, out.dtype, 2)
        if gate.shape != out.shape:
            raise AlofaError("shape_mismatch", "one gate per output", f"gate={tuple(gate.shape)} out={tuple(out.shape)}")
    T = x.shape[0]
    if not exact and out.dtype is torch.bfloat16 and w.dtype is torch.bfloat16 and din % 8 == 0 and _aligned_rows(x) and w.data_ptr() % 16 == 0 and T > 0:
        tile_rows = 64 if T >= GROUPED_BIG_TILES else 16      # (tiles of 64 rows, which use a fragment of the matrix four times, once there are rows for them)
        per = (T + tile_rows - 1) // tile_rows
        _grouped(out, dout, x, din, w, None, din, dout * din, dout, din, None, T, False, H * per, per, None, None, gate, None, 0.0, 0.0, 0.0,
                 GR_SIGMOID_GATE if gate is not None else GR_STORE, tile_rows)
        return
    for a in range(H):
        gemm(out[:, a * dout:(a + 1) * dout], x[:, a * din:(a + 1) * din], w[a], exact=exact)
    if gate is not None:
        sigmoid_gate(out, gate, exact)


class ExpertRows:
    """The rows of a step sorted by the experts they take (``expert_rows``): ``row_in`` int32 [slots] (the row in a slot, -1: none),
    ``slot_weight`` float32 [slots], ``slot_of`` int32 [T * top (+ T)] (the slot of row t's k-th choice; then, with a shared expert, of
    row t's place in it), ``tile_batch`` int32 [tiles] (the expert of every 16 slots, -1: none)."""

    def __init__(self, T: int, top: int, experts: int, shared: bool, scratch):
        self.T, self.top, self.experts, self.shared = T, top, experts, shared
        # an expert's rows fill whole tiles: of 64 rows where the experts get that many on average, else of 16
        pad = self.tile_rows = 64 if T >= GROUPED_BIG_TILES and T * top >= 64 * experts else 16
        self.slots = (T * top + pad - 1) // pad * pad + pad * experts + ((T + pad - 1) // pad * pad if shared else 0)
        self.tiles = self.slots // pad
        self.row_in, self.slot_weight = scratch("expert_row_in", (self.slots,), torch.int32), scratch("expert_slot_weight", (self.slots,), torch.float32)
        self.slot_of, self.tile_batch = scratch("expert_slot_of", (T * (top + 1),), torch.int32), scratch("expert_tile_batch", (self.tiles,), torch.int32)


def expert_rows(rows: ExpertRows, chosen: torch.Tensor, weights: torch.Tensor) -> None:
    _gpu("chosen", chosen, torch.int32, 2), _gpu("weights", weights, torch.float32, 2), _contig("chosen", chosen), _contig("weights", weights)
    if tuple(chosen.shape) != (rows.T, rows.top) or tuple(weights.shape) != (rows.T, rows.top):
        raise AlofaError("shape_mismatch", "one choice and one weight per row and place", f"chosen={tuple(chosen.shape)} weights={tuple(weights.shape)}")
    _call("alofa_expert_rows", _ptr(chosen), _ptr(weights), _ptr(rows.row_in), _ptr(rows.slot_weight), _ptr(rows.slot_of), _ptr(rows.tile_batch),
          _I(rows.T), _I(rows.top), _I(rows.experts), _I(int(rows.shared)), _I(rows.slots), _I(rows.tiles), _I(rows.tile_rows), _stream())


def can_group_experts(x: torch.Tensor, w_gate: torch.Tensor, ff: int, shared_ff: int) -> bool:
    """Whether the experts' products can run slot by slot on the matrix cores: bfloat16, every reduction a multiple of eight."""
    return (x.dtype is torch.bfloat16 and w_gate.dtype is torch.bfloat16 and _aligned_rows(x) and x.shape[1] % 8 == 0 and ff % 8 == 0 and shared_ff % 8 == 0)


def experts_gate_up(act: torch.Tensor, x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, rows: ExpertRows, ff: int, shared_ff: int,
                    limit: float, shared_limit: float, slope: float, offset: float = 1.0) -> None:
    """act[slot, :] = weight[slot] * a sigmoid(slope a) (b + offset) with a = min(gate_e(x[row]), limit), b = clamp(up_e(x[row]), -limit, limit)
    for the expert e of the slot; w_gate and w_up hold the experts' matrices one below the other ([E * ff (+ shared_ff), h])."""
    _gpu("act", act, torch.bfloat16, 2), _gpu("x", x, torch.bfloat16, 2), _gpu("w_gate", w_gate, torch.bfloat16, 2), _gpu("w_up", w_up, torch.bfloat16, 2)
    _contig("w_gate", w_gate), _contig("w_up", w_up), _contig("act", act)
    h = x.shape[1]
    F = rows.experts * ff + (shared_ff if rows.shared else 0)
    if tuple(w_gate.shape) != (F, h) or tuple(w_up.shape) != (F, h) or act.shape[0] < rows.slots or act.shape[1] < max(ff, shared_ff) or x.shape[0] != rows.T:
        raise AlofaError("shape_mismatch", "the experts' matrices or the slots' rows do not fit", f"act={tuple(act.shape)} x={tuple(x.shape)} w_gate={tuple(w_gate.shape)} F={F}")
    _grouped(act, 0, x, 0, w_gate, w_up, h, ff * h, ff, h, (rows.experts, shared_ff, h) if rows.shared else None, rows.slots, False, rows.tiles, 0,
             rows.tile_batch, rows.row_in, None, rows.slot_weight, limit, shared_limit, slope, GR_CLAMPED_GLU, rows.tile_rows, offset)


def experts_down(y: torch.Tensor, act: torch.Tensor, w_down: torch.Tensor, rows: ExpertRows, ff: int, shared_ff: int) -> None:
    """y[slot, :] = down_e(act[slot, :]) (float32); w_down holds the experts' matrices side by side ([h, E * ff (+ shared_ff)])."""
    _gpu("y", y, torch.float32, 2), _gpu("act", act, torch.bfloat16, 2), _gpu("w_down", w_down, torch.bfloat16, 2), _contig("w_down", w_down), _contig("y", y)
    h = w_down.shape[0]
    F = rows.experts * ff + (shared_ff if rows.shared else 0)
    if w_down.shape[1] != F or tuple(y.shape) != (rows.slots, h) or act.shape[0] < rows.slots or not _aligned_rows(act) or F % 8:
        raise AlofaError("shape_mismatch", "the experts' matrices or the slots' rows do not fit", f"y={tuple(y.shape)} act={tuple(act.shape)} w_down={tuple(w_down.shape)} F={F}")
    _grouped(y, 0, act, 0, w_down, None, F, ff, h, ff, (rows.experts, h, shared_ff) if rows.shared else None, rows.slots, True, rows.tiles, 0,
             rows.tile_batch, rows.row_in, None, None, 0.0, 0.0, 0.0, GR_STORE, rows.tile_rows)


def experts_sum(residual: torch.Tensor, y: torch.Tensor, rows: ExpertRows, scale: Optional[torch.Tensor] = None, passed: Optional[tuple] = None,
                assign: bool = False) -> None:
    """residual[t] += scale * (sum over row t's choices k, ascending, of y[slot of (t, k)], then its slot of the shared expert). A choice
    without a slot (an expert without matrices) adds nothing here; ``passed`` = (weight float32 [T], x bfloat16 [T, h]) adds weight[t] * x[t]
    to the sum: the row itself, handed on. ``assign``: the sum is stored instead of added."""
    _gpu("residual", residual, torch.float32, 2), _gpu("y", y, torch.float32, 2), _contig("residual", residual), _contig("y", y)
    T, h = residual.shape
    if T != rows.T or tuple(y.shape) != (rows.slots, h):
        raise AlofaError("shape_mismatch", "the slots' results do not fit the stream", f"residual={tuple(residual.shape)} y={tuple(y.shape)}")
    if scale is not None:
        _gpu("scale", scale, torch.float32, 1), _contig("scale", scale)
        if scale.shape[0] != h:
            raise AlofaError("shape_mismatch", "one factor per channel of the stream", f"scale={tuple(scale.shape)}")
    pw = px = None
    if passed is not None:
        pw, px = passed
        _gpu("pass weight", pw, torch.float32, 1), _contig("pass weight", pw), _gpu("passed rows", px, torch.bfloat16, 2)
        if pw.shape[0] != T or tuple(px.shape) != (T, h):
            raise AlofaError("shape_mismatch", "one weight and one row to hand on per row of the stream", f"weight={tuple(pw.shape)} rows={tuple(px.shape)}")
    _call("alofa_experts_sum", _ptr(residual), _ptr(y), _ptr(rows.slot_of), _ptr(scale), _I(T), _I(h), _I(rows.top), _I(int(rows.shared)),
          _ptr(pw), _ptr(px), _L(_rows("passed rows", px) if px is not None else 0), _I(int(assign)), _stream())


# ------------------------------------------------------------- attention over a window: norms before the turn, pooled blocks, a bias by distance, a sink

NORM_NONE, NORM_HEAD, NORM_ALL = 0, 1, 2
GATE_NONE, GATE_CHANNEL, GATE_HEAD = 0, 1, 2


def pooled_places(block_size: int, pool: int) -> int:
    """Places of a page for the blocks of ``pool`` tokens that begin in it."""
    return (block_size - 1) // pool + 1


def norm_turn_write(qkv: torch.Tensor, positions: torch.Tensor, table: Optional[tuple], heads: int, kv_heads: int, d: int, dv: int, scope: int,
                    wq: Optional[torch.Tensor], wk: Optional[torch.Tensor], eps: float, exact: bool, slots: Optional[torch.Tensor] = None,
                    k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None, values_are_keys: bool = False,
                    row_factors: Optional[torch.Tensor] = None, true_d: Optional[int] = None) -> None:
    """What a step's projections become before attention. ``qkv`` [T, heads * d + kv_heads * d (+ kv_heads * dv)]: query heads, key heads and (unless
    ``values_are_keys``) value heads side by side. Queries and keys are divided by a root mean square (``scope`` NORM_HEAD: every head's own over d;
    NORM_ALL: the whole query projection's, and the whole key projection's, of the row; NORM_NONE: not at all) and multiplied by ``wq`` / ``wk`` (float32,
    [d] per head alike for NORM_HEAD, [heads * d] / [kv_heads * d] for NORM_ALL, None: no weight), then turned by ``table`` (cos, sin float32 [n, pairs]:
    channel i with i + pairs; None: not turned). Queries are left in place; keys go to ``k_cache`` [pages, kv_heads, page, d] and values, transposed, to
    ``v_cache`` [pages, kv_heads, dv, page] at ``slots`` int64 [T]; with ``values_are_keys`` the values are the keys as projected, before norm and turn.
    ``row_factors``: float64 [T, 2], room that NORM_ALL needs. ``true_d``: how many of a head's d channels count in the mean (heads widened with zeros)."""
    _gpu("qkv", qkv, None, 2), _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
    T = qkv.shape[0]
    cos = sin = None
    half = 0
    if table is not None:
        cos, sin = table
        _gpu("cos", cos, torch.float32, 2), _gpu("sin", sin, torch.float32, 2), _contig("cos", cos), _contig("sin", sin)
        half = cos.shape[1]
        if cos.shape != sin.shape or 2 * half > d:
            raise AlofaError("shape_mismatch", "the table of angles does not fit the heads", f"table={tuple(cos.shape)} d={d}")
    width = heads * d + kv_heads * d + (0 if values_are_keys else kv_heads * dv)
    if qkv.shape[1] != width or positions.shape[0] != T or scope not in (NORM_NONE, NORM_HEAD, NORM_ALL) or (values_are_keys and d != dv):
        raise AlofaError("shape_mismatch", "rows or positions do not fit", f"qkv={tuple(qkv.shape)} heads={heads} kv_heads={kv_heads} d={d} dv={dv} scope={scope}")
    for name, w, n in (("wq", wq, heads), ("wk", wk, kv_heads)):
        if w is not None:
            _gpu(name, w, torch.float32, 1), _contig(name, w)
            if scope == NORM_NONE or w.shape[0] != (d if scope == NORM_HEAD else n * d):
                raise AlofaError("shape_mismatch", "a norm's weight does not fit its scope", f"operand={name} shape={tuple(w.shape)} scope={scope}")
    block = 0
    if kv_heads:
        _gpu("slots", slots, torch.int64, 1), _contig("slots", slots), _gpu("k_cache", k_cache, qkv.dtype, 4), _gpu("v_cache", v_cache, qkv.dtype, 4)
        _contig("k_cache", k_cache), _contig("v_cache", v_cache)
        block = k_cache.shape[2]
        if slots.shape[0] != T or tuple(k_cache.shape[1:]) != (kv_heads, block, d) or tuple(v_cache.shape) != (k_cache.shape[0], kv_heads, dv, block):
            raise AlofaError("shape_mismatch", "caches or slots do not fit", f"k={tuple(k_cache.shape)} v={tuple(v_cache.shape)} slots={tuple(slots.shape)}")
    if scope == NORM_ALL:
        _gpu("row_factors", row_factors, torch.float64, 2), _contig("row_factors", row_factors)
        if tuple(row_factors.shape) != (T, 2):
            raise AlofaError("shape_mismatch", "two factors per row", f"row_factors={tuple(row_factors.shape)}")
    _call("alofa_norm_turn_write", _ptr(qkv), _L(_rows("qkv", qkv)), _I(dtype_code(qkv)), _ptr(positions), _ptr(cos), _ptr(sin), _I(half), _I(scope), _ptr(wq), _ptr(wk),
          _F(eps), _ptr(row_factors if scope == NORM_ALL else None), _ptr(slots), _ptr(k_cache), _ptr(v_cache), _I(block), _I(T), _I(heads), _I(kv_heads), _I(d), _I(dv),
          _I(int(true_d or d)), _I(int(values_are_keys)), _I(int(exact)), _stream())


def _pooled_operands(pk, pv, pool_table, k_cache, kv_heads: int, d: int, dv: int, pool: int) -> int:
    block = k_cache.shape[2]
    places = pooled_places(block, pool)
    _gpu("pooled keys", pk, k_cache.dtype, 4), _gpu("pooled values", pv, k_cache.dtype, 4), _contig("pooled keys", pk), _contig("pooled values", pv)
    _gpu("pool_table", pool_table, torch.int32, 2), _contig("pool_table", pool_table)
    if tuple(pk.shape[1:]) != (kv_heads, places, d) or tuple(pv.shape) != (pk.shape[0], kv_heads, dv, places) or pool <= 0:
        raise AlofaError("shape_mismatch", "the pooled blocks' pages do not fit", f"keys={tuple(pk.shape)} values={tuple(pv.shape)} page={block} pool={pool} places={places}")
    return places


def pool_blocks(k_cache: torch.Tensor, v_cache: torch.Tensor, pk: torch.Tensor, pv: torch.Tensor, block_table: torch.Tensor, pool_table: torch.Tensor,
                req_of_token: Optional[torch.Tensor], positions: torch.Tensor, kv_heads: int, d: int, dv: int, pool: int, exact: bool = False) -> None:
    """Every row whose position ends a block of ``pool`` tokens leaves the mean of the block's keys and of its values, read from the pages
    (``k_cache`` [pages, kv_heads, page, d], ``v_cache`` [pages, kv_heads, dv, page] through ``block_table``), in ``pk`` [pages', kv_heads, places, d] and
    ``pv`` [pages', kv_heads, dv, places] through ``pool_table``: block b at the page of its first token, place ((b pool) % page) // pool."""
    _gpu("k_cache", k_cache, None, 4), _gpu("v_cache", v_cache, k_cache.dtype, 4), _contig("k_cache", k_cache), _contig("v_cache", v_cache)
    _gpu("block_table", block_table, torch.int32, 2), _contig("block_table", block_table), _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
    block = k_cache.shape[2]
    if tuple(k_cache.shape[1:]) != (kv_heads, block, d) or tuple(v_cache.shape) != (k_cache.shape[0], kv_heads, dv, block):
        raise AlofaError("shape_mismatch", "caches do not fit", f"k={tuple(k_cache.shape)} v={tuple(v_cache.shape)}")
    places = _pooled_operands(pk, pv, pool_table, k_cache, kv_heads, d, dv, pool)
    T = positions.shape[0]
    if req_of_token is not None:
        _gpu("req_of_token", req_of_token, torch.int32, 1), _contig("req_of_token", req_of_token)
    elif min(block_table.shape[0], pool_table.shape[0]) < T:
        raise AlofaError("shape_mismatch", "without a request per row every row is a request of its own", f"rows={T} tables={block_table.shape[0]}")
    _call("alofa_pool_blocks", _ptr(k_cache), _ptr(v_cache), _ptr(pk), _ptr(pv), _I(dtype_code(k_cache)), _ptr(block_table), _I(block_table.shape[1]), _ptr(pool_table),
          _I(pool_table.shape[1]), _ptr(req_of_token), _ptr(positions), _I(T), _I(kv_heads), _I(d), _I(dv), _I(block), _I(pool), _I(places), _I(int(exact)), _stream())


def span_attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor, req_of_token: Optional[torch.Tensor],
                   positions: torch.Tensor, heads: int, kv_heads: int, d: int, dv: int, window: Optional[int], scale: float, exact: bool = False,
                   pooled: Optional[tuple] = None, bias: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                   gate_kind: int = GATE_NONE) -> None:
    """The always-valid attention over a window: out[t, h] = (sum_e w_e v_e) * sigmoid(gate), the softmax weights w over the tokens row t may see (its request's, up to its
    position; the last ``window``) and, with ``pooled`` = (keys, values, table, pool), over the blocks of ``pool`` tokens that lie wholly behind the window (their mean keys
    and values, as ``pool_blocks`` left them); scores are scale * q . k, plus ``bias`` [heads, n] float32 by distance (the last entry for every distance from n - 1 on);
    ``sink`` [heads] float32 adds exp(sink) to the head's denominator. ``gate``: [T, heads * dv] (GATE_CHANNEL) or [T, heads] (GATE_HEAD). Rows ``q`` [T, heads * d],
    ``out`` [T, heads * dv] (row strides allowed)."""
    _gpu("out", out, None, 2), _gpu("q", q, out.dtype, 2), _gpu("k_cache", k_cache, out.dtype, 4), _gpu("v_cache", v_cache, out.dtype, 4)
    _contig("k_cache", k_cache), _contig("v_cache", v_cache), _gpu("block_table", block_table, torch.int32, 2), _contig("block_table", block_table)
    _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
    T, block = q.shape[0], k_cache.shape[2]
    if (tuple(q.shape) != (T, heads * d) or tuple(out.shape) != (T, heads * dv) or tuple(k_cache.shape[1:]) != (kv_heads, block, d)
            or tuple(v_cache.shape) != (k_cache.shape[0], kv_heads, dv, block) or positions.shape[0] != T):
        raise AlofaError("shape_mismatch", "attention operands do not fit", f"out={tuple(out.shape)} q={tuple(q.shape)} k={tuple(k_cache.shape)} v={tuple(v_cache.shape)} heads={heads} kv_heads={kv_heads} d={d} dv={dv}")
    pk = pv = pool_table = None
    pool = places = 0
    if pooled is not None:
        pk, pv, pool_table, pool = pooled
        places = _pooled_operands(pk, pv, pool_table, k_cache, kv_heads, d, dv, pool)
        if not window:
            raise AlofaError("invalid_argument", "pooled blocks lie behind a window")
    if req_of_token is not None:
        _gpu("req_of_token", req_of_token, torch.int32, 1), _contig("req_of_token", req_of_token)
    elif block_table.shape[0] < T or (pool_table is not None and pool_table.shape[0] < T):
        raise AlofaError("shape_mismatch", "without a request per row every row is a request of its own", f"rows={T} tables={block_table.shape[0]}")
    if bias is not None:
        _gpu("bias", bias, torch.float32, 2), _contig("bias", bias)
        if bias.shape[0] != heads or bias.shape[1] < 1:
            raise AlofaError("shape_mismatch", "the bias is [heads, distances]", f"bias={tuple(bias.shape)}")
    if sink is not None:
        _gpu("sink", sink, torch.float32, 1), _contig("sink", sink)
        if sink.shape[0] != heads:
            raise AlofaError("shape_mismatch", "one sink per head", f"sink={tuple(sink.shape)}")
    if gate_kind != GATE_NONE:
        _gpu("gate", gate, out.dtype, 2)
        if tuple(gate.shape) != (T, heads * dv if gate_kind == GATE_CHANNEL else heads):
            raise AlofaError("shape_mismatch", "the gate does not fit its kind", f"gate={tuple(gate.shape)} kind={gate_kind}")
    _call("alofa_span_attention", _ptr(out), _L(_rows("out", out)), _ptr(q), _L(_rows("q", q)), _ptr(k_cache), _ptr(v_cache), _ptr(pk), _ptr(pv), _I(dtype_code(out)),
          _ptr(block_table), _I(block_table.shape[1]), _ptr(pool_table), _I(pool_table.shape[1] if pool_table is not None else 0), _ptr(req_of_token), _ptr(positions),
          _I(T), _I(heads), _I(kv_heads), _I(d), _I(dv), _I(block), _I(int(window or 0)), _I(int(pool)), _I(places), _F(scale), _ptr(bias),
          _I(bias.shape[1] if bias is not None else 0), _ptr(sink), _ptr(gate if gate_kind != GATE_NONE else None),
          _L(_rows("gate", gate) if gate_kind != GATE_NONE else 0), _I(gate_kind), _I(int(exact)), _stream())


def head_gate(x: torch.Tensor, gate: torch.Tensor, heads: int, dv: int, per_head: bool, dv_stored: Optional[int] = None) -> None:
    """x[t, h, :dv] *= sigmoid(gate[t, h]) (``per_head``) or sigmoid(gate[t, h, :]); a head of x holds ``dv_stored`` channels (default dv)."""
    stored = dv if dv_stored is None else dv_stored
    _gpu("x", x, None, 2), _gpu("gate", gate, x.dtype, 2)
    T = x.shape[0]
    if x.shape[1] != heads * stored or tuple(gate.shape) != (T, heads if per_head else heads * dv):
        raise AlofaError("shape_mismatch", "the gate does not fit the heads", f"x={tuple(x.shape)} gate={tuple(gate.shape)} heads={heads} dv={dv}")
    _call("alofa_head_gate", _ptr(x), _L(_rows("x", x)), _ptr(gate), _L(_rows("gate", gate)), _I(dtype_code(x)), _L(T), _I(heads), _I(dv), _I(stored), _I(int(per_head)), _stream())


# ------------------------------------------------------------- a state-space mixer around the recurrence kernel

def conv_bias_act(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, rows: RowsOfRequests, silu: bool = True,
                  exact: bool = False) -> None:
    """out[t] = act(bias + sum_j w[:, j] * x[t - taps + 1 + j]) per channel, within each request; the inputs before a request's first row of this step come from
    ``state`` [slots, taps - 1, width] (x's dtype, contiguous; the newest last), which is not written (``conv_keep`` does that afterwards). Rows may have strides;
    ``out`` must not be ``x``. ``w`` float32 [width, taps], ``bias`` float32 [width] or None."""
    _gpu("out", out, x.dtype, 2), _gpu("x", x, None, 2), _gpu("w", w, torch.float32, 2), _gpu("state", state, x.dtype, 3), _contig("w", w), _contig("state", state)
    T, width = x.shape
    taps = w.shape[1]
    if tuple(out.shape) != (T, width) or w.shape[0] != width or tuple(state.shape[1:]) != (taps - 1, width) or T != rows.rows or not 1 <= taps <= CONV_MAX_TAPS:
        raise AlofaError("shape_mismatch", "convolution operands do not fit", f"out={tuple(out.shape)} x={tuple(x.shape)} w={tuple(w.shape)} state={tuple(state.shape)} rows={rows.rows}")
    if bias is not None:
        _gpu("bias", bias, torch.float32, 1), _contig("bias", bias)
        if bias.shape[0] != width:
            raise AlofaError("shape_mismatch", "one bias per channel", f"bias={tuple(bias.shape)}")
    if out.data_ptr() == x.data_ptr():
        raise AlofaError("invalid_argument", "the convolution does not run in place")
    rows.fits("state", state)
    _call("alofa_conv_bias_act", _ptr(out), _L(_rows("out", out)), _I(dtype_code(out)), _ptr(x), _L(_rows("x", x)), _I(dtype_code(x)), _ptr(w), _ptr(bias), _ptr(state),
          _ptr(rows.slots), _ptr(rows.offsets), _ptr(rows.req_of_row), _I(T), _I(width), _I(taps), _I(int(silu)), _I(int(exact)), _stream())


def conv_keep(state: torch.Tensor, x: torch.Tensor, rows: RowsOfRequests) -> None:
    """``keep_last_rows`` for rows with a stride: state[slot] = the last inputs its request has seen once this step's rows are in."""
    _gpu("state", state, x.dtype, 3), _gpu("x", x, None, 2), _contig("state", state)
    if state.shape[2] != x.shape[1] or x.shape[0] != rows.rows or state.shape[1] > CONV_MAX_TAPS - 1:
        raise AlofaError("shape_mismatch", "the kept rows do not fit", f"state={tuple(state.shape)} x={tuple(x.shape)} rows={rows.rows}")
    rows.fits("state", state)
    _call("alofa_conv_keep", _ptr(state), _ptr(x), _L(_rows("x", x)), _I(dtype_code(x)), _ptr(rows.slots), _ptr(rows.offsets), _I(rows.requests), _I(x.shape[1]),
          _I(state.shape[1]), _stream())


def ssd_operands(qf: torch.Tensor, kf: torch.Tensor, vf: torch.Tensor, decay: torch.Tensor, xbc: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor,
                 a_log: torch.Tensor, heads: int, groups: int, state: int, dv: int, exact: bool = False) -> None:
    """What ``linear_recurrence`` takes for a state-space mixer, as float32 rows: with dt = softplus(dt_raw + dt_bias) per row and head, decay = exp(-exp(a_log) dt) for every
    key channel of the head, kf = dt * B and qf = C of the head's group, vf = x. ``xbc`` [T, heads * dv + 2 * groups * state]: x, B, C side by side."""
    T = xbc.shape[0]
    for n, t, w in (("qf", qf, heads * state), ("kf", kf, heads * state), ("decay", decay, heads * state), ("vf", vf, heads * dv)):
        _gpu(n, t, torch.float32, 2), _contig(n, t)
        if tuple(t.shape) != (T, w):
            raise AlofaError("shape_mismatch", "the float operands do not fit", f"operand={n} shape={tuple(t.shape)} rows={T} width={w}")
    _gpu("xbc", xbc, None, 2), _gpu("dt_raw", dt_raw, xbc.dtype, 2), _gpu("dt_bias", dt_bias, torch.float32, 1), _gpu("a_log", a_log, torch.float32, 1)
    _contig("dt_bias", dt_bias), _contig("a_log", a_log)
    if xbc.shape[1] != heads * dv + 2 * groups * state or tuple(dt_raw.shape) != (T, heads) or dt_bias.shape[0] != heads or a_log.shape[0] != heads or heads % groups:
        raise AlofaError("shape_mismatch", "the rows do not fit", f"xbc={tuple(xbc.shape)} dt={tuple(dt_raw.shape)} heads={heads} groups={groups} state={state} dv={dv}")
    _call("alofa_ssd_operands", _ptr(qf), _ptr(kf), _ptr(vf), _ptr(decay), _ptr(xbc), _L(_rows("xbc", xbc)), _ptr(dt_raw), _L(_rows("dt_raw", dt_raw)), _I(dtype_code(xbc)),
          _ptr(dt_bias), _ptr(a_log), _L(T), _I(heads), _I(groups), _I(state), _I(dv), _I(int(exact)), _stream())


def ssd_finish(out: torch.Tensor, o: torch.Tensor, x: torch.Tensor, z: torch.Tensor, skip: torch.Tensor, weight: torch.Tensor, heads: int, dv: int, norm_parts: int,
               eps: float, exact: bool = False, parts: int = 1) -> None:
    """out = rms_parts((o + skip[head] * x) * silu(z)) * weight: the read-outs ``o`` float32 [T, heads * dv] (or [P, T, heads * dv], the first ``parts`` added), the
    values ``x`` and gates ``z`` [T, heads * dv] rows (strides allowed), ``skip`` float32 [heads], the row normed in ``norm_parts`` equal parts, ``weight`` float32 [heads * dv]."""
    _gpu("out", out, None, 2), _gpu("o", o, torch.float32), _contig("o", o), _gpu("x", x, out.dtype, 2), _gpu("z", z, out.dtype, 2)
    _gpu("skip", skip, torch.float32, 1), _gpu("weight", weight, torch.float32, 1), _contig("skip", skip), _contig("weight", weight)
    part_stride = 0
    if o.dim() == 3:
        if not 1 <= parts <= o.shape[0]:
            raise AlofaError("shape_mismatch", "more parts than the read-outs have room for", f"o={tuple(o.shape)} parts={parts}")
        part_stride, o = o.stride(0), o[0]
    elif o.dim() != 2 or parts != 1:
        raise AlofaError("shape_mismatch", "read-outs are [T, heads * dv] or parts of that", f"o={tuple(o.shape)} parts={parts}")
    T, inner = o.shape[0], heads * dv
    if o.shape[1] != inner or any(tuple(t.shape) != (T, inner) for t in (out, x, z)) or skip.shape[0] != heads or weight.shape[0] != inner or norm_parts <= 0 or inner % norm_parts:
        raise AlofaError("shape_mismatch", "the rows do not fit", f"out={tuple(out.shape)} o={tuple(o.shape)} x={tuple(x.shape)} z={tuple(z.shape)} heads={heads} dv={dv} norm_parts={norm_parts}")
    _call("alofa_ssd_finish", _ptr(out), _L(_rows("out", out)), _ptr(o), _I(parts), _L(part_stride), _ptr(x), _L(_rows("x", x)), _ptr(z), _L(_rows("z", z)), _I(dtype_code(out)),
          _ptr(skip), _ptr(weight), _L(T), _I(heads), _I(dv), _I(norm_parts), _F(eps), _I(int(exact)), _stream())


def rms_pair_sum(out: torch.Tensor, a: torch.Tensor, wa: torch.Tensor, sa: float, b: torch.Tensor, wb: torch.Tensor, sb: float, eps: float, exact: bool = False) -> None:
    """out[t] = sa * a[t] / rms(a[t]) * wa + sb * b[t] / rms(b[t]) * wb, all float32 [T, h] (weights [h]); rms(x) = sqrt(mean(x^2) + eps). ``out`` may be ``a`` or ``b``."""
    for n, t in (("out", out), ("a", a), ("b", b)):
        _gpu(n, t, torch.float32, 2), _contig(n, t)
    _gpu("wa", wa, torch.float32, 1), _gpu("wb", wb, torch.float32, 1), _contig("wa", wa), _contig("wb", wb)
    T, h = out.shape
    if a.shape != out.shape or b.shape != out.shape or wa.shape[0] != h or wb.shape[0] != h:
        raise AlofaError("shape_mismatch", "two branches of the output's shape, one weight per channel each", f"out={tuple(out.shape)} a={tuple(a.shape)} b={tuple(b.shape)}")
    _call("alofa_rms_pair_sum", _ptr(out), _ptr(a), _ptr(wa), _F(sa), _ptr(b), _ptr(wb), _F(sb), _L(T), _I(h), _F(eps), _I(int(exact)), _stream())


def span_attention_fast(d: int, block_size: int, dtype) -> bool:
    """Whether ``span_attention_mfma`` takes heads of d channels over pages of ``block_size`` tokens in this dtype."""
    return dtype is torch.bfloat16 and d % 16 == 0 and 16 <= d <= MAX_HEAD_DIM and block_size >= MIN_FAST_PAGE and block_size & (block_size - 1) == 0


def span_attention_mfma(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor, tiles: Optional[torch.Tensor],
                        req_of_token: Optional[torch.Tensor], positions: torch.Tensor, heads: int, kv_heads: int, d: int, window: Optional[int], scale: float,
                        pooled: Optional[tuple] = None, bias: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                        gate_kind: int = GATE_NONE, dv_true: Optional[int] = None) -> None:
    """``span_attention`` on the matrix cores, bfloat16: heads of d channels for keys and values alike (``dv_true`` of the value channels are the design's: the gate
    per channel is [T, heads * dv_true]). ``tiles`` int32 [n, 3]: (request, first row, rows <= 16) of every run of rows that a wavefront serves per head; None: every
    row is a run of its own (of request ``req_of_token[row]``, or of request ``row`` without it)."""
    _gpu("out", out, torch.bfloat16, 2), _gpu("q", q, torch.bfloat16, 2), _gpu("k_cache", k_cache, torch.bfloat16, 4), _gpu("v_cache", v_cache, torch.bfloat16, 4)
    _contig("k_cache", k_cache), _contig("v_cache", v_cache), _gpu("block_table", block_table, torch.int32, 2), _contig("block_table", block_table)
    _gpu("positions", positions, torch.int32, 1), _contig("positions", positions)
    T, block = q.shape[0], k_cache.shape[2]
    dv_true = d if dv_true is None else int(dv_true)
    if (tuple(q.shape) != (T, heads * d) or tuple(out.shape) != (T, heads * d) or tuple(k_cache.shape[1:]) != (kv_heads, block, d)
            or tuple(v_cache.shape) != (k_cache.shape[0], kv_heads, d, block) or positions.shape[0] != T or not span_attention_fast(d, block, q.dtype)):
        raise AlofaError("shape_mismatch", "attention operands do not fit the matrix-core kernel", f"out={tuple(out.shape)} q={tuple(q.shape)} k={tuple(k_cache.shape)} v={tuple(v_cache.shape)} heads={heads} kv_heads={kv_heads} d={d}")
    pk = pv = pool_table = None
    pool = places = 0
    if pooled is not None:
        pk, pv, pool_table, pool = pooled
        places = _pooled_operands(pk, pv, pool_table, k_cache, kv_heads, d, d, pool)
        if not window:
            raise AlofaError("invalid_argument", "pooled blocks lie behind a window")
    n_tiles = T
    if tiles is not None:
        _gpu("tiles", tiles, torch.int32, 2), _contig("tiles", tiles)
        if tiles.shape[1] != 3:
            raise AlofaError("shape_mismatch", "tiles are [n, 3]", f"tiles={tuple(tiles.shape)}")
        n_tiles = tiles.shape[0]
    elif req_of_token is not None:
        _gpu("req_of_token", req_of_token, torch.int32, 1), _contig("req_of_token", req_of_token)
    elif block_table.shape[0] < T or (pool_table is not None and pool_table.shape[0] < T):
        raise AlofaError("shape_mismatch", "without a request per row every row is a request of its own", f"rows={T} tables={block_table.shape[0]}")
    if bias is not None:
        _gpu("bias", bias, torch.float32, 2), _contig("bias", bias)
        if bias.shape[0] != heads or bias.shape[1] < 1:
            raise AlofaError("shape_mismatch", "the bias is [heads, distances]", f"bias={tuple(bias.shape)}")
    if sink is not None:
        _gpu("sink", sink, torch.float32, 1), _contig("sink", sink)
        if sink.shape[0] != heads:
            raise AlofaError("shape_mismatch", "one sink per head", f"sink={tuple(sink.shape)}")
    if gate_kind != GATE_NONE:
        _gpu("gate", gate, torch.bfloat16, 2)
        if tuple(gate.shape) != (T, heads * dv_true if gate_kind == GATE_CHANNEL else heads):
            raise AlofaError("shape_mismatch", "the gate does not fit its kind", f"gate={tuple(gate.shape)} kind={gate_kind}")
    _call("alofa_span_attention_mfma", _ptr(out), _L(_rows("out", out)), _ptr(q), _L(_rows("q", q)), _ptr(k_cache), _ptr(v_cache), _ptr(pk), _ptr(pv), _ptr(tiles), _I(n_tiles),
          _ptr(block_table), _I(block_table.shape[1]), _ptr(pool_table), _I(pool_table.shape[1] if pool_table is not None else 0), _ptr(req_of_token), _ptr(positions),
          _I(heads), _I(kv_heads), _I(d), _I(dv_true), _I(block), _I(int(window or 0)), _I(int(pool)), _I(places), _F(scale), _ptr(bias),
          _I(bias.shape[1] if bias is not None else 0), _ptr(sink), _ptr(gate if gate_kind != GATE_NONE else None),
          _L(_rows("gate", gate) if gate_kind != GATE_NONE else 0), _I(gate_kind), _stream())


def rms_pair_add_norm(residual: torch.Tensor, a: torch.Tensor, wa: torch.Tensor, sa: float, b: torch.Tensor, wb: torch.Tensor, sb: float, scale: Optional[torch.Tensor],
                      eps: float, exact: bool = False, then_norm: Optional[tuple] = None) -> None:
    """residual[t, c] += scale[c] * (sa * a[t] / rms(a[t]) * wa + sb * b[t] / rms(b[t]) * wb)[c] (``scale`` None: ones); with ``then_norm`` = (weight, eps, rows) the same
    launch leaves rows[t] = rmsnorm(residual[t]) * weight."""
    for n, t in (("residual", residual), ("a", a), ("b", b)):
        _gpu(n, t, torch.float32, 2), _contig(n, t)
    _gpu("wa", wa, torch.float32, 1), _gpu("wb", wb, torch.float32, 1), _contig("wa", wa), _contig("wb", wb)
    T, h = residual.shape
    if a.shape != residual.shape or b.shape != residual.shape or wa.shape[0] != h or wb.shape[0] != h:
        raise AlofaError("shape_mismatch", "two branches of the stream's shape, one weight per channel each", f"residual={tuple(residual.shape)} a={tuple(a.shape)} b={tuple(b.shape)}")
    if scale is not None:
        _gpu("scale", scale, torch.float32, 1), _contig("scale", scale)
        if scale.shape[0] != h:
            raise AlofaError("shape_mismatch", "one factor per channel", f"scale={tuple(scale.shape)}")
    nw = rows = None
    norm_eps = 0.0
    if then_norm is not None:
        nw, norm_eps, rows = then_norm
        _gpu("norm weight", nw, torch.float32, 1), _contig("norm weight", nw), _gpu("normed rows", rows, None, 2), _contig("normed rows", rows)
        if nw.shape[0] != h or rows.shape != residual.shape:
            raise AlofaError("shape_mismatch", "the norm behind the sum does not fit", f"weight={tuple(nw.shape)} rows={tuple(rows.shape)}")
    _call("alofa_rms_pair_add_norm", _ptr(residual), _ptr(a), _ptr(wa), _F(sa), _ptr(b), _ptr(wb), _F(sb), _ptr(scale), _L(T), _I(h), _F(eps), _ptr(rows),
          _I(dtype_code(rows) if rows is not None else F32), _ptr(nw), _F(norm_eps), _I(int(exact)), _stream())


def ssd_step(xbc: torch.Tensor, raw: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor], rows: RowsOfRequests, qf: torch.Tensor,
             kf: torch.Tensor, vf: torch.Tensor, decay: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, heads: int, groups: int,
             n_state: int, dv: int, exact: bool = False) -> None:
    """``conv_bias_act`` (with silu) and ``conv_keep`` in one launch, then ``ssd_operands``, for a step in which every request brings one row."""
    T, width = raw.shape
    taps = w.shape[1]
    _gpu("xbc", xbc, raw.dtype, 2), _gpu("raw", raw, None, 2), _gpu("w", w, torch.float32, 2), _contig("w", w)
    if rows.offsets is not None or rows.rows != T or tuple(xbc.shape) != (T, width) or width != heads * dv + 2 * groups * n_state or w.shape[0] != width or not 1 <= taps <= CONV_MAX_TAPS:
        raise AlofaError("shape_mismatch", "one row per request, rows of x, B, C side by side", f"raw={tuple(raw.shape)} xbc={tuple(xbc.shape)} w={tuple(w.shape)} heads={heads} groups={groups}")
    if taps > 1:
        _gpu("state", state, raw.dtype, 3), _contig("state", state)
        if tuple(state.shape[1:]) != (taps - 1, width):
            raise AlofaError("shape_mismatch", "the convolution's state does not fit", f"state={tuple(state.shape)}")
        rows.fits("state", state)
    if bias is not None:
        _gpu("bias", bias, torch.float32, 1), _contig("bias", bias)
    for n, t, wd in (("qf", qf, heads * n_state), ("kf", kf, heads * n_state), ("decay", decay, heads * n_state), ("vf", vf, heads * dv)):
        _gpu(n, t, torch.float32, 2), _contig(n, t)
        if tuple(t.shape) != (T, wd):
            raise AlofaError("shape_mismatch", "the float operands do not fit", f"operand={n} shape={tuple(t.shape)}")
    _gpu("dt_raw", dt_raw, raw.dtype, 2), _gpu("dt_bias", dt_bias, torch.float32, 1), _gpu("a_log", a_log, torch.float32, 1), _contig("dt_bias", dt_bias), _contig("a_log", a_log)
    if tuple(dt_raw.shape) != (T, heads) or dt_bias.shape[0] != heads or a_log.shape[0] != heads or (bias is not None and bias.shape[0] != width):
        raise AlofaError("shape_mismatch", "one step size, bias and rate per head", f"dt={tuple(dt_raw.shape)}")
    _call("alofa_ssd_step", _ptr(xbc), _L(_rows("xbc", xbc)), _ptr(raw), _L(_rows("raw", raw)), _I(dtype_code(raw)), _ptr(w), _ptr(bias), _ptr(state if taps > 1 else None),
          _ptr(rows.slots), _I(taps), _ptr(qf), _ptr(kf), _ptr(vf), _ptr(decay), _ptr(dt_raw), _L(_rows("dt_raw", dt_raw)), _ptr(dt_bias), _ptr(a_log), _L(T), _I(heads),
          _I(groups), _I(n_state), _I(dv), _I(int(exact)), _stream())
