"""Python faces of the HIP kernels.

Every function checks on the host that the operands are on the GPU, contiguous, of the
expected type and of shapes that fit what the kernel and its grid assume, and only then
launches on torch's current stream.  Nothing here falls back to another implementation: a
missing library or a refused size raises.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Iterable, Optional, Tuple

import torch

from .. import log
from .device import ARCH, COMPUTE_UNITS, N_XCD
from .library import KernelModule, Variant, load_module

P = ctypes.c_void_p
I = ctypes.c_int
F = ctypes.c_float
LL = ctypes.c_longlong

DT_F32, DT_BF16 = 0, 1
_DT = {torch.float32: DT_F32, torch.bfloat16: DT_BF16}

ROPE_NONE, ROPE_SPLIT_HALF, ROPE_CONSECUTIVE = 0, 1, 2

# The matrix-core attention module is compiled per head size, when a model with that head size
# first runs; these sizes are compiled ahead by build_all().
MFMA_HEAD_DIMS_PREBUILT = (16, 32, 64, 128)
MFMA_MAX_HEAD_DIM = 128
# The tile kernel's two tilings: 1 = tiles of 64 rows (four waves of 16), which give twice as many workgroups for
# short portions; 2 = tiles of 128 rows, in which every key and value fetched serves twice as many rows.  At head
# size 128 the tall tiles are the kernel of attn_prefill.hip (eight waves of 16 rows, tiles loaded straight into
# LDS), at the other head sizes attn_mfma.hip's with two query tiles per wave.
TILE_QTS = (1, 2)
# (that kernel is written in gfx950's own instructions, loads into LDS of 16 bytes a lane among them; built for anything
# else, the tall tiles of head size 128 are attn_mfma.hip's as well)
DIRECT_TILE_HEAD_DIM = 128 if ARCH == "gfx950" else None


class KernelError(RuntimeError):
    pass


def module_variants() -> Iterable[Tuple[str, Variant]]:
    yield ("cache_manager", ())       # host code: the cache's bookkeeping
    yield ("core", ())
    yield ("gemm_f32", ())
    yield ("attn_plain", ())
    yield ("sampling", ())
    yield ("gemm_bf16", ())
    yield ("gemm_wide", ())
    yield ("ceilings", ())            # measurement only: what the memory gives a kernel that just reads
    for d in MFMA_HEAD_DIMS_PREBUILT:
        for qt in TILE_QTS:
            yield _tile_module(d, qt)[:2]


def _tile_module(head_dim: int, qt: int):
    """(module, variant, entry point, the function that says its tile rows) of the tile kernel for a tiling."""
    if qt == 2 and head_dim == DIRECT_TILE_HEAD_DIM:
        return "attn_prefill", (("HEAD_DIM", head_dim),), "ifx_attn_prefill", "ifx_attn_prefill_tile_rows"
    return "attn_mfma", (("HEAD_DIM", head_dim), ("TILE_QT", qt)), "ifx_attn_tiles", "ifx_attn_tile_rows"


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported element type {t.dtype} (float32 or bfloat16)") from None


def _check(t: torch.Tensor, name: str, shape=None, dtype=None) -> None:
    # on every launch: written for the case that nothing is wrong
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous()):
        if not isinstance(t, torch.Tensor):
            raise KernelError(f"{name}: not a tensor")
        if not t.is_cuda:
            raise KernelError(f"{name}: tensor is on {t.device}; the kernels run on the GPU only")
        raise KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: element type {t.dtype}, expected {dtype}")
    if shape is not None:
        ts = t.shape
        ok = len(shape) == len(ts)
        if ok:
            for want, got in zip(shape, ts):
                if want is not None and want != got:
                    ok = False
                    break
        if not ok:
            raise KernelError(f"{name}: shape {tuple(ts)}, expected {tuple(shape)}")


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def _stream() -> int:
    # torch's current stream as a raw handle; the accessor that skips building a Stream object is used
    # where this torch has it (it is called once per launch)
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _call(mod: KernelModule, fname: str, argtypes, *args) -> None:
    rc = mod.fn(fname, argtypes)(*args)
    if rc != 0:
        raise KernelError(f"{fname}: {mod.last_error()} (code {rc})")


# ----------------------------------------------------------------------------------------
def embedding(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """float32 [T, H] rows of ``table`` [V, H] named by int32 ``ids`` [T] (ids are checked by the caller)."""
    _check(ids, "ids", (None,), torch.int32)
    _check(table, "table", (None, None))
    T, H = ids.shape[0], table.shape[1]
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _call(load_module("core"), "ifx_embedding", (P, P, I, P, I, I, P),
          ids.data_ptr(), table.data_ptr(), _dt(table), out.data_ptr(), T, H, _stream())
    return out


def embedding_scaled(ids: torch.Tensor, table: torch.Tensor, norm_weight: torch.Tensor, eps: float):
    """``embedding`` for up to 16 tokens that also prepares the RMS norm (bfloat16 weight ``norm_weight`` [H]) which
    reads the stream first: returns (the float32 stream [T, H], that norm's rows up to the factor per row)."""
    _check(ids, "ids", (None,), torch.int32)
    _check(table, "table", (None, None))
    T, H = ids.shape[0], table.shape[1]
    _check(norm_weight, "norm_weight", (H,), torch.bfloat16)
    if T > 16:
        raise KernelError(f"embedding_scaled: {T} rows (at most 16)")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    rows = torch.empty((T, H), dtype=torch.bfloat16, device=table.device)
    pieces = torch.empty((-(-H // 4096), 16), dtype=torch.float32, device=table.device)
    _call(load_module("core"), "ifx_embedding_norm", (P, P, I, P, P, P, P, I, I, P),
          ids.data_ptr(), table.data_ptr(), _dt(table), norm_weight.data_ptr(), out.data_ptr(), rows.data_ptr(),
          pieces.data_ptr(), T, H, _stream())
    return out, ScaledRows(rows, pieces, H, eps, norm_weight)


def add_rmsnorm(residual: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``residual`` [T, H] float32 (+= ``delta`` in place when given and no ``rows``), then RMSNorm.

    With ``rows`` (int32 [R]) only those rows are normalised, into [R, H], and the residual is
    left untouched.
    """
    _check(residual, "residual", (None, None), torch.float32)
    T, H = residual.shape
    _check(weight, "weight", (H,))
    n_slices = 1
    if isinstance(delta, SliceSums):               # partial sums: the kernel adds them in slice order
        _check(delta.parts, "delta", (None, T, H), torch.float32)
        n_slices, delta = delta.parts.shape[0], delta.parts
    elif delta is not None:
        _check(delta, "delta", (T, H))
    n = T
    if rows is not None:
        _check(rows, "rows", (None,), torch.int32)
        n = rows.shape[0]
    out = torch.empty((n, H), dtype=out_dtype, device=residual.device)
    _call(load_module("core"), "ifx_add_rmsnorm", (P, P, I, P, I, P, I, P, I, I, F, I, I, LL, P),
          residual.data_ptr(), _ptr(delta), _dt(delta) if delta is not None else 0, weight.data_ptr(),
          _dt(weight), out.data_ptr(), _DT[out_dtype], _ptr(rows), n, H, float(eps),
          1 if (delta is not None and rows is None) else 0, n_slices, T * H, _stream())
    return out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor):
    """cos and sin [T, pairs] of float(position) * inv_freq, computed in float."""
    _check(positions, "positions", (None,), torch.int32)
    _check(inv_freq, "inv_freq", (None,), torch.float32)
    T, n = positions.shape[0], inv_freq.shape[0]
    cs = torch.empty((T, n), dtype=torch.float32, device=positions.device)
    sn = torch.empty((T, n), dtype=torch.float32, device=positions.device)
    _call(load_module("core"), "ifx_rope_table", (P, P, P, P, I, I, P),
          positions.data_ptr(), inv_freq.data_ptr(), cs.data_ptr(), sn.data_ptr(), T, n, _stream())
    return cs, sn


def rope_append(qkv: torch.Tensor, bias: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], rope_style: int,
                rotary_dim: int, n_heads: int, n_kv_heads: int, head_dim: int,
                k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], page_size: int,
                v_head_dim: Optional[int] = None) -> torch.Tensor:
    """Bias, rotation and cache write of one step's projections; returns q [T, n_heads, head_dim].

    ``qkv`` is [T, (n_heads + n_kv_heads) head_dim + n_kv_heads v_head_dim] when the keys and values are
    written (``slots`` int32 [T] = page * page_size + offset; ``v_head_dim`` None: as wide as the keys), or
    [T, n_heads head_dim] with ``n_kv_heads`` = 0 for a mixer that only reads another's cache.  ``cos`` / ``sin``
    are the step's rotation table [T, rotary_dim / 2] (from rope_table).
    """
    T = qkv.shape[0]
    dv = head_dim if v_head_dim is None else int(v_head_dim)
    width = (n_heads + n_kv_heads) * head_dim + n_kv_heads * dv
    n_slices = 1
    if isinstance(qkv, SliceSums):                  # partial sums: the kernel adds them in slice order
        _check(qkv.parts, "qkv", (None, T, width), torch.float32)
        n_slices, dtype, qkv = qkv.parts.shape[0], qkv.dtype, qkv.parts
    else:
        _check(qkv, "qkv", (T, width))
        dtype = qkv.dtype
    if bias is not None:
        _check(bias, "bias", (width,))
    if rope_style != ROPE_NONE:
        _check(cos, "cos", (T, rotary_dim // 2), torch.float32)
        _check(sin, "sin", (T, rotary_dim // 2), torch.float32)
    if slots is not None:
        _check(slots, "slots", (T,), torch.int32)
        _check(k_cache, "k_cache", (None, n_kv_heads, page_size, head_dim), dtype)
        _check(v_cache, "v_cache", (k_cache.shape[0], n_kv_heads, dv, page_size), dtype)
    elif n_kv_heads != 0:
        raise KernelError("rope_append: keys and values given but no slots to write them to")
    q = torch.empty((T, n_heads, head_dim), dtype=dtype, device=qkv.device)
    _call(load_module("core"), "ifx_rope_append", (P, I, P, I, P, P, P, I, I, I, I, I, I, I, P, P, P, I, LL, I, P),
          qkv.data_ptr(), _DT[dtype], _ptr(bias), _dt(bias) if bias is not None else 0, _ptr(slots),
          _ptr(cos) if rope_style != ROPE_NONE else 0, _ptr(sin) if rope_style != ROPE_NONE else 0, rope_style,
          rotary_dim, T, n_heads, n_kv_heads, head_dim, page_size, q.data_ptr(), _ptr(k_cache), _ptr(v_cache),
          n_slices, T * width, dv, _stream())
    return q


def swiglu(gate_up: torch.Tensor, interleaved: bool = False) -> torch.Tensor:
    """silu(gate) * up [T, I] from [T, 2I] laid out [gate | up] or, interleaved, gate_0, up_0, gate_1, ..."""
    _check(gate_up, "gate_up", (None, None))
    T, two_i = gate_up.shape
    if two_i % 2:
        raise KernelError("swiglu: odd width")
    out = torch.empty((T, two_i // 2), dtype=gate_up.dtype, device=gate_up.device)
    _call(load_module("core"), "ifx_swiglu", (P, P, I, I, I, I, P),
          gate_up.data_ptr(), out.data_ptr(), _dt(gate_up), T, two_i // 2, 1 if interleaved else 0, _stream())
    return out


# ----------------------------------------------------------------------------------------
def gemm_f32(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
             out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """x [M, K] (float32 or bfloat16) times float32 ``weight`` [N, K] transposed, true 32-bit math."""
    _check(x, "x", (None, None))
    M, K = x.shape
    _check(weight, "weight", (None, K), torch.float32)
    N = weight.shape[0]
    if bias is not None:
        _check(bias, "bias", (N,), torch.float32)
    out_dtype = out_dtype or x.dtype
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _call(load_module("gemm_f32"), "ifx_gemm_f32", (P, I, P, P, P, I, I, I, I, P),
          x.data_ptr(), _dt(x), weight.data_ptr(), _ptr(bias), out.data_ptr(), _DT[out_dtype], M, N, K, _stream())
    return out


SKINNY_MAX_M = 64
WIDE_MAX_M = 128           # rows the product that shares x through LDS takes at most ...
WIDE_MANY_ROWS_MAX_N = 16384   # ... beyond 64 of them only for weights of up to this many rows (see _small_m_kernel)


def enable_library_gemm_tuning(max_ms_per_shape: int = 300, filename: Optional[str] = None) -> None:
    """Let the library pick, by timing, the fastest of its kernels for every matrix-product shape it
    meets (torch's TunableOp over hipBLASLt and rocBLAS).  The first product of a shape then takes
    up to ``max_ms_per_shape`` longer; worth it when shapes repeat (a fixed prefill portion, a steady
    decode batch), not for one-off shapes, so it is off unless asked for."""
    import torch.cuda.tunable as tunable
    tunable.enable(True)
    tunable.tuning_enable(True)
    tunable.set_max_tuning_duration(int(max_ms_per_shape))
    if not filename:
        import os
        from .library import _fallback_dir
        # this user's private folder under the temporary directory (refused if somebody else made it or may write it)
        filename = os.path.join(_fallback_dir(create=True), "tunableop.csv")
    tunable.set_filename(filename)     # choices are kept there and reused by later runs


def pause_library_gemm_tuning(paused: bool) -> None:
    """While paused, shapes already timed keep their chosen kernel and new shapes take the default."""
    import torch.cuda.tunable as tunable
    if tunable.is_enabled():
        tunable.tuning_enable(not paused)


def tile_weights(weight: torch.Tensor, order: Optional[torch.Tensor] = None, tile_rows: int = 16) -> torch.Tensor:
    """The tiled form of a bfloat16 ``weight`` [N, K] that the weight-streaming product reads in
    contiguous runs: a flat tensor of ceil(N / tile_rows) row tiles of ``tile_rows`` rows (even, 8 to 16) by
    cols64(K) k-values (zeros in the padding).  ``order`` (int32, a permutation of the row tiles, tiles of 16
    only): tile t of the copy is row tile order[t] of the weight."""
    _check(weight, "weight", (None, None), torch.bfloat16)
    N, K = weight.shape
    if K % 8:
        raise KernelError(f"tile_weights: K={K} must be a multiple of 8")
    if tile_rows not in TILE_ROWS or (order is not None and tile_rows != 16):
        raise KernelError(f"tile_weights: {tile_rows} rows to a tile (one of {TILE_ROWS}; 16 with a tile order)")
    mod = load_module("gemm_bf16")
    n_tiles = -(-N // tile_rows)
    if order is not None:
        _check(order, "order", (n_tiles,), torch.int32)
        if sorted(order.tolist()) != list(range(n_tiles)):
            raise KernelError("tile_weights: order is not a permutation of the weight's row tiles")
    out = torch.empty((_tiled_size(N, K, tile_rows),), dtype=torch.bfloat16, device=weight.device)
    _call(mod, "ifx_tile_weights", (P, P, I, I, P, I, P), weight.data_ptr(), out.data_ptr(), N, K, _ptr(order), tile_rows, _stream())
    return out


TILE_ROWS = (8, 10, 12, 14, 16)      # rows a tile of the copy may hold


def _tiled_size(N: int, K: int, tile_rows: int) -> int:
    return -(-N // tile_rows) * tile_rows * (-(-K // 64) * 64)


def choose_tile_rows(N: int) -> int:
    """Rows to a tile of a weight's streamed copy.  A workgroup of the products for few rows of x owns whole row
    tiles, and a compute unit can have only so many bytes on their way: a weight of 3,584 rows in tiles of 16
    gives 224 of the 256 units a tile and takes as long as one of 4,096 rows.  Where 16-row tiles leave units
    without one, the tiles are made as low as still gives every unit at most one (3,584 rows: 14; 2,048: 8).
    Measured at 1-64 rows of x: 3,584 x 18,944 takes 24.8 us instead of 25.9 at 8 rows, 2,048 x 11,008 16.3
    instead of 20.1 at 16 rows; weights with more tiles than units gain nothing from lower tiles or lose."""
    if N > 16 * COMPUTE_UNITS:
        return 16
    rows = -(-N // COMPUTE_UNITS)
    return min(16, max(8, rows + rows % 2))


class LinearWeight:
    """A projection's weight as the products want it: ``rows`` [N, K] as the model file has it, and for
    bfloat16 weights ``tiled``, the copy that products with few rows of x (decoding) stream from.  The
    copy doubles the weight's memory; it is left out when ``decode_weight_copy`` is off or when the
    card has no room for it, and products with few rows then read ``rows``."""

    __slots__ = ("rows", "tiled", "order", "tile_rows")

    def __init__(self, rows: torch.Tensor, tiled: Optional[torch.Tensor] = None, order: Optional[torch.Tensor] = None,
                 tile_rows: int = 16):
        # order: the copy's row-tile order, tile_rows: the rows to a tile of the copy (see tile_weights)
        self.rows, self.tiled, self.order, self.tile_rows = rows, tiled, order, tile_rows

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype


# Whether prepare_linear makes tiled copies, and how much memory it leaves free when it does.
decode_weight_copy = True
DECODE_COPY_RESERVE_BYTES = 8 << 30


def prepare_linear(weight: torch.Tensor, order: Optional[torch.Tensor] = None, tile_rows: int = 0) -> LinearWeight:
    """Wrap a projection's weight for ``linear`` / ``linear_swiglu``, with the tiled copy if wanted and possible
    (its row tiles in ``order``, if given, and then of 16 rows; else of ``tile_rows`` rows, 0: ``choose_tile_rows``)."""
    tiled = None
    if order is not None:
        tile_rows = 16
    elif tile_rows == 0:
        tile_rows = choose_tile_rows(weight.shape[0]) if weight.dim() == 2 else 16
    if (decode_weight_copy and weight.is_cuda and weight.dtype == torch.bfloat16 and weight.dim() == 2
            and weight.shape[1] % 8 == 0):
        free, _ = torch.cuda.mem_get_info(weight.device)
        if free >= weight.numel() * 2 + DECODE_COPY_RESERVE_BYTES:
            tiled = tile_weights(weight.contiguous(), order, tile_rows)
        else:
            log.warn("kernels", f"no room for the decode copy of a {tuple(weight.shape)} weight "
                                f"({free / 2**30:.1f} GiB free): decoding reads the plain rows")
    return LinearWeight(weight, tiled, order if tiled is not None else None, tile_rows if tiled is not None else 16)


class ScaledRows:
    """Rows of a normalised activation up to one factor per row: row t stands for
    ``rows[t] * rsqrt(sum(pieces[:, t]) / width + eps)``.  ``rows`` is bfloat16 [T <= 16, width] (the stream times
    the norm's weight), ``pieces`` float32 [n, 16] (sums of squares of the stream over runs of columns, one run
    per row tile of the product that made them; rows past T hold zeros).  A weight-streaming product that takes these multiplies its sums by the factor, which
    saves the norm a kernel of its own; ``linear_into_stream`` makes them."""

    __slots__ = ("rows", "pieces", "width", "eps", "norm_weight")

    def __init__(self, rows: torch.Tensor, pieces: torch.Tensor, width: int, eps: float,
                 norm_weight: Optional[torch.Tensor] = None):
        self.rows, self.pieces, self.width, self.eps = rows, pieces, int(width), float(eps)
        self.norm_weight = norm_weight      # the weight the rows were multiplied by: whose norm they stand for

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype


class SliceSums:
    """A product left as partial sums over slices of K: it stands for ``parts.sum(0)`` (float32 [S, M, N], added in
    slice order).  ``add_rmsnorm`` takes it as its delta and ``rope_append`` as its q/k/v, which saves the kernel
    that would add the slices; ``sum()`` adds them for everyone else."""

    __slots__ = ("parts", "dtype")

    def __init__(self, parts: torch.Tensor, dtype: torch.dtype):
        self.parts, self.dtype = parts, dtype      # dtype: what the sum would be rounded to

    @property
    def shape(self):
        return self.parts.shape[1:]

    def sum(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        S, M, N = self.parts.shape
        out = torch.empty((M, N), dtype=dtype or self.dtype, device=self.parts.device)
        _call(load_module("gemm_wide"), "ifx_sum_slices", (P, P, I, I, LL, P),
              self.parts.data_ptr(), out.data_ptr(), _DT[out.dtype], S, M * N, _stream())
        return out


def _scale_args(x):
    """(rows, the four row-factor arguments of the kernels) of a tensor or a ``ScaledRows``."""
    if isinstance(x, ScaledRows):
        _check(x.pieces, "pieces", (None, 16), torch.float32)
        if not 1 <= x.pieces.shape[0] <= x.width:
            raise KernelError(f"scaled rows: {x.pieces.shape[0]} pieces for a width of {x.width}")
        _check(x.rows, "rows", (None, x.width), torch.bfloat16)
        if x.rows.shape[0] > 16:
            raise KernelError(f"scaled rows: {x.rows.shape[0]} rows, at most 16")
        return x.rows, (x.pieces.data_ptr(), x.pieces.shape[0], float(x.width), x.eps)
    return x, (0, 0, 0.0, 0.0)


def takes_scaled_rows(n_rows: int, weight) -> bool:
    """Whether ``linear`` / ``linear_swiglu`` / ``qkv_rope_append`` take ``ScaledRows`` of ``n_rows`` rows with this weight."""
    if not isinstance(weight, LinearWeight):
        return False
    N, K = weight.rows.shape
    return (weight.rows.dtype == torch.bfloat16 and n_rows <= 16
            and _small_m_kernel(n_rows, N, K, weight.tiled is not None) in ("skinny", "wide"))


def adds_into_stream(n_rows: int, weight, norm_weight: torch.Tensor) -> bool:
    """Whether ``linear_into_stream`` takes this shape."""
    if not isinstance(weight, LinearWeight) or weight.order is not None:
        return False
    N, K = weight.rows.shape
    return (weight.rows.dtype == torch.bfloat16 and norm_weight.dtype == torch.bfloat16 and n_rows <= 16 and N % 4 == 0
            and _small_m_kernel(n_rows, N, K, weight.tiled is not None) == "skinny")


def linear_into_stream(x: torch.Tensor, weight: LinearWeight, stream: torch.Tensor, norm_weight: torch.Tensor,
                       eps: float) -> ScaledRows:
    """``stream`` [M <= 16, N] (float32) += x [M, K] W^T in place, as the product's epilogue, which also prepares
    the RMS norm that follows (weight ``norm_weight`` [N] bfloat16): returns its rows up to the factor per row."""
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    N = weight.rows.shape[0]
    if not adds_into_stream(M, weight, norm_weight) or weight.rows.shape[1] != K:
        raise KernelError(f"linear_into_stream: not for {M} rows times a {tuple(weight.rows.shape)} weight")
    _check(stream, "stream", (M, N), torch.float32)
    _check(norm_weight, "norm_weight", (N,), torch.bfloat16)
    rows = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    tile_rows = 16 if weight.tiled is None else weight.tile_rows
    pieces = torch.empty((-(-N // tile_rows), 16), dtype=torch.float32, device=x.device)    # one piece per row tile
    w = weight.rows if weight.tiled is None else weight.tiled
    _call(load_module("gemm_bf16"), "ifx_skinny_gemm", _SKINNY_ARGS,
          x.data_ptr(), w.data_ptr(), 0, DT_F32, M, N, K, 0, 0, 0, 2, 0 if weight.tiled is None else tile_rows, 0,
          0, 0, 0.0, 0.0, stream.data_ptr(), norm_weight.data_ptr(), rows.data_ptr(), pieces.data_ptr(), _stream())
    return ScaledRows(rows, pieces, N, eps, norm_weight)


_SKINNY_ARGS = (P, P, P, I, I, I, I, I, I, I, I, I, P, P, I, F, F, P, P, P, P, P)


def pair_tile_order(n_heads: int, head_dim: int) -> list:
    """Row-tile order of a projection whose rows are ``n_heads`` heads of ``head_dim`` (a multiple of 32) that
    puts the two halves of 16 split-half rotation pairs into consecutive tiles: for head h and j < d / 32,
    tiles h d/16 + j and h d/16 + j + d/32.  What ``qkv_rope_append`` expects of its tiled copy."""
    per, half = head_dim // 16, head_dim // 32
    return [h * per + j + s * half for h in range(n_heads) for j in range(half) for s in (0, 1)]


def qkv_rope_append(x: torch.Tensor, weight: LinearWeight, bias: Optional[torch.Tensor], slots: Optional[torch.Tensor],
                    cos: torch.Tensor, sin: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                    k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], page_size: int,
                    waves: int = 0, unroll: int = 0) -> torch.Tensor:
    """For up to 16 tokens: q, k, v = x W^T + bias from the pair-ordered tiled copy of the concatenated
    weight, q and k rotated (split-half pairs over the whole head, table cos/sin [M, d/2]), k and v written
    into the paged cache at ``slots``, q returned [M, nH, d] -- one kernel, the rotation and the cache
    write being the product's epilogue.  With ``slots`` None the weight holds the query rows only.
    ``x`` may be ``ScaledRows``."""
    x, scale = _scale_args(x)
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    heads = n_heads + (2 * n_kv_heads if slots is not None else 0)
    if weight.tiled is None or weight.order is None or tuple(weight.rows.shape) != (heads * head_dim, K):
        raise KernelError(f"qkv_rope_append: needs the pair-ordered tiled copy of a [{heads * head_dim}, {K}] weight")
    if M > 16 or head_dim % 32 or K % 8:
        raise KernelError(f"qkv_rope_append: M={M} must be <= 16, head_dim={head_dim} a multiple of 32, K={K} of 8")
    _check(cos, "cos", (M, head_dim // 2), torch.float32)
    _check(sin, "sin", (M, head_dim // 2), torch.float32)
    if bias is not None:
        _check(bias, "bias", (heads * head_dim,))
    if slots is not None:
        _check(slots, "slots", (M,), torch.int32)
        _check(k_cache, "k_cache", (None, n_kv_heads, page_size, head_dim), torch.bfloat16)
        _check(v_cache, "v_cache", (k_cache.shape[0], n_kv_heads, head_dim, page_size), torch.bfloat16)
    q = torch.empty((M, n_heads, head_dim), dtype=torch.bfloat16, device=x.device)
    _call(load_module("gemm_bf16"), "ifx_qkv_rope", (P, P, I, I, P, I, P, P, P, I, I, I, I, P, P, P, I, I, P, I, F, F, P),
          x.data_ptr(), weight.tiled.data_ptr(), M, K, _ptr(bias), _dt(bias) if bias is not None else 0, _ptr(slots),
          cos.data_ptr(), sin.data_ptr(), n_heads, n_kv_heads, head_dim, page_size, q.data_ptr(), _ptr(k_cache),
          _ptr(v_cache), waves, unroll, *scale, _stream())
    return q


def skinny_gemm(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                nt: int = 0, waves: int = 0, unroll: int = 0, swiglu_pairs: bool = False,
                tiled: Optional[torch.Tensor] = None, order: Optional[torch.Tensor] = None, tile_rows: int = 16) -> torch.Tensor:
    """bfloat16 x [M <= 64, K] times bfloat16 ``weight`` [N, K] transposed on the matrix cores, float
    accumulation, output bfloat16 or float32.  ``nt``, ``waves``, ``unroll`` = 0 lets the kernel choose.
    With ``swiglu_pairs`` the weight's rows alternate gate and up and the output is silu(gate) * up [M, N/2].
    With ``tiled`` (``tile_weights(weight, order, tile_rows)``) the kernel streams that copy instead of the rows.
    ``x`` may be ``ScaledRows``."""
    x, scale = _scale_args(x)
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    _check(weight, "weight", (None, K), torch.bfloat16)
    N = weight.shape[0]
    if tiled is not None:
        if tile_rows not in TILE_ROWS or (order is not None and tile_rows != 16):
            raise KernelError(f"skinny_gemm: {tile_rows} rows to a tile (one of {TILE_ROWS}; 16 with a tile order)")
        _check(tiled, "tiled", (_tiled_size(N, K, tile_rows),), torch.bfloat16)
    if M > SKINNY_MAX_M or K % 8:
        raise KernelError(f"skinny_gemm: M={M} must be <= {SKINNY_MAX_M} and K={K} a multiple of 8")
    if swiglu_pairs and N % 2:
        raise KernelError("skinny_gemm: gate/up pairs need an even number of weight rows")
    out = torch.empty((M, N // 2 if swiglu_pairs else N), dtype=out_dtype, device=x.device)
    if order is not None and (tiled is None or swiglu_pairs):
        raise KernelError("skinny_gemm: a tile order goes with a tiled copy and a plain product")
    _call(load_module("gemm_bf16"), "ifx_skinny_gemm", _SKINNY_ARGS,
          x.data_ptr(), (weight if tiled is None else tiled).data_ptr(), out.data_ptr(), _DT[out_dtype], M, N, K, nt, waves,
          unroll, 1 if swiglu_pairs else 0, 0 if tiled is None else tile_rows, _ptr(order), *scale, 0, 0, 0, 0, _stream())
    return out


def wide_gemm(x, weight: LinearWeight, out_dtype: torch.dtype = torch.bfloat16, waves: int = 0,
              slices: int = 0, swiglu_pairs: bool = False, keep_slices: bool = False):
    """bfloat16 x [M <= 128, K] times ``weight`` transposed from its tiled copy, x shared through LDS by the waves
    of a workgroup: the product for 17-64 rows, for 65-128 rows of weights with few rows, and for 9-16 rows of large
    tall weights.  ``waves`` (4-16 per workgroup, 8 beyond 64 rows; one tile of weight rows each) and ``slices`` of K
    (added in a fixed order): 0 lets the kernel choose.  With ``keep_slices`` a product of several slices comes back as
    ``SliceSums``.  ``x`` may be ``ScaledRows`` (up to 16 rows)."""
    x, scale = _scale_args(x)
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    N = weight.rows.shape[0]
    if weight.tiled is None or weight.rows.shape[1] != K or weight.rows.dtype != torch.bfloat16:
        raise KernelError(f"wide_gemm: needs the tiled copy of a bfloat16 [N, {K}] weight")
    if M > WIDE_MAX_M or K % 8:
        raise KernelError(f"wide_gemm: M={M} must be <= {WIDE_MAX_M} and K={K} a multiple of 8")
    if swiglu_pairs and (N % 2 or weight.order is not None):
        raise KernelError("wide_gemm: gate/up pairs need an even number of weight rows in their natural order")
    mod = load_module("gemm_wide")
    if _tiled_size(N, K, weight.tile_rows) != weight.tiled.numel():
        raise KernelError(f"wide_gemm: the copy is not that of a [{N}, {K}] weight in tiles of {weight.tile_rows} rows")
    plan = mod.fn("ifx_wide_gemm_plan", (I, I, I, I, I, I, I))(M, N, K, waves, slices, 1 if swiglu_pairs else 0, weight.tile_rows)
    n_waves, n_slices = plan // 256, plan % 256
    part = torch.empty((n_slices, M, N), dtype=torch.float32, device=x.device) if n_slices > 1 else None
    keep = keep_slices and n_slices > 1
    out = None if keep else torch.empty((M, N // 2 if swiglu_pairs else N), dtype=out_dtype, device=x.device)
    _call(mod, "ifx_wide_gemm", (P, P, P, I, P, I, I, I, I, I, I, P, I, P, I, F, F, P),
          x.data_ptr(), weight.tiled.data_ptr(), _ptr(out), _DT[out_dtype], _ptr(part), M, N, K, n_waves, n_slices,
          1 if swiglu_pairs else 0, _ptr(weight.order), weight.tile_rows, *scale, _stream())
    return SliceSums(part, out_dtype) if keep else out


def staged_gemm(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                slices: int = 0, unroll: int = 0, swiglu_pairs: bool = False) -> torch.Tensor:
    """The same product as skinny_gemm with x staged in LDS and shared by the waves of a workgroup
    (64 weight rows per workgroup, K cut into ``slices``; 0 lets the kernel choose)."""
    _check(x, "x", (None, None), torch.bfloat16)
    M, K = x.shape
    _check(weight, "weight", (None, K), torch.bfloat16)
    N = weight.shape[0]
    if M > SKINNY_MAX_M or K % 8:
        raise KernelError(f"staged_gemm: M={M} must be <= {SKINNY_MAX_M} and K={K} a multiple of 8")
    if swiglu_pairs and N % 2:
        raise KernelError("staged_gemm: gate/up pairs need an even number of weight rows")
    mod = load_module("gemm_bf16")
    n_slices = 1 if swiglu_pairs else mod.fn("ifx_staged_gemm_slices", (I, I, I, I))(M, N, K, slices)
    part = torch.empty((n_slices, M, N), dtype=torch.float32, device=x.device) if n_slices > 1 else None
    out = torch.empty((M, N // 2 if swiglu_pairs else N), dtype=out_dtype, device=x.device)
    _call(mod, "ifx_staged_gemm", (P, P, P, I, P, I, I, I, I, I, I, P),
          x.data_ptr(), weight.data_ptr(), out.data_ptr(), _DT[out_dtype], _ptr(part), M, N, K, slices, unroll,
          1 if swiglu_pairs else 0, _stream())
    return out


def linear(x: torch.Tensor, weight, out_dtype: Optional[torch.dtype] = None, keep_slices: bool = False):
    """x [M, K] times ``weight`` [N, K] transposed (a tensor or a ``LinearWeight``), chosen by the weight's
    type and by M.  With ``keep_slices`` the result may be ``SliceSums`` (the caller hands it to ``add_rmsnorm`` or
    ``rope_append``, or calls its ``sum()``).

    A float32 weight takes the true 32-bit kernel whatever the activation's type.  A bfloat16
    weight with bfloat16 activations takes the weight-streaming kernel for up to 64 rows and the
    library product with float accumulation beyond, as the reference does for every dense
    projection (runtime/backends/cuda/native/cublas_gemm.cpp:99-117).  float32 output (logits)
    always comes from float accumulators, never through a bfloat16 rounding.
    """
    tiled = order = None
    tile_rows = 16
    if isinstance(x, ScaledRows) and not takes_scaled_rows(x.shape[0], weight):
        raise KernelError(f"linear: scaled rows are not taken for {x.shape[0]} rows and this weight")
    if isinstance(weight, LinearWeight):
        weight, tiled, order, tile_rows = weight.rows, weight.tiled, weight.order, weight.tile_rows
    if weight.dtype == torch.float32:
        return gemm_f32(x, weight, None, out_dtype or x.dtype)
    if weight.dtype != torch.bfloat16 or x.dtype != torch.bfloat16:
        raise KernelError(f"linear: weight {weight.dtype} with activation {x.dtype} is not supported")
    _check(x if not isinstance(x, ScaledRows) else x.rows, "x", (None, weight.shape[1]))
    _check(weight, "weight", (None, None))
    out_dtype = out_dtype or torch.bfloat16
    M, K = x.shape
    kind = _small_m_kernel(M, weight.shape[0], K, tiled is not None)
    if kind == "skinny":
        return skinny_gemm(x, weight, out_dtype, tiled=tiled, order=order, tile_rows=tile_rows)
    if kind == "wide":
        return wide_gemm(x, LinearWeight(weight, tiled, order, tile_rows), out_dtype, keep_slices=keep_slices)
    if kind == "staged":
        return staged_gemm(x, weight, out_dtype)
    if out_dtype == torch.float32:
        return torch.mm(x, weight.t(), out_dtype=torch.float32)
    if keep_slices:
        S = library_k_slices(M, weight.shape[0], K)
        if S > 1 and not torch.cuda.is_current_stream_capturing():
            # K cut into S slices as one batched product of the library with float32 results: [S, M, N] partial sums
            xs = x.view(M, S, K // S).transpose(0, 1)
            ws = weight.view(weight.shape[0], S, K // S).permute(1, 2, 0)
            return SliceSums(torch.bmm(xs, ws, out_dtype=torch.float32), out_dtype)
    return torch.matmul(x, weight.t())


LIBRARY_SLICE_MIN_K = 2048      # k-values a slice of a library product keeps at least
LIBRARY_MAX_SLICES = 8


def library_k_slices(M: int, N: int, K: int) -> int:
    """Into how many slices of K a product that goes to the library is cut when the caller adds partial sums anyway.
    A product of many rows with a deep, narrow weight (down: 3,584 x 18,944) has few output tiles (the library's are
    about 256 x 256: 28 at 512 rows) and leaves most of the chip idle; cut into slices that still hold a few
    thousand k-values each, the same library fills it: at 512 rows 65 us instead of 124 (196 without tuning), at
    1,024 rows 112 instead of 188, at 2,048 rows 210 instead of 265.  A power of two, 1: not cut."""
    tiles = -(-M // 256) * -(-N // 256)
    S = 1
    while (2 * S <= LIBRARY_MAX_SLICES and 2 * S * tiles <= 256 and K % (16 * S) == 0
           and K // (2 * S) >= LIBRARY_SLICE_MIN_K):
        S *= 2
    return S


WIDE_FEW_ROWS_MIN_N = 16384               # rows of a weight (tall enough to fill the chip without slices of K) and ...
WIDE_FEW_ROWS_MIN_WEIGHT = 100_000_000    # ... its elements from which 9-16 rows take the product that shares x through LDS


def _tile_pairs_fit(N: int) -> bool:
    """Whether the product that splits K over a workgroup's waves takes the 16-row tiles of a weight of ``N`` rows in
    pairs (the rule of ifx_skinny_gemm: pairs halve its reads of x, and it takes them where they do not give the fullest
    of the 256 compute units more tiles than single tiles would)."""
    n_tiles = -(-N // 16)
    fullest = lambda nt: -(-(-(-n_tiles // nt)) // 256) * nt
    return -(-n_tiles // 2) >= 128 and fullest(2) <= fullest(1)


def _wide_for_few_rows(M: int, N: int, K: int) -> bool:
    """Whether up to 16 rows go to the product that shares x through LDS instead of the one that splits K over a
    workgroup's waves.  From 9 rows on the latter reads as much of x from the L2 as of W from memory; for large tall
    weights, which fill the chip without slices of K, the former then wins (both with the norm's factor per row; gate/up
    of the 7B shape at 9-16 rows 44.4 against 46.9 us, of the 14B shape 46 against 47-49, 32B 87 against 88-94 from 12
    rows, 72B 145 against 157-164; the heads of the 7B, 3B and 72B shapes from 12 rows: 177 against 185, 99 against 105
    and 385 against 414 at 16).  Where the other product cannot take tiles in pairs (gate/up of the 14B and 72B shapes)
    it reads x twice as often and loses from 6 rows on (14B 44.6 against 46.6-47.3 us at 6-8 rows, 72B 143-145 against
    146-149).  Smaller weights (gate/up of the 3B shape: 20 against 17 us) stay where they are."""
    if N < WIDE_FEW_ROWS_MIN_N:
        return _few_rows_in_slices(M, N, K)
    if N * K < WIDE_FEW_ROWS_MIN_WEIGHT:
        return False
    if M >= (12 if N >= 65536 else 9):
        return True
    return M >= 6 and N < 65536 and not _tile_pairs_fit(N)


UNEVEN_TILES_MIN_WEIGHT = 64_000_000      # elements from which a weight whose tiles lie unevenly on the chip is cut into slices of K


def _few_rows_in_slices(M: int, N: int, K: int) -> bool:
    """Whether 8-16 rows times a large weight of few rows go to the product that shares x through LDS and cuts K into slices
    (their sum left to the norm's kernel) instead of the one that adds into the stream itself.  The latter gives a
    workgroup whole row tiles: 5,120 rows are 320 tiles, two for 64 of the 256 compute units and one for the others,
    and the product takes as long as one of 8,192 rows (lower tiles do not help it: measured).  Slices of K fill the
    chip evenly whatever the number of tiles, at the price of the kernel that adds them (5.6 us).  down of the 32B shape
    (5,120 x 27,648) at 8 / 12 / 16 rows: 55 / 61 / 67 us against 43 + 5.6; of the 14B shape (5,120 x 13,824) 29 / 33 / 36
    against 24 + 5.6; its o (5,120 x 5,120: 14-17 against 11 + 5.6) is too small to gain, and weights whose tiles lie
    evenly (3,584 rows in tiles of 14, 8,192 rows) lose.  Decode steps: 8 requests at the 32B shape 13.4 -> 12.9 ms, 16 at
    the 14B shape 11.5 -> 11.3."""
    if M < (8 if N * K >= 2 * UNEVEN_TILES_MIN_WEIGHT else 9) or N * K < UNEVEN_TILES_MIN_WEIGHT:   # (8 rows: the smaller weight ties)
        return False
    tile_rows = choose_tile_rows(N)
    n_tiles = -(-N // tile_rows)
    return N < 0.7 * (-(-n_tiles // COMPUTE_UNITS) * COMPUTE_UNITS * tile_rows)


def _small_m_kernel(M: int, N: int, K: int, has_tiled: bool = False) -> Optional[str]:
    """Which of the streaming kernels takes a bfloat16 product of this shape, or None for the library.
    Measured on the 7B shapes: up to 16 rows the product that splits K over the waves of a workgroup (with x
    staged in LDS for very tall weights such as the head's when there is no tiled copy; 9-16 rows of large tall
    weights as from 17 rows, see _wide_for_few_rows); from 17 to 64 rows
    the product that shares x through LDS, which needs the tiled copy (without it, the first kernel up to 32
    rows on narrow weights); from 65 to 128 rows the same product for weights of few rows, whose K it cuts into
    slices to fill the chip where the library has too few output tiles to (down, o and q/k/v of the 7B shape:
    37-50, 15-21 and 16-22 us against 58-66, 30-34 and 30-37); beyond that, and for tall weights such as gate/up
    and the head, the library's tiles reuse the rows better."""
    if K % 8:
        return None
    if M <= 16:
        if has_tiled and _wide_for_few_rows(M, N, K):
            return "wide"
        return "staged" if N >= 65536 and not has_tiled else "skinny"
    if has_tiled and (M <= SKINNY_MAX_M or (M <= WIDE_MAX_M and N <= WIDE_MANY_ROWS_MAX_N)):
        return "wide"
    if M <= 32 and N <= 4096:
        return "skinny"
    return None


def linear_swiglu(x: torch.Tensor, weight_pairs) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) where ``weight_pairs`` [2I, K] (a tensor or a ``LinearWeight``) alternates the
    rows of Wg and Wu.  For few rows the activation is the product's epilogue; otherwise a second kernel
    applies it."""
    M, K = x.shape
    if isinstance(x, ScaledRows) and not takes_scaled_rows(M, weight_pairs):
        raise KernelError(f"linear_swiglu: scaled rows are not taken for {M} rows and this weight")
    rows, tiled, tile_rows = ((weight_pairs.rows, weight_pairs.tiled, weight_pairs.tile_rows) if isinstance(weight_pairs, LinearWeight)
                              else (weight_pairs, None, 16))
    if isinstance(weight_pairs, LinearWeight) and weight_pairs.order is not None:
        raise KernelError("linear_swiglu: a tile order is not supported for gate/up pairs")
    if rows.dtype == torch.bfloat16 and x.dtype == torch.bfloat16:
        kind = _small_m_kernel(M, rows.shape[0], K, tiled is not None)
        if kind == "skinny":
            return skinny_gemm(x, rows, torch.bfloat16, swiglu_pairs=True, tiled=tiled, tile_rows=tile_rows)
        if kind == "wide":
            return wide_gemm(x, weight_pairs, torch.bfloat16, swiglu_pairs=True)
        if kind == "staged":
            return staged_gemm(x, rows, torch.bfloat16, swiglu_pairs=True)
    return swiglu(linear(x, rows), interleaved=True)


# ----------------------------------------------------------------------------------------
def attention_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, row_req: torch.Tensor,
                    positions: torch.Tensor, block_table: torch.Tensor, window: Optional[int],
                    scale: float) -> torch.Tensor:
    """Causal (optionally windowed) attention of q [T, nH, d] over the paged cache (K [pages, nKV, page, d],
    V [pages, nKV, dv, page]; dv may differ from d); returns [T, nH*dv]."""
    _check(q, "q", (None, None, None))
    T, nH, d = q.shape
    _check(k_cache, "k_cache", (None, None, None, d), q.dtype)
    n_pages, nKV, page_size, _ = k_cache.shape
    _check(v_cache, "v_cache", (n_pages, nKV, None, page_size), q.dtype)
    dv = v_cache.shape[2]
    _check(row_req, "row_req", (T,), torch.int32)
    _check(positions, "positions", (T,), torch.int32)
    _check(block_table, "block_table", (None, None), torch.int32)
    out = torch.empty((T, nH * dv), dtype=q.dtype, device=q.device)
    _call(load_module("attn_plain"), "ifx_attn_plain", (P, P, P, P, I, P, P, P, I, I, I, I, I, I, I, I, F, P),
          q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _dt(q), row_req.data_ptr(),
          positions.data_ptr(), block_table.data_ptr(), block_table.shape[1], T, nH, nKV, d, dv, page_size,
          int(window or 0), float(scale), _stream())
    return out


def mfma_attention_supported(dtype: torch.dtype, head_dim: int, page_size: int) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and head_dim <= MFMA_MAX_HEAD_DIM
            and page_size >= 16 and page_size & (page_size - 1) == 0)


def _attn_common(q, k_cache, v_cache, qt=1):
    _check(q, "q", (None, None, None), torch.bfloat16)
    T, nH, d = q.shape
    _check(k_cache, "k_cache", (None, None, None, d), torch.bfloat16)
    n_pages, nKV, page_size, _ = k_cache.shape
    _check(v_cache, "v_cache", (n_pages, nKV, d, page_size), torch.bfloat16)
    if not mfma_attention_supported(q.dtype, d, page_size):
        raise KernelError(f"matrix-core attention needs bfloat16, head_dim a multiple of 16 up to {MFMA_MAX_HEAD_DIM} and "
                          f"page_size a power of two from 16; got head_dim {d}, page_size {page_size}")
    name, variant, _, _ = _tile_module(d, qt)
    return T, nH, d, nKV, page_size, load_module(name, variant)


ROW_MAX_WAVES = 8


def row_waves_fit(n_heads: int, n_kv_heads: int, head_dim: int, waves: int) -> int:
    """The most waves per workgroup, up to ``waves``, whose results fit the row kernel's 64 KB of LDS."""
    nc = min(16, n_heads // n_kv_heads)
    while waves > 1 and waves * nc * (head_dim + 6) * 4 > 65536:
        waves //= 2
    return waves


def attention_rows(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                   rows: Optional[torch.Tensor], n_rows: int, row_req: torch.Tensor, positions: torch.Tensor,
                   block_table: torch.Tensor, window: Optional[int], scale: float, chunk: int, max_splits: int,
                   waves: int = 0, req_is_row: bool = False) -> None:
    """Attention of single rows (``rows`` int32, or None for rows 0..n_rows-1) into ``out`` [T, nH*d].

    ``waves`` 0: split s of a row covers key positions [s*chunk, (s+1)*chunk), one wave each, and a second launch
    merges a row's splits; ``max_splits`` * chunk must reach past the largest position among the rows.
    ``waves`` 1-8: one workgroup of that many waves per (row, kv head) shares the row's keys evenly and writes the
    output itself (``chunk`` and ``max_splits`` are not used): for launches with pairs enough to fill the chip.
    ``req_is_row``: the caller vouches that ``row_req`` is 0, 1, 2, ... (every request brings one row), which lets
    a wave ask for its block-table entries before it knows anything else."""
    T, nH, d, nKV, page_size, mod = _attn_common(q, k_cache, v_cache)
    _check(out, "out", (T, nH * d), torch.bfloat16)
    _check(row_req, "row_req", (T,), torch.int32)
    _check(positions, "positions", (T,), torch.int32)
    _check(block_table, "block_table", (None, None), torch.int32)
    if rows is not None:
        _check(rows, "rows", (n_rows,), torch.int32)
    elif n_rows != T:
        raise KernelError("attention_rows: without a row list every row of the batch is handled")
    if not 0 <= waves <= ROW_MAX_WAVES or row_waves_fit(nH, nKV, d, waves) != waves:
        raise KernelError(f"attention_rows: {waves} waves per workgroup (0-{ROW_MAX_WAVES}, and their results within 64 KB of LDS: "
                          f"up to {row_waves_fit(nH, nKV, d, ROW_MAX_WAVES)} at these head counts)")
    part_o = part_ml = None
    if waves == 0:
        part_o = torch.empty((n_rows, nH, max_splits, d), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n_rows, nH, max_splits, 2), dtype=torch.float32, device=q.device)
    if req_is_row and block_table.shape[0] < T:
        raise KernelError("attention_rows: req_is_row needs a block-table row for every row of the step")
    _call(mod, "ifx_attn_rows", (P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, F, P, P, I, I, P),
          q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), _ptr(rows), row_req.data_ptr(),
          positions.data_ptr(), block_table.data_ptr(), block_table.shape[1], n_rows, nH, nKV, d, page_size,
          int(window or 0), chunk, max_splits, float(scale), _ptr(part_o), _ptr(part_ml), waves, 1 if req_is_row else 0, _stream())


def attention_tile_rows(head_dim: int, qt: int = 1) -> int:
    """Rows per tile of the tile kernel in tiling ``qt`` (see TILE_QTS; the compiled module says the same; asking it
    would compile a variant that a short step never runs)."""
    return 64 * qt


def attention_tiles(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                    tile_req: torch.Tensor, tile_q0: torch.Tensor, q_start: torch.Tensor, q_len: torch.Tensor,
                    kv_len: torch.Tensor, block_table: torch.Tensor, window: Optional[int], scale: float,
                    qt: int = 1, chunk: int = 0, max_splits: int = 1, rows: Optional[torch.Tensor] = None,
                    row_req: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None,
                    order: Optional[torch.Tensor] = None) -> None:
    """Attention of tiles of ``attention_tile_rows(d, qt)`` consecutive rows of one request each (tile t:
    request tile_req[t], rows from tile_q0[t] of that request's rows in this step) into ``out`` [T, nH*d].

    With ``max_splits`` > 1 every tile's keys are cut into splits of ``chunk`` keys (a multiple of 64;
    ``max_splits`` * chunk must reach past the largest position) that run as workgroups of their own, and
    the rows named by ``rows`` (int32: every row of every tiled request) are merged at the end; this
    needs the step's ``row_req`` and ``positions`` [T].

    ``order`` (int32 [8 * n], from ``attention.tile_order``) says which work item each workgroup of the launch
    takes; every item must appear exactly once (-1: a workgroup without work).  The result does not depend on it."""
    T, nH, d, nKV, page_size, mod = _attn_common(q, k_cache, v_cache, qt)
    _, _, entry, rows_fn = _tile_module(d, qt)
    if mod.fn(rows_fn, ())() != attention_tile_rows(d, qt):
        raise KernelError("attention_tiles: the compiled module's tile rows differ from attention_tile_rows()")
    _check(out, "out", (T, nH * d), torch.bfloat16)
    n_tiles = tile_req.shape[0]
    _check(tile_req, "tile_req", (n_tiles,), torch.int32)
    _check(tile_q0, "tile_q0", (n_tiles,), torch.int32)
    R = q_start.shape[0]
    for t, nm in ((q_start, "q_start"), (q_len, "q_len"), (kv_len, "kv_len")):
        _check(t, nm, (R,), torch.int32)
    _check(block_table, "block_table", (R, None), torch.int32)
    part_o = part_ml = None
    n_rows = 0
    if max_splits > 1:
        if chunk <= 0 or chunk % 64:
            raise KernelError(f"attention_tiles: splits need a chunk that is a multiple of 64, got {chunk}")
        if rows is None or row_req is None or positions is None:
            raise KernelError("attention_tiles: splits need the rows to merge, row_req and positions")
        n_rows = rows.shape[0]
        _check(rows, "rows", (n_rows,), torch.int32)
        _check(row_req, "row_req", (T,), torch.int32)
        _check(positions, "positions", (T,), torch.int32)
        part_o = torch.empty((T, nH, max_splits, d), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T, nH, max_splits, 2), dtype=torch.float32, device=q.device)
    per_xcd = 0
    if order is not None:
        _check(order, "order", (None,), torch.int32)
        if order.shape[0] % N_XCD:
            raise KernelError(f"attention_tiles: the order has a place for each of {N_XCD} XCDs' workgroups")
        per_xcd = order.shape[0] // N_XCD
    _call(mod, entry, (P, P, P, P, P, P, I, P, P, P, P, I, I, I, I, I, I, F, I, I, P, P, P, I, P, P, P, I, I, P),
          q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), tile_req.data_ptr(), tile_q0.data_ptr(),
          n_tiles, q_start.data_ptr(), q_len.data_ptr(), kv_len.data_ptr(), block_table.data_ptr(),
          block_table.shape[1], nH, nKV, d, page_size, int(window or 0), float(scale), int(chunk), int(max_splits),
          _ptr(part_o), _ptr(part_ml), _ptr(rows), n_rows, _ptr(row_req), _ptr(positions), _ptr(order), per_xcd, N_XCD, _stream())


# ----------------------------------------------------------------------------------------
def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Lowest index of the maximum of each row of float32 ``logits`` [R, V]; int32 [R]."""
    _check(logits, "logits", (None, None), torch.float32)
    R, V = logits.shape
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    pv = torch.empty((R, 32), dtype=torch.float32, device=logits.device)
    pi = torch.empty((R, 32), dtype=torch.int32, device=logits.device)
    _call(load_module("sampling"), "ifx_argmax", (P, I, I, P, P, P, P), logits.data_ptr(), R, V, out.data_ptr(),
          pv.data_ptr(), pi.data_ptr(), _stream())
    return out


def apply_penalties(logits: torch.Tensor, rows: torch.Tensor, ids: torch.Tensor, counts: torch.Tensor,
                    rep: torch.Tensor, freq: torch.Tensor, pres: torch.Tensor) -> None:
    _check(logits, "logits", (None, None), torch.float32)
    R, V = logits.shape
    n = rows.shape[0]
    for t, nm in ((rows, "rows"), (ids, "ids"), (counts, "counts")):
        _check(t, nm, (n,), torch.int32)
    for t, nm in ((rep, "rep"), (freq, "freq"), (pres, "pres")):
        _check(t, nm, (R,), torch.float32)
    _call(load_module("sampling"), "ifx_apply_penalties", (P, I, P, P, P, I, P, P, P, P),
          logits.data_ptr(), V, rows.data_ptr(), ids.data_ptr(), counts.data_ptr(), n, rep.data_ptr(),
          freq.data_ptr(), pres.data_ptr(), _stream())


def add_logit_bias(logits: torch.Tensor, rows: torch.Tensor, ids: torch.Tensor, bias: torch.Tensor) -> None:
    _check(logits, "logits", (None, None), torch.float32)
    n = rows.shape[0]
    _check(rows, "rows", (n,), torch.int32)
    _check(ids, "ids", (n,), torch.int32)
    _check(bias, "bias", (n,), torch.float32)
    _call(load_module("sampling"), "ifx_add_logit_bias", (P, I, P, P, P, I, P),
          logits.data_ptr(), logits.shape[1], rows.data_ptr(), ids.data_ptr(), bias.data_ptr(), n, _stream())


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, uniform: Optional[torch.Tensor] = None, draws: Optional[torch.Tensor] = None,
           any_greedy: bool = True, any_filters: bool = True) -> torch.Tensor:
    """One token per row of float32 ``logits`` [R, V]; rows with temperature <= 0 take the argmax (``any_greedy``
    False: the caller knows that there is no such row; ``any_filters`` False: that no row has top-k or top-p; both
    save launches that would find nothing to do).  The number in
    [0, 1) that a row's draw uses is either given (``uniform`` [R]) or made by the kernel from ``draws`` (int32
    [R, 4]: the row's seed and the count of its draws so far, 64 bits each, low word first), as
    ``sampling.params.philox_uniform`` makes it."""
    _check(logits, "logits", (None, None), torch.float32)
    R, V = logits.shape
    _check(temperature, "temperature", (R,), torch.float32)
    _check(top_k, "top_k", (R,), torch.int32)
    _check(top_p, "top_p", (R,), torch.float32)
    _check(min_p, "min_p", (R,), torch.float32)
    if (uniform is None) == (draws is None):
        raise KernelError("sample: either uniform numbers or seeds and counters")
    if uniform is not None:
        _check(uniform, "uniform", (R,), torch.float32)
    else:
        _check(draws, "draws", (R, 4), torch.int32)
    mod = load_module("sampling")
    weights = torch.empty_like(logits)
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    # large vocabularies are drawn by several workgroups a row, which hand each other their results in scratch memory
    n_scratch = mod.fn("ifx_sample_scratch_blocks", (I, I, I))(R, V, 1 if any_filters else 0)
    scratch = torch.empty((n_scratch * 256,), dtype=torch.uint8, device=logits.device) if n_scratch else None
    _call(mod, "ifx_sample", (P, P, P, P, P, P, P, P, P, I, I, P, I, I, P),
          logits.data_ptr(), weights.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
          min_p.data_ptr(), uniform.data_ptr() if uniform is not None else None,
          draws.data_ptr() if draws is not None else None, out.data_ptr(), R, V, _ptr(scratch), 1 if any_greedy else 0,
          1 if any_filters else 0, _stream())
    return out


def logprobs(logits: torch.Tensor, chosen: torch.Tensor, top_n: int):
    """log-softmax of the chosen token of each row and the row's ``top_n`` (<= 20) most probable tokens:
    (lp [R], top_ids [R, top_n] int32, top_lp [R, top_n]), descending, lowest index first among equals."""
    _check(logits, "logits", (None, None), torch.float32)
    R, V = logits.shape
    _check(chosen, "chosen", (R,), torch.int32)
    lp = torch.empty((R,), dtype=torch.float32, device=logits.device)
    top_ids = torch.empty((R, top_n), dtype=torch.int32, device=logits.device)
    top_lp = torch.empty((R, top_n), dtype=torch.float32, device=logits.device)
    _call(load_module("sampling"), "ifx_logprobs", (P, P, I, I, I, P, P, P, P),
          logits.data_ptr(), chosen.data_ptr(), R, V, top_n, lp.data_ptr(), top_ids.data_ptr(), top_lp.data_ptr(), _stream())
    return lp, top_ids, top_lp


# ----------------------------------------------------------------------------------------
_SINKS: Dict[int, torch.Tensor] = {}


def stream_read(region: torch.Tensor, waves: int, streaming: bool) -> None:
    """Measurement only: ``waves`` single-wave workgroups read the whole of ``region`` (a multiple of 8 KB) once."""
    _check(region, "region")
    sink = _SINKS.get(region.device.index)
    if sink is None:
        sink = _SINKS[region.device.index] = torch.zeros(1, dtype=torch.float32, device=region.device)
    _call(load_module("ceilings"), "ifx_stream_read", (P, LL, I, I, P, P),
          region.data_ptr(), region.numel() * region.element_size(), waves, int(streaming), sink.data_ptr(), _stream())


def stream_copy(src: torch.Tensor, dst: torch.Tensor, waves: int, streaming: bool) -> None:
    """Measurement only: copies ``src`` to ``dst`` (same size, a multiple of 8 KB) with ``waves`` single-wave workgroups."""
    _check(src, "src")
    _check(dst, "dst")
    n = src.numel() * src.element_size()
    if n != dst.numel() * dst.element_size():
        raise KernelError(f"stream_copy: {n} bytes into {dst.numel() * dst.element_size()}")
    _call(load_module("ceilings"), "ifx_stream_copy", (P, P, LL, I, I, P), src.data_ptr(), dst.data_ptr(), n, waves, int(streaming), _stream())
