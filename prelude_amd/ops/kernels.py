"""Python faces of the HIP kernels: shape and type checks on the host, then one launch.

Every function works on CUDA (HIP) tensors and launches on torch's current
stream.  Nothing here computes on the CPU or through a torch operator;
``linear`` in bfloat16 for tall inputs calls the library matrix product
(hipBLASLt, directly) where the reference calls its GEMM libraries
(crates/prelude-cuda/src/ops/gemm.rs:35-137).
"""
from __future__ import annotations

from typing import Optional

import torch

from .._native import NativeError, check, kernels

_CODES = {torch.float32: 0, torch.bfloat16: 1}


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise NativeError(f"element type {t.dtype} is not supported (float32 or bfloat16)") from None


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current stream's handle.  Asked for before every launch (a graph capture switches streams), so
    through torch's raw accessor where it has one: the Stream object costs several microseconds to build."""
    if _RAW_STREAM is not None:
        return _RAW_STREAM(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise NativeError("kernel operand is not on the GPU; there is no CPU path")
        if not t.is_contiguous():
            raise NativeError(f"kernel operand of shape {tuple(t.shape)} is not contiguous")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _i32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32:
        raise NativeError(f"{name} must be int32, got {t.dtype}")


def _f32(t: Optional[torch.Tensor], name: str) -> None:
    if t is not None and t.dtype != torch.float32:
        raise NativeError(f"{name} must be float32, got {t.dtype}")


# ---------------------------------------------------------------------------
def embed_gather(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]]; ids int32 [T], table [V, H]."""
    _dev(ids, table)
    _i32(ids, "ids")
    if ids.dim() != 1 or table.dim() != 2:
        raise NativeError(f"embed_gather: ids {tuple(ids.shape)} / table {tuple(table.shape)}")
    out = torch.empty((ids.shape[0], table.shape[1]), dtype=table.dtype, device=table.device)
    check(kernels().pa_embed_gather(_stream(), _code(table), _ptr(ids), _ptr(table), _ptr(out), ids.shape[0],
                                    table.shape[1], table.shape[0]))
    return out


def carry_tokens(sampled: torch.Tensor, src: torch.Tensor, dst: torch.Tensor, ids: torch.Tensor) -> None:
    """ids[dst[i]] = sampled[src[i]] where src[i] >= 0; all int32 on the device."""
    _dev(sampled, src, dst, ids)
    for t, name in ((sampled, "sampled"), (src, "src"), (dst, "dst"), (ids, "ids")):
        _i32(t, name)
    if src.shape != dst.shape or src.dim() != 1:
        raise NativeError(f"carry_tokens: src {tuple(src.shape)} / dst {tuple(dst.shape)}")
    check(kernels().pa_carry_tokens(_stream(), _ptr(sampled), _ptr(src), _ptr(dst), _ptr(ids), src.shape[0],
                                    sampled.numel(), ids.numel()))


def zero_fresh_rows(data: torch.Tensor, slots: torch.Tensor, fresh: torch.Tensor) -> None:
    """data[slots[i]] = 0 for every sequence i with fresh[i] != 0 and slots[i] >= 0; data [rows, ...] of a
    4-byte-multiple row size, slots / fresh int32 [B] on the device."""
    _dev(data, slots, fresh)
    _i32(slots, "slots")
    _i32(fresh, "fresh")
    if data.dim() < 1 or slots.shape != fresh.shape or slots.dim() != 1:
        raise NativeError(f"zero_fresh_rows: data {tuple(data.shape)} / slots {tuple(slots.shape)} / fresh {tuple(fresh.shape)}")
    if data.shape[0] == 0 or slots.shape[0] == 0:
        return
    row_bytes = data[0].numel() * data.element_size()
    check(kernels().pa_zero_fresh_rows(_stream(), _ptr(data), row_bytes, _ptr(slots), _ptr(fresh), slots.shape[0],
                                       data.shape[0]))


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm over the last axis of x [T, H] with a float32 weight [H].

    With ``residual`` the norm is taken of x + residual (32-bit sum) and the
    residual tensor receives the sum.  With ``rows`` (int32 [R]) only those
    rows are normed, into a compact [R, H] output, and the residual is read only.
    """
    if isinstance(x, SliceSums):
        return _rmsnorm_slices(x, weight, eps, residual, rows)
    _dev(x, weight, residual, rows)
    _f32(weight, "norm weight")
    if x.dim() != 2 or weight.shape != (x.shape[1],):
        raise NativeError(f"rmsnorm: x {tuple(x.shape)} / weight {tuple(weight.shape)}")
    if residual is not None and (residual.shape != x.shape or residual.dtype != x.dtype):
        raise NativeError(f"rmsnorm: residual {tuple(residual.shape)} {residual.dtype} does not match x")
    n = x.shape[0]
    if rows is not None:
        _i32(rows, "rows")
        n = rows.shape[0]
    out = torch.empty((n, x.shape[1]), dtype=x.dtype, device=x.device)
    check(kernels().pa_rmsnorm(_stream(), _code(x), _ptr(x), _ptr(residual), _ptr(weight), _ptr(out), _ptr(rows), n,
                               x.shape[1], float(eps)))
    return out


def _rmsnorm_slices(x, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor],
                    rows: Optional[torch.Tensor]) -> torch.Tensor:
    """``rmsnorm`` of a product that comes as partial sums: the slices are added in order as they are loaded."""
    parts = x.parts
    _dev(parts, weight, residual, rows)
    _f32(weight, "norm weight")
    s, m, h = parts.shape
    if weight.shape != (h,) or h % 4:
        raise NativeError(f"rmsnorm: slices {tuple(parts.shape)} / weight {tuple(weight.shape)}")
    if residual is not None and (tuple(residual.shape) != (m, h) or residual.dtype != x.dtype):
        raise NativeError(f"rmsnorm: residual {tuple(residual.shape)} {residual.dtype} does not match the product")
    n = m
    if rows is not None:
        _i32(rows, "rows")
        n = rows.shape[0]
    out = torch.empty((n, h), dtype=x.dtype, device=parts.device)
    check(kernels().pa_rmsnorm_slices(_stream(), _CODES[x.dtype], _ptr(parts), s, m * h, _ptr(residual), _ptr(weight),
                                      _ptr(out), _ptr(rows), n, h, float(eps)))
    return out


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}   # codes of the kernels' gated epilogues (common.h)


def gate_activation_code(name: str) -> int:
    try:
        return GATE_ACTIVATIONS[name]
    except KeyError:
        raise NativeError(f"gated activation {name!r} is not one of {sorted(GATE_ACTIVATIONS)}") from None


def silu_mul(gate_up: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """act(gate) * up for gate_up [T, 2I] whose columns alternate gate_j, up_j -> [T, I]; ``activation`` is
    ``"silu"`` or ``"gelu_tanh"``, here and in the gated epilogues of the products."""
    act = gate_activation_code(activation)
    _dev(gate_up)
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise NativeError(f"silu_mul: input {tuple(gate_up.shape)} is not [T, 2I]")
    inter = gate_up.shape[1] // 2
    out = torch.empty((gate_up.shape[0], inter), dtype=gate_up.dtype, device=gate_up.device)
    check(kernels().pa_silu_mul(_stream(), _code(gate_up), _ptr(gate_up), _ptr(out), gate_up.shape[0], inter, act))
    return out


def gather_rows(x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    _dev(x, rows)
    _i32(rows, "rows")
    if x.dim() != 2:
        raise NativeError(f"gather_rows: x {tuple(x.shape)}")
    out = torch.empty((rows.shape[0], x.shape[1]), dtype=x.dtype, device=x.device)
    check(kernels().pa_gather_rows(_stream(), _code(x), _ptr(x), _ptr(rows), _ptr(out), rows.shape[0], x.shape[1]))
    return out


def add_bias_(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    _dev(y, bias)
    _f32(bias, "bias")
    if y.dim() != 2 or bias.shape != (y.shape[1],):
        raise NativeError(f"add_bias: y {tuple(y.shape)} / bias {tuple(bias.shape)}")
    check(kernels().pa_add_bias(_stream(), _code(y), _ptr(y), _ptr(bias), y.shape[0], y.shape[1]))
    return y


def to_f32(x: torch.Tensor) -> torch.Tensor:
    _dev(x)
    if x.dtype == torch.float32:
        return x
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    check(kernels().pa_to_f32(_stream(), _code(x), _ptr(x), _ptr(out), x.numel()))
    return out


def _check_caches(k_cache, v_cache, num_kv_heads, head_dim, dtype, what) -> None:
    """K [pages, nkv, page, hd] and V [pages, nkv, hd, page] of the same pool."""
    ok = (k_cache is not None and v_cache is not None and k_cache.dim() == 4 and v_cache.dim() == 4
          and k_cache.shape[0] == v_cache.shape[0] and k_cache.shape[1] == v_cache.shape[1] == num_kv_heads
          and k_cache.shape[3] == v_cache.shape[2] == head_dim and k_cache.shape[2] == v_cache.shape[3]
          and k_cache.dtype == dtype and v_cache.dtype == dtype)
    if not ok:
        raise NativeError(f"{what}: caches must be K [pages, {num_kv_heads}, page, {head_dim}] and "
                          f"V [pages, {num_kv_heads}, {head_dim}, page] of {dtype}")


def qknorm_rope_kv(qkv: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                   cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
                   slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   num_heads: int, num_kv_heads: int, head_dim: int, rotary_dim: int, eps: float) -> torch.Tensor:
    """Per-head RMSNorm of Q and K, rotation by position, K and V into the paged cache.

    qkv [T, (nh + 2 nkv) * hd]; returns q [T, nh, hd].  With ``slots`` None
    nothing is written to the cache (then ``num_kv_heads`` may be 0 for a
    Q-only input).  K cache [pages, nkv, page_size, hd], V cache [pages, nkv, hd, page_size].
    """
    _dev(qkv, q_weight, k_weight, cos, sin, positions, slots, k_cache, v_cache)
    _i32(positions, "positions")
    _f32(q_weight, "q_norm weight")
    _f32(k_weight, "k_norm weight")
    _f32(cos, "cos table")
    _f32(sin, "sin table")
    t = qkv.shape[0]
    width = (num_heads + 2 * num_kv_heads) * head_dim
    if qkv.dim() != 2 or qkv.shape[1] != width:
        raise NativeError(f"qknorm_rope_kv: qkv {tuple(qkv.shape)} is not [T, {width}]")
    if positions.shape != (t,):
        raise NativeError(f"qknorm_rope_kv: positions {tuple(positions.shape)} for {t} tokens")
    for w, nm in ((q_weight, "q_norm"), (k_weight, "k_norm")):
        if w is not None and w.shape != (head_dim,):
            raise NativeError(f"qknorm_rope_kv: {nm} weight {tuple(w.shape)} is not [{head_dim}]")
    if rotary_dim:
        if cos is None or sin is None or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] != rotary_dim // 2:
            raise NativeError(f"qknorm_rope_kv: cos/sin tables must be [positions, {rotary_dim // 2}]")
    page_size = 1
    if slots is not None:
        _i32(slots, "slots")
        if slots.shape != (t,):
            raise NativeError(f"qknorm_rope_kv: slots {tuple(slots.shape)} for {t} tokens")
        _check_caches(k_cache, v_cache, num_kv_heads, head_dim, qkv.dtype, "qknorm_rope_kv")
        page_size = k_cache.shape[2]
    q_out = torch.empty((t, num_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    check(kernels().pa_qknorm_rope_kv(_stream(), _code(qkv), _ptr(qkv), _ptr(q_weight), _ptr(k_weight), _ptr(cos),
                                      _ptr(sin), _ptr(positions), _ptr(slots), _ptr(q_out), _ptr(k_cache),
                                      _ptr(v_cache), t, num_heads, num_kv_heads, head_dim, rotary_dim, page_size,
                                      float(eps)))
    return q_out


def gemm_plain(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
               out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """x [M, K] @ w[N, K]^T (+ bias) with 32-bit FMA arithmetic in a fixed order."""
    _dev(x, w, bias)
    _f32(bias, "bias")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.dtype != w.dtype:
        raise NativeError(f"gemm: x {tuple(x.shape)} {x.dtype} / w {tuple(w.shape)} {w.dtype}")
    out_dtype = out_dtype or x.dtype
    m, k = x.shape
    n = w.shape[0]
    if bias is not None and bias.shape != (n,):
        raise NativeError(f"gemm: bias {tuple(bias.shape)} is not [{n}]")
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    check(kernels().pa_gemm_plain(_stream(), _code(x), _CODES[out_dtype], _ptr(x), _ptr(w), _ptr(bias), _ptr(out), m, n,
                                  k, k, k, n))
    return out


SKINNY_MAX_ROWS = 16   # above this the library product is faster (the kernel itself takes up to 64) ...
# ... except for small weights in tiles, where the library's 19 us floor is what it takes: (rows, elements) up to
# which the streaming kernel measured faster -- [6144, 2560] and [2560, 4096] to 48 rows (11 against 19 us at 32),
# [6144, 4096] to 32 rows (15 against 19 us); weights beyond that go to the library, as do rows of 8192 columns or
# more -- unless they are very long: [5120, 25600] takes the library 143 to 155 us at 24 to 64 rows, the streaming
# kernel 67 to 118.  Inside a captured step, where no launch waits for the host, the library's floor is 11 us and
# the order is the same: [4096, 1024] takes the streaming kernel 4.6 to 8.0 us at 17 to 64 rows, [6144, 2560] 11.6
# to 14.4 at 17 to 48 rows against 12.5 to 15.5
TILED_LIMITS = ((64, 1 << 23), (48, 1 << 24), (32, 1 << 25))
TILED_LONG_ROWS = 16384


def _tiled_beyond_16(m: int, n: int, k: int) -> bool:
    if k % 8:
        return False
    if k >= TILED_LONG_ROWS:
        return m <= 64
    return k < 8192 and any(m <= rows and n * k <= size for rows, size in TILED_LIMITS)


class TiledWeight:
    """A bfloat16 weight [n, k] laid out in the tiles the weight-streaming kernel reads (``pack_tiles``)."""

    def __init__(self, data: torch.Tensor, n: int, k: int):
        self.data, self.n, self.k = data, n, k
        self.shape = (n, k)
        self.dtype, self.device = data.dtype, data.device


def pack_tiles(w: torch.Tensor) -> TiledWeight:
    """The weight in tiles of 16 rows x 64 columns, each stored in the order a wavefront's lanes load it."""
    _dev(w)
    if w.dim() != 2 or w.dtype != torch.bfloat16:
        raise NativeError(f"pack_tiles: w {tuple(w.shape)} {w.dtype}")
    n, k = w.shape
    out = torch.empty(((n + 15) // 16) * ((k + 63) // 64) * 1024, dtype=torch.bfloat16, device=w.device)
    check(kernels().pa_pack_tiles(_stream(), _ptr(w), _ptr(out), n, k))
    return TiledWeight(out, n, k)


WEIGHT_TILES = True   # keep a tiled copy of bfloat16 weights for products of few rows (``set_weight_tiles``)


def set_weight_tiles(on: bool) -> None:
    """Whether ``prepare_weight`` adds the tiled copy (a second copy of the weight in device memory)."""
    global WEIGHT_TILES
    WEIGHT_TILES = bool(on)


class LinearWeight:
    """A matrix [out, in] as the products read it: by rows for many-row products (the library's) and the
    32-bit path, and, for bfloat16, in tiles for the weight-streaming product of few rows."""

    def __init__(self, rows: torch.Tensor, tiles: Optional[TiledWeight] = None):
        self.rows, self.tiles = rows, tiles
        self.shape, self.dtype, self.device = tuple(rows.shape), rows.dtype, rows.device

    def first_rows(self, n: int) -> torch.Tensor:
        """The first n outputs as a plain matrix (a view)."""
        return self.rows[:n]


def prepare_weight(w: torch.Tensor) -> LinearWeight:
    """What a part keeps of a weight it multiplies by: called once when weights are loaded."""
    tiles = None
    if WEIGHT_TILES and w.dtype == torch.bfloat16 and w.is_cuda and w.dim() == 2:
        tiles = pack_tiles(w.contiguous())
    return LinearWeight(w, tiles)


def gemm_skinny(x: torch.Tensor, w, bias: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, silu_mul_epilogue: bool = False,
                activation: str = "silu") -> torch.Tensor:
    """x [M <= 64, K] @ w[N, K]^T in bfloat16 on the matrix cores, streaming w once.

    ``w`` is a tensor [N, K] or a ``TiledWeight``.  With
    ``silu_mul_epilogue`` the rows of w alternate gate_j, up_j and the
    result is act(gate) * up, [M, N/2], act being ``activation``."""
    epi = 1 + gate_activation_code(activation) if silu_mul_epilogue else 0
    tiled = isinstance(w, TiledWeight)
    wt = w.data if tiled else w
    _dev(x, wt, bias)
    _f32(bias, "bias")
    if x.dim() != 2 or len(w.shape) != 2 or x.shape[1] != w.shape[1] or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise NativeError(f"gemm_skinny: x {tuple(x.shape)} {x.dtype} / w {tuple(w.shape)} {w.dtype}")
    m, k = x.shape
    n = w.shape[0]
    out_dtype = out_dtype or torch.bfloat16
    if bias is not None and bias.shape != (n,):
        raise NativeError(f"gemm_skinny: bias {tuple(bias.shape)} is not [{n}]")
    cols = n // 2 if silu_mul_epilogue else n
    out = torch.empty((m, cols), dtype=out_dtype, device=x.device)
    check(kernels().pa_gemm_skinny(_stream(), _CODES[out_dtype], epi, _ptr(x), _ptr(wt),
                                   _ptr(bias), _ptr(out), m, n, k, k, cols, 1 if tiled else 0))
    return out


class SliceSums:
    """A product left as 32-bit partial sums of slices of its inner size, [slices, M, N]: what ``gemm_mid`` gives
    when its reader can add the slices itself (``rmsnorm`` does, as it loads them).  ``materialize()`` adds them
    for any other reader."""

    def __init__(self, parts: torch.Tensor, dtype: torch.dtype):
        self.parts = parts
        self.shape = tuple(parts.shape[1:])
        self.dtype, self.device = dtype, parts.device

    def materialize(self) -> torch.Tensor:
        s, m, n = self.parts.shape
        out = torch.empty((m, n), dtype=self.dtype, device=self.device)
        check(kernels().pa_sum_slices(_stream(), _CODES[self.dtype], _ptr(self.parts), _ptr(out), s, m * n))
        return out


def gemm_skinny_sliced(x: torch.Tensor, w: "TiledWeight", bias: Optional[torch.Tensor] = None, slices: int = 2,
                       waves: int = 0) -> SliceSums:
    """``gemm_skinny`` of up to 16 rows with K cut into slices, each a workgroup of its own a tile, left as 32-bit
    partial sums for a reader that adds them: a narrow weight has too few tiles to give every compute unit work."""
    _dev(x, w.data, bias)
    _f32(bias, "bias")
    m, k = x.shape
    n = w.shape[0]
    if x.dtype != torch.bfloat16 or w.shape[1] != k or not 1 <= m <= 16 or (bias is not None and bias.shape != (n,)):
        raise NativeError(f"gemm_skinny_sliced: x {tuple(x.shape)} {x.dtype} / w {w.shape}")
    made = int(kernels().pa_gemm_skinny_slices(k, int(slices)))
    parts = torch.empty((made, m, n), dtype=torch.float32, device=x.device)
    check(kernels().pa_gemm_skinny_sliced(_stream(), _ptr(x), _ptr(w.data), _ptr(bias), _ptr(parts), m, n, k, k, int(slices),
                                          int(waves)))
    return SliceSums(parts, torch.bfloat16)


GEMM_MID_MAX_ROWS = 128
# Where ``linear`` takes the product with X staged in LDS (measured at the shapes of 4B, 8B and 32B models, 17 to
# 128 rows).  Cut into slices, for a reader that adds them, wherever the weight's shape gives two slices or more:
# [2560, 4096] at 64 rows 9.2 against the library's 14.7 us, [2560, 9728] 14.4 against 28, [4096, 12288] 28 against
# 37, [5120, 25600] 50 against 155 (and 73 against 179 at 128 rows).  Uncut for very wide weights with 32-bit output
# (the head; figures at MID_WIDE_MAX_M).  The gated product with its activation in the epilogue: see
# ``linear_silu_mul``.
MID_MIN_SLICES = 2
MID_WIDE_ROWS = 65536
MID_WIDE_MAX_M = 64            # ... for rows of up to MID_WIDE_SHORT_K columns, half of it beyond.  (Alone inside a
#                                captured graph the head is ahead of the library up to 128 rows, 214 against 230 us at
#                                96 rows of 2,560 columns; in the decode step of 112 requests it is not: 7,380 against
#                                7,640 tok/s.  The step decides.)
MID_WIDE_SHORT_K = 4096
MID_SLICED_MIN_ROWS = 9        # ... for rows of MID_SLICED_LONG_K columns or more; 17 otherwise
MID_SLICED_LONG_K = 5120
MID_SLICED_MIN_ROWS_LONG = 8   # rows of TILED_LONG_ROWS columns or more: in slices from here on
# A reader that wants a tensor gets the slices too, added by a kernel of their own, where the pair is still ahead of
# the library: large weights ([10240, 5120] inside a captured step: 24.2 to 26.9 us at 24 to 64 rows against 28.4 to
# 32.4, 33.7 and 38.6 at 96 and 128 rows against 36.1 and 40.4; [6144, 4096] and [6144, 2560] are within a
# microsecond either way and stay with the library)
MID_SUMMED_MIN_ELEMENTS = 40 << 20
MID_PRODUCTS = True    # ``set_mid_products``: off sends these products where they went without this kernel (measurements)


def set_mid_products(on: bool) -> None:
    global MID_PRODUCTS
    MID_PRODUCTS = bool(on)


def gemm_mid_slices(n: int, k: int) -> int:
    """Into how many slices of its inner size ``gemm_mid`` cuts an [n, k] weight for a reader that adds slices."""
    return int(kernels().pa_gemm_mid_slices(int(n), int(k)))


def gemm_mid(x: torch.Tensor, w: "TiledWeight", bias: Optional[torch.Tensor] = None,
             out_dtype: Optional[torch.dtype] = None, silu_mul_epilogue: bool = False, slices: int = 1, waves: int = 0,
             activation: str = "silu"):
    """x [M <= 128, K] @ w[N, K]^T from the weight in tiles, X staged through LDS; with ``slices`` > 1 the result
    is a ``SliceSums`` (one 32-bit partial sum per slice of K) instead of a tensor.  ``waves``: wavefronts a
    workgroup (3, 4, 5, 6, 8; 0 lets the launcher choose by the weight's shape; the same bits at every number)."""
    if not isinstance(w, TiledWeight):
        raise NativeError("gemm_mid takes the weight in tiles (pack_tiles)")
    epi = 1 + gate_activation_code(activation) if silu_mul_epilogue else 0
    _dev(x, w.data, bias)
    _f32(bias, "bias")
    if x.dim() != 2 or x.shape[1] != w.k or x.dtype != torch.bfloat16:
        raise NativeError(f"gemm_mid: x {tuple(x.shape)} {x.dtype} / w {w.shape}")
    m, k = x.shape
    n = w.n
    out_dtype = out_dtype or torch.bfloat16
    if bias is not None and bias.shape != (n,):
        raise NativeError(f"gemm_mid: bias {tuple(bias.shape)} is not [{n}]")
    if slices > 1:
        parts = torch.empty((slices, m, n), dtype=torch.float32, device=x.device)
        check(kernels().pa_gemm_mid(_stream(), _CODES[out_dtype], 0, _ptr(x), _ptr(w.data), _ptr(bias), None, _ptr(parts),
                                    m, n, k, k, n, slices, waves))
        return SliceSums(parts, out_dtype)
    cols = n // 2 if silu_mul_epilogue else n
    out = torch.empty((m, cols), dtype=out_dtype, device=x.device)
    check(kernels().pa_gemm_mid(_stream(), _CODES[out_dtype], epi, _ptr(x), _ptr(w.data),
                                _ptr(bias), _ptr(out), None, m, n, k, k, cols, 1, waves))
    return out


def gemm_tall(x: torch.Tensor, w: "TiledWeight", bias: Optional[torch.Tensor] = None, silu_mul_epilogue: bool = False,
              slices: int = 1, shape=(0, 0), activation: str = "silu"):
    """x [M, K] @ w[N, K]^T for any number of rows from the weight in tiles, the output tiled both ways: a
    workgroup owns ``16 * shape[0]`` rows of X and ``64 * shape[1]`` rows of W ((0, 0): the launcher chooses by the
    product's size; the same bits at every shape).  bfloat16 out; with ``slices`` > 1 a ``SliceSums``."""
    if not isinstance(w, TiledWeight):
        raise NativeError("gemm_tall takes the weight in tiles (pack_tiles)")
    epi = 1 + gate_activation_code(activation) if silu_mul_epilogue else 0
    _dev(x, w.data, bias)
    _f32(bias, "bias")
    if x.dim() != 2 or x.shape[1] != w.k or x.dtype != torch.bfloat16:
        raise NativeError(f"gemm_tall: x {tuple(x.shape)} {x.dtype} / w {w.shape}")
    m, k = x.shape
    n = w.n
    if bias is not None and bias.shape != (n,):
        raise NativeError(f"gemm_tall: bias {tuple(bias.shape)} is not [{n}]")
    if slices > 1:
        parts = torch.empty((slices, m, n), dtype=torch.float32, device=x.device)
        check(kernels().pa_gemm_tall(_stream(), 0, _ptr(x), _ptr(w.data), _ptr(bias), None, _ptr(parts), m, n, k, k, n,
                                     slices, int(shape[0]), int(shape[1])))
        return SliceSums(parts, torch.bfloat16)
    cols = n // 2 if silu_mul_epilogue else n
    out = torch.empty((m, cols), dtype=torch.bfloat16, device=x.device)
    check(kernels().pa_gemm_tall(_stream(), epi, _ptr(x), _ptr(w.data), _ptr(bias), _ptr(out),
                                 None, m, n, k, k, cols, 1, int(shape[0]), int(shape[1])))
    return out


# Where ``linear`` takes the product tiled both ways (``gemm_tall``) beyond the 128 rows of ``gemm_mid``.  Alone, with
# the weights coming from memory, it is ahead of the library for most products of 129 to 320 rows at the shapes of 4B, 8B
# and 32B models ([2560, 9728] at 256 rows in four slices 35.1 against 41.7 us, [4096, 12288] 46.5 against 54.8,
# [5120, 25600] 108 against 261; the gated [19456, 2560] 46.9 against 51.7 with the separate activation kernel); what
# decides is the prompt step it runs in, where the reader of slices pays for them (the norm reads four 32-bit partial
# sums instead of one bfloat16 tensor) -- a whole prompt through 36 layers, same box, library against this kernel:
#  - in four slices for the norm that follows, wide outputs only: hidden 4,096 at 129 / 160 / 192 / 256 rows 7.29 /
#    8.00 / 9.27 / 8.21 against 6.96 / 6.85 / 7.42 / 8.02 ms, level at 320 rows and behind from 384 on; hidden 2,560
#    5.01 / 5.20 / 5.43 / 6.56 against 5.34 / 5.49 / 5.78 / 6.39: the library's.  The very large weights of a 32B
#    model (a [5120, 25600] product alone: 163 against 271 us at 512 rows) up to 576 rows;
#  - the gated product with its activation in the epilogue, rows shorter than 4,096 columns: hidden 2,560 at 129 / 192 /
#    256 rows 5.01 / 5.43 / 6.56 against 4.76 / 5.23 / 6.34 ms, behind from 288 rows on (6.16 against 6.43);
#    [24576, 4096] is the library's at every number of rows (256 rows: 68.2 against 71.9 us);
#  - slices added by a kernel of their own for a reader of tensors (the QKV projection) lost everywhere (hidden
#    2,560 at 256 rows: 6.56 against 8.01 ms) and are not dispatched.
TALL_MAX_ROWS = 256
TALL_SLICED_MIN_N = 4096       # outputs at least this wide go to it in slices for the norm ...
TALL_HUGE_MAX_ROWS = 576       # ... and weights of TALL_HUGE_ELEMENTS up to this many rows
TALL_HUGE_ELEMENTS = 80 << 20        # [5120, 17408] at 384 and 512 rows: 127 and 134 us against the library's 141 and 175
TALL_GATED_MAX_K = 4096
TALL_PRODUCTS = 3              # ``set_tall_products``: which of these products ``gemm_tall`` takes (measurements):
#                                1 in slices for a reader of slices, 2 the gated one


def set_tall_products(on) -> None:
    global TALL_PRODUCTS
    TALL_PRODUCTS = 3 if on is True else int(on)


def _tall_slices(k: int) -> int:
    """Slices of the inner size for ``gemm_tall``: four where every slice still has eight steps of 64 columns."""
    steps = (k + 63) // 64
    for s in (4, 2):
        if steps >= 8 * s and -(-steps // -(-steps // s)) == s:
            return s
    return 1


def _tall_sliced(m: int, n: int, k: int) -> bool:
    if not TALL_PRODUCTS & 1 or m <= GEMM_MID_MAX_ROWS or k % 8 or n % 4 or n < TALL_SLICED_MIN_N:
        return False
    return m <= TALL_MAX_ROWS or (m <= TALL_HUGE_MAX_ROWS and n * k >= TALL_HUGE_ELEMENTS)


LIBRARY_WORKSPACE_BYTES = 76 << 20   # what the library's stream-K kernels may use for partial sums
_library_workspaces: dict = {}


def library_workspace_reserve(device) -> int:
    """Bytes the library product will still allocate on ``device`` at its first call (0 once it has)."""
    return 0 if torch.device(device) in _library_workspaces else LIBRARY_WORKSPACE_BYTES


def gemm_library(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y = x W^T in bfloat16 with 32-bit accumulation by hipBLASLt, called directly (its plan is kept per shape:
    a call through ``torch.matmul`` costs the host some 20 us, this one 14)."""
    _dev(x, w)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise NativeError(f"gemm_library: x {tuple(x.shape)} {x.dtype} / w {tuple(w.shape)} {w.dtype}")
    m, k = x.shape
    n = w.shape[0]
    ws = _library_workspaces.get(x.device)
    if ws is None:
        ws = _library_workspaces[x.device] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
    out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    check(kernels().pa_gemm_library(_stream(), _ptr(x), _ptr(w), _ptr(out), m, n, k, k, n, _ptr(ws), LIBRARY_WORKSPACE_BYTES))
    return out


def linear(x: torch.Tensor, w, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, slices_ok: bool = False):
    """y = x W^T (+ b), W [out, in] as a tensor or a ``LinearWeight``.  float32: our own true 32-bit product.
    bfloat16: few rows our weight-streaming kernel (from the tiled copy if the weight has one), above that the
    library product or, for the shapes they suit, the products with X staged in LDS (``gemm_mid`` to 128 rows,
    ``gemm_tall`` beyond); 32-bit accumulation in all.

    ``slices_ok``: the caller's reader adds slices itself (``rmsnorm`` does): a narrow weight at 17 to 128 rows
    (a wide one beyond, see ``TALL_MAX_ROWS``) then comes back as ``SliceSums`` (the product cut along its inner size, a 32-bit partial sum per slice)
    instead of a tensor."""
    tiles = None
    if isinstance(w, LinearWeight):
        w, tiles = w.rows, w.tiles
    if x.dtype == torch.float32:
        return gemm_plain(x, w, bias, out_dtype)
    _dev(x, w, bias)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise NativeError(f"linear: x {x.dtype} / w {w.dtype}")
    m, k = x.shape
    n = w.shape[0]
    # what a reader of slices gets from the product with X in LDS: from MID_SLICED_MIN_ROWS rows on where the rows are
    # long (the streaming kernel sums such a row in one workgroup: [2560, 9728] with the norm behind it 20.2 us
    # at 16 rows against 17.7 in four or eight slices, [5120, 25600] 60.4 against 50.6; at 8 rows and fewer it is
    # the other way round), from 17 rows on everywhere
    sliced = (MID_PRODUCTS and slices_ok and tiles is not None and k % 8 == 0 and n % 4 == 0 and m <= GEMM_MID_MAX_ROWS
              and out_dtype in (None, torch.bfloat16)
              and (m > SKINNY_MAX_ROWS or (m >= MID_SLICED_MIN_ROWS and k >= MID_SLICED_LONG_K)
                   # rows of 16,384 columns and more from 8 rows on ([5120, 17408] with the norm behind it 40.0
                   # against 42.6 us at 8 rows, [5120, 25600] 54.3 against 57.9; level at 4 rows)
                   or (m >= MID_SLICED_MIN_ROWS_LONG and k >= TILED_LONG_ROWS)))
    # (with four slices at most this holds just beyond 16 rows too, where eight slices lost to the streaming kernel:
    # with the norm that reads it, at 20 and 24 rows, [2560, 4096] 11.3 and 11.4 us against 12.2 and 13.0, [2048, 2048]
    # 8.7 against 9.0 and 9.2, [5120, 5120] 17.6 and 17.5 against 20.2 and 21.2; [4096, 4096] 14.6 and 14.9 against
    # 13.9 and 14.7 is the one shape the other way round)
    if SKINNY_SLICED and slices_ok and tiles is not None and k % 8 == 0 and n % 4 == 0 and out_dtype in (None, torch.bfloat16):
        s = _skinny_slices(m, n, k)
        if s > 1:
            return gemm_skinny_sliced(x, tiles, bias, slices=s, waves=8)
    if sliced:
        s = gemm_mid_slices(n, k)
        if s >= MID_MIN_SLICES:
            return gemm_mid(x, tiles, bias, slices=s)
    if m <= SKINNY_MAX_ROWS and k % 8 == 0:
        # a large weight whose reader wants a tensor, 9 to 16 rows: [10240, 5120] 22.5 us against the streaming
        # kernel's 27.5 at 12 rows (22.9 against 22.3 at 8); [7168, 5120] is the streaming kernel's (15.4 against 20.8)
        if (MID_PRODUCTS and tiles is not None and m >= MID_SLICED_MIN_ROWS and bias is None and n % 4 == 0
                and out_dtype in (None, torch.bfloat16) and n * k >= MID_SUMMED_MIN_ELEMENTS and k < TILED_LONG_ROWS):
            return gemm_mid(x, tiles)
        return gemm_skinny(x, tiles if tiles is not None and m <= 16 else w, bias, out_dtype)
    if (MID_PRODUCTS and tiles is not None and bias is None and k % 8 == 0 and n % 4 == 0 and m <= GEMM_MID_MAX_ROWS
            and out_dtype in (None, torch.bfloat16) and n * k >= MID_SUMMED_MIN_ELEMENTS and k < TILED_LONG_ROWS):
        s = gemm_mid_slices(n, k)
        if s >= MID_MIN_SLICES:
            return gemm_mid(x, tiles, slices=s).materialize()
    if MID_PRODUCTS and tiles is not None and k % 8 == 0 and m <= GEMM_MID_MAX_ROWS:
        if n >= MID_WIDE_ROWS and m <= (MID_WIDE_MAX_M if k <= MID_WIDE_SHORT_K else MID_WIDE_MAX_M // 2):
            return gemm_mid(x, tiles, bias, out_dtype)
    if tiles is not None and _tiled_beyond_16(m, w.shape[0], k):
        return gemm_skinny(x, tiles, bias, out_dtype)
    if tiles is not None and slices_ok and out_dtype in (None, torch.bfloat16) and _tall_sliced(m, n, k):
        s = _tall_slices(k)
        if s > 1:
            return gemm_tall(x, tiles, bias, slices=s)
    if k % 8:
        # rows that are no multiple of 16 bytes: neither the streaming kernel's loads nor the library's fast
        # kernels take them; the plain product does (bfloat16 in, 32-bit sums), and only odd toy sizes come here
        return gemm_plain(x, w, bias, out_dtype)
    y = gemm_library(x, w)
    if bias is not None:
        add_bias_(y, bias)
    if out_dtype is not None and out_dtype != y.dtype:
        y = to_f32(y)
    return y


# A narrow weight has too few tiles of 16 rows to give every compute unit a workgroup of the streaming kernel (160
# for 2,560 outputs, 64 for 1,024): for a reader of slices K is cut so that there are 256 to 480 workgroups.  Measured
# with the norm behind it, inside a graph, against what was dispatched before (us): [2560, 9728] in three slices
# 16.0 -> 14.9 at 6 rows, 16.8 -> 15.0 at 8, 16.5 -> 15.5 at 10, level at 4 and 12 and behind at 1, 2 and 16;
# [2048, 6144] in two 9.7 -> 8.9 at one row, 10.5 -> 9.5 at 8, 11.0 -> 9.9 at 16; [1024, 3072] in four 7.0 -> 6.5,
# 7.8 -> 7.0, 8.8 -> 7.3; [1024, 2048] in four 6.5 -> 6.3, 7.2 -> 6.8, 7.8 -> 7.0; nothing for [2048, 2048], [4096, 4096],
# [5120, 8192], and for [5120, 5120] at 6 to 8 rows only.
# (most tiles, slices, least k-steps, rows from, rows to)
SKINNY_SLICED_SHAPES = ((64, 4, 32, 1, 16), (128, 2, 64, 1, 16), (160, 3, 128, 4, 12))
SKINNY_SLICED = True    # ``set_skinny_sliced``: off sends these products where they went before (measurements)


def set_skinny_sliced(on: bool) -> None:
    global SKINNY_SLICED
    SKINNY_SLICED = bool(on)


def _skinny_slices(m: int, n: int, k: int) -> int:
    tiles, steps = (n + 15) // 16, (k + 63) // 64
    if k >= TILED_LONG_ROWS:      # rows this long have rules of their own (MID_SLICED_MIN_ROWS_LONG), measured at their shapes
        return 1
    for most_tiles, slices, least_steps, rows_from, rows_to in SKINNY_SLICED_SHAPES:
        if tiles <= most_tiles:
            return slices if steps >= least_steps and rows_from <= m <= rows_to else 1
    return 1


def as_tensor(x):
    """A product that may have come back as ``SliceSums``, as a tensor."""
    return x.materialize() if isinstance(x, SliceSums) else x


def set_skinny_max_rows(n: int) -> None:
    """Up to how many rows ``linear`` uses the weight-streaming kernel (for measurements)."""
    global SKINNY_MAX_ROWS
    SKINNY_MAX_ROWS = max(0, min(int(n), 64))


# The gated product keeps its activation in the streaming kernel's epilogue, which saves the library's separate
# SiLU*up kernel: measured in the decode step, that is the faster way up to 24 rows for [19456, 2560] (5.76 against
# 5.79 ms a step at 24 rows, 6.76 against 6.71 at 32) and up to 32 rows for [24576, 4096] (6.94 against 7.26 ms at
# 24 rows, 7.98 against 8.18 at 32); for [51200, 5120] the library with the separate kernel is ahead from 12 rows on
# Beyond 16 rows the product with X staged in LDS takes it, activation in its epilogue too: [19456, 2560] 20.3 us at
# 32 rows, 22.9 at 64 and 33.0 at 128 against the library's 27.3, 31.0 and 35.3 with the separate kernel (the
# streaming kernel: 30 and 47 at 32 and 64); [24576, 4096] 37.6 at 64 rows against 47.7; [51200, 5120] stays with the
# library (110 against 105 at 64 rows, 163 against 119 at 128).  The bounds below are for weights without tiles
# for that kernel to read, and for measurements with it switched off.
# Up to 16 rows the two kernels are close: [19456, 2560] takes the product with X in LDS 19.4 us at any number of rows
# and the streaming kernel 18.7 at one row, 20.0 at 8, 23.2 at 16; [24576, 4096] 35.0 against 35.8 to 36.7
GATED_MID_MIN_ROWS = 8         # ... for rows shorter than GATED_TILED_LONG_K columns; 1 for longer ones
GATED_TILED_ROWS = 24          # ... and 32 for rows of GATED_TILED_LONG_K columns or more
GATED_TILED_LONG_K = 4096
GATED_TILED_ELEMENTS = 1 << 27
# ... a [34816, 5120] weight too, up to 96 rows (63.4 against the streaming kernel's 70.7 us at 16 rows, 65.3 against
# the library's 79.3 at 20, 75.0 against 85.8 at 48, 95.9 against 97.1 at 96; 116.9 against 101.6 at 128), while
# [51200, 5120] is the library's from 12 rows on
GATED_LARGE_ELEMENTS = 200 << 20
GATED_LARGE_MAX_ROWS = 96
# ... and below this size the streaming kernel keeps 8 rows ([12288, 2048] 10.8 against 12.1 us, [6144, 1024] 4.8
# against 5.5; from 12 rows on the product with X in LDS is level or ahead)
GATED_SMALL_ELEMENTS = 40 << 20


def _gated_tiled(m: int, n: int, k: int) -> bool:
    return n * k <= GATED_TILED_ELEMENTS and k < 8192 and (m <= GATED_TILED_ROWS or (m <= 32 and k >= GATED_TILED_LONG_K))


def linear_gated(x: torch.Tensor, w, activation: str = "silu") -> torch.Tensor:
    """act(x Wg^T) * (x Wu^T) for a weight [2I, K] whose rows alternate gate_j, up_j; ``activation`` is ``"silu"``
    or ``"gelu_tanh"`` (the same kernels, another epilogue code)."""
    gate_activation_code(activation)
    m, k = x.shape
    if x.dtype == torch.bfloat16 and k % 8 == 0:
        tiles = w.tiles if isinstance(w, LinearWeight) else None
        if m <= SKINNY_MAX_ROWS:
            first = 1 if k >= GATED_TILED_LONG_K else GATED_MID_MIN_ROWS
            if tiles is not None and tiles.n * k < GATED_SMALL_ELEMENTS:
                first = GATED_MID_MIN_ROWS + 1
            elif tiles is not None and tiles.n * k > GATED_TILED_ELEMENTS:
                first = MID_SLICED_MIN_ROWS
            if MID_PRODUCTS and tiles is not None and tiles.n * k <= GATED_LARGE_ELEMENTS and m >= first:
                return gemm_mid(x, tiles, silu_mul_epilogue=True, activation=activation)
            if isinstance(w, LinearWeight):
                w = tiles if tiles is not None and m <= 16 else w.rows
            return gemm_skinny(x, w, silu_mul_epilogue=True, activation=activation)
        if MID_PRODUCTS and tiles is not None and (
                (m <= GEMM_MID_MAX_ROWS and tiles.n * k <= GATED_TILED_ELEMENTS)
                or (m <= GATED_LARGE_MAX_ROWS and tiles.n * k <= GATED_LARGE_ELEMENTS)):
            return gemm_mid(x, tiles, silu_mul_epilogue=True, activation=activation)
        if tiles is not None and _gated_tiled(m, tiles.n, k):
            return gemm_skinny(x, tiles, silu_mul_epilogue=True, activation=activation)
        if (TALL_PRODUCTS & 2 and tiles is not None and GEMM_MID_MAX_ROWS < m <= TALL_MAX_ROWS and k < TALL_GATED_MAX_K
                and tiles.n % 2 == 0):
            return gemm_tall(x, tiles, silu_mul_epilogue=True, activation=activation)
    return silu_mul(linear(x, w), activation)


# The residual add and RMSNorm in front of the gated product, inside that product (``gemm_mid`` stages X through LDS
# once per workgroup, and there are a few hundred workgroups, so adding the residual and multiplying by the gain as
# it stages costs little; the row's scale is applied to the finished sums): one kernel less in a decode step's layer.
# For up to 16 rows whose mixer output comes as a tensor, and weights of 40 M to 200 M elements: measured against
# the two kernels apart it gains 1.3 to 3 us at [19456, 2560], 2.3 to 3.8 us at [24576, 4096], 2.5 us up to 8 rows
# at [34816, 5120] (nothing at 12 rows, and it loses 1.5 us at 16), and loses 0.3 to 1.6 us at [6144, 1024] and
# [12288, 2048], where the streaming kernel is the better product.
NORMED_GATED = True              # ``set_normed_gated``: off runs the norm and the product apart (measurements)
NORMED_GATED_MAX_ROWS = 16
NORMED_GATED_MAX_ROWS_LARGE = 12   # ... for weights of more than GATED_TILED_ELEMENTS elements


def set_normed_gated(on: bool) -> None:
    global NORMED_GATED
    NORMED_GATED = bool(on)


def gated_after_norm_supported(x, residual, w, activation: str = "silu") -> bool:
    """Whether ``linear_gated_after_norm`` takes these operands (else: the norm, then ``linear_gated``)."""
    if not (NORMED_GATED and MID_PRODUCTS and isinstance(x, torch.Tensor) and isinstance(residual, torch.Tensor)
            and isinstance(w, LinearWeight) and w.tiles is not None and activation in GATE_ACTIVATIONS):
        return False
    m, k = x.shape
    return (x.dtype == torch.bfloat16 and residual.dtype == torch.bfloat16 and residual.shape == x.shape and x.is_contiguous()
            and residual.is_contiguous() and k % 8 == 0 and w.tiles.n % 2 == 0
            and GATED_SMALL_ELEMENTS <= w.tiles.n * k <= GATED_LARGE_ELEMENTS
            and 1 <= m <= (NORMED_GATED_MAX_ROWS if w.tiles.n * k <= GATED_TILED_ELEMENTS else NORMED_GATED_MAX_ROWS_LARGE))


def linear_gated_after_norm(x: torch.Tensor, residual: torch.Tensor, gain: torch.Tensor, eps: float, w,
                            activation: str = "silu", waves: int = 0):
    """(residual + x rounded once, act(h Wg^T) * (h Wu^T)) for h = rmsnorm(residual + x; gain, eps): the residual add,
    the norm and the gated product in one kernel.  The new residual is a tensor of its own."""
    _dev(x, residual, gain, w.tiles.data)
    _f32(gain, "gain")
    m, k = x.shape
    n = w.tiles.n
    if gain.shape != (k,) or w.tiles.k != k:
        raise NativeError(f"linear_gated_after_norm: x {tuple(x.shape)} / gain {tuple(gain.shape)} / w {w.tiles.shape}")
    res_out = torch.empty_like(residual)
    out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    check(kernels().pa_gemm_mid_normed(_stream(), 1 + gate_activation_code(activation), _ptr(x), _ptr(residual), _ptr(gain),
                                       float(eps), _ptr(res_out), _ptr(w.tiles.data), _ptr(out), m, n, k, k, n // 2, int(waves)))
    return res_out, out


def linear_silu_mul(x: torch.Tensor, w) -> torch.Tensor:
    """``linear_gated`` with SiLU, the reference's own feed-forward (crates/prelude-core/src/models/qwen3.rs:429-447)."""
    return linear_gated(x, w, "silu")


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      seq_of_token: torch.Tensor, positions: torch.Tensor, window: int, scale: float,
                      softcap: float = 0.0) -> torch.Tensor:
    """Paged causal attention, any mix of portions and decode tokens.  ``softcap`` > 0 (here and in the other
    attention entry points) bends every scaled score to ``softcap * tanh(score / softcap)`` before the softmax;
    0, the default, leaves the scores alone (the same bits as without the parameter).

    q [T, nh, hd]; K cache [pages, nkv, page, hd], V cache [pages, nkv, hd, page]; block_table int32 [B, stride];
    seq_of_token / positions int32 [T].  window 0 = all keys.
    """
    _dev(q, k_cache, v_cache, block_table, seq_of_token, positions)
    _i32(block_table, "block_table")
    _i32(seq_of_token, "seq_of_token")
    _i32(positions, "positions")
    if q.dim() != 3:
        raise NativeError(f"attention: q {tuple(q.shape)} is not [T, heads, head_dim]")
    t, nh, hd = q.shape
    _check_caches(k_cache, v_cache, k_cache.shape[1] if k_cache is not None and k_cache.dim() == 4 else -1, hd, q.dtype,
                  "attention")
    if seq_of_token.shape != (t,) or positions.shape != (t,) or block_table.dim() != 2:
        raise NativeError("attention: index arrays do not match the number of tokens")
    out = torch.empty_like(q)
    check(kernels().pa_attn_generic(_stream(), _code(q), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                    block_table.shape[1], _ptr(seq_of_token), _ptr(positions), _ptr(out), t, nh,
                                    k_cache.shape[1], hd, k_cache.shape[2], int(window), float(scale), float(softcap)))
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Index of the largest logit per row (lowest index among equals); logits float32 [R, V] -> int32 [R]."""
    _dev(logits)
    _f32(logits, "logits")
    if logits.dim() != 2:
        raise NativeError(f"argmax: logits {tuple(logits.shape)}")
    out = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
    words = kernels().pa_argmax_scratch(logits.shape[0], logits.shape[1])
    scratch = torch.empty((words,), dtype=torch.float32, device=logits.device) if words else None
    check(kernels().pa_argmax(_stream(), _ptr(logits), _ptr(out), _ptr(scratch), logits.shape[0], logits.shape[1]))
    return out


# Keys per split of the decode kernel: fixed, so which keys a split sums never depends on the batch.  (The order in
# which a split's steps are added does, in the last bits: grids of 769 to 1,536 workgroups run with two wavefronts a
# workgroup instead of four.  Steps of the same size on the same side of those limits give the same bits.)
DECODE_SPLIT_KEYS = 256
DECODE_CONTEXT_STEP = 1024   # the longest context of a step counts rounded up to this many tokens (whole pages)


def decode_context_bound(max_context: int, page_size: int) -> int:
    """The longest context of a step of single tokens, rounded up: the number of splits the decode kernels are
    launched for follows this bound and not the context itself, and so do the choices that follow the grid's size
    (wavefronts a workgroup, groups of the merge), which change a sum's last bits.  A step replayed from a graph
    knows only such a bound (the width of its block tables); with the same rounding a step run directly is launched
    alike and gives the same bits.

    Contexts of up to one split (256 keys) are a class of their own: one split needs no workspace and no merge, a
    launch less per layer where a whole step is a few hundred short kernels (a 28-layer model at 128 to 160 tokens of
    context: 233 launches a step with the merge, 205 without)."""
    first = max(1, DECODE_SPLIT_KEYS // page_size) * page_size
    if max_context <= first:
        return first
    step = max(1, DECODE_CONTEXT_STEP // page_size) * page_size
    return -(-max(int(max_context), 1) // step) * step


def _decode_splits(max_context: int, window: int, page_size: int) -> int:
    bound = decode_context_bound(max_context, page_size)
    if bound <= DECODE_SPLIT_KEYS:
        return 1            # every context lies in the first split, window or not
    span = min(bound, window + DECODE_SPLIT_KEYS) if window else bound
    return max(1, -(-span // DECODE_SPLIT_KEYS) + (1 if window else 0))


def mfma_attention_supported(head_dim: int, page_size: int) -> bool:
    return bool(kernels().pa_attn_mfma_supports(int(head_dim), int(page_size)))


def attention_decode(q, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens, out, max_context: int,
                     window: int, scale: float, every_seq: bool = False, softcap: float = 0.0) -> None:
    """Matrix-core attention for the sequences ``seq_ids`` (each feeding one token); writes their rows of ``out``.
    ``every_seq``: ``seq_ids`` is 0, 1, .. (a step of single tokens only); the kernels then count for themselves
    instead of reading it, which is one trip to memory less before their first key."""
    _dev(q, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens, out)
    t, nh, hd = q.shape
    _check_caches(k_cache, v_cache, k_cache.shape[1], hd, torch.bfloat16, "attention_decode")
    n = seq_ids.shape[0]
    if n == 0:
        return
    max_splits = _decode_splits(max_context, window, k_cache.shape[2])
    words = kernels().pa_attn_decode_workspace(n, nh, hd, max_splits)
    ws = torch.empty((max(words, 1),), dtype=torch.float32, device=q.device)
    check(kernels().pa_attn_decode(_stream(), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                   block_table.shape[1], None if every_seq else _ptr(seq_ids), _ptr(cu_q),
                                   _ptr(context_lens), _ptr(out),
                                   _ptr(ws), n, nh, k_cache.shape[1], hd, k_cache.shape[2], int(window), float(scale),
                                   float(softcap), DECODE_SPLIT_KEYS, max_splits))


def attention_decode_fused_supported(nh: int, nkv: int, hd: int, rot: int, page_size: int) -> bool:
    return bool(kernels().pa_attn_decode_fused_supports(int(nh), int(nkv), int(hd), int(rot), int(page_size)))


def attention_decode_fused(qkv, q_weight, k_weight, cos, sin, slots, eps: float, k_cache, v_cache,
                           block_table, seq_ids, cu_q, context_lens, nh: int, max_context: int, window: int,
                           scale: float, every_seq: bool = False, softcap: float = 0.0) -> torch.Tensor:
    """``qknorm_rope_kv`` and ``attention_decode`` in one kernel, for a step in which every sequence feeds one
    token: takes the merged projection [T, (nh + 2 nkv) * hd], writes the tokens' keys and values into the caches
    and returns the attention output [T, nh, hd].  A token's position is its sequence's context length less one.
    ``every_seq``: as in ``attention_decode``."""
    _dev(qkv, q_weight, k_weight, cos, sin, slots, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens)
    nkv, page, hd = k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    _check_caches(k_cache, v_cache, nkv, hd, torch.bfloat16, "attention_decode_fused")
    t = qkv.shape[0]
    if qkv.dtype != torch.bfloat16 or qkv.dim() != 2 or qkv.shape[1] != (nh + 2 * nkv) * hd or not qkv.is_contiguous():
        raise NativeError(f"attention_decode_fused: qkv {tuple(qkv.shape)} {qkv.dtype} for nh={nh} nkv={nkv} hd={hd}")
    _f32(q_weight, "q_weight")
    _f32(k_weight, "k_weight")
    _f32(cos, "cos")
    _f32(sin, "sin")
    _i32(slots, "slots")
    if cos.shape[1] != hd // 2 or sin.shape != cos.shape or slots.shape[0] != t:
        raise NativeError("attention_decode_fused: rotary tables or slots do not match the tokens")
    out = torch.empty((t, nh, hd), dtype=torch.bfloat16, device=qkv.device)
    n = seq_ids.shape[0]
    if n == 0:
        return out
    max_splits = _decode_splits(max_context, window, page)
    words = kernels().pa_attn_decode_workspace(n, nh, hd, max_splits)
    ws = torch.empty((max(words, 1),), dtype=torch.float32, device=qkv.device)
    check(kernels().pa_attn_decode_fused(_stream(), _ptr(qkv), _ptr(q_weight), _ptr(k_weight), _ptr(cos), _ptr(sin),
                                         _ptr(slots), float(eps), _ptr(k_cache), _ptr(v_cache),
                                         _ptr(block_table), block_table.shape[1],
                                         None if every_seq else _ptr(seq_ids), _ptr(cu_q),
                                         _ptr(context_lens), _ptr(out), _ptr(ws), n, nh, nkv, hd, page, int(window),
                                         float(scale), float(softcap), DECODE_SPLIT_KEYS, max_splits))
    return out


def attention_prefill(q, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens, out, max_q_len: int,
                      window: int, scale: float, cut=None, min_prefix: int = 0, softcap: float = 0.0) -> None:
    """Matrix-core attention for the sequences ``seq_ids`` (portions of several tokens); writes their rows of ``out``.

    ``min_prefix`` is the fewest keys any of the sequences has before its portion: a hint for how the launcher
    cuts the work (portions far into their contexts need no pairing of early and late tiles).
    ``cut`` (tests and measurements) fixes the cut instead: ``(paired, heads a wavefront, head groups a
    workgroup, staged)``, -1 for the launcher's choice."""
    _dev(q, k_cache, v_cache, block_table, seq_ids, cu_q, context_lens, out)
    t, nh, hd = q.shape
    _check_caches(k_cache, v_cache, k_cache.shape[1], hd, torch.bfloat16, "attention_prefill")
    n = seq_ids.shape[0]
    if n == 0:
        return
    args = (_stream(), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(seq_ids),
            _ptr(cu_q), _ptr(context_lens), _ptr(out), n, int(max_q_len), int(min_prefix), nh, k_cache.shape[1], hd,
            k_cache.shape[2], int(window), float(scale), float(softcap))
    if cut is None:
        check(kernels().pa_attn_prefill(*args))
    else:
        check(kernels().pa_attn_prefill_cut(*args, *(int(c) for c in cut)))


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, group, step, window: int,
              scale: float, softcap: float = 0.0) -> torch.Tensor:
    """Attention of one step over one cache group; picks the kernel for the sizes at hand.

    ``group`` is the step's ``GroupStep`` of the cache group, ``step`` the ``StepBatch``.
    bfloat16 with a head_dim and page size the matrix-core kernels take: single
    tokens go to the split decode kernel, portions to the prefill kernel.
    Everything else (float32, other sizes) goes to the generic kernel.
    """
    if q.dtype == torch.bfloat16 and step.decode_seqs is not None \
            and mfma_attention_supported(q.shape[2], k_cache.shape[2]):
        out = torch.empty_like(q)
        if step.n_decode:
            attention_decode(q, k_cache, v_cache, group.block_table, step.decode_seqs, step.cu_q, step.context_lens,
                             out, step.max_decode_context, window, scale,
                             every_seq=step.n_prefill == 0 and step.n_decode == step.num_seqs, softcap=softcap)
        if step.n_prefill:
            attention_prefill(q, k_cache, v_cache, group.block_table, step.prefill_seqs, step.cu_q, step.context_lens,
                              out, step.max_prefill_q, window, scale, min_prefix=step.min_prefill_prefix, softcap=softcap)
        return out
    return attention_generic(q, k_cache, v_cache, group.block_table, step.seq_of_token, step.positions, window, scale,
                             softcap)


def logprobs(logits: torch.Tensor, ids: torch.Tensor, k: int = 0):
    """Log-probabilities under softmax(logits[r]) of the tokens ``ids`` [R] (int32; negative = none, gives 0).

    Returns ``(lp [R] float32, top)``; with ``k`` > 0, ``top`` is ``(values [R, cap], indices [R, cap], count [R])``:
    the entries among each row's k largest with their log-probabilities, ties at the k-th value included, in no
    particular order (the caller sorts the few there are); else ``None``.
    """
    _dev(logits, ids)
    _f32(logits, "logits")
    _i32(ids, "ids")
    if logits.dim() != 2 or ids.shape != (logits.shape[0],):
        raise NativeError(f"logprobs: logits {tuple(logits.shape)} / ids {tuple(ids.shape)}")
    r, vocab = logits.shape
    k = int(k)
    lp = torch.empty(r, dtype=torch.float32, device=logits.device)
    top = None
    cap = 0
    if k > 0:
        cap = min(vocab, k + 32)
        top = (torch.empty((r, cap), dtype=torch.float32, device=logits.device),
               torch.empty((r, cap), dtype=torch.int32, device=logits.device),
               torch.empty(r, dtype=torch.int32, device=logits.device))
    check(kernels().pa_logprobs(_stream(), _ptr(logits), _ptr(ids), _ptr(lp), _ptr(top[0]) if top else None,
                                _ptr(top[1]) if top else None, _ptr(top[2]) if top else None, r, vocab, k, cap))
    return lp, top


SAMPLE_WIDE_FROM = 32768   # rows this long are sampled with every pass spread over the chip,
SAMPLE_WIDE_ROWS = 32      # up to this many at a time (more rows fill the chip with a workgroup each)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, any_top_k: bool = True, any_top_p: bool = True,
           wide: Optional[bool] = None) -> torch.Tensor:
    """One token per row of float32 logits [R, V]; per-row float32 temperature / top_p / uniform and int32 top_k.

    temperature < 1e-7: argmax.  Else a draw from softmax(logits / T) kept to the
    top_k largest (0 = all) and the shortest descending prefix of mass top_p
    (>= 1 = all), by inverse CDF in index order at uniform[r] in [0, 1).

    ``any_top_k`` / ``any_top_p`` false promise that no row has one, which spares long rows the passes of
    that search.  ``wide`` picks the kernel (one workgroup a row, or rows cut into slices over many
    workgroups); by default it follows the row length.  Both give the same token except where 32-bit
    rounding of the sums decides between neighbours.
    """
    _dev(logits, temperature, top_k, top_p, uniform)
    _f32(logits, "logits")
    _f32(temperature, "temperature")
    _f32(top_p, "top_p")
    _f32(uniform, "uniform")
    _i32(top_k, "top_k")
    r = logits.shape[0]
    if logits.dim() != 2 or any(t.shape != (r,) for t in (temperature, top_k, top_p, uniform)):
        raise NativeError("sample: per-row parameters do not match the rows of logits")
    out = torch.empty((r,), dtype=torch.int32, device=logits.device)
    vocab = logits.shape[1]
    if wide is None:
        wide = vocab >= SAMPLE_WIDE_FROM and r <= SAMPLE_WIDE_ROWS
    if wide and r > 0:
        ws = torch.empty(int(kernels().pa_sample_wide_workspace(r, vocab)), dtype=torch.uint8, device=logits.device)
        check(kernels().pa_sample_wide(_stream(), _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p),
                                       _ptr(uniform), _ptr(out), _ptr(ws), r, vocab,
                                       (1 if any_top_k else 0) | (2 if any_top_p else 0)))
        return out
    check(kernels().pa_sample(_stream(), _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform),
                              _ptr(out), r, vocab))
    return out
