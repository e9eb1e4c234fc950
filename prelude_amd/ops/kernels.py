"""Python faces of the HIP kernels: shape and type checks on the host, then one launch.

Every function works on CUDA (HIP) tensors and launches on torch's current
stream.  Nothing here computes on the CPU or through a torch operator, except
``linear`` in bfloat16 for tall inputs, which calls the library matrix product
(hipBLASLt through ``torch.matmul``) where the reference calls its GEMM
libraries (crates/prelude-cuda/src/ops/gemm.rs:35-137).
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


def _stream() -> int:
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


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: Optional[torch.Tensor] = None,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm over the last axis of x [T, H] with a float32 weight [H].

    With ``residual`` the norm is taken of x + residual (32-bit sum) and the
    residual tensor receives the sum.  With ``rows`` (int32 [R]) only those
    rows are normed, into a compact [R, H] output, and the residual is read only.
    """
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


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up for gate_up [T, 2I] (gate columns first) -> [T, I]."""
    _dev(gate_up)
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise NativeError(f"silu_mul: input {tuple(gate_up.shape)} is not [T, 2I]")
    inter = gate_up.shape[1] // 2
    out = torch.empty((gate_up.shape[0], inter), dtype=gate_up.dtype, device=gate_up.device)
    check(kernels().pa_silu_mul(_stream(), _code(gate_up), _ptr(gate_up), _ptr(out), gate_up.shape[0], inter))
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


def qknorm_rope_kv(qkv: torch.Tensor, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                   cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
                   slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   num_heads: int, num_kv_heads: int, head_dim: int, rotary_dim: int, eps: float) -> torch.Tensor:
    """Per-head RMSNorm of Q and K, rotation by position, K and V into the paged cache.

    qkv [T, (nh + 2 nkv) * hd]; returns q [T, nh, hd].  With ``slots`` None
    nothing is written to the cache (then ``num_kv_heads`` may be 0 for a
    Q-only input).  Caches are [pages, nkv, page_size, hd].
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
        if k_cache is None or v_cache is None or k_cache.shape != v_cache.shape or k_cache.dim() != 4 \
                or k_cache.shape[1] != num_kv_heads or k_cache.shape[3] != head_dim \
                or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype:
            raise NativeError(f"qknorm_rope_kv: caches must be [pages, {num_kv_heads}, page, {head_dim}] of {qkv.dtype}")
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


def linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y = x W^T (+ b), W [out, in].  float32: our own true 32-bit product.
    bfloat16: the library product with 32-bit accumulation."""
    if x.dtype == torch.float32:
        return gemm_plain(x, w, bias, out_dtype)
    _dev(x, w, bias)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise NativeError(f"linear: x {x.dtype} / w {w.dtype}")
    y = torch.matmul(x, w.t())
    if bias is not None:
        add_bias_(y, bias)
    if out_dtype is not None and out_dtype != y.dtype:
        y = to_f32(y)
    return y


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_table: torch.Tensor,
                      seq_of_token: torch.Tensor, positions: torch.Tensor, window: int, scale: float) -> torch.Tensor:
    """Paged causal attention, any mix of portions and decode tokens.

    q [T, nh, hd]; caches [pages, nkv, page, hd]; block_table int32 [B, stride];
    seq_of_token / positions int32 [T].  window 0 = all keys.
    """
    _dev(q, k_cache, v_cache, block_table, seq_of_token, positions)
    _i32(block_table, "block_table")
    _i32(seq_of_token, "seq_of_token")
    _i32(positions, "positions")
    if q.dim() != 3 or k_cache.dim() != 4 or k_cache.shape != v_cache.shape or k_cache.shape[3] != q.shape[2] \
            or k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise NativeError(f"attention: q {tuple(q.shape)} {q.dtype} / cache {tuple(k_cache.shape)} {k_cache.dtype}")
    t, nh, hd = q.shape
    if seq_of_token.shape != (t,) or positions.shape != (t,) or block_table.dim() != 2:
        raise NativeError("attention: index arrays do not match the number of tokens")
    out = torch.empty_like(q)
    check(kernels().pa_attn_generic(_stream(), _code(q), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table),
                                    block_table.shape[1], _ptr(seq_of_token), _ptr(positions), _ptr(out), t, nh,
                                    k_cache.shape[1], hd, k_cache.shape[2], int(window), float(scale)))
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """Index of the largest logit per row (lowest index among equals); logits float32 [R, V] -> int32 [R]."""
    _dev(logits)
    _f32(logits, "logits")
    if logits.dim() != 2:
        raise NativeError(f"argmax: logits {tuple(logits.shape)}")
    out = torch.empty((logits.shape[0],), dtype=torch.int32, device=logits.device)
    check(kernels().pa_argmax(_stream(), _ptr(logits), _ptr(out), logits.shape[0], logits.shape[1]))
    return out


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, group, step, window: int,
              scale: float) -> torch.Tensor:
    """Attention of one step over one cache group; picks the kernel for the sizes at hand.

    ``group`` is the step's ``GroupStep`` of the cache group, ``step`` the ``StepBatch``.
    """
    return attention_generic(q, k_cache, v_cache, group.block_table, step.seq_of_token, step.positions, window, scale)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor) -> torch.Tensor:
    """One token per row of float32 logits [R, V]; per-row float32 temperature / top_p / uniform and int32 top_k.

    temperature < 1e-7: argmax.  Else a draw from softmax(logits / T) kept to the
    top_k largest (0 = all) and the shortest descending prefix of mass top_p
    (>= 1 = all), by inverse CDF in index order at uniform[r] in [0, 1).
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
    check(kernels().pa_sample(_stream(), _ptr(logits), _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(uniform),
                              _ptr(out), r, logits.shape[1]))
    return out
