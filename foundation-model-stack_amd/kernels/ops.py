"""The kernels as functions of torch tensors.

torch tensors are used as device buffers only; every computation below is a
HIP kernel of this package, with one exception that is named where it happens
(large bfloat16 matrix products go to the vendor library through
``torch.matmul``, as the reference's linear layers do).  Each wrapper checks on
the host what its kernel and grid assume before launching.
"""

from __future__ import annotations

import ctypes
import math
from typing import Optional

import torch

from .library import check, load

F32, BF16 = 0, 1
# the names of the reference (fms/utils/activation.py:14-24) and "identity"; the numbers are FMS_ACT_* of csrc/fmsamd.h
ACTIVATIONS = {"silu": 0, "swish": 0, "gelu": 1, "relu": 2, "identity": 3, "sigmoid": 4, "tanh": 5, "mish": 6,
               "gelu-tanh": 7, "gelu_pytorch_tanh": 7}
PAGE_TOKENS = 64


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise TypeError(f"fms_amd kernels take float32 and bfloat16, not {dtype}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need_cuda(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("fms_amd kernels run on the GPU only; got a CPU tensor (there is no CPU fallback)")


def _need_i32(name: str, t: torch.Tensor) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise TypeError(f"{name} must be a contiguous int32 tensor")


def _rows2d(name: str, t: torch.Tensor) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be 2-D with a contiguous last dimension, got shape {tuple(t.shape)} strides {t.stride()}")


# --------------------------------------------------------------------------
def embed(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """float32 rows of `table` for int32 `ids` [T] -> [T, width]."""
    _need_cuda(ids, table)
    _need_i32("ids", ids)
    if table.dim() != 2 or not table.is_contiguous():
        raise ValueError("embedding table must be a contiguous [vocab, width] tensor")
    out = torch.empty(ids.numel(), table.shape[1], dtype=torch.float32, device=table.device)
    check(load().fmsamd_embed(ids.data_ptr(), table.data_ptr(), _code(table.dtype), out.data_ptr(), ids.numel(),
                              table.shape[1], table.shape[0], _stream()))
    return out


def add_norm(
    resid: torch.Tensor,
    branch: Optional[torch.Tensor],
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    eps: float,
    out_dtype: torch.dtype,
    rows: Optional[torch.Tensor] = None,
    use_mean: bool = False,
) -> torch.Tensor:
    """resid += branch (in place, float32); returns norm(resid) * weight + bias in `out_dtype`.

    With `rows` (int32 indices) only those rows are produced and resid is left as it is.
    """
    _need_cuda(resid, branch, weight, bias, rows)
    if resid.dtype != torch.float32 or resid.dim() != 2 or not resid.is_contiguous():
        raise ValueError("the residual stream must be a contiguous float32 [T, width] tensor")
    T, width = resid.shape
    if branch is not None:
        if branch.shape != resid.shape or not branch.is_contiguous() or branch.dtype != out_dtype:
            raise ValueError(f"branch must be contiguous {tuple(resid.shape)} of {out_dtype}, got {tuple(branch.shape)} {branch.dtype}")
    wdtype = out_dtype
    for name, t in (("weight", weight), ("bias", bias)):
        if t is not None:
            if t.shape != (width,) or not t.is_contiguous():
                raise ValueError(f"norm {name} must be a contiguous [{width}] tensor, got {tuple(t.shape)}")
            wdtype = t.dtype
    if weight is not None and bias is not None and weight.dtype != bias.dtype:
        raise TypeError("norm weight and bias must have one dtype")
    n_out = T
    if rows is not None:
        _need_i32("rows", rows)
        n_out = rows.numel()
    out = torch.empty(n_out, width, dtype=out_dtype, device=resid.device)
    check(load().fmsamd_add_norm(resid.data_ptr(), _ptr(branch), _code(out_dtype), _ptr(weight), _ptr(bias), _code(wdtype),
                                 out.data_ptr(), _ptr(rows), n_out, width, float(eps), int(use_mean), _stream()))
    return out


def gated_act(gu: torch.Tensor, bias: Optional[torch.Tensor], activation: str) -> torch.Tensor:
    """[T, 2*hidden] (gate first) -> act(gate + b) * (up + b) [T, hidden]."""
    _need_cuda(gu, bias)
    if gu.dim() != 2 or not gu.is_contiguous() or gu.shape[1] % 2:
        raise ValueError("gated_act takes a contiguous [T, 2*hidden] tensor")
    T, hidden = gu.shape[0], gu.shape[1] // 2
    if bias is not None and (bias.shape != (2 * hidden,) or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous [{2 * hidden}] tensor")
    out = torch.empty(T, hidden, dtype=gu.dtype, device=gu.device)
    for t0 in range(0, T, 65535):
        n = min(65535, T - t0)
        check(load().fmsamd_gated_act(gu[t0:].data_ptr(), _ptr(bias), _code(bias.dtype) if bias is not None else 0,
                                      out[t0:].data_ptr(), _code(gu.dtype), n, hidden, ACTIVATIONS[activation], _stream()))
    return out


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    _need_cuda(x)
    if x.dtype == dtype:
        return x
    if not x.is_contiguous():
        raise ValueError("cast takes a contiguous tensor")
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    check(load().fmsamd_cast(x.data_ptr(), _code(x.dtype), out.data_ptr(), _code(dtype), x.numel(), _stream()))
    return out


def advance_positions_(positions: torch.Tensor, seq_of_token: torch.Tensor) -> None:
    """positions += 1 on the live rows (seq_of_token >= 0) of a fixed-size decode batch."""
    _need_cuda(positions, seq_of_token)
    _need_i32("positions", positions)
    _need_i32("seq_of_token", seq_of_token)
    if positions.numel() != seq_of_token.numel():
        raise ValueError("positions and seq_of_token must have one entry per row")
    check(load().fmsamd_advance_positions(positions.data_ptr(), seq_of_token.data_ptr(), positions.numel(), _stream()))


def bias_add_(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    _need_cuda(x, bias)
    if x.dim() != 2 or not x.is_contiguous() or bias.shape != (x.shape[1],) or not bias.is_contiguous():
        raise ValueError("bias_add_ takes a contiguous [rows, cols] tensor and a [cols] bias")
    check(load().fmsamd_bias_add(x.data_ptr(), _code(x.dtype), bias.data_ptr(), _code(bias.dtype), x.shape[0], x.shape[1], _stream()))
    return x


# --------------------------------------------------------------------------
def rope_table(freqs: torch.Tensor, max_pos: int):
    """cos and sin of position * freqs, float32 [max_pos, len(freqs)]."""
    _need_cuda(freqs)
    if freqs.dtype != torch.float32 or freqs.dim() != 1 or not freqs.is_contiguous():
        raise ValueError("freqs must be a contiguous float32 vector")
    half = freqs.numel()
    cos = torch.empty(max_pos, half, dtype=torch.float32, device=freqs.device)
    sin = torch.empty_like(cos)
    check(load().fmsamd_rope_table(freqs.data_ptr(), cos.data_ptr(), sin.data_ptr(), max_pos, half, _stream()))
    return cos, sin


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, kvheads: int, head_dim: int, dtype: torch.dtype) -> int:
    shape = (kvheads, PAGE_TOKENS, head_dim)
    if k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != shape or not k_cache.is_contiguous():
        raise ValueError(f"key cache must be contiguous [pages, {kvheads}, {PAGE_TOKENS}, {head_dim}], got {tuple(k_cache.shape)}")
    vshape = (kvheads, head_dim, PAGE_TOKENS)
    if v_cache.dim() != 4 or tuple(v_cache.shape[1:]) != vshape or not v_cache.is_contiguous():
        raise ValueError(f"value cache must be contiguous [pages, {kvheads}, {head_dim}, {PAGE_TOKENS}], got {tuple(v_cache.shape)}")
    if k_cache.dtype != dtype or v_cache.dtype != dtype or k_cache.shape[0] != v_cache.shape[0]:
        raise TypeError("key and value cache must have the dtype of the queries and equal page counts")
    return k_cache.shape[0]


def _check_batch_index(positions, seq_of_token, block_table, n_tokens: int) -> None:
    _need_i32("positions", positions)
    _need_i32("seq_of_token", seq_of_token)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise TypeError("block_table must be an int32 [sequences, pages] tensor")
    if positions.numel() < n_tokens or seq_of_token.numel() < n_tokens:
        raise ValueError("positions and seq_of_token must have an entry per token")


class RowNorm:
    """A row norm left to the product that reads the rows.  The rows hold stream * norm weight; `partials`
    [M, count] float32 are partial sums of squares of the stream's rows; the product multiplies its result
    by rsqrt(sum / K + eps) per row before the bias."""

    def __init__(self, partials: torch.Tensor, eps: float):
        if partials.dtype != torch.float32 or partials.dim() != 2 or not partials.is_contiguous():
            raise ValueError("the partial sums of a deferred row norm are a contiguous float32 [M, count] tensor")
        self.partials, self.eps = partials, float(eps)


def _skinny_workspace(rows: int, weight_rows: int, K: int, device):
    """(pointer, bytes) of the workspace a product for `rows` rows of x needs; (None, 0) up to 16 rows."""
    n = load().fmsamd_gemm_skinny_workspace(rows, weight_rows, K)
    if n <= 0:
        return None, 0
    ws = torch.empty(n // 4, dtype=torch.float32, device=device)
    return ws, n


class _RowScaleArg(ctypes.Structure):
    _fields_ = [("partials", ctypes.c_void_p), ("count", ctypes.c_int), ("eps", ctypes.c_float)]


def _row_scale(row_norm: Optional[RowNorm], rows: int):
    if row_norm is None:
        return None
    _need_cuda(row_norm.partials)
    if row_norm.partials.shape[0] != rows:
        raise ValueError(f"deferred row norm has {row_norm.partials.shape[0]} rows, the product {rows}")
    return ctypes.byref(_RowScaleArg(row_norm.partials.data_ptr(), row_norm.partials.shape[1], row_norm.eps))


def qkv_rope_write(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    positions: torch.Tensor,
    seq_of_token: torch.Tensor,
    block_table: torch.Tensor,
    cos: Optional[torch.Tensor],
    sin: Optional[torch.Tensor],
    rot_dim: int,
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    nheads: int,
    kvheads: int,
    head_dim: int,
    row_norm: Optional[RowNorm] = None,
) -> torch.Tensor:
    """The fused qkv projection of a decode step (at most QKV_ROPE_MAX_ROWS rows, bfloat16): x W^T (+ bias), q and k
    rotated, k and v written into their cache pages.  Returns the [M, (H+2K)*D] buffer whose query
    columns hold the rotated queries (its other columns are not written).  Equal to `linear` followed
    by `rope_kv_write`."""
    _need_cuda(x, weight, bias, positions, seq_of_token, block_table, cos, sin, k_cache, v_cache)
    _rows2d("x", x)
    M, K = x.shape
    N = (nheads + 2 * kvheads) * head_dim
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or tuple(weight.shape) != (N, K) or not weight.is_contiguous():
        raise ValueError(f"qkv_rope_write takes bfloat16 x [M, {K}] and a contiguous bfloat16 weight [{N}, {K}]")
    if M > QKV_ROPE_MAX_ROWS or K % 8 or x.stride(0) % 8 or N % 16:
        raise ValueError(f"qkv_rope_write: at most {QKV_ROPE_MAX_ROWS} rows, K a multiple of 8, the output row a multiple of 16")
    if bias is not None and (bias.shape != (N,) or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous [{N}] tensor")
    _check_batch_index(positions, seq_of_token, block_table, M)
    max_pos = 0
    if cos is not None:
        if cos.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] * 2 != rot_dim:
            raise ValueError("cos/sin tables must be float32 [max_pos, rot_dim/2]")
        if not (cos.is_contiguous() and sin.is_contiguous()):
            raise ValueError("cos/sin tables must be contiguous")
        max_pos = cos.shape[0]
    if k_cache is not None:
        _check_cache(k_cache, v_cache, kvheads, head_dim, torch.bfloat16)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    ws, ws_bytes = _skinny_workspace(M, N, K, x.device)
    check(load().fmsamd_qkv_rope_skinny_bf16(
        x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), _code(bias.dtype) if bias is not None else 0,
        out.data_ptr(), out.stride(0), M, K, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
        block_table.stride(0), _ptr(cos), _ptr(sin), rot_dim if cos is not None else 0, max_pos, _ptr(k_cache),
        _ptr(v_cache), nheads, kvheads, head_dim, _row_scale(row_norm, M), _ptr(ws), ws_bytes, _stream()))
    return out


QKV_ROPE_MAX_ROWS = 192


def rope_kv_write(
    qkv: torch.Tensor,
    positions: torch.Tensor,
    seq_of_token: torch.Tensor,
    block_table: torch.Tensor,
    cos: Optional[torch.Tensor],
    sin: Optional[torch.Tensor],
    rot_dim: int,
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    nheads: int,
    kvheads: int,
    head_dim: int,
) -> None:
    """Rotate q (in place, inside qkv) and k; write k and v of every token into its cache page.

    The caller guarantees (and the engine checks on the host) that every position is below the
    table length and that block_table holds a valid page for every (sequence, position // 64).
    """
    _need_cuda(qkv, positions, seq_of_token, block_table, cos, sin, k_cache, v_cache)
    _rows2d("qkv", qkv)
    T = qkv.shape[0]
    if qkv.shape[1] != (nheads + 2 * kvheads) * head_dim:
        raise ValueError(f"qkv has {qkv.shape[1]} columns, expected {(nheads + 2 * kvheads) * head_dim}")
    _check_batch_index(positions, seq_of_token, block_table, T)
    max_pos = 0
    if cos is not None:
        if cos.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] * 2 != rot_dim:
            raise ValueError("cos/sin tables must be float32 [max_pos, rot_dim/2]")
        if not (cos.is_contiguous() and sin.is_contiguous()):
            raise ValueError("cos/sin tables must be contiguous")
        max_pos = cos.shape[0]
    if k_cache is not None:
        _check_cache(k_cache, v_cache, kvheads, head_dim, qkv.dtype)
    check(load().fmsamd_rope_kv_write(qkv.data_ptr(), _code(qkv.dtype), qkv.stride(0), positions.data_ptr(),
                                      seq_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0),
                                      _ptr(cos), _ptr(sin), rot_dim if cos is not None else 0, max_pos, _ptr(k_cache),
                                      _ptr(v_cache), T, nheads, kvheads, head_dim, _stream()))


def attention(
    q: torch.Tensor,
    positions: torch.Tensor,
    seq_of_token: torch.Tensor,
    block_table: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    nheads: int,
    kvheads: int,
    head_dim: int,
    scale: float,
    window: int = 0,
    *,
    decode: bool = False,
    max_context: int = 0,
    qblock_start: Optional[torch.Tensor] = None,
    qblock_len: Optional[torch.Tensor] = None,
    qblock_tokens: int = 0,
    pages_per_block: int = 0,
    waves: int = 0,
    force_generic: bool = False,
    staged: Optional[bool] = None,
    row_order: Optional[torch.Tensor] = None,
    score_slopes: Optional[torch.Tensor] = None,
    soft_cap: float = 0.0,
) -> torch.Tensor:
    """Causal attention of every token over the cache of its sequence -> [T, nheads*head_dim].

    Further terms of the scores (a position encoding that acts on the scores, a capped attention): score_slopes,
    float32 [nheads], adds slope[head] * (key position - query position); soft_cap c > 0 turns a score s into
    c * tanh(s / c) first.  With either, both types run the generic kernel (the MFMA kernels have no such term).

    q is a [T, >= nheads*head_dim] view (the query columns of the qkv rows).  float32 runs the
    generic kernel; bfloat16 runs the MFMA kernels (prefill needs the query blocks, decode the
    largest context).  row_order (decode, optional): int32 [T], the token rows in the order in which the
    kernel's blocks are to take them, longest context first; the result does not depend on it.
    """
    _need_cuda(q, positions, seq_of_token, block_table, k_cache, v_cache)
    _rows2d("q", q)
    T = q.shape[0]
    _check_batch_index(positions, seq_of_token, block_table, T)
    _check_cache(k_cache, v_cache, kvheads, head_dim, q.dtype)
    out = torch.empty(T, nheads * head_dim, dtype=q.dtype, device=q.device)
    lib = load()
    common_tail = (T, nheads, kvheads, head_dim, float(scale), int(window), _stream())
    if score_slopes is not None:
        _need_cuda(score_slopes)
        if score_slopes.dtype != torch.float32 or tuple(score_slopes.shape) != (nheads,) or not score_slopes.is_contiguous():
            raise ValueError(f"score_slopes must be a contiguous float32 [{nheads}] tensor")
    if not (soft_cap >= 0.0 and math.isfinite(soft_cap)):
        raise ValueError(f"soft_cap {soft_cap} must be zero (none) or positive")
    if q.dtype == torch.float32 or force_generic or head_dim % 16 or score_slopes is not None or soft_cap > 0.0:
        for t0 in range(0, T, 65535):
            n = min(65535, T - t0)
            check(lib.fmsamd_attn_generic(q[t0:].data_ptr(), q.stride(0), out[t0:].data_ptr(), out.stride(0), _code(q.dtype),
                                          positions[t0:].data_ptr(), seq_of_token[t0:].data_ptr(), block_table.data_ptr(),
                                          block_table.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), n, *common_tail[1:-1],
                                          _ptr(score_slopes), float(soft_cap), common_tail[-1]))
        return out
    if decode:
        if max_context <= 0:
            raise ValueError("decode attention needs max_context (an upper bound of every context length)")
        n_pages = -(-max_context // PAGE_TOKENS)
        auto_pages, auto_waves = decode_split(T * kvheads, n_pages)
        if pages_per_block <= 0:
            pages_per_block = auto_pages
        if waves <= 0:
            waves = min(auto_waves, pages_per_block)
        n_splits = -(-n_pages // pages_per_block)
        if row_order is not None:
            _need_cuda(row_order)
            _need_i32("row_order", row_order)
            if row_order.numel() != T or not row_order.is_contiguous():
                raise ValueError(f"row_order has {row_order.numel()} entries for {T} tokens")
        ws_bytes = lib.fmsamd_attn_decode_workspace(T, nheads, head_dim, n_splits)
        ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.float32, device=q.device) if ws_bytes else None
        check(lib.fmsamd_attn_decode_bf16(q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), _ptr(ws), ws_bytes,
                                          positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
                                          block_table.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), T, nheads, kvheads,
                                          head_dim, float(scale), int(window), int(max_context), int(pages_per_block), int(waves),
                                          int(bool(staged)) if staged is not None else int(head_dim == 128), _ptr(row_order), _stream()))
        return out
    if qblock_start is None or qblock_len is None:
        raise ValueError("bfloat16 prefill attention needs the query blocks of the batch")
    _need_i32("qblock_start", qblock_start)
    _need_i32("qblock_len", qblock_len)
    check(lib.fmsamd_attn_prefill_bf16(q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), positions.data_ptr(),
                                       seq_of_token.data_ptr(), qblock_start.data_ptr(), qblock_len.data_ptr(),
                                       qblock_start.numel(), int(qblock_tokens), block_table.data_ptr(), block_table.stride(0),
                                       k_cache.data_ptr(), v_cache.data_ptr(), *common_tail))
    return out


def decode_split(rows: int, n_pages: int):
    """(pages per split, waves per block) of the decode attention kernel.

    rows = tokens x kv heads.  A compute unit pulls only a small share of the memory bandwidth, so
    the cache has to be spread over all of them: the context bound is cut into as many splits as give
    a few hundred blocks, and at least so many that a block has no more than 128 pages (every sequence
    deals its own pages out evenly over the splits; the waves of a block run their pages as a pipeline,
    so a block of many pages is cheaper than many blocks).  The waves of a block share its pages and merge in LDS, the blocks of a row
    merge in a second kernel."""
    by_rows = min(-(-256 // max(rows, 1)), max(1, n_pages // 8))  # but no splits of under 8 pages: one for each wave
    splits = max(1, min(max(by_rows, -(-n_pages // 128)), n_pages))
    pages = -(-n_pages // splits)
    waves = max(1, min(8 if rows * splits <= 512 else 4, pages))
    return pages, waves


def prefill_qblock(nheads: int, kvheads: int, head_dim: int, n_tokens: int) -> int:
    """The number of consecutive query tokens of one sequence that a block of the bfloat16 prefill
    kernel takes, for a step of n_tokens tokens; the step's query blocks are built with it."""
    return load().fmsamd_attn_prefill_qblock(nheads, kvheads, head_dim, n_tokens)


# --------------------------------------------------------------------------
# matrix products
# --------------------------------------------------------------------------
SKINNY_MAX_ROWS = 192
# Up to this many rows the skinny kernel, with the norms, rotation and activation fused into it, beats the
# vendor library followed by those as kernels of their own.
SKINNY_FAST_ROWS = 192


def linear(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
    allow_library: bool = True,
    row_norm: Optional[RowNorm] = None,
) -> torch.Tensor:
    """x [M, K] @ weight[N, K]^T (+ bias) -> [M, N].

    float32 x float32: the FMA kernel (true 32-bit).  bfloat16 x bfloat16: the weight-streaming
    skinny kernels up to 192 rows; above that the vendor library (hipBLASLt through torch.matmul,
    as the reference's nn.Linear does; for float32 output with the float32 sums as they are), or this
    package's MFMA kernel when allow_library is False.
    A float32 weight with bfloat16 activations (a tensor the checkpoint keeps in 32-bit) runs the
    float32 kernel on up-cast activations.
    """
    _need_cuda(x, weight, bias)
    _rows2d("x", x)
    if weight.dim() != 2 or not weight.is_contiguous():
        raise ValueError("weight must be a contiguous [N, K] tensor")
    M, K = x.shape
    N = weight.shape[0]
    if weight.shape[1] != K:
        raise ValueError(f"x has {K} columns, weight has {weight.shape[1]}")
    if bias is not None and (bias.shape != (N,) or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous [{N}] tensor")
    out_dtype = out_dtype or x.dtype
    lib = load()
    if row_norm is not None and not (weight.dtype == x.dtype == torch.bfloat16 and M <= SKINNY_FAST_ROWS):
        raise ValueError(f"a deferred row norm goes with the bfloat16 product of at most {SKINNY_FAST_ROWS} rows")
    if weight.dtype == torch.float32:
        xf = x if x.dtype == torch.float32 else cast(x.contiguous(), torch.float32)
        bf = bias if bias is None or bias.dtype == torch.float32 else cast(bias, torch.float32)
        out = torch.empty(M, N, dtype=torch.float32, device=x.device)
        for m0 in range(0, M, 65535 * 64):
            m = min(65535 * 64, M - m0)
            check(lib.fmsamd_gemm_f32(xf[m0:].data_ptr(), xf.stride(0), weight.data_ptr(), _ptr(bf), out[m0:].data_ptr(),
                                      out.stride(0), m, N, K, _stream()))
        return out if out_dtype == torch.float32 else cast(out, out_dtype)
    if weight.dtype != torch.bfloat16:
        raise TypeError(f"weights are float32 or bfloat16, not {weight.dtype}")
    if x.dtype != torch.bfloat16:
        raise TypeError("a bfloat16 weight takes bfloat16 activations")
    bcode = _code(bias.dtype) if bias is not None else 0
    if K % 8 or x.stride(0) % 8:
        # rows that are not 16-byte aligned: the element-wise kernel, so that no width is refused
        if row_norm is not None:
            raise ValueError("a deferred row norm goes with K and a row stride that are multiples of 8")
        out = torch.empty(M, N, dtype=out_dtype, device=x.device)
        for m0 in range(0, M, 65535 * 64):
            m = min(65535 * 64, M - m0)
            check(lib.fmsamd_gemm_bf16_any(x[m0:].data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), bcode,
                                           out[m0:].data_ptr(), _code(out_dtype), out.stride(0), m, N, K, _stream()))
        return out
    if M <= SKINNY_FAST_ROWS or (M <= SKINNY_MAX_ROWS and not (allow_library and out_dtype == torch.bfloat16)):
        out = torch.empty(M, N, dtype=out_dtype, device=x.device)
        ws, ws_bytes = _skinny_workspace(M, N, K, x.device)
        check(lib.fmsamd_gemm_skinny_bf16(x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), bcode, out.data_ptr(),
                                          _code(out_dtype), out.stride(0), M, N, K, _row_scale(row_norm, M), _ptr(ws),
                                          ws_bytes, _stream()))
        return out
    if allow_library and out_dtype in (torch.bfloat16, torch.float32):
        # vendor library GEMM, float32 accumulation; float32 results (the logits of many rows) come straight from the
        # accumulators, without a rounding to bfloat16 in between
        if out_dtype == torch.bfloat16:
            out = torch.matmul(x, weight.t())
        else:
            out = torch.mm(x, weight.t(), out_dtype=torch.float32)
        if bias is not None:
            bias_add_(out, bias)
        return out
    out = torch.empty(M, N, dtype=out_dtype, device=x.device)
    check(lib.fmsamd_gemm_bf16(x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), bcode, out.data_ptr(),
                               _code(out_dtype), out.stride(0), M, N, K, _stream()))
    return out


def linear_into_stream(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    resid: torch.Tensor,
    norm_weight: Optional[torch.Tensor],
    eps: float,
    row_norm: Optional[RowNorm] = None,
):
    """The last product of a residual branch with what follows it (bfloat16, at most SKINNY_FAST_ROWS rows):
    resid += x W^T (+ bias) in float32 in place.  Returns (scaled, RowNorm): scaled = resid * norm_weight in
    bfloat16 and the sums of squares of resid's rows by tiles of 16 columns, which a product takes as its
    `row_norm` to read the RMS-normed stream without a norm kernel in between."""
    _need_cuda(x, weight, bias, resid, norm_weight)
    _rows2d("x", x)
    _rows2d("resid", resid)
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.shape[1] != K or not weight.is_contiguous():
        raise ValueError(f"linear_into_stream takes bfloat16 x [M, {K}] and a contiguous bfloat16 weight [N, {K}]")
    if M > SKINNY_FAST_ROWS or K % 8 or x.stride(0) % 8:
        raise ValueError(f"linear_into_stream: at most {SKINNY_FAST_ROWS} rows, K and the row stride multiples of 8")
    if resid.dtype != torch.float32 or tuple(resid.shape) != (M, N):
        raise ValueError(f"the residual stream is float32 [{M}, {N}]")
    if bias is not None and (bias.shape != (N,) or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous [{N}] tensor")
    if norm_weight is not None and (norm_weight.shape != (N,) or not norm_weight.is_contiguous()
                                    or norm_weight.dtype not in (torch.float32, torch.bfloat16)):
        raise ValueError(f"the norm weight is a contiguous float32 or bfloat16 [{N}] tensor")
    scaled = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    lib = load()
    partials = torch.empty(M, lib.fmsamd_gemm_skinny_residual_partials(M, N, K), dtype=torch.float32, device=x.device)
    ws, ws_bytes = _skinny_workspace(M, N, K, x.device)
    check(lib.fmsamd_gemm_skinny_residual_bf16(
        x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), _code(bias.dtype) if bias is not None else 0,
        resid.data_ptr(), resid.stride(0), _ptr(norm_weight), _code(norm_weight.dtype) if norm_weight is not None else 0,
        scaled.data_ptr(), scaled.stride(0), partials.data_ptr(), partials.shape[1], M, N, K, _row_scale(row_norm, M),
        _ptr(ws), ws_bytes, _stream()))
    return scaled, RowNorm(partials, eps)


def gated_linear(
    x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], activation: str, allow_library: bool = True,
    row_norm: Optional[RowNorm] = None,
) -> torch.Tensor:
    """act(x Wg^T + bg) * (x Wu^T + bu) for weight = [Wg; Wu] stacked [2*hidden, K] -> [M, hidden]."""
    M = x.shape[0]
    if weight.shape[0] % 2:
        raise ValueError("the stacked gate/up weight needs an even number of rows")
    hidden = weight.shape[0] // 2
    if (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and M <= (SKINNY_FAST_ROWS if allow_library else SKINNY_MAX_ROWS)
            and x.dim() == 2 and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0):
        _need_cuda(x, weight, bias)
        _rows2d("x", x)
        K = x.shape[1]
        if weight.shape[1] != K or not weight.is_contiguous():
            raise ValueError("weight must be contiguous [2*hidden, K] with K the width of x")
        if bias is not None and (bias.shape != (2 * hidden,) or not bias.is_contiguous()):
            raise ValueError(f"bias must be a contiguous [{2 * hidden}] tensor")
        out = torch.empty(M, hidden, dtype=torch.bfloat16, device=x.device)
        ws, ws_bytes = _skinny_workspace(M, 2 * hidden, K, x.device)
        check(load().fmsamd_gemm_skinny_gated_bf16(x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias),
                                                   _code(bias.dtype) if bias is not None else 0, out.data_ptr(), BF16,
                                                   out.stride(0), M, hidden, K, ACTIVATIONS[activation],
                                                   _row_scale(row_norm, M), _ptr(ws), ws_bytes, _stream()))
        return out
    if row_norm is not None:
        raise ValueError(f"a deferred row norm goes with the bfloat16 product of at most {SKINNY_FAST_ROWS} rows")
    gu = linear(x, weight, None, allow_library=allow_library)
    return gated_act(gu, bias, activation)


# --------------------------------------------------------------------------
def sample(
    logits: torch.Tensor,
    do_sample: bool,
    temperature: float = 1.0,
    top_k: int = 0,
    rng_state: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """One token per row of float32 logits.  rng_state: int64 [rows, 2] (seed, counter), advanced in place."""
    _need_cuda(logits, rng_state, out)
    _rows2d("logits", logits)
    if logits.dtype != torch.float32:
        raise TypeError("logits are float32")
    rows, vocab = logits.shape
    if do_sample:
        if rng_state is None or rng_state.dtype != torch.int64 or tuple(rng_state.shape) != (rows, 2) or not rng_state.is_contiguous():
            raise ValueError("sampling needs a contiguous int64 [rows, 2] generator state")
        if not (temperature > 0 and math.isfinite(temperature)):
            raise ValueError(f"temperature {temperature} must be positive")
    if out is None:
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
    elif out.dtype != torch.int32 or out.numel() < rows or not out.is_contiguous():
        raise ValueError("out must be a contiguous int32 tensor with an entry per row")
    if not do_sample and vocab > 4096:
        lib = load()
        nbytes = lib.fmsamd_argmax_workspace(rows, vocab)
        ws = torch.empty(nbytes // 4, dtype=torch.float32, device=logits.device)
        check(lib.fmsamd_argmax(logits.data_ptr(), logits.stride(0), rows, vocab, ws.data_ptr(), nbytes, out.data_ptr(), _stream()))
        return out
    check(load().fmsamd_sample(logits.data_ptr(), logits.stride(0), rows, vocab, int(bool(do_sample)), float(temperature),
                               int(top_k or 0), _ptr(rng_state), out.data_ptr(), _stream()))
    return out


# --------------------------------------------------------------------------
def measured_peaks(read_mib: int = 1024, repeats: int = 5):
    """(bytes per second of a pure read, bfloat16 matrix flops per second) as measured on this GPU now: the best of
    `repeats` runs of a kernel that only reads a buffer of read_mib MiB, and of one that only issues matrix
    instructions on registers.  Takes about a tenth of a second."""
    lib = load()
    buffer = torch.empty(read_mib << 20, dtype=torch.uint8, device="cuda").zero_()
    out = torch.zeros(4, dtype=torch.float32, device="cuda")
    flops = ctypes.c_double(0.0)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best_ms(launch):
        launch()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(repeats):
            start.record()
            launch()
            end.record()
            torch.cuda.synchronize()
            best = min(best, start.elapsed_time(end))
        return best

    # the best of a few shapes of each: what the hardware can do, not what one launch shape happens to reach
    read_ms = min(best_ms(lambda b=blocks, c=contiguous: check(lib.fmsamd_probe_read(buffer.data_ptr(), buffer.numel(), b, c, out.data_ptr(), _stream())))
                  for blocks in (1024, 2048, 4096) for contiguous in (0, 1))
    mfma = 0.0
    for large in (0, 1):
        for blocks in (256 * 2, 256 * 4):
            ms = best_ms(lambda: check(lib.fmsamd_probe_mfma(blocks, 512, large, out.data_ptr(), ctypes.byref(flops), _stream())))
            mfma = max(mfma, flops.value / (ms / 1000))
    return buffer.numel() / (read_ms / 1000), mfma
