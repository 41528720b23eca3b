"""Typed Python entry points of the HIP kernels.

Each function checks on the host that the operands have the shapes, dtypes and
layout its kernel assumes (a kernel never sees a shape it was not written for),
then launches on torch's current HIP stream.  There is no CPU path: tensors must
live on the GPU.
"""
from __future__ import annotations

import ctypes
import dataclasses
import functools
import itertools
import math
import os

import torch

from . import lib

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}
MAX_HEAD_DIM = 512
_GRID_Y_MAX = 65535


class ShapeError(ValueError):
    """Operands that a kernel was not written for."""


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise ShapeError(f"unsupported element type {t.dtype}; kernels take float32 and bfloat16")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Handle of the current stream of the current device (the raw call is many times cheaper than building a
    Stream object, and this runs once per kernel launch)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ShapeError(msg)


def _gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ShapeError("arle_amd kernels run on the GPU only; got a CPU tensor")


def _rows(t: torch.Tensor, name: str) -> None:
    _need(t.dim() == 2 and t.stride(1) == 1, f"{name} must be 2-D with contiguous rows")


def _i32(t, name: str, n: int | None = None) -> None:
    _need(t.dtype == torch.int32 and t.dim() == 1 and t.is_contiguous(), f"{name} must be int32 1-D")
    if n is not None:
        _need(t.numel() == n, f"{name} must have {n} entries, has {t.numel()}")


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


# ------------------------------------------------------------------ embedding


def embed_gather(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor | None = None, scale: float = 1.0):
    """out[t, :] = float32(table[ids[t], :]) * scale.  ids must already be checked to lie in range."""
    _gpu(table, ids, out)
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [V, H]")
    _i32(ids, "ids")
    tokens, hidden = ids.numel(), table.shape[1]
    if out is None:
        out = torch.empty((tokens, hidden), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (tokens, hidden) and out.is_contiguous(),
          "embed_gather output must be contiguous float32 [T, H]")
    lib.call("arle_embed_gather", table.data_ptr(), _code(table), ids.data_ptr(), out.data_ptr(),
             tokens, hidden, float(scale), _stream())
    return out


def silu_mul_interleaved(gate_up: torch.Tensor, block: int = 16):
    """out[:, j] = silu(g_j) * u_j for a [T, 2I] buffer whose columns alternate between `block` gate
    columns and the `block` matching up columns."""
    _gpu(gate_up)
    _rows(gate_up, "gate_up")
    tokens, two_i = gate_up.shape
    _need(block > 0 and two_i % (2 * block) == 0, "interleaved gate/up width must be a multiple of 2*block")
    width = two_i // 2
    _need(math.ceil(width / 256) <= _GRID_Y_MAX, "silu_mul: width too large")
    out = torch.empty((tokens, width), dtype=gate_up.dtype, device=gate_up.device)
    lib.call("arle_silu_mul", gate_up.data_ptr(), gate_up.data_ptr(), gate_up.stride(0), out.data_ptr(),
             _code(gate_up), tokens, width, int(block), _stream())
    return out


def silu_mul(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor | None = None):
    """out = silu(gate) * up for two [T, I] views with the same row stride."""
    _gpu(gate, up, out)
    _rows(gate, "gate")
    _rows(up, "up")
    _need(gate.shape == up.shape and gate.dtype == up.dtype and gate.stride(0) == up.stride(0),
          "gate and up must agree in shape, dtype and row stride")
    tokens, width = gate.shape
    _need(math.ceil(width / 256) <= _GRID_Y_MAX, "silu_mul: width too large")
    if out is None:
        out = torch.empty((tokens, width), dtype=gate.dtype, device=gate.device)
    _need(out.shape == (tokens, width) and out.dtype == gate.dtype and out.is_contiguous(),
          "silu_mul output must be contiguous [T, I] of the input type")
    lib.call("arle_silu_mul", gate.data_ptr(), up.data_ptr(), gate.stride(0), out.data_ptr(),
             _code(gate), tokens, width, 0, _stream())
    return out


# ----------------------------------------------------------------------- norms


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
            rows: torch.Tensor | None = None, out: torch.Tensor | None = None):
    """out[r] = x[src(r)] / sqrt(mean(x^2) + eps) * weight;  src(r) = rows[r] or r."""
    _gpu(x, weight, rows, out)
    _rows(x, "x")
    width = x.shape[1]
    _need(weight.shape == (width,) and weight.is_contiguous(), "norm weight must be [width]")
    n_rows = x.shape[0]
    if rows is not None:
        _i32(rows, "rows")
        n_rows = rows.numel()
    if out is None:
        out = torch.empty((n_rows, width), dtype=out_dtype, device=x.device)
    _need(out.shape == (n_rows, width) and out.dtype == out_dtype and out.is_contiguous(),
          "rmsnorm output must be contiguous [rows, width]")
    lib.call("arle_rmsnorm", x.data_ptr(), _code(x), x.stride(0), weight.data_ptr(), _code(weight),
             out.data_ptr(), _code(out), _ptr(rows), n_rows, width, float(eps), _stream())
    return out


def add_rmsnorm(residual: torch.Tensor, delta: torch.Tensor, weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: torch.Tensor | None = None,
                out: torch.Tensor | None = None):
    """residual += delta (float32, in place unless `rows` is given); out = rmsnorm(residual).

    delta is [T, H], or a stack [S, T, H] of partial sums that are added in the order of the stack
    (what a matrix product with K split over workgroups leaves behind)."""
    _gpu(residual, delta, weight, rows, out)
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(),
          "residual must be contiguous float32 [T, H]")
    _need(delta.dim() in (2, 3) and tuple(delta.shape[-2:]) == tuple(residual.shape) and delta.is_contiguous()
          and delta.dtype in _CODES and (delta.dim() == 2 or delta.shape[0] >= 1),
          "delta must match the residual ([T, H] or a stack [S, T, H])")
    n_delta = delta.shape[0] if delta.dim() == 3 else 1
    width = residual.shape[1]
    _need(weight.shape == (width,) and weight.is_contiguous(), "norm weight must be [width]")
    n_rows = residual.shape[0]
    if rows is not None:
        _i32(rows, "rows")
        n_rows = rows.numel()
    if out is None:
        out = torch.empty((n_rows, width), dtype=out_dtype, device=residual.device)
    _need(out.shape == (n_rows, width) and out.dtype == out_dtype and out.is_contiguous(),
          "add_rmsnorm output must be contiguous [rows, width]")
    lib.call("arle_add_rmsnorm", residual.data_ptr(), delta.data_ptr(), n_delta, residual.numel(), _code(delta),
             weight.data_ptr(), _code(weight), out.data_ptr(), _code(out), _ptr(rows), n_rows, width,
             float(eps), _stream())
    return out


# ------------------------------------------------------------------- products


def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor | None = None):
    """out[M, N] = a[M, K] . w[N, K]^T in true float32, fixed k order."""
    _gpu(a, w, out)
    _rows(a, "a")
    _rows(w, "w")
    _need(a.dtype == torch.float32 and w.dtype == torch.float32, "gemm_f32 takes float32 operands")
    M, K = a.shape
    N = w.shape[0]
    _need(w.shape[1] == K, f"gemm_f32: inner sizes differ ({K} vs {w.shape[1]})")
    _need(math.ceil(M / 64) <= _GRID_Y_MAX, "gemm_f32: too many rows for one launch")
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=a.device)
    _rows(out, "out")
    _need(out.shape == (M, N) and out.dtype == torch.float32, "gemm_f32 output must be float32 [M, N]")
    lib.call("arle_gemm_f32", a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(),
             out.stride(0), M, N, K, _stream())
    return out


# ------------------------------------------------------ q/k preparation + cache


def qk_prep(q, k, v, *, num_q_heads: int, num_kv_heads: int, head_dim: int, eps: float,
            q_weight=None, k_weight=None, cos=None, sin=None, rotary_dim: int = 0,
            positions=None, slot_of_token=None, block_table=None, k_pages=None, v_pages=None,
            page_size: int = 0, parts=None):
    """Per-head norm + rotation of q and k in place; k and v written to the paged cache.

    q [T, nq*D], k, v [T, nkv*D] (row views of one fused buffer are fine).  With no
    cache given k is rewritten in place and v is left alone.

    parts: float32 [S, T, (nq + 2 nkv) * D], a stack of partial products of the fused q|k|v projection.
    Then the values are the sums over the stack (in order), q is an output only, and k, v are None:
    they go to the cache, which must be given unless num_kv_heads is 0 (a layer that only needs q).
    """
    _gpu(q, k, v, q_weight, k_weight, cos, sin, positions, slot_of_token, block_table, k_pages, v_pages, parts)
    tokens = q.shape[0]
    D = head_dim
    _need(0 < D <= MAX_HEAD_DIM, f"head_dim {D} is outside the supported range 1..{MAX_HEAD_DIM}")
    part_args = (0, 0, 0, 0)
    if parts is not None:
        width = (num_q_heads + 2 * num_kv_heads) * D
        _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[0] >= 1
              and tuple(parts.shape[1:]) == (tokens, width) and parts.is_contiguous(),
              f"parts must be contiguous float32 [S, {tokens}, {width}]")
        _need(k is None and v is None, "with parts, k and v are not given: they go to the cache")
        _need(num_kv_heads == 0 or k_pages is not None, "with parts, k and v need the cache to go to")
        _rows(q, "q")
        _need(q.shape == (tokens, num_q_heads * D), "q must be [T, heads*D]")
        part_args = (parts.data_ptr(), parts.shape[0], tokens * width, width)
        k = v = q   # never read or written in this mode
    else:
        for name, t, heads in (("q", q, num_q_heads), ("k", k, num_kv_heads), ("v", v, num_kv_heads)):
            _rows(t, name)
            _need(t.shape == (tokens, heads * D), f"{name} must be [T, heads*D]")
            _need(t.dtype == q.dtype, "q, k and v must share one element type")
    _need((q_weight is None) == (k_weight is None), "give both q and k norm weights or neither")
    w_code = F32
    if q_weight is not None:
        _need(q_weight.shape == (D,) and k_weight.shape == (D,) and q_weight.dtype == k_weight.dtype
              and q_weight.is_contiguous() and k_weight.is_contiguous(),
              "q/k norm weights must be [head_dim] of one type")
        w_code = _code(q_weight)
    _i32(positions, "positions", tokens)
    if rotary_dim:
        _need(rotary_dim % 2 == 0 and rotary_dim <= D, "rotary_dim must be even and <= head_dim")
        _need(cos is not None and sin is not None and cos.dtype == torch.float32
              and sin.dtype == torch.float32 and cos.dim() == 2 and cos.shape == sin.shape
              and cos.shape[1] == rotary_dim // 2 and cos.is_contiguous() and sin.is_contiguous(),
              "cos/sin must be contiguous float32 [positions, rotary_dim/2]")
    table_stride = 0
    if k_pages is not None or v_pages is not None:
        _need(k_pages is not None and v_pages is not None, "give both k and v pages or neither")
        _need(page_size > 0, "page_size must be positive")
        _check_pages(k_pages, v_pages, num_kv_heads, page_size, D, q.dtype)
        _i32(slot_of_token, "slot_of_token", tokens)
        _need(block_table is not None and block_table.dtype == torch.int32 and block_table.dim() == 2
              and block_table.is_contiguous(), "block_table must be contiguous int32 [slots, pages]")
        table_stride = block_table.shape[1]
    heads = num_q_heads + 2 * num_kv_heads
    _need(math.ceil(heads / 4) <= _GRID_Y_MAX, "too many heads")
    lib.call("arle_qk_prep", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(),
             v.stride(0), _code(q), _ptr(q_weight), _ptr(k_weight), w_code, _ptr(cos), _ptr(sin),
             int(rotary_dim), positions.data_ptr(), _ptr(slot_of_token), _ptr(block_table),
             table_stride, _ptr(k_pages), _ptr(v_pages), tokens, num_q_heads, num_kv_heads, D,
             int(page_size), float(eps), *part_args, _stream())


# ------------------------------------------------------------------ attention


def _check_pages(k_pages, v_pages, nkv, page_size, D, dtype):
    """Keys [pages, nkv, page_size, D]; values d-major inside a page [pages, nkv, D, page_size]."""
    _need(k_pages.dim() == 4 and tuple(k_pages.shape[1:]) == (nkv, page_size, D) and k_pages.is_contiguous()
          and k_pages.dtype == dtype, "k_pages must be contiguous [pages, nkv, page_size, D]")
    _need(v_pages.dim() == 4 and tuple(v_pages.shape[1:]) == (nkv, D, page_size) and v_pages.is_contiguous()
          and v_pages.dtype == dtype and v_pages.shape[0] == k_pages.shape[0],
          "v_pages must be contiguous [pages, nkv, D, page_size]")


def _check_paged(q, out, k_pages, v_pages, block_table, positions, slot_of_token, nq, nkv, D,
                 page_size):
    _gpu(q, out, k_pages, v_pages, block_table, positions, slot_of_token)
    tokens = q.shape[0]
    _rows(q, "q")
    _rows(out, "out")
    _need(q.shape == (tokens, nq * D) and out.shape == (tokens, nq * D) and out.dtype == q.dtype,
          "q and out must be [T, nq*D] of one type")
    _need(nkv > 0 and nq % nkv == 0, "number of q heads must be a multiple of the kv heads")
    _check_pages(k_pages, v_pages, nkv, page_size, D, q.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    _i32(positions, "positions", tokens)
    _i32(slot_of_token, "slot_of_token", tokens)


def attn_paged_simt(q, out, k_pages, v_pages, block_table, positions, slot_of_token, *,
                    num_q_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                    scale: float, window: int = 0, row_list=None):
    """Causal attention of every token row (or of `row_list`) over its request's cached keys."""
    _check_paged(q, out, k_pages, v_pages, block_table, positions, slot_of_token, num_q_heads,
                 num_kv_heads, head_dim, page_size)
    _need(0 < head_dim <= MAX_HEAD_DIM, f"head_dim {head_dim} outside 1..{MAX_HEAD_DIM}")
    _need(num_q_heads <= _GRID_Y_MAX, "too many heads")
    n_rows = q.shape[0]
    if row_list is not None:
        _gpu(row_list)
        _i32(row_list, "row_list")
        n_rows = row_list.numel()
    lib.call("arle_attn_paged_simt", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0),
             k_pages.data_ptr(), v_pages.data_ptr(), _code(q), block_table.data_ptr(),
             block_table.shape[1], positions.data_ptr(), slot_of_token.data_ptr(), _ptr(row_list),
             n_rows, num_q_heads, num_kv_heads, head_dim, page_size, float(scale), int(window),
             _stream())
    return out


MFMA_MAX_HEAD_DIM = 256
_MFMA_TARGET_WAVES = 768    # workgroups wanted for a decode launch: three a compute unit (measured in whole decode steps at batch 4..64; 2,048 gave 3 % less at batch 8, 5 % less at batch 32)


def attn_mfma_supported(dtype, head_dim: int, page_size: int) -> bool:
    return (dtype == torch.bfloat16 and head_dim % 16 == 0 and 0 < head_dim <= MFMA_MAX_HEAD_DIM
            and page_size >= 4 and page_size & (page_size - 1) == 0)


def decode_split_cap(max_kv_len: int) -> int:
    """Most splits worth making for keys up to max_kv_len: at least two 32-key blocks each, at most 64
    (the merge keeps the statistics of one split in each lane of a wave), and a power of two, so that a
    context that grows passes through few different values (a captured decode step is made for one)."""
    most = max(1, min(-(-max_kv_len // 32) // 2, 64))
    return 1 << (most.bit_length() - 1)


_ATTN_ROW_TILE = 16   # rows of the matrix-core tile: a segment with more rows goes to the LDS kernel


def decode_splits(segments: int, num_kv_heads: int, max_kv_len: int) -> int:
    """Split-KV factor of a step of single decoded tokens: enough waves to fill the chip."""
    return max(1, min(-(-_MFMA_TARGET_WAVES // (segments * num_kv_heads)), decode_split_cap(max_kv_len)))


_PORTION_SPLITS_MAX = 8         # parts into which the keys of a portion's row block may be cut
_PORTION_ROWS = 128             # rows of a row block of the portions kernel
_PORTION_LIST_MAX = 16384       # (row block, segment) pairs that its work list holds
_PORTION_WS_BYTES = 256 << 20   # most memory for the parts


@functools.lru_cache(maxsize=None)
def _compute_units(device_index: int) -> int:
    return int(torch.cuda.get_device_properties(device_index).multi_processor_count)


def portion_key_splits(tokens: int, max_qlen: int, long_segments: int, num_q_heads: int, num_kv_heads: int,
                       head_dim: int, max_kv_len: int, device) -> int:
    """Into how many parts the keys of every row block of a prompt portion are cut.

    The portions kernel gives a row block of 128 rows (tokens x q heads of a kv head) to a workgroup.  A short
    portion has fewer row blocks than the chip has compute units, however long its context: then the keys are
    cut too, each part about a thousand keys long at least (the parts are merged by a kernel of its own, which
    writes and reads every part's rows: for a fresh 512-token prompt two parts cost more than they save), and
    the parts are merged afterwards.  The number depends on the shape of the step and on the power-of-two class of
    the longest context only, like the split of decoded tokens, so that a captured step and an eager one choose
    alike.
    """
    group = num_q_heads // num_kv_heads
    blocks = -(-max_qlen * group // _PORTION_ROWS)
    items = blocks * num_kv_heads * max(1, long_segments)
    units = _compute_units(device.index if device.index is not None else torch.cuda.current_device())
    if items >= units or blocks * max(1, long_segments) > _PORTION_LIST_MAX:
        return 1
    most = max(1, (1 << (max(int(max_kv_len), 1).bit_length() - 1)) // 1024)    # 2 from 2,048 keys on, 4 from 4,096, ...
    parts = min(-(-2 * units // items), _PORTION_SPLITS_MAX, most)    # up to two items a compute unit
    while parts > 1 and tokens * num_q_heads * parts * (head_dim + 2) * 4 > _PORTION_WS_BYTES:
        parts -= 1
    return parts


def attn_paged_mfma(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, *,
                    max_qlen: int, max_kv_len: int, num_q_heads: int, num_kv_heads: int, head_dim: int,
                    page_size: int, scale: float, window: int = 0, splits: int | None = None,
                    min_qlen: int = 1, short_segments: int | None = None, portion_splits: int | None = None,
                    plan_token: int = 0, max_portion_kv_len: int | None = None):
    """Causal attention of a packed step on the matrix cores (bfloat16).

    Segments: rows seg_row0[s]..seg_row0[s+1] belong to block-table row seg_slot[s] and start at
    position seg_start[s].  Segments whose rows (tokens x q heads of a kv head) fit one row tile of 16,
    decoded tokens above all, are split over the keys (split-KV), also beside longer portions in one
    step; `short_segments` says how many there are (default: all), which sets the number of splits.
    Longer portions that are too few to fill the chip have their keys cut into `portion_splits` parts
    (default: portion_key_splits).  `plan_token` (new_plan_token()) names the step: with the same token and the
    same segments the portions kernels list their work once, for the first layer, and not once a layer.
    `max_portion_kv_len`: the longest context among the segments of more than one token (default: max_kv_len); what
    the portions kernels plan by, so that a fresh portion beside requests that decode deep into their contexts is
    not cut into parts for the decoders' sake.
    """
    _gpu(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start)
    tokens = q.shape[0]
    _rows(q, "q")
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "the MFMA attention takes bfloat16")
    _need(q.shape == (tokens, num_q_heads * head_dim) and out.shape == q.shape and out.is_contiguous(),
          "q must be [T, nq*D] and out contiguous [T, nq*D]")
    _need(attn_mfma_supported(q.dtype, head_dim, page_size),
          f"the MFMA attention needs head_dim % 16 == 0, head_dim <= {MFMA_MAX_HEAD_DIM} and a power-of-two page_size >= 4 "
          f"(got head_dim {head_dim}, page_size {page_size})")
    _need(q.data_ptr() % 16 == 0 and (q.stride(0) * 2) % 16 == 0, "q rows must be 16-byte aligned")
    _need(num_kv_heads > 0 and num_q_heads % num_kv_heads == 0, "q heads must be a multiple of kv heads")
    _check_pages(k_pages, v_pages, num_kv_heads, page_size, head_dim, q.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    segments = seg_slot.numel()
    _i32(seg_row0, "seg_row0", segments + 1)
    _i32(seg_slot, "seg_slot")
    _i32(seg_start, "seg_start", segments)
    _need(1 <= min_qlen <= max_qlen <= tokens, "need 1 <= min_qlen <= max_qlen <= tokens")
    group = num_q_heads // num_kv_heads
    if min_qlen * group > _ATTN_ROW_TILE:
        splits = 1                      # no segment is short enough for the kernel that splits the keys
    elif splits is None:
        short = segments if short_segments is None else max(1, min(short_segments, segments))
        splits = decode_splits(short, num_kv_heads, max_kv_len)
    _need(segments * splits <= _GRID_Y_MAX and num_kv_heads <= _GRID_Y_MAX, "too many segments for one launch")
    ws_o = ws_ml = None
    if splits > 1:
        ws_rows = segments * max(1, min(max_qlen, _ATTN_ROW_TILE // group))   # arle_attn_ws_rows a segment
        ws_o = torch.empty((ws_rows, num_q_heads, splits, head_dim), dtype=torch.float32, device=q.device)
        ws_ml = torch.empty((ws_rows, num_q_heads, splits, 2), dtype=torch.float32, device=q.device)
    if portion_splits is None:
        long_segments = segments if short_segments is None else max(1, segments - short_segments)
        portion_splits = portion_key_splits(tokens, max_qlen, long_segments, num_q_heads, num_kv_heads, head_dim,
                                            max_portion_kv_len or max_kv_len, q.device)
    if max_qlen * group <= _ATTN_ROW_TILE:
        portion_splits = 1              # no portion for the kernel that they are for
    _need(1 <= portion_splits <= _PORTION_SPLITS_MAX, f"portion_splits must be 1..{_PORTION_SPLITS_MAX}")
    pws_o = pws_ml = None
    if portion_splits > 1:
        pws_o = torch.empty((tokens, num_q_heads, portion_splits, head_dim), dtype=torch.float32, device=q.device)
        pws_ml = torch.empty((tokens, num_q_heads, portion_splits, 2), dtype=torch.float32, device=q.device)
    lib.call("arle_attn_paged_mfma", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0),
             k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1],
             seg_row0.data_ptr(), seg_slot.data_ptr(), seg_start.data_ptr(), segments, int(max_qlen),
             int(min_qlen), int(max_portion_kv_len or max_kv_len), tokens,
             num_q_heads, num_kv_heads, head_dim, page_size, float(scale), int(window), int(splits),
             _ptr(ws_o), _ptr(ws_ml), int(portion_splits), _ptr(pws_o), _ptr(pws_ml), int(plan_token), _stream())
    return out


_PREP_HEAD_DIMS = (64, 128)


def attn_decode_prep_supported(dtype, head_dim: int, page_size: int, group: int, rotary_dim: int) -> bool:
    """Whether attn_decode_prep takes these sizes: bfloat16 pages, a head_dim whose kernel is made for it, up to 16
    q heads a kv head, and a rotated width whose halves are whole chunks of 32 columns (or none)."""
    return (attn_mfma_supported(dtype, head_dim, page_size) and head_dim in _PREP_HEAD_DIMS and 1 <= group <= _ATTN_ROW_TILE
            and rotary_dim % 64 == 0 and 0 <= rotary_dim <= head_dim)


def attn_decode_prep(parts, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, *, max_kv_len: int,
                     num_q_heads: int, num_kv_heads: int, head_dim: int, page_size: int, scale: float, eps: float,
                     q_weight=None, k_weight=None, cos=None, sin=None, rotary_dim: int = 0, window: int = 0,
                     splits: int | None = None):
    """A step of single decoded tokens (segment s is token row s) from the float32 stack of partial products
    [S, T, (nq + 2 nkv) D] of its fused q|k|v projection, or from the projection itself in bfloat16 [T, (nq + 2 nkv) D]:
    what qk_prep and attn_paged_mfma do one after the other, in the attention's own kernel.  Every wave sums, norms and rotates its q heads itself; the wave whose keys end
    with the new token's does the same for the k head, writes key and value into the cache and uses them from its
    registers.  out: bfloat16 [T, nq*D]."""
    _gpu(parts, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, q_weight, k_weight, cos, sin)
    group = num_q_heads // max(num_kv_heads, 1)
    width = (num_q_heads + 2 * num_kv_heads) * head_dim
    whole = parts.dim() == 2     # the projection itself, not a stack of parts
    if whole:
        _rows(parts, "parts")
        _need(parts.dtype == torch.bfloat16 and parts.shape[1] == width and parts.stride(0) % 8 == 0
              and parts.data_ptr() % 16 == 0, f"a whole projection must be bfloat16 [T, {width}] with 16-byte aligned rows")
        n_parts, part_stride, row_stride, tokens = 1, 0, parts.stride(0), parts.shape[0]
    else:
        _need(parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[0] >= 1 and parts.shape[2] == width
              and parts.is_contiguous(), f"parts must be contiguous float32 [S, T, {width}]")
        n_parts, part_stride, row_stride, tokens = parts.shape[0], parts.stride(0), parts.stride(1), parts.shape[1]
    _need(out.dtype == torch.bfloat16 and out.shape == (tokens, num_q_heads * head_dim) and out.is_contiguous(),
          "out must be contiguous bfloat16 [T, nq*D]")
    _need(num_kv_heads > 0 and num_q_heads % num_kv_heads == 0, "q heads must be a multiple of kv heads")
    _need(attn_decode_prep_supported(out.dtype, head_dim, page_size, group, rotary_dim),
          f"attn_decode_prep takes head_dim {_PREP_HEAD_DIMS}, up to {_ATTN_ROW_TILE} q heads a kv head and a rotated width "
          f"that is a multiple of 64 (got head_dim {head_dim}, {group} heads, rotary_dim {rotary_dim})")
    _check_pages(k_pages, v_pages, num_kv_heads, page_size, head_dim, out.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    segments = seg_slot.numel()
    _need(segments == tokens, "attn_decode_prep takes one token a segment")
    _i32(seg_row0, "seg_row0", segments + 1)
    _i32(seg_slot, "seg_slot")
    _i32(seg_start, "seg_start", segments)
    _need((q_weight is None) == (k_weight is None), "give both q and k norm weights or neither")
    w_f32 = 0
    if q_weight is not None:
        _need(q_weight.shape == (head_dim,) and k_weight.shape == (head_dim,) and q_weight.dtype == k_weight.dtype
              and q_weight.dtype in (torch.float32, torch.bfloat16) and q_weight.is_contiguous() and k_weight.is_contiguous()
              and q_weight.data_ptr() % 16 == 0 and k_weight.data_ptr() % 16 == 0,
              "q/k norm weights must be 16-byte aligned [head_dim] of one type, float32 or bfloat16")
        w_f32 = int(q_weight.dtype == torch.float32)
    if rotary_dim:
        _need(cos is not None and sin is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32
              and cos.dim() == 2 and cos.shape == sin.shape and cos.shape[1] == rotary_dim // 2 and cos.is_contiguous()
              and sin.is_contiguous() and cos.data_ptr() % 16 == 0 and sin.data_ptr() % 16 == 0,
              "cos/sin must be contiguous 16-byte aligned float32 [positions, rotary_dim/2]")
    if splits is None:
        splits = decode_splits(segments, num_kv_heads, max_kv_len)
    _need(1 <= splits <= 64, "splits must be 1..64")
    _need(segments * splits <= _GRID_Y_MAX and num_kv_heads <= _GRID_Y_MAX, "too many segments for one launch")
    ws_o = ws_ml = None
    if splits > 1:
        ws_o = torch.empty((segments, num_q_heads, splits, head_dim), dtype=torch.float32, device=out.device)
        ws_ml = torch.empty((segments, num_q_heads, splits, 2), dtype=torch.float32, device=out.device)
    lib.call("arle_attn_decode_prep", parts.data_ptr(), int(whole), n_parts, part_stride, row_stride, _ptr(q_weight),
             _ptr(k_weight), w_f32, _ptr(cos), _ptr(sin), int(rotary_dim), float(eps), out.data_ptr(), out.stride(0),
             k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], seg_row0.data_ptr(),
             seg_slot.data_ptr(), seg_start.data_ptr(), segments, num_q_heads, num_kv_heads, head_dim, page_size,
             float(scale), int(window), int(splits), _ptr(ws_o), _ptr(ws_ml), _stream())
    return out


_plan_tokens = itertools.count(1)


def new_plan_token() -> int:
    """A number that no other step of this process has (attn_paged_mfma's plan_token)."""
    return next(_plan_tokens)


def attn_decode_static(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, *, max_qlen: int,
                       num_q_heads: int, num_kv_heads: int, head_dim: int, page_size: int, scale: float,
                       window: int = 0, splits: int = 1):
    """attn_paged_mfma for steps whose every segment fits one row tile of 16, with the split-KV partial results
    in the library's fixed device array: the call allocates nothing (for code under graph capture and other
    callers that cannot allocate).  Steps too large for the array raise with the library's reason; calls that
    overlap on one GPU race on the array."""
    _gpu(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start)
    tokens = q.shape[0]
    _rows(q, "q")
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "the MFMA attention takes bfloat16")
    _need(q.shape == (tokens, num_q_heads * head_dim) and out.shape == q.shape and out.is_contiguous(),
          "q must be [T, nq*D] and out contiguous [T, nq*D]")
    _need(q.data_ptr() % 16 == 0 and (q.stride(0) * 2) % 16 == 0, "q rows must be 16-byte aligned")
    _check_pages(k_pages, v_pages, num_kv_heads, page_size, head_dim, q.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    segments = seg_slot.numel()
    _i32(seg_row0, "seg_row0", segments + 1)
    _i32(seg_slot, "seg_slot")
    _i32(seg_start, "seg_start", segments)
    status = lib.function("arle_attn_decode_static")(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(), v_pages.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], seg_row0.data_ptr(), seg_slot.data_ptr(), seg_start.data_ptr(),
        segments, int(max_qlen), num_q_heads, num_kv_heads, head_dim, page_size, float(scale), int(window), int(splits),
        _stream())
    if status != 0:
        why = lib.function_raw("arle_attn_decode_static_error", ctypes.c_char_p)().decode()
        raise lib.KernelError(why or f"arle_attn_decode_static failed with HIP error {status}")
    return out


# ------------------------------------------------------------------- sampling


def _logits(logits):
    _gpu(logits)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.is_contiguous(),
          "logits must be contiguous float32 [rows, vocab]")
    return logits.shape


@functools.lru_cache(maxsize=None)
def _argmax_chunks(rows: int, vocab: int) -> int:
    """Into how many chunks the argmax kernel cuts each row (it wants scratch for more than one)."""
    return int(lib.function("arle_argmax_chunks")(rows, vocab))


def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    rows, vocab = _logits(logits)
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    chunks = _argmax_chunks(rows, vocab)
    parts = torch.empty((rows, chunks, 2), dtype=torch.int32, device=logits.device) if chunks > 1 else None
    lib.call("arle_argmax_rows", logits.data_ptr(), rows, vocab, out.data_ptr(),
             parts.data_ptr() if parts is not None else 0, _stream())
    return out


def token_logprobs(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """float32 [rows]: log softmax(logits[r])[tokens[r]], natural logarithm (tokens int32 [rows])."""
    rows, vocab = _logits(logits)
    _gpu(tokens)
    _i32(tokens, "tokens", rows)
    out = torch.empty((rows,), dtype=torch.float32, device=logits.device)
    lib.call("arle_token_logprobs", logits.data_ptr(), rows, vocab, tokens.data_ptr(), out.data_ptr(), _stream())
    return out


@functools.lru_cache(maxsize=None)
def _sample_scratch_bytes(rows: int, vocab: int) -> int:
    fn = lib.function("arle_sample_scratch_bytes")
    fn.restype = ctypes.c_longlong
    return int(fn(rows, vocab))


def sample_rows(logits, temperature, top_k, top_p, min_p, u, *, use_top_k: bool = True,
                use_top_p: bool = True) -> torch.Tensor:
    """One token id per row; per-row float32 temperature/top_p/min_p/u and int32 top_k.

    use_top_k / use_top_p = False promise that no row has that filter switched on (top_k in 1..vocab-1,
    top_p < 1): the passes over the row that look for its threshold are then not launched.
    """
    rows, vocab = _logits(logits)
    for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                        ("top_p", top_p, torch.float32), ("min_p", min_p, torch.float32),
                        ("u", u, torch.float32)):
        _gpu(t)
        _need(t.dtype == dt and t.shape == (rows,) and t.is_contiguous(), f"{name} must be {dt} [rows]")
    probs = torch.empty((rows, vocab), dtype=torch.float32, device=logits.device)
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    words = -(-_sample_scratch_bytes(rows, vocab) // 8)
    scratch = torch.zeros((words,), dtype=torch.int64, device=logits.device)   # histograms start at zero
    lib.call("arle_sample_rows", logits.data_ptr(), rows, vocab, probs.data_ptr(),
             temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(), min_p.data_ptr(),
             u.data_ptr(), out.data_ptr(), scratch.data_ptr(), int(bool(use_top_k)), int(bool(use_top_p)),
             _stream())
    return out


def apply_penalties(logits, indptr, tokens, counts, repetition, frequency, presence) -> None:
    """In place: repetition, frequency and presence penalties on the listed (row, token, count)."""
    rows, vocab = _logits(logits)
    _gpu(indptr, tokens, counts, repetition, frequency, presence)
    _i32(indptr, "indptr", rows + 1)
    _i32(tokens, "tokens")
    _i32(counts, "counts", tokens.numel())
    for name, t in (("repetition", repetition), ("frequency", frequency), ("presence", presence)):
        _need(t.dtype == torch.float32 and t.shape == (rows,) and t.is_contiguous(),
              f"{name} must be float32 [rows]")
    lib.call("arle_apply_penalties", logits.data_ptr(), rows, vocab, indptr.data_ptr(),
             tokens.data_ptr(), counts.data_ptr(), repetition.data_ptr(), frequency.data_ptr(),
             presence.data_ptr(), _stream())


# ------------------------------------------------------------ bfloat16 products


ROWS_KERNEL_MAX = 64          # most rows the hand-written few-rows kernel takes
EPI_NONE, EPI_SILU_MUL = 0, 1
# How the few-rows kernel is shaped for a product (measured on MI355X together with the kernel that adds
# the stack of partial products; see the kernel for the variants):
_ROWS_TARGET_WORKGROUPS = 640    # K is split until about this many workgroups stream W
_ROWS_MAX_SPLITS = 4             # ... the consumer pays for every part of the stack (4, 8, 16 measure alike)
_ROWS_PARTIAL_BYTES = 3 << 20    # ... and the float32 partial products stay below this
_ROWS_WIDE_N = 32768             # from here on (an output head) N alone gives enough workgroups
_ROWS_NARROW_N = 4096            # up to here N gives so few that one column tile a workgroup is best
_ROWS_FUSED_MAX = 32             # gate|up with the activation in one go: as many rows as fit into LDS with all of K (27 at K = 2560): 4.20 against 4.41 ms a step at batch 20; more rows: gemm_rows_rounds
_ROWS_PREFERRED = 16             # with more rows the library is at least as fast on MI355X
_V_GENERAL, _V_FUSED_FEW, _V_NARROW, _V_SHARED = 0, 1, 2, 3
ROWS_VARIANTS = 5


def gemm_rows_supported(rows: int, k: int, x_stride: int) -> bool:
    return 0 < rows <= ROWS_KERNEL_MAX and k % 8 == 0 and x_stride % 8 == 0


def _fused_variant(rows: int) -> int:
    return _V_FUSED_FEW if rows <= 4 else _V_SHARED   # 8 rows: 20.7 against 22.3 us for the eight-column-tile workgroups


def gemm_rows_preferred(rows: int, n: int, k: int, x_stride: int, fused: bool = False) -> bool:
    """Whether the hand-written kernel, not the library, should run this product."""
    if fused:   # the activation needs whole sums: the rows of all of K in LDS at once
        return (gemm_rows_supported(rows, k, x_stride) and rows <= _ROWS_FUSED_MAX
                and _rows_min_splits(_fused_variant(rows), rows, k) == 1)
    if not gemm_rows_supported(rows, k, x_stride) or rows > _ROWS_PREFERRED:
        return False
    return True


@functools.lru_cache(maxsize=None)
def _rows_geometry(variant: int):
    """(waves that share a k slice, output columns per workgroup, can apply the fused activation) of a variant."""
    packed = lib.function("arle_gemm_rows_geometry")(variant)
    _need(packed > 0, f"gemm_rows has no variant {variant}")
    return packed >> 20, (packed >> 4) & 0xFFFF, packed & 15


@functools.lru_cache(maxsize=4096)
def _rows_min_splits(variant: int, M: int, K: int) -> int:
    """Fewest k splits with which the X rows of one slice fit into LDS."""
    fn = lib.function("arle_gemm_rows_lds")
    fn.restype = ctypes.c_longlong
    cap_fn = lib.function("arle_gemm_rows_lds_max")
    cap_fn.restype = ctypes.c_longlong
    cap, steps = cap_fn(), -(-K // 32)
    splits = 1
    while fn(variant, M, -(-steps // splits)) > cap:
        splits += 1
        _need(splits <= steps, f"gemm_rows: {M} rows of one k step do not fit into LDS")
    return splits


@functools.lru_cache(maxsize=4096)
def gemm_rows_plan(M: int, N: int, K: int, fused: bool = False):
    """(variant, splits) for a product: small workgroups, K split across workgroups until enough of them
    stream W, within a budget for the stack of partial products that the consumer has to add."""
    if fused:
        return _fused_variant(M), 1
    if N >= _ROWS_WIDE_N:
        variant, want = (_V_NARROW if M <= 4 else _V_SHARED), 1
    else:
        variant = _V_NARROW if N <= _ROWS_NARROW_N else _V_GENERAL
        _, columns, _ = _rows_geometry(variant)
        groups = -(-N // columns)
        want = min(-(-_ROWS_TARGET_WORKGROUPS // groups), _ROWS_MAX_SPLITS, max(1, _ROWS_PARTIAL_BYTES // (M * N * 4)))
    return variant, max(want, _rows_min_splits(variant, M, K))


def pack_weight_tiles(w: torch.Tensor) -> torch.Tensor:
    """w [N, K] bfloat16 -> [ceil(N/16), ceil(K/32), 512]: the operand tiles that gemm_rows and gemm_stream read
    with one contiguous kilobyte a wave and k step.  Tile (t, s), element 128 g + 8 i + e = w[16 t + i, 32 s + 8 g + e]
    (lane 16 g + i of the wave reads its eight elements); zeros past N and K.  A rearrangement at load time, the
    values are untouched, and the product adds them in the same order as from rows."""
    _need(w.dim() == 2 and w.dtype == torch.bfloat16, "pack_weight_tiles takes a bfloat16 [N, K] matrix")
    N, K = w.shape
    Np, Kp = -(-N // 16) * 16, -(-K // 32) * 32
    if (Np, Kp) != (N, K):
        w = torch.nn.functional.pad(w, (0, Kp - K, 0, Np - N))
    return w.reshape(Np // 16, 16, Kp // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(Np // 16, Kp // 32, 512)


def _check_tiles(tiles, N: int, K: int) -> None:
    _need(tiles.dtype == torch.bfloat16 and tiles.is_contiguous() and tiles.dim() == 3 and tiles.shape[1:] == (-(-K // 32), 512)
          and tiles.shape[0] >= -(-N // 16) and tiles.data_ptr() % 16 == 0,
          f"operand tiles of a [{N}, {K}] matrix have the shape [{-(-N // 16)}, {-(-K // 32)}, 512], got {tuple(tiles.shape)}")


def gemm_rows(x, w, out_dtype=torch.bfloat16, epilogue: int = EPI_NONE, *, variant: int | None = None,
              splits: int | None = None, tiles: torch.Tensor | None = None):
    """x . w^T for 1..64 rows of x, with x shared through LDS inside a workgroup.

    splits == 1: returns [M, N] (or [M, N/2] with EPI_SILU_MUL) in `out_dtype`.
    splits > 1: K is also split across workgroups; returns float32 [S, M, N] partial products (S <= splits,
    no split is empty) for the consumer to add in the order of S.  With `variant` and `splits` left out
    the shape decides (gemm_rows_plan), so callers must be ready for either form.
    EPI_SILU_MUL: w holds gate and up rows interleaved in blocks of 16; out[m, j] = silu(gate_j) * up_j.
    tiles: pack_weight_tiles(w); the kernel then streams these instead of the rows of w (same sums, bit for bit).
    """
    _gpu(x, w)
    _rows(x, "x")
    _need(w.dim() == 2 and w.is_contiguous(), "w must be contiguous [N, K]")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_rows takes bfloat16 operands")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape[1] == K, f"gemm_rows: inner sizes differ ({K} vs {w.shape[1]})")
    _need(gemm_rows_supported(M, K, x.stride(0)),
          f"gemm_rows takes 1..{ROWS_KERNEL_MAX} rows and K % 8 == 0 (got {M} rows, K = {K})")
    _need(x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_rows writes bfloat16 or float32")
    fused = epilogue == EPI_SILU_MUL
    if variant is None or splits is None:
        plan = gemm_rows_plan(M, N, K, fused)
        variant = plan[0] if variant is None else variant
        splits = plan[1] if splits is None else splits
    _, _, can_fuse = _rows_geometry(variant)
    steps = -(-K // 32)
    per_split = -(-steps // max(1, min(splits, steps)))
    splits = -(-steps // per_split)
    if fused:
        _need(N % 32 == 0, "the fused activation needs gate/up interleaved in blocks of 16")
        _need(can_fuse == 1 and splits == 1,
              "the fused activation needs a variant with an even number of column tiles, and whole sums")
    _need(splits >= _rows_min_splits(variant, M, K),
          f"gemm_rows: {M} rows of {per_split * 32} columns do not fit into LDS; split K further")
    if splits > 1:
        out = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
        ldo, stride, code = N, M * N, F32
    else:
        out = torch.empty((M, N // 2 if fused else N), dtype=out_dtype, device=x.device)
        ldo, stride, code = out.stride(0), 0, _CODES[out_dtype]
    if tiles is not None:
        _check_tiles(tiles, N, K)
    lib.call("arle_gemm_rows", x.data_ptr(), x.stride(0), (w if tiles is None else tiles).data_ptr(), w.stride(0),
             int(tiles is not None), out.data_ptr(), ldo, stride,
             code, M, N, K, int(epilogue), variant, splits, per_split, _stream())
    return out


_ROUNDS_MAX_WORKGROUPS = 256     # one workgroup a compute unit (its x rows take most of a CU's LDS): more would run in two turns
_ROUNDS_TALL_MIN_N = 16384       # 33 to 64 rows (four row tiles a wave): only outputs this wide gain


def gemm_rows_rounds_preferred(rows: int, n: int, k: int, x_stride: int) -> bool:
    """Whether gate|up with its activation should run in the few-rows kernel that walks K in rounds (up to 64
    rows), not as the library's product and the activation kernel.  Measured on MI355X, in us, rounds against
    library, at 28 / 48 / 64 rows: 19,456 x 2,560 (Qwen3-4B) 24.4 / 27.1 / 31.0 against 27.7 / 30.4 / 31.8;
    24,576 x 4,096 (8B) 45.7 / 49.7 / 52.7 against 53.1 / 53.6 / 54.1; 6,144 x 1,024 (0.6B) 8.6 / 11.0 / 12.9
    against 12.1 / 12.8 / 12.6; 12,288 x 2,048 (1.7B, 96 workgroups) 19.9 / 22.6 / 24.9 against 20.5 / 21.4 / 21.8;
    51,200 x 5,120 (32B: 400 workgroups for 256 compute units, two turns) 105.7 / 113.8 / 123.6 against
    100.5 / 104.2 / 110.4.  So: no more workgroups than compute units, and beyond 32 rows a wide output.  Up to 16
    rows the x rows of a round are small enough for several workgroups a compute unit and the kernel is level with
    the library at every width (32B shape, 16 rows: 94 against 94 us), where the product alone without the
    activation, as a stack of parts of K, takes 123 + 5 + 5 us: so rows that the kernel without rounds cannot
    hold (14 to 16 rows at K = 5,120) come here."""
    if not (gemm_rows_supported(rows, k, x_stride) and n % 32 == 0):
        return False
    return rows <= _ROWS_PREFERRED or (-(-n // 128) <= _ROUNDS_MAX_WORKGROUPS and (rows <= 32 or n >= _ROUNDS_TALL_MIN_N))


@functools.lru_cache(maxsize=None)
def _rows_round_steps(rows: int, k: int) -> int:
    """Steps of 32 k whose x rows the fused few-rows kernel can hold in LDS at a time, cut so that the rounds
    that cover K are of one length."""
    steps = -(-k // 32)
    need = lib.function("arle_gemm_rows_lds")
    need.restype = ctypes.c_longlong
    cap_fn = lib.function("arle_gemm_rows_lds_max")
    cap_fn.restype = ctypes.c_longlong
    most, fit = cap_fn(), steps
    while fit > 1 and need(_V_SHARED, rows, fit) > most:
        fit -= 1
    _need(need(_V_SHARED, rows, fit) <= most, f"gemm_rows_rounds: {rows} rows of 32 columns do not fit into LDS")
    rounds = -(-steps // fit)
    return -(-steps // rounds)


def gemm_rows_rounds(x, w, out_dtype=torch.bfloat16, *, tiles: torch.Tensor | None = None, round_steps: int | None = None):
    """silu(x . gate^T) * (x . up^T) for 1..64 rows of x, w holding gate and up rows interleaved in blocks of 16:
    gemm_rows with the fused activation where the x rows of all of K do not fit into LDS at once (more than 27
    rows at K = 2,560).  K is walked in rounds of `round_steps` steps of 32, the sums stay in registers.
    Returns [M, N/2]."""
    _gpu(x, w)
    _rows(x, "x")
    _need(w.dim() == 2 and w.is_contiguous(), "w must be contiguous [N, K]")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_rows_rounds takes bfloat16 operands")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape[1] == K, f"gemm_rows_rounds: inner sizes differ ({K} vs {w.shape[1]})")
    _need(gemm_rows_supported(M, K, x.stride(0)),
          f"gemm_rows_rounds takes 1..{ROWS_KERNEL_MAX} rows and K % 8 == 0 (got {M} rows, K = {K})")
    _need(x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_rows_rounds writes bfloat16 or float32")
    _need(N % 32 == 0, "the fused activation needs gate/up interleaved in blocks of 16")
    if round_steps is None:
        round_steps = _rows_round_steps(M, K)
    _need(round_steps >= 1, "a round is at least one step of 32")
    round_steps = min(int(round_steps), -(-K // 32))
    need = lib.function("arle_gemm_rows_lds")
    need.restype = ctypes.c_longlong
    cap_fn = lib.function("arle_gemm_rows_lds_max")
    cap_fn.restype = ctypes.c_longlong
    _need(need(_V_SHARED, M, round_steps) <= cap_fn(),
          f"gemm_rows_rounds: {M} rows of {round_steps * 32} columns do not fit into LDS; take shorter rounds")
    if tiles is not None:
        _check_tiles(tiles, N, K)
    out = torch.empty((M, N // 2), dtype=out_dtype, device=x.device)
    lib.call("arle_gemm_rows_rounds", x.data_ptr(), x.stride(0), (w if tiles is None else tiles).data_ptr(), w.stride(0),
             int(tiles is not None), out.data_ptr(), out.stride(0), _CODES[out_dtype], M, N, K, int(round_steps), _stream())
    return out


STREAM_VARIANTS = 5


@functools.lru_cache(maxsize=None)
def _stream_geometry(variant: int):
    """(output columns of a column group, steps of a round) of a variant of the kernel whose workgroups stay."""
    packed = lib.function("arle_gemm_stream_geometry")(variant)
    _need(packed > 0, f"gemm_stream has no variant {variant}")
    return packed >> 8, packed & 255


@functools.lru_cache(maxsize=4096)
def _stream_min_splits(variant: int, M: int, K: int) -> int:
    fn = lib.function("arle_gemm_stream_lds")
    fn.restype = ctypes.c_longlong
    cap_fn = lib.function("arle_gemm_rows_lds_max")
    cap_fn.restype = ctypes.c_longlong
    cap, steps = cap_fn(), -(-K // 32)
    splits = 1
    while fn(variant, M, -(-steps // splits)) > cap:
        splits += 1
        _need(splits <= steps, f"gemm_stream: {M} rows of one round do not fit into LDS")
    return splits


def gemm_stream(x, w, out_dtype=torch.bfloat16, *, variant: int = 0, splits: int | None = None,
                workgroups: int | None = None, tiles: torch.Tensor | None = None):
    """x . w^T for 1..64 rows of x by workgroups that stay: each stages its slice of x once and walks several
    groups of output columns, so that w alone is streamed (see gemm_stream_kernel).

    Returns [M, N] in `out_dtype` for one k split, else float32 [S, M, N] partial products for the consumer
    to add in the order of S.  `workgroups`: how many of them work on every k split.
    """
    _gpu(x, w)
    _rows(x, "x")
    _need(w.dim() == 2 and w.is_contiguous(), "w must be contiguous [N, K]")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_stream takes bfloat16 operands")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape[1] == K, f"gemm_stream: inner sizes differ ({K} vs {w.shape[1]})")
    _need(gemm_rows_supported(M, K, x.stride(0)),
          f"gemm_stream takes 1..{ROWS_KERNEL_MAX} rows and K % 8 == 0 (got {M} rows, K = {K})")
    _need(x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_stream writes bfloat16 or float32")
    columns, _ = _stream_geometry(variant)
    least = _stream_min_splits(variant, M, K)
    steps = -(-K // 32)
    splits = max(least, splits or 1)
    per_split = -(-steps // max(1, min(splits, steps)))
    splits = -(-steps // per_split)
    _need(splits >= least, f"gemm_stream: {M} rows of {per_split * 32} columns do not fit into LDS; split K further")
    groups = -(-N // columns)
    if workgroups is None:
        workgroups = max(1, min(groups, -(-_STREAM_TARGET_WORKGROUPS // splits)))
    if splits > 1:
        out = torch.empty((splits, M, N), dtype=torch.float32, device=x.device)
        ldo, stride, code = N, M * N, F32
    else:
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
        ldo, stride, code = out.stride(0), 0, _CODES[out_dtype]
    if tiles is not None:
        _check_tiles(tiles, N, K)
    lib.call("arle_gemm_stream", x.data_ptr(), x.stride(0), (w if tiles is None else tiles).data_ptr(), w.stride(0),
             int(tiles is not None), out.data_ptr(), ldo, stride,
             code, M, N, K, variant, splits, per_split, int(workgroups), _stream())
    return out


_STREAM_TARGET_WORKGROUPS = 256   # staying workgroups in all: one for every compute unit


# The many-rows kernel that reads operand tiles takes over from the library only where whole prefill steps were
# measured faster with it on MI355X (same machine, both ways, 12 layers): gate|up with the activation fused, a hidden
# size of at most 2,560 and 2,048 to about 6,000 rows.  Qwen3-4B widths: 0.5 to 4.6 % of the step at 2,048 rows (the
# gain differs from machine to machine), 1.8 % at 4,096; hidden sizes 1,024 and 2,048: level; hidden sizes 4,096 and
# 5,120: 9 and 8 % slower, so the library keeps those.  Kernel against kernel with cold weights the library's product
# and the activation kernel take 234-272 us at 2,048 x 19,456 x 2,560 and this kernel 237-255 us; at 8,192 rows the
# library is ahead.  Plain products stay with the library (q|k|v at 2,048 rows: 85 against 60 us).
_TILES_MIN_ROWS = 2048
_TILES_MAX_ROWS = 6144
_TILES_MIN_N = 4096
_TILES_MAX_K = 2560
_TILES_BIG_ROWS = 4096      # from here on workgroups of 256 rows with the pipelined loop


def gemm_tiles_preferred(rows: int, n: int, k: int, x_stride: int, fused: bool = False) -> bool:
    """Whether the many-rows kernel that reads operand tiles, not the library, should run this product."""
    return (fused and _TILES_MIN_ROWS <= rows < _TILES_MAX_ROWS and n >= _TILES_MIN_N and k <= _TILES_MAX_K
            and k % 8 == 0 and x_stride % 8 == 0)


# (row tiles of 32 a workgroup, ring depths W|X; 1xx: the loop with the barrier in mid-step and four LDS stages[,
#  column tiles of 32 a wave: 2 unless given])
TILES_VARIANTS = ((4, 22), (4, 44), (8, 44), (8, 144), (4, 44, 1), (4, 84, 1))


def gemm_tiles(x, tiles, n: int, out_dtype=torch.bfloat16, epilogue: int = EPI_NONE, *, variant=None, splits: int = 1):
    """x [M, K] . W^T for many rows, W [n, K] given as its operand tiles (pack_weight_tiles): workgroups of
    128 or 256 rows x 256 (or 128) columns, W straight from memory into the matrix cores, x through LDS.
    EPI_SILU_MUL: gate and up rows of W interleaved in blocks of 16; returns [M, n/2].
    splits > 1: K cut into that many parts (of whole steps of 32), one workgroup each; returns the float32 stack
    [splits, M, n] for the caller to add in order."""
    _gpu(x, tiles)
    _rows(x, "x")
    _need(x.dtype == torch.bfloat16, "gemm_tiles takes bfloat16 operands")
    M, K = x.shape
    _need(K % 8 == 0 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0, "gemm_tiles: K and the row stride of x must be multiples of 8")
    _check_tiles(tiles, n, K)
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_tiles writes bfloat16 or float32")
    fused = epilogue == EPI_SILU_MUL
    _need(not fused or n % 32 == 0, "the fused activation needs gate/up interleaved in blocks of 16")
    if variant is None:
        variant = (8, 144) if M >= _TILES_BIG_ROWS else (4, 44)
    _need(tuple(variant) in TILES_VARIANTS, f"gemm_tiles has no variant {variant}")
    col_tiles = variant[2] if len(variant) > 2 else 2
    steps = -(-K // 32)
    _need(1 <= splits <= steps, f"gemm_tiles cannot cut {steps} steps of K into {splits} parts")
    per = -(-steps // splits)
    splits = -(-steps // per)   # parts of `per` steps cover K; the last one may be shorter
    if splits > 1:
        _need(not fused and out_dtype == torch.float32, "parts of K come back as a float32 stack without an epilogue")
        out = torch.empty((splits, M, n), dtype=torch.float32, device=x.device)
        ldo, stride = out.stride(1), out.stride(0)
    else:
        out = torch.empty((M, n // 2 if fused else n), dtype=out_dtype, device=x.device)
        ldo, stride = out.stride(0), 0
    lib.call("arle_gemm_tiles", x.data_ptr(), x.stride(0), tiles.data_ptr(), out.data_ptr(), ldo,
             _CODES[out_dtype], M, n, K, int(epilogue), variant[0], col_tiles, variant[1], splits, per, stride, _stream())
    return out


def sum_partials(parts: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[S, ...] float32 -> [...]: the stack added in order."""
    _gpu(parts)
    _need(parts.dtype == torch.float32 and parts.dim() >= 2 and parts.is_contiguous() and parts.shape[0] >= 1,
          "sum_partials takes a contiguous float32 stack")
    _need(out_dtype in _CODES, "sum_partials writes bfloat16 or float32")
    out = torch.empty(parts.shape[1:], dtype=out_dtype, device=parts.device)
    lib.call("arle_sum_partials", parts.data_ptr(), parts.shape[0], out.numel(), out.data_ptr(), _CODES[out_dtype],
             out.numel(), _stream())
    return out


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, partials_ok: bool = False,
              tiles: torch.Tensor | None = None):
    """out[M, N] = x[M, K] . w[N, K]^T, bfloat16 operands, float32 accumulation.

    Few rows (decode steps, short portions) run the hand-written weight-streaming kernels.  More rows go
    to the vendor library (hipBLASLt through torch.matmul), the matrix product the reference also leaves
    to a library (crates/cuda-kernels/csrc/gemm/gemv.cu:240-330).  Which kernel it is for a shape is decided in
    one place, `choose_product`: by a measured table where one is loaded for these widths, else by the rules.
    partials_ok: the caller adds a float32 stack [S, M, N] itself (in the order of S) if that is what the
    kernel leaves behind; otherwise the stack is added here by one more small kernel.
    tiles: pack_weight_tiles(w), for the hand-written kernels to stream instead of w.
    """
    _gpu(x, w)
    _rows(x, "x")
    _need(w.dim() == 2 and w.is_contiguous(), "w must be contiguous [N, K]")
    _need(x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16, "gemm_bf16 takes bfloat16 operands")
    _need(x.shape[1] == w.shape[1], f"gemm_bf16: inner sizes differ ({x.shape[1]} vs {w.shape[1]})")
    _need(out_dtype in (torch.bfloat16, torch.float32), "gemm_bf16 writes bfloat16 or float32")
    rows, n, k = x.shape[0], w.shape[0], x.shape[1]
    choice = choose_product(rows, n, k, x.stride(0), tiled=tiles is not None, fused=False, partials_ok=partials_ok,
                            aligned=x.data_ptr() % 16 == 0)
    return run_product(choice, x, w, tiles, out_dtype, partials_ok)


# The library runs a product with a narrow output and a long K (o and down: 2,560 columns) as a few dozen
# workgroups that each walk all of K, and takes as long for 128 rows as for 1,024 (down of the Qwen3-4B shape: 60 us
# at 512 rows, where reading the weights takes 10 and the products 17).  Cut into parts along K, as one batched
# product of the parts, it fills the chip: 33 us at 512 rows, 29 at 128.  The parts come back as a float32 stack
# for the consumer to add in order, like the stacks of the few-rows kernels (added in float32, where the single
# product rounds its sum to bfloat16).  More parts make a larger stack to write and read, so wide outputs and
# rows beyond 1,024 stay whole.  Outputs of 5,120 columns (the 14B and 32B shapes) gain most: down (5,120 x 25,600)
# whole takes 172 / 182 / 261 / 272 / 349 us at 65 / 128 / 256 / 512 / 1,024 rows and 60 / 63 / 79 / 120 / 247 in
# parts; o (5,120 x 8,192) 31 / 46 / 74 / 70 / 94 whole and 31 / 32 / 37 / 48 / 89 in parts.
_LIB_SPLIT_MAX_N = 5120
_LIB_SPLIT_MIN_K = 2048
_LIB_SPLIT_MAX_ROWS = 1024
_LIB_SPLIT_LONG_K = 8192
_LIB_SPLIT_LONG_K_MAX_ROWS = 3072
_BMM_OUT_DTYPE_OK = None


# A product with a narrow output and 65 to 256 rows (o and down of a large decode batch or a short portion) is a
# matter of streaming W, and the library gives it a few dozen workgroups.  gemm_tiles with workgroups of 128 rows x
# 128 columns and K cut into parts, so that about 160 to 200 workgroups stream at once, leaves a float32 stack like
# the few-rows kernels.  Measured on MI355X at the Qwen3-4B shape, in us: o (2,560 x 4,096) at 96 / 128 / 256 rows
# 13.0 / 14.7 / 19.3 against 23.4 / 23.8 / 22.0 for the library's batched parts; down (2,560 x 9,728) at 96 / 128 /
# 192 rows 20.7 / 23.7 / 30.2 against 28.4 / 30.1 / 33.7, and behind at 256 (34.7 against 25.8).  For q|k|v the
# larger stack costs the consumer what the product gains, and gate|up needs whole sums for its activation.
_NARROW_TILES_VARIANT = (4, 44, 1)
_NARROW_TILES_MAX_N = 4096
_NARROW_TILES_MIN_K = 2048
_NARROW_TILES_WORKGROUPS = 200


def narrow_tiles_splits(rows: int, n: int, k: int, x_stride: int) -> int:
    """Into how many parts along K gemm_tiles' narrow workgroups cut such a product; 0: they do not take it."""
    most_rows = 256 if k < 8192 else 192
    if not (ROWS_KERNEL_MAX < rows <= most_rows and n <= _NARROW_TILES_MAX_N and k >= _NARROW_TILES_MIN_K
            and k % 8 == 0 and x_stride % 8 == 0):
        return 0
    blocks = -(-n // 128) * -(-rows // 128)
    splits = 8
    while splits > 1 and (blocks * splits > _NARROW_TILES_WORKGROUPS or k < 320 * splits):
        splits //= 2
    return splits if splits > 1 else 0


def library_k_splits(rows: int, n: int, k: int) -> int:
    """Into how many parts along K the library's product is cut (1: not at all)."""
    if not (ROWS_KERNEL_MAX < rows and n <= _LIB_SPLIT_MAX_N and k >= _LIB_SPLIT_MIN_K):
        return 1
    if rows > _LIB_SPLIT_MAX_ROWS:
        # a very long K still gains from two parts: down of the Qwen3-4B shape 76 / 91 / 126 us at 1,536 / 2,048 /
        # 3,072 rows against 92 / 111 / 146 whole (the consumer pays 6 to 10 us for the stack); at 4,096 whole is ahead
        if not (k >= _LIB_SPLIT_LONG_K and rows <= _LIB_SPLIT_LONG_K_MAX_ROWS):
            return 1
        splits = 2
    elif k >= 8192:
        splits = 8 if rows <= 256 else 4
    else:
        splits = 4 if rows <= 512 else 2
    while splits > 1 and k % (32 * splits):
        splits //= 2
    return splits


def _bmm_takes_out_dtype(device) -> bool:
    """Whether this torch's batched product hands back float32 sums of bfloat16 operands; asked once, on a tiny
    product, so that no failure of a real call (out of memory, say) is taken for the answer."""
    global _BMM_OUT_DTYPE_OK
    if _BMM_OUT_DTYPE_OK is None:
        probe = torch.zeros((2, 16, 32), dtype=torch.bfloat16, device=device)
        try:
            torch.bmm(probe, probe.transpose(1, 2), out_dtype=torch.float32)
            _BMM_OUT_DTYPE_OK = True
        except (TypeError, RuntimeError):
            _BMM_OUT_DTYPE_OK = False
    return _BMM_OUT_DTYPE_OK


def _library_mm_split_k(x, w, splits: int):
    """float32 [splits, M, N]: part s is x[:, s-th part of K] . w[:, s-th part of K]^T; None if this torch cannot
    give a batched product float32 results."""
    if not _bmm_takes_out_dtype(x.device):
        return None
    m, k = x.shape
    n, part = w.shape[0], k // splits
    xs = x.as_strided((splits, m, part), (part, x.stride(0), 1))
    ws = w.as_strided((splits, part, n), (part, 1, w.stride(0)))
    return torch.bmm(xs, ws, out_dtype=torch.float32)


# 17..64 rows: the kernel whose workgroups stay beats the library where the output is narrow and K long (the
# o and down projections: 11 against 15 us and 19 against 29 us at 64 rows of the Qwen3-4B shapes); for wide
# outputs (q|k|v, gate|up) the two are level and the library stays.
_STREAM_VARIANT = 0
_STREAM_SPLITS = 6              # at least so many k splits ...
_STREAM_STEPS_A_SPLIT = 50      # ... and at most so many steps of 32 in one (the 32B shape's down, K = 25600: 16 splits)
_STREAM_MAX_N = 5120            # 60 against the library's 146 us there at 32 rows, 97 against 157 us at 64
_STREAM_MIN_K = 2048


_STREAM_PARTIAL_BYTES = 8 << 20  # a larger stack of partial products is added before it is handed on


# From operand tiles (one contiguous kilobyte a wave and k step) the staying kernel does better still, measured on
# MI355X at the Qwen3-4B shapes: narrow outputs from 9 rows on (down at 16 rows: 12.8 us against 21.1 us of the
# few-rows kernel, which stages x again for every column group); q|k|v (6144 columns) at 17..64 rows with eight
# waves a workgroup and four k splits: 10.1 against the library's 11.9 us at 32 rows, 12.1 against 16.3 us at 64;
# gate|up (19456 columns) stays level with the library, and stays there.
_STREAM_TILED_FROM_ROWS = 8
_STREAM_TILED_MAX_N = 8192
_STREAM_TILED_WIDE = (1, 4)     # (variant, k splits) for outputs wider than _STREAM_MAX_N
_STREAM_TILED_MANY_ROWS = 32    # from here on eight waves a workgroup (variant 1) for the narrow outputs too


def _stream_splits(rows: int, k: int, variant: int = _STREAM_VARIANT) -> int:
    return max(_STREAM_SPLITS, -(-k // (32 * _STREAM_STEPS_A_SPLIT)), _stream_min_splits(variant, rows, k))


def _stream_plan(rows: int, n: int, k: int, tiled: bool):
    """(variant, k splits) of the staying kernel for a product."""
    if tiled and n > _STREAM_MAX_N:
        variant, splits = _STREAM_TILED_WIDE
        return variant, max(splits, _stream_min_splits(variant, rows, k))
    variant = 1 if (tiled and rows > _STREAM_TILED_MANY_ROWS) else _STREAM_VARIANT
    return variant, _stream_splits(rows, k, variant)


def gemm_stream_preferred(rows: int, n: int, k: int, x_stride: int, tiled: bool = False) -> bool:
    """Whether the kernel whose workgroups stay should run this product: a long K, and from rows: 17..64 rows and a
    narrow output; from operand tiles: 9..64 rows and a narrow output, 17..64 rows and a middling one."""
    least = _STREAM_TILED_FROM_ROWS if (tiled and n <= _STREAM_MAX_N) else _ROWS_PREFERRED
    widest = _STREAM_TILED_MAX_N if tiled else _STREAM_MAX_N
    return (least < rows <= ROWS_KERNEL_MAX and n <= widest and k >= _STREAM_MIN_K
            and gemm_rows_supported(rows, k, x_stride))


_MM_OUT_DTYPE_OK = None


def _library_mm_f32out(x, w):
    """bfloat16 x bfloat16 -> float32 through the library.  With a torch that takes `out_dtype` the 32-bit
    accumulators are returned as they are; an older one hands back bfloat16, which is then only widened (the
    result has been rounded once).  Which torch this is, is asked once on a tiny product."""
    global _MM_OUT_DTYPE_OK
    if _MM_OUT_DTYPE_OK is None:
        probe = torch.zeros((16, 32), dtype=torch.bfloat16, device=x.device)
        try:
            torch.mm(probe, probe.t(), out_dtype=torch.float32)
            _MM_OUT_DTYPE_OK = True
        except (TypeError, RuntimeError):
            _MM_OUT_DTYPE_OK = False
    if _MM_OUT_DTYPE_OK:
        return torch.mm(x, w.t(), out_dtype=torch.float32)
    return torch.matmul(x, w.t()).float()


# ------------------------------------------------------ which kernel runs a product
#
# One place decides.  A choice names a kernel and what it needs to be launched; `product_by_rules` holds the
# thresholds that were measured at the Qwen3-4B, 8B and 32B widths (the constants above, each beside the numbers that
# set it); a table measured for a model's own widths (`arle_amd.kernels.tune`, `bench.py --tune-products`) takes
# their place where one is loaded: {(N, K, fused, tiled): [(most rows, choice), ...]}.  Another width then costs a
# run of the tuner, not a reading of these rules.


@dataclasses.dataclass(frozen=True)
class ProductChoice:
    kernel: str            # "rows", "stream", "rounds", "tiles", "tiles_parts", "library", "library_parts"
    variant: tuple = ()    # the kernel's own variant, where it has several
    splits: int = 0        # parts of K; 0: the kernel's own plan


PRODUCT_KERNELS = ("rows", "stream", "rounds", "tiles", "tiles_parts", "library", "library_parts")
_PRODUCT_TABLE: dict = {}


def product_by_rules(rows: int, n: int, k: int, x_stride: int, *, tiled: bool, fused: bool, partials_ok: bool,
                     aligned: bool = True) -> ProductChoice:
    """The kernel for x[rows, k] . w[n, k]^T by the measured thresholds.  fused: gate|up with SiLU·mul (w holds
    gate and up rows interleaved in blocks of 16), whose result is the activation [rows, n/2]."""
    if fused:
        if rows and aligned and gemm_rows_preferred(rows, n, k, x_stride, fused=True):
            return ProductChoice("rows", (_fused_variant(rows),), 1)
        if rows and aligned and tiled and gemm_rows_rounds_preferred(rows, n, k, x_stride):
            return ProductChoice("rounds")
        if aligned and tiled and gemm_tiles_preferred(rows, n, k, x_stride, fused=True):
            return ProductChoice("tiles", (8, 144) if rows >= _TILES_BIG_ROWS else (4, 44))
        return ProductChoice("library")
    staying = aligned and gemm_stream_preferred(rows, n, k, x_stride, tiled=tiled)
    if not staying and aligned and gemm_rows_preferred(rows, n, k, x_stride):
        return ProductChoice("rows")
    if staying:
        variant, splits = _stream_plan(rows, n, k, tiled)
        return ProductChoice("stream", (variant,), splits)
    if partials_ok and tiled and aligned:
        splits = narrow_tiles_splits(rows, n, k, x_stride)
        if splits:
            return ProductChoice("tiles_parts", _NARROW_TILES_VARIANT, splits)
    if partials_ok:
        splits = library_k_splits(rows, n, k)
        if splits > 1:
            return ProductChoice("library_parts", (), splits)
    return ProductChoice("library")


_CANDIDATE_STACK_BYTES = 32 << 20     # a candidate may leave a stack of partial products of at most this size


def product_candidates(rows: int, n: int, k: int, x_stride: int, *, tiled: bool, fused: bool) -> list:
    """Every choice that can run this shape (what a tuner times against each other): the library whole and in parts
    of K, and the hand-written kernels in their variants with several numbers of parts."""
    found = [ProductChoice("library")]
    eight = k % 8 == 0 and x_stride % 8 == 0
    few = gemm_rows_supported(rows, k, x_stride)
    steps = -(-k // 32)
    small = lambda parts: parts * rows * n * 4 <= _CANDIDATE_STACK_BYTES
    if fused:
        if few and n % 32 == 0:
            for variant in (_V_GENERAL, _V_FUSED_FEW, _V_SHARED, 4):
                if _rows_geometry(variant)[2] == 1 and _rows_min_splits(variant, rows, k) == 1:
                    found.append(ProductChoice("rows", (variant,), 1))
            if tiled:
                found.append(ProductChoice("rounds"))
                longest = _rows_round_steps(rows, k)
                for round_steps in (8, 13, 20, 27, 40):       # shorter rounds than the longest that fits
                    if round_steps < longest:
                        found.append(ProductChoice("rounds", (round_steps,)))
        if tiled and eight and n % 32 == 0 and rows > ROWS_KERNEL_MAX:
            found += [ProductChoice("tiles", v) for v in ((4, 44), (8, 144))]
        return found
    if few:
        for variant in range(ROWS_VARIANTS):
            least = _rows_min_splits(variant, rows, k)
            for parts in (1, 2, 3, 4, 6, 8):
                if least <= parts <= steps and small(parts):
                    found.append(ProductChoice("rows", (variant,), parts))
        for variant in range(STREAM_VARIANTS):
            least = _stream_min_splits(variant, rows, k)
            for parts in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16):
                if least <= parts <= steps and small(parts):
                    found.append(ProductChoice("stream", (variant,), parts))
                    if parts in (2, 4, 8):      # and with two workgroups for every compute unit
                        found.append(ProductChoice("stream", (variant, 2 * _STREAM_TARGET_WORKGROUPS // parts), parts))
    if rows > ROWS_KERNEL_MAX // 2:
        for parts in (2, 4, 8):
            if k % (32 * parts) == 0 and small(parts):
                found.append(ProductChoice("library_parts", (), parts))
            if tiled and eight and rows <= 1024 and k >= 320 * parts and small(parts):
                found.append(ProductChoice("tiles_parts", _NARROW_TILES_VARIANT, parts))
    return list(dict.fromkeys(found))


def load_product_table(table) -> None:
    """Take a measured table in: {"N,K,fused,tiled": [[most rows, kernel, variant, splits], ...]} (what the tuner
    writes, or the path of its JSON file).  Entries are looked up by the exact widths; other widths keep the rules."""
    import json

    if isinstance(table, (str, bytes)) or hasattr(table, "__fspath__"):
        with open(table, encoding="utf-8") as fh:
            table = json.load(fh)
    for key, entries in table.items():
        if isinstance(key, str):
            n, k, fused, tiled = key.split(",")
            key = (int(n), int(k), fused.strip() in ("1", "True", "true"), tiled.strip() in ("1", "True", "true"))
        parsed = []
        for most_rows, kernel, variant, splits in entries:
            _need(kernel in PRODUCT_KERNELS, f"a product table names the kernel {kernel!r}; known: {', '.join(PRODUCT_KERNELS)}")
            parsed.append((int(most_rows), ProductChoice(kernel, tuple(variant), int(splits))))
        _PRODUCT_TABLE[key] = sorted(parsed, key=lambda e: e[0])


def clear_product_table() -> None:
    _PRODUCT_TABLE.clear()


def choose_product(rows: int, n: int, k: int, x_stride: int, *, tiled: bool, fused: bool, partials_ok: bool,
                   aligned: bool = True) -> ProductChoice:
    """The table's entry for these widths and this many rows if there is one (the tables were measured with operands
    on the 16-byte grid: others go by the rules), else `product_by_rules`."""
    on_grid = aligned and k % 8 == 0 and x_stride % 8 == 0
    entries = _PRODUCT_TABLE.get((n, k, fused, tiled)) if on_grid and _PRODUCT_TABLE else None
    if entries:
        for most_rows, choice in entries:
            if rows <= most_rows:
                return choice
    return product_by_rules(rows, n, k, x_stride, tiled=tiled, fused=fused, partials_ok=partials_ok, aligned=aligned)


def run_product(choice: ProductChoice, x, w, tiles, out_dtype, partials_ok: bool, fused: bool = False):
    """Launch what `choice` names.  Plain products come back as [M, N] in out_dtype, or, where the caller said
    partials_ok, possibly as a float32 stack [S, M, N]; fused ones as the activation [M, N/2]."""
    kernel = choice.kernel
    if fused:
        if kernel == "rows":
            return gemm_rows(x, w, x.dtype, EPI_SILU_MUL, variant=choice.variant[0] if choice.variant else None,
                             splits=1 if choice.variant else None, tiles=tiles)
        if kernel == "rounds":
            return gemm_rows_rounds(x, w, x.dtype, tiles=tiles, round_steps=choice.variant[0] if choice.variant else None)
        if kernel == "tiles":
            return gemm_tiles(x, tiles, w.shape[0], x.dtype, EPI_SILU_MUL, variant=choice.variant or None)
        return silu_mul_interleaved(gemm_bf16(x, w, x.dtype, tiles=tiles), 16)
    if kernel == "rows":
        out = gemm_rows(x, w, out_dtype, variant=choice.variant[0] if choice.variant else None,
                        splits=choice.splits or None, tiles=tiles)
    elif kernel == "stream":
        out = gemm_stream(x, w, out_dtype, variant=choice.variant[0] if choice.variant else _STREAM_VARIANT,
                          splits=choice.splits or None, workgroups=choice.variant[1] if len(choice.variant) > 1 else None,
                          tiles=tiles)
    elif kernel == "tiles_parts":
        out = gemm_tiles(x, tiles, w.shape[0], torch.float32, variant=choice.variant or _NARROW_TILES_VARIANT,
                         splits=choice.splits)
    elif kernel == "tiles":
        out = gemm_tiles(x, tiles, w.shape[0], out_dtype, variant=choice.variant or None)
    elif kernel == "library_parts":
        out = _library_mm_split_k(x, w, choice.splits)
        if out is None:
            out = _library_mm_f32out(x, w) if out_dtype == torch.float32 else torch.matmul(x, w.t())
    else:
        out = _library_mm_f32out(x, w) if out_dtype == torch.float32 else torch.matmul(x, w.t())
    # a large stack is added here by many workgroups; the consumer would add it with one workgroup a row
    if out.dim() == 3 and (not partials_ok or (kernel in ("rows", "stream") and out.numel() * 4 > _STREAM_PARTIAL_BYTES)):
        out = sum_partials(out, out_dtype)
    elif out.dim() == 2 and out.dtype != out_dtype:
        out = out.to(out_dtype)
    return out


def gate_up_act(x: torch.Tensor, w: torch.Tensor, tiles: torch.Tensor | None = None, act: int = 0) -> torch.Tensor:
    """act(x . gate^T) * (x . up^T) for w [2I, K] holding gate and up rows interleaved in blocks of 16: [M, I];
    act 0: silu, 1: the tanh form of gelu."""
    _gpu(x, w)
    _rows(x, "x")
    rows, n, k = x.shape[0], w.shape[0], x.shape[1]
    if rows == 0:
        return torch.empty((0, n // 2), dtype=x.dtype, device=x.device)
    if act != 0:     # the products that apply the activation themselves know silu only
        return act_mul_interleaved(gemm_bf16(x, w, x.dtype, tiles=tiles), act, 16)
    choice = choose_product(rows, n, k, x.stride(0), tiled=tiles is not None, fused=True, partials_ok=False,
                            aligned=x.data_ptr() % 16 == 0)
    return run_product(choice, x, w, tiles, x.dtype, False, fused=True)


PRODUCT_TABLE_ENV = "ARLE_AMD_PRODUCT_TABLE"   # the path of a table that is taken in when this module is loaded ("none": no table at all)
PRODUCT_TABLE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tables")


def load_shipped_product_tables() -> int:
    """The tables that come with the package (measured on an MI355X for the widths of Qwen3-4B, 8B and 32B)."""
    count = 0
    if os.path.isdir(PRODUCT_TABLE_DIR):
        for name in sorted(os.listdir(PRODUCT_TABLE_DIR)):
            if name.endswith(".json"):
                load_product_table(os.path.join(PRODUCT_TABLE_DIR, name))
                count += 1
    return count


if os.environ.get(PRODUCT_TABLE_ENV, "") != "none":
    load_shipped_product_tables()
    if os.environ.get(PRODUCT_TABLE_ENV):
        load_product_table(os.environ[PRODUCT_TABLE_ENV])


# ------------------------------------------------- layer norm with the adds of a parallel block


def _term_args(term, bias, shape):
    """(pointer, stack depth, stack stride, type code, bias pointer, bias type code) of one addend of add_layernorm."""
    if term is None:
        _need(bias is None, "a bias without its term")
        return (0, 0, 0, 0, 0, 0)
    _need(term.dim() in (2, 3) and tuple(term.shape[-2:]) == tuple(shape) and term.is_contiguous() and term.dtype in _CODES,
          "an addend must match the residual ([T, H] or a float32 stack [S, T, H])")
    _need(term.dim() == 2 or (term.dtype == torch.float32 and term.shape[0] >= 1), "a stack of partial sums is float32")
    if bias is not None:
        _need(bias.shape == (shape[1],) and bias.is_contiguous() and bias.dtype in _CODES, "an addend's bias must be [H]")
    return (term.data_ptr(), term.shape[0] if term.dim() == 3 else 1, shape[0] * shape[1], _code(term),
            _ptr(bias), _code(bias) if bias is not None else 0)


LAYERNORM_MAX_WIDTH = 16384


def add_layernorm(residual: torch.Tensor, terms, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
                  weight_b: torch.Tensor | None = None, rows: torch.Tensor | None = None, *,
                  bias: torch.Tensor | None = None, bias_b: torch.Tensor | None = None):
    """residual += sum of `terms` (float32, in place unless `rows` is given); then the layer norm of
    every row (or of the rows named by `rows`), once with `weight` and, if given, once more with `weight_b`;
    `bias`, `bias_b`: the norms' own biases, of their weights' type (None: none).

    terms: up to two (tensor, bias or None); a tensor is [T, H] or a float32 stack [S, T, H] added in order.
    Returns out, or (out, out_b)."""
    terms = list(terms or [])
    _need(len(terms) <= 2, "add_layernorm adds at most two terms")
    _gpu(residual, weight, weight_b, rows, bias, bias_b, *[t for pair in terms for t in pair])
    for c in (bias, bias_b):
        _need(c is None or (c.shape == weight.shape and c.is_contiguous() and c.dtype == weight.dtype),
              "a norm's bias must be [width] of its weight's type")
    _need(bias_b is None or weight_b is not None, "a second bias without a second weight")
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(),
          "residual must be contiguous float32 [T, H]")
    width = residual.shape[1]
    _need(0 < width <= LAYERNORM_MAX_WIDTH, f"layer norm takes widths up to {LAYERNORM_MAX_WIDTH}")
    _need(weight.shape == (width,) and weight.is_contiguous(), "norm weight must be [width]")
    if weight_b is not None:
        _need(weight_b.shape == (width,) and weight_b.is_contiguous() and weight_b.dtype == weight.dtype,
              "the second norm weight must be [width] of the first one's type")
    n_rows = residual.shape[0]
    if rows is not None:
        _i32(rows, "rows")
        n_rows = rows.numel()
    out = torch.empty((n_rows, width), dtype=out_dtype, device=residual.device)
    out_b = torch.empty_like(out) if weight_b is not None else None
    args = []
    for i in range(2):
        args += _term_args(*(terms[i] if i < len(terms) else (None, None)), residual.shape)
    lib.call("arle_add_layernorm", residual.data_ptr(), *args, weight.data_ptr(), _ptr(weight_b), _code(weight),
             out.data_ptr(), _ptr(out_b), _code(out), _ptr(rows), n_rows, width, float(eps), _ptr(bias), _ptr(bias_b),
             _stream())
    return out if weight_b is None else (out, out_b)


# ------------------------------------------------------------- short causal convolution with state

CONV_MAX_TAPS = 16


def causal_conv(u: torch.Tensor, weight, state, slot_of_token: torch.Tensor, *, bias=None, add_input: bool = False,
                out_dtype: torch.dtype | None = None, silu: bool = False):
    """y_t = (u_t if add_input) + sum_j weight[:, j] * u_(t - taps + 1 + j) per channel, over the rows of each request
    (consecutive in u) and, further back, over its state [slots, taps-1, C]; u counts with `bias` added.  weight
    None: y = u + bias.  silu: y / (1 + exp(-y)) is what comes out.  The state is not changed: `conv_state_update`
    does that once the step's rows are done."""
    _gpu(u, weight, state, slot_of_token, bias)
    _rows(u, "u")
    tokens, channels = u.shape
    _i32(slot_of_token, "slot_of_token", tokens)
    taps = 1
    if weight is not None:
        _need(weight.dim() == 2 and weight.shape[0] == channels and weight.is_contiguous() and weight.dtype in _CODES,
              "a convolution weight must be contiguous [channels, taps]")
        taps = weight.shape[1]
        _need(1 <= taps <= CONV_MAX_TAPS, f"the short convolution takes 1..{CONV_MAX_TAPS} taps")
        if taps > 1:
            _need(state is not None and state.dim() == 3 and tuple(state.shape[1:]) == (taps - 1, channels)
                  and state.is_contiguous() and state.dtype in _CODES, "conv state must be [slots, taps-1, channels]")
    if bias is not None:
        _need(bias.shape == (channels,) and bias.is_contiguous() and bias.dtype in _CODES, "conv bias must be [channels]")
    out = torch.empty((tokens, channels), dtype=out_dtype or u.dtype, device=u.device)
    has_state = weight is not None and taps > 1
    lib.call("arle_causal_conv", u.data_ptr(), u.stride(0), _code(u), _ptr(bias), _code(bias) if bias is not None else 0,
             _ptr(weight), _code(weight) if weight is not None else 0, state.data_ptr() if has_state else 0,
             _code(state) if has_state else 0, slot_of_token.data_ptr(), out.data_ptr(), out.stride(0), _code(out),
             tokens, channels, taps, (1 if add_input else 0) | (2 if silu else 0), _stream())
    return out


def conv_state_update(u: torch.Tensor, state: torch.Tensor, seg_row0: torch.Tensor, seg_slot: torch.Tensor, *, bias=None):
    """state[slot] <- the last taps-1 rows of (state[slot], the request's rows of u (+ bias)), for every segment."""
    _gpu(u, state, seg_row0, seg_slot, bias)
    _rows(u, "u")
    channels = u.shape[1]
    _need(state.dim() == 3 and state.shape[2] == channels and state.is_contiguous() and state.dtype in _CODES
          and state.shape[1] < CONV_MAX_TAPS, "conv state must be [slots, taps-1, channels]")
    segments = seg_slot.numel()
    _i32(seg_slot, "seg_slot")
    _i32(seg_row0, "seg_row0", segments + 1)
    lib.call("arle_conv_state_update", u.data_ptr(), u.stride(0), _code(u), _ptr(bias),
             _code(bias) if bias is not None else 0, state.data_ptr(), _code(state), seg_row0.data_ptr(),
             seg_slot.data_ptr(), segments, channels, state.shape[1] + 1, _stream())


# ------------------------------------------------------------------------ PolyNorm activation


def polynorm(u: torch.Tensor, coef: torch.Tensor, eps: float, *, bias=None, out_dtype: torch.dtype | None = None):
    """a N(z) + b N(z^2) + c N(z^3) + e over rows of z = u + bias; N divides a row by its root mean square;
    coef = (a, b, c, e) on the GPU."""
    _gpu(u, coef, bias)
    _rows(u, "u")
    tokens, width = u.shape
    _need(coef.shape == (4,) and coef.is_contiguous() and coef.dtype in _CODES, "PolyNorm takes four coefficients")
    _need(0 < width <= 24576, "PolyNorm takes rows of up to 24,576 values")
    if bias is not None:
        _need(bias.shape == (width,) and bias.is_contiguous() and bias.dtype in _CODES, "the bias must be [width]")
    out = torch.empty((tokens, width), dtype=out_dtype or u.dtype, device=u.device)
    lib.call("arle_polynorm", u.data_ptr(), u.stride(0), _code(u), _ptr(bias), _code(bias) if bias is not None else 0,
             coef.data_ptr(), _code(coef), out.data_ptr(), _code(out), tokens, width, float(eps), _stream())
    return out


# ------------------------------------------------------------------------ mLSTM matrix memory

MLSTM_MAX_KEY_DIM = 256


def mlstm_scan(q, k, v, gates, bias_i, bias_f, cap: float, s_state, n_state, m_state, seg_row0, seg_slot, *,
               heads: int, key_dim: int, value_dim: int):
    """The matrix-memory recurrence over the rows of every segment, from and into the requests' states.  Returns
    (num float32 [T, heads * value_dim], nq float32 [T, heads], coefs float32 [T, heads, 3]): the numerators
    S_t^T q_t and n_t . q_t with q scaled by key_dim^(-1/2), and (keep, take, m_t) of every row and head, for
    `mlstm_output`.  gates float32 [T, 2 * heads]: pre-activations of the input gates, then of the forget gates."""
    _gpu(q, k, v, gates, bias_i, bias_f, s_state, n_state, m_state, seg_row0, seg_slot)
    H, D, Dv = heads, key_dim, value_dim
    tokens = q.shape[0]
    for name, t, width in (("q", q, H * D), ("k", k, H * D), ("v", v, H * Dv)):
        _rows(t, name)
        _need(t.shape == (tokens, width) and t.dtype == q.dtype, f"{name} must be [T, {width}] of one type")
    _need(0 < D <= MLSTM_MAX_KEY_DIM, f"the mLSTM kernels take key sizes up to {MLSTM_MAX_KEY_DIM}")
    _rows(gates, "gates")
    _need(gates.dtype == torch.float32 and gates.shape == (tokens, 2 * H), "gates must be float32 [T, 2 * heads]")
    _need(bias_i.shape == (H,) and bias_f.shape == (H,) and bias_i.dtype == bias_f.dtype == torch.float32
          and bias_i.is_contiguous() and bias_f.is_contiguous(), "gate biases must be float32 [heads]")
    slots = s_state.shape[0]
    _need(s_state.shape == (slots, H, D, Dv) and n_state.shape == (slots, H, D) and m_state.shape == (slots, H)
          and all(t.dtype == torch.float32 and t.is_contiguous() for t in (s_state, n_state, m_state)),
          "mLSTM states are float32 [slots, H, D, Dv], [slots, H, D] and [slots, H]")
    segments = seg_slot.numel()
    _i32(seg_slot, "seg_slot")
    _i32(seg_row0, "seg_row0", segments + 1)
    coefs = torch.empty((tokens, H, 3), dtype=torch.float32, device=q.device)
    num = torch.empty((tokens, H * Dv), dtype=torch.float32, device=q.device)
    nq = torch.empty((tokens, H), dtype=torch.float32, device=q.device)
    lib.call("arle_mlstm_scan", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), _code(q),
             gates.data_ptr(), gates.stride(0), bias_i.data_ptr(), bias_f.data_ptr(), float(cap),
             s_state.data_ptr(), n_state.data_ptr(), m_state.data_ptr(), seg_row0.data_ptr(), seg_slot.data_ptr(),
             segments, coefs.data_ptr(), num.data_ptr(), nq.data_ptr(), H, D, Dv, _stream())
    return num, nq, coefs


def mlstm_output(num, nq, coefs, gate, weight, eps: float, out_dtype, *, heads: int, value_dim: int):
    """o = num / (max(|nq|, exp(-m)) + 1e-6); then each head's o divided by its root mean square, times `weight`
    [heads * value_dim], times sigmoid(gate)."""
    _gpu(num, nq, coefs, gate, weight)
    tokens = num.shape[0]
    width = heads * value_dim
    _need(num.dtype == torch.float32 and num.shape == (tokens, width) and num.is_contiguous(), "num must be float32 [T, H * Dv]")
    _need(nq.dtype == torch.float32 and nq.shape == (tokens, heads) and nq.is_contiguous()
          and coefs.dtype == torch.float32 and coefs.shape == (tokens, heads, 3) and coefs.is_contiguous(),
          "nq [T, H] and coefs [T, H, 3] must be float32")
    _rows(gate, "gate")
    _need(gate.shape == (tokens, width) and gate.dtype in _CODES, "gate must be [T, H * Dv]")
    _need(weight.shape == (width,) and weight.is_contiguous() and weight.dtype in _CODES, "the norm weight must be [H * Dv]")
    out = torch.empty((tokens, width), dtype=out_dtype, device=num.device)
    lib.call("arle_mlstm_output", num.data_ptr(), nq.data_ptr(), coefs.data_ptr(), gate.data_ptr(), gate.stride(0),
             _code(gate), weight.data_ptr(), _code(weight), out.data_ptr(), _code(out), tokens, heads, value_dim,
             float(eps), _stream())
    return out


# --------------------------------------------------- soft-capped attention with a distance penalty


def _check_kv_pages(k_pages, v_pages, nkv, page_size, Dk, Dv, dtype):
    _need(k_pages.dim() == 4 and tuple(k_pages.shape[1:]) == (nkv, page_size, Dk) and k_pages.is_contiguous()
          and k_pages.dtype == dtype, "k_pages must be contiguous [pages, nkv, page_size, Dk]")
    _need(v_pages.dim() == 4 and tuple(v_pages.shape[1:]) == (nkv, Dv, page_size) and v_pages.is_contiguous()
          and v_pages.dtype == dtype and v_pages.shape[0] == k_pages.shape[0],
          "v_pages must be contiguous [pages, nkv, Dv, page_size]")


def qkv_norm_store(q, k, v, *, num_q_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, eps: float,
                   q_weight=None, k_weight=None, temp_coef: float = 0.0, temp_every: int = 1, positions=None,
                   slot_of_token=None, block_table=None, k_pages=None, v_pages=None, page_size: int = 0):
    """Per-head RMS norm of q (in place, then times 1 + temp_coef ln(floor((p + 1) / temp_every) + 1)) and of k;
    k and v go to the pages.  num_kv_heads 0 (k, v None): only q, for a layer that reads another layer's pages."""
    _gpu(q, k, v, q_weight, k_weight, positions, slot_of_token, block_table, k_pages, v_pages)
    tokens = q.shape[0]
    _rows(q, "q")
    _need(q.shape == (tokens, num_q_heads * key_dim) and q.dtype in _CODES, "q must be [T, heads * Dk]")
    _need(0 < key_dim <= MAX_HEAD_DIM and 0 < value_dim, "head sizes out of range")
    _i32(positions, "positions", tokens)
    w_code = 0
    for w in (q_weight, k_weight):
        if w is not None:
            _need(w.shape == (key_dim,) and w.is_contiguous() and w.dtype in _CODES, "a q/k norm weight must be [Dk]")
            w_code = _code(w)
    if q_weight is not None and k_weight is not None:
        _need(q_weight.dtype == k_weight.dtype, "q and k norm weights must be of one type")
    table_stride = 0
    if num_kv_heads:
        _rows(k, "k")
        _rows(v, "v")
        _need(k.shape == (tokens, num_kv_heads * key_dim) and v.shape == (tokens, num_kv_heads * value_dim)
              and k.dtype == q.dtype and v.dtype == q.dtype, "k, v must be [T, kv heads * Dk], [T, kv heads * Dv]")
        _check_kv_pages(k_pages, v_pages, num_kv_heads, page_size, key_dim, value_dim, q.dtype)
        _i32(slot_of_token, "slot_of_token", tokens)
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
              "block_table must be contiguous int32 [slots, pages]")
        table_stride = block_table.shape[1]
    _need(temp_coef == 0.0 or temp_every >= 1, "the query temperature's period must be positive")
    kk, vv = (k, v) if num_kv_heads else (q, q)
    lib.call("arle_qkv_norm_store", q.data_ptr(), q.stride(0), kk.data_ptr(), kk.stride(0), vv.data_ptr(), vv.stride(0),
             _code(q), _ptr(q_weight), _ptr(k_weight), w_code, float(eps), float(temp_coef), int(temp_every),
             positions.data_ptr(), _ptr(slot_of_token) if num_kv_heads else 0, _ptr(block_table) if num_kv_heads else 0,
             table_stride, _ptr(k_pages) if num_kv_heads else 0, _ptr(v_pages) if num_kv_heads else 0, tokens,
             num_q_heads, num_kv_heads, key_dim, value_dim, int(page_size), _stream())


def attn_softcap_simt(q, out, k_pages, v_pages, block_table, positions, slot_of_token, *, num_q_heads: int,
                      num_kv_heads: int, key_dim: int, value_dim: int, page_size: int, scale: float,
                      softcap: float = 0.0, r1=None, r2=None, window: int = 0, chunk: int = 0, sink=None,
                      keep_first: int = 0):
    """Causal attention of every row over its request's pages: scores scale (q . k), soft-capped (softcap > 0), less
    r1_h ln(1 + r2_h distance) (r1, r2 [heads] given), over the last `window` keys (0: all) and, with `chunk` > 0,
    over the keys of the row's own chunk of so many positions only; `sink` [heads]: exp(sink_h) joins the softmax's
    denominator; `keep_first` (with a window): the request's first so many keys stay visible behind the window."""
    _need(keep_first >= 0 and (keep_first == 0 or window > 0), "kept first keys go with a window")
    _gpu(q, out, k_pages, v_pages, block_table, positions, slot_of_token, r1, r2, sink)
    _check_sink(sink, num_q_heads, window, chunk)
    tokens = q.shape[0]
    _rows(q, "q")
    _rows(out, "out")
    _need(q.shape == (tokens, num_q_heads * key_dim) and out.shape == (tokens, num_q_heads * value_dim)
          and out.dtype == q.dtype, "q [T, nq*Dk] and out [T, nq*Dv] must be of one type")
    _need(num_kv_heads > 0 and num_q_heads % num_kv_heads == 0, "number of q heads must be a multiple of the kv heads")
    _need(max(key_dim, value_dim) <= CAP_SIMT_MAX_DIM and num_q_heads <= _GRID_Y_MAX, "head sizes or counts out of range")
    _check_kv_pages(k_pages, v_pages, num_kv_heads, page_size, key_dim, value_dim, q.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    _i32(positions, "positions", tokens)
    _i32(slot_of_token, "slot_of_token", tokens)
    _need((r1 is None) == (r2 is None), "give both distance constants or neither")
    if r1 is not None:
        _need(r1.shape == (num_q_heads,) and r2.shape == (num_q_heads,) and r1.dtype == r2.dtype and r1.dtype in _CODES
              and r1.is_contiguous() and r2.is_contiguous(), "r1, r2 must be [heads] of one type")
    lib.call("arle_attn_softcap_simt", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(),
             v_pages.data_ptr(), _code(q), block_table.data_ptr(), block_table.shape[1], positions.data_ptr(),
             slot_of_token.data_ptr(), tokens, num_q_heads, num_kv_heads, key_dim, value_dim, page_size, float(scale),
             float(softcap), _ptr(r1), _ptr(r2), _code(r1) if r1 is not None else 0, int(window), int(chunk), _ptr(sink),
             _code(sink) if sink is not None else 0, int(keep_first), _stream())
    return out


def _check_sink(sink, num_q_heads: int, window: int, chunk: int) -> None:
    _need(window >= 0 and chunk >= 0, "a window and a chunk size are not negative")
    if sink is not None:
        _need(sink.shape == (num_q_heads,) and sink.is_contiguous() and sink.dtype in _CODES, "sink must be [heads]")


def mask_span(window: int, chunk: int) -> int:
    """The most keys a row sees under a window and a chunk size (0 for either: none); 0: all earlier keys."""
    return min(window, chunk) if window > 0 and chunk > 0 else max(window, chunk)


CAP_MFMA_MAX_DIM = 256
CAP_SIMT_MAX_DIM = 1024     # the widest head the fixed-order kernel of this family takes


def attn_softcap_mfma_supported(dtype, key_dim: int, value_dim: int, page_size: int, group: int) -> bool:
    """Whether the matrix-core kernel of the soft-capped attention takes this shape."""
    return (dtype == torch.bfloat16 and key_dim % 8 == 0 and value_dim % 16 == 0 and page_size % 16 == 0
            and key_dim <= CAP_MFMA_MAX_DIM and value_dim <= CAP_MFMA_MAX_DIM)


def _softcap_page_ids(window: int, table_width: int, page_size: int, keep_first: int = 0) -> int:
    """Page ids that a work item of the matrix-core kernel keeps in LDS (the launcher's own count)."""
    mapped = table_width * page_size
    seen = (window + 16 if 0 < window and window + 16 < mapped else mapped) + 64
    return seen // page_size + 2 + (keep_first + 31) // page_size + 2


def attn_softcap_mfma_fits(window: int, table_width: int, page_size: int, keep_first: int = 0) -> bool:
    """Whether the ids of the pages that a row's keys span (its window, or all that the block table maps, and the
    kept first keys) fit where the matrix-core kernel keeps them."""
    return _softcap_page_ids(window, table_width, page_size, keep_first) * 4 <= 48 * 1024


@functools.lru_cache(maxsize=None)
def _softcap_lds_limit() -> int:
    return int(lib.function("arle_attn_softcap_lds_limit")())


def attn_softcap_mfma(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, *, max_qlen: int,
                      num_q_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, page_size: int, scale: float,
                      softcap: float = 0.0, r1=None, r2=None, window: int = 0, chunk: int = 0, sink=None,
                      keep_first: int = 0):
    """`attn_softcap_simt` on the matrix cores, bfloat16: sixteen rows of a segment a wave, or (when every segment is
    one decoded row) one row's q heads of a kv head, sixteen at a time, a wave.  keep_first (with a window and no
    chunks): the request's first so many keys stay visible to rows whose window has passed them."""
    _need(keep_first >= 0 and (keep_first == 0 or (window > 0 and chunk == 0)),
          "kept first keys go with a window and without chunks in the matrix-core kernel")
    _gpu(q, out, k_pages, v_pages, block_table, seg_row0, seg_slot, seg_start, r1, r2, sink)
    _check_sink(sink, num_q_heads, window, chunk)
    tokens = q.shape[0]
    _rows(q, "q")
    _rows(out, "out")
    group = num_q_heads // max(num_kv_heads, 1)
    _need(attn_softcap_mfma_supported(q.dtype, key_dim, value_dim, page_size, group), "shape outside the matrix-core kernel's")
    _need(q.shape == (tokens, num_q_heads * key_dim) and out.shape == (tokens, num_q_heads * value_dim)
          and out.dtype == q.dtype, "q [T, nq*Dk] and out [T, nq*Dv] must be bfloat16")
    _need(num_kv_heads > 0 and num_q_heads % num_kv_heads == 0 and num_q_heads <= _GRID_Y_MAX, "head counts out of range")
    _need(q.stride(0) % 8 == 0 and out.stride(0) % 8 == 0 and q.data_ptr() % 16 == 0 and out.data_ptr() % 16 == 0,
          "rows of q and out must be 16-byte aligned")
    _check_kv_pages(k_pages, v_pages, num_kv_heads, page_size, key_dim, value_dim, q.dtype)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    segments = seg_slot.numel()
    _i32(seg_slot, "seg_slot")
    _i32(seg_start, "seg_start", segments)
    _i32(seg_row0, "seg_row0", segments + 1)
    _need((r1 is None) == (r2 is None), "give both distance constants or neither")
    if r1 is not None:
        _need(r1.shape == (num_q_heads,) and r2.shape == (num_q_heads,) and r1.dtype == r2.dtype and r1.dtype in _CODES
              and r1.is_contiguous() and r2.is_contiguous(), "r1, r2 must be [heads] of one type")
    _need(attn_softcap_mfma_fits(mask_span(window, chunk), block_table.shape[1], page_size, keep_first),
          "the keys a row sees span more pages than the kernel holds ids for")
    # a decoded row's waves add their sums through LDS: that and the page ids have to fit a compute unit's
    page_ids = _softcap_page_ids(mask_span(window, chunk), block_table.shape[1], page_size, keep_first)
    heads_mode = (max_qlen == 1 and segments == tokens
                  and 8 * ((value_dim // 16) * 256 + 32) * 4 + page_ids * 4 <= _softcap_lds_limit())
    row_blocks = tokens // 16 + segments      # no fewer than the sixteen-row blocks of all segments together
    lib.call("arle_attn_softcap_mfma", q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), k_pages.data_ptr(),
             v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1], seg_row0.data_ptr(), seg_slot.data_ptr(),
             seg_start.data_ptr(), segments, row_blocks, 1 if heads_mode else 0, num_q_heads, num_kv_heads, key_dim,
             value_dim, page_size, float(scale), float(softcap), _ptr(r1), _ptr(r2),
             _code(r1) if r1 is not None else 0, int(window), int(chunk), _ptr(sink),
             _code(sink) if sink is not None else 0, int(keep_first), _stream())
    return out


def wide_norm_store(q, k, v, *, num_q_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, eps: float,
                    q_weight=None, k_weight=None, v_first=None, mix=None, positions, slot_of_token, block_table,
                    k_pages, v_pages, page_size: int, cos=None, sin=None, rotary_dim: int = 0, interleaved: bool = False):
    """RMS norm of q over its whole row (in place, weight [heads * Dk]) and of k over its whole row (weight
    [kv heads * Dk]); k goes to the pages, and so does v, as (1 - mix) v + mix v_first where v_first [T, kv heads * Dv]
    is given (`mix`: a tensor of one number).  rotary_dim > 0: behind the norm the first so many entries of every head
    of q and k turn by the angles of the float32 tables cos, sin [positions, rotary_dim / 2] (entry i with
    i + rotary_dim / 2, or with `interleaved` 2i with 2i + 1)."""
    _need(0 <= rotary_dim <= key_dim and rotary_dim % 2 == 0, "rotary_dim must be even and at most the head's size")
    _need(max(num_q_heads, num_kv_heads) * key_dim * 4 <= 64 * 1024 or not rotary_dim,
          "a rotated row of more than 16,384 entries is not taken")
    if rotary_dim:
        _gpu(cos, sin)
        for name, t in (("cos", cos), ("sin", sin)):
            _need(t is not None and t.dtype == torch.float32 and t.dim() == 2 and t.shape[1] == rotary_dim // 2
                  and t.is_contiguous(), f"{name} must be contiguous float32 [positions, rotary_dim / 2]")
    _gpu(q, k, v, q_weight, k_weight, v_first, mix, positions, slot_of_token, block_table, k_pages, v_pages)
    tokens = q.shape[0]
    for name, t, width in (("q", q, num_q_heads * key_dim), ("k", k, num_kv_heads * key_dim),
                           ("v", v, num_kv_heads * value_dim)):
        _rows(t, name)
        _need(t.shape == (tokens, width) and t.dtype == q.dtype and t.dtype in _CODES, f"{name} must be [T, {width}]")
    w_code = 0
    for w, width in ((q_weight, num_q_heads * key_dim), (k_weight, num_kv_heads * key_dim)):
        if w is not None:
            _need(w.shape == (width,) and w.is_contiguous() and w.dtype in _CODES, "a whole-row norm weight spans the row")
            w_code = _code(w)
    if q_weight is not None and k_weight is not None:
        _need(q_weight.dtype == k_weight.dtype, "q and k norm weights must be of one type")
    if v_first is not None:
        _rows(v_first, "v_first")
        _need(v_first.shape == v.shape and v_first.dtype == v.dtype, "v_first must match v")
        _need(mix is not None and mix.numel() == 1 and mix.dtype in _CODES, "the mixing weight is one number")
    _check_kv_pages(k_pages, v_pages, num_kv_heads, page_size, key_dim, value_dim, q.dtype)
    _i32(positions, "positions", tokens)
    _i32(slot_of_token, "slot_of_token", tokens)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    lib.call("arle_wide_norm_store", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
             _ptr(v_first), v_first.stride(0) if v_first is not None else 0, _code(q), _ptr(q_weight), _ptr(k_weight),
             w_code, _ptr(mix) if v_first is not None else 0, _code(mix) if v_first is not None else 0, float(eps),
             positions.data_ptr(), slot_of_token.data_ptr(), block_table.data_ptr(), block_table.shape[1],
             k_pages.data_ptr(), v_pages.data_ptr(), tokens, num_q_heads, num_kv_heads, key_dim, value_dim,
             int(page_size), _ptr(cos) if rotary_dim else 0, _ptr(sin) if rotary_dim else 0, int(rotary_dim),
             0 if interleaved else 1, _stream())


# ------------------------------------------------------------------ a norm on a sublayer's output

NORM_ADD_MAX_WIDTH = 16384


def _addend_args(term, rows: int, width: int):
    """(pointer, parts, part stride, row stride, weights pointer) of one float32 addend of `norm_add`: a tensor [T, W];
    a stack [S, T, W] of partial sums; or (outputs [T, n, W], weights [T, n])."""
    if term is None:
        return (0, 0, 0, 0, 0)
    if isinstance(term, tuple):
        outs, weights = term
        _need(outs.dim() == 3 and outs.shape[0] == rows and outs.shape[2] == width and outs.is_contiguous()
              and outs.dtype == torch.float32, "weighted outputs must be contiguous float32 [T, n, W]")
        _need(weights.shape == outs.shape[:2] and weights.dtype == torch.float32 and weights.is_contiguous(),
              "their weights must be contiguous float32 [T, n]")
        return (outs.data_ptr(), outs.shape[1], width, outs.shape[1] * width, weights.data_ptr())
    _need(term.dim() in (2, 3) and tuple(term.shape[-2:]) == (rows, width) and term.is_contiguous()
          and term.dtype == torch.float32 and term.shape[0] >= 1,
          "an addend must match the residual (float32 [T, W] or a stack [S, T, W])")
    return (term.data_ptr(), term.shape[0] if term.dim() == 3 else 1, rows * width, width, 0)


def norm_add(residual: torch.Tensor, terms, weight: torch.Tensor, eps: float, *, one_plus: bool = False,
             act_dtype: torch.dtype | None = None, center: bool = False, bias: torch.Tensor | None = None,
             mult: float = 1.0):
    """residual += mult * y / sqrt(mean(y^2) + eps) * weight (or 1 + weight) for y the sum of up to two `terms`, in
    place; with `center` the layer norm mult * ((y - mean) / sqrt(var + eps) * weight + bias) instead (bias [width] of
    the weight's type, or None); returns the updated residual rounded to `act_dtype` (None: nothing is returned)."""
    terms = [t for t in (terms if isinstance(terms, list) else [terms]) if t is not None]
    _need(1 <= len(terms) <= 2, "norm_add takes one or two addends")
    # what a sublayer leaves for the residual is 32-bit sums; an output that was rounded on its way is widened first
    terms = [t.float() if torch.is_tensor(t) and t.dtype == torch.bfloat16 else t for t in terms]
    _gpu(residual, weight, *[x for t in terms for x in (t if isinstance(t, tuple) else (t,))])
    _need(residual.dtype == torch.float32 and residual.dim() == 2 and residual.is_contiguous(),
          "residual must be contiguous float32 [T, W]")
    rows, width = residual.shape
    _need(0 < width <= NORM_ADD_MAX_WIDTH, f"norm_add takes widths up to {NORM_ADD_MAX_WIDTH}")
    _need(weight.shape == (width,) and weight.is_contiguous() and weight.dtype in _CODES, "norm weight must be [width]")
    _need(bias is None or (bias.is_cuda and bias.shape == (width,) and bias.is_contiguous() and bias.dtype == weight.dtype),
          "a norm's bias must be [width] of its weight's type")
    act = torch.empty((rows, width), dtype=act_dtype, device=residual.device) if act_dtype is not None else None
    args = []
    for i in range(2):
        args += _addend_args(terms[i] if i < len(terms) else None, rows, width)
    lib.call("arle_norm_add", residual.data_ptr(), *args, weight.data_ptr(), _code(weight), 1 if one_plus else 0,
             1 if center else 0, _ptr(bias), float(mult), _ptr(act), _code(act) if act is not None else 0, rows, width, float(eps), _stream())
    return act


def tanh_cap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap tanh(x / cap) in place on contiguous float32."""
    _gpu(x)
    _need(x.dtype == torch.float32 and x.is_contiguous() and cap > 0, "tanh_cap_ takes contiguous float32 and a positive cap")
    lib.call("arle_tanh_cap", x.data_ptr(), x.numel(), float(cap), _stream())
    return x


# ------------------------------------------------------------------ latent attention's operands

HEAD_PROJ_MAX_K = 1024


def latent_prep(q, dkv, q_full, *, heads: int, dim: int, rot_dim: int, rank: int, c_weight, eps: float, cos, sin,
                rotary_dims: int, positions, slot_of_token, block_table, k_pages, v_pages, page_size: int,
                halves: bool = False):
    """dkv [T, rank + rot_dim]: the first `rank` entries RMS-normed (c), the rest rotated (interleaved pairs over the
    first `rotary_dims`, or with `halves` entry i with i + rotary_dims / 2), [c | k_rot] to the key pages and c to the value pages; the rotated part of every head of
    q [T, heads * (dim + rot_dim)] goes, rotated, to the last rot_dim entries of its head in
    q_full [T, heads * (rank + rot_dim)]."""
    _gpu(q, dkv, q_full, c_weight, cos, sin, positions, slot_of_token, block_table, k_pages, v_pages)
    tokens = q.shape[0]
    for name, t, width in (("q", q, heads * (dim + rot_dim)), ("dkv", dkv, rank + rot_dim),
                           ("q_full", q_full, heads * (rank + rot_dim))):
        _rows(t, name)
        _need(t.shape == (tokens, width) and t.dtype == q.dtype and t.dtype in _CODES, f"{name} must be [T, {width}]")
    _need(c_weight.shape == (rank,) and c_weight.is_contiguous() and c_weight.dtype in _CODES, "the latent's norm weight must be [rank]")
    _need(0 <= rotary_dims <= rot_dim and rotary_dims % 2 == 0, "rotary dims must be even and within the rotated part")
    if rotary_dims:
        for name, t in (("cos", cos), ("sin", sin)):
            _need(t.dtype == torch.float32 and t.dim() == 2 and t.shape[1] == rotary_dims // 2 and t.is_contiguous(),
                  f"{name} must be contiguous float32 [positions, rotary_dims / 2]")
    _check_kv_pages(k_pages, v_pages, 1, page_size, rank + rot_dim, rank, q.dtype)
    _i32(positions, "positions", tokens)
    _i32(slot_of_token, "slot_of_token", tokens)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    lib.call("arle_latent_prep", q.data_ptr(), q.stride(0), dkv.data_ptr(), dkv.stride(0), q_full.data_ptr(),
             q_full.stride(0), _code(q), c_weight.data_ptr(), _code(c_weight), float(eps), _ptr(cos), _ptr(sin),
             int(rotary_dims), positions.data_ptr(), slot_of_token.data_ptr(), block_table.data_ptr(),
             block_table.shape[1], k_pages.data_ptr(), v_pages.data_ptr(), tokens, heads, dim, rot_dim, rank,
             int(page_size), 1 if halves else 0, _stream())


def head_proj(x, wt, out, *, heads: int, in_head: int, out_head: int):
    """out[t, h * out_head + n] = sum_k x[t, h * in_head + k] wt[h, k, n] for wt [heads, K, N]: a matrix of its own
    for every head, one fixed-order chain over k an output."""
    _gpu(x, wt, out)
    _rows(x, "x")
    _rows(out, "out")
    _need(wt.dim() == 3 and wt.shape[0] == heads and wt.is_contiguous(), "wt must be contiguous [heads, K, N]")
    K, N = wt.shape[1], wt.shape[2]
    _need(x.dtype == wt.dtype == out.dtype and x.dtype in _CODES, "x, wt and out must be of one type")
    _need(K <= HEAD_PROJ_MAX_K, f"head_proj takes inner sizes up to {HEAD_PROJ_MAX_K}")
    _need(x.shape[0] == out.shape[0] and (heads - 1) * in_head + K <= x.shape[1]
          and (heads - 1) * out_head + N <= out.shape[1], "a head's numbers must lie inside its row")
    lib.call("arle_head_proj", x.data_ptr(), x.stride(0), int(in_head), wt.data_ptr(), out.data_ptr(), out.stride(0),
             int(out_head), _code(x), x.shape[0], heads, K, N, _stream())
    return out


def head_proj_mfma_supported(x, heads: int, in_head: int, K: int) -> bool:
    """Whether the matrix-core form of `head_proj` takes these operands (bfloat16, 16-byte pieces)."""
    return (x.dtype == torch.bfloat16 and K % 8 == 0 and K >= 8 and in_head % 8 == 0 and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0)


def head_proj_mfma(x, wnk, out, *, heads: int, in_head: int, out_head: int):
    """`head_proj` on the matrix cores: bfloat16, every head's matrix stored wnk [heads, N, K]."""
    _gpu(x, wnk, out)
    _rows(x, "x")
    _rows(out, "out")
    _need(wnk.dim() == 3 and wnk.shape[0] == heads and wnk.is_contiguous(), "wnk must be contiguous [heads, N, K]")
    N, K = wnk.shape[1], wnk.shape[2]
    _need(x.dtype == wnk.dtype == out.dtype == torch.bfloat16, "x, wnk and out must be bfloat16")
    _need(head_proj_mfma_supported(x, heads, in_head, K), "operands outside the matrix-core kernel's")
    _need(x.shape[0] == out.shape[0] and (heads - 1) * in_head + K <= x.shape[1]
          and (heads - 1) * out_head + N <= out.shape[1], "a head's numbers must lie inside its row")
    lib.call("arle_head_proj_mfma", x.data_ptr(), x.stride(0), int(in_head), wnk.data_ptr(), out.data_ptr(),
             out.stride(0), int(out_head), x.shape[0], heads, K, N, _stream())
    return out


# ------------------------------------------------------------------ mixture of experts

MOE_MAX_EXPERTS = 1024
MOE_MAX_TOP = 64


def moe_route(x, router, correction, *, top: int, scale: float, score: str = "sigmoid", groups: int = 1,
              keep_groups: int = 1, normalize: bool = True):
    """(ids int32 [T, top], weights float32 [T, top]) of a router: z = router x in 32-bit sums, s = sigmoid(z) or
    (score "softmax") softmax(z) over all rows of the router, the `top` largest s + correction chosen (ties: the lower
    index) among the experts of the `keep_groups` best of `groups` equal groups of neighbours (a group's number: the
    largest s + correction in it), weights s / (sum + 1e-20) * scale, or s * scale without `normalize`, in the order
    they were chosen."""
    _need(score in ("sigmoid", "softmax"), "a router's scores are sigmoid or softmax")
    _gpu(x, router, correction)
    _rows(x, "x")
    experts, width = router.shape
    _need(router.dim() == 2 and router.is_contiguous() and router.dtype in _CODES and x.shape[1] == width and x.dtype in _CODES,
          "router must be contiguous [experts, width]")
    _need(1 <= top <= min(experts, MOE_MAX_TOP) and experts <= MOE_MAX_EXPERTS,
          f"the router takes up to {MOE_MAX_EXPERTS} experts and {MOE_MAX_TOP} choices a token")
    _need(groups >= 1 and experts % groups == 0 and 1 <= keep_groups <= groups and top <= keep_groups * (experts // groups),
          "groups divide the experts evenly, and the kept groups hold at least `top` experts")
    if correction is not None:
        _need(correction.shape == (experts,) and correction.is_contiguous() and correction.dtype in _CODES,
              "correction must be [experts]")
    ids = torch.empty((x.shape[0], top), dtype=torch.int32, device=x.device)
    weights = torch.empty((x.shape[0], top), dtype=torch.float32, device=x.device)
    lib.call("arle_moe_route", x.data_ptr(), x.stride(0), _code(x), router.data_ptr(), _code(router), _ptr(correction),
             _code(correction) if correction is not None else 0, ids.data_ptr(), weights.data_ptr(), x.shape[0], width,
             experts, int(top), float(scale), 1 if score == "softmax" else 0, int(groups), int(keep_groups),
             1 if normalize else 0, _stream())
    return ids, weights


def moe_identity(x, ids, outs, first: int):
    """Rows of experts that hand back their input: where ids [T, top] names a router output from `first` on, the row
    t * top + k of outs (float32 [T * top, W]) becomes x[t] (in 32 bits)."""
    _gpu(x, ids, outs)
    _rows(x, "x")
    tokens, top = ids.shape
    _need(ids.dtype == torch.int32 and ids.is_contiguous() and x.shape[0] == tokens and x.dtype in _CODES,
          "ids must be contiguous int32 [T, top] over the rows of x")
    _need(outs.dtype == torch.float32 and outs.is_contiguous() and outs.shape == (tokens * top, x.shape[1]),
          "outs must be contiguous float32 [T * top, W]")
    lib.call("arle_moe_identity", x.data_ptr(), x.stride(0), _code(x), ids.data_ptr(), outs.data_ptr(), tokens, top,
             x.shape[1], int(first), _stream())
    return outs


def moe_expert(x, w, ids, *, gate_up: bool):
    """The chosen experts' products.  gate_up: x [T, K], w [experts, 2N, K] (gate rows, then up rows) ->
    silu(gate) * up as [T * top, N] of x's type, row t * top + k for token t's k-th choice.  Else: x [T * top, K],
    w [experts, N, K] -> float32 [T * top, N]."""
    _gpu(x, w, ids)
    _rows(x, "x")
    _need(ids.dtype == torch.int32 and ids.dim() == 2 and ids.is_contiguous(), "ids must be contiguous int32 [T, top]")
    tokens, top = ids.shape
    _need(w.dim() == 3 and w.is_contiguous() and w.dtype == x.dtype and x.dtype in _CODES and w.shape[2] == x.shape[1],
          "w must be contiguous [experts, N, K] of x's type")
    _need(x.shape[0] == (tokens if gate_up else tokens * top), "x has a row a token (gate|up) or a row a choice (down)")
    _need(not gate_up or w.shape[1] % 2 == 0, "gate|up has an even number of rows")
    N = w.shape[1] // 2 if gate_up else w.shape[1]
    out = torch.empty((tokens * top, N), dtype=x.dtype if gate_up else torch.float32, device=x.device)
    lib.call("arle_moe_expert", x.data_ptr(), x.stride(0), w.data_ptr(), ids.data_ptr(), out.data_ptr(), _code(x),
             1 if gate_up else 0, tokens, w.shape[0], top, N, x.shape[1], _stream())
    return out


# ------------------------------------------------------------- gated feed-forward activations

ACT_SILU, ACT_GELU_TANH, ACT_SIGMOID = 0, 1, 2
ACTIVATIONS = {"silu": ACT_SILU, "gelu_tanh": ACT_GELU_TANH}      # of a gated feed-forward's gate
GATES = dict(ACTIVATIONS, sigmoid=ACT_SIGMOID)                    # of a gate on something that is not its own input


def gate_mul(gate: torch.Tensor, x: torch.Tensor, act: int = ACT_SIGMOID):
    """out = act(gate) * x for two [T, W] views of one type, each with a row stride of its own; out is contiguous."""
    _gpu(gate, x)
    _rows(gate, "gate")
    _rows(x, "x")
    _need(gate.shape == x.shape and gate.dtype == x.dtype and gate.dtype in _CODES, "gate and x must agree in shape and type")
    _need(act in GATES.values(), "unknown activation code")
    tokens, width = gate.shape
    _need(math.ceil(width / 256) <= _GRID_Y_MAX, "gate_mul: width too large")
    out = torch.empty((tokens, width), dtype=gate.dtype, device=gate.device)
    lib.call("arle_gate_mul", gate.data_ptr(), gate.stride(0), x.data_ptr(), x.stride(0), out.data_ptr(), _code(gate),
             tokens, width, int(act), _stream())
    return out


def token_gate(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, first: int, act: int = ACT_GELU_TANH):
    """out[t, j] = act(z[t, j]) * table[ids[t], first + j]: z [T, W], table [rows, >= first + W] (bfloat16 or float32),
    ids int32 [T] inside the table (the step's token ids, which the engine has checked against the vocabulary)."""
    _gpu(z, table, ids)
    _rows(z, "z")
    tokens, width = z.shape
    _need(z.dtype in _CODES and table.dtype in _CODES and table.dim() == 2 and table.stride(1) == 1, "table must be [rows, columns]")
    _need(0 <= first and first + width <= table.shape[1], "the slice does not lie in the table's columns")
    _i32(ids, "ids", tokens)
    _need(act in GATES.values(), "unknown activation code")
    out = torch.empty((tokens, width), dtype=z.dtype, device=z.device)
    lib.call("arle_token_gate", z.data_ptr(), z.stride(0), _code(z), table.data_ptr(), table.stride(0), _code(table),
             int(first), ids.data_ptr(), out.data_ptr(), tokens, width, int(act), _stream())
    return out


def act_mul(gate: torch.Tensor, up: torch.Tensor, act: int = ACT_SILU):
    """out = act(gate) * up for two [T, I] views with the same row stride; act: ACT_SILU or ACT_GELU_TANH
    (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))))."""
    _gpu(gate, up)
    _rows(gate, "gate")
    _rows(up, "up")
    _need(gate.shape == up.shape and gate.dtype == up.dtype and gate.stride(0) == up.stride(0),
          "gate and up must agree in shape, dtype and row stride")
    _need(act in (ACT_SILU, ACT_GELU_TANH), "unknown activation code")
    tokens, width = gate.shape
    _need(math.ceil(width / 256) <= _GRID_Y_MAX, "act_mul: width too large")
    out = torch.empty((tokens, width), dtype=gate.dtype, device=gate.device)
    lib.call("arle_act_mul", gate.data_ptr(), up.data_ptr(), gate.stride(0), out.data_ptr(), _code(gate), tokens, width,
             0, int(act), _stream())
    return out


def act_mul_interleaved(gate_up: torch.Tensor, act: int = ACT_SILU, block: int = 16):
    """`act_mul` for a [T, 2I] buffer whose columns alternate between `block` gate columns and the matching up columns."""
    _gpu(gate_up)
    _rows(gate_up, "gate_up")
    tokens, two_i = gate_up.shape
    _need(block > 0 and two_i % (2 * block) == 0, "interleaved gate/up width must be a multiple of 2*block")
    width = two_i // 2
    _need(math.ceil(width / 256) <= _GRID_Y_MAX, "act_mul: width too large")
    out = torch.empty((tokens, width), dtype=gate_up.dtype, device=gate_up.device)
    lib.call("arle_act_mul", gate_up.data_ptr(), gate_up.data_ptr(), gate_up.stride(0), out.data_ptr(), _code(gate_up),
             tokens, width, int(block), int(act), _stream())
    return out


# ------------------------------------------------------- residual streams with learned connections

HYPER_MAX_STREAMS = 16
HYPER_MAX_WIDTH = 16000


def _stack_args(y, rows: int, width: int, name: str):
    """(pointer, type code, row stride, parts, part stride) of a sublayer's output: a tensor [T, W] of a kernel type
    or a contiguous float32 stack [P, T, W] of partial sums."""
    if y.dim() == 3:
        _need(y.dtype == torch.float32 and y.is_contiguous() and tuple(y.shape[1:]) == (rows, width) and y.shape[0] >= 1,
              f"{name}: a stack of partial sums must be contiguous float32 [P, T, W]")
        return y.data_ptr(), F32, width, y.shape[0], rows * width
    _rows(y, name)
    _need(y.shape == (rows, width) and y.dtype in _CODES, f"{name} must be [T, W]")
    return y.data_ptr(), _code(y), y.stride(0), 1, 0


def hyper_step(streams: torch.Tensor, y, mix, out_w, in_w, norm_w: torch.Tensor, eps: float, out_dtype: torch.dtype, *,
               num_streams: int, rows=None):
    """One step of a residual of `num_streams` streams (see csrc/hyper.hip): write the output y of the sublayer before
    through its connection (mix [S, S] indexed [from, to], out_w [S]; y None: nothing to write), then read through the
    next sublayer's connection (in_w [S]; None: the plain sum) and RMS-norm with norm_w.

    streams: float32 [T, S, W], updated in place, or float32 [T, W] (every stream starts as a copy of it; a new
    [T, S, W] tensor is made).  rows (int32 [R]): only these tokens are read, nothing is written.  Returns
    (streams [T, S, W], normed [T or R, W] in out_dtype)."""
    _gpu(streams, y, mix, out_w, in_w, norm_w, rows)
    S = int(num_streams)
    _need(1 <= S <= HYPER_MAX_STREAMS, f"1..{HYPER_MAX_STREAMS} streams")
    _need(streams.dtype == torch.float32 and streams.is_contiguous() and streams.dim() in (2, 3),
          "streams must be contiguous float32 [T, S, W] or [T, W]")
    tokens, width = streams.shape[0], streams.shape[-1]
    _need(0 < width <= HYPER_MAX_WIDTH, f"hyper_step takes widths up to {HYPER_MAX_WIDTH}")
    if streams.dim() == 3:
        _need(streams.shape[1] == S, "streams must be [T, S, W]")
        src_strides, dst = (S * width, width), streams
    else:
        src_strides = (width, 0)
        dst = streams if rows is not None else torch.empty((tokens, S, width), dtype=torch.float32, device=streams.device)
    for name, t, shape in (("mix", mix, (S, S)), ("out_w", out_w, (S,)), ("in_w", in_w, (S,)), ("norm_w", norm_w, (width,))):
        if t is not None:
            _need(tuple(t.shape) == shape and t.dtype == torch.float32 and t.is_contiguous(), f"{name} must be float32 {shape}")
    y_args = (0, 0, 0, 0, 0)
    if y is not None:
        _need(mix is not None and out_w is not None, "an output is written through a connection")
        y_args = _stack_args(y, tokens, width, "y")
    grid = tokens
    if rows is not None:
        _i32(rows, "rows")
        grid = rows.numel()
    out = torch.empty((grid, width), dtype=out_dtype, device=streams.device)
    vec = (width % 4 == 0 and (y is None or (y_args[2] % 4 == 0 and y_args[0] % 16 == 0)))
    lib.call("arle_hyper_step", streams.data_ptr(), src_strides[0], src_strides[1],
             0 if rows is not None else dst.data_ptr(), *y_args, _ptr(mix), _ptr(out_w), _ptr(in_w), norm_w.data_ptr(),
             float(eps), _ptr(rows), out.data_ptr(), _CODES[out_dtype], width, grid, S, width, 1 if vec else 0, _stream())
    return dst, out


def pair_norm(a, b, weight_a, weight_b, eps: float, coef: float = 0.5):
    """float32 [T, W]: coef * (a / rms(a) * weight_a + b / rms(b) * weight_b), rms over W with eps inside the root;
    a and b are tensors [T, W] of one type or float32 stacks [P, T, W] of partial sums."""
    _gpu(a, b, weight_a, weight_b)
    tokens, width = a.shape[-2], a.shape[-1]
    if a.dtype != b.dtype:
        a, b = a.float(), b.float()
    pa, ca, sa, na, nsa = _stack_args(a, tokens, width, "a")
    pb, cb, sb, nb, nsb = _stack_args(b, tokens, width, "b")
    for w in (weight_a, weight_b):
        _need(w.shape == (width,) and w.dtype == torch.float32 and w.is_contiguous(), "the weights must be float32 [W]")
    out = torch.empty((tokens, width), dtype=torch.float32, device=a.device)
    vec = width % 4 == 0 and sa % 4 == 0 and sb % 4 == 0 and pa % 16 == 0 and pb % 16 == 0
    lib.call("arle_pair_norm", pa, sa, na, nsa, pb, sb, nb, nsb, ca, weight_a.data_ptr(), weight_b.data_ptr(), float(eps),
             float(coef), out.data_ptr(), tokens, width, 1 if vec else 0, _stream())
    return out


# ------------------------------------------------------ attention operands with rotary positions

ROTARY_MAX_HEAD_DIM = 1024


def rotary_qkv_store(q, k, v, *, num_q_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, eps: float,
                     q_weight=None, k_weight=None, unit_after: bool = False, cos=None, sin=None, rotary_dim: int = 0,
                     interleaved: bool = False, positions, slot_of_token, block_table, k_pages, v_pages, page_size: int):
    """Per head of q (in place) and k (to the pages): an RMS norm with a weight [Dk] in front of the rotation
    (q_weight, k_weight given), the rotation of the first `rotary_dim` entries by the angles of float32 tables
    cos, sin [positions, rotary_dim / 2] (pairs (i, i + rotary_dim / 2), or (2i, 2i + 1) if `interleaved`), and a
    division by the root mean square behind it (`unit_after`); v goes to the pages as it is."""
    _gpu(q, k, v, q_weight, k_weight, cos, sin, positions, slot_of_token, block_table, k_pages, v_pages)
    tokens = q.shape[0]
    for name, t, width in (("q", q, num_q_heads * key_dim), ("k", k, num_kv_heads * key_dim), ("v", v, num_kv_heads * value_dim)):
        _rows(t, name)
        _need(t.shape == (tokens, width) and t.dtype == q.dtype and t.dtype in _CODES, f"{name} must be [T, {width}]")
    _need(0 < key_dim <= ROTARY_MAX_HEAD_DIM and value_dim > 0 and num_q_heads + 2 * num_kv_heads <= _GRID_Y_MAX,
          "head sizes or counts out of range")
    _need((q_weight is None) == (k_weight is None), "give both norm weights or neither")
    w_code = 0
    if q_weight is not None:
        for w in (q_weight, k_weight):
            _need(w.shape == (key_dim,) and w.is_contiguous() and w.dtype in _CODES, "a q/k norm weight must be [Dk]")
        _need(q_weight.dtype == k_weight.dtype, "q and k norm weights must be of one type")
        w_code = _code(q_weight)
    _need(0 <= rotary_dim <= key_dim and rotary_dim % 2 == 0, "rotary_dim must be even and at most the key size")
    if rotary_dim:
        for name, t in (("cos", cos), ("sin", sin)):
            _need(t is not None and t.dtype == torch.float32 and t.dim() == 2 and t.shape[1] == rotary_dim // 2
                  and t.is_contiguous(), f"{name} must be contiguous float32 [positions, rotary_dim / 2]")
    _check_kv_pages(k_pages, v_pages, num_kv_heads, page_size, key_dim, value_dim, q.dtype)
    _i32(positions, "positions", tokens)
    _i32(slot_of_token, "slot_of_token", tokens)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be contiguous int32 [slots, pages]")
    lib.call("arle_rotary_qkv_store", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
             _code(q), _ptr(q_weight), _ptr(k_weight), w_code, float(eps), 1 if unit_after else 0, _ptr(cos), _ptr(sin),
             int(rotary_dim), 1 if interleaved else 0, positions.data_ptr(), slot_of_token.data_ptr(),
             block_table.data_ptr(), block_table.shape[1], k_pages.data_ptr(), v_pages.data_ptr(), tokens, num_q_heads,
             num_kv_heads, key_dim, value_dim, int(page_size), _stream())


# ------------------------------------------------------------------------- gated delta rule

GATED_DELTA_MAX_KEY_DIM = 256


def gated_delta_scan(q, k, v, gates, a_log, dt_bias, s_state, seg_row0, seg_slot, *, heads: int, kv_heads: int,
                     key_dim: int, value_dim: int, unit_eps: float = 1e-6, channel_decay=None):
    """The gated delta rule over the rows of every segment, from and into the requests' states (see
    csrc/gated_delta.hip).  q, k [T, kv_heads * D] and v [T, heads * Dv] as the convolutions left them; gates float32
    [T, >= 2 * heads]: the pre-activations of beta, then those of the decay; a_log, dt_bias float32 [heads]; s_state
    float32 [slots, heads, D, Dv].  channel_decay: float32 [T, heads * D], the pre-activations of a decay for every
    head and key entry; gates then holds beta's alone ([T, >= heads]) and dt_bias is [heads * D].
    Returns o float32 [T, heads * Dv]."""
    _gpu(q, k, v, gates, a_log, dt_bias, s_state, seg_row0, seg_slot, channel_decay)
    H, G, D, Dv = heads, kv_heads, key_dim, value_dim
    tokens = q.shape[0]
    for name, t, width in (("q", q, G * D), ("k", k, G * D), ("v", v, H * Dv)):
        _rows(t, name)
        _need(t.shape == (tokens, width) and t.dtype == q.dtype and t.dtype in _CODES, f"{name} must be [T, {width}] of one type")
    _need(0 < D <= GATED_DELTA_MAX_KEY_DIM and G > 0 and H % G == 0 and H <= _GRID_Y_MAX,
          f"key sizes up to {GATED_DELTA_MAX_KEY_DIM}, heads a multiple of the q/k heads")
    _rows(gates, "gates")
    channel = channel_decay is not None
    _need(gates.dtype == torch.float32 and gates.shape[0] == tokens and gates.shape[1] >= (H if channel else 2 * H),
          "gates must be float32 [T, >= 2 * heads] (with a decay a channel: [T, >= heads])")
    decays = H * D if channel else H
    if channel:
        _rows(channel_decay, "channel_decay")
        _need(channel_decay.dtype == torch.float32 and channel_decay.shape == (tokens, decays),
              "the channels' decays must be float32 [T, heads * D]")
    _need(a_log.shape == (H,) and dt_bias.shape == (decays,) and a_log.dtype == dt_bias.dtype == torch.float32
          and a_log.is_contiguous() and dt_bias.is_contiguous(), "A_log must be float32 [heads], dt_bias float32 [decays]")
    _need(s_state.dim() == 4 and tuple(s_state.shape[1:]) == (H, D, Dv) and s_state.dtype == torch.float32
          and s_state.is_contiguous(), "the state is float32 [slots, heads, D, Dv]")
    segments = seg_slot.numel()
    _i32(seg_slot, "seg_slot")
    _i32(seg_row0, "seg_row0", segments + 1)
    out = torch.empty((tokens, H * Dv), dtype=torch.float32, device=q.device)
    decay_ptr = channel_decay.data_ptr() if channel else gates.data_ptr() + 4 * H
    decay_stride = channel_decay.stride(0) if channel else gates.stride(0)
    lib.call("arle_gated_delta_scan", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
             _code(q), gates.data_ptr(), gates.stride(0), decay_ptr, decay_stride, a_log.data_ptr(), dt_bias.data_ptr(),
             float(unit_eps), s_state.data_ptr(), seg_row0.data_ptr(), seg_slot.data_ptr(), segments,
             1 if tokens == segments else 0, out.data_ptr(), H, G, D, Dv, 1 if channel else 0, _stream())
    return out


def gated_delta_output(o, gate, weight, eps: float, *, heads: int, value_dim: int, act: int = 0):
    """Each head's o [T, heads * Dv] (float32) divided by its root mean square, times weight [Dv], times act(gate)
    (act 0: silu; one of GATES' codes); in the type of `gate`."""
    _need(act in (0, 1, 2), "unknown activation code")
    _gpu(o, gate, weight)
    tokens = o.shape[0]
    width = heads * value_dim
    _need(o.dtype == torch.float32 and o.shape == (tokens, width) and o.is_contiguous(), "o must be float32 [T, H * Dv]")
    _rows(gate, "gate")
    _need(gate.shape == (tokens, width) and gate.dtype in _CODES, "gate must be [T, H * Dv]")
    _need(weight.shape == (value_dim,) and weight.is_contiguous() and weight.dtype in _CODES, "the norm weight must be [Dv]")
    _need(heads <= _GRID_Y_MAX, "too many heads")
    out = torch.empty((tokens, width), dtype=gate.dtype, device=o.device)
    lib.call("arle_gated_delta_output", o.data_ptr(), gate.data_ptr(), gate.stride(0), _code(gate), weight.data_ptr(),
             _code(weight), float(eps), out.data_ptr(), tokens, heads, value_dim, int(act), _stream())
    return out
