"""Tensor-level wrappers over the C ABI (libmi355_decode.so).

PyTorch is used only as the owner of device memory and streams: each wrapper
checks dtype/layout, then passes raw device pointers, sizes and the current HIP
stream to the library.  Every call is asynchronous on
``torch.cuda.current_stream()`` and allocates nothing unless it has to return a
new tensor (pass ``out=`` to avoid that, e.g. under HIP graph capture).
"""
from __future__ import annotations

import os

import torch

from . import _lib
from ._lib import BLOCK_SIZE, check, lib

_DT = {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_F16, torch.float32: _lib.DTYPE_F32}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got {t.device})")


def _dt16(t: torch.Tensor, name: str) -> int:
    _dev(t, name)
    if t.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"{name}: dtype {t.dtype} not supported (bfloat16/float16)")
    return _DT[t.dtype]


def _rows(t: torch.Tensor, name: str) -> int:
    """Row stride (elements) of a 2-D view whose last dim is contiguous."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be 2-D with a contiguous last dim (shape {tuple(t.shape)}, "
                         f"strides {t.stride()})")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor | None = None):
    dt = _dt16(x, "x")
    _dev(weight, "weight")
    if weight.dtype != x.dtype or weight.numel() != x.shape[1] or not weight.is_contiguous():
        raise ValueError("weight must be contiguous [hidden] in the dtype of x")
    if out is None:
        out = torch.empty_like(x, memory_format=torch.contiguous_format)
    check(lib.mi355_rms_norm(out.data_ptr(), x.data_ptr(), weight.data_ptr(), x.shape[0], x.shape[1],
                             _rows(x, "x"), _rows(out, "out"), float(eps), dt, _stream()))
    return out


def fused_add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float,
                       out: torch.Tensor | None = None):
    """residual <- x + residual (in place); returns rms_norm(residual).  ``out`` defaults to ``x``."""
    dt = _dt16(x, "x")
    _dev(residual, "residual"), _dev(weight, "weight")
    if residual.dtype != x.dtype or residual.shape != x.shape or weight.dtype != x.dtype:
        raise ValueError("residual must match x; weight must have the dtype of x")
    if weight.numel() != x.shape[1] or not weight.is_contiguous():
        raise ValueError("weight must be contiguous [hidden]")
    if out is None:
        out = x
    check(lib.mi355_fused_add_rms_norm(out.data_ptr(), x.data_ptr(), residual.data_ptr(), weight.data_ptr(),
                                       x.shape[0], x.shape[1], _rows(x, "x"), _rows(out, "out"),
                                       _rows(residual, "residual"), float(eps), dt, _stream()))
    return out


def _check_partial(partial: torch.Tensor, num_slabs: int, rows: int, width: int) -> None:
    _dev(partial, "partial")
    if (partial.dtype != torch.float32 or not partial.is_contiguous() or num_slabs < 1
            or partial.numel() < num_slabs * rows * width):
        raise ValueError("partial must be contiguous float32 holding [num_slabs, rows, width]")


def fused_add_rms_norm_partial(partial: torch.Tensor, num_slabs: int, residual: torch.Tensor,
                               weight: torch.Tensor, eps: float, out: torch.Tensor,
                               bias: torch.Tensor | None = None):
    """fused_add_rms_norm whose x is round(sum of the fp32 slabs partial[:num_slabs] (+ bias)):
    the partial-sum output of linear_tiled(..., epilogue=EPI_PARTIAL) over the same rows."""
    dt = _dt16(residual, "residual")
    _dev(weight, "weight"), _dev(out, "out")
    T, H = residual.shape
    _check_partial(partial, num_slabs, T, H)
    if weight.dtype != residual.dtype or weight.numel() != H or not weight.is_contiguous():
        raise ValueError("weight must be contiguous [hidden] in the dtype of residual")
    if out.dtype != residual.dtype or tuple(out.shape) != (T, H):
        raise ValueError("out must match residual")
    if bias is not None and (bias.dtype != residual.dtype or bias.numel() != H or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous [hidden] in the dtype of residual")
    check(lib.mi355_fused_add_rms_norm_partial(out.data_ptr(), partial.data_ptr(), num_slabs, T * H,
                                               bias.data_ptr() if bias is not None else 0, residual.data_ptr(),
                                               weight.data_ptr(), T, H, _rows(out, "out"),
                                               _rows(residual, "residual"), float(eps), dt, _stream()))
    return out


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor,
                  slot_mapping: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  num_heads: int, num_kv_heads: int, head_dim: int, partial: torch.Tensor | None = None,
                  num_slabs: int = 0, bias: torch.Tensor | None = None) -> None:
    """In-place rotary embedding on the q|k parts of ``qkv`` + paged store of k, v.
    k_cache [blocks, kv_heads, 16, head_dim]; v_cache [blocks, kv_heads, head_dim, 16].
    With ``partial`` (fp32 [num_slabs, tokens, width], the partial-sum output of
    linear_tiled) the rows are first formed as round(sum of slabs (+ bias)) and
    written to ``qkv`` in full."""
    dt = _dt16(qkv, "qkv")
    T = qkv.shape[0]
    for t, n in ((positions, "positions"), (slot_mapping, "slot_mapping")):
        _dev(t, n)
        if t.dtype != torch.int64 or t.numel() != T or not t.is_contiguous():
            raise ValueError(f"{n} must be contiguous int64 [num_tokens]")
    nb = k_cache.shape[0]
    if (tuple(k_cache.shape) != (nb, num_kv_heads, BLOCK_SIZE, head_dim)
            or tuple(v_cache.shape) != (nb, num_kv_heads, head_dim, BLOCK_SIZE)
            or not k_cache.is_contiguous() or not v_cache.is_contiguous()
            or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype):
        raise ValueError("k_cache/v_cache must be contiguous [blocks, kv_heads, 16, d] / [blocks, kv_heads, d, 16]")
    if cos_sin.dtype != qkv.dtype or cos_sin.dim() != 2 or cos_sin.shape[1] != head_dim or not cos_sin.is_contiguous():
        raise ValueError("cos_sin must be contiguous [max_position, head_dim] in the dtype of qkv")
    if qkv.shape[1] != (num_heads + 2 * num_kv_heads) * head_dim:
        raise ValueError("qkv width must be (num_heads + 2*num_kv_heads) * head_dim")
    if partial is not None:
        _check_partial(partial, num_slabs, T, qkv.shape[1])
        if bias is not None and (bias.dtype != qkv.dtype or bias.numel() != qkv.shape[1] or not bias.is_contiguous()):
            raise ValueError("bias must be contiguous [width] in the dtype of qkv")
        check(lib.mi355_rope_kv_write_partial(
            qkv.data_ptr(), _rows(qkv, "qkv"), partial.data_ptr(), num_slabs, T * qkv.shape[1],
            bias.data_ptr() if bias is not None else 0, positions.data_ptr(), cos_sin.data_ptr(), cos_sin.shape[0],
            slot_mapping.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), nb, T, num_heads, num_kv_heads,
            head_dim, dt, _stream()))
        return
    check(lib.mi355_rope_kv_write(qkv.data_ptr(), _rows(qkv, "qkv"), positions.data_ptr(), cos_sin.data_ptr(),
                                  cos_sin.shape[0], slot_mapping.data_ptr(), k_cache.data_ptr(),
                                  v_cache.data_ptr(), nb, T, num_heads, num_kv_heads, head_dim, dt, _stream()))


def decode_workspace_bytes(num_seqs: int, num_heads: int, head_dim: int, num_splits: int) -> int:
    return int(lib.mi355_paged_attn_decode_workspace(num_seqs, num_heads, head_dim, num_splits))


def _check_cache(q, k_cache, v_cache, block_tables, num_kv_heads, head_dim):
    nb = k_cache.shape[0]
    if (tuple(k_cache.shape) != (nb, num_kv_heads, BLOCK_SIZE, head_dim)
            or tuple(v_cache.shape) != (nb, num_kv_heads, head_dim, BLOCK_SIZE)
            or not k_cache.is_contiguous() or not v_cache.is_contiguous()
            or k_cache.dtype != q.dtype or v_cache.dtype != q.dtype):
        raise ValueError("k_cache/v_cache must be contiguous [blocks, kv_heads, 16, d] / [blocks, kv_heads, d, 16]")
    _dev(block_tables, "block_tables")
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be contiguous int32 [num_seqs, max_blocks]")
    return nb


def paged_attn_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, context_lens: torch.Tensor, num_heads: int,
                      num_kv_heads: int, head_dim: int, scale: float, num_splits: int = 1,
                      workspace: torch.Tensor | None = None, out: torch.Tensor | None = None):
    """q: 2-D view [num_seqs, >= num_heads*head_dim] (e.g. the q part of the qkv rows)."""
    dt = _dt16(q, "q")
    B = q.shape[0]
    nb = _check_cache(q, k_cache, v_cache, block_tables, num_kv_heads, head_dim)
    _dev(context_lens, "context_lens")
    if context_lens.dtype != torch.int32 or context_lens.numel() != B or not context_lens.is_contiguous():
        raise ValueError("context_lens must be contiguous int32 [num_seqs]")
    if block_tables.shape[0] != B:
        raise ValueError("block_tables rows must equal num_seqs")
    if out is None:
        out = torch.empty((B, num_heads * head_dim), dtype=q.dtype, device=q.device)
    elif not out.is_contiguous() or out.numel() != B * num_heads * head_dim or out.dtype != q.dtype:
        raise ValueError("out must be contiguous [num_seqs, num_heads*head_dim]")
    ws_ptr, ws_bytes = 0, 0
    if num_splits > 1:
        need = decode_workspace_bytes(B, num_heads, head_dim, num_splits)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
        ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    check(lib.mi355_paged_attn_decode(out.data_ptr(), q.data_ptr(), _rows(q, "q"), k_cache.data_ptr(),
                                      v_cache.data_ptr(), nb, block_tables.data_ptr(), block_tables.shape[1],
                                      context_lens.data_ptr(), B, num_heads, num_kv_heads, head_dim,
                                      float(scale), num_splits, ws_ptr, ws_bytes, dt, _stream()))
    return out


STATIC_SCRATCH_BYTES = 16 * 1024 * 1024       # MI355_PAGED_ATTN_DECODE_STATIC_MAX_BYTES


def paged_attn_decode_static(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                             block_tables: torch.Tensor, context_lens: torch.Tensor, num_heads: int,
                             num_kv_heads: int, head_dim: int, scale: float, num_splits: int, out: torch.Tensor):
    """paged_attn_decode through the entry point that allocates nothing: the split-KV partials live in
    the library's built-in device array, `out` must be given (this wrapper creates no tensor either)."""
    dt = _dt16(q, "q")
    B = q.shape[0]
    nb = _check_cache(q, k_cache, v_cache, block_tables, num_kv_heads, head_dim)
    _dev(context_lens, "context_lens")
    if context_lens.dtype != torch.int32 or context_lens.numel() != B or not context_lens.is_contiguous():
        raise ValueError("context_lens must be contiguous int32 [num_seqs]")
    if block_tables.shape[0] != B:
        raise ValueError("block_tables rows must equal num_seqs")
    if not out.is_contiguous() or out.numel() != B * num_heads * head_dim or out.dtype != q.dtype:
        raise ValueError("out must be contiguous [num_seqs, num_heads*head_dim]")
    check(lib.mi355_paged_attn_decode_static(out.data_ptr(), q.data_ptr(), _rows(q, "q"), k_cache.data_ptr(),
                                             v_cache.data_ptr(), nb, block_tables.data_ptr(), block_tables.shape[1],
                                             context_lens.data_ptr(), B, num_heads, num_kv_heads, head_dim,
                                             float(scale), num_splits, dt, _stream()))
    return out


def paged_attn_decode_fused(qkv: torch.Tensor | None, cos_sin: torch.Tensor, slot_mapping: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_tables: torch.Tensor, context_lens: torch.Tensor, num_heads: int,
                            num_kv_heads: int, head_dim: int, scale: float, num_splits: int = 1,
                            workspace: torch.Tensor | None = None, out: torch.Tensor | None = None,
                            partial: torch.Tensor | None = None, num_slabs: int = 0,
                            bias: torch.Tensor | None = None):
    """rope_kv_write + paged_attn_decode in one launch; the new token of a sequence is
    the one at position context_lens - 1.  The step's projection is either
    ``qkv`` (packed 16-bit rows [num_seqs, (nh + 2 nkv) d], left untouched) or ``partial``
    (fp32 [num_slabs, num_seqs, width] from linear_tiled, + ``bias``)."""
    B = slot_mapping.numel()
    width = (num_heads + 2 * num_kv_heads) * head_dim
    if partial is None:
        dt = _dt16(qkv, "qkv")
        if qkv.shape != (B, width):
            raise ValueError("qkv must be [num_seqs, (num_heads + 2*num_kv_heads) * head_dim]")
        ref = qkv
    else:
        dt = _dt16(k_cache, "k_cache")
        _check_partial(partial, num_slabs, B, width)
        if bias is not None and (bias.dtype != k_cache.dtype or bias.numel() != width or not bias.is_contiguous()):
            raise ValueError("bias must be contiguous [width] in the cache dtype")
        ref = k_cache
    nb = _check_cache(ref, k_cache, v_cache, block_tables, num_kv_heads, head_dim)
    _dev(slot_mapping, "slot_mapping")
    if slot_mapping.dtype != torch.int64 or not slot_mapping.is_contiguous():
        raise ValueError("slot_mapping must be contiguous int64 [num_seqs]")
    _dev(context_lens, "context_lens")
    if context_lens.dtype != torch.int32 or context_lens.numel() != B or not context_lens.is_contiguous():
        raise ValueError("context_lens must be contiguous int32 [num_seqs]")
    if block_tables.shape[0] != B:
        raise ValueError("block_tables rows must equal num_seqs")
    if cos_sin.dtype != ref.dtype or cos_sin.dim() != 2 or cos_sin.shape[1] != head_dim or not cos_sin.is_contiguous():
        raise ValueError("cos_sin must be contiguous [max_position, head_dim] in the model dtype")
    if out is None:
        out = torch.empty((B, num_heads * head_dim), dtype=ref.dtype, device=ref.device)
    elif not out.is_contiguous() or out.numel() != B * num_heads * head_dim or out.dtype != ref.dtype:
        raise ValueError("out must be contiguous [num_seqs, num_heads*head_dim]")
    ws_ptr, ws_bytes = 0, 0
    if num_splits > 1:
        need = decode_workspace_bytes(B, num_heads, head_dim, num_splits)
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=ref.device)
        ws_ptr, ws_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    check(lib.mi355_paged_attn_decode_fused(
        out.data_ptr(), qkv.data_ptr() if qkv is not None else 0, _rows(qkv, "qkv") if qkv is not None else 0,
        partial.data_ptr() if partial is not None else 0, num_slabs, B * width,
        bias.data_ptr() if bias is not None else 0, cos_sin.data_ptr(), cos_sin.shape[0],
        slot_mapping.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), nb, block_tables.data_ptr(),
        block_tables.shape[1], context_lens.data_ptr(), B, num_heads, num_kv_heads, head_dim, float(scale),
        num_splits, ws_ptr, ws_bytes, dt, _stream()))
    return out


def paged_attn_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                       block_tables: torch.Tensor, cu_seqlens: torch.Tensor, context_lens: torch.Tensor,
                       max_q_len: int, num_heads: int, num_kv_heads: int, head_dim: int, scale: float,
                       out: torch.Tensor | None = None):
    dt = _dt16(q, "q")
    T = q.shape[0]
    nb = _check_cache(q, k_cache, v_cache, block_tables, num_kv_heads, head_dim)
    S = block_tables.shape[0]
    for t, n, cnt in ((cu_seqlens, "cu_seqlens", S + 1), (context_lens, "context_lens", S)):
        _dev(t, n)
        if t.dtype != torch.int32 or t.numel() != cnt or not t.is_contiguous():
            raise ValueError(f"{n} must be contiguous int32 [{cnt}]")
    if out is None:
        out = torch.empty((T, num_heads * head_dim), dtype=q.dtype, device=q.device)
    check(lib.mi355_paged_attn_prefill(out.data_ptr(), _rows(out, "out"), q.data_ptr(), _rows(q, "q"),
                                       k_cache.data_ptr(), v_cache.data_ptr(), nb, block_tables.data_ptr(),
                                       block_tables.shape[1], cu_seqlens.data_ptr(), context_lens.data_ptr(),
                                       S, int(max_q_len), num_heads, num_kv_heads, head_dim, float(scale), dt,
                                       _stream()))
    return out


def chunk_attn_prefill_ok(dtype: torch.dtype, num_heads: int, num_kv_heads: int, head_dim: int, v_dim: int) -> bool:
    """Whether paged_attn_prefill_ext covers these sizes (16-bit storage, equal key and value sizes of 64 or 128,
    at most 16 query heads to a kv head)."""
    return dtype in (torch.bfloat16, torch.float16) and head_dim == v_dim and head_dim in (64, 128) \
        and num_heads % num_kv_heads == 0 and num_heads // num_kv_heads <= 16


def paged_attn_prefill_ext(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                           cu_seqlens: torch.Tensor, context_lens: torch.Tensor, max_q_len: int, num_heads: int,
                           num_kv_heads: int, head_dim: int, scale: float, chunk: int = 0, sink: torch.Tensor | None = None,
                           gate: torch.Tensor | None = None, out: torch.Tensor | None = None):
    """paged_attn_prefill (K/V steps staged through LDS for a workgroup's query tile) for attention inside
    chunks of `chunk` positions counted from position 0 (0: plain causal), with one more value-less term
    exp(sink[h]) in the softmax denominator (float32 [heads]) and the output times sigmoid(gate[t, h])
    (gate [tokens, heads], a column slice is fine).  q and out may be column slices on 16-byte boundaries."""
    dt = _dt16(q, "q")
    T = q.shape[0]
    nb = _check_cache(q, k_cache, v_cache, block_tables, num_kv_heads, head_dim)
    S = block_tables.shape[0]
    for t, n, cnt in ((cu_seqlens, "cu_seqlens", S + 1), (context_lens, "context_lens", S)):
        _dev(t, n)
        if t.dtype != torch.int32 or t.numel() != cnt or not t.is_contiguous():
            raise ValueError(f"{n} must be contiguous int32 [{cnt}]")
    if out is None:
        out = torch.empty((T, num_heads * head_dim), dtype=q.dtype, device=q.device)
    if out.dtype != q.dtype or tuple(out.shape) != (T, num_heads * head_dim):
        raise ValueError("out must be [tokens, heads * head_dim] in the dtype of q")
    check(lib.mi355_paged_attn_prefill_ext(
        out.data_ptr(), _rows(out, "out"), q.data_ptr(), _cols(q, "q", num_heads * head_dim), k_cache.data_ptr(),
        v_cache.data_ptr(), nb, block_tables.data_ptr(), block_tables.shape[1], cu_seqlens.data_ptr(), context_lens.data_ptr(),
        S, int(max_q_len), num_heads, num_kv_heads, head_dim, float(scale), int(chunk),
        None if sink is None else _f32(sink, "sink", num_heads), None if gate is None else _same(gate, q, "gate"),
        0 if gate is None else _cols(gate, "gate", num_heads), dt, _stream()))
    return out


def silu_and_mul(x: torch.Tensor, out: torch.Tensor | None = None):
    dt = _dt16(x, "x")
    T, two_f = x.shape
    if two_f % 2:
        raise ValueError("x must be [num_tokens, 2*inter]")
    inter = two_f // 2
    if out is None:
        out = torch.empty((T, inter), dtype=x.dtype, device=x.device)
    elif not out.is_contiguous() or tuple(out.shape) != (T, inter):
        raise ValueError("out must be contiguous [num_tokens, inter]")
    check(lib.mi355_silu_and_mul(out.data_ptr(), x.data_ptr(), _rows(x, "x"), T, inter, dt, _stream()))
    return out


def sum_slabs(partial: torch.Tensor, num_slabs: int, out: torch.Tensor, bias: torch.Tensor | None = None):
    """out[M, N] = round(sum of the first num_slabs fp32 slabs of `partial` ([num_slabs, M, N], flat is fine) + bias),
    slabs added in slab order: the 16-bit tensor an all-reduce needs from a K-split projection."""
    dt = _dt16(out, "out")
    M, N = out.shape
    _check_partial(partial, num_slabs, M, N)
    if bias is not None and (bias.dtype != out.dtype or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous [N] in the dtype of out")
    check(lib.mi355_sum_slabs(out.data_ptr(), _rows(out, "out"), partial.data_ptr(), num_slabs,
                              bias.data_ptr() if bias is not None else 0, M, N, dt, _stream()))
    return out


def silu_and_mul_slabs(partial: torch.Tensor, num_slabs: int, out: torch.Tensor):
    """SwiGLU from the slabs of a K-split gate_up projection on weights tiled with interleave_halves
    ([num_slabs, M, 2F], 16-column tiles alternating gate / up): out[M, F], the values the GEMM's own
    SwiGLU epilogue would have produced from the same sums."""
    dt = _dt16(out, "out")
    M, F = out.shape
    _check_partial(partial, num_slabs, M, 2 * F)
    check(lib.mi355_silu_and_mul_slabs(out.data_ptr(), _rows(out, "out"), partial.data_ptr(), num_slabs, M, 2 * F, dt,
                                       _stream()))
    return out


def argmax(logits: torch.Tensor, out: torch.Tensor | None = None):
    _dev(logits, "logits")
    if logits.dtype not in _DT:
        raise TypeError(f"logits dtype {logits.dtype} not supported")
    B, V = logits.shape
    if out is None:
        out = torch.empty(B, dtype=torch.int64, device=logits.device)
    check(lib.mi355_argmax(out.data_ptr(), logits.data_ptr(), _rows(logits, "logits"), B, V,
                           _DT[logits.dtype], _stream()))
    return out


def argmax_chunked(logits: torch.Tensor, keys: torch.Tensor, out: torch.Tensor, out2: torch.Tensor | None = None):
    """argmax for a decode batch: rows cut into column ranges over many workgroups.  `keys` int64
    [>= rows] must be zero before the first call (every call leaves it zero); `out2` gets the ids too."""
    _dev(logits, "logits"), _dev(keys, "keys"), _dev(out, "out")
    if logits.dtype not in _DT:
        raise TypeError(f"logits dtype {logits.dtype} not supported")
    B, V = logits.shape
    for t, n in ((keys, "keys"), (out, "out")) + (((out2, "out2"),) if out2 is not None else ()):
        if t.dtype != torch.int64 or t.numel() < B or not t.is_contiguous():
            raise ValueError(f"{n} must be contiguous int64 with at least one element per row")
    check(lib.mi355_argmax_chunked(out.data_ptr(), out2.data_ptr() if out2 is not None else 0, keys.data_ptr(),
                                   logits.data_ptr(), _rows(logits, "logits"), B, V, _DT[logits.dtype], _stream()))
    return out


def embed_rms_norm(embed: torch.Tensor, token_ids: torch.Tensor, weight: torch.Tensor, eps: float,
                   residual: torch.Tensor, out: torch.Tensor):
    """residual <- embed[token_ids]; out <- rms_norm(residual): the first launch of a decode step."""
    dt = _dt16(embed, "embed")
    _dev(token_ids, "token_ids"), _dev(weight, "weight"), _dev(residual, "residual"), _dev(out, "out")
    T = token_ids.numel()
    H = embed.shape[1]
    if token_ids.dtype != torch.int64 or not token_ids.is_contiguous():
        raise ValueError("token_ids must be contiguous int64")
    if weight.dtype != embed.dtype or weight.numel() != H or not weight.is_contiguous():
        raise ValueError("weight must be contiguous [hidden] in the dtype of embed")
    for t, n in ((residual, "residual"), (out, "out")):
        if t.dtype != embed.dtype or tuple(t.shape) != (T, H):
            raise ValueError(f"{n} must be [num_tokens, hidden] in the dtype of embed")
    check(lib.mi355_embed_rms_norm(out.data_ptr(), residual.data_ptr(), embed.data_ptr(), token_ids.data_ptr(),
                                   embed.shape[0], weight.data_ptr(), T, H, _rows(embed, "embed"), _rows(out, "out"),
                                   _rows(residual, "residual"), float(eps), dt, _stream()))
    return out


def _affine(weight: torch.Tensor, bias: torch.Tensor, hidden: int, dtype) -> None:
    for t, n in ((weight, "weight"), (bias, "bias")):
        _dev(t, n)
        if t.dtype != dtype or t.numel() != hidden or not t.is_contiguous():
            raise ValueError(f"{n} must be contiguous [hidden] in the dtype of the rows")


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float,
               out: torch.Tensor | None = None):
    """LayerNorm with weight and bias over the rows of x (OPT-style decoders)."""
    dt = _dt16(x, "x")
    _affine(weight, bias, x.shape[1], x.dtype)
    if out is None:
        out = torch.empty_like(x, memory_format=torch.contiguous_format)
    check(lib.mi355_layer_norm(out.data_ptr(), x.data_ptr(), weight.data_ptr(), bias.data_ptr(), x.shape[0], x.shape[1],
                               _rows(x, "x"), _rows(out, "out"), float(eps), dt, _stream()))
    return out


def fused_add_layer_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float,
                         out: torch.Tensor | None = None):
    """residual <- x + residual (in place); returns layer_norm(residual).  ``out`` defaults to ``x``."""
    dt = _dt16(x, "x")
    _dev(residual, "residual")
    if residual.dtype != x.dtype or residual.shape != x.shape:
        raise ValueError("residual must match x")
    _affine(weight, bias, x.shape[1], x.dtype)
    if out is None:
        out = x
    check(lib.mi355_fused_add_layer_norm(out.data_ptr(), x.data_ptr(), residual.data_ptr(), weight.data_ptr(),
                                         bias.data_ptr(), x.shape[0], x.shape[1], _rows(x, "x"), _rows(out, "out"),
                                         _rows(residual, "residual"), float(eps), dt, _stream()))
    return out


def embed_pos_layer_norm(embed: torch.Tensor, token_ids: torch.Tensor, pos_embed: torch.Tensor,
                         positions: torch.Tensor, position_offset: int, weight: torch.Tensor, bias: torch.Tensor,
                         eps: float, residual: torch.Tensor, out: torch.Tensor):
    """residual <- embed[token_ids] + pos_embed[positions + position_offset]; out <- layer_norm(residual):
    the first launch of an OPT-style step."""
    dt = _dt16(embed, "embed")
    _dev(token_ids, "token_ids"), _dev(positions, "positions"), _dev(residual, "residual"), _dev(out, "out")
    _dev(pos_embed, "pos_embed")
    T, H = token_ids.numel(), embed.shape[1]
    for t, n in ((token_ids, "token_ids"), (positions, "positions")):
        if t.dtype != torch.int64 or t.numel() != T or not t.is_contiguous():
            raise ValueError(f"{n} must be contiguous int64 [num_tokens]")
    if pos_embed.dtype != embed.dtype or pos_embed.dim() != 2 or pos_embed.shape[1] != H:
        raise ValueError("pos_embed must be [num_positions, hidden] in the dtype of embed")
    _affine(weight, bias, H, embed.dtype)
    for t, n in ((residual, "residual"), (out, "out")):
        if t.dtype != embed.dtype or tuple(t.shape) != (T, H):
            raise ValueError(f"{n} must be [num_tokens, hidden] in the dtype of embed")
    check(lib.mi355_embed_pos_layer_norm(out.data_ptr(), residual.data_ptr(), embed.data_ptr(), token_ids.data_ptr(),
                                         embed.shape[0], _rows(embed, "embed"), pos_embed.data_ptr(),
                                         positions.data_ptr(), pos_embed.shape[0], int(position_offset),
                                         _rows(pos_embed, "pos_embed"), weight.data_ptr(), bias.data_ptr(), T, H,
                                         _rows(out, "out"), _rows(residual, "residual"), float(eps), dt, _stream()))
    return out


def relu(x: torch.Tensor, out: torch.Tensor | None = None):
    """x < 0 ? 0 : x (NaN and -0.0 kept); in place by default."""
    dt = _dt16(x, "x")
    if out is None:
        out = x
    _dev(out, "out")
    if not x.is_contiguous() or not out.is_contiguous() or out.dtype != x.dtype or out.numel() != x.numel():
        raise ValueError("x and out must be contiguous tensors of one size and dtype")
    check(lib.mi355_relu(out.data_ptr(), x.data_ptr(), x.numel(), dt, _stream()))
    return out


def argmax_shard_key(logits: torch.Tensor, index_offset: int, out: torch.Tensor | None = None):
    """Key of the best token of a vocabulary slice whose first row is token `index_offset`:
    a signed 64-bit max over the slices' keys is the key of the argmax of the whole vocabulary
    (argmax_key_to_index turns it into the token id)."""
    _dev(logits, "logits")
    if logits.dtype not in _DT:
        raise TypeError(f"logits dtype {logits.dtype} not supported")
    B, V = logits.shape
    if out is None:
        out = torch.empty(B, dtype=torch.int64, device=logits.device)
    check(lib.mi355_argmax_shard_key(out.data_ptr(), logits.data_ptr(), _rows(logits, "logits"), B, V,
                                     _DT[logits.dtype], int(index_offset), _stream()))
    return out


def argmax_key_to_index(keys: torch.Tensor, out: torch.Tensor | None = None):
    _dev(keys, "keys")
    if keys.dtype != torch.int64 or not keys.is_contiguous():
        raise TypeError("keys must be contiguous int64")
    if out is None:
        out = torch.empty_like(keys)
    check(lib.mi355_argmax_key_to_index(out.data_ptr(), keys.data_ptr(), keys.numel(), _stream()))
    return out


LINEAR_DECODE_MAX_M = 128


def token_logprobs(logits: torch.Tensor, token_ids: torch.Tensor):
    """(logprob of token_ids[b] in row b, logsumexp of row b), both float32 [rows]."""
    _dev(logits, "logits"), _dev(token_ids, "token_ids")
    ldt = _DT.get(logits.dtype)
    if ldt is None or logits.dim() != 2 or logits.stride(1) != 1:
        raise TypeError("logits must be a 2-D bf16/fp16/fp32 tensor with unit column stride")
    B, V = logits.shape
    if token_ids.dtype != torch.int64 or token_ids.numel() != B or not token_ids.is_contiguous():
        raise ValueError("token_ids must be contiguous int64 [rows]")
    lp = torch.empty(B, dtype=torch.float32, device=logits.device)
    lse = torch.empty(B, dtype=torch.float32, device=logits.device)
    check(lib.mi355_token_logprobs(lp.data_ptr(), lse.data_ptr(), logits.data_ptr(), _rows(logits, "logits"), B, V,
                                   ldt, token_ids.data_ptr(), _stream()))
    return lp, lse


TOPK_MAX = 64


def topk_logits(logits: torch.Tensor, k: int, lse: torch.Tensor | None = None):
    """(token ids int64 [rows, k], values float32 [rows, k]) of the k largest logits of every row, most likely
    first, ties to the lower id; with `lse` (float32 [rows]) the values are log-probabilities."""
    _dev(logits, "logits")
    ldt = _DT.get(logits.dtype)
    if ldt is None or logits.dim() != 2 or logits.stride(1) != 1:
        raise TypeError("logits must be a 2-D bf16/fp16/fp32 tensor with unit column stride")
    B, V = logits.shape
    if lse is not None and (lse.dtype != torch.float32 or lse.numel() != B or not lse.is_contiguous() or not lse.is_cuda):
        raise ValueError("lse must be contiguous float32 [rows] on the device")
    ids = torch.empty((B, k), dtype=torch.int64, device=logits.device)
    vals = torch.empty((B, k), dtype=torch.float32, device=logits.device)
    check(lib.mi355_topk_logits(ids.data_ptr(), vals.data_ptr(), logits.data_ptr(), _rows(logits, "logits"), B, V, ldt,
                                int(k), lse.data_ptr() if lse is not None else 0, _stream()))
    return ids, vals


def linear_decode(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
                  out: torch.Tensor | None = None, k_slices: int = 0):
    """y = x @ weight.T (+ bias) for decode batches (M <= 128): weights streamed once."""
    dt = _dt16(x, "x")
    _dev(weight, "weight")
    M, K = x.shape
    if weight.dtype != x.dtype or weight.dim() != 2 or weight.shape[1] != K or not weight.is_contiguous():
        raise ValueError("weight must be contiguous [N, K] in the dtype of x")
    N = weight.shape[0]
    if bias is not None and (bias.dtype != x.dtype or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous [N] in the dtype of x")
    if out is None:
        out = torch.empty((M, N), dtype=x.dtype, device=x.device)
    elif out.dtype != x.dtype or tuple(out.shape) != (M, N):
        raise ValueError("out must be [M, N] in the dtype of x")
    check(lib.mi355_linear_decode(out.data_ptr(), _rows(out, "out"), x.data_ptr(), _rows(x, "x"), weight.data_ptr(),
                                  bias.data_ptr() if bias is not None else 0, M, N, K, int(k_slices), dt, _stream()))
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           seeds: torch.Tensor, steps: torch.Tensor, out: torch.Tensor | None = None, cut_rows: bool = True):
    """Per-row sampling (greedy where temperature <= 0).  temperature/top_p float32 [B], top_k int32 [B],
    seeds/steps int64 [B], all on the device.  cut_rows=False: the caller knows that no row has an active
    top-k / top-p, so the follow-up launches that serve rows with huge kept sets are left out (same tokens)."""
    _dev(logits, "logits")
    if logits.dtype not in _DT:
        raise TypeError(f"logits dtype {logits.dtype} not supported")
    B, V = logits.shape
    for t, n, dt in ((temperature, "temperature", torch.float32), (top_k, "top_k", torch.int32),
                     (top_p, "top_p", torch.float32), (seeds, "seeds", torch.int64), (steps, "steps", torch.int64)):
        _dev(t, n)
        if t.dtype != dt or t.numel() != B or not t.is_contiguous():
            raise ValueError(f"{n} must be contiguous {dt} [num_rows]")
    if out is None:
        out = torch.empty(B, dtype=torch.int64, device=logits.device)
    check(lib.mi355_sample_topk_topp_hinted(out.data_ptr(), logits.data_ptr(), _rows(logits, "logits"), B, V,
                                            _DT[logits.dtype], temperature.data_ptr(), top_k.data_ptr(),
                                            top_p.data_ptr(), seeds.data_ptr(), steps.data_ptr(),
                                            1 if cut_rows else 0, _stream()))
    return out


EPI_STORE, EPI_SILU_MUL, EPI_PARTIAL, EPI_REDUCE_STORE, EPI_REDUCE_RESID = 0, 1, 2, 3, 4
SUMSQ_ROWS = 32                      # row pitch of the sum-of-squares tables
LINEAR_TILED_MAX_M = 256             # beyond 128 rows: two row blocks of one launch


KW_CODES = (302, 304, 308, 402, 404)   # K split across 2 / 4 / 8 waves of an 8-wave workgroup (4xx: 512-wide x slices)


def row_block_rows(tiles_per_wg: int) -> int:
    """Rows of a row block (one workgroup's rows) for a tiles_per_wg code: 128, + 1000: 64, + 2000: 32."""
    return (128, 64, 32)[tiles_per_wg // 1000]


def tiled_slice_width(M: int, tiles_per_wg: int) -> int:
    """K slice of x a workgroup of linear_tiled stages at a time."""
    M = min(M, row_block_rows(tiles_per_wg))
    tiles_per_wg %= 1000
    mt = 1 if M <= 16 else 2 if M <= 32 else 4 if M <= 64 else 8
    narrow = tiles_per_wg in (104, 108, 208, 402, 404)      # 210 .. 216 (two tiles per wave, 5 .. 8 waves) stage the wide slice
    return (512 if narrow else 1024) // (1 if mt <= 2 else mt // 2)


def tiles_per_workgroup(tiles_per_wg: int) -> int:
    """Weight tiles one workgroup covers for a tiles_per_wg code (208 .. 216: two tiles per wave;
    30x / 40x: 8 waves, x waves per tile; + 1000 / + 2000: the same in row blocks of 64 / 32)."""
    tiles_per_wg %= 1000
    if tiles_per_wg in KW_CODES:
        return 8 // (tiles_per_wg % 100)
    return tiles_per_wg % 100


def plan_linear_tiled(N: int, K: int, split_k: bool, M: int = 32):
    """(tiles_per_wg, k_groups) for linear_tiled on an [N, K] weight and M rows, or None when
    the kernel does not cover the shape.  One workgroup per CU (>= ~192 workgroups) is what
    saturates the weight stream: wide layers take 8 tiles per workgroup, unsplit; narrower
    ones take 4 tiles and the narrow x slice (two workgroups per CU; 8 tiles beyond 64 rows)
    and, when the caller can consume or reduce fp32 partial sums, split K over workgroups
    until there are enough of them."""
    if M > LINEAR_TILED_MAX_M:
        return None
    tiles_total = (N + 15) // 16
    if M > 64:
        candidates = [8]
    elif tiles_total >= 8 * 160:
        candidates = [8, 104]
    else:
        candidates = [104]
    for tiles in candidates:
        ksl = tiled_slice_width(M, tiles)
        if K % ksl:
            continue
        units = K // ksl
        wgs = -(-tiles_total // (tiles % 100)) * (-(-M // 128))          # beyond 128 rows: two row blocks
        groups = 1
        if split_k and wgs < 160:
            # at most 8 slabs: the consumers (attention, norm) sum up to 8 with straight-line loads
            groups = max(1, min(-(-192 // wgs), units, 8))
            # an even deal of the slices if one is near; otherwise K just does not divide evenly
            for g in range(groups, min(2 * groups, units, 8) + 1):
                if units % g == 0:
                    groups = g
                    break
        return tiles, groups
    return None


def linear_tiled_candidates(N: int, K: int, split_k: bool, M: int = 32, swiglu: bool = False):
    """Every (tiles_per_wg, k_groups) worth timing for linear_tiled on an [N, K] weight and M rows:
    both workgroup shapes that every kernel form (fp8, fused epilogues) is built for, K split into
    1, 2, 4 or 8 groups when the caller can take partial sums, beyond 32 rows also the forms with
    two tiles per wave (208 .. 216: 4 .. 8 waves, so that a tile count that 16 per workgroup would
    spread over too few CUs finds a better deal), kept if the launch has between 64 and 1024 workgroups; up to 32
    rows and few tiles also the forms that split K across the waves of a workgroup (`swiglu`: the
    gate / up pair must share a workgroup, at most 4 waves per tile); beyond 64 / 32 rows also the forms of
    the 64- / 32-row class run in row blocks of 64 / 32 (tiles_per_wg + 1000 / + 2000).  Not
    every form exists for every code (fp8 at up to 32 rows: 8 and 104 only): the caller skips a
    candidate the library refuses.  plan_linear_tiled's choice comes first."""
    first = plan_linear_tiled(N, K, split_k, M)
    if first is None:
        return []
    out = [first]
    tiles_total = (N + 15) // 16
    row_blocks = -(-M // 128)
    for tiles in ((8, 104, 108) if M <= 32 else (8, 104, 108, 208, 216, 210, 212, 214) if M <= 64
                  else (8, 216, 210, 212, 214)):
        ksl = tiled_slice_width(M, tiles)
        if K % ksl:
            continue
        wgs = -(-tiles_total // tiles_per_workgroup(tiles)) * row_blocks
        for g in ((1, 2, 4, 8) if split_k else (1,)):
            if g <= K // ksl and 64 <= wgs * g <= 1024 and (tiles, g) not in out:
                out.append((tiles, g))
    # beyond 64 / 32 rows: the forms of the 64- / 32-row class in row blocks of 64 / 32 rows (tiles_per_wg + 1000 / + 2000)
    for rb_code, rb, forms in ((1000, 64, (8, 104, 108, 208, 216, 210, 212, 214, 302, 304, 402)),
                               (2000, 32, (8, 104, 108, 302, 304, 402))):
        if M <= rb or os.environ.get("MI355_ROW_BLOCKS", "1") == "0":      # (the switch: for A/B timing)
            continue
        blocks = -(-M // rb)
        for tiles in forms:
            code = rb_code + tiles
            ksl = tiled_slice_width(M, code)
            if K % ksl or (tiles in KW_CODES and ((swiglu and tiles % 100 > 4) or (tiles % 100) * 128 > ksl)):
                continue
            wgs = -(-tiles_total // tiles_per_workgroup(code)) * blocks
            for g in ((1, 2, 4, 8) if split_k else (1,)):
                if g <= K // ksl and 96 <= wgs * g <= 1024 and (code, g) not in out:
                    out.append((code, g))
    if tiles_total < 8 * 160:
        # few tiles (a tensor-parallel rank's slice): K split across the waves of a workgroup, the
        # only way to more waves when the output must be 16-bit or gated (no slabs)
        for tiles in KW_CODES:
            ksl = tiled_slice_width(M, tiles)
            if K % ksl or (swiglu and tiles % 100 > 4) or (tiles % 100) * 128 > ksl:   # a wave needs a register group of the slice
                continue
            wgs = -(-tiles_total // tiles_per_workgroup(tiles)) * row_blocks
            for g in ((1, 2, 4, 8) if split_k else (1,)):
                if g <= K // ksl and 48 <= wgs * g <= 1024 and (tiles, g) not in out:
                    out.append((tiles, g))
    return out


def tile_weights(weight: torch.Tensor, interleave_halves: bool = False) -> torch.Tensor:
    """Row-major [N, K] -> fragment-tiled flat tensor for linear_tiled (done once at load)."""
    _dt16(weight, "weight")
    if weight.dim() != 2 or not weight.is_contiguous():
        raise ValueError("weight must be contiguous [N, K]")
    N, K = weight.shape
    n = int(lib.mi355_tiled_weight_elems(N, K))
    if n == 0:
        raise ValueError(f"K {K} must be a multiple of 128")
    out = torch.empty(n, dtype=weight.dtype, device=weight.device)
    check(lib.mi355_tile_weights(out.data_ptr(), weight.data_ptr(), N, K, int(bool(interleave_halves)), _stream()))
    return out


def untile_weights(w_tiled, N: int, K: int, dtype: torch.dtype, interleave_halves: bool = False,
                   out: torch.Tensor | None = None) -> torch.Tensor:
    """Row-major [N, K] matrix from a tiled weight: a 16-bit tensor of tile_weights (the same bits
    back), or the (fp8 bytes, row scales) pair of tile_weights_fp8 (decoded: round(fp8 * scale))."""
    fp8 = isinstance(w_tiled, tuple)
    src = w_tiled[0] if fp8 else w_tiled
    _dev(src, "w_tiled")
    if dtype not in _DT:
        raise TypeError(f"dtype {dtype} not supported")
    want = int(lib.mi355_tiled_weight_fp8_bytes(N, K)) if fp8 else int(lib.mi355_tiled_weight_elems(N, K))
    if want == 0 or src.numel() != want or (not fp8 and src.dtype != dtype) or (fp8 and src.dtype != torch.uint8):
        raise ValueError("w_tiled does not match (N, K) / dtype")
    if out is None:
        out = torch.empty((N, K), dtype=dtype, device=src.device)
    elif out.dtype != dtype or tuple(out.shape) != (N, K) or not out.is_contiguous():
        raise ValueError("out must be contiguous [N, K] in the model dtype")
    if fp8:
        check(lib.mi355_untile_weights_fp8(out.data_ptr(), src.data_ptr(), w_tiled[1].data_ptr(), N, K,
                                           int(bool(interleave_halves)), _DT[dtype], _stream()))
    else:
        check(lib.mi355_untile_weights(out.data_ptr(), src.data_ptr(), N, K, int(bool(interleave_halves)), _stream()))
    return out


def linear_tiled(x: torch.Tensor, w_tiled: torch.Tensor, N: int, bias: torch.Tensor | None = None,
                 out: torch.Tensor | None = None, partial: torch.Tensor | None = None, tiles_per_wg: int = 0,
                 k_groups: int = 1, epilogue: int = EPI_STORE):
    """y = x @ W.T on fragment-tiled weights (M <= 256).  Returns `out`
    ([M, N], or [M, N/2] with the SwiGLU epilogue) or `partial` ([k_groups, M, N] fp32)."""
    dt = _dt16(x, "x")
    _dev(w_tiled, "w_tiled")
    M, K = x.shape
    if w_tiled.dtype != x.dtype or w_tiled.numel() != int(lib.mi355_tiled_weight_elems(N, K)):
        raise ValueError("w_tiled does not match (N, K) / dtype")
    tiles_total = (N + 15) // 16
    if tiles_per_wg == 0:                         # 8 tiles (waves) per workgroup once that still fills the chip
        tiles_per_wg = 8 if M > 64 or -(-tiles_total // 8) * k_groups >= 160 else (4 if M <= 32 else 104)
    y_ptr = p_ptr = 0
    y_stride = 0
    if epilogue == EPI_PARTIAL:
        if partial is None:
            partial = torch.empty((k_groups, M, N), dtype=torch.float32, device=x.device)
        elif partial.dtype != torch.float32 or partial.numel() < k_groups * M * N or not partial.is_contiguous():
            raise ValueError("partial must be contiguous float32 [k_groups, M, N]")
        p_ptr = partial.data_ptr()
        ret = partial
    else:
        width = N // 2 if epilogue == EPI_SILU_MUL else N
        if out is None:
            out = torch.empty((M, width), dtype=x.dtype, device=x.device)
        elif out.dtype != x.dtype or tuple(out.shape) != (M, width):
            raise ValueError(f"out must be [M, {width}] in the dtype of x")
        y_ptr, y_stride, ret = out.data_ptr(), _rows(out, "out"), out
    if bias is not None and (bias.dtype != x.dtype or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous [N] in the dtype of x")
    check(lib.mi355_linear_tiled(y_ptr, y_stride, p_ptr, x.data_ptr(), _rows(x, "x"), w_tiled.data_ptr(),
                                 bias.data_ptr() if bias is not None else 0, M, N, K, tiles_per_wg, k_groups,
                                 epilogue, dt, _stream()))
    return ret


def linear_tiled_fused(x: torch.Tensor, w_tiled: torch.Tensor, N: int, *, tiles_per_wg: int, k_groups: int = 1,
                       epilogue: int = EPI_STORE, bias: torch.Tensor | None = None, out: torch.Tensor | None = None,
                       partial: torch.Tensor | None = None, norm_weight: torch.Tensor | None = None,
                       norm_sumsq: torch.Tensor | None = None, norm_parts: int = 0, eps: float = 0.0,
                       residual: torch.Tensor | None = None, sumsq_out: torch.Tensor | None = None,
                       counters: torch.Tensor | None = None):
    """linear_tiled with the RMSNorm before it (norm_weight + norm_sumsq: x is the residual
    stream, normalised while it is staged) and/or the K-split reduction, residual add and
    sum of squares after it (epilogues EPI_REDUCE_STORE / EPI_REDUCE_RESID) in the same launch."""
    dt = _dt16(x, "x")
    _dev(w_tiled, "w_tiled")
    M, K = x.shape
    if w_tiled.dtype != x.dtype or w_tiled.numel() != int(lib.mi355_tiled_weight_elems(N, K)):
        raise ValueError("w_tiled does not match (N, K) / dtype")
    nw = tiles_per_wg % 100
    groups = -(-((N + 15) // 16) // max(nw, 1))
    y_ptr, y_stride = 0, 0
    if epilogue in (EPI_STORE, EPI_SILU_MUL, EPI_REDUCE_STORE):
        width = N // 2 if epilogue == EPI_SILU_MUL else N
        if out is None:
            out = torch.empty((M, width), dtype=x.dtype, device=x.device)
        elif out.dtype != x.dtype or tuple(out.shape) != (M, width):
            raise ValueError(f"out must be [M, {width}] in the dtype of x")
        y_ptr, y_stride = out.data_ptr(), _rows(out, "out")
    if epilogue in (EPI_PARTIAL, EPI_REDUCE_STORE, EPI_REDUCE_RESID):
        if partial is None:
            partial = torch.empty((k_groups, M, N), dtype=torch.float32, device=x.device)
        _check_partial(partial, k_groups, M, N)
    if epilogue in (EPI_REDUCE_STORE, EPI_REDUCE_RESID):
        if counters is None or counters.dtype != torch.int32 or counters.numel() < groups or not counters.is_cuda:
            raise ValueError(f"counters must be a zero-initialised int32 device tensor with >= {groups} elements")
    if epilogue == EPI_REDUCE_RESID:
        if residual is None or residual.dtype != x.dtype or tuple(residual.shape) != (M, N):
            raise ValueError("residual must be [M, N] in the dtype of x")
        if (sumsq_out is None or sumsq_out.dtype != torch.float32 or sumsq_out.numel() < groups * SUMSQ_ROWS
                or not sumsq_out.is_contiguous()):
            raise ValueError(f"sumsq_out must be contiguous float32 with >= {groups} x {SUMSQ_ROWS} elements")
    if norm_weight is not None:
        if norm_weight.dtype != x.dtype or norm_weight.numel() != K or not norm_weight.is_contiguous():
            raise ValueError("norm_weight must be contiguous [K] in the dtype of x")
        if (norm_sumsq is None or norm_sumsq.dtype != torch.float32 or norm_parts < 1
                or norm_sumsq.numel() < norm_parts * SUMSQ_ROWS or not norm_sumsq.is_contiguous()):
            raise ValueError("norm_sumsq must be contiguous float32 [norm_parts, 32]")
    if bias is not None and (bias.dtype != x.dtype or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous [N] in the dtype of x")
    ptr = lambda t: t.data_ptr() if t is not None else 0  # noqa: E731
    check(lib.mi355_linear_tiled_fused(
        y_ptr, y_stride, ptr(partial), x.data_ptr(), _rows(x, "x"), w_tiled.data_ptr(), ptr(bias), M, N, K,
        tiles_per_wg, k_groups, epilogue, ptr(norm_weight), ptr(norm_sumsq), norm_parts, float(eps), ptr(residual),
        _rows(residual, "residual") if residual is not None else 0, ptr(sumsq_out), ptr(counters), dt, _stream()))
    if epilogue == EPI_PARTIAL:
        return partial
    if epilogue == EPI_REDUCE_RESID:
        return residual
    return out


def tile_weights_fp8(weight: torch.Tensor, interleave_halves: bool = False):
    """Row-major 16-bit [N, K] -> (fp8 e4m3fn fragment-tiled bytes, fp32 row scales in tiled row order)."""
    dt = _dt16(weight, "weight")
    if weight.dim() != 2 or not weight.is_contiguous():
        raise ValueError("weight must be contiguous [N, K]")
    N, K = weight.shape
    n = int(lib.mi355_tiled_weight_fp8_bytes(N, K))
    if n == 0:
        raise ValueError(f"K {K} must be a multiple of 128")
    q = torch.empty(n, dtype=torch.uint8, device=weight.device)
    scale = torch.empty((N + 15) // 16 * 16, dtype=torch.float32, device=weight.device)
    check(lib.mi355_tile_weights_fp8(q.data_ptr(), scale.data_ptr(), weight.data_ptr(), N, K,
                                     int(bool(interleave_halves)), dt, _stream()))
    return q, scale


def linear_tiled_w8(x: torch.Tensor, w_fp8: torch.Tensor, w_scale: torch.Tensor, N: int,
                    bias: torch.Tensor | None = None, out: torch.Tensor | None = None,
                    partial: torch.Tensor | None = None, tiles_per_wg: int = 0, k_groups: int = 1,
                    epilogue: int = EPI_STORE):
    """linear_tiled on fp8 weights from tile_weights_fp8 (x stays 16-bit; M <= 128)."""
    dt = _dt16(x, "x")
    _dev(w_fp8, "w_fp8"), _dev(w_scale, "w_scale")
    M, K = x.shape
    if w_fp8.dtype != torch.uint8 or w_fp8.numel() != int(lib.mi355_tiled_weight_fp8_bytes(N, K)):
        raise ValueError("w_fp8 does not match (N, K)")
    if w_scale.dtype != torch.float32 or w_scale.numel() != (N + 15) // 16 * 16 or not w_scale.is_contiguous():
        raise ValueError("w_scale must be contiguous float32 [ceil(N/16)*16]")
    if tiles_per_wg == 0:
        tiles_per_wg = 8 if M > 64 or -(-((N + 15) // 16) // 8) * k_groups >= 160 else 104
    y_ptr = p_ptr = y_stride = 0
    if epilogue == EPI_PARTIAL:
        if partial is None:
            partial = torch.empty((k_groups, M, N), dtype=torch.float32, device=x.device)
        _check_partial(partial, k_groups, M, N)
        p_ptr, ret = partial.data_ptr(), partial
    else:
        width = N // 2 if epilogue == EPI_SILU_MUL else N
        if out is None:
            out = torch.empty((M, width), dtype=x.dtype, device=x.device)
        elif out.dtype != x.dtype or tuple(out.shape) != (M, width):
            raise ValueError(f"out must be [M, {width}] in the dtype of x")
        y_ptr, y_stride, ret = out.data_ptr(), _rows(out, "out"), out
    if bias is not None and (bias.dtype != x.dtype or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous [N] in the dtype of x")
    check(lib.mi355_linear_tiled_w8(y_ptr, y_stride, p_ptr, x.data_ptr(), _rows(x, "x"), w_fp8.data_ptr(),
                                    w_scale.data_ptr(), bias.data_ptr() if bias is not None else 0, M, N, K,
                                    tiles_per_wg, k_groups, epilogue, dt, _stream()))
    return ret


def quant_rows_fp8(x: torch.Tensor, out: torch.Tensor | None = None, scale: torch.Tensor | None = None):
    """16-bit rows [M, K] -> (e4m3fn rows as uint8 [M, K], one fp32 scale per row): the activation
    input of linear_tiled_w8a8."""
    dt = _dt16(x, "x")
    M, K = x.shape
    if out is None:
        out = torch.empty((M, K), dtype=torch.uint8, device=x.device)
    elif out.dtype != torch.uint8 or tuple(out.shape) != (M, K):
        raise ValueError("out must be uint8 [M, K]")
    if scale is None:
        scale = torch.empty(M, dtype=torch.float32, device=x.device)
    elif scale.dtype != torch.float32 or scale.numel() != M or not scale.is_contiguous():
        raise ValueError("scale must be contiguous float32 [M]")
    check(lib.mi355_quant_rows_fp8(out.data_ptr(), _rows(out, "out"), scale.data_ptr(), x.data_ptr(), _rows(x, "x"),
                                   M, K, dt, _stream()))
    return out, scale


def linear_tiled_w8a8(xq: torch.Tensor, x_scale: torch.Tensor, w_fp8: torch.Tensor, w_scale: torch.Tensor, N: int,
                      dtype: torch.dtype = torch.bfloat16, bias: torch.Tensor | None = None,
                      out: torch.Tensor | None = None, partial: torch.Tensor | None = None, tiles_per_wg: int = 0,
                      k_groups: int = 1, epilogue: int = EPI_STORE):
    """fp8 activations (quant_rows_fp8) x fp8 weights (tile_weights_fp8) on the fp8 matrix instruction;
    `dtype`: the 16-bit type of the output and the bias.  M <= 128."""
    _dev(xq, "xq"), _dev(x_scale, "x_scale"), _dev(w_fp8, "w_fp8"), _dev(w_scale, "w_scale")
    if xq.dtype != torch.uint8 or xq.dim() != 2:
        raise ValueError("xq must be uint8 [M, K]")
    M, K = xq.shape
    dt = _DT.get(dtype)
    if dt is None:
        raise ValueError("dtype must be bfloat16 or float16")
    if x_scale.dtype != torch.float32 or x_scale.numel() != M or not x_scale.is_contiguous():
        raise ValueError("x_scale must be contiguous float32 [M]")
    if w_fp8.dtype != torch.uint8 or w_fp8.numel() != int(lib.mi355_tiled_weight_fp8_bytes(N, K)):
        raise ValueError("w_fp8 does not match (N, K)")
    if w_scale.dtype != torch.float32 or w_scale.numel() != (N + 15) // 16 * 16 or not w_scale.is_contiguous():
        raise ValueError("w_scale must be contiguous float32 [ceil(N/16)*16]")
    if tiles_per_wg == 0:
        tiles_per_wg = 216 if M <= 32 or -(-((N + 15) // 16) // 16) * k_groups >= 200 else 210
    y_ptr = p_ptr = y_stride = 0
    if epilogue == EPI_PARTIAL:
        if partial is None:
            partial = torch.empty((k_groups, M, N), dtype=torch.float32, device=xq.device)
        _check_partial(partial, k_groups, M, N)
        p_ptr, ret = partial.data_ptr(), partial
    else:
        width = N // 2 if epilogue == EPI_SILU_MUL else N
        if out is None:
            out = torch.empty((M, width), dtype=dtype, device=xq.device)
        elif out.dtype != dtype or tuple(out.shape) != (M, width):
            raise ValueError(f"out must be [M, {width}] in `dtype`")
        y_ptr, y_stride, ret = out.data_ptr(), _rows(out, "out"), out
    if bias is not None and (bias.dtype != dtype or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous [N] in `dtype`")
    check(lib.mi355_linear_tiled_w8a8(y_ptr, y_stride, p_ptr, xq.data_ptr(), _rows(xq, "xq"), x_scale.data_ptr(),
                                      w_fp8.data_ptr(), w_scale.data_ptr(), bias.data_ptr() if bias is not None else 0,
                                      M, N, K, tiles_per_wg, k_groups, epilogue, dt, _stream()))
    return ret


# ---------------------------------------------------------------------------------------------- #
# decoders with an fp32 residual stream; sequence mixers over packed chunks (csrc/resid32.hip,
# csrc/seqmix.hip).  Activations and weights are bf16, fp16 or fp32; the residual, recurrent
# state and the small per-head parameters are fp32 tensors.
# ---------------------------------------------------------------------------------------------- #
def _dt3(t: torch.Tensor, name: str) -> int:
    _dev(t, name)
    if t.dtype not in _DT:
        raise TypeError(f"{name}: dtype {t.dtype} not supported (bfloat16/float16/float32)")
    return _DT[t.dtype]


def _f32(t: torch.Tensor, name: str, numel: int | None = None) -> int:
    _dev(t, name)
    if t.dtype != torch.float32 or not t.is_contiguous() or (numel is not None and t.numel() != numel):
        raise ValueError(f"{name} must be a contiguous float32 tensor" + (f" of {numel} elements" if numel else ""))
    return t.data_ptr()


def _idx(t: torch.Tensor, name: str, dtype: torch.dtype, numel: int | None = None) -> int:
    _dev(t, name)
    if t.dtype != dtype or not t.is_contiguous() or (numel is not None and t.numel() < numel):
        raise ValueError(f"{name} must be a contiguous {dtype} tensor" + (f" of >= {numel} elements" if numel else ""))
    return t.data_ptr()


def _same(t: torch.Tensor, ref: torch.Tensor, name: str) -> int:
    _dev(t, name)
    if t.dtype != ref.dtype:
        raise TypeError(f"{name}: dtype {t.dtype}, expected {ref.dtype}")
    return t.data_ptr()


def embed_scale_f32(embed: torch.Tensor, ids: torch.Tensor, scale: float, out: torch.Tensor | None = None):
    """out[t] = embed[ids[t]] * scale as float32 rows."""
    dt = _dt3(embed, "embed")
    if embed.dim() != 2 or not embed.is_contiguous():
        raise ValueError("embed must be contiguous [vocab, width]")
    T, W = ids.numel(), embed.shape[1]
    if out is None:
        out = torch.empty(T, W, dtype=torch.float32, device=embed.device)
    check(lib.mi355_embed_scale_f32(_f32(out, "out", T * W), embed.data_ptr(), _idx(ids, "ids", torch.int64), T, W,
                                    embed.shape[0], float(scale), dt, _stream()))
    return out


def embed_scale_pos_f32(embed: torch.Tensor, ids: torch.Tensor, scale: float, pos_table: torch.Tensor,
                        positions: torch.Tensor):
    """float32 rows embed[ids[t]] * scale + pos_table[positions[t]] (learned positions, unscaled)."""
    dt = _dt3(embed, "embed")
    if embed.dim() != 2 or not embed.is_contiguous():
        raise ValueError("embed must be contiguous [vocab, width]")
    T, W = ids.numel(), embed.shape[1]
    if pos_table.dtype != embed.dtype or pos_table.dim() != 2 or pos_table.shape[1] != W or not pos_table.is_contiguous():
        raise ValueError("pos_table must be contiguous [positions, width] in the dtype of embed")
    out = torch.empty(T, W, dtype=torch.float32, device=embed.device)
    check(lib.mi355_embed_scale_pos_f32(out.data_ptr(), embed.data_ptr(), pos_table.data_ptr(), _idx(ids, "ids", torch.int64),
                                        _idx(positions, "positions", torch.int64, T), T, W, embed.shape[0],
                                        pos_table.shape[0], float(scale), dt, _stream()))
    return out


def resid_add_f32(resid: torch.Tensor, other: torch.Tensor | None = None, rows: torch.Tensor | None = None,
                  vec: torch.Tensor | None = None):
    """resid (float32, in place) += other (float32 rows) + rows (activation rows) + vec (one row)."""
    T, W = resid.shape
    dt = None
    if T == 0:
        return resid
    for name, t, shape in (("rows", rows, (T, W)), ("vec", vec, (W,))):
        if t is None:
            continue
        if (dt is not None and _DT[t.dtype] != dt) or t.numel() != T * W // (T if name == "vec" else 1) \
                or not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous {shape}, rows and vec in one dtype")
        dt = _dt3(t, name)
    check(lib.mi355_resid_add_f32(_f32(resid, "resid"), None if other is None else _f32(other, "other", T * W),
                                  None if rows is None else rows.data_ptr(), None if vec is None else vec.data_ptr(),
                                  T, W, _DT[torch.float32] if dt is None else dt, _stream()))
    return resid


def add_rms_norm_f32(resid: torch.Tensor, weight: torch.Tensor, eps: float, add: torch.Tensor | None = None,
                     out: torch.Tensor | None = None):
    """resid (float32, in place) += add; returns resid / rms(resid) * weight in the dtype of weight.
    weight: one number (numel 1) or one per column."""
    T, W = resid.shape
    dt = _dt3(weight, "weight")
    if weight.numel() not in (1, W) or not weight.is_contiguous():
        raise ValueError("weight must be one number or one contiguous row")
    if out is None:
        out = torch.empty(T, W, dtype=weight.dtype, device=resid.device)
    if out.dtype != weight.dtype or not out.is_contiguous() or out.shape != resid.shape:
        raise ValueError("out must be contiguous, shaped like resid, in the dtype of weight")
    if add is not None and (add.dtype != weight.dtype or not add.is_contiguous() or add.shape != resid.shape):
        raise ValueError("add must be contiguous, shaped like resid, in the dtype of weight")
    check(lib.mi355_add_rms_norm_f32(out.data_ptr(), _f32(resid, "resid"), None if add is None else add.data_ptr(),
                                     weight.data_ptr(), weight.numel(), T, W, float(eps), dt, _stream()))
    return out


def rms_norm_mix_f32(resid: torch.Tensor, xa: torch.Tensor, wa: torch.Tensor, xb: torch.Tensor | None,
                     wb: torch.Tensor | None, eps: float, alpha: float):
    """resid (float32, in place) += alpha * (rmsnorm(xa) * wa + rmsnorm(xb) * wb)."""
    T, W = resid.shape
    dt = _dt3(xa, "xa")
    for n, t, shape in (("xa", xa, (T, W)), ("wa", wa, (W,)), ("xb", xb, (T, W)), ("wb", wb, (W,))):
        if t is None:
            continue
        if t.dtype != xa.dtype or not t.is_contiguous() or tuple(t.shape) != shape:
            raise ValueError(f"{n} must be contiguous {shape} in the dtype of xa")
    check(lib.mi355_rms_norm_mix_f32(_f32(resid, "resid"), xa.data_ptr(), wa.data_ptr(),
                                     None if xb is None else xb.data_ptr(), None if wb is None else wb.data_ptr(),
                                     T, W, float(eps), float(alpha), dt, _stream()))
    return resid


def gelu_tanh_and_mul(x: torch.Tensor, out: torch.Tensor | None = None):
    """x [tokens, 2 * inter] holding gate | up -> gelu_tanh(gate) * up."""
    dt = _dt3(x, "x")
    inter = x.shape[1] // 2
    if out is None:
        out = torch.empty(x.shape[0], inter, dtype=x.dtype, device=x.device)
    check(lib.mi355_gelu_tanh_and_mul(out.data_ptr(), x.data_ptr(), _rows(x, "x"), x.shape[0], inter, dt, _stream()))
    return out


ACT_SILU, ACT_SIGMOID = 0, 1


def gated_head_rms_norm(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float, activation: int,
                        out: torch.Tensor | None = None):
    """o float32 [tokens, heads, dim]; gate [tokens, >= heads * dim] (a column slice is fine);
    weight float32 [dim] (shared by the heads) or [heads * dim].  Returns o / rms(o) * weight * act(gate)
    as [tokens, heads * dim] in gate's dtype."""
    T, H, D = o.shape
    wh = H if weight.numel() == H * D and H > 1 else 1
    dt = _dt3(gate, "gate")
    if gate.dim() != 2 or gate.shape[1] != H * D or gate.stride(1) != 1:
        raise ValueError("gate must be [tokens, heads * dim] with a contiguous last dim")
    if out is None:
        out = torch.empty(T, H * D, dtype=gate.dtype, device=o.device)
    check(lib.mi355_gated_head_rms_norm(out.data_ptr(), _f32(o, "o"), gate.data_ptr(), gate.stride(0) if T > 1 else H * D,
                                        _f32(weight, "weight", wh * D), wh, T, H, D, float(eps), int(activation), dt,
                                        _stream()))
    return out


def softcap(z: torch.Tensor, cap: float):
    """z <- cap * tanh(z / cap), in place."""
    dt = _dt3(z, "z")
    if not z.is_contiguous():
        raise ValueError("z must be contiguous")
    check(lib.mi355_softcap(z.data_ptr(), z.numel(), float(cap), dt, _stream()))
    return z


def _cols(t: torch.Tensor, name: str, width: int) -> int:
    """Row stride of a [rows, width] column slice."""
    if t.dim() != 2 or t.shape[1] != width or t.stride(1) != 1:
        raise ValueError(f"{name} must be [rows, {width}] with a contiguous last dim (shape {tuple(t.shape)})")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), width)


def rope_partial_kv_write(q: torch.Tensor, k: torch.Tensor | None, v: torch.Tensor | None, cos_sin: torch.Tensor,
                          positions: torch.Tensor, slot_mapping: torch.Tensor, k_cache: torch.Tensor | None,
                          v_cache: torch.Tensor | None, num_heads: int, num_kv_heads: int, head_dim: int, v_dim: int):
    """Rotates q in place and k into its page by the float32 table cos_sin [max_pos, rot_dims]; copies v
    into its page.  q / k / v may be column slices of one projection output.  k, v and the caches None:
    only q is rotated (a layer that attends to another layer's pages)."""
    dt = _dt3(q, "q")
    T = q.shape[0]
    rot = cos_sin.shape[1]
    if k is None:
        if v is not None or k_cache is not None or v_cache is not None:
            raise ValueError("k, v and both caches go together")
        check(lib.mi355_rope_partial_kv_write(
            q.data_ptr(), _cols(q, "q", num_heads * head_dim), None, 0, None, 0, _f32(cos_sin, "cos_sin") or q.data_ptr(),
            max(cos_sin.shape[0], 1), _idx(positions, "positions", torch.int64, T),
            _idx(slot_mapping, "slot_mapping", torch.int64, T), None, None, T, num_heads, num_kv_heads, head_dim, v_dim,
            rot, dt, _stream()))
        return
    if tuple(k_cache.shape[1:]) != (num_kv_heads, BLOCK_SIZE, head_dim) or tuple(v_cache.shape[1:]) != (num_kv_heads, v_dim, BLOCK_SIZE) \
            or k_cache.shape[0] != v_cache.shape[0] or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise ValueError("K pages must be [blocks, kv_heads, 16, head_dim] and V pages [blocks, kv_heads, v_dim, 16]")
    check(lib.mi355_rope_partial_kv_write(
        q.data_ptr(), _cols(q, "q", num_heads * head_dim), _same(k, q, "k"), _cols(k, "k", num_kv_heads * head_dim),
        _same(v, q, "v"), _cols(v, "v", num_kv_heads * v_dim),
        _f32(cos_sin, "cos_sin") or q.data_ptr(),            # rot_dims 0: the table is empty and never read
        max(cos_sin.shape[0], 1),
        _idx(positions, "positions", torch.int64, T), _idx(slot_mapping, "slot_mapping", torch.int64, T),
        _same(k_cache, q, "k_cache"), _same(v_cache, q, "v_cache"), T, num_heads, num_kv_heads, head_dim, v_dim, rot,
        dt, _stream()))


def sigmoid_window_attn(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                        tok_seq: torch.Tensor, positions: torch.Tensor, temp: torch.Tensor, bias: torch.Tensor,
                        gate: torch.Tensor | None, num_heads: int, window: int, scale: float,
                        out: torch.Tensor | None = None, tiles: torch.Tensor | None = None,
                        partial: torch.Tensor | None = None, num_splits: int = 1):
    """Sliding-window attention with sigmoid weights over the paged K/V of each packed row's
    sequence.  Returns [tokens, heads * v_dim].  `tiles` (int32 [n, 3], see query_tiles) selects the
    matrix-core form where the shapes allow it; there `partial` (float32, >= num_splits * tokens *
    heads * v_dim elements) with num_splits > 1 spreads each tile's keys over num_splits workgroups."""
    dt = _dt3(q, "q")
    T = q.shape[0]
    G, d, dv = k_cache.shape[1], k_cache.shape[3], v_cache.shape[2]
    if tiles is not None and (tiles.dtype != torch.int32 or tiles.dim() != 2 or tiles.shape[1] != 3
                              or not tiles.is_contiguous() or not tiles.is_cuda):
        raise ValueError("tiles must be a contiguous int32 [n, 3] tensor on the GPU")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be contiguous int32 [chunks, max_blocks]")
    if out is None:
        out = torch.empty(T, num_heads * dv, dtype=q.dtype, device=q.device)
    check(lib.mi355_sigmoid_window_attn(
        out.data_ptr(), q.data_ptr(), _cols(q, "q", num_heads * d), _same(k_cache, q, "k_cache"),
        _same(v_cache, q, "v_cache"), block_tables.data_ptr(), block_tables.shape[1],
        _idx(tok_seq, "tok_seq", torch.int32, T), _idx(positions, "positions", torch.int64, T),
        _f32(temp, "temp", num_heads), _f32(bias, "bias", num_heads),
        None if gate is None else _same(gate, q, "gate"), 0 if gate is None else _cols(gate, "gate", num_heads),
        T, num_heads, G, d, dv, int(window), float(scale), None if tiles is None else tiles.data_ptr(),
        0 if tiles is None else tiles.shape[0],
        None if partial is None or num_splits <= 1 else _f32(partial[: num_splits * T * num_heads * dv], "partial",
                                                             num_splits * T * num_heads * dv),
        int(num_splits), dt, _stream()))
    return out


def query_tiles(cu_seqlens) -> "np.ndarray":
    """(chunk, first packed row, rows <= 16) for every 16-row tile of a packed batch, from the host
    copy of cu_seqlens: the work list of the matrix-core window attention."""
    import numpy as np
    cu = np.asarray(cu_seqlens, dtype=np.int64)
    out = []
    for s in range(len(cu) - 1):
        for a in range(int(cu[s]), int(cu[s + 1]), 16):
            out.append((s, a, min(16, int(cu[s + 1]) - a)))
    return np.asarray(out, dtype=np.int32).reshape(-1, 3)


def causal_conv_silu(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, tok_seq: torch.Tensor,
                     positions: torch.Tensor, cu_seqlens: torch.Tensor, state_slots: torch.Tensor,
                     out: torch.Tensor | None = None):
    """Depthwise causal convolution + SiLU over packed chunks, then the state update: state
    [slots, taps - 1, channels] float32 holds each sequence's last taps - 1 inputs."""
    dt = _dt3(x, "x")
    T, C = x.shape
    taps = weight.shape[1]
    if tuple(weight.shape) != (C, taps) or weight.dtype != x.dtype or not weight.is_contiguous():
        raise ValueError("weight must be contiguous [channels, taps] in the dtype of x")
    if state.dim() != 3 or tuple(state.shape[1:]) != (max(taps - 1, 0), C):
        raise ValueError("state must be [slots, taps - 1, channels]")
    S = cu_seqlens.numel() - 1
    if out is None:
        out = torch.empty(T, C, dtype=x.dtype, device=x.device)
    args = (_idx(cu_seqlens, "cu_seqlens", torch.int32), _idx(state_slots, "state_slots", torch.int32, S))
    st = _f32(state, "state") or x.data_ptr()                # one tap: the state is empty and never read
    check(lib.mi355_causal_conv_silu(out.data_ptr(), x.data_ptr(), _cols(x, "x", C), weight.data_ptr(),
                                     st, _idx(tok_seq, "tok_seq", torch.int32, T),
                                     _idx(positions, "positions", torch.int64, T), *args, T, C, taps, dt, _stream()))
    check(lib.mi355_conv_state_update(st, x.data_ptr(), _cols(x, "x", C), *args, S, C, taps, dt,
                                      _stream()))
    return out


def gated_delta_rule(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, beta: torch.Tensor, decay: torch.Tensor,
                     a_log: torch.Tensor, dt_bias: torch.Tensor, state: torch.Tensor, cu_seqlens: torch.Tensor,
                     positions: torch.Tensor, state_slots: torch.Tensor, num_heads: int, num_kv_heads: int,
                     head_dim: int, v_dim: int, per_channel: bool = False, out: torch.Tensor | None = None,
                     long_chunks: bool = False):
    """The gated delta rule over packed chunks.  qkv [tokens, C] holds q (kv_heads x head_dim) at column
    q_off, k at k_off, v (heads x v_dim) at v_off; beta [tokens, heads] and decay [tokens, heads] or
    [tokens, heads * head_dim] are raw projection outputs (column slices are fine); a_log [heads] and
    dt_bias (decay's width) float32; state float32 [slots, heads, head_dim, v_dim].
    Returns o float32 [tokens, heads, v_dim].  long_chunks: the batch holds chunks of many tokens -- take
    the form that splits the state rows over lanes (it allocates a float32 workspace; not for graphs)."""
    dt = _dt3(qkv, "qkv")
    T = qkv.shape[0]
    S = cu_seqlens.numel() - 1
    width = num_heads * head_dim if per_channel else num_heads
    if tuple(state.shape[1:]) != (num_heads, head_dim, v_dim):
        raise ValueError("state must be [slots, heads, head_dim, v_dim]")
    need = max(q_off + num_kv_heads * head_dim, k_off + num_kv_heads * head_dim, v_off + num_heads * v_dim)
    if qkv.dim() != 2 or qkv.shape[1] < need or not qkv.is_contiguous():
        raise ValueError("qkv must be contiguous [tokens, >= the q / k / v columns]")
    if out is None:
        out = torch.empty(T, num_heads, v_dim, dtype=torch.float32, device=qkv.device)
    ws = None
    if long_chunks and T > 0:
        ws = torch.empty(lib.mi355_gated_delta_rule_workspace(T, num_heads, num_kv_heads, head_dim), dtype=torch.float32,
                         device=qkv.device)
    check(lib.mi355_gated_delta_rule(
        _f32(out, "out", T * num_heads * v_dim), qkv.data_ptr(), qkv.shape[1], q_off, k_off, v_off,
        _same(beta, qkv, "beta"), _cols(beta, "beta", num_heads), _same(decay, qkv, "decay"), _cols(decay, "decay", width),
        _f32(a_log, "a_log", num_heads), _f32(dt_bias, "dt_bias", width), int(per_channel), _f32(state, "state"),
        _idx(cu_seqlens, "cu_seqlens", torch.int32), _idx(positions, "positions", torch.int64, T),
        _idx(state_slots, "state_slots", torch.int32, S), S, num_heads, num_kv_heads, head_dim, v_dim, T,
        None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), dt, _stream()))
    return out


def general_delta_rule(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, decay_bias: torch.Tensor,
                       rate: torch.Tensor, rate_bias: torch.Tensor, state: torch.Tensor, cu_seqlens: torch.Tensor,
                       positions: torch.Tensor, state_slots: torch.Tensor, num_heads: int, head_dim: int,
                       out: torch.Tensor | None = None, long_chunks: bool = True):
    """The general delta rule over packed chunks: S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r with
    w = exp(-exp(-1/2) sigmoid(decay + decay_bias)), a = sigmoid(rate + rate_bias), u the unit key.
    r / k / v / decay / rate [tokens, heads * head_dim] (column slices are fine); the biases float32;
    state float32 [slots, heads, head_dim, head_dim].  Returns o float32 [tokens, heads, head_dim].
    long_chunks False: the form for chunks of a token or two (one state column per lane)."""
    dt = _dt3(r, "r")
    T, C = r.shape[0], num_heads * head_dim
    S = cu_seqlens.numel() - 1
    if tuple(state.shape[1:]) != (num_heads, head_dim, head_dim):
        raise ValueError("state must be [slots, heads, head_dim, head_dim]")
    if out is None:
        out = torch.empty(T, num_heads, head_dim, dtype=torch.float32, device=r.device)
    if T == 0:
        return out
    ws = None
    if long_chunks:
        ws = torch.empty(lib.mi355_general_delta_rule_workspace(T, num_heads, head_dim), dtype=torch.float32, device=r.device)
    check(lib.mi355_general_delta_rule(
        _f32(out, "out", T * C), r.data_ptr(), _cols(r, "r", C), _same(k, r, "k"), _cols(k, "k", C), _same(v, r, "v"),
        _cols(v, "v", C), _same(decay, r, "decay"), _cols(decay, "decay", C), _f32(decay_bias, "decay_bias", C),
        _same(rate, r, "rate"), _cols(rate, "rate", C), _f32(rate_bias, "rate_bias", C), _f32(state, "state"),
        _idx(cu_seqlens, "cu_seqlens", torch.int32), _idx(positions, "positions", torch.int64, T),
        _idx(state_slots, "state_slots", torch.int32, S), S, num_heads, head_dim, T, int(bool(long_chunks)),
        None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), dt, _stream()))
    return out


def group_rms_norm_f32(x: torch.Tensor, weight: torch.Tensor, groups: int, eps: float, dtype: torch.dtype | None = None,
                       out: torch.Tensor | None = None):
    """RMS norm over each of `groups` equal consecutive parts of the float32 rows x, times weight
    (float32 [width]).  dtype None: float32 rows (out may be x itself); otherwise activation rows."""
    T, W = x.shape
    if out is None:
        out = torch.empty(T, W, dtype=dtype or torch.float32, device=x.device)
    if not out.is_contiguous() or out.shape != x.shape or out.dtype != (dtype or torch.float32):
        raise ValueError("out must be contiguous, shaped like x, in the requested dtype")
    to32 = dtype is None
    check(lib.mi355_group_rms_norm_f32(None if to32 else out.data_ptr(), out.data_ptr() if to32 else None, _f32(x, "x"),
                                       _f32(weight, "weight", W), T, W, int(groups), float(eps),
                                       _DT[torch.float32] if to32 else _dt3(out, "out"), _stream()))
    return out


def gated_norm_resid_f32(resid: torch.Tensor, y: torch.Tensor, gate: torch.Tensor, bias: torch.Tensor,
                         weight: torch.Tensor, groups: int, eps: float, mult: float):
    """resid (float32, in place) += mult * gn(y * sigmoid(gate + bias)) * weight, gn the RMS norm in
    `groups` parts.  y [tokens, width] contiguous; gate the same shape (a column slice is fine)."""
    T, W = resid.shape
    dt = _dt3(y, "y")
    if y.shape != resid.shape or not y.is_contiguous():
        raise ValueError("y must be contiguous, shaped like resid")
    check(lib.mi355_gated_norm_resid_f32(_f32(resid, "resid"), y.data_ptr(), _same(gate, y, "gate"), _cols(gate, "gate", W),
                                         _f32(bias, "bias", W), _f32(weight, "weight", W), T, W, int(groups), float(eps),
                                         float(mult), dt, _stream()))
    return resid


def rms_norm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float):
    """x [rows, n] (a column slice is fine) / rms * weight (float32 [n]) -> contiguous [rows, n] in x's dtype."""
    dt = _dt3(x, "x")
    T, n = x.shape
    out = torch.empty(T, n, dtype=x.dtype, device=x.device)
    check(lib.mi355_rms_norm_rows(out.data_ptr(), x.data_ptr(), _cols(x, "x", n), _f32(weight, "weight", n), T, n,
                                  float(eps), dt, _stream()))
    return out


def tanh_rows(x: torch.Tensor):
    """tanh of x [rows, n] (a column slice is fine) -> contiguous [rows, n]."""
    dt = _dt3(x, "x")
    T, n = x.shape
    out = torch.empty(T, n, dtype=x.dtype, device=x.device)
    check(lib.mi355_tanh_rows(out.data_ptr(), x.data_ptr(), _cols(x, "x", n), T, n, dt, _stream()))
    return out


def latent_kv_write(x: torch.Tensor, norm_weight: torch.Tensor, cos_sin: torch.Tensor, positions: torch.Tensor,
                    slot_mapping: torch.Tensor, cache: torch.Tensor, rank: int, rot: int, eps: float,
                    cache_t: torch.Tensor | None = None):
    """x [tokens, rank + rot] (a column slice is fine): the first rank columns RMS-normed with norm_weight
    (float32), the last rot rotated by the table cos_sin [max_pos, rot_dims], both into the row's slot of
    cache [blocks, 16, rank + rot]; the latent also into cache_t [blocks, rank, 16] if given."""
    dt = _dt3(x, "x")
    T = x.shape[0]
    if cache.dim() != 3 or tuple(cache.shape[1:]) != (BLOCK_SIZE, rank + rot) or not cache.is_contiguous():
        raise ValueError("latent pages must be contiguous [blocks, 16, rank + rot]")
    if cache_t is not None and (tuple(cache_t.shape) != (cache.shape[0], rank, BLOCK_SIZE) or not cache_t.is_contiguous()):
        raise ValueError("the channel-major latent pages must be contiguous [blocks, rank, 16]")
    check(lib.mi355_latent_kv_write(_same(cache, x, "cache"), None if cache_t is None else _same(cache_t, x, "cache_t"),
                                    x.data_ptr(), _cols(x, "x", rank + rot),
                                    _f32(norm_weight, "norm_weight", rank), _f32(cos_sin, "cos_sin") or x.data_ptr(),
                                    max(cos_sin.shape[0], 1), _idx(positions, "positions", torch.int64, T),
                                    _idx(slot_mapping, "slot_mapping", torch.int64, T), T, rank, rot, cos_sin.shape[1],
                                    float(eps), dt, _stream()))


def pair_tiles(cu_seqlens, num_heads: int) -> "np.ndarray":
    """(chunk, first pair, pairs <= 16) for every tile of 16 consecutive (packed row, head) pairs of a
    packed batch, pair number = row * num_heads + head, from the host copy of cu_seqlens: the work
    list of the matrix-core latent attention."""
    import numpy as np
    cu = np.asarray(cu_seqlens, dtype=np.int64) * num_heads
    out = []
    for s in range(len(cu) - 1):
        first = np.arange(cu[s], cu[s + 1], 16, dtype=np.int64)
        out.append(np.stack([np.full_like(first, s), first, np.minimum(16, cu[s + 1] - first)], axis=1))
    return (np.concatenate(out) if out else np.zeros((0, 3))).astype(np.int32).reshape(-1, 3)


def latent_tiles_ok(dtype: torch.dtype, rank: int, rot: int) -> bool:
    """Whether the matrix-core latent attention covers these sizes."""
    return dtype in (torch.bfloat16, torch.float16) and rank % 16 == 0 and (rank + rot) % 8 == 0 and rank <= 512 \
        and rank + rot <= 640


def latent_q_pack(q_latent: torch.Tensor, q: torch.Tensor, q_head_width: int, q_rot_offset: int, rot: int,
                  cos_sin: torch.Tensor, positions: torch.Tensor):
    """[tokens, heads, rank + rot] = q_latent [heads, tokens, rank] | the rotated `rot` columns of q at
    q_rot_offset of every head: the query as latent_window_attn_tiles reads it."""
    dt = _dt3(q, "q")
    H, T, rank = q_latent.shape
    if q_latent.stride(2) != 1 or q.shape[0] != T:
        raise ValueError("q_latent must be [heads, tokens, rank] with a contiguous last dim")
    out = torch.empty(T, H, rank + rot, dtype=q.dtype, device=q.device)
    check(lib.mi355_latent_q_pack(out.data_ptr(), _same(q_latent, q, "q_latent"), max(q_latent.stride(1), rank),
                                  max(q_latent.stride(0), rank), q.data_ptr(), _cols(q, "q", H * q_head_width), q_head_width,
                                  q_rot_offset, _f32(cos_sin, "cos_sin") or q.data_ptr(), max(cos_sin.shape[0], 1),
                                  _idx(positions, "positions", torch.int64, T), T, H, rank, rot, cos_sin.shape[1], dt,
                                  _stream()))
    return out


def latent_window_attn_tiles(q_packed: torch.Tensor, cache: torch.Tensor, cache_t: torch.Tensor, block_tables: torch.Tensor,
                             tiles: torch.Tensor, positions: torch.Tensor, sink: torch.Tensor, gate: torch.Tensor | None,
                             window: int, scale: float, num_splits: int = 1, out: torch.Tensor | None = None):
    """The matrix-core form of latent_window_attn: q_packed [tokens, heads, rank + rot] (latent_q_pack),
    both copies of the latent pages, tiles from pair_tiles.  Returns [heads, tokens, rank]."""
    dt = _dt16(q_packed, "q_packed")
    T, H, dq = q_packed.shape
    rank = cache_t.shape[1]
    if not q_packed.is_contiguous() or tuple(cache.shape[1:]) != (BLOCK_SIZE, dq) or not cache.is_contiguous() \
            or tuple(cache_t.shape) != (cache.shape[0], rank, BLOCK_SIZE) or not cache_t.is_contiguous():
        raise ValueError("q_packed [tokens, heads, rank + rot], pages [blocks, 16, rank + rot] and [blocks, rank, 16]")
    if tiles.dtype != torch.int32 or tiles.dim() != 2 or tiles.shape[1] != 3 or not tiles.is_contiguous() or not tiles.is_cuda:
        raise ValueError("tiles must be a contiguous int32 [n, 3] tensor on the GPU")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be contiguous int32 [chunks, max_blocks]")
    if out is None:
        out = torch.empty(H, T, rank, dtype=q_packed.dtype, device=q_packed.device)
    partial = None
    if num_splits > 1:
        partial = torch.empty(num_splits * T * H * (rank + 2), dtype=torch.float32, device=q_packed.device)
    check(lib.mi355_latent_window_attn_tiles(
        out.data_ptr(), max(out.stride(1), rank), max(out.stride(0), rank), q_packed.data_ptr(),
        _same(cache, q_packed, "cache"), _same(cache_t, q_packed, "cache_t"), block_tables.data_ptr(), block_tables.shape[1],
        tiles.data_ptr(), tiles.shape[0], _idx(positions, "positions", torch.int64, T), _f32(sink, "sink", H),
        None if gate is None else _same(gate, q_packed, "gate"), 0 if gate is None else _cols(gate, "gate", H), T, H, rank,
        dq - rank, int(window), float(scale), None if partial is None else partial.data_ptr(), int(num_splits), dt,
        _stream()))
    return out


def latent_window_attn(q_latent: torch.Tensor, q: torch.Tensor, q_head_width: int, q_rot_offset: int, cache: torch.Tensor,
                       block_tables: torch.Tensor, tok_seq: torch.Tensor, positions: torch.Tensor, sink: torch.Tensor,
                       gate: torch.Tensor | None, cos_sin: torch.Tensor, window: int, scale: float,
                       out: torch.Tensor | None = None):
    """Sliding-window softmax attention with a sink over latent pages (see latent_kv_write).  q_latent
    [heads, tokens, rank]: the unrotated query part multiplied into the latent space; q [tokens, heads *
    q_head_width] holds the part to rotate at q_rot_offset of every head.  Returns the gated weighted
    latent [heads, tokens, rank]."""
    dt = _dt3(q, "q")
    T = q.shape[0]
    H, _, rank = q_latent.shape
    rot = cache.shape[2] - rank
    if q_latent.shape[1] != T or q_latent.stride(2) != 1:
        raise ValueError("q_latent must be [heads, tokens, rank] with a contiguous last dim")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be contiguous int32 [chunks, max_blocks]")
    if cache.dim() != 3 or cache.shape[1] != BLOCK_SIZE or rot < 0 or not cache.is_contiguous():
        raise ValueError("latent pages must be contiguous [blocks, 16, rank + rot]")
    if out is None:
        out = torch.empty(H, T, rank, dtype=q.dtype, device=q.device)
    if out.shape != q_latent.shape or out.stride(2) != 1 or out.dtype != q.dtype:
        raise ValueError("out must be shaped like q_latent")
    check(lib.mi355_latent_window_attn(
        out.data_ptr(), max(out.stride(1), rank), max(out.stride(0), rank), _same(q_latent, q, "q_latent"),
        max(q_latent.stride(1), rank), max(q_latent.stride(0), rank), q.data_ptr(), _cols(q, "q", H * q_head_width),
        q_head_width, q_rot_offset, _same(cache, q, "cache"),
        block_tables.data_ptr(), block_tables.shape[1], _idx(tok_seq, "tok_seq", torch.int32, T),
        _idx(positions, "positions", torch.int64, T), _f32(sink, "sink", H),
        None if gate is None else _same(gate, q, "gate"), 0 if gate is None else _cols(gate, "gate", H),
        _f32(cos_sin, "cos_sin") or q.data_ptr(), max(cos_sin.shape[0], 1), T, H, rank, rot, cos_sin.shape[1],
        int(window), float(scale), dt, _stream()))
    return out


def moe_route(logits: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int, softmax: bool = False,
              group_max: bool = False, weight_scale: float = 1.0, experts: int | None = None, chosen_softmax: bool = False):
    """float32 router logits [tokens, >= experts] (rows may carry more columns than router outputs:
    `experts` says how many count) -> (ids int32 [tokens, top], weights float32 [tokens, top]).
    Scores are a sigmoid per logit or (softmax) a softmax over the router outputs; a group scores the
    sum of its two best choice scores or (group_max) its best.  chosen_softmax: the choice is by the
    logits themselves and the weights are a softmax over the chosen logits alone."""
    T = logits.shape[0]
    E = int(experts) if experts is not None else logits.shape[1]
    _dev(logits, "logits")
    if logits.dtype != torch.float32 or logits.dim() != 2 or logits.stride(1) != 1 or logits.shape[1] < E:
        raise ValueError("logits must be float32 [tokens, >= experts] with a contiguous last dim")
    ids = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    wts = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    check(lib.mi355_moe_route(ids.data_ptr(), wts.data_ptr(), logits.data_ptr(), logits.stride(0) if T > 1 else logits.shape[1],
                              _f32(correction, "correction", E), T, E, int(top), int(groups), int(keep),
                              2 if chosen_softmax else int(bool(softmax)),
                              int(bool(group_max)), float(weight_scale), _stream()))
    return ids, wts


def moe_sort(ids: torch.Tensor, experts: int):
    """Routed rows by expert: (offsets int32 [experts + 1], perm [rows], inv [rows])."""
    rows = ids.numel()
    dev = ids.device
    offsets = torch.empty(experts + 1, dtype=torch.int32, device=dev)
    perm = torch.empty(max(rows, 1), dtype=torch.int32, device=dev)
    inv = torch.empty(max(rows, 1), dtype=torch.int32, device=dev)
    check(lib.mi355_moe_sort(offsets.data_ptr(), perm.data_ptr(), inv.data_ptr(), _idx(ids, "ids", torch.int32), rows,
                             int(experts), _stream()))
    return offsets, perm, inv


def moe_gather_rows(x: torch.Tensor, perm: torch.Tensor, rows: int, top: int, offsets: torch.Tensor | None = None,
                    pad_to: int = 0, experts: int | None = None):
    """The routed rows of x in expert order [rows, width]; with pad_to > 0 every expert's rows padded
    with zero rows to pad_to: [experts * pad_to, width] (`experts`: the first so many of offsets')."""
    dt = _dt3(x, "x")
    if not x.is_contiguous():
        raise ValueError("x must be contiguous")
    n = rows if pad_to <= 0 else (int(experts) if experts is not None else offsets.numel() - 1) * pad_to
    xs = torch.empty(n, x.shape[1], dtype=x.dtype, device=x.device)
    check(lib.mi355_moe_gather_rows(xs.data_ptr(), x.data_ptr(), _idx(perm, "perm", torch.int32, rows),
                                    None if pad_to <= 0 else _idx(offsets, "offsets", torch.int32), max(int(pad_to), 0), n,
                                    int(top), x.shape[1], dt, _stream()))
    return xs


ACT_SILU_MUL, ACT_LIMITED = 0, 1


def _gate_act(limit) -> tuple:
    return (ACT_SILU_MUL, 0.0) if limit is None else (ACT_LIMITED, float(limit))


def moe_gate_up_rows(x: torch.Tensor, w_gate_up: torch.Tensor, offsets: torch.Tensor, perm: torch.Tensor, top: int,
                     limit: float | None = None):
    """a(Wg[e] x, Wu[e] x) for every routed row, in expert order: [tokens * top, ff].  a(g, u) is
    silu(g) * u, or with a limit g' sigmoid(1.702 g') (u' + 1), g' = min(g, limit), u' = clamp(u, -limit, limit).
    offsets may list more bins than w_gate_up has experts (identity experts): their rows are left alone."""
    dt = _dt3(x, "x")
    E, F2, W = w_gate_up.shape
    if not x.is_contiguous() or x.shape[1] != W or not w_gate_up.is_contiguous():
        raise ValueError("x must be contiguous [tokens, width], w_gate_up contiguous [experts, 2 ff, width]")
    rows = x.shape[0] * top
    act = torch.empty(rows, F2 // 2, dtype=x.dtype, device=x.device)
    fn, lim = _gate_act(limit)
    check(lib.mi355_moe_gate_up_rows(act.data_ptr(), x.data_ptr(), _same(w_gate_up, x, "w_gate_up"),
                                     _idx(offsets, "offsets", torch.int32, E + 1), _idx(perm, "perm", torch.int32, rows),
                                     E, int(top), W, F2 // 2, fn, lim, dt, _stream()))
    return act


def moe_down_rows(act: torch.Tensor, w_down: torch.Tensor, offsets: torch.Tensor):
    dt = _dt3(act, "act")
    E, W, F = w_down.shape
    if not act.is_contiguous() or act.shape[1] != F or not w_down.is_contiguous():
        raise ValueError("act must be contiguous [rows, ff], w_down contiguous [experts, width, ff]")
    y = torch.empty(act.shape[0], W, dtype=act.dtype, device=act.device)
    check(lib.mi355_moe_down_rows(y.data_ptr(), act.data_ptr(), _same(w_down, act, "w_down"),
                                  _idx(offsets, "offsets", torch.int32, E + 1), E, W, F, dt, _stream()))
    return y


def moe_silu_and_mul(x: torch.Tensor, limit: float | None = None):
    """x [rows, 2 ff] holding gate | up -> a(gate, up) (see moe_gate_up_rows)."""
    dt = _dt3(x, "x")
    if not x.is_contiguous():
        raise ValueError("x must be contiguous [rows, 2 ff]")
    out = torch.empty(x.shape[0], x.shape[1] // 2, dtype=x.dtype, device=x.device)
    fn, lim = _gate_act(limit)
    check(lib.mi355_moe_silu_and_mul(out.data_ptr(), x.data_ptr(), x.shape[0], x.shape[1] // 2, fn, lim, dt, _stream()))
    return out


def gated_act_rows(gate: torch.Tensor, up: torch.Tensor, limit: float | None = None, out: torch.Tensor | None = None):
    """a(gate, up) (see moe_gate_up_rows) for [rows, ff] column slices of one buffer (equal row
    strides), into `out` [rows, ff], which may be a column slice of a wider buffer."""
    dt = _dt3(gate, "gate")
    R, F = gate.shape
    if up.shape != gate.shape or up.dtype != gate.dtype or gate.stride(1) != 1 or up.stride(1) != 1 \
            or (R > 1 and gate.stride(0) != up.stride(0)):
        raise ValueError("gate and up must be [rows, ff] slices with equal row strides and contiguous columns")
    if out is None:
        out = torch.empty(R, F, dtype=gate.dtype, device=gate.device)
    if out.shape != gate.shape or out.dtype != gate.dtype or out.stride(1) != 1:
        raise ValueError("out must be [rows, ff] with contiguous columns in the dtype of gate")
    fn, lim = _gate_act(limit)
    check(lib.mi355_gated_act_rows(out.data_ptr(), _cols(out, "out", F), gate.data_ptr(), up.data_ptr(), _cols(gate, "gate", F),
                                   R, F, fn, lim, dt, _stream()))
    return out


def moe_combine(y: torch.Tensor, inv: torch.Tensor, weights: torch.Tensor, num_tokens: int, top: int,
                ids: torch.Tensor | None = None, offsets: torch.Tensor | None = None, pad_to: int = 0,
                x: torch.Tensor | None = None, num_real: int = 0, shared: torch.Tensor | None = None,
                shared_gate: torch.Tensor | None = None):
    """out[t] = sum_k weights[t, k] * y[inv[t * top + k]]; with pad_to > 0, y holds every expert's rows
    padded to pad_to (moe_gather_rows) and ids / offsets locate them.  x: chosen ids >= num_real are
    identity experts whose row is x[t].  shared [tokens, width]: added, times the sigmoid of
    shared_gate (float32, one number per token; any row stride) if given."""
    dt = _dt3(y, "y")
    if not y.is_contiguous():
        raise ValueError("y must be contiguous")
    W = y.shape[1]
    out = torch.empty(num_tokens, W, dtype=y.dtype, device=y.device)
    pad = max(int(pad_to), 0)
    need_ids = pad > 0 or x is not None
    for n, t in (("x", x), ("shared", shared)):
        if t is not None and (t.dtype != y.dtype or not t.is_contiguous() or tuple(t.shape) != (num_tokens, W)):
            raise ValueError(f"{n} must be contiguous [tokens, width] in the dtype of y")
    sg, sgs = None, 0
    if shared_gate is not None:
        _dev(shared_gate, "shared_gate")
        if shared is None or shared_gate.dtype != torch.float32 or shared_gate.shape[0] != num_tokens:
            raise ValueError("shared_gate: float32, one number per token, with shared rows")
        sg, sgs = shared_gate.data_ptr(), (shared_gate.stride(0) if num_tokens > 1 else 1)
    check(lib.mi355_moe_combine(out.data_ptr(), y.data_ptr(), _idx(inv, "inv", torch.int32, num_tokens * top),
                                _f32(weights, "weights", num_tokens * top),
                                None if not need_ids else _idx(ids, "ids", torch.int32, num_tokens * top),
                                None if pad == 0 else _idx(offsets, "offsets", torch.int32), pad, num_tokens, int(top),
                                W, None if x is None else x.data_ptr(), int(num_real),
                                None if shared is None else shared.data_ptr(), sg, sgs, dt, _stream()))
    return out


# ---- hashed previous-token embedding, block attention with a distance penalty, per-channel gated recurrence
def embed_bigram_pos_f32(embed: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, bigram: torch.Tensor | None = None,
                         hash_consts: tuple | None = None, cu_seqlens: torch.Tensor | None = None,
                         tok_seq: torch.Tensor | None = None, state_slots: torch.Tensor | None = None,
                         prev_tokens: torch.Tensor | None = None, freq: torch.Tensor | None = None):
    """float32 rows embed[id] + bigram[(prev * mul_prev + id * mul_cur) % buckets] + sinusoid(position).
    hash_consts = (buckets, mul_prev, mul_cur); bigram [buckets + 1, width], its last row for position
    0.  The previous token of a chunk's first row is prev_tokens[state slot] (int32; see
    prev_token_update).  freq float32 [ceil(width / 2)]: entries 2i / 2i + 1 get sin / cos of
    position * freq[i]."""
    dt = _dt3(embed, "embed")
    if embed.dim() != 2 or not embed.is_contiguous():
        raise ValueError("embed must be contiguous [vocab, width]")
    T, W = ids.numel(), embed.shape[1]
    out = torch.empty(T, W, dtype=torch.float32, device=embed.device)
    buckets = mp = mc = 0
    if bigram is not None:
        buckets, mp, mc = (int(v) for v in hash_consts)
        if bigram.dtype != embed.dtype or not bigram.is_contiguous() or tuple(bigram.shape) != (buckets + 1, W):
            raise ValueError("bigram must be contiguous [buckets + 1, width] in the dtype of embed")
        S = cu_seqlens.numel() - 1
        _idx(cu_seqlens, "cu_seqlens", torch.int32), _idx(tok_seq, "tok_seq", torch.int32, T)
        _idx(state_slots, "state_slots", torch.int32, S), _idx(prev_tokens, "prev_tokens", torch.int32)
    if freq is not None:
        _f32(freq, "freq", (W + 1) // 2)
    check(lib.mi355_embed_bigram_pos_f32(
        out.data_ptr(), embed.data_ptr(), None if bigram is None else bigram.data_ptr(), _idx(ids, "ids", torch.int64),
        _idx(positions, "positions", torch.int64, T), None if bigram is None else cu_seqlens.data_ptr(),
        None if bigram is None else tok_seq.data_ptr(), None if bigram is None else state_slots.data_ptr(),
        None if bigram is None else prev_tokens.data_ptr(), None if freq is None else freq.data_ptr(), T, W, embed.shape[0],
        buckets, mp, mc, dt, _stream()))
    return out


def prev_token_update(prev_tokens: torch.Tensor, ids: torch.Tensor, cu_seqlens: torch.Tensor, state_slots: torch.Tensor):
    """prev_tokens[state slot of chunk s] = the last token of chunk s."""
    S = cu_seqlens.numel() - 1
    check(lib.mi355_prev_token_update(_idx(prev_tokens, "prev_tokens", torch.int32), _idx(ids, "ids", torch.int64),
                                      _idx(cu_seqlens, "cu_seqlens", torch.int32), _idx(state_slots, "state_slots", torch.int32, S),
                                      S, _stream()))
    return prev_tokens


def relu_squared(x: torch.Tensor):
    """max(x, 0)^2."""
    dt = _dt3(x, "x")
    if not x.is_contiguous():
        raise ValueError("x must be contiguous")
    out = torch.empty_like(x)
    check(lib.mi355_relu_squared(out.data_ptr(), x.data_ptr(), x.numel(), dt, _stream()))
    return out


def qk_norm_kv_write(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor,
                     slot_mapping: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, num_heads: int,
                     num_kv_heads: int, head_dim: int, v_dim: int, eps: float):
    """q [tokens, heads * dim] is RMS-normed per head in place (weight float32 [dim]); the normed k goes
    to the K pages, v (as given; it may be k itself) to the V pages.  q / k / v may be column slices."""
    dt = _dt3(q, "q")
    T = q.shape[0]
    check(lib.mi355_qk_norm_kv_write(
        q.data_ptr(), _cols(q, "q", num_heads * head_dim), _same(k, q, "k"), _cols(k, "k", num_kv_heads * head_dim),
        _same(v, q, "v"), _cols(v, "v", num_kv_heads * v_dim), _f32(q_weight, "q_weight", head_dim),
        _f32(k_weight, "k_weight", head_dim), _idx(slot_mapping, "slot_mapping", torch.int64, T),
        _same(k_cache, q, "k_cache"), _same(v_cache, q, "v_cache"), T, num_heads, num_kv_heads, head_dim, v_dim, float(eps),
        dt, _stream()))


def softmax_bias_attn(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                      tok_seq: torch.Tensor, positions: torch.Tensor, r1: torch.Tensor | None, r2: torch.Tensor | None,
                      gate: torch.Tensor | None, num_heads: int, scale: float, block: int = 0, window: int = 0,
                      tiles: torch.Tensor | None = None, num_splits: int = 0, sink: torch.Tensor | None = None,
                      out: torch.Tensor | None = None):
    """Softmax attention over the paged K/V [blocks, kv_heads, 16, dim] / [blocks, kv_heads, vdim, 16] with
    the score q.k * scale - r1[h] ln(1 + r2[h] * distance); a row at position p sees the keys j <= p of
    its block of `block` positions (0: all) and, window > 0, the last `window` of them.  gate
    [tokens, heads] or [tokens, heads * vdim]: the output is multiplied by its sigmoid.  tiles
    (query_tiles) selects the matrix-core form where the sizes allow; num_splits > 1 spreads a
    tile's keys over that many workgroups.  sink (float32 [heads]): the softmax denominator holds one
    more term exp(sink[h]) without a value.  out: [tokens, heads * vdim], may be a column slice of a
    wider buffer.  Returns [tokens, heads * vdim]."""
    dt = _dt3(q, "q")
    T = q.shape[0]
    G, d, dv = k_cache.shape[1], k_cache.shape[3], v_cache.shape[2]
    if k_cache.shape[2] != BLOCK_SIZE or v_cache.shape[3] != BLOCK_SIZE or v_cache.shape[1] != G \
            or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise ValueError("k_cache [blocks, kv_heads, 16, dim] and v_cache [blocks, kv_heads, vdim, 16], contiguous")
    if block_tables.dim() != 2 or not block_tables.is_contiguous():
        raise ValueError("block_tables must be contiguous [chunks, max_blocks]")
    if out is None:
        out = torch.empty(T, num_heads * dv, dtype=q.dtype, device=q.device)
    elif out.dtype != q.dtype or tuple(out.shape) != (T, num_heads * dv) or out.stride(1) != 1:
        raise ValueError("out must be [tokens, heads * vdim] with contiguous columns in the dtype of q")
    per_channel, gs = 0, 0
    if gate is not None:
        per_channel = int(gate.shape[1] == num_heads * dv and dv > 1)
        gs = _cols(gate, "gate", num_heads * dv if per_channel else num_heads)
    ws, n = None, 0
    if tiles is not None and num_splits > 1 and q.dtype != torch.float32:
        n = int(num_splits)
        ws = torch.empty(lib.mi355_softmax_bias_attn_workspace(T, num_heads, dv, n), dtype=torch.float32, device=q.device)
    check(lib.mi355_softmax_bias_attn(
        out.data_ptr(), q.data_ptr(), _cols(q, "q", num_heads * d), _same(k_cache, q, "k_cache"), _same(v_cache, q, "v_cache"),
        _idx(block_tables, "block_tables", torch.int32), block_tables.shape[1], _idx(tok_seq, "tok_seq", torch.int32, T),
        _idx(positions, "positions", torch.int64, T), None if r1 is None else _f32(r1, "r1", num_heads),
        None if r2 is None else _f32(r2, "r2", num_heads), None if gate is None else _same(gate, q, "gate"), gs, per_channel,
        T, num_heads, G, d, dv, int(block), int(window), float(scale),
        None if tiles is None else _idx(tiles, "tiles", torch.int32), 0 if tiles is None else tiles.shape[0],
        None if ws is None else ws.data_ptr(), n, None if sink is None else _f32(sink, "sink", num_heads),
        _cols(out, "out", num_heads * dv), dt, _stream()))
    return out


def mingru_scan(proj: torch.Tensor, z_off: int, x_off: int, g_off: int, channels: int, z_bias: torch.Tensor | None,
                x_bias: torch.Tensor | None, state: torch.Tensor, cu_seqlens: torch.Tensor, positions: torch.Tensor,
                state_slots: torch.Tensor, long_chunks: bool = True, num_parts: int | None = None):
    """The per-channel gated recurrence over a packed batch: proj [tokens, >= ...] holds the z, x and
    gate projections at the given column offsets; state float32 [slots, channels] is read (unless the
    chunk starts at position 0) and left at the chunk's last token.  long_chunks: some chunk holds
    several rows.  num_parts: workgroups a chunk is dealt out to (None: enough to fill the chip when
    the step has few, long chunks).  Returns S * silu(gate) [tokens, channels] in proj's dtype."""
    dt = _dt3(proj, "proj")
    T, S = proj.shape[0], cu_seqlens.numel() - 1
    if proj.dim() != 2 or proj.stride(1) != 1:
        raise ValueError("proj must be [tokens, columns] with a contiguous last dim")
    if state.dim() != 2 or state.shape[1] != channels:
        raise ValueError("state must be float32 [slots, channels]")
    out = torch.empty(T, channels, dtype=proj.dtype, device=proj.device)
    if num_parts is None:                                      # about 16 rows per wave at least, about 512 workgroups at most
        num_parts = min(16, max(T // max(S, 1) // 256, 1), max(512 // max(S * ((channels + 63) // 64), 1), 1))
    num_parts = int(num_parts) if long_chunks else 1
    ws = torch.empty(lib.mi355_mingru_scan_workspace(S, channels, num_parts), dtype=torch.float32, device=proj.device) \
        if num_parts > 1 else None
    check(lib.mi355_mingru_scan(
        out.data_ptr(), proj.data_ptr(), proj.stride(0) if T > 1 else proj.shape[1], int(z_off), int(x_off), int(g_off),
        None if z_bias is None else _f32(z_bias, "z_bias", channels), None if x_bias is None else _f32(x_bias, "x_bias", channels),
        _f32(state, "state"), _idx(cu_seqlens, "cu_seqlens", torch.int32), _idx(positions, "positions", torch.int64, T),
        _idx(state_slots, "state_slots", torch.int32, S), S, T, int(channels), int(bool(long_chunks)),
        None if ws is None else ws.data_ptr(), num_parts, dt, _stream()))
    return out
