"""Python callables over the C ABI, shaped like the reference's kernel objects.

The reference reaches its kernels through tilelang ``JITKernel`` callables that
take the non-output tensors positionally, allocate the tensors listed in
``out_idx`` with ``torch.empty`` and return them, read dynamic sizes from the
tensor shapes and launch on the current torch stream
(EfficientKascadeStrategy.py:24-70, kernel_utils.py:50-81).  The functions here
keep those call shapes; each one names the reference callable it stands for.

PyTorch is used for device memory and the stream handle only.  Every function
raises ``KascadeError`` when libkascade_hip.so is missing or a call fails.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import Strides, KascadeError
from . import budgets

H, G, D, TILE = 32, 8, 128, 32      # the reference's shape (EfficientKascadeStrategy.py:19-21)
GROUP = 4                             # query heads per KV head of the reference's shape
GROUPS_OK = tuple(range(1, 17))       # ... and what the kernels take
_ELEM = {torch.float16: 0, torch.bfloat16: 1}


def _shape(Q: torch.Tensor, K: torch.Tensor):
    """(query heads, KV heads, head_dim, dtype) of a call, from Q [..., H, D] and K [..., G, D]:
    fp16 or bf16, head_dim 64 or 128, 1 to 16 query heads per KV head."""
    Hq, Dh, Gk = Q.shape[-2], Q.shape[-1], K.shape[-2]
    if Q.dtype not in _ELEM or K.dtype != Q.dtype:
        raise KascadeError(f"Q and K must both be float16 or bfloat16, got {Q.dtype} / {K.dtype}")
    if Dh not in (64, 128) or K.shape[-1] != Dh:
        raise KascadeError(f"head_dim must be 64 or 128 for Q and K, got {Dh} / {K.shape[-1]}")
    if Gk < 1 or Hq % Gk or Hq // Gk not in GROUPS_OK:
        raise KascadeError(f"need 1 to 16 query heads per KV head, got {Hq} query / {Gk} KV heads")
    return Hq, Gk, Dh, Q.dtype


_entry = {}     # (name, shaped) -> bound library function: attribute look-ups are per-call cost


def _call(lib, name: str, shape, *args):
    """The plain entry point for the reference's shape, its *_shaped_call twin otherwise."""
    Hq, Gk, Dh, dt = shape
    if Gk == G and Dh == D and dt is torch.float16 and Hq == H:
        fn = _entry.get((name, False))
        if fn is None:
            fn = _entry[(name, False)] = getattr(lib, f"kascade_{name}_call")
        return fn(*args)
    fn = _entry.get((name, True))
    if fn is None:
        fn = _entry[(name, True)] = getattr(lib, f"kascade_{name}_shaped_call")
    return fn(ctypes.byref(_lib.Shape(Gk, Dh, _ELEM[dt], Hq // Gk)), *args)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Handle of the current stream of the current device.  The raw accessor skips the stream
    object torch.cuda.current_stream() builds (several microseconds per kernel call)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _req(t: torch.Tensor, dtype, name: str, contiguous: bool = True):
    if t.is_cuda and t.dtype is dtype and (not contiguous or t.is_contiguous()):
        return
    if not t.is_cuda:
        raise KascadeError(f"{name} must be a device tensor")
    if t.dtype != dtype:
        raise KascadeError(f"{name} must be {dtype}, got {t.dtype}")
    raise KascadeError(f"{name} must be contiguous")


def _blhd_strides(t: torch.Tensor, name: str) -> Strides:
    """Strides of a [B,L,heads,D] view whose innermost dimension is contiguous."""
    if t.dim() != 4 or t.stride(-1) != 1:
        raise KascadeError(f"{name} must be [B,L,heads,D] with a contiguous last dimension")
    return Strides(t.stride(0), t.stride(1), t.stride(2))


GATHER_ROWS_PER_SPLIT = 1664


def default_num_split(total_rows: int, max_rows: int, wgs_per_cu: int = 2, min_rows: int = 512,
                      cap_rows: Optional[int] = None, row_counts=None, heads: int = G) -> int:
    """Split count for a decode launch.  Every split covers the same number of rows
    (ceil(max_rows/num_split)), so the number of non-empty workgroups is about
    total_rows / rows_per_split; aim at wgs_per_cu of them per compute unit without
    dropping below min_rows rows per workgroup (per-workgroup set-up is not free).
    total_rows = sum over (sequence, KV head) of the rows visited; max_rows = longest list.
    cap_rows: upper limit on the rows of a split.  Gather launches keep a split at about
    GATHER_ROWS_PER_SPLIT rows: twice that is 1-3 % faster on uniform batches (batch 16 x 26240
    rows: 307 us against 316 us) but 6 % slower on the ragged batch of four long sequences
    (109 us against 103 us); the streaming kernels do not care.
    row_counts: the rows of every sequence (per KV head), when the caller knows them."""
    cus = _lib.init().kascade_device_cu_count() or 256
    target_wgs = wgs_per_cu * cus
    if row_counts is not None and len(row_counts) > 1 and total_rows / max(min_rows, 1) >= cus:
        # Ragged batch with known lengths: count the workgroups exactly.  Each sequence rounds its
        # split count up, and a few workgroups beyond what is resident at once run when almost
        # everything else has finished, far below the device's bandwidth (four sequences of
        # 131072..524288 tokens, 10 % gathered: 86 us with 512 workgroups, 100 us with 544).  So
        # take the largest split count whose workgroups still fit `rounds` residencies, more
        # than one only when a split would otherwise exceed about 4096 rows.
        def count(ns):
            rps = ((-(-max_rows // ns) + 63) // 64) * 64
            return heads * sum(max(1, -(-int(n) // rps)) for n in row_counts), rps
        rounds = 1
        while True:
            best = 1
            for ns in range(1, 257):
                wgs, rps = count(ns)
                if wgs <= rounds * target_wgs and rps >= min(min_rows, max_rows):
                    best = ns
            if not cap_rows or count(best)[1] <= 4096 or rounds >= 8:
                return best
            rounds += 1
    rows_per_split = max(min_rows, total_rows / target_wgs)
    if cap_rows:
        rows_per_split = min(rows_per_split, cap_rows)
    if total_rows / rows_per_split < cus:
        # small launch (short lists, small batch): latency, not set-up, is what counts, so
        # spread down to 128 rows per workgroup to put one workgroup on every compute unit
        rows_per_split = max(min(128, min_rows), total_rows / cus)
    # round to nearest: one workgroup more than a whole number per compute unit costs a
    # full extra wave of workgroups on a few units (tail), one fewer costs nothing
    return int(max(1, min(256, round(max_rows / rows_per_split))))


# ---------------------------------------------------------------- decode
def _out_buffer(out, B, device, shape=(H, G, D, torch.float16)) -> torch.Tensor:
    """The caller's [B,H,D] output buffer, or a fresh one."""
    Hq, _, Dh, dt = shape
    if out is None:
        return torch.empty(B, Hq, Dh, device=device, dtype=dt)
    _req(out, dt, "out")
    if tuple(out.shape) != (B, Hq, Dh):
        raise KascadeError(f"out must be [{B},{Hq},{Dh}]")
    return out


def _decode_kv(K, V, block_table, shape=(H, G, D, torch.float16)):
    """dtype / layout check of the decode K and V operands; returns the optional strides argument.
    Pages must be contiguous.  Without a block table any [B,L,G,D] view with a contiguous last
    dimension is read in place (e.g. a head-major [B,G,L,D] cache transposed), and the strides
    are passed only when the view is not the plain contiguous layout."""
    _, Gk, Dh, dt = shape
    for t, name in ((K, "K"), (V, "V")):
        _req(t, dt, name, contiguous=block_table is not None)
    if K.shape != V.shape or tuple(K.shape[-2:]) != (Gk, Dh):
        raise KascadeError(f"K and V must share one [..., {Gk}, {Dh}] shape")
    if block_table is not None or (K.is_contiguous() and V.is_contiguous()):
        return None
    ks, vs = _blhd_strides(K, "K"), _blhd_strides(V, "V")
    if (ks.b, ks.l, ks.h) != (vs.b, vs.l, vs.h):
        raise KascadeError("K and V must share one set of strides")
    return ctypes.byref(ks)


def _new_rows(k_new, v_new, B, shape=(H, G, D, torch.float16)):
    """Optional [B,G,D] rows of the newest token for the fused append (both or neither)."""
    if k_new is None and v_new is None:
        return None, None
    if k_new is None or v_new is None:
        raise KascadeError("k_new and v_new come together")
    _, Gk, Dh, dt = shape
    for t, name in ((k_new, "k_new"), (v_new, "v_new")):
        _req(t, dt, name)
        if tuple(t.shape) != (B, Gk, Dh):
            raise KascadeError(f"{name} must be [{B},{Gk},{Dh}]")
    return _ptr(k_new), _ptr(v_new)


def decode_budgets(cache_seqlens, topk_percent: float, advance: int = 0, valid_out=None, n_sel_out=None,
                   kv_heads: int = G):
    """One small launch for the bookkeeping of a ragged decode step: adds ``advance`` to the
    lengths in place and returns (valid_len, n_sel) per (sequence, KV head) row as the selection
    takes them.  The reference's benchmark glue does this on the host
    (recompute_kascade_gqa_decode_with_kvcache.py:368-377)."""
    lib = _lib.init()
    _req(cache_seqlens, torch.int32, "cache_seqlens")
    B = cache_seqlens.numel()
    n = B * kv_heads
    if valid_out is None:
        valid_out = torch.empty(n, device=cache_seqlens.device, dtype=torch.int32)
    if n_sel_out is None:
        n_sel_out = torch.empty(n, device=cache_seqlens.device, dtype=torch.int32)
    for t, name in ((valid_out, "valid_out"), (n_sel_out, "n_sel_out")):
        _req(t, torch.int32, name)
        if t.numel() < n:
            raise KascadeError(f"{name} needs {n} entries")
    # only the KV-head count of the shape matters here
    _lib.check(_call(lib, "decode_budgets", (GROUP * kv_heads, kv_heads, D, torch.float16),
                     _ptr(cache_seqlens), int(advance), float(topk_percent), B, _ptr(valid_out), _ptr(n_sel_out),
                     _stream()))
    return valid_out[:n], n_sel_out[:n]


def _decode_shapes(Q, shape, idx=None, head_mapping=None, glse=None, Output_partial=None,
                   block_table=None, cache_seqlens=None) -> None:
    """Tensor metadata of a decode call against the shape the kernels will index with: a scratch or
    index tensor sized for another head count would be read or written out of bounds on the device."""
    Hq, Gk, Dh, _ = shape
    B = Q.shape[0]
    if tuple(Q.shape) != (B, Hq, Dh):
        raise KascadeError(f"Q must be [B,{Hq},{Dh}]")
    if idx is not None and (idx.dim() != 3 or tuple(idx.shape[:2]) != (B, Gk)):
        raise KascadeError(f"index lists must be [{B},{Gk},topk]")
    if head_mapping is not None and head_mapping.numel() != Gk:
        raise KascadeError(f"head_mapping must have {Gk} entries")
    if glse is not None:
        ns = glse.shape[2] if glse.dim() == 3 else -1
        if tuple(glse.shape) != (B, Hq, ns) or Output_partial is None or tuple(Output_partial.shape) != (B, Hq, ns, Dh):
            raise KascadeError(f"glse must be [{B},{Hq},S] and Output_partial [{B},{Hq},S,{Dh}]")
    if block_table is not None and (block_table.dim() != 2 or block_table.shape[0] != B):
        raise KascadeError(f"block_table must be [{B},max_pages]")
    if cache_seqlens is not None and cache_seqlens.numel() != B:
        raise KascadeError(f"cache_seqlens must have {B} entries")


def _sync_arg(sync, B, groups: int = G):
    """Optional [B*G] int32 counter array for the fused combine (zero-initialised by the caller)."""
    if sync is None:
        return None
    _req(sync, torch.int32, "sync_counters")
    if sync.numel() < B * groups:
        raise KascadeError(f"sync_counters needs {B * groups} entries")
    return _ptr(sync)


def _log_sum_arg(log_sum, B, Hq):
    """Optional [B,H] fp32 output: the merged log-sum of the rows every head attended to."""
    if log_sum is None:
        return None
    _req(log_sum, torch.float32, "log_sum")
    if tuple(log_sum.shape) != (B, Hq):
        raise KascadeError(f"log_sum must be [{B},{Hq}]")
    return _ptr(log_sum)


def decode_reuse(Q, K, V, topk_indices, head_mapping, glse, Output_partial, sync=None, log_sum=None) -> torch.Tensor:
    """``decode_reuse_kernel(Q, K, V, topk_indices, head_mapping, glse, Output_partial) -> O``
    (out_idx=[7]; EfficientKascadeStrategy.py:30-38, 113, 122).  Contiguous cache
    K,V [B,L,G,D]; the split count is glse.shape[2].  log_sum: optional [B,H] fp32 output."""
    lib = _lib.init()
    B = Q.shape[0]
    L = K.shape[1]
    shape = _shape(Q, K)
    Hq, Gk, Dh, dt = shape
    _req(Q, dt, "Q")
    kv_strides = _decode_kv(K, V, None, shape)
    _req(topk_indices, torch.int32, "topk_indices"); _req(head_mapping, torch.int32, "head_mapping")
    _req(glse, torch.float32, "glse"); _req(Output_partial, torch.float32, "Output_partial")
    ns = glse.shape[2]
    if tuple(glse.shape) != (B, Hq, ns) or tuple(Output_partial.shape) != (B, Hq, ns, Dh):
        raise KascadeError("glse must be [B,H,S] and Output_partial [B,H,S,D]")
    out = torch.empty(B, Hq, Dh, device=Q.device, dtype=dt)
    if kv_strides is None and shape == (H, G, D, torch.float16) and log_sum is None:
        _lib.check(lib.kascade_decode_reuse_call(
            _ptr(Q), _ptr(K), _ptr(V), _ptr(topk_indices), _ptr(head_mapping), _ptr(glse),
            _ptr(Output_partial), _ptr(out), B, L, topk_indices.shape[-1], ns, _sync_arg(sync, B), _stream()))
    else:
        _lib.check(_call(lib, "decode_reuse_paged", shape,
            _ptr(Q), _ptr(K), _ptr(V), None, _ptr(topk_indices), _ptr(head_mapping), 0.0, _ptr(glse),
            _ptr(Output_partial), _ptr(out), B, L, topk_indices.shape[-1], ns, None, 0, 1, kv_strides,
            None, None, _sync_arg(sync, B, Gk), _log_sum_arg(log_sum, B, Hq), _stream()))
    return out


def decode_reuse_paged(Q, K, V, cache_seqlens, topk_indices, head_mapping, topk_percent, glse,
                       Output_partial, block_table=None, page_size: int = 16, out=None,
                       sync=None, k_new=None, v_new=None, log_sum=None) -> torch.Tensor:
    """``reuse kvcache kernel(Q, K, V, cache_seqlens, topk_indices, head_mapping, topk_percent,
    glse, Output_partial) -> O`` (out_idx=[9]; reuse_kascade_gqa_decode_with_kvcache.py:160-173)
    with an optional block table.  Without one K,V are the padded [B,maxL,G,D] cache;
    with one they are pages [P,page_size,G,D]."""
    lib = _lib.init()
    B = Q.shape[0]
    shape = _shape(Q, K)
    _req(Q, shape[3], "Q")
    kv_strides = _decode_kv(K, V, block_table, shape)
    _req(topk_indices, torch.int32, "topk_indices"); _req(head_mapping, torch.int32, "head_mapping")
    _req(glse, torch.float32, "glse"); _req(Output_partial, torch.float32, "Output_partial")
    if cache_seqlens is not None:
        _req(cache_seqlens, torch.int32, "cache_seqlens")
    _decode_shapes(Q, shape, topk_indices, head_mapping, glse, Output_partial, block_table, cache_seqlens)
    ns = glse.shape[2]
    if block_table is not None:
        _req(block_table, torch.int32, "block_table")
        stride_tokens, max_pages = 0, block_table.shape[1]
    else:
        stride_tokens, max_pages = K.shape[1], 0
    out = _out_buffer(out, B, Q.device, shape)
    _lib.check(_call(lib, "decode_reuse_paged", shape,
        _ptr(Q), _ptr(K), _ptr(V), _ptr(cache_seqlens), _ptr(topk_indices), _ptr(head_mapping),
        float(topk_percent), _ptr(glse), _ptr(Output_partial), _ptr(out), B, stride_tokens,
        topk_indices.shape[-1], ns, _ptr(block_table), max_pages, page_size, kv_strides,
        *_new_rows(k_new, v_new, B, shape), _sync_arg(sync, B, shape[1]), _log_sum_arg(log_sum, B, shape[0]),
        _stream()))
    return out


def decode_reuse_rows(Q, K_pages, V_pages, cache_seqlens, cache_rows, head_mapping, topk_percent, glse,
                      Output_partial, block_table, page_size: int = 16, out=None, sync=None,
                      k_new=None, v_new=None, log_sum=None) -> torch.Tensor:
    """Reuse decode over a paged cache from index lists already translated to cache rows
    (``translate_indices`` of the anchor's selection): one dependent load fewer per row than
    ``decode_reuse_paged``.  cache_rows [B,G,topk] int32."""
    lib = _lib.init()
    B = Q.shape[0]
    shape = _shape(Q, K_pages)
    Hq, Gk, Dh, dt = shape
    _req(Q, dt, "Q"); _req(K_pages, dt, "K_pages"); _req(V_pages, dt, "V_pages")
    _req(cache_rows, torch.int32, "cache_rows"); _req(head_mapping, torch.int32, "head_mapping")
    _req(glse, torch.float32, "glse"); _req(Output_partial, torch.float32, "Output_partial")
    _req(block_table, torch.int32, "block_table")
    if cache_seqlens is not None:
        _req(cache_seqlens, torch.int32, "cache_seqlens")
    if K_pages.dim() != 4 or K_pages.shape[1] != page_size or K_pages.shape != V_pages.shape:
        raise KascadeError(f"pages must be [num_pages,{page_size},{Gk},{Dh}]")
    _decode_shapes(Q, shape, cache_rows, head_mapping, glse, Output_partial, block_table, cache_seqlens)
    ns = glse.shape[2]
    out = _out_buffer(out, B, Q.device, shape)
    _lib.check(_call(lib, "decode_reuse_rows", shape,
        _ptr(Q), _ptr(K_pages), _ptr(V_pages), _ptr(cache_seqlens), _ptr(cache_rows), _ptr(head_mapping),
        float(topk_percent), _ptr(glse), _ptr(Output_partial), _ptr(out), B, cache_rows.shape[-1], ns,
        _ptr(block_table), block_table.shape[1], page_size, K_pages.shape[0], *_new_rows(k_new, v_new, B, shape),
        _sync_arg(sync, B, Gk), _log_sum_arg(log_sum, B, Hq), _stream()))
    return out


NOALLOC_MAX_UNITS = 1024   # batch * num_split the library's built-in scratch holds


def decode_reuse_paged_noalloc(Q, K, V, cache_seqlens, topk_indices, head_mapping, topk_percent,
                               num_split: int, out: torch.Tensor, block_table=None, page_size: int = 16,
                               k_new=None, v_new=None) -> torch.Tensor:
    """``decode_reuse_paged`` for callers that cannot allocate: the splits' partial results live in
    a buffer built into the library (batch * num_split <= NOALLOC_MAX_UNITS), the output buffer is
    the caller's, and nothing is allocated on the way -- not by this wrapper either."""
    lib = _lib.init()
    B = Q.shape[0]
    shape = _shape(Q, K)
    if shape != (H, G, D, torch.float16):
        raise KascadeError(f"the no-allocation entry exists for {H} query / {G} KV heads, head_dim {D}, float16 only")
    _req(Q, torch.float16, "Q")
    kv_strides = _decode_kv(K, V, block_table)
    _req(topk_indices, torch.int32, "topk_indices"); _req(head_mapping, torch.int32, "head_mapping")
    if cache_seqlens is not None:
        _req(cache_seqlens, torch.int32, "cache_seqlens")
    _decode_shapes(Q, shape, topk_indices, head_mapping, None, None, block_table, cache_seqlens)
    if block_table is not None:
        _req(block_table, torch.int32, "block_table")
        stride_tokens, max_pages = 0, block_table.shape[1]
    else:
        stride_tokens, max_pages = K.shape[1], 0
    out = _out_buffer(out, B, Q.device)
    _lib.check(lib.kascade_decode_reuse_paged_noalloc_call(
        _ptr(Q), _ptr(K), _ptr(V), _ptr(cache_seqlens), _ptr(topk_indices), _ptr(head_mapping),
        float(topk_percent), _ptr(out), B, stride_tokens, topk_indices.shape[-1], int(num_split),
        _ptr(block_table), max_pages, page_size, kv_strides, *_new_rows(k_new, v_new, B), _stream()))
    return out


def decode_dense_paged(Q, K, V, cache_seqlens, glse, Output_partial, block_table=None,
                       page_size: int = 16, kv_len: Optional[int] = None, out=None,
                       sync=None, k_new=None, v_new=None) -> torch.Tensor:
    """Dense split-K decode, the baseline of gqa_decode.py / gqa_decode_with_kvcache.py:
    ``kernel(Q, K, V, [cache_seqlens,] glse, Output_partial) -> O``."""
    lib = _lib.init()
    B = Q.shape[0]
    shape = _shape(Q, K)
    _req(Q, shape[3], "Q")
    kv_strides = _decode_kv(K, V, block_table, shape)
    _req(glse, torch.float32, "glse"); _req(Output_partial, torch.float32, "Output_partial")
    _decode_shapes(Q, shape, None, None, glse, Output_partial, block_table, cache_seqlens)
    ns = glse.shape[2]
    if block_table is not None:
        _req(block_table, torch.int32, "block_table")
        stride_tokens, max_pages = (kv_len or 0), block_table.shape[1]
    else:
        stride_tokens, max_pages = K.shape[1], 0
    out = _out_buffer(out, B, Q.device, shape)
    _lib.check(_call(lib, "decode_dense_paged", shape,
        _ptr(Q), _ptr(K), _ptr(V), _ptr(cache_seqlens), _ptr(glse), _ptr(Output_partial), _ptr(out),
        B, stride_tokens, ns, _ptr(block_table), max_pages, page_size, kv_strides,
        *_new_rows(k_new, v_new, B, shape), _sync_arg(sync, B, shape[1]), _stream()))
    return out


def decode_recompute(Q, K, V, glse, Output_partial, row_sums, scores, layer: int,
                     cache_seqlens=None, block_table=None, page_size: int = 16,
                     kv_len: Optional[int] = None, out=None,
                     sync=None, k_new=None, v_new=None) -> Tuple[Optional[torch.Tensor], torch.Tensor]:
    """``decode_recomp{0,1}_kernel(Q, K, V, glse, Output_partial, row_sums, scores) -> (O, agg)``
    (out_idx=[7,8]; EfficientKascadeStrategy.py:24-28, 107-110) and its kvcache form
    (recompute_kascade_gqa_decode_with_kvcache.py:302-333).  ``scores`` is scratch of
    [B,H,stride] fp32 elements whose contents are private to the library (the raw scores travel
    in a compact form); agg is [B,G,stride] fp16.  layer == 0 also computes the dense output;
    otherwise O is None."""
    lib = _lib.init()
    B = Q.shape[0]
    shape = _shape(Q, K)
    _req(Q, shape[3], "Q")
    kv_strides = _decode_kv(K, V, block_table, shape)
    _req(glse, torch.float32, "glse"); _req(row_sums, torch.float32, "row_sums")
    _req(scores, torch.float32, "scores")
    with_out = 1 if layer == 0 else 0
    _decode_shapes(Q, shape, None, None, glse, Output_partial if with_out else None, block_table, cache_seqlens) \
        if with_out else _decode_shapes(Q, shape, None, None, None, None, block_table, cache_seqlens)
    Hq = shape[0]
    if glse.dim() != 3 or tuple(glse.shape[:2]) != (B, Hq) or tuple(row_sums.shape) != (B, Hq) \
            or scores.dim() != 3 or tuple(scores.shape[:2]) != (B, Hq):
        raise KascadeError(f"glse must be [{B},{Hq},S], row_sums [{B},{Hq}] and scores [{B},{Hq},stride]")
    ns = glse.shape[2]
    stride = scores.shape[2]
    if block_table is not None:
        _req(block_table, torch.int32, "block_table")
        stride_tokens, max_pages = (kv_len or 0), block_table.shape[1]
    else:
        stride_tokens, max_pages = K.shape[1], 0
    out = _out_buffer(out, B, Q.device, shape) if with_out else None
    agg = torch.empty(B, shape[1], stride, device=Q.device, dtype=torch.float16)
    _lib.check(_call(lib, "decode_recompute_paged", shape,
        _ptr(Q), _ptr(K), _ptr(V), _ptr(cache_seqlens), _ptr(glse), _ptr(Output_partial),
        _ptr(row_sums), _ptr(scores), _ptr(out), _ptr(agg), B, stride_tokens, stride, ns, with_out,
        _ptr(block_table), max_pages, page_size, kv_strides, *_new_rows(k_new, v_new, B, shape),
        _sync_arg(sync, B, shape[1]), _stream()))
    return out, agg


# ----------------------------------------------------------------- top-k
_TOPK_WS = {}


def _topk_workspace(nbytes: int, device) -> torch.Tensor:
    """Scratch for the multi-workgroup selection, grown on demand and kept per (device, stream):
    selections that run concurrently on different streams must not share it."""
    key = (str(device), torch.cuda.current_stream(device).cuda_stream)
    ws = _TOPK_WS.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(nbytes, device=device, dtype=torch.uint8)
        _TOPK_WS[key] = ws
    return ws


def topk_indices(scores: torch.Tensor, k: int, valid_len=None, n_sel=None,
                 uniform_len: Optional[int] = None, fill_value: Optional[int] = None,
                 block_table: Optional[torch.Tensor] = None, page_size: int = 16,
                 rows_out: Optional[torch.Tensor] = None):
    """Stands for ``torch.topk(scores, k, dim=-1).indices.to(int32)``
    (EfficientKascadeStrategy.py:82, 111) as an exact selection: row r delivers the
    n_sel largest of its first valid_len entries in slots [0, n_sel), ascending by
    index; remaining slots hold fill_value.  valid_len / n_sel are int32 device
    tensors indexed by (row % len) or None for uniform rows.
    With ``block_table`` [B,max_pages] (scores [B, ..., L]) the call returns (indices, cache_rows):
    the same selection also as rows of the paged cache (``translate_indices`` without its
    launch), written to ``rows_out`` when given."""
    lib = _lib.init()
    _req(scores, torch.float16, "scores", contiguous=False)
    if scores.stride(-1) != 1:
        raise KascadeError("scores rows must be contiguous")
    Lrow = scores.shape[-1]
    lead = scores.shape[:-1]
    rows = int(math.prod(lead)) if len(lead) else 1
    # rows must be evenly strided
    flat = scores.reshape(rows, Lrow) if scores.is_contiguous() else None
    if flat is None:
        row_stride = scores.stride(-2)
        exp = row_stride
        for dim in range(scores.dim() - 2, -1, -1):
            if scores.stride(dim) != exp and scores.shape[dim] != 1:
                raise KascadeError("scores must have uniformly strided rows")
            exp *= scores.shape[dim]
    else:
        row_stride = Lrow
    period = 1
    if valid_len is not None:
        _req(valid_len, torch.int32, "valid_len"); period = valid_len.numel()
    if n_sel is not None:
        _req(n_sel, torch.int32, "n_sel")
        if valid_len is not None and n_sel.numel() != period:
            raise KascadeError("valid_len and n_sel must have the same length")
        period = n_sel.numel()
    out = torch.empty(*lead, k, device=scores.device, dtype=torch.int32)
    ulen = Lrow if uniform_len is None else uniform_len
    ws_bytes = lib.kascade_topk_workspace_bytes(rows, ulen)
    ws = _topk_workspace(ws_bytes, scores.device) if ws_bytes > 0 else None
    fill = (Lrow - 1) if fill_value is None else fill_value
    if block_table is None:
        _lib.check(lib.kascade_topk_call(
            _ptr(scores), _ptr(out), rows, row_stride, ulen,
            _ptr(valid_len), _ptr(n_sel), period, k, fill, _ptr(ws), _stream()))
        return out
    _req(block_table, torch.int32, "block_table")
    nseq = block_table.shape[0]
    if scores.shape[0] != nseq or rows % nseq:
        raise KascadeError("block_table needs one row per sequence (the leading dimension of scores)")
    if rows_out is None:
        rows_out = torch.empty_like(out)
    else:
        _req(rows_out, torch.int32, "rows_out")
        if tuple(rows_out.shape) != tuple(out.shape):
            raise KascadeError("rows_out must have the shape of the index tensor")
    _lib.check(lib.kascade_topk_rows_call(
        _ptr(scores), _ptr(out), rows, row_stride, ulen, _ptr(valid_len), _ptr(n_sel), period, k, fill,
        _ptr(ws), _ptr(rows_out), _ptr(block_table), block_table.shape[1], page_size, rows // nseq, _stream()))
    return out, rows_out


def topk_sorted(scores: torch.Tensor, k: int, valid_len=None, uniform_len: Optional[int] = None) -> torch.Tensor:
    """``torch.topk(scores[..., :uniform_len], k, dim=-1).indices.to(int32)`` in the reference's own
    form (EfficientKascadeStrategy.py:82, 90, 111): full-width rows, largest score first, equal
    scores by ascending position; a row with fewer than k valid entries (valid_len, an int32
    device tensor indexed by row % len) continues with the positions past its end.  For a
    consumer that slices its own prefix of a row; the kernels here take ``topk_indices``."""
    lib = _lib.init()
    _req(scores, torch.float16, "scores")
    Lrow = scores.shape[-1]
    lead = scores.shape[:-1]
    rows = int(math.prod(lead)) if len(lead) else 1
    ulen = Lrow if uniform_len is None else uniform_len
    period = 1
    if valid_len is not None:
        _req(valid_len, torch.int32, "valid_len"); period = valid_len.numel()
    out = torch.empty(*lead, k, device=scores.device, dtype=torch.int32)
    ws = torch.empty(max(1, lib.kascade_topk_sorted_workspace_bytes(rows, ulen, k)), dtype=torch.uint8,
                     device=scores.device)
    _lib.check(lib.kascade_topk_sorted_call(_ptr(scores), _ptr(out), rows, Lrow, ulen, _ptr(valid_len), period, k,
                                            _ptr(ws), _stream()))
    return out


# --------------------------------------------------------------- prefill
def prefill_recompute0(Q, K, V) -> Tuple[torch.Tensor, torch.Tensor]:
    """``prefill_recomp0_kernel(Q, K, V) -> (log_sum, O)`` (out_idx=[3,4];
    EfficientKascadeStrategy.py:40-43, 78).  Q [B,L,H,D], K,V [B,L,G,D] (strided views allowed)."""
    lib = _lib.init()
    shape = _shape(Q, K)
    Hq, _, Dh, dt = shape
    _req(Q, dt, "Q", False); _req(K, dt, "K", False); _req(V, dt, "V", False)
    B, L = Q.shape[0], Q.shape[1]
    qs, ks = _blhd_strides(Q, "Q"), _blhd_strides(K, "K")
    if tuple(V.stride()) != tuple(K.stride()) or V.shape != K.shape:
        raise KascadeError("K and V must share shape and strides")
    log_sum = torch.empty(B, L, Hq, device=Q.device, dtype=torch.float32)
    out = torch.empty(B, L, Hq, Dh, device=Q.device, dtype=dt)
    _lib.check(_call(lib, "prefill_dense", shape, _ptr(Q), _ptr(K), _ptr(V), _ptr(log_sum), _ptr(out),
                     B, L, qs, ks, 1, _stream()))
    return log_sum, out


def prefill_recompute1(Q, K) -> torch.Tensor:
    """``prefill_recomp1_kernel(Q, K) -> log_sum`` (out_idx=[2]; EfficientKascadeStrategy.py:44-47, 80)."""
    lib = _lib.init()
    shape = _shape(Q, K)
    _req(Q, shape[3], "Q", False); _req(K, shape[3], "K", False)
    B, L = Q.shape[0], Q.shape[1]
    qs, ks = _blhd_strides(Q, "Q"), _blhd_strides(K, "K")
    log_sum = torch.empty(B, L, shape[0], device=Q.device, dtype=torch.float32)
    _lib.check(_call(lib, "prefill_dense", shape, _ptr(Q), _ptr(K), None, _ptr(log_sum), None,
                     B, L, qs, ks, 0, _stream()))
    return log_sum


def prefill_dense(Q, K, V) -> torch.Tensor:
    """Dense causal prefill baseline (example_gqa_fwd_bshd_wgmma_pipelined.py:121-166):
    ``kernel(Q, K, V) -> O``; no log-sum is written."""
    lib = _lib.init()
    shape = _shape(Q, K)
    Hq, _, Dh, dt = shape
    _req(Q, dt, "Q", False); _req(K, dt, "K", False); _req(V, dt, "V", False)
    B, L = Q.shape[0], Q.shape[1]
    qs, ks = _blhd_strides(Q, "Q"), _blhd_strides(K, "K")
    if tuple(V.stride()) != tuple(K.stride()) or V.shape != K.shape:
        raise KascadeError("K and V must share shape and strides")
    out = torch.empty(B, L, Hq, Dh, device=Q.device, dtype=dt)
    _lib.check(_call(lib, "prefill_dense", shape, _ptr(Q), _ptr(K), _ptr(V), None, _ptr(out),
                     B, L, qs, ks, 1, _stream()))
    return out


def prefill_aggregate(Q, K, log_sum, scores, fill_invalid: bool = False) -> None:
    """``aggregate_kernel(Q, K, log_sum, scores)`` (out_idx=None; in place;
    EfficientKascadeStrategy.py:49-59, 81).  scores [B,G,ceil(L/32),L] fp16."""
    lib = _lib.init()
    shape = _shape(Q, K)
    Hq, Gk, _, dt = shape
    _req(Q, dt, "Q", False); _req(K, dt, "K", False)
    _req(log_sum, torch.float32, "log_sum"); _req(scores, torch.float16, "scores")
    B, L = Q.shape[0], Q.shape[1]
    T = (L + TILE - 1) // TILE
    if tuple(scores.shape) != (B, Gk, T, L) or tuple(log_sum.shape) != (B, L, Hq):
        raise KascadeError("scores must be [B,G,ceil(L/32),L] and log_sum [B,L,H]")
    qs, ks = _blhd_strides(Q, "Q"), _blhd_strides(K, "K")
    _lib.check(_call(lib, "prefill_aggregate", shape, _ptr(Q), _ptr(K), _ptr(log_sum), _ptr(scores), B, L,
                     qs, ks, 1 if fill_invalid else 0, _stream()))


def prefill_aggregate_range(Q, K, log_sum, scores, q_start: int, q_len: int, fill_invalid: bool = False) -> None:
    """``aggregate_kernel`` for the query tiles of rows [q_start, q_start+q_len) of a long prompt:
    Q [B,L,H,D] and log_sum [B,L,H] are the whole prompt's, scores is
    [B,G,ceil(q_len/32),q_start+q_len] fp16.  Lets an anchor layer pool and select a few hundred
    tiles at a time instead of holding L^2/4 bytes of scores."""
    lib = _lib.init()
    shape = _shape(Q, K)
    Hq, Gk, _, dt = shape
    _req(Q, dt, "Q", False); _req(K, dt, "K", False)
    _req(log_sum, torch.float32, "log_sum"); _req(scores, torch.float16, "scores")
    B, L = Q.shape[0], Q.shape[1]
    if q_start % TILE or q_start < 0 or q_len <= 0 or q_start + q_len > L:
        raise KascadeError("q_start must be a multiple of 32 and the range must lie inside the prompt")
    T = (q_len + TILE - 1) // TILE
    if tuple(scores.shape) != (B, Gk, T, q_start + q_len) or tuple(log_sum.shape) != (B, L, Hq):
        raise KascadeError("scores must be [B,G,ceil(q_len/32),q_start+q_len] and log_sum [B,L,H]")
    qs, ks = _blhd_strides(Q, "Q"), _blhd_strides(K, "K")
    q_rows = Q[:, q_start:q_start + q_len]
    ls_rows = log_sum[:, q_start:q_start + q_len].contiguous()      # a view for batch 1
    _lib.check(_call(lib, "prefill_aggregate_range", shape, _ptr(q_rows), _ptr(K), _ptr(ls_rows), _ptr(scores), B,
                     q_start, q_len, qs, ks, 1 if fill_invalid else 0, _stream()))


def prefill_reuse(Q, K, V, topk_idx, head_mapping, topk_percent, rolling: bool, return_log_sum: bool = False):
    """``prefill_reuse_kernel(Q, K, V, topk_indices, head_mapping, topk_percent) -> O``
    (out_idx=[6]; EfficientKascadeStrategy.py:61-70, 92, 97); ``rolling`` selects between the
    reference's two compiled objects.  With return_log_sum also the [B,L,H] fp32 log2-domain
    log-sum over the keys every row attended to: returns (O, log_sum)."""
    lib = _lib.init()
    shape = _shape(Q, K)
    Hq, Gk, Dh, dt = shape
    _req(Q, dt, "Q", False); _req(K, dt, "K", False); _req(V, dt, "V", False)
    _req(topk_idx, torch.int32, "topk_indices"); _req(head_mapping, torch.int32, "head_mapping")
    B, L = Q.shape[0], Q.shape[1]
    T = (L + TILE - 1) // TILE
    if tuple(topk_idx.shape[:3]) != (B, Gk, T) or head_mapping.numel() != Gk:
        raise KascadeError("topk_indices must be [B,G,ceil(L/32),max_topk] and head_mapping [G]")
    qs, ks = _blhd_strides(Q, "Q"), _blhd_strides(K, "K")
    if tuple(V.stride()) != tuple(K.stride()) or V.shape != K.shape:
        raise KascadeError("K and V must share shape and strides")
    out = torch.empty(B, L, Hq, Dh, device=Q.device, dtype=dt)
    log_sum = torch.empty(B, L, Hq, device=Q.device, dtype=torch.float32) if return_log_sum else None
    _lib.check(_call(lib, "prefill_reuse", shape,
        _ptr(Q), _ptr(K), _ptr(V), _ptr(topk_idx), _ptr(head_mapping), float(topk_percent), _ptr(out),
        B, L, topk_idx.shape[-1], 1 if rolling else 0, qs, ks, _ptr(log_sum), _stream()))
    return (out, log_sum) if return_log_sum else out


# ------------------------------------------------------------- KV append
def paged_kv_append(K_pages, V_pages, k_new, v_new, start_pos, block_table, page_size: int = 16,
                    n_new_rows=None):
    """Write k_new/v_new [B,n_new,G,D] into the paged cache at positions start_pos[b]+t.
    n_new_rows [B] int32: sequence b brings only its first n_new_rows[b] rows."""
    lib = _lib.init()
    dt = K_pages.dtype
    if dt not in _ELEM:
        raise KascadeError("pages must be float16 or bfloat16")
    _req(K_pages, dt, "K_pages"); _req(V_pages, dt, "V_pages")
    _req(k_new, dt, "k_new", False); _req(v_new, dt, "v_new", False)
    _req(start_pos, torch.int32, "start_pos"); _req(block_table, torch.int32, "block_table")
    if tuple(k_new.stride()) != tuple(v_new.stride()):
        raise KascadeError("k_new and v_new must share strides")
    Gk, Dh = K_pages.shape[-2], K_pages.shape[-1]
    if Dh not in (64, 128) or tuple(k_new.shape[2:]) != (Gk, Dh) or K_pages.shape != V_pages.shape:
        raise KascadeError("pages [num_pages,page,G,D] and new rows [B,n,G,D] must agree, D 64 or 128")
    B, n_new = k_new.shape[0], k_new.shape[1]
    st = _blhd_strides(k_new, "k_new")
    if start_pos.numel() != B or block_table.shape[0] != B:
        raise KascadeError("start_pos and block_table must have one row per sequence")
    if n_new_rows is not None:
        _req(n_new_rows, torch.int32, "n_new_rows")
        if n_new_rows.numel() != B:
            raise KascadeError("n_new_rows must have one entry per sequence")
    _lib.check(_call(lib, "paged_kv_append", (GROUP * Gk, Gk, Dh, dt),
        _ptr(K_pages), _ptr(V_pages), _ptr(k_new), _ptr(v_new), _ptr(start_pos), _ptr(block_table),
        B, n_new, block_table.shape[1], page_size, st, _ptr(n_new_rows), _stream()))


def rope_table(max_pos: int, theta: float = 1e6, device="cuda", round_to=torch.float16,
               head_dim: int = D) -> torch.Tensor:
    """[max_pos, D] fp32: cos of position * theta^(-2i/D) for the D/2 pairs, then the sines.  The
    angles are formed in fp32 and the values rounded to ``round_to`` (what the transformers
    rotary module hands an fp16 model; None keeps fp32)."""
    inv = (1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))).to(device)
    ang = torch.arange(max_pos, device=device, dtype=torch.float32)[:, None] * inv
    table = torch.cat((ang.cos(), ang.sin()), dim=1)
    if round_to is not None:
        table = table.to(round_to).float()
    return table.contiguous()


def rope_append_paged(q_in, k_in, v_in, cos_sin, start_pos, K_pages, V_pages, block_table,
                      page_size: int = 16, pos_offset: int = 0, q_norm_weight=None, k_norm_weight=None,
                      norm_eps: float = 1e-6, out=None) -> torch.Tensor:
    """What a decoder's attention module does between its projections and the attention call
    (normalise q/k heads, rotate by position, extend the cache), in one launch.  q_in [B,n,H,D],
    k_in/v_in [B,n,G,D] may be views of one packed projection output.  Returns the rotated
    queries [B,n,H,D]; the rotated keys and the values land in their page slots, token t of
    sequence b at position start_pos[b] + pos_offset + t."""
    lib = _lib.init()
    shape = _shape(q_in, k_in)
    Hq, Gk, Dh, dt = shape
    for t, name in ((q_in, "q_in"), (k_in, "k_in"), (v_in, "v_in")):
        _req(t, dt, name, False)
    _req(cos_sin, torch.float32, "cos_sin"); _req(start_pos, torch.int32, "start_pos")
    _req(K_pages, dt, "K_pages"); _req(V_pages, dt, "V_pages")
    _req(block_table, torch.int32, "block_table")
    B, n = q_in.shape[0], q_in.shape[1]
    if tuple(q_in.shape) != (B, n, Hq, Dh) or tuple(k_in.shape) != (B, n, Gk, Dh) or k_in.shape != v_in.shape:
        raise KascadeError(f"q_in must be [B,n,{Hq},{Dh}] and k_in/v_in [B,n,{Gk},{Dh}]")
    if tuple(k_in.stride()) != tuple(v_in.stride()):
        raise KascadeError("k_in and v_in must share strides")
    if cos_sin.dim() != 2 or cos_sin.shape[1] != Dh:
        raise KascadeError(f"cos_sin must be [max_pos,{Dh}]")
    if start_pos.numel() != B or block_table.shape[0] != B:
        raise KascadeError("start_pos and block_table must have one row per sequence")
    if K_pages.dim() != 4 or K_pages.shape[1] != page_size or tuple(K_pages.shape[2:]) != (Gk, Dh) \
            or K_pages.shape != V_pages.shape:
        raise KascadeError(f"pages must be [num_pages,{page_size},{Gk},{Dh}]")
    for w, name in ((q_norm_weight, "q_norm_weight"), (k_norm_weight, "k_norm_weight")):
        if w is not None:
            _req(w, dt, name)
            if w.numel() != Dh:
                raise KascadeError(f"{name} must have {Dh} elements")
    if out is None:
        out = torch.empty(B, n, Hq, Dh, device=q_in.device, dtype=dt)
    else:
        _req(out, dt, "out")
        if tuple(out.shape) != (B, n, Hq, Dh):
            raise KascadeError("out must be [B,n,H,D]")
    qs, ks = _blhd_strides(q_in, "q_in"), _blhd_strides(k_in, "k_in")
    _lib.check(_call(lib, "rope_append_paged", shape,
        _ptr(q_in), ctypes.byref(qs), _ptr(k_in), _ptr(v_in), ctypes.byref(ks), _ptr(cos_sin), cos_sin.shape[0],
        _ptr(q_norm_weight), _ptr(k_norm_weight), float(norm_eps), _ptr(start_pos), int(pos_offset),
        _ptr(out), _ptr(K_pages), _ptr(V_pages), _ptr(block_table), block_table.shape[1], page_size,
        B, n, _stream()))
    return out


# ------------------------------------------- chunked prefill over the paged cache
def _chunk_args(Q, K_pages, block_table, q_start: int, page_size: int, q_starts=None, q_lens=None):
    shape = _shape(Q, K_pages)
    _req(Q, shape[3], "Q", False); _req(K_pages, shape[3], "K_pages")
    _req(block_table, torch.int32, "block_table")
    if K_pages.dim() != 4 or K_pages.shape[1] != page_size:
        raise KascadeError(f"pages must be [num_pages,{page_size},G,D]")
    if q_start % TILE:
        raise KascadeError(f"q_start must be a multiple of {TILE}")
    if block_table.shape[0] != Q.shape[0]:
        raise KascadeError("block_table must have one row per sequence")
    for t, name in ((q_starts, "q_starts"), (q_lens, "q_lens")):
        if t is not None:
            _req(t, torch.int32, name)
            if t.numel() != Q.shape[0]:
                raise KascadeError(f"{name} must have one entry per sequence")
    if q_lens is not None and q_starts is None:
        raise KascadeError("q_lens comes with q_starts")
    return Q.shape[0], Q.shape[1], _blhd_strides(Q, "Q"), shape


def prefill_chunk_dense(Q, K_pages, V_pages, block_table, q_start: int, page_size: int = 16,
                        with_output: bool = True, q_starts=None, q_lens=None
                        ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Dense causal attention of a chunk's queries (global positions q_start..q_start+Lq-1) over
    cache positions [0, q_start+Lq): the chunked form of ``prefill_recomp0_kernel`` /
    ``prefill_recomp1_kernel`` (EfficientKascadeStrategy.py:78, 80).  Returns (log_sum, O);
    O is None without with_output.
    q_starts / q_lens [B] int32 (device): a batch whose sequences stand at different positions --
    sequence b's rows start at q_starts[b] (a multiple of 32, at most q_start) and the first
    q_lens[b] rows of Q are its own; rows beyond are not written."""
    lib = _lib.init()
    B, Lq, qs, shape = _chunk_args(Q, K_pages, block_table, q_start, page_size, q_starts, q_lens)
    Hq, _, Dh, dt = shape
    log_sum = torch.empty(B, Lq, Hq, device=Q.device, dtype=torch.float32)
    out = torch.empty(B, Lq, Hq, Dh, device=Q.device, dtype=dt) if with_output else None
    if with_output:
        _req(V_pages, dt, "V_pages")
        if V_pages.shape != K_pages.shape:
            raise KascadeError("K_pages and V_pages must share one shape")
    _lib.check(_call(lib, "prefill_chunk_dense", shape,
        _ptr(Q), _ptr(K_pages), _ptr(V_pages) if with_output else None, _ptr(log_sum), _ptr(out), B,
        q_start, Lq, qs, _ptr(block_table), block_table.shape[1], page_size, K_pages.shape[0],
        1 if with_output else 0, _ptr(q_starts), _ptr(q_lens), _stream()))
    return log_sum, out


def prefill_chunk_aggregate(Q, K_pages, log_sum, scores, block_table, q_start: int,
                            page_size: int = 16, fill_invalid: bool = False, q_starts=None, q_lens=None) -> None:
    """Chunked ``aggregate_kernel`` (EfficientKascadeStrategy.py:81): scores
    [B,G,ceil(Lq/32),q_start+Lq] fp16, row t valid for keys < q_start + 32 t."""
    lib = _lib.init()
    B, Lq, qs, shape = _chunk_args(Q, K_pages, block_table, q_start, page_size, q_starts, q_lens)
    Hq, Gk = shape[0], shape[1]
    _req(log_sum, torch.float32, "log_sum"); _req(scores, torch.float16, "scores")
    T = (Lq + TILE - 1) // TILE
    if tuple(scores.shape) != (B, Gk, T, q_start + Lq) or tuple(log_sum.shape) != (B, Lq, Hq):
        raise KascadeError("scores must be [B,G,ceil(Lq/32),q_start+Lq] and log_sum [B,Lq,H]")
    _lib.check(_call(lib, "prefill_chunk_aggregate", shape,
        _ptr(Q), _ptr(K_pages), _ptr(log_sum), _ptr(scores), B, q_start, Lq, qs, _ptr(block_table),
        block_table.shape[1], page_size, K_pages.shape[0], 1 if fill_invalid else 0, _ptr(q_starts),
        _ptr(q_lens), _stream()))


def translate_indices(token_idx, block_table, kv_len: int, page_size: int = 16, out=None):
    """Token positions [B, ...] -> rows of the paged cache (block_table[b, t // page] * page +
    t % page), what the chunked reuse kernel gathers from."""
    lib = _lib.init()
    _req(token_idx, torch.int32, "token_idx"); _req(block_table, torch.int32, "block_table")
    B = token_idx.shape[0]
    if out is None:
        out = torch.empty_like(token_idx)
    _lib.check(lib.kascade_translate_indices_call(
        _ptr(token_idx), _ptr(out), _ptr(block_table), B, token_idx.numel() // B,
        block_table.shape[1], page_size, kv_len, _stream()))
    return out


def prefill_chunk_reuse(Q, K_pages, V_pages, physical_rows, head_mapping, topk_percent,
                        rolling: bool, block_table, q_start: int, page_size: int = 16,
                        q_starts=None, q_lens=None, return_log_sum: bool = False):
    """Chunked ``prefill_reuse_kernel`` (EfficientKascadeStrategy.py:92, 97): physical_rows
    [B,G,ceil(Lq/32),max_topk] comes from ``translate_indices``."""
    lib = _lib.init()
    B, Lq, qs, shape = _chunk_args(Q, K_pages, block_table, q_start, page_size, q_starts, q_lens)
    Hq, Gk, Dh, dt = shape
    _req(V_pages, dt, "V_pages")
    if V_pages.shape != K_pages.shape:
        raise KascadeError("K_pages and V_pages must share one shape")
    _req(physical_rows, torch.int32, "physical_rows"); _req(head_mapping, torch.int32, "head_mapping")
    T = (Lq + TILE - 1) // TILE
    if tuple(physical_rows.shape[:3]) != (B, Gk, T) or head_mapping.numel() != Gk:
        raise KascadeError("physical_rows must be [B,G,ceil(Lq/32),max_topk] and head_mapping [G]")
    out = torch.empty(B, Lq, Hq, Dh, device=Q.device, dtype=dt)
    log_sum = torch.empty(B, Lq, Hq, device=Q.device, dtype=torch.float32) if return_log_sum else None
    _lib.check(_call(lib, "prefill_chunk_reuse", shape,
        _ptr(Q), _ptr(K_pages), _ptr(V_pages), _ptr(physical_rows), _ptr(head_mapping),
        float(topk_percent), _ptr(out), B, q_start, Lq, physical_rows.shape[-1], 1 if rolling else 0,
        qs, _ptr(block_table), block_table.shape[1], page_size, K_pages.shape[0], _ptr(q_starts),
        _ptr(q_lens), _ptr(log_sum), _stream()))
    return (out, log_sum) if return_log_sum else out


# ------------------------------------------------- benchmark / correctness glue
def prefill_full_kernel(Q, K, V, topk, tile_size=TILE, layer=0, topk_percent=10, rolling=False,
                        fill_invalid=True):
    """``full_kernel(recompute_kernel, aggregate_kernel, reuse_kernel, Q, K, V, topk, tile_size,
    layer, topk_percent)`` of recompute_kascade_gqa_prefill.py:340-361: runs an anchor layer and
    returns the three observables the reference's correctness mode compares, (O, indices, scores).
    scores holds -inf at and after each tile's start when fill_invalid is set."""
    if tile_size != TILE:
        raise KascadeError(f"tile_size must be {TILE}")
    B, L = Q.shape[:2]
    Gk = K.shape[2]
    T = (L + TILE - 1) // TILE
    if layer == 0:
        log_sum, o = prefill_recompute0(Q, K, V)
    else:
        log_sum = prefill_recompute1(Q, K)
    scores = torch.empty(B, Gk, T, L, device=Q.device, dtype=torch.float16)
    prefill_aggregate(Q, K, log_sum, scores, fill_invalid=fill_invalid)
    valid, nsel = budgets.prefill_tile_budgets(L, TILE, topk_percent, rolling, topk)
    indices = topk_indices(scores, topk,
                           valid_len=torch.tensor(valid, dtype=torch.int32, device=Q.device),
                           n_sel=torch.tensor(nsel, dtype=torch.int32, device=Q.device))
    if layer != 0:
        o = prefill_reuse(Q, K, V, indices, torch.arange(Gk, device=Q.device, dtype=torch.int32),
                          topk_percent, rolling)
    return o, indices, scores


def decode_full_kernel(Q, K, V, topk, glse, Output_partial, row_sums, scores, layer=0):
    """``full_kernel(recompute_kernel, reuse_kernel, Q, K, V, topk, glse, Output_partial, row_sums,
    scores, layer)`` of recompute_kascade_gqa_decode.py:396-402 over a contiguous cache:
    returns (O, topk_indices, aggregated scores)."""
    L = K.shape[1]
    o, agg = decode_recompute(Q, K, V, glse, Output_partial, row_sums, scores, layer)
    indices = topk_indices(agg[:, :, :L], topk, fill_value=0)
    if layer != 0:
        o = decode_reuse(Q, K, V, indices, torch.arange(K.shape[2], device=Q.device, dtype=torch.int32), glse,
                         Output_partial)
    return o, indices, agg[:, :, :L]


def decode_full_kernel_kvcache(Q, K, V, cache_seqlens, topk_percent, glse, Output_partial, row_sums, scores,
                               layer=0, block_table=None, page_size: int = 16, max_seqlen: Optional[int] = None):
    """kvcache ``full_kernel`` of recompute_kascade_gqa_decode_with_kvcache.py:368-377 over a padded
    or paged cache: anchor pass, selection over agg[:, :, :max_seqlen] with row width
    128*ceil(floor(p*max_seqlen/100)/128), per-sequence prefix budgets, and on layers > 0 the
    reuse pass with the identity head map.  max_seqlen avoids a device->host copy of the lengths."""
    if max_seqlen is None:
        max_seqlen = int(cache_seqlens.max().item())
    o, agg = decode_recompute(Q, K, V, glse, Output_partial, row_sums, scores, layer,
                              cache_seqlens=cache_seqlens, block_table=block_table, page_size=page_size,
                              kv_len=max_seqlen)
    width = budgets.decode_budget(max_seqlen, topk_percent)
    if float(topk_percent).is_integer():
        fl = (cache_seqlens.to(torch.int64) * int(topk_percent)) // 100
    else:
        fl = torch.floor(cache_seqlens.to(torch.float64) * float(topk_percent) / 100.0).to(torch.int64)
    counts = (((fl + 127) // 128) * 128).to(torch.int32)
    Gk = K.shape[-2]
    indices = topk_indices(agg[:, :, :max_seqlen], width, valid_len=cache_seqlens.repeat_interleave(Gk),
                           n_sel=counts.repeat_interleave(Gk), fill_value=0)
    if layer != 0:
        o = decode_reuse_paged(Q, K, V, cache_seqlens, indices,
                               torch.arange(Gk, device=Q.device, dtype=torch.int32), topk_percent, glse,
                               Output_partial, block_table=block_table, page_size=page_size)
    return o, indices, agg[:, :, :max_seqlen]
