"""Host side of the Kascade hot path: the ``efficient_kascade`` attention strategy.

``EfficientKascadeStrategy`` keeps the reference class's constructor, attributes,
method seams and HF registration (src/strategies/EfficientKascadeStrategy.py:16-168,
parents KascadeStrategy.py:11-16, 174-183 and Strategy.py:8-11), with the HIP
kernels of libkascade_hip.so behind the seams:

    attention_forward(module, query[B,H,Lq,D], key[B,G,Lk,D], value, mask, scaling)
        -> (attn_output[B,Lq,H,D], None)
    _prefill_recomp_forward / _prefill_reuse_forward
    _decode_recomp_forward  / _decode_reuse_forward

Differences, all inside the seams: strided [B,L,H,D] views of HF's [B,H,L,D]
tensors go to the prefill kernels as they are (no copy); the anchor's top-k is an
exact selection kernel that delivers each row's consumed prefix instead of a full
sort; the decode split count adapts to the device instead of the fixed 8.

``PagedKascadeDecoder`` is the paged-cache decode backend (block table, per
sequence lengths) with the reference's kvcache call order
(recompute_kascade_gqa_decode_with_kvcache.py:368-377).  ``PagedKascadePrefill`` is
the chunked-prefill backend over the same paged cache.
"""
from __future__ import annotations

import math
import os
from pathlib import Path
from typing import List, Optional, Sequence

import numpy as np
import torch

from . import budgets, kernels
from ._lib import KascadeError

H, G, D, TILE = 32, 8, 128, 32
FUSED_MERGE_MAX_SPLITS = 32
ANCHOR_ROWS_PER_SPLIT = 8192


def get_head_mapping(model_name: str, recompute_layers: Sequence[int],
                     search_dirs: Optional[Sequence[os.PathLike]] = None) -> List[List[int]]:
    """int32 [num_layers][G] head maps (KascadeStrategy.py:174-183).  Looked up as
    ``{basename}_layers_{a_b_c}.npy`` in ./results/head_mappings (the reference's cwd-relative
    location) and then in the package's own head_mappings directory."""
    base = model_name.split("/")[-1]
    fname = f"{base}_layers_{'_'.join(map(str, recompute_layers))}.npy"
    dirs = list(search_dirs or []) + [Path("./results/head_mappings"),
                                      Path(__file__).resolve().parent / "head_mappings"]
    for d in dirs:
        path = Path(d) / fname
        if path.exists():
            return np.load(path, allow_pickle=False).tolist()
    raise ValueError(f"Head mapping file not found for model {model_name} with layers {list(recompute_layers)}.")


def _head_map_tensor(row, groups: int, layer, device) -> torch.Tensor:
    """One layer's head map as a device tensor: one entry per KV head, each naming a KV head."""
    row = [int(x) for x in row]
    if len(row) != groups:
        raise KascadeError(f"head mapping of layer {layer} has {len(row)} entries for {groups} KV heads")
    if any(x < 0 or x >= groups for x in row):
        raise KascadeError(f"head mapping of layer {layer} names a KV head outside 0..{groups - 1}")
    return torch.tensor(row, device=device, dtype=torch.int32)


class EfficientKascadeStrategy:
    """Drop-in for the reference's EfficientKascadeStrategy (name ``efficient_kascade``)."""

    WHOLE_PROMPT_SCORES = 65536   # prompts up to this length pool their tile scores in one tensor
    SCORE_CHUNK_TILES = 512       # longer ones this many query tiles (16384 queries) at a time

    def __init__(self, recompute_layers: List[int], model_name: Optional[str], k=1, tile_size=1,
                 rolling_prefill=False, block_size=12288, head_mapping: Optional[List[List[int]]] = None,
                 register: bool = True):
        if recompute_layers is None:
            raise ValueError("recompute_layers cannot be None for KascadeStrategy")
        if not (0 <= k <= 100):
            raise ValueError(f"Invalid k: {k}. It should be between 0 and 100%.")
        if tile_size != TILE:
            raise KascadeError(f"the kernels are specialised to tile_size={TILE}, got {tile_size}")
        if 0 not in recompute_layers:
            raise KascadeError("layer 0 must be a recompute (anchor) layer for the efficient path")
        self.name = "efficient_kascade"
        self.k = k
        self.tile_size = tile_size
        self.rolling_prefill = rolling_prefill
        self.recompute_layers = list(recompute_layers)
        self._block_size = block_size
        self._head_mapping = head_mapping if head_mapping is not None else \
            get_head_mapping(model_name, self.recompute_layers)
        self._heads, self._dim, self._groups = H, D, G
        self._topk_to_reuse = None
        self._hm_cache = {}
        self._budget_cache = {}
        if register:
            self.register_attention()

    # ------------------------------------------------------------------ helpers
    def _hm(self, layer, device, groups: int = G) -> torch.Tensor:
        key = (layer, str(device), groups)
        if key not in self._hm_cache:
            row = list(range(groups)) if layer is None else self._head_mapping[layer]
            self._hm_cache[key] = _head_map_tensor(row, groups, layer, device)
        return self._hm_cache[key]

    def _tile_budgets(self, L, width, device):
        key = (L, width, self.rolling_prefill, float(self.k), str(device))
        if key not in self._budget_cache:
            valid, nsel = budgets.prefill_tile_budgets(L, self.tile_size, self.k, self.rolling_prefill, width)
            self._budget_cache[key] = (torch.tensor(valid, device=device, dtype=torch.int32),
                                       torch.tensor(nsel, device=device, dtype=torch.int32))
        return self._budget_cache[key]

    # ------------------------------------------------------------------ prefill
    def _prefill_recomp_forward(self, Q, K, V, topk, tile_size, layer, topk_percent):
        """Anchor prefill (EfficientKascadeStrategy.py:72-93): log-sum pass (+ dense output on
        layer 0), pooled tile scores, per-tile selection, and on layers > 0 the sparse pass with
        the fresh indices and the identity head map."""
        B, L = Q.shape[:2]
        G = K.shape[2]                      # KV heads of this model (8 for the reference's shape)
        T = math.ceil(L / tile_size)
        if layer == 0:
            log_sum, o = kernels.prefill_recompute0(Q, K, V)
        else:
            log_sum = kernels.prefill_recompute1(Q, K)
        valid, nsel = self._tile_budgets(L, topk, Q.device)
        if L <= self.WHOLE_PROMPT_SCORES:
            scores = torch.empty((B, G, T, L), device=Q.device, dtype=torch.float16)
            kernels.prefill_aggregate(Q, K, log_sum, scores)
            self._topk_to_reuse = kernels.topk_indices(scores, topk, valid_len=valid, n_sel=nsel)
        else:
            # Long prompts: pool and select SCORE_CHUNK_TILES tiles at a time.  The whole score
            # tensor would take L^2/4 bytes (8 GiB at 131072 tokens), and rows beyond 65536 entries
            # go to the multi-workgroup selection, which takes a few thousand rows per call.  The
            # reference keeps the whole tensor and chunks its torch.topk by rows above 131072
            # tokens (EfficientKascadeStrategy.py:83-90); the indices are the same.
            idx = torch.empty((B, G, T, topk), device=Q.device, dtype=torch.int32)
            step = max(32, self.SCORE_CHUNK_TILES // B)
            buf = torch.empty(B * G * step * L, device=Q.device, dtype=torch.float16)
            for t0 in range(0, T, step):
                t1 = min(t0 + step, T)
                s, e = t0 * tile_size, min(t1 * tile_size, L)
                scores = buf[:B * G * (t1 - t0) * e].view(B, G, t1 - t0, e)
                kernels.prefill_aggregate_range(Q, K, log_sum, scores, s, e - s)
                idx[:, :, t0:t1] = kernels.topk_indices(scores, topk, valid_len=valid[t0:t1].contiguous(),
                                                        n_sel=nsel[t0:t1].contiguous(), fill_value=L - 1)
            self._topk_to_reuse = idx
        if layer != 0:
            o = kernels.prefill_reuse(Q, K, V, self._topk_to_reuse, self._hm(None, Q.device, G), topk_percent,
                                      self.rolling_prefill)
        return o

    def _prefill_reuse_forward(self, Q, K, V, topk_percent, layer):
        """Reuse prefill (EfficientKascadeStrategy.py:95-98)."""
        if self._topk_to_reuse is None:
            raise KascadeError("reuse layer called before any anchor layer")
        return kernels.prefill_reuse(Q, K, V, self._topk_to_reuse, self._hm(layer, Q.device, K.shape[2]), topk_percent,
                                     self.rolling_prefill)

    # ------------------------------------------------------------------- decode
    def _decode_scratch(self, Q, ns):
        B, heads, dim = Q.shape
        return (torch.empty(B, heads, ns, device=Q.device, dtype=torch.float32),
                torch.empty(B, heads, ns, dim, device=Q.device, dtype=torch.float32))

    def _decode_recomp_forward(self, Q, K, V, topk, layer):
        """Anchor decode (EfficientKascadeStrategy.py:100-115) over a contiguous [B,L,G,D] cache."""
        B, L, G = K.shape[:3]
        H = Q.shape[1]
        ns = kernels.default_num_split(B * G * L, L, heads=G)
        glse, part = self._decode_scratch(Q, ns)
        row_sums = torch.empty(B, H, device=Q.device, dtype=torch.float32)
        stride = ((L + 7) // 8) * 8
        scores = torch.empty(B, H, stride, device=Q.device, dtype=torch.float32)
        o, agg = kernels.decode_recompute(Q, K, V, glse, part, row_sums, scores, layer)
        self._topk_to_reuse = kernels.topk_indices(agg[:, :, :L], topk, fill_value=0)
        if layer != 0:
            ns = kernels.default_num_split(B * G * topk, topk, cap_rows=kernels.GATHER_ROWS_PER_SPLIT, heads=G)
            glse, part = self._decode_scratch(Q, ns)
            o = kernels.decode_reuse(Q, K, V, self._topk_to_reuse, self._hm(None, Q.device, G), glse, part)
        return o

    def _decode_reuse_forward(self, Q, K, V, layer):
        """Reuse decode (EfficientKascadeStrategy.py:117-123)."""
        if self._topk_to_reuse is None:
            raise KascadeError("reuse layer called before any anchor layer")
        B, G = Q.shape[0], K.shape[2]
        topk = self._topk_to_reuse.shape[-1]
        ns = kernels.default_num_split(B * G * topk, topk, cap_rows=kernels.GATHER_ROWS_PER_SPLIT, heads=G)
        glse, part = self._decode_scratch(Q, ns)
        return kernels.decode_reuse(Q, K, V, self._topk_to_reuse, self._hm(layer, Q.device, G), glse, part)

    # --------------------------------------------------------------- HF boundary
    def attention_forward(self, module, query, key, value, attention_mask, scaling, dropout=0.0, **kwargs):
        """EfficientKascadeStrategy.py:126-161.  query [B,H,Lq,D], key/value [B,G,Lk,D]."""
        if key.shape[-2] <= 128:
            from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
            return ALL_ATTENTION_FUNCTIONS["sdpa"](module, query, key, value, attention_mask,
                                                   scaling=scaling, dropout=dropout, **kwargs)
        # the reference's kernels exist for fp16, 32 query / 8 KV heads, head_dim 128 only
        # (EfficientKascadeStrategy.py:19-21); here any model with 1 to 16 query heads per KV head,
        # head_dim 64 or 128, in fp16 or bf16
        if query.shape[1] % key.shape[1] or query.shape[1] // key.shape[1] not in kernels.GROUPS_OK \
                or query.shape[-1] not in (64, 128) or query.dtype not in (torch.float16, torch.bfloat16):
            raise KascadeError("efficient_kascade needs fp16 or bf16, 1 to 16 query heads per KV head, "
                               "head_dim 64 or 128")
        is_decode = (query.shape[2] == 1)
        Lk = key.shape[-2]
        rounded_k = budgets.topk_width(Lk, self.k)
        query = query.transpose(1, 2)   # B, L, H, D (strided view)
        key = key.transpose(1, 2)
        value = value.transpose(1, 2)
        layer = module.layer_idx
        if is_decode:
            query = query.squeeze(1).contiguous()
            # The reference copies the whole cache to [B,L,G,D] here on every step
            # (EfficientKascadeStrategy.py:149-150); the decode kernels take the strided view of
            # HF's head-major cache instead and read it in place.
            if key.stride(-1) != 1 or value.stride() != key.stride():
                key, value = key.contiguous(), value.contiguous()
            if layer in self.recompute_layers:
                o = self._decode_recomp_forward(query, key, value, rounded_k, layer)
            else:
                o = self._decode_reuse_forward(query, key, value, layer)
            o = o.unsqueeze(1)
        else:
            if query.shape[1] != Lk:
                raise KascadeError("prefill needs Lq == Lk (no cached prefix), as in the reference kernels")
            if layer in self.recompute_layers:
                o = self._prefill_recomp_forward(query, key, value, rounded_k, self.tile_size, layer, self.k)
            else:
                o = self._prefill_reuse_forward(query, key, value, self.k, layer)
        return o, None

    def register_attention(self):
        """EfficientKascadeStrategy.py:163-168."""
        from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
        from transformers.masking_utils import ALL_MASK_ATTENTION_FUNCTIONS

        def _attention_forward(module, query, key, value, attention_mask, scaling, dropout=0.0, **kwargs):
            return self.attention_forward(module, query, key, value, attention_mask, scaling,
                                          dropout=dropout, **kwargs)
        ALL_MASK_ATTENTION_FUNCTIONS.register(self.name, ALL_MASK_ATTENTION_FUNCTIONS["sdpa"])
        ALL_ATTENTION_FUNCTIONS.register(self.name, _attention_forward)


class PagedKascadeDecoder:
    """Paged decode backend: anchor and reuse decode over K/V pages [P,page,G,D] with a block
    table [B,max_pages] and per-sequence lengths.  Scratch is allocated once for a maximum
    batch / context and reused by every call (the C ABI never allocates).

    Call order per decode step follows the reference's kvcache ``full_kernel``
    (recompute_kascade_gqa_decode_with_kvcache.py:368-377): anchor -> selection over
    agg[:, :, :max_len] with row width max_topk -> (layers > 0) reuse with the identity map;
    reuse layers read rows head_mapping[layer] of the last anchor's indices."""

    def __init__(self, k: float, head_mapping: List[List[int]], recompute_layers: Sequence[int],
                 max_batch: int, max_seqlen: int, page_size: int = 16, device="cuda",
                 num_split_dense: Optional[int] = None, num_split_reuse: Optional[int] = None,
                 total_tokens: Optional[int] = None, fused_combine: bool = True,
                 seqlens_hint: Optional[Sequence[int]] = None, kv_heads: int = G, head_dim: int = D,
                 group_size: int = kernels.GROUP):
        """kv_heads, head_dim, group_size: the model's shape (query heads = group_size * kv_heads;
        the element type is that of the tensors of each call).
        fused_combine: merge the splits inside the split launch (one launch fewer per layer).
        total_tokens: expected sum of the sequence lengths of a batch (default
        max_batch*max_seqlen); with ragged batches it sizes the splits so that the non-empty
        workgroups, not the grid, cover the device about twice.
        seqlens_hint: the (approximate) lengths themselves, as a serving engine's scheduler knows
        them; then the workgroups of a ragged batch are counted exactly."""
        self.k = k
        self.page_size = page_size
        self.recompute_layers = list(recompute_layers)
        self._head_mapping = head_mapping
        self.device = torch.device(device)
        self.max_batch, self.max_seqlen = max_batch, max_seqlen
        G, D = kv_heads, head_dim            # this model's, from here on
        H = group_size * G
        self.G, self.H, self.D = G, H, D
        self.stride = ((max_seqlen + 7) // 8) * 8
        self.max_topk = budgets.decode_budget(max_seqlen, k)
        if seqlens_hint is not None and total_tokens is None:
            total_tokens = sum(seqlens_hint)
        total = total_tokens if total_tokens is not None else max_batch * max_seqlen
        dense_rows = list(seqlens_hint) if seqlens_hint is not None else None
        reuse_rows = [budgets.decode_budget(n, k) for n in seqlens_hint] if seqlens_hint is not None else None
        self.ns_dense = num_split_dense or kernels.default_num_split(G * total, max_seqlen, row_counts=dense_rows,
                                                                         heads=G)
        # A batch of equal lengths gathers fastest with one workgroup per compute unit (16 x 65536:
        # 76.9 us with 256 workgroups against 78.6 with 512; 8 x 65536: 44.0 against 45.0); ragged
        # batches want two, so that the short sequences' workgroups fill in behind the long ones.
        uniform = seqlens_hint is not None and len(set(int(n) for n in seqlens_hint)) == 1
        self.ns_reuse = num_split_reuse or kernels.default_num_split(
            G * budgets.decode_budget(total, k), self.max_topk, wgs_per_cu=1 if uniform else 2,
            cap_rows=kernels.GATHER_ROWS_PER_SPLIT, row_counts=reuse_rows, heads=G)
        # The anchor passes (which also write their score codes) run 2 % faster with twice the
        # splits where two workgroups per compute unit leave a split more than 8192 rows
        # (16 x 65536: 795 / 508 us with 8 splits against 815 / 521 with 4); dense decode does not
        # care, and beyond 32 splits the merge inside the launch would be lost.
        self.ns_anchor = self.ns_dense
        if (not num_split_dense and -(-max_seqlen // self.ns_dense) > ANCHOR_ROWS_PER_SPLIT
                and 2 * self.ns_dense <= FUSED_MERGE_MAX_SPLITS):
            self.ns_anchor = 2 * self.ns_dense
        ns = max(self.ns_dense, self.ns_reuse, self.ns_anchor)
        dev = self.device
        self._glse = torch.empty(max_batch * H * ns, device=dev, dtype=torch.float32)
        self._part = torch.empty(max_batch * H * ns * D, device=dev, dtype=torch.float32)
        self._row_sums = torch.empty(max_batch, H, device=dev, dtype=torch.float32)
        self._scores = torch.empty(max_batch * H * self.stride, device=dev, dtype=torch.float32)
        self._scratch_views = {}
        self._hm = {None: torch.arange(G, device=dev, dtype=torch.int32)}
        for l, row in enumerate(head_mapping):
            self._hm[l] = _head_map_tensor(row, G, l, dev)
        self._topk_to_reuse = None      # the last anchor's selection as token positions
        self._rows_to_reuse = None      # ... translated to cache rows, what the reuse launches gather from
        widest = max(self.max_topk, budgets.topk_width(max_seqlen, k), budgets.CHUNK)
        self._rows_buf = torch.empty(max_batch * G * widest, device=dev, dtype=torch.int32)
        self._counts = None
        self._valid_rows = torch.empty(max_batch * G, device=dev, dtype=torch.int32)
        self._nsel_rows = torch.empty(max_batch * G, device=dev, dtype=torch.int32)
        # arrival counters of the fused combine: zero now, set back to zero by every launch
        self._sync = torch.zeros(max_batch * G, device=dev, dtype=torch.int32) if fused_combine else None
        # one workgroup merges all splits of a (sequence, KV head), 16 partial outputs per trip to
        # memory: a win up to about 32 splits; beyond that the combine launch, which spreads the
        # merge over 32 workgroups per sequence, is faster
        self._sync_dense = self._sync if self.ns_dense <= FUSED_MERGE_MAX_SPLITS else None
        self._sync_anchor = self._sync if self.ns_anchor <= FUSED_MERGE_MAX_SPLITS else None
        self._sync_reuse = self._sync if self.ns_reuse <= FUSED_MERGE_MAX_SPLITS else None

    def _scratch(self, B, ns):
        H, D = self.H, self.D
        views = self._scratch_views.get((B, ns))
        if views is None:   # a view costs a microsecond or two of host time per layer call
            views = self._scratch_views[(B, ns)] = (self._glse[:B * H * ns].view(B, H, ns),
                                                    self._part[:B * H * ns * D].view(B, H, ns, D))
        return views

    def dense(self, q, k_pages, v_pages, block_table, seqlens, max_len: int, out=None,
              k_new=None, v_new=None):
        B = q.shape[0]
        glse, part = self._scratch(B, self.ns_dense)
        return kernels.decode_dense_paged(q, k_pages, v_pages, seqlens, glse, part, block_table,
                                          self.page_size, kv_len=max_len, out=out, sync=self._sync_dense,
                                          k_new=k_new, v_new=v_new)

    def begin_step(self, seqlens: torch.Tensor, advance: int = 1):
        """One launch at the start of a decode step: the lengths grow by ``advance`` in place
        (the new token, which the layer calls append themselves when handed ``k_new``/``v_new``)
        and the per-row budgets of the step's anchor layers are computed from the new lengths."""
        self._counts = (self._budget_key(seqlens),
                        *kernels.decode_budgets(seqlens, float(self.k), advance, self._valid_rows, self._nsel_rows,
                                                kv_heads=self.G))

    @staticmethod
    def _budget_key(seqlens):
        return (seqlens.data_ptr(), seqlens._version, seqlens.numel())

    def anchor(self, layer, q, k_pages, v_pages, block_table, seqlens, max_len: int,
               ragged: bool = True, out=None, k_new=None, v_new=None):
        """Anchor layer: returns the attention output [B,H,D] (written to ``out`` when given);
        keeps indices for reuse layers.  ``k_new``/``v_new`` [B,G,D]: rows of the newest token
        (position seqlens-1), appended to the cache by the anchor launch itself."""
        B = q.shape[0]
        G, H = self.G, self.H
        stride = ((max_len + 7) // 8) * 8
        glse, part = self._scratch(B, self.ns_anchor)
        scores = self._scores[:B * H * stride].view(B, H, stride)
        o, agg = kernels.decode_recompute(q, k_pages, v_pages, glse, part, self._row_sums[:B], scores, layer,
                                          cache_seqlens=seqlens, block_table=block_table,
                                          page_size=self.page_size, kv_len=max_len, out=out, sync=self._sync_anchor,
                                          k_new=k_new, v_new=v_new)
        if ragged:
            width = budgets.decode_budget(max_len, self.k)
            lens_rows, counts = self._row_budgets(seqlens)
        else:
            width = budgets.topk_width(max_len, self.k)
            lens_rows = counts = None
        # One translation per anchor, inside the selection launch: every reuse launch up to the
        # next anchor reads the same block table, so the selection also leaves its lists as cache
        # rows and the gathers skip the table.
        self._topk_to_reuse, self._rows_to_reuse = kernels.topk_indices(
            agg[:, :, :max_len], width, valid_len=lens_rows, n_sel=counts, fill_value=0,
            block_table=block_table, page_size=self.page_size,
            rows_out=self._rows_buf[:B * G * width].view(B, G, width))
        self._pct = float(self.k) if ragged else 0.0
        if layer != 0:
            o = self._reuse(q, k_pages, v_pages, block_table, seqlens, self._hm[None], out)
        return o

    def _row_budgets(self, seqlens: torch.Tensor):
        """Per (sequence, KV head) row: valid length and selection count.  The anchors of one
        decode step see the same lengths, so the tensors are kept until seqlens is written again
        (a dozen tiny launches otherwise, as long as an anchor pass at short contexts)."""
        key = self._budget_key(seqlens)
        if self._counts is None or self._counts[0] != key:
            self._counts = (key, *kernels.decode_budgets(seqlens, float(self.k), 0, self._valid_rows,
                                                         self._nsel_rows, kv_heads=self.G))
        return self._counts[1], self._counts[2]

    def _reuse(self, q, k_pages, v_pages, block_table, seqlens, hm, out=None, k_new=None, v_new=None):
        B = q.shape[0]
        glse, part = self._scratch(B, self.ns_reuse)
        return kernels.decode_reuse_rows(q, k_pages, v_pages, seqlens, self._rows_to_reuse, hm, self._pct,
                                         glse, part, block_table, page_size=self.page_size, out=out,
                                         sync=self._sync_reuse, k_new=k_new, v_new=v_new)

    def reuse(self, layer, q, k_pages, v_pages, block_table, seqlens, out=None, k_new=None, v_new=None):
        """Reuse layer: attends to rows head_mapping[layer] of the last anchor's indices."""
        if self._topk_to_reuse is None:
            raise KascadeError("reuse layer called before any anchor layer")
        return self._reuse(q, k_pages, v_pages, block_table, seqlens, self._hm[layer], out, k_new, v_new)

    def forward(self, layer, q, k_pages, v_pages, block_table, seqlens, max_len: int, ragged: bool = True,
                out=None, k_new=None, v_new=None):
        if layer in self.recompute_layers:
            return self.anchor(layer, q, k_pages, v_pages, block_table, seqlens, max_len, ragged, out,
                               k_new, v_new)
        return self.reuse(layer, q, k_pages, v_pages, block_table, seqlens, out, k_new, v_new)


class PagedKascadePrefill:
    """Chunked prefill backend over the paged cache: a prompt arrives in 32-aligned chunks, each
    chunk's K/V are appended to the cache (``kernels.paged_kv_append``) and its queries then
    attend to every cached position.  Per chunk the layer sequence is the reference's prefill
    sequence (EfficientKascadeStrategy.py:72-98): an anchor layer runs the log-sum pass (dense
    output on layer 0), pools tile scores, selects each tile's top-k and, on layers > 0, runs
    its own sparse pass with the identity head map; reuse layers gather rows
    head_mapping[layer] of the last anchor's indices.  A prompt processed this way gives the
    rows a whole-prompt call gives."""

    def __init__(self, k: float, head_mapping: List[List[int]], recompute_layers: Sequence[int],
                 page_size: int = 16, rolling_prefill: bool = True, device="cuda", kv_heads: int = G):
        self.k = k
        self.page_size = page_size
        self.rolling_prefill = rolling_prefill
        self.recompute_layers = list(recompute_layers)
        self.device = torch.device(device)
        self.G = kv_heads
        self._hm = {None: torch.arange(kv_heads, device=self.device, dtype=torch.int32)}
        for l, row in enumerate(head_mapping):
            self._hm[l] = _head_map_tensor(row, kv_heads, l, self.device)
        self._rows_to_reuse = None      # physical rows [B,G,T,width] of the last anchor
        self._topk_to_reuse = None      # the same selection as token positions
        self._budget_cache = {}
        self._geom_cache = {}
        self._scores = None

    def _tile_budgets(self, q_start: int, Lq: int, width: int):
        key = (q_start, Lq, width)
        hit = self._budget_cache.get(key)
        if hit is None:
            Lk = q_start + Lq
            T = (Lq + TILE - 1) // TILE
            valid = [q_start + TILE * t for t in range(T)]
            if self.rolling_prefill and Lk > budgets.CHUNK:
                nsel = [min(budgets.rolling_budget(s, self.k), width) for s in valid]
            else:
                nsel = [width] * T
            hit = (torch.tensor(valid, dtype=torch.int32, device=self.device),
                   torch.tensor(nsel, dtype=torch.int32, device=self.device))
            self._budget_cache[key] = hit
        return hit

    def _geometry(self, q_start, q_lens, Lq: int):
        """Where the rows of a call stand.  q_start: one int for the whole batch, or one per
        sequence (the scheduler's view: host ints, multiples of 32); q_lens: how many of the Lq
        rows belong to each sequence (default all).  Returns (largest start, device starts,
        device lengths, host starts, host lengths); the device tensors are None for a uniform batch."""
        if isinstance(q_start, int) and q_lens is None:
            return q_start, None, None, None, None
        starts = [int(q_start)] * len(q_lens) if isinstance(q_start, int) else [int(x) for x in q_start]
        lens = [Lq] * len(starts) if q_lens is None else [int(x) for x in q_lens]
        if len(lens) != len(starts) or any(x % TILE or x < 0 for x in starts) or any(n < 0 or n > Lq for n in lens):
            raise KascadeError("per-sequence chunk starts must be multiples of 32 and lengths within the rows of Q")
        key = (tuple(starts), tuple(lens))
        hit = self._geom_cache.get(key)
        if hit is None:
            if len(self._geom_cache) > 64:
                self._geom_cache.clear()
            hit = (torch.tensor(starts, dtype=torch.int32, device=self.device),
                   torch.tensor(lens, dtype=torch.int32, device=self.device))
            self._geom_cache[key] = hit
        return max(starts), hit[0], hit[1], starts, lens

    def _ragged_budgets(self, starts, lens, Lq: int, width: int):
        """(valid_len, n_sel) per (sequence, KV head, tile) row of the pooled scores of a mixed
        batch: every sequence gets the budgets of a call of its own."""
        key = (tuple(starts), tuple(lens), Lq, width)
        hit = self._budget_cache.get(key)
        if hit is None:
            T = (Lq + TILE - 1) // TILE
            valid, nsel = [], []
            for s, n in zip(starts, lens):
                Lk = s + n
                own = min(width, budgets.topk_width(Lk, self.k)) if Lk > 0 else 0
                v_row, n_row = [], []
                for t in range(T):
                    if TILE * t >= n:                      # a tile past the sequence's rows selects nothing
                        v_row.append(0); n_row.append(0)
                        continue
                    v_row.append(s + TILE * t)
                    roll = self.rolling_prefill and Lk > budgets.CHUNK
                    n_row.append(min(budgets.rolling_budget(s + TILE * t, self.k), own) if roll else own)
                valid += v_row * self.G
                nsel += n_row * self.G
            if len(self._budget_cache) > 64:
                self._budget_cache.clear()
            hit = (torch.tensor(valid, dtype=torch.int32, device=self.device),
                   torch.tensor(nsel, dtype=torch.int32, device=self.device))
            self._budget_cache[key] = hit
        return hit

    def _score_buffer(self, B, T, Lk):
        G = self.G
        n = B * G * T * Lk
        if self._scores is None or self._scores.numel() < n:
            self._scores = torch.empty(n, device=self.device, dtype=torch.float16)
        return self._scores[:n].view(B, G, T, Lk)

    def anchor(self, layer, q, k_pages, v_pages, block_table, q_start, q_lens=None):
        B, Lq = q.shape[:2]
        qs_max, qs_dev, ql_dev, starts, lens = self._geometry(q_start, q_lens, Lq)
        Lk = qs_max + Lq
        T = (Lq + TILE - 1) // TILE
        width = budgets.topk_width(Lk, self.k)
        log_sum, o = kernels.prefill_chunk_dense(q, k_pages, v_pages, block_table, qs_max,
                                                 self.page_size, with_output=(layer == 0),
                                                 q_starts=qs_dev, q_lens=ql_dev)
        scores = self._score_buffer(B, T, Lk)
        kernels.prefill_chunk_aggregate(q, k_pages, log_sum, scores, block_table, qs_max, self.page_size,
                                        q_starts=qs_dev, q_lens=ql_dev)
        if qs_dev is None:
            valid, nsel = self._tile_budgets(qs_max, Lq, width)
        else:
            valid, nsel = self._ragged_budgets(starts, lens, Lq, width)
        self._topk_to_reuse, self._rows_to_reuse = kernels.topk_indices(
            scores, width, valid_len=valid, n_sel=nsel, block_table=block_table, page_size=self.page_size)
        if layer != 0:
            o = self._reuse(q, k_pages, v_pages, block_table, qs_max, self._hm[None], qs_dev, ql_dev)
        return o

    def _reuse(self, q, k_pages, v_pages, block_table, q_start, hm, q_starts=None, q_lens=None):
        return kernels.prefill_chunk_reuse(q, k_pages, v_pages, self._rows_to_reuse, hm, float(self.k),
                                           self.rolling_prefill, block_table, q_start, self.page_size,
                                           q_starts=q_starts, q_lens=q_lens)

    def reuse(self, layer, q, k_pages, v_pages, block_table, q_start, q_lens=None):
        if self._rows_to_reuse is None:
            raise KascadeError("reuse layer called before any anchor layer")
        qs_max, qs_dev, ql_dev, _, _ = self._geometry(q_start, q_lens, q.shape[1])
        return self._reuse(q, k_pages, v_pages, block_table, qs_max, self._hm[layer], qs_dev, ql_dev)

    def dense(self, q, k_pages, v_pages, block_table, q_start, q_lens=None):
        qs_max, qs_dev, ql_dev, _, _ = self._geometry(q_start, q_lens, q.shape[1])
        return kernels.prefill_chunk_dense(q, k_pages, v_pages, block_table, qs_max, self.page_size,
                                           q_starts=qs_dev, q_lens=ql_dev)[1]

    def forward(self, layer, q, k_pages, v_pages, block_table, q_start, q_lens=None):
        """q [B,Lq,H,D] at global positions q_start.. (K/V of the chunk already in the cache).
        q_start: one int, or one per sequence; q_lens: rows of q that belong to each sequence."""
        if layer in self.recompute_layers:
            return self.anchor(layer, q, k_pages, v_pages, block_table, q_start, q_lens)
        return self.reuse(layer, q, k_pages, v_pages, block_table, q_start, q_lens)
