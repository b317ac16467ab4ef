"""Attention layer with the reference's interface (layers/attention/attention_v4.py:21-52, 316-410)
running on the HIP operators: `Attention(num_heads, head_dim, scale, num_kv_heads,
model_type).forward(q, k, v)` reads the thread-local ContextForDiffusionLM, stores K/V into the
paged cache through the slot mapping, and attends

  * prefill: every sequence of the packed batch to itself (block-diagonal; full, causal or the
    dense block mask of the context) -- attention_v4.py:336-367;
  * decode: the active rows to [visible prefix pages || active rows] without the dense
    load_kvcache staging copy -- attention_v4.py:368-397.

The experimental corrections of the reference (default off) are here too: the decode delta
(attention_v4.py:86-166: anchors re-attend to the full prompt, the difference is spread over their
neighbours) and the sparse prefill with its anchor delta (attention_v4.py:168-293).  The denser
attention is computed for every row and read at the anchors."""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Optional

import torch
from torch import nn

from . import ops
from .context import ContextForDiffusionLM, get_context_diffusion_lm


class Attention(nn.Module):
    def __init__(self, num_heads, head_dim, scale, num_kv_heads, model_type="diffusion_lm"):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.scale = scale
        self.num_kv_heads = num_kv_heads
        self.k_cache = self.v_cache = torch.tensor([])
        self.model_type = model_type
        if model_type != "diffusion_lm":
            raise NotImplementedError("the causal-LM branch of the reference layer is not part of this build")
        # the reference switches flex / sdpa here (attention_v4.py:38); this layer is the third value
        self.attention_backend = os.environ.get("PREFILLING_DLLM_ENGINE_ATTENTION_BACKEND", "hip").lower()
        self.layer_idx = -1

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask=None) -> torch.Tensor:
        q = q.view(-1, self.num_heads, self.head_dim)
        k = k.view(-1, self.num_kv_heads, self.head_dim)
        v = v.view(-1, self.num_kv_heads, self.head_dim)
        context: ContextForDiffusionLM = get_context_diffusion_lm()
        if context.kv_cache_layout != "unified":
            raise NotImplementedError("only kv_cache_layout='unified' is supported")
        k_cache, v_cache = self.k_cache, self.v_cache
        has_cache = k_cache.numel() > 0 and v_cache.numel() > 0

        # A decode step over a cached prefix stores its active rows inside the attention call (their slots lie
        # behind the context the same call reads, ENG:497); every other case stores first, as the reference does.
        max_ctx = 0 if context.is_prefill else int(context.max_context_len) or max(int(context.max_seqlen_k) - 1, 0)
        # (precondition: no active slot lies inside a visible prefix range; `context.store_before_attention`
        # restores the reference's order for callers that break it, PDLLM_DEBUG_CHECKS=1 verifies it on the host)
        store_in_call = (has_cache and context.need_kv_cache_store and not context.is_prefill and max_ctx > 0
                         and context.slot_mapping is not None and not context.store_before_attention)
        if store_in_call and os.environ.get("PDLLM_DEBUG_CHECKS", "0") == "1":
            self._check_store_after_attention(context, k_cache.shape[1])
        if has_cache and context.need_kv_cache_store and not store_in_call:
            ops.store_kvcache_unified_layout(k, v, k_cache, v_cache, context.slot_mapping, self.model_type, context)

        mask_mode, dense = context.mask_kind, None
        if context.block_mask is not None:
            mask_mode, dense = "dense", context.block_mask
            if dense.dim() != 2 or dense.shape[0] != q.shape[0]:
                raise ValueError(f"block_mask must be [rows, keys] with one row per active token, got {tuple(dense.shape)}")
            if dense.shape[1] != q.shape[0]:
                # the reference's decode form [Nq, sum(ctx + Sq)] (utils/context.py:85-98): keep the active columns
                # (reduced once per context, not once per layer: every layer of a step passes the same mask)
                held = getattr(context, "_active_mask_of", None)
                if held is None or held[0] is not dense:
                    held = (dense, self._active_columns(dense, context))
                    context._active_mask_of = held
                dense = held[1]
                if dense is None:          # nothing hidden: the bidirectional block needs no mask tensor
                    mask_mode = "full"
        if context.is_prefill:
            o = self._maybe_prefill_sparse_attention(q, k, v, context)
            if o is not None:
                pass
            elif mask_mode == "dense":
                o = ops.sparse_decode_attention(q, k, v, None, None, None, context.cu_seqlens_q,
                                                max_q_len=int(context.max_seqlen_q), max_ctx_len=0,
                                                mask_mode="dense", mask=dense, sm_scale=self.scale)
            else:
                o = ops.chunk_prefill_attention(q, k, v, context.cu_seqlens_q, max_seqlen=int(context.max_seqlen_q),
                                                causal=(mask_mode == "causal"), sm_scale=self.scale)
        else:
            o = ops.sparse_decode_attention(q, k, v, k_cache if has_cache else None, v_cache if has_cache else None,
                                            context.block_tables, context.cu_seqlens_q,
                                            max_q_len=int(context.max_seqlen_q), max_ctx_len=max_ctx if has_cache else 0,
                                            context_lens=context.context_lens, ranges=context.ranges,
                                            mask_mode=mask_mode, mask=dense, sm_scale=self.scale,
                                            active_slot_mapping=context.slot_mapping if store_in_call else None)
            o = self._maybe_apply_decode_delta(o, q, k, v, context, mask_mode, dense)
        return o.view(-1, self.num_heads * self.head_dim)

    @staticmethod
    def _check_store_after_attention(context: ContextForDiffusionLM, page_size: int) -> None:
        """Debug check of the in-call store's precondition: no slot that receives an active row is the slot of a
        visible prefix key of the same call (host-side, synchronises)."""
        slots = context.slot_mapping[context.slot_mapping >= 0].long()
        if slots.numel() == 0 or context.block_tables is None:
            return
        if context.ranges is not None:
            ptr, start, length = (t.tolist() for t in context.ranges[:3])
            spans = [[(start[i], length[i]) for i in range(ptr[r], ptr[r + 1])] for r in range(len(ptr) - 1)]
        else:
            spans = [[(0, int(n))] for n in context.context_lens.tolist()]
        for r, req_spans in enumerate(spans):
            table = context.block_tables[r].long()
            for first, n in req_spans:
                if n <= 0:
                    continue
                tok = torch.arange(first, first + n, device=slots.device)
                visible = table[tok // page_size] * page_size + tok % page_size
                if torch.isin(visible, slots).any().item():
                    raise RuntimeError("an active row's slot lies inside a visible prefix range: set "
                                       "context.store_before_attention to store in front of the attention")

    @staticmethod
    def _active_columns(mask: torch.Tensor, context: ContextForDiffusionLM):
        """[Nq, sum(ctx_s + Sq_s)] block-diagonal decode mask of the reference -> [Nq, Nq] over the active keys
        (None when no active key is hidden)."""
        from .context import active_block_mask
        if context.is_prefill or context.context_lens is None or context.cu_seqlens_q is None:
            raise ValueError(f"block_mask of shape {tuple(mask.shape)} does not match {mask.shape[0]} active rows")
        # (the context's host-side lengths when it carries them: no transfer)
        if context.seq_lens is not None and len(context.seq_lens) == context.context_lens.numel():
            cu = [0]
            for n in context.seq_lens:
                cu.append(cu[-1] + int(n))
        else:
            cu = [int(x) for x in context.cu_seqlens_q.tolist()]
        ctx = [int(x) for x in context.context_lens.tolist()]
        if mask.shape[1] != sum(ctx) + cu[-1]:
            raise ValueError(f"block_mask has {mask.shape[1]} key columns, expected {cu[-1]} (active) or "
                             f"{sum(ctx) + cu[-1]} (contexts + active)")
        parts, col = [], 0
        for s, c in enumerate(ctx):
            h = cu[s + 1] - cu[s]
            parts.append(mask[cu[s]:cu[s + 1], col:col + c + h])
            col += c + h
        return active_block_mask(parts)

    # ---- experimental corrections (default off) ----

    @staticmethod
    def _debug_stats(state, delta_abs_max: float, n_anchors: int) -> None:
        state["calls"] = int(state.get("calls", 0)) + 1
        state["nonzero_calls"] = int(state.get("nonzero_calls", 0)) + int(delta_abs_max > 0.0)
        state["max_abs"] = max(float(state.get("max_abs", 0.0)), delta_abs_max)
        state["anchor_count"] = int(state.get("anchor_count", 0)) + n_anchors

    def _paged_prompt(self, state, full_k, full_v, extra: int):
        """The layer's full prompt K/V [S, Hkv, d] as pages of a cache of its own (where the reference concatenates,
        attention_v4.py:120-125) with room for `extra` more tokens.  The copy lives in the state between steps and
        is tied to the prompt tensor *objects* it was made from (the entry holds them, so their storage cannot be
        freed and handed to another tensor while the copy is in use) and to their version counters, so an in-place
        update of the prompt tensors makes a new copy.  Tensors made under torch.inference_mode() -- the reference
        builds full_k / full_v there (fastdllm_engine.py:656-662) -- have no version counter: a caller that
        rewrites those in place bumps `state["prompt_generation"]`.  The copy doubles the prompt K/V of the layer in
        device memory for as long as the state lives."""
        page, n_prompt = 256, int(full_k.shape[0])
        pages = (n_prompt + extra + page - 1) // page
        def version(t):
            try:
                return t._version
            except RuntimeError:      # inference tensors do not track a version counter
                return -1
        generation = (state.get("prompt_generation", 0), version(full_k), version(full_v))
        held = state.setdefault("_paged_prompt", {})
        ent = held.get(self.layer_idx)
        fresh = (ent is not None and ent["k"] is full_k and ent["v"] is full_v and ent["n"] == n_prompt
                 and ent["generation"] == generation and ent["kc"].shape[0] >= pages)
        if not fresh:
            kc = torch.empty((pages, page, self.num_kv_heads, self.head_dim), dtype=full_k.dtype, device=full_k.device)
            vc = torch.empty_like(kc)
            kc.view(-1, self.num_kv_heads, self.head_dim)[:n_prompt].copy_(full_k)
            vc.view(-1, self.num_kv_heads, self.head_dim)[:n_prompt].copy_(full_v)
            ent = {"k": full_k, "v": full_v, "n": n_prompt, "generation": generation, "kc": kc, "vc": vc}
            held[self.layer_idx] = ent
        return ent["kc"], ent["vc"]

    def _maybe_apply_decode_delta(self, o, q, k_new, v_new, context, mask_mode="full", active_mask=None):
        """attention_v4.py:86-166.  The packed active rows are one sequence, as in the reference; active_mask is the
        [Nq, Nq] mask over the active keys (attention_v4.py:131-133 takes those columns of the block mask)."""
        state = getattr(context, "decode_delta_state", None)
        if not state or not state.get("enabled", False) or self.layer_idx < 0:
            return o
        full_k_by_layer, full_v_by_layer = state.get("full_k"), state.get("full_v")
        if full_k_by_layer is None or full_v_by_layer is None or self.layer_idx >= len(full_k_by_layer):
            return o
        full_k, full_v = full_k_by_layer[self.layer_idx], full_v_by_layer[self.layer_idx]
        if full_k is None or full_v is None or full_k.numel() == 0:
            return o
        seq_len = q.shape[0]
        ap = ops.anchor_params(state, seq_len)
        if ap is None:
            return o
        stride, offset, left, right, direction = ap
        dev = q.device
        n_prompt = int(full_k.shape[0])
        anchors = torch.arange(offset, seq_len, stride, device=dev)
        n_a = int(anchors.numel())
        if mask_mode == "full" and active_mask is None and 0 < n_a < seq_len:
            # Only the anchor rows are attended, as in the reference (attention_v4.py:127): the active K/V rows are
            # appended to the paged copy of the prompt, so that every key is a prefix key and the anchors are a
            # compact batch of queries whose own "active" keys are all masked.
            kc, vc = self._paged_prompt(state, full_k, full_v, seq_len)
            kc.view(-1, self.num_kv_heads, self.head_dim)[n_prompt:n_prompt + seq_len].copy_(k_new)
            vc.view(-1, self.num_kv_heads, self.head_dim)[n_prompt:n_prompt + seq_len].copy_(v_new)
            n_keys = n_prompt + seq_len
            dense_a = ops.sparse_decode_attention(
                q.index_select(0, anchors), k_new.index_select(0, anchors), v_new.index_select(0, anchors), kc, vc,
                torch.arange(kc.shape[0], dtype=torch.int32, device=dev).view(1, -1),
                torch.tensor([0, n_a], dtype=torch.int32, device=dev), max_q_len=n_a, max_ctx_len=n_keys,
                context_lens=torch.tensor([n_keys], dtype=torch.int32, device=dev), mask_mode="dense",
                mask=torch.zeros((n_a, n_a), dtype=torch.bool, device=dev), sm_scale=self.scale)
            dense = torch.empty_like(o)   # only the anchor rows are read below
            dense.index_copy_(0, anchors, dense_a)
        else:
            # a mask over the active keys applies to keys, not to rows: every active row goes through the kernel
            kc, vc = self._paged_prompt(state, full_k, full_v, 0)
            dense = ops.sparse_decode_attention(q, k_new, v_new, kc, vc,
                                                torch.arange(kc.shape[0], dtype=torch.int32, device=dev).view(1, -1),
                                                torch.tensor([0, seq_len], dtype=torch.int32, device=dev),
                                                max_q_len=seq_len, max_ctx_len=n_prompt,
                                                context_lens=torch.tensor([n_prompt], dtype=torch.int32, device=dev),
                                                mask_mode=mask_mode, mask=active_mask, sm_scale=self.scale)
        one_seq = torch.tensor([0, seq_len], dtype=torch.int32, device=dev)
        scale = float(state.get("scale", 1.0))
        if state.get("debug", False):
            delta = (dense.index_select(0, anchors) - o.index_select(0, anchors)) * scale
            self._debug_stats(state, float(delta.abs().max().item()) if delta.numel() else 0.0, int(anchors.numel()))
        return ops.anchor_delta_add(o, dense, one_seq, max_q_len=seq_len, stride=stride, anchor_offset=offset,
                                    left=left, right=right, direction=direction, scale=scale)

    def _maybe_prefill_sparse_attention(self, q, k, v, context):
        """attention_v4.py:168-293.  None = not active, the caller runs the ordinary prefill."""
        if self.model_type != "diffusion_lm":
            return None
        state = getattr(context, "prefill_sparse_state", None)
        plan = _SparsePrefill.parse(state, self.layer_idx, q.shape[0], self.num_heads, context.block_mask, q.device,
                                    q.dtype)
        if plan is None:
            return None
        seq_len = q.shape[0]
        one_seq = torch.tensor([0, seq_len], dtype=torch.int32, device=q.device)

        def attend(mask):
            return ops.sparse_decode_attention(q, k, v, None, None, None, one_seq, max_q_len=seq_len, max_ctx_len=0,
                                               mask_mode="dense", mask=mask, sm_scale=self.scale)

        if plan.debug:
            n_keys = int(plan.keys.sum().item())
            state["union_min"] = min(int(state.get("union_min", n_keys)), n_keys)
            state["union_max"] = max(int(state.get("union_max", n_keys)), n_keys)
        o_sparse = attend(plan.rows_mask & plan.keys.unsqueeze(0))
        if plan.anchor is None:            # no correction asked for, or no anchor row in this sequence
            return o_sparse
        stride, offset, left, right, direction = plan.anchor
        kw = dict(max_q_len=seq_len, stride=stride, anchor_offset=offset, left=left, right=right, direction=direction,
                  scale=plan.scale)
        anchors = torch.arange(offset, seq_len, stride, device=q.device)

        if plan.mode == "replace":
            # the selection's rows stand in for the dense attention of the anchors; without a usable row: no correction
            if plan.sel is None or not plan.selection_covers(anchors):
                return o_sparse
            out = ops.anchor_delta_add(o_sparse, None, one_seq, sel=plan.sel, sel_counts=plan.sel_counts,
                                       sel_mode="replace", **kw)
            state["selection_used_calls"] = int(state.get("selection_used_calls", 0)) + 1
        elif plan.mode == "add" and plan.sel is not None:
            out = ops.anchor_delta_add(o_sparse, attend(plan.rows_mask), one_seq, sel=plan.sel,
                                       sel_counts=plan.sel_counts, sel_mode="add", sel_scale=plan.sel_scale, **kw)
            state["selection_used_calls"] = int(state.get("selection_used_calls", 0)) + 1
        else:
            out = ops.anchor_delta_add(o_sparse, attend(plan.rows_mask), one_seq, **kw)
        if plan.debug:
            # largest |out - o_sparse| over the anchor rows stands in for the reference's max |delta|
            diff = (out.index_select(0, anchors).float() - o_sparse.index_select(0, anchors).float()).abs()
            self._debug_stats(state, float(diff.max().item()) if diff.numel() else 0.0, int(anchors.numel()))
        return out


_DELTA_OFF = frozenset({"none", "off", "0", ""})
_DELTA_ON = frozenset({"s4_left3", "delta_s4_left3", "sampled_delta_s4_left3"})
_SELECTION_MODES = {"selection_dense_replace": "replace", "selection_dense_add": "add"}


@dataclass
class _SparsePrefill:
    """One layer's view of the `prefill_sparse_state` dictionary (attention_v4.py:171-232), read once.

    keys        [S] bool, the key columns the sparse pass may see: the layer's keep list and everything from
                `full_prompt_len` on
    rows_mask   [S, S] bool, the context's block mask
    anchor      (stride, offset, left, right, direction) of the correction, None = sparse pass only
    mode        "plain" | "replace" | "add": where the anchors' denser rows come from
    sel         [n, Hq, d] ready-made anchor rows of this layer (selection modes), with per-row counts
    """
    keys: torch.Tensor
    rows_mask: torch.Tensor
    anchor: Optional[tuple] = None
    mode: str = "plain"
    sel: Optional[torch.Tensor] = None
    sel_counts: Optional[torch.Tensor] = None
    scale: float = 1.0
    sel_scale: float = 1.0
    debug: bool = False

    @staticmethod
    def _layer_entry(table, layer_idx):
        if table is None or not 0 <= layer_idx < len(table):
            return None
        return table[layer_idx]

    @classmethod
    def parse(cls, state, layer_idx, seq_len, num_heads, block_mask, dev, dtype):
        if not state or not state.get("enabled", False) or layer_idx < 0 or block_mask is None:
            return None
        keep = cls._layer_entry(state.get("keep_indices"), layer_idx)
        if keep is None or keep.numel() == 0:
            return None
        keep = keep.to(device=dev, dtype=torch.long).flatten()
        keep = keep[(keep >= 0) & (keep < seq_len)]
        if keep.numel() == 0:
            return None
        keys = torch.zeros(seq_len, dtype=torch.bool, device=dev).index_fill_(0, keep, True)
        prompt_end = int(state.get("full_prompt_len", seq_len))
        if 0 <= prompt_end < seq_len:
            keys[prompt_end:] = True
        plan = cls(keys=keys, rows_mask=block_mask.to(device=dev, dtype=torch.bool),
                   scale=float(state.get("scale", 1.0)), sel_scale=float(state.get("selection_scale", 1.0)),
                   debug=bool(state.get("debug", False)))
        delta_mode = (state.get("delta_mode") or "none").lower()
        if delta_mode in _DELTA_OFF:
            return plan
        if delta_mode not in _DELTA_ON:
            raise ValueError(f"Unsupported prefill_delta_mode: {delta_mode}")
        plan.anchor = ops.anchor_params(state, seq_len)
        plan.mode = _SELECTION_MODES.get((state.get("selection_mode") or "none").lower(), "plain")
        ready = state.get("selection_dense")
        if plan.mode != "plain" and isinstance(ready, dict):
            rows = cls._layer_entry(ready.get("outputs"), layer_idx)
            if rows is not None and rows.dim() == 3 and rows.shape[0] > 0 and rows.shape[1] == num_heads:
                plan.sel = rows.to(device=dev, dtype=dtype).contiguous()
                counts = cls._layer_entry(ready.get("counts"), layer_idx)
                plan.sel_counts = None if counts is None else counts.to(dev)
        return plan

    def selection_covers(self, anchors) -> bool:
        """Does the selection hold a usable row (in range, count > 0) for at least one anchor?"""
        n = self.sel.shape[0]
        usable = anchors < n
        if self.sel_counts is not None:
            usable = usable & (self.sel_counts.index_select(0, anchors.clamp_max(n - 1)) > 0)
        return bool(usable.any().item())
