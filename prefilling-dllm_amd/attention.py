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
        store_in_call = (has_cache and context.need_kv_cache_store and not context.is_prefill and max_ctx > 0
                         and context.slot_mapping is not None)
        if has_cache and context.need_kv_cache_store and not store_in_call:
            ops.store_kvcache_unified_layout(k, v, k_cache, v_cache, context.slot_mapping, self.model_type, context)

        mask_mode, dense = context.mask_kind, None
        if context.block_mask is not None:
            mask_mode, dense = "dense", context.block_mask
            if dense.dim() != 2 or dense.shape[0] != q.shape[0]:
                raise ValueError(f"block_mask must be [rows, keys] with one row per active token, got {tuple(dense.shape)}")
            if dense.shape[1] != q.shape[0]:
                # the reference's decode form [Nq, sum(ctx + Sq)] (utils/context.py:85-98): keep the active columns
                dense = self._active_columns(dense, context)
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
    def _active_columns(mask: torch.Tensor, context: ContextForDiffusionLM):
        """[Nq, sum(ctx_s + Sq_s)] block-diagonal decode mask of the reference -> [Nq, Nq] over the active keys
        (None when no active key is hidden)."""
        from .context import active_block_mask
        if context.is_prefill or context.context_lens is None or context.cu_seqlens_q is None:
            raise ValueError(f"block_mask of shape {tuple(mask.shape)} does not match {mask.shape[0]} active rows")
        ctx = [int(x) for x in context.context_lens.tolist()]
        cu = [int(x) for x in context.cu_seqlens_q.tolist()]
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
        attention_v4.py:120-125) with room for `extra` more tokens.  The copy is kept in the state between steps and
        made again when the prompt tensors change."""
        page, n_prompt = 256, int(full_k.shape[0])
        pages = (n_prompt + extra + page - 1) // page
        key = (full_k.data_ptr(), full_v.data_ptr(), n_prompt, full_k._version, full_v._version)
        held = state.setdefault("_paged_prompt", {})
        ent = held.get(self.layer_idx)
        if ent is None or ent[0] != key or ent[1].shape[0] < pages:
            kc = torch.empty((pages, page, self.num_kv_heads, self.head_dim), dtype=full_k.dtype, device=full_k.device)
            vc = torch.empty_like(kc)
            kc.view(-1, self.num_kv_heads, self.head_dim)[:n_prompt].copy_(full_k)
            vc.view(-1, self.num_kv_heads, self.head_dim)[:n_prompt].copy_(full_v)
            ent = (key, kc, vc)
            held[self.layer_idx] = ent
        return ent[1], ent[2]

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
        state = getattr(context, "prefill_sparse_state", None)
        if not state or not state.get("enabled", False):
            return None
        if self.model_type != "diffusion_lm" or self.layer_idx < 0:
            return None
        keep_by_layer = state.get("keep_indices")
        if keep_by_layer is None or self.layer_idx >= len(keep_by_layer):
            return None
        base_mask = context.block_mask
        if base_mask is None:
            return None
        seq_len, dev = q.shape[0], q.device
        layer_keep = keep_by_layer[self.layer_idx]
        if layer_keep is None or layer_keep.numel() == 0:
            return None
        valid_keep = layer_keep.to(device=dev, dtype=torch.long).reshape(-1)
        valid_keep = valid_keep[(valid_keep >= 0) & (valid_keep < seq_len)]
        if valid_keep.numel() == 0:
            return None
        key_mask = torch.zeros(seq_len, dtype=torch.bool, device=dev)
        key_mask[valid_keep] = True
        full_prompt_len = int(state.get("full_prompt_len", seq_len))
        if 0 <= full_prompt_len < seq_len:
            key_mask[full_prompt_len:] = True
        if state.get("debug", False):
            active_keys = int(key_mask.sum().item())
            state["union_min"] = min(int(state.get("union_min", active_keys)), active_keys)
            state["union_max"] = max(int(state.get("union_max", active_keys)), active_keys)
        base_mask = base_mask.to(device=dev, dtype=torch.bool)
        one_seq = torch.tensor([0, seq_len], dtype=torch.int32, device=dev)

        def attend(mask):
            return ops.sparse_decode_attention(q, k, v, None, None, None, one_seq, max_q_len=seq_len, max_ctx_len=0,
                                               mask_mode="dense", mask=mask, sm_scale=self.scale)

        o_sparse = attend(base_mask & key_mask.unsqueeze(0))
        delta_mode = (state.get("delta_mode") or "none").lower()
        if delta_mode in {"none", "off", "0", ""}:
            return o_sparse
        if delta_mode not in {"s4_left3", "delta_s4_left3", "sampled_delta_s4_left3"}:
            raise ValueError(f"Unsupported prefill_delta_mode: {delta_mode}")
        ap = ops.anchor_params(state, seq_len)
        if ap is None:
            return o_sparse
        stride, offset, left, right, direction = ap

        selection_mode = (state.get("selection_mode") or "none").lower()
        selection_dense = state.get("selection_dense")
        sel = counts = None
        if selection_mode in {"selection_dense_replace", "selection_dense_add"} and selection_dense:
            outputs_by_layer = selection_dense.get("outputs") if isinstance(selection_dense, dict) else None
            counts_by_layer = selection_dense.get("counts") if isinstance(selection_dense, dict) else None
            if outputs_by_layer is not None and self.layer_idx < len(outputs_by_layer):
                layer_outputs = outputs_by_layer[self.layer_idx]
                if layer_outputs is not None and layer_outputs.shape[0] > 0 and layer_outputs.shape[1] == self.num_heads:
                    sel = layer_outputs.to(device=dev, dtype=o_sparse.dtype).contiguous()
                    if counts_by_layer is not None and self.layer_idx < len(counts_by_layer) and \
                            counts_by_layer[self.layer_idx] is not None:
                        counts = counts_by_layer[self.layer_idx].to(dev)
        scale = float(state.get("scale", 1.0))
        kw = dict(max_q_len=seq_len, stride=stride, anchor_offset=offset, left=left, right=right, direction=direction,
                  scale=scale)
        anchors = torch.arange(offset, seq_len, stride, device=dev)

        def any_valid():
            in_range = anchors < sel.shape[0]
            if counts is None:
                return bool(in_range.any().item())
            safe = anchors.clamp_max(sel.shape[0] - 1)
            return bool(((counts.index_select(0, safe) > 0) & in_range).any().item())

        if selection_mode == "selection_dense_replace":
            if sel is None or not any_valid():
                return o_sparse
            out = ops.anchor_delta_add(o_sparse, None, one_seq, sel=sel, sel_counts=counts, sel_mode="replace", **kw)
            state["selection_used_calls"] = int(state.get("selection_used_calls", 0)) + 1
            dense = None
        else:
            dense = attend(base_mask)
            if selection_mode == "selection_dense_add" and sel is not None:
                out = ops.anchor_delta_add(o_sparse, dense, one_seq, sel=sel, sel_counts=counts, sel_mode="add",
                                           sel_scale=float(state.get("selection_scale", 1.0)), **kw)
                state["selection_used_calls"] = int(state.get("selection_used_calls", 0)) + 1
            else:
                out = ops.anchor_delta_add(o_sparse, dense, one_seq, **kw)
        if state.get("debug", False):
            # largest |out - o_sparse| over the anchor rows stands in for the reference's max |delta|
            diff = (out.index_select(0, anchors).float() - o_sparse.index_select(0, anchors).float()).abs()
            self._debug_stats(state, float(diff.max().item()) if diff.numel() else 0.0, int(anchors.numel()))
        return out
