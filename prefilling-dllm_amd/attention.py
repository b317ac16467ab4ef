"""Attention layer with the reference's interface (layers/attention/attention_v4.py:21-52, 316-410)
running on the HIP operators: `Attention(num_heads, head_dim, scale, num_kv_heads,
model_type).forward(q, k, v)` reads the thread-local ContextForDiffusionLM, stores K/V into the
paged cache through the slot mapping, and attends

  * prefill: every sequence of the packed batch to itself (block-diagonal; full, causal or the
    dense block mask of the context) -- attention_v4.py:336-367;
  * decode: the active rows to [visible prefix pages || active rows] without the dense
    load_kvcache staging copy -- attention_v4.py:368-397.

The experimental decode-delta / sparse-prefill corrections of the reference (default off) are not
part of this layer."""
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

        if has_cache and context.need_kv_cache_store:
            ops.store_kvcache_unified_layout(k, v, k_cache, v_cache, context.slot_mapping, self.model_type, context)

        mask_mode, dense = context.mask_kind, None
        if context.block_mask is not None:
            mask_mode, dense = "dense", context.block_mask
        if context.is_prefill:
            if mask_mode == "dense":
                o = ops.sparse_decode_attention(q, k, v, None, None, None, context.cu_seqlens_q,
                                                max_q_len=int(context.max_seqlen_q), max_ctx_len=0,
                                                mask_mode="dense", mask=dense, sm_scale=self.scale)
            else:
                o = ops.chunk_prefill_attention(q, k, v, context.cu_seqlens_q, max_seqlen=int(context.max_seqlen_q),
                                                causal=(mask_mode == "causal"), sm_scale=self.scale)
        else:
            max_ctx = int(context.max_context_len) or max(int(context.max_seqlen_k) - 1, 0)
            o = ops.sparse_decode_attention(q, k, v, k_cache if has_cache else None, v_cache if has_cache else None,
                                            context.block_tables, context.cu_seqlens_q,
                                            max_q_len=int(context.max_seqlen_q), max_ctx_len=max_ctx if has_cache else 0,
                                            context_lens=context.context_lens, ranges=context.ranges,
                                            mask_mode=mask_mode, mask=dense, sm_scale=self.scale)
        return o.view(-1, self.num_heads * self.head_dim)
