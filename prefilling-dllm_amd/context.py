"""Thread-local operator descriptor: the fields of the reference's ContextForDiffusionLM
(prefilling_dllm/utils/context.py:8-24, 58-98, 126-155) that the attention operators consume.

The reference assembles a dense block-diagonal boolean mask in __post_init__ (context.py:69-98).
Here the mask stays a per-sequence description (`mask_kind` "full" / "causal", or a dense tensor
in `block_mask` when the caller really has one), because the HIP kernels take the mask mode and
read a dense mask only when one is given."""
from __future__ import annotations

import threading
from dataclasses import dataclass
from typing import Any, List, Optional

import torch

_THREAD_CONTEXT = threading.local()


@dataclass
class ContextForDiffusionLM:
    is_prefill: bool = False
    cu_seqlens_q: Optional[torch.Tensor] = None
    cu_seqlens_k: Optional[torch.Tensor] = None
    max_seqlen_q: int = 0
    max_seqlen_k: int = 0
    slot_mapping: Optional[torch.Tensor] = None
    context_lens: Optional[torch.Tensor] = None
    block_tables: Optional[torch.Tensor] = None
    seqs: Optional[List[Any]] = None
    seq_lens: Optional[List[int]] = None
    seq_lens_ts: Optional[torch.Tensor] = None
    kv_cache_layout: str = "unified"
    need_kv_cache_store: bool = True
    block_mask: Optional[torch.Tensor] = None      # dense [Nq, Nq] over the active rows, or None
    decode_delta_state: Any = None
    prefill_sparse_state: Any = None
    mask_kind: str = "full"                        # "full" | "causal" | "dense"
    # visible prefix as token ranges (range_ptr, range_start, range_len, max_ranges); None = the
    # first context_lens[r] tokens of each page table (the reference's decode context)
    ranges: Any = None
    max_context_len: int = 0
    # A decode step over a cached prefix normally stores its active rows inside the attention call, after the
    # kernel has read the cache.  That equals the reference's store-then-attend order (attention_v4.py:328-331)
    # only while no active slot lies inside a visible prefix range -- true for the reference's own callers
    # (fastdllm_engine.py:497: the block's slots follow the context).  A caller that rewrites visible context
    # rows sets this flag: the store then runs as a launch of its own in front of the attention.
    store_before_attention: bool = False

    def __post_init__(self):
        if self.seq_lens_ts is not None and self.context_lens is not None:
            self.total_lens = self.seq_lens_ts + self.context_lens
        if self.block_mask is None and self.seqs:
            # the reference's form: every sequence carries its own mask (utils/context.py:69-98)
            masks = [getattr(seq, "current_block_mask", None) for seq in self.seqs]
            if all(m is not None for m in masks):
                self.block_mask = active_block_mask(masks)
        if self.block_mask is not None:
            self.mask_kind = "dense"

    @property
    def total_num_seqs(self) -> int:
        return len(self.seqs) if self.seqs is not None else 0


def active_block_mask(masks) -> Optional[torch.Tensor]:
    """Per-sequence masks of the reference -> the dense [Nq, Nq] mask over the active rows that the HIP operators
    take, or None when every active key is visible to every active row of its sequence (the "full" mode).

    A sequence's mask is [..., h, w] with h active rows and w = h keys (prefill) or w = ctx + h keys (decode,
    unified layout: the cached context in the leading columns, engine/sequence.py:489-493,
    fastdllm_engine.py:496-503).  The reference lays them out block-diagonally (utils/context.py:73-98); so does
    this, on the active columns only.  The cached context is always visible to the HIP kernels -- it is in every
    mask the reference builds -- so a mask that hides a context column is refused."""
    parts, ctx_ok, act_ok = [], [], []
    for m in masks:
        m = m.reshape(m.shape[-2], m.shape[-1]).to(torch.bool)
        h, w = m.shape
        if w < h:
            raise ValueError(f"sequence mask of {h} rows has only {w} key columns")
        if w > h:
            ctx_ok.append(m[:, :w - h].all())
        a = m[:, w - h:]
        act_ok.append(a.all())
        parts.append(a)
    if not parts:
        return None
    # one transfer to the host for all sequences: [every context column visible, every active column visible]
    one = torch.ones((), dtype=torch.bool, device=parts[0].device)
    flags = torch.stack([torch.stack(ctx_ok).all() if ctx_ok else one, torch.stack(act_ok).all()]).tolist()
    if not flags[0]:
        raise ValueError("a sequence mask hides cached context keys; the HIP attention always sees the "
                         "visible prefix (pass a shorter context or other ranges instead)")
    if flags[1]:
        return None
    n = sum(p.shape[0] for p in parts)
    out = torch.zeros((n, n), dtype=torch.bool, device=parts[0].device)
    r = 0
    for a in parts:
        out[r:r + a.shape[0], r:r + a.shape[0]] = a
        r += a.shape[0]
    return out


def get_context_diffusion_lm() -> ContextForDiffusionLM:
    ctx = getattr(_THREAD_CONTEXT, "diffusion_lm", None)
    if ctx is None:
        ctx = ContextForDiffusionLM()
        _THREAD_CONTEXT.diffusion_lm = ctx
    return ctx


def set_context_diffusion_lm(is_prefill, cu_seqlens_q=None, cu_seqlens_k=None, max_seqlen_q=0, max_seqlen_k=0,
                             slot_mapping=None, context_lens=None, block_tables=None, seqs=None, seq_lens=None,
                             seq_lens_ts=None, kv_cache_layout="unified", need_kv_cache_store=True,
                             decode_delta_state=None, prefill_sparse_state=None, block_mask=None, mask_kind="full",
                             ranges=None, max_context_len=0, store_before_attention=False) -> None:
    """Same positional/keyword surface as the reference (context.py:135-152) plus the mask / range
    description the HIP path uses instead of a materialised mask."""
    _THREAD_CONTEXT.diffusion_lm = ContextForDiffusionLM(
        is_prefill, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, slot_mapping, context_lens, block_tables,
        seqs, seq_lens, seq_lens_ts, kv_cache_layout, need_kv_cache_store, block_mask, decode_delta_state,
        prefill_sparse_state, mask_kind, ranges, max_context_len, store_before_attention)


def reset_context_diffusion_lm() -> None:
    _THREAD_CONTEXT.diffusion_lm = ContextForDiffusionLM()
