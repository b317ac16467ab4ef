"""Operator layer: the names the reference exports from layers/attention/ops/__init__.py
(store_kvcache_unified_layout, load_kvcache, diffusion_lm_parallel_flash_decoding,
query_to_chunk_attention_scores) plus the tensor-level helpers of fastdllm_engine.py,
all running the hand-written HIP kernels through the C ABI (libpdllm_hip.so).

PyTorch is used only for device memory and the current stream.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import AttnDesc, check, lib

PAGE_SIZE = 256  # reference default, config.py:39


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need_cuda(*ts: torch.Tensor) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("HIP operators require device tensors (the product path has no CPU fallback).")


def _scale_layout(k_scale: torch.Tensor, v_scale: torch.Tensor, n_pages: int, num_kv_heads: int,
                  device) -> Tuple[int, int]:
    """(page stride, head stride) of the fp8 scales, the same for the store and for the attention: one scalar
    (what the reference passes, prefix_prefill.py:118-121), scale[n_pages], or scale[n_pages, Hkv]."""
    for name, t in (("k_scale", k_scale), ("v_scale", v_scale)):
        if not isinstance(t, torch.Tensor) or t.dtype != torch.float32 or t.device != device:
            raise ValueError(f"{name} must be an fp32 tensor on the device of the cache")
    if k_scale.shape != v_scale.shape or k_scale.stride() != v_scale.stride():
        raise ValueError("k_scale and v_scale must have the same layout")
    if k_scale.numel() == 1:
        return 0, 0
    if k_scale.dim() == 1 and k_scale.shape[0] >= n_pages:
        return k_scale.stride(0), 0
    if k_scale.dim() == 2 and k_scale.shape[0] >= n_pages and k_scale.shape[1] == num_kv_heads:
        return k_scale.stride(0), k_scale.stride(1)
    raise ValueError(f"fp8 scales must be a scalar, [n_pages] or [n_pages, Hkv] with n_pages >= {n_pages}, "
                     f"Hkv = {num_kv_heads}; got {tuple(k_scale.shape)}")


_WORKSPACES: dict = {}


def _workspace(device: torch.device, nbytes: int) -> Optional[torch.Tensor]:
    """A per-(device, stream) scratch tensor, grown on demand (torch owns the memory)."""
    if nbytes <= 0:
        return None
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = ws
    return ws


# ----------------------------------------------------------------------------------------
# KV store / load  (reference: layers/attention/ops/kv_cache_kernels.py)
# ----------------------------------------------------------------------------------------

def store_kvcache_unified_layout(key: torch.Tensor, value: torch.Tensor, k_cache: torch.Tensor,
                                 v_cache: torch.Tensor, slot_mapping: torch.Tensor,
                                 model_type: str = "diffusion_lm", context=None,
                                 k_scale: Optional[torch.Tensor] = None,
                                 v_scale: Optional[torch.Tensor] = None) -> None:
    """kv_cache_kernels.py:150-172.  slot < 0 skips the token (diffusion_lm semantics, :46-48).

    With an fp8 (float8_e4m3fn) cache and per-page scales the rows are quantised on the way."""
    _need_cuda(key, value, k_cache, v_cache, slot_mapping)
    N, num_heads, head_dim = key.shape
    D = num_heads * head_dim
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == head_dim and value.stride(1) == head_dim
    assert k_cache.stride(1) == D and v_cache.stride(1) == D
    assert N == slot_mapping.numel(), f"`N`: {N}, `slot_mapping.numel()`: {slot_mapping.numel()}"
    if model_type not in ("causal_lm", "diffusion_lm"):
        return
    if slot_mapping.dtype != torch.int32:
        slot_mapping = slot_mapping.to(torch.int32)
    slot_mapping = slot_mapping.contiguous()
    n_slots = k_cache.shape[0] * k_cache.shape[1]
    if not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise ValueError("unified KV cache must be contiguous")
    if k_cache.dtype == torch.float8_e4m3fn:
        if k_scale is None or v_scale is None:
            raise ValueError("fp8 KV cache needs k_scale / v_scale")
        if key.dtype != torch.bfloat16 or value.dtype != torch.bfloat16:
            raise ValueError("the fp8 store quantises bf16 rows")
        sps, shs = _scale_layout(k_scale, v_scale, k_cache.shape[0], num_heads, k_cache.device)
        st = lib.pdllm_kv_store_fp8(key.data_ptr(), value.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                    k_scale.data_ptr(), v_scale.data_ptr(), slot_mapping.data_ptr(), N, D,
                                    key.stride(0), value.stride(0), n_slots, k_cache.shape[1], head_dim, sps, shs,
                                    _stream(key))
    else:
        if key.dtype != k_cache.dtype or key.element_size() != 2:
            raise ValueError("KV store expects 16-bit rows of the cache dtype")
        st = lib.pdllm_kv_store(key.data_ptr(), value.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                slot_mapping.data_ptr(), N, D, key.stride(0), value.stride(0), n_slots,
                                _stream(key))
    check(st, "store_kvcache_unified_layout")


def store_kvcache_distinct_layout(*args, **kwargs):
    raise NotImplementedError("the distinct (x-split K / transposed V) layout is not part of this build; "
                              "use kv_cache_layout='unified'")


def slot_mapping_from_pages(page_ids: torch.Tensor, num_tokens: int, start_token: int = 0,
                            page_size: int = PAGE_SIZE) -> torch.Tensor:
    """fastdllm_engine.py:331-337, 434-441 on device: slot = page_ids[t // P] * P + t % P."""
    _need_cuda(page_ids)
    page_ids = page_ids.to(torch.int32).contiguous()
    out = torch.empty(num_tokens, dtype=torch.int32, device=page_ids.device)
    check(lib.pdllm_slot_mapping(page_ids.data_ptr(), page_ids.numel(), start_token, num_tokens, page_size,
                                 out.data_ptr(), _stream(page_ids)), "slot_mapping_from_pages")
    return out


def load_kvcache(k_cache: torch.Tensor, v_cache: torch.Tensor, context, k_new: torch.Tensor,
                 v_new: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """kv_cache_kernels.py:278-327: dense [sum(ctx+active), Hkv, d] staging copy.

    Kept for callers that want the dense tensors; the attention operator below reads the
    pages directly and does not need it."""
    _need_cuda(k_cache, v_cache, k_new, v_new)
    assert k_cache.shape == v_cache.shape
    assert k_new.shape == v_new.shape
    n_blocks, page_size, h_kv, head_dim = k_cache.shape
    num_seqs, _ = context.block_tables.shape
    ctxlens = context.context_lens
    seqlens = context.seq_lens_ts
    seq_lens_host = [int(x) for x in context.seq_lens]
    assert sum(seq_lens_host) == k_new.shape[0]
    dbs = context.seqs[0].diffusion_block_size
    assert max(seq_lens_host) % dbs == 0
    cu_q, cu_k = context.cu_seqlens_q, context.cu_seqlens_k
    assert cu_q.shape == cu_k.shape and cu_q.shape[0] == num_seqs + 1
    total = int(cu_k[-1].item())
    max_total = int((ctxlens + seqlens).max().item())
    k_out = torch.empty((total, h_kv, head_dim), device=k_cache.device, dtype=k_cache.dtype)
    v_out = torch.empty_like(k_out)
    _need_cuda(context.block_tables, ctxlens, cu_q, cu_k)
    # converted copies stay bound to locals until the call has been enqueued
    bt = context.block_tables.to(torch.int32).contiguous()
    ctx32, cuq32, cuk32 = (t.to(torch.int32).contiguous() for t in (ctxlens, cu_q, cu_k))
    D = h_kv * head_dim
    check(lib.pdllm_kv_load(k_cache.data_ptr(), v_cache.data_ptr(), k_new.data_ptr(), v_new.data_ptr(),
                            k_out.data_ptr(), v_out.data_ptr(), bt.data_ptr(), bt.stride(0),
                            ctx32.data_ptr(), cuq32.data_ptr(), cuk32.data_ptr(), num_seqs, max_total, D, page_size,
                            n_blocks, k_new.stride(0), D, _stream(k_cache)), "load_kvcache")
    del bt, ctx32, cuq32, cuk32
    return k_out, v_out


# ----------------------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------------------

def _fill_desc(q, k_new, v_new, out, k_cache, v_cache, block_table, q_start_loc, ranges, mask, mask_mode,
               max_q_len, max_ctx_len, sm_scale, k_scale, v_scale, num_splits, rows_per_group,
               tiles_per_workgroup=0) -> AttnDesc:
    n_tokens, Hq, d = q.shape
    Hkv = k_new.shape[1]
    for t in (q, k_new, v_new, out):
        if t.dtype != torch.bfloat16 or t.stride(-1) != 1 or t.stride(1) != d:
            raise ValueError("q / k / v / out must be bf16 [tokens, heads, head_dim] with contiguous heads")
    desc = AttnDesc()
    desc.q, desc.k_new, desc.v_new, desc.out = q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), out.data_ptr()
    desc.q_stride, desc.kn_stride, desc.vn_stride, desc.o_stride = q.stride(0), k_new.stride(0), v_new.stride(0), out.stride(0)
    desc.n_tokens = n_tokens
    desc.num_q_heads, desc.num_kv_heads, desc.head_dim = Hq, Hkv, d
    desc.q_start_loc = q_start_loc.data_ptr()
    desc.n_req = q_start_loc.numel() - 1
    desc.max_q_len, desc.max_ctx_len = int(max_q_len), int(max_ctx_len)
    desc.mask_mode = mask_mode
    desc.sm_scale = float(sm_scale)
    desc.num_splits, desc.rows_per_group = int(num_splits), int(rows_per_group)
    desc.tiles_per_workgroup = int(tiles_per_workgroup)
    if mask_mode == _lib.MASK_DENSE:
        if mask is None:
            raise ValueError("dense mask mode needs a mask")
        desc.mask, desc.mask_stride = mask.data_ptr(), mask.stride(0)
    if k_cache is not None and max_ctx_len > 0:
        if k_cache.dim() != 4 or k_cache.stride(-1) != 1:
            raise NotImplementedError("only the unified cache layout [pages, page_size, Hkv, d] is supported")
        desc.k_cache, desc.v_cache = k_cache.data_ptr(), v_cache.data_ptr()
        desc.n_pages, desc.page_size = k_cache.shape[0], k_cache.shape[1]
        desc.cache_page_stride, desc.cache_token_stride, desc.cache_head_stride = k_cache.stride(0), k_cache.stride(1), k_cache.stride(2)
        if k_cache.dtype == torch.bfloat16:
            desc.kv_dtype = _lib.KV_BF16
        elif k_cache.dtype in (torch.float8_e4m3fn, torch.uint8):
            desc.kv_dtype = _lib.KV_FP8_E4M3
            if k_scale is None or v_scale is None:
                raise ValueError("fp8 KV cache needs k_scale / v_scale tensors")
            desc.k_scale, desc.v_scale = k_scale.data_ptr(), v_scale.data_ptr()
            desc.scale_page_stride, desc.scale_head_stride = _scale_layout(k_scale, v_scale, k_cache.shape[0], Hkv,
                                                                           k_cache.device)
        else:
            raise ValueError(f"unsupported KV cache dtype {k_cache.dtype}")
        desc.block_table, desc.bt_stride = block_table.data_ptr(), block_table.stride(0)
        rp, rs, rl, max_ranges = ranges
        desc.range_ptr, desc.range_start, desc.range_len = rp.data_ptr(), rs.data_ptr(), rl.data_ptr()
        desc.max_ranges = int(max_ranges)
    return desc


def _active_mask(mask: Optional[torch.Tensor], n_tokens: int) -> Optional[torch.Tensor]:
    """The dense mask the kernels index as mask[q_start + i, q_start + j] over the ACTIVE rows and keys only."""
    if mask is None:
        return None
    if mask.dim() != 2 or tuple(mask.shape) != (n_tokens, n_tokens):
        raise ValueError(f"mask must be [n_tokens, n_tokens] = [{n_tokens}, {n_tokens}] over the active rows and "
                         f"active keys, got {tuple(mask.shape)}; a mask with context columns "
                         "([Sq, ctx + Sq], the reference's decode form) goes through context.active_block_mask")
    _need_cuda(mask)
    return mask.to(torch.bool).contiguous().view(torch.uint8)


def sparse_decode_attention(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
                            k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                            block_table: Optional[torch.Tensor], q_start_loc: torch.Tensor, *,
                            max_q_len: int, max_ctx_len: int,
                            context_lens: Optional[torch.Tensor] = None,
                            ranges: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int]] = None,
                            mask_mode: str = "full", mask: Optional[torch.Tensor] = None,
                            sm_scale: Optional[float] = None, k_scale: Optional[torch.Tensor] = None,
                            v_scale: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                            num_splits: int = 0, rows_per_group: int = 0,
                            tiles_per_workgroup: int = 0,
                            active_slot_mapping: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of the active block over [selected prefix pages || active block].

    active_slot_mapping: int32 [n_tokens] cache slots of the active rows; when given the call also stores
    k_new / v_new there (store_kvcache_unified_layout of the decode forward, attention_v4.py:328-331).

    The visible prefix of request r is either `context_lens[r]` leading tokens of its page
    table (the reference's decode context, attention_v4.py:368-397) or an explicit list of
    token ranges `ranges = (range_ptr[n_req+1], range_start[], range_len[], max_ranges)`,
    which is how a top-K chunk selection reads its non-contiguous chunks in place.
    mask_mode: "full" (bidirectional block), "causal", or "dense" with mask[n_tok, n_tok]."""
    _need_cuda(q, k_new, v_new, q_start_loc, k_cache, v_cache, block_table, context_lens, k_scale, v_scale, out)
    if ranges is not None:
        _need_cuda(*ranges[:3])
    n_tokens, Hq, d = q.shape
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    if out is None:
        out = torch.empty_like(q)
    q_start_loc = q_start_loc.to(torch.int32).contiguous()
    n_req = q_start_loc.numel() - 1
    mode = {"full": _lib.MASK_FULL, "causal": _lib.MASK_CAUSAL, "dense": _lib.MASK_DENSE}[mask_mode]
    mask = _active_mask(mask, n_tokens)
    if k_cache is not None and max_ctx_len > 0:
        block_table = block_table.to(torch.int32).contiguous()
        if ranges is None:
            if context_lens is None:
                raise ValueError("give context_lens or ranges")
            dev = q.device
            ranges = (torch.arange(n_req + 1, dtype=torch.int32, device=dev),
                      torch.zeros(n_req, dtype=torch.int32, device=dev),
                      context_lens.to(torch.int32).contiguous(), 1)
        else:
            ranges = tuple(t.to(torch.int32).contiguous() for t in ranges[:3]) + (int(ranges[3]),)
    desc = _fill_desc(q, k_new, v_new, out, k_cache, v_cache, block_table, q_start_loc, ranges, mask, mode,
                      max_q_len, max_ctx_len, sm_scale, k_scale, v_scale, num_splits, rows_per_group,
                      tiles_per_workgroup)
    active_slot_mapping = _slot_mapping_arg(desc, active_slot_mapping, n_tokens)
    need = lib.pdllm_attn_workspace_bytes(C.byref(desc))
    if need < 0:
        check(int(need), "sparse_decode_attention")
    ws = _workspace(q.device, int(need))
    if ws is not None:
        desc.workspace, desc.workspace_bytes = ws.data_ptr(), ws.numel()
    check(lib.pdllm_sparse_decode_attn(C.byref(desc), _stream(q)), "sparse_decode_attention")
    return out


def _slot_mapping_arg(desc: AttnDesc, slots: Optional[torch.Tensor], n_tokens: int) -> Optional[torch.Tensor]:
    """Bind the cache slots of the active rows to the descriptor (the store rides in the attention call).  Returns
    the tensor the descriptor points at; the caller keeps it alive until the launch has been enqueued."""
    if slots is None:
        return None
    _need_cuda(slots)
    if slots.numel() != n_tokens:
        raise ValueError(f"active_slot_mapping must name one slot per active row: {slots.numel()} vs {n_tokens}")
    if not desc.k_cache:
        raise ValueError("active_slot_mapping needs a KV cache to store into")
    slots = slots.to(torch.int32).contiguous()
    desc.active_slot_mapping = slots.data_ptr()
    return slots


class PreparedAttention:
    """A filled attention descriptor bound to its tensors, for loops that run the same shapes
    again and again (every denoise step reuses the page table, ranges and buffers): `run()` is one
    ctypes call into pdllm_sparse_decode_attn with no per-call tensor bookkeeping."""

    def __init__(self, q, k_new, v_new, k_cache, v_cache, block_table, q_start_loc, *, max_q_len, max_ctx_len,
                 context_lens=None, ranges=None, mask_mode="full", mask=None, sm_scale=None, k_scale=None,
                 v_scale=None, out=None, num_splits=0, rows_per_group=0, workspace=None, slot_table=None,
                 tiles_per_workgroup=0, active_slot_mapping=None):
        """slot_table: an int32 tensor from `new_slot_table` shared by every layer of a step; the caller
        refreshes it with `build_slot_table()` of any one of the prepared layers whenever the page table
        or the ranges change.  Without it every `run()` rebuilds the table in its workspace."""
        _need_cuda(q, k_new, v_new, q_start_loc, k_cache, v_cache, block_table, context_lens, k_scale, v_scale, out,
                   workspace, slot_table)
        if ranges is not None:
            _need_cuda(*ranges[:3])
        n_tokens, Hq, d = q.shape
        self.out = torch.empty_like(q) if out is None else out
        q_start_loc = q_start_loc.to(torch.int32).contiguous()
        n_req = q_start_loc.numel() - 1
        mode = {"full": _lib.MASK_FULL, "causal": _lib.MASK_CAUSAL, "dense": _lib.MASK_DENSE}[mask_mode]
        mask = _active_mask(mask, n_tokens)
        if k_cache is not None and max_ctx_len > 0:
            block_table = block_table.to(torch.int32).contiguous()
            if ranges is None:
                if context_lens is None:
                    raise ValueError("give context_lens or ranges")
                ranges = (torch.arange(n_req + 1, dtype=torch.int32, device=q.device),
                          torch.zeros(n_req, dtype=torch.int32, device=q.device),
                          context_lens.to(torch.int32).contiguous(), 1)
            else:
                ranges = tuple(t.to(torch.int32).contiguous() for t in ranges[:3]) + (int(ranges[3]),)
        self.desc = _fill_desc(q, k_new, v_new, self.out, k_cache, v_cache, block_table, q_start_loc, ranges,
                               mask, mode, max_q_len, max_ctx_len,
                               1.0 / math.sqrt(d) if sm_scale is None else sm_scale, k_scale, v_scale,
                               num_splits, rows_per_group, tiles_per_workgroup)
        active_slot_mapping = _slot_mapping_arg(self.desc, active_slot_mapping, n_tokens)
        self.slot_table = slot_table
        if slot_table is not None and k_cache is not None and max_ctx_len > 0:
            if slot_table.dtype != torch.int32 or slot_table.dim() != 2 or slot_table.stride(1) != 1:
                raise ValueError("slot_table must be an int32 [n_req, stride] tensor (see new_slot_table)")
            self.desc.slot_table, self.desc.slot_table_stride = slot_table.data_ptr(), slot_table.stride(0)
        need = lib.pdllm_attn_workspace_bytes(C.byref(self.desc))
        if need < 0:
            check(int(need), "PreparedAttention")
        self.workspace_bytes = int(need)
        if need > 0:
            if workspace is None or workspace.numel() * workspace.element_size() < need:
                workspace = torch.empty(int(need), dtype=torch.uint8, device=q.device)
            self.desc.workspace, self.desc.workspace_bytes = workspace.data_ptr(), int(need)
        # keep every tensor the descriptor points at alive
        self._keep = (q, k_new, v_new, k_cache, v_cache, block_table, q_start_loc, ranges, mask, k_scale, v_scale,
                      workspace, slot_table, active_slot_mapping)
        self._ref = C.byref(self.desc)
        self._fn = lib.pdllm_sparse_decode_attn

    def run(self, stream: Optional[int] = None) -> torch.Tensor:
        st = self._fn(self._ref, torch.cuda.current_stream().cuda_stream if stream is None else stream)
        if st != 0:
            check(st, "PreparedAttention.run")
        return self.out

    def describe_plan(self) -> str:
        """One line naming the kernel and the cut of the launch this descriptor leads to (pdllm_attn_plan_describe)."""
        buf = C.create_string_buffer(256)
        check(lib.pdllm_attn_plan_describe(self._ref, 0, buf, 256), "PreparedAttention.describe_plan")
        return buf.value.decode()

    def build_slot_table(self, stream: Optional[int] = None) -> None:
        """(Re)build the shared slot table from this layer's page table and ranges."""
        if self.slot_table is None:
            raise ValueError("this PreparedAttention was made without a slot_table")
        st = lib.pdllm_attn_build_slot_table(self._ref, self.slot_table.data_ptr(), self.slot_table.stride(0),
                                             torch.cuda.current_stream().cuda_stream if stream is None else stream)
        if st != 0:
            check(st, "PreparedAttention.build_slot_table")


def new_slot_table(n_req: int, max_ctx_len: int, device) -> torch.Tensor:
    """An int32 [n_req, stride] tensor of the size pdllm_attn_build_slot_table needs."""
    desc = AttnDesc()
    desc.max_ctx_len = int(max_ctx_len)
    stride = lib.pdllm_attn_slot_table_stride(C.byref(desc))
    if stride < 0:
        check(int(stride), "new_slot_table")
    return torch.zeros((int(n_req), int(stride)), dtype=torch.int32, device=device)


def attention_plan(n_req: int, num_q_heads: int, num_kv_heads: int, *, max_q_len: int, max_ctx_len: int,
                   prefill: bool = False, num_splits: int = 0, rows_per_group: int = 0) -> Tuple[int, int]:
    """(rows per workgroup, KV splits) the library would pick for these sizes; no launch."""
    d = 128
    dummy = torch.empty(16, dtype=torch.int32)  # only non-NULL, 16-byte aligned addresses are needed
    desc = AttnDesc()
    desc.q = desc.k_new = desc.v_new = desc.out = desc.q_start_loc = dummy.data_ptr() & ~15
    desc.q_stride = desc.o_stride = num_q_heads * d
    desc.kn_stride = desc.vn_stride = num_kv_heads * d
    desc.n_tokens = n_req * max_q_len
    desc.num_q_heads, desc.num_kv_heads, desc.head_dim = num_q_heads, num_kv_heads, d
    desc.n_req, desc.max_q_len, desc.max_ctx_len = n_req, int(max_q_len), int(max_ctx_len)
    desc.num_splits, desc.rows_per_group = num_splits, rows_per_group
    desc.sm_scale = 1.0 / math.sqrt(d)
    rows, splits = C.c_int32(0), C.c_int32(0)
    check(lib.pdllm_attn_plan(C.byref(desc), 1 if prefill else 0, C.byref(rows), C.byref(splits)), "attention_plan")
    return rows.value, splits.value


def chunk_prefill_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor, *,
                            max_seqlen: int, causal: bool = True, sm_scale: Optional[float] = None,
                            k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None,
                            slot_mapping: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                            rows_per_group: int = 0, num_splits: int = 0) -> torch.Tensor:
    """Block-diagonal self-attention over a packed batch of independent chunks
    (attention_v4.py:336-367 with the block mask of utils/context.py:73-84), causal or full
    inside each chunk, with the paged store of K/V (kv_cache_kernels.py:150-172) when
    slot_mapping is given.  num_splits = 0 lets the library choose the kernel (resident workgroups that stream
    through their columns for large batches, one workgroup per column otherwise); 1 asks for one workgroup per
    column."""
    _need_cuda(q, k, v, cu_seqlens)
    n_tokens, Hq, d = q.shape
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    if out is None:
        out = torch.empty_like(q)
    cu = cu_seqlens.to(torch.int32).contiguous()
    mode = _lib.MASK_CAUSAL if causal else _lib.MASK_FULL
    desc = _fill_desc(q, k, v, out, None, None, None, cu, None, None, mode, max_seqlen, 0, sm_scale, None, None,
                      num_splits, rows_per_group)
    slots_ptr = None
    if slot_mapping is not None:
        if k_cache is None or v_cache is None:
            raise ValueError("slot_mapping given without caches")
        if not k_cache.is_contiguous() or not v_cache.is_contiguous() or k_cache.dtype != torch.bfloat16:
            raise ValueError("prefill store needs contiguous bf16 unified caches")
        assert slot_mapping.numel() == n_tokens
        slot_mapping = slot_mapping.to(torch.int32).contiguous()
        slots_ptr = slot_mapping.data_ptr()
        desc.k_cache, desc.v_cache = k_cache.data_ptr(), v_cache.data_ptr()
        desc.n_pages, desc.page_size = k_cache.shape[0], k_cache.shape[1]
        desc.cache_page_stride, desc.cache_token_stride, desc.cache_head_stride = k_cache.stride(0), k_cache.stride(1), k_cache.stride(2)
        desc.kv_dtype = _lib.KV_BF16
    check(lib.pdllm_chunk_prefill_attn(C.byref(desc), slots_ptr, _stream(q)), "chunk_prefill_attention")
    return out


def describe_prefill_plan(n_chunks: int, num_q_heads: int, num_kv_heads: int, max_seqlen: int, n_tokens: int,
                          causal: bool = True, num_splits: int = 0) -> str:
    """The launch pdllm_chunk_prefill_attn would make for such a batch, as pdllm_attn_plan_describe words it
    (which kernel, grid, team or split).  Needs no device memory."""
    desc = AttnDesc()
    desc.q = desc.k_new = desc.v_new = desc.out = desc.q_start_loc = 16   # non-NULL, aligned; never dereferenced
    d = 128
    desc.q_stride = desc.o_stride = num_q_heads * d
    desc.kn_stride = desc.vn_stride = num_kv_heads * d
    desc.n_tokens, desc.n_req = int(n_tokens), int(n_chunks)
    desc.num_q_heads, desc.num_kv_heads, desc.head_dim = num_q_heads, num_kv_heads, d
    desc.max_q_len, desc.max_ctx_len = int(max_seqlen), 0
    desc.mask_mode = _lib.MASK_CAUSAL if causal else _lib.MASK_FULL
    desc.sm_scale = 1.0 / math.sqrt(d)
    desc.num_splits = int(num_splits)
    text = C.create_string_buffer(256)
    check(lib.pdllm_attn_plan_describe(C.byref(desc), 1, text, 256), "describe_prefill_plan")
    return text.value.decode()


def diffusion_lm_parallel_flash_decoding(query, key, value, output, kv_cache_dtype, key_cache, value_cache,
                                         block_table, query_start_loc, seq_lens, max_seq_len, max_query_len,
                                         k_scale, v_scale, diffusion_blk_sz=32, alibi_slopes=None,
                                         sliding_window=None, sm_scale=None, mask=None, bidirectional=False):
    """Signature of chunked_prefill_paged_decode (chunked_prefill_decoding_unified_kernel.py:220-241).

    seq_lens = context + query length per sequence; the cache is the unified layout.  `mask` is the
    [Nq, Nq] boolean mask over the active rows (block-diagonal per sequence); with `bidirectional`
    and no mask every active key is visible."""
    if alibi_slopes is not None or (sliding_window is not None and sliding_window > 0):
        raise NotImplementedError("alibi / sliding window are not used by the diffusion path")
    if max_query_len <= 1:
        raise NotImplementedError("single-token decode is the causal-LM path, not part of this build")
    if sm_scale is None:
        sm_scale = 1.0 / (query.shape[1] ** 0.5)  # sic: the reference scales by heads here (:243-244)
    qsl = query_start_loc.to(torch.int32)
    ctx = seq_lens.to(torch.int32) - (qsl[1:] - qsl[:-1])
    has_cache = key_cache is not None and key_cache.numel() > 0 and int(max_seq_len) > 0
    max_ctx = int(max_seq_len) if has_cache else 0
    if mask is not None:
        mode = "dense"
    else:
        mode = "full" if bidirectional else "causal"
    ks = k_scale if isinstance(k_scale, torch.Tensor) else None
    vs = v_scale if isinstance(v_scale, torch.Tensor) else None
    if has_cache and key_cache.dtype in (torch.float8_e4m3fn, torch.uint8):
        # the reference passes Python floats (1.0, 1.0): one scalar scale for the whole cache
        if ks is None and k_scale is not None:
            ks = torch.tensor(float(k_scale), dtype=torch.float32, device=key_cache.device)
        if vs is None and v_scale is not None:
            vs = torch.tensor(float(v_scale), dtype=torch.float32, device=key_cache.device)
    sparse_decode_attention(query, key, value, key_cache if has_cache else None,
                            value_cache if has_cache else None, block_table, qsl,
                            max_q_len=int(max_query_len), max_ctx_len=max_ctx, context_lens=ctx,
                            mask_mode=mode, mask=mask, sm_scale=sm_scale, k_scale=ks, v_scale=vs, out=output)


# ----------------------------------------------------------------------------------------
# chunk scoring / selection
# ----------------------------------------------------------------------------------------

def selfinfo_logprob(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """log_softmax(logits.float())[row, label[row]] for bf16 logits [rows, vocab]
    (fastdllm_engine.py:1148-1152)."""
    _need_cuda(logits, labels)
    if logits.dtype != torch.bfloat16 or logits.stride(-1) != 1 or logits.dim() != 2:
        raise ValueError("logits must be bf16 [rows, vocab] with contiguous vocab")
    n, vocab = logits.shape
    labels = labels.to(torch.int64).contiguous()
    out = torch.empty(n, dtype=torch.float32, device=logits.device)
    need = lib.pdllm_vocab_workspace_bytes(n, vocab)
    ws = _workspace(logits.device, int(need))
    check(lib.pdllm_selfinfo_logprob(logits.data_ptr(), logits.stride(0), labels.data_ptr(), n, vocab,
                                     _ptr(ws), 0 if ws is None else ws.numel(), out.data_ptr(),
                                     _stream(logits)), "selfinfo_logprob")
    return out


def chunk_scores_from_logits(logits: torch.Tensor, labels: torch.Tensor, mean: bool = True) -> torch.Tensor:
    """logits [n_chunks, n_labels, vocab] bf16, labels [n_chunks, n_labels] -> score per chunk
    (mean log-probability of the labels, fastdllm_engine.py:1150-1152; sum with mean=False)."""
    c, j, vocab = logits.shape
    lp = selfinfo_logprob(logits.reshape(c * j, vocab), labels.reshape(c * j))
    out = torch.empty(c, dtype=torch.float32, device=logits.device)
    check(lib.pdllm_chunk_score_reduce(lp.data_ptr(), c, j, 1 if mean else 0, out.data_ptr(), _stream(logits)),
          "chunk_scores_from_logits")
    return out


def chunk_select_from_logits(logits: torch.Tensor, labels: torch.Tensor, k: int, mean: bool = True,
                             sorted_ascending: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """chunk_scores_from_logits followed by topk_lowest_index in one library call (two launches):
    logits [n_chunks, n_labels, vocab] bf16, labels [n_chunks, n_labels] -> (scores fp32 [n_chunks],
    indices int64 [min(k, n_chunks)]); fastdllm_engine.py:1148-1152 and 1199-1204."""
    _need_cuda(logits, labels)
    if logits.dtype != torch.bfloat16 or logits.dim() != 3 or not logits.is_contiguous():
        raise ValueError("logits must be contiguous bf16 [n_chunks, n_labels, vocab]")
    c, j, vocab = logits.shape
    k = min(int(k), c)
    if k <= 0:
        raise ValueError("k must be positive")
    labels = labels.to(torch.int64).reshape(c * j).contiguous()
    scores = torch.empty(c, dtype=torch.float32, device=logits.device)
    idx = torch.empty(k, dtype=torch.int64, device=logits.device)
    need = lib.pdllm_vocab_workspace_bytes(c * j, vocab)
    ws = _workspace(logits.device, int(need))
    check(lib.pdllm_chunk_select(logits.data_ptr(), vocab, labels.data_ptr(), c, j, vocab, 1 if mean else 0, k,
                                 1 if sorted_ascending else 0, _ptr(ws), 0 if ws is None else ws.numel(), None,
                                 scores.data_ptr(), idx.data_ptr(), _stream(logits)), "chunk_select_from_logits")
    return scores, idx


def topk_lowest_index(scores: torch.Tensor, k: int, sorted_ascending: bool = True) -> torch.Tensor:
    """Top-k indices per row by (score desc, index asc); non-finite scores rank as -inf
    (fastdllm_engine.py:1199-1204)."""
    _need_cuda(scores)
    squeeze = scores.dim() == 1
    s2 = scores.reshape(1, -1) if squeeze else scores
    if s2.dtype != torch.float32 or s2.stride(-1) != 1:
        s2 = s2.float().contiguous()
    rows, n = s2.shape
    k = min(int(k), n)      # the reference takes ranked[:k] of n chunks
    if k <= 0:
        return torch.empty((0,) if squeeze else (rows, 0), dtype=torch.int64, device=scores.device)
    out = torch.empty((rows, k), dtype=torch.int64, device=scores.device)
    check(lib.pdllm_topk_lowest_index(s2.data_ptr(), rows, n, s2.stride(0), k, 1 if sorted_ascending else 0,
                                      out.data_ptr(), _stream(scores)), "topk_lowest_index")
    return out[0] if squeeze else out


# ----------------------------------------------------------------------------------------
# token eviction
# ----------------------------------------------------------------------------------------

def evict_colsum(probs: torch.Tensor, heads_per_group: Optional[int] = None) -> torch.Tensor:
    """probs [n_chunks, H, Q, K] fp32 -> [n_chunks, H/heads_per_group, K]: per head the sum over
    queries, then the sum over the heads of a group (both in index order)."""
    _need_cuda(probs)
    if probs.dim() == 3:
        probs = probs.unsqueeze(0)
    if probs.dtype != torch.float32 or not probs.is_contiguous():
        raise ValueError("probs must be contiguous fp32 [chunks, heads, queries, keys]")
    c, h, nq, nk = probs.shape
    hpg = h if heads_per_group is None else heads_per_group
    out = torch.empty((c, h // hpg, nk), dtype=torch.float32, device=probs.device)
    ws = _workspace(probs.device, int(lib.pdllm_evict_colsum_workspace_bytes(c, h, nk)))
    check(lib.pdllm_evict_colsum(probs.data_ptr(), c, h, nq, nk, hpg, _ptr(ws), 0 if ws is None else ws.numel(),
                                 out.data_ptr(), _stream(probs)), "evict_colsum")
    return out


def evict_keep_from_probs(probs: torch.Tensor, capacity: int, heads_per_group: Optional[int] = None,
                          keep_high: bool = True, force_keep_first: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """One eviction step from ready-made attention probabilities in one library call: evict_colsum followed by
    topb_keep_bos, same bits (fastdllm_engine.py:1230-1322 summed over queries and heads, then :903-927).
    probs [chunks, H, Q, K] fp32 -> (scores [chunks, groups, K] fp32, keep indices [chunks * groups, keep] int64,
    ascending)."""
    _need_cuda(probs)
    if probs.dim() == 3:
        probs = probs.unsqueeze(0)
    if probs.dtype != torch.float32 or not probs.is_contiguous():
        raise ValueError("probs must be contiguous fp32 [chunks, heads, queries, keys]")
    c, h, nq, nk = probs.shape
    hpg = h if heads_per_group is None else heads_per_group
    if hpg <= 0 or h % hpg:
        raise ValueError(f"{h} heads do not split into groups of {hpg}")
    keep = min(max(1, int(capacity)), nk)
    scores = torch.empty((c, h // hpg, nk), dtype=torch.float32, device=probs.device)
    idx = torch.empty((c * (h // hpg), keep), dtype=torch.int64, device=probs.device)
    ws = _workspace(probs.device, int(lib.pdllm_evict_colsum_workspace_bytes(c, h, nk)))
    check(lib.pdllm_evict_keep_from_probs(probs.data_ptr(), c, h, nq, nk, hpg, int(capacity), 1 if keep_high else 0,
                                          1 if force_keep_first else 0, _ptr(ws), 0 if ws is None else ws.numel(),
                                          scores.data_ptr(), idx.data_ptr(), _stream(probs)), "evict_keep_from_probs")
    return scores, idx


def query_to_chunk_attention_scores(q: torch.Tensor, k: torch.Tensor, *, prefix_len: int, chunk_len: int,
                                    query_len: int, scale: float, reduce_mode: str = "sum",
                                    attention_mask: str = "causal", block_n: int = 64,
                                    block_chunk: int = 64) -> torch.Tensor:
    """Signature and error behaviour of triton_eviction_scorer.py:114-210."""
    if not q.is_cuda or not k.is_cuda:
        raise ValueError("HIP eviction scorer requires device tensors.")
    if q.ndim != 3 or k.ndim != 3:
        raise ValueError(f"Expected q/k as [seq, heads, dim], got {tuple(q.shape)} / {tuple(k.shape)}")
    if chunk_len <= 0 or query_len <= 0:
        return torch.empty(0, device=q.device)
    if int(q.shape[0]) != int(k.shape[0]):
        raise ValueError("q and k must use the same sequence length.")
    hq, hkv, d = int(q.shape[1]), int(k.shape[1]), int(q.shape[2])
    if int(k.shape[2]) != d:
        raise ValueError("q and k must use the same head dimension.")
    if hq % hkv != 0:
        raise ValueError("num_query_heads must be divisible by num_kv_heads.")
    if d > 256:
        raise ValueError(f"Unsupported head_dim for eviction scorer: {d}")
    if query_len > 64:
        raise ValueError(f"query_len={query_len} is too large for the eviction scorer.")
    mask = (attention_mask or "full").lower()
    if mask in {"full", "none", "query_to_chunk"}:
        causal = 0
    elif mask == "causal":
        causal = 1
    else:
        raise ValueError(f"Unsupported token attention mask for scorer: {attention_mask}")
    if int(q.shape[0]) != prefix_len + chunk_len + query_len:
        raise ValueError("sequence length must equal prefix_len + chunk_len + query_len")
    q = q.to(torch.bfloat16).contiguous()
    k = k.to(torch.bfloat16).contiguous()
    out = torch.empty((hq, int(chunk_len)), device=q.device, dtype=torch.float32)
    need = int(lib.pdllm_evict_score_qk_workspace_bytes(prefix_len, chunk_len, query_len, hq, hkv, d))
    if need < 0:
        check(need, "query_to_chunk_attention_scores")
    ws = _workspace(q.device, need)
    check(lib.pdllm_evict_score_qk(q.data_ptr(), k.data_ptr(), prefix_len, chunk_len, query_len, hq, hkv, d,
                                   float(scale), 1 if (reduce_mode or "sum").lower() == "mean" else 0, causal,
                                   ws.data_ptr(), ws.numel(), out.data_ptr(), _stream(q)),
          "query_to_chunk_attention_scores")
    return out


def token_score_pool_group(scores: torch.Tensor, pooling: str = "none", kernel: int = 7,
                           num_kv_heads: Optional[int] = None) -> torch.Tensor:
    """fastdllm_engine.py:1405-1433: pooling over [heads, n] then mean per KV-head group."""
    _need_cuda(scores)
    scores = scores.float().contiguous()
    h, n = scores.shape
    pool = {"none": 0, "maxpool": 1, "avgpool": 2}.get((pooling or "none").lower())
    if pool is None:
        raise ValueError(f"Unsupported token_score_pooling: {pooling}")
    kernel = max(1, min(int(kernel or 1), n))
    groups = h if num_kv_heads is None else int(num_kv_heads)
    if h % groups != 0:
        raise ValueError(f"Cannot group {h} query-head scores into {groups} KV heads.")
    out = torch.empty((groups, n), dtype=torch.float32, device=scores.device)
    check(lib.pdllm_token_score_pool_group(scores.data_ptr(), h, n, pool, kernel, h // groups, out.data_ptr(),
                                           _stream(scores)), "token_score_pool_group")
    return out


def topb_keep_bos(scores: torch.Tensor, capacity: int, keep_high: bool = True,
                  force_keep_first: bool = True) -> torch.Tensor:
    """Rows of scores [rows, chunk_len] -> ascending keep indices [rows, keep_count]
    (fastdllm_engine.py:903-927, ties broken by lowest index)."""
    _need_cuda(scores)
    squeeze = scores.dim() == 1
    s2 = scores.reshape(1, -1) if squeeze else scores
    if s2.dtype != torch.float32 or s2.stride(-1) != 1:
        s2 = s2.float().contiguous()
    rows, n = s2.shape
    keep = min(max(1, int(capacity)), n)
    out = torch.empty((rows, keep), dtype=torch.int64, device=scores.device)
    check(lib.pdllm_topb_keep_bos(s2.data_ptr(), rows, n, s2.stride(0), capacity, 1 if keep_high else 0,
                                  1 if force_keep_first else 0, out.data_ptr(), _stream(scores)), "topb_keep_bos")
    return out[0] if squeeze else out


def vote_histogram(indices: torch.Tensor, length: int) -> torch.Tensor:
    """fp32 [length] counts of how often each position occurs in `indices` (any shape, int64); positions
    outside [0, length) are ignored (preevict_votetopk.sh:231-239)."""
    _need_cuda(indices)
    idx = indices.to(torch.int64).reshape(-1).contiguous()
    votes = torch.zeros(int(length), dtype=torch.float32, device=indices.device)
    check(lib.pdllm_vote_histogram(idx.data_ptr(), idx.numel(), int(length), votes.data_ptr(), _stream(indices)),
          "vote_histogram")
    return votes


# ----------------------------------------------------------------------------------------
# KV gather / scatter (compaction, snapshot, load)
# ----------------------------------------------------------------------------------------

def kv_gather(layer_cache: torch.Tensor, page_ids: torch.Tensor, n_tokens: int,
              token_idx: Optional[torch.Tensor] = None, src_offset: int = 0) -> torch.Tensor:
    """layer_cache [pages, P, Hkv, d] -> dense [n_tokens, Hkv, d]; token j of head h comes from
    logical token token_idx[h, j] + src_offset (or j + src_offset) of the page list."""
    _need_cuda(layer_cache, page_ids)
    if not layer_cache.is_contiguous():
        raise ValueError("cache must be contiguous")
    pages, P, hkv, d = layer_cache.shape
    page_ids = page_ids.to(torch.int32).contiguous()
    out = torch.empty((n_tokens, hkv, d), dtype=layer_cache.dtype, device=layer_cache.device)
    idx_ptr, stride = None, 0
    if token_idx is not None:
        token_idx = token_idx.to(torch.int64).contiguous()
        if token_idx.dim() == 1:
            stride = 0
        else:
            assert token_idx.shape[0] == hkv
            stride = token_idx.stride(0)
        assert token_idx.shape[-1] == n_tokens
        idx_ptr = token_idx.data_ptr()
    check(lib.pdllm_kv_gather(layer_cache.data_ptr(), page_ids.data_ptr(), page_ids.numel(), idx_ptr, stride,
                              src_offset, n_tokens, hkv, d, P, pages, layer_cache.element_size(),
                              out.data_ptr(), _stream(layer_cache)), "kv_gather")
    return out


def kv_scatter(layer_cache: torch.Tensor, page_ids: torch.Tensor, src: torch.Tensor, dst_start: int = 0) -> None:
    """cache[page_ids[(dst_start+j)/P], (dst_start+j)%P] = src[j] for dense src [n, Hkv, d]."""
    _need_cuda(layer_cache, page_ids, src)
    if not layer_cache.is_contiguous():
        raise ValueError("cache must be contiguous")
    pages, P, hkv, d = layer_cache.shape
    src = src.to(layer_cache.dtype).contiguous()
    if tuple(src.shape[1:]) != (hkv, d):
        raise ValueError(f"shape mismatch: src {tuple(src.shape)} cache heads/dim {(hkv, d)}")
    page_ids = page_ids.to(torch.int32).contiguous()
    check(lib.pdllm_kv_scatter(layer_cache.data_ptr(), page_ids.data_ptr(), page_ids.numel(), dst_start,
                               src.shape[0], hkv, d, P, pages, layer_cache.element_size(), src.data_ptr(),
                               _stream(layer_cache)), "kv_scatter")


def kv_compact_per_head(kv_cache: torch.Tensor, page_ids: torch.Tensor, keep: torch.Tensor,
                        max_workspace_bytes: int = 256 << 20) -> None:
    """In place on the unified cache kv_cache [2, layers, n_pages, page_size, Hkv, d]: token j of KV head h of
    layer l <- token keep[l, h, j] of the request's pages, for K and V (fastdllm_engine.py:607-638 for all layers:
    two launches per round of layers instead of two per layer and tensor).  keep: int64 [layers, Hkv, n_keep]."""
    _need_cuda(kv_cache, page_ids, keep)
    if kv_cache.dim() != 6 or not kv_cache.is_contiguous() or kv_cache.shape[0] != 2:
        raise ValueError("kv_cache must be contiguous [2, layers, n_pages, page_size, Hkv, d]")
    _, layers, n_pages, P, hkv, d = kv_cache.shape
    keep = keep.to(torch.int64).contiguous()
    if keep.dim() != 3 or keep.shape[0] != layers or keep.shape[1] != hkv:
        raise ValueError(f"keep must be [layers, Hkv, n_keep] = [{layers}, {hkv}, n], got {tuple(keep.shape)}")
    n_keep = int(keep.shape[2])
    if n_keep == 0:
        return
    page_ids = page_ids.to(torch.int32).contiguous()
    esz = kv_cache.element_size()
    per_layer = int(lib.pdllm_kv_compact_per_head_workspace_bytes(n_keep, hkv, d, esz))
    ws = _workspace(kv_cache.device, min(max(per_layer, int(max_workspace_bytes)), per_layer * layers))
    check(lib.pdllm_kv_compact_per_head(kv_cache.data_ptr(), kv_cache.stride(1) * esz, layers, page_ids.data_ptr(),
                                        page_ids.numel(), keep.data_ptr(), keep.stride(0), keep.stride(1), n_keep,
                                        hkv, d, P, n_pages, esz, ws.data_ptr(), ws.numel(), _stream(kv_cache)),
          "kv_compact_per_head")


def kv_copy_pages(src_kv_cache: torch.Tensor, dst_kv_cache: torch.Tensor, src_page_ids: torch.Tensor,
                  dst_page_ids: torch.Tensor) -> None:
    """dst[:, :, dst_page_ids[i]] = src[:, :, src_page_ids[i]] for two unified caches
    [2, layers, n_pages, page_size, Hkv, d] of the same page geometry and dtype, all layers in one
    launch (the page-granular form of the copies in fastdllm_engine.py:845-859)."""
    _need_cuda(src_kv_cache, dst_kv_cache, src_page_ids, dst_page_ids)
    if src_kv_cache.dim() != 6 or dst_kv_cache.dim() != 6 or not src_kv_cache.is_contiguous() or \
            not dst_kv_cache.is_contiguous():
        raise ValueError("caches must be contiguous [2, layers, n_pages, page_size, Hkv, d]")
    if src_kv_cache.shape[:2] != dst_kv_cache.shape[:2] or src_kv_cache.shape[3:] != dst_kv_cache.shape[3:] or \
            src_kv_cache.dtype != dst_kv_cache.dtype:
        raise ValueError("source and destination caches differ in layers, page geometry or dtype")
    if src_page_ids.numel() != dst_page_ids.numel():
        raise ValueError("page id lists differ in length")
    sp = src_page_ids.to(torch.int32).contiguous()
    dp = dst_page_ids.to(torch.int32).contiguous()
    planes = src_kv_cache.shape[0] * src_kv_cache.shape[1]
    page_bytes = src_kv_cache.stride(2) * src_kv_cache.element_size()
    check(lib.pdllm_kv_copy_pages(src_kv_cache.data_ptr(), dst_kv_cache.data_ptr(), sp.data_ptr(), dp.data_ptr(),
                                  sp.numel(), page_bytes, planes,
                                  src_kv_cache.stride(1) * src_kv_cache.element_size(),
                                  dst_kv_cache.stride(1) * dst_kv_cache.element_size(),
                                  src_kv_cache.shape[2], dst_kv_cache.shape[2], _stream(dst_kv_cache)),
          "kv_copy_pages")


# ----------------------------------------------------------------------------------------
# confidence / unmask / rope
# ----------------------------------------------------------------------------------------

def conf_argmax(logits: torch.Tensor, block_len: int, shift: bool = False,
                last_logit: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 logits [n_seqs*block_len, vocab] -> (confidence fp32, token int64) per row:
    max softmax probability in fp32 and its first index (fastdllm_engine.py:1658-1681, T=0),
    reading rows through the Dream logit shift of :1647-1656 when shift is set."""
    _need_cuda(logits)
    if logits.dtype != torch.bfloat16 or logits.stride(-1) != 1 or logits.dim() != 2:
        raise ValueError("logits must be bf16 [rows, vocab]")
    rows, vocab = logits.shape
    if rows % block_len:
        raise ValueError("rows must be a multiple of block_len")
    n_seqs = rows // block_len
    ll_ptr, ll_stride = None, 0
    if last_logit is not None:
        last_logit = last_logit.to(torch.bfloat16).reshape(n_seqs, vocab).contiguous()
        ll_ptr, ll_stride = last_logit.data_ptr(), last_logit.stride(0)
    conf = torch.empty(rows, dtype=torch.float32, device=logits.device)
    tok = torch.empty(rows, dtype=torch.int64, device=logits.device)
    need = lib.pdllm_vocab_workspace_bytes(rows, vocab)
    ws = _workspace(logits.device, int(need))
    check(lib.pdllm_conf_argmax(logits.data_ptr(), logits.stride(0), ll_ptr, ll_stride, n_seqs, block_len, vocab,
                                1 if shift else 0, _ptr(ws), 0 if ws is None else ws.numel(), conf.data_ptr(),
                                tok.data_ptr(), _stream(logits)), "conf_argmax")
    return conf, tok


def threshold_unmask(conf: torch.Tensor, token: torch.Tensor, block_ids: torch.Tensor, mask_token_id: int,
                     threshold: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """In-place transfer rule of fastdllm_engine.py:2146-2157 for block_ids [n_seqs, block_len] int64.
    Returns (transfer bool [n_seqs, block_len], masked positions left int32 [n_seqs])."""
    _need_cuda(conf, token, block_ids)
    if block_ids.dtype != torch.int64 or not block_ids.is_contiguous():
        raise ValueError("block_ids must be contiguous int64")
    n_seqs, block_len = block_ids.shape
    conf = conf.float().contiguous()
    token = token.to(torch.int64).contiguous()
    transfer = torch.empty((n_seqs, block_len), dtype=torch.uint8, device=block_ids.device)
    left = torch.empty(n_seqs, dtype=torch.int32, device=block_ids.device)
    check(lib.pdllm_threshold_unmask(conf.data_ptr(), token.data_ptr(), block_ids.data_ptr(), n_seqs, block_len,
                                     int(mask_token_id), float(threshold), transfer.data_ptr(), left.data_ptr(),
                                     _stream(block_ids)), "threshold_unmask")
    return transfer.view(torch.bool), left


def denoise_unmask(logits: torch.Tensor, block_ids: torch.Tensor, mask_token_id: int, threshold: float,
                   shift: bool = False, last_logit: Optional[torch.Tensor] = None
                   ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """conf_argmax followed by threshold_unmask in one library call (two launches, no host sync):
    bf16 logits [n_seqs*block_len, vocab], block_ids int64 [n_seqs, block_len] updated in place.
    Returns (confidence fp32 [rows], token int64 [rows], transfer bool [n_seqs, block_len], masked left int32
    [n_seqs]); fastdllm_engine.py:1647-1681 and 2146-2157."""
    _need_cuda(logits, block_ids)
    if logits.dtype != torch.bfloat16 or logits.stride(-1) != 1 or logits.dim() != 2:
        raise ValueError("logits must be bf16 [rows, vocab]")
    if block_ids.dtype != torch.int64 or not block_ids.is_contiguous() or block_ids.dim() != 2:
        raise ValueError("block_ids must be contiguous int64 [n_seqs, block_len]")
    rows, vocab = logits.shape
    n_seqs, block_len = block_ids.shape
    if rows != n_seqs * block_len:
        raise ValueError("logits rows must equal n_seqs * block_len")
    ll_ptr, ll_stride = None, 0
    if last_logit is not None:
        last_logit = last_logit.to(torch.bfloat16).reshape(n_seqs, vocab).contiguous()
        ll_ptr, ll_stride = last_logit.data_ptr(), last_logit.stride(0)
    dev = logits.device
    conf = torch.empty(rows, dtype=torch.float32, device=dev)
    tok = torch.empty(rows, dtype=torch.int64, device=dev)
    transfer = torch.empty((n_seqs, block_len), dtype=torch.uint8, device=dev)
    left = torch.empty(n_seqs, dtype=torch.int32, device=dev)
    need = lib.pdllm_vocab_workspace_bytes(rows, vocab)
    ws = _workspace(dev, int(need))
    check(lib.pdllm_denoise_unmask(logits.data_ptr(), logits.stride(0), ll_ptr, ll_stride, n_seqs, block_len, vocab,
                                   1 if shift else 0, block_ids.data_ptr(), int(mask_token_id), float(threshold),
                                   _ptr(ws), 0 if ws is None else ws.numel(), conf.data_ptr(), tok.data_ptr(),
                                   transfer.data_ptr(), left.data_ptr(), _stream(logits)), "denoise_unmask")
    return conf, tok, transfer.view(torch.bool), left


class PreparedDenoiseUnmask:
    """denoise_unmask with everything a step needs resolved once: the engine runs it after every model
    forward on the same logits buffer and block, so outputs and workspace are allocated here and run()
    is one library call (fastdllm_engine.py:2133-2157 without its host syncs)."""

    def __init__(self, logits: torch.Tensor, block_ids: torch.Tensor, mask_token_id: int, threshold: float,
                 shift: bool = False, last_logit: Optional[torch.Tensor] = None):
        _need_cuda(logits, block_ids)
        if logits.dtype != torch.bfloat16 or logits.stride(-1) != 1 or logits.dim() != 2:
            raise ValueError("logits must be bf16 [rows, vocab]")
        if block_ids.dtype != torch.int64 or not block_ids.is_contiguous() or block_ids.dim() != 2:
            raise ValueError("block_ids must be contiguous int64 [n_seqs, block_len]")
        rows, vocab = logits.shape
        n_seqs, block_len = block_ids.shape
        if rows != n_seqs * block_len:
            raise ValueError("logits rows must equal n_seqs * block_len")
        dev = logits.device
        self.logits, self.block_ids = logits, block_ids
        self.last_logit = None
        ll_ptr, ll_stride = None, 0
        if last_logit is not None:
            self.last_logit = last_logit.to(torch.bfloat16).reshape(n_seqs, vocab).contiguous()
            ll_ptr, ll_stride = self.last_logit.data_ptr(), self.last_logit.stride(0)
        self.conf = torch.empty(rows, dtype=torch.float32, device=dev)
        self.token = torch.empty(rows, dtype=torch.int64, device=dev)
        self._transfer = torch.empty((n_seqs, block_len), dtype=torch.uint8, device=dev)
        self.transfer = self._transfer.view(torch.bool)
        self.left = torch.empty(n_seqs, dtype=torch.int32, device=dev)
        need = int(lib.pdllm_vocab_workspace_bytes(rows, vocab))
        self._ws = torch.empty(max(need, 8), dtype=torch.uint8, device=dev)
        self._args = (logits.data_ptr(), logits.stride(0), ll_ptr, ll_stride, n_seqs, block_len, vocab,
                      1 if shift else 0, block_ids.data_ptr(), int(mask_token_id), float(threshold),
                      self._ws.data_ptr(), self._ws.numel(), self.conf.data_ptr(), self.token.data_ptr(),
                      self._transfer.data_ptr(), self.left.data_ptr())

    def run(self, stream: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """Updates block_ids in place; returns (transfer mask, masked positions left)."""
        st = lib.pdllm_denoise_unmask(*self._args,
                                      torch.cuda.current_stream().cuda_stream if stream is None else stream)
        if st != 0:
            check(st, "PreparedDenoiseUnmask.run")
        return self.transfer, self.left


def rope_inplace(x: torch.Tensor, positions: torch.Tensor, cos_sin_cache: torch.Tensor) -> torch.Tensor:
    """neox rotary embedding (layers/rotary_embedding.py:6-17, 39-65) in place on bf16 x [n, heads, d]."""
    _need_cuda(x, positions, cos_sin_cache)
    n, h, d = x.shape
    if x.dtype != torch.bfloat16 or x.stride(-1) != 1 or x.stride(1) != d:
        raise ValueError("x must be bf16 [tokens, heads, d] with contiguous heads")
    positions = positions.to(torch.int64).contiguous()
    cs = cos_sin_cache.float().contiguous()
    check(lib.pdllm_rope_inplace(x.data_ptr(), x.stride(0), positions.data_ptr(), cs.data_ptr(), cs.shape[0], n, h,
                                 d, _stream(x)), "rope_inplace")
    return x


def rope_qk_store(q: torch.Tensor, k: torch.Tensor, v: Optional[torch.Tensor], positions: torch.Tensor,
                  cos_sin_cache: torch.Tensor, k_cache: Optional[torch.Tensor] = None,
                  v_cache: Optional[torch.Tensor] = None, slot_mapping: Optional[torch.Tensor] = None) -> None:
    """rope_inplace on q and k and store_kvcache_unified_layout of (rotated k, v) in one launch
    (layers/rotary_embedding.py:39-65 then kv_cache_kernels.py:150-172).  q [n, Hq, d], k / v [n, Hkv, d]
    bf16; without slot_mapping only the rotation is done."""
    _need_cuda(q, k, positions, cos_sin_cache)
    n, hq, d = q.shape
    hkv = k.shape[1]
    for name, x in (("q", q), ("k", k)) + ((("v", v),) if v is not None else ()):
        if x.dtype != torch.bfloat16 or x.stride(-1) != 1 or x.stride(1) != d or x.shape[0] != n or x.shape[2] != d:
            raise ValueError(f"{name} must be bf16 [tokens, heads, d] with contiguous heads")
    positions = positions.to(torch.int64).contiguous()
    cs = cos_sin_cache.float().contiguous()
    slots_ptr, n_slots, kc_ptr, vc_ptr, v_ptr, v_stride = None, 0, None, None, None, 0
    if slot_mapping is not None:
        if v is None or k_cache is None or v_cache is None:
            raise ValueError("slot_mapping needs v and both caches")
        if not k_cache.is_contiguous() or not v_cache.is_contiguous() or k_cache.dtype != torch.bfloat16 or \
                tuple(k_cache.shape[2:]) != (hkv, d):
            raise ValueError("the fused store needs contiguous bf16 unified caches [pages, page_size, Hkv, d]")
        slot_mapping = slot_mapping.to(torch.int32).contiguous()
        if slot_mapping.numel() != n:
            raise ValueError("slot_mapping must have one entry per token")
        slots_ptr, n_slots = slot_mapping.data_ptr(), k_cache.shape[0] * k_cache.shape[1]
        kc_ptr, vc_ptr, v_ptr, v_stride = k_cache.data_ptr(), v_cache.data_ptr(), v.data_ptr(), v.stride(0)
    check(lib.pdllm_rope_qk_store(q.data_ptr(), q.stride(0), hq, k.data_ptr(), k.stride(0), v_ptr, v_stride, hkv, d,
                                  positions.data_ptr(), cs.data_ptr(), cs.shape[0], n, kc_ptr, vc_ptr, slots_ptr,
                                  n_slots, _stream(q)), "rope_qk_store")


# ----------------------------------------------------------------------------------------------
# anchor corrections of the attention output
# ----------------------------------------------------------------------------------------------

def anchor_params(state: dict, seq_len: int) -> Optional[Tuple[int, int, int, int, int]]:
    """(stride, anchor_offset, left, right, direction) from a decode-delta / sparse-prefill state dict with the
    reference's defaults and clamps (attention_v4.py:113-125, 226-236), or None when the sequence has no anchor.
    direction: 0 left, 1 right, 2 both."""
    stride = max(1, int(state.get("stride", 4)))
    left = max(0, int(state.get("left", stride - 1)))
    right = max(0, int(state.get("right", 0)))
    direction = {"right": 1, "both": 2}.get((state.get("direction") or "left").lower(), 0)
    anchor_offset = int(state.get("anchor_offset", stride - 1))
    if anchor_offset < 0:
        anchor_offset = stride - 1
    anchor_offset = min(anchor_offset, stride - 1)
    if seq_len <= anchor_offset:
        return None
    return stride, anchor_offset, left, right, direction


def anchor_delta_add(base: torch.Tensor, dense: Optional[torch.Tensor], q_start_loc: torch.Tensor, *, max_q_len: int,
                     stride: int, anchor_offset: int, left: int, right: int, direction: int, scale: float = 1.0,
                     sel: Optional[torch.Tensor] = None, sel_counts: Optional[torch.Tensor] = None,
                     sel_scale: float = 1.0, sel_mode: str = "none") -> torch.Tensor:
    """base + the window sums of the anchor deltas (attention_v4.py:139-166, 263-293), rounded to bf16 where the
    reference's bf16 tensor operations round.  base / dense [n_rows, heads, d] bf16 (dense is read at the anchor rows
    only); sel [n_sel_rows, heads, d] bf16 with sel_mode "replace" / "add".  Returns a new tensor."""
    _need_cuda(base, q_start_loc)
    mode = {"none": 0, "replace": 1, "add": 2}[sel_mode]
    rows = base.shape[0]
    row_elems = base.numel() // max(rows, 1)
    b2 = base.reshape(rows, row_elems)
    if b2.dtype != torch.bfloat16 or b2.stride(-1) != 1:
        raise ValueError("base must be bf16 with contiguous rows")
    out = torch.empty_like(b2)

    def rows_of(t, name):
        if t is None:
            return None, 0, 0
        t2 = t.reshape(t.shape[0], row_elems)
        if t2.dtype != torch.bfloat16 or t2.stride(-1) != 1:
            raise ValueError(f"{name} must be bf16 with contiguous rows of {row_elems} elements")
        return t2, t2.stride(0), t2.shape[0]

    d2, d_stride, d_rows = rows_of(dense, "dense")
    if d2 is not None and d_rows != rows:
        raise ValueError("dense must have one row per base row")
    s2, s_stride, s_rows = rows_of(sel, "sel")
    cnt = None if sel_counts is None else sel_counts.to(device=base.device, dtype=torch.int64).contiguous()
    if cnt is not None and cnt.numel() < s_rows:
        raise ValueError("sel_counts must have one entry per selection row")
    qsl = q_start_loc.to(torch.int32).contiguous()
    check(lib.pdllm_anchor_delta_add(b2.data_ptr(), b2.stride(0), _ptr(d2), d_stride, _ptr(s2), s_stride, s_rows,
                                     _ptr(cnt), out.data_ptr(), out.stride(0), qsl.data_ptr(), qsl.numel() - 1,
                                     int(max_q_len), rows, row_elems, int(stride), int(anchor_offset), int(left), int(right),
                                     int(direction), float(scale), float(sel_scale), mode, _stream(base)),
          "anchor_delta_add")
    return out.view(base.shape)
