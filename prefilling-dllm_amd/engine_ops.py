"""Host-side mirror of the tensor-math helpers of the reference engine (fastdllm_engine.py) on top of
the HIP operators: chunk ranking, token keep-set selection, per-head KV compaction, KV snapshot /
load, chunk-local KV copy and the confidence-threshold unmask step.  Names, argument meaning and
error behaviour follow the reference methods (cited per function; ENG = fastdllm_engine.py).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import ops
from .page_pool import PageAllocator, PagePool, PrefixPageAllocator, _CachedPrefix  # noqa: F401  (re-exported)

PAGE_SIZE = ops.PAGE_SIZE


# ------------------------------------------------------------------------------------------
# PD boundary types (ENG:33-61) -- field for field
# ------------------------------------------------------------------------------------------

@dataclass
class FastDLLMEngineOutput:
    text: str
    token_ids: List[int]
    n_diff_steps: int


@dataclass
class DreamPrefillRecord:
    """Boundary state between prefill and decode (ENG:33-49)."""

    prompt_ids: List[int]
    prompt_positions: List[int]
    suffix_positions: List[int]
    prompt_len: int
    full_prompt_len: int
    decode_len: int
    prompt_page_ids: List[int]
    block_page_ids: List[int]
    first_token_id: int
    last_context_logit: Optional[torch.Tensor]
    decode_delta_state: Optional[dict]
    owns_prompt_pages: bool
    cached_prefix: Optional["_CachedPrefix"] = None
    kv_mode: str = "full_dense"


@dataclass
class DreamKVSnapshot:
    """Transferable prompt KV payload (ENG:52-61): per layer [prompt_len, Hkv, d]."""

    prompt_len: int
    page_size: int
    kv_mode: str
    k_by_layer: List[torch.Tensor]
    v_by_layer: List[torch.Tensor]
    last_context_logit: Optional[torch.Tensor] = None


# ------------------------------------------------------------------------------------------
# chunk ranking (ENG:1199-1204)
# ------------------------------------------------------------------------------------------

def split_token_chunks(token_ids: Sequence[int], chunk_size: int, split_from_tail: bool = False) -> List[List[int]]:
    """Prompt -> consecutive chunks of chunk_size tokens (prefilling_dllm_eval/fastdllm_parallelcomp.py:158-180).
    The short chunk is the last one, or the first one with split_from_tail; a non-positive chunk_size or a prompt
    that fits gives one chunk, an empty prompt none."""
    ids = list(token_ids)
    n = len(ids)
    if n == 0:
        return []
    if chunk_size <= 0 or n <= chunk_size:
        return [ids]
    first = n % chunk_size if split_from_tail else 0
    cuts = ([0] if first else []) + list(range(first, n, chunk_size)) + [n]
    return [ids[a:b] for a, b in zip(cuts[:-1], cuts[1:])]


def select_chunks_from_scores(scores: torch.Tensor, topk_chunks: int, keep_first_chunk: bool = False) -> torch.Tensor:
    """Ranking tail of select_chunks_by_engine: non-finite -> -inf, stable descending order
    (lowest index first on ties), the top `topk_chunks` of the non-forced chunks plus chunk 0 when
    keep_first_chunk, returned in ascending chunk order.  scores: device fp32 [n_chunks]."""
    n = int(scores.numel())
    if n == 0:
        return torch.empty(0, dtype=torch.int64, device=scores.device)
    scores = scores.float().reshape(-1)
    if keep_first_chunk:
        rest = scores[1:]
        k = rest.numel() if int(topk_chunks or 0) <= 0 else min(int(topk_chunks), rest.numel())
        if k == 0:
            return torch.zeros(1, dtype=torch.int64, device=scores.device)
        sel = ops.topk_lowest_index(rest.contiguous(), k, sorted_ascending=True) + 1
        return torch.cat([torch.zeros(1, dtype=torch.int64, device=scores.device), sel])
    k = n if int(topk_chunks or 0) <= 0 else min(int(topk_chunks), n)
    return ops.topk_lowest_index(scores.contiguous(), k, sorted_ascending=True)


def select_chunks_from_logits(logits: torch.Tensor, labels: torch.Tensor, topk_chunks: int,
                              mean: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """score_chunk_self_information_engine (ENG:1098-1152) for all chunks of a draft round and the
    ranking of select_chunks_by_engine (ENG:1199-1204) in one library call: logits
    [n_chunks, n_labels, vocab] bf16 (the rows that predict the labels), labels [n_chunks, n_labels].
    Returns (scores fp32 [n_chunks], selected chunk indices ascending)."""
    n = int(logits.shape[0])
    k = n if int(topk_chunks or 0) <= 0 else min(int(topk_chunks), n)
    return ops.chunk_select_from_logits(logits, labels, k, mean=mean, sorted_ascending=True)


# ------------------------------------------------------------------------------------------
# token keep set (ENG:903-927)
# ------------------------------------------------------------------------------------------

def select_positions_from_token_scores(token_scores: torch.Tensor, *, capacity: int, chunk_len: int,
                                       keep_high: bool = True, force_keep_first: bool = True) -> torch.Tensor:
    """_select_positions_from_token_scores with ties broken by lowest index.  token_scores is one
    row [chunk_len] or a batch [rows, chunk_len] on the device."""
    keep_count = min(max(1, int(capacity)), int(chunk_len))
    if token_scores.shape[-1] != chunk_len:
        head = keep_count // 2
        tail = keep_count - head
        keep = sorted(set(list(range(head)) + list(range(chunk_len - tail, chunk_len))))
        return torch.tensor(keep[:keep_count], device=token_scores.device, dtype=torch.long)
    return ops.topb_keep_bos(token_scores, capacity, keep_high=keep_high,
                             force_keep_first=force_keep_first and chunk_len > 0)


# ------------------------------------------------------------------------------------------
# compaction / snapshot / load / chunk-local copy (ENG:525-558, 607-698)
# ------------------------------------------------------------------------------------------

def preevict_vote_topk_indices(keep_indices_per_layer_per_head: Sequence[torch.Tensor], full_prompt_len: int,
                               chunk_spans: Sequence[Tuple[int, int]], capacity: int) -> torch.Tensor:
    """Vote variant of the keep set (preevict_votetopk.sh:231-258): every (layer, KV head) votes for the
    positions it kept; inside each chunk [start, end) the first token and the capacity - 1 positions with the
    most votes (lowest index on ties) survive, tokens outside the chunks always do.  keep_indices: one int64
    tensor [heads, keep] of prompt positions per layer (device).  Returns ascending int64 positions."""
    n = int(full_prompt_len)
    dev = keep_indices_per_layer_per_head[0].device if len(keep_indices_per_layer_per_head) else None
    if n <= 0:
        return torch.empty(0, dtype=torch.int64, device=dev)
    if dev is None:
        return torch.arange(n, dtype=torch.int64)
    votes = ops.vote_histogram(torch.cat([k.reshape(-1) for k in keep_indices_per_layer_per_head]), n)
    cap = int(capacity or 0)
    keep = torch.zeros(n, dtype=torch.bool, device=dev)
    cursor = 0
    by_len: Dict[int, List[int]] = {}
    for start, end in chunk_spans:
        start, end = int(start), int(end)
        if start > cursor:
            keep[cursor:start] = True
        if end > start:
            by_len.setdefault(end - start, []).append(start)
        cursor = end
    if cursor < n:
        keep[cursor:] = True
    for length, starts in by_len.items():
        if cap <= 0 or cap >= length:
            for s0 in starts:
                keep[s0:s0 + length] = True
            continue
        st = torch.as_tensor(starts, dtype=torch.int64, device=dev)
        rows = votes[(st[:, None] + torch.arange(length, device=dev)[None, :])]       # [chunks, length]
        sel = ops.topb_keep_bos(rows.contiguous(), max(1, cap)) + st[:, None]
        keep[sel.reshape(-1)] = True
    if not bool(keep.any()):
        keep[:] = True
    return torch.nonzero(keep).reshape(-1)


def compact_prompt_cache_per_head(layer_cache: torch.Tensor, page_ids: torch.Tensor, keep: torch.Tensor) -> int:
    """One layer, one of K/V: token j of head h <- token keep[h][j]; gather completes before the
    write (the reference clones), so overlapping source and destination slots are safe."""
    active_len = int(keep.shape[1])
    if active_len <= 0:
        return 0
    compacted = ops.kv_gather(layer_cache, page_ids, active_len, token_idx=keep)
    ops.kv_scatter(layer_cache, page_ids, compacted, dst_start=0)
    return active_len


def _as_one_stack(tensors: Sequence[torch.Tensor], device) -> Optional[torch.Tensor]:
    """The [L, H, n] tensor the given per-layer tensors are consecutive slices of, or None.  normalize_per_head_keep_indices
    returns such slices (as the reference's engine passes the output of its _normalize_per_head_keep_indices on to
    the compaction, ENG:1940 -> 2081): stacking them again would copy 28 tensors for nothing."""
    first = tensors[0]
    if not isinstance(first, torch.Tensor) or first.dtype != torch.long or first.device != torch.device(device) \
            or first.dim() != 2 or not first.is_contiguous():
        return None
    step = first.numel()
    store = first.untyped_storage().data_ptr()
    for l, t in enumerate(tensors):
        if (not isinstance(t, torch.Tensor) or t.dtype != torch.long or t.device != first.device or t.shape != first.shape
                or not t.is_contiguous() or t.untyped_storage().data_ptr() != store
                or t.storage_offset() != first.storage_offset() + l * step):
            return None
    return torch.as_strided(first, (len(tensors),) + tuple(first.shape), (step, first.shape[1], 1))


def compact_prompt_cache_per_layer_per_head(kv_cache: torch.Tensor, prompt_page_ids: Sequence[int],
                                            keep_indices_per_layer_per_head: Sequence[torch.Tensor]) -> int:
    """_compact_prompt_cache_per_layer_per_head (ENG:607-638) on kv_cache [2, L, pages, P, Hkv, d]: all layers, K and
    V in one library call."""
    if not keep_indices_per_layer_per_head:
        return 0
    page_ids = torch.as_tensor(list(prompt_page_ids), dtype=torch.int32, device=kv_cache.device)
    active_len = int(keep_indices_per_layer_per_head[0].shape[1])
    if active_len <= 0:
        return 0
    keep = _as_one_stack(keep_indices_per_layer_per_head, kv_cache.device)
    if keep is None:
        keep = torch.stack([k.to(device=kv_cache.device, dtype=torch.long) for k in keep_indices_per_layer_per_head])
    if kv_cache.is_contiguous() and keep.shape[0] == kv_cache.shape[1]:
        ops.kv_compact_per_head(kv_cache, page_ids, keep)
    else:       # a view of a larger cache, or fewer keep lists than layers: layer by layer
        for layer_idx in range(keep.shape[0]):
            for kv in range(2):
                compact_prompt_cache_per_head(kv_cache[kv, layer_idx], page_ids, keep[layer_idx])
    return active_len


def normalize_per_head_keep_indices(keep_indices_per_layer_per_head, *, num_layers: int, num_heads: int,
                                    full_prompt_len: int, device) -> Tuple[List[torch.Tensor], int]:
    """The contract of _normalize_per_head_keep_indices (ENG:560-605): `num_layers` index tensors
    [num_heads, active_len] of one common active_len with entries in [0, full_prompt_len); returns them as
    contiguous int64 tensors on `device` and the active length.  Any violation is a ValueError that names the
    first offending layer.

    The layers are stacked into one [L, H, n] tensor, so the range check is one pass over all of them and one
    transfer to the host instead of two per layer."""
    given = list(keep_indices_per_layer_per_head)
    if len(given) != num_layers:
        raise ValueError(f"keep indices for {len(given)} layers were passed, the model has {num_layers}")
    if num_layers == 0:
        return [], 0
    per_layer = [torch.as_tensor(x, dtype=torch.long, device=device) for x in given]
    shapes = [tuple(t.shape) for t in per_layer]
    want_tail = shapes[0][1:] if len(shapes[0]) == 2 else None
    for l, shp in enumerate(shapes):
        if len(shp) != 2 or shp[0] != num_heads:
            raise ValueError(f"layer {l}: keep indices have shape {shp}, expected [{num_heads}, active_len]")
        if shp[1:] != want_tail:
            raise ValueError(f"layer {l}: {shp[1]} kept tokens per head, layer 0 keeps {want_tail[0]}")
    stacked = torch.stack(per_layer)                                   # [L, H, n]
    n_keep = int(stacked.shape[2])
    if n_keep > 0:
        bad = ((stacked < 0) | (stacked >= full_prompt_len)).flatten(1).any(dim=1)   # [L]
        bad_layers = torch.nonzero(bad).flatten().tolist()                          # the one host transfer
        if bad_layers:
            raise ValueError(f"layer {bad_layers[0]}: a keep index lies outside the prompt of {full_prompt_len} tokens")
    return list(stacked.unbind(0)), n_keep


def snapshot_prompt_cache_per_layer(kv_cache: torch.Tensor, prompt_page_ids: Sequence[int],
                                    prompt_len: int) -> Tuple[List[torch.Tensor], List[torch.Tensor]]:
    """_snapshot_prompt_cache_per_layer (ENG:640-662): per layer [prompt_len, Hkv, d] for K and V."""
    if prompt_len <= 0:
        return [], []
    page_ids = torch.as_tensor(list(prompt_page_ids), dtype=torch.int32, device=kv_cache.device)
    full_k = [ops.kv_gather(kv_cache[0, l], page_ids, int(prompt_len)) for l in range(kv_cache.shape[1])]
    full_v = [ops.kv_gather(kv_cache[1, l], page_ids, int(prompt_len)) for l in range(kv_cache.shape[1])]
    return full_k, full_v


def load_prompt_cache_per_layer(kv_cache: torch.Tensor, prompt_page_ids: Sequence[int], prompt_len: int,
                                k_by_layer: Sequence[torch.Tensor], v_by_layer: Sequence[torch.Tensor]) -> None:
    """_load_prompt_cache_per_layer (ENG:664-698) with its shape checks."""
    if prompt_len <= 0:
        return
    L = int(kv_cache.shape[1])
    if len(k_by_layer) != L or len(v_by_layer) != L:
        raise ValueError(f"PD KV snapshot layer count mismatch: k={len(k_by_layer)} v={len(v_by_layer)} expected={L}")
    page_ids = torch.as_tensor(list(prompt_page_ids), dtype=torch.int32, device=kv_cache.device)
    expected = (int(prompt_len), int(kv_cache.shape[4]), int(kv_cache.shape[5]))
    for l, (lk, lv) in enumerate(zip(k_by_layer, v_by_layer)):
        lk = lk.to(device=kv_cache.device, dtype=kv_cache.dtype)
        lv = lv.to(device=kv_cache.device, dtype=kv_cache.dtype)
        if tuple(lk.shape) != expected or tuple(lv.shape) != expected:
            raise ValueError(f"PD KV snapshot shape mismatch at layer {l}: k={tuple(lk.shape)} "
                             f"v={tuple(lv.shape)} expected={expected}")
        ops.kv_scatter(kv_cache[0, l], page_ids, lk)
        ops.kv_scatter(kv_cache[1, l], page_ids, lv)


def snapshot_pd_record_kv(kv_cache: torch.Tensor, record: DreamPrefillRecord, *, page_size: int = PAGE_SIZE,
                          device="cpu") -> DreamKVSnapshot:
    """snapshot_pd_record_kv (ENG:700-726): gather the record's prompt KV and move it to `device`."""
    k, v = snapshot_prompt_cache_per_layer(kv_cache, record.prompt_page_ids, record.prompt_len)
    ll = record.last_context_logit
    return DreamKVSnapshot(prompt_len=record.prompt_len, page_size=page_size, kv_mode=record.kv_mode,
                           k_by_layer=[t.to(device) for t in k], v_by_layer=[t.to(device) for t in v],
                           last_context_logit=None if ll is None else ll.to(device))


def _allocate_record_pages(allocator: PageAllocator, prompt_len: int, decode_len: int,
                           page_size: int) -> Tuple[List[int], List[int]]:
    """Pages for a record on the decode side: evict unreferenced cached prefixes until both lists fit
    (ENG:746-751), then take the prompt pages and the block pages."""
    n_prompt = math.ceil(prompt_len / page_size)
    n_block = math.ceil(decode_len / page_size)
    while allocator.num_free_pages < n_prompt + n_block:
        if not allocator.evict_one():
            break
    return allocator.allocate_pages(n_prompt), allocator.allocate_pages(n_block)


def _decode_side_record(source: DreamPrefillRecord, prompt_page_ids: List[int], block_page_ids: List[int],
                        last_context_logit: Optional[torch.Tensor]) -> DreamPrefillRecord:
    return DreamPrefillRecord(
        prompt_ids=list(source.prompt_ids), prompt_positions=list(source.prompt_positions),
        suffix_positions=list(source.suffix_positions), prompt_len=source.prompt_len,
        full_prompt_len=source.full_prompt_len, decode_len=source.decode_len, prompt_page_ids=prompt_page_ids,
        block_page_ids=block_page_ids, first_token_id=source.first_token_id, last_context_logit=last_context_logit,
        decode_delta_state=source.decode_delta_state, owns_prompt_pages=True, cached_prefix=None,
        kv_mode=source.kv_mode)


def make_pd_record_from_kv_snapshot(kv_cache: torch.Tensor, allocator: PageAllocator,
                                    source: DreamPrefillRecord, snapshot: DreamKVSnapshot, *,
                                    page_size: int = PAGE_SIZE) -> DreamPrefillRecord:
    """make_pd_record_from_kv_snapshot (ENG:728-781): allocate local pages, load the snapshot into them
    and return the record the decode side works on; the same three consistency checks."""
    if snapshot.page_size != page_size:
        raise ValueError(f"PD KV snapshot page_size mismatch: snapshot={snapshot.page_size}, engine={page_size}")
    if snapshot.prompt_len != source.prompt_len:
        raise ValueError(f"PD KV snapshot prompt_len mismatch: snapshot={snapshot.prompt_len}, "
                         f"source={source.prompt_len}")
    if snapshot.kv_mode != source.kv_mode:
        raise ValueError(f"PD KV snapshot mode mismatch: snapshot={snapshot.kv_mode}, source={source.kv_mode}")
    prompt_pages, block_pages = _allocate_record_pages(allocator, source.prompt_len, source.decode_len, page_size)
    load_prompt_cache_per_layer(kv_cache, prompt_pages, source.prompt_len, snapshot.k_by_layer, snapshot.v_by_layer)
    ll = snapshot.last_context_logit
    if ll is not None:
        ll = ll.to(device=kv_cache.device).contiguous()
    return _decode_side_record(source, prompt_pages, block_pages, ll)


def make_pd_record_from_remote_cache(src_kv_cache: torch.Tensor, dst_kv_cache: torch.Tensor,
                                     allocator: PageAllocator, source: DreamPrefillRecord, *,
                                     page_size: int = PAGE_SIZE) -> DreamPrefillRecord:
    """make_pd_record_from_remote_engine (ENG:800-881) for two caches on this GPU: the prompt KV moves
    page by page, all layers in one launch, instead of one gather and one indexed write per layer."""
    if int(src_kv_cache.shape[3]) != page_size or int(dst_kv_cache.shape[3]) != page_size:
        raise ValueError(f"remote-engine PD page_size mismatch: source={int(src_kv_cache.shape[3])}, "
                         f"target={int(dst_kv_cache.shape[3])}")
    if int(src_kv_cache.shape[1]) != int(dst_kv_cache.shape[1]):
        raise ValueError(f"remote-engine PD layer mismatch: source={int(src_kv_cache.shape[1])}, "
                         f"target={int(dst_kv_cache.shape[1])}")
    prompt_pages, block_pages = _allocate_record_pages(allocator, source.prompt_len, source.decode_len, page_size)
    n = len(prompt_pages)
    dev = dst_kv_cache.device
    ops.kv_copy_pages(src_kv_cache, dst_kv_cache,
                      torch.as_tensor(list(source.prompt_page_ids)[:n], dtype=torch.int32, device=dev),
                      torch.as_tensor(prompt_pages, dtype=torch.int32, device=dev))
    ll = source.last_context_logit
    if ll is not None:
        ll = ll.to(device=dev).contiguous()
    return _decode_side_record(source, prompt_pages, block_pages, ll)


def release_pd_record(allocator: PageAllocator, record: DreamPrefillRecord) -> None:
    """release_pd_record (ENG:2192-2198): block pages always go back, prompt pages when the record owns
    them, and a shared prefix loses one reference."""
    allocator.release_pages(record.block_page_ids)
    if record.owns_prompt_pages:
        allocator.release_pages(record.prompt_page_ids)
    if record.cached_prefix is not None:
        record.cached_prefix.ref_count -= 1


def copy_chunk_local_kv_to_prompt_pages(kv_cache: torch.Tensor, *, src_page_ids: Sequence[int],
                                        dst_page_ids: Sequence[int], src_chunk_start: int, dst_start: int,
                                        keep_indices_per_layer_per_head: Sequence[torch.Tensor]) -> int:
    """_copy_chunk_local_kv_to_prompt_pages (ENG:525-558): kept tokens of a chunk prefilled into
    temporary pages are copied, per layer and KV head, behind dst_start of the request's pages."""
    if not keep_indices_per_layer_per_head:
        return 0
    dev = kv_cache.device
    src_pages = torch.as_tensor(list(src_page_ids), dtype=torch.int32, device=dev)
    dst_pages = torch.as_tensor(list(dst_page_ids), dtype=torch.int32, device=dev)
    keep_count = int(keep_indices_per_layer_per_head[0].shape[1])
    if keep_count <= 0:
        return 0
    for layer_idx, keep in enumerate(keep_indices_per_layer_per_head):
        keep = keep.to(device=dev, dtype=torch.long)
        if int(keep.shape[1]) != keep_count:
            raise ValueError(f"Layer {layer_idx} keep_count mismatch in chunk-local KV copy")
        for kv in range(2):
            gathered = ops.kv_gather(kv_cache[kv, layer_idx], src_pages, keep_count, token_idx=keep,
                                     src_offset=int(src_chunk_start))
            ops.kv_scatter(kv_cache[kv, layer_idx], dst_pages, gathered, dst_start=int(dst_start))
    return keep_count


# ------------------------------------------------------------------------------------------
# rotary positions of chunks and queries (prefilling_dllm_eval/fastdllm_parallelcomp.py:919-948)
# ------------------------------------------------------------------------------------------

def chunk_rope_start(mode: str, prefix_len: int, chunk_order: int, chunk_index: int, chunk_size: int) -> int:
    """First rotary position of a chunk (_chunk_rope_start): "reuse" puts every chunk right behind the
    prefix, "continuous" lines the chunks up in the order they are processed, "absolute" by their index in
    the document."""
    step = max(1, int(chunk_size))
    if mode == "reuse":
        return int(prefix_len)
    if mode == "continuous":
        return int(prefix_len) + int(chunk_order) * step
    if mode == "absolute":
        return int(prefix_len) + int(chunk_index) * step
    raise ValueError(f"Unsupported chunk_position_mode: {mode}")


def chunk_query_rope_start(mode: str, prefix_len: int, chunk_start: int, chunk_len: int, chunk_size: int) -> int:
    """First rotary position of the query appended to a chunk while it is scored (_chunk_query_rope_start)."""
    if mode == "after_reused_window":
        return int(prefix_len) + max(1, int(chunk_size))
    if mode == "after_chunk":
        return int(chunk_start) + int(chunk_len)
    raise ValueError(f"Unsupported chunk_query_position_mode: {mode}")


def final_query_rope_start(mode: str, prefix_len: int, cache_positions: Sequence[int], selected_count: int,
                           chunk_size: int) -> int:
    """First rotary position of the query + response block of the decode (_final_query_rope_start)."""
    if mode == "after_reused_window":
        return int(prefix_len) + max(1, int(chunk_size))
    if mode == "after_selected_chunks":
        return int(prefix_len) + int(selected_count) * max(1, int(chunk_size))
    if mode == "after_cache":
        return (max(cache_positions) + 1) if len(cache_positions) else int(prefix_len)
    raise ValueError(f"Unsupported query_position_mode: {mode}")


def chunk_positions(mode: str, prefix_len: int, chunk_lens: Sequence[int], chunk_indices: Sequence[int],
                    chunk_size: int, device=None) -> torch.Tensor:
    """Rotary positions of a packed batch of chunks (int64 [sum(chunk_lens)]): chunk j, the j-th processed
    and chunk_indices[j]-th of the document, gets chunk_rope_start(...) + 0 .. len-1."""
    out = []
    for order, (n, ci) in enumerate(zip(chunk_lens, chunk_indices)):
        s0 = chunk_rope_start(mode, prefix_len, order, ci, chunk_size)
        out.append(torch.arange(s0, s0 + int(n), dtype=torch.int64))
    pos = torch.cat(out) if out else torch.empty(0, dtype=torch.int64)
    return pos if device is None else pos.to(device)


# ------------------------------------------------------------------------------------------
# one denoise step after the model forward (ENG:2143-2157), no host synchronisation
# ------------------------------------------------------------------------------------------

def denoise_unmask_step(logits: torch.Tensor, block_ids: torch.Tensor, *, mask_token_id: int, threshold: float,
                        last_context_logit: Optional[torch.Tensor] = None,
                        shift: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """logits [n_seqs*block_len, vocab] bf16, block_ids [n_seqs, block_len] int64 (updated in place).
    shift=True applies the Dream logit shift (_shift_logits, ENG:1647-1656) while reading; LLaDA
    uses shift=False.  Confidence = fp32 max-softmax, token = first argmax (_sample_tokens at
    temperature 0, ENG:1675-1681); transfer = most confident masked position plus every masked
    position with confidence >= threshold (ENG:2146-2157).  Returns (transfer mask, masked left)."""
    _, _, transfer, left = ops.denoise_unmask(logits, block_ids, mask_token_id, threshold, shift=shift,
                                              last_logit=last_context_logit)
    return transfer, left


# ------------------------------------------------------------------------------------------
# draft rounds for chunk selection (ENG:1013-1059)
# ------------------------------------------------------------------------------------------

def partial_draft_round(logits: torch.Tensor, block_ids: torch.Tensor, *, prompt_len: int, mask_token_id: int,
                        first: bool = False) -> torch.Tensor:
    """One round of generate_partial_draft_rounds_for_selection (ENG:1043-1059) on the device, no host sync.

    logits [prompt_len + draft_len, vocab] bf16 is the model output for prompt + block, block_ids [draft_len] or
    [1, draft_len] int64 is updated in place.  A round confirms exactly one position: the still-masked position
    whose shifted logits are the most confident (first one on ties) receives its argmax token -- the unmask step
    with a threshold no confidence reaches.  first=True is the opening move of the reference (ENG:1034-1036): position
    0 is confirmed whatever its confidence.  Returns the bool transfer mask of the round, shaped like block_ids.

    The shift needs no copy: shifted row prompt_len + i is logits row prompt_len + i - 1 (ENG:1647-1656), so the
    block's shifted rows are the slice starting at prompt_len - 1; with an empty prompt row 0 stands for itself."""
    ids = block_ids.view(1, -1)
    draft_len = ids.shape[1]
    if logits.dim() != 2 or logits.shape[0] != prompt_len + draft_len:
        raise ValueError("logits must be [prompt_len + draft_len, vocab]")
    if prompt_len > 0:
        rows, shift = logits[prompt_len - 1:prompt_len - 1 + draft_len], False
    else:
        rows, shift = logits, True
    if first:
        rows, ids = rows[:1], ids[:, :1]
        if not bool(ids.is_contiguous()):
            raise ValueError("block_ids must be contiguous")
    _, _, transfer, _ = ops.denoise_unmask(rows, ids, mask_token_id, 2.0, shift=shift)
    if first:
        full = torch.zeros(draft_len, dtype=torch.bool, device=logits.device)
        full[:1] = transfer.view(-1)
        transfer = full
    return transfer.view(block_ids.shape)


def generate_partial_draft_rounds_for_selection(forward_logits, prompt_ids: Sequence[int], *, max_new_tokens: int,
                                                partial_rounds: int, mask_token_id: int,
                                                device=None) -> Tuple[List[int], List[bool]]:
    """generate_partial_draft_rounds_for_selection (ENG:1013-1059) around a caller-supplied model forward:
    forward_logits(token_ids int64 [prompt_len + draft_len]) -> logits [prompt_len + draft_len, vocab] bf16 stands
    for _forward_prefill_for_selection with a full mask.  The block stays on the device between rounds; the only
    host transfers are the two result lists at the end (the reference reads one scalar per round to find the masked
    positions).  A round after the last mask is gone changes nothing, as the reference's early exit."""
    draft_len = int(max_new_tokens or 0)
    if draft_len <= 0:
        return [], []
    prompt = torch.as_tensor([int(x) for x in prompt_ids], dtype=torch.int64, device=device)
    dev = prompt.device
    block = torch.full((draft_len,), int(mask_token_id), dtype=torch.int64, device=dev)
    confirmed = torch.zeros(draft_len, dtype=torch.bool, device=dev)
    n = int(prompt.numel())
    for r in range(1 + max(0, int(partial_rounds or 0))):
        logits = forward_logits(torch.cat([prompt, block]))
        confirmed |= partial_draft_round(logits, block, prompt_len=n, mask_token_id=mask_token_id, first=(r == 0))
    return block.tolist(), confirmed.tolist()


# ------------------------------------------------------------------------------------------
# per-chunk keep lists -> global keep lists (ENG:1524-1546)
# ------------------------------------------------------------------------------------------

def assemble_global_keep_indices(layer_chunk_keeps: Sequence[Sequence[torch.Tensor]],
                                 chunk_spans: Sequence[Tuple[int, int]], full_prompt_len: int, num_kv_heads: int,
                                 as_lists: bool = True):
    """Global keep lists per layer and KV head from the keep lists of the evicted chunks (ENG:1524-1546).

    layer_chunk_keeps[layer][c] is int64 [Hkv, kept_c]: the positions kept of chunk c, already global (the engine
    adds the chunk start, ENG:1514); chunk_spans[c] = (start, end) in the order the chunks were processed.
    Everything outside the spans is kept by every head: the result of a head is, span after span, the gap in front
    of the span (cursor .. start) followed by the span's kept positions, then the tail up to full_prompt_len.  A
    layer without keep lists keeps every position.  Returns List[layer][head][position] (as_lists, the reference's
    form, the input of normalize_per_head_keep_indices / compact_prompt_cache_per_layer_per_head) or a list of
    int64 tensors [Hkv, n] on the device of the keep lists."""
    spans = [(int(s[0]), int(s[1])) if not isinstance(s, dict) else (int(s["start"]), int(s["end"]))
             for s in chunk_spans]
    out = []
    for parts in layer_chunk_keeps:
        parts = list(parts)
        if not parts:
            t = torch.arange(full_prompt_len, dtype=torch.int64).unsqueeze(0).repeat(int(num_kv_heads), 1)
            out.append(t.tolist() if as_lists else t)
            continue
        if len(parts) != len(spans):
            raise ValueError("one keep tensor per chunk span expected")
        dev, heads = parts[0].device, int(parts[0].shape[0])
        cols, cursor = [], 0
        for (start, end), keep in zip(spans, parts):
            if keep.dim() != 2 or int(keep.shape[0]) != heads:
                raise ValueError("keep lists must be [Hkv, kept] with the same Hkv for every chunk")
            if start > cursor:                      # whole rows of columns: the gap is the same for every head
                cols.append(torch.arange(cursor, start, dtype=torch.int64, device=dev).expand(heads, -1))
            cols.append(keep.to(device=dev, dtype=torch.int64))
            cursor = end
        if cursor < full_prompt_len:
            cols.append(torch.arange(cursor, full_prompt_len, dtype=torch.int64, device=dev).expand(heads, -1))
        t = torch.cat(cols, dim=1)
        out.append(t.tolist() if as_lists else t)
    return out
