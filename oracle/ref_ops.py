"""CPU oracle: a plain PyTorch / numpy restatement of the reference algorithm for the hot path.

THIS IS TEST INFRASTRUCTURE.  Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
bench.py may import it; the product path (prefilling_dllm_amd) never does.

Every function cites the reference lines it restates.  Path shorthand (under the reference root):
  ENG = prefilling_dllm_engine/prefilling_dllm/fastdllm_engine.py
  OPS = prefilling_dllm_engine/prefilling_dllm/layers/attention/ops
  ATT = prefilling_dllm_engine/prefilling_dllm/layers/attention/attention_v4.py
  CTX = prefilling_dllm_engine/prefilling_dllm/utils/context.py
  ROT = prefilling_dllm_engine/prefilling_dllm/layers/rotary_embedding.py
  RES = prefilling_dllm_eval/fastdllm_parallelcomp.py

How each function is pinned (tests/test_oracle_*.py):
  slot mapping / store / load / gather / scatter / compaction / chunk-local copy : closed form page*P + t%P,
      token-by-token loops over plain indices (overlapping source and destination pages included),
      gather(scatter(x)) == x, the reference's slot-mapping fixture (examples/mimic_data) and the
      procedures of examples/test_dllm_kv_cache_store.py:41-43, test_dllm_kv_cache_load.py:63-65
  attention : torch SDPA in fp64, V == 1 => O == 1, key permutation invariance, split/merge
      identity, causal block-diagonal == independent per-chunk SDPA, the procedure of
      examples/test_dllm_decoding_kernel.py:84-97
  self-information : scipy.special.logsumexp in fp64
  top-K / top-B : brute force over all subsets on tiny inputs, the degenerate branches of ENG:903-927
  eviction scores : closed form column sums; sum over keys == query_len * mass invariant
  confidence / unmask : 1 / sum exp(x - max), first-max index; set formula {argmax} U {conf >= thr}
  rope : rotation preserves the norm of each (x_i, x_{i+d/2}) pair; position 0 is the identity
  fp8 : torch.float8_e4m3fn casts
  vote keep set : numpy bincount + stable argsort, and the invariants of the definition (first token of a
      chunk and tokens outside the chunks survive, min(capacity, length) per chunk, no dropped token
      outvotes a kept one)
  draft rounds : a hand-computed 3-round trace on a 5-token vocabulary (which position wins each round, ties)
  keep-list assembly : a hand-listed example with a leading gap, adjacent chunks and a tail
  anchor corrections : hand-listed anchor / window tables for the three directions, stride 1 with a zero window
      reproduces the dense result, an unchanged prompt gives a zero delta, the selection modes reduce to the plain
      mode for selection == dense
Unpinned: nothing in this file is "parity unpinned".
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

PAGE_SIZE = 256  # prefilling_dllm/config.py:39


# --------------------------------------------------------------------------------------
# paged addressing, store, load  (ENG:331-351, 434-441; OPS/kv_cache_kernels.py)
# --------------------------------------------------------------------------------------

def slot_mapping(page_ids: Sequence[int], num_tokens: int, start_token: int = 0,
                 page_size: int = PAGE_SIZE) -> torch.Tensor:
    """ENG:331-337 (_page_ids_to_slot_mapping) and :434-441 (_range_slot_mapping)."""
    slots = []
    for local_idx in range(int(num_tokens)):
        token_idx = int(start_token) + local_idx
        slots.append(int(page_ids[token_idx // page_size]) * page_size + token_idx % page_size)
    return torch.tensor(slots, dtype=torch.int32)


def split_slot_mapping(prompt_page_ids, block_page_ids, prompt_len, block_len, page_size=PAGE_SIZE):
    """ENG:339-351: prompt tokens -> prompt pages, block tokens -> block pages."""
    return torch.cat([slot_mapping(prompt_page_ids, prompt_len, 0, page_size),
                      slot_mapping(block_page_ids, block_len, 0, page_size)])


def store_kvcache(key, value, k_cache, v_cache, slots) -> None:
    """OPS/kv_cache_kernels.py:34-55: per token, slot < 0 skips, else copy the whole [Hkv*d] row."""
    kc = k_cache.view(-1, k_cache.shape[-2] * k_cache.shape[-1])
    vc = v_cache.view(-1, v_cache.shape[-2] * v_cache.shape[-1])
    for t, slot in enumerate(slots.tolist()):
        if slot < 0:
            continue
        kc[slot] = key[t].reshape(-1)
        vc[slot] = value[t].reshape(-1)


def load_kvcache(k_cache, v_cache, block_tables, ctx_lens, seq_lens, k_new, v_new):
    """OPS/kv_cache_kernels.py:175-327: per sequence the first ctx_len tokens of its pages, then
    its active rows; sequences concatenated.  Same loop as CHECK_LOADING (:365-394)."""
    P = k_cache.shape[1]
    ks, vs = [], []
    q0 = 0
    for s, (ctx, n_act) in enumerate(zip(ctx_lens, seq_lens)):
        ctx, n_act = int(ctx), int(n_act)
        for t in range(ctx):
            page = int(block_tables[s][t // P])
            ks.append(k_cache[page, t % P])
            vs.append(v_cache[page, t % P])
        for t in range(n_act):
            ks.append(k_new[q0 + t])
            vs.append(v_new[q0 + t])
        q0 += n_act
    return torch.stack(ks), torch.stack(vs)


def gather_tokens(layer_cache, page_ids, token_idx, page_size=PAGE_SIZE):
    """ENG:640-662 (_snapshot_prompt_cache_per_layer): cache[pages[t // P], t % P] for a token list."""
    page_ids = torch.as_tensor(page_ids, dtype=torch.long)
    token_idx = torch.as_tensor(token_idx, dtype=torch.long)
    pages = page_ids.index_select(0, token_idx // page_size)
    offsets = token_idx % page_size
    return layer_cache[pages, offsets].clone()


def scatter_tokens(layer_cache, page_ids, src, dst_start=0, page_size=PAGE_SIZE) -> None:
    """ENG:664-698 (_load_prompt_cache_per_layer)."""
    page_ids = torch.as_tensor(page_ids, dtype=torch.long)
    token_idx = torch.arange(dst_start, dst_start + src.shape[0], dtype=torch.long)
    layer_cache[page_ids.index_select(0, token_idx // page_size), token_idx % page_size] = src


def compact_per_head(layer_cache, page_ids, keep, page_size=PAGE_SIZE) -> None:
    """ENG:607-638: per KV head h, token j of the compacted cache = token keep[h][j] of the old one
    (gather is cloned before the write, exactly as the reference)."""
    page_ids = torch.as_tensor(page_ids, dtype=torch.long)
    keep = torch.as_tensor(keep, dtype=torch.long)
    active_len = keep.shape[1]
    dst = torch.arange(active_len, dtype=torch.long)
    dst_pages = page_ids.index_select(0, dst // page_size)
    dst_off = dst % page_size
    for h in range(keep.shape[0]):
        src = keep[h]
        compacted = layer_cache[page_ids.index_select(0, src // page_size), src % page_size, h, :].clone()
        layer_cache[dst_pages, dst_off, h, :] = compacted


def copy_chunk_local_kv(layer_cache, src_page_ids, dst_page_ids, src_chunk_start, dst_start, keep,
                        page_size=PAGE_SIZE) -> None:
    """ENG:525-558 (_copy_chunk_local_kv_to_prompt_pages) for one layer and one of K/V."""
    src_pages = torch.as_tensor(src_page_ids, dtype=torch.long)
    dst_pages_all = torch.as_tensor(dst_page_ids, dtype=torch.long)
    keep = torch.as_tensor(keep, dtype=torch.long)
    n = keep.shape[1]
    dst = torch.arange(dst_start, dst_start + n, dtype=torch.long)
    dst_pages = dst_pages_all.index_select(0, dst // page_size)
    dst_off = dst % page_size
    for h in range(keep.shape[0]):
        src = keep[h] + int(src_chunk_start)
        gathered = layer_cache[src_pages.index_select(0, src // page_size), src % page_size, h, :].clone()
        layer_cache[dst_pages, dst_off, h, :] = gathered


# --------------------------------------------------------------------------------------
# fp8 e4m3 pages with a per-page scale (extension of OPS/prefix_prefill.py:118-121, 159-162)
# --------------------------------------------------------------------------------------

def quantize_pages_fp8(cache: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """cache [pages, P, Hkv, d] float -> (e4m3 cache, scale[pages] fp32), scale = amax(page)/448."""
    c = cache.float()
    amax = c.abs().amax(dim=(1, 2, 3))
    scale = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax)).float()
    q = (c / scale.view(-1, 1, 1, 1)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q, scale


def dequantize_pages_fp8(q: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """float(e4m3) * scale[page], then rounded to bf16 as the kernel input precision
    (prefix_prefill.py:118-121 converts `(k_load.to(fp32) * scale).to(q.dtype)`)."""
    return (q.float() * scale.view(-1, 1, 1, 1)).to(torch.bfloat16)


# --------------------------------------------------------------------------------------
# attention  (ATT:54-78, 316-410; OPS/prefix_prefill.py:25-230; CTX:69-98)
# --------------------------------------------------------------------------------------

def _sdpa(q, k, v, mask, scale, dtype=torch.float32):
    """softmax(q k^T * scale + mask) v with GQA by head grouping (prefix_prefill.py:62,
    ATT:69-71).  q [Sq, Hq, d], k/v [Sk, Hkv, d], mask [Sq, Sk] bool or None.  Rows with no
    visible key give zeros."""
    Sq, Hq, d = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    qf = q.to(dtype).permute(1, 0, 2)                                # [Hq, Sq, d]
    kf = k.to(dtype).permute(1, 0, 2).repeat_interleave(G, dim=0)    # [Hq, Sk, d]
    vf = v.to(dtype).permute(1, 0, 2).repeat_interleave(G, dim=0)
    s = torch.matmul(qf, kf.transpose(1, 2)) * scale
    if mask is not None:
        s = s.masked_fill(~mask.unsqueeze(0), float("-inf"))
    m = s.amax(dim=-1, keepdim=True)
    m = torch.where(torch.isinf(m), torch.zeros_like(m), m)
    p = torch.exp(s - m)
    den = p.sum(dim=-1, keepdim=True)
    o = torch.matmul(p, vf) / torch.where(den > 0, den, torch.ones_like(den))
    return o.permute(1, 0, 2)                                        # [Sq, Hq, d]


def gather_prefix(k_cache, v_cache, block_table_row, ranges, page_size=PAGE_SIZE):
    """Rows of the visible prefix: logical tokens of every (start, len) range mapped through the
    request's page table (page_table[t // P], t % P) -- the addressing of prefix_prefill.py:100-109.
    A page-table entry outside [0, n_pages) names no page; its tokens are left out, as load_kvcache skips -1
    entries (kv_cache_kernels.py:208)."""
    toks: List[int] = []
    for start, length in ranges:
        toks.extend(range(int(start), int(start) + int(length)))
    if not toks:
        empty = k_cache.new_zeros((0,) + tuple(k_cache.shape[2:]))
        return empty, empty.clone()
    t = torch.tensor(toks, dtype=torch.long)
    pages = torch.as_tensor(block_table_row, dtype=torch.long).index_select(0, t // page_size)
    named = (pages >= 0) & (pages < k_cache.shape[0])
    pages, t = pages[named], t[named]
    return k_cache[pages, t % page_size], v_cache[pages, t % page_size]


def sparse_decode_attention(q, k_new, v_new, k_cache, v_cache, block_table, q_start_loc, ranges_per_req,
                            *, mask_mode="full", mask=None, sm_scale=None, dtype=torch.float32,
                            out_dtype=None):
    """Decode branch of Attention.forward (ATT:368-397): every request's active rows attend to
    [its visible prefix tokens || its active rows].  Prefix keys are always visible
    (prefix_prefill.py:96-176); the active keys follow mask_mode: "full" (all ones mask of
    ENG:392-396), "causal", or "dense" with mask[n_tok, n_tok] indexed by absolute row numbers."""
    n_tok, Hq, d = q.shape
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    out = torch.zeros((n_tok, Hq, d), dtype=dtype)
    qsl = [int(x) for x in q_start_loc]
    for r in range(len(qsl) - 1):
        a, b = qsl[r], qsl[r + 1]
        Sq = b - a
        if Sq <= 0:
            continue
        if k_cache is not None and ranges_per_req is not None and len(ranges_per_req[r]) > 0:
            kp, vp = gather_prefix(k_cache, v_cache, block_table[r], ranges_per_req[r], k_cache.shape[1])
        else:
            kp = k_new.new_zeros((0,) + tuple(k_new.shape[1:]))
            vp = kp.clone()
        k_all = torch.cat([kp.to(dtype), k_new[a:b].to(dtype)], dim=0)
        v_all = torch.cat([vp.to(dtype), v_new[a:b].to(dtype)], dim=0)
        n_ctx = kp.shape[0]
        if mask_mode == "full":
            am = torch.ones((Sq, Sq), dtype=torch.bool)
        elif mask_mode == "causal":
            am = torch.tril(torch.ones((Sq, Sq), dtype=torch.bool))
        elif mask_mode == "dense":
            am = mask[a:b, a:b].to(torch.bool)
        else:
            raise ValueError(mask_mode)
        full = torch.cat([torch.ones((Sq, n_ctx), dtype=torch.bool), am], dim=1)
        out[a:b] = _sdpa(q[a:b], k_all, v_all, full, sm_scale, dtype)
    return out if out_dtype is None else out.to(out_dtype)


def chunk_prefill_attention(q, k, v, cu_seqlens, *, causal=True, sm_scale=None, dtype=torch.float32):
    """Prefill branch (ATT:336-367) with the block-diagonal mask of CTX:73-84: each chunk attends
    only to itself, causal (ENG:943-944 selection mask) or full (ENG:256-281)."""
    cu = [int(x) for x in cu_seqlens]
    return sparse_decode_attention(q, k, v, None, None, None, cu, None,
                                   mask_mode="causal" if causal else "full", sm_scale=sm_scale, dtype=dtype)


# --------------------------------------------------------------------------------------
# experimental anchor corrections (ATT:86-293, default off)
# --------------------------------------------------------------------------------------

def anchor_windows(seq_len: int, state: dict):
    """Anchors and the rows each one corrects: ATT:113-125 (defaults and clamps) and ATT:151-165 (windows)."""
    stride = max(1, int(state.get("stride", 4)))
    left = max(0, int(state.get("left", stride - 1)))
    right = max(0, int(state.get("right", 0)))
    direction = (state.get("direction") or "left").lower()
    anchor_offset = int(state.get("anchor_offset", stride - 1))
    if anchor_offset < 0:
        anchor_offset = stride - 1
    anchor_offset = min(anchor_offset, stride - 1)
    anchors = list(range(anchor_offset, seq_len, stride))
    windows = []
    for anchor in anchors:
        if direction == "right":
            rows = range(anchor, min(seq_len - 1, anchor + right) + 1)
        elif direction == "both":
            rows = range(max(0, anchor - left), min(seq_len - 1, anchor + right) + 1)
        else:
            rows = range(max(0, anchor - left), anchor + 1)
        windows.append(list(rows))
    return anchors, windows


def anchor_delta_add(base, delta, windows):
    """ATT:150-166: correction = zeros_like(base); correction[rows] += delta[idx] per anchor, ascending; base +
    correction.  base [S, H, d], delta [A, H, d]; computed in the dtype of the tensors (bf16 tensors round after every
    operation, as the reference's do)."""
    correction = torch.zeros_like(base)
    for idx, rows in enumerate(windows):
        if rows:
            correction[rows] += delta[idx:idx + 1]
    return base + correction


def decode_delta(o, q, k_new, v_new, full_k, full_v, state, *, active_mask=None, sm_scale=None):
    """Attention._maybe_apply_decode_delta (ATT:86-166): the anchor rows attend to [full prompt || active rows]
    (prompt keys all visible, active keys by active_mask[anchors] or all), delta = (dense - o[anchors]) * scale is
    spread over each anchor's window.  o / q [S, Hq, d], k_new / v_new [S, Hkv, d], full_k / full_v [P, Hkv, d].
    Arithmetic in the dtype of o."""
    S, _, d = q.shape
    anchors, windows = anchor_windows(S, state)
    if not anchors:
        return o
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    k_all = torch.cat([full_k.to(k_new.dtype), k_new], dim=0)
    v_all = torch.cat([full_v.to(v_new.dtype), v_new], dim=0)
    am = torch.ones((len(anchors), S), dtype=torch.bool) if active_mask is None else active_mask[anchors].to(torch.bool)
    mask = torch.cat([torch.ones((len(anchors), full_k.shape[0]), dtype=torch.bool), am], dim=1)
    dense_anchor = _sdpa(q[anchors], k_all, v_all, mask, sm_scale, torch.float32).to(o.dtype)
    delta = (dense_anchor - o[anchors]) * float(state.get("scale", 1.0))
    return anchor_delta_add(o, delta, windows)


def prefill_sparse_attention(q, k, v, base_mask, keep, state, *, sm_scale=None, selection_outputs=None,
                             selection_counts=None, out_dtype=torch.float32):
    """Attention._maybe_prefill_sparse_attention (ATT:168-293) for one layer: keys outside `keep` (and before
    full_prompt_len) are masked on top of base_mask; with a delta mode the anchor rows are corrected towards the
    dense result (or the stored selection outputs).  q [S, Hq, d], k / v [S, Hkv, d], base_mask [S, S] bool.
    The attention is computed in fp32 and cast to out_dtype, the correction runs in out_dtype."""
    S, Hq, d = q.shape
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    key_mask = torch.zeros(S, dtype=torch.bool)
    valid_keep = keep.reshape(-1).long()
    valid_keep = valid_keep[(valid_keep >= 0) & (valid_keep < S)]
    key_mask[valid_keep] = True
    full_prompt_len = int(state.get("full_prompt_len", S))
    if 0 <= full_prompt_len < S:
        key_mask[full_prompt_len:] = True
    base_mask = base_mask.to(torch.bool)
    o_sparse = _sdpa(q, k, v, base_mask & key_mask.unsqueeze(0), sm_scale, torch.float32).to(out_dtype)
    delta_mode = (state.get("delta_mode") or "none").lower()
    if delta_mode in {"none", "off", "0", ""}:
        return o_sparse
    anchors, windows = anchor_windows(S, state)
    if not anchors:
        return o_sparse
    sparse_anchor = o_sparse[anchors]
    selection_mode = (state.get("selection_mode") or "none").lower()
    selection_anchor = selection_valid = None
    if selection_mode in {"selection_dense_replace", "selection_dense_add"} and selection_outputs is not None \
            and selection_outputs.shape[0] > 0 and selection_outputs.shape[1] == Hq:
        at = torch.tensor(anchors)
        in_range = at < selection_outputs.shape[0]
        safe = at.clamp_max(selection_outputs.shape[0] - 1)
        selection_anchor = torch.zeros_like(sparse_anchor)
        selection_anchor[in_range] = selection_outputs.to(out_dtype)[safe][in_range]
        selection_valid = ((selection_counts[safe] > 0) & in_range) if selection_counts is not None else in_range
    dense_anchor = None
    if selection_mode != "selection_dense_replace":
        dense_anchor = _sdpa(q[anchors], k, v, base_mask[anchors], sm_scale, torch.float32).to(out_dtype)
    if selection_mode == "selection_dense_replace":
        if selection_anchor is None or not bool(selection_valid.any()):
            return o_sparse
        delta = (selection_anchor - sparse_anchor) * float(state.get("scale", 1.0))
        delta = delta * selection_valid.view(-1, 1, 1).to(delta.dtype)
    else:
        delta = (dense_anchor - sparse_anchor) * float(state.get("scale", 1.0))
        if selection_mode == "selection_dense_add" and selection_anchor is not None:
            sd = (selection_anchor - dense_anchor) * float(state.get("selection_scale", 1.0))
            delta = delta + sd * selection_valid.view(-1, 1, 1).to(sd.dtype)
    return anchor_delta_add(o_sparse, delta, windows)


def split_token_chunks(token_ids: Sequence[int], chunk_size: int, split_from_tail: bool = False):
    """RES:158-180."""
    ids = list(token_ids)
    if not ids:
        return []
    if chunk_size <= 0 or len(ids) <= chunk_size:
        return [ids]
    chunks, cursor = [], 0
    if split_from_tail:
        lead = len(ids) % chunk_size
        if lead > 0:
            chunks.append(ids[:lead])
            cursor = lead
    while cursor < len(ids):
        chunks.append(ids[cursor:cursor + chunk_size])
        cursor += chunk_size
    return chunks


# --------------------------------------------------------------------------------------
# rotary embedding (ROT:6-17, 39-65)
# --------------------------------------------------------------------------------------

def rope_cos_sin_cache(head_dim: int, max_pos: int, base: float = 10000.0) -> torch.Tensor:
    """ROT:31-38: [max_pos, head_dim] = cos(d/2) | sin(d/2) in fp32."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim))
    t = torch.arange(max_pos, dtype=torch.float)
    freqs = torch.einsum("i,j -> ij", t, inv_freq)
    return torch.cat((freqs.cos(), freqs.sin()), dim=-1)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, cos_sin_cache: torch.Tensor) -> torch.Tensor:
    """ROT:6-17 neox split-half rotation in fp32, result cast back to x.dtype."""
    cos_sin = cos_sin_cache[positions]
    cos, sin = cos_sin.chunk(2, dim=-1)
    cos, sin = cos.unsqueeze(-2), sin.unsqueeze(-2)
    x1, x2 = torch.chunk(x.to(torch.float32), 2, dim=-1)
    y1 = x1 * cos - x2 * sin
    y2 = x2 * cos + x1 * sin
    return torch.cat((y1, y2), dim=-1).to(x.dtype)


# --------------------------------------------------------------------------------------
# chunk scoring and ranking (ENG:1098-1152, 1199-1204)
# --------------------------------------------------------------------------------------

def selfinfo_logprob(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """ENG:1150-1151: log_softmax(query_logits.float())[label]."""
    lp = F.log_softmax(logits.float(), dim=-1)
    return lp.gather(dim=-1, index=labels.long().unsqueeze(-1)).squeeze(-1)


def chunk_scores(logits: torch.Tensor, labels: torch.Tensor, mean: bool = True) -> torch.Tensor:
    """ENG:1152: score = -mean(nll) = mean(log p[label]).  logits [chunks, labels, vocab].
    The per-chunk reduction runs over the labels in index order in fp32."""
    lp = selfinfo_logprob(logits.reshape(-1, logits.shape[-1]), labels.reshape(-1)).reshape(labels.shape)
    acc = torch.zeros(lp.shape[0], dtype=torch.float32)
    for j in range(lp.shape[1]):
        acc = acc + lp[:, j]
    return acc / lp.shape[1] if mean else acc


def topk_lowest_index(scores: Sequence[float], k: int, sorted_ascending: bool = True) -> List[int]:
    """ENG:1199-1204: non-finite -> -inf; Python's stable sort with reverse=True keeps the
    original (lowest-index-first) order among equal scores; top k; ascending index order."""
    vals = [float(s) if math.isfinite(float(s)) else float("-inf") for s in scores]
    ranked = sorted(range(len(vals)), key=lambda i: vals[i], reverse=True)
    top = ranked[:k]
    return sorted(top) if sorted_ascending else top


# --------------------------------------------------------------------------------------
# token eviction (ENG:1230-1322, 1405-1433, 903-927; OPS/triton_eviction_scorer.py)
# --------------------------------------------------------------------------------------

def evict_colsum(probs: torch.Tensor, heads_per_group: Optional[int] = None) -> torch.Tensor:
    """Column sums of attention probabilities [chunks, H, Q, K] -> [chunks, H/hpg, K]:
    per head the sum over the query rows (`query_to_chunk.sum(dim=1)`, ENG:1305), then the heads
    of a group added up (the global head sum of RES:1607-1637; the per-KV-head mean of
    ENG:1418-1432 is this sum / hpg).  Both sums run in index order in fp32, which makes the
    result reproducible bit for bit."""
    p = probs.numpy() if isinstance(probs, torch.Tensor) else probs
    if p.ndim == 3:
        p = p[None]
    c, h, nq, nk = p.shape
    hpg = h if heads_per_group is None else heads_per_group
    out = np.zeros((c, h // hpg, nk), dtype=np.float32)
    for g in range(h // hpg):
        gacc = np.zeros((c, nk), dtype=np.float32)
        for hh in range(hpg):
            acc = np.zeros((c, nk), dtype=np.float32)
            for qi in range(nq):
                acc = acc + p[:, g * hpg + hh, qi, :]
            gacc = gacc + acc
        out[:, g, :] = gacc
    return torch.from_numpy(out)


def chunk_attention_head_scores(q, k, *, prefix_len, chunk_len, query_len, scale, reduce_mode="sum",
                                attention_mask="causal"):
    """Torch path of _engine_chunk_attention_head_scores (ENG:1279-1310), direction
    query_to_chunk: per q-head softmax over the visible keys of each of the last query_len rows,
    chunk columns summed (or averaged) over those rows -> [Hq, chunk_len] fp32."""
    Hq, Hkv = q.shape[1], k.shape[1]
    G = Hq // Hkv
    key_len = k.shape[0]
    query_start = prefix_len + chunk_len
    rows = torch.arange(query_start, query_start + query_len)
    per_head = []
    mode = (attention_mask or "full").lower()
    for kvh in range(Hkv):
        qg = q.index_select(0, rows)[:, kvh * G:(kvh + 1) * G, :]
        logits = torch.einsum("rgd,sd->rgs", qg.float(), k[:, kvh, :].float()) * float(scale)
        if mode == "causal":
            for li, row in enumerate(rows.tolist()):
                allowed = torch.arange(key_len) <= row
                logits[li, :, ~allowed] = torch.finfo(logits.dtype).min
        probs = torch.softmax(logits, dim=-1)
        per_head.append(probs.permute(1, 0, 2))
    probs = torch.cat(per_head, dim=0)                       # [Hq, query_len, key_len]
    q2c = probs[:, :, prefix_len:prefix_len + chunk_len]
    return q2c.mean(dim=1) if reduce_mode == "mean" else q2c.sum(dim=1)


def token_score_pool_group(scores: torch.Tensor, pooling: str = "none", kernel: int = 7,
                           num_kv_heads: Optional[int] = None) -> torch.Tensor:
    """ENG:1405-1433: optional max/avg pooling (kernel, padding kernel//2, stride 1) then the mean of
    each KV head's group of q-head rows (summed in index order)."""
    chunk_len = scores.shape[-1]
    pooling = (pooling or "none").lower()
    if pooling != "none":
        kernel = max(1, min(int(kernel or 1), chunk_len))
        pooled = scores.unsqueeze(1)
        if pooling == "avgpool":
            pooled = F.avg_pool1d(pooled, kernel_size=kernel, padding=kernel // 2, stride=1)
        elif pooling == "maxpool":
            pooled = F.max_pool1d(pooled, kernel_size=kernel, padding=kernel // 2, stride=1)
        else:
            raise ValueError(pooling)
        scores = pooled.squeeze(1)[..., :chunk_len]
    if num_kv_heads is not None and scores.shape[0] != num_kv_heads:
        hpg = scores.shape[0] // num_kv_heads
        grouped = []
        for g in range(num_kv_heads):
            acc = torch.zeros(chunk_len, dtype=scores.dtype)
            for hh in range(hpg):
                acc = acc + scores[g * hpg + hh]
            grouped.append(acc / hpg)
        scores = torch.stack(grouped, dim=0)
    return scores


def select_positions_from_token_scores(token_scores: torch.Tensor, *, capacity: int, chunk_len: int,
                                       keep_high: bool = True, force_keep_first: bool = True) -> torch.Tensor:
    """ENG:903-927 with the tie rule made explicit: candidates ranked by (score desc, index asc)
    [keep_high] or (score asc, index asc); BOS (position 0) always kept; result ascending."""
    keep_count = min(max(1, int(capacity)), int(chunk_len))
    if token_scores.numel() != chunk_len:
        head = keep_count // 2
        tail = keep_count - head
        keep = sorted(set(list(range(head)) + list(range(chunk_len - tail, chunk_len))))
        return torch.tensor(keep[:keep_count], dtype=torch.long)
    vals = token_scores.float().tolist()

    def rank(cands, k):
        key = (lambda i: (-vals[i], i)) if keep_high else (lambda i: (vals[i], i))
        # NaN ranks as the largest value, as torch.topk does
        def k2(i):
            v = vals[i]
            if math.isnan(v):
                return (float("-inf"), i) if keep_high else (float("inf"), i)
            return key(i)
        return sorted(cands, key=k2)[:k]

    if force_keep_first and chunk_len > 0:
        if keep_count == 1:
            return torch.zeros(1, dtype=torch.long)
        cands = list(range(1, chunk_len))
        if len(cands) <= keep_count - 1:
            return torch.arange(chunk_len, dtype=torch.long)
        sel = rank(cands, keep_count - 1)
        return torch.tensor(sorted([0] + sel), dtype=torch.long)
    return torch.tensor(sorted(rank(list(range(chunk_len)), keep_count)), dtype=torch.long)


# --------------------------------------------------------------------------------------
# logits -> confidence -> unmask (ENG:1647-1681, 2146-2157)
# --------------------------------------------------------------------------------------

def preevict_vote_topk_indices(keep_indices, full_prompt_len: int, chunk_spans, capacity: int) -> List[int]:
    """Vote variant of the keep set, after scripts/run_dream_longbench_task_fastdllm_engine_full_bridge_
    preevict_votetopk.sh:231-258: keep_indices[layer][head] = kept prompt positions; per chunk (start, end)
    keep its first token and the capacity - 1 positions with the most votes, ties to the lowest index; tokens
    between and after the chunks are all kept."""
    votes = [0] * int(full_prompt_len)
    for layer in keep_indices or []:
        for head in layer or []:
            for idx in head or []:
                if 0 <= int(idx) < full_prompt_len:
                    votes[int(idx)] += 1
    keep, cursor, cap = set(), 0, int(capacity or 0)
    for start, end in chunk_spans:
        if start > cursor:
            keep.update(range(cursor, start))
        chunk_len = max(0, end - start)
        keep_count = min(max(1, cap), chunk_len) if cap > 0 else chunk_len
        if chunk_len > 0:
            ranked = sorted(range(start + 1, end), key=lambda i: (-votes[i], i))
            keep.add(start)
            keep.update(ranked[:max(0, keep_count - 1)])
        cursor = end
    if cursor < full_prompt_len:
        keep.update(range(cursor, full_prompt_len))
    if not keep:
        keep.update(range(full_prompt_len))
    return sorted(keep)


def shift_logits(logits: torch.Tensor, last_logit: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ENG:1647-1656."""
    shifted = torch.empty_like(logits)
    if logits.shape[0] > 1:
        shifted[1:, :] = logits[:-1, :]
    if last_logit is None:
        shifted[0, :] = logits[0, :]
    else:
        shifted[0, :] = last_logit.reshape(-1)
    return shifted


def sample_tokens(logits: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """ENG:1658-1681 at temperature 0, no top-k/top-p: fp32 softmax, (max prob, first argmax)."""
    probs = F.softmax(logits.float(), dim=-1)
    confidence, sampled = probs.max(dim=-1)
    return confidence, sampled


def threshold_unmask(block_ids: torch.Tensor, confidence: torch.Tensor, sampled: torch.Tensor,
                     mask_token_id: int, threshold: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """ENG:2146-2157 for one block.  confidence / sampled are given for EVERY position of the block
    (the reference computes them for masked positions only; unmasked ones are ignored here).
    Ties for the rank-0 position resolve to the lowest index.  Returns (new block_ids, transfer)."""
    block_ids = block_ids.clone()
    mask_index = block_ids == mask_token_id
    transfer = torch.zeros_like(block_ids, dtype=torch.bool)
    n_mask = int(mask_index.sum())
    if n_mask == 0:
        return block_ids, transfer
    full_conf = torch.full(block_ids.shape, float("-inf"), dtype=torch.float32)
    full_conf[mask_index] = confidence.float()[mask_index]
    order = sorted(range(block_ids.numel()), key=lambda i: (-float(full_conf[i]), i))[:n_mask]
    transfer[order[0]] = True
    for idx in order[1:]:
        if np.float32(full_conf[idx]) >= np.float32(threshold):  # torch compares in the tensor dtype (fp32)
            transfer[idx] = True
    block_ids[transfer] = sampled[transfer]
    return block_ids, transfer


def partial_draft_rounds(logits_of, prompt_ids: Sequence[int], max_new_tokens: int, partial_rounds: int,
                         mask_token_id: int) -> Tuple[List[int], List[bool]]:
    """ENG:1013-1059 with the model forward abstracted: logits_of(ids list) -> [len(ids), vocab] tensor.
    First the token at block position 0 is confirmed, then one masked position per round: the one whose
    (shifted) confidence is the highest, first on ties."""
    draft_len = int(max_new_tokens or 0)
    if draft_len <= 0:
        return [], []
    prompt_ids = [int(x) for x in prompt_ids]
    block_ids = [int(mask_token_id)] * draft_len
    confirmed = [False] * draft_len
    n = len(prompt_ids)
    shifted = shift_logits(logits_of(prompt_ids + block_ids))
    _, first = sample_tokens(shifted[n:n + 1])
    block_ids[0] = int(first[0])
    confirmed[0] = True
    for _ in range(max(0, int(partial_rounds or 0))):
        mask_positions = [i for i, t in enumerate(block_ids) if t == mask_token_id]
        if not mask_positions:
            break
        shifted = shift_logits(logits_of(prompt_ids + block_ids))
        conf, tok = sample_tokens(shifted[n:n + draft_len][mask_positions])
        best = int(torch.argmax(conf))
        block_ids[mask_positions[best]] = int(tok[best])
        confirmed[mask_positions[best]] = True
    return block_ids, confirmed


def assemble_global_keep_indices(layer_chunk_keeps, chunk_spans, full_prompt_len: int, num_kv_heads: int):
    """ENG:1524-1546, head by head: gaps between the processed chunks are kept whole, each chunk contributes its
    (already global) keep list.  layer_chunk_keeps[layer][chunk] = [Hkv][kept] ints; returns [layer][head][pos]."""
    out = []
    for parts in layer_chunk_keeps:
        if not parts:
            out.append([list(range(full_prompt_len)) for _ in range(num_kv_heads)])
            continue
        heads = []
        for h in range(len(parts[0])):
            pieces, cursor = [], 0
            for (start, end), keep in zip(chunk_spans, parts):
                if start > cursor:
                    pieces += list(range(cursor, start))
                pieces += [int(x) for x in keep[h]]
                cursor = end
            if cursor < full_prompt_len:
                pieces += list(range(cursor, full_prompt_len))
            heads.append(pieces)
        out.append(heads)
    return out
