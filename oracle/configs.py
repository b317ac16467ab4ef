"""Seeded synthetic inputs for the five benchmark configurations (test infrastructure).

Each generator returns CPU tensors; tests move them to the GPU, bench.py generates the full-size
workload directly on the device with the same recipe.  Shapes follow the reference engine:
pages of 256 tokens (config.py:39), Dream-7B GQA 28/4 x 128 and LLaDA-8B MHA 32/32 x 128 as used
by examples/test_dllm_decoding_kernel.py:27-28.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import torch

PAGE = 256


@dataclass
class AttnCase:
    q: torch.Tensor            # [n_tok, Hq, d] bf16
    k_new: torch.Tensor        # [n_tok, Hkv, d] bf16
    v_new: torch.Tensor
    k_cache: torch.Tensor      # [pages, P, Hkv, d] bf16 (or fp8)
    v_cache: torch.Tensor
    block_table: torch.Tensor  # [n_req, max_pages] int32
    q_start_loc: torch.Tensor  # [n_req+1] int32
    ranges: List[List[Tuple[int, int]]]  # per request: (logical start, length)
    k_scale: Optional[torch.Tensor] = None
    v_scale: Optional[torch.Tensor] = None
    k_cache_ref: Optional[torch.Tensor] = None  # what the kernel should see (dequantised) for fp8
    v_cache_ref: Optional[torch.Tensor] = None
    meta: dict = field(default_factory=dict)

    def range_tensors(self):
        ptr, start, length = [0], [], []
        for rr in self.ranges:
            for s, l in rr:
                start.append(s)
                length.append(l)
            ptr.append(len(start))
        mk = lambda x: torch.tensor(x, dtype=torch.int32)
        return mk(ptr), mk(start), mk(length), max(len(r) for r in self.ranges)

    @property
    def max_ctx(self):
        return max(sum(l for _, l in rr) for rr in self.ranges)

    @property
    def max_q(self):
        q = self.q_start_loc
        return int((q[1:] - q[:-1]).max())


def _randn(gen, *shape, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(torch.bfloat16)


def chunked_prefix_case(seed: int, *, n_req: int, n_chunks: int, chunk_tokens: int, topk: int,
                        q_len: int, Hq: int = 28, Hkv: int = 4, d: int = 128, shared_prefix: bool = True,
                        fp8: bool = False, extra_pages: int = 1) -> AttnCase:
    """Prefix = n_chunks chunks of chunk_tokens tokens (chunk c holds logical tokens
    [c*chunk_tokens, (c+1)*chunk_tokens)), stored in a paged cache whose page order is shuffled by
    the seed; each request attends to `topk` seeded distinct chunks plus its own active block."""
    gen = torch.Generator().manual_seed(seed)
    std = 1.0 / math.sqrt(d)
    prefix_tokens = n_chunks * chunk_tokens
    pages_per_req = (prefix_tokens + PAGE - 1) // PAGE
    n_prefixes = 1 if shared_prefix else n_req
    n_pages = n_prefixes * pages_per_req + extra_pages
    k_cache = _randn(gen, n_pages, PAGE, Hkv, d, scale=std)
    v_cache = _randn(gen, n_pages, PAGE, Hkv, d, scale=std)
    perm = torch.randperm(n_pages, generator=gen)
    block_table = torch.empty((n_req, pages_per_req), dtype=torch.int32)
    for r in range(n_req):
        base = 0 if shared_prefix else r * pages_per_req
        block_table[r] = perm[base:base + pages_per_req].to(torch.int32)
    ranges = []
    for r in range(n_req):
        sel = sorted(torch.randperm(n_chunks, generator=gen)[:topk].tolist())
        ranges.append([(c * chunk_tokens, chunk_tokens) for c in sel])
    n_tok = n_req * q_len
    q = _randn(gen, n_tok, Hq, d, scale=std)
    k_new = _randn(gen, n_tok, Hkv, d, scale=std)
    v_new = _randn(gen, n_tok, Hkv, d, scale=std)
    qsl = torch.arange(0, n_tok + 1, q_len, dtype=torch.int32)
    case = AttnCase(q, k_new, v_new, k_cache, v_cache, block_table, qsl, ranges,
                    meta=dict(seed=seed, n_chunks=n_chunks, chunk_tokens=chunk_tokens, topk=topk))
    if fp8:
        from . import ref_ops
        kq, ks = ref_ops.quantize_pages_fp8(k_cache)
        vq, vs = ref_ops.quantize_pages_fp8(v_cache)
        case.k_cache_ref = ref_ops.dequantize_pages_fp8(kq, ks)
        case.v_cache_ref = ref_ops.dequantize_pages_fp8(vq, vs)
        case.k_cache, case.v_cache, case.k_scale, case.v_scale = kq, vq, ks, vs
    return case


def config1(seed: int = 0) -> AttnCase:
    """C1: 8 chunks x (1 BOS + 1024), top-K = 4, 64 query + 32 response rows, batch 1."""
    return chunked_prefix_case(seed, n_req=1, n_chunks=8, chunk_tokens=1025, topk=4, q_len=96)


def config3_small(seed: int = 0, n_req: int = 2) -> AttnCase:
    """C3 shape at reduced batch: 32 chunks compacted to 512 tokens (2 pages) each, top-K = 8,
    128 query + 32 response rows per request."""
    return chunked_prefix_case(seed, n_req=n_req, n_chunks=32, chunk_tokens=512, topk=8, q_len=160,
                               shared_prefix=False)


def config5_small(seed: int = 0, n_req: int = 1, n_chunks: int = 8, topk: int = 4) -> AttnCase:
    """C5 shape at reduced size: MHA 32/32, fp8 e4m3 pages with a per-page scale."""
    return chunked_prefix_case(seed, n_req=n_req, n_chunks=n_chunks, chunk_tokens=1025, topk=topk, q_len=160,
                               Hq=32, Hkv=32, fp8=True, shared_prefix=True)


def draft_logits(seed: int, n_chunks: int = 32, n_tokens: int = 4, vocab: int = 152064):
    """C2 scoring input: N(0, 2) bf16 logits with one +8 peak per row; labels = the peak for even
    rows, a seeded other index for odd rows."""
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(n_chunks, n_tokens, vocab, generator=gen) * 2.0
    peak = torch.randint(0, vocab, (n_chunks, n_tokens), generator=gen)
    logits.scatter_add_(2, peak.unsqueeze(-1), torch.full((n_chunks, n_tokens, 1), 8.0))
    other = torch.randint(0, vocab, (n_chunks, n_tokens), generator=gen)
    rows = torch.arange(n_chunks * n_tokens).reshape(n_chunks, n_tokens)
    labels = torch.where(rows % 2 == 0, peak, other)
    return logits.to(torch.bfloat16), labels


def eviction_probs(seed: int, n_chunks: int = 2, H: int = 28, Q: int = 64, K: int = 1025):
    """C2 eviction input: softmax(N(0,1) logits [H, Q, K]) per chunk in fp32."""
    gen = torch.Generator().manual_seed(seed)
    return torch.softmax(torch.randn(n_chunks, H, Q, K, generator=gen), dim=-1).contiguous()


def unmask_logits(seed: int, n_seqs: int = 4, block_len: int = 32, vocab: int = 126464, peaks: int = 10):
    """C5 unmask input: N(0, 3) bf16 logits; `peaks` seeded rows per sequence get a +30 peak (their
    confidence goes above 0.9), a few more get a +14 peak (confidence well inside (0, 0.9))."""
    gen = torch.Generator().manual_seed(seed)
    logits = torch.randn(n_seqs, block_len, vocab, generator=gen) * 3.0
    for b in range(n_seqs):
        rows = torch.randperm(block_len, generator=gen)
        for i, r in enumerate(rows[:peaks + 4].tolist()):
            idx = int(torch.randint(0, vocab, (1,), generator=gen))
            logits[b, r, idx] += 30.0 if i < peaks else 14.0
    return logits.to(torch.bfloat16).reshape(n_seqs * block_len, vocab)


def staircase_case(seed: int, *, n_req: int = 2, n_chunks: int = 4, topk: int = 3, q_len: int = 40, gran: int = 64,
                   Hq: int = 28, Hkv: int = 4, fp8: bool = False, step: float = 9.0) -> AttnCase:
    """A case whose softmax maximum rises by about 9 log2 units from one group of `gran` visible keys to the next
    (every tile for gran = 64, every page for gran = 256) while the values shrink by 2^-9 per group, so that every
    group contributes a comparable share of the result: an error in the rescaling of the running accumulators, or in
    the log-sum-exp weights of partial results, shows up at full size instead of vanishing below the last group.
    Key group g of a request has k[..., 0] = step * g; row (token, head) has q[..., 0] in {6.5, 8, 8.5}, which with
    sm_scale = 1/sqrt(128) gives 7.5 / 9.2 / 9.8 log2 units per group (the first stays below the kernel's lazy
    rescale threshold of 8, the others cross it every group)."""
    from . import ref_ops
    case = chunked_prefix_case(seed, n_req=n_req, n_chunks=n_chunks, chunk_tokens=PAGE, topk=topk, q_len=q_len,
                               Hq=Hq, Hkv=Hkv, shared_prefix=False)
    kc, vc = case.k_cache.float(), case.v_cache.float()
    vc *= math.sqrt(case.q.shape[-1])                      # values of order one at group 0
    kn, vn = case.k_new.float(), case.v_new.float() * math.sqrt(case.q.shape[-1])
    q = case.q.float()
    for r in range(n_req):
        v_idx = 0
        for s, l in case.ranges[r]:
            for t in range(s, s + l):
                g = v_idx // gran
                page, off = int(case.block_table[r][t // PAGE]), t % PAGE
                kc[page, off, :, 0] = step * g
                vc[page, off] *= 2.0 ** (-9 * g)
                v_idx += 1
        a, b = int(case.q_start_loc[r]), int(case.q_start_loc[r + 1])
        for i in range(b - a):
            g = (v_idx + i) // gran
            kn[a + i, :, 0] = step * g
            vn[a + i] *= 2.0 ** (-9 * g)
    rows = torch.arange(q.shape[0]).view(-1, 1) + torch.arange(Hq).view(1, -1)
    q[:, :, 0] = torch.tensor([6.5, 8.0, 8.5])[rows % 3]
    case.q, case.k_new, case.v_new = q.to(torch.bfloat16), kn.to(torch.bfloat16), vn.to(torch.bfloat16)
    case.k_cache, case.v_cache = kc.to(torch.bfloat16), vc.to(torch.bfloat16)
    if fp8:
        kq, ks = ref_ops.quantize_pages_fp8(case.k_cache)
        vq, vs = ref_ops.quantize_pages_fp8(case.v_cache)
        case.k_cache_ref = ref_ops.dequantize_pages_fp8(kq, ks)
        case.v_cache_ref = ref_ops.dequantize_pages_fp8(vq, vs)
        case.k_cache, case.v_cache, case.k_scale, case.v_scale = kq, vq, ks, vs
    case.meta.update(gran=gran, step=step, fp8=fp8)
    return case
