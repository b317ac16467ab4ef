"""Pins the CPU oracle (oracle/ref_ops.py) against closed forms, library routines, invariants and
brute force, so that a dropped term, a wrong sign or index, or a transposed operand fails here.
Runs on CPU only."""
import itertools
import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import configs, ref_ops

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ---------------------------------------------------------------- paged addressing / store / load

def test_slot_mapping_closed_form_and_fixture():
    pages = [5, 2, 9]
    s = ref_ops.slot_mapping(pages, 600, start_token=100)
    for i in (0, 155, 156, 411, 412, 599):
        t = 100 + i
        assert int(s[i]) == pages[t // 256] * 256 + t % 256
    # the reference's own slot-mapping fixture: 160 skipped rows, slots 882..913, 896 skipped rows
    with open(os.path.join(GOLDEN, "mimic_slot_mapping.json")) as f:
        fx = json.load(f)
    assert fx["length"] == 1088 and fx["runs"] == [["skip", 0, 160], ["run", 882, 32], ["skip", 0, 896]]
    # slots 882..913 are tokens 114..145 of page 3 (882 = 3*256 + 114): the active block of a sequence
    # with context 114 stored behind its context, as the reference's load test expects
    assert torch.equal(ref_ops.slot_mapping([0, 1, 2, 3], 32, start_token=3 * 256 + 114),
                       torch.arange(882, 914, dtype=torch.int32))


def test_store_skips_negative_slots_and_load_roundtrip():
    gen = torch.Generator().manual_seed(0)
    kc = torch.zeros(4, 256, 2, 8)
    vc = torch.zeros(4, 256, 2, 8)
    k = torch.randn(300, 2, 8, generator=gen)
    v = torch.randn(300, 2, 8, generator=gen)
    slots = ref_ops.slot_mapping([3, 1], 300)
    slots[7] = -1
    ref_ops.store_kvcache(k, v, kc, vc, slots)
    assert torch.equal(kc[3, :7], k[:7]) and kc[3, 7].abs().sum() == 0 and torch.equal(kc[1, :44], k[256:])
    # load == brute-force gather of the context followed by the active rows (CHECK_LOADING semantics)
    kn = torch.randn(64, 2, 8, generator=gen)
    ko, vo = ref_ops.load_kvcache(kc, vc, [[3, 1], [1, 0]], [300, 10], [32, 32], kn, kn)
    assert ko.shape[0] == 300 + 32 + 10 + 32
    assert torch.equal(ko[:256], kc[3]) and torch.equal(ko[256:300], kc[1, :44]) and torch.equal(ko[300:332], kn[:32])
    assert torch.equal(ko[332:342], kc[1, :10]) and torch.equal(ko[342:], kn[32:])


def test_gather_scatter_compaction_invariants():
    gen = torch.Generator().manual_seed(1)
    cache = torch.randn(6, 256, 2, 4, generator=gen)
    pages = [4, 0, 5]
    snap = ref_ops.gather_tokens(cache, pages, torch.arange(700))
    fresh = torch.zeros_like(cache)
    ref_ops.scatter_tokens(fresh, [1, 2, 3], snap)
    assert torch.equal(ref_ops.gather_tokens(fresh, [1, 2, 3], torch.arange(700)), snap)  # gather(scatter(x)) == x
    # per-head compaction: brute force, head by head, token by token
    keep = torch.stack([torch.sort(torch.randperm(700, generator=gen)[:300]).values for _ in range(2)])
    before = cache.clone()
    ref_ops.compact_per_head(cache, pages, keep)
    for h in range(2):
        for j in (0, 1, 150, 299):
            t = int(keep[h, j])
            assert torch.equal(cache[pages[j // 256], j % 256, h], before[pages[t // 256], t % 256, h])
    # tokens beyond the kept length are untouched
    assert torch.equal(cache[pages[2], 100:], before[pages[2], 100:])


def test_chunk_local_kv_copy_token_by_token():
    """copy_chunk_local_kv against a token-by-token loop over plain Python indices: source chunk that starts in
    the middle of a page, destination that starts in the middle of another, source and destination page lists
    that share pages (the copy of a head reads everything before it writes), a different keep list per head."""
    gen = torch.Generator().manual_seed(6)
    P, H, d = 256, 3, 4
    cache = torch.randn(7, P, H, d, generator=gen)
    src_pages, dst_pages = [5, 2, 6], [2, 0, 3]          # page 2 is both read and written
    src_chunk_start, dst_start, chunk_len, keep_n = 200, 130, 500, 330
    keep = torch.stack([torch.sort(torch.randperm(chunk_len, generator=gen)[:keep_n]).values for _ in range(H)])
    keep[1] = torch.arange(keep_n)                        # one head keeps a plain prefix
    before = cache.clone()
    ref_ops.copy_chunk_local_kv(cache, src_pages, dst_pages, src_chunk_start, dst_start, keep)
    want = before.clone()
    for h in range(H):
        for j in range(keep_n):
            s = int(keep[h, j]) + src_chunk_start
            t = dst_start + j
            want[dst_pages[t // P], t % P, h] = before[src_pages[s // P], s % P, h]
    assert torch.equal(cache, want)
    # some destination slot really lay inside the source range of page 2 (the overlap is exercised) ...
    assert any(dst_pages[(dst_start + j) // P] == 2 for j in range(keep_n))
    assert any(src_pages[(int(keep[0, j]) + src_chunk_start) // P] == 2 for j in range(keep_n))
    # ... and nothing outside the destination range changed
    touched = torch.zeros(7, P, dtype=torch.bool)
    for j in range(keep_n):
        touched[dst_pages[(dst_start + j) // P], (dst_start + j) % P] = True
    assert torch.equal(cache[~touched], before[~touched])


# ---------------------------------------------------------------- attention

def _sdpa64(q, k, v, mask, scale):
    G = q.shape[1] // k.shape[1]
    qq = q.double().permute(1, 0, 2).unsqueeze(0)
    kk = k.double().permute(1, 0, 2).repeat_interleave(G, 0).unsqueeze(0)
    vv = v.double().permute(1, 0, 2).repeat_interleave(G, 0).unsqueeze(0)
    o = F.scaled_dot_product_attention(qq, kk, vv, attn_mask=mask, scale=scale)
    return o[0].permute(1, 0, 2)


def test_attention_matches_torch_sdpa_fp64_gqa_and_paging():
    case = configs.chunked_prefix_case(3, n_req=2, n_chunks=3, chunk_tokens=130, topk=2, q_len=24, Hq=6, Hkv=2, d=16,
                                       shared_prefix=False)
    out = ref_ops.sparse_decode_attention(case.q, case.k_new, case.v_new, case.k_cache, case.v_cache, case.block_table,
                                          case.q_start_loc, case.ranges, sm_scale=0.3)
    for r in range(2):
        a, b = r * 24, (r + 1) * 24
        toks = [t for s, l in case.ranges[r] for t in range(s, s + l)]
        kp = torch.stack([case.k_cache[int(case.block_table[r][t // 256]), t % 256] for t in toks])
        vp = torch.stack([case.v_cache[int(case.block_table[r][t // 256]), t % 256] for t in toks])
        ref = _sdpa64(case.q[a:b], torch.cat([kp, case.k_new[a:b]]), torch.cat([vp, case.v_new[a:b]]), None, 0.3)
        assert (out[a:b].double() - ref).abs().max() < 1e-5
    # GQA grouping is head // G, not head % Hkv: swapping two KV heads changes exactly their q-head groups
    k2 = case.k_cache.clone()
    k2[:, :, 0] = case.k_cache[:, :, 1]
    out2 = ref_ops.sparse_decode_attention(case.q, case.k_new, case.v_new, k2, case.v_cache, case.block_table,
                                           case.q_start_loc, case.ranges, sm_scale=0.3)
    assert (out2[:, 3:] - out[:, 3:]).abs().max() == 0 and (out2[:, :3] - out[:, :3]).abs().max() > 0


def test_attention_masks_and_invariants():
    case = configs.chunked_prefix_case(4, n_req=1, n_chunks=2, chunk_tokens=70, topk=1, q_len=20, Hq=4, Hkv=2, d=16)
    # causal == SDPA with [ones(ctx) | tril]
    out = ref_ops.sparse_decode_attention(case.q, case.k_new, case.v_new, case.k_cache, case.v_cache, case.block_table,
                                          case.q_start_loc, case.ranges, mask_mode="causal")
    s, l = case.ranges[0][0]
    kp = torch.stack([case.k_cache[int(case.block_table[0][t // 256]), t % 256] for t in range(s, s + l)])
    vp = torch.stack([case.v_cache[int(case.block_table[0][t // 256]), t % 256] for t in range(s, s + l)])
    m = torch.cat([torch.ones(20, 70, dtype=torch.bool), torch.tril(torch.ones(20, 20, dtype=torch.bool))], 1)
    ref = _sdpa64(case.q, torch.cat([kp, case.k_new]), torch.cat([vp, case.v_new]), m, 0.25)
    assert (out.double() - ref).abs().max() < 1e-5
    # rows of a softmax sum to one: V == 1 gives O == 1
    ones = ref_ops.sparse_decode_attention(case.q, case.k_new, torch.ones_like(case.v_new), case.k_cache,
                                           torch.ones_like(case.v_cache), case.block_table, case.q_start_loc,
                                           case.ranges)
    assert (ones - 1).abs().max() < 1e-5
    # split / merge identity: attention over two key sets merges by log-sum-exp weights
    q, k, v = case.q[:, :2].float(), case.k_new.float(), case.v_new.float()
    full = ref_ops._sdpa(q, k, v, None, 0.25)

    def part(ks, vs):
        s_ = torch.einsum("qhd,khd->hqk", q, ks) * 0.25
        m_ = s_.amax(-1)
        p_ = torch.exp(s_ - m_[..., None])
        return m_, p_.sum(-1), torch.einsum("hqk,khd->hqd", p_, vs)

    m1, l1, o1 = part(k[:7], v[:7])
    m2, l2, o2 = part(k[7:], v[7:])
    mm = torch.maximum(m1, m2)
    o = (o1 * torch.exp(m1 - mm)[..., None] + o2 * torch.exp(m2 - mm)[..., None]) / \
        (l1 * torch.exp(m1 - mm) + l2 * torch.exp(m2 - mm))[..., None]
    assert (o.permute(1, 0, 2) - full).abs().max() < 1e-5


def test_chunk_prefill_is_block_diagonal():
    gen = torch.Generator().manual_seed(5)
    lens = [5, 9, 1]
    n = sum(lens)
    q = torch.randn(n, 4, 8, generator=gen)
    k = torch.randn(n, 2, 8, generator=gen)
    v = torch.randn(n, 2, 8, generator=gen)
    cu = [0, 5, 14, 15]
    out = ref_ops.chunk_prefill_attention(q, k, v, cu, causal=True)
    for a, b in zip(cu[:-1], cu[1:]):
        m = torch.tril(torch.ones(b - a, b - a, dtype=torch.bool))
        ref = _sdpa64(q[a:b], k[a:b], v[a:b], m, 1 / math.sqrt(8))
        assert (out[a:b].double() - ref).abs().max() < 1e-5
    # a dense [S, S] block-diagonal causal mask over the packed batch gives the same (context.py:73-84)
    dense = torch.zeros(n, n, dtype=torch.bool)
    for a, b in zip(cu[:-1], cu[1:]):
        dense[a:b, a:b] = torch.tril(torch.ones(b - a, b - a, dtype=torch.bool))
    ref = _sdpa64(q, k, v, dense, 1 / math.sqrt(8))
    assert (out.double() - ref).abs().max() < 1e-5


def test_split_token_chunks():
    assert ref_ops.split_token_chunks(list(range(10)), 4) == [[0, 1, 2, 3], [4, 5, 6, 7], [8, 9]]
    assert ref_ops.split_token_chunks(list(range(10)), 4, split_from_tail=True) == [[0, 1], [2, 3, 4, 5], [6, 7, 8, 9]]
    assert ref_ops.split_token_chunks([1, 2], 4) == [[1, 2]] and ref_ops.split_token_chunks([], 4) == []


# ---------------------------------------------------------------- rope

def test_rope_is_a_rotation_and_matches_complex_form():
    cs = ref_ops.rope_cos_sin_cache(16, 64, base=10000.0)
    gen = torch.Generator().manual_seed(6)
    x = torch.randn(5, 3, 16, generator=gen)
    pos = torch.tensor([0, 1, 7, 33, 63])
    y = ref_ops.apply_rope(x, pos, cs)
    assert torch.equal(y[0], x[0])                                   # position 0 is the identity
    assert ((y[..., :8] ** 2 + y[..., 8:] ** 2) - (x[..., :8] ** 2 + x[..., 8:] ** 2)).abs().max() < 1e-5
    # complex form: (x1 + i x2) * exp(i pos * base^(-2j/d))
    inv = 1.0 / (10000.0 ** (torch.arange(0, 16, 2).double() / 16))
    ang = pos.double()[:, None] * inv[None, :]
    z = torch.complex(x[..., :8].double(), x[..., 8:].double()) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    assert (y[..., :8].double() - z.real).abs().max() < 1e-5 and (y[..., 8:].double() - z.imag).abs().max() < 1e-5


# ---------------------------------------------------------------- scoring / ranking

def test_selfinfo_matches_scipy_logsumexp():
    from scipy.special import logsumexp
    gen = torch.Generator().manual_seed(7)
    logits = (torch.randn(6, 5000, generator=gen) * 4).to(torch.bfloat16)
    labels = torch.randint(0, 5000, (6,), generator=gen)
    got = ref_ops.selfinfo_logprob(logits, labels)
    x = logits.double().numpy()
    ref = x[np.arange(6), labels.numpy()] - logsumexp(x, axis=1)
    assert np.abs(got.numpy() - ref).max() < 1e-5
    sc = ref_ops.chunk_scores(logits.view(3, 2, 5000), labels.view(3, 2), mean=True)
    assert np.abs(sc.numpy() - ref.reshape(3, 2).mean(1)).max() < 1e-5


def test_topk_bruteforce_with_ties_and_nonfinite():
    vals = [1.0, 2.0, 2.0, float("nan"), -1.0, 2.0, float("inf"), 0.5]
    clean = [v if math.isfinite(v) else float("-inf") for v in vals]
    for k in range(1, 9):
        # brute force: the k-subset maximising the score multiset, then preferring low indices
        best = max(itertools.combinations(range(8), k),
                   key=lambda c: (sorted((clean[i] for i in c), reverse=True), [-i for i in c]))
        assert ref_ops.topk_lowest_index(vals, k) == sorted(best)
    assert ref_ops.topk_lowest_index(vals, 3, sorted_ascending=False) == [1, 2, 5]


def test_select_positions_branches_match_reference_semantics():
    s = torch.tensor([0.1, 0.9, 0.3, 0.9, 0.2, 0.05])
    f = ref_ops.select_positions_from_token_scores
    assert f(s, capacity=1, chunk_len=6).tolist() == [0]
    assert f(s, capacity=3, chunk_len=6).tolist() == [0, 1, 3]                  # BOS + two best
    assert f(s, capacity=2, chunk_len=6).tolist() == [0, 1]                     # tie 0.9 -> lowest index
    assert f(s, capacity=6, chunk_len=6).tolist() == [0, 1, 2, 3, 4, 5]         # everything fits
    assert f(s, capacity=0, chunk_len=6).tolist() == [0]                        # max(1, capacity)
    assert f(s, capacity=3, chunk_len=6, force_keep_first=False).tolist() == [1, 2, 3]
    assert f(s, capacity=3, chunk_len=6, keep_high=False).tolist() == [0, 4, 5]
    assert f(s[:4], capacity=4, chunk_len=6).tolist() == [0, 1, 4, 5]           # wrong length -> head/tail
    # agrees with torch.topk wherever torch's answer is unique (no ties at the cut)
    gen = torch.Generator().manual_seed(8)
    r = torch.rand(100, generator=gen)
    sel = torch.arange(1, 100)[torch.topk(r[1:], 19).indices]
    ref = torch.sort(torch.cat([torch.zeros(1, dtype=torch.long), sel])).values
    assert f(r, capacity=20, chunk_len=100).tolist() == ref.tolist()


def test_evict_colsum_closed_form_and_mass():
    p = configs.eviction_probs(1, n_chunks=2, H=4, Q=6, K=33)
    got = ref_ops.evict_colsum(p)
    assert (got[:, 0] - p.sum(dim=(1, 2))).abs().max() < 1e-5
    assert (got.sum(-1) - 4 * 6).abs().max() < 1e-4                     # every softmax row sums to one
    g2 = ref_ops.evict_colsum(p, heads_per_group=2)
    assert (g2[:, 1] - p[:, 2:4].sum(dim=(1, 2))).abs().max() < 1e-5


def test_head_scores_match_closed_form():
    gen = torch.Generator().manual_seed(9)
    prefix, chunk, ql = 2, 11, 3
    S = prefix + chunk + ql
    q = torch.randn(S, 4, 8, generator=gen)
    k = torch.randn(S, 2, 8, generator=gen)
    got = ref_ops.chunk_attention_head_scores(q, k, prefix_len=prefix, chunk_len=chunk, query_len=ql, scale=0.3)
    ref = torch.zeros(4, chunk, dtype=torch.float64)
    for h in range(4):
        for r in range(prefix + chunk, S):
            logit = (q[r, h].double() @ k[:r + 1, h // 2].double().T) * 0.3    # causal: keys <= row
            ref[h] += torch.softmax(logit, -1)[prefix:prefix + chunk]
    assert (got.double() - ref).abs().max() < 1e-5
    full = ref_ops.chunk_attention_head_scores(q, k, prefix_len=prefix, chunk_len=chunk, query_len=ql, scale=0.3,
                                               attention_mask="full", reduce_mode="mean")
    ref = torch.zeros(4, chunk, dtype=torch.float64)
    for h in range(4):
        for r in range(prefix + chunk, S):
            ref[h] += torch.softmax((q[r, h].double() @ k[:, h // 2].double().T) * 0.3, -1)[prefix:prefix + chunk] / ql
    assert (full.double() - ref).abs().max() < 1e-5


def test_pool_group_brute_force():
    gen = torch.Generator().manual_seed(10)
    s = torch.rand(4, 9, generator=gen)
    mp = ref_ops.token_score_pool_group(s, "maxpool", 3)
    ap = ref_ops.token_score_pool_group(s, "avgpool", 3)
    for i in range(9):
        w = s[:, max(0, i - 1):i + 2]
        assert torch.equal(mp[:, i], w.max(1).values)
        assert (ap[:, i] - w.sum(1) / 3).abs().max() < 1e-6            # zero padding counts in the average
    g = ref_ops.token_score_pool_group(s, "none", 1, num_kv_heads=2)
    assert (g[1] - (s[2] + s[3]) / 2).abs().max() < 1e-7


# ---------------------------------------------------------------- confidence / unmask / fp8

def test_shift_sample_unmask():
    gen = torch.Generator().manual_seed(11)
    logits = (torch.randn(4, 50, generator=gen) * 3).to(torch.bfloat16)
    last = (torch.randn(50, generator=gen) * 3).to(torch.bfloat16)
    sh = ref_ops.shift_logits(logits, last)
    assert torch.equal(sh[0], last) and torch.equal(sh[1:], logits[:-1])
    assert torch.equal(ref_ops.shift_logits(logits)[0], logits[0])
    conf, tok = ref_ops.sample_tokens(logits)
    x = logits.double()
    assert (conf.double() - 1.0 / torch.exp(x - x.max(-1, keepdim=True).values).sum(-1)).abs().max() < 1e-6
    assert torch.equal(tok, x.argmax(-1))
    tie = torch.zeros(1, 10, dtype=torch.bfloat16)
    assert int(ref_ops.sample_tokens(tie)[1]) == 0                      # first index of the maximum
    # transfer set == {most confident masked position} U {masked positions with confidence >= threshold}
    block = torch.tensor([7, 99, 99, 99, 8, 99])
    c = torch.tensor([1.0, 0.95, 0.2, 0.95, 1.0, 0.91])
    t = torch.tensor([1, 2, 3, 4, 5, 6])
    nb, tr = ref_ops.threshold_unmask(block, c, t, 99, 0.9)
    assert tr.tolist() == [False, True, False, True, False, True] and nb.tolist() == [7, 2, 99, 4, 8, 6]
    nb, tr = ref_ops.threshold_unmask(block, c * 0.5, t, 99, 0.9)
    assert tr.tolist() == [False, True, False, False, False, False]     # ties -> lowest index, exactly one
    nb, tr = ref_ops.threshold_unmask(torch.tensor([1, 2]), c[:2], t[:2], 99, 0.9)
    assert not tr.any()


def test_fp8_page_quantisation():
    gen = torch.Generator().manual_seed(12)
    cache = torch.randn(3, 256, 2, 16, generator=gen)
    cache[1] *= 100
    q, scale = ref_ops.quantize_pages_fp8(cache)
    assert q.dtype == torch.float8_e4m3fn and (scale - cache.abs().amax(dim=(1, 2, 3)) / 448).abs().max() < 1e-6
    deq = q.float() * scale.view(-1, 1, 1, 1)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 for normal values, absolute <= scale * 2^-10 below
    err = (deq - cache).abs()
    assert (err <= cache.abs() * 2 ** -4 + scale.view(-1, 1, 1, 1) * 2 ** -9).all()
    assert ref_ops.dequantize_pages_fp8(q, scale).dtype == torch.bfloat16


def test_vote_topk_against_an_independent_formulation():
    """The vote keep set (preevict_votetopk.sh:231-258) against numpy: bincount for the votes and a stable
    argsort of the negated votes for the order, plus what the definition fixes: the first token of every chunk
    and every token outside the chunks survive, a chunk keeps min(capacity, length) tokens, and no dropped token
    has more votes than a kept non-first one."""
    import numpy as np
    rng = np.random.default_rng(3)
    n = 90
    spans = [(5, 30), (30, 31), (40, 80)]
    keep_idx = [[sorted(rng.choice(n + 5, size=20, replace=False).tolist()) for _ in range(3)] for _ in range(4)]
    votes = np.bincount(np.array([i for l in keep_idx for h in l for i in h if i < n]), minlength=n)
    for cap in (0, 1, 4, 10, 100):
        got = ref_ops.preevict_vote_topk_indices(keep_idx, n, spans, cap)
        want = set(range(0, 5)) | set(range(31, 40)) | set(range(80, n))
        for s0, e0 in spans:
            length = e0 - s0
            k = length if cap <= 0 else min(max(1, cap), length)
            order = np.argsort(-votes[s0 + 1:e0], kind="stable") + s0 + 1
            want |= {s0} | set(order[:k - 1].tolist())
            kept = [i for i in got if s0 <= i < e0]
            assert s0 in kept and len(kept) == k
            dropped = [i for i in range(s0 + 1, e0) if i not in kept]
            if dropped and len(kept) > 1:
                assert max(votes[dropped]) <= min(votes[[i for i in kept if i != s0]])
        assert got == sorted(want)
    assert ref_ops.preevict_vote_topk_indices([], 4, [], 2) == [0, 1, 2, 3]


# ---- experimental anchor corrections ----

def test_anchor_windows_hand_listed_tables():
    """Anchors and windows read off the reference loops by hand (ATT:113-125, 151-165)."""
    aw = ref_ops.anchor_windows
    assert aw(10, {}) == ([3, 7], [[0, 1, 2, 3], [4, 5, 6, 7]])                     # stride 4, left 3, offset 3
    assert aw(10, dict(direction="right", right=2)) == ([3, 7], [[3, 4, 5], [7, 8, 9]])
    assert aw(9, dict(direction="right", right=3)) == ([3, 7], [[3, 4, 5, 6], [7, 8]])   # clipped at the end
    assert aw(10, dict(direction="both", left=1, right=1)) == ([3, 7], [[2, 3, 4], [6, 7, 8]])
    assert aw(9, dict(anchor_offset=0)) == ([0, 4, 8], [[0], [1, 2, 3, 4], [5, 6, 7, 8]])
    assert aw(10, dict(anchor_offset=-5))[0] == [3, 7]                              # negative -> stride - 1
    assert aw(10, dict(anchor_offset=99))[0] == [3, 7]                              # clamped to stride - 1
    assert aw(10, dict(stride=2, left=5))[1][1] == [0, 1, 2, 3]                      # overlapping windows
    assert aw(3, {}) == ([], [])
    assert aw(7, dict(stride=0, left=0))[0] == list(range(7))                       # stride < 1 -> 1


def test_decode_delta_reduces_to_known_cases():
    gen = torch.Generator().manual_seed(5)
    Hq, Hkv, d, S, P = 8, 2, 32, 12, 40
    q = torch.randn(S, Hq, d, generator=gen)
    k, v = torch.randn(S, Hkv, d, generator=gen), torch.randn(S, Hkv, d, generator=gen)
    fk, fv = torch.randn(P, Hkv, d, generator=gen), torch.randn(P, Hkv, d, generator=gen)
    keep = torch.arange(0, P, 3)                                                    # the sparse prefix: every third key
    full = torch.ones(S, S + keep.numel(), dtype=torch.bool)
    o = ref_ops._sdpa(q, torch.cat([fk[keep], k]), torch.cat([fv[keep], v]), full, d ** -0.5)
    dense_all = ref_ops._sdpa(q, torch.cat([fk, k]), torch.cat([fv, v]), torch.ones(S, S + P, dtype=torch.bool), d ** -0.5)
    # every row an anchor with a window of one row and scale 1: the result is the dense attention itself
    got = ref_ops.decode_delta(o, q, k, v, fk, fv, dict(stride=1, left=0))
    assert (got - dense_all).abs().max() < 1e-5
    # scale 0.5 moves every row half way
    got = ref_ops.decode_delta(o, q, k, v, fk, fv, dict(stride=1, left=0, scale=0.5))
    assert (got - (o + dense_all) / 2).abs().max() < 1e-5
    # a "full" prompt equal to the sparse prefix changes nothing
    got = ref_ops.decode_delta(o, q, k, v, fk[keep], fv[keep], {})
    assert (got - o).abs().max() < 1e-5
    # default windows: rows 0-3 receive the delta of row 3, rows 4-7 that of row 7, rows 8-11 that of row 11
    got = ref_ops.decode_delta(o, q, k, v, fk, fv, {})
    for r in range(S):
        a = r // 4 * 4 + 3
        assert (got[r] - (o[r] + dense_all[a] - o[a])).abs().max() < 1e-5
    # an active mask only changes the anchors' view of the active keys
    am = torch.tril(torch.ones(S, S, dtype=torch.bool))
    got = ref_ops.decode_delta(o, q, k, v, fk, fv, dict(stride=1, left=0), active_mask=am)
    causal = ref_ops._sdpa(q, torch.cat([fk, k]), torch.cat([fv, v]),
                           torch.cat([torch.ones(S, P, dtype=torch.bool), am], 1), d ** -0.5)
    assert (got - causal).abs().max() < 1e-5


def test_prefill_sparse_reduces_to_known_cases():
    gen = torch.Generator().manual_seed(6)
    Hq, Hkv, d, S = 4, 2, 32, 14
    q = torch.randn(S, Hq, d, generator=gen)
    k, v = torch.randn(S, Hkv, d, generator=gen), torch.randn(S, Hkv, d, generator=gen)
    causal = torch.tril(torch.ones(S, S, dtype=torch.bool))
    dense = ref_ops._sdpa(q, k, v, causal, d ** -0.5)
    every = torch.arange(S)
    # all keys kept: the sparse prefill is the dense one, with or without the delta
    for st in ({}, dict(delta_mode="s4_left3")):
        assert (ref_ops.prefill_sparse_attention(q, k, v, causal, every, st) - dense).abs().max() < 1e-6
    # a subset: the same as attention over the gathered keys with the causal mask gathered alike
    keep = torch.tensor([0, 2, 3, 7, 8, 12, 40, -1])                                 # out-of-range entries are ignored
    kk = keep[(keep >= 0) & (keep < S)]
    sub = ref_ops._sdpa(q, k[kk], v[kk], causal[:, kk], d ** -0.5)
    got = ref_ops.prefill_sparse_attention(q, k, v, causal, keep, {})
    assert (got - sub).abs().max() < 1e-6
    # keys from full_prompt_len on are always visible
    got = ref_ops.prefill_sparse_attention(q, k, v, causal, keep, dict(full_prompt_len=10))
    kk2 = torch.tensor([0, 2, 3, 7, 8, 10, 11, 12, 13])
    assert (got - ref_ops._sdpa(q, k[kk2], v[kk2], causal[:, kk2], d ** -0.5)).abs().max() < 1e-6
    # delta: anchors 3, 7, 11 land on the dense result, their windows move by the same amount; rows 12, 13 stay
    got = ref_ops.prefill_sparse_attention(q, k, v, causal, keep, dict(delta_mode="s4_left3"))
    for r in range(S):
        a = r // 4 * 4 + 3
        want = sub[r] + (dense[a] - sub[a]) if a < S else sub[r]
        assert (got[r] - want).abs().max() < 1e-5
    with_sel = dict(delta_mode="s4_left3", selection_mode="selection_dense_add", selection_scale=0.7)
    # selection outputs equal to the dense result: both selection modes give the plain correction
    g_add = ref_ops.prefill_sparse_attention(q, k, v, causal, keep, with_sel, selection_outputs=dense)
    assert (g_add - got).abs().max() < 1e-5
    rep = dict(delta_mode="s4_left3", selection_mode="selection_dense_replace")
    g_rep = ref_ops.prefill_sparse_attention(q, k, v, causal, keep, rep, selection_outputs=dense)
    assert (g_rep - got).abs().max() < 1e-5
    # replace with counts == 0 everywhere, or no selection at all: the sparse result is returned
    g0 = ref_ops.prefill_sparse_attention(q, k, v, causal, keep, rep, selection_outputs=dense,
                                          selection_counts=torch.zeros(S, dtype=torch.long))
    assert torch.equal(g0, sub.to(g0.dtype)) or (g0 - sub).abs().max() < 1e-6
    # a selection shorter than the sequence: anchors past its end are not valid (replace: no correction there)
    g_short = ref_ops.prefill_sparse_attention(q, k, v, causal, keep, rep, selection_outputs=dense[:8])
    assert (g_short[:8] - got[:8]).abs().max() < 1e-5 and (g_short[8:] - sub[8:]).abs().max() < 1e-6


def test_partial_draft_rounds_hand_trace():
    """fastdllm_engine.py:1013-1059 on a hand-computed trace.  Vocabulary of 5, prompt of 2, draft of 4, mask id 4.
    The stand-in model returns fixed rows: the logits row at position p decides block position p - prompt_len + 1
    (the shift).  Row sharpness: block position 0 <- row 1 (weak), 1 <- row 2 (sharpest), 2 <- row 3 and 3 <- row 4
    (equal, medium).  Position 0 is confirmed first although it is the weakest; then position 1; then the tie of
    positions 2 and 3 goes to position 2; a fourth round takes 3; a fifth finds no mask."""
    import torch
    rows = torch.zeros(6, 5)
    rows[1, 3] = 0.5     # -> block position 0: token 3
    rows[2, 1] = 9.0     # -> block position 1: token 1
    rows[3, 2] = 4.0     # -> block position 2: token 2
    rows[4, 0] = 4.0     # -> block position 3: token 0 (same confidence as position 2)
    calls = []

    def logits_of(ids):
        calls.append(list(ids))
        return rows.clone()

    ids, conf = ref_ops.partial_draft_rounds(logits_of, [7, 8], 4, 0, 4)
    assert ids == [3, 4, 4, 4] and conf == [True, False, False, False]
    ids, conf = ref_ops.partial_draft_rounds(logits_of, [7, 8], 4, 1, 4)
    assert ids == [3, 1, 4, 4] and conf == [True, True, False, False]
    ids, conf = ref_ops.partial_draft_rounds(logits_of, [7, 8], 4, 2, 4)
    assert ids == [3, 1, 2, 4] and conf == [True, True, True, False]
    calls.clear()
    ids, conf = ref_ops.partial_draft_rounds(logits_of, [7, 8], 4, 9, 4)
    assert ids == [3, 1, 2, 0] and conf == [True] * 4
    assert len(calls) == 4 and calls[-1] == [7, 8, 3, 1, 2, 4]     # stops when no mask is left
    assert ref_ops.partial_draft_rounds(logits_of, [7, 8], 0, 3, 4) == ([], [])


def test_assemble_global_keep_indices_hand_listed():
    """fastdllm_engine.py:1524-1546: prompt of 12, chunks [2,5) and [5,9) (adjacent), 2 heads.  Head 0 keeps {2,4}
    and {5,8}, head 1 keeps {3,4} and {6,7}; positions 0-1 and 9-11 lie outside every chunk."""
    keeps = [[[[2, 4], [3, 4]], [[5, 8], [6, 7]]], []]
    out = ref_ops.assemble_global_keep_indices(keeps, [(2, 5), (5, 9)], 12, 2)
    assert out[0] == [[0, 1, 2, 4, 5, 8, 9, 10, 11], [0, 1, 3, 4, 6, 7, 9, 10, 11]]
    assert out[1] == [list(range(12)), list(range(12))]
    # a chunk that starts at 0 and one that ends at the prompt end: no gap, no tail
    out = ref_ops.assemble_global_keep_indices([[[[0]], [[3]]]], [(0, 2), (2, 4)], 4, 1)
    assert out == [[[0, 3]]]
