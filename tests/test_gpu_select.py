"""GPU parity of scoring / top-K / eviction / unmask / rope kernels against the CPU oracle."""
import pytest
import torch

from oracle import configs, ref_ops

pytestmark = pytest.mark.gpu


def _ops():
    from prefilling_dllm_amd import ops
    return ops


def test_selfinfo_and_chunk_topk_config2(dev):
    """BASELINE config 2 scoring: [32 chunks, 4 draft tokens, vocab 152064] bf16 logits -> per chunk
    summed log-probability of the labels -> top-4 chunk indices, bit exact."""
    logits, labels = configs.draft_logits(seed=0)
    ops = _ops()
    lp = ops.selfinfo_logprob(logits.reshape(-1, logits.shape[-1]).to(dev), labels.reshape(-1).to(dev)).cpu()
    lp_ref = ref_ops.selfinfo_logprob(logits.reshape(-1, logits.shape[-1]), labels.reshape(-1))
    assert (lp - lp_ref).abs().max() <= 2e-5 * lp_ref.abs().max()
    for mean in (False, True):
        sc = ops.chunk_scores_from_logits(logits.to(dev), labels.to(dev), mean=mean)
        sc_ref = ref_ops.chunk_scores(logits, labels, mean=mean)
        assert (sc.cpu() - sc_ref).abs().max() <= 1e-4
        idx = ops.topk_lowest_index(sc, 4).cpu().tolist()
        assert idx == ref_ops.topk_lowest_index(sc_ref.tolist(), 4)
        # the separation of the scores around the cut must exceed the reduction error
        srt = sorted(sc_ref.tolist(), reverse=True)
        assert srt[3] - srt[4] > 1e-3


def test_chunk_select_single_call_equals_the_three_calls(dev):
    """pdllm_chunk_select = selfinfo_logprob + chunk_score_reduce + topk_lowest_index, bit for bit, and the
    oracle's selection; also with tied and non-finite chunk scores (labels outside the vocabulary give -inf)."""
    ops = _ops()
    logits, labels = configs.draft_logits(seed=4)
    dl, dlab = logits.to(dev), labels.to(dev)
    for mean in (False, True):
        for asc in (True, False):
            sc, idx = ops.chunk_select_from_logits(dl, dlab, 4, mean=mean, sorted_ascending=asc)
            sc3 = ops.chunk_scores_from_logits(dl, dlab, mean=mean)
            assert torch.equal(sc, sc3)
            assert torch.equal(idx, ops.topk_lowest_index(sc3, 4, sorted_ascending=asc))
            ref = ref_ops.chunk_scores(logits, labels, mean=mean)
            assert idx.cpu().tolist() == ref_ops.topk_lowest_index(ref.tolist(), 4, sorted_ascending=asc)
    # ties and -inf: chunks 1 and 2 are identical rows, chunk 3 has a label outside the vocabulary
    gen = torch.Generator().manual_seed(9)
    small = (torch.randn(6, 2, 5000, generator=gen) * 2).to(torch.bfloat16)
    small[2] = small[1]
    lab = torch.randint(0, 5000, (6, 2), generator=gen)
    lab[2] = lab[1]
    lab[3, 0] = -1
    for k in range(1, 7):
        sc, idx = ops.chunk_select_from_logits(small.to(dev), lab.to(dev), k, mean=False)
        assert torch.isinf(sc[3]) and sc[3] < 0 and sc[1] == sc[2]
        assert idx.cpu().tolist() == ref_ops.topk_lowest_index(sc.cpu().tolist(), k), k
        assert torch.equal(idx, ops.topk_lowest_index(sc, k))


def test_selfinfo_ragged_vocab_and_bad_label(dev):
    gen = torch.Generator().manual_seed(2)
    logits = (torch.randn(5, 1003, generator=gen) * 3).to(torch.bfloat16)  # rows not 16-byte aligned
    labels = torch.tensor([0, 1002, 17, -1, 5000])
    got = _ops().selfinfo_logprob(logits.to(dev), labels.to(dev)).cpu()
    ref = ref_ops.selfinfo_logprob(logits[:3], labels[:3])
    assert (got[:3] - ref).abs().max() <= 1e-5 * ref.abs().max() + 1e-6
    assert torch.isinf(got[3]) and got[3] < 0 and torch.isinf(got[4]) and got[4] < 0


def test_topk_ties_and_nonfinite(dev):
    ops = _ops()
    s = torch.tensor([1.0, 3.0, 3.0, float("nan"), 2.0, 3.0, float("inf"), -float("inf"), 2.0])
    for k in range(0, 10):
        if k == 0:
            continue
        got = ops.topk_lowest_index(s.to(dev), k).cpu().tolist()
        assert got == ref_ops.topk_lowest_index(s.tolist(), k), k
        got_r = ops.topk_lowest_index(s.to(dev), k, sorted_ascending=False).cpu().tolist()
        assert got_r == ref_ops.topk_lowest_index(s.tolist(), k, sorted_ascending=False), k
    # many equal scores: the selection is the k lowest indices
    z = torch.zeros(64)
    assert ops.topk_lowest_index(z.to(dev), 16).cpu().tolist() == list(range(16))
    # batched rows
    gen = torch.Generator().manual_seed(1)
    b = torch.randint(0, 5, (7, 33), generator=gen).float()
    got = ops.topk_lowest_index(b.to(dev), 8).cpu()
    for r in range(7):
        assert got[r].tolist() == ref_ops.topk_lowest_index(b[r].tolist(), 8)


def test_topk_long_rows_radix(dev):
    gen = torch.Generator().manual_seed(4)
    s = torch.randint(0, 50, (3, 5000), generator=gen).float()  # heavy ties
    got = _ops().topk_lowest_index(s.to(dev), 700).cpu()
    for r in range(3):
        assert got[r].tolist() == ref_ops.topk_lowest_index(s[r].tolist(), 700)


def test_eviction_config2_bit_exact(dev):
    """BASELINE config 2 eviction: probabilities [28, 64, 1025] per chunk, column sums over heads
    and queries, BOS + top-255 kept, indices bit exact."""
    probs = configs.eviction_probs(seed=0, n_chunks=3)
    ops = _ops()
    sc = ops.evict_colsum(probs.to(dev))
    sc_ref = ref_ops.evict_colsum(probs)
    assert torch.equal(sc.cpu(), sc_ref)                    # same summation order => same bits
    assert (sc_ref[:, 0].sum(-1) - 28 * 64).abs().max() < 1e-1  # rows of a softmax sum to one
    keep = ops.topb_keep_bos(sc[:, 0], 256).cpu()
    for c in range(3):
        ref = ref_ops.select_positions_from_token_scores(sc_ref[c, 0], capacity=256, chunk_len=1025)
        assert keep[c].tolist() == ref.tolist()
        assert keep[c, 0] == 0
    # per-KV-head grouping (7 q-heads per group)
    g = ops.evict_colsum(probs.to(dev), heads_per_group=7).cpu()
    assert torch.equal(g, ref_ops.evict_colsum(probs, heads_per_group=7))


def test_topb_degenerate_branches(dev):
    from prefilling_dllm_amd import engine_ops
    gen = torch.Generator().manual_seed(6)
    s = torch.rand(40, generator=gen)
    s[7] = s[9] = s[3]  # ties
    cases = [dict(capacity=1), dict(capacity=0), dict(capacity=39), dict(capacity=40), dict(capacity=100),
             dict(capacity=10), dict(capacity=10, keep_high=False), dict(capacity=10, force_keep_first=False),
             dict(capacity=10, keep_high=False, force_keep_first=False)]
    for kw in cases:
        got = engine_ops.select_positions_from_token_scores(s.to(dev), chunk_len=40, **kw).cpu().tolist()
        ref = ref_ops.select_positions_from_token_scores(s, chunk_len=40, **kw).tolist()
        assert got == ref, kw
    # wrong-length scores -> head/tail fallback
    got = engine_ops.select_positions_from_token_scores(s[:5].to(dev), capacity=6, chunk_len=40).cpu().tolist()
    assert got == ref_ops.select_positions_from_token_scores(s[:5], capacity=6, chunk_len=40).tolist()


@pytest.mark.parametrize("shape", [(8, 28, 64, 1025, 28), (8, 28, 64, 1025, 7), (3, 8, 5, 2048, 2), (2, 4, 3, 1024, 4),
                                   (5, 6, 7, 37, 3), (2, 4, 3, 2049, 2), (1, 2, 2, 1, 2)])
def test_evict_keep_from_probs_equals_the_two_calls(dev, shape):
    """One eviction step in one library call (fastdllm_engine.py:1230-1322 summed, then :903-927): the scores and the
    keep indices must be the bits of evict_colsum followed by topb_keep_bos, and the indices those of the oracle's
    selection on the same scores -- for one and several head groups, rows of 1 to 2049 keys (2049: the step falls
    back to the launches of the two calls), both score orders, with and without the forced first position, keep
    counts from 1 to the whole row, and rows in which most scores tie."""
    ops = _ops()
    c, h, nq, nk, hpg = shape
    gen = torch.Generator().manual_seed(sum(shape))
    probs = torch.rand(c, h, nq, nk, generator=gen)
    probs[0] = torch.round(probs[0] * 4) / 4                       # chunk 0: few distinct values, many ties
    if c > 1:
        probs[1] = 0.125                                           # chunk 1: every score equal
    dp = probs.to(dev)
    caps = sorted({0, 1, 2, nk // 4, nk - 1, nk, nk + 5} & set(range(0, nk + 6)))
    for cap in caps:
        for keep_high, force in ((True, True), (False, True), (True, False), (False, False)):
            sc, idx = ops.evict_keep_from_probs(dp, cap, hpg, keep_high=keep_high, force_keep_first=force)
            sc2 = ops.evict_colsum(dp, hpg)
            idx2 = ops.topb_keep_bos(sc2.view(-1, nk), cap, keep_high, force)
            assert torch.equal(sc, sc2) and torch.equal(idx, idx2), (shape, cap, keep_high, force)
    ref_sc = ref_ops.evict_colsum(probs, hpg)
    assert torch.equal(sc.cpu(), ref_sc)
    # a caller without a workspace gets the launches of the two calls: the same bits
    from prefilling_dllm_amd._lib import lib, check
    keep = min(max(1, nk // 3), nk)
    sc3 = torch.empty_like(sc2)
    idx3 = torch.empty((sc2.shape[0] * sc2.shape[1], keep), dtype=torch.int64, device=dev)
    check(lib.pdllm_evict_keep_from_probs(dp.data_ptr(), c, h, nq, nk, hpg, nk // 3, 1, 1, None, 0, sc3.data_ptr(),
                                          idx3.data_ptr(), torch.cuda.current_stream().cuda_stream), "no workspace")
    assert torch.equal(sc3, sc2) and torch.equal(idx3, ops.topb_keep_bos(sc2.view(-1, nk), nk // 3, True, True))
    cap = max(1, nk // 4)
    sc, idx = ops.evict_keep_from_probs(dp, cap, hpg)
    rows = ref_sc.view(-1, nk)
    for r in range(rows.shape[0]):
        assert idx[r].cpu().tolist() == ref_ops.select_positions_from_token_scores(rows[r], capacity=cap,
                                                                                   chunk_len=nk).tolist()


def test_query_to_chunk_scores(dev):
    gen = torch.Generator().manual_seed(9)
    prefix, chunk, ql = 3, 300, 8
    S = prefix + chunk + ql
    q = torch.randn(S, 28, 128, generator=gen).to(torch.bfloat16)
    k = torch.randn(S, 4, 128, generator=gen).to(torch.bfloat16)
    scale = 128 ** -0.5
    ops = _ops()
    for mask in ("causal", "full"):
        for red in ("sum", "mean"):
            got = ops.query_to_chunk_attention_scores(q.to(dev), k.to(dev), prefix_len=prefix, chunk_len=chunk,
                                                      query_len=ql, scale=scale, reduce_mode=red,
                                                      attention_mask=mask).cpu()
            ref = ref_ops.chunk_attention_head_scores(q, k, prefix_len=prefix, chunk_len=chunk, query_len=ql,
                                                      scale=scale, reduce_mode=red, attention_mask=mask)
            assert (got - ref).abs().max() <= 1e-4 * ref.abs().max() + 1e-7
    with pytest.raises(ValueError):
        ops.query_to_chunk_attention_scores(q.to(dev), k.to(dev), prefix_len=prefix, chunk_len=chunk - 1,
                                            query_len=65, scale=scale)


@pytest.mark.parametrize("prefix,chunk,ql,Hq,Hkv,d", [
    (0, 1025, 64, 28, 4, 128), (700, 1025, 8, 28, 4, 128), (5, 130, 1, 28, 4, 128), (33, 257, 20, 8, 8, 128),
    (0, 64, 13, 32, 2, 128),      # 16 q-heads per KV head
    (10, 100, 8, 4, 2, 64),       # another head dim: the vector-unit kernels
])
def test_query_to_chunk_scores_shapes(dev, prefix, chunk, ql, Hq, Hkv, d):
    """The matrix-core scorer (head dim 128) and the vector-unit one over ragged shapes: padding rows (query_len
    not a multiple of 8), several key segments, chunk lengths that are no multiple of 32, causal and full, and
    the same bits on a second run (fixed order of additions)."""
    gen = torch.Generator().manual_seed(prefix + chunk + ql)
    S = prefix + chunk + ql
    q = torch.randn(S, Hq, d, generator=gen).to(torch.bfloat16)
    k = torch.randn(S, Hkv, d, generator=gen).to(torch.bfloat16)
    scale = d ** -0.5
    ops = _ops()
    for mask in ("causal", "full"):
        for red in ("sum", "mean"):
            kw = dict(prefix_len=prefix, chunk_len=chunk, query_len=ql, scale=scale, reduce_mode=red, attention_mask=mask)
            got = ops.query_to_chunk_attention_scores(q.to(dev), k.to(dev), **kw).cpu()
            again = ops.query_to_chunk_attention_scores(q.to(dev), k.to(dev), **kw).cpu()
            ref = ref_ops.chunk_attention_head_scores(q, k, **kw)
            assert got.shape == ref.shape == (Hq, chunk)
            assert (got - ref).abs().max() <= 1e-4 * ref.abs().max() + 1e-7, (mask, red, (got - ref).abs().max())
            assert torch.equal(got, again)
    # every key column's mass over all heads and rows: a causal row sees itself, so the chunk columns of a row
    # never hold all of its mass; a full row's mass over chunk + the rest is 1
    full = ops.query_to_chunk_attention_scores(q.to(dev), k.to(dev), prefix_len=prefix, chunk_len=chunk, query_len=ql,
                                               scale=scale, attention_mask="full").cpu()
    assert (full.sum(dim=1) <= ql + 1e-3).all() and (full >= 0).all()


def test_pool_and_group(dev):
    gen = torch.Generator().manual_seed(10)
    s = torch.rand(28, 1025, generator=gen)
    ops = _ops()
    for pooling in ("none", "maxpool", "avgpool"):
        got = ops.token_score_pool_group(s.to(dev), pooling, 7, num_kv_heads=4).cpu()
        ref = ref_ops.token_score_pool_group(s, pooling, 7, num_kv_heads=4)
        assert (got - ref).abs().max() <= 1e-6, pooling
    got = ops.token_score_pool_group(s.to(dev), "maxpool", 7).cpu()
    assert torch.equal(got, ref_ops.token_score_pool_group(s, "maxpool", 7))


def test_unmask_config5_bit_exact(dev):
    """BASELINE config 5 unmask: bf16 logits [4*32, 126464], fp32 max-softmax >= 0.9 unmasks with the
    argmax token (LLaDA: no logit shift); decisions and tokens bit exact."""
    logits = configs.unmask_logits(seed=0)
    ops = _ops()
    conf, tok = ops.conf_argmax(logits.to(dev), 32)
    conf_ref, tok_ref = ref_ops.sample_tokens(logits)
    assert torch.equal(tok.cpu(), tok_ref)
    # fp32 sums in a different order and the hardware exp2: confidences agree to ~1e-5 relative
    assert (conf.cpu() - conf_ref).abs().max() <= 5e-5
    assert ((conf_ref - 0.9).abs() > 1e-3).all()  # no row sits on the threshold
    mask_id = 126336
    block = torch.full((4, 32), mask_id, dtype=torch.int64)
    block[:, 0] = 11  # already decoded positions stay
    block[2, 5] = 12
    dblock = block.to(dev)
    from prefilling_dllm_amd import engine_ops
    transfer, left = engine_ops.denoise_unmask_step(logits.to(dev), dblock, mask_token_id=mask_id, threshold=0.9,
                                                    shift=False)
    for b in range(4):
        nb, tr = ref_ops.threshold_unmask(block[b], conf_ref.view(4, 32)[b], tok_ref.view(4, 32)[b], mask_id, 0.9)
        assert torch.equal(dblock[b].cpu(), nb)
        assert torch.equal(transfer[b].cpu(), tr)
        assert int(left[b]) == int((nb == mask_id).sum())
        assert tr.sum() >= 1


def test_unmask_with_dream_shift(dev):
    gen = torch.Generator().manual_seed(12)
    vocab, L = 4096, 32
    logits = (torch.randn(2 * L, vocab, generator=gen) * 4).to(torch.bfloat16)
    last = (torch.randn(2, vocab, generator=gen) * 4).to(torch.bfloat16)
    conf, tok = _ops().conf_argmax(logits.to(dev), L, shift=True, last_logit=last.to(dev))
    for b in range(2):
        sh = ref_ops.shift_logits(logits[b * L:(b + 1) * L], last[b])
        c_ref, t_ref = ref_ops.sample_tokens(sh)
        assert torch.equal(tok[b * L:(b + 1) * L].cpu(), t_ref)
        assert (conf[b * L:(b + 1) * L].cpu() - c_ref).abs().max() <= 5e-5
    conf2, tok2 = _ops().conf_argmax(logits.to(dev), L, shift=True)
    sh = ref_ops.shift_logits(logits[:L], None)
    assert torch.equal(tok2[:L].cpu(), ref_ops.sample_tokens(sh)[1])


def test_denoise_unmask_single_call_equals_the_two_calls(dev):
    """pdllm_denoise_unmask = conf_argmax + threshold_unmask, bit for bit, with the Dream shift, a last
    context logit, partly decoded blocks and a block with nothing left to unmask."""
    ops = _ops()
    gen = torch.Generator().manual_seed(14)
    vocab, L, n_seqs, mask_id = 9000, 32, 3, 8999
    logits = (torch.randn(n_seqs * L, vocab, generator=gen) * 2).to(torch.bfloat16)
    rows = torch.randperm(n_seqs * L, generator=gen)[:40]
    logits[rows, torch.randint(0, vocab - 1, (40,), generator=gen)] = 20.0   # confident rows
    last = (torch.randn(n_seqs, vocab, generator=gen) * 2).to(torch.bfloat16)
    block = torch.full((n_seqs, L), mask_id, dtype=torch.int64)
    block[0, :7] = 5
    block[2] = 6                                                               # nothing masked
    for shift, ll in ((False, None), (True, None), (True, last)):
        a_ids, b_ids = block.clone().to(dev), block.clone().to(dev)
        lld = None if ll is None else ll.to(dev)
        conf, tok, tr, left = ops.denoise_unmask(logits.to(dev), a_ids, mask_id, 0.9, shift=shift, last_logit=lld)
        conf2, tok2 = ops.conf_argmax(logits.to(dev), L, shift=shift, last_logit=lld)
        tr2, left2 = ops.threshold_unmask(conf2.view(n_seqs, L), tok2.view(n_seqs, L), b_ids, mask_id, 0.9)
        assert torch.equal(conf, conf2) and torch.equal(tok, tok2)
        assert torch.equal(tr, tr2) and torch.equal(left, left2) and torch.equal(a_ids, b_ids)
        assert int(left[2]) == 0 and not bool(tr[2].any())
        assert int(tr[0, :7].sum()) == 0 and int(tr[0].sum()) >= 1
        # the prepared form of the same call, run over several denoise steps until nothing is masked
        c_ids = block.clone().to(dev)
        prep = ops.PreparedDenoiseUnmask(logits.to(dev), c_ids, mask_id, 0.9, shift=shift, last_logit=lld)
        tr3, left3 = prep.run()
        assert torch.equal(tr3, tr) and torch.equal(left3, left) and torch.equal(c_ids, a_ids)
        assert torch.equal(prep.conf, conf) and torch.equal(prep.token, tok)
        for _ in range(L):
            prep.run()
        assert int(prep.left.sum()) == 0 and not bool((c_ids == mask_id).any())


def test_argmax_first_index_on_ties(dev):
    logits = torch.zeros(3, 70000, dtype=torch.bfloat16)
    logits[0, 69999] = 5; logits[0, 123] = 5
    logits[1, 40000] = 2; logits[1, 40001] = 2
    conf, tok = _ops().conf_argmax(logits.to(dev), 1)
    assert tok.cpu().tolist() == [123, 40000, 0]
    assert torch.equal(tok.cpu(), ref_ops.sample_tokens(logits)[1])


def test_unmask_all_below_threshold_moves_exactly_one(dev):
    conf = torch.tensor([[0.2, 0.5, 0.5, 0.1]])
    tok = torch.tensor([[7, 8, 9, 10]])
    block = torch.full((1, 4), 99, dtype=torch.int64, device=dev)
    tr, left = _ops().threshold_unmask(conf.to(dev), tok.to(dev), block, 99, 0.9)
    assert block.cpu().tolist() == [[99, 8, 99, 99]] and int(left[0]) == 3
    nb, _ = ref_ops.threshold_unmask(torch.full((4,), 99), conf[0], tok[0], 99, 0.9)
    assert nb.tolist() == [99, 8, 99, 99]


def _toy_model(vocab, seed):
    """A deterministic stand-in for the model forward: logits row p depends on the token ids at positions <= p
    (so confirming a token changes the later rows, as a real forward does).  bf16 logits on the CPU."""
    gen = torch.Generator().manual_seed(seed)
    emb = torch.randn(vocab + 1, 48, generator=gen)
    out = torch.randn(48, vocab, generator=gen) * 0.6

    def logits_of(ids):
        ids = torch.as_tensor(ids, dtype=torch.int64).cpu()
        x = emb[ids.clamp(max=vocab)]
        ctx = torch.cumsum(x, 0) / torch.arange(1, len(ids) + 1).unsqueeze(1)
        return ((x + ctx) @ out).to(torch.bfloat16)

    return logits_of


@pytest.mark.parametrize("prompt_len,draft_len,rounds", [(7, 4, 0), (7, 4, 2), (5, 6, 5), (9, 3, 8), (0, 5, 3),
                                                         (33, 32, 12)])
def test_partial_draft_rounds_for_selection(dev, prompt_len, draft_len, rounds):
    """engine_ops.generate_partial_draft_rounds_for_selection against the restatement of
    fastdllm_engine.py:1013-1059: same tokens, same confirmed positions, round by round (each round is the device
    unmask step with a threshold no confidence reaches, position 0 first)."""
    from prefilling_dllm_amd import engine_ops as eo
    vocab, mask_id = 3000, 3000
    model = _toy_model(vocab, 100 + prompt_len)
    prompt = list(range(11, 11 + prompt_len))
    ref_ids, ref_conf = ref_ops.partial_draft_rounds(lambda ids: model(ids).float(), prompt, draft_len, rounds, mask_id)
    got_ids, got_conf = eo.generate_partial_draft_rounds_for_selection(
        lambda ids: model(ids).to(dev), prompt, max_new_tokens=draft_len, partial_rounds=rounds,
        mask_token_id=mask_id, device=dev)
    assert got_ids == ref_ids and got_conf == ref_conf
    assert sum(ref_conf) == min(draft_len, 1 + rounds)
    assert eo.generate_partial_draft_rounds_for_selection(None, prompt, max_new_tokens=0, partial_rounds=3,
                                                          mask_token_id=mask_id) == ([], [])


def test_partial_draft_round_confirms_one_position(dev):
    """One round on the device: exactly one masked position changes, the transfer mask names it, and a block
    without masks is left alone."""
    from prefilling_dllm_amd import engine_ops as eo
    vocab, mask_id, n, d = 500, 500, 6, 8
    model = _toy_model(vocab, 3)
    block = torch.full((d,), mask_id, dtype=torch.int64, device=dev)
    ids = torch.cat([torch.arange(n, device=dev), block])
    tr = eo.partial_draft_round(model(ids).to(dev), block, prompt_len=n, mask_token_id=mask_id, first=True)
    assert tr.cpu().tolist() == [True] + [False] * (d - 1) and int((block != mask_id).sum()) == 1
    before = block.clone()
    tr = eo.partial_draft_round(model(torch.cat([ids[:n], block])).to(dev), block, prompt_len=n, mask_token_id=mask_id)
    assert int(tr.sum()) == 1 and int((block != before).sum()) == 1 and bool((block[tr] != mask_id).all())
    full = torch.arange(d, dtype=torch.int64, device=dev)
    tr = eo.partial_draft_round(model(torch.cat([ids[:n], full])).to(dev), full, prompt_len=n, mask_token_id=mask_id)
    assert int(tr.sum()) == 0 and full.cpu().tolist() == list(range(d))
    with pytest.raises(ValueError):
        eo.partial_draft_round(model(ids).to(dev)[:-1], block, prompt_len=n, mask_token_id=mask_id)


def test_rope_matches_reference_formula(dev):
    gen = torch.Generator().manual_seed(14)
    cs = ref_ops.rope_cos_sin_cache(128, 40000, base=1000000.0)
    x = torch.randn(100, 4, 128, generator=gen).to(torch.bfloat16)
    pos = torch.randint(0, 40000, (100,), generator=gen)
    got = _ops().rope_inplace(x.clone().to(dev), pos.to(dev), cs.to(dev)).cpu()
    assert torch.equal(got, ref_ops.apply_rope(x, pos, cs))


def test_rope_qk_store_single_launch_equals_the_three_calls(dev):
    """pdllm_rope_qk_store = rope on q, rope on k, paged store of (rotated k, v): same bits as the three calls and
    as the oracle; continuous chunk positions as in BASELINE config 4; slots < 0 are not stored; strided q/k/v
    (views of a fused qkv projection)."""
    from prefilling_dllm_amd import engine_ops as eo
    ops = _ops()
    gen = torch.Generator().manual_seed(15)
    Hq, Hkv, d, P = 28, 4, 128, 256
    lens = [300, 257, 1]
    n = sum(lens)
    cs = ref_ops.rope_cos_sin_cache(d, 4096, base=1000000.0)
    qkv = torch.randn(n, (Hq + 2 * Hkv) * d, generator=gen).to(torch.bfloat16)
    pos = eo.chunk_positions("continuous", 5, lens, [4, 0, 2], 1025)
    assert pos[:3].tolist() == [5, 6, 7] and int(pos[300]) == 5 + 1025 and int(pos[-1]) == 5 + 2 * 1025
    pages = torch.randperm(4, generator=gen).to(torch.int32)
    slots = ops.slot_mapping_from_pages(pages.to(dev), n).clone()
    slots[10:20] = -1

    def views(t):
        q = t[:, :Hq * d].view(n, Hq, d)
        k = t[:, Hq * d:(Hq + Hkv) * d].view(n, Hkv, d)
        v = t[:, (Hq + Hkv) * d:].view(n, Hkv, d)
        return q, k, v

    a = qkv.clone().to(dev)
    qa, ka, va = views(a)
    kc = torch.zeros(4, P, Hkv, d, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    ops.rope_qk_store(qa, ka, va, pos.to(dev), cs.to(dev), kc, vc, slots)

    b = qkv.clone().to(dev)
    qb, kb, vb = views(b)
    qb2, kb2 = qb.contiguous(), kb.contiguous()
    ops.rope_inplace(qb2, pos.to(dev), cs.to(dev))
    ops.rope_inplace(kb2, pos.to(dev), cs.to(dev))
    kc2 = torch.zeros_like(kc)
    vc2 = torch.zeros_like(kc)
    ops.store_kvcache_unified_layout(kb2, vb.contiguous(), kc2, vc2, slots, model_type="diffusion_lm")
    assert torch.equal(qa, qb2) and torch.equal(ka, kb2) and torch.equal(va, vb)
    assert torch.equal(kc, kc2) and torch.equal(vc, vc2)
    q0, k0, _ = views(qkv)
    assert torch.equal(qa.cpu(), ref_ops.apply_rope(q0, pos, cs))
    assert torch.equal(ka.cpu(), ref_ops.apply_rope(k0, pos, cs))
    # rotation only
    c = qkv.clone().to(dev)
    qc, kc_, _ = views(c)
    ops.rope_qk_store(qc, kc_, None, pos.to(dev), cs.to(dev))
    assert torch.equal(qc, qa) and torch.equal(kc_, ka)


def test_vote_topk_keep_set(dev):
    """Votes of all (layer, KV head) keep lists, then per chunk the first token + the most voted positions,
    lowest index on ties: bit-exact with the oracle; chunks of different lengths, gaps between chunks, a
    capacity larger than a chunk and capacity 0 (keep everything)."""
    from prefilling_dllm_amd import engine_ops as eo
    gen = torch.Generator().manual_seed(21)
    n, L, H, keep = 3000, 5, 4, 600
    spans = [(4, 1029), (1029, 2054), (2060, 2061), (2100, 2900)]
    keep_idx = [torch.stack([torch.randperm(n + 50, generator=gen)[:keep].sort().values for _ in range(H)])
                for _ in range(L)]
    votes = _ops().vote_histogram(torch.cat([k.reshape(-1) for k in keep_idx]).to(dev), n).cpu()
    want_votes = torch.bincount(torch.cat([k.reshape(-1) for k in keep_idx]).clamp(max=n), minlength=n + 1)[:n]
    assert torch.equal(votes, want_votes.float())
    as_lists = [[h.tolist() for h in layer] for layer in keep_idx]
    for cap in (0, 1, 256, 900, 5000):
        got = eo.preevict_vote_topk_indices([k.to(dev) for k in keep_idx], n, spans, cap).cpu().tolist()
        assert got == ref_ops.preevict_vote_topk_indices(as_lists, n, spans, cap), cap
