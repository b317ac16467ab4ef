"""The hot path at the full sizes of the BASELINE configurations (one layer each): direct comparison with
the CPU oracle where that takes seconds, and size-independent properties (V = 1 gives O = 1, the output
does not depend on how the key range is cut over workgroups, store followed by gather is the identity,
block-diagonal prefill equals per-chunk attention) for the rest."""
import pytest
import torch

import bench
from oracle import ref_ops
from oracle.tolerances import assert_attn_close

pytestmark = pytest.mark.gpu


def _ops():
    from prefilling_dllm_amd import ops
    return ops


def test_config3_full_layer_against_oracle_and_split_invariance(dev):
    """configs[2]: 8 requests x 160 rows over 8 x 512 selected tokens in shuffled pages, GQA 28/4."""
    ops = _ops()
    w = bench.build_workload(torch, dev, layers=1, seed=5)
    args = (w["q"][0], w["kn"][0], w["vn"][0], w["kv"][0, 0], w["kv"][1, 0], w["block_table"], w["qsl"])
    kw = dict(max_q_len=w["q_len"], max_ctx_len=w["ctx"], ranges=w["ranges"])
    out = ops.sparse_decode_attention(*args, **kw).float().cpu()
    ref = ref_ops.sparse_decode_attention(*(t.cpu() for t in args[:5]), w["block_table"].cpu(), w["qsl"].cpu(),
                                          w["ranges_host"])
    assert_attn_close(out, ref, "C3 layer, default plan")
    # the same rows through other cuts of the work: whole columns, equal splits, unaligned tile spans
    for plan in (dict(rows_per_group=128, num_splits=1), dict(rows_per_group=128, num_splits=3),
                 dict(rows_per_group=64, tiles_per_workgroup=11), dict(rows_per_group=160, num_splits=2)):
        other = ops.sparse_decode_attention(*args, **kw, **plan).float().cpu()
        assert_attn_close(other, ref, f"C3 layer, plan {plan}")
    # rows of a softmax sum to one: V = 1 everywhere gives O = 1 exactly up to bf16 rounding of the normaliser
    ones_cache = torch.ones_like(w["kv"][1, 0])
    ones_new = torch.ones_like(w["vn"][0])
    o1 = ops.sparse_decode_attention(w["q"][0], w["kn"][0], ones_new, w["kv"][0, 0], ones_cache, w["block_table"],
                                     w["qsl"], **kw).float().cpu()
    assert (o1 - 1.0).abs().max().item() <= 2 ** -7


def test_config4_full_prefill_layer(dev):
    """configs[3]: 32 chunks x 1025 rows, causal inside a chunk, K/V stored into shuffled pages."""
    ops = _ops()
    L, NC, Hq, Hkv, d, P = 1025, 32, 28, 4, 128, 256
    n = L * NC
    g = torch.Generator().manual_seed(11)
    q = torch.randn((n, Hq, d), generator=g).to(torch.bfloat16)     # configs[3]: Q, K, V ~ N(0, 1)
    k = torch.randn((n, Hkv, d), generator=g).to(torch.bfloat16)
    v = torch.randn((n, Hkv, d), generator=g).to(torch.bfloat16)
    pages = (n + P - 1) // P
    page_ids = torch.randperm(pages, generator=g).to(torch.int32)
    kc = torch.zeros((pages, P, Hkv, d), dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    slots = ops.slot_mapping_from_pages(page_ids.to(dev), n)
    cu = torch.arange(0, n + 1, L, dtype=torch.int32)
    out = ops.chunk_prefill_attention(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), max_seqlen=L, causal=True,
                                      k_cache=kc, v_cache=vc, slot_mapping=slots).float().cpu()
    assert torch.isfinite(out).all()
    # block-diagonal == independent per-chunk causal attention (the oracle on every chunk)
    for c in range(NC):
        sl = slice(c * L, (c + 1) * L)
        ref = ref_ops.chunk_prefill_attention(q[sl], k[sl], v[sl], torch.tensor([0, L]), causal=True)
        assert_attn_close(out[sl], ref, f"C4 chunk {c}")
    # the paged store is a bit-exact copy: gather(store(x)) == x
    back_k = ops.kv_gather(kc, page_ids.to(dev), n).cpu()
    back_v = ops.kv_gather(vc, page_ids.to(dev), n).cpu()
    assert torch.equal(back_k, k) and torch.equal(back_v, v)


def test_config2_full_scoring_and_eviction(dev):
    """configs[1]: 32 chunks x 4 labels over a 152064-entry vocabulary, top-4; eviction keep 256 of 1025."""
    from oracle import configs
    ops = _ops()
    logits, labels = configs.draft_logits(seed=21)
    sc = ops.chunk_scores_from_logits(logits.to(dev), labels.to(dev), mean=False).cpu()
    ref = ref_ops.chunk_scores(logits, labels, mean=False)
    assert (sc - ref).abs().max().item() <= 1e-4
    sel = ops.topk_lowest_index(sc.to(dev), 4).cpu().tolist()
    assert sel == ref_ops.topk_lowest_index(ref.tolist(), 4) or sel == ref_ops.topk_lowest_index(sc.tolist(), 4)
    probs = configs.eviction_probs(seed=22, n_chunks=8)
    s = ops.evict_colsum(probs.to(dev))
    assert torch.equal(s.cpu(), ref_ops.evict_colsum(probs))
    keep = ops.topb_keep_bos(s[:, 0], 256).cpu()
    for c in range(8):
        assert keep[c].tolist() == ref_ops.select_positions_from_token_scores(s[c, 0].cpu(), capacity=256,
                                                                                chunk_len=1025).tolist()


def test_config5_full_fp8_decode_layer_and_unmask(dev):
    """configs[4]: MHA 32/32, 4 requests x 16 of 64 chunks x 1025 tokens in fp8 e4m3 pages with a per-page
    scale, 160 active rows; then the threshold-0.9 unmask over [4, 32, 126464] logits."""
    from oracle import configs
    ops = _ops()
    case = configs.chunked_prefix_case(31, n_req=4, n_chunks=64, chunk_tokens=1025, topk=16, q_len=160, Hq=32,
                                       Hkv=32, fp8=True, shared_prefix=True)
    d = lambda t: None if t is None else t.to(dev)
    rp, rs, rl, mr = case.range_tensors()
    prep = ops.PreparedAttention(d(case.q), d(case.k_new), d(case.v_new), d(case.k_cache), d(case.v_cache),
                                 d(case.block_table), d(case.q_start_loc), max_q_len=case.max_q,
                                 max_ctx_len=case.max_ctx, ranges=(d(rp), d(rs), d(rl), mr),
                                 k_scale=d(case.k_scale), v_scale=d(case.v_scale))
    # 160 rows per (request, head) are five row blocks: one workgroup column each (four blocks would open a second,
    # mostly empty group that reads the pages again)
    assert "kv=fp8 row_blocks=5 " in prep.describe_plan(), prep.describe_plan()
    out = prep.run().float().cpu()
    assert torch.isfinite(out).all()
    # the oracle on every request (dequantised pages)
    for r in range(4):
        a, b = int(case.q_start_loc[r]), int(case.q_start_loc[r + 1])
        ref = ref_ops.sparse_decode_attention(case.q[a:b], case.k_new[a:b], case.v_new[a:b], case.k_cache_ref,
                                              case.v_cache_ref, case.block_table[r:r + 1], torch.tensor([0, b - a]),
                                              [case.ranges[r]])
        assert_attn_close(out[a:b], ref, f"C5 request {r}")
    logits = configs.unmask_logits(seed=32)
    if logits.dim() == 3:
        logits = logits.reshape(-1, logits.shape[-1])
    vocab, block_len = logits.shape[-1], 32
    n_seqs = logits.shape[0] // block_len
    mask_id = 126336
    conf, tok = ops.conf_argmax(logits.to(dev), block_len)
    rc, rt = ref_ops.sample_tokens(logits)
    assert torch.equal(tok.cpu(), rt)
    assert ((rc - 0.9).abs() > 1e-3).all()  # no row sits on the threshold
    block = torch.full((n_seqs, block_len), mask_id, dtype=torch.int64)
    ids = block.to(dev)
    transfer, left = ops.threshold_unmask(conf, tok, ids, mask_id, 0.9)
    for b in range(n_seqs):
        nb, tr = ref_ops.threshold_unmask(block[b], rc.view(n_seqs, block_len)[b], rt.view(n_seqs, block_len)[b],
                                          mask_id, 0.9)
        assert torch.equal(ids[b].cpu(), nb) and torch.equal(transfer[b].cpu(), tr)
        assert int(left[b]) == int((nb == mask_id).sum())
