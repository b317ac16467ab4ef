"""GPU parity of the paged KV data movement (store / load / gather / scatter / compaction)."""
import json
import os

import pytest
import torch

from oracle import ref_ops

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _ops():
    from prefilling_dllm_amd import ops
    return ops


def test_store_reference_procedure(dev):
    """examples/test_dllm_kv_cache_store.py:8-43 of the reference: 20 sequences, contexts 81..120,
    32 active rows each mapped to -1, cache (307, 256, 4, 128) bf16, seed 114514."""
    torch.manual_seed(114514)
    ctx = [119, 110, 81, 114, 112, 119, 110, 81, 114, 112, 119, 110, 81, 114, 112, 120, 111, 82, 115, 113]
    total = [c + 32 for c in ctx]
    k = torch.randn(sum(total), 4, 128).to(torch.bfloat16)
    v = torch.randn(sum(total), 4, 128).to(torch.bfloat16)
    slots = []
    for i, c in enumerate(ctx):
        slots.extend(range(i * 256, i * 256 + c))
        slots.extend([-1] * 32)
    slots = torch.tensor(slots, dtype=torch.int64)
    kc = torch.zeros(307, 256, 4, 128, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    _ops().store_kvcache_unified_layout(k.to(dev), v.to(dev), kc, vc, slots.to(dev), model_type="diffusion_lm")
    torch.cuda.synchronize()
    start = 0
    for i, (l, c) in enumerate(zip(total, ctx)):
        assert torch.equal(kc[i, :c].cpu(), k[start:start + c])
        assert torch.equal(vc[i, :c].cpu(), v[start:start + c])
        assert kc[i, c:].abs().max() == 0  # masked (-1) rows were not written
        start += l
    kc_ref = torch.zeros(307, 256, 4, 128, dtype=torch.bfloat16)
    vc_ref = torch.zeros_like(kc_ref)
    ref_ops.store_kvcache(k, v, kc_ref, vc_ref, slots)
    assert torch.equal(kc.cpu(), kc_ref) and torch.equal(vc.cpu(), vc_ref)


def test_store_then_load_reference_fixture(dev):
    """examples/test_dllm_kv_cache_load.py:28-65 with the reference's slot-mapping fixture
    (examples/mimic_data/mimic_slot_mapping.py, committed as run-length JSON)."""
    with open(os.path.join(GOLDEN, "mimic_slot_mapping.json")) as f:
        fx = json.load(f)
    slots = []
    for value, start, count in fx["runs"]:
        slots.extend([-1] * count if value == "skip" else range(start, start + count))
    assert len(slots) == fx["length"]
    torch.manual_seed(114514)
    seq = [64, 64, 32, 64, 64, 32, 64, 32, 64, 64, 32, 64, 64, 64, 64, 64, 32, 32, 64, 64]
    ctx = [119, 110, 81, 114, 112, 119, 110, 81, 114, 112, 119, 110, 81, 114, 112, 120, 111, 82, 115, 113]
    assert sum(seq) == len(slots)
    n_pages = 1342
    k_cache = torch.randn(n_pages, 256, 4, 128).to(torch.bfloat16)
    v_cache = torch.randn(n_pages, 256, 4, 128).to(torch.bfloat16)
    k_new = torch.randn(sum(seq), 4, 128).to(torch.bfloat16)
    v_new = torch.randn(sum(seq), 4, 128).to(torch.bfloat16)
    bt = torch.arange(20, dtype=torch.int32).view(20, 1)
    ops = _ops()
    kc, vc = k_cache.to(dev), v_cache.to(dev)
    slots_t = torch.tensor(slots, dtype=torch.int64)
    ops.store_kvcache_unified_layout(k_new.to(dev), v_new.to(dev), kc, vc, slots_t.to(dev), model_type="diffusion_lm")
    ref_ops.store_kvcache(k_new, v_new, k_cache, v_cache, slots_t)
    torch.cuda.synchronize()
    assert torch.equal(kc.cpu(), k_cache) and torch.equal(vc.cpu(), v_cache)

    class Seq:
        diffusion_block_size = 32

    class Ctx:
        pass

    c = Ctx()
    c.block_tables = bt.to(dev)
    c.context_lens = torch.tensor(ctx, dtype=torch.int32, device=dev)
    c.seq_lens_ts = torch.tensor(seq, dtype=torch.int32, device=dev)
    c.seq_lens = seq
    c.seqs = [Seq()]
    cu = lambda x: torch.tensor([0] + list(torch.tensor(x).cumsum(0)), dtype=torch.int32, device=dev)
    c.cu_seqlens_q = cu(seq)
    c.cu_seqlens_k = cu([a + b for a, b in zip(seq, ctx)])
    k_comb, v_comb = ops.load_kvcache(kc, vc, c, k_new.to(dev), v_new.to(dev))
    torch.cuda.synchronize()
    k_ref, v_ref = ref_ops.load_kvcache(k_cache, v_cache, bt, ctx, seq, k_new, v_new)
    assert torch.equal(k_comb.cpu(), k_ref) and torch.equal(v_comb.cpu(), v_ref)


def test_slot_mapping_matches_closed_form(dev):
    pages = [7, 3, 11, 0, 5]
    got = _ops().slot_mapping_from_pages(torch.tensor(pages, device=dev), 700, start_token=300).cpu()
    assert torch.equal(got, ref_ops.slot_mapping(pages, 700, 300))
    # tokens beyond the page list are not mapped
    got = _ops().slot_mapping_from_pages(torch.tensor(pages[:2], device=dev), 600).cpu()
    assert (got[512:] == -1).all() and torch.equal(got[:512], ref_ops.slot_mapping(pages, 512))


def test_gather_scatter_roundtrip_and_snapshot(dev):
    gen = torch.Generator().manual_seed(3)
    n_pages, Hkv, d = 12, 4, 128
    cache = torch.randn(n_pages, 256, Hkv, d, generator=gen).to(torch.bfloat16)
    page_ids = torch.randperm(n_pages, generator=gen)[:5]
    prompt_len = 1100
    ops = _ops()
    snap = ops.kv_gather(cache.to(dev), page_ids.to(dev), prompt_len).cpu()
    assert torch.equal(snap, ref_ops.gather_tokens(cache, page_ids, torch.arange(prompt_len)))
    # load into fresh pages of another cache and read back
    cache2 = torch.zeros_like(cache).to(dev)
    page_ids2 = torch.randperm(n_pages, generator=gen)[:5]
    ops.kv_scatter(cache2, page_ids2.to(dev), snap.to(dev))
    back = ops.kv_gather(cache2, page_ids2.to(dev), prompt_len).cpu()
    assert torch.equal(back, snap)
    ref2 = torch.zeros_like(cache)
    ref_ops.scatter_tokens(ref2, page_ids2, snap)
    assert torch.equal(cache2.cpu(), ref2)


def test_pd_handoff_snapshot_and_page_copy(dev):
    """The prefill/decode hand-off both ways the reference has it (fastdllm_engine.py:700-881): through a host
    snapshot loaded into freshly allocated pages, and cache to cache page by page.  Either way the decode side
    reads back exactly the prompt KV of the prefill side; pages it did not receive stay untouched."""
    from prefilling_dllm_amd import engine_ops as eo
    ops = _ops()
    gen = torch.Generator().manual_seed(8)
    L, n_pages, P, Hkv, d = 3, 10, 256, 4, 128
    src = torch.randn(2, L, n_pages, P, Hkv, d, generator=gen).to(torch.bfloat16).to(dev)
    prompt_len, decode_len = 700, 96
    src_pages = [7, 2, 5]
    rec = eo.DreamPrefillRecord(prompt_ids=list(range(prompt_len)), prompt_positions=list(range(prompt_len)),
                                suffix_positions=list(range(prompt_len, prompt_len + decode_len)),
                                prompt_len=prompt_len, full_prompt_len=prompt_len, decode_len=decode_len,
                                prompt_page_ids=src_pages, block_page_ids=[9], first_token_id=1,
                                last_context_logit=torch.arange(8, dtype=torch.float32, device=dev),
                                decode_delta_state=None, owns_prompt_pages=True)
    want_k, want_v = eo.snapshot_prompt_cache_per_layer(src, src_pages, prompt_len)
    for l in range(L):
        idx = torch.arange(prompt_len)
        assert torch.equal(want_k[l].cpu(), ref_ops.gather_tokens(src[0, l].cpu(), torch.tensor(src_pages), idx))

    # (1) host snapshot -> another engine's cache
    snap = eo.snapshot_pd_record_kv(src, rec, device="cpu")
    assert snap.k_by_layer[0].device.type == "cpu" and tuple(snap.k_by_layer[0].shape) == (prompt_len, Hkv, d)
    dst = torch.zeros_like(src)
    alloc = eo.PagePool(n_pages, P)
    alloc.allocate_pages(2)                                     # pages 0, 1 are taken by someone else
    rec2 = eo.make_pd_record_from_kv_snapshot(dst, alloc, rec, snap)
    assert rec2.prompt_page_ids == [2, 3, 4] and rec2.block_page_ids == [5] and rec2.owns_prompt_pages
    got_k, got_v = eo.snapshot_prompt_cache_per_layer(dst, rec2.prompt_page_ids, prompt_len)
    for l in range(L):
        assert torch.equal(got_k[l], want_k[l]) and torch.equal(got_v[l], want_v[l])
    assert int(dst[:, :, [0, 1, 5, 6, 7, 8, 9]].abs().sum()) == 0
    assert torch.equal(rec2.last_context_logit, rec.last_context_logit)
    with pytest.raises(ValueError, match="page_size mismatch"):
        eo.make_pd_record_from_kv_snapshot(dst, alloc, rec, snap, page_size=128)
    snap.prompt_len += 1
    with pytest.raises(ValueError, match="prompt_len mismatch"):
        eo.make_pd_record_from_kv_snapshot(dst, alloc, rec, snap)
    eo.release_pd_record(alloc, rec2)
    assert alloc.num_free_pages == n_pages - 2

    # (2) cache to cache, whole pages, all layers in one launch
    dst2 = torch.zeros_like(src)
    alloc2 = eo.PagePool(n_pages, P)
    alloc2.allocate_pages(4)
    rec3 = eo.make_pd_record_from_remote_cache(src, dst2, alloc2, rec)
    assert rec3.prompt_page_ids == [4, 5, 6]
    for a, b in zip(src_pages, rec3.prompt_page_ids):
        assert torch.equal(dst2[:, :, b], src[:, :, a])
    assert int(dst2[:, :, [0, 1, 2, 3, 7, 8, 9]].abs().sum()) == 0
    got_k, got_v = eo.snapshot_prompt_cache_per_layer(dst2, rec3.prompt_page_ids, prompt_len)
    for l in range(L):
        assert torch.equal(got_k[l], want_k[l]) and torch.equal(got_v[l], want_v[l])
    # page ids outside either cache are skipped, not written
    ops.kv_copy_pages(src, dst2, torch.tensor([1, 99], dtype=torch.int32, device=dev),
                      torch.tensor([-1, 0], dtype=torch.int32, device=dev))
    torch.cuda.synchronize()
    assert int(dst2[:, :, 0].abs().sum()) == 0


def test_per_head_compaction_matches_reference_order(dev):
    """fastdllm_engine.py:607-638: gather with per-head keep lists, rewrite into the first slots."""
    gen = torch.Generator().manual_seed(5)
    n_pages, Hkv, d = 10, 4, 128
    cache = torch.randn(n_pages, 256, Hkv, d, generator=gen).to(torch.bfloat16)
    page_ids = torch.randperm(n_pages, generator=gen)[:6]
    full_len, keep_n = 1400, 520
    keep = torch.stack([torch.sort(torch.randperm(full_len, generator=gen)[:keep_n]).values for _ in range(Hkv)])
    ops = _ops()
    dc = cache.to(dev)
    from prefilling_dllm_amd import engine_ops
    engine_ops.compact_prompt_cache_per_head(dc, page_ids.to(dev), keep.to(dev))
    torch.cuda.synchronize()
    ref = cache.clone()
    ref_ops.compact_per_head(ref, page_ids, keep)
    assert torch.equal(dc.cpu(), ref)


@pytest.mark.parametrize("sorted_keep,ws_layers", [(True, 3), (False, 1), (True, 99)])
def test_per_head_compaction_all_layers_in_one_call(dev, sorted_keep, ws_layers):
    """compact_prompt_cache_per_layer_per_head on a whole cache: K and V of every layer, each KV head with its own
    keep list, in rounds of as many layers as the workspace holds; unsorted keep lists too (the gather of a round
    is complete before its first row is overwritten, as in the reference, which clones)."""
    from prefilling_dllm_amd import engine_ops
    ops = _ops()
    gen = torch.Generator().manual_seed(31 + ws_layers)
    L, n_pages, Hkv, d = 5, 9, 4, 128
    kv = torch.randn(2, L, n_pages, 256, Hkv, d, generator=gen).to(torch.bfloat16)
    page_ids = torch.randperm(n_pages, generator=gen)[:6]
    full_len, keep_n = 1400, 520
    def one():
        idx = torch.randperm(full_len, generator=gen)[:keep_n]
        return torch.sort(idx).values if sorted_keep else idx
    keeps = [torch.stack([one() for _ in range(Hkv)]) for _ in range(L)]
    ref = kv.clone()
    for l in range(L):
        for which in range(2):
            ref_ops.compact_per_head(ref[which, l], page_ids, keeps[l])
    dkv = kv.to(dev)
    per_layer = 2 * keep_n * Hkv * d * 2
    ops.kv_compact_per_head(dkv, page_ids.to(dev), torch.stack(keeps).to(dev), max_workspace_bytes=per_layer * ws_layers)
    torch.cuda.synchronize()
    assert torch.equal(dkv.cpu(), ref)
    dkv2 = kv.to(dev)
    assert engine_ops.compact_prompt_cache_per_layer_per_head(dkv2, page_ids.tolist(), [k.to(dev) for k in keeps]) == keep_n
    assert torch.equal(dkv2.cpu(), ref)


def test_chunk_local_kv_copy_matches_reference_order(dev):
    """fastdllm_engine.py:525-558: the kept tokens of a chunk that was prefilled into temporary pages go, per layer
    and KV head, behind dst_start of the request's pages.  Source chunk and destination both start inside a page,
    the page lists overlap, every head has its own keep list, K and V of two layers."""
    from prefilling_dllm_amd import engine_ops
    gen = torch.Generator().manual_seed(12)
    L, n_pages, P, Hkv, d = 2, 9, 256, 4, 128
    kv = torch.randn(2, L, n_pages, P, Hkv, d, generator=gen).to(torch.bfloat16)
    src_pages, dst_pages = [7, 3, 8], [3, 1, 4, 0]
    src_chunk_start, dst_start, chunk_len, keep_n = 77, 190, 640, 410
    keeps = [torch.stack([torch.sort(torch.randperm(chunk_len, generator=gen)[:keep_n]).values for _ in range(Hkv)])
             for _ in range(L)]
    dkv = kv.to(dev)
    n = engine_ops.copy_chunk_local_kv_to_prompt_pages(dkv, src_page_ids=src_pages, dst_page_ids=dst_pages,
                                                       src_chunk_start=src_chunk_start, dst_start=dst_start,
                                                       keep_indices_per_layer_per_head=[k.to(dev) for k in keeps])
    torch.cuda.synchronize()
    assert n == keep_n
    ref = kv.clone()
    for l in range(L):
        for which in range(2):
            ref_ops.copy_chunk_local_kv(ref[which, l], src_pages, dst_pages, src_chunk_start, dst_start, keeps[l])
    assert torch.equal(dkv.cpu(), ref)
    # degenerate inputs of the reference: no layers, an empty keep list, a layer of another length
    assert engine_ops.copy_chunk_local_kv_to_prompt_pages(dkv, src_page_ids=src_pages, dst_page_ids=dst_pages,
                                                          src_chunk_start=0, dst_start=0,
                                                          keep_indices_per_layer_per_head=[]) == 0
    empty = torch.empty(Hkv, 0, dtype=torch.long, device=dev)
    assert engine_ops.copy_chunk_local_kv_to_prompt_pages(dkv, src_page_ids=src_pages, dst_page_ids=dst_pages,
                                                          src_chunk_start=0, dst_start=0,
                                                          keep_indices_per_layer_per_head=[empty, empty]) == 0
    with pytest.raises(ValueError, match="keep_count mismatch"):
        engine_ops.copy_chunk_local_kv_to_prompt_pages(dkv, src_page_ids=src_pages, dst_page_ids=dst_pages,
                                                       src_chunk_start=0, dst_start=0,
                                                       keep_indices_per_layer_per_head=[keeps[0].to(dev),
                                                                                        keeps[1][:, :5].to(dev)])


def test_fp8_store_matches_torch_cast(dev):
    gen = torch.Generator().manual_seed(8)
    n, Hkv, d, n_pages = 600, 4, 128, 4
    k = torch.randn(n, Hkv, d, generator=gen).to(torch.bfloat16)
    v = torch.randn(n, Hkv, d, generator=gen).to(torch.bfloat16)
    page_ids = [2, 0, 3]
    slots = ref_ops.slot_mapping(page_ids, n)
    ks = torch.tensor([0.01, 0.02, 0.013, 0.017])
    vs = torch.tensor([0.011, 0.009, 0.02, 0.015])
    kc = torch.zeros(n_pages, 256, Hkv, d, dtype=torch.float8_e4m3fn, device=dev)
    vc = torch.zeros_like(kc)
    _ops().store_kvcache_unified_layout(k.to(dev), v.to(dev), kc, vc, slots.to(dev), k_scale=ks.to(dev),
                                        v_scale=vs.to(dev))
    torch.cuda.synchronize()
    page_of = (slots // 256).long()
    kq = (k.float() / ks[page_of].view(-1, 1, 1)).clamp(-448, 448).to(torch.float8_e4m3fn)
    vq = (v.float() / vs[page_of].view(-1, 1, 1)).clamp(-448, 448).to(torch.float8_e4m3fn)
    got_k = kc.view(-1, Hkv, d)[slots.long().to(dev)].cpu().view(torch.uint8)
    got_v = vc.view(-1, Hkv, d)[slots.long().to(dev)].cpu().view(torch.uint8)
    assert torch.equal(got_k, kq.view(torch.uint8)) and torch.equal(got_v, vq.view(torch.uint8))


@pytest.mark.parametrize("layout", ["scalar", "per_page", "per_head"])
def test_fp8_store_then_attention_with_each_scale_layout(dev, layout):
    """The quantising store and the dequantising attention address the scales the same way: one scalar (what the
    reference passes, prefix_prefill.py:118-121), one scale per page, one per page and KV head.  Rows are stored
    through the C ABI, then attended to; the oracle sees float(e4m3(x / scale)) * scale."""
    ops = _ops()
    gen = torch.Generator().manual_seed(15)
    n, Hq, Hkv, d, n_pages = 700, 8, 4, 128, 5
    k = (torch.randn(n, Hkv, d, generator=gen) * torch.tensor([0.5, 1.0, 2.0, 4.0]).view(1, Hkv, 1)).to(torch.bfloat16)
    v = (torch.randn(n, Hkv, d, generator=gen) * torch.tensor([3.0, 0.3, 1.0, 2.0]).view(1, Hkv, 1)).to(torch.bfloat16)
    page_ids = [3, 0, 4]
    slots = ref_ops.slot_mapping(page_ids, n)
    if layout == "scalar":
        ks, vs = torch.tensor(0.05), torch.tensor(0.04)
        ks_full, vs_full = ks.expand(n_pages, Hkv), vs.expand(n_pages, Hkv)
    elif layout == "per_page":
        ks, vs = torch.linspace(0.03, 0.06, n_pages), torch.linspace(0.05, 0.02, n_pages)
        ks_full, vs_full = ks.view(-1, 1).expand(n_pages, Hkv), vs.view(-1, 1).expand(n_pages, Hkv)
    else:
        ks = torch.linspace(0.01, 0.04, n_pages).view(-1, 1) * torch.tensor([0.5, 1.0, 2.0, 4.0]).view(1, -1)
        vs = torch.linspace(0.02, 0.03, n_pages).view(-1, 1) * torch.tensor([3.0, 0.3, 1.0, 2.0]).view(1, -1)
        ks, vs = ks.contiguous(), vs.contiguous()
        ks_full, vs_full = ks, vs
    kc = torch.zeros(n_pages, 256, Hkv, d, dtype=torch.float8_e4m3fn, device=dev)
    vc = torch.zeros_like(kc)
    ops.store_kvcache_unified_layout(k.to(dev), v.to(dev), kc, vc, slots.to(dev), k_scale=ks.to(dev), v_scale=vs.to(dev))
    torch.cuda.synchronize()
    page_of = (slots // 256).long()
    kq = (k.float() / ks_full[page_of].unsqueeze(-1)).clamp(-448, 448).to(torch.float8_e4m3fn)
    vq = (v.float() / vs_full[page_of].unsqueeze(-1)).clamp(-448, 448).to(torch.float8_e4m3fn)
    got_k = kc.view(-1, Hkv, d)[slots.long().to(dev)].cpu()
    got_v = vc.view(-1, Hkv, d)[slots.long().to(dev)].cpu()
    assert torch.equal(got_k.view(torch.uint8), kq.view(torch.uint8))
    assert torch.equal(got_v.view(torch.uint8), vq.view(torch.uint8))
    # attention over the stored rows
    q = (torch.randn(32, Hq, d, generator=gen) / 8).to(torch.bfloat16)
    kn = (torch.randn(32, Hkv, d, generator=gen) / 8).to(torch.bfloat16)
    vn = torch.randn(32, Hkv, d, generator=gen).to(torch.bfloat16)
    bt = torch.tensor([page_ids], dtype=torch.int32)
    qsl = torch.tensor([0, 32], dtype=torch.int32)
    out = ops.sparse_decode_attention(q.to(dev), kn.to(dev), vn.to(dev), kc, vc, bt.to(dev), qsl.to(dev),
                                      max_q_len=32, max_ctx_len=n, context_lens=torch.tensor([n], dtype=torch.int32,
                                                                                             device=dev),
                                      k_scale=ks.to(dev), v_scale=vs.to(dev)).float().cpu()
    k_ref = torch.zeros(n_pages, 256, Hkv, d, dtype=torch.bfloat16)
    v_ref = torch.zeros_like(k_ref)
    k_ref.view(-1, Hkv, d)[slots.long()] = (kq.float() * ks_full[page_of].unsqueeze(-1)).to(torch.bfloat16)
    v_ref.view(-1, Hkv, d)[slots.long()] = (vq.float() * vs_full[page_of].unsqueeze(-1)).to(torch.bfloat16)
    ref = ref_ops.sparse_decode_attention(q, kn, vn, k_ref, v_ref, bt, qsl, [[(0, n)]])
    from oracle.tolerances import assert_attn_close
    assert_attn_close(out, ref, layout, abs_tol=3e-2)
    # a scale tensor of another layout, dtype or device is refused instead of being read out of bounds
    with pytest.raises(ValueError):
        ops.store_kvcache_unified_layout(k.to(dev), v.to(dev), kc, vc, slots.to(dev),
                                         k_scale=torch.ones(2, device=dev), v_scale=torch.ones(2, device=dev))
    with pytest.raises(ValueError):
        ops.store_kvcache_unified_layout(k.to(dev), v.to(dev), kc, vc, slots.to(dev),
                                         k_scale=torch.ones(n_pages), v_scale=torch.ones(n_pages))
    with pytest.raises(ValueError):
        ops.store_kvcache_unified_layout(k.to(dev), v.to(dev), kc, vc, slots.to(dev),
                                         k_scale=torch.ones(n_pages, dtype=torch.float64, device=dev),
                                         v_scale=torch.ones(n_pages, dtype=torch.float64, device=dev))
