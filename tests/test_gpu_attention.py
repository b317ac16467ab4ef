"""GPU parity of the sparse-prefix attention kernels against the CPU oracle (through the C ABI)."""
import math

import pytest
import torch

from oracle import configs, ref_ops
from oracle.tolerances import assert_attn_close

pytestmark = pytest.mark.gpu

TOL_BF16 = 2e-2   # max-abs tolerance of bf16 attention outputs (north star)


def _ops():
    from prefilling_dllm_amd import ops
    return ops


def run_case(case, dev, *, mask_mode="full", mask=None, rows_per_group=0, num_splits=0, use_ctx_lens=False,
             sm_scale=None, tiles_per_workgroup=0):
    ops = _ops()
    d = lambda t: None if t is None else t.to(dev)
    rp, rs, rl, mr = case.range_tensors()
    kwargs = dict(max_q_len=case.max_q, max_ctx_len=case.max_ctx, mask_mode=mask_mode, mask=d(mask),
                  sm_scale=sm_scale, k_scale=d(case.k_scale), v_scale=d(case.v_scale),
                  rows_per_group=rows_per_group, num_splits=num_splits, tiles_per_workgroup=tiles_per_workgroup)
    if use_ctx_lens:
        kwargs["context_lens"] = d(torch.tensor([sum(l for _, l in rr) for rr in case.ranges], dtype=torch.int32))
    else:
        kwargs["ranges"] = (d(rp), d(rs), d(rl), mr)
    out = ops.sparse_decode_attention(d(case.q), d(case.k_new), d(case.v_new), d(case.k_cache), d(case.v_cache),
                                      d(case.block_table), d(case.q_start_loc), **kwargs)
    torch.cuda.synchronize()
    return out.float().cpu()


def oracle_case(case, *, mask_mode="full", mask=None, sm_scale=None):
    kc = case.k_cache_ref if case.k_cache_ref is not None else case.k_cache
    vc = case.v_cache_ref if case.v_cache_ref is not None else case.v_cache
    return ref_ops.sparse_decode_attention(case.q, case.k_new, case.v_new, kc, vc, case.block_table,
                                           case.q_start_loc, case.ranges, mask_mode=mask_mode, mask=mask,
                                           sm_scale=sm_scale)


def check(out, ref, tol=TOL_BF16, what=""):
    """max|out - ref| <= max(2e-2 max|ref|, 2 bf16 ulp) and <= tol, and a norm-wise relative bound."""
    assert_attn_close(out, ref, what, abs_tol=tol)
    rel = (out - ref).norm() / ref.norm().clamp_min(1e-12)
    assert rel <= 1e-2, f"{what}: relative error {rel}"


def test_config1_parity(dev):
    """BASELINE config 1: 8 x 1025-token chunks in shuffled pages, top-K 4, 96 active rows."""
    case = configs.config1(seed=1)
    check(run_case(case, dev), oracle_case(case))


@pytest.mark.parametrize("rows", [32, 64, 128, 160, 192, 256])
@pytest.mark.parametrize("splits", [1, 2, 3])
def test_row_group_and_split_variants(dev, rows, splits):
    """Every row-group shape (own / shared row blocks, LDS merge) and the workspace split path on
    a ragged case: chunks of 300 tokens (not page aligned, partial last tile), 40 active rows."""
    case = configs.chunked_prefix_case(7, n_req=2, n_chunks=5, chunk_tokens=300, topk=2, q_len=40,
                                       shared_prefix=False)
    ref = oracle_case(case)
    check(run_case(case, dev, rows_per_group=rows, num_splits=splits), ref)


@pytest.mark.parametrize("rows", [32, 64, 128, 160])
@pytest.mark.parametrize("tiles", [1, 2, 3, 5, 7, 100])
def test_tile_spans_across_columns(dev, rows, tiles):
    """Workgroups that take a fixed number of tiles of the line of all columns' tiles: pieces of a
    column end up in different workgroups, one workgroup finishes a column and starts the next, and
    columns of unequal length (ragged requests) leave empty pieces."""
    case = configs.chunked_prefix_case(13, n_req=3, n_chunks=5, chunk_tokens=300, topk=2, q_len=40,
                                       shared_prefix=False)
    check(run_case(case, dev, rows_per_group=rows, tiles_per_workgroup=tiles), oracle_case(case))


def test_tile_spans_causal_dense(dev):
    case = configs.chunked_prefix_case(17, n_req=2, n_chunks=4, chunk_tokens=200, topk=2, q_len=70,
                                       shared_prefix=False)
    check(run_case(case, dev, mask_mode="causal", tiles_per_workgroup=3), oracle_case(case, mask_mode="causal"))


def test_shared_slot_table_matches_per_call_table(dev):
    """A slot table built once (pdllm_attn_build_slot_table) and handed to the prepared descriptor gives
    the same output as the table the call builds for itself."""
    ops = _ops()
    case = configs.chunked_prefix_case(19, n_req=3, n_chunks=6, chunk_tokens=260, topk=3, q_len=48,
                                       shared_prefix=False)
    d = lambda t: None if t is None else t.to(dev)
    rp, rs, rl, mr = case.range_tensors()
    args = (d(case.q), d(case.k_new), d(case.v_new), d(case.k_cache), d(case.v_cache), d(case.block_table),
            d(case.q_start_loc))
    kw = dict(max_q_len=case.max_q, max_ctx_len=case.max_ctx, ranges=(d(rp), d(rs), d(rl), mr))
    base = ops.sparse_decode_attention(*args, **kw).clone()
    table = ops.new_slot_table(case.q_start_loc.numel() - 1, case.max_ctx, dev)
    prep = ops.PreparedAttention(*args, slot_table=table, **kw)
    prep.build_slot_table()
    out = prep.run()
    torch.cuda.synchronize()
    assert torch.equal(out, base)
    # the table itself: slot of every visible key, then the count
    t = table.cpu()
    for r, rr in enumerate(case.ranges):
        toks = [s + i for s, l in rr for i in range(l)]
        assert int(t[r, -1]) == len(toks)
        bt = case.block_table[r]
        want = [int(bt[tk // 256]) * 256 + tk % 256 for tk in toks]
        assert t[r, :len(toks)].tolist() == want


@pytest.mark.parametrize("fp8", [False, True])
def test_page_table_entries_that_name_no_page_are_left_out(dev, fp8):
    """The reference skips page-table entries of -1 (kv_cache_kernels.py:208).  Entries outside [0, n_pages) inside
    the visible ranges -- a whole chunk's pages, the page in the middle of a range, the page a range ends in --
    contribute no keys: the output equals the oracle's over the remaining keys, the slot table lists only those,
    and a request whose visible pages are all gone attends to its active block alone."""
    ops = _ops()
    case = configs.chunked_prefix_case(23, n_req=4, n_chunks=6, chunk_tokens=300, topk=3, q_len=48,
                                       shared_prefix=False, fp8=fp8)
    n_pages = case.k_cache.shape[0]
    bt = case.block_table.clone()
    r0, r1, r3 = case.ranges[0], case.ranges[1], case.ranges[3]
    bt[0, r0[0][0] // 256] = -1                                   # the page the first range starts in
    bt[0, (r0[1][0] + 150) // 256] = n_pages + 5                  # a page in the middle of the second range
    bt[1, (r1[2][0] + r1[2][1] - 1) // 256] = -1                  # the page the last range ends in
    for start, length in r3:                                      # request 3: every visible page
        bt[3, start // 256:(start + length - 1) // 256 + 1] = -1
    case.block_table = bt
    ref = oracle_case(case)
    for kw in (dict(), dict(num_splits=3), dict(rows_per_group=256) if not fp8 else dict(rows_per_group=64)):
        check(run_case(case, dev, **kw), ref, what=f"{kw}")
    # request 3 sees its active block only
    d = lambda t: None if t is None else t.to(dev)
    a, b = int(case.q_start_loc[3]), int(case.q_start_loc[4])
    alone = ref_ops.sparse_decode_attention(case.q[a:b], case.k_new[a:b], case.v_new[a:b], None, None, None,
                                            [0, b - a], None)
    assert_attn_close(run_case(case, dev)[a:b], alone, "request without a page")
    # the table: the slots of the keys that remain, in order, then their number
    rp, rs, rl, mr = case.range_tensors()
    table = ops.new_slot_table(4, case.max_ctx, dev)
    prep = ops.PreparedAttention(d(case.q), d(case.k_new), d(case.v_new), d(case.k_cache), d(case.v_cache), d(bt),
                                 d(case.q_start_loc), max_q_len=case.max_q, max_ctx_len=case.max_ctx,
                                 ranges=(d(rp), d(rs), d(rl), mr), slot_table=table, k_scale=d(case.k_scale),
                                 v_scale=d(case.v_scale))
    prep.build_slot_table()
    torch.cuda.synchronize()
    t = table.cpu()
    for r, rr in enumerate(case.ranges):
        toks = [s + i for s, l in rr for i in range(l)]
        want = [int(bt[r, tk // 256]) * 256 + tk % 256 for tk in toks if 0 <= int(bt[r, tk // 256]) < n_pages]
        assert int(t[r, -1]) == len(want) and t[r, :len(want)].tolist() == want
        pad = (len(want) + 63) // 64 * 64
        assert all(0 <= x < n_pages * 256 for x in t[r, len(want):pad].tolist())


@pytest.mark.parametrize("rows", [0, 160, 256])
def test_config3_shape_small_batch(dev, rows):
    case = configs.config3_small(seed=3, n_req=2)
    check(run_case(case, dev, rows_per_group=rows), oracle_case(case))


@pytest.mark.parametrize("rows", [0, 128, 256])
def test_ragged_requests_under_the_default_cut(dev, rows):
    """Requests of one batch with very different numbers of selected keys (one with none at all) and the default
    plan, whose workgroups take the first tiles of each row group side by side and then the remaining tiles:
    a request shorter than that first part leaves the later workgroups empty pieces."""
    case = configs.chunked_prefix_case(29, n_req=4, n_chunks=8, chunk_tokens=512, topk=6, q_len=160,
                                       shared_prefix=False)
    case.ranges[1] = case.ranges[1][:1]              # 512 keys
    case.ranges[2] = []                              # only the active block
    case.ranges[3] = [(s, l - 37) for s, l in case.ranges[3][:3]]   # ranges that end inside a page
    ref = oracle_case(case)
    out = run_case(case, dev, rows_per_group=rows)
    check(out, ref)
    # the same through the shared slot table
    ops = _ops()
    d = lambda t: None if t is None else t.to(dev)
    rp, rs, rl, mr = case.range_tensors()
    table = ops.new_slot_table(4, case.max_ctx, dev)
    prep = ops.PreparedAttention(d(case.q), d(case.k_new), d(case.v_new), d(case.k_cache), d(case.v_cache),
                                 d(case.block_table), d(case.q_start_loc), max_q_len=case.max_q,
                                 max_ctx_len=case.max_ctx, ranges=(d(rp), d(rs), d(rl), mr), slot_table=table,
                                 rows_per_group=rows)
    prep.build_slot_table()
    assert torch.equal(prep.run().float().cpu(), out)


def test_context_lens_path_matches_ranges(dev):
    """The reference's decode context (first ctx_len tokens of the page table) is the single-range case."""
    case = configs.chunked_prefix_case(11, n_req=3, n_chunks=1, chunk_tokens=333, topk=1, q_len=32,
                                       shared_prefix=False)
    ref = oracle_case(case)
    check(run_case(case, dev, use_ctx_lens=True), ref)
    check(run_case(case, dev), ref)


def test_mha_group_of_one(dev):
    case = configs.chunked_prefix_case(5, n_req=2, n_chunks=3, chunk_tokens=257, topk=2, q_len=64, Hq=8, Hkv=8)
    check(run_case(case, dev), oracle_case(case))


def test_causal_and_dense_masks(dev):
    case = configs.chunked_prefix_case(9, n_req=2, n_chunks=2, chunk_tokens=100, topk=1, q_len=70,
                                       shared_prefix=False)
    check(run_case(case, dev, mask_mode="causal"), oracle_case(case, mask_mode="causal"))
    gen = torch.Generator().manual_seed(0)
    n = case.q.shape[0]
    mask = torch.rand(n, n, generator=gen) < 0.5
    check(run_case(case, dev, mask_mode="dense", mask=mask), oracle_case(case, mask_mode="dense", mask=mask))


def test_reference_decoding_test_procedure(dev):
    """The procedure of the reference's examples/test_dllm_decoding_kernel.py:11-97: 20 sequences of
    64 active rows over contexts of 81..120 tokens (one page each), block-causal dense mask, checked
    on every sequence (the reference checks sequence 0 only)."""
    torch.manual_seed(114514)
    seq = torch.tensor([64] * 20, dtype=torch.int32)
    ctx = torch.tensor([119, 110, 81, 114, 112, 119, 110, 81, 114, 112, 119, 110, 81, 114, 112, 120, 111, 82, 115,
                        113], dtype=torch.int32)
    n = int(seq.sum())
    q = torch.randn(n, 28, 128).to(torch.bfloat16)
    k = torch.randn(n, 4, 128).to(torch.bfloat16)
    v = torch.randn(n, 4, 128).to(torch.bfloat16)
    k_cache = torch.randn(20, 256, 4, 128).to(torch.bfloat16)
    v_cache = torch.randn(20, 256, 4, 128).to(torch.bfloat16)
    bt = torch.arange(20, dtype=torch.int32).view(20, 1)
    cu = torch.cat([torch.zeros(1, dtype=torch.int32), torch.cumsum(seq, 0).to(torch.int32)])
    mask = torch.zeros(n, n, dtype=torch.bool)
    for i in range(20):
        s = int(cu[i])
        for b in range(2):
            mask[s + 32 * b:s + 32 * b + 32, s:s + 32 * b + 32] = True
    ops = _ops()
    out = torch.empty(n, 28, 128, dtype=torch.bfloat16, device=dev)
    scale = 1.0 / math.sqrt(128)
    ops.diffusion_lm_parallel_flash_decoding(q.to(dev), k.to(dev), v.to(dev), out, "torch.bfloat16",
                                             k_cache.to(dev), v_cache.to(dev), bt.to(dev), cu.to(dev),
                                             (seq + ctx).to(dev), int((seq + ctx).max()), 64, 1.0, 1.0,
                                             diffusion_blk_sz=32, sm_scale=scale, mask=mask.to(dev))
    torch.cuda.synchronize()
    ranges = [[(0, int(c))] for c in ctx]
    ref = ref_ops.sparse_decode_attention(q, k, v, k_cache, v_cache, bt, cu, ranges, mask_mode="dense", mask=mask,
                                          sm_scale=scale)
    # N(0,1) inputs give outputs of magnitude ~1; bf16 rounding of O dominates
    check(out.float().cpu(), ref, tol=3e-2)


def test_fully_masked_rows_give_zeros(dev):
    case = configs.chunked_prefix_case(2, n_req=1, n_chunks=1, chunk_tokens=64, topk=1, q_len=32)
    case.ranges = [[]]  # no visible prefix
    n = case.q.shape[0]
    mask = torch.ones(n, n, dtype=torch.bool)
    mask[5, :] = False
    ops = _ops()
    d = lambda t: t.to(dev)
    out = ops.sparse_decode_attention(d(case.q), d(case.k_new), d(case.v_new), None, None, None,
                                      d(case.q_start_loc), max_q_len=32, max_ctx_len=0, mask_mode="dense",
                                      mask=d(mask)).float().cpu()
    ref = oracle_case(case, mask_mode="dense", mask=mask)
    assert out[5].abs().max() == 0
    check(out, ref)


def test_fp8_pages_with_per_page_scale(dev):
    """BASELINE config 5 shape (MHA, fp8 e4m3 pages, fp32 scale per page) at reduced size; the
    oracle sees float(e4m3) * scale rounded to bf16, i.e. exactly what the kernel dequantises."""
    case = configs.config5_small(seed=4, n_req=2, n_chunks=6, topk=3)
    check(run_case(case, dev), oracle_case(case))


@pytest.mark.parametrize("q_len,Hq,Hkv,blocks", [(160, 32, 32, 5), (176, 8, 8, 6), (90, 8, 4, 6), (65, 8, 4, 5)])
def test_fp8_groups_of_five_and_six_row_blocks(dev, q_len, Hq, Hkv, blocks):
    """fp8 pages have no 8-block kernel: 129-192 rows per (request, KV head) can run as one group of 5 or 6 row
    blocks (the planner's choice for large shapes; forced here), MHA and grouped heads, cut and uncut."""
    case = configs.chunked_prefix_case(21 + q_len, n_req=2, n_chunks=5, chunk_tokens=300, topk=3, q_len=q_len,
                                       Hq=Hq, Hkv=Hkv, fp8=True)
    ref = oracle_case(case)
    for splits in (0, 1, 3):
        check(run_case(case, dev, rows_per_group=32 * blocks, num_splits=splits), ref, what=f"splits={splits}")


@pytest.mark.parametrize("plan", [dict(), dict(num_splits=2), dict(tiles_per_workgroup=7), dict(tiles_per_workgroup=1)],
                         ids=["default", "split2", "span7", "span1"])
def test_fp8_five_row_blocks_masks_and_ragged_pieces(dev, plan):
    """The fp8 kernel for five row blocks has waves that only fill the tile buffers for the others: causal and
    dense masks over the active block, 150 rows (the last row block and the last active tile ragged), prefixes that
    end inside a tile, and workgroups whose span covers pieces of two columns or a single tile."""
    case = configs.chunked_prefix_case(57, n_req=3, n_chunks=4, chunk_tokens=210, topk=2, q_len=150, Hq=4, Hkv=4,
                                       fp8=True, shared_prefix=False)
    check(run_case(case, dev, rows_per_group=160, **plan), oracle_case(case), what="full")
    check(run_case(case, dev, rows_per_group=160, mask_mode="causal", **plan), oracle_case(case, mask_mode="causal"),
          what="causal")
    gen = torch.Generator().manual_seed(3)
    n = case.q.shape[0]
    mask = torch.rand(n, n, generator=gen) < 0.5
    mask |= torch.eye(n, dtype=torch.bool)
    check(run_case(case, dev, rows_per_group=160, mask_mode="dense", mask=mask, **plan),
          oracle_case(case, mask_mode="dense", mask=mask), what="dense")


@pytest.mark.parametrize("q_len,Hq,Hkv,mode", [(160, 28, 4, "full"), (80, 8, 2, "causal"), (75, 8, 4, "full")])
def test_fp8_default_plan_takes_groups_of_five_where_they_fill(dev, q_len, Hq, Hkv, mode):
    """With fp8 pages the planner cuts the rows of a (request, KV head) into groups of five row blocks (the kernel
    with producer waves) when that leaves no more empty blocks than groups of four: 35 blocks (7 groups), 10 blocks
    (2 groups), 10 blocks with a ragged last one.  Several row groups per (request, KV head), by default and forced."""
    ops = _ops()
    case = configs.chunked_prefix_case(71 + q_len, n_req=2, n_chunks=5, chunk_tokens=300, topk=3, q_len=q_len,
                                       Hq=Hq, Hkv=Hkv, fp8=True, shared_prefix=False)
    d = lambda t: t.to(dev)
    rp, rs, rl, mr = case.range_tensors()
    pr = ops.PreparedAttention(d(case.q), d(case.k_new), d(case.v_new), d(case.k_cache), d(case.v_cache),
                               d(case.block_table), d(case.q_start_loc), max_q_len=case.max_q, max_ctx_len=case.max_ctx,
                               ranges=(d(rp), d(rs), d(rl), mr), k_scale=d(case.k_scale), v_scale=d(case.v_scale),
                               mask_mode=mode)
    if Hq == 28:  # (the smaller shapes take shorter row groups by default, to fill the compute units)
        assert "kv=fp8 row_blocks=5" in pr.describe_plan(), pr.describe_plan()
    ref = oracle_case(case, mask_mode=mode)
    check(run_case(case, dev, mask_mode=mode), ref, what="default plan")
    check(run_case(case, dev, mask_mode=mode, rows_per_group=160), ref, what="groups of 160 rows")
    # 7 row blocks (32 response rows of 7 query heads each) stay with groups of four
    small = configs.chunked_prefix_case(72, n_req=2, n_chunks=5, chunk_tokens=300, topk=3, q_len=32, fp8=True)
    rp, rs, rl, mr = small.range_tensors()
    pr = ops.PreparedAttention(d(small.q), d(small.k_new), d(small.v_new), d(small.k_cache), d(small.v_cache),
                               d(small.block_table), d(small.q_start_loc), max_q_len=small.max_q,
                               max_ctx_len=small.max_ctx, ranges=(d(rp), d(rs), d(rl), mr), k_scale=d(small.k_scale),
                               v_scale=d(small.v_scale))
    assert "row_blocks=5" not in pr.describe_plan(), pr.describe_plan()


@pytest.mark.parametrize("plan", [dict(), dict(num_splits=1), dict(num_splits=4)], ids=["default", "unsplit", "split4"])
def test_fp8_five_row_blocks_ragged_requests(dev, plan):
    """The kernel with producer waves on requests of very different prefix lengths: one with a single chunk, one with
    no visible key at all (its pieces hold tiles of the active block only, or nothing), one whose ranges end inside a
    page; pieces past the end of a short request are empty."""
    case = configs.chunked_prefix_case(83, n_req=4, n_chunks=6, chunk_tokens=330, topk=5, q_len=140, Hq=8, Hkv=8,
                                       fp8=True, shared_prefix=False)
    case.ranges[1] = case.ranges[1][:1]
    case.ranges[2] = []
    case.ranges[3] = [(s, l - 37) for s, l in case.ranges[3][:3]]
    check(run_case(case, dev, rows_per_group=160, **plan), oracle_case(case))


def test_fp8_codes_decode_like_torch(dev):
    """All 256 e4m3 codes through the kernel's dequantisation == torch.float8_e4m3fn -> float."""
    ops = _ops()
    codes = torch.arange(0x7f, dtype=torch.uint8)  # every positive code (0x7f is NaN); mean is far from 0
    n = codes.numel()
    # one key per code: V row = the code in every element, K = 0 so softmax is uniform over n keys
    Hkv, dd = 1, 128
    pages = (n + 255) // 256
    v8 = torch.zeros(pages * 256, Hkv, dd, dtype=torch.uint8)
    v8[:n] = codes.view(n, 1, 1)
    k8 = torch.zeros_like(v8)
    scale = torch.tensor([0.5] * pages, dtype=torch.float32)
    q = torch.zeros(32, 1, dd, dtype=torch.bfloat16)
    knew = torch.zeros(32, 1, dd, dtype=torch.bfloat16)
    # active block fully masked out so only the cache is averaged
    mask = torch.zeros(32, 32, dtype=torch.bool)
    bt = torch.arange(pages, dtype=torch.int32).view(1, pages)
    out = ops.sparse_decode_attention(q.to(dev), knew.to(dev), knew.to(dev),
                                      k8.view(pages, 256, Hkv, dd).view(torch.float8_e4m3fn).to(dev),
                                      v8.view(pages, 256, Hkv, dd).view(torch.float8_e4m3fn).to(dev), bt.to(dev),
                                      torch.tensor([0, 32], dtype=torch.int32, device=dev), max_q_len=32,
                                      max_ctx_len=n, context_lens=torch.tensor([n], dtype=torch.int32, device=dev),
                                      mask_mode="dense", mask=mask.to(dev), k_scale=scale.to(dev),
                                      v_scale=scale.to(dev)).float().cpu()
    vals = (codes.view(torch.float8_e4m3fn).float() * 0.5).to(torch.bfloat16).float()
    expect = vals.mean().item()
    assert abs(out[0, 0, 0].item() - expect) <= 2e-2 * max(1.0, abs(expect))


@pytest.mark.parametrize("causal", [True, False])
def test_chunk_prefill_block_diagonal(dev, causal):
    """BASELINE config 4 shape at reduced size: independent chunks of ragged length, causal inside a
    chunk, K/V written to shuffled pages through a slot mapping."""
    gen = torch.Generator().manual_seed(21)
    lens = [257, 64, 1, 130, 300]
    n = sum(lens)
    Hq, Hkv, dd = 28, 4, 128
    q = (torch.randn(n, Hq, dd, generator=gen)).to(torch.bfloat16)
    k = (torch.randn(n, Hkv, dd, generator=gen)).to(torch.bfloat16)
    v = (torch.randn(n, Hkv, dd, generator=gen)).to(torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    n_pages = (n + 255) // 256 + 2
    page_ids = torch.randperm(n_pages, generator=gen)[:(n + 255) // 256].tolist()
    slots = ref_ops.slot_mapping(page_ids, n)
    slots[10] = -1  # a skipped token
    ops = _ops()
    kc = torch.zeros(n_pages, 256, Hkv, dd, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    out = ops.chunk_prefill_attention(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), max_seqlen=max(lens),
                                      causal=causal, k_cache=kc, v_cache=vc, slot_mapping=slots.to(dev))
    torch.cuda.synchronize()
    ref = ref_ops.chunk_prefill_attention(q, k, v, cu, causal=causal)
    check(out.float().cpu(), ref, tol=3e-2)
    kc_ref = torch.zeros(n_pages, 256, Hkv, dd, dtype=torch.bfloat16)
    vc_ref = torch.zeros_like(kc_ref)
    ref_ops.store_kvcache(k, v, kc_ref, vc_ref, slots)
    assert torch.equal(kc.cpu(), kc_ref) and torch.equal(vc.cpu(), vc_ref)


@pytest.mark.parametrize("lens,heads,causal", [
    ([300] * 8, (28, 4), True), ([300] * 8, (28, 4), False),
    ([1025, 700, 64, 1, 333, 1024, 1000, 129] * 2, (28, 4), True),        # ragged: empty columns, single-tile columns
    ([1025, 700, 64, 1, 333, 1024, 1000, 129] * 2, (28, 4), False),
    ([2000, 1950], (32, 32), True),                                        # MHA: a column spans two to three key tiles
    ([4100] * 2, (28, 4), True),                                           # few units: teams of 64 workgroups
    ([700, 650, 600, 590], (28, 4), True),                                 # 16 units: teams of 32 workgroups
])
def test_chunk_prefill_stream_kernel(dev, lens, heads, causal):
    """Large batches of chunks run on resident workgroups that stream through their columns
    (attn_prefill_stream_kernel); one workgroup per column (num_splits = 1) is the same arithmetic in the same
    order: the two must agree bit for bit on every row, and with the oracle within the attention bound."""
    from prefilling_dllm_amd._lib import AttnDesc  # noqa: F401  (the library is loaded)
    ops = _ops()
    Hq, Hkv = heads
    gen = torch.Generator().manual_seed(len(lens) * 131 + Hq + int(causal))
    n, dd = sum(lens), 128
    q = torch.randn(n, Hq, dd, generator=gen).to(torch.bfloat16)
    k = torch.randn(n, Hkv, dd, generator=gen).to(torch.bfloat16)
    v = torch.randn(n, Hkv, dd, generator=gen).to(torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    a = ops.chunk_prefill_attention(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), max_seqlen=max(lens), causal=causal)
    b = ops.chunk_prefill_attention(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), max_seqlen=max(lens), causal=causal,
                                    num_splits=1)
    torch.cuda.synchronize()
    assert "attn_prefill_stream_kernel" in ops.describe_prefill_plan(len(lens), Hq, Hkv, max(lens), n, causal)
    assert "attn_fwd_kernel" in ops.describe_prefill_plan(len(lens), Hq, Hkv, max(lens), n, causal, num_splits=1)
    assert torch.equal(a, b)
    if n * Hq <= 16 * 1100 * 28 and max(lens) <= 2000:        # the oracle in a few seconds
        ref = ref_ops.chunk_prefill_attention(q, k, v, cu, causal=causal)
        check(a.float().cpu(), ref, tol=3e-2)


@pytest.mark.parametrize("seed", range(6))
def test_chunk_prefill_stream_kernel_random_batches(dev, seed):
    """Seeded random batches for the stream kernel: ragged chunk lengths with empty chunks, one-token chunks and
    lengths on both sides of a tile boundary, 1 to 16 query heads per KV head, logits that grow along the keys (the
    running maximum moves in late tiles: accumulators that carry weight are rescaled), causal and full masks.  The
    result must equal one workgroup per column up to the rounding of the output: the decision to rescale is taken
    per wave, and in a wave that also holds rows past the end of its chunk it depends on what those lanes hold, which
    the two kernels fill differently -- such rows may differ by one bf16 step, every other row is equal bit for bit."""
    ops = _ops()
    rng = torch.Generator().manual_seed(1000 + seed)
    Hq, Hkv = [(28, 4), (8, 8), (16, 8), (32, 8), (16, 2), (32, 2)][seed]
    G = Hq // Hkv
    pick = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=rng))
    special = [0, 1, 63, 64, 65, 127, 128, 129, 1024, 1025]
    # enough rows per chunk for 16 columns of 128 rows (R >= team) at the largest chunk, enough units for the teams
    lmax = max(pick(1100, 1600), (16 * 128 + G - 1) // G + 1)
    n_chunks = max(8, 2 * (512 // 16) // Hkv + pick(0, 3))
    lens = [lmax] + [special[pick(0, len(special) - 1)] if pick(0, 3) == 0 else pick(1, lmax) for _ in range(n_chunks - 1)]
    causal = seed % 2 == 0
    n, dd = sum(lens), 128
    q = torch.randn(n, Hq, dd, generator=rng).to(torch.bfloat16)
    k = torch.randn(n, Hkv, dd, generator=rng)
    # keys late in a chunk carry larger logits: ramp their norm along the chunk
    pos = torch.cat([torch.arange(l) for l in lens]).float()
    k = (k * (1.0 + pos[:, None, None] / 400.0)).to(torch.bfloat16)
    v = torch.randn(n, Hkv, dd, generator=rng).to(torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    plan = ops.describe_prefill_plan(len(lens), Hq, Hkv, max(lens), n, causal)
    assert "attn_prefill_stream_kernel" in plan, (plan, lens, Hq, Hkv)
    a = ops.chunk_prefill_attention(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), max_seqlen=max(lens), causal=causal)
    b = ops.chunk_prefill_attention(q.to(dev), k.to(dev), v.to(dev), cu.to(dev), max_seqlen=max(lens), causal=causal,
                                    num_splits=1)
    torch.cuda.synchronize()
    af, bf = a.float().cpu(), b.float().cpu()
    assert torch.isfinite(af).all()
    differ = (af != bf).flatten(1).any(dim=1)
    assert int(differ.sum()) <= len(lens) * max(1, 32 // G + 1), (seed, int(differ.sum()))   # last row blocks of chunks at most
    row_scale = bf.abs().amax(dim=2, keepdim=True).clamp_min(2.0 ** -7)          # one bf16 step of the row's largest
    assert ((af - bf).abs() <= 2.0 ** -7 * row_scale).all(), (seed, (af - bf).abs().max())
    # one mid-sized chunk against the oracle
    c = max(range(len(lens)), key=lambda i: lens[i] if lens[i] <= 700 else 0)
    if lens[c] > 0:
        lo, hi = int(cu[c]), int(cu[c + 1])
        ref = ref_ops.chunk_prefill_attention(q[lo:hi], k[lo:hi], v[lo:hi], [0, hi - lo], causal=causal)
        check(a[lo:hi].float().cpu(), ref, tol=3e-2)


def test_permuting_pages_leaves_output_unchanged(dev):
    """Size-independent property: the physical page order is irrelevant (same logical tokens)."""
    case = configs.chunked_prefix_case(13, n_req=1, n_chunks=4, chunk_tokens=512, topk=4, q_len=32)
    out1 = run_case(case, dev)
    perm = torch.randperm(case.k_cache.shape[0], generator=torch.Generator().manual_seed(1))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(perm.numel())
    case.k_cache = case.k_cache[perm]
    case.v_cache = case.v_cache[perm]
    case.block_table = inv[case.block_table.long()].to(torch.int32)
    out2 = run_case(case, dev)
    assert torch.equal(out1, out2)


def test_value_of_ones_gives_ones(dev):
    """Rows of the softmax sum to one: V == 1 everywhere => O == 1 (up to bf16 rounding of P)."""
    case = configs.config3_small(seed=5, n_req=1)
    case.v_cache = torch.ones_like(case.v_cache)
    case.v_new = torch.ones_like(case.v_new)
    out = run_case(case, dev)
    assert (out - 1.0).abs().max() <= 1e-2


def test_limits_many_ranges_single_row_and_empty_request(dev):
    """The edges of what a descriptor may hold: 128 ranges per request (the most the table builder accepts;
    129 is refused), ranges of a few tokens that start and end anywhere inside pages, a request with a single
    query row next to one with none, and a request whose ranges are empty."""
    ops = _ops()
    case = configs.chunked_prefix_case(37, n_req=3, n_chunks=4, chunk_tokens=512, topk=4, q_len=8,
                                       shared_prefix=False)
    gen = torch.Generator().manual_seed(1)
    starts = sorted(torch.randperm(2048 - 16, generator=gen)[:128].tolist())
    many = []
    for i, s0 in enumerate(starts):
        nxt = starts[i + 1] if i + 1 < len(starts) else 2048
        many.append((s0, max(1, min(1 + i % 7, nxt - s0))))
    case.ranges[0] = many
    case.ranges[1] = [(5, 1)]
    case.ranges[2] = []
    # request 0: 8 rows, request 1: one row, request 2: no rows at all
    case.q_start_loc = torch.tensor([0, 8, 9, 9], dtype=torch.int32)
    case.q, case.k_new, case.v_new = case.q[:9], case.k_new[:9], case.v_new[:9]
    ref = oracle_case(case)
    for rows in (0, 32, 128):
        check(run_case(case, dev, rows_per_group=rows), ref)
    case.ranges[0] = many + [(2040, 2)]
    with pytest.raises(NotImplementedError):
        run_case(case, dev)


def test_cache_beyond_four_gib_uses_wide_addresses(dev):
    """The K/V copies use 32-bit byte offsets when every source tensor is below 4 GiB and 64-bit addresses
    otherwise: the same request through a small cache and through pages at the far end of a 4.3 GB cache
    must give the same bits."""
    ops = _ops()
    case = configs.chunked_prefix_case(41, n_req=2, n_chunks=6, chunk_tokens=512, topk=3, q_len=160,
                                       shared_prefix=False)
    ref = oracle_case(case)
    small = run_case(case, dev)
    check(small, ref)
    n_small = case.k_cache.shape[0]
    n_big = 16400                                   # x 256 tokens x 1 KiB = 4.3 GB per cache
    shift = n_big - n_small
    kc = torch.empty((n_big, 256, 4, 128), dtype=torch.bfloat16, device=dev)
    vc = torch.empty_like(kc)
    kc[shift:] = case.k_cache.to(dev)
    vc[shift:] = case.v_cache.to(dev)
    rp, rs, rl, mr = case.range_tensors()
    d = lambda t: t.to(dev)
    out = ops.sparse_decode_attention(d(case.q), d(case.k_new), d(case.v_new), kc, vc,
                                      d(case.block_table + shift), d(case.q_start_loc), max_q_len=case.max_q,
                                      max_ctx_len=case.max_ctx, ranges=(d(rp), d(rs), d(rl), mr))
    torch.cuda.synchronize()
    assert torch.equal(out.float().cpu(), small)
    del kc, vc


def test_fp8_cache_beyond_four_gib_takes_the_register_staged_kernel(dev):
    """Five row blocks on fp8 pages run with producer waves that address the caches with 32-bit offsets; a cache
    of 4 GiB or more takes the kernel that dequantises through registers with 64-bit addresses.  The same
    request through a small cache and through pages at the far end of a 4.3 GB cache: both match the oracle."""
    ops = _ops()
    case = configs.chunked_prefix_case(43, n_req=2, n_chunks=5, chunk_tokens=300, topk=3, q_len=150, Hq=8, Hkv=8,
                                       fp8=True)
    ref = oracle_case(case)
    check(run_case(case, dev), ref, what="small cache")
    n_small, page = case.k_cache.shape[0], case.k_cache.shape[1]
    n_big = (1 << 32) // (page * 8 * 128) + 64      # pages of page x 8 heads x 128 bytes: a little over 4 GiB
    shift = n_big - n_small
    kc = torch.empty((n_big, page, 8, 128), dtype=case.k_cache.dtype, device=dev)
    vc = torch.empty_like(kc)
    kc[shift:] = case.k_cache.to(dev)
    vc[shift:] = case.v_cache.to(dev)
    ks = torch.ones((n_big,) + tuple(case.k_scale.shape[1:]), dtype=torch.float32, device=dev)
    vs = torch.ones_like(ks)
    ks[shift:] = case.k_scale.to(dev)
    vs[shift:] = case.v_scale.to(dev)
    rp, rs, rl, mr = case.range_tensors()
    d = lambda t: t.to(dev)
    out = ops.sparse_decode_attention(d(case.q), d(case.k_new), d(case.v_new), kc, vc,
                                      d(case.block_table + shift), d(case.q_start_loc), max_q_len=case.max_q,
                                      max_ctx_len=case.max_ctx, ranges=(d(rp), d(rs), d(rl), mr), k_scale=ks, v_scale=vs)
    torch.cuda.synchronize()
    check(out.float().cpu(), ref, what="4.3 GB cache")
    del kc, vc


def test_error_codes(dev):
    ops = _ops()
    q = torch.zeros(32, 4, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(NotImplementedError):
        ops.sparse_decode_attention(q, q, q, None, None, None, torch.tensor([0, 32], dtype=torch.int32, device=dev),
                                    max_q_len=32, max_ctx_len=0)
    q = torch.zeros(32, 6, 128, dtype=torch.bfloat16, device=dev)
    k = torch.zeros(32, 4, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        ops.sparse_decode_attention(q, k, k, None, None, None, torch.tensor([0, 32], dtype=torch.int32, device=dev),
                                    max_q_len=32, max_ctx_len=0)
    with pytest.raises(ValueError):
        ops.sparse_decode_attention(q.cpu(), k.cpu(), k.cpu(), None, None, None,
                                    torch.tensor([0, 32], dtype=torch.int32), max_q_len=32, max_ctx_len=0)


def test_attention_layer_interface(dev):
    """The layer mirror of attention_v4.Attention: a prefill that stores K/V into pages, then a decode
    step of a 32-token block against that paged context, both checked against the oracle."""
    from prefilling_dllm_amd.attention import Attention
    from prefilling_dllm_amd.context import set_context_diffusion_lm, reset_context_diffusion_lm
    gen = torch.Generator().manual_seed(31)
    Hq, Hkv, d, P = 28, 4, 128, 256
    prompt, block = 300, 32
    scale = d ** -0.5
    layer = Attention(Hq, d, scale, Hkv, "diffusion_lm")
    layer.k_cache = torch.zeros(6, P, Hkv, d, dtype=torch.bfloat16, device=dev)
    layer.v_cache = torch.zeros_like(layer.k_cache)
    prompt_pages, block_pages = [4, 1], [3]
    mk = lambda n, h: (torch.randn(n, h * d, generator=gen) / 3).to(torch.bfloat16)
    q, k, v = mk(prompt + block, Hq), mk(prompt + block, Hkv), mk(prompt + block, Hkv)
    slots = ref_ops.split_slot_mapping(prompt_pages, block_pages, prompt, block)
    cu = torch.tensor([0, prompt + block], dtype=torch.int32, device=dev)
    set_context_diffusion_lm(True, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_q=prompt + block,
                             max_seqlen_k=prompt + block, slot_mapping=slots.to(dev), mask_kind="full")
    try:
        o = layer(q.to(dev), k.to(dev), v.to(dev))
    finally:
        reset_context_diffusion_lm()
    ref = ref_ops.chunk_prefill_attention(q.view(-1, Hq, d), k.view(-1, Hkv, d), v.view(-1, Hkv, d),
                                          [0, prompt + block], causal=False, sm_scale=scale)
    check(o.view(-1, Hq, d).float().cpu(), ref, tol=3e-2)
    # decode step: replace the block, context = the prompt tokens in pages [4, 1]
    q2, k2, v2 = mk(block, Hq), mk(block, Hkv), mk(block, Hkv)
    slots2 = ref_ops.slot_mapping(block_pages, block)
    cu2 = torch.tensor([0, block], dtype=torch.int32, device=dev)
    bt = torch.tensor([prompt_pages + block_pages], dtype=torch.int32, device=dev)
    set_context_diffusion_lm(False, cu_seqlens_q=cu2, max_seqlen_q=block, max_seqlen_k=prompt + block,
                             slot_mapping=slots2.to(dev), context_lens=torch.tensor([prompt], dtype=torch.int32, device=dev),
                             block_tables=bt, mask_kind="full")
    try:
        o2 = layer(q2.to(dev), k2.to(dev), v2.to(dev))
    finally:
        reset_context_diffusion_lm()
    kc, vc = layer.k_cache.cpu(), layer.v_cache.cpu()
    ref2 = ref_ops.sparse_decode_attention(q2.view(-1, Hq, d), k2.view(-1, Hkv, d), v2.view(-1, Hkv, d), kc, vc,
                                           bt.cpu(), [0, block], [[(0, prompt)]], sm_scale=scale)
    check(o2.view(-1, Hq, d).float().cpu(), ref2, tol=3e-2)
    # the decode step stored the new block rows behind the prompt pages
    assert torch.equal(kc[3, :block], k2.view(-1, Hkv, d))


def test_store_before_attention_for_callers_that_rewrite_visible_rows(dev, monkeypatch):
    """A decode step normally stores its active rows inside the attention call, after the kernel has read the cache;
    that equals the reference's store-then-attend order (attention_v4.py:328-331) only while no active slot is a
    visible prefix slot.  A caller that rewrites visible context rows sets `store_before_attention`: the output is then
    the oracle's over the cache *after* the store.  Without the flag the debug check names the violation."""
    from prefilling_dllm_amd.attention import Attention
    from prefilling_dllm_amd.context import set_context_diffusion_lm, reset_context_diffusion_lm
    gen = torch.Generator().manual_seed(53)
    Hq, Hkv, d, P = 28, 4, 128, 256
    ctx, block = 300, 32
    layer = Attention(Hq, d, d ** -0.5, Hkv, "diffusion_lm")
    kc0 = (torch.randn(4, P, Hkv, d, generator=gen) / 3).to(torch.bfloat16)
    vc0 = (torch.randn(4, P, Hkv, d, generator=gen) / 3).to(torch.bfloat16)
    bt = torch.tensor([[2, 0]], dtype=torch.int32)
    mk = lambda n, h: (torch.randn(n, h * d, generator=gen) / 3).to(torch.bfloat16)
    q, k, v = mk(block, Hq), mk(block, Hkv), (mk(block, Hkv).float() + 2.0).to(torch.bfloat16)
    # the block overwrites context tokens 100 .. 131 (page 2 of the cache), which every row can see
    slots = (2 * P + 100 + torch.arange(block)).to(torch.int32)
    cu = torch.tensor([0, block], dtype=torch.int32, device=dev)
    common = dict(cu_seqlens_q=cu, max_seqlen_q=block, max_seqlen_k=ctx + block, slot_mapping=slots.to(dev),
                  context_lens=torch.tensor([ctx], dtype=torch.int32, device=dev), block_tables=bt.to(dev),
                  mask_kind="full")
    kc_ref, vc_ref = kc0.clone(), vc0.clone()
    ref_ops.store_kvcache(k.view(-1, Hkv, d), v.view(-1, Hkv, d), kc_ref, vc_ref, slots)
    ref = ref_ops.sparse_decode_attention(q.view(-1, Hq, d), k.view(-1, Hkv, d), v.view(-1, Hkv, d), kc_ref, vc_ref,
                                          bt, [0, block], [[(0, ctx)]])
    stale = ref_ops.sparse_decode_attention(q.view(-1, Hq, d), k.view(-1, Hkv, d), v.view(-1, Hkv, d), kc0, vc0,
                                            bt, [0, block], [[(0, ctx)]])
    assert (ref - stale).abs().max() > 0.05            # the order matters for this input
    layer.k_cache, layer.v_cache = kc0.to(dev), vc0.to(dev)
    set_context_diffusion_lm(False, store_before_attention=True, **common)
    try:
        o = layer(q.to(dev), k.to(dev), v.to(dev))
    finally:
        reset_context_diffusion_lm()
    check(o.view(-1, Hq, d).float().cpu(), ref, tol=3e-2)
    assert torch.equal(layer.k_cache.cpu(), kc_ref) and torch.equal(layer.v_cache.cpu(), vc_ref)
    # without the flag, under the debug check: refused before anything is launched or stored
    layer.k_cache, layer.v_cache = kc0.to(dev), vc0.to(dev)
    monkeypatch.setenv("PDLLM_DEBUG_CHECKS", "1")
    set_context_diffusion_lm(False, **common)
    try:
        with pytest.raises(RuntimeError, match="store_before_attention"):
            layer(q.to(dev), k.to(dev), v.to(dev))
    finally:
        reset_context_diffusion_lm()
    assert torch.equal(layer.k_cache.cpu(), kc0)


def test_reference_form_decode_masks_with_context_columns(dev):
    """The reference hands the layer per-sequence masks [Sq, ctx + Sq] (fastdllm_engine.py:496-507: all ones, with
    the keys behind `valid_tokens` hidden from the first `valid_tokens` rows) through `seqs`, or the block-diagonal
    [Nq, sum(ctx + Sq)] tensor its context assembles from them (utils/context.py:85-98).  Both must reach the kernel
    as the [Nq, Nq] mask over the active keys; a mask of the wrong shape or one that hides context keys is refused."""
    from types import SimpleNamespace
    from prefilling_dllm_amd.attention import Attention
    from prefilling_dllm_amd.context import set_context_diffusion_lm, reset_context_diffusion_lm
    ops = _ops()
    gen = torch.Generator().manual_seed(41)
    Hq, Hkv, d, P = 28, 4, 128, 256
    ctxs, lens, valid = [300, 70], [40, 32], [25, 32]
    n = sum(lens)
    layer = Attention(Hq, d, d ** -0.5, Hkv, "diffusion_lm")
    kc = (torch.randn(5, P, Hkv, d, generator=gen) / 3).to(torch.bfloat16)
    vc = (torch.randn(5, P, Hkv, d, generator=gen) / 3).to(torch.bfloat16)
    layer.k_cache, layer.v_cache = kc.to(dev), vc.to(dev)
    bt = torch.tensor([[4, 1], [2, 0]], dtype=torch.int32)
    mk = lambda rows, h: (torch.randn(rows, h * d, generator=gen) / 3).to(torch.bfloat16)
    q, k, v = mk(n, Hq), mk(n, Hkv), mk(n, Hkv)
    masks = []
    for c, l, va in zip(ctxs, lens, valid):
        m = torch.ones(l, c + l, dtype=torch.bool)
        m[:va, c + va:] = False
        masks.append(m)
    cu = torch.tensor([0, lens[0], n], dtype=torch.int32, device=dev)
    common = dict(cu_seqlens_q=cu, max_seqlen_q=max(lens), max_seqlen_k=max(c + l for c, l in zip(ctxs, lens)),
                  context_lens=torch.tensor(ctxs, dtype=torch.int32, device=dev), block_tables=bt.to(dev),
                  need_kv_cache_store=False)
    # the oracle's mask: [Nq, Nq] over the active keys
    act = torch.zeros(n, n, dtype=torch.bool)
    act[:lens[0], :lens[0]] = masks[0][:, ctxs[0]:]
    act[lens[0]:, lens[0]:] = masks[1][:, ctxs[1]:]
    ref = ref_ops.sparse_decode_attention(q.view(-1, Hq, d), k.view(-1, Hkv, d), v.view(-1, Hkv, d), kc, vc, bt,
                                          [0, lens[0], n], [[(0, ctxs[0])], [(0, ctxs[1])]], mask_mode="dense",
                                          mask=act)
    # (1) through seqs, as the engine does
    seqs = [SimpleNamespace(current_block_mask=m.to(dev).view(1, 1, *m.shape), diffusion_block_size=32) for m in masks]
    set_context_diffusion_lm(False, seqs=seqs, seq_lens=lens, **common)
    try:
        o1 = layer(q.to(dev), k.to(dev), v.to(dev))
    finally:
        reset_context_diffusion_lm()
    check(o1.view(-1, Hq, d).float().cpu(), ref, tol=3e-2, what="seqs")
    # (2) the assembled block-diagonal tensor with context columns
    wide = torch.zeros(n, sum(c + l for c, l in zip(ctxs, lens)), dtype=torch.bool)
    wide[:lens[0], :ctxs[0] + lens[0]] = masks[0]
    wide[lens[0]:, ctxs[0] + lens[0]:] = masks[1]
    set_context_diffusion_lm(False, block_mask=wide.to(dev), **common)
    try:
        o2 = layer(q.to(dev), k.to(dev), v.to(dev))
    finally:
        reset_context_diffusion_lm()
    assert torch.equal(o1, o2)
    # the operator itself takes [Nq, Nq] only
    with pytest.raises(ValueError, match="n_tokens"):
        ops.sparse_decode_attention(q.view(-1, Hq, d).to(dev), k.view(-1, Hkv, d).to(dev), v.view(-1, Hkv, d).to(dev),
                                    layer.k_cache, layer.v_cache, bt.to(dev), cu, max_q_len=40, max_ctx_len=300,
                                    context_lens=common["context_lens"], mask_mode="dense", mask=wide.to(dev))
    # a mask that hides a context key cannot be honoured: refused, not ignored
    bad = masks[0].clone()
    bad[3, 10] = False
    with pytest.raises(ValueError, match="context"):
        set_context_diffusion_lm(False, seqs=[SimpleNamespace(current_block_mask=bad)], seq_lens=[lens[0]], **common)
    reset_context_diffusion_lm()


def test_seeded_random_shapes_and_plans(dev):
    """40 seeded random decode cases: head layouts from MHA to 32:1 GQA, 1-9 requests, chunk lengths that are not page or
    tile aligned, 1-200 active rows, bf16 and fp8 pages, full and causal active blocks, default and forced plans."""
    import random
    rnd = random.Random(20240)
    heads = [(28, 4), (32, 32), (8, 8), (16, 2), (4, 4), (32, 1), (12, 4)]
    for i in range(40):
        Hq, Hkv = rnd.choice(heads)
        n_chunks = rnd.randint(2, 10)
        q_len = rnd.choice([1, 7, 32, 33, 64, 96, 129, 160, 200])
        if Hq // Hkv * q_len > 2048:
            q_len = 32
        plan = rnd.choice([{}, {}, {}, dict(rows_per_group=rnd.choice([32, 64, 128, 256])),
                           dict(rows_per_group=128, num_splits=rnd.randint(1, 4)),
                           dict(rows_per_group=rnd.choice([64, 128, 256]), tiles_per_workgroup=rnd.randint(1, 9))])
        mode = rnd.choice(["full", "full", "causal"])
        case = configs.chunked_prefix_case(3000 + i, n_req=rnd.randint(1, 9), n_chunks=n_chunks,
                                           chunk_tokens=rnd.choice([17, 64, 100, 255, 256, 300, 513, 640]),
                                           topk=rnd.randint(1, n_chunks), q_len=q_len, Hq=Hq, Hkv=Hkv,
                                           fp8=rnd.random() < 0.3, shared_prefix=rnd.random() < 0.5)
        out = run_case(case, dev, mask_mode=mode, **plan)
        ref = oracle_case(case, mask_mode=mode)
        check(out, ref, what=f"case {i} {case.meta} plan {plan} mask {mode}")


def test_prefill_layer_replays_from_a_hip_graph(dev):
    """A prefill layer (rotary on Q and K with the paged store of K and V in one launch, then the chunk attention on
    the resident-workgroup kernel) captured once and replayed three times with new activations in the same buffers,
    with eager launches and synchronisations in between; every replay equals the eager result bit for bit and the
    pages hold the rotated keys of that replay."""
    ops = _ops()
    gen = torch.Generator().manual_seed(77)
    Hq, Hkv, dd, P = 28, 4, 128, 256
    lens = [700, 650, 600, 590, 1025, 129, 64, 1]
    n = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
    assert "attn_prefill_stream_kernel" in ops.describe_prefill_plan(len(lens), Hq, Hkv, max(lens), n, True)
    q = torch.empty(n, Hq, dd, dtype=torch.bfloat16, device=dev)
    k = torch.empty(n, Hkv, dd, dtype=torch.bfloat16, device=dev)
    v = torch.empty(n, Hkv, dd, dtype=torch.bfloat16, device=dev)
    out = torch.empty_like(q)
    pages = (n + P - 1) // P
    kc = torch.zeros(pages, P, Hkv, dd, dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    page_ids = torch.randperm(pages, generator=gen).to(torch.int32).to(dev)
    slots = ops.slot_mapping_from_pages(page_ids, n)
    pos = torch.cat([torch.arange(l) for l in lens]).to(dev)
    inv = 1.0 / (10000.0 ** (torch.arange(0, dd, 2).float() / dd))
    ang = torch.arange(max(lens)).float()[:, None] * inv[None, :]
    cos_sin = torch.cat([ang.cos(), ang.sin()], dim=-1).to(dev)

    def fill():
        q.copy_(torch.randn(q.shape, generator=gen).to(torch.bfloat16))
        k.copy_(torch.randn(k.shape, generator=gen).to(torch.bfloat16))
        v.copy_(torch.randn(v.shape, generator=gen).to(torch.bfloat16))

    def layer():
        ops.rope_qk_store(q, k, v, pos, cos_sin, kc, vc, slots)
        ops.chunk_prefill_attention(q, k, v, cu, max_seqlen=max(lens), causal=True, out=out)

    fill()
    q0, k0 = q.clone(), k.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer()                                  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    q.copy_(q0); k.copy_(k0)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer()
    for rep in range(3):
        fill()
        q_in, k_in = q.clone(), k.clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got, got_k, got_q = out.clone(), ops.kv_gather(kc, page_ids, n), q.clone()
        out.zero_(); kc.zero_()
        q.copy_(q_in); k.copy_(k_in)             # the rotation is in place: start again from the same activations
        layer()
        torch.cuda.synchronize()
        assert torch.equal(got_q, q) and torch.equal(got, out), rep
        assert torch.equal(got_k, ops.kv_gather(kc, page_ids, n)) and torch.equal(got_k, k), rep
    assert torch.isfinite(out.float()).all() and out.float().abs().max() > 0.1


def test_decode_step_replays_from_a_hip_graph(dev):
    """The library allocates nothing and never synchronises, so a denoise step (slot-table build + the layers'
    attention and merge launches) can be captured once and replayed: three replays with new queries and a new chunk
    selection written into the same buffers in between, each compared bit for bit with the eager launches."""
    ops = _ops()
    case = configs.config3_small(seed=21, n_req=3)
    d = lambda t: t.to(dev)
    rp, rs, rl, mr = (x.to(dev) if torch.is_tensor(x) else x for x in case.range_tensors())
    layers = 3
    gen = torch.Generator().manual_seed(5)
    qs = [d(case.q.clone()) for _ in range(layers)]
    table = ops.new_slot_table(3, case.max_ctx, dev)
    kc, vc, kn, vn, bt, qsl = d(case.k_cache), d(case.v_cache), d(case.k_new), d(case.v_new), d(case.block_table), d(case.q_start_loc)
    preps = [ops.PreparedAttention(qs[l], kn, vn, kc, vc, bt, qsl, max_q_len=case.max_q, max_ctx_len=case.max_ctx,
                                   ranges=(rp, rs, rl, mr), slot_table=table) for l in range(layers)]

    def step():
        preps[0].build_slot_table()
        for p in preps:
            p.run()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()                                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    starts = preps[0]._keep[7][1]                # the int32 range_start tensor the descriptors point at
    base_starts = starts.clone()
    for rep in range(3):
        for l in range(layers):
            qs[l].copy_((torch.randn(case.q.shape, generator=gen) / 11.3).to(torch.bfloat16))
        # another selection: rotate the chunk starts of every request
        for p in preps:
            p._keep[7][1].copy_(torch.roll(base_starts, rep + 1))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replayed = [p.out.clone() for p in preps]
        for p in preps:
            p.out.zero_()
        step()
        torch.cuda.synchronize()
        for l in range(layers):
            assert torch.equal(replayed[l], preps[l].out), (rep, l)
        # and the eager result is the oracle's for the current selection
        sel = p._keep[7][1].cpu().tolist()
        lens = rl.cpu().tolist()
        ptr = rp.cpu().tolist()
        ranges = [[(sel[i], lens[i]) for i in range(ptr[r], ptr[r + 1])] for r in range(3)]
        ref = ref_ops.sparse_decode_attention(qs[0].cpu(), case.k_new, case.v_new, case.k_cache, case.v_cache,
                                              case.block_table, case.q_start_loc, ranges)
        check(preps[0].out.float().cpu(), ref)


def test_seeded_random_ragged_requests_cut_ranges_and_dense_masks(dev):
    """30 seeded random cases on top of the shapes above: requests of different lengths, selections of different
    sizes, a range that starts inside a chunk, and random dense masks over the active rows."""
    import random
    rnd = random.Random(77)
    heads = [(28, 4), (32, 32), (8, 8), (16, 2), (4, 4), (32, 1), (12, 4)]
    for i in range(30):
        Hq, Hkv = rnd.choice(heads)
        n_req, n_chunks = rnd.randint(1, 7), rnd.randint(2, 8)
        q_len = rnd.choice([7, 32, 33, 64, 96, 129, 160])
        if Hq // Hkv * q_len > 2048:
            q_len = 32
        case = configs.chunked_prefix_case(5000 + i, n_req=n_req, n_chunks=n_chunks,
                                           chunk_tokens=rnd.choice([17, 100, 255, 256, 300, 513]),
                                           topk=rnd.randint(1, n_chunks), q_len=q_len, Hq=Hq, Hkv=Hkv,
                                           fp8=rnd.random() < 0.3, shared_prefix=rnd.random() < 0.5)
        lens = [rnd.randint(1, q_len) for _ in range(n_req)]
        keep = torch.cat([torch.arange(r * q_len, r * q_len + lens[r]) for r in range(n_req)])
        case.q, case.k_new, case.v_new = case.q[keep], case.k_new[keep], case.v_new[keep]
        case.q_start_loc = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
        for r in range(n_req):
            if rnd.random() < 0.5 and len(case.ranges[r]) > 1:
                case.ranges[r] = case.ranges[r][:rnd.randint(1, len(case.ranges[r]))]
            if rnd.random() < 0.3:
                a0, l0 = case.ranges[r][0]
                cut = rnd.randint(0, l0 - 1)
                case.ranges[r][0] = (a0 + cut, l0 - cut)
        mode, mask = rnd.choice(["full", "causal"]), None
        if rnd.random() < 0.4:
            n_tok = case.q.shape[0]
            mask = torch.rand(n_tok, n_tok, generator=torch.Generator().manual_seed(i)) < 0.6
            mask |= torch.eye(n_tok, dtype=torch.bool)
            mode = "dense"
        plan = rnd.choice([{}, {}, dict(rows_per_group=rnd.choice([32, 64, 128, 256])),
                           dict(rows_per_group=128, tiles_per_workgroup=rnd.randint(1, 9))])
        out = run_case(case, dev, mask_mode=mode, mask=mask, **plan)
        ref = oracle_case(case, mask_mode=mode, mask=mask)
        check(out, ref, what=f"case {i} lens {lens} plan {plan} mask {mode}")


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("plan", [dict(), dict(num_splits=1), dict(rows_per_group=256), dict(rows_per_group=32, num_splits=3)],
                         ids=["default", "unsplit", "wide", "split3"])
def test_active_rows_stored_inside_the_attention_call(dev, fp8, plan):
    """desc.active_slot_mapping: the call stores k_new / v_new like store_kvcache_unified_layout
    (attention_v4.py:328-331, OPS/kv_cache_kernels.py:150-172) and attends like the call without it.  The store is
    compared bit for bit with the separate store operator on a copy of the cache; rows with slot -1 are skipped and
    every other cache row stays as it was (with and without a merge launch, bf16 and fp8 pages)."""
    ops = _ops()
    case = configs.chunked_prefix_case(21, n_req=2, n_chunks=6, chunk_tokens=512, topk=3, q_len=40,
                                       shared_prefix=False, fp8=fp8, extra_pages=3)
    d = lambda t: None if t is None else t.to(dev)
    n_tok = case.q.shape[0]
    n_pages = case.k_cache.shape[0]
    used = set(case.block_table.flatten().tolist())
    free = [p for p in range(n_pages) if p not in used]
    assert len(free) >= 2
    slots = torch.cat([torch.arange(40, dtype=torch.int32) + free[r] * 256 + 7 for r in range(2)])
    slots[3] = -1
    slots[55] = -1
    rp, rs, rl, mr = case.range_tensors()
    kc, vc = d(case.k_cache), d(case.v_cache)
    kc2, vc2 = kc.clone(), vc.clone()
    args = (d(case.q), d(case.k_new), d(case.v_new))
    kw = dict(max_q_len=case.max_q, max_ctx_len=case.max_ctx, ranges=(d(rp), d(rs), d(rl), mr),
              k_scale=d(case.k_scale), v_scale=d(case.v_scale), **plan)
    plain = ops.sparse_decode_attention(*args, kc2, vc2, d(case.block_table), d(case.q_start_loc), **kw)
    ops.store_kvcache_unified_layout(args[1], args[2], kc2, vc2, d(slots), k_scale=d(case.k_scale), v_scale=d(case.v_scale))
    fused = ops.sparse_decode_attention(*args, kc, vc, d(case.block_table), d(case.q_start_loc),
                                        active_slot_mapping=d(slots), **kw)
    torch.cuda.synchronize()
    assert torch.equal(fused, plain)
    as_bits = lambda t: t.view(torch.uint8) if t.dtype != torch.bfloat16 else t.view(torch.int16)
    assert torch.equal(as_bits(kc), as_bits(kc2)) and torch.equal(as_bits(vc), as_bits(vc2))
    assert not torch.equal(as_bits(kc), as_bits(d(case.k_cache)))          # something was stored
    check(fused.float().cpu(), oracle_case(case))
    with pytest.raises(ValueError):
        ops.sparse_decode_attention(*args, kc, vc, d(case.block_table), d(case.q_start_loc),
                                    active_slot_mapping=d(slots[:-1]), **kw)
