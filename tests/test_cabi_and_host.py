"""CPU-only checks: the C-ABI library loads and exports every symbol include/pdllm.h declares, error
codes map to the reference's exception classes, and the host-side mirrors (allocator, record types)
behave like the reference.  No kernel is launched here."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pdllm.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pdllm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from prefilling_dllm_amd import _lib
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(_lib.lib, n), f"{n} declared in pdllm.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert _lib.lib.pdllm_abi_version() == 5
    assert _lib.lib.pdllm_status_string(0) == b"ok"


def test_header_compiles_as_c():
    """The boundary is a plain C header: no C++ or HIP types in the signatures."""
    src = '#include "pdllm.h"\nint main(void){ pdllm_attn_desc d; (void)d; return PDLLM_OK; }\n'
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-I", os.path.dirname(HEADER), "-x", "c",
                        "-"], input=src.encode(), capture_output=True)
    assert r.returncode == 0, r.stderr.decode()


def test_struct_mirror_matches_header_layout():
    """sizeof(pdllm_attn_desc) as the C compiler sees it == the ctypes mirror."""
    from prefilling_dllm_amd import _lib
    src = '#include <stdio.h>\n#include "pdllm.h"\nint main(void){ printf("%zu %zu %zu", sizeof(pdllm_attn_desc), ' \
          '__builtin_offsetof(pdllm_attn_desc, q_stride), __builtin_offsetof(pdllm_attn_desc, sm_scale)); return 0; }\n'
    exe = "/tmp/pdllm_sizeof"
    r = subprocess.run(["gcc", "-I", os.path.dirname(HEADER), "-x", "c", "-", "-o", exe], input=src.encode(),
                       capture_output=True)
    assert r.returncode == 0, r.stderr.decode()
    size, off_q, off_s = map(int, subprocess.check_output([exe]).split())
    assert ctypes.sizeof(_lib.AttnDesc) == size
    assert _lib.AttnDesc.q_stride.offset == off_q and _lib.AttnDesc.sm_scale.offset == off_s


def test_status_codes_map_to_reference_exception_classes():
    from prefilling_dllm_amd import _lib
    _lib.check(0, "x")
    for code, exc in ((-1, ValueError), (-2, ValueError), (-3, ValueError), (-5, RuntimeError), (-7, NotImplementedError)):
        with pytest.raises(exc):
            _lib.check(code, "x")


def test_argument_errors_are_reported_without_a_gpu():
    """Validation happens on the host before any launch: NULL pointers and bad shapes return codes."""
    from prefilling_dllm_amd import _lib
    lib = _lib.lib
    assert lib.pdllm_kv_store(None, None, None, None, None, 1, 512, 512, 512, 10, None) == -1
    assert lib.pdllm_topk_lowest_index(None, 1, 4, 4, 2, 1, None, None) == -1
    assert lib.pdllm_attn_workspace_bytes(None) == -1
    d = _lib.AttnDesc()
    assert lib.pdllm_sparse_decode_attn(ctypes.byref(d), None) == -1
    buf = (ctypes.c_char * 64)()
    p = (ctypes.addressof(buf) + 15) & ~15
    d.q = d.k_new = d.v_new = d.out = d.q_start_loc = p
    d.head_dim, d.num_q_heads, d.num_kv_heads = 64, 4, 4
    assert lib.pdllm_sparse_decode_attn(ctypes.byref(d), None) == -7            # head_dim != 128
    d.head_dim, d.num_q_heads, d.num_kv_heads = 128, 6, 4
    assert lib.pdllm_sparse_decode_attn(ctypes.byref(d), None) == -2            # heads not divisible
    assert lib.pdllm_selfinfo_logprob(p, 10, p, 1, 100, p, 1 << 20, p, None) == -2   # stride < vocab
    assert lib.pdllm_vocab_workspace_bytes(128, 152064) > 0
    ada = lib.pdllm_anchor_delta_add
    big = (ctypes.c_char * 256)()
    o = (ctypes.addressof(big) + 15) & ~15
    assert ada(None, 128, p, 128, None, 0, 0, None, o, 128, p, 1, 4, 4, 128, 4, 3, 3, 0, 0, 1.0, 1.0, 0, None) == -1
    assert ada(p, 128, None, 128, None, 0, 0, None, o, 128, p, 1, 4, 4, 128, 4, 3, 3, 0, 0, 1.0, 1.0, 0, None) == -1  # no dense
    assert ada(p, 128, p, 128, None, 0, 0, None, o, 128, p, 1, 4, 4, 128, 4, 4, 3, 0, 0, 1.0, 1.0, 0, None) == -2   # offset >= stride
    assert ada(p, 128, p, 128, None, 0, 0, None, o, 128, p, 1, 4, 4, 100, 4, 3, 3, 0, 0, 1.0, 1.0, 0, None) == -2   # row_elems % 8
    assert ada(p, 128, p, 128, None, 0, 0, None, p, 128, p, 1, 4, 4, 128, 4, 3, 3, 0, 0, 1.0, 1.0, 0, None) == -3   # out aliases base
    assert ada(p, 128, p, 128, p, 128, 4, None, o, 128, p, 2, 4, 8, 128, 4, 3, 3, 0, 0, 1.0, 1.0, 2, None) == -7    # selection, 2 sequences
    assert ada(p, 128, p, 128, None, 0, 0, None, o, 128, p, 0, 4, 0, 128, 4, 3, 3, 0, 0, 1.0, 1.0, 0, None) == 0    # nothing to do


def test_store_only_descriptor_needs_aligned_cache():
    """A decode call without a visible prefix that still stores its active rows (active_slot_mapping set,
    max_ctx_len 0) writes 16 bytes per lane (8 of fp8 bytes): a cache base that is not aligned to that is refused on
    the host, as it is when a prefix is read."""
    from prefilling_dllm_amd import _lib
    lib = _lib.lib
    buf = (ctypes.c_char * 256)()
    p = (ctypes.addressof(buf) + 63) & ~63
    d = _lib.AttnDesc()
    d.q = d.k_new = d.v_new = d.out = d.q_start_loc = d.active_slot_mapping = p
    d.head_dim, d.num_q_heads, d.num_kv_heads = 128, 28, 4
    d.q_stride = d.o_stride = 28 * 128
    d.kn_stride = d.vn_stride = 4 * 128
    d.n_tokens, d.n_req, d.max_q_len, d.max_ctx_len = 32, 1, 32, 0
    d.mask_mode, d.sm_scale = _lib.MASK_FULL, 0.088
    d.kv_dtype, d.page_size, d.n_pages = _lib.KV_BF16, 256, 2
    d.cache_head_stride, d.cache_token_stride, d.cache_page_stride = 128, 512, 512 * 256
    d.k_cache = d.v_cache = p
    assert lib.pdllm_attn_workspace_bytes(ctypes.byref(d)) >= 0
    d.k_cache = p + 8
    assert lib.pdllm_attn_workspace_bytes(ctypes.byref(d)) == -3
    d.kv_dtype = _lib.KV_FP8_E4M3                      # fp8 rows: 8-byte stores
    d.k_scale = d.v_scale = p
    assert lib.pdllm_attn_workspace_bytes(ctypes.byref(d)) >= 0
    d.k_cache = p + 4
    assert lib.pdllm_attn_workspace_bytes(ctypes.byref(d)) == -3


def test_attention_plan_is_host_only():
    from prefilling_dllm_amd import ops
    rows, splits = ops.attention_plan(8, 28, 4, max_q_len=160, max_ctx_len=4096)
    assert rows in (32, 64, 128, 160, 192, 256) and splits >= 1
    rows, splits = ops.attention_plan(1, 28, 4, max_q_len=32, max_ctx_len=32768)
    assert splits > 1                                                            # few rows, long prefix: split KV
    assert ops.attention_plan(8, 28, 4, max_q_len=160, max_ctx_len=4096, rows_per_group=128, num_splits=2) == (128, 2)


def _decode_desc(n_req, q_len, ctx, hq=28, hkv=4, fp8=False):
    """A decode descriptor over a paged cache with made-up (non-NULL, aligned) addresses: the planner and the
    validation only read sizes and strides."""
    import torch
    from prefilling_dllm_amd import _lib
    dummy = torch.empty(64, dtype=torch.int32)
    a = (dummy.data_ptr() + 15) & ~15
    d = _lib.AttnDesc()
    for f in ("q", "k_new", "v_new", "out", "q_start_loc", "k_cache", "v_cache", "block_table", "range_ptr",
              "range_start", "range_len"):
        setattr(d, f, a)
    if fp8:
        d.k_scale = d.v_scale = a
    d.q_stride = d.o_stride = hq * 128
    d.kn_stride = d.vn_stride = hkv * 128
    d.cache_head_stride, d.cache_token_stride, d.cache_page_stride = 128, hkv * 128, 256 * hkv * 128
    d.n_tokens, d.n_pages, d.bt_stride, d.page_size = n_req * q_len, 4096, 1024, 256
    d.n_req, d.max_q_len, d.max_ctx_len, d.max_ranges = n_req, q_len, ctx, 16
    d.num_q_heads, d.num_kv_heads, d.head_dim = hq, hkv, 128
    d.kv_dtype = _lib.KV_FP8_E4M3 if fp8 else _lib.KV_BF16
    d.sm_scale = 128 ** -0.5
    return d


def _plan_text(desc):
    from prefilling_dllm_amd import _lib
    buf = ctypes.create_string_buffer(256)
    _lib.check(_lib.lib.pdllm_attn_plan_describe(ctypes.byref(desc), 0, buf, 256), "plan")
    return dict(kv.split("=") for kv in buf.value.decode().split()[1:]), buf.value.decode().split()[0]


def test_planner_lays_out_the_set_cut_without_a_gpu():
    """The cut of the benchmark's decode step (8 requests x 160 rows x 7 heads per KV head over 4096 + 160 keys, 256
    compute units assumed without a device): 16 workgroups per (request, KV head), nine of them on the leading 40
    tiles of one row group each, the other seven on spans of 36 tiles of the nine tails of 27 -- every third cut
    falls on the end of a column, so no workgroup has more than two pieces and no row more than three."""
    f, kernel = _plan_text(_decode_desc(8, 160, 4096))
    assert kernel == "attn_fwd_kernel" and f["kv"] == "bf16" and f["row_blocks"] == "4"
    assert (f["grid"], f["set"], f["head"], f["span"], f["tiles"], f["pieces"]) == ("512", "16", "40", "36", "67", "3")
    assert f["partial_row_bytes"] == "276"
    head, span, tiles, rt, k = 40, 36, 67, 9, 16
    tail = tiles - head
    loads = [(min(a + span, rt * tail) - a, (min(a + span, rt * tail) - 1) // tail - a // tail + 1)
             for a in range(0, rt * tail, span)]
    assert len(loads) == k - rt and max(p for _, p in loads) == 2 and sum(p for _, p in loads) == 13
    # 32 response rows only: the 224 rows of a (request, KV head) are two row groups, each cut into eight aligned
    # pieces (two workgroups per CU); the eight-wave kernel on request
    f, kernel = _plan_text(_decode_desc(8, 32, 4096))
    assert kernel == "attn_fwd_kernel" and (f["row_blocks"], f["grid"], f["span"], f["head"], f["pieces"]) == ("4", "512", "9", "0", "8")
    d = _decode_desc(8, 32, 4096)
    d.rows_per_group = 256
    f, kernel = _plan_text(d)
    assert kernel == "attn_fwd2_kernel" and (f["row_blocks"], f["grid"], f["span"], f["head"]) == ("8", "256", "9", "0")
    # fp8 pages, 160 rows per head: one group of five row blocks, two aligned pieces
    f, kernel = _plan_text(_decode_desc(4, 160, 16 * 1025, hq=32, hkv=32, fp8=True))
    assert kernel == "attn_fwd_kernel" and (f["kv"], f["row_blocks"], f["grid"], f["pieces"]) == ("fp8", "5", "256", "2")
    # one workgroup per column when the columns fill the chip: no partial rows
    f, _ = _plan_text(_decode_desc(64, 128, 1024))
    assert f["pieces"] == "1" and f["partial_row_bytes"] == "0"


def test_remembered_plans_equal_fresh_ones():
    """The library remembers the last eight plans per host thread.  More shapes than that, visited twice in an order
    that evicts every entry in between, and from a second thread: every answer equals the first one."""
    import threading
    shapes = [(n, q, c, hq, hkv, fp8) for n in (1, 3, 8) for q in (32, 160) for c in (1024, 4096)
              for hq, hkv, fp8 in ((28, 4, False), (32, 32, True))]
    assert len(shapes) > 8
    first = [_plan_text(_decode_desc(n, q, c, hq=hq, hkv=hkv, fp8=fp8)) for n, q, c, hq, hkv, fp8 in shapes]
    assert len({str(x) for x in first}) > 8          # the shapes really have different plans
    again = [_plan_text(_decode_desc(n, q, c, hq=hq, hkv=hkv, fp8=fp8)) for n, q, c, hq, hkv, fp8 in shapes]
    assert again == first
    for n, q, c, hq, hkv, fp8 in shapes[:3]:         # the same shape back to back: served from the memory
        d = _decode_desc(n, q, c, hq=hq, hkv=hkv, fp8=fp8)
        assert _plan_text(d) == _plan_text(d)
        d.rows_per_group = 128                       # a forced field is part of the key
        forced = _plan_text(d)
        d.rows_per_group = 0
        assert _plan_text(d) == first[shapes.index((n, q, c, hq, hkv, fp8))] and forced[0]["row_blocks"] == "4"
    other = []
    t = threading.Thread(target=lambda: other.extend(
        _plan_text(_decode_desc(n, q, c, hq=hq, hkv=hkv, fp8=fp8)) for n, q, c, hq, hkv, fp8 in shapes))
    t.start(); t.join()
    assert other == first


def test_page_pool_semantics():
    """What callers of the reference's allocator observe (fastdllm_engine.py:88-167): pages are handed out in the
    order they became free, refcounts, the exhaustion error, hash-keyed prefix reuse and eviction."""
    from prefilling_dllm_amd.page_pool import PageAllocator, PagePool, prompt_digest
    from prefilling_dllm_amd import engine_ops
    import torch
    assert engine_ops.PrefixPageAllocator is PagePool
    a = PagePool(4, 256)
    assert isinstance(a, PageAllocator)
    p = a.allocate_pages(3)
    assert p == [0, 1, 2] and a.num_free_pages == 1
    with pytest.raises(RuntimeError, match="Cannot allocate 2 pages, only 1 free"):
        a.allocate_pages(2)
    assert a.num_free_pages == 1                                      # all or nothing
    a.ref_pages([1])
    a.release_pages([0, 1])
    assert a.num_free_pages == 2 and a.page_ref_count[1] == 1        # page 1 still referenced
    a.release_pages([1])
    assert list(a.free_pages) == [3, 0, 1]
    with pytest.raises(RuntimeError, match="released more often"):
        a.release_pages([3])
    ids = [5, 6, 7]
    e = a.register_prefix(ids, [2], 3, torch.zeros(4))
    assert a.lookup_prefix(ids) is e and a.lookup_prefix([5, 6]) is None
    assert a.compute_prompt_hash(ids) == prompt_digest(tuple(ids))
    # the digest is xxh64 over the ids as little-endian int64 (known answer: the empty prompt, and one id)
    import xxhash
    assert prompt_digest([]) == 0xEF46DB3751D8E999
    assert prompt_digest([1]) == xxhash.xxh64((1).to_bytes(8, "little")).intdigest()
    e.ref_count = 1
    assert not a.evict_one()
    a.release_prefix(ids)
    assert a.evict_one() and a.lookup_prefix(ids) is None and a.num_free_pages == 4
    assert list(a.free_pages) == [3, 0, 1, 2]
    assert a.allocate_pages(4) == [3, 0, 1, 2] and a.num_free_pages == 0 and list(a.free_pages) == []
    a.release_pages([1])
    assert list(a.free_pages) == [1]


def test_page_pool_edge_cases():
    """Nothing asked for is nothing done (the reference returns [] for n <= 0, fastdllm_engine.py:112-119), and a
    release that must be refused leaves the pool as it was."""
    from prefilling_dllm_amd.page_pool import PagePool
    a = PagePool(4, 256)
    assert a.allocate_pages(0) == [] and a.allocate_pages(-2) == [] and a.num_free_pages == 4
    assert list(a.free_pages) == [0, 1, 2, 3]
    p = a.allocate_pages(3)                                       # [0, 1, 2], one holder each
    a.ref_pages([1])
    before = (a.num_free_pages, list(a.free_pages), [a.page_ref_count[i] for i in range(4)])
    with pytest.raises(RuntimeError, match="released more often"):
        a.release_pages([0, 1, 1, 1])                             # page 1 has two holders, three are dropped
    with pytest.raises(RuntimeError, match="released more often"):
        a.release_pages([2, 2])
    with pytest.raises(RuntimeError, match="not all pages of this pool"):
        a.release_pages([0, 7])
    assert (a.num_free_pages, list(a.free_pages), [a.page_ref_count[i] for i in range(4)]) == before
    a.release_pages([])                                           # nothing listed
    a.release_pages([1, 1, 0])                                    # a page listed twice drops two holders
    assert list(a.free_pages) == [3, 1, 0] and p == [0, 1, 2]


def test_normalised_keep_indices_are_taken_as_one_stack():
    """What normalize_per_head_keep_indices returns is a list of slices of one [L, H, n] tensor; the compaction
    recognises that and uses the tensor as it is.  Anything else (copies, another order, another dtype) is stacked."""
    import torch
    from prefilling_dllm_amd.engine_ops import _as_one_stack, normalize_per_head_keep_indices as norm
    given = [torch.randint(0, 50, (3, 7)) for _ in range(4)]
    views, n = norm(given, num_layers=4, num_heads=3, full_prompt_len=50, device="cpu")
    one = _as_one_stack(views, "cpu")
    assert n == 7 and one is not None and one.shape == (4, 3, 7) and torch.equal(one, torch.stack(given))
    assert one.data_ptr() == views[0].data_ptr()
    assert _as_one_stack(given, "cpu") is None                                # separate tensors
    assert _as_one_stack([views[1], views[0], views[2], views[3]], "cpu") is None   # not in layer order
    assert _as_one_stack([v.to(torch.int32) for v in views], "cpu") is None
    assert _as_one_stack([v.t() for v in views], "cpu") is None


def test_normalize_per_head_keep_indices_contract():
    """_normalize_per_head_keep_indices (fastdllm_engine.py:560-605): one [heads, n] index tensor per layer, one
    common n, entries inside the prompt; the error names the first offending layer."""
    import torch
    from prefilling_dllm_amd.engine_ops import normalize_per_head_keep_indices as norm
    kw = dict(num_layers=3, num_heads=2, full_prompt_len=10, device="cpu")
    good = [[[0, 3, 9], [1, 2, 3]], torch.tensor([[4, 5, 6], [7, 8, 9]], dtype=torch.int32), [[0, 1, 2], [0, 1, 2]]]
    out, n = norm(good, **kw)
    assert n == 3 and len(out) == 3 and all(t.dtype == torch.int64 and t.is_contiguous() for t in out)
    assert out[1].tolist() == [[4, 5, 6], [7, 8, 9]]
    assert norm([], num_layers=0, num_heads=2, full_prompt_len=10, device="cpu") == ([], 0)
    empty, n0 = norm([torch.zeros(2, 0, dtype=torch.long)] * 3, **kw)
    assert n0 == 0 and len(empty) == 3
    with pytest.raises(ValueError, match="2 layers"):
        norm(good[:2], **kw)
    with pytest.raises(ValueError, match="layer 1"):
        norm([good[0], [[1, 2, 3]], good[2]], **kw)                      # one head instead of two
    with pytest.raises(ValueError, match="layer 2"):
        norm([good[0], good[1], [[0, 1], [0, 1]]], **kw)                 # another active length
    with pytest.raises(ValueError, match="layer 0"):
        norm([[0, 1, 2], good[1], good[2]], **kw)                        # not two-dimensional
    with pytest.raises(ValueError, match="layer 1.*outside the prompt of 10"):
        norm([good[0], [[4, 5, 10], [7, 8, 9]], [[0, 1, -1], [0, 1, 2]]], **kw)
    with pytest.raises(ValueError, match="layer 2.*outside"):
        norm([good[0], good[1], [[0, 1, -1], [0, 1, 2]]], **kw)


def test_active_block_mask_from_per_sequence_masks():
    """Per-sequence masks [h, ctx + h] (engine/sequence.py:489-493) -> the block-diagonal [Nq, Nq] mask over the
    active keys that utils/context.py:73-98 lays out, None when nothing is hidden; a hidden context key is refused."""
    import torch
    from prefilling_dllm_amd.context import active_block_mask, ContextForDiffusionLM
    from types import SimpleNamespace
    assert active_block_mask([]) is None
    full = [torch.ones(1, 1, 3, 8, dtype=torch.bool), torch.ones(2, 2, dtype=torch.bool)]
    assert active_block_mask(full) is None
    a = torch.ones(3, 8, dtype=torch.bool)
    a[0, 6:] = False                                   # row 0 does not see active keys 1, 2
    b = torch.tensor([[1, 0], [1, 1]], dtype=torch.bool)
    got = active_block_mask([a.view(1, 1, 3, 8), b])
    want = torch.zeros(5, 5, dtype=torch.bool)
    want[:3, :3] = a[:, 5:]
    want[3:, 3:] = b
    assert torch.equal(got, want)
    hidden_ctx = torch.ones(3, 8, dtype=torch.bool)
    hidden_ctx[1, 2] = False
    with pytest.raises(ValueError, match="hides cached context keys"):
        active_block_mask([hidden_ctx])
    with pytest.raises(ValueError, match="only 2 key columns"):
        active_block_mask([torch.ones(3, 2, dtype=torch.bool)])
    # the context assembles it from its sequences, as the reference's __post_init__ does
    ctx = ContextForDiffusionLM(seqs=[SimpleNamespace(current_block_mask=a), SimpleNamespace(current_block_mask=b)])
    assert ctx.mask_kind == "dense" and torch.equal(ctx.block_mask, want)
    ctx = ContextForDiffusionLM(seqs=[SimpleNamespace(current_block_mask=m) for m in full])
    assert ctx.block_mask is None and ctx.mask_kind == "full"


def test_record_helpers_take_any_allocator():
    """The PD record helpers only use allocate_pages / release_pages / evict_one / num_free_pages."""
    from prefilling_dllm_amd import engine_ops as eo

    class Counting:
        def __init__(self):
            self.free, self.log = list(range(10)), []
        num_free_pages = property(lambda self: len(self.free))
        def allocate_pages(self, n):
            out, self.free = self.free[:n], self.free[n:]
            return out
        def release_pages(self, pages):
            self.log.append(list(pages)); self.free += list(pages)
        def evict_one(self):
            return False

    a = Counting()
    prompt, block = eo._allocate_record_pages(a, 600, 32, 256)
    assert prompt == [0, 1, 2] and block == [3]
    rec = eo.DreamPrefillRecord([], [], [], 600, 600, 32, prompt, block, 0, None, None, True)
    eo.release_pd_record(a, rec)
    assert a.log == [[3], [0, 1, 2]]


def test_record_types_keep_the_reference_fields():
    from prefilling_dllm_amd import engine_ops as e
    import dataclasses
    assert [f.name for f in dataclasses.fields(e.DreamPrefillRecord)] == [
        "prompt_ids", "prompt_positions", "suffix_positions", "prompt_len", "full_prompt_len", "decode_len",
        "prompt_page_ids", "block_page_ids", "first_token_id", "last_context_logit", "decode_delta_state",
        "owns_prompt_pages", "cached_prefix", "kv_mode"]
    assert [f.name for f in dataclasses.fields(e.DreamKVSnapshot)] == [
        "prompt_len", "page_size", "kv_mode", "k_by_layer", "v_by_layer", "last_context_logit"]
    assert [f.name for f in dataclasses.fields(e.FastDLLMEngineOutput)] == ["text", "token_ids", "n_diff_steps"]


def test_product_path_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "prefilling-dllm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("# oracle", ""), f"{f} mentions the oracle"


def test_rotary_position_modes_follow_the_reference_formulas():
    """fastdllm_parallelcomp.py:919-948: the three chunk modes, the two chunk-query modes and the three final
    query modes, on values a wrong branch or a swapped argument would change."""
    from prefilling_dllm_amd import engine_ops as eo
    assert eo.chunk_rope_start("reuse", 7, 3, 9, 1025) == 7
    assert eo.chunk_rope_start("continuous", 7, 3, 9, 1025) == 7 + 3 * 1025
    assert eo.chunk_rope_start("absolute", 7, 3, 9, 1025) == 7 + 9 * 1025
    assert eo.chunk_rope_start("continuous", 7, 3, 9, 0) == 10          # chunk_size 0 counts as 1
    assert eo.chunk_query_rope_start("after_reused_window", 7, 100, 50, 1025) == 7 + 1025
    assert eo.chunk_query_rope_start("after_chunk", 7, 100, 50, 1025) == 150
    assert eo.final_query_rope_start("after_reused_window", 7, [1, 2], 8, 1025) == 7 + 1025
    assert eo.final_query_rope_start("after_selected_chunks", 7, [1, 2], 8, 1025) == 7 + 8 * 1025
    assert eo.final_query_rope_start("after_cache", 7, [3, 40, 12], 8, 1025) == 41
    assert eo.final_query_rope_start("after_cache", 7, [], 8, 1025) == 7
    for fn, args in ((eo.chunk_rope_start, ("x", 0, 0, 0, 1)), (eo.chunk_query_rope_start, ("x", 0, 0, 0, 1)),
                     (eo.final_query_rope_start, ("x", 0, [], 0, 1))):
        with pytest.raises(ValueError):
            fn(*args)
    pos = eo.chunk_positions("absolute", 2, [3, 2], [5, 1], 10)
    assert pos.tolist() == [52, 53, 54, 12, 13]


def test_split_token_chunks_cases():
    """Chunking of the prompt (fastdllm_parallelcomp.py:158-180): hand-listed cases and the oracle on a sweep."""
    from oracle import ref_ops
    from prefilling_dllm_amd import engine_ops
    f = engine_ops.split_token_chunks
    assert f([], 4) == []
    assert f([1, 2, 3], 4) == [[1, 2, 3]] and f([1, 2, 3], 0) == [[1, 2, 3]] and f([1, 2, 3], -2) == [[1, 2, 3]]
    assert f(range(10), 4) == [[0, 1, 2, 3], [4, 5, 6, 7], [8, 9]]
    assert f(range(10), 4, split_from_tail=True) == [[0, 1], [2, 3, 4, 5], [6, 7, 8, 9]]
    assert f(range(8), 4, split_from_tail=True) == [[0, 1, 2, 3], [4, 5, 6, 7]]
    for n in range(0, 40):
        for c in (1, 2, 3, 7, 16):
            for tail in (False, True):
                assert f(range(n), c, tail) == ref_ops.split_token_chunks(range(n), c, tail)


def test_anchor_params_follow_the_reference_defaults_and_clamps():
    """ops.anchor_params (attention_v4.py:113-125) against the oracle's anchor list for the same state."""
    from oracle import ref_ops
    from prefilling_dllm_amd import ops
    states = [{}, dict(stride=2), dict(stride=0, left=0), dict(anchor_offset=-3), dict(anchor_offset=99),
              dict(stride=5, anchor_offset=1, left=7, right=2, direction="both"), dict(direction="RIGHT", right=3),
              dict(direction=None), dict(stride=8, left=-4, right=-1)]
    for st in states:
        for seq_len in (1, 3, 4, 9, 33):
            anchors, windows = ref_ops.anchor_windows(seq_len, st)
            got = ops.anchor_params(st, seq_len)
            if not anchors:
                assert got is None, (st, seq_len)
                continue
            stride, offset, left, right, direction = got
            assert list(range(offset, seq_len, stride)) == anchors, (st, seq_len)
            for a, rows in zip(anchors, windows):
                lo = a - (left if direction in (0, 2) else 0)
                hi = a + (right if direction in (1, 2) else 0)
                assert rows == list(range(max(0, lo), min(seq_len - 1, hi) + 1)), (st, seq_len, a)


def test_assemble_global_keep_indices_against_the_oracle():
    """engine_ops.assemble_global_keep_indices (fastdllm_engine.py:1524-1546) on random spans and keep lists."""
    import random
    import torch
    from oracle import ref_ops
    from prefilling_dllm_amd import engine_ops as eo
    rng = random.Random(5)
    for case in range(20):
        L, H, n = rng.randint(1, 3), rng.randint(1, 4), rng.randint(8, 60)
        cuts = sorted(rng.sample(range(n + 1), rng.randint(2, 6)))
        spans = [(a, b) for a, b in zip(cuts[:-1], cuts[1:]) if rng.random() < 0.7 and b > a] or [(cuts[0], cuts[1])]
        layers = []
        for layer in range(L):
            if rng.random() < 0.2:
                layers.append([])
                continue
            parts = []
            for a, b in spans:
                k = rng.randint(1, b - a)
                parts.append(torch.tensor([sorted(rng.sample(range(a, b), k)) for _ in range(H)], dtype=torch.int64))
            layers.append(parts)
        ref = ref_ops.assemble_global_keep_indices([[p.tolist() for p in parts] for parts in layers], spans, n, H)
        got = eo.assemble_global_keep_indices(layers, spans, n, H)
        assert got == ref, case
        tens = eo.assemble_global_keep_indices(layers, [{"start": a, "end": b} for a, b in spans], n, H, as_lists=False)
        assert [t.tolist() for t in tens] == ref
    with pytest.raises(ValueError):
        eo.assemble_global_keep_indices([[torch.zeros(2, 1, dtype=torch.int64)]], [(0, 1), (1, 2)], 4, 2)
