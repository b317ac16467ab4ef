"""GPU parity of the experimental anchor corrections (decode delta, sparse prefill) against the oracle."""
import pytest
import torch

from oracle import ref_ops

pytestmark = pytest.mark.gpu


def _bf16_reference(base, dense, state, sel=None, counts=None, mode="none"):
    """The reference's tensor operations on bf16 tensors (attention_v4.py:139-166, 263-293)."""
    S = base.shape[0]
    anchors, windows = ref_ops.anchor_windows(S, state)
    at = torch.tensor(anchors, dtype=torch.long)
    base_anchor = base[at]
    scale = float(state.get("scale", 1.0))
    sel_anchor = valid = None
    if mode != "none":
        in_range = at < sel.shape[0]
        safe = at.clamp_max(sel.shape[0] - 1)
        sel_anchor = torch.zeros_like(base_anchor)
        sel_anchor[in_range] = sel[safe][in_range]
        valid = ((counts[safe] > 0) & in_range) if counts is not None else in_range
    if mode == "replace":
        delta = (sel_anchor - base_anchor) * scale
        delta = delta * valid.view(-1, 1, 1).to(delta.dtype)
    else:
        delta = (dense[at] - base_anchor) * scale
        if mode == "add":
            sd = (sel_anchor - dense[at]) * float(state.get("selection_scale", 1.0))
            delta = delta + sd * valid.view(-1, 1, 1).to(sd.dtype)
    return ref_ops.anchor_delta_add(base, delta, windows)


@pytest.mark.parametrize("state", [
    {}, dict(scale=0.37), dict(direction="right", right=2), dict(direction="both", left=1, right=1),
    dict(stride=2, left=5, scale=1.3), dict(stride=1, left=0), dict(anchor_offset=0), dict(stride=7, left=2, right=9, direction="both"),
])
def test_anchor_delta_add_same_bits_as_bf16_tensor_ops(dev, state):
    from prefilling_dllm_amd import ops
    gen = torch.Generator().manual_seed(3)
    S, H, d = 45, 6, 128
    base = torch.randn(S, H, d, generator=gen).to(torch.bfloat16)
    dense = (base.float() + 0.3 * torch.randn(S, H, d, generator=gen)).to(torch.bfloat16)
    sel = (base.float() + 0.3 * torch.randn(S, H, d, generator=gen)).to(torch.bfloat16)[:30]
    counts = torch.randint(0, 2, (30,), generator=gen)
    qsl = torch.tensor([0, S], dtype=torch.int32, device=dev)
    stride, offset, left, right, direction = ops.anchor_params(state, S)
    kw = dict(max_q_len=S, stride=stride, anchor_offset=offset, left=left, right=right, direction=direction,
              scale=float(state.get("scale", 1.0)))
    got = ops.anchor_delta_add(base.to(dev), dense.to(dev), qsl, **kw).cpu()
    assert torch.equal(got, _bf16_reference(base, dense, state))
    st2 = dict(state, selection_scale=0.6)
    for mode, cnt in (("add", counts), ("add", None), ("replace", counts), ("replace", None)):
        got = ops.anchor_delta_add(base.to(dev), None if mode == "replace" else dense.to(dev), qsl, sel=sel.to(dev),
                                   sel_counts=None if cnt is None else cnt.to(dev), sel_scale=0.6, sel_mode=mode, **kw).cpu()
        assert torch.equal(got, _bf16_reference(base, dense, st2, sel, cnt, mode)), (mode, cnt is None)


def test_anchor_delta_add_per_sequence_and_errors(dev):
    from prefilling_dllm_amd import ops
    gen = torch.Generator().manual_seed(4)
    lens = [9, 1, 14, 3]
    S, H, d = sum(lens), 2, 64
    base = torch.randn(S, H, d, generator=gen).to(torch.bfloat16)
    dense = torch.randn(S, H, d, generator=gen).to(torch.bfloat16)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    got = ops.anchor_delta_add(base.to(dev), dense.to(dev), cu.to(dev), max_q_len=max(lens), stride=4, anchor_offset=3,
                               left=3, right=0, direction=0).cpu()
    for a, b in zip(cu[:-1].tolist(), cu[1:].tolist()):
        assert torch.equal(got[a:b], _bf16_reference(base[a:b], dense[a:b], {}))
    with pytest.raises(ValueError):      # dense missing without a replacing selection
        ops.anchor_delta_add(base.to(dev), None, cu.to(dev), max_q_len=14, stride=4, anchor_offset=3, left=3, right=0,
                             direction=0)
    with pytest.raises(ValueError):      # anchor offset outside the stride
        ops.anchor_delta_add(base.to(dev), dense.to(dev), cu.to(dev), max_q_len=14, stride=4, anchor_offset=4, left=3,
                             right=0, direction=0)
    with pytest.raises(NotImplementedError):  # selection rows are per sequence
        ops.anchor_delta_add(base.to(dev), dense.to(dev), cu.to(dev), max_q_len=14, stride=4, anchor_offset=3, left=3,
                             right=0, direction=0, sel=dense.to(dev), sel_mode="add")


def _layer(dev, Hq, Hkv, d):
    from prefilling_dllm_amd.attention import Attention
    layer = Attention(Hq, d, d ** -0.5, Hkv, "diffusion_lm")
    layer.layer_idx = 1
    return layer


@pytest.mark.parametrize("state", [dict(enabled=True), dict(enabled=True, stride=2, left=1, scale=0.5, debug=True),
                                   dict(enabled=True, direction="both", left=2, right=2)])
def test_decode_delta_layer(dev, state):
    """Decode step against a sparse prefix (every other 64-token chunk) with the delta towards the full prompt."""
    from prefilling_dllm_amd.context import set_context_diffusion_lm, reset_context_diffusion_lm
    gen = torch.Generator().manual_seed(8)
    Hq, Hkv, d, P = 28, 4, 128, 256
    prompt, block = 700, 32
    mk = lambda n, h, std=1.0: (torch.randn(n, h, d, generator=gen) * std).to(torch.bfloat16)
    fk, fv = mk(prompt, Hkv, 1.5), mk(prompt, Hkv, 0.2)         # peaked softmax rows: the missing keys matter
    q, k, v = mk(block, Hq, 2.0), mk(block, Hkv, 1.5), mk(block, Hkv, 0.2)
    pages = (prompt + P - 1) // P
    kc = torch.zeros(pages + 1, P, Hkv, d, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    kc.view(-1, Hkv, d)[:prompt] = fk
    vc.view(-1, Hkv, d)[:prompt] = fv
    ranges = [[(c * 64, 64) for c in range(0, prompt // 64, 2)]]
    rp = torch.tensor([0, len(ranges[0])], dtype=torch.int32)
    rs = torch.tensor([a for a, _ in ranges[0]], dtype=torch.int32)
    rl = torch.tensor([b for _, b in ranges[0]], dtype=torch.int32)
    layer = _layer(dev, Hq, Hkv, d)
    layer.k_cache, layer.v_cache = kc.to(dev), vc.to(dev)
    st = dict(state, full_k=[None, fk.to(dev)], full_v=[None, fv.to(dev)])
    bt = torch.arange(pages + 1, dtype=torch.int32).view(1, -1)
    cu = torch.tensor([0, block], dtype=torch.int32)
    n_ctx = sum(b for _, b in ranges[0])
    set_context_diffusion_lm(False, cu_seqlens_q=cu.to(dev), max_seqlen_q=block, max_seqlen_k=n_ctx + block,
                             block_tables=bt.to(dev), need_kv_cache_store=False, decode_delta_state=st,
                             ranges=(rp.to(dev), rs.to(dev), rl.to(dev), len(ranges[0])), max_context_len=n_ctx)
    try:
        got = layer(q.to(dev).view(block, -1), k.to(dev).view(block, -1), v.to(dev).view(block, -1))
    finally:
        reset_context_diffusion_lm()
    got = got.view(block, Hq, d).float().cpu()
    base = ref_ops.sparse_decode_attention(q, k, v, kc, vc, bt, [0, block], ranges)
    ref = ref_ops.decode_delta(base, q.float(), k.float(), v.float(), fk.float(), fv.float(), state)
    assert (ref - base).abs().max() > 5e-2                       # the correction is not a no-op here
    assert (got - ref).abs().max() <= 3e-2, (got - ref).abs().max()
    if state.get("debug"):
        assert st["calls"] == 1 and st["nonzero_calls"] == 1 and st["anchor_count"] == len(ref_ops.anchor_windows(block, state)[0])
    # the paged copy of the prompt is kept between steps and made again when the prompt changes in place
    def again():
        set_context_diffusion_lm(False, cu_seqlens_q=cu.to(dev), max_seqlen_q=block, max_seqlen_k=n_ctx + block,
                                 block_tables=bt.to(dev), need_kv_cache_store=False, decode_delta_state=st,
                                 ranges=(rp.to(dev), rs.to(dev), rl.to(dev), len(ranges[0])), max_context_len=n_ctx)
        try:
            return layer(q.to(dev).view(block, -1), k.to(dev).view(block, -1), v.to(dev).view(block, -1)) \
                .view(block, Hq, d).float().cpu()
        finally:
            reset_context_diffusion_lm()
    held = st["_paged_prompt"][1]["kc"]
    assert torch.equal(again(), got) and st["_paged_prompt"][1]["kc"] is held
    st["full_v"][1].mul_(-1.0)
    ref_neg = ref_ops.decode_delta(base, q.float(), k.float(), v.float(), fk.float(), -fv.float(), state)
    assert (again() - ref_neg).abs().max() <= 3e-2 and st["_paged_prompt"][1]["kc"] is not held
    st["full_v"][1].mul_(-1.0)
    # disabled or without a prompt for this layer: the plain decode result
    for off in (dict(st, enabled=False), dict(st, full_k=[None, None])):
        set_context_diffusion_lm(False, cu_seqlens_q=cu.to(dev), max_seqlen_q=block, max_seqlen_k=n_ctx + block,
                                 block_tables=bt.to(dev), need_kv_cache_store=False, decode_delta_state=off,
                                 ranges=(rp.to(dev), rs.to(dev), rl.to(dev), len(ranges[0])), max_context_len=n_ctx)
        try:
            plain = layer(q.to(dev).view(block, -1), k.to(dev).view(block, -1), v.to(dev).view(block, -1))
        finally:
            reset_context_diffusion_lm()
        assert (plain.view(block, Hq, d).float().cpu() - base).abs().max() <= 2e-2


def test_decode_delta_layer_under_inference_mode(dev):
    """The reference builds full_k / full_v under torch.inference_mode() (fastdllm_engine.py:656-662) and runs the
    layer there: inference tensors have no version counter, the layer must not ask for one."""
    from prefilling_dllm_amd.context import set_context_diffusion_lm, reset_context_diffusion_lm
    gen = torch.Generator().manual_seed(11)
    Hq, Hkv, d, P = 28, 4, 128, 256
    prompt, block = 300, 32
    mk = lambda n, h, std=1.0: (torch.randn(n, h, d, generator=gen) * std).to(torch.bfloat16)
    fk, fv = mk(prompt, Hkv, 1.5), mk(prompt, Hkv, 0.2)
    q, k, v = mk(block, Hq, 2.0), mk(block, Hkv, 1.5), mk(block, Hkv, 0.2)
    pages = (prompt + P - 1) // P
    kc = torch.zeros(pages + 1, P, Hkv, d, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    kc.view(-1, Hkv, d)[:prompt] = fk
    vc.view(-1, Hkv, d)[:prompt] = fv
    ranges = [[(c * 64, 64) for c in range(0, prompt // 64, 2)]]
    rp = torch.tensor([0, len(ranges[0])], dtype=torch.int32)
    rs = torch.tensor([a for a, _ in ranges[0]], dtype=torch.int32)
    rl = torch.tensor([b for _, b in ranges[0]], dtype=torch.int32)
    bt = torch.arange(pages + 1, dtype=torch.int32).view(1, -1)
    cu = torch.tensor([0, block], dtype=torch.int32)
    n_ctx = sum(b for _, b in ranges[0])
    state = dict(enabled=True)
    layer = _layer(dev, Hq, Hkv, d)
    layer.k_cache, layer.v_cache = kc.to(dev), vc.to(dev)
    with torch.inference_mode():
        st = dict(state, full_k=[None, fk.to(dev).clone()], full_v=[None, fv.to(dev).clone()])
        assert st["full_k"][1].is_inference()
        outs = []
        for _ in range(2):      # the second call reuses the paged copy of the prompt
            set_context_diffusion_lm(False, cu_seqlens_q=cu.to(dev), max_seqlen_q=block, max_seqlen_k=n_ctx + block,
                                     block_tables=bt.to(dev), need_kv_cache_store=False, decode_delta_state=st,
                                     ranges=(rp.to(dev), rs.to(dev), rl.to(dev), len(ranges[0])), max_context_len=n_ctx)
            try:
                outs.append(layer(q.to(dev).view(block, -1), k.to(dev).view(block, -1), v.to(dev).view(block, -1))
                            .view(block, Hq, d).float().cpu())
            finally:
                reset_context_diffusion_lm()
    base = ref_ops.sparse_decode_attention(q, k, v, kc, vc, bt, [0, block], ranges)
    ref = ref_ops.decode_delta(base, q.float(), k.float(), v.float(), fk.float(), fv.float(), state)
    assert (outs[0] - ref).abs().max() <= 3e-2 and torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("state,selection", [
    (dict(enabled=True), None),
    (dict(enabled=True, delta_mode="s4_left3", debug=True), None),
    (dict(enabled=True, delta_mode="s4_left3", full_prompt_len=300, scale=0.8), None),
    (dict(enabled=True, delta_mode="s4_left3", selection_mode="selection_dense_add", selection_scale=0.5), "counts"),
    (dict(enabled=True, delta_mode="s4_left3", selection_mode="selection_dense_replace"), "counts"),
    (dict(enabled=True, delta_mode="s4_left3", selection_mode="selection_dense_replace"), "short"),
])
def test_prefill_sparse_layer(dev, state, selection):
    from prefilling_dllm_amd.context import set_context_diffusion_lm, reset_context_diffusion_lm
    gen = torch.Generator().manual_seed(9)
    Hq, Hkv, d, S = 28, 4, 128, 333
    mk = lambda n, h, std=1.0: (torch.randn(n, h, d, generator=gen) * std).to(torch.bfloat16)
    q, k, v = mk(S, Hq, 2.0), mk(S, Hkv, 1.5), mk(S, Hkv, 0.2)   # outputs below 2: three bf16 roundings stay under the tolerance
    base_mask = torch.tril(torch.ones(S, S, dtype=torch.bool))
    keep = torch.cat([torch.tensor([0]), torch.randperm(S - 1, generator=gen)[:120] + 1, torch.tensor([-1, 5000])])
    sel_out = sel_cnt = None
    st = dict(state, keep_indices=[None, keep.to(dev)])
    if selection is not None:
        n_sel = S if selection == "counts" else 150
        sel_out = mk(n_sel, Hq, 0.2)
        sel_cnt = torch.randint(0, 3, (n_sel,), generator=gen) if selection == "counts" else None
        st["selection_dense"] = dict(outputs=[None, sel_out.to(dev)],
                                     counts=None if sel_cnt is None else [None, sel_cnt.to(dev)])
    layer = _layer(dev, Hq, Hkv, d)
    cu = torch.tensor([0, S], dtype=torch.int32, device=dev)
    set_context_diffusion_lm(True, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_q=S, max_seqlen_k=S,
                             block_mask=base_mask.to(dev), prefill_sparse_state=st)
    try:
        got = layer(q.to(dev).view(S, -1), k.to(dev).view(S, -1), v.to(dev).view(S, -1))
    finally:
        reset_context_diffusion_lm()
    got = got.view(S, Hq, d).float().cpu()
    ref = ref_ops.prefill_sparse_attention(q.float(), k.float(), v.float(), base_mask, keep, state,
                                           selection_outputs=None if sel_out is None else sel_out.float(),
                                           selection_counts=sel_cnt)
    dense = ref_ops._sdpa(q, k, v, base_mask, d ** -0.5)
    assert (ref - dense).abs().max() > 5e-2                      # sparsity matters in this case
    assert torch.isfinite(got).all() and (got - ref).abs().max() <= 3e-2, (got - ref).abs().max()
    if state.get("debug"):
        assert st["calls"] == 1 and st["union_min"] == st["union_max"] == 121
    if selection is not None:
        assert st.get("selection_used_calls", 0) == 1
    # an unsupported delta mode raises like the reference
    bad = dict(st, delta_mode="something_else")
    set_context_diffusion_lm(True, cu_seqlens_q=cu, cu_seqlens_k=cu, max_seqlen_q=S, max_seqlen_k=S,
                             block_mask=base_mask.to(dev), prefill_sparse_state=bad)
    try:
        with pytest.raises(ValueError):
            layer(q.to(dev).view(S, -1), k.to(dev).view(S, -1), v.to(dev).view(S, -1))
    finally:
        reset_context_diffusion_lm()
