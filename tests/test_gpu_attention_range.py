"""Attention parity where the softmax is far from uniform: logits with a large spread, a running maximum that
has to be advanced on accumulators that already hold weight (and partial results of very different log-sum-exp),
and the partial results of a cut column before the output is rounded to bf16.  All through the C ABI, against the CPU oracle."""
import ctypes as C
import math

import pytest
import torch

from oracle import configs, ref_ops
from oracle.tolerances import REL_TOL_BF16, REL_TOL_FP32, assert_attn_close

pytestmark = pytest.mark.gpu


def _ops():
    from prefilling_dllm_amd import ops
    return ops


def _run(case, dev, **kw):
    ops = _ops()
    d = lambda t: None if t is None else t.to(dev)
    rp, rs, rl, mr = case.range_tensors()
    out = ops.sparse_decode_attention(d(case.q), d(case.k_new), d(case.v_new), d(case.k_cache), d(case.v_cache),
                                      d(case.block_table), d(case.q_start_loc), max_q_len=case.max_q,
                                      max_ctx_len=case.max_ctx, ranges=(d(rp), d(rs), d(rl), mr),
                                      k_scale=d(case.k_scale), v_scale=d(case.v_scale), **kw)
    torch.cuda.synchronize()
    return out.float().cpu()


def _oracle(case, **kw):
    kc = case.k_cache_ref if case.k_cache_ref is not None else case.k_cache
    vc = case.v_cache_ref if case.v_cache_ref is not None else case.v_cache
    return ref_ops.sparse_decode_attention(case.q, case.k_new, case.v_new, kc, vc, case.block_table,
                                           case.q_start_loc, case.ranges, **kw)


def _rowwise_rel(out, ref):
    """Largest error of a row relative to the largest value of that row (rows differ by many orders of magnitude)."""
    assert torch.isfinite(out).all()
    scale = ref.abs().amax(dim=-1, keepdim=True)
    assert (scale > 0).all()
    return float(((out - ref).abs() / scale).max())


PLANS = [dict(), dict(rows_per_group=32), dict(rows_per_group=64), dict(rows_per_group=128),
         dict(rows_per_group=256), dict(rows_per_group=32, num_splits=3), dict(rows_per_group=64, num_splits=2),
         dict(rows_per_group=128, num_splits=4), dict(rows_per_group=256, num_splits=3),
         dict(rows_per_group=128, tiles_per_workgroup=3), dict(rows_per_group=256, tiles_per_workgroup=5)]


@pytest.mark.parametrize("plan", PLANS, ids=lambda p: "-".join(f"{k[0]}{v}" for k, v in p.items()) or "default")
@pytest.mark.parametrize("how", ["sm_scale", "inputs"])
def test_logits_with_a_large_spread(dev, plan, how):
    """Logits of standard deviation ~9 (natural units) over 1536 + 40 keys: a handful of keys carry a row, the
    running maximum jumps by more than the lazy-rescale slack in the first tiles and now and then later."""
    case = configs.chunked_prefix_case(51, n_req=2, n_chunks=5, chunk_tokens=512, topk=3, q_len=40,
                                       shared_prefix=False)
    base = 1.0 / math.sqrt(128)
    if how == "sm_scale":
        sm = base * 9.0 * 128            # q.k of the N(0,1)/sqrt(128) inputs has std 1/sqrt(128)
    else:
        case.q = (case.q.float() * 34).to(torch.bfloat16)
        case.k_new = (case.k_new.float() * 34).to(torch.bfloat16)
        case.k_cache = (case.k_cache.float() * 34).to(torch.bfloat16)
        sm = base
    ref = _oracle(case, sm_scale=sm)
    out = _run(case, dev, sm_scale=sm, **plan)
    assert_attn_close(out, ref, f"{how} {plan}")
    assert _rowwise_rel(out, ref) <= REL_TOL_BF16


@pytest.mark.parametrize("fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("plan", PLANS, ids=lambda p: "-".join(f"{k[0]}{v}" for k, v in p.items()) or "default")
def test_rising_maximum_rescales_accumulators_that_carry_weight(dev, plan, fp8):
    """The planted staircase of oracle.configs.staircase_case: the maximum rises by 7.5 / 9.2 / 9.8 log2 units per
    tile (per page for fp8 pages, whose scale is per page) for different rows of one wave, the values shrink by 2^-9
    per step, so every step carries a visible share of the result.  A wrong rescale factor of the accumulators or the
    row sum, or a wrong log-sum-exp weight of a piece (in LDS for the shared row blocks, in the workspace for
    splits and tile spans), changes the result by far more than the bound; every row is checked relative to its
    own magnitude."""
    case = configs.staircase_case(3, gran=256 if fp8 else 64, fp8=fp8, n_chunks=8 if fp8 else 4,
                                  topk=8 if fp8 else 3)
    ref = _oracle(case)
    out = _run(case, dev, **plan)
    rel = _rowwise_rel(out, ref)
    assert rel <= REL_TOL_BF16, f"plan {plan}: row-wise relative error {rel}"


def test_causal_staircase(dev):
    case = configs.staircase_case(5, gran=64, q_len=70)
    ref = _oracle(case, mask_mode="causal")
    for plan in (dict(), dict(rows_per_group=128, num_splits=2), dict(rows_per_group=256)):
        out = _run(case, dev, mask_mode="causal", **plan)
        rel = _rowwise_rel(out, ref)
        assert rel <= REL_TOL_BF16, f"plan {plan}: row-wise relative error {rel}"


def _partials(case, dev, num_splits, rows_per_group, sm_scale=None):
    """Run one split launch through the C ABI with a workspace of our own and read the partial results back:
    o[row, piece, 0:128] (normalised; stored as fp16 with a power-of-two scale per 32 columns) and lse[row, piece]
    in log2 units, row = token * Hq + head."""
    from prefilling_dllm_amd import _lib, ops
    d = lambda t: None if t is None else t.to(dev)
    rp, rs, rl, mr = (d(x) if torch.is_tensor(x) else x for x in case.range_tensors())
    q, kn, vn = d(case.q), d(case.k_new), d(case.v_new)
    kc, vc, bt, qsl = d(case.k_cache), d(case.v_cache), d(case.block_table).contiguous(), d(case.q_start_loc)
    ks, vs = d(case.k_scale), d(case.v_scale)      # (every tensor the descriptor points at stays alive in a local)
    out = torch.empty_like(q)
    n_tok, Hq, dd = q.shape
    desc = ops._fill_desc(q, kn, vn, out, kc, vc, bt, qsl, (rp, rs, rl, mr), None, _lib.MASK_FULL, case.max_q,
                          case.max_ctx, 1.0 / math.sqrt(dd) if sm_scale is None else sm_scale, ks, vs,
                          num_splits, rows_per_group)
    rows_out, splits_out = C.c_int32(0), C.c_int32(0)
    _lib.check(_lib.lib.pdllm_attn_plan(C.byref(desc), 0, C.byref(rows_out), C.byref(splits_out)), "plan")
    assert splits_out.value == num_splits and rows_out.value == rows_per_group
    need = int(_lib.lib.pdllm_attn_workspace_bytes(C.byref(desc)))
    ws = torch.zeros(need, dtype=torch.uint8, device=dev)
    desc.workspace, desc.workspace_bytes = ws.data_ptr(), need
    _lib.check(_lib.lib.pdllm_sparse_decode_attn(C.byref(desc), torch.cuda.current_stream().cuda_stream), "attn")
    torch.cuda.synchronize()
    rows = n_tok * Hq
    n = rows * num_splits
    # workspace: fp16 rows [n, 128], then fp32 log-sum-exps [n], then fp32 scales [n, 4] (one per 32 columns)
    o16 = ws[:n * dd * 2].view(torch.float16).view(rows, num_splits, 4, dd // 4).cpu().double()
    f = ws[n * dd * 2:n * dd * 2 + n * 20].view(torch.float32)
    lse = f[:n].view(rows, num_splits).cpu().double()
    scale = f[n:n * 5].view(rows, num_splits, 4, 1).cpu().double()
    o = (o16 * scale).view(rows, num_splits, dd)
    return o, lse, out.float().cpu()


@pytest.mark.parametrize("splits,rows", [(2, 128), (3, 256), (4, 64)])
def test_fp32_partials_before_bf16_rounding(dev, splits, rows):
    """The split-KV partial results (accumulated in fp32, stored in the workspace as fp16 with a power-of-two scale
    per 32 columns) merged on the host in fp64 against the oracle in fp64: 1e-3 relative, the bound stated for fp32
    accumulation.  The values have a mean of 1 so that the result of a
    row is a well-conditioned average (with zero-mean values the result is itself a rounding-size residue of the
    cancellation and "relative" has no meaning); the probabilities are rounded to bf16 for the second MFMA, as in
    every bf16 attention kernel, which is what the remaining error consists of."""
    case = configs.chunked_prefix_case(61, n_req=2, n_chunks=5, chunk_tokens=512, topk=3, q_len=40,
                                       shared_prefix=False)
    case.v_cache = (case.v_cache.float() * 2 + 1).to(torch.bfloat16)
    case.v_new = (case.v_new.float() * 2 + 1).to(torch.bfloat16)
    case.q = (case.q.float() * 20).to(torch.bfloat16)          # logits of std ~ 1.8: a peaked but broad softmax
    case.k_cache = (case.k_cache.float() * 12).to(torch.bfloat16)
    case.k_new = (case.k_new.float() * 12).to(torch.bfloat16)
    for r in range(2):                                          # the second selected chunk of a request has logits of
        c0 = case.ranges[r][1][0] // 256                        # twice the spread: its piece outweighs the others
        for pg in case.block_table[r][c0:c0 + 2].tolist():
            case.k_cache[pg] = (case.k_cache[pg].float() * 2).to(torch.bfloat16)
    o, lse, out = _partials(case, dev, splits, rows)
    n_tok, Hq, dd = case.q.shape
    m = lse.amax(dim=1, keepdim=True)
    w = torch.where(torch.isinf(lse), torch.zeros_like(lse), torch.exp2(lse - m))
    merged = ((w.unsqueeze(-1) * torch.nan_to_num(o)).sum(1) / w.sum(1, keepdim=True)).view(n_tok, Hq, dd)
    ref = _oracle(case, dtype=torch.float64)
    err = float((merged - ref).abs().max() / ref.abs().max())
    print(f"partials, {splits} splits, {rows} rows per group: relative error {err:.2e}")
    assert err <= REL_TOL_FP32, f"partials, {splits} splits: relative error {err}"
    # every piece saw keys, and the pieces of a row do not all weigh the same
    assert torch.isfinite(lse).all() and float((lse.amax(1) - lse.amin(1)).max()) > 0.5
    # the bf16 output of the same launch is the merged result rounded
    assert_attn_close(out, ref.float(), f"{splits} splits")
    assert float((out.double() - merged).abs().max()) <= 2.0 ** -8 * float(ref.abs().max()) * 1.01


@pytest.mark.parametrize("plan", [dict(rows_per_group=128, num_splits=3), dict(rows_per_group=256, num_splits=2),
                                  dict(rows_per_group=32, num_splits=4), dict(rows_per_group=128, tiles_per_workgroup=5),
                                  dict()],
                         ids=lambda p: "-".join(f"{k[0]}{v}" for k, v in p.items()) or "default")
@pytest.mark.parametrize("shift", [100, -60, 17, -33])
def test_values_scaled_by_a_power_of_two_scale_the_output_exactly(dev, plan, shift):
    """V * 2^k gives out * 2^k bit for bit: every product and sum of the kernel scales exactly, and the partial rows
    of a cut column (fp16 with a power-of-two scale per 32 columns) must follow the magnitude of V whatever it is --
    values of 1e29 and of 1e-19 alike.  (Far below 2^-60 single products leave the normal range of fp32 and the
    scaling stops being exact.)"""
    case = configs.chunked_prefix_case(71, n_req=2, n_chunks=4, chunk_tokens=512, topk=3, q_len=40,
                                       shared_prefix=False)
    base = _run(case, dev, **plan)
    f = 2.0 ** shift
    case.v_cache = (case.v_cache.float() * f).to(torch.bfloat16)
    case.v_new = (case.v_new.float() * f).to(torch.bfloat16)
    assert torch.isfinite(case.v_cache.float()).all() and float(case.v_cache.float().abs().max()) > 0
    scaled = _run(case, dev, **plan)
    assert torch.isfinite(scaled).all()
    assert torch.equal(scaled, base * f), float((scaled / f - base).abs().max())
    assert_attn_close(scaled / f, _oracle(_unscaled(case, f)), f"V * 2^{shift}")


def _unscaled(case, f):
    import copy
    c = copy.copy(case)
    c.v_cache = (case.v_cache.float() / f).to(torch.bfloat16)
    c.v_new = (case.v_new.float() / f).to(torch.bfloat16)
    return c
