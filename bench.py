#!/usr/bin/env python3
"""Benchmark of the sparse-prefix decode attention hot path on one MI355X.

Workload (BASELINE.json configs[2], "C3"): one denoise step = the attention of all 28 layers for 8
requests, each with 128 query + 32 response rows (Dream-7B GQA 28/4, d=128, bf16) over its
top-K = 8 of 32 chunks compacted to 512 tokens (16 non-contiguous 256-token pages per request out
of a shared, seeded page pool) plus the active block itself, preceded -- as in the reference's decode forward
(attention_v4.py:328-331) -- by the paged store of the active block's K/V rows into the request's block page.
The prefix KV stays fixed over the steps.  Inputs are synthetic (N(0,1)/sqrt(128)) and resident in HBM before
the timed region.

Prints ONE JSON line: metric = microseconds per denoise step (lower is better), with the roofline
of the dominant kernel (attn_fwd_kernel) and the CPU oracle timed on a bounded sample next to it.
"""
import argparse
import collections
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0        # MI355X HBM3E, published
PEAK_BF16_TFLOPS = 2500.0    # MI355X dense bf16 MFMA, published
# L2-miss bytes of one launch (attention + merge kernels) of this workload, from two rocprofv3 --pmc runs
# (FETCH_SIZE, WRITE_SIZE, scaled by what the same counters read for a plain copy).  The summary of those runs
# names the launch plan it was taken on ("plan: ..." as pdllm_attn_plan_describe prints it) and the resulting
# figure ("traffic_bytes_per_launch: ..."); the figure is reported only while the library still picks that plan.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "attn_fwd_kernel_c3_decode_hbm_traffic.txt")


def measured_traffic(plan_text):
    """Bytes per launch from the committed counter summary, or None when it was taken on another plan."""
    try:
        lines = open(TRAFFIC_PROFILE).read().splitlines()
    except OSError:
        return None
    plan = [ln.split(":", 1)[1].strip() for ln in lines if ln.startswith("plan:")]
    val = [ln.split(":", 1)[1].strip() for ln in lines if ln.startswith("traffic_bytes_per_launch:")]
    if len(plan) != 1 or len(val) != 1 or plan[0] != plan_text:
        return None
    return float(val[0])


Layer = collections.namedtuple("Layer", "store attn")   # one layer of a step (store: a separate call, if any)

HQ, HKV, D, PAGE = 28, 4, 128, 256
LAYERS, N_REQ, N_CHUNKS, TOPK, CHUNK_TOKENS = 28, 8, 32, 8, 512
Q_LEN = 160


def build_workload(torch, dev, q_len=Q_LEN, layers=LAYERS, n_req=N_REQ, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    pages_per_req = N_CHUNKS * CHUNK_TOKENS // PAGE            # logical pages of a request's prefix
    sel_pages = TOPK * CHUNK_TOKENS // PAGE                    # 16 pages actually read
    n_pages = n_req * pages_per_req + 1 + n_req                # + one block page per request for the active rows
    std = 1.0 / math.sqrt(D)
    gd = torch.Generator(device=dev).manual_seed(seed)
    kv = torch.empty((2, layers, n_pages, PAGE, HKV, D), dtype=torch.bfloat16, device=dev)
    for l in range(layers):  # fill per layer to bound the fp32 temporary
        kv[:, l] = (torch.randn((2, n_pages, PAGE, HKV, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    perm = torch.randperm(n_pages - n_req, generator=g)
    block_table = torch.stack([perm[r * pages_per_req:(r + 1) * pages_per_req] for r in range(n_req)]).to(torch.int32)
    ptr, start, length = [0], [], []
    for r in range(n_req):
        sel = sorted(torch.randperm(N_CHUNKS, generator=g)[:TOPK].tolist())
        for c in sel:
            start.append(c * CHUNK_TOKENS)
            length.append(CHUNK_TOKENS)
        ptr.append(len(start))
    mk = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    n_tok = n_req * q_len
    q = (torch.randn((layers, n_tok, HQ, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    kn = (torch.randn((layers, n_tok, HKV, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    vn = (torch.randn((layers, n_tok, HKV, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    out = torch.empty_like(q)
    qsl = torch.arange(0, n_tok + 1, q_len, dtype=torch.int32, device=dev)
    # slot of active row i of request r: offset i of the request's block page (the pages behind the prefix pool)
    block_page = torch.arange(n_pages - n_req, n_pages, dtype=torch.int32)
    store_slots = (block_page.repeat_interleave(q_len) * PAGE + torch.arange(q_len, dtype=torch.int32).repeat(n_req))
    return dict(store_slots=store_slots.to(dev), kv=kv, block_table=block_table.to(dev), ranges=(mk(ptr), mk(start), mk(length), TOPK), q=q, kn=kn,
                vn=vn, out=out, qsl=qsl, q_len=q_len, ctx=TOPK * CHUNK_TOKENS, n_req=n_req, layers=layers,
                ranges_host=[[(start[i], length[i]) for i in range(ptr[r], ptr[r + 1])] for r in range(n_req)],
                sel_pages=sel_pages)


def algorithmic_work(q_len, ctx, n_req):
    """Algorithmic work of one launch (= one layer, all requests): bytes = K/V pages of the selected keys + new K/V
    read (once for the store and the attention) and written to the block page + Q read + output written;
    FLOPs = 4 * rows * keys * d * heads (QK^T and PV, multiply and add)."""
    by = n_req * (2 * ctx * HKV * D * 2 + 2 * 2 * q_len * HKV * D * 2 + 2 * q_len * HQ * D * 2)
    fl = n_req * 4 * q_len * (ctx + q_len) * D * HQ
    return by, fl


def prepare(ops, w, rows_per_group=0, num_splits=0, tiles_per_workgroup=0):
    """One prepared descriptor per layer.  All layers of a step read the same page table and chunk
    ranges, so they share one slot table, which every step rebuilds once (inside the timed region)."""
    table = ops.new_slot_table(w["n_req"], w["ctx"], w["q"].device)
    preps = []
    for l in range(w["layers"]):
        preps.append(Layer(None, ops.PreparedAttention(w["q"][l], w["kn"][l], w["vn"][l], w["kv"][0, l], w["kv"][1, l],
                                           w["block_table"], w["qsl"], max_q_len=w["q_len"], max_ctx_len=w["ctx"],
                                           ranges=w["ranges"], out=w["out"][l], rows_per_group=rows_per_group,
                                           num_splits=num_splits, slot_table=table,
                                           tiles_per_workgroup=tiles_per_workgroup,
                                           active_slot_mapping=w["store_slots"])))
    return preps


def run_step(preps, stream):
    """One denoise step: the slot table once, then per layer one library call = the store of the active K/V rows
    and the attention."""
    preps[0].attn.build_slot_table(stream)
    for p in preps:
        p.attn.run(stream)


def time_steps(torch, preps, steps, warmup):
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(warmup):
        run_step(preps, stream)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        run_step(preps, stream)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) * 1e-3


def cpu_baseline(torch, w, sample_layers=8):
    """The CPU oracle (a PyTorch restatement of the reference path: page-table gather + fp32
    masked softmax attention with GQA repeat) on the first `sample_layers` layers of the same step
    (about 10 s of CPU work with the warm-up and three timed passes).  Returns the seconds per
    layer (median pass), the thread count and the oracle's output of layer 0."""
    from oracle import ref_ops
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    n = min(sample_layers, w["layers"])
    host = [([w[k][l].cpu() for k in ("q", "kn", "vn")], w["kv"][0, l].cpu(), w["kv"][1, l].cpu()) for l in range(n)]
    bt, qsl = w["block_table"].cpu(), w["qsl"].cpu()
    ref0 = ref_ops.sparse_decode_attention(*host[0][0], host[0][1], host[0][2], bt, qsl, w["ranges_host"])  # warm-up
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        for args, kc, vc in host:
            ref_ops.sparse_decode_attention(*args, kc, vc, bt, qsl, w["ranges_host"])
        times.append(time.perf_counter() - t0)
    return sorted(times)[1] / n, cores, ref0, n


def _time_us(torch, fn, iters=10, warmup=2, warm_seconds=0.05):
    """Average launch-to-launch time of fn.  The secondary shapes run after the CPU leg, on an idle GPU whose clocks
    have dropped: besides the `warmup` calls fn is repeated for warm_seconds before the timed calls."""
    t0 = time.perf_counter()
    n = 0
    while n < warmup or time.perf_counter() - t0 < warm_seconds:
        fn()
        n += 1
        if n % 4 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / iters


def _graph_us(torch, fn, iters=20):
    """Device time of fn per call when it is captured once as a HIP graph and replayed: what the launches cost
    without the host's share (Python, ctypes, allocations) between them."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):       # warm-up on the capture stream (lazy initialisation must not be captured)
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        fn()
    return _time_us(torch, g.replay, iters)


def _hbm(by, us):
    return {"hbm_GBps": by / us / 1e3, "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS}


def x_decode_32_rows(torch, ops, dev, gd):
    """Response-only block (the reference engine's real decode shape, 32 rows): the HBM-bound case."""
    w32 = build_workload(torch, dev, q_len=32, layers=4)
    p32 = prepare(ops, w32)
    _, g32 = time_steps(torch, p32, 32, 200)   # 200 warm-up steps of 4 layers = 40 ms: the clocks are up again
    b32, f32_ = algorithmic_work(32, w32["ctx"], w32["n_req"])
    l32 = g32 / (32 * 4)
    return {"us_per_launch": l32 * 1e6, "us_per_step_28_layers": l32 * 28e6, "hbm_GBps": b32 / l32 / 1e9,
            "hbm_frac": b32 / l32 / 1e9 / PEAK_HBM_GBS, "bf16_TFLOPs": f32_ / l32 / 1e12,
            "plan": p32[0].attn.describe_plan()}


PREFILL_NUM_SPLITS = 0   # --num-splits with --only prefill: 1 = one workgroup per column (attn_fwd_kernel)


def _prefill_inputs(torch, ops, dev, gd):
    """configs[3]: 32 chunks x (1 BOS + 1024) tokens, Q/K/V drawn N(0,1), a seeded page table."""
    L, NC = 1025, 32
    n = L * NC
    q = torch.randn((n, HQ, D), generator=gd, device=dev).to(torch.bfloat16)
    k = torch.randn((n, HKV, D), generator=gd, device=dev).to(torch.bfloat16)
    v = torch.randn((n, HKV, D), generator=gd, device=dev).to(torch.bfloat16)
    pages = (n + PAGE - 1) // PAGE
    kc = torch.zeros((pages + 1, PAGE, HKV, D), dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    page_ids = torch.randperm(pages, generator=torch.Generator().manual_seed(2)).to(torch.int32).to(dev)
    slots = ops.slot_mapping_from_pages(page_ids, n)
    cu = torch.arange(0, n + 1, L, dtype=torch.int32, device=dev)
    return L, NC, q, k, v, kc, vc, slots, cu


def x_prefill(torch, ops, dev, gd):
    """configs[3]: chunked BOS-prefixed prefill, causal inside a chunk, with the paged store of K/V (one layer;
    a prefill is 28 of these)."""
    L, NC, q, k, v, kc, vc, slots, cu = _prefill_inputs(torch, ops, dev, gd)
    o = torch.empty_like(q)
    ns = PREFILL_NUM_SPLITS
    us = _time_us(torch, lambda: ops.chunk_prefill_attention(q, k, v, cu, max_seqlen=L, causal=True, k_cache=kc,
                                                             v_cache=vc, slot_mapping=slots, out=o, num_splits=ns), 5, 1)
    fl = 2.0 * NC * L * L * D * HQ
    return {"us_per_layer": us, "bf16_TFLOPs": fl / us / 1e6, "mfma_frac": fl / us / 1e6 / PEAK_BF16_TFLOPS,
            "us_per_prefill_28_layers": us * 28, "inputs": "N(0,1)",
            "plan": ops.describe_prefill_plan(NC, HQ, HKV, L, NC * L, causal=True, num_splits=ns)}


def x_prefill_full(torch, ops, dev, gd):
    """The rows of configs[3] with every key of their chunk visible and no store (17 tiles per column, no mask):
    the rate of the prefill kernel's tile loop without the short columns of the causal case."""
    L, NC, q, k, v, kc, vc, slots, cu = _prefill_inputs(torch, ops, dev, gd)
    o = torch.empty_like(q)
    ns = PREFILL_NUM_SPLITS
    us = _time_us(torch, lambda: ops.chunk_prefill_attention(q, k, v, cu, max_seqlen=L, causal=False, out=o,
                                                             num_splits=ns), 5, 1)
    fl = 4.0 * NC * L * L * D * HQ
    return {"us_per_layer": us, "bf16_TFLOPs": fl / us / 1e6, "mfma_frac": fl / us / 1e6 / PEAK_BF16_TFLOPS,
            "plan": ops.describe_prefill_plan(NC, HQ, HKV, L, NC * L, causal=False, num_splits=ns)}


def x_rope_qk_store(torch, ops, dev, gd):
    """Rotary embedding of Q and K and the paged store of rotated K and V of the configs[3] layer in one launch
    (layers/rotary_embedding.py:39-65 + kv_cache_kernels.py:150-172).  Bytes: Q read and written, K and V read,
    K and V written to the pages."""
    L, NC, q, k, v, kc, vc, slots, cu = _prefill_inputs(torch, ops, dev, gd)
    n = L * NC
    pos = torch.arange(n, device=dev)
    inv = 1.0 / (1e6 ** (torch.arange(0, D, 2, device=dev).float() / D))
    ang = torch.arange(n, device=dev).float()[:, None] * inv[None, :]
    cs = torch.cat([ang.cos(), ang.sin()], dim=-1)
    us = _time_us(torch, lambda: ops.rope_qk_store(q, k, v, pos, cs, kc, vc, slots), 5, 1)
    by = n * (2 * HQ * D * 2 + 2 * 2 * HKV * D * 2 + 2 * HKV * D * 2)  # q r+w, k r+w(in place) + v r, pages w
    return {"us_per_layer": us, **_hbm(by, us)}


def x_score(torch, ops, dev, gd):
    """configs[1]: draft self-information scores of 32 chunks x 4 labels over a 152064 vocabulary + top-4."""
    V2 = 152064
    logits = (torch.randn((32, 4, V2), generator=gd, device=dev) * 2.0).to(torch.bfloat16)
    labels = torch.randint(0, V2, (32, 4), generator=gd, device=dev)
    fn = lambda: ops.chunk_select_from_logits(logits, labels, 4)
    us = _time_us(torch, fn)
    by = logits.numel() * 2
    return {"us": us, **_hbm(by, us), "us_graph_replay": _graph_us(torch, fn)}


def x_evict(torch, ops, dev, gd):
    """configs[1]: column-sum eviction scores of 8 chunks (28 heads x 64 queries x 1025 keys fp32) + keep 256."""
    probs = torch.softmax(torch.randn((8, HQ, 64, 1025), generator=gd, device=dev), dim=-1)
    fn = lambda: ops.evict_keep_from_probs(probs, 256)
    us = _time_us(torch, fn)
    by = probs.numel() * 4
    return {"us": us, **_hbm(by, us), "us_graph_replay": _graph_us(torch, fn)}


def x_evict_qk(torch, ops, dev, gd):
    """The eviction scorer from q and k (triton_eviction_scorer.py:114-210) at the reference's shape: 28 heads,
    the last Lq = 8 / 64 query rows over prefix + 1025-token chunk + queries, causal.  Bytes: K of every visible
    key once per pass over it (the scorer makes two: row maxima and sums, then the chunk columns) + Q."""
    out = {}
    for lq, prefix in ((8, 0), (64, 0), (8, 4096)):
        n = prefix + 1025 + lq
        q = (torch.randn((n, HQ, D), generator=gd, device=dev)).to(torch.bfloat16)
        k = (torch.randn((n, HKV, D), generator=gd, device=dev)).to(torch.bfloat16)
        fn = lambda: ops.query_to_chunk_attention_scores(q, k, prefix_len=prefix, chunk_len=1025, query_len=lq,
                                                         scale=D ** -0.5)
        us = _time_us(torch, fn)
        by = (n + 1025) * HKV * D * 2 + lq * HQ * D * 2 + HQ * 1025 * 4
        out[f"Lq{lq}_prefix{prefix}"] = {"us": us, **_hbm(by, us)}
    return out


def x_compact(torch, ops, dev, gd):
    """Per-head compaction of one configs[2] request (fastdllm_engine.py:607-638): 28 layers x K and V x 4 KV
    heads, 4096 kept of 32800 prompt tokens gathered and written to the front of the request's pages.  Bytes:
    the kept rows read and written."""
    from prefilling_dllm_amd import engine_ops
    layers, n_tok, kept = LAYERS, 32 * 1025, 4096
    pages = (n_tok + PAGE - 1) // PAGE
    kv = torch.randn((2, layers, pages + 1, PAGE, HKV, D), generator=gd, device=dev, dtype=torch.bfloat16)
    page_ids = torch.randperm(pages, generator=torch.Generator().manual_seed(4)).tolist()
    g = torch.Generator().manual_seed(5)
    keep = [torch.stack([torch.randperm(n_tok, generator=g)[:kept].sort().values for _ in range(HKV)]).to(dev)
            for _ in range(layers)]
    # (the engine hands the compaction what its normalisation step returned: fastdllm_engine.py:1940 -> 2081)
    keep, _ = engine_ops.normalize_per_head_keep_indices(keep, num_layers=layers, num_heads=HKV, full_prompt_len=n_tok,
                                                         device=dev)
    us = _time_us(torch, lambda: engine_ops.compact_prompt_cache_per_layer_per_head(kv, page_ids, keep), 3, 1)
    by = 2 * layers * HKV * kept * D * 2 * 2
    return {"us_per_request": us, **_hbm(by, us)}


def x_copy_pages(torch, ops, dev, gd):
    """Page-granular cache-to-cache copy of one request's prompt KV (fastdllm_engine.py:845-859 as pages): 129
    pages x 28 layers x K and V, one launch.  Bytes: the pages read and written."""
    layers, pages = LAYERS, (32 * 1025 + PAGE - 1) // PAGE
    src = torch.randn((2, layers, pages + 3, PAGE, HKV, D), generator=gd, device=dev, dtype=torch.bfloat16)
    dst = torch.zeros_like(src)
    sp = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(6))[:pages].to(torch.int32).to(dev)
    dp = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(7))[:pages].to(torch.int32).to(dev)
    us = _time_us(torch, lambda: ops.kv_copy_pages(src, dst, sp, dp), 5, 1)
    by = 2 * 2 * layers * pages * PAGE * HKV * D * 2
    return {"us_per_request": us, **_hbm(by, us)}


def x_unmask(torch, ops, dev, gd):
    """configs[4]: confidence + argmax over [4 x 32, 126464] logits and the threshold-0.9 unmask decision."""
    V5 = 126464
    lg = (torch.randn((128, V5), generator=gd, device=dev) * 3.0).to(torch.bfloat16)
    ids = torch.full((4, 32), V5 - 1, dtype=torch.int64, device=dev)
    prepared_unmask = ops.PreparedDenoiseUnmask(lg, ids, V5 - 1, 0.9)

    def unmask():
        ids.fill_(V5 - 1)
        prepared_unmask.run()
    us = _time_us(torch, unmask)
    by = lg.numel() * 2
    return {"us": us, **_hbm(by, us), "us_graph_replay": _graph_us(torch, unmask)}


def x_fp8(torch, ops, dev, gd):
    """configs[4]: fp8 e4m3 KV pages with a per-page fp32 scale, MHA 32/32, 4 requests x 16 of 64 chunks x 1025
    tokens, 160 rows.  The pages hold N(0,1)/sqrt(128) values quantised page by page with scale = amax / 448, as
    the quantising store writes them."""
    Hm, n_req, ctx5, ql = 32, 4, 16 * 1025, 160
    std = 1.0 / math.sqrt(D)
    ppr = 64 * 1025 // PAGE + 1
    n_pages = n_req * ppr + 1
    kc8 = torch.empty((n_pages, PAGE, Hm, D), dtype=torch.uint8, device=dev)
    vc8 = torch.empty_like(kc8)
    ks = torch.empty((n_pages,), dtype=torch.float32, device=dev)
    vs = torch.empty_like(ks)
    for cache, scale in ((kc8, ks), (vc8, vs)):
        for p0 in range(0, n_pages, 64):       # in slabs, to bound the fp32 temporary
            x = torch.randn((min(64, n_pages - p0), PAGE, Hm, D), generator=gd, device=dev) * std
            sc = x.abs().amax(dim=(1, 2, 3)) / 448.0
            scale[p0:p0 + x.shape[0]] = sc
            cache[p0:p0 + x.shape[0]] = (x / sc.view(-1, 1, 1, 1)).to(torch.float8_e4m3fn).view(torch.uint8)
    bt = torch.arange(n_req * ppr, dtype=torch.int32, device=dev).view(n_req, ppr)
    g = torch.Generator().manual_seed(3)
    ptr, start, length = [0], [], []
    for r in range(n_req):
        for c in sorted(torch.randperm(64, generator=g)[:16].tolist()):
            start.append(c * 1025)
            length.append(1025)
        ptr.append(len(start))
    mk = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    q5 = (torch.randn((n_req * ql, Hm, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    k5 = (torch.randn((n_req * ql, Hm, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    v5 = (torch.randn((n_req * ql, Hm, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    qsl = torch.arange(0, n_req * ql + 1, ql, dtype=torch.int32, device=dev)
    table = ops.new_slot_table(n_req, ctx5, dev)
    pr = ops.PreparedAttention(q5, k5, v5, kc8, vc8, bt, qsl, max_q_len=ql, max_ctx_len=ctx5,
                               ranges=(mk(ptr), mk(start), mk(length), 16), k_scale=ks, v_scale=vs, slot_table=table)
    pr.build_slot_table()
    us = _time_us(torch, pr.run, 5, 1)
    by = n_req * (2 * ctx5 * Hm * D * 1 + 2 * ql * Hm * D * 2 + 2 * ql * Hm * D * 2)
    fl = n_req * 4.0 * ql * (ctx5 + ql) * D * Hm
    return {"us_per_layer": us, **_hbm(by, us), "bf16_TFLOPs": fl / us / 1e6,
            "mfma_frac": fl / us / 1e6 / PEAK_BF16_TFLOPS, "plan": pr.describe_plan()}


# name in the JSON line -> (short name for --only, function)
EXTRAS = collections.OrderedDict([
    ("decode_32_rows", ("decode32", x_decode_32_rows)),
    ("prefill_32x1025_causal_layer", ("prefill", x_prefill)),
    ("prefill_32x1025_full_mask_layer_no_store", ("prefillfull", x_prefill_full)),
    ("rope_qk_store_32x1025_layer", ("rope", x_rope_qk_store)),
    ("score_32x4x152064_top4", ("score", x_score)),
    ("evict_8x28x64x1025_keep256", ("evict", x_evict)),
    ("evict_score_qk_28_heads_chunk_1025", ("evictqk", x_evict_qk)),
    ("compact_per_head_28_layers_4096_of_32800", ("compact", x_compact)),
    ("kv_copy_pages_129_pages_28_layers", ("copypages", x_copy_pages)),
    ("unmask_4x32x126464", ("unmask", x_unmask)),
    ("decode_fp8_kv_4x16x1025_mha32_layer", ("fp8", x_fp8)),
])


def secondary_shapes(torch, ops, dev, only=None):
    """The other BASELINE configs and the operators around them, one launch (or one layer) each: reported next to
    the headline number.  `only`: short names to run (the rest is skipped)."""
    out = {}
    for name, (short, fn) in EXTRAS.items():
        if only is not None and short not in only:
            continue
        gd = torch.Generator(device=dev).manual_seed(1)
        out[name] = fn(torch, ops, dev, gd)
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=16)   # 16 steps = 55 ms: the GPU clocks need about 50 ms to settle
    ap.add_argument("--rows-per-group", type=int, default=0, help="override the row-group size (tuning)")
    ap.add_argument("--num-splits", type=int, default=0, help="override the KV split count (tuning)")
    ap.add_argument("--tiles-per-wg", type=int, default=0, help="override the tiles per workgroup (tuning)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip the secondary shapes")
    ap.add_argument("--only", default="", metavar="NAMES",
                    help="run only these secondary shapes (comma-separated short names: "
                         + ", ".join(v[0] for v in EXTRAS.values()) + ") and print their results; the headline "
                         "step is not run (for profiling one kernel)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="also run a plain device copy of this many MiB (a kernel of known traffic, used to "
                         "scale the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build is single-GPU (one MI355X); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from prefilling_dllm_amd import ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_calibration > 0:
        n = args.copy_calibration << 20
        src = torch.empty(n, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.only:
        global PREFILL_NUM_SPLITS
        PREFILL_NUM_SPLITS = args.num_splits
        only = set(args.only.split(","))
        unknown = only - {v[0] for v in EXTRAS.values()}
        if unknown:
            print(f"bench.py: unknown shape(s) {sorted(unknown)}", file=sys.stderr)
            sys.exit(2)
        print(json.dumps({"extras": secondary_shapes(torch, ops, dev, only)}))
        return

    w = build_workload(torch, dev)
    preps = prepare(ops, w, args.rows_per_group, args.num_splits, args.tiles_per_wg)
    wall, gpu_s = time_steps(torch, preps, args.steps, args.warmup)
    launches = args.steps * w["layers"]
    us_per_step = gpu_s / args.steps * 1e6
    launch_s = gpu_s / launches
    by, fl = algorithmic_work(w["q_len"], w["ctx"], w["n_req"])
    tflops = fl / launch_s / 1e12
    gbs = by / launch_s / 1e9

    # the active rows of layer 0 now sit in the block pages
    stored = w["kv"][0, 0].view(-1, HKV, D)[w["store_slots"].long()]
    if not torch.equal(stored, w["kn"][0]):
        print("bench.py: the active K rows were not stored into the block pages", file=sys.stderr)
        sys.exit(4)

    # parity spot check of the timed outputs against the oracle (layer 0), and the CPU baseline
    cpu = None
    if not args.no_cpu:
        per_layer, cores, ref, n_sample = cpu_baseline(torch, w)
        from oracle.tolerances import attn_bound
        err = (w["out"][0].float().cpu() - ref).abs().max().item()
        bound = attn_bound(ref)   # max(2e-2 max|ref|, 2 bf16 ulp), at most 2e-2: an all-zero output fails
        if not err <= bound:
            print(f"bench.py: parity check failed, max abs err {err} > {bound}", file=sys.stderr)
            sys.exit(4)
        cpu = {"value": per_layer * w["layers"] * 1e6, "unit": "us/step", "cores": cores, "kind": "port",
               "sample": f"{n_sample} of {w['layers']} layers x {w['n_req']} requests of the same step (median of 3 "
                         f"passes), extrapolated to {w['layers']} layers", "max_abs_err_vs_gpu": err}

    extras = secondary_shapes(torch, ops, dev) if not args.no_extras else {}

    rows, splits = ops.attention_plan(w["n_req"], HQ, HKV, max_q_len=w["q_len"], max_ctx_len=w["ctx"],
                                      num_splits=args.num_splits, rows_per_group=args.rows_per_group)
    plan_text = preps[0].attn.describe_plan()
    line = {
        "metric": "us/denoise-step sparse-KV attention, 32K prefix top-K=8 (28 layers, 8 requests, 160 rows)",
        "value": us_per_step, "unit": "us/step", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": us_per_step / 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: 28-layer sparse-prefix decode step, 8 req x (128 query + 32 "
                               "response rows) over 8x512 non-contiguous KV tokens in 256-token pages, GQA 28/4 d128",
                   "rows_per_workgroup": rows, "kv_splits": splits},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / PEAK_BF16_TFLOPS,
                     "traffic": measured_traffic(plan_text), "plan": plan_text,
                     "kernel": plan_text.split()[0], "avg_launch_us": launch_s * 1e6,
                     "algorithmic_flops_per_launch": fl, "algorithmic_bytes_per_launch": by},
        "hbm": {"achieved_GBps": gbs, "peak_GBps": PEAK_HBM_GBS, "frac": gbs / PEAK_HBM_GBS},
        "cpu_baseline": cpu,
        "wall_s_timed_region": wall,
        "extras": extras,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
