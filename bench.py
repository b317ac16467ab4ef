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


def secondary_shapes(torch, ops, dev):
    """The other BASELINE configs, one launch (or one layer) each: reported next to the headline number."""
    out = {}
    gd = torch.Generator(device=dev).manual_seed(1)
    std = 1.0 / math.sqrt(D)

    # response-only block (the reference engine's real decode shape, 32 rows): the HBM-bound case
    w32 = build_workload(torch, dev, q_len=32, layers=4)
    p32 = prepare(ops, w32)
    _, g32 = time_steps(torch, p32, 32, 200)   # 200 warm-up steps of 4 layers = 40 ms: the clocks are up again
    b32, f32_ = algorithmic_work(32, w32["ctx"], w32["n_req"])
    l32 = g32 / (32 * 4)
    out["decode_32_rows"] = {"us_per_launch": l32 * 1e6, "us_per_step_28_layers": l32 * 28e6,
                             "hbm_GBps": b32 / l32 / 1e9, "hbm_frac": b32 / l32 / 1e9 / PEAK_HBM_GBS,
                             "bf16_TFLOPs": f32_ / l32 / 1e12}
    del w32, p32

    # configs[3]: chunked BOS-prefixed prefill, 32 chunks x 1025 rows, causal inside a chunk, with the paged
    # store of K/V (one layer; a prefill is 28 of these)
    L, NC = 1025, 32
    n = L * NC
    q = (torch.randn((n, HQ, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    k = (torch.randn((n, HKV, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    v = (torch.randn((n, HKV, D), generator=gd, device=dev) * std).to(torch.bfloat16)
    o = torch.empty_like(q)
    pages = (n + PAGE - 1) // PAGE
    kc = torch.zeros((pages + 1, PAGE, HKV, D), dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    page_ids = torch.randperm(pages, generator=torch.Generator().manual_seed(2)).to(torch.int32).to(dev)
    slots = ops.slot_mapping_from_pages(page_ids, n)
    cu = torch.arange(0, n + 1, L, dtype=torch.int32, device=dev)
    us = _time_us(torch, lambda: ops.chunk_prefill_attention(q, k, v, cu, max_seqlen=L, causal=True, k_cache=kc,
                                                             v_cache=vc, slot_mapping=slots, out=o), 5, 1)
    fl = 2.0 * NC * L * L * D * HQ
    out["prefill_32x1025_causal_layer"] = {"us_per_layer": us, "bf16_TFLOPs": fl / us / 1e6,
                                           "mfma_frac": fl / us / 1e6 / PEAK_BF16_TFLOPS,
                                           "us_per_prefill_28_layers": us * 28}
    del q, k, v, o, kc, vc

    # configs[1]: draft self-information scores of 32 chunks x 4 labels over a 152064 vocabulary + top-4,
    # and the column-sum eviction scores of 8 chunks (28 heads x 64 queries x 1025 keys fp32) + keep 256
    V2 = 152064
    logits = (torch.randn((32, 4, V2), generator=gd, device=dev) * 2.0).to(torch.bfloat16)
    labels = torch.randint(0, V2, (32, 4), generator=gd, device=dev)
    us = _time_us(torch, lambda: ops.chunk_select_from_logits(logits, labels, 4))
    by = logits.numel() * 2
    out["score_32x4x152064_top4"] = {"us": us, "hbm_GBps": by / us / 1e3, "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS}
    probs = torch.softmax(torch.randn((8, HQ, 64, 1025), generator=gd, device=dev), dim=-1)
    us = _time_us(torch, lambda: ops.topb_keep_bos(ops.evict_colsum(probs).reshape(8, 1025), 256))
    by = probs.numel() * 4
    out["evict_8x28x64x1025_keep256"] = {"us": us, "hbm_GBps": by / us / 1e3, "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS}
    del logits, probs

    # configs[4]: confidence + argmax over [4 x 32, 126464] logits and the threshold-0.9 unmask decision
    V5 = 126464
    lg = (torch.randn((128, V5), generator=gd, device=dev) * 3.0).to(torch.bfloat16)
    ids = torch.full((4, 32), V5 - 1, dtype=torch.int64, device=dev)

    prepared_unmask = ops.PreparedDenoiseUnmask(lg, ids, V5 - 1, 0.9)

    def unmask():
        ids.fill_(V5 - 1)
        prepared_unmask.run()
    us = _time_us(torch, unmask)
    by = lg.numel() * 2
    out["unmask_4x32x126464"] = {"us": us, "hbm_GBps": by / us / 1e3, "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS}
    del lg

    # configs[4]: fp8 e4m3 KV pages with a per-page scale, MHA 32/32, 4 requests x 16 chunks x 1025 tokens, 160 rows
    Hm, n_req, ctx5, ql = 32, 4, 16 * 1025, 160
    ppr = 64 * 1025 // PAGE + 1
    n_pages = n_req * ppr + 1
    kc8 = torch.randint(0, 0x78, (n_pages, PAGE, Hm, D), dtype=torch.uint8, device=dev, generator=gd)
    vc8 = torch.randint(0, 0x78, (n_pages, PAGE, Hm, D), dtype=torch.uint8, device=dev, generator=gd)
    ks = torch.full((n_pages,), 1.0 / 448, dtype=torch.float32, device=dev)
    vs = torch.full((n_pages,), 1.0 / 448, dtype=torch.float32, device=dev)
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
    out["decode_fp8_kv_4x16x1025_mha32_layer"] = {"us_per_layer": us, "hbm_GBps": by / us / 1e3,
                                                  "hbm_frac": by / us / 1e3 / PEAK_HBM_GBS,
                                                  "bf16_TFLOPs": fl / us / 1e6}
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
