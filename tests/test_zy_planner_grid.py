"""The attention planner against forced plans: over a grid of 1-16 requests x 32 / 160 active rows (the decode
shapes of BASELINE configs[2] and the reference engine's response-only block) the plan the library picks by itself
must run within a few per cent of the best plan that can be forced through the descriptor (row-group size, number
of KV splits).  A mis-fit of the planner's cost model after a kernel change shows up here.

This is a timing test: it measures every plan for tens of milliseconds after a warm-up and measures a losing
default plan a second time before it fails."""
import os
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FORCED = [(128, 0), (256, 0), (128, 1), (256, 1), (128, 2), (128, 4), (256, 2), (256, 4), (128, 8), (256, 8),
          (128, 12), (256, 12), (256, 16)]
BOUND = 1.06     # the default plan may lose this much to the best forced one (the target is 5 %; 1 % for noise)


def _time(bench, torch, ops, w, rows, splits):
    preps = bench.prepare(ops, w, rows, splits, 0)
    _, gpu_s = bench.time_steps(torch, preps, 24, 40)       # 4 layers a step: 160 warm-up and 96 timed launches
    return gpu_s / (24 * w["layers"]) * 1e6


@pytest.mark.parametrize("q_len", [32, 160])
def test_default_plan_close_to_best_forced_plan(dev, q_len):
    import bench
    from prefilling_dllm_amd import ops
    report = []
    for n_req in (1, 2, 4, 8, 16):
        w = bench.build_workload(torch, dev, q_len=q_len, layers=4, n_req=n_req)
        _time(bench, torch, ops, w, 0, 0)                    # clocks up
        default = _time(bench, torch, ops, w, 0, 0)
        forced = {}
        for rows, splits in FORCED:
            try:
                forced[(rows, splits)] = _time(bench, torch, ops, w, rows, splits)
            except (ValueError, RuntimeError, NotImplementedError):
                continue                                     # a plan this shape does not admit
        best_plan, best = min(forced.items(), key=lambda kv: kv[1])
        if default > BOUND * best:                           # once more, both, back to back
            default = min(default, _time(bench, torch, ops, w, 0, 0))
            best = max(best, _time(bench, torch, ops, w, *best_plan))
        report.append((n_req, default, best, best_plan))
        del w
        torch.cuda.empty_cache()
    print(f"rows {q_len}: " + "; ".join(f"{n} req: default {d:.1f} us, best forced {b:.1f} us {p}" for n, d, b, p in report))
    for n_req, default, best, best_plan in report:
        assert default <= BOUND * best, (f"{n_req} requests x {q_len} rows: default plan {default:.1f} us, forced "
                                         f"rows_per_group={best_plan[0]} num_splits={best_plan[1]} {best:.1f} us")
