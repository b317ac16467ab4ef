"""Host-side prefill/decode lookahead and the thread-local operator context: the behaviours the reference's own
tests check (prefilling_dllm_engine/tests/test_pd_pipeline.py:48-160), restated against this package."""
import threading

import pytest

from prefilling_dllm_amd import context as ctx
from prefilling_dllm_amd.pd_pipeline import ordered_prefetch_map


def test_next_item_is_prepared_while_the_current_one_is_consumed():
    order, releases = [], []
    second_prepared = threading.Event()

    def prepare(item):
        order.append(("prepare", item))
        if item == 2:
            second_prepared.set()
        return f"record-{item}"

    def consume(item, record):
        if item == 1:
            assert second_prepared.wait(timeout=2.0), "item 2 must be prepared while item 1 is consumed"
        return f"{item}:{record}"

    out = list(ordered_prefetch_map([1, 2, 3], prepare=prepare, consume=consume, release_prepared=releases.append))
    assert out == ["1:record-1", "2:record-2", "3:record-3"]
    assert releases == []
    assert order == [("prepare", 1), ("prepare", 2), ("prepare", 3)]


def test_prepared_ahead_item_is_released_when_consume_fails():
    releases = []
    second_prepared = threading.Event()

    def prepare(item):
        if item == 2:
            second_prepared.set()
        return f"record-{item}"

    def consume(item, record):
        if item == 1:
            assert second_prepared.wait(timeout=2.0)
            raise RuntimeError("decode failed")
        return record

    with pytest.raises(RuntimeError, match="decode failed"):
        list(ordered_prefetch_map([1, 2], prepare=prepare, consume=consume, release_prepared=releases.append))
    assert releases == ["record-2"]


def test_empty_input_single_item_and_early_close():
    assert list(ordered_prefetch_map([], prepare=lambda i: i, consume=lambda i, r: r)) == []
    assert list(ordered_prefetch_map([7], prepare=lambda i: i * 2, consume=lambda i, r: (i, r))) == [(7, 14)]
    releases = []
    gen = ordered_prefetch_map([1, 2, 3], prepare=lambda i: f"r{i}", consume=lambda i, r: r,
                               release_prepared=releases.append)
    assert next(gen) == "r1"
    gen.close()                       # the consumer stops early: the record prepared ahead goes back
    assert releases == ["r2"]


def test_prepare_failure_propagates_in_order():
    def prepare(item):
        if item == 2:
            raise ValueError("prefill failed")
        return item

    got = []
    with pytest.raises(ValueError, match="prefill failed"):
        for r in ordered_prefetch_map([1, 2, 3], prepare=prepare, consume=lambda i, r: r):
            got.append(r)
    assert got == [1]


def test_operator_context_is_isolated_between_threads():
    ctx.reset_context_diffusion_lm()
    ctx.set_context_diffusion_lm(True, max_seqlen_q=11)
    ready, done, seen = threading.Event(), threading.Event(), {}

    def worker():
        ctx.reset_context_diffusion_lm()
        ctx.set_context_diffusion_lm(False, max_seqlen_q=22)
        seen["worker"] = ctx.get_context_diffusion_lm().max_seqlen_q
        ready.set()
        done.wait(timeout=2.0)

    t = threading.Thread(target=worker)
    t.start()
    assert ready.wait(timeout=2.0)
    assert ctx.get_context_diffusion_lm().max_seqlen_q == 11
    done.set()
    t.join(timeout=2.0)
    assert seen == {"worker": 22}
    ctx.reset_context_diffusion_lm()
