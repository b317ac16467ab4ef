"""One-item lookahead between the prefill side and the decode side of a prefill/decode split.

Mirror of the reference's helper (prefilling_dllm/pd_pipeline.py:22-64): while the consumer works on item i
(decode from a prefill record), the producer already prepares item i + 1 (its prefill and KV snapshot) on one
background thread; results come back in input order; when the consumer fails, the record that was prepared
ahead is handed to `release_prepared` so that its pages return to the allocator."""
from __future__ import annotations

import queue
import threading
from typing import Callable, Iterable, Iterator, Optional, TypeVar

ItemT = TypeVar("ItemT")
PreparedT = TypeVar("PreparedT")
ResultT = TypeVar("ResultT")

_STOP = object()


class _Lookahead:
    """A worker thread that runs `prepare` for the items it is handed, one at a time."""

    def __init__(self, prepare: Callable):
        self._prepare = prepare
        self._todo: "queue.Queue" = queue.Queue()
        self._done: "queue.Queue" = queue.Queue()
        self._thread = threading.Thread(target=self._run, name="pd-prefetch", daemon=True)
        self._thread.start()

    def _run(self) -> None:
        while True:
            item = self._todo.get()
            if item is _STOP:
                return
            try:
                self._done.put((True, self._prepare(item[0])))
            except BaseException as exc:  # handed to the caller of collect()
                self._done.put((False, exc))

    def submit(self, item) -> None:
        self._todo.put((item,))

    def collect(self):
        ok, value = self._done.get()
        if not ok:
            raise value
        return value

    def close(self) -> None:
        self._todo.put(_STOP)
        self._thread.join()


def ordered_prefetch_map(items: Iterable[ItemT], *, prepare: Callable[[ItemT], PreparedT],
                         consume: Callable[[ItemT, PreparedT], ResultT],
                         release_prepared: Optional[Callable[[PreparedT], None]] = None) -> Iterator[ResultT]:
    """Yield consume(item, prepare(item)) for every item, in order.  prepare(item i+1) is started before
    consume(item i) and runs beside it.  If consume raises, the item prepared ahead is released and the
    exception propagates."""
    it = iter(items)
    try:
        current = next(it)
    except StopIteration:
        return
    worker = _Lookahead(prepare)
    try:
        worker.submit(current)
        while True:
            prepared = worker.collect()
            try:
                following = next(it)
                ahead = True
            except StopIteration:
                following, ahead = None, False
            if ahead:
                worker.submit(following)
            try:
                yield consume(current, prepared)
            except BaseException:
                if ahead and release_prepared is not None:
                    try:
                        release_prepared(worker.collect())
                    except BaseException:
                        pass  # the lookahead itself failed: nothing was prepared
                raise
            if not ahead:
                return
            current = following
    finally:
        worker.close()
