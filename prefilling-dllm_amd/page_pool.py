"""Page bookkeeping for the paged KV cache: which pages are free, how many holders a page has, and which
prompt prefixes are cached under which pages.

The attention and cache operators only ever see page ids; any object with the four members of `PageAllocator`
can hand them out (the record helpers in engine_ops take the allocator as an argument).  `PagePool` is the
implementation that ships: it keeps the interface of the reference's allocator (fastdllm_engine.py:88-167 --
method names, the order in which pages are handed out, the text of the exhaustion error and the prompt hash are
part of what callers observe) over array-based state: the free pages form a first-in-first-out queue threaded
through one int32 array, reference counts live in another.
"""
from __future__ import annotations

import threading
from dataclasses import dataclass
from typing import Dict, Iterator, List, Optional, Protocol, Sequence, runtime_checkable

import numpy as np
import torch

_NIL = -1


@runtime_checkable
class PageAllocator(Protocol):
    """What the record helpers need from an allocator."""

    @property
    def num_free_pages(self) -> int: ...

    def allocate_pages(self, n: int) -> List[int]: ...

    def release_pages(self, pages: Sequence[int]) -> None: ...

    def evict_one(self) -> bool: ...


@dataclass
class _CachedPrefix:
    """A prompt prefix whose KV stays in the cache for reuse (fields as fastdllm_engine.py:64-86)."""

    prompt_hash: int
    page_ids: List[int]
    prompt_len: int
    last_context_logit: torch.Tensor
    ref_count: int = 1


def prompt_digest(prompt_ids: Sequence[int]) -> int:
    """Key of a cached prefix: xxh64 of the token ids as little-endian int64, the digest the reference uses
    (fastdllm_engine.py:100-105), so that keys computed on either side agree."""
    import xxhash
    return xxhash.xxh64(np.asarray(list(prompt_ids), dtype="<i8").tobytes()).intdigest()


class PagePool:
    def __init__(self, num_pages: int, page_size: int):
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self.num_pages = int(num_pages)
        self.page_size = int(page_size)
        self._lock = threading.RLock()
        # queue of free pages: _link[p] is the page behind p, pages leave at _front and join at _back
        self._link = np.arange(1, self.num_pages + 1, dtype=np.int32)
        if self.num_pages:
            self._link[-1] = _NIL
        self._front = 0 if self.num_pages else _NIL
        self._back = self.num_pages - 1 if self.num_pages else _NIL
        self._n_free = self.num_pages
        self._holders = np.zeros(self.num_pages, dtype=np.int32)
        self._prefixes: Dict[int, _CachedPrefix] = {}

    # ---- views of the state ----
    @property
    def num_free_pages(self) -> int:
        with self._lock:
            return self._n_free

    @property
    def free_pages(self) -> Iterator[int]:
        """The free pages in the order they will be handed out."""
        with self._lock:
            order, p = [], self._front
            while p != _NIL:
                order.append(int(p))
                p = int(self._link[p])
        return iter(order)

    @property
    def page_ref_count(self) -> np.ndarray:
        return self._holders

    @property
    def hash_to_prefix(self) -> Dict[int, _CachedPrefix]:
        return self._prefixes

    compute_prompt_hash = staticmethod(prompt_digest)

    # ---- pages ----
    def allocate_pages(self, n: int) -> List[int]:
        """The n pages that have been free the longest, each with one holder; all or nothing."""
        n = int(n)
        if n <= 0:
            return []          # nothing asked for: no state is touched (the reference returns [] as well, ENG:112-119)
        with self._lock:
            if n > self._n_free:
                raise RuntimeError(f"Cannot allocate {n} pages, only {self._n_free} free")
            taken = []
            for _ in range(n):
                p = self._front
                self._front = int(self._link[p])
                self._link[p] = _NIL
                self._holders[p] = 1
                taken.append(int(p))
            self._n_free -= n
            if self._front == _NIL:
                self._back = _NIL
            return taken

    def ref_pages(self, pages: Sequence[int]) -> None:
        with self._lock:
            np.add.at(self._holders, np.asarray(list(pages), dtype=np.int64), 1)

    def release_pages(self, pages: Sequence[int]) -> None:
        """One holder less per listed page; a page without holders joins the back of the free queue."""
        with self._lock:
            # all or nothing: the whole list is checked (a page listed twice needs two holders) before any
            # count changes, so a refused call leaves the pool as it was
            listed = np.asarray([int(p) for p in pages], dtype=np.int64)
            if listed.size == 0:
                return
            if listed.min() < 0 or listed.max() >= self._holders.shape[0]:
                raise RuntimeError(f"page ids {listed.tolist()} are not all pages of this pool")
            drop = np.bincount(listed, minlength=self._holders.shape[0])
            over = np.nonzero(drop > self._holders)[0]
            if over.size:
                raise RuntimeError(f"page {int(over[0])} released more often than it was held")
            for p in listed.tolist():
                self._holders[p] -= 1
                if self._holders[p] == 0:
                    if self._back == _NIL:
                        self._front = int(p)
                    else:
                        self._link[self._back] = p
                    self._back = int(p)
                    self._n_free += 1

    # ---- cached prefixes ----
    def lookup_prefix(self, prompt_ids: Sequence[int]) -> Optional[_CachedPrefix]:
        with self._lock:
            return self._prefixes.get(prompt_digest(prompt_ids))

    def register_prefix(self, prompt_ids: Sequence[int], page_ids: Sequence[int], prompt_len: int,
                        last_context_logit: torch.Tensor) -> _CachedPrefix:
        """Remember that `page_ids` hold the KV of this prompt.  The entry starts without users: it can be
        evicted until somebody raises its ref_count."""
        key = prompt_digest(prompt_ids)
        kept = _CachedPrefix(key, [int(p) for p in page_ids], int(prompt_len), last_context_logit.detach(), 0)
        with self._lock:
            self._prefixes[key] = kept
        return kept

    def release_prefix(self, prompt_ids: Sequence[int]) -> None:
        with self._lock:
            kept = self._prefixes.get(prompt_digest(prompt_ids))
            if kept is not None:
                kept.ref_count -= 1

    def evict_one(self) -> bool:
        """Drop the oldest cached prefix nobody uses and release its pages; False when there is none."""
        with self._lock:
            victim = next((k for k, e in self._prefixes.items() if e.ref_count <= 0), None)
            if victim is None:
                return False
            self.release_pages(self._prefixes.pop(victim).page_ids)
            return True


PrefixPageAllocator = PagePool  # the name callers of the reference know
