"""Timeouts for ``torch.futures.Future`` (host-side timer, no GPU work).

Same contract as the reference's helpers (torchft/futures.py:123-165):
``future_timeout`` returns a future that resolves like the given one, or fails
with ``TimeoutError("future did not complete within <timeout>")`` when the
deadline passes first; ``future_wait`` blocks with a deadline.
"""

from __future__ import annotations

import heapq
import itertools
import threading
import time
from datetime import timedelta
from typing import Callable, List, Optional, Tuple, TypeVar

from torch.futures import Future

T = TypeVar("T")


class _Deadlines:
    """One daemon thread that fires callbacks at their deadlines."""

    def __init__(self) -> None:
        self._cv = threading.Condition()
        self._heap: List[Tuple[float, int, List[Optional[Callable[[], None]]]]] = []
        self._ids = itertools.count()
        self._thread: Optional[threading.Thread] = None

    def add(self, delay_s: float, fn: Callable[[], None]) -> List[Optional[Callable[[], None]]]:
        slot: List[Optional[Callable[[], None]]] = [fn]  # slot[0] = None cancels
        with self._cv:
            if self._thread is None:
                self._thread = threading.Thread(target=self._run, name="tft_deadlines", daemon=True)
                self._thread.start()
            heapq.heappush(self._heap, (time.monotonic() + delay_s, next(self._ids), slot))
            self._cv.notify()
        return slot

    def _run(self) -> None:
        while True:
            with self._cv:
                while not self._heap:
                    self._cv.wait()
                due, _, slot = self._heap[0]
                now = time.monotonic()
                if due > now:
                    self._cv.wait(timeout=due - now)
                    continue
                heapq.heappop(self._heap)
            fn = slot[0]
            if fn is not None:
                try:
                    fn()
                except Exception:  # a callback must not kill the timer thread
                    pass


_DEADLINES = _Deadlines()


def future_timeout(fut: "Future[T]", timeout: timedelta) -> "Future[T]":
    """A future with the value (or error) of ``fut``, or a ``TimeoutError`` after ``timeout``."""
    if fut.done():
        return fut  # nothing left to time (stream-ordered work completes its future at launch)
    timed: Future = Future()
    lock = threading.Lock()
    done = [False]

    def settle(action: Callable[[], None]) -> None:
        with lock:
            if done[0]:
                return
            done[0] = True
        action()

    def on_deadline() -> None:
        settle(
            lambda: timed.set_exception(TimeoutError(f"future did not complete within {timeout}"))
        )

    slot = _DEADLINES.add(timeout.total_seconds(), on_deadline)

    def on_done(f: "Future[T]") -> None:
        slot[0] = None
        try:
            value = f.value()
        except Exception as e:  # propagate the original failure
            settle(lambda: timed.set_exception(e))
            return
        settle(lambda: timed.set_result(value))

    fut.add_done_callback(on_done)
    return timed


def future_wait(fut: "Future[T]", timeout: timedelta) -> T:
    """Blocks until ``fut`` is done or raises ``TimeoutError`` after ``timeout``."""
    event = threading.Event()
    fut.add_done_callback(lambda _f: event.set())
    if not event.wait(timeout=timeout.total_seconds()):
        raise TimeoutError(f"future did not complete within {timeout}")
    return fut.wait()
