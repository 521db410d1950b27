"""A thread that keeps a scheduler stepping, for callers that want to submit from elsewhere (a
server's event loop, a test). The scheduler itself is single-threaded; this helper is the only
place where a second thread appears, and it is the caller's to use or not (the reference keeps
such a loop inside its scheduler: pytorch/src/mini_llm/scheduler.py:104-129)."""

from __future__ import annotations

import threading

from .scheduler import Request, Scheduler


class SchedulerThread:
    def __init__(self, scheduler: Scheduler, idle_wait_s: float = 0.05):
        self._scheduler = scheduler
        self._idle_wait_s = idle_wait_s
        self._news = threading.Event()     # set by submit() and stop(): the loop sleeps on it while idle
        self._leaving = False
        self._thread: threading.Thread | None = None

    def start(self) -> None:
        if self.is_running():
            raise RuntimeError("the scheduler thread is running already")
        self._leaving = False
        self._thread = threading.Thread(target=self._work, name="mini-llm-scheduler", daemon=True)
        self._thread.start()

    def is_running(self) -> bool:
        return self._thread is not None and self._thread.is_alive()

    def submit(self, request: Request) -> None:
        self._scheduler.submit(request)
        self._news.set()

    def stop(self, message: str = "the engine is shutting down") -> None:
        """Ends the loop after the step it is in, then fails whatever is live or waiting."""
        self._leaving = True
        self._news.set()
        if self._thread is not None:
            self._thread.join()
            self._thread = None
        self._scheduler.shutdown(message)

    def _work(self) -> None:
        while not self._leaving:
            self._news.clear()
            if not self._scheduler.step() and not self._scheduler.has_work():
                # nothing to do: sleep until something is submitted (the timeout covers a submit
                # that slipped in between the step and the clear above)
                self._news.wait(self._idle_wait_s)
