"""Runs a function in a forked child with a time limit (the job abstraction of the reference's multi.py:10-49).

``Job(func, args, timeout)``: ``start(args)`` forks, ``get()`` returns the child's result, or 0 when the child
raised, died or outlived ``timeout`` seconds - in which case the child and everything it started are killed.
Forking copies the parent's task and constraint solver for free, which is why sampling uses it; the children must
never call into the HIP library (not fork-safe once initialised) - they only run the solver.
"""
import multiprocessing
import signal
import traceback

import psutil

_ctx = multiprocessing.get_context("fork")
multi = _ctx        # kept: callers that want the same start method


def _child(func, conn, args):
    try:
        out = func(*args)
    except Exception:  # noqa: BLE001 - the parent gets "no result" at once instead of waiting for the limit
        traceback.print_exc()
        out = 0
    try:
        conn.send(out)
    finally:
        conn.close()


def kill_child_processes(parent_pid, sig=signal.SIGTERM):
    """Signals every descendant of ``parent_pid``."""
    try:
        descendants = psutil.Process(parent_pid).children(recursive=True)
    except psutil.NoSuchProcess:
        return
    for proc in descendants:
        try:
            proc.send_signal(sig)
        except psutil.NoSuchProcess:
            pass


class Job:
    def __init__(self, func, attach_info, timeout=10):
        self.func = func
        self.attach_info = attach_info
        self.timeout = timeout
        self._proc = None
        self._conn = None

    def start(self, inputs):
        self._conn, child_end = _ctx.Pipe(duplex=False)
        self._proc = _ctx.Process(target=_child, args=(self.func, child_end, inputs))
        self._proc.start()
        child_end.close()

    def get(self):
        result = 0
        try:
            if self._conn.poll(self.timeout):
                result = self._conn.recv()
        except (EOFError, OSError):
            result = 0                      # the child died before it could answer
        if self._proc.is_alive():
            kill_child_processes(self._proc.pid)
            self._proc.terminate()
        self._proc.join()
        self._conn.close()
        self._proc = self._conn = None
        return result
