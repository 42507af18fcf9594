"""Fork-per-chunk parallel sampling with a timeout (multi.py:10-49 of the reference).

A ``Job`` forks a child that runs ``func(*inputs)`` and sends the result through a queue; ``get``
waits ``timeout`` seconds, returns 0 on failure and kills the child's whole process tree.
Children must never call into the HIP library (it is not fork-safe once initialised); sampling
only touches the constraint solver.
"""
import multiprocessing as _multi
import signal

import psutil

multi = _multi.get_context("fork")


class Job:
    def __init__(self, func, attach_info, timeout=10):
        self.func = func
        self.attach_info = attach_info
        self.timeout = timeout

    def start(self, inputs):
        self.queue = multi.Queue(2)
        self.process = multi.Process(target=exec, args=(self.func, self.queue, inputs,))
        self.process.start()

    def get(self):
        try:
            res = self.queue.get(block=True, timeout=self.timeout)
        except Exception:  # noqa: BLE001 - timeout or a broken pipe both mean "no result"
            res = 0
        if self.process.is_alive():
            kill_child_processes(self.process.pid)
            self.process.terminate()
        self.process.join()
        self.queue.close()
        self.queue.join_thread()
        del self.process
        del self.queue
        return res


def exec(func, queue, args):
    try:
        res = func(*args)
    except Exception:  # noqa: BLE001 - report the failure at once instead of letting the parent wait for the timeout
        import traceback
        traceback.print_exc()
        res = 0
    queue.put(res)


def kill_child_processes(parent_pid, sig=signal.SIGTERM):
    try:
        parent = psutil.Process(parent_pid)
    except psutil.NoSuchProcess:
        return
    for process in parent.children(recursive=True):
        try:
            process.send_signal(sig)
        except psutil.NoSuchProcess:
            return
