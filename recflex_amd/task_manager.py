"""Runs tasks in child processes, at most one at a time per resource (a GPU id, a compile slot).

The interface of ``RecFlex/task_manager.py:19-53``: ``TaskManager(resources, max_threads)``,
``add_task(target, args, ident_key)`` -- run ``target(*args)`` in a spawned process, with the
resource it was given as keyword ``ident_key`` if that is set -- and ``join()``.  The structure
is another one: every resource has a serving thread that takes tasks from one shared queue for
as long as there are any, so a thousand tasks cost as many processes but only ``len(resources)``
threads, and a resource can never be handed to two tasks.  ``join`` waits until the queue has
drained and the serving threads have ended; the next ``add_task`` starts them again.  More than
``max_threads`` unfinished tasks make ``add_task`` wait for all of them first, as in the reference.
Added: ``exit_codes`` keeps the exit code of every child (``None`` if it could not be started), so
that a caller can tell a crashed worker from a finished one.
"""

import multiprocessing as mp
import queue
import threading
from typing import Any, Callable, List, Optional, Sequence, Tuple

_Task = Tuple[Callable, Sequence[Any], Optional[str]]


class TaskManager:
    def __init__(self, resources: List[Any], max_threads: int = 256):
        assert mp.get_start_method() == 'spawn', \
            "Please add multiprocessing.set_start_method('spawn') at the start of your program!"
        self.resources: List[Any] = list(resources)
        self.max_threads = max_threads
        self.exit_codes: List[Optional[int]] = []
        self._tasks: "queue.Queue[Optional[_Task]]" = queue.Queue()
        self._servers: List[threading.Thread] = []
        self._busy: List[Any] = []
        self._lock = threading.Lock()

    # ---- one serving thread per resource --------------------------------------------------

    def _serve(self, resource: Any) -> None:
        while True:
            task = self._tasks.get()
            if task is None:                    # join() is over: nothing more will come
                self._tasks.task_done()
                return
            target, args, ident_key = task
            code: Optional[int] = None
            with self._lock:
                self._busy.append(resource)
            try:
                child = mp.Process(target=target, args=tuple(args),
                                   kwargs={ident_key: resource} if ident_key else {})
                child.start()
                child.join()
                code = child.exitcode
            except Exception as exc:            # e.g. an argument that cannot be pickled: this
                # task is lost (exit code None), the resource goes on serving the others
                print(f"TaskManager: could not run {getattr(target, '__name__', target)}: "
                      f"{type(exc).__name__}: {exc}", flush=True)
            finally:
                with self._lock:
                    self._busy.remove(resource)
                    self.exit_codes.append(code)
                self._tasks.task_done()

    def _start_servers(self) -> None:
        if not self._servers:
            self._servers = [threading.Thread(target=self._serve, args=(r,), daemon=True)
                             for r in self.resources]
            for server in self._servers:
                server.start()

    # ---- the reference's interface --------------------------------------------------------

    def add_task(self, target: Callable, args: Sequence[Any], ident_key: str = None) -> None:
        if self._tasks.unfinished_tasks >= self.max_threads:
            print("Too many tasks have been added! Forced to wait for previous tasks finishing.")
            self.join()
        self._start_servers()
        self._tasks.put((target, args, ident_key))

    def join(self) -> None:
        """Returns when every task added so far has run."""
        self._tasks.join()
        for _ in self._servers:
            self._tasks.put(None)
        for server in self._servers:
            server.join()
        self._servers = []

    @property
    def resource_queue(self) -> "queue.Queue[Any]":
        """The resources no task holds right now (a snapshot, in the reference's form)."""
        with self._lock:
            idle = [r for r in self.resources if r not in self._busy]
        snapshot: "queue.Queue[Any]" = queue.Queue(len(self.resources))
        for resource in idle:
            snapshot.put(resource)
        return snapshot
