"""Pool of worker processes gated by a queue of resources (GPU ids, compile slots).

Same interface and behaviour as ``RecFlex/task_manager.py:19-53``: ``add_task`` starts a thread
that takes one resource from the queue, runs the target in a spawned process (passing the
resource as keyword ``ident_key`` if given), waits for it and puts the resource back even if
starting the process fails; ``join`` waits for all threads; more than ``max_threads``
outstanding tasks force a join.  Added: the exit codes of the child processes are kept in
``exit_codes`` so that a caller can tell a crashed worker from a finished one.
"""

import multiprocessing as mp
import queue
import threading
from typing import Any, List


class TaskManager:
    def __init__(self, resources: List[Any], max_threads: int = 256):
        self.resource_queue = queue.Queue(len(resources))
        for resource in resources:
            self.resource_queue.put(resource)
        self.task_threads: List[threading.Thread] = []
        self.max_threads = max_threads
        self.exit_codes: List[int] = []
        self._lock = threading.Lock()

        assert mp.get_start_method() == 'spawn', \
            "Please add multiprocessing.set_start_method('spawn') at the start of your program!"

    def _exec(self, target, args, ident_key: str = None):
        ident = self.resource_queue.get()
        try:
            kwargs = {ident_key: ident} if ident_key else {}
            p = mp.Process(target=target, args=args, kwargs=kwargs)
            p.start()
            p.join()
            with self._lock:
                self.exit_codes.append(p.exitcode)
        finally:
            self.resource_queue.put(ident)

    def add_task(self, target, args, ident_key: str = None):
        thread = threading.Thread(target=self._exec, args=(target, args, ident_key))
        self.task_threads.append(thread)
        thread.start()

        if len(self.task_threads) >= self.max_threads:
            print("Too many tasks have been added! Forced to wait for previous threads finishing.")
            self.join()

    def join(self):
        for thread in self.task_threads:
            thread.join()
        self.task_threads = []
