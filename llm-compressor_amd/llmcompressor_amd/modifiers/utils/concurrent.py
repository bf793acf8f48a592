"""Running independent per-module compression jobs side by side on one GPU.

A module's compression (the Cholesky chain, then the blocked column loop) is a long run of small, serially
dependent kernels that leaves most of the chip idle; the modules of one layer are independent.  Each worker is
one host thread with its own HIP stream (default priority): the side streams start behind everything queued on
the caller's stream, and the caller's stream waits for all of them at the end.  Per job the kernels and their
order are those of the sequential loop, so results do not change.
"""
from __future__ import annotations

import threading
from typing import Callable, Dict, List

import torch

__all__ = ["run_on_streams", "SIDE_STREAMS"]

# the side streams of every device, shared by all modifiers of the process: creating a stream and giving it its
# first submission costs about 0.4 ms, and one modifier after the other uses them, never two at a time
SIDE_STREAMS: Dict[torch.device, list] = {}


def run_on_streams(jobs: List, work: Callable, workers: int, device: torch.device,
                   stream_cache: Dict[torch.device, list]) -> None:
    """``work(job, produced_on=side_stream, consumed_on=caller_stream)`` for every job, in list order, at most
    ``workers`` at a time.  The first exception stops the remaining jobs and is re-raised on the caller."""
    jobs = list(jobs)
    streams = stream_cache.setdefault(device, [])
    while len(streams) < max(workers, 4):
        # the runtime binds a stream to one of its few hardware queues at the stream's first submission; two
        # streams first used at the same moment from two threads have been seen to land on the same queue and
        # then run strictly one after the other.  One tiny submission per new stream, in turn, spreads them.
        streams.append(torch.cuda.Stream(device=device))
        with torch.cuda.stream(streams[-1]):
            torch.zeros(1, device=device)
    main = torch.cuda.current_stream(device)
    ready = main.record_event()
    lock = threading.Lock()
    errors = []

    def worker(stream):
        try:
            with torch.cuda.device(device), torch.cuda.stream(stream):
                stream.wait_event(ready)
                while True:
                    with lock:
                        if not jobs or errors:
                            return
                        job = jobs.pop(0)
                    work(job, produced_on=stream, consumed_on=main)
        except BaseException as err:  # re-raised on the calling thread
            errors.append(err)

    threads = [threading.Thread(target=worker, args=(s,), daemon=True) for s in streams[:workers]]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for s in streams[:workers]:
        main.wait_stream(s)
    if errors:
        raise errors[0]
