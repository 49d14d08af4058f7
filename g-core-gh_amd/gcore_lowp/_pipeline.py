"""Host <-> device pipeline of the checkpoint converters.

A converter's kernels take microseconds per tensor; what it waits for is the host: paging the tensor in from the
safetensors file, the copy to the GPU and the copy back.  Three stages run side by side, each on its own thread and
(for the two copies) its own stream of default priority:

  feeder   reads job i+1 from the checkpoint, stages it in pinned memory, starts its host-to-device copy
  caller   waits for job i's copy on the current stream and launches its kernels (all library calls stay on the
           calling thread)
  drainer  copies job i-1's results into pinned host memory and hands them back

Pinned buffers come from torch's caching host allocator (hipHostMalloc underneath), so after the first few jobs no
allocation reaches the driver.  Results are returned in pinned memory; the caller drops them after writing the shard.
"""
from __future__ import annotations

import queue
import threading

import torch

_END = object()


def run_pipelined(dev, jobs, compute, depth: int = 2):
    """jobs: iterable of (tag, host_tensors, on_gpu); host_tensors is a tuple of CPU tensors (None entries pass
    through), consumed on the feeder thread.  compute(tag, tensors) -> {name: tensor} is called on the calling
    thread, in job order, with GPU copies of the tensors when on_gpu, else with the host tensors themselves.
    Yields (tag, {name: CPU tensor}) as results become available (not necessarily in job order).  An exception on
    any stage stops the others and is raised here."""
    s_in, s_out = torch.cuda.Stream(dev), torch.cuda.Stream(dev)
    staged: queue.Queue = queue.Queue(maxsize=depth)
    to_drain: queue.Queue = queue.Queue(maxsize=depth)
    results: queue.Queue = queue.Queue()
    stop = threading.Event()
    errors: list[BaseException] = []

    def put(q, item) -> bool:
        while not stop.is_set():
            try:
                q.put(item, timeout=0.05)
                return True
            except queue.Full:
                continue
        return False

    def get(q):
        while not stop.is_set():
            try:
                return q.get(timeout=0.05)
            except queue.Empty:
                continue
        return _END

    def feeder():
        try:
            with torch.cuda.device(dev), torch.cuda.stream(s_in):
                for tag, host, on_gpu in jobs:
                    if not on_gpu:
                        if not put(staged, (tag, host, None)):
                            return
                        continue
                    gpu = []
                    for t in host:
                        if t is None:
                            gpu.append(None)
                            continue
                        pinned = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
                        pinned.copy_(t)                               # pages the file in; host memcpy
                        gpu.append(pinned.to(dev, non_blocking=True))
                    ready = torch.cuda.Event()
                    ready.record(s_in)
                    if not put(staged, (tag, gpu, ready)):
                        return
            put(staged, _END)
        except BaseException as e:  # noqa: BLE001 - handed to the caller
            errors.append(e)
            stop.set()

    def drainer():
        try:
            with torch.cuda.device(dev), torch.cuda.stream(s_out):
                while True:
                    item = get(to_drain)
                    if item is _END:
                        return
                    tag, outs, computed = item
                    s_out.wait_event(computed)
                    host = {}
                    for name, t in outs.items():
                        if not t.is_cuda:
                            host[name] = t
                            continue
                        h = torch.empty(t.shape, dtype=t.dtype, pin_memory=True)
                        h.copy_(t, non_blocking=True)
                        t.record_stream(s_out)
                        host[name] = h
                    s_out.synchronize()
                    results.put((tag, host))
        except BaseException as e:  # noqa: BLE001
            errors.append(e)
            stop.set()

    threads = [threading.Thread(target=feeder, daemon=True), threading.Thread(target=drainer, daemon=True)]
    for th in threads:
        th.start()
    try:
        with torch.cuda.device(dev):
            cur = torch.cuda.current_stream(dev)
            while True:
                item = get(staged)
                if item is _END:
                    break
                tag, tensors, ready = item
                if ready is None:
                    results.put((tag, compute(tag, tensors)))
                else:
                    cur.wait_event(ready)
                    for t in tensors:
                        if t is not None:
                            t.record_stream(cur)
                    outs = compute(tag, tensors)
                    computed = torch.cuda.Event()
                    computed.record(cur)
                    if not put(to_drain, (tag, outs, computed)):
                        break
                while not results.empty():
                    yield results.get()
        if not stop.is_set():
            put(to_drain, _END)
            threads[1].join()
    except BaseException:
        stop.set()
        raise
    finally:
        if errors:
            stop.set()
        for th in threads:
            th.join(timeout=5)
    if errors:
        raise errors[0]
    while not results.empty():
        yield results.get()
