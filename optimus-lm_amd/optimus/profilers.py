"""optimus.profilers — the hot path's timing hook, same name and tag scheme as the reference
(optimus/profilers.py:99-119): record_pcl_function("a--b--c") starts/stops the nested timers
"a", "a--b", "a--b--c" on optimus.globals.profiler and is a no-op when that is None.

The reference marks events with a SYCL profiling tag on the XPU queue
(pytorch_xpu_extensions/pcl.xpu.profiler/csrc/profiler/profile.dp.cpp:36-42); here an event is a
HIP event recorded on PyTorch's current stream, so nothing synchronises until `summary()`.
"""
from contextlib import contextmanager

import torch

import optimus.globals


@contextmanager
def record_pcl_function(full_name, tag=None, exclude_from_trace=False, key="", ignore=False):
    profiler = optimus.globals.profiler
    if ignore or profiler is None:
        yield
        return
    tokens = full_name.split("--")
    names = ["--".join(tokens[0:i + 1]) for i in range(len(tokens))]
    try:
        for name in names:
            if name not in profiler.timers:
                profiler.register_timer(name, tag=tag, exclude_from_trace=exclude_from_trace)
            profiler.start(name, key=key)
        yield
    finally:
        for name in names:
            profiler.stop(name)


class PclProfiler:
    """Hierarchical stream timers: start/stop record HIP events; summary() resolves them."""

    def __init__(self, process="GPU", rank=0, world_size=1):
        self.process = process
        self.rank = rank
        self.world_size = world_size
        self.timers = {}

    def register_timer(self, name, tag=None, exclude_from_trace=False):
        self.timers[name] = {"tag": tag, "exclude_from_trace": exclude_from_trace, "open": None,
                             "pairs": []}

    def start(self, name, key=""):
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self.timers[name]["open"] = ev

    def stop(self, name):
        t = self.timers[name]
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        t["pairs"].append((t["open"], ev))
        t["open"] = None

    def summary(self, reset=True):
        """-> {name: (calls, total_ms)}; synchronises the device once."""
        torch.cuda.synchronize()
        out = {}
        for name, t in self.timers.items():
            out[name] = (len(t["pairs"]), sum(a.elapsed_time(b) for a, b in t["pairs"]))
            if reset:
                t["pairs"] = []
        return out
