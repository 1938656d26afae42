"""HIP graphs over runs of fixed-shape Sinkhorn steps.

On small problems a solve is bound by launch latency: 2000 x 2000 x 3 takes 0.02 ms of kernel
time per step and two launches.  A run of steps between two convergence checks is a fixed
sequence of kernels on fixed shapes (``fs_symmetric_steps`` / ``fs_self_pair_steps`` enqueue
everything without looking at device data), so it is captured once into a graph and replayed.

A graph bakes in addresses, so each one owns static copies of its inputs (filled by device
copies before a replay), its operand planes, work vectors and outputs (cloned after a replay:
the next replay overwrites them).  Keys hold everything that shapes the launches: device,
shapes, the per-step (eps, weight, damping) tuples, flags, and which arguments alias.  The first
call with a key runs eagerly (it also loads the kernels), the second captures, later ones replay;
an LRU bound keeps the memory of forgotten shapes from piling up.  Nothing is captured while the
caller is itself capturing.  An entry's static tensors are written, replayed into and cloned on
the caller's stream, so an entry belongs to one (thread, stream) pair: both are part of the key,
and two threads or streams solving the same shape each capture a graph of their own; the cache
itself is guarded by a lock.  No counterpart in the reference, whose solver loop launches one
Triton kernel per step (sinkhorn_solvers.py:497-531).
"""
from __future__ import annotations

import os
import threading
from collections import OrderedDict
from typing import Callable, Optional, Sequence, Tuple

import torch

# FLASH_SINKHORN_GRAPHS=0 switches graphs off; runs shorter than MIN_STEPS or on more than
# MAX_LOGITS = n * m logits per half-update are launch by launch anyway
ENABLED = os.environ.get("FLASH_SINKHORN_GRAPHS", "1") != "0"
MIN_STEPS = 8
MAX_LOGITS = 1 << 25
MAX_ENTRIES = 16


class _Entry:
    __slots__ = ("graph", "inputs", "outputs", "calls")

    def __init__(self):
        self.graph = None
        self.inputs = None
        self.outputs = None
        self.calls = 0


_cache: "OrderedDict[tuple, _Entry]" = OrderedDict()
_lock = threading.Lock()


def eligible(n: int, m: int, n_steps: int, device: torch.device) -> bool:
    return (ENABLED and n_steps >= MIN_STEPS and n * m <= MAX_LOGITS and device.type == "cuda"
            and not torch.cuda.is_current_stream_capturing())


def clear() -> None:
    with _lock:
        _cache.clear()


def run(key: tuple, fn: Callable[..., Tuple[torch.Tensor, ...]],
        inputs: Sequence[Optional[torch.Tensor]]) -> Tuple[torch.Tensor, ...]:
    """``fn(*inputs)`` through a graph: ``fn`` must enqueue the same kernels for the same key
    whatever the values in ``inputs`` (contiguous tensors or None), allocate what it needs with
    torch, and return a tuple of tensors."""
    key = key + (torch.cuda.current_stream().cuda_stream, threading.get_ident())
    with _lock:
        entry = _cache.get(key)
        if entry is None:
            entry = _cache[key] = _Entry()
            while len(_cache) > MAX_ENTRIES:
                _cache.popitem(last=False)
        _cache.move_to_end(key)
    entry.calls += 1
    if entry.calls == 1:  # eager: loads the kernels, and one-off shapes never pay for a capture
        return fn(*inputs)
    if entry.graph is None:
        entry.inputs = [None if t is None else t.clone() for t in inputs]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            entry.outputs = fn(*entry.inputs)
        entry.graph = graph
    else:
        for dst, src in zip(entry.inputs, inputs):
            if dst is not None:
                dst.copy_(src)
    entry.graph.replay()
    return tuple(t.clone() for t in entry.outputs)
