"""Replaying a network as one HIP graph.

On small graphs a compiled plan is a dozen short kernels and the time of an
inference is the time to launch them (the reference's Cora / Pubmed rows,
examples/GAT/GAT.py:87-137, are of that kind).  ``Graphed`` records one call of
``fn(*args)`` into a HIP graph (``torch.cuda.CUDAGraph``) and replays it: one
launch per inference, no Python, no TorchScript interpreter, no allocator.

Contract of a replay: the tensors in ``args`` (and every tensor ``fn`` reaches
through them, e.g. a graph's feature dictionaries and the weights of a network)
are read at their recorded addresses, so new inputs are written into them in
place (``x.copy_(new)``); the result is the same output object every time, valid
until the next replay.  The operators of this package qualify: they enqueue on
the current stream, never synchronise, take their scratch memory from a
per-graph workspace that has reached its final size once ``fn`` has run, and
clear memory with fill kernels, never with memset nodes.  ``fn`` must not read
values back to the host.
"""
from __future__ import annotations

import torch


class Graphed:
    def __init__(self, fn, args=(), warmup: int = 3):
        self.fn, self.args = fn, tuple(args)
        # lazy state (row ids of the graph, workspaces, library handles) is built
        # by ordinary calls first, on a side stream as capture requires
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):
                fn(*self.args)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.output = fn(*self.args)

    def __call__(self):
        """Replay; returns the recorded output object (overwritten by the next replay)."""
        self.graph.replay()
        return self.output
