"""A training step of many small launches, captured once into a HIP graph and replayed.

The per-relation models of the heterogeneous path and the temporal attention step are
hundreds of kernels of a few microseconds each; issued one by one, the host is the
bottleneck (the reference's executor issues them the same way, xgnn_h/executor.py:9-66).
Every kernel of this library is launched on torch's current stream and takes its scratch
from torch's allocator, so a whole forward + backward can be recorded by
``torch.cuda.graph`` and replayed as one submission.

Replay is only handed out after it has been checked: graph replays on this platform have
given wrong results after the first one when the recording held a memset node, and torch
ops record such nodes in places one does not see (column reductions, for one). So the
recording is replayed several times, with eager runs of the same step in between, and every
replay must reproduce the eager results; otherwise ``ReplayedStep`` raises and the caller
keeps the eager step.
"""
import torch


class ReplayedStep:
    """``step()`` runs forward + backward on tensors that keep their addresses (inputs,
    parameters) and returns the list of tensors it produces (outputs, gradients); it must
    drop old gradients itself (``p.grad = None``) so that the recorded step writes them
    instead of accumulating. Deterministic steps only: dropout off, or the check fails.

    ``replay()`` runs the recorded step and returns the same list of (static) result
    tensors; their contents are overwritten by the next replay."""

    def __init__(self, step, warmup=3, checks=3, rtol=1e-5, atol=1e-6):
        want = [t.detach().clone() for t in step()]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # graph-private allocations settle on a side stream
            for _ in range(warmup):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self._results = list(step())
        if len(self._results) != len(want):
            raise RuntimeError("the step returned %d tensors when recorded, %d before"
                               % (len(self._results), len(want)))
        for round_ in range(checks):
            for t in self._results:
                t.detach().fill_(float("nan"))
            self._graph.replay()
            torch.cuda.synchronize()
            bad = [i for i, (got, ref) in enumerate(zip(self._results, want))
                   if got.shape != ref.shape or not torch.allclose(got, ref, rtol=rtol, atol=atol)]
            if bad:
                raise RuntimeError("replay %d of the recorded step differs from the eager step in "
                                   "results %s" % (round_, bad))
            step()  # the program's own eager work between replays
            torch.cuda.synchronize()

    def replay(self):
        self._graph.replay()
        return self._results
