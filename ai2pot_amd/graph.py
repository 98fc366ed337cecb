"""Replay of an energy / force / virial operator call as a HIP graph.

A small system is launch-bound: one call is a dozen short kernels (zero fills, the model kernel,
the pair reduction, the partial-sum reductions) and at a few thousand atoms their launch latency
is several times their run time.  ``GraphedCall`` records one call into a HIP graph on first use
and replays it afterwards with a single launch.

The operators qualify because they enqueue kernels only: no host synchronisation, no memset
nodes, and no allocation once the library's workspace has reached its size (it has after the
eager warm-up calls made here before the capture).  What a caller has to respect:

* the input tensors are the graph's static buffers: write new coordinates / lists into them in
  place (``tensor.copy_(...)``), keep shapes, dtypes and scalar arguments unchanged;
* the outputs are overwritten by every replay: consume or clone them before the next one;
* input checks that read back from the device are skipped (``validate=False`` is forced), so a
  list that violates the contract is not reported from inside the graph;
* the graph names the library's per-device workspace by address.  A later call that needs a larger
  workspace (a bigger system, another ``GraphedCall`` with bigger shapes) or ``a2p_workspace_release``
  frees those buffers; ``replay`` notices (the library counts such events) and records the call
  again instead of replaying onto freed memory.  The output tensors are then new objects: use what
  ``replay`` returns.
"""
import ctypes

import torch

from . import _lib


def _generation():
    fn = _lib.lib().a2p_workspace_generation
    fn.restype = ctypes.c_ulonglong
    return int(fn())


class GraphedCall:
    def __init__(self, op, *args, warmup=3, **kwargs):
        """op: one of the ``ai2pot_amd.ops`` operators without host synchronisation (the E/F/V,
        descriptor and site-energy operators); args / kwargs: its arguments, tensors on one device."""
        kwargs = dict(kwargs, validate=False)
        tensors = [a for a in args if isinstance(a, torch.Tensor) and a.is_cuda]
        if not tensors:
            raise RuntimeError("GraphedCall needs at least one tensor argument on a HIP device")
        self.device = tensors[0].device
        self._op, self._args, self._kwargs = op, args, kwargs
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):       # sizes the library workspace and torch's pools
                op(*args, **kwargs)
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        self.recaptures = 0
        self._capture()

    def _capture(self):
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.outputs = self._op(*self._args, **self._kwargs)
        self._generation = _generation()

    def valid(self):
        """False once the workspace the graph names has been freed or replaced."""
        return _generation() == self._generation

    def replay(self):
        """Runs the recorded call on the current stream and returns the (static) output tensors.  If
        the library's workspace changed since the capture, the call is first run eagerly (which sizes
        the workspace again) and recorded anew."""
        if not self.valid():
            self._op(*self._args, **self._kwargs)
            torch.cuda.synchronize(self.device)
            self._capture()
            self.recaptures += 1
        self.graph.replay()
        return self.outputs
