"""Replay of an inference forward as a HIP graph.

A forward over CACHED kernel maps queues a fixed sequence of launches: nothing is read back,
nothing depends on the host.  ``GraphedForward`` records that sequence once and replays it with one
call per forward, so the ~100 launches of a U-Net cost the host one launch: what remains is
the kernels' own time.  (A forward that BUILDS its maps cannot be recorded: the number of
output rows of every strided layer comes back to the host, and the sizes of everything after it
depend on it.)

    runner = GraphedForward(model, x)          # x: SparseTensor; builds the maps, records
    out = runner(new_feats)                    # same coordinates, new features

The recording runs on a stream of its own, and so do the warm-up forwards before it: the
library keeps its scratch buffers and per-map products per stream, and the warm-up leaves them
where the recording finds them (nothing is allocated for them while recording).  Replays are
ordered after the work queued on the caller's current stream and the caller's stream after the
replay.  The output tensors are the graph's own: a replay overwrites them, so copy what must
outlive the next call.

The recording holds ADDRESSES.  Those of the kernel maps stay valid because the input's caches
are kept here; those of buffers the library owns (a stream's scratch and tile counters, identity
maps, pair segments, grouped maps, packed weights) because every such tensor handed to a launch
during warm-up and recording is collected (``backend.pinned``) and referenced by this object:
``backend.release_scratch()`` and the eviction of the library's tables drop THEIR references, the
memory stays.  A replay first checks that the collected tensors still sit where they were
recorded (``resize_`` or ``set_`` on one of them would move it) and raises otherwise."""
from typing import Any, Callable, Optional

import torch

from torchsparse_amd import backend
from torchsparse_amd.tensor import SparseTensor

__all__ = ["GraphedForward"]


def _tensors_of(out) -> list:
    if isinstance(out, torch.Tensor):
        return [out]
    if isinstance(out, SparseTensor):
        return [out.feats]
    if isinstance(out, dict):
        return [t for v in out.values() for t in _tensors_of(v)]
    if isinstance(out, (list, tuple)):
        return [t for v in out for t in _tensors_of(v)]
    return []


class GraphedForward:
    """``fn(x)`` over the cached kernel maps of the SparseTensor ``x``, recorded as a HIP graph.

    ``fn`` is a module or any callable of one SparseTensor; it must run under ``torch.no_grad``
    semantics (inference) and must not synchronise.  ``warmup`` eager forwards run first (at
    least one: it builds and caches the kernel maps, packs the weights and sizes the scratch
    buffers)."""

    def __init__(self, fn: Callable[[SparseTensor], Any], x: SparseTensor, warmup: int = 2):
        if not x.feats.is_cuda:
            raise RuntimeError("GraphedForward needs GPU tensors")
        if warmup < 1:
            raise ValueError("at least one warm-up forward is needed: it builds the kernel maps")
        self.fn = fn
        self.feats = x.feats.detach().clone()  # the graph's input buffer
        self.x = SparseTensor._make(self.feats, x.coords, x.stride, x.spatial_range, x._caches)
        dev = x.feats.device
        caller = torch.cuda.current_stream(dev)
        self.stream = torch.cuda.Stream(device=dev)
        self.stream.wait_stream(caller)
        with backend.pinned() as held:
            with torch.no_grad(), torch.cuda.stream(self.stream):
                for _ in range(warmup):
                    fn(self.x)
            self.stream.synchronize()
            self.graph = torch.cuda.CUDAGraph()
            with torch.no_grad(), torch.cuda.graph(self.graph, stream=self.stream):
                self.out = fn(self.x)
        caller.wait_stream(self.stream)
        self._outputs = _tensors_of(self.out)
        # the library's buffers the recorded launches read and write, and where they were
        self.pinned = tuple(held)
        self._pinned_at = tuple(t.data_ptr() for t in held)

    def __call__(self, feats: Optional[torch.Tensor] = None):
        """Replay with ``feats`` (same shape and dtype as the recorded input; None: whatever the
        input buffer holds).  Returns the recorded output object, whose tensors now hold this
        replay's results."""
        if feats is not None:
            if feats.shape != self.feats.shape or feats.dtype != self.feats.dtype:
                raise ValueError(f"the graph was recorded for features of shape {tuple(self.feats.shape)} "
                                 f"and dtype {self.feats.dtype}")
            self.feats.copy_(feats)
        for t, at in zip(self.pinned, self._pinned_at):
            if t.data_ptr() != at:
                raise RuntimeError("a buffer this graph was recorded over has been moved (resize_/set_ on a "
                                   "tensor of the library): record a new GraphedForward")
        self.graph.replay()
        return self.out
