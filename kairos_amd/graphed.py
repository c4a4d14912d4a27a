"""HIP-graph replay of a fixed sequence of switched linears.

Decode-sized calls are bound by the host (about 9 us of Python, allocation and launch per linear against
4-15 us of kernel time), not by the kernels.  A caller whose step has fixed shapes -- one decode step at a
given batch size -- can capture it once and replay it with a single graph launch.  The lookup table is
consulted while capturing, so a graph is tied to the M it was captured with: capture one per batch bucket,
exactly as serving stacks do with CUDA graphs.

Capture rules this module enforces or relies on:
  * every kernel of the library launches on torch's current stream, so torch's stream capture records it;
  * the library records no memset nodes (none of its entry points clears memory);
  * the temp cache is created BEFORE capture, by warm-up calls on the capture stream (it must not come from the
    graph's private pool: it is shared with eager calls);
  * the split-K and small-M scratch of the captured kernels belongs to the GraphedCallable (an ops.Scratch made or
    given at construction), not to a stream: a replay runs on whatever stream is current, so scratch looked up by
    the capture stream's handle could be in use by eager work, or by another graph, on a different stream at that
    moment.  Replays of ONE instance, and of instances that share a Scratch, must be ordered on one stream;
  * the temp cache is invalidated right before capture, so every conversion the step needs is part of the
    graph, and after every replay, because the graph rewrites the cache behind the host-side tag's back;
  * inputs are copied into static buffers before each replay; outputs are the static tensors captured.
"""
import torch

from . import ops
from .temp_cache import default_cache


class GraphedCallable:
    """Captures `fn(*static_inputs)` once; `__call__(*inputs)` copies the inputs in and replays.

    `fn` must be a pure function of its tensor arguments over modules of this package (fixed shapes, no
    host-side data dependence).  The returned tensors are reused by every replay: consume or clone them
    before the next call.
    """

    def __init__(self, fn, example_inputs, warmup=3, caches=None, scratch=None):
        """caches: the TempCache objects the captured modules use (default: the process-wide one).  scratch: the
        ops.Scratch whose buffers the captured kernels use (default: a new one, 96 MiB, owned by this instance);
        pass one Scratch to several instances whose replays are ordered on one stream (e.g. the batch buckets of
        one decode loop) to share it."""
        if not torch.cuda.is_available():
            raise RuntimeError("GraphedCallable: needs a GPU")
        self._static_in = [x.clone() for x in example_inputs]
        self.scratch = scratch if scratch is not None else ops.Scratch(self._static_in[0].device)
        side = torch.cuda.Stream()                      # default priority; warm-up AND capture run on it
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), self.scratch:
            for _ in range(warmup):                     # sizes the temp cache and settles the LUT memo
                fn(*self._static_in)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self._caches = list(caches) if caches is not None else [default_cache()]
        self._invalidate()
        for c in self._caches:
            c.prepare_for_capture(self._static_in[0].device)
        self._graph = torch.cuda.CUDAGraph()
        with self.scratch, torch.cuda.graph(self._graph, stream=side):
            self._static_out = fn(*self._static_in)
        self._invalidate()
        self.replays = 0

    def _invalidate(self):
        dev = self._static_in[0].device
        for c in self._caches:
            c.invalidate()
            c.touch(dev)                                # the replay used the cache's buffer on the current stream

    def __call__(self, *inputs):
        if len(inputs) != len(self._static_in):
            raise ValueError(f"GraphedCallable: captured with {len(self._static_in)} inputs, got {len(inputs)}")
        for dst, src in zip(self._static_in, inputs):
            if dst.shape != src.shape or dst.dtype != src.dtype:
                raise ValueError(f"GraphedCallable: captured for {tuple(dst.shape)} {dst.dtype}, "
                                 f"got {tuple(src.shape)} {src.dtype}")
            if dst.data_ptr() != src.data_ptr():
                dst.copy_(src)
        self._graph.replay()
        self._invalidate()
        self.replays += 1
        return self._static_out

    def replay(self):
        """Replays on the inputs already in the static buffers (no copies)."""
        self._graph.replay()
        self._invalidate()
        self.replays += 1
        return self._static_out

    @property
    def static_inputs(self):
        return self._static_in


def graph_layer(linears, example_input_for, scratch=None):
    """Convenience: one graph over `[lin(x) for lin in linears]`, `example_input_for(lin)` giving each input."""
    xs = [example_input_for(l) for l in linears]

    def step(*inputs):
        return tuple(l(x) for l, x in zip(linears, inputs))

    return GraphedCallable(step, xs, scratch=scratch)
