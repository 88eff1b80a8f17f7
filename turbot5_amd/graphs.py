"""Forward passes of fixed shape as one HIP graph.

A T5 encoder pass on a short input is a hundred launches of a few microseconds each; the host cannot
issue them as fast as the device retires them.  ``GraphedForward`` captures one call of a module on
static input buffers and replays it for every later call of the same shapes: the inputs are copied into
the static buffers, the graph runs, the static output is returned (valid until the next call).

Only tensors may vary between calls, and only in their values: shapes, dtypes, ``None``-ness and every
non-tensor argument are fixed at capture.  Host-side decisions of the module (is the mask all ones,
how many tokens are valid) are taken once, at capture, from the example inputs -- so a mask must keep
the pattern it had at capture.  Arguments that look like one ((B, L) tensors that are not integer ids:
floating, bool or int32 and smaller) are compared with the captured pattern on every call, which costs one
host synchronisation, and a different pattern raises.  Inference only.
"""
from __future__ import annotations

import torch


class GraphedForward:
    def __init__(self, module: torch.nn.Module, *example_args, **example_kwargs):
        self.module = module
        self._args = [a.clone() if torch.is_tensor(a) else a for a in example_args]
        self._kwargs = {k: (v.clone() if torch.is_tensor(v) else v) for k, v in example_kwargs.items()}
        tensors = [a for a in list(self._args) + list(self._kwargs.values()) if torch.is_tensor(a)]
        if not tensors or not all(t.is_cuda for t in tensors):
            raise ValueError("GraphedForward needs at least one tensor argument, all on a ROCm device")
        dev = tensors[0].device
        # the graph holds the addresses of the parameters: remember them to notice a module that moved
        self._weights = tuple(p.data_ptr() for p in module.parameters())
        with torch.no_grad():
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side):     # warm-up outside the capture: library handles, caches, allocator
                module(*self._args, **self._kwargs)
            torch.cuda.current_stream(dev).wait_stream(side)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.output = module(*self._args, **self._kwargs)

    @staticmethod
    def _load(static, new, name):
        if torch.is_tensor(static):
            if not torch.is_tensor(new) or new.shape != static.shape or new.dtype != static.dtype:
                raise ValueError(f"argument {name}: the captured graph takes a {tuple(static.shape)} {static.dtype} tensor")
            if static.dim() == 2 and static.dtype != torch.long and not torch.equal(new != 0, static != 0):
                raise ValueError(f"argument {name} looks like an attention mask and its pattern differs from the one "
                                 "the graph was captured with; capture a graph for this pattern or run the module itself")
            static.copy_(new)
        elif torch.is_tensor(new) or new != static:
            raise ValueError(f"argument {name} was {static!r} at capture and cannot change")

    def __call__(self, *args, **kwargs):
        if len(args) != len(self._args) or set(kwargs) != set(self._kwargs):
            raise ValueError("the captured graph takes the arguments of the example call")
        if tuple(p.data_ptr() for p in self.module.parameters()) != self._weights:
            raise RuntimeError("the module's parameters moved since the capture; build a new GraphedForward")
        for i, (s, n) in enumerate(zip(self._args, args)):
            self._load(s, n, i)
        for k, s in self._kwargs.items():
            self._load(s, kwargs[k], k)
        self.graph.replay()
        return self.output
