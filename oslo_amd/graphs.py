"""Replaying a fused model's forward as one HIP graph.

Small models and short sequences are bound by kernel launches, not by the
kernels: a GPT-2-small forward of 2048 tokens is a few hundred launches of
microseconds each. Every kernel of this package only enqueues work on the
caller's stream and allocates nothing, so a whole forward can be captured once
with ``torch.cuda.CUDAGraph`` and replayed with one launch. The capture holds
the shapes, the mode (``eval``) and the weights' storage fixed; inputs are
copied into the captured input tensors before each replay and the outputs are
the captured output tensors, overwritten by the next call.
"""

import torch


class GraphedForward(object):
    """``graphed = GraphedForward(model, input_ids, attention_mask=...)`` captures
    ``model(*args, **kwargs)`` for tensors of these shapes and dtypes;
    ``graphed(input_ids, attention_mask=...)`` replays it. Tensor arguments may
    change in value between calls, not in shape; non-tensor arguments are fixed
    at capture. The result (any nesting of dicts, tuples, lists and tensors) is
    returned as captured: copy what has to outlive the next call."""

    def __init__(self, model, *args, warmup=3, **kwargs):
        if model.training:
            raise RuntimeError("GraphedForward captures inference: call model.eval() first "
                               "(dropout draws its Philox offsets on the host, outside any graph)")
        tensors = [a for a in list(args) + list(kwargs.values()) if isinstance(a, torch.Tensor)]
        if not tensors or not all(t.is_cuda for t in tensors):
            raise RuntimeError("GraphedForward needs its tensor arguments on a ROCm device")
        self._model = model
        self._args = tuple(a.clone() if isinstance(a, torch.Tensor) else a for a in args)
        self._kwargs = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in kwargs.items()}
        device = tensors[0].device
        # warm-up on a side stream: lazy initialisation (library handles, caches
        # of masks and tables) must not happen inside the capture
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(max(1, warmup)):
                model(*self._args, **self._kwargs)
        torch.cuda.current_stream(device).wait_stream(side)
        torch.cuda.synchronize(device)
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph), torch.no_grad():
            self._out = model(*self._args, **self._kwargs)

    @staticmethod
    def _copy_in(static, given, what):
        if isinstance(static, torch.Tensor):
            if not isinstance(given, torch.Tensor) or given.shape != static.shape or given.dtype != static.dtype:
                raise RuntimeError(f"{what}: the graph was captured for a {tuple(static.shape)} "
                                   f"{static.dtype} tensor")
            static.copy_(given)
        elif given != static:
            raise RuntimeError(f"{what}: non-tensor arguments are fixed at capture ({static!r})")

    def __call__(self, *args, **kwargs):
        if len(args) != len(self._args) or set(kwargs) != set(self._kwargs):
            raise RuntimeError("GraphedForward: call with the arguments it was captured with")
        for i, (static, given) in enumerate(zip(self._args, args)):
            self._copy_in(static, given, f"argument {i}")
        for k, given in kwargs.items():
            self._copy_in(self._kwargs[k], given, f"argument {k!r}")
        self._graph.replay()
        return self._out
