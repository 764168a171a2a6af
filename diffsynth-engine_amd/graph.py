"""One denoising step recorded once as a HIP graph and replayed.

The block runners issue about 1500 kernel launches per Flux step from Python.  At 4096 + 512 tokens the
GPU is the slower side and the launches hide behind it; at small latents (or on a busy host) the host is
the slower side.  libdsx allocates nothing, synchronises nothing and launches on the stream it is handed,
so a whole ``runner(**inputs)`` call can be recorded into a graph on torch's capture stream and replayed
with one submission.  The reference has no counterpart (its loop is eager, pipelines/flux_image.py:506-533).

Recording fixes shapes, the runner's weights and every option that selects a kernel; only the contents of
the input tensors may change between replays.
"""
from typing import Dict

import torch


class GraphedStep:
    """``GraphedStep(runner, **example_inputs)`` records ``runner(**inputs)``; calling the object with
    tensors of the same shapes copies them into the recorded input buffers, replays the graph and returns
    the recorded output tensor (overwritten by the next replay: clone it to keep it)."""

    def __init__(self, runner, warmup: int = 2, **example_inputs):
        self.static_in: Dict[str, torch.Tensor] = {}
        self.other: Dict[str, object] = {}
        for k, v in example_inputs.items():
            if isinstance(v, torch.Tensor):
                if not v.is_cuda:
                    raise RuntimeError(f"GraphedStep: input '{k}' must be on the GPU (a host copy cannot be recorded)")
                self.static_in[k] = v.clone()
            else:
                self.other[k] = v
        # Lazy one-time work (kernel attribute set-up, device queries, torch's own workspace allocations) has
        # to happen before recording: run the step eagerly on a side stream first.
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(1, warmup)):
                runner(**self.static_in, **self.other)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.static_out = runner(**self.static_in, **self.other)

    def __call__(self, **inputs):
        for k, v in inputs.items():
            if k in self.static_in:
                buf = self.static_in[k]
                if v.shape != buf.shape:
                    raise ValueError(f"GraphedStep: '{k}' was recorded with shape {tuple(buf.shape)}, got {tuple(v.shape)}")
                buf.copy_(v)
            elif k not in self.other or self.other[k] is not v and self.other[k] != v:
                raise ValueError(f"GraphedStep: '{k}' is not a recorded tensor input and cannot change")
        self.graph.replay()
        return self.static_out
