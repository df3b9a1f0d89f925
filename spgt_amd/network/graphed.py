"""HIP-graph replay of an inference forward.

A forward of the accelerated model is ~100 short launches; issuing them from Python takes about as long
as the GPU needs to run them.  `GraphedInference` records one forward (fixed shapes, no autograd) into a
HIP graph through torch's stream capture and replays it: one host call per forward.  Everything the
library launches goes to torch's current stream and takes its scratch from torch's caching allocator,
so its kernels are captured like torch's own.
"""
from typing import Sequence

import torch
from torch import Tensor, nn


class GraphedInference:
    """`g = GraphedInference(model, *example_inputs)`; `g(*inputs)` copies the inputs into the captured
    buffers, replays the graph and returns the captured output tensor(s), which the next call overwrites.

    Inputs must keep the example's shapes and dtypes.  Every replay reads the module's parameters where they
    were at capture: kernels that take a parameter as stored read it in place, and the launch that rewrites the
    derived layouts (transposed and packed weights, see derived.py) is part of the graph.  In-place updates
    (optimizer steps, `copy_`, writes through `.data`, `load_state_dict`) are therefore seen by the next replay;
    a parameter that moves to new storage (`.to()`, `load_state_dict(assign=True)`) needs a new capture."""

    def __init__(self, module: nn.Module, *example_inputs: Tensor, warmup: int = 3) -> None:
        if not example_inputs or not all(isinstance(x, Tensor) and x.is_cuda for x in example_inputs):
            raise ValueError("GraphedInference needs example inputs on a GPU")
        self.module = module
        self.static_inputs = [x.detach().clone() for x in example_inputs]
        device = example_inputs[0].device
        with torch.no_grad(), torch.cuda.device(device):
            # library autotuning, lazy initialisation and the allocator's growth happen outside the capture
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(max(1, warmup)):
                    module(*self.static_inputs)
            torch.cuda.current_stream().wait_stream(side)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self.static_output = module(*self.static_inputs)

    def __call__(self, *inputs: Tensor):
        if len(inputs) != len(self.static_inputs):
            raise ValueError(f"expected {len(self.static_inputs)} inputs, got {len(inputs)}")
        for dst, src in zip(self.static_inputs, inputs):
            if src.shape != dst.shape or src.dtype != dst.dtype:
                raise ValueError(f"input of shape {tuple(src.shape)} / {src.dtype} does not match the captured "
                                 f"{tuple(dst.shape)} / {dst.dtype}")
            if src.data_ptr() != dst.data_ptr():
                dst.copy_(src)
        self.graph.replay()
        return self.static_output
