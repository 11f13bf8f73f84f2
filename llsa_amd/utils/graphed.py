"""A forward + backward step captured in one HIP graph.

The operators launch ~25 small kernels per step through Python; at the sizes where those
kernels take a few hundred microseconds in total, issuing them costs about as much host
time as they take to run.  Replaying a captured graph issues the whole step with one call.
Everything the kernels of this package do is capturable: no allocation inside the library,
no host synchronisation, no memset nodes, all work on the stream it is given (the lists for
the backward are built on a second stream that forks from and joins the capturing one).

Status: SWITCHED OFF.  Capture and replay were checked bit for bit against the eager step at
B=2,H=6,N=16384 (llsa_l2, top-k 16/16, RoPE) and B=4,H=6,N=4096 (llsa_l1, top-k 16), but at
B=1,H=2,N=16384 with top-k 8/4 the host process died twice inside torch.cuda.graph's capture_end
(hipStreamEndCapture) and the cause has not been found: reading the launch parameters of that
shape against the two that captured cleanly shows no empty grid, no dynamic-LDS attribute call
and no second stream in it.  Until a cause is shown the constructor raises; the class is not
exported by the package and nothing in it uses it.
"""
from __future__ import annotations

from typing import Callable, Sequence

import torch


class GraphedStep:
    """fn(*inputs) -> output, then output.backward(grad_out), captured once and replayed.

    `inputs` and `grad_out` are the static buffers of the graph: write new values into them
    (copy_) before replay().  After replay(), `output` and `grads` (one per input that requires
    grad, in order) hold the results; they are overwritten by the next replay."""

    def __init__(self, fn: Callable, inputs: Sequence[torch.Tensor], grad_out: torch.Tensor, warmup: int = 3):
        raise RuntimeError("GraphedStep is switched off: capturing one shape (B=1, H=2, N=16384, top-k 8/4) crashed the host "
                           "process inside hipStreamEndCapture and the cause is not known")
        self.inputs, self.grad_out = list(inputs), grad_out
        needs = [t for t in self.inputs if t.requires_grad]

        def step():
            for t in needs:
                t.grad = None
            out = fn(*self.inputs)
            out.backward(self.grad_out)
            return out

        # warm up on a side stream (allocator pools, lazy initialisation), as graph capture asks for
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                step()
        torch.cuda.current_stream().wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.output = step()
            self.grads = [t.grad for t in needs]
        for t in needs:             # the graph owns these buffers; do not leave them attached as .grad
            t.grad = None

    def replay(self):
        self.graph.replay()
        return self.output, self.grads
