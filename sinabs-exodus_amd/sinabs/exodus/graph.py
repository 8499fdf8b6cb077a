"""Record one training-style step of a model with EXODUS layers into a HIP graph and replay it.

Every entry point of the kernel library only enqueues kernels on the stream it is handed, so a recording made
with ``torch.cuda.CUDAGraph`` holds the hand-written kernels themselves and a replay skips the host side of the
step altogether -- what a small layer needs, whose forward + backward pass is a few tens of microseconds of kernels
behind a few hundred microseconds of Python.  The reference has no counterpart.

    static_x = torch.zeros(batch, steps, features, device="cuda")
    def step():
        for layer in model: layer.reset_states() if hasattr(layer, "reset_states") else None
        out = model(static_x)
        loss_fn(out).backward()
        return out
    graphed = GraphedStep(model, step)
    for x in batches:
        static_x.copy_(x)
        out = graphed.replay()        # gradients are in the parameters' .grad tensors, as after step()

What the recording needs, and what ``GraphedStep`` takes care of:

* the warm-up passes and the capture run on ONE side stream.  Autograd binds the gradient accumulator of every
  parameter to the stream it was first used on; a capture on another stream would make the engine wait on a stream
  outside the capture, which ends the capture with an error;
* the layers' states and ``firing_rate`` carry the autograd graph of the last pass they saw (and with it every
  accumulator that pass created); they are detached before the warm-up -- a pass that the program ran earlier on
  another stream would otherwise hand its accumulators on to the warm-up's graph and from there to the capture's --
  and again before the capture, so the capture creates its own;
* the state tensors that exist at capture time are the ones the recording reads and zeroes; the layers replace them
  by new tensors during the pass, so the object keeps the old ones alive for as long as it lives;
* the ``.grad`` tensors are released before the capture, so the recorded pass creates them inside the graph's own
  memory pool and every replay writes them afresh (``optimizer.zero_grad(set_to_none=False)`` between replays would
  be wasted work; setting them to None would detach them from the graph).

The step must not make the host wait for the device.  The layers' range checks of decay factors, threshold and
lower bound do that once per parameter version, during the warm-up passes; after that they launch nothing.
"""
from typing import Any, Callable, Optional

import torch


class GraphedStep:
    def __init__(self, model: torch.nn.Module, step: Callable[[], Any], warmup: int = 3,
                 stream: Optional["torch.cuda.Stream"] = None):
        if warmup < 1:
            raise ValueError("at least one warm-up pass is needed (it also runs the layers' one-time range checks)")
        self.model, self.step = model, step
        self.stream = torch.cuda.Stream() if stream is None else stream
        self.stream.wait_stream(torch.cuda.current_stream())
        self._cut_loose()
        with torch.cuda.stream(self.stream):
            for _ in range(warmup):
                step()
                model.zero_grad(set_to_none=True)
            self._cut_loose()
        torch.cuda.current_stream().wait_stream(self.stream)
        self._held = list(model.buffers())
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=self.stream):
            self.output = step()

    def _cut_loose(self) -> None:
        """Detach everything the layers keep from their last pass: the states (``layer.zero_grad()``) and the
        firing rate, whose autograd graphs would keep that pass's gradient accumulators alive."""
        for m in self.model.modules():
            if hasattr(m, "reset_states"):
                m.zero_grad()
                rate = getattr(m, "firing_rate", None)
                if isinstance(rate, torch.Tensor) and rate.grad_fn is not None:
                    m.firing_rate = rate.detach()
                if getattr(m, "recordings", None):
                    m.recordings = {k: v.detach() for k, v in m.recordings.items()}

    def replay(self):
        """Run the recorded step once more on whatever the static input tensors hold now; returns the output
        tensor(s) of the recorded ``step`` (the same objects every time, rewritten by the replay)."""
        self.graph.replay()
        return self.output
