"""Inference through a captured HIP graph: at small batch sizes a forward pass is ~250 short kernels and the
Python / launch overhead, not the GPU, sets the latency.  Capturing the pass once for a fixed input shape and
replaying it removes that overhead.  The library's kernels allocate nothing and record no memset, so they capture
as they are; what the surrounding torch ops record is their own business, which is why :class:`GraphedInference`
checks the first replays against eager results before it trusts the graph."""
from __future__ import annotations

import torch


class GraphedInference:
    """``model(x)`` (or ``model(x, lens)``) for one input shape, replayed from a captured graph.

    ``example`` fixes the shape and dtype of ``x`` (and ``lens``); ``autocast`` is the dtype the pass runs under.
    ``verify`` replays the graph that many times on perturbed inputs, with eager passes and synchronisations in
    between, and raises if a replay differs from the eager result by more than rounding - a graph that records
    an op which does not replay faithfully is not handed out.
    """

    def __init__(self, model, example, lens=None, autocast=torch.bfloat16, verify=3, warmup=3):
        assert not model.training, "graphed inference is for model.eval()"
        self.model, self.autocast = model, autocast
        self.x = example.clone()
        self.lens = None if lens is None else lens.clone()
        stream = torch.cuda.Stream(device=example.device)          # default priority
        stream.wait_stream(torch.cuda.current_stream(example.device))
        with torch.cuda.stream(stream):
            for _ in range(warmup):                                # allocator, library handles, prepared weights
                self._eager(self.x, self.lens)
        torch.cuda.current_stream(example.device).wait_stream(stream)
        torch.cuda.synchronize(example.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.out = self._eager(self.x, self.lens)
        for i in range(verify):
            x = example + 0.01 * (i + 1) * torch.randn_like(example)
            want = self._eager(x, lens)
            torch.cuda.synchronize(example.device)
            got = self(x, lens).clone()
            torch.cuda.synchronize(example.device)
            cos = torch.nn.functional.cosine_similarity(got.float(), want.float(), dim=-1).min().item()
            if not cos > 0.9999:
                raise RuntimeError("graph replay %d differs from the eager pass (cosine %.6f)" % (i, cos))

    def _eager(self, x, lens):
        with torch.no_grad(), torch.autocast(x.device.type, dtype=self.autocast):
            return self.model(x) if lens is None else self.model(x, lens)

    def __call__(self, x, lens=None):
        """Copies the inputs into the graph's buffers, replays, and returns the graph's output buffer (valid until
        the next call; clone it to keep it)."""
        assert x.shape == self.x.shape and (lens is None) == (self.lens is None)
        self.x.copy_(x)
        if lens is not None:
            self.lens.copy_(lens)
        self.graph.replay()
        return self.out
