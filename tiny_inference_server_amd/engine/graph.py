"""Captured decode steps.

A step in which every request brings exactly one token, far enough into its sequence that every stage has
one row per request, always launches the same kernels on arrays of the same shapes. Such a step is
captured once per (number of requests, block-table width) as a HIP graph over a fixed device buffer that
holds the step's integer arrays; later steps of the same shape copy their arrays into that buffer and
replay the graph, which removes the launch cost of several hundred small kernels.

Nothing is cleared inside the graph with a memset, and the first step of a shape runs without a graph (it
also sizes the kernels' workspace), so a capture records kernel launches only.
"""
from __future__ import annotations

import torch

from .batch import StepPlan, materialize


class DecodeGraph:
    def __init__(self, engine, plan: StepPlan, kv_capacity: int):
        self.layout = plan.layout()
        dev = engine.device
        self.host = torch.zeros(max(plan.packer.total, 4), dtype=torch.int32, pin_memory=True)
        self.dev = torch.zeros(max(plan.packer.total, 4), dtype=torch.int32, device=dev)
        self.copied = torch.cuda.Event()
        self.step = materialize(plan, dev, self.host, self.dev)
        for st in self.step.stages:
            st.max_kv_len = kv_capacity
        n = self.step.n_wanted
        self.graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize(dev)
        with torch.cuda.graph(self.graph):
            outs = engine.model.forward(self.step, engine.cache)
            self.logits = engine.model.logits(outs[0].hidden, self.step.stages[0].want_index, n)
        self.copied.record()

    def run(self, plan: StepPlan) -> torch.Tensor:
        if plan.layout() != self.layout:
            raise RuntimeError("this step's arrays do not have the captured layout")
        self.copied.synchronize()            # the previous copy out of the pinned buffer has finished
        plan.packer.fill(self.host)
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()
        self.graph.replay()
        return self.logits
