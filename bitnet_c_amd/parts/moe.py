"""Mixture-of-experts feed-forward: n_experts small feed-forwards without a gate, of which every token uses top_k.

    z = W_router h                         float32 (h in the activations' type)
    s = sigmoid(z)   or   softmax(z)       `scoring`
    the top_k experts with the largest scores; their weights w are the scores themselves, or, with `renormalize`, the
    scores divided by their sum
    y = sum over the chosen e of  W_down,e act(W_up,e (w_e h))     weight_on "input": the weight multiplies what the expert reads
      = sum over the chosen e of  w_e W_down,e act(W_up,e h)       weight_on "output"

The experts' matrices are stacked on the device ([E, F, D] and [E, D, F]); the model folder holds them one by one
(e<n>.w_up [F, D], e<n>.w_down [D, F]).  The router runs one workgroup a token and chooses on the device; steps of few rows
read each chosen expert once per (token, choice) pair (ops.moe_experts), steps of many rows order the pairs by expert and
run the two products as grouped matrix products over tiles whose rows share an expert (ops.moe_experts_grouped).  Nothing waits
for the host, so the part's steps are captured like any other.  The result is handed on as the top_k slabs of float32
rows (ops.PartialSums) that the consumer's kernel adds.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import FEED_FORWARDS, ParamSpec, Part
from .linear import upload


@FEED_FORWARDS.register("moe")
class MoEFFN(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    def __init__(self, hidden: int, n_experts: int, top_k: int, intermediate: int, activation: str = "relu2",
                 scoring: str = "sigmoid", renormalize: bool = False, weight_on: str = "input"):
        if activation not in ops.UNARY_ACTIVATIONS:
            raise ValueError(f"moe: unknown activation {activation!r}; known: {sorted(ops.UNARY_ACTIVATIONS)}")
        if scoring not in ops.MOE_SCORINGS:
            raise ValueError(f"moe: unknown scoring {scoring!r}; known: {sorted(ops.MOE_SCORINGS)}")
        if weight_on not in ("input", "output"):
            raise ValueError(f"moe: weight_on {weight_on!r} is neither 'input' nor 'output'")
        self.hidden, self.E, self.K, self.F = int(hidden), int(n_experts), int(top_k), int(intermediate)
        if not 1 <= self.K <= self.E or self.E > ops.MOE_MAX_EXPERTS:
            raise ValueError(f"moe: top_k {self.K} of {self.E} experts (at most {ops.MOE_MAX_EXPERTS})")
        self.activation, self.scoring, self.renormalize = activation, scoring, bool(renormalize)
        self.weight_on_input = weight_on == "input"
        self.router = self.w_up = self.w_down = None

    def tensors(self):
        t = {"router": ParamSpec((self.E, self.hidden))}
        for e in range(self.E):
            t[f"e{e}.w_up"] = ParamSpec((self.F, self.hidden))
            t[f"e{e}.w_down"] = ParamSpec((self.hidden, self.F))
        return t

    def load(self, tensors, device, dtype):
        self.router = upload(tensors["router"], device, torch.float32)
        self.w_up = torch.empty((self.E, self.F, self.hidden), dtype=dtype, device=device)
        self.w_down = torch.empty((self.E, self.hidden, self.F), dtype=dtype, device=device)
        for e in range(self.E):                              # one by one: the host holds no stacked copy
            self.w_up[e].copy_(upload(tensors[f"e{e}.w_up"], device, dtype))
            self.w_down[e].copy_(upload(tensors[f"e{e}.w_down"], device, dtype))

    def forward(self, h, ctx, lazy_ok: bool = False):
        if isinstance(h, ops.DeferredNorm):
            h = h.materialize()
        ids, wts = ops.moe_route(h, self.router, self.K, self.scoring, self.renormalize)
        if ops.moe_grouped_supported(h.shape[0], self.hidden, self.F, h.dtype):
            return ops.moe_experts_grouped(h, self.w_up, self.w_down, ids, wts, self.activation, self.weight_on_input)
        return ops.moe_experts(h, self.w_up, self.w_down, ids, wts, self.activation, self.weight_on_input)
