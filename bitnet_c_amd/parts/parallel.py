"""Two mixers side by side: both read the same input, each output goes through an RMSNorm of its own over the model
width (plain weights "left_out" / "right_out", eps inside the root), and the result is half their sum:

    y = 1/2 (rmsnorm(left(h)) * w_left + rmsnorm(right(h)) * w_right)

The two are any registered mixers; between them they may keep one set of keys and values and one state of fixed size
(the cache gives an entry of the schedule one of each), which is what an attention beside a recurrence needs.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import MIXERS, CacheNeed, ParamSpec, Part, PartSpec
from .linear import upload


@MIXERS.register("parallel")
class ParallelMixer(Part):
    def __init__(self, hidden: int, left: PartSpec, right: PartSpec, eps: float):
        self.hidden, self.eps = int(hidden), float(eps)
        self.left, self.right = MIXERS.build(left), MIXERS.build(right)
        needs = [self.left.cache_need(), self.right.cache_need()]
        if sum(n.kv is not None for n in needs) > 1 or sum(n.state is not None for n in needs) > 1:
            raise ValueError("parallel mixer: its two mixers may keep one set of keys and values and one state between them")
        self.w_left = self.w_right = None

    @property
    def prompt_capturable(self) -> bool:
        return all(getattr(m, "prompt_capturable", False) for m in (self.left, self.right))

    def children(self):
        return {"left": self.left, "right": self.right}

    def tensors(self):
        t = {f"{cn}.{tn}": spec for cn, c in self.children().items() for tn, spec in c.tensors().items()}
        t.update({"left_out": ParamSpec((self.hidden,), "ones"), "right_out": ParamSpec((self.hidden,), "ones")})
        return t

    def load(self, tensors, device, dtype):
        for cn, c in self.children().items():
            c.load({k[len(cn) + 1:]: v for k, v in tensors.items() if k.startswith(cn + ".")}, device, dtype)
        self.w_left = upload(tensors["left_out"], device, torch.float32)
        self.w_right = upload(tensors["right_out"], device, torch.float32)

    def linears(self):
        return [l for c in self.children().values() for l in c.linears()]

    def cache_need(self) -> CacheNeed:
        a, b = self.left.cache_need(), self.right.cache_need()
        return CacheNeed(kv=a.kv or b.kv, state=a.state or b.state)

    def forward(self, h, ctx, kv):
        a = self.left.forward(h, ctx, kv)
        b = self.right.forward(h, ctx, kv)
        return ops.rmsnorm_mean(a, self.w_left, b, self.w_right, self.eps)
