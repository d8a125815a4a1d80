"""RMSNorm: out = x * 1/sqrt(mean(x^2) + eps) * w, eps inside the root
(src/transformer/rmsnorm_scalar.c:4-13).  Computed in float32 whatever the activation
type; the weight is kept in float32.  `scalar`: the model folder holds one number for all
coordinates (a tensor without dimensions); it is spread over the coordinates at load, and
every kernel that takes this norm, folded into a product or not, sees a weight vector."""
from __future__ import annotations

import torch

from .. import ops
from .base import NORMS, ParamSpec, Part
from .linear import upload


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone
    deferrable = True        # a product may fold this norm around itself (weight and eps are all it needs)
    takes_partial_sums = True    # apply() accepts ops.PartialSums as the delta
    normed_delta = True          # weight and eps are all that ops.add_normed_rmsnorm needs: it may be a block's output norm

    def __init__(self, dim: int, eps: float, scalar: bool = False):
        self.dim, self.eps, self.scalar = int(dim), float(eps), bool(scalar)
        self.weight = None

    def tensors(self):
        return {"weight": ParamSpec(() if self.scalar else (self.dim,), init="ones")}

    def load(self, tensors, device, dtype):
        w = upload(tensors["weight"], device, torch.float32)
        self.weight = w.reshape(1).expand(self.dim).contiguous() if self.scalar else w

    def apply(self, x, delta, out_dtype, rows=None):
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, out_dtype, rows)
