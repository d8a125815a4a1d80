"""Configurations and model folders of the Sunusun tests: sizes of this file's own choosing and weights of its own making."""
import json
import math
import os

import torch


def _wkv(heads, dim, rank, ff=None, **kw):
    return dict(type="wkv", mixer=dict(heads=heads, dim=dim, decay_rank=rank), mlp=None if ff is None else dict(kind="dense", ff=ff), **kw)


def _par(heads, kv, dim, vdim, scale, coef, every, width, ff=None, **kw):
    return dict(type="parallel", mlp=None if ff is None else dict(kind="dense", ff=ff),
                mixer=dict(left=dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale, q_temp=dict(coef=coef, every=every)),
                           right=dict(width=width)), **kw)


# Sizes that differ from layer to layer and between the configurations: values wider and narrower than keys, one and three
# query heads per kv head, head counts and sizes that are no powers of two, an odd recurrence width, layers without a
# feed-forward, shared weights of either kind (also pointing forward), a parallel layer first and last.
CONFIGS = {
    "P": dict(architecture="Sunusun", vocab=97, width=64, norm=dict(eps=1e-5), logit_scale=0.5, layers=[
        _par(4, 2, 16, 24, 0.31, 0.2, 3, 40, ff=72),
        _wkv(2, 24, 8),
        _wkv(3, 20, 5, ff=50),
        _par(4, 2, 16, 24, 0.31, 0.2, 3, 40, ff=72, weights_of=0),
        _wkv(3, 20, 5, ff=50, weights_of=2)]),
    # recurrent layers alone (no keys or values anywhere: a cache without pages) and parallel layers alone
    "R": dict(architecture="Sunusun", vocab=50, width=40, norm=dict(eps=1e-5), logit_scale=0.7, layers=[
        _wkv(2, 16, 3, ff=48), _wkv(5, 8, 2), _wkv(2, 16, 3, ff=48, weights_of=0)]),
    "S": dict(architecture="Sunusun", vocab=70, width=24, norm=dict(eps=1e-5), logit_scale=1.5, layers=[
        _par(8, 1, 4, 2, 0.6, -0.2, 9, 8, ff=30), _par(2, 2, 32, 32, 0.2, 0.4, 100, 64)]),
    # the head sizes of real models (64 for the recurrence, 64 and 128 for attention: sizes at which other kernels of the
    # library would claim bf16 pages of another order), a parallel layer first, a feed-forward narrower than the width
    "T": dict(architecture="Sunusun", vocab=211, width=128, norm=dict(eps=1e-6), logit_scale=0.25, layers=[
        _par(4, 2, 64, 64, 0.125, 0.3, 16, 96, ff=64), _wkv(2, 64, 16, ff=192), _par(2, 1, 128, 32, 0.09, 0.2, 50, 128),
        _wkv(2, 64, 16, ff=192, weights_of=1)]),
    "Q": dict(architecture="Sunusun", vocab=131, width=48, norm=dict(eps=1e-6), logit_scale=1.0, layers=[
        _wkv(1, 32, 4, ff=64, weights_of=2),
        _par(3, 3, 8, 6, 0.9, 0.5, 1, 33),
        _wkv(1, 32, 4, ff=64),
        _par(6, 2, 10, 16, 0.5, 0.1, 40, 56, ff=40)]),
}


def write_folder(path, cfg, seed, dtype=torch.bfloat16, name_rank=True):
    """A model folder with weights of this file's own making: matrices N(0, 1/in), norm weights near 1, shift weights in
    (0, 1), decay offsets around -1, biases and bonuses of order 1/2, positive distance-bias numbers."""
    from bitnet_c_amd.config import SunusunConfig
    from bitnet_c_amd.config.sunusun import build_sunusun_plan
    from bitnet_c_amd.weights import write_file
    plan = build_sunusun_plan(SunusunConfig.from_dict(cfg))
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, spec in plan.expected_tensors().items():
        shape = tuple(spec.shape)
        leaf = name.split(".", 1)[1] if name.startswith("l") and name[1].isdigit() else name
        if leaf in ("norm1", "norm2") or name == "final.norm" or leaf.endswith(".norm") or leaf.endswith(".out"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif ".mu." in leaf:
            t = torch.rand(shape, generator=g)
        elif leaf.endswith("w0"):
            t = -1.0 + 0.7 * torch.randn(shape, generator=g)
        elif leaf.endswith(".u") or leaf.endswith(".b"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf.endswith("r1"):
            t = 0.4 * torch.rand(shape, generator=g)
        elif leaf.endswith("r2"):
            t = 0.05 + torch.rand(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        tensors[name] = t.to(dtype)
    os.makedirs(path, exist_ok=True)
    raw = json.loads(json.dumps(cfg))
    if not name_rank:                              # the rank of the decay projection is then read from the tensor's shape
        for L in raw["layers"]:
            L["mixer"].pop("decay_rank", None)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f)
    write_file(os.path.join(path, "model.safetensors"), tensors)
    return str(path)
