"""Configurations and model folders of the Sonodra tests: sizes of this file's own choosing and weights of its own making."""
import json
import math
import os

import torch


def _att(heads, kv, dim, vdim, scale, window, rot, mlp):
    m = dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale)
    if window:
        m["mask"] = dict(size=window)
    if rot:
        m["rot"] = dict(base=rot[0], dims=rot[1])
    return dict(type="attention", mixer=m, mlp=mlp)


def _lat(heads, dim, vdim, rank, scale, mlp, kv_from=None):
    m = dict(heads=heads, dim=dim, vdim=vdim, kv_rank=rank, scale=scale)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return dict(type="latent_attention", mixer=m, mlp=mlp)


def _dense(ff):
    return dict(kind="dense", ff=ff)


def _moe(experts, top, ff):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


# Sizes that differ from layer to layer and between the configurations: several kv heads and one, three and six query
# heads per kv head, values wider and narrower than keys, windows shorter than a page, longer than a page and of one
# token, a rotation over part of a head, over the whole head and none, latent widths that the matrix-core prompt kernel
# takes (32, 128) and that it does not (24, 8), several experts per token, all experts per token, a single expert, expert
# widths that the grouped products take and that they do not, layers without a feed-forward, a layer that reads another's
# latent vectors (also two that read the same), a latent layer first and last.
CONFIGS = {
    "A": dict(architecture="Sonodra", vocab=101, width=64, norm=dict(eps=1e-5), layers=[
        _att(4, 2, 16, 24, 0.3, 20, (10000.0, 8), _dense(72)),
        _lat(3, 16, 8, 32, 0.25, _moe(6, 2, 32)),
        _lat(2, 8, 16, 32, 0.4, _moe(5, 1, 40), kv_from=1),
        _att(4, 4, 16, 16, 0.25, 70, (300.0, 16), None)]),
    "B": dict(architecture="Sonodra", vocab=77, width=48, norm=dict(eps=1e-6), layers=[
        _lat(5, 12, 12, 24, 0.3, _dense(50)),
        _att(6, 1, 8, 6, 0.5, 3, (50.0, 2), _moe(3, 3, 16)),
        _att(2, 2, 32, 32, 0.2, 129, None, _moe(9, 4, 8)),
        _lat(1, 20, 30, 24, 0.2, None, kv_from=0)]),
    # the head sizes of real models: the matrix-core prompt kernels and the grouped products take every layer
    "C": dict(architecture="Sonodra", vocab=211, width=128, norm=dict(eps=1e-6), layers=[
        _att(4, 2, 64, 64, 0.125, 64, (500000.0, 32), _moe(8, 2, 64)),
        _lat(4, 64, 32, 128, 0.1, _dense(256)),
        _att(2, 1, 128, 128, 0.09, 100, (10000.0, 128), _moe(4, 1, 128)),
        _lat(2, 32, 64, 128, 0.15, _moe(16, 3, 32), kv_from=1),
        _lat(3, 32, 32, 128, 0.15, None, kv_from=1)]),
    # sizes that fit no kernel's favourite shape: a width that is no multiple of 8, seven and 32 heads, a latent 96 wide,
    # a rotation over 30 of 32 dimensions, a window of 33, three of eleven experts
    "E": dict(architecture="Sonodra", vocab=90, width=100, norm=dict(eps=1e-6), layers=[
        _lat(7, 18, 22, 96, 0.2, _moe(11, 3, 44)),
        _att(14, 7, 32, 64, 0.17, 33, (1e6, 30), _dense(130)),
        _att(8, 2, 96, 32, 0.1, 200, (1000.0, 96), _moe(5, 2, 72)),
        _lat(32, 8, 8, 96, 0.3, None, kv_from=0)]),
    # ones everywhere: one head, a window of one token (a query sees itself alone), one expert, a latent as wide as a head
    "D": dict(architecture="Sonodra", vocab=40, width=32, norm=dict(eps=1e-5), layers=[
        _att(1, 1, 8, 8, 0.35, 1, (100.0, 8), _moe(1, 1, 8)),
        _lat(1, 8, 8, 8, 1.0, _moe(2, 1, 4)),
        _att(3, 1, 6, 10, 0.4, 2, (7.0, 4), _dense(20))]),
}


def write_folder(path, cfg, seed, dtype=torch.bfloat16, overrides=None):
    """A model folder with weights of this file's own making: matrices N(0, 1/in), norm weights near 1, router rows three
    times larger (scores spread over (0, 1)), the embedding N(0, 1).  overrides: name -> tensor, put in place of what is drawn."""
    from bitnet_c_amd.config import SonodraConfig
    from bitnet_c_amd.config.sonodra import build_sonodra_plan
    from bitnet_c_amd.weights import write_file
    plan = build_sonodra_plan(SonodraConfig.from_dict(cfg))
    g = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, spec in plan.expected_tensors().items():
        shape = tuple(spec.shape)
        if len(shape) == 1:
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        elif name.endswith(".router"):
            t = 3.0 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        tensors[name] = t.to(dtype)
    for name, t in (overrides or {}).items():
        assert tuple(t.shape) == tuple(tensors[name].shape), name
        tensors[name] = t.to(dtype)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_file(os.path.join(path, "model.safetensors"), tensors)
    return str(path)


_settled = {}


def settled_tokens(folder, n, seed, margin=0.05):
    """n token ids for which no expert choice of the model in `folder` is a close call: built from left to right, a few
    tokens at a time; whatever follows the first token whose smallest routing margin (plain implementation, float64) is
    below `margin` of its logits' root mean square is drawn again.  Routing is causal, so a sequence's beginning stays settled
    however it goes on, and one sequence per (folder, seed) serves every length.  A model that rounds its activations to 8
    bits (its router's logits are then off by well under a hundredth of their size) chooses as the plain implementation
    does, and a difference between the two is a fault and not a coin that fell the other way."""
    import plain_sonodra as ps
    key = (folder, seed)
    if key not in _settled:
        _settled[key] = ([], torch.Generator().manual_seed(seed))
    toks, g = _settled[key]
    if len(toks) < n:
        cfg, W = ps.read_config(folder), ps.read_weights(folder)
        if not any(L.get("mlp") and L["mlp"]["kind"] == "moe" for L in cfg["layers"]):
            toks += torch.randint(0, cfg["vocab"], (n - len(toks),), generator=g).tolist()
        tries = 0
        while len(toks) < n:
            tries += 1
            assert tries < 100 * n, "no sequence without a close expert choice was found"
            more = torch.randint(0, cfg["vocab"], (min(16, n - len(toks)),), generator=g).tolist()
            margins = []
            ps.forward(cfg, W, toks + more, margins=margins)
            good = 0
            while good < len(more) and margins[len(toks) + good] >= margin:
                good += 1
            toks += more[:good]
    return list(toks[:n])
