"""Plain, slow implementation of the Sonodra decoder, for tests only.

Whole sequences, no cache, nothing carried between calls, one function per mechanism, CPU tensors in float64.  It shares
no code with the package under test: its own reading of config.json, its own safetensors reading (through the
`safetensors` library), its own greedy loop.  Notation: h is a mixer's input [T, D]; positions count from 0; linear
weights are [out, in]; attention is written query by query, the way its definition reads.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def read_weights(folder: str) -> dict:
    from safetensors.torch import load_file
    return {k: v.to(F64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


# ---- small pieces ----------------------------------------------------------------------------------------------

def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis; eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softmax_over(scores: torch.Tensor) -> torch.Tensor:
    """Weights of lists of scores [..., n], each list by itself."""
    e = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
    return e / e.sum(dim=-1, keepdim=True)


def rotate_pairs(x: torch.Tensor, positions, dims: int, base: float, angle_dtype=F64) -> torch.Tensor:
    """x [T, heads, d] at the given positions [T]: dimensions 2i and 2i + 1 (i < dims / 2) of every head turned by the
    angle position * base^(-2i/dims); the rest of the vector passes.  angle_dtype float32: frequency and angle rounded as
    an engine that keeps them in 32 bits forms them."""
    out = x.clone()
    pos = torch.as_tensor(positions, dtype=F64).to(angle_dtype)
    for i in range(dims // 2):
        f = torch.tensor(float(base) ** (-2.0 * i / dims), dtype=F64).to(angle_dtype)
        a = (pos * f).to(F64)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * torch.cos(a) - v * torch.sin(a)
        out[..., 2 * i + 1] = v * torch.cos(a) + u * torch.sin(a)
    return out


# ---- mixers ----------------------------------------------------------------------------------------------------

def window_attention(h, W, p, m, eps, angle_dtype=F64):
    """Grouped-query attention over the last mask.size positions, with one norm over the whole query projection and one
    over the whole key projection, then a rotation of every head's first rot.dims dimensions."""
    T = h.shape[0]
    H, G, d, vd = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = unit_rms(h @ W[p + "q"].T, eps) * W[p + "q.norm"]
    k = unit_rms(h @ W[p + "k"].T, eps) * W[p + "k.norm"]
    v = (h @ W[p + "v"].T).reshape(T, G, vd)
    q, k = q.reshape(T, H, d), k.reshape(T, G, d)
    rot = m.get("rot")
    if rot:
        q = rotate_pairs(q, range(T), rot["dims"], rot["base"], angle_dtype)
        k = rotate_pairs(k, range(T), rot["dims"], rot["base"], angle_dtype)
    window = m["mask"]["size"] if m.get("mask") else T + 1
    out = torch.zeros(T, H, vd, dtype=F64)
    group = [a // (H // G) for a in range(H)]           # the kv head of every query head
    for t in range(T):
        first = max(0, t - window + 1)                  # j with 0 <= t - j < window
        keys, vals = k[first:t + 1, group], v[first:t + 1, group]                 # [n, H, d], [n, H, vd]
        w = softmax_over(torch.einsum("nhd,hd->hn", keys, q[t]) * m["scale"])    # [H, n]
        out[t] = torch.einsum("hn,nhe->he", w, vals)
    return out.reshape(T, H * vd) @ W[p + "o"].T


def latent_of(h, W, p, eps):
    """The normed down-projection that a latent attention layer keeps per token."""
    return unit_rms(h @ W[p + "dkv"].T, eps) * W[p + "dkv.norm"]


def latent_attention(h, c, W, p, m):
    """Causal attention whose keys and values of head a are W_uk[a] c and W_uv[a] c; no positions; an output gate that
    reads h."""
    T = h.shape[0]
    H, d, vd = m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = (h @ W[p + "q"].T).reshape(T, H, d)
    k = (c @ W[p + "uk"].T).reshape(T, H, d)
    v = (c @ W[p + "uv"].T).reshape(T, H, vd)
    out = torch.zeros(T, H, vd, dtype=F64)
    for t in range(T):
        w = softmax_over(torch.einsum("nhd,hd->hn", k[:t + 1], q[t]) * m["scale"])    # [H, n]
        out[t] = torch.einsum("hn,nhe->he", w, v[:t + 1])
    gated = out.reshape(T, H * vd) * sigmoid(h @ W[p + "g"].T)
    return gated @ W[p + "o"].T


# ---- feed-forwards -----------------------------------------------------------------------------------------------

def gated_ffn(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def expert(x, W, p):
    return (torch.clamp(x @ W[p + "up"].T, min=0.0) ** 2) @ W[p + "down"].T


def moe_ffn(h, W, p, m, margins: list | None = None):
    """Every token to its `top` experts of largest sigmoid score; the score multiplies what the expert reads.  margins
    collects, per token, how far the last chosen logit lies above the first one left out, over the logits' root mean
    square."""
    n, top = m["router"]["experts"], m["router"]["top"]
    z = h @ W[p + "router"].T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(n), key=lambda e: (-float(z[t, e]), e))
        for e in order[:top]:
            out[t] += expert(sigmoid(z[t, e]) * h[t], W, f"{p}e{e}.")
        if margins is not None:
            if top < n:
                margins.append(float(z[t, order[top - 1]] - z[t, order[top]]) / max(float(z[t].pow(2).mean().sqrt()), 1e-30))
            else:
                margins.append(float("inf"))              # every expert is chosen: nothing to decide
    return out


# ---- the model --------------------------------------------------------------------------------------------------

def forward(cfg: dict, W: dict, tokens, streams: list | None = None, angle_dtype=F64, margins: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] for one whole sequence; `streams` collects the residual stream after every layer, `margins`
    [T] the smallest routing margin of every token over the layers (moe_ffn)."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    latents = {}
    per_layer = []
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = unit_rms(x, eps) * W[p + "norm1"]
        if L["type"] == "attention":
            y = window_attention(h, W, p + "mix.", m, eps, angle_dtype)
        else:
            if "kv_from" in m:
                c = latents[m["kv_from"]]
            else:
                c = latents[i] = latent_of(h, W, p + "mix.", eps)
            y = latent_attention(h, c, W, p + "mix.", m)
        x = x + unit_rms(y, eps) * W[p + "norm1b"]
        if L.get("mlp") is not None:
            h = unit_rms(x, eps) * W[p + "norm2"]
            if L["mlp"]["kind"] == "dense":
                y = gated_ffn(h, W, p + "mlp.")
            else:
                mg = []
                y = moe_ffn(h, W, p + "mlp.", L["mlp"], mg)
                per_layer.append(mg)
            x = x + unit_rms(y, eps) * W[p + "norm2b"]
        if streams is not None:
            streams.append(x.clone())
    if margins is not None:
        margins.extend(min(col) for col in zip(*per_layer)) if per_layer else margins.extend([float("inf")] * len(tokens))
    return (unit_rms(x, eps) * W["final.norm"]) @ W["head"].T


def generate(cfg: dict, W: dict, prompt, n_new: int) -> list:
    """Greedy: the largest logit, ties to the lower index."""
    seq, out = list(prompt), []
    for _ in range(n_new):
        tok = int(torch.argmax(forward(cfg, W, seq)[-1]))
        out.append(tok)
        seq.append(tok)
    return out
