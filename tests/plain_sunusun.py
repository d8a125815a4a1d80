"""Plain, slow implementation of the Sunusun decoder, for tests only.

Whole sequences, no cache, no state carried between calls, one function per mechanism, CPU tensors in float64.  It
shares no code with the package under test: its own reading of config.json, its own safetensors reading (through the
`safetensors` library), its own greedy loop.  Notation: h is a mixer's input [T, D]; positions count from 0; linear
weights are [out, in].
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


def sinusoid(n_tokens: int, width: int, angle_dtype=F64) -> torch.Tensor:
    """[T, width]: entry 2i = sin(p / 10000^(2i/width)), entry 2i+1 = cos of the same angle.  angle_dtype float32: the
    frequency and the angle p * frequency are rounded to float32, as an engine that keeps positions and angles in 32
    bits forms them (at position 2,000 that alone moves an angle by 1e-4)."""
    out = torch.zeros(n_tokens, width, dtype=F64)
    for e in range(width):
        i = e // 2
        freq = torch.tensor(10000.0 ** (-2.0 * i / width), dtype=F64).to(angle_dtype)
        angle = (torch.arange(n_tokens, dtype=angle_dtype) * freq).to(F64)
        out[:, e] = torch.sin(angle) if e % 2 == 0 else torch.cos(angle)
    return out


def gelu_exact(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def dense_ffn(h, w_up, w_down):
    return gelu_exact(h @ w_up.T) @ w_down.T


# ---- wkv --------------------------------------------------------------------------------------------------------

def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """h_t + (h_{t-1} - h_t) * mu, with h_{-1} = 0."""
    before = torch.zeros_like(h)
    before[1:] = h[:-1]
    return h + (before - h) * mu


def wkv_decay(x_w, w1, w2, w0):
    """exp(-exp(W2 tanh(W1 x) + w0)): a number in (0, 1) per head and key channel."""
    return torch.exp(-torch.exp(torch.tanh(x_w @ w1.T) @ w2.T + w0))


def wkv_recurrence(r, k, v, w, u):
    """r, k, v, w: [T, H, d]; u: [H, d].  Token by token, per head, with S [d, d] starting at zero:
    o_t[j] = sum_i r_t[i] (S[i, j] + u[i] k_t[i] v_t[j]);  then S[i, j] <- w_t[i] S[i, j] + k_t[i] v_t[j]."""
    T, H, d = r.shape
    o = torch.zeros(T, H, d, dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, d, dtype=F64)
        for t in range(T):
            outer = k[t, hd][:, None] * v[t, hd][None, :]
            o[t, hd] = r[t, hd] @ (S + u[hd][:, None] * outer)
            S = w[t, hd][:, None] * S + outer
    return o


def wkv_mixer(h, W, p, heads, dim, eps):
    T = h.shape[0]
    x = {s: token_shift(h, W[p + "mu." + s]) for s in "rkvgw"}
    r = (x["r"] @ W[p + "r"].T).view(T, heads, dim)
    k = (x["k"] @ W[p + "k"].T).view(T, heads, dim)
    v = (x["v"] @ W[p + "v"].T).view(T, heads, dim)
    gate = silu(x["g"] @ W[p + "g"].T)
    w = wkv_decay(x["w"], W[p + "w1"], W[p + "w2"], W[p + "w0"]).view(T, heads, dim)
    o = wkv_recurrence(r, k, v, w, W[p + "u"])
    o = unit_rms(o, eps).reshape(T, heads * dim) * W[p + "norm"] * gate
    return o @ W[p + "o"].T


# ---- the attention of a parallel layer ---------------------------------------------------------------------------

def query_temperature(n_tokens: int, coef: float, every: int) -> torch.Tensor:
    p = torch.arange(n_tokens)
    return 1.0 + coef * torch.log(torch.div(p + 1, every, rounding_mode="floor").to(F64) + 1.0)


def distance_bias(n_tokens: int, a: float, b: float) -> torch.Tensor:
    """[T, T]: a * ln(1 + b * (i - j)) for j <= i (0 elsewhere; those places are masked)."""
    p = torch.arange(n_tokens)
    dist = (p[:, None] - p[None, :]).clamp(min=0).to(F64)
    return a * torch.log(1.0 + b * dist)


def sink_softmax(scores: torch.Tensor, visible: torch.Tensor) -> torch.Tensor:
    """exp(s_j) / (1 + sum over visible j of exp(s_j)), row by row; 0 where not visible."""
    e = torch.where(visible, torch.exp(scores), torch.zeros_like(scores))
    return e / (1.0 + e.sum(dim=-1, keepdim=True))


def attention_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ W[p + "q"].T).view(T, H, d), eps) * W[p + "q.norm"]
    k = unit_rms((h @ W[p + "k"].T).view(T, G, d), eps) * W[p + "k.norm"]
    v = (h @ W[p + "v"].T).view(T, G, vd)
    q = q * query_temperature(T, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    pos = torch.arange(T)
    visible = pos[:, None] >= pos[None, :]
    out = torch.zeros(T, H, vd, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"] - distance_bias(T, float(W[p + "r1"][hd]), float(W[p + "r2"][hd]))
        out[:, hd] = sink_softmax(s, visible) @ v[:, g]
    return out.reshape(T, H * vd) @ W[p + "o"].T


# ---- min-GRU --------------------------------------------------------------------------------------------------

def mingru_mixer(h, W, p):
    z = torch.sigmoid(h @ W[p + "z"].T + W[p + "z.b"])
    c = h @ W[p + "x"].T + W[p + "x.b"]
    cand = torch.where(c >= 0, c + 0.5, torch.sigmoid(c))
    gate = silu(h @ W[p + "g"].T)
    S = torch.zeros(z.shape[1], dtype=F64)
    y = torch.zeros_like(z)
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        y[t] = S * gate[t]
    return y @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    a = attention_mixer(h, W, p + "left.", m["left"], eps)
    b = mingru_mixer(h, W, p + "right.")
    return 0.5 * (unit_rms(a, eps) * W[p + "left.out"] + unit_rms(b, eps) * W[p + "right.out"])


# ---- the model --------------------------------------------------------------------------------------------------

def forward(cfg: dict, W: dict, tokens, streams: list | None = None, angle_dtype=F64) -> torch.Tensor:
    """Logits [T, vocab] for one whole sequence; `streams` collects the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(list(tokens), dtype=torch.long)] + sinusoid(len(tokens), cfg["width"], angle_dtype)
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % L.get("weights_of", i)
        h = unit_rms(x, eps) * W[p + "norm1"]
        if L["type"] == "wkv":
            x = x + wkv_mixer(h, W, p + "mix.", L["mixer"]["heads"], L["mixer"]["dim"], eps)
        else:
            x = x + parallel_mixer(h, W, p + "mix.", L["mixer"], eps)
        if L.get("mlp") is not None:
            h = unit_rms(x, eps) * W[p + "norm2"]
            x = x + dense_ffn(h, W[p + "mlp.up"], W[p + "mlp.down"])
        if streams is not None:
            streams.append(x.clone())
    return (unit_rms(x, eps) * W["final.norm"]) @ W["head"].T * cfg.get("logit_scale", 1.0)


def generate(cfg: dict, W: dict, prompt, n_new: int) -> list:
    """Greedy: the largest logit, ties to the lower index."""
    seq, out = list(prompt), []
    for _ in range(n_new):
        tok = int(torch.argmax(forward(cfg, W, seq)[-1]))
        out.append(tok)
        seq.append(tok)
    return out
