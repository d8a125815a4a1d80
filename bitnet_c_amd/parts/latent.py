"""Latent attention: causal attention without positions whose keys and values are projections of one vector per token.

With h the mixer's input, per head i of n_heads (query/key size head_dim, value size v_head_dim):
    q_i = W_q,i h
    c   = rmsnorm(W_dkv h) * dkv_norm          the latent, kv_rank wide; eps inside the root, float32
    k_i = W_uk,i c;   v_i = W_uv,i c
    o_i = sum_j softmax_j((q_i . k_i,j) * scale) v_i,j       over the positions j <= the query's
    y   = W_o (concat(o) * sigmoid(W_g h))     the gate reads the mixer's input (gate False: no gate)

Only c is kept: the cache holds it as the one "kv head" of an attention whose keys and values are the same vectors
(a key row per position and, for the kernels' second product, the same numbers transposed inside the page).  Since k and
v are linear in c the mixer never forms them: the query goes into the latent's space, q'_i = W_uk,i^T q_i, all heads attend
over the cached c (score = q'_i . c_j), and the value projection runs on the attended latent, o_i = W_uv,i (sum_j p_j c_j).
That is the same sum in another order; scores, softmax and the norm are float32, the products accumulate in float32.
The attention itself is the attention mixer's general form (ops.attention / ops.attention_general_prompt) with one kv
head of size kv_rank and values as wide.

own_latent False: the layer has no W_dkv; its schedule entry reads the cache of the entry that has (ScheduleEntry.kv_from),
with its own W_uk and W_uv, queries, gate and output projection.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import MIXERS, CacheNeed, KVNeed, ParamSpec, Part
from .linear import Linear, upload


@MIXERS.register("latent_attention")
class LatentAttention(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    def __init__(self, hidden: int, n_heads: int, head_dim: int, kv_rank: int, scale: float, eps: float,
                 v_head_dim: int = 0, own_latent: bool = True, gate: bool = True):
        self.hidden, self.H, self.hs, self.rank = int(hidden), int(n_heads), int(head_dim), int(kv_rank)
        self.vd = int(v_head_dim) or self.hs
        self.scale, self.eps, self.own, self.gated = float(scale), float(eps), bool(own_latent), bool(gate)
        if self.rank % 2 or self.rank < 2 or self.rank > ops.MAX_HEAD_DIM:
            raise ValueError(f"latent attention: kv_rank {self.rank} is not supported by the attention kernels "
                             f"(even, at most {ops.MAX_HEAD_DIM})")
        if max(self.hs, self.rank) > ops.HEAD_LINEAR_MAX_IN:
            raise ValueError(f"latent attention: head_dim {self.hs} / kv_rank {self.rank} above {ops.HEAD_LINEAR_MAX_IN}")
        self.proj, self.o = Linear(), Linear()      # proj: [W_q; W_g; W_dkv] stacked, one product
        self.uk = self.uv_t = self.dkv_norm = None   # [H, head_dim, rank] and [H, rank, v_head_dim]: both [head, in, out]

    @property
    def q_dim(self):
        return self.H * self.hs

    @property
    def o_dim(self):
        return self.H * self.vd

    def tensors(self):
        D = self.hidden
        t = {"wq": ParamSpec((self.q_dim, D)), "wuk": ParamSpec((self.q_dim, self.rank)),
             "wuv": ParamSpec((self.o_dim, self.rank)), "wo": ParamSpec((D, self.o_dim))}
        if self.gated:
            t["wg"] = ParamSpec((self.o_dim, D))
        if self.own:
            t.update({"wdkv": ParamSpec((self.rank, D)), "dkv_norm": ParamSpec((self.rank,), "ones")})
        return t

    def load(self, tensors, device, dtype):
        names = ["wq"] + (["wg"] if self.gated else []) + (["wdkv"] if self.own else [])
        w = torch.cat([upload(tensors[n], device, dtype) for n in names], dim=0).contiguous()
        self.proj.load(w, None, device, dtype)
        self.o.load(tensors["wo"], None, device, dtype)
        # W_uk of head i is [head_dim, rank]: already [in, out] for q' = W_uk^T q; W_uv of head i is [v_head_dim, rank]:
        # turned once to [rank, v_head_dim]
        self.uk = upload(tensors["wuk"], device, dtype).reshape(self.H, self.hs, self.rank).contiguous()
        self.uv_t = upload(tensors["wuv"], device, dtype).reshape(self.H, self.vd, self.rank).transpose(1, 2).contiguous()
        if self.own:
            self.dkv_norm = upload(tensors["dkv_norm"], device, torch.float32)

    def linears(self):
        return [self.proj, self.o]

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv=KVNeed(1, self.rank, 0, v_head_dim=self.rank, v_layout="transposed"))

    def forward(self, h, ctx, kv):
        H, hs, vd, R = self.H, self.hs, self.vd, self.rank
        if isinstance(h, ops.DeferredNorm):
            h = h.materialize()
        if kv.writes != self.own:
            raise ValueError("latent attention: a layer with a down-projection writes its own cache, one without reads another's")
        p = self.proj(h)                                    # [T, H hs (+ H vd) (+ R)]
        if self.own:
            ops.latent_store(p, self.q_dim + (self.o_dim if self.gated else 0), R, self.dkv_norm, self.eps, ctx.positions,
                             ctx.seq_index, kv.block_table, kv.k_pages, kv.v_pages)
        q = ops.head_linear(p[:, :self.q_dim], self.uk)      # [T, H R]: the queries in the latent's space
        out = torch.empty((h.shape[0], H * R), dtype=h.dtype, device=h.device)
        on_matrix_cores = ops.attention_general_supported(h.dtype, R, R) and ops.GENERAL_PROMPT_ON_MATRIX_CORES
        if ctx.is_decode and on_matrix_cores:
            n_splits, chunk, _ = ops.general_decode_plan(ctx.n_rows, H, 1, kv.max_len)
            ops.attention_general_decode(q, out, kv.k_pages, kv.v_pages, kv.block_table, ctx.seq_lens, H, 1, R, R, self.scale,
                                         n_splits=n_splits, chunk=chunk, max_len_dev=ctx.max_len_dev if n_splits > 1 else None)
        elif ctx.is_decode:
            n_splits, chunk = ops.decode_splits(ctx.n_rows, H, 1, kv.max_len, h.dtype, target_wgs=ops.VECTOR_DECODE_TARGET_WGS)
            ops.attention(q, out, kv.k_pages, kv.v_pages, kv.block_table, H, 1, R, self.scale, seq_lens=ctx.seq_lens,
                          n_splits=n_splits, chunk=chunk, max_len_dev=ctx.max_len_dev if n_splits > 1 else None,
                          v_transposed=True, blocked=False, v_dim=R)
        elif on_matrix_cores:
            ops.attention_general_prompt(q, out, kv.k_pages, kv.v_pages, kv.block_table, H, 1, R, R, self.scale,
                                         ctx.tiles(ops.GENERAL_PROMPT_TILE))
        else:
            _, _, qt = ops.attention_row_shape(H, 1, False)
            ops.attention(q, out, kv.k_pages, kv.v_pages, kv.block_table, H, 1, R, self.scale, tiles=ctx.tiles(qt), qt=qt,
                          v_transposed=True, blocked=False, v_dim=R)
        gate = p[:, self.q_dim:self.q_dim + self.o_dim] if self.gated else None
        return self.o(ops.head_linear(out, self.uv_t, gate))
