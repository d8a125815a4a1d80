"""Arrangement of the parts of one layer.

"prenorm": x += mixer(norm(x)); x += ffn(norm(x)) -- the order of the reference's layer
(src/transformer/cpu.c:536-939 and :1247-1303): norm, mixer, add, norm, feed-forward, add.
A layer without a feed-forward (ffn None; ffn_norm None with it) is the first half alone.
With output norms (mixer_out_norm, ffn_out_norm) a half's output goes through a norm of its own before it joins the
stream: x += norm_out(mixer(norm(x))).  The stream holds such an output back with its norm (NormedDelta), and the
kernel of the next norm forms the normed output, the sum and the next half's input in one pass."""
from __future__ import annotations

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, NormedDelta, Part, PartSpec


@BLOCKS.register("prenorm")
class PreNormBlock(Part):
    def __init__(self, mixer: PartSpec, ffn: PartSpec | None, mixer_norm: PartSpec, ffn_norm: PartSpec | None = None,
                 mixer_out_norm: PartSpec | None = None, ffn_out_norm: PartSpec | None = None):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("prenorm block: a feed-forward and its norm come together or not at all")
        if ffn is None and ffn_out_norm is not None:
            raise ValueError("prenorm block: an output norm of a feed-forward that is not there")
        self.mixer = MIXERS.build(mixer)
        self.ffn = FEED_FORWARDS.build(ffn) if ffn is not None else None
        self.mixer_norm = NORMS.build(mixer_norm)
        self.ffn_norm = NORMS.build(ffn_norm) if ffn_norm is not None else None
        self.mixer_out_norm = NORMS.build(mixer_out_norm) if mixer_out_norm is not None else None
        self.ffn_out_norm = NORMS.build(ffn_out_norm) if ffn_out_norm is not None else None
        for n in (self.mixer_out_norm, self.ffn_out_norm):
            if n is not None and not getattr(n, "normed_delta", False):
                raise ValueError("prenorm block: an output norm must be one that the stream can apply to a held-back output")

    @property
    def prompt_capturable(self) -> bool:
        return all(getattr(c, "prompt_capturable", False) for c in self.children().values())

    def children(self):
        c = {"mixer": self.mixer, "ffn": self.ffn, "mixer_norm": self.mixer_norm, "ffn_norm": self.ffn_norm,
             "mixer_out_norm": self.mixer_out_norm, "ffn_out_norm": self.ffn_out_norm}
        return {k: v for k, v in c.items() if v is not None}

    def linears(self):
        return [l for part in self.children().values() for l in getattr(part, "linears", list)()]

    def tensors(self):
        return {f"{cn}.{tn}": spec for cn, c in self.children().items() for tn, spec in c.tensors().items()}

    def load(self, tensors, device, dtype):
        for cn, c in self.children().items():
            c.load({k[len(cn) + 1:]: v for k, v in tensors.items() if k.startswith(cn + ".")}, device, dtype)

    def cache_need(self):
        return self.mixer.cache_need()

    def forward(self, stream, ctx, kv):
        # A part that says so may get its norm undone (it applies it inside its first product) and may hand
        # its last product in undone (it then adds itself to the stream): see ResidualStream.
        tap = getattr(ctx, "tap", None)        # diagnostics (StepContext.tap): the stream at the reference's three dump points
        if tap is not None:
            tap("layer_in", ctx.entry, stream, ctx)
        h = stream.normed(self.mixer_norm, ctx.act_dtype, consumer=self.mixer, ctx=ctx)
        if self.mixer_out_norm is not None:
            stream.add(NormedDelta(self.mixer.forward(h, ctx, kv), self.mixer_out_norm))
        elif getattr(self.mixer, "gives_lazy_delta", False):
            stream.add(self.mixer.forward(h, ctx, kv, lazy_ok=True))
        else:
            stream.add(self.mixer.forward(h, ctx, kv))
        if tap is not None:
            tap("ffn_in", ctx.entry, stream, ctx)
        if self.ffn is None:
            if tap is not None:
                tap("layer_out", ctx.entry, stream, ctx)
            return
        h = stream.normed(self.ffn_norm, ctx.act_dtype, consumer=self.ffn, ctx=ctx)
        if self.ffn_out_norm is not None:
            stream.add(NormedDelta(self.ffn.forward(h, ctx), self.ffn_out_norm))
        elif getattr(self.ffn, "gives_lazy_delta", False):
            stream.add(self.ffn.forward(h, ctx, lazy_ok=True))
        else:
            stream.add(self.ffn.forward(h, ctx))
        if tap is not None:
            tap("layer_out", ctx.entry, stream, ctx)
