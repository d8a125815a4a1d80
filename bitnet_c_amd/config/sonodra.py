"""Sonodra: a decoder whose config.json lists its layers one by one.  Every layer is a block with a norm in front of and
behind each of its two halves (parts/block.py, "prenorm" with output norms):

    x += norm1b(mixer(norm1(x)));   x += norm2b(ff(norm2(x)))          all four plain RMSNorms with weights [width]

Two kinds of mixers:

  "attention"         grouped-query attention over a sliding window: an RMSNorm over the whole query projection and one
                      over the whole key projection (weights as wide as the projection), then a rotation of the first
                      rot.dims dimensions of every head in neighbouring pairs (2i, 2i + 1), value heads of a width of
                      their own (parts/attention.py)
  "latent_attention"  causal attention without positions whose keys and values are both projections of one normed latent
                      vector per token, which is all the cache keeps; an output gate; a layer that says "kv_from": j
                      reads layer j's latent vectors and has no down-projection of its own (parts/latent.py)

and two kinds of feed-forwards: "dense" (silu-gated) and "moe" (experts without a gate, squared relu, chosen by the
largest sigmoid scores, the score multiplying the expert's input; parts/moe.py); "mlp": null leaves the second half out.

config.json keys: architecture, vocab, width, norm.eps, layers[] = {type, mixer, mlp} with
  attention mixer         {heads, kv_heads, dim, vdim, scale, mask: {size}, rot: {base, dims}}
  latent_attention mixer  {heads, dim, vdim, kv_rank, scale, kv_from?}
  mlp                     {kind: "dense", ff} | {kind: "moe", expert: {ff}, router: {experts, top}} | null

Tensor names of the folder (linear weights [out, in]): embed, head, final.norm, and for layer i under l<i>.:
  norm1, norm1b, norm2, norm2b
  attention:         mix.{q,k,v,o}, mix.q.norm, mix.k.norm
  latent_attention:  mix.{q,uk,uv,g,o} and, unless kv_from, mix.dkv, mix.dkv.norm
  dense:             mlp.{gate,up,down}
  moe:               mlp.router, mlp.e<n>.{up,down}
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple, Union

from ..engine.plan import LayerPlan, ModelPlan, ScheduleEntry
from ..parts.base import PartSpec
from .base import Architecture, ConfigError, _positive_int, register_architecture

NAME = "Sonodra"


def _number(raw: dict, key: str, what: str, positive: bool = True) -> float:
    v = raw.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not v > 0):
        raise ConfigError(f"config.json: {what}.{key} must be a {'positive ' if positive else ''}number, got {v!r}")
    return float(v)


def _object(raw, what: str) -> dict:
    if not isinstance(raw, dict):
        raise ConfigError(f"config.json: {what} must be an object, got {raw!r}")
    return raw


@dataclass(frozen=True)
class WindowAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int                 # 0: every earlier position is visible
    rot_base: float
    rot_dims: int               # 0: no rotation

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.window:
            d["mask"] = {"size": self.window}
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return d


@dataclass(frozen=True)
class LatentAttentionSizes:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    kv_from: Optional[int] = None

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "kv_rank": self.kv_rank, "scale": self.scale}
        if self.kv_from is not None:
            d["kv_from"] = self.kv_from
        return d


@dataclass(frozen=True)
class DenseSizes:
    ff: int

    def to_dict(self):
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class MoeSizes:
    experts: int
    top: int
    ff: int

    def to_dict(self):
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class SonodraLayer:
    type: str                                                   # "attention" | "latent_attention"
    mixer: Union[WindowAttentionSizes, LatentAttentionSizes]
    mlp: Union[DenseSizes, MoeSizes, None]

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class SonodraConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[SonodraLayer, ...]

    MIXER_TYPES = ("attention", "latent_attention")
    MLP_KINDS = ("dense", "moe")

    @staticmethod
    def _mixer(kind: str, raw, where: str, n_layers: int, index: int):
        m = _object(raw, where + ".mixer")
        heads, dim = _positive_int(m, "heads"), _positive_int(m, "dim")
        vdim = _positive_int(m, "vdim", dim)
        scale = _number(m, "scale", where + ".mixer")
        if kind == "attention":
            kv_heads = _positive_int(m, "kv_heads", heads)
            if heads % kv_heads:
                raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
            window = _positive_int(_object(m["mask"], where + ".mixer.mask"), "size") if m.get("mask") is not None else 0
            base, dims = 0.0, 0
            if m.get("rot") is not None:
                rot = _object(m["rot"], where + ".mixer.rot")
                base, dims = _number(rot, "base", where + ".mixer.rot"), _positive_int(rot, "dims")
                if dims % 2 or dims > dim:
                    raise ConfigError(f"config.json: {where}.mixer.rot.dims {dims} must be even and at most dim {dim}")
            return WindowAttentionSizes(heads, kv_heads, dim, vdim, scale, window, base, dims)
        src = m.get("kv_from")
        if src is not None and (isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < n_layers or src == index):
            raise ConfigError(f"config.json: {where}.mixer.kv_from {src!r} names no other layer")
        return LatentAttentionSizes(heads, dim, vdim, _positive_int(m, "kv_rank"), scale, src)

    @classmethod
    def _mlp(cls, raw, where: str):
        if raw is None:
            return None
        m = _object(raw, where + ".mlp")
        kind = m.get("kind")
        if kind == "dense":
            return DenseSizes(_positive_int(m, "ff"))
        if kind == "moe":
            router = _object(m.get("router"), where + ".mlp.router")
            experts, top = _positive_int(router, "experts"), _positive_int(router, "top")
            if top > experts:
                raise ConfigError(f"config.json: {where}.mlp.router: top {top} of {experts} experts")
            return MoeSizes(experts, top, _positive_int(_object(m.get("expert"), where + ".mlp.expert"), "ff"))
        raise ConfigError(f"config.json: {where}.mlp.kind {kind!r} is not one of {cls.MLP_KINDS}")

    @classmethod
    def from_dict(cls, raw: dict) -> "SonodraConfig":
        norm = _object(raw.get("norm"), "norm")
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: layers must be a list with at least one entry")
        layers = []
        for i, L in enumerate(layers_raw):
            where = f"layers[{i}]"
            L = _object(L, where)
            kind = L.get("type")
            if kind not in cls.MIXER_TYPES:
                raise ConfigError(f"config.json: {where}.type {kind!r} is not one of {cls.MIXER_TYPES}")
            layers.append(SonodraLayer(kind, cls._mixer(kind, L.get("mixer"), where, len(layers_raw), i),
                                       cls._mlp(L.get("mlp"), where)))
        for i, L in enumerate(layers):
            src = getattr(L.mixer, "kv_from", None)
            if src is None:
                continue
            if src > i:
                raise ConfigError(f"config.json: layers[{i}] reads the latent vectors of layers[{src}], which runs after it")
            S = layers[src]
            if S.type != "latent_attention" or S.mixer.kv_from is not None:
                raise ConfigError(f"config.json: layers[{i}] reads the latent vectors of layers[{src}], which keeps none of its own")
            if S.mixer.kv_rank != L.mixer.kv_rank:
                raise ConfigError(f"config.json: layers[{i}] (kv_rank {L.mixer.kv_rank}) reads the latent vectors of "
                                  f"layers[{src}] (kv_rank {S.mixer.kv_rank})")
        return cls(vocab=_positive_int(raw, "vocab"), width=_positive_int(raw, "width"), eps=_number(norm, "eps", "norm"),
                   layers=tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": NAME, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "layers": [L.to_dict() for L in self.layers]}


def _mixer_spec(c: SonodraConfig, L: SonodraLayer):
    """(mixer spec, the mixer's local tensor names -> names under l<i>.mix.)"""
    m = L.mixer
    if L.type == "attention":
        position = (PartSpec.of("rope", head_dim=m.dim, theta=m.rot_base, rope_dims=m.rot_dims, interleaved=True)
                    if m.rot_dims else PartSpec.of("none"))
        spec = PartSpec.of("attention", hidden=c.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, scale=m.scale,
                           position=position, window=m.window, v_head_dim=m.vdim, qk_norm_eps=c.eps, qk_norm_span="projection")
        return spec, {"wq": "q", "wk": "k", "wv": "v", "wo": "o", "q_norm": "q.norm", "k_norm": "k.norm"}
    own = m.kv_from is None
    spec = PartSpec.of("latent_attention", hidden=c.width, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim,
                       kv_rank=m.kv_rank, scale=m.scale, eps=c.eps, own_latent=own, gate=True)
    names = {"wq": "q", "wuk": "uk", "wuv": "uv", "wg": "g", "wo": "o"}
    if own:
        names.update({"wdkv": "dkv", "dkv_norm": "dkv.norm"})
    return spec, names


def _ffn_spec(c: SonodraConfig, mlp, prefix: str):
    """(feed-forward spec, its local tensor names -> names of the folder)"""
    if isinstance(mlp, DenseSizes):
        spec = PartSpec.of("gated", hidden=c.width, intermediate=mlp.ff, activation="silu")
        return spec, {"w_gate": prefix + "gate", "w_up": prefix + "up", "w_down": prefix + "down"}
    spec = PartSpec.of("moe", hidden=c.width, n_experts=mlp.experts, top_k=mlp.top, intermediate=mlp.ff, activation="relu2",
                       scoring="sigmoid", renormalize=False, weight_on="input")
    names = {"router": prefix + "router"}
    for e in range(mlp.experts):
        names.update({f"e{e}.w_up": f"{prefix}e{e}.up", f"e{e}.w_down": f"{prefix}e{e}.down"})
    return spec, names


def build_sonodra_plan(c: SonodraConfig) -> ModelPlan:
    norm = PartSpec.of("rmsnorm", dim=c.width, eps=c.eps)
    layers, schedule = [], []
    for i, L in enumerate(c.layers):
        p = f"l{i}."
        mixer, mixer_names = _mixer_spec(c, L)
        names = {"mixer_norm.weight": p + "norm1", "mixer_out_norm.weight": p + "norm1b"}
        names.update({"mixer." + local: p + "mix." + name for local, name in mixer_names.items()})
        ffn = None
        if L.mlp is not None:
            ffn, ffn_names = _ffn_spec(c, L.mlp, p + "mlp.")
            names.update({"ffn_norm.weight": p + "norm2", "ffn_out_norm.weight": p + "norm2b"})
            names.update({"ffn." + local: name for local, name in ffn_names.items()})
        block = PartSpec.of("prenorm", mixer=mixer, ffn=ffn, mixer_norm=norm, ffn_norm=norm if ffn is not None else None,
                            mixer_out_norm=norm, ffn_out_norm=norm if ffn is not None else None)
        layers.append(LayerPlan(block=block, names=names))
        schedule.append(ScheduleEntry(i, kv_from=getattr(L.mixer, "kv_from", None)))
    plan = ModelPlan(vocab_size=c.vocab, hidden_size=c.width, layers=layers, schedule=schedule, final_norm=norm,
                     embedding_name="embed", final_norm_names={"weight": "final.norm"}, lm_head_name="head")
    plan.validate()
    return plan


SONODRA = register_architecture(Architecture(name=NAME, config_cls=SonodraConfig, build_plan=build_sonodra_plan,
                                             aliases=("sonodra",)))
