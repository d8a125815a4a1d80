"""Sunusun: a decoder whose config.json lists its layers one by one.  Every layer is a pre-norm block (RMSNorm with one
number as its weight) around a mixer and, unless the entry says null, a dense feed-forward with the exact gelu.  A
sinusoidal position vector is added to the embedding; no mixer rotates anything.  Two kinds of layers:

  "wkv"       time mixing with a matrix state per head (parts/recurrent.py, "wkv")
  "parallel"  an attention without rotation (query/key head norms, a query temperature, a logarithmic distance bias, a
              sink in the softmax) beside a min-GRU, each output normed, half their sum (parts/parallel.py)

A layer with "weights_of": j has no tensors of its own: it runs layer j's weights with a cache or state of its own,
which the plan's schedule says by naming layer j twice.

config.json keys: architecture, vocab, width, norm.eps, logit_scale, layers[] = {type, mixer, mlp, weights_of?} with
  wkv mixer       {heads, dim}; the rank of the decay's low-rank projection is the first size of tensor l<i>.mix.w1
                  (a folder written by this library also names it, "decay_rank")
  parallel mixer  {left: {heads, kv_heads, dim, vdim, scale, q_temp: {coef, every}}, right: {width}}
  mlp             {kind: "dense", ff} or null

Tensor names of the folder (linear weights [out, in]): embed, head, final.norm, and for layer i under l<i>.:
  norm1, norm2, mlp.up, mlp.down
  wkv:       mix.mu.{r,k,v,g,w}, mix.{r,k,v,g}, mix.w1, mix.w2, mix.w0, mix.u, mix.norm, mix.o
  parallel:  mix.left.{q,k,v,o}, mix.left.q.norm, mix.left.k.norm, mix.left.r1, mix.left.r2, mix.left.out,
             mix.right.{z,x,g,o}, mix.right.z.b, mix.right.x.b, mix.right.out
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from ..engine.plan import LayerPlan, ModelPlan, ScheduleEntry
from ..parts.base import PartSpec
from .base import Architecture, ConfigError, _positive_int, register_architecture

SINUSOID_BASE = 10000.0           # the position vector's base; the design fixes it
NAME = "Sunusun"


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
class WkvSizes:
    heads: int
    dim: int
    decay_rank: int

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "decay_rank": self.decay_rank}


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp_coef: float
    q_temp_every: int

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "q_temp": {"coef": self.q_temp_coef, "every": self.q_temp_every}}


@dataclass(frozen=True)
class ParallelSizes:
    left: AttentionSizes
    right_width: int

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": {"width": self.right_width}}


@dataclass(frozen=True)
class SunusunLayer:
    type: str                                  # "wkv" | "parallel"
    mixer: object                              # WkvSizes | ParallelSizes
    ff: Optional[int]                          # the dense feed-forward's inner width; None: the layer has none
    weights_of: Optional[int] = None

    def to_dict(self):
        d = {"type": self.type, "mixer": self.mixer.to_dict(),
             "mlp": None if self.ff is None else {"kind": "dense", "ff": self.ff}}
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class SunusunConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: Tuple[SunusunLayer, ...]

    MIXER_TYPES = ("wkv", "parallel")

    @staticmethod
    def sizes_from_tensors(raw: dict, shapes: dict) -> dict:
        """config.json completed by the sizes that only a tensor's shape gives: the rank of every wkv layer's decay
        projection (tensor l<i>.mix.w1 of the layer whose weights the entry uses)."""
        layers = raw.get("layers")
        if not isinstance(layers, list):
            return raw
        out = []
        for i, L in enumerate(layers):
            if isinstance(L, dict) and L.get("type") == "wkv" and isinstance(L.get("mixer"), dict) \
                    and "decay_rank" not in L["mixer"]:
                j = L.get("weights_of", i)
                shape = shapes.get(f"l{j}.mix.w1")
                if shape is not None and len(shape) == 2:
                    L = dict(L, mixer=dict(L["mixer"], decay_rank=int(shape[0])))
            out.append(L)
        return dict(raw, layers=out)

    @staticmethod
    def _mixer(kind: str, raw, where: str):
        m = _object(raw, where + ".mixer")
        if kind == "wkv":
            if "decay_rank" not in m:
                raise ConfigError(f"config.json: {where}.mixer: the decay projection's rank is neither named (decay_rank) "
                                  f"nor given by the shape of the layer's tensor mix.w1")
            return WkvSizes(_positive_int(m, "heads"), _positive_int(m, "dim"), _positive_int(m, "decay_rank"))
        left, right = _object(m.get("left"), where + ".mixer.left"), _object(m.get("right"), where + ".mixer.right")
        temp = _object(left.get("q_temp"), where + ".mixer.left.q_temp")
        a = AttentionSizes(_positive_int(left, "heads"), _positive_int(left, "kv_heads"), _positive_int(left, "dim"),
                           _positive_int(left, "vdim"), _number(left, "scale", where + ".mixer.left"),
                           _number(temp, "coef", where + ".mixer.left.q_temp", positive=False),
                           _positive_int(temp, "every"))
        if a.heads % a.kv_heads:
            raise ConfigError(f"config.json: {where}: {a.heads} heads are not a multiple of {a.kv_heads} kv_heads")
        return ParallelSizes(a, _positive_int(right, "width"))

    @classmethod
    def from_dict(cls, raw: dict) -> "SunusunConfig":
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
            mlp = L.get("mlp")
            ff = None
            if mlp is not None:
                mlp = _object(mlp, where + ".mlp")
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp.kind {mlp.get('kind')!r} is not supported (supported: 'dense')")
                ff = _positive_int(mlp, "ff")
            wo = L.get("weights_of")
            if wo is not None and (isinstance(wo, bool) or not isinstance(wo, int) or not 0 <= wo < len(layers_raw) or wo == i):
                raise ConfigError(f"config.json: {where}.weights_of {wo!r} names no other layer")
            layers.append(SunusunLayer(kind, cls._mixer(kind, L.get("mixer"), where), ff, wo))
        for i, L in enumerate(layers):
            if L.weights_of is not None:
                src = layers[L.weights_of]
                if src.weights_of is not None:
                    raise ConfigError(f"config.json: layers[{i}] uses the weights of layers[{L.weights_of}], which has none of its own")
                if (src.type, src.mixer, src.ff) != (L.type, L.mixer, L.ff):
                    raise ConfigError(f"config.json: layers[{i}] uses the weights of layers[{L.weights_of}] but differs from it")
        return cls(vocab=_positive_int(raw, "vocab"), width=_positive_int(raw, "width"), eps=_number(norm, "eps", "norm"),
                   logit_scale=_number(raw, "logit_scale", "config") if "logit_scale" in raw else 1.0, layers=tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": NAME, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "logit_scale": self.logit_scale, "layers": [L.to_dict() for L in self.layers]}


def _mixer_spec(c: SunusunConfig, L: SunusunLayer):
    """(mixer spec, the mixer's local tensor names -> names under l<i>.mix.)"""
    if L.type == "wkv":
        m = L.mixer
        spec = PartSpec.of("wkv", hidden=c.width, n_heads=m.heads, head_dim=m.dim, decay_rank=m.decay_rank, eps=c.eps)
        names = {f"mu_{s}": f"mu.{s}" for s in "rkvgw"}
        names.update({"wr": "r", "wk": "k", "wv": "v", "wg": "g", "w1": "w1", "w2": "w2", "w0": "w0", "u": "u",
                      "norm": "norm", "wo": "o"})
        return spec, names
    a = L.mixer.left
    left = PartSpec.of("attention", hidden=c.width, n_heads=a.heads, n_kv_heads=a.kv_heads, head_dim=a.dim, scale=a.scale,
                       position=PartSpec.of("none"), v_head_dim=a.vdim, qk_norm_eps=c.eps, q_temp_coef=a.q_temp_coef,
                       q_temp_every=a.q_temp_every, distance_bias=True, sink=True)
    right = PartSpec.of("mingru", hidden=c.width, width=L.mixer.right_width, bias=True)
    spec = PartSpec.of("parallel", hidden=c.width, left=left, right=right, eps=c.eps)
    names = {"left.wq": "left.q", "left.wk": "left.k", "left.wv": "left.v", "left.wo": "left.o",
             "left.q_norm": "left.q.norm", "left.k_norm": "left.k.norm", "left.dist_a": "left.r1", "left.dist_b": "left.r2",
             "right.wz": "right.z", "right.bz": "right.z.b", "right.wx": "right.x", "right.bx": "right.x.b",
             "right.wg": "right.g", "right.wo": "right.o", "left_out": "left.out", "right_out": "right.out"}
    return spec, names


def build_sunusun_plan(c: SunusunConfig) -> ModelPlan:
    norm = PartSpec.of("rmsnorm", dim=c.width, eps=c.eps, scalar=True)
    layers, index = [], {}                  # index: config layer -> its place among the layers that own tensors
    for i, L in enumerate(c.layers):
        if L.weights_of is not None:
            continue
        mixer, mixer_names = _mixer_spec(c, L)
        ffn = PartSpec.of("dense", hidden=c.width, intermediate=L.ff, activation="gelu_erf") if L.ff is not None else None
        block = PartSpec.of("prenorm", mixer=mixer, ffn=ffn, mixer_norm=norm, ffn_norm=norm if ffn is not None else None)
        p = f"l{i}."
        names = {"mixer_norm.weight": p + "norm1"}
        names.update({"mixer." + local: p + "mix." + name for local, name in mixer_names.items()})
        if ffn is not None:
            names.update({"ffn_norm.weight": p + "norm2", "ffn.w_up": p + "mlp.up", "ffn.w_down": p + "mlp.down"})
        index[i] = len(layers)
        layers.append(LayerPlan(block=block, names=names))
    schedule = [ScheduleEntry(index[L.weights_of if L.weights_of is not None else i]) for i, L in enumerate(c.layers)]
    plan = ModelPlan(vocab_size=c.vocab, hidden_size=c.width, layers=layers, schedule=schedule, final_norm=norm,
                     embedding_name="embed", final_norm_names={"weight": "final.norm"}, lm_head_name="head",
                     position_sinusoid_base=SINUSOID_BASE, logit_scale=c.logit_scale)
    plan.validate()
    return plan


SUNUSUN = register_architecture(Architecture(name=NAME, config_cls=SunusunConfig, build_plan=build_sunusun_plan,
                                             aliases=("sunusun",)))
