"""The configuration of a Sazilorn model, read from its ``config.json``.

The file lists the layers one by one; every size and every constant that may differ between
two models of the design is taken from it.  Keys:

    architecture: "Sazilorn"      vocab, width, max_positions      norm.eps      canon.taps (absent: no convolution)
    layers[i].type: "attention" | "hgrn2" | "parallel"
    layers[i].mlp: null | {"kind": "dense", "ff": n}
                        | {"kind": "moe", "expert": {ff}, "router": {experts, top, scale}, "shared": absent or null | {ff}}
    attention mixer: heads, kv_heads, dim, vdim, scale, bias_max (the distance at which the bias reaches its last bucket;
                     the number of buckets is the first size of the checkpoint's ``l<i>.mix.rel``, or ``bias_buckets``)
    hgrn2 mixer:     heads, dim, vdim
    parallel mixer:  left: {heads, kv_heads, dim, vdim, scale, softcap}, right: {heads, dim, vdim, decay: [one a head]},
                     left_scale, right_scale
"""

from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any

from tokasaurus_amd.config.kupuzen_config import _need
from tokasaurus_amd.config.model_config import ConfigError


@dataclass(frozen=True)
class BiasedAttentionLayer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: int
    bias_buckets: int | None = None  # rows of the table of biases; None: not known yet (the checkpoint's shapes say)


@dataclass(frozen=True)
class HGRN2Layer:
    heads: int
    dim: int
    vdim: int


@dataclass(frozen=True)
class CappedAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float | None


@dataclass(frozen=True)
class LightningAttentionPart:
    heads: int
    dim: int
    vdim: int
    decay: tuple[float, ...]


@dataclass(frozen=True)
class ParallelLayer:
    left: CappedAttention
    right: LightningAttentionPart
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class DenseFF:
    ff: int


@dataclass(frozen=True)
class ExpertsFF:
    ff: int
    experts: int
    top: int
    scale: float
    shared_ff: int | None


@dataclass(frozen=True)
class SazilornLayer:
    kind: str
    mixer: BiasedAttentionLayer | HGRN2Layer | ParallelLayer
    ff: DenseFF | ExpertsFF | None


def _ints(d: dict, keys: tuple[str, ...], where: str) -> dict[str, int]:
    return {k: int(_need(d, k, where)) for k in keys}


@dataclass(frozen=True)
class SazilornConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    taps: int  # of the convolution in front of every mixer; 0: none
    layers: tuple[SazilornLayer, ...]
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "SazilornConfig":
        layers = []
        for i, layer in enumerate(_need(d, "layers", "the file")):
            where = f"layers[{i}]"
            kind = _need(layer, "type", where)
            m = _need(layer, "mixer", where)
            mw = f"{where}.mixer"
            if kind == "attention":
                buckets = m.get("bias_buckets")
                mixer: Any = BiasedAttentionLayer(**_ints(m, ("heads", "kv_heads", "dim", "vdim"), mw), scale=float(_need(m, "scale", mw)),
                                                  bias_max=int(_need(m, "bias_max", mw)),
                                                  bias_buckets=int(buckets) if buckets else None)
            elif kind == "hgrn2":
                mixer = HGRN2Layer(**_ints(m, ("heads", "dim", "vdim"), mw))
            elif kind == "parallel":
                a, b = _need(m, "left", mw), _need(m, "right", mw)
                cap = a.get("softcap")
                mixer = ParallelLayer(
                    left=CappedAttention(**_ints(a, ("heads", "kv_heads", "dim", "vdim"), f"{mw}.left"),
                                         scale=float(_need(a, "scale", f"{mw}.left")), softcap=float(cap) if cap else None),
                    right=LightningAttentionPart(**_ints(b, ("heads", "dim", "vdim"), f"{mw}.right"),
                                                 decay=tuple(float(x) for x in _need(b, "decay", f"{mw}.right"))),
                    left_scale=float(_need(m, "left_scale", mw)), right_scale=float(_need(m, "right_scale", mw)))
            else:
                raise ConfigError(f"config.json: {where} has type {kind!r}; known: attention, hgrn2, parallel")
            mlp = layer.get("mlp")
            ff: Any = None
            if mlp is not None:
                mk = mlp.get("kind")
                if mk == "dense":
                    ff = DenseFF(int(_need(mlp, "ff", f"{where}.mlp")))
                elif mk == "moe":
                    r = _need(mlp, "router", f"{where}.mlp")
                    sh = mlp.get("shared")
                    ff = ExpertsFF(ff=int(_need(_need(mlp, "expert", f"{where}.mlp"), "ff", f"{where}.mlp.expert")),
                                   experts=int(_need(r, "experts", f"{where}.mlp.router")), top=int(_need(r, "top", f"{where}.mlp.router")),
                                   scale=float(_need(r, "scale", f"{where}.mlp.router")),
                                   shared_ff=int(_need(sh, "ff", f"{where}.mlp.shared")) if sh else None)
                else:
                    raise ConfigError(f"config.json: {where}.mlp has kind {mk!r}; known: dense, moe")
            layers.append(SazilornLayer(kind, mixer, ff))
        eos = d.get("eos_token_id")
        canon = d.get("canon")
        cfg = cls(
            vocab=int(_need(d, "vocab", "the file")),
            width=int(_need(d, "width", "the file")),
            max_positions=int(_need(d, "max_positions", "the file")),
            norm_eps=float(_need(_need(d, "norm", "the file"), "eps", "norm")),
            taps=int(_need(canon, "taps", "canon")) if canon else 0,
            layers=tuple(layers),
            eos_token_ids=() if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos)),
        )
        cfg.validate()
        return cfg

    def with_tensor_shapes(self, shapes: dict[str, tuple[int, ...]]) -> "SazilornConfig":
        """The sizes that only the checkpoint knows, from the shapes of its tensors: the rows of an attention
        layer's table of biases by distance (``l<i>.mix.rel``)."""
        layers = []
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            rel = shapes.get(f"l{i}.mix.rel")
            if isinstance(m, BiasedAttentionLayer) and rel:
                m = replace(m, bias_buckets=int(rel[0]))
            layers.append(replace(layer, mixer=m))
        return replace(self, layers=tuple(layers))

    def validate(self) -> None:
        if min(self.vocab, self.width, self.max_positions) <= 0 or not self.layers:
            raise ConfigError("config.json: vocab, width, max_positions and the number of layers must be positive")
        if self.taps < 0:
            raise ConfigError(f"config.json: a convolution of {self.taps} taps")
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            heads = [m] if not isinstance(m, ParallelLayer) else [m.left, m.right]
            for p in heads:
                if min(p.heads, p.dim, p.vdim) <= 0 or (hasattr(p, "kv_heads") and (p.kv_heads <= 0 or p.heads % p.kv_heads)):
                    raise ConfigError(f"config.json: layers[{i}]: bad head counts or sizes")
            if isinstance(m, ParallelLayer) and len(m.right.decay) != m.right.heads:
                raise ConfigError(f"config.json: layers[{i}]: {len(m.right.decay)} decays for {m.right.heads} heads")
            if isinstance(m, BiasedAttentionLayer):
                if m.bias_buckets is not None and (m.bias_buckets < 2 or m.bias_max <= m.bias_buckets // 2):
                    raise ConfigError(f"config.json: layers[{i}]: {m.bias_buckets} buckets reaching to a distance of {m.bias_max}")
            f = layer.ff
            if isinstance(f, ExpertsFF) and not 0 < f.top <= f.experts:
                raise ConfigError(f"config.json: layers[{i}]: {f.top} of {f.experts} experts")
