"""The configuration of a Sakevik model, read from its ``config.json``.

The file lists the layers one by one; every size and every constant that may differ between
two models of the design is taken from it.  Keys:

    architecture: "Sakevik"       vocab, width       norm.eps       logit_scale (absent: 1)
    embedding: {scale, bigram: absent or null | {buckets, mul_prev, mul_cur}}
    layers[i].type: "mingru" | "attention" | "latent_attention"
    layers[i].mlp: null | {"kind": "dense", "ff": n, "limit": x}
    mingru mixer:           width
    attention mixer:        heads, kv_heads, dim, vdim, scale, mask: absent or null | {size},
                            rot: {base, dims, scaling: absent or null | as below (queries and keys only)}
    latent_attention mixer: heads, dim, rot_dim, vdim, kv_rank, scale, mask: absent or null | {size},
                            rot: {base, dims, scaling: absent or null | {factor, original, fast, slow}}
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

from tokasaurus_amd.config.kupuzen_config import _need
from tokasaurus_amd.config.model_config import ConfigError


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int
    scaling: tuple[float, float, float, float] | None = None  # factor, original, fast, slow


@dataclass(frozen=True)
class MinGRULayer:
    width: int


@dataclass(frozen=True)
class SigmoidAttentionLayer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int  # 0: every earlier key
    rot: Rotation


@dataclass(frozen=True)
class RotatedLatentAttentionLayer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int
    rot: Rotation


@dataclass(frozen=True)
class ClampedFF:
    ff: int
    limit: float


@dataclass(frozen=True)
class SakevikLayer:
    kind: str
    mixer: MinGRULayer | SigmoidAttentionLayer | RotatedLatentAttentionLayer
    ff: ClampedFF | None


@dataclass(frozen=True)
class Bigram:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class SakevikConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    bigram: Bigram | None
    logit_scale: float
    layers: tuple[SakevikLayer, ...]
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "SakevikConfig":
        def rotation(m: dict, where: str) -> Rotation:
            rot = _need(m, "rot", where)
            sc = rot.get("scaling")
            scaling = None
            if sc:
                scaling = tuple(float(_need(sc, k, f"{where}.rot.scaling")) for k in ("factor", "original", "fast", "slow"))
            r = Rotation(float(_need(rot, "base", f"{where}.rot")), int(_need(rot, "dims", f"{where}.rot")), scaling)
            if r.dims <= 0 or r.dims % 2:
                raise ConfigError(f"config.json: {where}.rot.dims must be a positive even number, got {r.dims}")
            return r

        def window(m: dict) -> int:
            mask = m.get("mask")
            return int(mask.get("size") or 0) if mask else 0

        layers = []
        for i, layer in enumerate(_need(d, "layers", "the file")):
            where = f"layers[{i}]"
            kind = _need(layer, "type", where)
            m = _need(layer, "mixer", where)
            mw = f"{where}.mixer"
            if kind == "mingru":
                mixer: Any = MinGRULayer(int(_need(m, "width", mw)))
            elif kind == "attention":
                mixer = SigmoidAttentionLayer(
                    heads=int(_need(m, "heads", mw)), kv_heads=int(_need(m, "kv_heads", mw)), dim=int(_need(m, "dim", mw)),
                    vdim=int(_need(m, "vdim", mw)), scale=float(_need(m, "scale", mw)), window=window(m), rot=rotation(m, mw))
                if mixer.heads % mixer.kv_heads:
                    raise ConfigError(f"config.json: {mw}: {mixer.heads} heads are no multiple of {mixer.kv_heads} kv_heads")
                if mixer.rot.dims > mixer.dim or mixer.vdim % 2:
                    raise ConfigError(f"config.json: {mw}: rot.dims beyond a head's size, or an odd vdim that cannot be turned in pairs")
            elif kind == "latent_attention":
                mixer = RotatedLatentAttentionLayer(
                    heads=int(_need(m, "heads", mw)), dim=int(_need(m, "dim", mw)), rot_dim=int(_need(m, "rot_dim", mw)),
                    vdim=int(_need(m, "vdim", mw)), kv_rank=int(_need(m, "kv_rank", mw)), scale=float(_need(m, "scale", mw)),
                    window=window(m), rot=rotation(m, mw))
                if mixer.rot.dims > mixer.rot_dim or mixer.rot_dim % 2:
                    raise ConfigError(f"config.json: {mw}: rot.dims beyond the rotated part rot_dim, or an odd rot_dim")
            else:
                raise ConfigError(f"config.json: {where} has type {kind!r}; known: mingru, attention, latent_attention")
            mlp = layer.get("mlp")
            ff = None
            if mlp is not None:
                fw = f"{where}.mlp"
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"config.json: {fw} has kind {mlp.get('kind')!r}; known: dense")
                ff = ClampedFF(int(_need(mlp, "ff", fw)), float(_need(mlp, "limit", fw)))
            layers.append(SakevikLayer(kind, mixer, ff))
        if not layers:
            raise ConfigError("config.json: a model needs at least one layer")
        emb = _need(d, "embedding", "the file")
        bg = emb.get("bigram")
        bigram = None
        if bg:
            bigram = Bigram(int(_need(bg, "buckets", "embedding.bigram")), int(_need(bg, "mul_prev", "embedding.bigram")),
                            int(_need(bg, "mul_cur", "embedding.bigram")))
            if bigram.buckets <= 0:
                raise ConfigError("config.json: embedding.bigram.buckets must be positive")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        return cls(
            vocab=int(_need(d, "vocab", "the file")), width=int(_need(d, "width", "the file")),
            norm_eps=float(_need(_need(d, "norm", "the file"), "eps", "norm")),
            embedding_scale=float(emb.get("scale") if emb.get("scale") is not None else 1.0), bigram=bigram,
            logit_scale=float(d.get("logit_scale") if d.get("logit_scale") is not None else 1.0),
            layers=tuple(layers), eos_token_ids=eos_ids)
