"""Sakevik as a choice of parts: a scaled embedding plus a hashed table of token pairs into a 32-bit
residual stream; blocks that norm a sublayer's output only (the sublayers read the stream itself);
per layer a gated recurrence whose gates read the current token only (minGRU), grouped-query attention
with sigmoid weights (norms of queries and keys head by head, a rotation of the halves of a head's
leading part, values turned by their own positions and turned back behind the sum, a bias per head on
the scores, a sliding window, a gate per head), or attention over a cached latent beside a rotated key
part that all heads share (a rotation of neighbouring elements with a ramp between two frequency
scales, a sliding window, ordinary softmax); per layer a gated feed-forward with clamps, or none; a
final norm and a head whose logits are scaled.  Checkpoint names: ``embed``, ``bigram``,
``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from tokasaurus_amd.config.sakevik_config import MinGRULayer, RotatedLatentAttentionLayer, SakevikConfig, SigmoidAttentionLayer
from tokasaurus_amd.models.spec import ModelSpec, RunEntry
from tokasaurus_amd.parts.base import PartSpec

MAX_POSITIONS = 1 << 30  # the rotations compute their angles from the position: no table ends them
GLU_ALPHA = 1.702  # the feed-forward's gate is g * sigmoid(GLU_ALPHA * g)


def sakevik_spec(cfg: SakevikConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("stream_rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "name": name})

    def ramp_of(rot) -> dict | None:
        return dict(zip(("factor", "original", "fast", "slow"), rot.scaling)) if rot.scaling is not None else None

    layers, unused = [], []
    for i, layer in enumerate(cfg.layers):
        m, p = layer.mixer, f"l{i}.mix"
        if isinstance(m, MinGRULayer):
            mixer = PartSpec("min_gru", {
                "hidden_size": cfg.width, "width": m.width,
                "names": {"z": f"{p}.z", "x": f"{p}.x", "g": f"{p}.g", "z_bias": f"{p}.z.b", "x_bias": f"{p}.x.b", "o": f"{p}.o"}})
        elif isinstance(m, SigmoidAttentionLayer):
            mixer = PartSpec("grouped_attention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim, "value_dim": m.vdim,
                "scale": m.scale, "window": m.window, "key_chunk": 256,
                # (a ramp between frequency scales, where the file gives one, is the queries' and keys' alone: the values turn
                # by the plain frequencies of the same base)
                "position": PartSpec("rotary_halves", {"dims": m.rot.dims, "base": m.rot.base, "ramp": ramp_of(m.rot)}),
                "names": {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o"},
                "bias_names": {"q": f"{p}.q.b", "k": f"{p}.k.b", "v": f"{p}.v.b", "o": f"{p}.o.b"},
                "head_norm": {"q": f"{p}.q.norm", "k": f"{p}.k.norm", "eps": cfg.norm_eps},
                "score_bias_name": f"{p}.pb",
                "value_rotation": {"base": m.rot.base, "pair_halves": True},
                "gate_name": f"{p}.g"})
        else:
            assert isinstance(m, RotatedLatentAttentionLayer)
            mixer = PartSpec("latent_attention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "q_rank": 0,
                "kv_rank": m.kv_rank, "rot_dim": m.rot_dim, "scale": m.scale, "norm_eps": cfg.norm_eps, "window": m.window,
                "position": PartSpec("rotary_interleaved", {"dims": m.rot.dims, "base": m.rot.base, "ramp": ramp_of(m.rot)}),
                "names": {"q": f"{p}.q", "dkv": f"{p}.dkv", "dkv_norm": f"{p}.dkv.norm", "uk": f"{p}.uk", "uv": f"{p}.uv",
                          "o": f"{p}.o"}})
        params = {"mixer": mixer, "mixer_post_norm": norm(f"l{i}.norm1")}
        if layer.ff is None:
            unused.append(f"l{i}.norm2")
        else:
            q = f"l{i}.mlp"
            params["ff_post_norm"] = norm(f"l{i}.norm2")
            params["feed_forward"] = PartSpec("clamped_glu", {
                "hidden_size": cfg.width, "intermediate_size": layer.ff.ff, "limit": layer.ff.limit, "alpha": GLU_ALPHA,
                "names": {"gate": f"{q}.gate", "up": f"{q}.up", "down": f"{q}.down"}})
        layers.append(PartSpec("post_norm", params))
    if cfg.bigram is not None:
        embedding = PartSpec("bigram_embedding", {
            "vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "embed", "pairs_name": "bigram", "scale": cfg.embedding_scale,
            "buckets": cfg.bigram.buckets, "mul_prev": cfg.bigram.mul_prev, "mul_cur": cfg.bigram.mul_cur})
    else:
        embedding = PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "embed",
                                                 "scale": cfg.embedding_scale, "stream_f32": True})
    return ModelSpec(
        vocab_size=cfg.vocab,
        embedding=embedding,
        head=PartSpec("norm_linear", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "name": "head", "norm": norm("final.norm"),
                                      "scale": cfg.logit_scale}),
        layers=tuple(layers),
        run_order=tuple(RunEntry(i) for i in range(len(layers))),
        max_positions=MAX_POSITIONS,
        eos_token_ids=cfg.eos_token_ids,
        # a layer without a feed-forward may still carry the norm behind it
        ignorable_tensors=tuple(unused),
    )
