"""Sazilorn as a choice of parts: token rows plus learned rows of the positions into a 32-bit residual stream;
blocks whose mixer and feed-forward run side by side on ONE norm of the stream (weights stored around zero),
the mixer behind a short causal convolution that is added to its input; behind every block a weighted sum over
the embedding's output and all blocks' results so far, which is what goes on.  Per layer the mixer is grouped
attention without positions in the keys (norms over the whole query and key projections, a learned bias by
distance), HGRN2 (linear attention whose forget gate also decides what is written), or soft-capped gated
attention and lightning attention side by side; the feed-forward is gated with the tanh form of gelu, a
mixture of silu-gated experts with normalised weights and a shared expert, or absent.  Checkpoint names:
``embed``, ``pos``, ``l<i>.norm1``, ``l<i>.canon1``, ``l<i>.dwa``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.

The rows of an attention layer's table of biases come with the configuration when it says them or has taken
them from the checkpoint's shapes (``SazilornConfig.with_tensor_shapes``); a model made without either takes
``DEFAULT_BUCKETS``.
"""

from __future__ import annotations

from tokasaurus_amd.config.sazilorn_config import BiasedAttentionLayer, DenseFF, ExpertsFF, HGRN2Layer, SazilornConfig
from tokasaurus_amd.models.spec import ModelSpec, RunEntry
from tokasaurus_amd.parts.base import PartSpec

DEFAULT_BUCKETS = 32


def default_buckets(bias_max: int) -> int:
    """Rows of a table of biases by distance when no checkpoint says: ``DEFAULT_BUCKETS``, fewer for a short reach."""
    b = DEFAULT_BUCKETS
    while b > 2 and bias_max <= b // 2:
        b //= 2
    return b


def sazilorn_spec(cfg: SazilornConfig) -> ModelSpec:
    W = cfg.width

    def norm(name: str) -> PartSpec:
        return PartSpec("stream_rmsnorm", {"size": W, "eps": cfg.norm_eps, "name": name, "unit_offset": True})

    layers, order, connectors = [], [], []
    for i, layer in enumerate(cfg.layers):
        m, p = layer.mixer, f"l{i}.mix"
        if isinstance(m, BiasedAttentionLayer):
            mixer = PartSpec("grouped_attention", {
                "hidden_size": W, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim, "value_dim": m.vdim,
                "scale": m.scale, "projection_norm": {"q": f"{p}.q.norm", "k": f"{p}.k.norm", "eps": cfg.norm_eps},
                "distance_bias": {"name": f"{p}.rel", "buckets": m.bias_buckets or default_buckets(m.bias_max), "far": m.bias_max},
                "key_chunk": 256, "names": {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "o": f"{p}.o"}})
        elif isinstance(m, HGRN2Layer):
            mixer = PartSpec("hgrn2", {
                "hidden_size": W, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "norm_eps": cfg.norm_eps,
                "names": {"q": f"{p}.q", "f": f"{p}.f", "f_bias": f"{p}.f.b", "lower": f"{p}.lower", "v": f"{p}.v",
                          "norm": f"{p}.norm", "o": f"{p}.o"}})
        else:
            a, b = m.left, m.right
            left = PartSpec("grouped_attention", {
                "hidden_size": W, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "key_dim": a.dim, "value_dim": a.vdim,
                "scale": a.scale, "softcap": a.softcap, "element_gate_name": f"{p}.left.g", "key_chunk": 256,
                "names": {"q": f"{p}.left.q", "k": f"{p}.left.k", "v": f"{p}.left.v", "o": f"{p}.left.o"}})
            right = PartSpec("lightning_attention", {
                "hidden_size": W, "num_heads": b.heads, "key_dim": b.dim, "value_dim": b.vdim, "decays": list(b.decay),
                "norm_eps": cfg.norm_eps,
                "names": {"q": f"{p}.right.q", "k": f"{p}.right.k", "v": f"{p}.right.v", "g": f"{p}.right.g",
                          "norm": f"{p}.right.norm", "o": f"{p}.right.o"}})
            mixer = PartSpec("mixer_pair", {"hidden_size": W, "left": left, "right": right, "left_scale": m.left_scale,
                                            "right_scale": m.right_scale})
        params = {"mixer_norm": norm(f"l{i}.norm1"), "mixer": mixer, "shared_norm": True}
        if cfg.taps:
            params["input_conv"] = {"taps": cfg.taps, "name": f"l{i}.canon1"}
        f, q = layer.ff, f"l{i}.mlp"
        if isinstance(f, DenseFF):
            params["feed_forward"] = PartSpec("swiglu", {
                "hidden_size": W, "intermediate_size": f.ff, "activation": "gelu_tanh",
                "names": {"gate": f"{q}.gate", "up": f"{q}.up", "down": f"{q}.down"}})
        elif isinstance(f, ExpertsFF):
            names = {"router": f"{q}.router", "correction": f"{q}.correction", "expert": q + ".e{e}"}
            if f.shared_ff:
                names["shared"] = f"{q}.shared"
            params["feed_forward"] = PartSpec("routed_experts", {
                "hidden_size": W, "expert_size": f.ff, "num_experts": f.experts, "top": f.top, "shared_size": f.shared_ff,
                "normalize_scale": f.scale, "names": names})
        layers.append(PartSpec("parallel_residual", params))
        # behind block i: the weighted sum over the embedding's output and the results of blocks 0 .. i
        connectors.append(PartSpec("depth_average", {"streams": i + 2, "name": f"l{i}.dwa"}))
        order.append(RunEntry(i, after=i))
    return ModelSpec(
        vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "embed", "stream_f32": True,
                                               "position_name": "pos", "max_positions": cfg.max_positions}),
        head=PartSpec("norm_linear", {"vocab_size": cfg.vocab, "hidden_size": W, "name": "head", "norm": norm("final.norm")}),
        layers=tuple(layers),
        run_order=tuple(order),
        connectors=tuple(connectors),
        max_positions=cfg.max_positions,
        eos_token_ids=cfg.eos_token_ids,
    )
