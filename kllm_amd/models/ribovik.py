"""The Ribovik decoder, put together from parts.

Token embedding with an RMS norm behind it; layers in the order the configuration lists them,
each with its norm behind the sub-layer (a = x + Norm1(Mixer(x)), x' = a + Norm2(FeedForward(a)),
the sub-layers reading the stream itself); the mixer is attention with biases, a partial rotation
of neighbouring pairs with stretched frequencies, queries and keys divided by their root mean
square after the rotation, a chunked mask and a softmax whose denominator has one more term; the
feed-forward is gated and dense with biases, or a mixture of clamped experts with identity
experts and a shared expert, or absent; a final norm, and the embedding table as output matrix.
Tensor names: ``embed``, ``embed.norm``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``final.norm``.
"""

from __future__ import annotations

from ..config.registry import register_architecture
from ..config.ribovik import RibovikConfig
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, Run

# The experts' gate is g sigmoid(SWISH_ALPHA g).
SWISH_ALPHA = 1.702


def build_ribovik(cfg: RibovikConfig) -> ModelSpec:
    d = cfg.width

    def norm(name):
        return PartSpec("rmsnorm", size=d, eps=cfg.norm_eps, names={"weight": name})

    positions = {}      # layers that rotate alike share one position part (and its tables of a step)
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}.mix"
        position = None
        if layer.rot_dims:
            s = layer.rot_scaling
            key = (layer.rot_dims, layer.rot_base, s)
            if key not in positions:
                positions[key] = PartSpec("rotary_scaled", rotary_dim=layer.rot_dims, base=layer.rot_base, interleaved=True,
                                          scaling=(s.factor, s.original, s.fast, s.slow) if s is not None else None)
            position = positions[key]
        names = {f"{t}.weight": f"{p}.{t}" for t in ("q", "k", "v", "o")}
        names.update({f"{t}.bias": f"{p}.{t}.b" for t in ("q", "k", "v")})
        mixer = PartSpec("attention_unit_qk", p, hidden=d, heads=layer.heads, kv_heads=layer.kv_heads, head_dim=layer.dim,
                         value_dim=layer.vdim, scale=layer.scale, eps=cfg.norm_eps, position=position, chunk=layer.chunk,
                         sink=True, names=names)
        ff = None
        mlp = layer.mlp
        if mlp is not None:
            m = f"l{i}.mlp"
            if mlp.kind == "dense":
                names = {f"{t}.weight": f"{m}.{t}" for t in ("gate", "up", "down")}
                names.update({f"{t}.bias": f"{m}.{t}.b" for t in ("gate", "up", "down")})
                ff = PartSpec("gated_mlp_bias", m, hidden=d, intermediate=mlp.ff, activation="silu", names=names)
            else:
                ff = PartSpec("routed_experts", m, hidden=d, experts=mlp.experts, identity=mlp.identity, top=mlp.top,
                              intermediate=mlp.ff, limit=mlp.limit, activation="clamped_swish", alpha=SWISH_ALPHA,
                              shared_intermediate=mlp.shared_ff, shared_limit=mlp.shared_limit)
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm_mixer=norm(f"l{i}.norm1"),
                                norm_feed_forward=norm(f"l{i}.norm2") if ff is not None else None,
                                block="sublayer_norm"))
    return ModelSpec(
        embedding=PartSpec("token_embedding", vocab=cfg.vocab, hidden=d, norm_eps=cfg.norm_eps,
                           names={"weight": "embed", "norm": "embed.norm"}),
        layers=layers,
        schedule=[Run(i) for i in range(len(layers))],
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", vocab=cfg.vocab, hidden=d, names={"weight": "embed"}),
        vocab_size=cfg.vocab,
        hidden_size=d,
    )


register_architecture("Ribovik", RibovikConfig, build_ribovik)
