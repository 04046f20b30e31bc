"""The Nusilix decoder, put together from parts.

Token embedding plus sinusoidal positions; layers in the order the configuration lists them,
each with one grouped RMS norm whose output both the mixer and the feed-forward read
(x' = x + residual_mult * (mixer + feed-forward)); a mixer is attention whose values are its
keys (biases, whole-projection query and key norms, a query temperature, a distance bias, no
rotation) or a generalized-delta-rule recurrence; the feed-forward is dense with the xIELU
activation, or absent; a final grouped norm and the output projection.  Tensor names:
``embed``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from ..config.nusilix import NusilixConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, Run

# The distance bias of head h of H is 2^(-8 (h + 1) / H) per position.
DISTANCE_SLOPE_BITS = 8


def build_nusilix(cfg: NusilixConfig) -> ModelSpec:
    d = cfg.width

    def norm(name):
        return PartSpec("group_rmsnorm", size=d, eps=cfg.norm_eps, groups=cfg.norm_groups, names={"weight": name})

    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}.mix"
        if layer.type == "attention":
            names = {f"{t}.weight": f"{p}.{t}" for t in ("q", "k", "o")}
            names.update({f"{t}.bias": f"{p}.{t}.b" for t in ("q", "k", "o")})
            mixer = PartSpec("attention_keys_as_values", p, hidden=d, heads=layer.heads, kv_heads=layer.kv_heads,
                             head_dim=layer.dim, scale=layer.scale, eps=cfg.norm_eps, q_temp=layer.q_temp,
                             distance_slope_bits=DISTANCE_SLOPE_BITS, names=names)
        else:
            names = {f"{t}.weight": f"{p}.{t}" for t in ("r", "k", "v", "g", "a", "w1", "w2", "o")}
            names["a.bias"] = f"{p}.a.b"
            mixer = PartSpec("general_delta", p, hidden=d, heads=layer.heads, head_dim=layer.dim, eps=cfg.norm_eps,
                             rank=layer.rank, names=names)
        ff = None
        if layer.ff is not None:
            m = f"l{i}.mlp"
            ff = PartSpec("dense_mlp", m, hidden=d, intermediate=layer.ff, activation="xielu",
                          names={"up.weight": f"{m}.up", "down.weight": f"{m}.down"})
        layers.append(LayerSpec(mixer=mixer, feed_forward=ff, norm_mixer=norm(f"l{i}.norm1"), block="parallel",
                                block_params={"mult": cfg.residual_mult}))
    return ModelSpec(
        embedding=PartSpec("token_embedding", vocab=cfg.vocab, hidden=d, names={"weight": "embed"},
                           position=PartSpec("sinusoidal", base=10000.0)),
        layers=layers,
        schedule=[Run(i) for i in range(len(layers))],
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", vocab=cfg.vocab, hidden=d, names={"weight": "head"}),
        vocab_size=cfg.vocab,
        hidden_size=d,
    )


register_architecture("Nusilix", NusilixConfig, build_nusilix)
