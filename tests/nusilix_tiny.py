"""Small Nusilix configurations for the tests, each unlike the others in every size and
constant, and helpers to write them as model folders.

N1: both mixers, grouped KV heads, heads of 16, a feed-forward on every layer.
N2: heads of 64 (the bfloat16 prompt and decode kernels), one KV head, one norm group, factor 1,
    a recurrent layer first, a layer without feed-forward, a query temperature that changes
    every 8 positions.
N3: heads of 32 and of 128, as many KV heads as heads on one layer, three norm groups, a width
    that is no power of two, a recurrence with heads of 64 and a low-rank width that is no
    multiple of 8.
N5: recurrent layers only (no pages at all), heads of 20, a low-rank width of 5.
N6: attention only (no state slots), as many KV heads as heads, heads of 20 (the kernel for every
    size in both number formats), an odd vocabulary, a temperature step at every position.
N7: a width of 50 in five norm groups (no multiple of 4 or 8 anywhere: the plain products and the
    norm kernel for every size), heads of 8 and 12, a low-rank width of 3, a factor above 1.
N4: heads of 24 in both mixers (sizes that only the kernel for every size takes in bfloat16),
    three recurrent heads, two recurrent layers in a row.
"""

import json
import os

import torch

import plain_nusilix as P


def attn(heads, kv, dim, coef=0.35, every=8, scale=None, ff=None):
    return {"type": "attention",
            "mixer": {"dim": dim, "vdim": dim, "heads": heads, "kv_heads": kv, "scale": scale or dim ** -0.5 * 1.5,
                      "q_temp": {"coef": coef, "every": every}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta(heads, dim, rank=8, ff=None):
    return {"type": "general_delta", "mixer": {"dim": dim, "heads": heads, "rank": rank},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def _cfg(vocab, width, layers, eps, groups, mult):
    return {"architecture": "Nusilix", "vocab": vocab, "width": width, "layers": layers,
            "norm": {"eps": eps, "groups": groups}, "residual_mult": mult}


CONFIGS = {
    "N1": _cfg(96, 64, [attn(4, 2, 16, ff=80), delta(2, 16, rank=8, ff=72), attn(4, 2, 16, every=5, ff=80)],
               1e-5, 2, 0.45),
    "N2": _cfg(128, 128, [delta(2, 32, rank=16, ff=96), attn(4, 1, 64, coef=0.5, every=8),
                          attn(4, 1, 64, coef=0.5, every=8, ff=160)], 1e-6, 1, 1.0),
    "N3": _cfg(101, 96, [attn(8, 1, 32, every=16, ff=64), delta(1, 64, rank=12, ff=56),
                         attn(2, 2, 128, coef=0.1, every=3)], 1e-4, 3, 0.7),
    "N5": _cfg(50, 40, [delta(2, 20, rank=5, ff=24), delta(2, 20, rank=5)], 1e-6, 2, 0.6),
    "N6": _cfg(61, 48, [attn(5, 5, 20, coef=0.25, every=1, ff=32), attn(5, 5, 20, coef=0.25, every=1, ff=32)],
               1e-5, 1, 1.0),
    "N7": _cfg(33, 50, [attn(2, 1, 8, every=4, ff=30), delta(2, 12, rank=3, ff=22), attn(2, 1, 8, every=4)],
               1e-5, 5, 1.3),
    "N4": _cfg(77, 72, [attn(6, 3, 24, every=7, ff=40), delta(3, 24, rank=4), delta(3, 24, rank=4, ff=48)],
               1e-5, 4, 0.35),
}


def rank_of(cfg):
    return [l["mixer"].get("rank") for l in cfg["layers"]]


def write_model(out_dir, cfg, seed, store="float32", weights=None, drop_rank=False):
    """A model folder written with the safetensors library.  ``drop_rank``: the configuration
    does not name the recurrence's low-rank width (the tensors' shapes give it)."""
    from safetensors.torch import save_file
    w = weights if weights is not None else P.random_weights(cfg, seed)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[store]
    os.makedirs(out_dir, exist_ok=True)
    save_file({k: v.to(dt).contiguous() for k, v in w.items()}, os.path.join(out_dir, "model.safetensors"))
    out = json.loads(json.dumps(cfg))
    if drop_rank:
        for layer in out["layers"]:
            layer["mixer"].pop("rank", None)
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(out, f)
    return out_dir


def read_weights(model_dir, as_stored_in=None):
    """The folder's weights as float32 CPU tensors; with as_stored_in="bfloat16" every matrix is
    rounded to bfloat16 first, as a bfloat16 engine keeps it (vectors stay in 32-bit)."""
    from safetensors.torch import load_file
    out = {}
    for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items():
        v = v.float()
        if as_stored_in == "bfloat16" and v.dim() > 1:
            v = v.to(torch.bfloat16).float()
        out[k] = v
    return out


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
