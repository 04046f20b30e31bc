"""Small Ribovik configurations for the tests, each unlike the others in every size and constant,
and helpers to write them as model folders.

R1: grouped KV heads, heads of 32 of which 16 elements turn, stretched frequencies, chunks of 24
    (no multiple of the page), a dense layer, then experts with identity experts and a shared
    expert.
R2: heads of 64 with one KV head and values of 32 (the kernel for every size in both number
    formats), plain frequencies, chunks of 40, a layer without feed-forward, one expert a token
    without identity or shared experts.
R3: two heads of 128 that turn by half, no mask at all, more identity experts in the choice than
    real ones, a width of 72.
R4: a width of 50 (no multiple of 4 or 8 anywhere: the plain products), five heads of 20 with
    values of 12, chunks of 7, an odd vocabulary, experts of 22.
R5: heads of 16 that turn whole, chunks of 16 (the page), stretched by 1.5 with a short ramp, dense
    layers only, another eps.
R6: heads of 96 of which 64 turn, ten heads on two KV heads, chunks of 100, experts whose limit
    clamps often, top 3 of 4 + 2.
R7: every layer unlike the others: heads of 32, 16 and 64, values of their own width on one layer,
    chunks of 12 and 30 and none, rotation whole, partial and none, two different mixtures, a layer
    without feed-forward; the first and the last layer alike.
"""

import json
import os

import torch

import plain_ribovik as P


def attn(heads, kv, dim, vdim=None, rot=None, base=10000.0, scaling=None, chunk=0, scale=None, mlp=None):
    mixer = {"dim": dim, "vdim": vdim or dim, "heads": heads, "kv_heads": kv, "scale": scale or 1.4 * dim ** -0.5}
    if rot:
        mixer["rot"] = {"base": base, "dims": rot}
        if scaling:
            mixer["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if chunk:
        mixer["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, limit, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
           "router": {"experts": experts, "identity": identity, "top": top}}
    if shared:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def _cfg(vocab, width, eps, layers):
    return {"architecture": "Ribovik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


CONFIGS = {
    "R1": _cfg(90, 64, 1e-5, [
        attn(4, 2, 32, rot=16, base=5000.0, scaling=(4.0, 64, 16.0, 2.0), chunk=24, mlp=dense(80)),
        attn(4, 2, 32, rot=16, base=5000.0, scaling=(4.0, 64, 16.0, 2.0), chunk=24,
             mlp=moe(6, 2, 2, 48, 3.0, shared=(40, 2.5)))]),
    "R2": _cfg(128, 128, 1e-6, [
        attn(4, 1, 64, vdim=32, rot=64, chunk=40, mlp=moe(4, 0, 1, 32, 1.0)),
        attn(4, 1, 64, vdim=32, rot=64, chunk=40),
        attn(4, 1, 64, vdim=32, rot=64, chunk=40, mlp=dense(96))]),
    "R3": _cfg(101, 72, 1e-4, [
        attn(2, 2, 128, rot=64, base=200.0, mlp=moe(2, 3, 4, 24, 2.0, shared=(16, 4.0))),
        attn(2, 2, 128, rot=64, base=200.0, mlp=dense(40))]),
    "R4": _cfg(61, 50, 1e-5, [
        attn(5, 5, 20, vdim=12, rot=10, chunk=7, mlp=dense(30)),
        attn(5, 5, 20, vdim=12, rot=10, chunk=7, mlp=moe(3, 1, 2, 22, 1.5, shared=(18, 1.0)))]),
    "R5": _cfg(77, 48, 1e-3, [
        attn(6, 3, 16, rot=16, base=1000.0, scaling=(1.5, 32, 8.0, 4.0), chunk=16, mlp=dense(56)),
        attn(6, 3, 16, rot=16, base=1000.0, scaling=(1.5, 32, 8.0, 4.0), chunk=16, mlp=dense(56))]),
    "R6": _cfg(150, 160, 1e-6, [
        attn(10, 2, 96, rot=64, base=100000.0, scaling=(8.0, 128, 24.0, 1.5), chunk=100,
             mlp=moe(4, 2, 3, 40, 0.3, shared=(64, 0.5))),
        attn(10, 2, 96, rot=64, base=100000.0, scaling=(8.0, 128, 24.0, 1.5), chunk=100, mlp=dense(72))]),
    "R7": _cfg(70, 96, 1e-5, [
        attn(4, 2, 32, rot=32, chunk=12, mlp=dense(64)),
        attn(6, 1, 16, rot=8, base=777.0, scaling=(3.0, 48, 12.0, 2.0), chunk=30, mlp=moe(5, 1, 2, 24, 2.5, shared=(32, 1.25))),
        attn(2, 2, 64, vdim=48),
        attn(4, 2, 32, rot=32, chunk=12, mlp=moe(3, 2, 3, 40, 0.8))]),
}


def write_model(out_dir, cfg, seed, store="float32", weights=None, spaced_correction=False):
    """A model folder written with the safetensors library."""
    from safetensors.torch import save_file
    w = weights if weights is not None else P.random_weights(cfg, seed, spaced_correction)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[store]
    os.makedirs(out_dir, exist_ok=True)
    save_file({k: v.to(dt).contiguous() for k, v in w.items()}, os.path.join(out_dir, "model.safetensors"))
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(cfg, f)
    return out_dir


def read_weights(model_dir, as_stored_in=None):
    """The folder's weights as float64 CPU tensors; with as_stored_in="bfloat16" every matrix is
    rounded to bfloat16 first, as a bfloat16 engine keeps it (vectors stay in 32-bit)."""
    from safetensors.torch import load_file
    out = {}
    for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items():
        v = v.float()
        if as_stored_in == "bfloat16" and v.dim() > 1:
            v = v.to(torch.bfloat16).float()
        out[k] = v.double()
    return out


def tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
