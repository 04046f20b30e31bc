"""A plain, slow Ribovik in float64 torch on the CPU: the oracle of the Ribovik tests.

One function per mechanism, written from the equations; nothing here is shared with the
package.  ``cfg`` is the config.json dict, ``w`` a dict of float64 tensors by checkpoint name.
Sequences are handled one at a time and whole.

    x_0     = N(E[token]) g_e                    N(v) = v / sqrt(mean(v^2) + eps)
    a       = x + N(Mixer(x)) g_1                the sub-layers read x itself
    x'      = a + N(FeedForward(a)) g_2          (a layer may have no feed-forward)
    logits  = E (N(x_L) g_f)                     the embedding table is the output matrix
"""

import math

import torch

F64 = torch.float64


# ----------------------------------------------------------------------------- mechanisms

def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms(x, eps) * weight


def yarn_frequencies(rot):
    """Per pair i of the rotated part: the angle per position, and the factor on cos and sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64), 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate_neighbours(x, positions, rot):
    """x [n, heads, d]: the first rot.dims channels of every head turn in neighbouring pairs."""
    if not rot:
        return x
    dims = int(rot["dims"])
    freq, mag = yarn_frequencies(rot)
    ang = torch.as_tensor(positions, dtype=F64)[:, None] * freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(i, j, chunk):
    """Whether the query at position i reads the key at position j."""
    return j <= i and (not chunk or i // chunk == j // chunk)


def softmax_with_sink(s):
    """Rows of scores (-inf where masked): exp(s_j) / (1 + sum exp(s_j))."""
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def masked_attention(q, k, v, scale, chunk, positions):
    """q [n, H, d], k [n, G, d], v [n, G, dv] of one sequence at ``positions``: softmax with a sink
    of the scaled scores of the keys a query reads, times the values; [n, H, dv]."""
    n, H, _ = q.shape
    G = k.shape[1]
    mask = torch.tensor([[visible(i, j, chunk) for j in positions] for i in positions])
    out = torch.zeros(n, H, v.shape[2], dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(scale)
        s = s.masked_fill(~mask, float("-inf"))
        out[:, hd] = softmax_with_sink(s) @ v[:, g]
    return out


def attention(h, w, p, m, eps, positions):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = (h @ w[p + ".q"].T + w[p + ".q.b"]).reshape(n, H, d)
    k = (h @ w[p + ".k"].T + w[p + ".k.b"]).reshape(n, G, d)
    v = (h @ w[p + ".v"].T + w[p + ".v.b"]).reshape(n, G, dv)
    q = rms(rotate_neighbours(q, positions, m.get("rot")), eps)
    k = rms(rotate_neighbours(k, positions, m.get("rot")), eps)
    chunk = int((m.get("mask") or {}).get("size", 0))
    out = masked_attention(q, k, v, m["scale"], chunk, positions)
    return out.reshape(n, H * dv) @ w[p + ".o"].T


def dense_ff(h, w, p):
    g = h @ w[p + ".gate"].T + w[p + ".gate.b"]
    u = h @ w[p + ".up"].T + w[p + ".up.b"]
    return (g * torch.sigmoid(g) * u) @ w[p + ".down"].T + w[p + ".down.b"]


def clamped_expert(h, w, p, limit):
    g = torch.clamp(h @ w[p + ".gate"].T, max=limit)
    u = torch.clamp(h @ w[p + ".up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + ".down"].T


def route(h, w, p, top):
    """(chosen experts [n, top], their weights [n, top])."""
    s = torch.softmax(h @ w[p + ".router"].T, dim=-1)
    choice = s + w[p + ".correction"]
    idx = torch.topk(choice, top, dim=-1).indices
    picked = torch.gather(s, 1, idx)
    return idx, picked / (picked.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, w, p, mlp):
    r = mlp["router"]
    E, ident, top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
    idx, wt = route(h, w, p, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wt[t]):
            if e >= E:
                out[t] += a * h[t]
            else:
                out[t] += a * clamped_expert(h[t:t + 1], w, f"{p}.e{e}", float(mlp["expert"]["limit"]))[0]
    if mlp.get("shared"):
        out = out + clamped_expert(h, w, p + ".shared", float(mlp["shared"]["limit"]))
    return out


def feed_forward(h, w, p, mlp):
    return dense_ff(h, w, p) if mlp["kind"] == "dense" else moe_ff(h, w, p, mlp)


# ----------------------------------------------------------------------------- the model

def forward(cfg, w, tokens, layers_out=None):
    """Logits [n, vocab] of one whole sequence; ``layers_out`` collects the stream after each layer."""
    eps = float(cfg["norm"]["eps"])
    positions = list(range(len(tokens)))
    x = rms_norm(w["embed"][torch.as_tensor(tokens)], w["embed.norm"], eps)
    for i, layer in enumerate(cfg["layers"]):
        x = x + rms_norm(attention(x, w, f"l{i}.mix", layer["mixer"], eps, positions), w[f"l{i}.norm1"], eps)
        if layer.get("mlp"):
            x = x + rms_norm(feed_forward(x, w, f"l{i}.mlp", layer["mlp"]), w[f"l{i}.norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T


def tensor_shapes(cfg):
    """name -> shape of every tensor of a checkpoint of this configuration."""
    d = cfg["width"]
    out = {"embed": (cfg["vocab"], d), "embed.norm": (d,), "final.norm": (d,)}
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}.mix"
        out[f"l{i}.norm1"] = (d,)
        for t, rows in (("q", m["heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]), ("v", m["kv_heads"] * m["vdim"])):
            out[f"{p}.{t}"] = (rows, d)
            out[f"{p}.{t}.b"] = (rows,)
        out[p + ".o"] = (d, m["heads"] * m["vdim"])
        mlp = layer.get("mlp")
        if not mlp:
            continue
        out[f"l{i}.norm2"] = (d,)
        p = f"l{i}.mlp"

        def three(q, ff, bias):
            for t, shape in (("gate", (ff, d)), ("up", (ff, d)), ("down", (d, ff))):
                out[f"{q}.{t}"] = shape
                if bias:
                    out[f"{q}.{t}.b"] = (shape[0],)
        if mlp["kind"] == "dense":
            three(p, mlp["ff"], True)
        else:
            r = mlp["router"]
            for e in range(r["experts"]):
                three(f"{p}.e{e}", mlp["expert"]["ff"], False)
            out[p + ".router"] = (r["experts"] + r.get("identity", 0), d)
            out[p + ".correction"] = (r["experts"] + r.get("identity", 0),)
            if mlp.get("shared"):
                three(p + ".shared", mlp["shared"]["ff"], False)
    return out


def random_weights(cfg, seed, spaced_correction=False):
    """Random float32 tensors of a checkpoint.  ``spaced_correction``: the corrections of a
    router lie 1.5 apart in a shuffled order, more than two scores can differ, so that which
    experts are chosen does not rest on small differences of the scores (the weights of the
    chosen still do): for comparisons in bfloat16, where a close call falls either way."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith(".correction"):
            n = shape[0]
            if spaced_correction:
                out[name] = 1.5 * torch.randperm(n, generator=g).float() - 0.75 * n
            else:
                out[name] = 0.05 * torch.randn(n, generator=g)
        elif len(shape) == 1:
            norm = "norm" in name.rsplit(".", 1)[-1] or name.endswith("norm")
            out[name] = (1.0 + 0.2 * torch.randn(shape, generator=g)) if norm else 0.3 * torch.randn(shape, generator=g)
        elif name == "embed":
            out[name] = torch.randn(shape, generator=g)
        elif name.endswith(".router"):
            out[name] = 2.0 * torch.randn(shape, generator=g) / math.sqrt(shape[1])
        else:
            out[name] = 1.5 * torch.randn(shape, generator=g) / math.sqrt(shape[1])
    return out


def greedy(cfg, w, prompt, steps):
    ids = list(prompt)
    for _ in range(steps):
        ids.append(int(forward(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]
