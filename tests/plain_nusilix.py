"""A plain, slow Nusilix in float64 torch on the CPU: the oracle of the Nusilix tests.

One function per mechanism, written from the equations; nothing here is shared with the
package.  ``cfg`` is the config.json dict.  Sequences are handled one at a time; the recurrent
mixer can be fed in pieces (``state`` in and out), the rest is whole-sequence.

    x_0       = E[token] + P(position)           P[2i] = sin(p b^(-2i/D)), P[2i+1] = cos(same), b = 10000
    h         = GroupNorm(x) * g                 groups of D/n channels, each / sqrt(mean^2 + eps)
    x'        = x + m (Mixer(h) + FeedForward(h))
    logits    = Head GroupNorm(x_L)
"""

import math

import torch

F64 = torch.float64


# ----------------------------------------------------------------------------- mechanisms

def sinusoid(positions, width, base=10000.0):
    p = torch.as_tensor(positions, dtype=F64)[:, None]
    out = torch.zeros(len(positions), width, dtype=F64)
    for c in range(width):
        angle = p[:, 0] * base ** (-2.0 * (c // 2) / width)
        out[:, c] = torch.cos(angle) if c % 2 else torch.sin(angle)
    return out


def group_norm(x, weight, groups, eps):
    n, d = x.shape
    parts = x.reshape(n, groups, d // groups)
    parts = parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)
    return parts.reshape(n, d) * weight


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def xielu(z, p, q):
    sp = lambda v: math.log1p(math.exp(v))
    pos = sp(p) * z * z + z / 2
    neg = (0.5 + sp(q)) * (torch.exp(torch.clamp(z, max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def dense_mlp(h, w_up, w_down, act):
    return xielu(h @ w_up.T, float(act[0]), float(act[1])) @ w_down.T


def slopes(heads, bits=8.0):
    return [2.0 ** (-bits * (h + 1) / heads) for h in range(heads)]


def query_temperature(positions, coef, every):
    p = torch.as_tensor(positions, dtype=torch.int64)
    return 1.0 + coef * torch.log(torch.div(p + 1, every, rounding_mode="floor").to(F64) + 1.0)


def attention_scores_to_output(q, k, v, scale, head_slopes, positions):
    """q [n, H, d], k and v [n, G, d] of one sequence at ``positions`` (increasing): causal
    softmax of q.k * scale - slope_h * (i - j), times v."""
    n, H, d = q.shape
    G = k.shape[1]
    pos = torch.as_tensor(positions, dtype=F64)
    dist = pos[:, None] - pos[None, :]
    out = torch.zeros(n, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale - head_slopes[h] * dist
        s = s.masked_fill(dist < 0, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def attention_keys_as_values(h, w, prefix, m, eps, positions):
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    n = h.shape[0]
    q = h @ w[prefix + "q"].T + w[prefix + "q.b"]
    k = h @ w[prefix + "k"].T + w[prefix + "k.b"]
    v = k.clone()                                             # the value is the key as projected
    q = rms(q, eps) * w[prefix + "q.norm"]                    # over all heads at once
    k = rms(k, eps) * w[prefix + "k.norm"]
    if m.get("q_temp"):
        q = q * query_temperature(positions, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None]
    o = attention_scores_to_output(q.reshape(n, H, d), k.reshape(n, G, d), v.reshape(n, G, d), m["scale"],
                                   slopes(H), positions)
    return o.reshape(n, H * d) @ w[prefix + "o"].T + w[prefix + "o.b"]


def delta_inputs(h, w, prefix, heads, dim):
    """r, k, v, decay, removal rate [n, heads, dim] and the output gate [n, heads * dim]."""
    n = h.shape[0]
    r, k, v = (h @ w[prefix + t].T for t in ("r", "k", "v"))
    low = torch.tanh(h @ w[prefix + "w1"].T) @ w[prefix + "w2"].T + w[prefix + "w0"]
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(low))
    rate = torch.sigmoid(h @ w[prefix + "a"].T + w[prefix + "a.b"])
    gate = torch.sigmoid(h @ w[prefix + "g"].T)
    shape = (n, heads, dim)
    return r.reshape(shape), k.reshape(shape), v.reshape(shape), decay.reshape(shape), rate.reshape(shape), gate


def delta_recurrence(r, k, v, decay, rate, state=None):
    """S_t = diag(decay) S - (rate * u)(u^T S) + k v^T with u = k / sqrt(k.k + 1e-6), both terms
    reading the old S; o_t = S_t^T r.  Returns (o [n, heads, dim], last S [heads, dim, dim])."""
    n, heads, dim = r.shape
    S = torch.zeros(heads, dim, dim, dtype=F64) if state is None else state.clone()
    o = torch.zeros(n, heads, dim, dtype=F64)
    for t in range(n):
        for h in range(heads):
            u = k[t, h] / torch.sqrt((k[t, h] * k[t, h]).sum() + 1e-6)
            old = S[h]
            S[h] = decay[t, h][:, None] * old - torch.outer(rate[t, h] * u, u @ old) + torch.outer(k[t, h], v[t, h])
            o[t, h] = S[h].T @ r[t, h]
    return o, S


def general_delta(h, w, prefix, m, eps, state=None):
    heads, dim = m["heads"], m["dim"]
    r, k, v, decay, rate, gate = delta_inputs(h, w, prefix, heads, dim)
    o, S = delta_recurrence(r, k, v, decay, rate, state)
    o = rms(o, eps).reshape(h.shape[0], heads * dim) * w[prefix + "norm"] * gate
    return o @ w[prefix + "o"].T, S


# ----------------------------------------------------------------------------- the model

def forward(w, cfg, tokens, layers_out=None):
    """Logits [n, vocab] of one whole sequence from position 0; ``layers_out`` (a list)
    receives the residual stream after every layer."""
    w = {k: v.to(F64) for k, v in w.items()}
    D, eps, groups, mult = cfg["width"], cfg["norm"]["eps"], cfg["norm"].get("groups", 1), cfg.get("residual_mult", 1.0)
    n = len(tokens)
    positions = list(range(n))
    x = w["embed"][torch.tensor(tokens)] + sinusoid(positions, D)
    for i, layer in enumerate(cfg["layers"]):
        h = group_norm(x, w[f"l{i}.norm1"], groups, eps)
        if layer["type"] == "attention":
            y = attention_keys_as_values(h, w, f"l{i}.mix.", layer["mixer"], eps, positions)
        else:
            y, _ = general_delta(h, w, f"l{i}.mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            y = y + dense_mlp(h, w[f"l{i}.mlp.up"], w[f"l{i}.mlp.down"], w[f"l{i}.mlp.act"])
        x = x + mult * y
        if layers_out is not None:
            layers_out.append(x.clone())
    return group_norm(x, w["final.norm"], groups, eps) @ w["head"].T


def greedy(w, cfg, prompt, new_tokens):
    ids = list(prompt)
    for _ in range(new_tokens):
        ids.append(int(forward(w, cfg, ids)[-1].argmax()))
    return ids[len(prompt):]


# ----------------------------------------------------------------------------- weights

def tensor_shapes(cfg, rank=8):
    D, V = cfg["width"], cfg["vocab"]
    shapes = {"embed": (V, D), "final.norm": (D,), "head": (V, D)}
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}."
        shapes[p + "norm1"] = (D,)
        if layer["type"] == "attention":
            q, k = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
            shapes.update({p + "mix.q": (q, D), p + "mix.q.b": (q,), p + "mix.k": (k, D), p + "mix.k.b": (k,),
                           p + "mix.q.norm": (q,), p + "mix.k.norm": (k,), p + "mix.o": (D, q), p + "mix.o.b": (D,)})
        else:
            hd, low = m["heads"] * m["dim"], m.get("rank", rank)
            for t in ("r", "k", "v", "g", "a"):
                shapes[p + "mix." + t] = (hd, D)
            shapes.update({p + "mix.a.b": (hd,), p + "mix.w1": (low, D), p + "mix.w2": (hd, low), p + "mix.w0": (hd,),
                           p + "mix.norm": (hd,), p + "mix.o": (D, hd)})
        if layer.get("mlp") is not None:
            f = layer["mlp"]["ff"]
            shapes.update({p + "mlp.up": (f, D), p + "mlp.down": (D, f), p + "mlp.act": (2,)})
    return shapes


def random_weights(cfg, seed, rank=8, std=None):
    """Float32 weights large enough that every mechanism shows in the logits: matrices
    N(0, 1/fan_in) times 1.5, norm weights around 1, biases and the embedding of size 0.5."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, rank).items():
        if len(shape) == 2 and name != "embed":
            t = torch.randn(shape, generator=g) * (1.5 / math.sqrt(shape[1]) if std is None else std)
        elif name.endswith("norm1") or name.endswith(".norm") or name == "final.norm":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g)
        else:
            t = 0.5 * torch.randn(shape, generator=g)
        out[name] = t
    return out
