"""A recurrent mixer with a matrix state per head, updated by a generalized delta rule.

Per head, with r, k, v projections of the input, a decay w and a removal rate a per key
channel, and the unit key u = k / sqrt(sum(k^2) + key_eps):

    S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T      o_t = S_t^T r_t

    w = exp(-decay_scale * sigmoid(W_w2 tanh(W_w1 x) + w0))       a = sigmoid(W_a x + a_bias)

Each head's o is divided by its root mean square, the heads are concatenated, multiplied by
a weight and by sigmoid(W_g x), and projected by W_o.  The state [heads, dim, dim] is 32-bit,
one per request, kept in a state slot between steps and started from zero at position 0;
everything that enters the recurrence besides the projections is 32-bit.

Parameters: ``hidden``, ``heads``, ``head_dim``, ``eps`` (of the output norm), ``rank`` (width
of the decay's low-rank path; None: read from the checkpoint), ``decay_scale`` (default
exp(-1/2)), ``key_eps`` (default 1e-6).  Tensors: ``<prefix>.{r,k,v,g,a,w1,w2,o}.weight``,
``.a.bias``, ``.w0``, ``.norm``.  The six input projections are kept as one matrix.
"""

from __future__ import annotations

import math

import torch

from .. import kernels as K
from .base import Part, register_part
from .linear import decode_linear, linear, tiled_copy
from .spec import CacheNeed, WeightSpec


@register_part("mixer", "general_delta")
class GeneralDeltaMixer(Part):
    graph_safe = True
    records_launches = True
    # From this many tokens on the second product of the decay's low-rank path is a matrix
    # product of its own (tanh rounded to the compute dtype in between, as any activation that
    # feeds a product); below, the kernel that prepares the recurrence's inputs does it.
    LOW_RANK_PRODUCT_ROWS = 17

    def __init__(self, spec, runtime):
        super().__init__(spec, runtime)
        self.hidden = int(self.param("hidden"))
        self.heads = int(self.param("heads"))
        self.head_dim = int(self.param("head_dim"))
        self.eps = float(self.param("eps"))
        rank = self.param("rank", None)
        self.rank = int(rank) if rank else -1
        self.decay_scale = float(self.param("decay_scale", math.exp(-0.5)))
        self.key_eps = float(self.param("key_eps", 1e-6))
        self.width = self.heads * self.head_dim
        self.w_in = self.w2 = self.w0 = self.a_bias = self.norm_weight = self.w_o = None

    def weight_specs(self):
        wide = (self.width, self.hidden)
        return ([WeightSpec(self.tensor_name(f"{n}.weight"), wide) for n in ("r", "k", "v", "g", "a")]
                + [WeightSpec(self.tensor_name("w1.weight"), (self.rank, self.hidden)),
                   WeightSpec(self.tensor_name("w2.weight"), (self.width, self.rank)),
                   WeightSpec(self.tensor_name("o.weight"), (self.hidden, self.width)),
                   WeightSpec(self.tensor_name("a.bias"), (self.width,), "vector"),
                   WeightSpec(self.tensor_name("w0"), (self.width,), "vector"),
                   WeightSpec(self.tensor_name("norm"), (self.width,), "vector")])

    def bind(self, weights):
        self.w_in = torch.cat([weights[self.tensor_name(f"{n}.weight")] for n in ("r", "k", "v", "g", "a", "w1")],
                              dim=0).contiguous()
        self.w2 = weights[self.tensor_name("w2.weight")]
        if self.w2.shape[1] != self.w_in.shape[0] - 5 * self.width:
            raise ValueError("general_delta: the two matrices of the decay's low-rank path do not fit")
        self.w_o = weights[self.tensor_name("o.weight")]
        self.a_bias = weights[self.tensor_name("a.bias")]
        self.w0 = weights[self.tensor_name("w0")]
        self.norm_weight = weights[self.tensor_name("norm")]
        # second copies for decode batches, in the order that kernel reads them
        self._tiled = {"in": tiled_copy(self.runtime, self.w_in, K.LINEAR_PARTS),
                       "o": tiled_copy(self.runtime, self.w_o, K.LINEAR_PARTS)}

    def cache_need(self):
        return CacheNeed("state", state_shape=(self.heads, self.head_dim, self.head_dim))

    def check_cache(self, page_size):
        if self.head_dim > K.delta_scan_max_dim():
            raise ValueError(f"general_delta: heads of {self.head_dim} are not built (up to {K.delta_scan_max_dim()})")

    def flops(self, tokens, keys_read=0.0):
        # the projections, and per token and head three passes over the state
        return super().flops(tokens) + 8.0 * tokens * self.heads * self.head_dim * self.head_dim

    def forward(self, ctx, xn, cache):
        n = xn.shape[0]
        f32 = torch.float32
        proj = decode_linear(ctx, xn, self.w_in, "delta.proj", self._tiled.get("in"))
        low = None
        if n >= self.LOW_RANK_PRODUCT_ROWS:
            rank = self.w2.shape[1]
            t = ctx.buf("delta.tanh", (n, rank), self.runtime.dtype)
            K.unary_act(proj, t, K.ACT_TANH, first_column=5 * self.width)
            low = linear(ctx, t, self.w2, "delta.low")
        scan_in = ctx.buf("delta.scan_in", (self.heads, n, K.DELTA_SCAN_FIELDS, self.head_dim), f32)
        gate = ctx.buf("delta.gate", (n, self.width), f32)
        K.delta_prep(proj, self.a_bias, self.w2, self.w0, self.decay_scale, self.key_eps, scan_in, gate,
                     self.heads, self.head_dim, low=low)
        o = ctx.buf("delta.o", (n, self.width), f32)
        K.delta_scan(scan_in, o, cache.state, cache.slots, ctx.span_start, ctx.span_pos, ctx.n_spans)
        out = ctx.buf("delta.out", (n, self.width), self.runtime.dtype)
        K.delta_out(o, gate, self.norm_weight, self.eps, out, self.heads, self.head_dim)
        return decode_linear(ctx, out, self.w_o, "delta.o_proj", self._tiled.get("o"))
