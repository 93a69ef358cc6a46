"""Grouped-query softmax attention over the paged cache with, as the spec asks, a sink in the softmax's
denominator, q and k as unit vectors (divided by their root mean square over a head, with or without a
gain), biases on the projections, a query temperature that grows with the logarithm of the position, a
penalty a head on the distance between query and key, and a window or a mask of blocks (a query sees the
keys of its own block of positions, blocks counted from the request's position 0).

weights_ij = exp(s_ij) / (exp(sink_h) + sum over the visible j of exp(s_ij)),
s_ij = scale (q_i . k_j) - slope_h (i - j); a sink has no key and no value, so a row's weights sum to
less than one.  One kernel stands between the projection and the attention kernel (unit vectors,
temperature, queries out, keys and values into the pages), all in 32-bit from the projection's 32-bit
sums, one rounding at the store.  Query/key heads and value heads may differ in size: every head is
stored in a row of ``padded`` values with zeros behind its own, and the output projection's columns are
padded alike once, at load.
"""

from __future__ import annotations

import math

import torch

from .. import kernels
from ..cache.layout import KVCacheSpec
from ..errors import UnsupportedError
from ..weights.loader import ParamDecl
from .linear import Linear
from .registry import register_mixer


def head_sinks(kind, heads: int, params: dict, device):
    """The sink of every head as 32-bit numbers: zeros, the tensor ``sink``, or None where there is none."""
    if kind is None:
        return None
    if kind == "zero":
        return torch.zeros((heads,), dtype=torch.float32, device=device)
    if kind == "learned":
        return params["sink"].to(torch.float32).contiguous()
    raise UnsupportedError(f"a sink of kind {kind!r} (zero, learned or none)")


def head_slopes(kind, heads: int, span: float, device):
    """The distance penalty of every head: ``geometric`` is 2^(-span (h + 1) / heads)."""
    if kind is None:
        return None
    if kind != "geometric":
        raise UnsupportedError(f"distance slopes of kind {kind!r} (geometric or none)")
    return torch.tensor([2.0 ** (-span * (h + 1) / heads) for h in range(heads)], dtype=torch.float64).to(
        torch.float32).to(device)


class SinkAttention:
    graph_safe = True
    short_portion = kernels.SHORT_PORTION
    # forward takes a norm still to run in place of rows (its one product, ``proj``, reads them)
    takes_pending_norm = True

    @staticmethod
    def declare(spec, hidden: int) -> list:
        H, G, D, V = spec.num_heads, spec.num_kv_heads, spec.head_dim, spec.value_dim
        decls = [ParamDecl("q", (H * D, hidden)), ParamDecl("k", (G * D, hidden)), ParamDecl("v", (G * V, hidden)),
                 ParamDecl("o", (hidden, H * V))]
        if spec.sink == "learned":
            decls.append(ParamDecl("sink", (H,), "bias"))
        if spec.qk_gain:
            decls += [ParamDecl("q.norm", (D,), "gain"), ParamDecl("k.norm", (D,), "gain")]
        if spec.qkv_bias:
            decls += [ParamDecl("q.b", (H * D,), "bias"), ParamDecl("k.b", (G * D,), "bias"), ParamDecl("v.b", (G * V,), "bias")]
        return decls

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        H, G, D, V = spec.num_heads, spec.num_kv_heads, spec.head_dim, spec.value_dim
        if spec.mask not in ("window", "block"):
            raise UnsupportedError(f"a mask of kind {spec.mask!r} (window or block)")
        if spec.qk_gain and spec.qk_unit_eps is None:
            raise UnsupportedError("a gain on q and k that are not divided by their root mean square")
        if H < 1 or G < 1 or H % G:
            raise UnsupportedError(f"{H} query heads over {G} key heads, which do not group evenly")
        unit = 1 if dtype == torch.float32 else 16       # the bfloat16 attention kernels take head sizes in 16s
        self.padded = (max(D, V) + unit - 1) // unit * unit
        if not 1 <= self.padded <= 1024:
            raise UnsupportedError(f"heads of {D} and {V}: the attention kernels take head sizes up to 1024")
        if spec.temperature_coef is not None and spec.temperature_every < 1:
            raise UnsupportedError(f"a query temperature every {spec.temperature_every} positions")
        self.spec, self.dtype = spec, dtype
        self.H, self.G, self.D, self.V = H, G, D, V
        self.scale = float(spec.scale) if spec.scale is not None else 1.0 / math.sqrt(D)
        self.window = int(spec.window or 0)
        # what the attention kernels are told: a window as it is, blocks of positions as a negative number
        self.mask = -self.window if spec.mask == "block" else self.window
        # (the biases are added where the projection's 32-bit sums are read next, in the prepare kernel: the product
        # keeps what it fuses, and a pass over the rows is saved)
        self.bias = (torch.cat([params["q.b"], params["k.b"], params["v.b"]]).to(torch.float32).contiguous()
                     if spec.qkv_bias else None)
        self.proj = Linear.fused([params["q"], params["k"], params["v"]])
        self.q_gain = params["q.norm"].to(torch.float32).contiguous() if spec.qk_gain else None
        self.k_gain = params["k.norm"].to(torch.float32).contiguous() if spec.qk_gain else None
        self.sinks = head_sinks(spec.sink, H, params, device)
        self.slopes = head_slopes(spec.distance_slopes, H, float(spec.slope_span), device)
        self.temperature = ((float(spec.temperature_coef), int(spec.temperature_every))
                            if spec.temperature_coef is not None else None)
        w_o = params["o"]
        if self.padded != V:
            wide = torch.zeros((hidden, H, self.padded), dtype=w_o.dtype, device=w_o.device)
            wide[:, :, :V] = w_o.view(hidden, H, V)
            w_o = wide.view(hidden, H * self.padded)
        self.o_proj = Linear(w_o)

    def cache_spec(self):
        # (no key further back than the block's size is ever read: pages behind it come back as behind a window)
        return KVCacheSpec(self.G, self.padded, self.window or None)

    def state_spec(self):
        return None

    def forward(self, x, ctx):
        """``x``: the normed rows, or a norm still to run.  The output comes back as 32-bit sums, or None where the output projection
        added them into ``ctx.residual`` itself."""
        batch, kv = ctx.batch, ctx.kv()
        rows = self.proj.forward(x, out_dtype=torch.float32)
        n = rows.shape[0]
        q = torch.empty((n, self.H * self.padded), dtype=self.dtype, device=rows.device)
        kernels.head_prepare(rows, 0, batch, kv, q, self.H, self.G, self.D, self.V, self.padded,
                             unit_eps=self.spec.qk_unit_eps, q_gain=self.q_gain, k_gain=self.k_gain,
                             temperature=self.temperature, write_kv=ctx.writes_cache, bias=self.bias)
        out = torch.empty((n, self.H * self.padded), dtype=self.dtype, device=rows.device)
        kernels.sink_attention(q, out, batch, kv, self.H, self.G, self.padded, self.scale, self.mask,
                               sinks=self.sinks, slopes=self.slopes)
        return self.o_proj.forward(out, out_dtype=torch.float32, add_into=getattr(ctx, "residual", None))


register_mixer("sink_attention", SinkAttention)
