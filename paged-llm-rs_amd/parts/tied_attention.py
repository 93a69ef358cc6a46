"""Grouped-query softmax attention over the paged cache without a value projection: a token's values are its
keys as projected (with the bias), before the keys are normed and turned.

q and k may carry biases.  q is normed over ALL its heads at once, one root mean square over the whole
projection with a gain a column, and k likewise.  The first ``rotary_dims`` values of every head turn in
neighbouring pairs (2i, 2i + 1) by position * f_i; the frequencies may be rescaled by their wavelength
(``rotary.rotary_frequencies``).  The mask is a window or blocks of positions, as the attention kernels take
either.  One kernel stands between the projection and the attention kernel (``kernels.wide_prepare``): biases, the
two statistics, gains, rotation, queries out, keys into the key pool and the raw keys into the value pool, all
in 32-bit from the projection's 32-bit sums, one rounding at the store.
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
from .rotary import rotary_frequencies


class TiedAttention:
    graph_safe = True
    short_portion = kernels.SHORT_PORTION
    # forward takes a norm still to run in place of rows (its one product, ``proj``, reads them)
    takes_pending_norm = True

    @staticmethod
    def declare(spec, hidden: int) -> list:
        H, G, D = spec.num_heads, spec.num_kv_heads, spec.head_dim
        decls = [ParamDecl("q", (H * D, hidden)), ParamDecl("k", (G * D, hidden))]
        if spec.qk_bias:
            decls += [ParamDecl("q.b", (H * D,), "bias"), ParamDecl("k.b", (G * D,), "bias")]
        if spec.qk_norm_eps is not None:
            decls += [ParamDecl("q.norm", (H * D,), "gain"), ParamDecl("k.norm", (G * D,), "gain")]
        decls.append(ParamDecl("o", (hidden, H * D)))
        return decls

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        H, G, D = spec.num_heads, spec.num_kv_heads, spec.head_dim
        if spec.mask not in ("window", "block"):
            raise UnsupportedError(f"a mask of kind {spec.mask!r} (window or block)")
        if H < 1 or G < 1 or H % G:
            raise UnsupportedError(f"{H} query heads over {G} key heads, which do not group evenly")
        if spec.rotary_dims % 2 or not 0 <= spec.rotary_dims <= D:
            raise UnsupportedError(f"a rotation over {spec.rotary_dims} values of a head of {D}")
        unit = 1 if dtype == torch.float32 else 16       # the bfloat16 attention kernels take head sizes in 16s
        self.padded = (D + unit - 1) // unit * unit
        if not 1 <= self.padded <= 1024:
            raise UnsupportedError(f"heads of {D}: the attention kernels take head sizes up to 1024")
        self.spec, self.dtype = spec, dtype
        self.H, self.G, self.D = H, G, D
        self.scale = float(spec.scale) if spec.scale is not None else 1.0 / math.sqrt(D)
        self.window = int(spec.window or 0)
        # what the attention kernels are told: a window as it is, blocks of positions as a negative number
        self.mask = -self.window if spec.mask == "block" else self.window
        # (the biases are added where the projection's 32-bit sums are read next, in the prepare kernel)
        self.bias = (torch.cat([params["q.b"], params["k.b"]]).to(torch.float32).contiguous() if spec.qk_bias else None)
        self.proj = Linear.fused([params["q"], params["k"]])
        normed = spec.qk_norm_eps is not None
        self.q_gain = params["q.norm"].to(torch.float32).contiguous() if normed else None
        self.k_gain = params["k.norm"].to(torch.float32).contiguous() if normed else None
        self.freq = (rotary_frequencies(spec.rotary_dims, spec.rotary_base, spec.rotary_scaling, device)
                     if spec.rotary_dims else None)
        w_o = params["o"]
        if self.padded != D:
            wide = torch.zeros((hidden, H, self.padded), dtype=w_o.dtype, device=w_o.device)
            wide[:, :, :D] = w_o.view(hidden, H, D)
            w_o = wide.view(hidden, H * self.padded)
        self.o_proj = Linear(w_o)

    def cache_spec(self):
        # (no key further back than the window's or the block's size is ever read: pages behind it come back)
        return KVCacheSpec(self.G, self.padded, self.window or None)

    def state_spec(self):
        return None

    def forward(self, x, ctx):
        """``x``: the normed rows, or a norm still to run.  The output comes back as 32-bit sums, or None where the
        output projection added them into ``ctx.residual`` itself."""
        batch, kv = ctx.batch, ctx.kv()
        rows = self.proj.forward(x, out_dtype=torch.float32)
        n = rows.shape[0]
        q = torch.empty((n, self.H * self.padded), dtype=self.dtype, device=rows.device)
        kernels.wide_prepare(rows, 0, batch, kv, q, self.H, self.G, self.D, self.padded, norm_eps=self.spec.qk_norm_eps,
                             q_gain=self.q_gain, k_gain=self.k_gain, freq=self.freq, rot=self.spec.rotary_dims,
                             write_kv=ctx.writes_cache, bias=self.bias)
        out = torch.empty((n, self.H * self.padded), dtype=self.dtype, device=rows.device)
        kernels.sink_attention(q, out, batch, kv, self.H, self.G, self.padded, self.scale, self.mask)
        return self.o_proj.forward(out, out_dtype=torch.float32, add_into=getattr(ctx, "residual", None))


register_mixer("tied_attention", TiedAttention)
