"""Attention whose pages hold one small vector a token.

A layer projects its input onto ``kv_rank`` values, normalises them (c), and onto one rotated key part of
``rotary_dim`` values that all heads share; the token's row of the pages is [c | rotated key part].  A head's
keys and values are linear in c, k_h = U_h c and v_h = W_h c, so they are never built: a query's unrotated
part is carried into c's space once, q~_h = U_h^T q_h, and

    score_ij = scale (q~_ih . c_j + rot(q)_ih . rot(k)_j),     read-out_ih = W_h (sum_j weight_ij c_j),

which is attention of H query heads over ONE key head whose keys are the pages' rows and whose values are the
first kv_rank values of those same rows (``KVCacheSpec.values_in_keys``).  The softmax may have a learned
sink a head, the read-out a gate a head (the sigmoid of a projection of the layer's input).  A layer built
with ``borrows`` has no projection onto c: the schedule names the layer whose pages it reads, with its own
queries, U, W, sinks and gates.
"""

from __future__ import annotations

import math

import torch

from .. import kernels
from ..cache.layout import KVCacheSpec
from ..config.specs import PositionSpec
from ..errors import UnsupportedError
from ..weights.loader import ParamDecl
from .linear import Linear
from .registry import register_mixer
from .rotary import rotary_frequencies, rotary_tables
from .sink_attention import head_sinks


class LatentAttention:
    graph_safe = True
    short_portion = kernels.SHORT_PORTION
    # forward takes a norm still to run in place of rows (its one product, ``proj``, reads them)
    takes_pending_norm = True

    @staticmethod
    def declare(spec, hidden: int) -> list:
        H, D, rot, V, R = spec.num_heads, spec.head_dim, spec.rotary_dim, spec.value_dim, spec.kv_rank
        decls = [ParamDecl("q", (H * (D + rot), hidden))]
        if not spec.borrows:
            decls += [ParamDecl("dkv", (R + rot, hidden)), ParamDecl("dkv.norm", (R,), "gain")]
        decls += [ParamDecl("uk", (H * D, R)), ParamDecl("uv", (H * V, R))]
        if spec.sink == "learned":
            decls.append(ParamDecl("sink", (H,), "bias"))
        if spec.gated:
            decls.append(ParamDecl("g", (H * V if spec.gate_each == "element" else H, hidden)))
        decls.append(ParamDecl("o", (hidden, H * V)))
        return decls

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        H, D, rot, V, R = spec.num_heads, spec.head_dim, spec.rotary_dim, spec.value_dim, spec.kv_rank
        unit = 1 if dtype == torch.float32 else 16       # the bfloat16 attention kernels take head sizes in 16s
        self.padded = (R + rot + unit - 1) // unit * unit
        if not 1 <= self.padded <= 1024:
            raise UnsupportedError(f"vectors of {R} with a rotated part of {rot}: the attention kernels take rows up to 1024")
        if spec.rotary_turned % 2 or not 0 <= spec.rotary_turned <= rot:
            raise UnsupportedError(f"a rotation over {spec.rotary_turned} values of a part of {rot}")
        if spec.gate_each not in ("head", "element"):
            raise UnsupportedError(f"a gate a {spec.gate_each!r} (head or element)")
        self.spec, self.dtype = spec, dtype
        self.H, self.D, self.rot, self.V, self.R = H, D, rot, V, R
        self.scale = float(spec.scale) if spec.scale is not None else 1.0 / math.sqrt(D + rot)
        self.window = int(spec.window or 0)
        # one product for everything the layer's input is projected onto: the row is [q | gates | c, key part]
        pieces = [params["q"]]
        self.gate_off = self.kv_off = 0
        if spec.gated:
            self.gate_off = H * (D + rot)
            pieces.append(params["g"])
        if not spec.borrows:
            self.kv_off = sum(p.shape[0] for p in pieces)
            pieces.append(params["dkv"])
            self.gain = params["dkv.norm"].to(torch.float32).contiguous()
        else:
            self.gain = None
        self.proj = Linear.fused(pieces)
        # U_h^T as the weights of a product a head, [H, R, D], and W_h, [H, V, R]
        self.uk_t = params["uk"].view(H, D, R).transpose(1, 2).contiguous()
        self.uv = params["uv"].view(H, V, R).contiguous()
        self.sinks = head_sinks(spec.sink, H, params, device)
        # the rotation's angles: tables of cosines and sines where the spec bounds the positions, otherwise the
        # frequencies alone (rounded from 64-bit), and the kernel multiplies by the position in 32-bit
        self.cos = self.sin = None
        if spec.rotary_turned and spec.max_positions:
            if getattr(spec, "rotary_scaling", None) is not None:
                raise UnsupportedError("rescaled rotation frequencies with tables of angles (max_positions = 0 works the angles out)")
            rotary = rotary_tables(PositionSpec("rotary_neighbours", spec.rotary_turned, float(spec.rotary_base),
                                                int(spec.max_positions)), device, shared)
            self.cos, self.sin = rotary.cos, rotary.sin
        elif spec.rotary_turned:
            self.cos = rotary_frequencies(spec.rotary_turned, spec.rotary_base, getattr(spec, "rotary_scaling", None), device)
        self.o_proj = Linear(params["o"])

    def cache_spec(self):
        return KVCacheSpec(1, self.padded, self.window or None, values_in_keys=True)

    def state_spec(self):
        return None

    def forward(self, x, ctx):
        """``x``: the normed rows, or a norm still to run.  The output comes back as 32-bit sums, or None where the output projection
        added them into ``ctx.residual`` itself."""
        batch, kv = ctx.batch, ctx.kv()
        H, D, rot, V, R, P = self.H, self.D, self.rot, self.V, self.R, self.padded
        rows = self.proj.forward(x, out_dtype=torch.float32)
        n = rows.shape[0]
        q = torch.empty((n, H * P), dtype=self.dtype, device=rows.device)
        q_plain = torch.empty((H, n, D), dtype=self.dtype, device=rows.device)
        kernels.latent_prepare(rows, 0, self.kv_off, self.gain, self.spec.norm_eps, self.cos, self.sin, self.spec.rotary_turned,
                               batch, kv, q_plain, q, H, D, rot, R, P,
                               write_kv=ctx.writes_cache and not self.spec.borrows)
        kernels.gemm_heads(q_plain.transpose(0, 1), self.uk_t, q.view(n, H, P)[:, :, :R])
        out = torch.empty((n, H * P), dtype=self.dtype, device=rows.device)
        kernels.sink_attention(q, out, batch, kv, H, 1, P, self.scale, self.window, sinks=self.sinks)
        values = torch.empty((n, H * V), dtype=self.dtype, device=rows.device)
        kernels.gemm_heads(out.view(n, H, P)[:, :, :R], self.uv, values.view(n, H, V))
        if self.spec.gated:
            kernels.head_gate_(values, rows, self.gate_off, batch.positions, H, V,
                               each_element=self.spec.gate_each == "element")
        return self.o_proj.forward(values, out_dtype=torch.float32, add_into=getattr(ctx, "residual", None))


register_mixer("latent_attention", LatentAttention)
