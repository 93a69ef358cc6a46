"""The pre-norm arrangement of a layer: norm, mixer, residual, norm,
feed-forward, residual (reference: model/mod.rs:84-136).

The residual stream is 32-bit.  A block receives the stream and the previous
block's output that has not been added yet, adds it inside its first norm, and
returns its own feed-forward output unadded, so that every residual sum is
fused with the norm that follows it.  With few rows the fusion goes the other
way: a part that can adds its output into the stream as the last stage of its
product kernel and the norm becomes the first stage of the next product.
"""

from __future__ import annotations

import torch

from .. import kernels
from ..errors import ConfigError
from .norm import PendingNorm
from .registry import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, lookup, prefixed, register_block, scoped)


class PreNormBlock:
    NAMES = {"norm1": "input_layernorm", "mixer": "self_attn", "norm2": "post_attention_layernorm",
             "feed_forward": "mlp"}

    @classmethod
    def names_of(cls, layer) -> dict:
        """The name parts of the members' tensors: this architecture's, or the layer spec's own."""
        given = getattr(layer, "names", None) or {}
        unknown = sorted(set(given) - set(cls.NAMES))
        if unknown:
            raise ConfigError(f"a layer names members that this arrangement does not have: {unknown}")
        return {**cls.NAMES, **given}

    @classmethod
    def declare(cls, layer, hidden: int) -> list:
        norm = lookup(NORMS, layer.norm.kind, "norm")
        mixer = lookup(MIXERS, layer.mixer.kind, "mixer")
        ffn = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")
        n = cls.names_of(layer)
        return (prefixed(norm.declare(layer.norm, hidden), n["norm1"])
                + prefixed(mixer.declare(layer.mixer, hidden), n["mixer"])
                + prefixed(norm.declare(layer.norm, hidden), n["norm2"])
                + prefixed(ffn.declare(layer.feed_forward, hidden), n["feed_forward"]))

    def __init__(self, layer, hidden: int, params: dict, dtype, device, shared: dict):
        n = self.names = self.names_of(layer)
        norm = lookup(NORMS, layer.norm.kind, "norm")
        self.dtype = dtype
        self.norm1 = norm(layer.norm, hidden, scoped(params, n["norm1"]), dtype, device)
        self.mixer = lookup(MIXERS, layer.mixer.kind, "mixer")(
            layer.mixer, hidden, scoped(params, n["mixer"]), dtype, device, shared)
        self.norm2 = norm(layer.norm, hidden, scoped(params, n["norm2"]), dtype, device)
        self.feed_forward = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")(
            layer.feed_forward, hidden, scoped(params, n["feed_forward"]), dtype, device, shared)

    @property
    def graph_safe(self) -> bool:
        """Whether a step through this block may be captured as a HIP graph: a part that
        reads device values on the host, or allocates by data, sets ``graph_safe = False``."""
        return getattr(self.mixer, "graph_safe", True) and getattr(self.feed_forward, "graph_safe", True)

    @property
    def first_norm(self):
        """The norm this block applies to the stream first: the block before may leave its work behind."""
        return self.norm1

    @staticmethod
    def _room(norm, resid):
        """Room for ``norm`` handed forward over the rows of ``resid``, where the norm has such a thing."""
        make = getattr(norm, "handoff", None)
        return make(resid.shape[0], resid.device) if make is not None else None

    def forward(self, resid, delta, ctx):
        """``delta``: what the block before has not added to the stream yet, or None.  Returns this
        block's own unadded output, or None when the feed-forward added it itself."""
        if ctx.trace is not None:
            return self._forward_recorded(resid, delta, ctx)
        mixer_fuses = getattr(self.mixer, "fuses", False)
        ffn_fuses = getattr(self.feed_forward, "fuses", False)
        half = self.dtype == torch.bfloat16
        if delta is None and mixer_fuses:
            # every sum is in the stream already (and the product that added the last may have left this norm's work)
            x = PendingNorm(self.norm1, resid, self.dtype, handed=getattr(ctx, "handed", None))
        else:
            x = self.norm1.apply(resid, delta, self.dtype)
        ctx.residual = resid if mixer_fuses else None
        # a mixer that adds into the stream may leave the second norm's work behind ...
        ctx.hand = self._room(self.norm2, resid) if half and mixer_fuses and ffn_fuses else None
        mixed = self.mixer.forward(x, ctx)
        left, ctx.residual, ctx.hand = ctx.hand, None, None
        if mixed is None and ffn_fuses:
            x = PendingNorm(self.norm2, resid, self.dtype, handed=left)
        else:
            x = self.norm2.apply(resid, mixed, self.dtype)
        if ffn_fuses:
            # ... and a feed-forward that does, the next layer's first norm's
            after = getattr(ctx, "norm_after", None)
            if half and after is not None and getattr(self.feed_forward, "hands_forward", False):
                room = self._room(after, resid)
                out = self.feed_forward.forward(x, residual=resid, hand=room)
                ctx.handed_out = room if out is None and room is not None and room.filled else None
                return out
            return self.feed_forward.forward(x, residual=resid)
        return self.feed_forward.forward(x)

    def _forward_recorded(self, resid, delta, ctx):
        """The same layer with every module's output recorded under its name: nothing is fused, so
        every norm runs as a kernel and no part adds into the stream itself.  A part whose class sets
        ``records = True`` takes the recorder (``ctx.trace`` for a mixer, ``trace=`` for a feed-forward)
        and records what happens inside it."""
        n, trace = self.names, ctx.trace
        x = self.norm1.apply(resid, delta, self.dtype)
        trace.record(f"{n['norm1']}.out", x)
        ctx.trace = trace.child(n["mixer"]) if getattr(self.mixer, "records", False) else None
        mixed = self.mixer.forward(x, ctx)
        ctx.trace = trace
        trace.record(f"{n['mixer']}.out", mixed)
        x = self.norm2.apply(resid, mixed, self.dtype)
        trace.record(f"{n['norm2']}.out", x)
        if getattr(self.feed_forward, "records", False):
            out = self.feed_forward.forward(x, trace=trace.child(n["feed_forward"]))
        else:
            out = self.feed_forward.forward(x)
        trace.record(f"{n['feed_forward']}.out", out)
        return out


register_block("pre_norm", PreNormBlock)


class SublayerNormBlock:
    """The arrangement that normalises what a sublayer gives instead of what it gets:
    x <- x + norm1(mixer(x)), then x <- x + norm2(feed_forward(x)); the sublayers read the stream itself.
    A layer whose spec has no feed-forward has the first sublayer only.

    The stream is 32-bit; the parts multiply its rows in the model's type, which the norm kernel that
    updates the stream leaves behind for the next part (``ctx.stream_rows`` carries them from layer to
    layer).  Mixers and feed-forwards hand back 32-bit rows, the unrounded sums of their last product.
    Tensor names: the norms' gains are stored under the norms' own names."""

    NAMES = {"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp"}

    @classmethod
    def names_of(cls, layer) -> dict:
        given = getattr(layer, "names", None) or {}
        unknown = sorted(set(given) - set(cls.NAMES))
        if unknown:
            raise ConfigError(f"a layer names members that this arrangement does not have: {unknown}")
        return {**cls.NAMES, **given}

    @classmethod
    def declare(cls, layer, hidden: int) -> list:
        from ..weights.loader import ParamDecl

        n = cls.names_of(layer)
        mixer = lookup(MIXERS, layer.mixer.kind, "mixer")
        decls = [ParamDecl(n["norm1"], (hidden,), "gain")] + prefixed(mixer.declare(layer.mixer, hidden), n["mixer"])
        if layer.feed_forward is not None:
            ffn = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")
            decls += [ParamDecl(n["norm2"], (hidden,), "gain")] + prefixed(ffn.declare(layer.feed_forward, hidden), n["feed_forward"])
        return decls

    def __init__(self, layer, hidden: int, params: dict, dtype, device, shared: dict):
        n = self.names = self.names_of(layer)
        norm = lookup(NORMS, layer.norm.kind, "norm")
        if not hasattr(norm, "apply_onto"):
            raise ConfigError(f"norm {layer.norm.kind!r} cannot normalise a sublayer's output onto the stream")
        self.dtype = dtype
        self.norm1 = norm(layer.norm, hidden, {"weight": params[n["norm1"]]}, dtype, device)
        self.mixer = lookup(MIXERS, layer.mixer.kind, "mixer")(
            layer.mixer, hidden, scoped(params, n["mixer"]), dtype, device, shared)
        self.norm2 = self.feed_forward = None
        if layer.feed_forward is not None:
            self.norm2 = norm(layer.norm, hidden, {"weight": params[n["norm2"]]}, dtype, device)
            self.feed_forward = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")(
                layer.feed_forward, hidden, scoped(params, n["feed_forward"]), dtype, device, shared)

    @property
    def graph_safe(self) -> bool:
        return getattr(self.mixer, "graph_safe", True) and getattr(self.feed_forward, "graph_safe", True)

    def _rows(self, resid, ctx):
        """The stream's rows in the model's type: what the part before left, or a pass of their own."""
        if self.dtype == torch.float32:
            return resid
        rows = getattr(ctx, "stream_rows", None)
        return rows if rows is not None else kernels.to_bf16(resid)

    def forward(self, resid, delta, ctx):
        if delta is not None:
            kernels.residual_add(resid, delta)
            ctx.stream_rows = None
        rows_dtype = None if self.dtype == torch.float32 else self.dtype
        mixed = self.mixer.forward(self._rows(resid, ctx), ctx)
        ctx.stream_rows = self.norm1.apply_onto(resid, mixed, rows_dtype)
        if self.feed_forward is not None:
            out = self.feed_forward.forward(self._rows(resid, ctx))
            ctx.stream_rows = self.norm2.apply_onto(resid, out, rows_dtype)
        return None


register_block("sublayer_norm", SublayerNormBlock)


class SharedNormBlock:
    """The arrangement with one norm a layer, read by both sublayers: with n = norm1(x),
    x <- x + mixer(n) + feed_forward(n).  A layer whose spec has no feed-forward adds the mixer's output only.

    The stream is 32-bit and every sum into it is: a sublayer's last product adds its 32-bit sums into the
    stream itself where its kernel can, and hands them back 32-bit to be added here where it cannot.
    Tensor names: the norm's gain is stored under the norm's own name."""

    NAMES = {"norm1": "norm1", "mixer": "mix", "feed_forward": "mlp"}

    @classmethod
    def names_of(cls, layer) -> dict:
        given = getattr(layer, "names", None) or {}
        unknown = sorted(set(given) - set(cls.NAMES))
        if unknown:
            raise ConfigError(f"a layer names members that this arrangement does not have: {unknown}")
        return {**cls.NAMES, **given}

    @classmethod
    def declare(cls, layer, hidden: int) -> list:
        from ..weights.loader import ParamDecl

        n = cls.names_of(layer)
        mixer = lookup(MIXERS, layer.mixer.kind, "mixer")
        decls = [ParamDecl(n["norm1"], (hidden,), "gain")] + prefixed(mixer.declare(layer.mixer, hidden), n["mixer"])
        if layer.feed_forward is not None:
            ffn = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")
            decls += prefixed(ffn.declare(layer.feed_forward, hidden), n["feed_forward"])
        return decls

    def __init__(self, layer, hidden: int, params: dict, dtype, device, shared: dict):
        n = self.names = self.names_of(layer)
        norm = lookup(NORMS, layer.norm.kind, "norm")
        self.dtype = dtype
        self.norm1 = norm(layer.norm, hidden, {"weight": params[n["norm1"]]}, dtype, device)
        self.mixer = lookup(MIXERS, layer.mixer.kind, "mixer")(
            layer.mixer, hidden, scoped(params, n["mixer"]), dtype, device, shared)
        self.feed_forward = None
        if layer.feed_forward is not None:
            self.feed_forward = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")(
                layer.feed_forward, hidden, scoped(params, n["feed_forward"]), dtype, device, shared)

    @property
    def graph_safe(self) -> bool:
        return getattr(self.mixer, "graph_safe", True) and getattr(self.feed_forward, "graph_safe", True)

    @property
    def first_norm(self):
        return self.norm1

    def _norm_into_products(self, rows: int) -> bool:
        """Whether the norm runs as the first stage of the two products that read it (few rows of a bfloat16
        model, where both products are the hand-written kernel's) instead of as a kernel of its own."""
        if self.dtype != torch.bfloat16 or not getattr(self.norm1, "fuses_into_product", False):
            return False
        readers = [getattr(self.mixer, "proj", None) if getattr(self.mixer, "takes_pending_norm", False) else None]
        if self.feed_forward is not None:
            readers.append(getattr(self.feed_forward, "gate_up_proj", None) if hasattr(self.feed_forward, "begin") else None)
        return all(r is not None and r.bias is None and kernels.fused_norm_applies(rows, r.in_features, r.weight)
                   and r.out_features <= kernels.FUSED_NORM_MAX_COLUMNS for r in readers)

    def forward(self, resid, delta, ctx):
        ffn = self.feed_forward
        if delta is None and ctx.trace is None and self._norm_into_products(resid.shape[0]):
            # Few rows: the norm is the first stage of the products that read it.  Both read the stream as the layer
            # found it, so the feed-forward's first half runs before the mixer adds its output into the stream.
            rows = PendingNorm(self.norm1, resid, self.dtype)
            act = ffn.begin(rows) if ffn is not None else None
        else:
            # (the norm's rows are written out: two sublayers read them, and the first adds into the stream
            # before the second runs)
            rows, act = self.norm1.apply(resid, delta, self.dtype), None
        ctx.residual = resid
        mixed = self.mixer.forward(rows, ctx)
        ctx.residual = None
        if mixed is not None:
            kernels.residual_add(resid, mixed)
        if ffn is not None:
            if act is not None:
                out = ffn.finish(act, residual=resid, out_dtype=torch.float32)
            elif getattr(ffn, "fuses", False):
                out = ffn.forward(rows, residual=resid, out_dtype=torch.float32)
            else:
                out = ffn.forward(rows)
            if out is not None:
                kernels.residual_add(resid, out)
        return None


register_block("shared_norm", SharedNormBlock)


class PendingCopies:
    """A rebuild of the copies of the stream that has not run yet: the last sublayer's output and its weights.  The
    layer behind runs it in the pass that reads out its own first rows."""

    __slots__ = ("y", "mix", "out")
    filled = True            # (what a layer hands to the next is looked at only when it says it holds something)

    def __init__(self, y, mix, out):
        self.y, self.mix, self.out = y, mix, out


class HyperConnectionBlock:
    """The pre-norm arrangement over several copies of the stream.  The stream a layer gets is [rows, S * width]:
    S copies x_1 .. x_S of every row, one behind the other.  A sublayer (1: the mixer, 2: the feed-forward, where
    the layer has one) reads u = sum_s in[s] x_s through its norm, and its output y rebuilds every copy from all
    of them, x_t <- sum_s mix[s, t] x_s + out[t] y.  A layer spec without ``stream_copies`` has the one stream
    and the plain sums x <- x + y, computed as one copy with weights of one.

    Everything about the copies is 32-bit.  One kernel rebuilds the copies behind a sublayer and reads out the
    next sublayer's normed rows in the same pass (``kernels.hc_step``), also from one layer to the next: a layer
    that is followed by another of this arrangement leaves its last rebuild to that layer's first pass
    (``PendingCopies``), so a layer with a feed-forward is two passes over the copies.  Sublayers hand back 32-bit rows.
    Tensor names: the norms' gains under the norms' own names; ``hc1.in`` [S], ``hc1.out`` [S], ``hc1.mix`` [S, S]
    (from, to) for the mixer and ``hc2.*`` for the feed-forward."""

    NAMES = {"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp", "copies1": "hc1", "copies2": "hc2"}

    @classmethod
    def names_of(cls, layer) -> dict:
        given = getattr(layer, "names", None) or {}
        unknown = sorted(set(given) - set(cls.NAMES))
        if unknown:
            raise ConfigError(f"a layer names members that this arrangement does not have: {unknown}")
        return {**cls.NAMES, **given}

    @staticmethod
    def _copy_decls(name: str, copies: int) -> list:
        from ..weights.loader import ParamDecl

        return [ParamDecl(f"{name}.in", (copies,), "copy_in"), ParamDecl(f"{name}.out", (copies,), "copy_out"),
                ParamDecl(f"{name}.mix", (copies, copies), "copy_mix")]

    @classmethod
    def declare(cls, layer, hidden: int) -> list:
        from ..weights.loader import ParamDecl

        n = cls.names_of(layer)
        copies = layer.stream_copies
        mixer = lookup(MIXERS, layer.mixer.kind, "mixer")
        gain = lookup(NORMS, layer.norm.kind, "norm").declare(layer.norm, hidden)[0].role
        decls = [ParamDecl(n["norm1"], (hidden,), gain)] + prefixed(mixer.declare(layer.mixer, hidden), n["mixer"])
        if copies is not None:
            decls += cls._copy_decls(n["copies1"], copies)
        if layer.feed_forward is not None:
            ffn = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")
            decls += [ParamDecl(n["norm2"], (hidden,), gain)] + prefixed(ffn.declare(layer.feed_forward, hidden), n["feed_forward"])
            if copies is not None:
                decls += cls._copy_decls(n["copies2"], copies)
        return decls

    def __init__(self, layer, hidden: int, params: dict, dtype, device, shared: dict):
        n = self.names = self.names_of(layer)
        norm = lookup(NORMS, layer.norm.kind, "norm")
        if not getattr(norm, "fuses_into_product", False):
            raise ConfigError(f"norm {layer.norm.kind!r} cannot run inside the pass over the copies of the stream "
                              "(it needs a 32-bit gain and an eps, nothing else)")
        self.dtype, self.hidden = dtype, hidden
        self.copies = int(layer.stream_copies or 1)
        if not 1 <= self.copies <= kernels.HC_MAX_COPIES:
            raise ConfigError(f"{self.copies} copies of the stream (1 to {kernels.HC_MAX_COPIES})")
        self.norm1 = norm(layer.norm, hidden, {"weight": params[n["norm1"]]}, dtype, device)
        self.norm1.takes_pending_copies = self.copies       # (how the layer before learns that its last rebuild can wait)
        self.mixer = lookup(MIXERS, layer.mixer.kind, "mixer")(
            layer.mixer, hidden, scoped(params, n["mixer"]), dtype, device, shared)
        self.weights1 = self._copy_weights(params, n["copies1"], layer.stream_copies, device)
        self.norm2 = self.feed_forward = self.weights2 = None
        if layer.feed_forward is not None:
            self.norm2 = norm(layer.norm, hidden, {"weight": params[n["norm2"]]}, dtype, device)
            self.feed_forward = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")(
                layer.feed_forward, hidden, scoped(params, n["feed_forward"]), dtype, device, shared)
            self.weights2 = self._copy_weights(params, n["copies2"], layer.stream_copies, device)

    @staticmethod
    def _copy_weights(params: dict, name: str, copies, device) -> tuple:
        """(in, mix, out) in 32-bit; for the one plain stream all three are one."""
        if copies is None:
            one = torch.ones((1,), dtype=torch.float32, device=device)
            return one, one.view(1, 1), one
        return tuple(params[f"{name}.{part}"].to(torch.float32).contiguous() for part in ("in", "mix", "out"))

    @property
    def graph_safe(self) -> bool:
        return getattr(self.mixer, "graph_safe", True) and getattr(self.feed_forward, "graph_safe", True)

    @property
    def first_norm(self):
        return self.norm1

    def _finish(self, resid, y, mix, out, ctx):
        """The layer's last rebuild: now, or, where the next layer is of this arrangement, in that layer's first pass."""
        after = getattr(ctx, "norm_after", None)
        if ctx.trace is None and after is not None and getattr(after, "takes_pending_copies", None) == self.copies:
            ctx.handed_out = PendingCopies(y, mix, out)
        else:
            kernels.hc_step(resid, self.copies, y=y, mix=mix, out=out)
        return None

    def _feed(self, rows, ctx):
        ffn = self.feed_forward
        if getattr(ffn, "takes_batch", False):
            return ffn.forward(rows, batch=ctx.batch)
        return ffn.forward(rows)

    def forward(self, resid, delta, ctx):
        if delta is not None:
            raise ConfigError("a layer over copies of the stream behind a layer that left its output unadded")
        if resid.shape[1] != self.copies * self.hidden:
            raise ConfigError(f"a stream of rows of {resid.shape[1]} for {self.copies} copies of {self.hidden}")
        S = self.copies
        in1, mix1, out1 = self.weights1
        before = getattr(ctx, "handed", None)
        if isinstance(before, PendingCopies):
            rows = kernels.hc_step(resid, S, y=before.y, mix=before.mix, out=before.out, read=in1, gain=self.norm1.gain32,
                                   eps=self.norm1.eps, read_dtype=self.dtype)
        else:
            rows = kernels.hc_step(resid, S, read=in1, gain=self.norm1.gain32, eps=self.norm1.eps, read_dtype=self.dtype)
        mixed = self.mixer.forward(rows, ctx)
        if self.feed_forward is None:
            return self._finish(resid, mixed, mix1, out1, ctx)
        in2, mix2, out2 = self.weights2
        rows = kernels.hc_step(resid, S, y=mixed, mix=mix1, out=out1, read=in2, gain=self.norm2.gain32,
                               eps=self.norm2.eps, read_dtype=self.dtype)
        return self._finish(resid, self._feed(rows, ctx), mix2, out2, ctx)


register_block("hyper_connections", HyperConnectionBlock)


class PendingSums:
    """What a layer whose sublayers stand side by side has not added to the stream yet: its sublayers' 32-bit outputs
    and their gains a column.  The layer behind adds them in the pass that norms its own rows."""

    __slots__ = ("a", "ls1", "b", "ls2")
    filled = True            # (what a layer hands to the next is looked at only when it says it holds something)

    def __init__(self, a, ls1, b, ls2):
        self.a, self.ls1, self.b, self.ls2 = a, ls1, b, ls2


class ParallelBlock:
    """The arrangement whose sublayers read the same stream through a norm each: with a = norm1(x) and b = norm2(x),
    x <- x + ls1 * mixer(a) + ls2 * feed_forward(b).  ``LayerSpec.layer_scale`` says whether the gains a column ls1 and
    ls2 exist (tensors ``ls1``, ``ls2``); without it the outputs are added as they are.  A layer whose spec has no
    feed-forward adds the mixer's output only (``norm2`` and ``ls2``, if a checkpoint carries them, are not used).

    The stream and every sum into it are 32-bit; sublayers hand back 32-bit rows.  One kernel adds a layer's two outputs
    into the stream and norms the next layer's two rows in the same pass (``kernels.parallel_step``): a layer that is
    followed by another of this arrangement leaves its sums to that layer's pass (``PendingSums``), so a layer is one
    pass over the stream.  ``ctx.stream_addend`` (rows the decoder wants added to the stream before this run) joins
    that pass too.  Tensor names: the norms' gains under the norms' own names."""

    NAMES = {"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp", "scale1": "ls1", "scale2": "ls2"}
    # the decoder may hand this block rows to add to the stream before it runs (``LayerContext.stream_addend``)
    takes_stream_addend = True

    @classmethod
    def names_of(cls, layer) -> dict:
        given = getattr(layer, "names", None) or {}
        unknown = sorted(set(given) - set(cls.NAMES))
        if unknown:
            raise ConfigError(f"a layer names members that this arrangement does not have: {unknown}")
        return {**cls.NAMES, **given}

    @classmethod
    def declare(cls, layer, hidden: int) -> list:
        from ..weights.loader import ParamDecl

        n = cls.names_of(layer)
        mixer = lookup(MIXERS, layer.mixer.kind, "mixer")
        gain = lookup(NORMS, layer.norm.kind, "norm").declare(layer.norm, hidden)[0].role
        scaled = bool(getattr(layer, "layer_scale", False))
        has_ffn = layer.feed_forward is not None
        decls = [ParamDecl(n["norm1"], (hidden,), gain), ParamDecl(n["norm2"], (hidden,), gain, optional=not has_ffn)]
        decls += prefixed(mixer.declare(layer.mixer, hidden), n["mixer"])
        if has_ffn:
            ffn = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")
            decls += prefixed(ffn.declare(layer.feed_forward, hidden), n["feed_forward"])
        if scaled:
            decls += [ParamDecl(n["scale1"], (hidden,), "gain"), ParamDecl(n["scale2"], (hidden,), "gain", optional=not has_ffn)]
        return decls

    def __init__(self, layer, hidden: int, params: dict, dtype, device, shared: dict):
        n = self.names = self.names_of(layer)
        norm = lookup(NORMS, layer.norm.kind, "norm")
        if not getattr(norm, "fuses_into_product", False):
            raise ConfigError(f"norm {layer.norm.kind!r} cannot run inside the pass over the stream of a layer whose "
                              "sublayers stand side by side (it needs a 32-bit gain and an eps, nothing else)")
        self.dtype, self.hidden = dtype, hidden
        self.norm1 = norm(layer.norm, hidden, {"weight": params[n["norm1"]]}, dtype, device)
        self.norm1.takes_pending_sums = True       # (how the layer before learns that its sums can wait)
        self.mixer = lookup(MIXERS, layer.mixer.kind, "mixer")(
            layer.mixer, hidden, scoped(params, n["mixer"]), dtype, device, shared)
        scaled = bool(getattr(layer, "layer_scale", False))
        self.ls1 = params[n["scale1"]].to(torch.float32).contiguous() if scaled else None
        self.norm2 = self.feed_forward = self.ls2 = None
        if layer.feed_forward is not None:
            self.norm2 = norm(layer.norm, hidden, {"weight": params[n["norm2"]]}, dtype, device)
            self.feed_forward = lookup(FEED_FORWARDS, layer.feed_forward.kind, "feed-forward")(
                layer.feed_forward, hidden, scoped(params, n["feed_forward"]), dtype, device, shared)
            self.ls2 = params[n["scale2"]].to(torch.float32).contiguous() if scaled else None

    @property
    def graph_safe(self) -> bool:
        return getattr(self.mixer, "graph_safe", True) and getattr(self.feed_forward, "graph_safe", True)

    @property
    def first_norm(self):
        return self.norm1

    def forward(self, resid, delta, ctx):
        if delta is not None:
            kernels.residual_add(resid, delta)
        before = getattr(ctx, "handed", None)
        if not isinstance(before, PendingSums):
            before = PendingSums(None, None, None, None)
        eps = self.norm1.eps
        rows1, rows2 = kernels.parallel_step(
            resid, a=before.a, ls1=before.ls1, b=before.b, ls2=before.ls2, more=getattr(ctx, "stream_addend", None),
            gain1=self.norm1.gain32, gain2=self.norm2.gain32 if self.norm2 is not None else None, eps=eps,
            out_dtype=self.dtype)
        ctx.stream_addend = None
        mixed = self.mixer.forward(rows1, ctx)
        out = None
        if self.feed_forward is not None:
            ffn = self.feed_forward
            out = ffn.forward(rows2, batch=ctx.batch) if getattr(ffn, "takes_batch", False) else ffn.forward(rows2)
            if out.dtype != torch.float32:
                out = out.float()
        after = getattr(ctx, "norm_after", None)
        if ctx.trace is None and after is not None and getattr(after, "takes_pending_sums", False):
            ctx.handed_out = PendingSums(mixed, self.ls1, out, self.ls2)
        else:
            kernels.parallel_step(resid, a=mixed, ls1=self.ls1, b=out, ls2=self.ls2)
        return None


register_block("parallel", ParallelBlock)
