"""The gated feed-forward: down(act(gate(x)) * up(x)), the activation on the
gate branch (reference: model/layers.rs:72-107, where it is SiLU; the spec names it)."""

from __future__ import annotations

import torch

from .. import kernels
from ..errors import UnsupportedError
from ..weights.loader import ParamDecl
from .linear import Linear
from .registry import register_feed_forward


class GatedMlp:
    NAMES = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")

    @classmethod
    def names_of(cls, spec) -> tuple:
        names = getattr(spec, "names", None) or cls.NAMES
        if len(names) != 3:
            raise UnsupportedError(f"a gated feed-forward has three tensors (gate, up, down), the spec names {len(names)}")
        return tuple(names)

    @classmethod
    def declare(cls, spec, hidden: int) -> list:
        i = spec.intermediate_size
        gate, up, down = cls.names_of(spec)
        return [ParamDecl(gate, (i, hidden)), ParamDecl(up, (i, hidden)), ParamDecl(down, (hidden, i))]

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        if spec.activation not in kernels.ACTIVATIONS:
            raise UnsupportedError(f"activation {spec.activation!r}, the kernels know {', '.join(sorted(kernels.ACTIVATIONS))}")
        self.activation = spec.activation
        gate, up, down = self.names_of(spec)
        # one product for gate and up: the output row is [gate | up]
        self.gate_up_proj = Linear.fused([params[gate], params[up]])
        self.down_proj = Linear(params[down])

    # forward takes a norm still to run in place of rows, and may add its result into the stream
    fuses = True
    # ... and a recorder of named activations
    records = True
    # ... and room for the norm that follows the stream, which the product that adds into it may fill
    hands_forward = True

    def forward(self, x, residual: torch.Tensor | None = None, trace=None, hand=None, out_dtype=None):
        """``x``: normalised rows, or a PendingNorm.  With ``residual`` (the 32-bit stream) the
        result is added there where the product kernel can do it, and None comes back; ``hand``
        (``kernels.HandedNorm``) is then filled where that kernel can leave the next norm's work behind."""
        if trace is not None:
            both = self.gate_up_proj.forward(x)
            inter = both.shape[1] // 2
            trace.record("gate_proj.out", both[:, :inter])
            trace.record("up_proj.out", both[:, inter:])
            act = kernels.swiglu(both, activation=self.activation)
            trace.record("down_proj.in", act)
            out = self.down_proj.forward(act)
            trace.record("down_proj.out", out)
            return out
        return self.finish(self.begin(x), residual=residual, hand=hand, out_dtype=out_dtype)

    def begin(self, x):
        """The first half, act(gate x) * (up x): all that reads the feed-forward's input.  A layer whose mixer
        adds into the stream that ``x`` is a norm of may run this half before the mixer and ``finish`` behind it."""
        # (few rows: the activation is the product's epilogue)
        return self.gate_up_proj.forward(x, swiglu=True, activation=self.activation)

    def finish(self, act, residual: torch.Tensor | None = None, hand=None, out_dtype=None):
        """The second half, down(act), added into ``residual`` where the product kernel can (None comes back)."""
        # (``out_dtype``: the type of what comes back where the product could not add it into the stream itself)
        return self.down_proj.forward(act, out_dtype=out_dtype, add_into=residual,
                                      hand=hand if residual is not None else None)


register_feed_forward("gated_mlp", GatedMlp)


class DenseMlp:
    """down(act(up(x))): two products with an activation between them.  The result comes back in 32-bit
    (the sums of the second product, unrounded) for a layer that normalises it before it joins the stream."""

    @staticmethod
    def declare(spec, hidden: int) -> list:
        return [ParamDecl("up", (spec.intermediate_size, hidden)), ParamDecl("down", (hidden, spec.intermediate_size))]

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        if spec.activation not in kernels.ACTIVATIONS:
            raise UnsupportedError(f"activation {spec.activation!r}, the kernels know {', '.join(sorted(kernels.ACTIVATIONS))}")
        self.activation = spec.activation
        self.up_proj = Linear(params["up"])
        self.down_proj = Linear(params["down"])

    def forward(self, x):
        return self.down_proj.forward(kernels.activation(self.up_proj.forward(x), self.activation),
                                      out_dtype=torch.float32)


register_feed_forward("dense_mlp", DenseMlp)


class TableExperts:
    """Small gated feed-forwards of which a token uses the few that a table names for its id, each with the
    same weight: the mean over the chosen e of down_e(act(gate_e x) * (up_e x)).  Nothing is learned about the
    choice and nothing depends on the other rows of the step.  The result comes back in 32-bit.
    Tensors: ``e<i>.gate``, ``e<i>.up`` [ff, width], ``e<i>.down`` [width, ff]; ``table`` [vocabulary, top], integers."""

    # forward needs the step's token ids
    takes_batch = True
    graph_safe = True

    @staticmethod
    def declare(spec, hidden: int) -> list:
        decls = []
        for e in range(spec.experts):
            decls += [ParamDecl(f"e{e}.gate", (spec.intermediate_size, hidden)),
                      ParamDecl(f"e{e}.up", (spec.intermediate_size, hidden)),
                      ParamDecl(f"e{e}.down", (hidden, spec.intermediate_size))]
        decls.append(ParamDecl("table", (spec.vocab_size, spec.top), f"choice_table:{spec.experts}"))
        return decls

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        if spec.activation not in kernels.ACTIVATIONS:
            raise UnsupportedError(f"activation {spec.activation!r}, the kernels know {', '.join(sorted(kernels.ACTIVATIONS))}")
        if not 1 <= spec.top <= spec.experts:
            raise UnsupportedError(f"{spec.top} of {spec.experts} experts a token")
        self.spec, self.activation = spec, spec.activation
        E = spec.experts
        # [E, 2 F, W]: an expert's gate rows, then its up rows; [E, W, F]
        self.w_gate_up = torch.stack([torch.cat([params[f"e{e}.gate"], params[f"e{e}.up"]], 0) for e in range(E)]).contiguous()
        self.w_down = torch.stack([params[f"e{e}.down"] for e in range(E)]).contiguous()
        table = params["table"]
        if table.dtype != torch.int32:
            raise UnsupportedError(f"a table of experts of type {table.dtype}")
        low, high = int(table.min()), int(table.max())
        if low < 0 or high >= E:
            raise UnsupportedError(f"the table of experts names experts {low} to {high} of {E}")
        self.table = table.contiguous()

    def forward(self, x, batch):
        if kernels.moe_grouped_applies(x, x.shape[1], self.spec.intermediate_size):
            return kernels.moe_grouped(x, batch, self.table, self.w_gate_up, self.w_down, self.activation)
        return kernels.moe_rows(x, batch, self.table, self.w_gate_up, self.w_down, self.activation)


register_feed_forward("table_experts", TableExperts)


class RoutedExperts:
    """Small gated feed-forwards behind a router, with identity experts behind the real ones: a token's output is the
    sum over its chosen e of weight_e * expert_e(x), where an identity expert's output is x itself.  The router's
    logits are one product with 32-bit sums out; scores, the correction for the choice, the groups, the choice and
    the weights are one kernel in 32-bit (``kernels.router_select``); the chosen pairs then run as the experts by table
    do: dealt to their experts and multiplied as grouped products on the matrix cores, or a pair at a time.  Nothing
    depends on the other rows of the step.  The result comes back in 32-bit.
    Tensors: ``e<i>.gate``, ``e<i>.up`` [ff, width], ``e<i>.down`` [width, ff]; ``router`` [experts + identity, width];
    ``correction`` [experts + identity]."""

    # forward needs the step (padding rows choose nothing)
    takes_batch = True
    graph_safe = True

    @staticmethod
    def declare(spec, hidden: int) -> list:
        decls = []
        for e in range(spec.experts):
            decls += [ParamDecl(f"e{e}.gate", (spec.intermediate_size, hidden)),
                      ParamDecl(f"e{e}.up", (spec.intermediate_size, hidden)),
                      ParamDecl(f"e{e}.down", (hidden, spec.intermediate_size))]
        total = spec.experts + spec.identity
        decls.append(ParamDecl("router", (total, hidden), "router"))
        if spec.corrected:
            decls.append(ParamDecl("correction", (total,), "bias"))
        return decls

    def __init__(self, spec, hidden: int, params: dict, dtype, device, shared: dict):
        if spec.activation not in kernels.ACTIVATIONS:
            raise UnsupportedError(f"activation {spec.activation!r}, the kernels know {', '.join(sorted(kernels.ACTIVATIONS))}")
        if spec.score != "softmax":
            raise UnsupportedError(f"router scores of kind {spec.score!r} (softmax)")
        E, total = spec.experts, spec.experts + spec.identity
        if E < 1 or spec.identity < 0 or not 1 <= spec.top <= total:
            raise UnsupportedError(f"{spec.top} of {E} + {spec.identity} experts a token")
        if spec.groups < 1 or total % spec.groups or not 1 <= spec.groups_kept <= spec.groups \
                or spec.top > spec.groups_kept * (total // spec.groups):
            raise UnsupportedError(f"{total} router outputs in {spec.groups} groups of which {spec.groups_kept} are kept, "
                                   f"{spec.top} chosen")
        self.spec, self.activation = spec, spec.activation
        # [E, 2 F, W]: an expert's gate rows, then its up rows; [E, W, F]
        self.w_gate_up = torch.stack([torch.cat([params[f"e{e}.gate"], params[f"e{e}.up"]], 0) for e in range(E)]).contiguous()
        self.w_down = torch.stack([params[f"e{e}.down"] for e in range(E)]).contiguous()
        self.router = Linear(params["router"])
        self.correction = params["correction"].to(torch.float32).contiguous() if spec.corrected else None

    def forward(self, x, batch):
        spec = self.spec
        if kernels.router_fuses(x.shape[0], self.router.out_features, x.shape[1]):
            # (few rows: the kernel that chooses works the logits out itself)
            choice, weight = kernels.router_select(None, self.correction, batch.positions, spec.top, spec.groups, spec.groups_kept,
                                                   spec.normalised, spec.weight_eps, x=x, w=self.router.weight)
        else:
            logits = self.router.forward(x, out_dtype=torch.float32)
            choice, weight = kernels.router_select(logits, self.correction, batch.positions, spec.top, spec.groups,
                                                   spec.groups_kept, spec.normalised, spec.weight_eps)
        run = kernels.moe_grouped if kernels.moe_grouped_applies(x, x.shape[1], spec.intermediate_size) else kernels.moe_rows
        return run(x, batch, None, self.w_gate_up, self.w_down, self.activation, choice=choice, weight=weight,
                   identity=spec.identity)


register_feed_forward("routed_experts", RoutedExperts)
