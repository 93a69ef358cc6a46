"""Transforms of the stream behind the embedding and of the logits that ship with the package."""

from __future__ import annotations

import torch

from .. import kernels
from ..errors import ConfigError
from ..weights.loader import ParamDecl
from .registry import NORMS, lookup, register_embed_transform, register_final_transform, register_logit_transform


class EmbeddingScale:
    """x <- x * extra["embedding_scale"], on the 32-bit stream."""

    graph_safe = True

    def __init__(self, spec, params: dict, dtype, device):
        self.scale = float(spec.extra["embedding_scale"])

    def __call__(self, x, batch):
        return kernels.scale_(x, self.scale) if self.scale != 1.0 else x


register_embed_transform("scale", EmbeddingScale)


class LearnedPosition:
    """x[t] <- x[t] + table[position of t]: a learned vector a position, added to the 32-bit stream unscaled.
    The table's checkpoint name is ``extra["position_table_name"]``; it has ``max_positions`` rows."""

    graph_safe = True

    @staticmethod
    def declare(spec) -> list:
        return [ParamDecl(spec.extra["position_table_name"], (spec.max_positions, spec.hidden_size), "embedding")]

    def __init__(self, spec, params: dict, dtype, device):
        self.table = params[spec.extra["position_table_name"]]

    def __call__(self, x, batch):
        return kernels.add_position_rows_(x, self.table, batch.positions)


class StreamNorm:
    """x <- norm(x) on the stream right behind the embedding; the norm is ``extra["stream_norm"]`` (a NormSpec),
    its gain the tensor ``extra["stream_norm_name"]``."""

    graph_safe = True

    @staticmethod
    def declare(spec) -> list:
        norm = lookup(NORMS, spec.extra["stream_norm"].kind, "norm")
        decls = norm.declare(spec.extra["stream_norm"], spec.hidden_size)
        if len(decls) != 1:
            raise ConfigError(f"a norm of {len(decls)} tensors cannot be stored under one name")
        return [ParamDecl(spec.extra["stream_norm_name"], decls[0].shape, decls[0].role)]

    def __init__(self, spec, params: dict, dtype, device):
        norm = lookup(NORMS, spec.extra["stream_norm"].kind, "norm")
        local = norm.declare(spec.extra["stream_norm"], spec.hidden_size)[0].name
        self.norm = norm(spec.extra["stream_norm"], spec.hidden_size, {local: params[spec.extra["stream_norm_name"]]},
                         dtype, device)

    def __call__(self, x, batch):
        # (the normalised rows in 32-bit are the stream from here on)
        return self.norm.apply(x, None, torch.float32)


class LogitScale:
    """logits <- logits * extra["logit_scale"]."""

    graph_safe = True

    def __init__(self, spec, params: dict, dtype, device):
        self.scale = float(spec.extra["logit_scale"])

    def __call__(self, logits, batch):
        return kernels.scale_(logits, self.scale) if self.scale != 1.0 and logits.numel() else logits


register_embed_transform("learned_position", LearnedPosition)
register_embed_transform("stream_norm", StreamNorm)
register_logit_transform("scale", LogitScale)


class StreamCopies:
    """The stream behind the embedding ``extra["stream_copies"]`` times, [rows, copies * width]: what layers over
    several copies of the stream start from."""

    graph_safe = True

    def __init__(self, spec, params: dict, dtype, device):
        self.copies = int(spec.extra["stream_copies"])

    def __call__(self, x, batch):
        return kernels.stream_copies(x, self.copies)


class StreamCopiesSum:
    """Before the final norm: the sum of the copies of the stream, for the rows whose logits are wanted."""

    graph_safe = True

    def __init__(self, spec, params: dict, dtype, device):
        self.copies = int(spec.extra["stream_copies"])
        self.ones = torch.ones((self.copies,), dtype=torch.float32, device=device)

    def __call__(self, x, batch):
        return kernels.hc_step(x, self.copies, read=self.ones, rows=batch.logit_rows)


class LogitSoftcap:
    """logits <- cap * tanh(logits / cap), cap = extra["logit_softcap"]."""

    graph_safe = True

    def __init__(self, spec, params: dict, dtype, device):
        self.cap = float(spec.extra["logit_softcap"])
        if not self.cap > 0:
            raise ConfigError(f"a soft cap of {self.cap} on the logits")

    def __call__(self, logits, batch):
        return kernels.softcap_(logits, self.cap) if logits.numel() else logits


register_embed_transform("stream_copies", StreamCopies)
register_final_transform("stream_copies_sum", StreamCopiesSum)
register_logit_transform("softcap", LogitSoftcap)
