"""The typed configuration of the Mukenex design, read from the keys of its own config.json.

A Mukenex model is a list of layers in the pre-norm arrangement, x <- x + mixer(norm1(x)) and then
x <- x + ff(norm2(x)), with norm gains stored around zero.  With ``streams`` the model keeps that many
copies of the stream instead of one: a sublayer reads a weighted sum of the copies and its output
rebuilds every copy from all of them.  Three kinds of mixer: ``latent_attention`` keeps one small
vector and one rotated key part a token and rebuilds every head's keys and values from them, under a
window, with a learned sink a head and a gate an element; ``attention`` is grouped-query attention
with biases, a norm with a gain on q and k, no positions, and a mask of blocks (a query sees the keys
of its own block of positions); ``lightning`` is linear attention with a fixed decay a head.  A
feed-forward is dense (the erf gelu) or a set of experts of which a table over token ids names a
token's few.  ``loop`` runs a stretch of the layers several times in a row with the same weights,
every run with pages and state of its own.  The logits may pass a soft cap.  Inside a mixer or a
feed-forward a key this reader does not know is refused: a model that ignores a constant runs and is wrong.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..errors import ConfigError, UnsupportedError
from .papivik import _count, _number, _object
from .specs import (DenseMlpSpec, LatentAttentionSpec, LayerSpec, LinearAttentionSpec, ModelSpec, NormSpec,
                    ScheduleEntry, SinkAttentionSpec, TableExpertsSpec)


def _mask(m, what: str):
    if m.get("mask") is None:
        return None
    _object(m["mask"], what + ".mask", ("size",))
    return _count(m["mask"], "size", what + ".mask")


def _latent(m, what: str, eps: float):
    _object(m, what, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "rot", "scale"), ("mask",))
    _object(m["rot"], what + ".rot", ("dims", "base"))
    rot_dim = _count(m, "rot_dim", what)
    turned, base = _count(m["rot"], "dims", what + ".rot"), _number(m["rot"], "base", what + ".rot")
    if turned % 2 or turned > rot_dim or not base > 0:
        raise ConfigError(f"{what}: a rotation over {turned} of {rot_dim} values with base {base}")
    return LatentAttentionSpec(num_heads=_count(m, "heads", what), head_dim=_count(m, "dim", what), rotary_dim=rot_dim,
                               value_dim=_count(m, "vdim", what), kv_rank=_count(m, "kv_rank", what),
                               rotary_turned=turned, rotary_base=base, max_positions=0,
                               scale=_number(m, "scale", what), norm_eps=eps, sink="learned", gated=True,
                               gate_each="element", window=_mask(m, what))


def _attention(m, what: str, eps: float):
    _object(m, what, ("heads", "kv_heads", "dim", "vdim", "scale"), ("mask",))
    heads, kv_heads = _count(m, "heads", what), _count(m, "kv_heads", what)
    if heads % kv_heads:
        raise ConfigError(f"{what}: {heads} heads over {kv_heads} kv_heads")
    return SinkAttentionSpec(num_heads=heads, num_kv_heads=kv_heads, head_dim=_count(m, "dim", what),
                             value_dim=_count(m, "vdim", what), scale=_number(m, "scale", what), qk_unit_eps=eps,
                             qk_gain=True, qkv_bias=True, window=_mask(m, what), mask="block", sink=None)


def _lightning(m, what: str, eps: float):
    _object(m, what, ("heads", "dim", "vdim", "decay"))
    heads = _count(m, "heads", what)
    decay = m["decay"]
    if not isinstance(decay, list) or len(decay) != heads:
        raise ConfigError(f"{what}: decay has to list one number a head ({heads})")
    return LinearAttentionSpec(num_heads=heads, head_dim=_count(m, "dim", what), value_dim=_count(m, "vdim", what),
                               decay=tuple(_number({"decay": x}, "decay", what) for x in decay), eps=eps)


_MIXERS = {"latent_attention": _latent, "attention": _attention, "lightning": _lightning}


def _feed_forward(mlp, what: str, vocab: int):
    if mlp is None:
        return None
    if not isinstance(mlp, dict) or "kind" not in mlp:
        raise ConfigError(f"{what} is no object with a kind")
    if mlp["kind"] == "dense":
        _object(mlp, what, ("kind", "ff"))
        return DenseMlpSpec(intermediate_size=_count(mlp, "ff", what), activation="gelu")
    if mlp["kind"] == "moe":
        _object(mlp, what, ("kind", "expert", "router"))
        _object(mlp["expert"], what + ".expert", ("ff",))
        _object(mlp["router"], what + ".router", ("experts", "top"))
        experts, top = _count(mlp["router"], "experts", what + ".router"), _count(mlp["router"], "top", what + ".router")
        if top > experts:
            raise ConfigError(f"{what}.router: {top} of {experts} experts a token")
        return TableExpertsSpec(experts=experts, top=top, intermediate_size=_count(mlp["expert"], "ff", what + ".expert"),
                                vocab_size=vocab, activation="silu")
    raise UnsupportedError(f"{what}: kind {mlp['kind']!r}, this design has dense and moe")


@dataclass(frozen=True)
class MukenexConfig:
    raw: dict
    width: int
    vocab: int
    eps: float
    streams: int | None       # copies of the stream; None: the one plain stream
    softcap: float | None
    loop: tuple | None        # (start, stop, times)
    layers: tuple             # (mixer spec, feed-forward spec or None) a layer

    architecture = "Mukenex"

    @classmethod
    def from_dict(cls, d: dict) -> "MukenexConfig":
        _object(d, "config.json", ("architecture", "layers", "norm", "vocab", "width"),
                ("streams", "loop", "logit_softcap"), others=True)
        _object(d["norm"], "norm", ("eps",))
        eps = _number(d["norm"], "eps", "norm")
        if not eps >= 0:
            raise ConfigError(f"norm: an eps of {eps}")
        vocab = _count(d, "vocab", "config.json")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("layers has to be a list of at least one layer")
        layers = []
        for i, layer in enumerate(d["layers"]):
            what = f"layers[{i}]"
            _object(layer, what, ("type", "mixer"), ("mlp",), others=True)
            if layer["type"] not in _MIXERS:
                raise UnsupportedError(f"{what}: a mixer of type {layer['type']!r}, this design has {', '.join(_MIXERS)}")
            layers.append((_MIXERS[layer["type"]](layer["mixer"], what + ".mixer", eps),
                           _feed_forward(layer.get("mlp"), what + ".mlp", vocab)))
        streams = _count(d, "streams", "config.json") if d.get("streams") is not None else None
        softcap = None
        if d.get("logit_softcap") is not None:
            softcap = _number(d, "logit_softcap", "config.json")
            if not softcap > 0:
                raise ConfigError(f"a logit_softcap of {softcap}")
        loop = None
        if d.get("loop") is not None:
            _object(d["loop"], "loop", ("start", "stop", "times"))
            start, stop, times = d["loop"]["start"], d["loop"]["stop"], _count(d["loop"], "times", "loop")
            for name, v in (("start", start), ("stop", stop)):
                if isinstance(v, bool) or not isinstance(v, int):
                    raise ConfigError(f"loop: {name} {v!r}, which has to be an integer")
            if not 0 <= start <= stop <= len(layers):
                raise ConfigError(f"loop: layers {start} to {stop} of {len(layers)}")
            loop = (start, stop, times)
        return cls(raw=d, width=_count(d, "width", "config.json"), vocab=vocab, eps=eps, streams=streams,
                   softcap=softcap, loop=loop, layers=tuple(layers))

    def to_dict(self) -> dict:
        return self.raw

    def schedule(self) -> tuple:
        """The runs of the layers in their order.  A layer of the looped stretch runs ``times`` times; every
        run after the first keeps its pages and state under a key of its own, past the layers' indices."""
        count = len(self.layers)
        if self.loop is None:
            return tuple(ScheduleEntry(i) for i in range(count))
        start, stop, times = self.loop
        runs = [ScheduleEntry(i) for i in range(start)]
        for again in range(times):
            for i in range(start, stop):
                runs.append(ScheduleEntry(i, cache_key=None if again == 0 else count + (again - 1) * (stop - start) + (i - start)))
        runs += [ScheduleEntry(i) for i in range(stop, count)]
        return tuple(runs)

    def model_spec(self) -> ModelSpec:
        norm = NormSpec("rms_norm", self.eps, gain_offset=1.0)
        layers = tuple(LayerSpec(block="hyper_connections", mixer=mixer, feed_forward=mlp, norm=norm,
                                 weight_prefix=f"l{i}", stream_copies=self.streams)
                       for i, (mixer, mlp) in enumerate(self.layers))
        extra = {"bare_norm_names": True}
        if self.streams is not None:
            extra.update({"embed_transform": "stream_copies", "final_transform": "stream_copies_sum",
                          "stream_copies": self.streams})
        if self.softcap is not None:
            extra.update({"logit_transform": "softcap", "logit_softcap": self.softcap})
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, layers=layers, schedule=self.schedule(),
                         final_norm=norm, tie_word_embeddings=False, max_positions=0, embed_name="embed",
                         final_norm_name="final.norm", head_name="head", extra=extra)
