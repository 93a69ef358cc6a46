"""The typed configuration of the Dimalix design, read from the keys of its own config.json.

A Dimalix model is a list of parallel layers: with a = norm1(x) and b = norm2(x) of the same x,
x <- x + ls1 * mixer(a) + ls2 * ff(b), where ls1 and ls2 are gains a column.  The embedding is scaled.
Two kinds of mixer: ``attention`` is grouped-query attention whose values are the keys as projected
(there is no value projection), with biases on q and k, one norm over all heads of q and one over all
heads of k, a rotation of the first values of every head in neighbouring pairs whose frequencies may be
rescaled by wavelength, and a mask of chunks (a query sees the keys of its own chunk of positions);
``latent_attention`` keeps one small normed vector and one rotated key part a token and rebuilds every
head's keys and values from them, under a sliding window.  A feed-forward is dense (the tanh gelu) or a
set of experts behind a router: softmax scores, a correction that counts for the choice alone, groups of
neighbouring experts of which the best may be chosen from, identity experts behind the real ones.
``loop`` runs a stretch of the layers several times in a row with the same weights, every run with
pages of its own, every pass but the first starting from the stream plus the embedding output.  Inside
a mixer or a feed-forward a key this reader does not know is refused: a model that ignores a constant
runs and is wrong.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..errors import ConfigError, UnsupportedError
from .papivik import _count, _number, _object
from .specs import (DenseMlpSpec, LatentAttentionSpec, LayerSpec, ModelSpec, NormSpec, RoutedExpertsSpec, ScheduleEntry,
                    TiedAttentionSpec)


def _mask(m, what: str):
    if m.get("mask") is None:
        return None
    _object(m["mask"], what + ".mask", ("size",))
    return _count(m["mask"], "size", what + ".mask")


def _rotation(rot, what: str, most: int):
    """(dims, base, scaling or None) of a mixer's ``rot``."""
    _object(rot, what, ("dims", "base"), ("scaling",))
    dims, base = _count(rot, "dims", what), _number(rot, "base", what)
    if dims % 2 or dims > most or not base > 0:
        raise ConfigError(f"{what}: a rotation over {dims} of {most} values with base {base}")
    scaling = None
    if rot.get("scaling") is not None:
        s = _object(rot["scaling"], what + ".scaling", ("factor", "low", "high", "original"))
        scaling = tuple(_number(s, key, what + ".scaling") for key in ("factor", "low", "high", "original"))
        factor, low, high, original = scaling
        if not (factor > 0 and high > low >= 0 and original > 0):
            raise ConfigError(f"{what}.scaling: factor {factor}, low {low}, high {high}, original {original}")
    return dims, base, scaling


def _attention(m, what: str, eps: float):
    _object(m, what, ("heads", "dim", "scale", "rot"), ("kv_heads", "vdim", "mask"))
    heads, dim = _count(m, "heads", what), _count(m, "dim", what)
    kv_heads = _count(m, "kv_heads", what) if m.get("kv_heads") is not None else heads
    if heads % kv_heads:
        raise ConfigError(f"{what}: {heads} heads over {kv_heads} kv_heads")
    if m.get("vdim") is not None and _count(m, "vdim", what) != dim:
        raise ConfigError(f"{what}: values of {m['vdim']} where the values are the keys, of {dim}")
    dims, base, scaling = _rotation(m["rot"], what + ".rot", dim)
    return TiedAttentionSpec(num_heads=heads, num_kv_heads=kv_heads, head_dim=dim, scale=_number(m, "scale", what),
                             qk_bias=True, qk_norm_eps=eps, rotary_dims=dims, rotary_base=base, rotary_scaling=scaling,
                             window=_mask(m, what), mask="block")


def _latent(m, what: str, eps: float):
    _object(m, what, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "rot", "scale"), ("mask",))
    rot_dim = _count(m, "rot_dim", what)
    dims, base, scaling = _rotation(m["rot"], what + ".rot", rot_dim)
    return LatentAttentionSpec(num_heads=_count(m, "heads", what), head_dim=_count(m, "dim", what), rotary_dim=rot_dim,
                               value_dim=_count(m, "vdim", what), kv_rank=_count(m, "kv_rank", what), rotary_turned=dims,
                               rotary_base=base, rotary_scaling=scaling, max_positions=0, scale=_number(m, "scale", what),
                               norm_eps=eps, sink=None, gated=False, window=_mask(m, what))


_MIXERS = {"attention": _attention, "latent_attention": _latent}


def _feed_forward(mlp, what: str):
    if mlp is None:
        return None
    if not isinstance(mlp, dict) or "kind" not in mlp:
        raise ConfigError(f"{what} is no object with a kind")
    if mlp["kind"] == "dense":
        _object(mlp, what, ("kind", "ff"))
        return DenseMlpSpec(intermediate_size=_count(mlp, "ff", what), activation="gelu_tanh")
    if mlp["kind"] == "moe":
        _object(mlp, what, ("kind", "expert", "router"))
        _object(mlp["expert"], what + ".expert", ("ff",))
        r = _object(mlp["router"], what + ".router", ("experts", "top"), ("identity", "groups"))
        experts, top = _count(r, "experts", what + ".router"), _count(r, "top", what + ".router")
        identity = r.get("identity") or 0
        if isinstance(identity, bool) or not isinstance(identity, int) or identity < 0:
            raise ConfigError(f"{what}.router: identity {identity!r}")
        groups = kept = 1
        if r.get("groups") is not None:
            _object(r["groups"], what + ".router.groups", ("count", "keep"))
            groups, kept = _count(r["groups"], "count", what + ".router.groups"), _count(r["groups"], "keep", what + ".router.groups")
        total = experts + identity
        if total % groups or kept > groups:
            raise ConfigError(f"{what}.router: {total} router outputs in {groups} groups of which {kept} are kept")
        if top > kept * (total // groups):
            raise ConfigError(f"{what}.router: {top} a token of the {kept * (total // groups)} that can be chosen")
        return RoutedExpertsSpec(experts=experts, identity=identity, top=top, intermediate_size=_count(mlp["expert"], "ff", what + ".expert"),
                                 activation="silu", score="softmax", corrected=True, groups=groups, groups_kept=kept)
    raise UnsupportedError(f"{what}: kind {mlp['kind']!r}, this design has dense and moe")


@dataclass(frozen=True)
class DimalixConfig:
    raw: dict
    width: int
    vocab: int
    eps: float
    embedding_scale: float
    loop: tuple | None        # (start, stop, times)
    layers: tuple             # (mixer spec, feed-forward spec or None) a layer

    architecture = "Dimalix"

    @classmethod
    def from_dict(cls, d: dict) -> "DimalixConfig":
        _object(d, "config.json", ("architecture", "layers", "norm", "vocab", "width"), ("embedding", "loop"), others=True)
        _object(d["norm"], "norm", ("eps",))
        eps = _number(d["norm"], "eps", "norm")
        if not eps >= 0:
            raise ConfigError(f"norm: an eps of {eps}")
        scale = 1.0
        if d.get("embedding") is not None:
            _object(d["embedding"], "embedding", ("scale",))
            scale = _number(d["embedding"], "scale", "embedding")
        if not isinstance(d["layers"], list) or not d["layers"]:
            raise ConfigError("layers has to be a list of at least one layer")
        layers = []
        for i, layer in enumerate(d["layers"]):
            what = f"layers[{i}]"
            _object(layer, what, ("type", "mixer"), ("mlp",), others=True)
            if layer["type"] not in _MIXERS:
                raise UnsupportedError(f"{what}: a mixer of type {layer['type']!r}, this design has {', '.join(_MIXERS)}")
            layers.append((_MIXERS[layer["type"]](layer["mixer"], what + ".mixer", eps),
                           _feed_forward(layer.get("mlp"), what + ".mlp")))
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
        return cls(raw=d, width=_count(d, "width", "config.json"), vocab=_count(d, "vocab", "config.json"), eps=eps,
                   embedding_scale=scale, loop=loop, layers=tuple(layers))

    def to_dict(self) -> dict:
        return self.raw

    def schedule(self) -> tuple:
        """The runs of the layers in their order.  A layer of the looped stretch runs ``times`` times; every run after
        the first keeps its pages under a key of its own, past the layers' indices, and the first run of every
        pass but the first stands behind the sum of the stream and the embedding output."""
        count = len(self.layers)
        if self.loop is None:
            return tuple(ScheduleEntry(i) for i in range(count))
        start, stop, times = self.loop
        runs = [ScheduleEntry(i) for i in range(start)]
        for again in range(times):
            for i in range(start, stop):
                runs.append(ScheduleEntry(i, cache_key=None if again == 0 else count + (again - 1) * (stop - start) + (i - start),
                                          add_embedding=again > 0 and i == start))
        runs += [ScheduleEntry(i) for i in range(stop, count)]
        return tuple(runs)

    def model_spec(self) -> ModelSpec:
        norm = NormSpec("rms_norm", self.eps)
        layers = tuple(LayerSpec(block="parallel", mixer=mixer, feed_forward=mlp, norm=norm, weight_prefix=f"l{i}",
                                 layer_scale=True)
                       for i, (mixer, mlp) in enumerate(self.layers))
        extra = {"bare_norm_names": True}
        if self.embedding_scale != 1.0:
            extra.update({"embed_transform": "scale", "embedding_scale": self.embedding_scale})
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, layers=layers, schedule=self.schedule(),
                         final_norm=norm, tie_word_embeddings=False, max_positions=0, embed_name="embed",
                         final_norm_name="final.norm", head_name="head", extra=extra)
