"""The Dimalix design without a GPU: its configuration reader and what it refuses, the tensors it declares, the
random-weights mode, the schedule and cache layout of a stretch of layers that runs several times, and properties of
the plain implementation's mechanisms."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import dimalix_util as du
import plain_dimalix as plain
from paged_llm_rs_amd.config import load_config
from paged_llm_rs_amd.config.specs import DenseMlpSpec, LatentAttentionSpec, RoutedExpertsSpec, TiedAttentionSpec
from paged_llm_rs_amd.errors import ConfigError, UnsupportedError
from paged_llm_rs_amd.parts.model import declare_parameters


def test_the_reader_takes_every_size_and_constant_from_the_config():
    spec = load_config(copy.deepcopy(du.ODD)).model_spec()
    assert spec.hidden_size == 72 and spec.vocab_size == 211 and spec.max_positions == 0
    assert spec.extra["embed_transform"] == "scale" and spec.extra["embedding_scale"] == 3.0
    latent, tied = spec.layers[0].mixer, spec.layers[1].mixer
    assert isinstance(latent, LatentAttentionSpec) and isinstance(tied, TiedAttentionSpec)
    assert (latent.num_heads, latent.head_dim, latent.rotary_dim, latent.value_dim, latent.kv_rank) == (3, 24, 8, 40, 40)
    assert latent.scale == 0.21 and latent.rotary_base == 500.0 and latent.rotary_turned == 8 and latent.norm_eps == 1e-5
    assert latent.sink is None and not latent.gated and latent.window == 37 and latent.rotary_scaling is None
    assert latent.max_positions == 0, "nothing bounds the positions: no tables of angles"
    assert (tied.num_heads, tied.num_kv_heads, tied.head_dim, tied.scale) == (6, 2, 24, 0.3)
    assert tied.qk_bias and tied.qk_norm_eps == 1e-5 and tied.window == 5 and tied.mask == "block"
    assert (tied.rotary_dims, tied.rotary_base, tied.rotary_scaling) == (10, 100.0, (4.0, 1.0, 3.0, 64.0))
    assert spec.layers[3].mixer.rotary_scaling is None and spec.layers[3].mixer.rotary_dims == 40
    experts, dense = spec.layers[0].feed_forward, spec.layers[2].feed_forward
    assert isinstance(experts, RoutedExpertsSpec) and isinstance(dense, DenseMlpSpec)
    assert (experts.experts, experts.identity, experts.top, experts.intermediate_size) == (7, 2, 2, 24)
    assert (experts.groups, experts.groups_kept, experts.corrected, experts.score) == (3, 2, True, "softmax")
    assert experts.normalised and experts.weight_eps == 1e-20 and experts.activation == "silu"
    assert dense.intermediate_size == 96 and dense.activation == "gelu_tanh" and spec.layers[3].feed_forward is None
    assert all(layer.block == "parallel" and layer.layer_scale for layer in spec.layers)
    # the stretch 0..2 runs three times; every run after the first has a cache key of its own, and every pass
    # but the first starts behind the sum with the embedding output
    assert [e.layer for e in spec.schedule] == [0, 1, 2, 0, 1, 2, 0, 1, 2, 3, 4]
    assert [e.add_embedding for e in spec.schedule] == [False, False, False, True, False, False, True, False, False, False, False]
    keys = [e.layer if e.cache_key is None else e.cache_key for e in spec.schedule]
    assert len(set(keys)) == 11 and keys[:3] == [0, 1, 2] and keys[-2:] == [3, 4]
    plain_one = load_config(copy.deepcopy(du.PLAIN)).model_spec()
    assert "embed_transform" not in plain_one.extra and [e.layer for e in plain_one.schedule] == [0, 1, 2, 3, 4]
    assert plain_one.layers[0].mixer.window is None and plain_one.layers[1].mixer.window is None
    first = plain_one.layers[0].feed_forward
    assert (first.identity, first.groups, first.groups_kept) == (0, 1, 1)
    ones = load_config(copy.deepcopy(du.ONES)).model_spec()
    assert [(e.layer, e.add_embedding) for e in ones.schedule] == [(0, False), (1, False), (2, False), (3, False)]
    without = copy.deepcopy(du.ONES)
    without["layers"][0]["mixer"].pop("kv_heads")
    assert load_config(without).model_spec().layers[0].mixer.num_kv_heads == 4


@pytest.mark.parametrize("damage, error", [
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), ConfigError),
    (lambda c: c["layers"][0]["mixer"].update(extra=1), UnsupportedError),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), ConfigError),
    (lambda c: c["layers"][1]["mixer"].update(vdim=16), ConfigError),            # the values are the keys
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), ConfigError),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=26), ConfigError),      # more than a head
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), ConfigError),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("low"), ConfigError),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].update(high=1.0), ConfigError),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), ConfigError),      # more than the rotated part
    (lambda c: c["layers"][0].update(type="lightning"), UnsupportedError),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), UnsupportedError),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=7), ConfigError),       # more than the kept groups hold
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), ConfigError),   # 9 outputs in 4 groups
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=4), ConfigError),
    (lambda c: c["layers"][0]["mlp"]["router"].update(identity=-1), ConfigError),
    (lambda c: c["layers"][0]["mlp"]["router"].update(kind="learned"), UnsupportedError),
    (lambda c: c["loop"].update(stop=7), ConfigError),
    (lambda c: c["loop"].update(start=4), ConfigError),
    (lambda c: c["loop"].update(times=0), ConfigError),
    (lambda c: c["embedding"].update(scale="big"), ConfigError),
    (lambda c: c["norm"].update(eps=-1.0), ConfigError),
])
def test_what_the_reader_refuses(damage, error):
    config = copy.deepcopy(du.ODD)
    damage(config)
    with pytest.raises(error):
        load_config(config)


def test_declared_tensors():
    found = declare_parameters(load_config(copy.deepcopy(du.ODD)).model_spec())
    decls = {d.name: tuple(d.shape) for d in found}
    optional = {d.name for d in found if d.optional}
    assert decls["embed"] == (211, 72) and decls["final.norm"] == (72,) and decls["head"] == (211, 72)
    assert decls["l0.mix.q"] == (3 * 32, 72) and decls["l0.mix.dkv"] == (48, 72) and decls["l0.mix.dkv.norm"] == (40,)
    assert decls["l0.mix.uk"] == (72, 40) and decls["l0.mix.uv"] == (120, 40) and decls["l0.mix.o"] == (72, 120)
    assert "l0.mix.sink" not in decls and "l0.mix.g" not in decls
    assert decls["l0.mlp.e6.gate"] == (24, 72) and decls["l0.mlp.e6.down"] == (72, 24) and "l0.mlp.e7.up" not in decls
    assert decls["l0.mlp.router"] == (9, 72) and decls["l0.mlp.correction"] == (9,), "identity experts have router rows and nothing else"
    assert decls["l1.mix.q"] == (144, 72) and decls["l1.mix.k"] == (48, 72) and "l1.mix.v" not in decls
    assert decls["l1.mix.q.b"] == (144,) and decls["l1.mix.k.b"] == (48,)
    assert decls["l1.mix.q.norm"] == (144,) and decls["l1.mix.k.norm"] == (48,), "one norm over all heads"
    assert decls["l1.mix.o"] == (72, 144)
    assert decls["l2.mlp.up"] == (96, 72) and decls["l2.mlp.down"] == (72, 96) and "l2.mlp.gate" not in decls
    for i in range(5):
        assert decls[f"l{i}.norm1"] == decls[f"l{i}.norm2"] == decls[f"l{i}.ls1"] == decls[f"l{i}.ls2"] == (72,)
    # a layer without a feed-forward needs neither its second norm nor its second gain
    assert {"l3.norm2", "l3.ls2"} <= optional and "l2.norm2" not in optional and not any(n.startswith("l3.mlp") for n in decls)


def test_the_random_weights_mode_and_the_plain_implementation(tmp_path):
    folder = du.write_model(tmp_path / "m", du.ODD, seed=3)
    config, weights = du.load_plain(folder)
    tokens = [5, 17, 3, 200, 0, 44, 9, 9, 120]
    streams = []
    logits = plain.forward(config, weights, tokens, streams)
    assert logits.shape == (9, 211) and len(streams) == 11 and torch.isfinite(logits).all()
    # causal: a prefix gives the same logits
    assert torch.allclose(plain.forward(config, weights, tokens[:5]), logits[:5], atol=1e-12)
    # a stretch that runs once is no loop, and the embedding output is then never added again
    once = copy.deepcopy(config)
    once["loop"]["times"] = 1
    other = copy.deepcopy(config)
    other.pop("loop")
    assert torch.equal(plain.forward(once, weights, tokens), plain.forward(other, weights, tokens))
    assert not torch.allclose(plain.forward(once, weights, tokens), logits)
    # the embedding output joins the stream once a further pass, right before the pass's first layer
    assert plain.layer_runs(config) == [(0, False), (1, False), (2, False), (0, True), (1, False), (2, False),
                                        (0, True), (1, False), (2, False), (3, False), (4, False)]
    unscaled = copy.deepcopy(config)
    unscaled["embedding"]["scale"] = 1.0
    assert not torch.allclose(plain.forward(unscaled, weights, tokens), logits)


def test_the_cache_layout_of_the_design():
    from paged_llm_rs_amd.cache.layout import CacheLayout, KVCacheSpec

    class Mixer:
        def __init__(self, spec):
            self.spec = spec

        def cache_spec(self):
            return self.spec

        def state_spec(self):
            return None

    class Block:
        def __init__(self, spec):
            self.mixer = Mixer(spec)

    spec = load_config(copy.deepcopy(du.ODD)).model_spec()
    small, heads = KVCacheSpec(1, 48, 37, values_in_keys=True), KVCacheSpec(2, 32, 5)
    other = KVCacheSpec(1, 48, 9, values_in_keys=True)
    blocks = [Block(small), Block(heads), Block(other), Block(KVCacheSpec(3, 48, 37)), Block(KVCacheSpec(1, 16, 64))]
    layout = CacheLayout.from_blocks(blocks, spec.schedule)
    # every run of a looped layer has pools of its own in its layer's group
    assert sorted(len(g.layers) for g in layout.groups) == [1, 1, 3, 3, 3] and not layout.states


def test_properties_of_the_plain_mechanisms():
    g = torch.Generator().manual_seed(0)
    positions = torch.arange(12)
    # a window sees itself and size - 1 before it; a chunk its own chunk up to itself
    w = plain.window_mask(positions, 4)
    assert w[7].nonzero().flatten().tolist() == [4, 5, 6, 7] and w[2].nonzero().flatten().tolist() == [0, 1, 2]
    b = plain.chunk_mask(positions, 5)
    assert b[7].nonzero().flatten().tolist() == [5, 6, 7] and b[5].nonzero().flatten().tolist() == [5]
    assert b[4].nonzero().flatten().tolist() == [0, 1, 2, 3, 4] and b[11].nonzero().flatten().tolist() == [10, 11]
    # chunks are counted from position 0, not from where the positions given start
    assert plain.chunk_mask(torch.arange(3, 9), 5)[3].nonzero().flatten().tolist() == [2, 3]
    # rotation: lengths of pairs stay, position 0 stays, values behind the turned ones stay, scores depend on the distance
    rot = {"dims": 8, "base": 100.0}
    x = torch.randn(7, 3, 12, generator=g, dtype=torch.float64)
    turned = plain.rotate_neighbours(x, torch.arange(7), rot)
    assert torch.allclose(turned[..., 8:], x[..., 8:]) and torch.allclose(turned[0], x[0])
    pairs = lambda t: t[..., 0:8:2] ** 2 + t[..., 1:8:2] ** 2
    assert torch.allclose(pairs(turned), pairs(x))
    a, c = torch.randn(1, 8, generator=g, dtype=torch.float64), torch.randn(1, 8, generator=g, dtype=torch.float64)
    dot = lambda p, q: float((plain.rotate_neighbours(a, torch.tensor([p]), rot) * plain.rotate_neighbours(c, torch.tensor([q]), rot)).sum())
    assert abs(dot(9, 4) - dot(25, 20)) < 1e-12 and abs(dot(9, 4) - dot(9, 5)) > 1e-6
    # the pair (u, v) at position 1 with frequency 1 turns by one radian, u towards v
    one = plain.rotate_neighbours(torch.tensor([[1.0, 0.0]], dtype=torch.float64), torch.tensor([1]), {"dims": 2, "base": 7.0})
    assert torch.allclose(one, torch.tensor([[math.cos(1.0), math.sin(1.0)]], dtype=torch.float64))
    # rescaled frequencies: short waves stay, long ones are divided by the factor, those between lie between
    plainf = plain.frequencies({"dims": 16, "base": 10000.0})
    scaled = plain.frequencies({"dims": 16, "base": 10000.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 256}})
    kinds = set()
    for f, s in zip(plainf, scaled):
        length = 2 * math.pi / f
        if length < 256 / 4.0:
            kinds.add("kept")
            assert s == f
        elif length > 256 / 1.0:
            kinds.add("stretched")
            assert abs(s - f / 8.0) < 1e-15
        else:
            kinds.add("between")
            assert f / 8.0 < s < f
    assert kinds == {"kept", "stretched", "between"}
    assert abs(float(plain.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12


def test_properties_of_the_plain_router():
    g = torch.Generator().manual_seed(1)
    h = torch.randn(40, 12, generator=g, dtype=torch.float64)
    w = {"router": torch.randn(8, 12, generator=g, dtype=torch.float64), "correction": torch.zeros(8, dtype=torch.float64)}
    router = {"experts": 6, "identity": 2, "top": 3}
    chosen, weight = plain.route(h, w, "", router)
    score = torch.softmax(h @ w["router"].T, -1)
    assert torch.equal(chosen, score.topk(3, -1).indices) and torch.allclose(weight.sum(-1), torch.ones(40, dtype=torch.float64))
    assert torch.allclose(weight, score.gather(1, chosen) / score.gather(1, chosen).sum(-1, keepdim=True))
    # the correction moves the choice and not the weights
    w["correction"] = torch.tensor([0, 0, 0, 0, 0, 0, 0, 5.0], dtype=torch.float64)
    chosen2, weight2 = plain.route(h, w, "", router)
    assert (chosen2[:, 0] == 7).all() and torch.allclose(weight2[:, 0], score[:, 7] / score.gather(1, chosen2).sum(-1))
    # groups: with one of four groups kept, all chosen lie in the group that holds the best choice score, also where
    # a better expert than the group's second lies elsewhere
    w["correction"] = torch.tensor([-0.5, 0.3, 0, 0, 0.2, -3.0, 0, 0], dtype=torch.float64)     # (negative choice scores too)
    grouped = dict(router, top=2, groups={"count": 4, "keep": 1})
    chosen3, _ = plain.route(h, w, "", grouped)
    best = (score + w["correction"]).argmax(-1)
    assert ((chosen3 // 2) == (best // 2)[:, None]).all()
    free, _ = plain.route(h, w, "", dict(router, top=2))
    assert not torch.equal(free, chosen3)
    # an identity expert hands its input through with its weight
    mlp = {"kind": "moe", "expert": {"ff": 5}, "router": {"experts": 1, "identity": 1, "top": 2}}
    w2 = {"router": torch.randn(2, 12, generator=g, dtype=torch.float64), "correction": torch.zeros(2, dtype=torch.float64),
          "e0.gate": torch.zeros(5, 12, dtype=torch.float64), "e0.up": torch.zeros(5, 12, dtype=torch.float64),
          "e0.down": torch.zeros(12, 5, dtype=torch.float64)}
    out = plain.routed_experts(h, w2, "", mlp)
    assert torch.allclose(out, h * torch.softmax(h @ w2["router"].T, -1)[:, 1:2])


def test_a_chunk_of_the_plain_attention_ends_at_multiples_of_its_size(tmp_path):
    """Changing a token changes the logits of the positions in its own chunk from it on and of no other (one layer
    without a feed-forward)."""
    config = du.model(40, 50, [du.attention(2, 1, 16, 0.7, chunk=4)])
    folder = du.write_model(tmp_path / "m", config, seed=5, std=0.3)
    cfg, weights = du.load_plain(folder)
    tokens = list(range(10, 30))
    base = plain.forward(cfg, weights, tokens)
    changed = list(tokens)
    changed[5] = 49
    moved = (plain.forward(cfg, weights, changed) - base).abs().max(-1).values > 1e-9
    assert moved.tolist() == [5 <= p < 8 for p in range(20)]


def test_the_values_of_the_plain_attention_are_its_keys_as_projected(tmp_path):
    """With one key to see (a chunk of one position) a head's read-out is the key as projected, bias and all, whatever
    the norm's gains and the rotation do."""
    config = du.model(24, 30, [du.attention(3, 1, 8, 0.7, chunk=1, base=10.0)])
    folder = du.write_model(tmp_path / "m", config, seed=6, std=0.3)
    cfg, w = du.load_plain(folder)
    tokens = torch.tensor([3, 9, 27, 1])
    x = w["embed"][tokens]
    h = plain.rms(x, 1e-6) * w["l0.norm1"]
    key = h @ w["l0.mix.k"].T + w["l0.mix.k.b"]
    want = key.repeat(1, 3) @ w["l0.mix.o"].T
    got = plain.attention_mixer(h, w, "l0.mix.", cfg["layers"][0]["mixer"], 1e-6, torch.arange(4))
    assert torch.allclose(got, want, atol=1e-12)
    w["l0.mix.k.norm"] = w["l0.mix.k.norm"] * 3
    assert torch.allclose(plain.attention_mixer(h, w, "l0.mix.", cfg["layers"][0]["mixer"], 1e-6, torch.arange(4)), want, atol=1e-12)
