"""The Mukenex design without a GPU: its configuration reader and what it refuses, the tensors it declares, the
random-weights mode, the schedule and cache layout of a stretch of layers that runs several times, and properties of
the plain implementation's mechanisms."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import mukenex_util as mu
import plain_mukenex as plain
from paged_llm_rs_amd.config import load_config
from paged_llm_rs_amd.config.specs import (DenseMlpSpec, LatentAttentionSpec, LinearAttentionSpec, ScheduleEntry,
                                           SinkAttentionSpec, TableExpertsSpec)
from paged_llm_rs_amd.errors import ConfigError, UnsupportedError
from paged_llm_rs_amd.parts.model import declare_parameters


def test_the_reader_takes_every_size_and_constant_from_the_config():
    spec = load_config(copy.deepcopy(mu.ODD)).model_spec()
    assert spec.hidden_size == 72 and spec.vocab_size == 211 and spec.max_positions == 0
    state, latent, blocks = (layer.mixer for layer in spec.layers[:3])
    assert isinstance(state, LinearAttentionSpec) and isinstance(latent, LatentAttentionSpec) and isinstance(blocks, SinkAttentionSpec)
    assert (state.num_heads, state.head_dim, state.value_dim, state.decay, state.eps) == (3, 24, 40, (0.6, 0.9, 0.999), 1e-5)
    assert (latent.num_heads, latent.head_dim, latent.rotary_dim, latent.value_dim, latent.kv_rank) == (3, 24, 8, 40, 40)
    assert latent.scale == 0.21 and latent.rotary_base == 500.0 and latent.rotary_turned == 8 and latent.norm_eps == 1e-5
    assert latent.sink == "learned" and latent.gated and latent.gate_each == "element" and latent.window == 37
    assert latent.max_positions == 0, "nothing bounds the positions: no tables of angles"
    assert (blocks.num_heads, blocks.num_kv_heads, blocks.head_dim, blocks.value_dim) == (6, 2, 24, 40)
    assert blocks.window == 5 and blocks.mask == "block" and blocks.sink is None and blocks.distance_slopes is None
    assert blocks.qk_gain and blocks.qkv_bias and blocks.qk_unit_eps == 1e-5 and blocks.scale == 0.3
    dense, experts = spec.layers[0].feed_forward, spec.layers[1].feed_forward
    assert isinstance(dense, DenseMlpSpec) and dense.intermediate_size == 100 and dense.activation == "gelu"
    assert isinstance(experts, TableExpertsSpec) and (experts.experts, experts.top, experts.intermediate_size) == (5, 2, 24)
    assert experts.vocab_size == 211 and experts.activation == "silu" and spec.layers[3].feed_forward is None
    assert all(layer.norm.gain_offset == 1.0 and layer.stream_copies == 4 for layer in spec.layers)
    assert spec.extra["logit_softcap"] == 20.0 and spec.extra["stream_copies"] == 4
    # the stretch 1..3 runs three times; every run after the first has a cache key of its own
    assert [e.layer for e in spec.schedule] == [0, 1, 2, 3, 1, 2, 3, 1, 2, 3, 4, 5]
    keys = [e.layer if e.cache_key is None else e.cache_key for e in spec.schedule]
    assert len(set(keys)) == 12 and keys[:4] == [0, 1, 2, 3] and keys[-2:] == [4, 5]
    plain_one = load_config(copy.deepcopy(mu.PLAIN)).model_spec()
    assert "embed_transform" not in plain_one.extra and "logit_transform" not in plain_one.extra
    assert all(layer.stream_copies is None for layer in plain_one.layers)
    assert plain_one.layers[0].mixer.window is None and plain_one.layers[1].mixer.window is None
    assert [e.layer for e in plain_one.schedule] == [0, 1, 2, 3, 4]
    ones = load_config(copy.deepcopy(mu.ONES)).model_spec()
    assert ones.layers[0].stream_copies == 1 and [e.layer for e in ones.schedule] == [0, 1, 2, 3, 4]
    assert ones.layers[3].mixer.rotary_turned == 8 and ones.layers[3].mixer.rotary_dim == 16


@pytest.mark.parametrize("damage, error", [
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), ConfigError),
    (lambda c: c["layers"][1]["mixer"].update(extra=1), UnsupportedError),
    (lambda c: c["layers"][2]["mixer"].update(kv_heads=4), ConfigError),
    (lambda c: c["layers"][2]["mixer"]["mask"].update(size=0), ConfigError),
    (lambda c: c["layers"][0]["mixer"].update(decay=[0.5]), ConfigError),
    (lambda c: c["layers"][0].update(type="other"), UnsupportedError),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), UnsupportedError),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), ConfigError),        # more than there are
    (lambda c: c["layers"][1]["mlp"]["router"].update(kind="learned"), UnsupportedError),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), ConfigError),       # more than the rotated part
    (lambda c: c["loop"].update(stop=7), ConfigError),
    (lambda c: c["loop"].update(start=5), ConfigError),
    (lambda c: c["loop"].update(times=0), ConfigError),
    (lambda c: c.update(streams=0), ConfigError),
    (lambda c: c.update(logit_softcap=-1.0), ConfigError),
    (lambda c: c["norm"].update(eps=-1.0), ConfigError),
])
def test_what_the_reader_refuses(damage, error):
    config = copy.deepcopy(mu.ODD)
    damage(config)
    with pytest.raises(error):
        load_config(config)


def test_declared_tensors():
    found = declare_parameters(load_config(copy.deepcopy(mu.ODD)).model_spec())
    decls = {d.name: tuple(d.shape) for d in found}
    assert decls["embed"] == (211, 72) and decls["final.norm"] == (72,) and decls["head"] == (211, 72)
    assert decls["l0.mix.q"] == (72, 72) and decls["l0.mix.v"] == (120, 72) and decls["l0.mix.g"] == (120, 72)
    assert decls["l0.mix.norm"] == (120,) and decls["l0.mix.o"] == (72, 120)
    assert decls["l0.mlp.up"] == (100, 72) and decls["l0.mlp.down"] == (72, 100) and "l0.mlp.gate" not in decls
    assert decls["l1.mix.q"] == (3 * 32, 72) and decls["l1.mix.dkv"] == (48, 72) and decls["l1.mix.dkv.norm"] == (40,)
    assert decls["l1.mix.uk"] == (72, 40) and decls["l1.mix.uv"] == (120, 40) and decls["l1.mix.sink"] == (3,)
    assert decls["l1.mix.g"] == (120, 72), "a gate an element of the read-out"
    assert decls["l1.mlp.e4.gate"] == (24, 72) and decls["l1.mlp.e4.down"] == (72, 24) and "l1.mlp.e5.up" not in decls
    assert decls["l1.mlp.table"] == (211, 2)
    assert decls["l2.mix.q"] == (144, 72) and decls["l2.mix.k.b"] == (48,) and decls["l2.mix.v.b"] == (80,)
    assert decls["l2.mix.q.norm"] == (24,) and decls["l2.mix.k.norm"] == (24,) and decls["l2.mix.o"] == (72, 240)
    assert "l2.mix.sink" not in decls and "l3.norm2" not in decls and "l3.hc2.in" not in decls
    for part in ("hc1", "hc2"):
        assert decls[f"l0.{part}.in"] == (4,) and decls[f"l0.{part}.out"] == (4,) and decls[f"l0.{part}.mix"] == (4, 4)
    without = {d.name for d in declare_parameters(load_config(copy.deepcopy(mu.PLAIN)).model_spec())}
    assert not any(".hc" in name for name in without)


def test_the_random_weights_mode_and_the_plain_implementation(tmp_path):
    folder = mu.write_model(tmp_path / "m", mu.ODD, seed=3)
    config, weights = mu.load_plain(folder)
    table = weights["l1.mlp.table"]
    assert table.dtype == torch.int32 and int(table.min()) >= 0 and int(table.max()) < 5
    assert all(len(set(row)) == 2 for row in table.tolist()), "a row names different experts"
    assert abs(float(weights["l0.norm1"].mean())) < 0.2, "norm gains are stored around zero"
    assert abs(float(weights["l0.hc1.mix"].diagonal().mean()) - 1) < 0.3
    tokens = [5, 17, 3, 200, 0, 44, 9, 9, 120]
    streams = []
    logits = plain.forward(config, weights, tokens, streams)
    assert logits.shape == (9, 211) and len(streams) == 12 and torch.isfinite(logits).all()
    assert float(logits.abs().max()) < 20.0
    # causal: a prefix gives the same logits
    assert torch.allclose(plain.forward(config, weights, tokens[:5]), logits[:5], atol=1e-12)
    # the soft cap bends the logits and nothing else
    other = copy.deepcopy(config)
    other.pop("logit_softcap")
    assert torch.allclose(20.0 * torch.tanh(plain.forward(other, weights, tokens) / 20.0), logits, atol=1e-12)
    # a stretch that runs once is no loop
    once = copy.deepcopy(config)
    once["loop"]["times"] = 1
    other = copy.deepcopy(config)
    other.pop("loop")
    assert torch.equal(plain.forward(once, weights, tokens), plain.forward(other, weights, tokens))
    assert not torch.allclose(plain.forward(once, weights, tokens), logits)


def test_one_copy_with_weights_of_one_is_the_plain_stream(tmp_path):
    config = mu.model(40, 50, [mu.lightning(2, 8, 8, (0.9, 0.5), mlp=mu.dense(24)), mu.attention(2, 1, 16, 8, 0.3, block=4)], streams=1)
    folder = mu.write_model(tmp_path / "m", config, seed=5, std=0.3)
    cfg, weights = mu.load_plain(folder)
    for name in list(weights):
        if ".hc" in name:
            weights[name] = torch.ones_like(weights[name])
    without = copy.deepcopy(cfg)
    without.pop("streams")
    tokens = list(range(10, 30))
    assert torch.allclose(plain.forward(cfg, weights, tokens), plain.forward(without, weights, tokens), atol=1e-12)


def test_the_cache_layout_of_a_layer_that_runs_several_times():
    from paged_llm_rs_amd.cache.layout import CacheLayout, KVCacheSpec, StateSpec

    class Mixer:
        def __init__(self, spec, state=None):
            self.spec, self.state = spec, state

        def cache_spec(self):
            return self.spec

        def state_spec(self):
            return self.state

    class Block:
        def __init__(self, spec, state=None):
            self.mixer = Mixer(spec, state)

    small, heads = KVCacheSpec(1, 48, 9, values_in_keys=True), KVCacheSpec(2, 32, 5)
    blocks = [Block(None, StateSpec((64,))), Block(small), Block(heads)]
    runs = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2), ScheduleEntry(0, cache_key=3), ScheduleEntry(1, cache_key=4),
            ScheduleEntry(2, cache_key=5))
    layout = CacheLayout.from_blocks(blocks, runs)
    assert [g.layers for g in layout.groups] == [[1, 4], [2, 5]] and sorted(layout.states) == [0, 3]
    assert layout.bytes_per_token(2) == 2 * 48 * 2 + 2 * 2 * 2 * 32 * 2
    with pytest.raises(ConfigError):       # two runs that would write the same pages
        CacheLayout.from_blocks(blocks, (ScheduleEntry(1), ScheduleEntry(1)))
    with pytest.raises(ConfigError):       # ... or the same state
        CacheLayout.from_blocks(blocks, (ScheduleEntry(0), ScheduleEntry(0, cache_key=0)))
    # a run may still read what a run with a key of its own wrote
    CacheLayout.from_blocks(blocks, (ScheduleEntry(1), ScheduleEntry(1, cache_key=7), ScheduleEntry(1, cache_from=7)))


def test_properties_of_the_plain_mechanisms():
    g = torch.Generator().manual_seed(0)
    positions = torch.arange(12)
    # a window sees itself and size - 1 before it; a block its own block up to itself
    w = plain.window_mask(positions, 4)
    assert w[7].nonzero().flatten().tolist() == [4, 5, 6, 7] and w[2].nonzero().flatten().tolist() == [0, 1, 2]
    b = plain.block_mask(positions, 5)
    assert b[7].nonzero().flatten().tolist() == [5, 6, 7] and b[5].nonzero().flatten().tolist() == [5]
    assert b[4].nonzero().flatten().tolist() == [0, 1, 2, 3, 4] and b[11].nonzero().flatten().tolist() == [10, 11]
    # blocks are counted from position 0, not from where the positions given start
    assert plain.block_mask(torch.arange(3, 9), 5)[3].nonzero().flatten().tolist() == [2, 3]
    # rotation: lengths of pairs stay, position 0 stays, scores depend on the distance alone
    x = torch.randn(7, 3, 12, generator=g, dtype=torch.float64)
    turned = plain.rotate_neighbours(x, torch.arange(7), 8, 100.0)
    assert torch.allclose(turned[..., 8:], x[..., 8:]) and torch.allclose(turned[0], x[0])
    pairs = lambda t: t[..., 0:8:2] ** 2 + t[..., 1:8:2] ** 2
    assert torch.allclose(pairs(turned), pairs(x))
    a, c = torch.randn(1, 8, generator=g, dtype=torch.float64), torch.randn(1, 8, generator=g, dtype=torch.float64)
    dot = lambda p, q: float((plain.rotate_neighbours(a, torch.tensor([p]), 8, 100.0) * plain.rotate_neighbours(c, torch.tensor([q]), 8, 100.0)).sum())
    assert abs(dot(9, 4) - dot(25, 20)) < 1e-12 and abs(dot(9, 4) - dot(9, 5)) > 1e-6
    # a sink takes its share and has no value; without one the weights sum to one
    score = torch.randn(5, 5, generator=g, dtype=torch.float64)
    visible = torch.tril(torch.ones(5, 5, dtype=torch.bool))
    s = plain.softmax_with_sink(score, visible, 0.3)
    assert (s.sum(-1) < 1).all() and (s[~visible] == 0).all()
    assert torch.allclose(s.sum(-1), 1 - math.exp(0.3) / (math.exp(0.3) + torch.exp(score.masked_fill(~visible, -math.inf)).sum(-1)))
    assert torch.allclose(plain.softmax_with_sink(score, visible).sum(-1), torch.ones(5, dtype=torch.float64))
    # the norm's stored gain is the distance from one
    v = torch.randn(3, 16, generator=g, dtype=torch.float64)
    assert torch.allclose(plain.norm_around_zero(v, torch.zeros(16, dtype=torch.float64), 0.0), plain.rms(v, 0.0))
    assert abs(float(plain.gelu_erf(torch.tensor(1.0, dtype=torch.float64))) - 0.8413447460685429) < 1e-12
    # the copies: with mix the identity, in and out (1, 0) the first copy is the plain stream and the second never moves
    copies = torch.randn(2, 4, 6, generator=g, dtype=torch.float64)
    weights = {"in": torch.tensor([1.0, 0.0], dtype=torch.float64), "out": torch.tensor([1.0, 0.0], dtype=torch.float64),
               "mix": torch.eye(2, dtype=torch.float64)}
    after = plain.sublayer_over_copies(copies, weights, "", lambda u: 2 * u)
    assert torch.allclose(after[0], 3 * copies[0]) and torch.equal(after[1], copies[1])
    # mix is indexed from, to
    weights["mix"] = torch.tensor([[0.0, 1.0], [0.0, 0.0]], dtype=torch.float64)
    after = plain.sublayer_over_copies(copies, weights, "", lambda u: 0 * u)
    assert torch.equal(after[1], copies[0]) and torch.equal(after[0], torch.zeros_like(after[0]))


def test_a_block_of_the_plain_attention_ends_at_multiples_of_its_size(tmp_path):
    """Changing a token changes the logits of the positions in its own block from it on and of no other (one layer)."""
    config = mu.model(40, 50, [mu.attention(2, 1, 16, 16, 0.7, block=4)])
    folder = mu.write_model(tmp_path / "m", config, seed=5, std=0.3)
    cfg, weights = mu.load_plain(folder)
    tokens = list(range(10, 30))
    base = plain.forward(cfg, weights, tokens)
    changed = list(tokens)
    changed[5] = 49
    moved = (plain.forward(cfg, weights, changed) - base).abs().max(-1).values > 1e-9
    assert moved.tolist() == [5 <= p < 8 for p in range(20)]


def test_a_state_layer_of_the_plain_implementation_remembers(tmp_path):
    """With a decay near one the first token moves the last position's logits; with a small one it does not reach it."""
    for decay, reaches in ((0.999, True), (0.05, False)):
        config = mu.model(40, 50, [mu.lightning(2, 8, 8, (decay, decay))])
        folder = mu.write_model(tmp_path / f"m{reaches}", config, seed=5, std=0.3)
        cfg, weights = mu.load_plain(folder)
        tokens = list(range(10, 40))
        base = plain.forward(cfg, weights, tokens)
        changed = [49] + tokens[1:]
        moved = float((plain.forward(cfg, weights, changed) - base)[-1].abs().max())
        assert (moved > 1e-4) == reaches, (decay, moved)
