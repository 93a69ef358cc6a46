"""The Dimalix design in the engine against the plain implementation: the new kernels alone (the pass that adds a
layer's outputs and norms the next layer's rows, the router's choice, the kernel between the projections of an attention
layer whose values are its keys and the attention kernels, routed experts with identity experts), every mixer and
feed-forward alone, whole prompts, tokens decoded one by one, portions down to two tokens, mixed batches with pages used
again, keys far away under a sharp softmax, keys just inside and just outside a window and a chunk (in prompts and while
decoding, at page borders), gains, corrections and biases that carry weight, the first tokens of a request, long
decoding, other sizes, and greedy generation through the engine's own entry point and the command line."""

from __future__ import annotations

import copy
import json
import math
import random
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import dimalix_util as du
import replay_util as ru

pytestmark = pytest.mark.gpu

# Against the plain implementation (64-bit): 32-bit runs are held tightly.  In bfloat16 a run gets a loose bound there
# and a tight one against the engine's own whole-prompt run of the same requests (the same roundings; what differs
# between schedules is the cache and the batch: a lost key shows there in full).  All bounds are for a position that
# amplifies rounding as the median position does, and grow with a position's own amplification.  A position at which a
# router decides by less than MARGIN of choice score is left out: the choice may fall the other way under rounding.
TOLERANCE = {"float32": 5e-5, "bfloat16": 0.1}
MARGIN = {"float32": 1e-5, "bfloat16": 8e-3}
BETWEEN_SCHEDULES = 4e-2
DTYPES = ["float32", "bfloat16"]


def replayer(folder, dtype, prompts, live=4, block_size=16, graphs=True):
    from paged_llm_rs_amd.engine.replay import Replayer

    return Replayer(folder, dtype, max_tokens=ru.pool_tokens(prompts, live), block_size=block_size, max_live=live,
                    graphs=graphs)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    made = {}

    def get(name, dtype):
        if (name, dtype) not in made:
            made[name, dtype] = du.write_model(tmp_path_factory.mktemp(f"dimalix_{name}_{dtype}"), du.CONFIGS[name],
                                               seed=sorted(du.CONFIGS).index(name) + 1, dtype=dtype)
        return made[name, dtype]
    return get


_whole: dict = {}
_factor: dict = {}
_plain: dict = {}
_close: dict = {}


def check(folder, dtype, prompts, steps, live=4, block_size=16, tolerance=None, between=BETWEEN_SCHEDULES, most_close=0.35):
    r = replayer(folder, dtype, prompts, live, block_size)
    got = ru.collect(r, steps)
    key = (str(folder), repr(sorted(prompts.items())))
    if key not in _plain:
        _plain[key] = du.plain_logits(folder, prompts)
        _factor[key] = du.sensitivity(folder, prompts)
    if (key, dtype) not in _close:
        _close[key, dtype] = du.close_calls(folder, prompts, MARGIN[dtype])
    want, factor, close = _plain[key], _factor[key], _close[key, dtype]
    compared = {k: row for k, row in got.items() if not bool(close[k[0]][k[1]])}
    assert len(compared) >= (1 - most_close) * len(got), f"{len(got) - len(compared)} of {len(got)} positions are close calls of a router"
    scale = max(float(want[n][p].abs().max()) for (n, p) in got)
    bound = tolerance or TOLERANCE[dtype]
    for (n, p), row in compared.items():
        ref = want[n][p].numpy()
        assert row.shape == ref.shape
        err = float(np.abs(row.astype(np.float64) - ref).max()) / scale
        assert err <= bound * float(factor[n][p]), f"{err:.3e} at {(n, p)}, where the bound is {bound * float(factor[n][p]):.3e}"
    assert r.cache.manager.live_sequences == 0, "every request's pages came back"
    if dtype == "bfloat16":
        if key not in _whole:
            _whole[key] = ru.collect(replayer(folder, dtype, prompts, live), ru.whole(prompts))
        spread = float(np.mean([want[n][p].std() for (n, p) in got]))
        over = {}
        for (n, p), row in compared.items():
            gap = float(np.sqrt(np.mean((row - _whole[key][(n, p)]) ** 2))) / spread
            if gap > between * float(factor[n][p]):
                over[n, p] = gap / (between * float(factor[n][p]))
        assert len(over) <= max(1, len(got) // 50) and all(x <= 3.0 for x in over.values()), \
            f"between this schedule and the whole prompt, over the bound by {sorted(over.items(), key=lambda x: -x[1])[:5]} of {len(got)}"
    return r, got


# --- the new kernels alone --------------------------------------------------------------------------------------------

@pytest.mark.parametrize("width", [52, 75, 200, 1024, 4096, 5000])
def test_the_pass_that_adds_a_layers_outputs_and_norms_the_next_layers_rows(width):
    """Sums and norms together and each alone, with and without gains a column, rows to add as they are, the norms of
    chosen rows, both types of normed rows, against 64-bit arithmetic."""
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(width)
    n = 37
    x, a, b, more = (torch.randn((n, width), generator=g, dtype=torch.float64) * s for s in (3, 1, 2, 1.5))
    ls1, ls2, gain1, gain2 = (1 + 0.4 * torch.randn((width,), generator=g, dtype=torch.float64) for _ in range(4))
    eps = 1e-5
    dev = lambda t: t.to(torch.float32).cuda().contiguous()
    norm = lambda u, gain: u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * gain
    summed = x + ls1 * a + ls2 * b + more
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 8e-3)):
        stream = dev(x)
        rows1, rows2 = kernels.parallel_step(stream, a=dev(a), ls1=dev(ls1), b=dev(b), ls2=dev(ls2), more=dev(more),
                                             gain1=dev(gain1), gain2=dev(gain2), eps=eps, out_dtype=dtype)
        assert (stream.double().cpu() - summed).abs().max() <= 2e-6 * summed.abs().max()
        for rows, gain in ((rows1, gain1), (rows2, gain2)):
            want = norm(summed, gain)
            assert rows.dtype == dtype and (rows.double().cpu() - want).abs().max() <= tol * want.abs().max()
    stream = dev(x)
    rows1, rows2 = kernels.parallel_step(stream, gain1=dev(gain1), eps=eps)
    assert rows2 is None and torch.equal(stream, dev(x)), "norms alone change nothing"
    assert (rows1.double().cpu() - norm(x, gain1)).abs().max() <= 2e-6 * norm(x, gain1).abs().max()
    assert kernels.parallel_step(stream, a=dev(a), b=dev(b), ls2=dev(ls2)) == (None, None)
    want = x + a + ls2 * b
    assert (stream.double().cpu() - want).abs().max() <= 2e-6 * want.abs().max()
    kernels.parallel_step(stream, more=dev(more))
    assert (stream.double().cpu() - (want + more)).abs().max() <= 2e-6 * want.abs().max()
    chosen = torch.tensor([5, 0, 36, 5], dtype=torch.int32).cuda()
    rows1, _ = kernels.parallel_step(stream, gain1=dev(gain2), eps=eps, rows=chosen)
    picked = norm(want + more, gain2)[chosen.cpu().long()]
    assert (rows1.double().cpu() - picked).abs().max() <= 2e-6 * picked.abs().max()


def _route64(z, correction, top, groups, kept):
    score = torch.softmax(z, -1)
    choice = score + (correction if correction is not None else 0)
    if groups > 1:
        size = z.shape[1] // groups
        best = choice.view(-1, groups, size).max(-1).values
        keep = best.topk(kept, -1).indices
        allowed = torch.zeros_like(best, dtype=torch.bool).scatter_(1, keep, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(size, 1), -math.inf)
    chosen = choice.topk(top, -1).indices
    weight = score.gather(1, chosen)
    return chosen, weight / (weight.sum(-1, keepdim=True) + 1e-20)


@pytest.mark.parametrize("total,top,groups,kept", [(12, 2, 3, 1), (9, 2, 3, 2), (1, 1, 1, 1), (4, 4, 4, 4), (64, 6, 8, 3), (256, 8, 8, 4),
                                                   (300, 5, 1, 1), (6, 3, 2, 1), (5, 3, 1, 1), (128, 1, 128, 1)])
def test_a_routers_choice(total, top, groups, kept):
    """Chosen experts, their order and weights against 64-bit arithmetic over the same 32-bit logits, with a correction
    that moves the choice (negative choice scores among them), without one, and for rows of padding."""
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(total * 31 + top)
    n = 200
    z = (torch.randn((n, total), generator=g) * 2.5).float()
    correction = (torch.randn((total,), generator=g) * 0.3).float()
    positions = torch.arange(n, dtype=torch.int32)
    positions[17] = -1
    for corr in (correction, None):
        chosen, weight = kernels.router_select(z.cuda(), corr.cuda() if corr is not None else None, positions.cuda(), top, groups, kept)
        want_c, want_w = _route64(z.double(), corr.double() if corr is not None else None, top, groups, kept)
        chosen, weight = chosen.cpu(), weight.cpu()
        assert (chosen[17] == -1).all() and (weight[17] == 0).all(), "a row of padding chooses nothing"
        rows = [t for t in range(n) if t != 17]
        assert torch.equal(chosen[rows].long(), want_c[rows]), "the same experts in the same order"
        assert (weight[rows].double() - want_w[rows]).abs().max() <= 1e-6
    # without normalising, the weights are the scores themselves
    chosen, weight = kernels.router_select(z.cuda(), None, None, top, groups, kept, normalised=False)
    score = torch.softmax(z.double(), -1)
    assert (weight.cpu().double() - score.gather(1, chosen.cpu().long())).abs().max() <= 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("total,top,groups,kept,width", [(12, 3, 3, 1, 320), (9, 3, 3, 2, 72), (64, 6, 8, 3, 1024), (4, 2, 1, 1, 100)])
def test_a_router_that_works_its_logits_out_itself(dtype, total, top, groups, kept, width):
    """The kernel that chooses, given rows and the router's matrix instead of logits, against the same kernel over logits
    from 64-bit arithmetic: the same experts and weights but for close calls."""
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(total + width)
    n = 120
    assert kernels.router_fuses(n, total, width)
    x = torch.randn((n, width), generator=g).to(dtype)
    w = (torch.randn((total, width), generator=g) * 2.5 * width ** -0.5).to(dtype)
    correction = (torch.randn((total,), generator=g) * 0.2).float()
    positions = torch.arange(n, dtype=torch.int32)
    positions[40] = -1
    z = (x.double() @ w.double().T).float()
    want_c, want_w = kernels.router_select(z.cuda(), correction.cuda(), positions.cuda(), top, groups, kept)
    got_c, got_w = kernels.router_select(None, correction.cuda(), positions.cuda(), top, groups, kept, x=x.cuda(), w=w.cuda())
    same = (got_c == want_c).all(-1).cpu()
    assert int(same.sum()) >= n - 2 and bool(same[40]) and (got_c[40] == -1).all()
    assert (got_w - want_w)[same.cuda()].abs().max() <= 2e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,rot,page", [(6, 2, 24, 10, 16), (4, 1, 16, 16, 4), (16, 1, 128, 128, 16), (3, 3, 40, 0, 8), (8, 2, 64, 32, 16),
                                            (2, 2, 22, 22, 16), (1, 1, 30, 2, 16), (64, 32, 128, 64, 16)])
def test_between_the_projections_and_the_attention_kernels_where_the_values_are_the_keys(dtype, H, G, D, rot, page):
    """Queries out, keys and values into scattered pages, against 64-bit arithmetic: the biases first, one statistic
    over all heads of q and one over all heads of k, a gain a column, the first values of every head turned in pairs,
    heads in padded rows with zeros behind them, the values the keys as they were before norm and rotation; rows of
    padding write nothing.  (The last case's rows take more of a workgroup's LDS than a launch gets unasked.)"""
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.cache.pools import LayerKV

    g = torch.Generator().manual_seed(H * 100 + D)
    n, eps = 23, 1e-5
    off, behind = (4, 8) if D % 8 == 0 else (3, 5)       # (rows that the kernel reads four values at a time, and rows it cannot)
    padded = D if dtype == torch.float32 else (D + 15) // 16 * 16
    rows = torch.randn((n, off + (H + G) * D + behind), generator=g, dtype=torch.float64)
    bias = torch.randn(((H + G) * D,), generator=g, dtype=torch.float64)
    q_gain = 1 + 0.3 * torch.randn((H * D,), generator=g, dtype=torch.float64)
    k_gain = 1 + 0.3 * torch.randn((G * D,), generator=g, dtype=torch.float64)
    freq = torch.tensor([50.0 ** (-2.0 * i / max(rot, 2)) for i in range(rot // 2)], dtype=torch.float64)
    positions = torch.randperm(40, generator=g)[:n]
    pages = -(-40 // page)
    order = torch.randperm(pages + 2, generator=g)[:pages]

    class Step:
        pass

    b = Step()
    pos = positions.clone()
    pos[5] = -1
    b.positions = pos.to(torch.int32).cuda()
    b.seq_of = torch.zeros(n, dtype=torch.int32).cuda()
    k_pool = torch.full(((pages + 2) * page, G * padded), 7.0, dtype=dtype).cuda()
    v_pool = torch.full(((pages + 2) * page, G * padded), 7.0, dtype=dtype).cuda()
    kv = LayerKV(k_pool, v_pool, order.to(torch.int32).view(1, pages).cuda(), page, 0)
    q_out = torch.full((n, H * padded), 7.0, dtype=dtype).cuda()
    f32 = lambda t: t.to(torch.float32).cuda().contiguous()
    kernels.wide_prepare(f32(rows), off, b, kv, q_out, H, G, D, padded, norm_eps=eps, q_gain=f32(q_gain), k_gain=f32(k_gain),
                         freq=f32(freq) if rot else None, rot=rot, bias=f32(bias))
    both = rows[:, off:off + (H + G) * D].float().double() + bias.float().double()
    q_raw, k_raw = both[:, :H * D], both[:, H * D:]
    unit = lambda t: t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps)

    def turn(t, heads):
        t = t.view(n, heads, D).clone()
        if rot:
            angle = positions.double()[:, None] * freq.float().double()[None, :]
            cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
            u, v = t[..., 0:rot:2].clone(), t[..., 1:rot:2].clone()
            t[..., 0:rot:2], t[..., 1:rot:2] = u * cos - v * sin, v * cos + u * sin
        return t

    q_want = turn(unit(q_raw) * q_gain.float().double(), H)
    k_want = turn(unit(k_raw) * k_gain.float().double(), G)
    tol = 3e-6 if dtype == torch.float32 else 8e-3
    q_got = q_out.double().cpu().view(n, H, padded)
    live = [t for t in range(n) if t != 5]
    assert (q_got[live][..., :D] - q_want[live]).abs().max() <= tol * q_want.abs().max()
    assert (q_got[live][..., D:] == 0).all() and (q_got[5] == 7.0).all()
    k_got, v_got = k_pool.double().cpu(), v_pool.double().cpu()
    written = set()
    for t in live:
        p = int(positions[t])
        row = int(order[p // page]) * page + p % page
        written.add(row)
        assert (k_got[row].view(G, padded)[:, :D] - k_want[t]).abs().max() <= tol * k_want.abs().max()
        assert (v_got[row].view(G, padded)[:, :D] - k_raw[t].view(G, D)).abs().max() <= tol * k_raw.abs().max()
        assert (k_got[row].view(G, padded)[:, D:] == 0).all() and (v_got[row].view(G, padded)[:, D:] == 0).all()
    others = [r for r in range(k_got.shape[0]) if r not in written]
    assert (k_got[others] == 7.0).all() and (v_got[others] == 7.0).all(), "no other row of the pages is touched"


class _Rows:
    """What the experts' kernels read of a step."""

    def __init__(self, n, positions=None):
        self.token_ids = torch.zeros(n, dtype=torch.int32).cuda()
        self.positions = torch.tensor(positions if positions is not None else list(range(n)), dtype=torch.int32).cuda()
        self.fed_tokens = None
        self.token_src = None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,identity,top,ff,width,rows", [(8, 2, 3, 64, 160, 50), (3, 0, 3, 44, 52, 7), (1, 3, 2, 24, 100, 9),
                                                               (16, 4, 4, 128, 256, 300), (4, 1, 1, 256, 512, 129), (6, 2, 8, 64, 96, 33)])
def test_experts_behind_a_router(dtype, experts, identity, top, ff, width, rows):
    """Every row against 64-bit arithmetic over its own chosen experts with their weights; an identity expert hands the
    row through; a pair without an expert adds nothing; rows of padding give zeros.  In bfloat16, where the sizes
    allow, the grouped products on the matrix cores against the kernel that takes a pair at a time."""
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(experts * 100 + rows)
    w_gu = (torch.randn((experts, 2 * ff, width), generator=g) * width ** -0.5).to(dtype)
    w_down = (torch.randn((experts, width, ff), generator=g) * ff ** -0.5).to(dtype)
    x = torch.randn((rows, width), generator=g).to(dtype)
    choice = torch.rand((rows, experts + identity), generator=g).argsort(1)[:, :top].to(torch.int32)
    choice[3, 0] = -1
    weight = torch.rand((rows, top), generator=g).float()
    positions = list(range(rows))
    positions[rows // 2] = -1
    batch = _Rows(rows, positions)
    got = kernels.moe_rows(x.cuda(), batch, None, w_gu.cuda(), w_down.cuda(), "silu", choice=choice.cuda(), weight=weight.cuda(),
                           identity=identity).double().cpu()
    want = torch.zeros((rows, width), dtype=torch.float64)
    for t in range(rows):
        for c, e in enumerate(choice[t].tolist()):
            if e < 0:
                continue
            if e >= experts:
                want[t] += x[t].double() * weight[t, c].double()
                continue
            both = w_gu[e].double() @ x[t].double()
            hidden = torch.nn.functional.silu(both[:ff]) * both[ff:]
            if dtype == torch.bfloat16:
                hidden = hidden.to(torch.bfloat16).double()      # (what lies between the two products is stored in the rows' type)
            want[t] += (w_down[e].double() @ hidden) * weight[t, c].double()
    want[rows // 2] = 0
    assert (got - want).abs().max() <= (1e-5 if dtype == torch.float32 else 2e-2) * want.abs().max()
    if dtype == torch.bfloat16 and kernels.moe_grouped_applies(x.cuda(), width, ff):
        for _ in range(2):
            dealt = kernels.moe_grouped(x.cuda(), batch, None, w_gu.cuda(), w_down.cuda(), "silu", choice=choice.cuda(),
                                        weight=weight.cuda(), identity=identity).double().cpu()
            assert (dealt - got).abs().max() <= 1e-2 * got.abs().max()
            assert float(dealt[rows // 2].abs().max()) == 0.0


# --- every mixer and feed-forward alone, in 32-bit, the stream behind the layer against the plain implementation's ----

ALONE = {
    "latent, a window": [du.latent(3, 24, 8, 40, 56, 0.3, base=300.0, window=11)],
    "latent, no window": [du.latent(2, 16, 12, 16, 20, 0.4, base=40.0)],
    "latent, rescaled frequencies": [du.latent(2, 16, 12, 16, 20, 0.4, base=40.0, window=30, scaling=(5.0, 1.0, 2.0, 30))],
    "attention, chunks of 7, part of a head turns, rescaled frequencies": [du.attention(6, 3, 24, 0.4, chunk=7, turned=14, base=60.0,
                                                                                         scaling=(4.0, 1.0, 3.0, 40))],
    "attention, no mask": [du.attention(2, 1, 40, 0.2, base=500.0)],
    "dense feed-forward": [du.attention(1, 1, 16, 0.5, mlp=du.dense(136))],
    "experts": [du.attention(1, 1, 16, 0.5, mlp=du.moe(6, 3, 40))],
    "experts, identity experts and groups": [du.attention(1, 1, 16, 0.5, mlp=du.moe(5, 3, 40, identity=3, groups=(4, 2)))],
    "two layers that run three times": [du.latent(2, 16, 8, 16, 24, 0.3, window=6, mlp=du.dense(40)),
                                        du.attention(2, 2, 16, 0.3, chunk=9, mlp=du.moe(3, 2, 24, identity=1))],
}


@pytest.mark.parametrize("which", sorted(ALONE))
def test_a_layer_alone_against_its_plain_function(tmp_path, which):
    """32-bit, the stream behind every run of a layer against the plain implementation's: whole, and again in portions (the
    later portions read what the earlier ones left in the pages)."""
    layers = ALONE[which]
    config = du.model(88, 61, layers, eps=1e-5, scale=2.5, loop=(0, 2, 3) if len(layers) == 2 else None)
    folder = du.write_model(tmp_path / "m", config, seed=7, std=0.2)
    tokens = [random.Random(3).randrange(61) for _ in range(45)]
    cfg, weights = du.load_plain(folder)
    want = []
    du.plain.forward(cfg, weights, tokens, want)
    names = ["l0.out"] if len(layers) == 1 else ["l0.out", "l1.out", "l0.run1.out", "l1.run1.out", "l0.run2.out", "l1.run2.out"]
    r = replayer(folder, "float32", {"a": tokens}, graphs=False)
    rec = {}
    r.step([{"id": "a", "tokens": tokens, "want": []}], ["a"], trace=rec)
    for name, stream in zip(names, want):
        assert (rec[name].double().cpu() - stream).abs().max() <= 5e-5 * stream.abs().max(), (which, name)
    pieces, at = {name: [] for name in names}, 0
    for n in (1, 2, 17, 3, 22):
        rec = {}
        r.step([{"id": "b", "tokens": tokens[at:at + n], "want": []}], ["b"] if at + n == 45 else [], trace=rec)
        for name in names:
            pieces[name].append(rec[name].double().cpu())
        at += n
    for name, stream in zip(names, want):
        assert (torch.cat(pieces[name]) - stream).abs().max() <= 5e-5 * stream.abs().max(), (which, name, "in portions")


# --- whole models of other sizes under every schedule ------------------------------------------------------------------

LENGTHS = [70, 3, 41, 18, 1, 33, 57]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(du.CONFIGS))
def test_whole_prompts(folders, name, dtype):
    prompts = ru.make_prompts(du.CONFIGS[name]["vocab"], LENGTHS, seed=1)
    check(folders(name, dtype), dtype, prompts, ru.whole(prompts))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(du.CONFIGS))
def test_prefill_then_tokens_one_by_one(folders, name, dtype):
    prompts = ru.make_prompts(du.CONFIGS[name]["vocab"], LENGTHS, seed=1)
    check(folders(name, dtype), dtype, prompts, ru.tail_decoded(prompts, tail=40))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(du.CONFIGS))
@pytest.mark.parametrize("block_size", [16, 8])
def test_portions_down_to_two_tokens(folders, name, dtype, block_size):
    prompts = ru.make_prompts(du.CONFIGS[name]["vocab"], LENGTHS, seed=1)
    check(folders(name, dtype), dtype, prompts, ru.portions(prompts), block_size=block_size)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(du.CONFIGS))
@pytest.mark.parametrize("seed", [0, 1])
def test_unequal_requests_together_with_pages_used_again(folders, name, dtype, seed):
    """Nine requests of unequal length through a pool that holds four: portions of some beside single tokens of others,
    requests left out of steps, pages of finished requests taken by the next."""
    prompts = ru.make_prompts(du.CONFIGS[name]["vocab"], [70, 3, 41, 18, 1, 33, 57, 64, 22], seed=2 + seed)
    check(folders(name, dtype), dtype, prompts, ru.mixed(prompts, seed=seed, max_live=4, tail=14))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(tmp_path, seed, dtype):
    """Ten drawn models (order of layers, looped stretch, sizes, head counts, windows, chunks, rotations, experts, groups,
    identity experts, constants; `dimalix_util.drawn_config`) under a mixed schedule and whole, over pages of 16, 8 and 32."""
    config = du.drawn_config(100 + seed)
    folder = du.write_model(tmp_path / "m", config, seed=seed, dtype=dtype, std=0.1)
    prompts = ru.make_prompts(config["vocab"], [75, 9, 130, 33, 2], seed=seed)
    block_size = (16, 8, 32)[seed % 3]
    check(folder, dtype, prompts, ru.mixed(prompts, seed=seed, max_live=3, tail=20), live=3, block_size=block_size, most_close=0.5)
    check(folder, dtype, prompts, ru.whole(prompts), live=3, block_size=block_size, most_close=0.5)


def test_schedules_agree_with_each_other_in_32_bit(folders):
    folder = folders("odd", "float32")
    prompts = ru.make_prompts(du.ODD["vocab"], LENGTHS, seed=1)
    close = du.close_calls(folder, prompts, 1e-4)
    whole = ru.collect(replayer(folder, "float32", prompts), ru.whole(prompts))
    scale = max(float(np.abs(row).max()) for row in whole.values())
    for steps in (ru.tail_decoded(prompts, tail=40), ru.portions(prompts), ru.mixed(prompts, seed=5)):
        for key, row in ru.collect(replayer(folder, "float32", prompts), steps).items():
            if not bool(close[key[0]][key[1]]):
                assert float(np.abs(row - whole[key]).max()) <= 2e-5 * scale, key


# --- keys far away, edges of windows and chunks, gains and corrections ---------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_one_key_among_hundreds_under_a_sharp_softmax(tmp_path, dtype):
    """Scales several times the usual make every softmax sharp: a position's weight lies on one or two keys, often
    hundreds of tokens back (the first layer sees the whole prompt, the second whole chunks of 400 positions), so a key
    lost at a page border, at the edge of a tile of keys or between shares of the context moves the logits in full."""
    config = du.model(64, 90, [du.latent(4, 16, 16, 16, 48, 2.5, base=1000.0, mlp=du.dense(64)),
                               du.attention(4, 2, 32, 1.5, chunk=400, base=1000.0, mlp=du.moe(4, 2, 32, identity=1)),
                               du.latent(2, 32, 16, 32, 48, 2.0, base=1000.0, window=300)], scale=2.0)
    folder = du.write_model(tmp_path / "m", config, seed=11, dtype=dtype, std=0.15)
    prompts = ru.make_prompts(90, [700, 333], seed=4)
    cfg, weights = du.load_plain(folder)
    # the test's own premise: the first layer's softmaxes are sharp and their heaviest keys lie far back
    x = weights["embed"][torch.tensor(prompts["r0"])] * 2.0
    h = du.plain.rms(x, 1e-6) * weights["l0.norm1"]
    m = cfg["layers"][0]["mixer"]
    both = h @ weights["l0.mix.dkv"].T
    c = du.plain.rms(both[:, :48], 1e-6) * weights["l0.mix.dkv.norm"]
    k_rot = du.plain.rotate_neighbours(both[:, 48:], torch.arange(700), m["rot"])
    q = (h @ weights["l0.mix.q"].T).view(700, 4, 32)
    score = (q[:, 0, :16] @ (c @ weights["l0.mix.uk"].T).view(700, 4, 16)[:, 0].T
             + du.plain.rotate_neighbours(q[:, 0, 16:], torch.arange(700), m["rot"]) @ k_rot.T) * m["scale"]
    score = score.masked_fill(~torch.tril(torch.ones(700, 700, dtype=torch.bool)), -np.inf)
    far = (torch.arange(700) - score.argmax(-1))[400:]
    assert (far > 100).float().mean() > 0.3 and torch.softmax(score, -1).max(-1).values[400:].median() > 0.3
    steps = ru.tail_decoded(prompts, tail=48)
    for s in steps:            # every seventh position of the long first steps is compared, and every decoded token
        for e in s["entries"]:
            e["want"] = list(range(0, len(e["tokens"]), 7)) + ([len(e["tokens"]) - 1] if (len(e["tokens"]) - 1) % 7 else [])
    # (angles are position times frequency in 32-bit: 700 positions in, under softmaxes this sharp, that alone is 1e-4)
    loose = 0.5 if dtype == "bfloat16" else 2e-4
    check(folder, dtype, prompts, steps, live=2, tolerance=loose, between=5 * BETWEEN_SCHEDULES)
    check(folder, dtype, prompts, ru.portions(prompts, sizes=(130, 2, 61, 16, 17, 300, 5)), live=2, tolerance=loose,
          between=5 * BETWEEN_SCHEDULES)


def _edges(tmp_path, dtype, layer, size):
    """A layer alone whose scale is small, so that its softmax is flat and every key it sees carries its share of the
    weight: the engine's logits are the plain implementation's with this size of the mask, and clearly not those with
    a mask one token larger or smaller, in prompts, in portions and for tokens decoded one by one, with pages of 16 and
    of 4 tokens (the first key seen at a page's border, before it and behind it)."""
    config = du.model(48, 70, [layer])
    folder = du.write_model(tmp_path / "m", config, seed=20 + size, dtype=dtype, std=0.25)
    prompts = ru.make_prompts(70, [90, 49], seed=6)
    want = du.plain_logits(folder, prompts)
    others = []
    for other in (size - 1, size + 1):
        if other >= 1:
            changed = copy.deepcopy(config)
            changed["layers"][0]["mixer"]["mask"]["size"] = other
            others.append(du.plain_logits(folder, prompts, changed))
    for block_size in (16, 4):
        for steps in (ru.whole(prompts), ru.tail_decoded(prompts, tail=45), ru.portions(prompts, sizes=(18, 2, 15, 33, 3))):
            got = ru.collect(replayer(folder, dtype, prompts, live=2, block_size=block_size), steps)
            closer = total = 0
            for (n, p), row in got.items():
                if p < size + 1:
                    continue
                err = float(np.abs(row - want[n][p].numpy()).max())
                for o in others:
                    if float((want[n][p] - o[n][p]).abs().max()) < 1e-9:
                        continue          # (a position that sees the same keys under both sizes)
                    total += 1
                    closer += err < 0.25 * float((want[n][p] - o[n][p]).abs().max())
            assert total > 10 and closer >= (total if dtype == "float32" else 0.9 * total), (block_size, closer, total)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 2, 16, 17, 33])
def test_keys_just_inside_and_just_outside_a_window(tmp_path, dtype, window):
    _edges(tmp_path, dtype, du.latent(8, 16, 8, 16, 24, 0.05, base=100.0, window=window), window)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk", [2, 3, 16, 17, 33])
def test_keys_just_inside_and_just_outside_a_chunk(tmp_path, dtype, chunk):
    _edges(tmp_path, dtype, du.attention(8, 2, 16, 0.05, chunk=chunk, base=100.0), chunk)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gains_corrections_biases_and_positions_that_carry_weight(tmp_path, dtype):
    """The engine agrees with the plain implementation, whose logits move by far more than the engine's error when a
    layer's gains a column are set to one, the corrections or the biases to zero, the identity experts' router rows are
    swapped with real experts', the embedding is not scaled, the rescaling of the frequencies is taken away, the keys'
    norm gains are applied to the values too (by scaling the values' source), or the looped stretch runs once."""
    config = du.model(64, 80, [du.latent(4, 16, 8, 16, 32, 0.3, base=100.0, window=20, mlp=du.moe(5, 2, 32, identity=1, groups=(3, 2))),
                               du.attention(4, 2, 16, 0.4, chunk=20, turned=12, base=30.0, scaling=(6.0, 1.0, 4.0, 24),
                                            mlp=du.moe(3, 2, 32, identity=2))], scale=4.0, loop=(0, 2, 2))
    folder = du.write_model(tmp_path / "m", config, seed=31, dtype=dtype, std=0.2)
    prompts = ru.make_prompts(80, [60, 5], seed=8)
    _, got = check(folder, dtype, prompts, ru.tail_decoded(prompts, tail=20), live=2, most_close=0.5)
    cfg, weights = du.load_plain(folder)
    close = du.close_calls(folder, prompts, MARGIN[dtype])
    compared = [(n, p) for (n, p) in got if not bool(close[n][p])]
    want = {n: du.plain.forward(cfg, weights, t) for n, t in prompts.items()}
    err = np.sqrt(np.mean([np.mean((got[n, p] - want[n][p].numpy()) ** 2) for (n, p) in compared]))

    def without(path, value=None):
        changed = copy.deepcopy(cfg)
        at = changed
        for key in path[:-1]:
            at = at[key]
        if value is None:
            at.pop(path[-1])
        else:
            at[path[-1]] = value
        return changed

    tensor_changes = (lambda k, v: torch.ones_like(v) if k.endswith(".ls1") or k.endswith(".ls2") else v,
                      lambda k, v: v * 0 if k.endswith(".correction") else v,
                      lambda k, v: v * 0 if k.endswith(".b") else v,
                      lambda k, v: v.flip(0) if k.endswith(".router") else v,
                      lambda k, v: torch.ones_like(v) if k.endswith(".k.norm") or k.endswith(".q.norm") else v)
    config_changes = (without(["embedding", "scale"], 1.0), without(["layers", 1, "mixer", "rot", "scaling"]),
                      without(["loop", "times"], 1), without(["layers", 1, "mixer", "rot", "dims"], 16))
    moved_all = [{n: du.plain.forward(cfg, {k: change(k, v) for k, v in weights.items()}, t) for n, t in prompts.items()}
                 for change in tensor_changes]
    moved_all += [{n: du.plain.forward(changed, weights, t) for n, t in prompts.items()} for changed in config_changes]
    for at, moved in enumerate(moved_all):
        part = 0.01 if dtype == "float32" else 0.3
        shift = np.sqrt(np.mean([float(((want[n][p] - moved[n][p]) ** 2).mean()) for (n, p) in compared]))
        assert err < part * shift, (at, err, shift)


def test_the_first_tokens_of_a_request(folders):
    """Requests of one, two and three tokens, whole and token by token, in pages that others have just left."""
    folder = folders("ones", "float32")
    prompts = ru.make_prompts(du.ONES["vocab"], [1, 2, 3, 1, 2, 3, 1], seed=9)
    want = du.plain_logits(folder, prompts)
    r = replayer(folder, "float32", prompts, live=2)
    for steps in (ru.whole(prompts), ru.tail_decoded(prompts, tail=3), ru.whole(prompts)):
        got = ru.collect(r, steps)
        worst, where = ru.worst_error(got, want)
        assert worst <= 5e-5, where


def test_long_decoding(folders):
    """Two hundred tokens decoded one by one from captured steps, beside a second request, past windows, chunks and page
    borders, against the plain implementation, in bfloat16 against the engine's own whole prompts as well."""
    for dtype in DTYPES:
        folder = folders("odd", dtype)
        prompts = ru.make_prompts(du.ODD["vocab"], [230, 215], seed=12)
        steps = []
        for name, toks in prompts.items():
            steps.append({"step": len(steps), "entries": [{"id": name, "tokens": toks[:15], "want": [14]}], "end": []})
        for p in range(15, 230):
            entries = [{"id": n, "tokens": [t[p]], "want": [0]} for n, t in prompts.items() if p < len(t)]
            steps.append({"step": len(steps), "entries": entries, "end": [n for n, t in prompts.items() if p == len(t) - 1]})
        check(folder, dtype, prompts, steps, live=2)


# --- the engine's own entry point ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_greedy_generation_through_the_engine(folders, dtype):
    """Prompts of unequal length through Engine.generate (scheduler, portions of 8 tokens, batches, captured steps,
    steps queued ahead) against greedy decoding with the plain implementation."""
    from paged_llm_rs_amd import Engine

    folder = folders("odd", "float32" if dtype == "f32" else "bfloat16")
    prompts = list(ru.make_prompts(du.ODD["vocab"], [5, 23, 1, 40, 12, 9], seed=10).values())
    engine = Engine(folder, dtype=dtype, block_size=16, num_blocks=24, max_batch=4, chunk=8)
    got = engine.generate(prompts, max_tokens=12, temperature=0.0, stop_tokens=[])
    cfg, weights = du.load_plain(folder)
    for prompt, result in zip(prompts, got):
        # (the chosen token is the plain implementation's best or within rounding of it: a router's close call or a
        # near tie of two logits may fall either way, and from then on the two continue differently)
        logits = du.plain.forward(cfg, weights, prompt + result["tokens"])[len(prompt) - 1:-1]
        chosen = logits[torch.arange(12), torch.tensor(result["tokens"])]
        bound = 1e-3 if dtype == "f32" else 0.05
        assert (logits.max(-1).values - chosen).max() <= bound * logits.abs().max(), prompt
    if dtype == "f32":
        same = sum(result["tokens"] == du.plain_greedy(folder, prompt, 12) for prompt, result in zip(prompts, got))
        assert same >= len(prompts) - 1
    assert engine.cache.manager.live_sequences == 0


def test_requests_that_give_way_are_computed_again(folders):
    """A pool too small for all residents: the newest gives way, comes back and recomputes its prompt; the tokens are
    those of an engine with room to spare."""
    from paged_llm_rs_amd import Engine

    folder = folders("odd", "float32")
    prompts = list(ru.make_prompts(du.ODD["vocab"], [30, 28, 26, 31], seed=13).values())
    roomy = Engine(folder, dtype="f32", block_size=8, num_blocks=64, max_batch=4, chunk=16)
    want = roomy.generate(prompts, max_tokens=24, temperature=0.0, stop_tokens=[])
    tight = Engine(folder, dtype="f32", block_size=8, num_blocks=19, max_batch=4, chunk=16)
    got = tight.generate(prompts, max_tokens=24, temperature=0.0, stop_tokens=[])
    assert sum(r["preemptions"] for r in got) > 0, "the pool was meant to run dry"
    assert [r["tokens"] for r in got] == [r["tokens"] for r in want]


def test_the_trace_runner_and_the_command_line_run_the_design(tmp_path):
    folder = du.write_model(tmp_path / "m", du.ODD, seed=2, dtype="bfloat16")
    repo = Path(__file__).resolve().parent.parent
    prompts = ru.make_prompts(du.ODD["vocab"], [20, 9], seed=3)
    steps = ru.mixed(prompts, seed=1, max_live=2, tail=4)
    out = tmp_path / "out"
    done = subprocess.run([sys.executable, str(repo / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
                           "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]
    want = du.plain_logits(folder, prompts)
    close = du.close_calls(folder, prompts, 1e-4)
    fed: dict = {}
    for s in steps:
        rows = [(e["id"], fed.get(e["id"], 0) + w) for e in s["entries"] for w in e["want"]]
        for e in s["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
        if rows:
            got = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(len(rows), -1)
            for row, (n, p) in zip(got, rows):
                if not bool(close[n][p]):
                    assert np.abs(row - want[n][p].numpy()).max() <= 1e-4 * float(want[n][p].abs().max())


def test_the_command_line_generates_with_the_design(tmp_path):
    config = tmp_path / "config.json"
    config.write_text(json.dumps(du.ONES))
    root = Path(__file__).resolve().parent.parent
    done = subprocess.run([sys.executable, str(root / "bin" / "pagedllm"), "--model", str(tmp_path / "m"), "--random-weights",
                           str(config), "--dtype", "bf16", "--prompt-ids", "1,2,3,4,5", "--prompt-ids", "9,8",
                           "--max-tokens", "5", "--temperature", "0", "--stop-ids", ""],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [json.loads(x) for x in done.stdout.splitlines() if x.startswith("{")]
    assert len(lines) == 2 and all(len(x["tokens"]) == 5 for x in lines), done.stdout
