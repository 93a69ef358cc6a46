"""The Mukenex design in the engine against the plain implementation: the new kernels alone (the pass over the copies
of the stream, experts by table, the mask of blocks in every attention kernel), every mixer and feed-forward alone,
whole prompts, tokens decoded one by one, portions down to two tokens, mixed batches with pages and state slots used
again, keys far away under a sharp softmax, keys just inside and just outside a window and a block (in prompts and
while decoding, at page borders), sinks that carry weight, the first tokens of a request, long decoding, other sizes,
and greedy generation through the engine's own entry point and the command line."""

from __future__ import annotations

import copy
import json
import random
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import mukenex_util as mu
import replay_util as ru

pytestmark = pytest.mark.gpu

# Against the plain implementation (64-bit): 32-bit runs are held tightly.  In bfloat16 a run gets a loose bound there
# and a tight one against the engine's own whole-prompt run of the same requests (the same roundings; what differs
# between schedules is the cache, the state and the batch: a lost key or state shows there in full).  All bounds are for
# a position that amplifies rounding as the median position does, and grow with a position's own amplification.
TOLERANCE = {"float32": 5e-5, "bfloat16": 0.1}
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
            made[name, dtype] = mu.write_model(tmp_path_factory.mktemp(f"mukenex_{name}_{dtype}"), mu.CONFIGS[name],
                                               seed=sorted(mu.CONFIGS).index(name) + 1, dtype=dtype, edit=mu.wide_sinks)
        return made[name, dtype]
    return get


_whole: dict = {}
_factor: dict = {}
_plain: dict = {}


def check(folder, dtype, prompts, steps, live=4, block_size=16, tolerance=None, between=BETWEEN_SCHEDULES):
    r = replayer(folder, dtype, prompts, live, block_size)
    got = ru.collect(r, steps)
    key = (str(folder), repr(sorted(prompts.items())))
    if key not in _plain:
        _plain[key] = mu.plain_logits(folder, prompts)
        _factor[key] = mu.sensitivity(folder, prompts)
    want, factor = _plain[key], _factor[key]
    scale = max(float(want[n][p].abs().max()) for (n, p) in got)
    bound = tolerance or TOLERANCE[dtype]
    for (n, p), row in got.items():
        ref = want[n][p].numpy()
        assert row.shape == ref.shape
        err = float(np.abs(row.astype(np.float64) - ref).max()) / scale
        assert err <= bound * float(factor[n][p]), f"{err:.3e} at {(n, p)}, where the bound is {bound * float(factor[n][p]):.3e}"
    assert r.cache.manager.live_sequences == 0, "every request's pages and slot came back"
    if dtype == "bfloat16":
        if key not in _whole:
            _whole[key] = ru.collect(replayer(folder, dtype, prompts, live), ru.whole(prompts))
        spread = float(np.mean([want[n][p].std() for (n, p) in got]))
        over = {}
        for (n, p), row in got.items():
            gap = float(np.sqrt(np.mean((row - _whole[key][(n, p)]) ** 2))) / spread
            if gap > between * float(factor[n][p]):
                over[n, p] = gap / (between * float(factor[n][p]))
        assert len(over) <= max(1, len(got) // 50) and all(x <= 3.0 for x in over.values()), \
            f"between this schedule and the whole prompt, over the bound by {sorted(over.items(), key=lambda x: -x[1])[:5]} of {len(got)}"
    return r, got


# --- the new kernels alone --------------------------------------------------------------------------------------------

@pytest.mark.parametrize("copies", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("width", [52, 200, 1000, 4096])
def test_the_pass_over_the_copies_of_the_stream(copies, width):
    """Rebuild and read-out together and each alone, the read-out of chosen rows, both types of normed rows, against
    64-bit arithmetic."""
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(copies * 7 + width)
    n = 37
    x = torch.randn((n, copies, width), generator=g, dtype=torch.float64) * 3
    y = torch.randn((n, width), generator=g, dtype=torch.float64)
    mix = torch.eye(copies, dtype=torch.float64) + 0.3 * torch.randn((copies, copies), generator=g, dtype=torch.float64)
    out, into = torch.randn((copies,), generator=g, dtype=torch.float64), torch.randn((copies,), generator=g, dtype=torch.float64)
    gain = 1 + 0.2 * torch.randn((width,), generator=g, dtype=torch.float64)
    eps = 1e-5
    rebuilt = torch.einsum("sr,nsw->nrw", mix, x) + out[None, :, None] * y[:, None, :]

    def read(copies_of, weights):
        u = torch.einsum("s,nsw->nw", weights, copies_of)
        return u, u / torch.sqrt((u * u).mean(-1, keepdim=True) + eps) * gain

    dev = lambda t: t.to(torch.float32).cuda().contiguous()
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 8e-3)):
        streams = dev(x.reshape(n, copies * width))
        rows = kernels.hc_step(streams, copies, y=dev(y), mix=dev(mix), out=dev(out), read=dev(into), gain=dev(gain),
                               eps=eps, read_dtype=dtype)
        assert (streams.double().cpu().view(n, copies, width) - rebuilt).abs().max() <= 2e-6 * rebuilt.abs().max()
        want = read(rebuilt, into)[1]
        assert rows.dtype == dtype and (rows.double().cpu() - want).abs().max() <= tol * want.abs().max()
    streams = dev(x.reshape(n, copies * width))
    rows = kernels.hc_step(streams, copies, read=dev(into), gain=dev(gain), eps=eps)
    assert torch.equal(streams, dev(x.reshape(n, copies * width))), "a read-out alone changes nothing"
    assert (rows.double().cpu() - read(x, into)[1]).abs().max() <= 2e-6 * read(x, into)[1].abs().max()
    assert kernels.hc_step(streams, copies, y=dev(y), mix=dev(mix), out=dev(out)) is None
    assert (streams.double().cpu().view(n, copies, width) - rebuilt).abs().max() <= 2e-6 * rebuilt.abs().max()
    chosen = torch.tensor([5, 0, 36, 5], dtype=torch.int32).cuda()
    sums = kernels.hc_step(streams, copies, read=torch.ones(copies, device="cuda"), rows=chosen)
    want = rebuilt.sum(1)[chosen.cpu().long()]
    assert (sums.double().cpu() - want).abs().max() <= 2e-6 * want.abs().max()
    wide = kernels.stream_copies(dev(y), copies)
    assert torch.equal(wide.view(n, copies, width), dev(y)[:, None, :].expand(n, copies, width))


@pytest.mark.parametrize("width,group,gains", [(120, 120, 120), (1024, 1024, 1024), (2048, 1024, 2048), (2560, 2560, 2560),
                                                (640, 640, 640), (3000, 1500, 1500), (1024, 128, 128)])
@pytest.mark.parametrize("act", [None, "sigmoid", "silu"])
def test_the_norm_over_all_heads_of_a_state_layers_read_out(width, group, gains, act):
    """Groups of a head up to the whole row (above 512 columns a workgroup of four waves takes a group, above 2,048 in two
    rounds), a gain a column of the row or of a group, no gate and both kinds, against 64-bit arithmetic."""
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(width + group)
    n, off = 19, 5
    x = torch.randn((n, width), generator=g, dtype=torch.float64) * 2
    gain = 1 + 0.3 * torch.randn((gains,), generator=g, dtype=torch.float64)
    gate = torch.randn((n, off + width + 3), generator=g, dtype=torch.float64)
    eps = 1e-5
    grouped = x.view(n, width // group, group)
    want = (grouped / torch.sqrt((grouped * grouped).mean(-1, keepdim=True) + eps)).reshape(n, width)
    want = want * (gain if gains == width else gain.repeat(width // group))
    if act is not None:
        chosen = gate[:, off:off + width]
        want = want * (torch.sigmoid(chosen) if act == "sigmoid" else chosen * torch.sigmoid(chosen))
    for dtype, tol in ((torch.float32, 3e-6), (torch.bfloat16, 8e-3)):
        got = kernels.gated_group_norm(x.float().cuda(), group, gain.float().cuda(), eps, dtype,
                                       gate=gate.float().cuda() if act else None, gate_off=off if act else 0, gate_act=act)
        assert got.dtype == dtype and (got.double().cpu() - want).abs().max() <= tol * want.abs().max()


class _Rows:
    """What the experts' kernels read of a step."""

    def __init__(self, ids, positions=None):
        self.token_ids = torch.tensor(ids, dtype=torch.int32).cuda()
        self.positions = torch.tensor(positions if positions is not None else list(range(len(ids))), dtype=torch.int32).cuda()
        self.fed_tokens = None
        self.token_src = None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,top,ff,width,rows", [(8, 3, 64, 160, 50), (3, 3, 44, 52, 7), (1, 1, 24, 100, 3), (16, 4, 40, 256, 300),
                                                      (32, 4, 128, 1024, 700), (4, 1, 256, 512, 129)])
def test_experts_by_table(dtype, experts, top, ff, width, rows):
    """Every row against 64-bit arithmetic over its own experts; rows of padding give zeros; a row whose id was left on the
    device by the step before takes that id."""
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(experts * 100 + rows)
    vocab = 41
    w_gu = (torch.randn((experts, 2 * ff, width), generator=g) * width ** -0.5).to(dtype)
    w_down = (torch.randn((experts, width, ff), generator=g) * ff ** -0.5).to(dtype)
    x = torch.randn((rows, width), generator=g).to(dtype)
    table = torch.rand((vocab, experts), generator=g).argsort(1)[:, :top].to(torch.int32)
    ids = torch.randint(0, vocab, (rows,), generator=g).tolist()
    positions = list(range(rows))
    positions[rows // 2] = -1
    batch = _Rows(ids, positions)
    got = kernels.moe_rows(x.cuda(), batch, table.cuda(), w_gu.cuda(), w_down.cuda(), "silu").double().cpu()
    want = torch.zeros((rows, width), dtype=torch.float64)
    hidden = torch.zeros((rows, top, ff), dtype=torch.float64)
    for t in range(rows):
        for c, e in enumerate(table[ids[t]].tolist()):
            both = w_gu[e].double() @ x[t].double()
            hidden[t, c] = torch.nn.functional.silu(both[:ff]) * both[ff:]
            if dtype == torch.bfloat16:
                hidden[t, c] = hidden[t, c].to(torch.bfloat16).double()      # (what lies between the two products is stored in the rows' type)
            want[t] += w_down[e].double() @ hidden[t, c] / top
    want[rows // 2] = 0
    assert (got - want).abs().max() <= (1e-5 if dtype == torch.float32 else 2e-2) * want.abs().max()
    if rows >= 7:
        batch.fed_tokens = torch.tensor([3, 40, 17], dtype=torch.int32).cuda()
        src = [-1] * rows
        src[1], src[4] = 2, 0
        batch.token_src = torch.tensor(src, dtype=torch.int32).cuda()
        fed = kernels.moe_rows(x.cuda(), batch, table.cuda(), w_gu.cuda(), w_down.cuda(), "silu").double().cpu()
        ids2 = list(ids)
        ids2[1], ids2[4] = 17, 3
        again = kernels.moe_rows(x.cuda(), _Rows(ids2, positions), table.cuda(), w_gu.cuda(), w_down.cuda(), "silu").double().cpu()
        assert torch.equal(fed, again)


@pytest.mark.parametrize("experts,top,ff,width,rows", [(8, 3, 64, 160, 50), (8, 3, 64, 160, 1), (16, 4, 128, 256, 300), (32, 4, 128, 1024, 700),
                                                      (4, 1, 256, 512, 129), (64, 8, 64, 96, 5), (3, 3, 192, 160, 1000), (2, 2, 1536, 1024, 64)])
def test_experts_by_table_dealt_to_their_experts(experts, top, ff, width, rows):
    """The grouped products on the matrix cores against the kernel that takes a row at a time (bfloat16): the same
    pairs, the same weights, sums in another order.  Rows of padding give zeros; ids left on the device are taken;
    an expert that nobody chose, experts with more than a tile of rows, more experts than pairs."""
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(experts * 100 + rows)
    vocab = 53
    w_gu = (torch.randn((experts, 2 * ff, width), generator=g) * width ** -0.5).to(torch.bfloat16).cuda()
    w_down = (torch.randn((experts, width, ff), generator=g) * ff ** -0.5).to(torch.bfloat16).cuda()
    x = torch.randn((rows, width), generator=g).to(torch.bfloat16).cuda()
    assert kernels.moe_grouped_applies(x, width, ff)
    table = torch.rand((vocab, experts), generator=g).argsort(1)[:, :top].to(torch.int32)
    if experts > 2:
        table[table == 1] = 0 if top == 1 else table[table == 1]      # (with one choice a row, expert 1 is never chosen)
    table = table.cuda()
    ids = torch.randint(0, vocab, (rows,), generator=g).tolist()
    positions = list(range(rows))
    if rows > 2:
        positions[rows // 2] = -1
    batch = _Rows(ids, positions)
    if rows >= 7:
        batch.fed_tokens = torch.tensor([3, 40, 17], dtype=torch.int32).cuda()
        src = [-1] * rows
        src[1], src[4] = 2, 0
        batch.token_src = torch.tensor(src, dtype=torch.int32).cuda()
    want = kernels.moe_rows(x, batch, table, w_gu, w_down, "silu")
    for _ in range(2):           # (which slot a pair gets may differ from run to run; what it computes may not)
        got = kernels.moe_grouped(x, batch, table, w_gu, w_down, "silu")
        assert got.shape == want.shape and torch.isfinite(got).all()
        assert (got - want).abs().max() <= 1e-2 * want.abs().max()
        if rows > 2:
            assert float(got[rows // 2].abs().max()) == 0.0
    again = kernels.moe_grouped(x, batch, table, w_gu, w_down, "silu")
    assert torch.equal(got, again), "a row's result does not depend on its place in a tile"


def _blocks_oracle(q, k, v, positions, block, scale):
    """Softmax attention of one request's queries at ``positions`` over keys 0 .. T - 1 inside the query's own block."""
    T = k.shape[0]
    kp = torch.arange(T)
    seen = (kp[None, :] <= positions[:, None]) & ((kp[None, :] // block) == (positions[:, None] // block))
    out = torch.zeros(q.shape[0], q.shape[1], v.shape[-1], dtype=torch.float64)
    group = q.shape[1] // k.shape[1]
    for h in range(q.shape[1]):
        s = (q[:, h] @ k[:, h // group].T) * scale
        out[:, h] = torch.softmax(s.masked_fill(~seen, -np.inf), -1) @ v[:, h // group]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("block,heads,kv_heads,d,page", [(64, 4, 2, 64, 16), (70, 8, 1, 128, 16), (5, 2, 2, 32, 4), (100, 16, 2, 64, 8),
                                                         (128, 4, 4, 128, 16), (1, 2, 1, 16, 16), (37, 8, 1, 48, 16)])
def test_a_mask_of_blocks_in_every_attention_kernel(dtype, block, heads, kv_heads, d, page):
    """One request of 300 keys; queries as a long portion (the matrix-core kernel in bfloat16), as a short portion and as
    single tokens (the kernels for single tokens and for groups of heads), at the first and last positions of blocks and
    in their middle.  In some rows one key just outside the query's block is made to answer the query with a huge
    score: seen, it would take all the weight."""
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.cache.pools import LayerKV

    g = torch.Generator().manual_seed(block * 13 + heads)
    T = 300
    k = torch.randn((T, kv_heads, d), generator=g)
    v = torch.randn((T, kv_heads, d), generator=g)
    pages = -(-T // page)
    order = torch.randperm(pages + 3, generator=g)[:pages]
    k_pool = torch.full(((pages + 3) * page, kv_heads * d), float("nan"))
    v_pool = torch.full(((pages + 3) * page, kv_heads * d), float("nan"))
    for j in range(T):
        row = int(order[j // page]) * page + j % page
        k_pool[row], v_pool[row] = k[j].reshape(-1), v[j].reshape(-1)
    k_pool, v_pool = k_pool.to(dtype).cuda(), v_pool.to(dtype).cuda()
    k64, v64 = k.to(dtype).double(), v.to(dtype).double()
    table = order.to(torch.int32).view(1, pages).cuda()
    scale = d ** -0.5

    class Step:
        pass

    def run(first, count):
        """Queries at positions first .. first + count - 1 of a request whose context then ends there."""
        positions = torch.arange(first, first + count)
        q = torch.randn((count, heads, d), generator=g)
        for i, p in enumerate(positions.tolist()):
            outside = (p // block) * block - 1
            if outside >= 0 and i % 3 == 0:
                q[i] = k[outside, :, None, :].expand(kv_heads, heads // kv_heads, d).reshape(heads, d) * 40
        q = q.to(dtype)
        b = Step()
        b.positions = positions.to(torch.int32).cuda()
        b.seq_of = torch.zeros(count, dtype=torch.int32).cuda()
        b.q_start = torch.zeros(1, dtype=torch.int32).cuda()
        b.q_len = torch.tensor([count], dtype=torch.int32).cuda()
        b.ctx_len = torch.tensor([first + count], dtype=torch.int32).cuda()
        b.max_q_len, b.max_ctx_len, b.num_tokens, b.num_seqs, b.live_seqs = count, 1024, count, 1, 1
        b.tokens_of_short_requests = lambda limit: count if count < limit else 0
        kv = LayerKV(k_pool, v_pool, table, page, 0)
        out = torch.empty((count, heads * d), dtype=dtype, device="cuda")
        kernels.sink_attention(q.reshape(count, heads * d).cuda().contiguous(), out, b, kv, heads, kv_heads, d, scale, -block)
        want = _blocks_oracle(q.double(), k64, v64, positions, block, scale).reshape(count, heads * d)
        err = (out.double().cpu() - want).abs().max() / want.abs().max()
        assert err <= (3e-5 if dtype == torch.float32 else 2e-2), (first, count, float(err))      # (queries times 40 amplify rounding)

    run(0, 300)                       # a whole prompt
    run(130, 170)                     # a long portion behind a context
    run(max(block * 2 - 3, 0) if block * 2 - 3 + 9 <= T else 0, 9)     # a short portion across a block's edge
    for first in sorted({0, block - 1, block, 2 * block - 1, 2 * block, T - 1, T // 2} & set(range(T))):
        run(first, 1)                 # single tokens: first and last of blocks


# --- every mixer and feed-forward alone, in 32-bit, the stream behind the layer against the plain implementation's ----

ALONE = {
    "latent, a window": [mu.latent(3, 24, 8, 40, 56, 0.3, base=300.0, window=11)],
    "latent, no window, part of the rotated values turn": [mu.latent(2, 16, 12, 16, 20, 0.4, base=40.0, turned=6)],
    "attention, blocks of 7": [mu.attention(6, 3, 24, 40, 0.4, block=7)],
    "attention, no mask": [mu.attention(2, 1, 40, 24, 0.2)],
    "lightning": [mu.lightning(3, 24, 40, (0.5, 0.9, 0.999))],
    "dense feed-forward": [mu.attention(1, 1, 16, 16, 0.5, mlp=mu.dense(136))],
    "experts": [mu.lightning(1, 16, 16, (0.9,), mlp=mu.moe(6, 3, 40))],
}


@pytest.mark.parametrize("streams", [None, 3])
@pytest.mark.parametrize("which", sorted(ALONE))
def test_a_layer_alone_against_its_plain_function(tmp_path, which, streams):
    """32-bit, the stream behind the layer (the sum of its copies) against the plain implementation's: whole, and again
    in portions (the later portions read what the earlier ones left in pages and state)."""
    config = mu.model(88, 61, ALONE[which], eps=1e-5, streams=streams, softcap=9.0)
    folder = mu.write_model(tmp_path / "m", config, seed=7, std=0.2, edit=mu.wide_sinks)
    tokens = [random.Random(3).randrange(61) for _ in range(45)]
    cfg, weights = mu.load_plain(folder)
    want = []
    mu.plain.forward(cfg, weights, tokens, want)
    summed = lambda t: t.double().cpu().view(t.shape[0], streams or 1, 88).sum(1)
    r = replayer(folder, "float32", {"a": tokens}, graphs=False)
    rec = {}
    r.step([{"id": "a", "tokens": tokens, "want": []}], ["a"], trace=rec)
    assert (summed(rec["l0.out"]) - want[0]).abs().max() <= 5e-5 * want[0].abs().max(), which
    pieces, at = [], 0
    for n in (1, 2, 17, 3, 22):
        rec = {}
        r.step([{"id": "b", "tokens": tokens[at:at + n], "want": []}], ["b"] if at + n == 45 else [], trace=rec)
        pieces.append(summed(rec["l0.out"]))
        at += n
    assert (torch.cat(pieces) - want[0]).abs().max() <= 5e-5 * want[0].abs().max(), (which, "in portions")


# --- whole models of other sizes under every schedule ------------------------------------------------------------------

LENGTHS = [70, 3, 41, 18, 1, 33, 57]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(mu.CONFIGS))
def test_whole_prompts(folders, name, dtype):
    prompts = ru.make_prompts(mu.CONFIGS[name]["vocab"], LENGTHS, seed=1)
    check(folders(name, dtype), dtype, prompts, ru.whole(prompts))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(mu.CONFIGS))
def test_prefill_then_tokens_one_by_one(folders, name, dtype):
    prompts = ru.make_prompts(mu.CONFIGS[name]["vocab"], LENGTHS, seed=1)
    check(folders(name, dtype), dtype, prompts, ru.tail_decoded(prompts, tail=40))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(mu.CONFIGS))
@pytest.mark.parametrize("block_size", [16, 8])
def test_portions_down_to_two_tokens(folders, name, dtype, block_size):
    prompts = ru.make_prompts(mu.CONFIGS[name]["vocab"], LENGTHS, seed=1)
    check(folders(name, dtype), dtype, prompts, ru.portions(prompts), block_size=block_size)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(mu.CONFIGS))
@pytest.mark.parametrize("seed", [0, 1])
def test_unequal_requests_together_with_pages_and_slots_used_again(folders, name, dtype, seed):
    """Nine requests of unequal length through a pool and state slots that hold four: portions of some beside single
    tokens of others, requests left out of steps, pages and slots of finished requests taken by the next."""
    prompts = ru.make_prompts(mu.CONFIGS[name]["vocab"], [70, 3, 41, 18, 1, 33, 57, 64, 22], seed=2 + seed)
    check(folders(name, dtype), dtype, prompts, ru.mixed(prompts, seed=seed, max_live=4, tail=14))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(tmp_path, seed, dtype):
    """Ten drawn models (order of layers, copies, looped stretch, sizes, head counts, windows, blocks, experts, constants;
    `mukenex_util.drawn_config`) under a mixed schedule and whole, over pages of 16, 8 and 32 tokens."""
    config = mu.drawn_config(100 + seed)
    folder = mu.write_model(tmp_path / "m", config, seed=seed, dtype=dtype, std=0.1, edit=mu.wide_sinks)
    prompts = ru.make_prompts(config["vocab"], [75, 9, 130, 33, 2], seed=seed)
    block_size = (16, 8, 32)[seed % 3]
    check(folder, dtype, prompts, ru.mixed(prompts, seed=seed, max_live=3, tail=20), live=3, block_size=block_size)
    check(folder, dtype, prompts, ru.whole(prompts), live=3, block_size=block_size)


def test_schedules_agree_with_each_other_in_32_bit(folders):
    folder = folders("odd", "float32")
    prompts = ru.make_prompts(mu.ODD["vocab"], LENGTHS, seed=1)
    whole = ru.collect(replayer(folder, "float32", prompts), ru.whole(prompts))
    scale = max(float(np.abs(row).max()) for row in whole.values())
    for steps in (ru.tail_decoded(prompts, tail=40), ru.portions(prompts), ru.mixed(prompts, seed=5)):
        for key, row in ru.collect(replayer(folder, "float32", prompts), steps).items():
            assert float(np.abs(row - whole[key]).max()) <= 2e-5 * scale, key


# --- keys far away, edges of windows and blocks, sinks, tables -------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_one_key_among_hundreds_under_a_sharp_softmax(tmp_path, dtype):
    """Scales several times the usual make every softmax sharp: a position's weight lies on one or two keys, often
    hundreds of tokens back (the first layer sees the whole prompt, the third whole blocks of 400 positions), so a key
    lost at a page border, at the edge of a tile of keys or between shares of the context moves the logits in full; a
    state layer whose decay is near one carries the first tokens to the last."""
    config = mu.model(64, 90, [mu.latent(4, 16, 16, 16, 48, 2.5, base=1000.0, mlp=mu.dense(64)),
                               mu.lightning(2, 16, 16, (0.9995, 0.99)),
                               mu.attention(4, 2, 32, 32, 1.5, block=400, mlp=mu.moe(4, 2, 32)),
                               mu.latent(2, 32, 16, 32, 48, 2.0, base=1000.0, window=300)], streams=2)
    folder = mu.write_model(tmp_path / "m", config, seed=11, dtype=dtype, std=0.15, edit=mu.wide_sinks)
    prompts = ru.make_prompts(90, [700, 333], seed=4)
    cfg, weights = mu.load_plain(folder)
    # the test's own premise: the first layer's softmaxes are sharp and their heaviest keys lie far back
    x = weights["embed"][torch.tensor(prompts["r0"])]
    h = mu.plain.norm_around_zero(x * weights["l0.hc1.in"].sum(), weights["l0.norm1"], 1e-6)
    m = cfg["layers"][0]["mixer"]
    both = h @ weights["l0.mix.dkv"].T
    c = mu.plain.rms(both[:, :48], 1e-6) * weights["l0.mix.dkv.norm"]
    k_rot = mu.plain.rotate_neighbours(both[:, 48:], torch.arange(700), 16, 1000.0)
    q = (h @ weights["l0.mix.q"].T).view(700, 4, 32)
    score = (q[:, 0, :16] @ (c @ weights["l0.mix.uk"].T).view(700, 4, 16)[:, 0].T
             + mu.plain.rotate_neighbours(q[:, 0, 16:], torch.arange(700), 16, 1000.0) @ k_rot.T) * m["scale"]
    score = score.masked_fill(~torch.tril(torch.ones(700, 700, dtype=torch.bool)), -np.inf)
    far = (torch.arange(700) - score.argmax(-1))[400:]
    assert (far > 100).float().mean() > 0.3 and torch.softmax(score, -1).max(-1).values[400:].median() > 0.3
    steps = ru.tail_decoded(prompts, tail=48)
    for s in steps:            # every seventh position of the long first steps is compared, and every decoded token
        for e in s["entries"]:
            e["want"] = list(range(0, len(e["tokens"]), 7)) + ([len(e["tokens"]) - 1] if (len(e["tokens"]) - 1) % 7 else [])
    loose = 0.5 if dtype == "bfloat16" else None
    check(folder, dtype, prompts, steps, live=2, tolerance=loose, between=5 * BETWEEN_SCHEDULES)
    check(folder, dtype, prompts, ru.portions(prompts, sizes=(130, 2, 61, 16, 17, 300, 5)), live=2, tolerance=loose,
          between=5 * BETWEEN_SCHEDULES)


def _edges(tmp_path, dtype, layer, size, resize):
    """A layer alone whose scale is small, so that its softmax is flat and every key it sees carries its share of the
    weight: the engine's logits are the plain implementation's with this size of the mask, and clearly not those with
    a mask one token larger or smaller, in prompts, in portions and for tokens decoded one by one, with pages of 16 and
    of 4 tokens (the first key seen at a page's border, before it and behind it)."""
    config = mu.model(48, 70, [layer], streams=2)
    folder = mu.write_model(tmp_path / "m", config, seed=20 + size, dtype=dtype, std=0.25)
    prompts = ru.make_prompts(70, [90, 49], seed=6)
    want = mu.plain_logits(folder, prompts)
    others = []
    for other in (size - 1, size + 1):
        if other >= 1:
            changed = copy.deepcopy(config)
            changed["layers"][0]["mixer"]["mask"]["size"] = other
            others.append(mu.plain_logits(folder, prompts, changed))
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
    _edges(tmp_path, dtype, mu.latent(8, 16, 8, 16, 24, 0.05, base=100.0, window=window), window, None)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("block", [2, 3, 16, 17, 33])
def test_keys_just_inside_and_just_outside_a_block(tmp_path, dtype, block):
    _edges(tmp_path, dtype, mu.attention(8, 2, 16, 16, 0.05, block=block), block, None)


@pytest.mark.parametrize("dtype", DTYPES)
def test_sinks_tables_and_copies_that_carry_weight(tmp_path, dtype):
    """Sinks between -1.5 and 2.5 beside scores of the same size, a table that decides which experts a token uses, and
    weights between the copies of the stream: the engine agrees with the plain implementation, whose logits move by far
    more than the engine's error when the sinks are set to zero or taken away, the table's rows are turned round, or the
    copies are mixed the other way."""
    config = mu.model(64, 80, [mu.latent(4, 16, 8, 16, 32, 0.3, base=100.0, window=20, mlp=mu.moe(6, 2, 32)),
                               mu.attention(4, 2, 16, 16, 0.4, block=20, mlp=mu.moe(4, 1, 32))], streams=3, loop=(0, 2, 2))
    folder = mu.write_model(tmp_path / "m", config, seed=31, dtype=dtype, std=0.2, edit=mu.wide_sinks)
    prompts = ru.make_prompts(80, [60, 5], seed=8)
    _, got = check(folder, dtype, prompts, ru.tail_decoded(prompts, tail=20), live=2)
    cfg, weights = mu.load_plain(folder)
    want = {n: mu.plain.forward(cfg, weights, t) for n, t in prompts.items()}
    changes = (lambda k, v: v * 0 if k.endswith(".sink") else v,
               lambda k, v: v - 50 if k.endswith(".sink") else v,
               lambda k, v: (v + 1) % (6 if k.startswith("l0.") else 4) if k.endswith(".table") else v,
               lambda k, v: v.T.contiguous() if k.endswith(".mix") and ".hc" in k else v,
               lambda k, v: v * 0 if k.endswith(".b") else v)
    for change in changes:
        moved = {n: mu.plain.forward(cfg, {k: change(k, v) for k, v in weights.items()}, t) for n, t in prompts.items()}
        part = 0.01 if dtype == "float32" else 0.3
        err = np.sqrt(np.mean([np.mean((row - want[n][p].numpy()) ** 2) for (n, p), row in got.items()]))
        shift = np.sqrt(np.mean([float(((want[n][p] - moved[n][p]) ** 2).mean()) for (n, p) in got]))
        assert err < part * shift, (err, shift)


def test_the_first_tokens_of_a_request(folders):
    """Requests of one, two and three tokens, whole and token by token, in slots and pages that others have just left."""
    folder = folders("ones", "float32")
    prompts = ru.make_prompts(mu.ONES["vocab"], [1, 2, 3, 1, 2, 3, 1], seed=9)
    want = mu.plain_logits(folder, prompts)
    r = replayer(folder, "float32", prompts, live=2)
    for steps in (ru.whole(prompts), ru.tail_decoded(prompts, tail=3), ru.whole(prompts)):
        got = ru.collect(r, steps)
        worst, where = ru.worst_error(got, want)
        assert worst <= 5e-5, where


def test_long_decoding(folders):
    """Two hundred tokens decoded one by one from captured steps, beside a second request, past windows, blocks and page
    borders, against the plain implementation, in bfloat16 against the engine's own whole prompts as well."""
    for dtype in DTYPES:
        folder = folders("odd", dtype)
        prompts = ru.make_prompts(mu.ODD["vocab"], [230, 215], seed=12)
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
    steps queued ahead: a decoded token's experts are then looked up from an id that never left the device) against
    greedy decoding with the plain implementation."""
    from paged_llm_rs_amd import Engine

    folder = folders("odd", "float32" if dtype == "f32" else "bfloat16")
    prompts = list(ru.make_prompts(mu.ODD["vocab"], [5, 23, 1, 40, 12, 9], seed=10).values())
    engine = Engine(folder, dtype=dtype, block_size=16, num_blocks=24, max_batch=4, chunk=8)
    got = engine.generate(prompts, max_tokens=12, temperature=0.0, stop_tokens=[])
    if dtype == "f32":
        for prompt, result in zip(prompts, got):
            assert result["tokens"] == mu.plain_greedy(folder, prompt, 12), prompt
    else:
        cfg, weights = mu.load_plain(folder)
        for prompt, result in zip(prompts, got):
            logits = mu.plain.forward(cfg, weights, prompt + result["tokens"])[len(prompt) - 1:-1]
            chosen = logits[torch.arange(12), torch.tensor(result["tokens"])]
            assert (logits.max(-1).values - chosen).max() <= 0.05 * logits.abs().max(), prompt
    assert engine.cache.manager.live_sequences == 0


def test_requests_that_give_way_are_computed_again(folders):
    """A pool too small for all residents: the newest gives way, comes back and recomputes its prompt into a cleared
    state slot; the tokens are those of an engine with room to spare."""
    from paged_llm_rs_amd import Engine

    folder = folders("odd", "float32")
    prompts = list(ru.make_prompts(mu.ODD["vocab"], [30, 28, 26, 31], seed=13).values())
    roomy = Engine(folder, dtype="f32", block_size=8, num_blocks=64, max_batch=4, chunk=16)
    want = roomy.generate(prompts, max_tokens=24, temperature=0.0, stop_tokens=[])
    tight = Engine(folder, dtype="f32", block_size=8, num_blocks=19, max_batch=4, chunk=16)
    got = tight.generate(prompts, max_tokens=24, temperature=0.0, stop_tokens=[])
    assert sum(r["preemptions"] for r in got) > 0, "the pool was meant to run dry"
    assert [r["tokens"] for r in got] == [r["tokens"] for r in want]


def test_the_trace_runner_and_the_command_line_run_the_design(tmp_path):
    folder = mu.write_model(tmp_path / "m", mu.ODD, seed=2, dtype="bfloat16")
    repo = Path(__file__).resolve().parent.parent
    prompts = ru.make_prompts(mu.ODD["vocab"], [20, 9], seed=3)
    steps = ru.mixed(prompts, seed=1, max_live=2, tail=4)
    out = tmp_path / "out"
    done = subprocess.run([sys.executable, str(repo / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
                           "--out", str(out), "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]
    want = mu.plain_logits(folder, prompts)
    fed: dict = {}
    for s in steps:
        rows = [(e["id"], fed.get(e["id"], 0) + w) for e in s["entries"] for w in e["want"]]
        for e in s["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
        if rows:
            got = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(len(rows), -1)
            for row, (n, p) in zip(got, rows):
                assert np.abs(row - want[n][p].numpy()).max() <= 1e-4 * float(want[n][p].abs().max())


def test_the_command_line_generates_with_the_design(tmp_path):
    config = tmp_path / "config.json"
    config.write_text(json.dumps(mu.ONES))
    root = Path(__file__).resolve().parent.parent
    done = subprocess.run([sys.executable, str(root / "bin" / "pagedllm"), "--model", str(tmp_path / "m"), "--random-weights",
                           str(config), "--dtype", "bf16", "--prompt-ids", "1,2,3,4,5", "--prompt-ids", "9,8",
                           "--max-tokens", "5", "--temperature", "0", "--stop-ids", ""],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [json.loads(x) for x in done.stdout.splitlines() if x.startswith("{")]
    assert len(lines) == 2 and all(len(x["tokens"]) == 5 for x in lines), done.stdout
