"""Configurations, model folders and comparisons for the tests of the Dimalix design."""

from __future__ import annotations

import copy
import json
import math
from pathlib import Path

import torch

import plain_dimalix as plain


def attention(heads, kv_heads, dim, scale, chunk=None, turned=None, base=10000.0, scaling=None, mlp=None):
    rot = {"dims": dim if turned is None else turned, "base": base}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "rot": rot}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, window=None, scaling=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"dims": rot_dim, "base": base}}
    if scaling is not None:
        m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if window is not None:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, identity=None, groups=None):
    router = {"experts": experts, "top": top}
    if identity is not None:
        router["identity"] = identity
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def model(width, vocab, layers, eps=1e-6, scale=None, loop=None):
    config = {"architecture": "Dimalix", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if scale is not None:
        config["embedding"] = {"scale": scale}
    if loop is not None:
        config["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return config


# Odd sizes: a stretch of three layers that runs three times (layers of both kinds of pages in it), heads of 24 of which
# 10 values turn, three query heads a key head, chunks of 5 and 37 positions and windows of 9 and 37 (inside a page,
# across page borders), rescaled frequencies whose three ranges are all met, 7 experts and 2 identity experts in 3 groups
# of which 2 are kept, 6 + 0 in 2 groups of which 1, a layer without a feed-forward.
ODD = model(72, 211, [
    latent(3, 24, 8, 40, 40, 0.21, base=500.0, window=37, mlp=moe(7, 2, 24, identity=2, groups=(3, 2))),
    attention(6, 2, 24, 0.3, chunk=5, turned=10, base=100.0, scaling=(4.0, 1.0, 3.0, 64), mlp=moe(4, 3, 40, identity=1)),
    latent(5, 16, 8, 24, 40, 0.3, base=500.0, window=9, mlp=dense(96)),
    attention(3, 3, 40, 0.2, chunk=37, base=3000.0),
    attention(4, 1, 16, 0.25, chunk=64, turned=16, base=50.0, scaling=(8.0, 1.0, 4.0, 32), mlp=moe(6, 2, 16, identity=0, groups=(2, 1))),
], eps=1e-5, scale=3.0, loop=(0, 3, 3))

# What a small model tends to make equal or 1 is different here: one head, one expert of one, one expert beside three
# identity experts, a stretch that "loops" once, a window and a chunk of one position, a rotated part of two values, a
# scale of one, a width that is no multiple of eight, no embedding scale, groups of one expert each, every group kept.
ONES = model(100, 97, [
    attention(4, 1, 16, 1.0, chunk=1, mlp=moe(1, 1, 48)),
    latent(1, 48, 2, 48, 30, 1.0, base=50.0, window=1, mlp=moe(1, 2, 24, identity=3, groups=(4, 4))),
    attention(1, 1, 64, 0.5, turned=2, mlp=dense(32)),
    latent(2, 16, 16, 16, 30, 0.25, base=50.0, mlp=moe(3, 1, 40, groups=(3, 1))),
], eps=1e-6, loop=(2, 4, 1))

# Without loop, embedding scale, masks, groups and identity experts (the keys are absent); larger sizes: pages' rows of
# 256 (a vector of 192 with a rotated part of 64), heads of 128, sixteen query heads a key head, expert widths and a
# width that the grouped products on the matrix cores take.
PLAIN = model(256, 300, [
    latent(8, 64, 64, 64, 192, 0.09, base=10000.0, mlp=moe(8, 2, 64)),
    attention(16, 1, 128, 0.1, mlp=dense(352)),
    attention(4, 2, 64, 0.15, chunk=64, turned=32, scaling=(8.0, 1.0, 4.0, 2048), mlp=moe(8, 4, 128, identity=2, groups=(5, 3))),
    latent(2, 128, 64, 128, 192, 0.07, base=10000.0, window=64, mlp=dense(256)),
    attention(8, 8, 32, 0.2, chunk=100, mlp=moe(16, 3, 64, identity=4, groups=(4, 2))),
], eps=1e-6)

# Rows of the pages beyond what the matrix-core kernels take (a vector of 272 with a rotated part of 16), head sizes that
# are no multiple of 4 (30, 22) or of 8 (20, 36), a rotation over 10 of 30 values, a width that is a multiple of 4 only,
# experts whose width is no multiple of 8, a looped stretch that is the whole model.
UNEVEN = model(52, 75, [
    latent(2, 20, 16, 36, 272, 0.2, base=123.0, window=100, mlp=moe(3, 2, 44, identity=1)),
    attention(3, 1, 30, 0.3, chunk=50, turned=10, base=77.0, mlp=dense(44)),
    attention(2, 2, 22, 0.3, chunk=3, mlp=moe(2, 2, 12, identity=2, groups=(2, 2))),
    latent(3, 22, 12, 30, 50, 0.21, base=123.0, window=3),
], eps=3e-6, scale=0.5, loop=(0, 4, 2))

CONFIGS = {"odd": ODD, "ones": ONES, "plain": PLAIN, "uneven": UNEVEN}


def telling(tensors) -> None:
    """Tensors as drawn would hide faults: biases and corrections near zero, layer scales and gains near one, routers whose
    scores are all alike.  Biases as large as what they are added to, corrections that move the choice, layer scales
    between 0.3 and 1.7, routers whose softmax has a clear order (a close call between two experts may fall either
    way under rounding)."""
    for name in list(tensors):
        t = tensors[name]
        if name.endswith(".b"):
            tensors[name] = (t.float() * 6).to(t.dtype)
        elif name.endswith(".correction"):
            tensors[name] = (t.float() * 2).to(t.dtype)
        elif name.endswith(".router"):
            tensors[name] = (t.float() * 3).to(t.dtype)
        elif name.endswith(".ls1") or name.endswith(".ls2"):
            tensors[name] = (1.0 + (t.float() - 1.0) * 3.5).clamp(0.3, 1.7).to(t.dtype)


def write_model(folder, config, seed=0, dtype="float32", std=0.08, gain_std=0.2, edit=telling) -> Path:
    """A model folder with random weights from the package's random-weights mode; ``edit(tensors)`` changes them."""
    from paged_llm_rs_amd.weights import write_random_model

    folder = write_random_model(Path(folder), copy.deepcopy(config), seed=seed, std=std, gain_std=gain_std, dtype=dtype)
    if edit is not None:
        from safetensors.torch import load_file, save_file

        tensors = load_file(str(folder / "model.safetensors"))
        edit(tensors)
        save_file({k: v.contiguous() for k, v in tensors.items()}, str(folder / "model.safetensors"))
    return folder


def load_plain(folder):
    from safetensors.torch import load_file

    config = json.loads((Path(folder) / "config.json").read_text())
    weights = {k: (v.to(torch.float64) if v.is_floating_point() else v)
               for k, v in load_file(str(Path(folder) / "model.safetensors")).items()}
    return config, weights


def plain_logits(folder, prompts: dict, config=None) -> dict:
    """``config``: another config.json to read the same weights with (a window one larger, say)."""
    own, weights = load_plain(folder)
    return {name: plain.forward(config or own, weights, tokens) for name, tokens in prompts.items()}


def plain_greedy(folder, prompt, count: int) -> list:
    config, weights = load_plain(folder)
    tokens, out = list(prompt), []
    for _ in range(count):
        nxt = int(plain.forward(config, weights, tokens)[-1].argmax())
        out.append(nxt)
        tokens.append(nxt)
    return out


def sensitivity(folder, prompts: dict) -> dict:
    """name -> a factor a position (>= 1): how much more than the median position this position's logits move when
    every weight matrix is disturbed by 2^-9 of itself (root mean square over the vocabulary; the larger of two
    disturbances).  Random models have single positions where rounding is amplified many times (a score near a tie
    under a sharp softmax, a router's close call); a bound on an engine's error there has to grow with it."""
    config, weights = load_plain(folder)
    out = {name: None for name in prompts}
    for sample in range(2):
        g = torch.Generator().manual_seed(1234 + sample)
        shaken = {k: v * (1 + (torch.rand(v.shape, generator=g, dtype=v.dtype) - 0.5) * 2.0 ** -8)
                  if v.dim() == 2 and v.is_floating_point() else v for k, v in weights.items()}
        for name, tokens in prompts.items():
            base = plain.forward(config, weights, tokens)
            moved = ((plain.forward(config, shaken, tokens) - base) ** 2).mean(-1).sqrt() / base.std()
            factor = torch.clamp(moved / (2 * moved.median()), min=1.0)
            out[name] = factor if out[name] is None else torch.maximum(out[name], factor)
    return out


def close_calls(folder, prompts: dict, margin: float, share: float = 0.03) -> dict:
    """name -> a mask a position: whether some router of the model, in some run of its layer, decides this position's
    experts (or kept groups) by less than ``margin`` of choice score between candidates of which one would weigh
    more than ``share`` of the chosen.  Such a choice may fall the other way under rounding, and the position's logits
    then are another function's.  (Two experts whose scores are both next to nothing may change places freely.)"""
    config, weights = load_plain(folder)
    eps = config["norm"]["eps"]
    out = {}
    for name, tokens in prompts.items():
        streams = []
        plain.forward(config, weights, tokens, streams)
        T = len(tokens)
        first = weights["embed"][torch.as_tensor(tokens)] * (config.get("embedding") or {}).get("scale", 1.0)
        close = torch.zeros(T, dtype=torch.bool)
        before = first
        for run, (i, again) in enumerate(plain.layer_runs(config)):
            x = before + first if again else before
            mlp = config["layers"][i].get("mlp")
            if mlp is not None and mlp["kind"] == "moe":
                p = f"l{i}.mlp."
                router = mlp["router"]
                h = plain.rms(x, eps) * weights[f"l{i}.norm2"]
                plain_score = torch.softmax(h @ weights[p + "router"].T, -1)
                score = plain_score + weights[p + "correction"]
                chosen, _ = plain.route(h, weights, p, router)
                total = plain_score.gather(1, chosen).sum(-1)
                groups = router.get("groups")
                if groups and groups["keep"] < groups["count"]:
                    size = score.shape[1] // groups["count"]
                    best = score.view(T, groups["count"], size).max(-1).values
                    order = best.argsort(-1, descending=True)
                    last, nxt = order[:, groups["keep"] - 1], order[:, groups["keep"]]
                    gap = best.gather(1, last[:, None])[:, 0] - best.gather(1, nxt[:, None])[:, 0]
                    heavy = plain_score.view(T, groups["count"], size).max(-1).values
                    weighs = torch.maximum(heavy.gather(1, last[:, None])[:, 0], heavy.gather(1, nxt[:, None])[:, 0]) / total
                    close |= (gap < margin) & (weighs > share)
                    allowed = torch.zeros(T, groups["count"], dtype=torch.bool).scatter_(1, order[:, :groups["keep"]], True)
                    score = score.masked_fill(~allowed.repeat_interleave(size, 1), -math.inf)
                if router["top"] < score.shape[1]:
                    order = score.argsort(-1, descending=True)
                    last, nxt = order[:, router["top"] - 1], order[:, router["top"]]
                    gap = score.gather(1, last[:, None])[:, 0] - score.gather(1, nxt[:, None])[:, 0]
                    weighs = torch.maximum(plain_score.gather(1, last[:, None])[:, 0], plain_score.gather(1, nxt[:, None])[:, 0]) / total
                    close |= (gap < margin) & (weighs > share)
            before = streams[run]
        out[name] = close
    return out


def drawn_config(seed: int) -> dict:
    """A configuration drawn from the sizes and constants a model of the design may have: any order of layers, a looped
    stretch anywhere, head counts from 1 to 16, groups of 1 to 8, heads from 8 to 128, vectors from 16 to 224, windows and
    chunks from 3 to beyond the prompts or none, rotations over part of a head, rescaled frequencies, dense feed-forwards,
    experts with and without identity experts and groups, or none."""
    import random

    rng = random.Random(seed)
    width = rng.choice([64, 96, 128, 192, 200])

    def feed_forward():
        kind = rng.random()
        if kind < 0.2:
            return None
        if kind < 0.4:
            return dense(rng.choice([64, 200]))
        count = rng.choice([1, 2, 4])
        size = rng.choice([1, 2, 3, 4])
        total = count * size
        identity = rng.randint(0, min(total - 1, 3))
        keep = rng.randint(1, count)
        return moe(total - identity, rng.randint(1, min(keep * size, 4)), rng.choice([16, 40, 64]),
                   identity=identity if identity or rng.random() < 0.5 else None,
                   groups=(count, keep) if count > 1 or rng.random() < 0.5 else None)

    layers = []
    for _ in range(rng.randint(3, 6)):
        if rng.random() < 0.5:
            heads, dim, vdim = rng.choice([1, 2, 4, 8, 12, 16]), rng.choice([8, 16, 32, 48, 64]), rng.choice([8, 16, 32, 64])
            rank, rot = rng.choice([16, 32, 48, 64, 96, 112, 160, 192, 224]), rng.choice([2, 8, 16, 32, 64])
            layers.append(latent(heads, dim, rot, vdim, rank, (dim + rot) ** -0.5, base=rng.choice([100.0, 10000.0, 250000.0]),
                                 window=rng.choice([None, 3, 20, 64, 70, 100, 500]), mlp=feed_forward()))
        else:
            kv_heads, group = rng.choice([1, 2, 4]), rng.choice([1, 2, 4, 8])
            dim = rng.choice([16, 24, 32, 48, 64, 96, 128])
            turned = dim if rng.random() < 0.6 else rng.randrange(2, dim, 2)
            scaling = None if rng.random() < 0.5 else (rng.choice([2.0, 8.0]), 1.0, rng.choice([2.0, 4.0]), rng.choice([16, 64, 2048]))
            layers.append(attention(kv_heads * group, kv_heads, dim, rng.choice([0.5, 1.0, 2.0]) * dim ** -0.5,
                                    chunk=rng.choice([None, 3, 20, 48, 70, 100, 500]), turned=turned,
                                    base=rng.choice([100.0, 10000.0, 500000.0]), scaling=scaling, mlp=feed_forward()))
    loop = None
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        loop = (start, rng.randint(start + 1, len(layers)), rng.randint(1, 3))
    return model(width, rng.choice([101, 256, 333]), layers, eps=rng.choice([1e-6, 1e-5]),
                 scale=rng.choice([None, 1.0, 4.0, 12.0]), loop=loop)
