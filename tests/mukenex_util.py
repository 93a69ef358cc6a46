"""Configurations, model folders and comparisons for the tests of the Mukenex design."""

from __future__ import annotations

import copy
import json
from pathlib import Path

import torch

import plain_mukenex as plain


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, turned=None, window=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"dims": rot_dim if turned is None else turned, "base": base}}
    if window is not None:
        m["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def attention(heads, kv_heads, dim, vdim, scale, block=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if block is not None:
        m["mask"] = {"size": block}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def lightning(heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def model(width, vocab, layers, eps=1e-6, streams=None, loop=None, softcap=None):
    config = {"architecture": "Mukenex", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if streams is not None:
        config["streams"] = streams
    if loop is not None:
        config["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    if softcap is not None:
        config["logit_softcap"] = softcap
    return config


# Odd sizes: four copies of the stream, a stretch of three layers that runs three times (a layer with state and layers of
# both kinds of pages in it), head parts of 24 and 8 with a vector of 40 (rows of 48 in pages of bfloat16), value heads
# larger than key heads, three query heads a key head, blocks of 5 and 37 positions and windows of 9 and 37 (inside a
# page, across page borders), five experts of which two and four of which three, a layer without a feed-forward.
ODD = model(72, 211, [
    lightning(3, 24, 40, (0.6, 0.9, 0.999), mlp=dense(100)),
    latent(3, 24, 8, 40, 40, 0.21, base=500.0, window=37, mlp=moe(5, 2, 24)),
    attention(6, 2, 24, 40, 0.3, block=5, mlp=moe(4, 3, 40)),
    lightning(2, 40, 24, (0.95, 0.7)),
    latent(5, 16, 8, 24, 40, 0.3, base=500.0, window=9, mlp=dense(96)),
    attention(3, 3, 40, 24, 0.2, block=37, mlp=moe(6, 2, 16)),
], eps=1e-5, streams=4, loop=(1, 4, 3), softcap=20.0)

# What a small model tends to make equal or 1 is different here: one copy of the stream (with its weights), one head, one
# expert of one, one of three, a stretch that "loops" once, a window and a block of one position, a rotated part of two
# values, a scale of one, a width that is no multiple of eight, no soft cap.
ONES = model(100, 97, [
    attention(4, 1, 16, 16, 1.0, block=1, mlp=moe(1, 1, 48)),
    latent(1, 48, 2, 48, 30, 1.0, base=50.0, window=1),
    lightning(1, 16, 16, (0.9,), mlp=moe(3, 1, 24)),
    latent(2, 16, 16, 16, 30, 0.25, base=50.0, turned=8, mlp=dense(40)),
    attention(1, 1, 64, 16, 0.5, mlp=dense(32)),
], eps=1e-6, streams=1, loop=(2, 4, 1))

# Without copies, loop and soft cap (the keys are absent), without masks; larger sizes: pages' rows of 256 (a vector of 192
# with a rotated part of 64), heads of 128, sixteen query heads a key head, state heads of 128 by 64, blocks of 64.
PLAIN = model(256, 300, [
    latent(8, 64, 64, 64, 192, 0.09, base=10000.0, mlp=moe(8, 2, 64)),
    attention(16, 1, 128, 128, 0.1, mlp=dense(320)),
    lightning(2, 128, 64, (0.97, 0.999), mlp=moe(4, 2, 128)),
    attention(4, 2, 64, 128, 0.15, block=64, mlp=moe(8, 4, 32)),
    latent(2, 128, 64, 128, 192, 0.07, base=10000.0, window=64, mlp=dense(256)),
], eps=1e-6)

# Rows of the pages beyond what the matrix-core kernels take (a vector of 272 with a rotated part of 16), head sizes that
# are no multiple of 4 (30, 22) or of 8 (20, 36), a rotation over 10 of 12 values, a width that is a multiple of 4 only,
# five copies, experts whose width is no multiple of 8, a looped stretch that is the whole model.
UNEVEN = model(52, 75, [
    latent(2, 20, 16, 36, 272, 0.2, base=123.0, window=100, mlp=moe(3, 2, 44)),
    attention(3, 1, 30, 22, 0.3, block=50, mlp=dense(44)),
    lightning(2, 20, 36, (0.8, 0.99), mlp=moe(2, 2, 12)),
    latent(3, 22, 12, 30, 50, 0.21, base=123.0, turned=10, window=3),
], eps=3e-6, streams=5, loop=(0, 4, 2), softcap=7.5)

CONFIGS = {"odd": ODD, "ones": ONES, "plain": PLAIN, "uneven": UNEVEN}


def write_model(folder, config, seed=0, dtype="float32", std=0.08, gain_std=0.2, edit=None) -> Path:
    """A model folder with random weights from the package's random-weights mode; ``edit(tensors)`` may change
    them (the folder is then written again)."""
    from paged_llm_rs_amd.weights import write_random_model

    folder = write_random_model(Path(folder), copy.deepcopy(config), seed=seed, std=std, gain_std=gain_std, dtype=dtype)
    if edit is not None:
        from safetensors.torch import load_file, save_file

        tensors = load_file(str(folder / "model.safetensors"))
        edit(tensors)
        save_file({k: v.contiguous() for k, v in tensors.items()}, str(folder / "model.safetensors"))
    return folder


def wide_sinks(tensors) -> None:
    """Sinks as drawn are near zero; spread them so that a sink left out, scaled or counted twice shows.  Biases too are
    drawn small: make them as large as what they are added to."""
    for name in tensors:
        if name.endswith(".sink"):
            heads = tensors[name].shape[0]
            tensors[name] = torch.linspace(-1.5, 2.5, heads).to(tensors[name].dtype)
        elif name.endswith(".b"):
            tensors[name] = (tensors[name].float() * 6).to(tensors[name].dtype)


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
    every weight matrix is disturbed by 2^-9 of itself (root mean square over the vocabulary).  Random models have single
    positions where rounding is amplified many times (a score near a tie under a sharp softmax); a bound on an engine's
    error there has to grow with it, as the error that rounding alone causes does."""
    config, weights = load_plain(folder)
    g = torch.Generator().manual_seed(1234)
    shaken = {k: v * (1 + (torch.rand(v.shape, generator=g, dtype=v.dtype) - 0.5) * 2.0 ** -8)
              if v.dim() == 2 and v.is_floating_point() and ".hc" not in k else v for k, v in weights.items()}
    out = {}
    for name, tokens in prompts.items():
        base = plain.forward(config, weights, tokens)
        moved = ((plain.forward(config, shaken, tokens) - base) ** 2).mean(-1).sqrt() / base.std()
        out[name] = torch.clamp(moved / (2 * moved.median()), min=1.0)
    return out


def drawn_config(seed: int) -> dict:
    """A configuration drawn from the sizes and constants a model of the design may have: any order of layers, with and
    without copies of the stream, a looped stretch anywhere, head counts from 1 to 16, groups of 1 to 8, head parts from 8
    to 128, vectors from 16 to 224, windows and blocks from 3 to beyond the prompts or none, dense feed-forwards, experts
    or none, with and without a soft cap."""
    import random

    rng = random.Random(seed)
    width = rng.choice([64, 96, 128, 192, 200])

    def feed_forward():
        kind = rng.random()
        if kind < 0.25:
            return None
        if kind < 0.5:
            return dense(rng.choice([64, 200]))
        experts = rng.choice([2, 4, 8, 16])
        return moe(experts, rng.randint(1, min(experts, 4)), rng.choice([16, 40, 64]))

    layers = []
    for _ in range(rng.randint(3, 6)):
        kind = rng.random()
        if kind < 0.35:
            heads, dim, vdim = rng.choice([1, 2, 4, 8, 12, 16]), rng.choice([8, 16, 32, 48, 64]), rng.choice([8, 16, 32, 64])
            rank, rot = rng.choice([16, 32, 48, 64, 96, 112, 160, 192, 224]), rng.choice([2, 8, 16, 32, 64])
            turned = rot if rng.random() < 0.8 else max(2, rot // 2 // 2 * 2)
            layers.append(latent(heads, dim, rot, vdim, rank, (dim + rot) ** -0.5, base=rng.choice([100.0, 10000.0, 250000.0]),
                                 turned=turned, window=rng.choice([None, 3, 20, 64, 70, 100, 500]), mlp=feed_forward()))
        elif kind < 0.7:
            kv_heads, group = rng.choice([1, 2, 4]), rng.choice([1, 2, 4, 8])
            dim, vdim = rng.choice([16, 32, 48, 64, 96, 128]), rng.choice([16, 32, 48, 64, 96, 128])
            layers.append(attention(kv_heads * group, kv_heads, dim, vdim, rng.choice([0.5, 1.0, 2.0]) * dim ** -0.5,
                                    block=rng.choice([None, 3, 20, 48, 70, 100, 500]), mlp=feed_forward()))
        else:
            heads = rng.choice([1, 2, 4, 6])
            layers.append(lightning(heads, rng.choice([8, 16, 32, 64]), rng.choice([8, 16, 32, 64]),
                                    [rng.choice([0.5, 0.9, 0.97, 0.999]) for _ in range(heads)], mlp=feed_forward()))
    loop = None
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        loop = (start, rng.randint(start, len(layers)), rng.randint(1, 3))
    return model(width, rng.choice([101, 256, 333]), layers, eps=rng.choice([1e-6, 1e-5]),
                 streams=rng.choice([None, 1, 2, 3, 4]), loop=loop, softcap=rng.choice([None, 10.0, 30.0]))
