"""A plain, slow implementation of the Dimalix design: whole sequences, no cache, no batches, one
function a mechanism, 64-bit arithmetic.  It shares no code with the package; the tests hold the
engine against it.

``config`` is the dict of a config.json; ``w`` maps tensor names to 64-bit tensors.

The embedding is scaled.  A layer is parallel: with a = norm1(x) and b = norm2(x) of the same x,
x <- x + ls1 * mixer(a) + ls2 * ff(b), ls1 and ls2 a gain a column.  Two mixers: ``attention`` (grouped
heads, biases on q and k, the values are the keys as projected, one norm over all heads of q and one over
all heads of k, neighbour rotation of the first values of a head with frequencies that may be rescaled,
keys seen inside the query's own chunk of positions) and ``latent_attention`` (keys and values rebuilt
from one small normed vector a token, a rotated key part shared by the heads, a sliding window).
Feed-forwards: dense with the tanh gelu, or routed experts: softmax scores, a correction added for the
choice alone, groups of neighbouring experts of which only the best may be chosen from, identity experts
at the end, weights renormalised over the chosen.  A stretch of the layers may run several times in a row,
each further pass starting from x plus the embedding output.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def frequencies(rot) -> list:
    """f_i = base^(-2i/dims); with ``scaling`` the long wavelengths are stretched by ``factor``, the short ones
    kept, and those between blended by where original/wavelength lies between ``low`` and ``high``."""
    dims, base = rot["dims"], rot["base"]
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        s = rot.get("scaling")
        if s:
            length = 2.0 * math.pi / f
            if length > s["original"] / s["low"]:
                f = f / s["factor"]
            elif length >= s["original"] / s["high"]:
                blend = (s["original"] / length - s["low"]) / (s["high"] - s["low"])
                f = (1.0 - blend) * f / s["factor"] + blend * f
        out.append(f)
    return out


def rotate_neighbours(x, positions, rot):
    """x [T, ..., n]: of the first ``dims`` values, value 2i turns with value 2i + 1 by position * f_i."""
    dims = rot["dims"]
    angle = positions.to(F)[:, None] * torch.tensor(frequencies(rot), dtype=F)[None, :]
    while angle.dim() < x.dim():
        angle = angle.unsqueeze(1)
    cos, sin = angle.cos(), angle.sin()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * cos - v * sin, v * cos + u * sin], -1).flatten(-2)
    return torch.cat([turned, x[..., dims:]], -1)


def window_mask(positions, size):
    """[i, j]: 0 <= i - j < size."""
    distance = positions[:, None] - positions[None, :]
    return (distance >= 0) & (distance < size)


def chunk_mask(positions, size):
    """[i, j]: j <= i and both in the same chunk of ``size`` positions counted from position 0."""
    same = (positions[:, None] // size) == (positions[None, :] // size)
    return same & (positions[:, None] >= positions[None, :])


def causal_mask(positions):
    return positions[:, None] >= positions[None, :]


def softmax_over(score, visible):
    score = score.masked_fill(~visible, -math.inf)
    e = torch.exp(score - score.max(-1, keepdim=True).values)
    return e / e.sum(-1, keepdim=True)


def attention_mixer(h, w, p, m, eps, positions):
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q_raw = h @ w[p + "q"].T + w[p + "q.b"]
    k_raw = h @ w[p + "k"].T + w[p + "k.b"]
    v = k_raw.view(T, G, D)                                   # the values are the keys as projected
    q = rotate_neighbours((rms(q_raw, eps) * w[p + "q.norm"]).view(T, H, D), positions, m["rot"])
    k = rotate_neighbours((rms(k_raw, eps) * w[p + "k.norm"]).view(T, G, D), positions, m["rot"])
    visible = chunk_mask(positions, m["mask"]["size"]) if m.get("mask") else causal_mask(positions)
    each = H // G
    out = torch.zeros(T, H, D, dtype=F)
    for head in range(H):
        score = (q[:, head] @ k[:, head // each].T) * m["scale"]
        out[:, head] = softmax_over(score, visible) @ v[:, head // each]
    return out.reshape(T, H * D) @ w[p + "o"].T


def latent_attention_mixer(h, w, p, m, eps, positions):
    T = h.shape[0]
    H, D, rot, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    both = h @ w[p + "dkv"].T
    c = rms(both[:, :R], eps) * w[p + "dkv.norm"]
    k_rot = rotate_neighbours(both[:, R:R + rot], positions, m["rot"])
    q = (h @ w[p + "q"].T).view(T, H, D + rot)
    q_plain = q[..., :D]
    q_rot = rotate_neighbours(q[..., D:], positions, m["rot"])
    k_plain = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, V)
    visible = window_mask(positions, m["mask"]["size"]) if m.get("mask") else causal_mask(positions)
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        score = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * m["scale"]
        out[:, head] = softmax_over(score, visible) @ v[:, head]
    return out.reshape(T, H * V) @ w[p + "o"].T


def dense_feed_forward(h, w, p):
    return gelu_tanh(h @ w[p + "up"].T) @ w[p + "down"].T


def expert(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w, p, router):
    """(chosen [T, top], weights [T, top]).  Outputs 0 .. experts - 1 of the router are experts, the ``identity``
    behind them identity experts; all of them are scored, grouped and chosen alike."""
    total = router["experts"] + router.get("identity", 0)
    score = torch.softmax(h @ w[p + "router"].T, -1)
    choice = score + w[p + "correction"]
    groups = router.get("groups")
    if groups:
        size = total // groups["count"]
        best = choice.view(-1, groups["count"], size).max(-1).values
        kept = best.topk(groups["keep"], -1).indices
        allowed = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(size, 1), -math.inf)
    chosen = choice.topk(router["top"], -1).indices
    weight = score.gather(1, chosen)
    return chosen, weight / (weight.sum(-1, keepdim=True) + 1e-20)


def routed_experts(h, w, p, mlp):
    router = mlp["router"]
    chosen, weight = route(h, w, p, router)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t].tolist(), weight[t]):
            out[t] += g * (h[t] if e >= router["experts"] else expert(h[t:t + 1], w, f"{p}e{e}.")[0])
    return out


def feed_forward(h, w, p, mlp):
    if mlp["kind"] == "dense":
        return dense_feed_forward(h, w, p)
    if mlp["kind"] == "moe":
        return routed_experts(h, w, p, mlp)
    raise ValueError(f"a feed-forward of kind {mlp['kind']!r}")


def mixer(layer, h, w, p, eps, positions):
    if layer["type"] == "attention":
        return attention_mixer(h, w, p, layer["mixer"], eps, positions)
    if layer["type"] == "latent_attention":
        return latent_attention_mixer(h, w, p, layer["mixer"], eps, positions)
    raise ValueError(f"a mixer of type {layer['type']!r}")


def layer_runs(config) -> list:
    """(layer, whether the embedding output joins the stream right before it) in the order the layers run."""
    count = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(count)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(start)]
    for again in range(times):
        runs += [(i, again > 0 and i == start) for i in range(start, stop)]
    return runs + [(i, False) for i in range(stop, count)]


def forward(config, w, tokens, streams=None):
    """Logits [T, vocab] of one whole sequence.  ``streams``: a list that receives the stream after every run of a layer."""
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    first = w["embed"][tokens] * (config.get("embedding") or {}).get("scale", 1.0)
    x = first.clone()
    for i, again in layer_runs(config):
        layer = config["layers"][i]
        p = f"l{i}."
        if again:
            x = x + first
        y = w[p + "ls1"] * mixer(layer, rms(x, eps) * w[p + "norm1"], w, p + "mix.", eps, positions)
        if layer.get("mlp") is not None:
            y = y + w[p + "ls2"] * feed_forward(rms(x, eps) * w[p + "norm2"], w, p + "mlp.", layer["mlp"])
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    return (rms(x, eps) * w["final.norm"]) @ w["head"].T
