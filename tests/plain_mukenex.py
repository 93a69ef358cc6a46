"""A plain, slow implementation of the Mukenex design: whole sequences, no cache, no batches, one
function a mechanism, 64-bit arithmetic.  It shares no code with the package; the tests hold the
engine against it.

``config`` is the dict of a config.json; ``w`` maps tensor names to 64-bit tensors (integer tables stay
integers).

The model keeps ``streams`` copies of the residual stream.  A sublayer reads a weighted sum of the
copies through a norm whose gain is stored around zero, and every copy is then rebuilt from all copies
and the sublayer's output.  Three mixers: ``latent_attention`` (keys and values rebuilt from one small
vector a token, a rotated key part shared by the heads, a window, a learned sink a head, a gate an
element), ``attention`` (grouped heads with biases and a norm a head on q and k, no positions, keys
seen inside the query's own block of positions only), ``lightning`` (a matrix of state a head with a
fixed decay).  Feed-forwards: dense with the erf gelu, or experts chosen by a table over token ids.
A stretch of the layers may run several times in a row.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, gain, eps):
    """The layers' norm: the stored gain is the distance from one."""
    return rms(x, eps) * (1.0 + gain)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate_neighbours(x, positions, dims, base):
    """x [T, ..., n]: of the first ``dims`` values, value 2i turns with value 2i + 1 by position * base^(-2i/dims)."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    angle = positions.to(F)[:, None] * freq[None, :]
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


def block_mask(positions, size):
    """[i, j]: j <= i and both in the same block of ``size`` positions counted from position 0."""
    same = (positions[:, None] // size) == (positions[None, :] // size)
    return same & (positions[:, None] >= positions[None, :])


def softmax_with_sink(score, visible, sink=None):
    """Weights exp(s_j) / (exp(sink) + sum over the visible j of exp(s_j)); without a sink the ordinary softmax."""
    score = score.masked_fill(~visible, -math.inf)
    top = score.max(-1, keepdim=True).values
    if sink is not None:
        sink = torch.as_tensor(sink, dtype=F)
        top = torch.clamp(top, min=float(sink))
    e = torch.exp(score - top)
    total = e.sum(-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink - top)
    return e / total


def latent_attention_mixer(h, w, p, m, eps, positions):
    T = h.shape[0]
    H, D, rot, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    dims, base = m["rot"]["dims"], m["rot"]["base"]
    both = h @ w[p + "dkv"].T
    c = rms(both[:, :R], eps) * w[p + "dkv.norm"]
    k_rot = rotate_neighbours(both[:, R:R + rot], positions, dims, base)
    q = (h @ w[p + "q"].T).view(T, H, D + rot)
    q_plain = q[..., :D]
    q_rot = rotate_neighbours(q[..., D:], positions, dims, base)
    k_plain = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, V)
    visible = window_mask(positions, m["mask"]["size"]) if m.get("mask") else window_mask(positions, 1 << 60)
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        score = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * m["scale"]
        out[:, head] = softmax_with_sink(score, visible, w[p + "sink"][head]) @ v[:, head]
    gated = out.reshape(T, H * V) * torch.sigmoid(h @ w[p + "g"].T)
    return gated @ w[p + "o"].T


def block_attention_mixer(h, w, p, m, eps, positions):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms((h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, D), eps) * w[p + "q.norm"]
    k = rms((h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, D), eps) * w[p + "k.norm"]
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, V)
    visible = block_mask(positions, m["mask"]["size"]) if m.get("mask") else window_mask(positions, 1 << 60)
    each = H // G
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        score = (q[:, head] @ k[:, head // each].T) * m["scale"]
        out[:, head] = softmax_with_sink(score, visible) @ v[:, head // each]
    return out.reshape(T, H * V) @ w[p + "o"].T


def lightning_mixer(h, w, p, m, eps):
    """S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, token by token."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).view(T, H, D)
    k = silu(h @ w[p + "k"].T).view(T, H, D)
    v = silu(h @ w[p + "v"].T).view(T, H, V)
    decay = torch.tensor(m["decay"], dtype=F)
    state = torch.zeros(H, D, V, dtype=F)
    read = torch.zeros(T, H, V, dtype=F)
    for t in range(T):
        state = decay[:, None, None] * state + k[t][:, :, None] * v[t][:, None, :]
        read[t] = torch.einsum("hdv,hd->hv", state, q[t])
    normed = rms(read.reshape(T, H * V), eps) * w[p + "norm"]
    return (normed * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def dense_feed_forward(h, w, p):
    return gelu_erf(h @ w[p + "up"].T) @ w[p + "down"].T


def expert(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def table_experts(h, w, p, tokens):
    """Every token's experts are the row of the table that its id names; each counts 1/top."""
    table = w[p + "table"]
    top = table.shape[1]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in table[int(tokens[t])].tolist():
            out[t] += expert(h[t:t + 1], w, f"{p}e{int(e)}.")[0] / top
    return out


def feed_forward(h, w, p, mlp, tokens):
    if mlp["kind"] == "dense":
        return dense_feed_forward(h, w, p)
    if mlp["kind"] == "moe":
        return table_experts(h, w, p, tokens)
    raise ValueError(f"a feed-forward of kind {mlp['kind']!r}")


def mixer(layer, h, w, p, eps, positions):
    m = layer["mixer"]
    if layer["type"] == "latent_attention":
        return latent_attention_mixer(h, w, p, m, eps, positions)
    if layer["type"] == "attention":
        return block_attention_mixer(h, w, p, m, eps, positions)
    if layer["type"] == "lightning":
        return lightning_mixer(h, w, p, m, eps)
    raise ValueError(f"a mixer of type {layer['type']!r}")


def sublayer_over_copies(copies, w, p, fn):
    """copies [S, T, W]: the sublayer reads sum_s in[s] x_s; copy t becomes sum_s mix[s, t] x_s + out[t] y."""
    u = torch.einsum("s,stw->tw", w[p + "in"], copies)
    y = fn(u)
    return torch.einsum("sr,stw->rtw", w[p + "mix"], copies) + w[p + "out"][:, None, None] * y[None]


def layer_order(config) -> list:
    """The layers in the order they run: a stretch may run several times in a row."""
    count = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(count))
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    return list(range(start)) + list(range(start, stop)) * times + list(range(stop, count))


def forward(config, w, tokens, streams=None):
    """Logits [T, vocab] of one whole sequence.  ``streams``: a list that receives the stream (the sum of its
    copies) after every run of a layer."""
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    x = w["embed"][tokens]
    copies = config.get("streams")
    if copies is not None:
        x = x[None].repeat(copies, 1, 1)
    for i in layer_order(config):
        layer = config["layers"][i]
        p = f"l{i}."
        first = lambda u: mixer(layer, norm_around_zero(u, w[p + "norm1"], eps), w, p + "mix.", eps, positions)
        second = lambda u: feed_forward(norm_around_zero(u, w[p + "norm2"], eps), w, p + "mlp.", layer["mlp"], tokens)
        if copies is not None:
            x = sublayer_over_copies(x, w, p + "hc1.", first)
            if layer.get("mlp") is not None:
                x = sublayer_over_copies(x, w, p + "hc2.", second)
        else:
            x = x + first(x)
            if layer.get("mlp") is not None:
                x = x + second(x)
        if streams is not None:
            streams.append((x.sum(0) if copies is not None else x).clone())
    if copies is not None:
        x = x.sum(0)
    logits = norm_around_zero(x, w["final.norm"], eps) @ w["head"].T
    cap = config.get("logit_softcap")
    if cap is not None:
        logits = cap * torch.tanh(logits / cap)
    return logits
