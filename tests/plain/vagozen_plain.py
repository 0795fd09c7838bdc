"""A plain, slow implementation of the Vagozen decoder, one function per mechanism, in float64 on the CPU.

It shares no code with the engine: it reads a model folder's config.json as a plain dict and its tensors by
name, and runs a whole sequence at once (no cache, no pages, no state slots).  The tests compare the engine
with it; `forward` also returns the residual stream after every layer run.

Notation: W x means `x @ W.T` for a weight stored [out, in]; positions count from 0; n tokens.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch

F = torch.float64


def read_folder(folder):
    from safetensors import safe_open

    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    tensors = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt", device="cpu") as source:
        for name in source.keys():
            value = source.get_tensor(name)
            tensors[name] = value.to(F) if value.dtype.is_floating_point else value
    return config, tensors


# ---------------------------------------------------------------------------- small functions


def rms_normalise(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


# ---------------------------------------------------------------------------- rotary


def plain_frequencies(dims, base):
    return [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]


def yarn_frequencies(dims, base, scaling):
    """(frequencies, what cos and sin are multiplied by).  Pair i keeps f_i where ramp_i is 0, has it divided by
    `factor` where ramp_i is 1; the ramp runs over the pair index between the pairs that make `fast` and `slow`
    turns over the original context."""
    plain = plain_frequencies(dims, base)
    if not scaling:
        return torch.tensor(plain, dtype=F), 1.0
    factor, original, fast, slow = (float(scaling[name]) for name in ("factor", "original", "fast", "slow"))

    def pair_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(pair_of(fast)), 0)
    hi = min(math.ceil(pair_of(slow)), dims - 1)
    out = []
    for i, f in enumerate(plain):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return torch.tensor(out, dtype=F), 0.1 * math.log(factor) + 1.0


def rotate(x, positions, frequencies, magnitude, layout):
    """x [n, heads, width]: the first 2 len(frequencies) dimensions of every head turn by position * frequency;
    `layout` "interleaved" pairs (2i, 2i + 1), "halves" pairs (i, i + dims / 2).  The rest passes unchanged."""
    dims = 2 * len(frequencies)
    angles = positions.to(F)[:, None] * frequencies[None, :]
    cos, sin = magnitude * angles.cos()[:, None, :], magnitude * angles.sin()[:, None, :]
    out = x.clone()
    if layout == "interleaved":
        first, second = slice(0, dims, 2), slice(1, dims, 2)
    else:
        first, second = slice(0, dims // 2), slice(dims // 2, dims)
    u, v = x[..., first], x[..., second]
    out[..., first] = u * cos - v * sin
    out[..., second] = v * cos + u * sin
    return out


# ---------------------------------------------------------------------------- mixers


def softmax_attention(q, k, v, scale, visible):
    """q [n, H, d], k [n, G, d], v [n, G, dv]; visible [n, n] bool (query row, key column)."""
    n, heads, _ = q.shape
    per = heads // k.shape[1]
    out = torch.zeros((n, heads, v.shape[-1]), dtype=F)
    for h in range(heads):
        g = h // per
        scores = (q[:, h] @ k[:, g].T) * scale
        scores = scores.masked_fill(~visible, -math.inf)
        out[:, h] = torch.softmax(scores, dim=-1) @ v[:, g]
    return out


def window_mask(n, size, keep_first):
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    seen = j <= i
    if size is not None:
        seen &= (i - j < size) | (j < keep_first)
    return seen


def attention_mixer(h, positions, m, t, prefix):
    heads, kv_heads, dim, vdim = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    n = h.shape[0]
    q = (h @ t[prefix + "q"].T + t[prefix + "q.b"]).view(n, heads, dim)
    k = (h @ t[prefix + "k"].T + t[prefix + "k.b"]).view(n, kv_heads, dim)
    v = (h @ t[prefix + "v"].T + t[prefix + "v.b"]).view(n, kv_heads, vdim)
    rot = m.get("rot")
    if rot:
        frequencies, magnitude = yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q = rotate(q, positions, frequencies, magnitude, "interleaved")
        k = rotate(k, positions, frequencies, magnitude, "interleaved")
    mask = m.get("mask")
    seen = window_mask(n, mask["size"] if mask else None, mask.get("keep_first", 0) if mask else 0)
    mixed = softmax_attention(q, k, v, m["scale"], seen)
    return mixed.reshape(n, heads * vdim) @ t[prefix + "o"].T


def retention_mixer(h, positions, m, t, prefix, eps):
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = (h @ t[prefix + "q"].T).view(n, heads, dim)
    k = (h @ t[prefix + "k"].T).view(n, heads, dim)
    v = (h @ t[prefix + "v"].T).view(n, heads, vdim)
    rot = m.get("rot")
    if rot:
        frequencies = torch.tensor(plain_frequencies(rot["dims"], rot["base"]), dtype=F)
        q = rotate(q, positions, frequencies, 1.0, "halves")
        k = rotate(k, positions, frequencies, 1.0, "halves")
    k = k * dim ** -0.5
    read = torch.zeros((n, heads, vdim), dtype=F)
    for head in range(heads):
        read[:, head] = retention_head(q[:, head], k[:, head], v[:, head], float(m["decay"][head]))
    read = rms_normalise(read, eps).reshape(n, heads * vdim)
    return (read * silu(h @ t[prefix + "g"].T)) @ t[prefix + "o"].T


def retention_head(q, k, v, decay):
    """S_t = decay S_(t-1) + k_t v_t^T from S = 0, o_t = S_t^T q_t, for one head: q, k [n, d], v [n, dv].  Short
    sequences token by token, as the recurrence is written; long ones by its closed form, o_t = sum over s <= t of
    decay^(t-s) (q_t . k_s) v_s, which is the same sum."""
    n = q.shape[0]
    if n <= 48:
        state = torch.zeros((q.shape[1], v.shape[1]), dtype=F)
        out = torch.zeros((n, v.shape[1]), dtype=F)
        for step in range(n):
            state = decay * state + torch.outer(k[step], v[step])
            out[step] = state.T @ q[step]
        return out
    distance = (torch.arange(n)[:, None] - torch.arange(n)[None, :]).clamp(min=0).to(F)
    fade = torch.tril(torch.tensor(decay, dtype=F) ** distance)
    return ((q @ k.T) * fade) @ v


def latent_mixer(h, positions, m, t, prefix, eps):
    heads, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    n = h.shape[0]
    latent_q = rms_normalise(h @ t[prefix + "dq"].T, eps) * t[prefix + "dq.norm"]
    q = (latent_q @ t[prefix + "uq"].T).view(n, heads, dim + rot_dim)
    down = h @ t[prefix + "dkv"].T
    c = rms_normalise(down[:, :rank], eps) * t[prefix + "dkv.norm"]
    shared = down[:, rank:].view(n, 1, rot_dim)
    rot = m["rot"]
    frequencies, magnitude = yarn_frequencies(rot.get("dims", rot_dim), rot["base"], rot.get("scaling"))
    q_turned = rotate(q[..., dim:], positions, frequencies, magnitude, "interleaved")
    shared = rotate(shared, positions, frequencies, magnitude, "interleaved")
    keys = (c @ t[prefix + "uk"].T).view(n, heads, dim)
    values = (c @ t[prefix + "uv"].T).view(n, heads, vdim)
    full_q = torch.cat([q[..., :dim], q_turned], dim=-1)
    full_k = torch.cat([keys, shared.expand(n, heads, rot_dim)], dim=-1)
    mixed = softmax_attention(full_q, full_k, values, m["scale"], window_mask(n, None, 0))
    return mixed.reshape(n, heads * vdim) @ t[prefix + "o"].T


# ---------------------------------------------------------------------------- feed-forwards


def limited_gate(gate, up, limit):
    g = gate.clamp(max=limit)
    u = up.clamp(-limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def dense_feed_forward(h, mlp, t, prefix):
    y = limited_gate(h @ t[prefix + "gate"].T, h @ t[prefix + "up"].T, mlp["limit"])
    return y @ t[prefix + "down"].T


def expert_feed_forward(h, mlp, t, prefix):
    router, limit = mlp["router"], mlp["expert"]["limit"]
    logits = h @ t[prefix + "router"].T + t[prefix + "router.b"]
    best, chosen = torch.topk(logits, router["top"], dim=-1)
    weights = torch.softmax(best, dim=-1)
    out = torch.zeros_like(h)
    for expert in range(router["experts"]):
        name = f"{prefix}e{expert}."
        share = (weights * (chosen == expert)).sum(-1, keepdim=True)  # the token's weight for this expert, 0 if it is not chosen
        y = limited_gate(h @ t[name + "gate"].T, h @ t[name + "up"].T, limit)
        out += share * (y @ t[name + "down"].T)
    return out


# ---------------------------------------------------------------------------- the model


def run_order(config):
    """[(layer, number of the pass it begins or None)]"""
    count = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(index, None) for index in range(count)]
    order = [(index, None) for index in range(loop["start"])]
    for number in range(loop["times"]):
        order += [(index, number if index == loop["start"] else None) for index in range(loop["start"], loop["stop"])]
    return order + [(index, None) for index in range(loop["stop"], count)]


def forward(config, t, tokens):
    """(logits [n, vocab], the stream after every layer run [runs, n, width])."""
    eps = config["norm"]["eps"]
    positions = torch.arange(len(tokens))
    x = t["embed"][torch.tensor(tokens)]
    embedded = x.clone()
    streams = []

    def norm(values, name):
        return rms_normalise(values, eps) * t[name]

    for index, begins in run_order(config):
        if begins is not None:
            if begins > 0:
                x = x + embedded
            x = x + t["loop.step"][begins]
        layer, prefix = config["layers"][index], f"l{index}."
        h = norm(x, prefix + "norm1")
        if layer["type"] == "attention":
            mixed = attention_mixer(h, positions, layer["mixer"], t, prefix + "mix.")
        elif layer["type"] == "retention":
            mixed = retention_mixer(h, positions, layer["mixer"], t, prefix + "mix.", eps)
        else:
            mixed = latent_mixer(h, positions, layer["mixer"], t, prefix + "mix.", eps)
        x = x + norm(mixed, prefix + "norm1b") * t[prefix + "ls1"]
        mlp = layer.get("mlp")
        if mlp:
            h = norm(x, prefix + "norm2")
            fed = dense_feed_forward(h, mlp, t, prefix + "mlp.") if mlp["kind"] == "dense" else expert_feed_forward(h, mlp, t, prefix + "mlp.")
            x = x + norm(fed, prefix + "norm2b") * t[prefix + "ls2"]
        streams.append(x.clone())
    logits = (norm(x, "final.norm") @ t["embed"].T) * config.get("logit_scale", 1.0)
    return logits, torch.stack(streams)
