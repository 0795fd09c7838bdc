"""A plain implementation of the Katenex decoder for the tests: float64, whole sequences, no cache, no batching,
one function per mechanism.  `config` is config.json as a plain mapping, `tensors` maps a tensor's name in the
model folder to a float64 tensor.  Nothing here is shared with the engine."""

from __future__ import annotations

import math

import torch


def rms_norm(x, weight, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def short_convolution(x, taps, bias=None):
    """x [T, C], taps [C, K] (the last column is the current token's); zeros before the sequence starts."""
    tokens, width = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros((width - 1, x.shape[1]), dtype=x.dtype), x])
    out = torch.zeros_like(x)
    for j in range(width):
        out += padded[j : j + tokens] * taps[:, j]
    return out if bias is None else out + bias


def rotate_half_pairs(x, positions, dims, base, factor):
    """x [T, heads, dim]: dimension i of the first `dims` turns with dimension i + dims / 2 by position * base^(-2i/dims) / factor."""
    half = dims // 2
    frequencies = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=torch.float64)
    angles = positions.to(torch.float64)[:, None] * frequencies[None, :]
    cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = a * cos - b * sin
    out[..., half:dims] = b * cos + a * sin
    return out


def softmax_attention(h, tensors, prefix, spec):
    tokens = h.shape[0]
    heads, kv_heads, dim, vdim = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    q = (h @ tensors[prefix + "q"].T).view(tokens, heads, dim)
    k = (h @ tensors[prefix + "k"].T).view(tokens, kv_heads, dim)
    v = (h @ tensors[prefix + "v"].T).view(tokens, kv_heads, vdim)
    rot = spec.get("rot")
    if rot:
        factor = (rot.get("scaling") or {}).get("factor", 1.0)
        positions = torch.arange(tokens)
        q = rotate_half_pairs(q, positions, rot["dims"], rot["base"], factor)
        k = rotate_half_pairs(k, positions, rot["dims"], rot["base"], factor)
    out = torch.zeros((tokens, heads, vdim), dtype=torch.float64)
    group = heads // kv_heads
    for head in range(heads):
        scores = (q[:, head] @ k[:, head // group].T) * spec["scale"]
        visible = torch.tril(torch.ones((tokens, tokens), dtype=torch.bool))
        scores = scores.masked_fill(~visible, -math.inf)
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, head // group]
    return out.reshape(tokens, heads * vdim) @ tensors[prefix + "o"].T


def gated_linear_recurrence(h, tensors, prefix, spec):
    """Two branches of `width`: a gelu branch, and a convolved branch that drives a diagonal recurrence whose decay
    and input gate come from block-diagonal products of the convolved branch itself."""
    tokens, width, blocks = h.shape[0], spec["width"], spec["blocks"]
    y = gelu_tanh(h @ tensors[prefix + "y"].T + tensors[prefix + "y.b"])
    u = short_convolution(h @ tensors[prefix + "x"].T + tensors[prefix + "x.b"], tensors[prefix + "conv"], tensors[prefix + "conv.b"])
    part = width // blocks
    split = u.view(tokens, blocks, part)
    r = torch.sigmoid(torch.einsum("bop,tbp->tbo", tensors[prefix + "ra"], split) + tensors[prefix + "ra.b"]).reshape(tokens, width)
    i = torch.sigmoid(torch.einsum("bop,tbp->tbo", tensors[prefix + "ri"], split) + tensors[prefix + "ri.b"]).reshape(tokens, width)
    log_a = -8.0 * r * softplus(tensors[prefix + "lam"])
    a = torch.exp(log_a)
    state = torch.zeros(width, dtype=torch.float64)
    read = torch.zeros((tokens, width), dtype=torch.float64)
    for t in range(tokens):
        state = a[t] * state + torch.sqrt(1.0 - a[t] ** 2) * i[t] * u[t]
        read[t] = state
    return (read * y) @ tensors[prefix + "o"].T


def parallel_mixer(h, tensors, prefix, spec):
    left = softmax_attention(h, tensors, prefix + "left.", spec["left"])
    right = gated_linear_recurrence(h, tensors, prefix + "right.", spec["right"])
    return spec["left_scale"] * left + spec["right_scale"] * right


def channel_delta(h, tensors, prefix, spec, eps):
    """The gated delta rule with a decay for every key channel of every head."""
    tokens = h.shape[0]
    heads, kv_heads, dim, vdim = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    q = silu(short_convolution(h @ tensors[prefix + "q"].T, tensors[prefix + "q.conv"])).view(tokens, kv_heads, dim)
    k = silu(short_convolution(h @ tensors[prefix + "k"].T, tensors[prefix + "k.conv"])).view(tokens, kv_heads, dim)
    v = silu(short_convolution(h @ tensors[prefix + "v"].T, tensors[prefix + "v.conv"])).view(tokens, heads, vdim)
    q = q / torch.sqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim**-0.5
    k = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ tensors[prefix + "b"].T)  # [T, heads]
    step = softplus((h @ tensors[prefix + "a1"].T) @ tensors[prefix + "a2"].T + tensors[prefix + "dt_bias"]).view(tokens, heads, dim)
    decay = torch.exp(-torch.exp(tensors[prefix + "A_log"])[None, :, None] * step)  # [T, heads, dim]
    group = heads // kv_heads
    read = torch.zeros((tokens, heads, vdim), dtype=torch.float64)
    for head in range(heads):
        S = torch.zeros((dim, vdim), dtype=torch.float64)
        for t in range(tokens):
            kt, qt = k[t, head // group], q[t, head // group]
            S = decay[t, head][:, None] * S
            u = beta[t, head] * (v[t, head] - S.T @ kt)
            S = S + torch.outer(kt, u)
            read[t, head] = S.T @ qt
    normed = read / torch.sqrt(read.pow(2).mean(-1, keepdim=True) + eps) * tensors[prefix + "norm"]
    gate = torch.sigmoid((h @ tensors[prefix + "g1"].T) @ tensors[prefix + "g2"].T).view(tokens, heads, vdim)
    return (normed * gate).reshape(tokens, heads * vdim) @ tensors[prefix + "o"].T


def gated_expert(h, tensors, prefix):
    return (silu(h @ tensors[prefix + "gate"].T) * (h @ tensors[prefix + "up"].T)) @ tensors[prefix + "down"].T


def choose_experts(scores, top, groups, keep):
    """scores [E] -> the indices of the `top` largest among the experts of the `keep` best of `groups` equal groups of
    neighbours (a group's score is its largest)."""
    experts = scores.shape[0]
    allowed = torch.ones(experts, dtype=torch.bool)
    if groups > 1:
        size = experts // groups
        best = scores.view(groups, size).max(-1).values
        kept = torch.sort(best, descending=True, stable=True).indices[:keep]
        allowed = torch.zeros(groups, dtype=torch.bool)
        allowed[kept] = True
        allowed = allowed.repeat_interleave(size)
    masked = torch.where(allowed, scores, torch.full_like(scores, -math.inf))
    return torch.sort(masked, descending=True, stable=True).indices[:top]


def mixture_of_experts(h, tensors, prefix, spec):
    router = spec["router"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    out = torch.zeros((h.shape[0], tensors[prefix + "e0.down"].shape[0]), dtype=torch.float64)
    scores = torch.softmax(h @ tensors[prefix + "router"].T, dim=-1)
    for t in range(h.shape[0]):
        chosen = choose_experts(scores[t], router["top"], groups["count"], groups["keep"])
        weights = scores[t][chosen] / (scores[t][chosen].sum() + 1e-20) * router["scale"]
        for weight, expert in zip(weights, chosen):
            out[t] += weight * gated_expert(h[t], tensors, f"{prefix}e{int(expert)}.")
    if spec.get("shared"):
        out += gated_expert(h, tensors, prefix + "shared.")
    return out


def mixer_of(layer, h, tensors, prefix, eps):
    if layer["type"] == "parallel":
        return parallel_mixer(h, tensors, prefix, layer["mixer"])
    if layer["type"] == "channel_delta":
        return channel_delta(h, tensors, prefix, layer["mixer"], eps)
    raise ValueError(layer["type"])


def forward(config, tensors, tokens):
    """-> (logits [T, vocab], the sum of the streams after every layer [layers, T, width])."""
    eps = config["norm"]["eps"]
    x = tensors["embed"][torch.as_tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    streams = [x.clone() for _ in range(config.get("streams") or 1)]
    count = len(streams)
    after = []

    def sublayer(name, norm, run):
        nonlocal streams
        if config.get("streams") is None:  # one stream and the plain residual sum: x <- x + sublayer(norm(x))
            streams = [streams[0] + run(rms_norm(streams[0], tensors[norm], eps))]
            return
        read, write, mix = tensors[name + ".in"], tensors[name + ".out"], tensors[name + ".mix"]
        u = sum(read[s] * streams[s] for s in range(count))
        y = run(rms_norm(u, tensors[norm], eps))
        streams = [sum(mix[s, t] * streams[s] for s in range(count)) + write[t] * y for t in range(count)]

    for index, layer in enumerate(config["layers"]):
        prefix = f"l{index}."
        sublayer(prefix + "hc1", prefix + "norm1", lambda h: mixer_of(layer, h, tensors, prefix + "mix.", eps))
        if layer.get("mlp") is not None:
            sublayer(prefix + "hc2", prefix + "norm2", lambda h: mixture_of_experts(h, tensors, prefix + "mlp.", layer["mlp"]))
        after.append(sum(streams))
    final = rms_norm(sum(streams), tensors["final.norm"], eps)
    return final @ tensors["head"].T, torch.stack(after)
