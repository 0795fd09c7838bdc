"""A stand-in for the HIP kernel library, in elementary torch on the CPU.

It exists only so that the tests which need no GPU can run the engine's parts,
cache manager, step function, scheduler and entry points here; the product
never selects it.  It rounds to the run dtype at the same places as the HIP
kernels (activations between operations), and computes everything in float32.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch


@dataclass
class _Linear:
    weight: torch.Tensor  # [N, K] float32
    bias: torch.Tensor | None


def _limited_swish(gate, up, limit):
    g = gate.clamp(max=limit)
    return g * torch.sigmoid(1.702 * g) * (up.clamp(-limit, limit) + 1.0)


class TorchKernels:
    def __init__(self, dtype: torch.dtype = torch.float32) -> None:
        self.device = torch.device("cpu")
        self.dtype = dtype
        self.calls: list[str] = []

    def to_device(self, tensor):
        return tensor

    def queued_to_device(self, tensor):
        return tensor

    def embedding(self, table, token_ids):
        return table[token_ids.long()].float()

    def add_rms_norm(self, hidden, delta, weight, eps):
        if delta is not None:
            hidden += delta if delta.ndim == 2 else delta.sum(0)
        variance = hidden.pow(2).mean(-1, keepdim=True)
        return (hidden * torch.rsqrt(variance + eps) * weight.float()).to(self.dtype)

    def prepare_linear(self, weights, biases):
        weight = torch.cat([w.float() for w in weights], dim=0)
        bias = torch.cat([b.float() for b in biases], dim=0) if biases else None
        return _Linear(weight, bias)

    def prepare_gated_linear(self, gate, up, activation="silu", limit=None):
        acts = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "relu": torch.relu,
                "gelu_tanh": lambda z: torch.nn.functional.gelu(z, approximate="tanh")}
        if activation == "limited_swish":
            if limit is None or not limit > 0:
                raise ValueError("gated_linear: limited_swish has a positive limit")
            return (_Linear(gate.float(), None), _Linear(up.float(), None), lambda g, u: _limited_swish(g, u, float(limit)), True)
        if activation not in acts:
            raise ValueError(f"gated_linear: no activation {activation!r}")
        return (_Linear(gate.float(), None), _Linear(up.float(), None), acts[activation])

    def linear(self, x, weights, out_dtype=None, partial=False):
        y = x.float() @ weights.weight.T
        if weights.bias is not None:
            y = y + weights.bias
        return y.to(out_dtype or self.dtype)

    def gated_linear(self, x, weights):
        gate = x.float() @ weights[0].weight.T
        up = x.float() @ weights[1].weight.T
        if len(weights) > 3:  # a function of gate and up both
            return weights[2](gate, up).to(self.dtype)
        return (weights[2](gate) * up).to(self.dtype)

    def rotate_and_store(self, qkv, layout, batch, cell, inverse_frequencies, pairing):
        tokens = qkv.shape[0]
        heads, kv_heads, dim = layout.num_heads, layout.num_kv_heads, layout.head_dim
        view = qkv.view(tokens, heads + 2 * kv_heads, dim)
        if pairing != "none":
            angles = batch.positions.float()[:, None] * inverse_frequencies[None, :]
            cos, sin = angles.cos()[:, None, :], angles.sin()[:, None, :]
            part = view[:, : heads + kv_heads].float()
            if pairing == "adjacent":
                a, b = part[..., 0::2], part[..., 1::2]
                out = torch.empty_like(part)
                out[..., 0::2] = a * cos - b * sin
                out[..., 1::2] = b * cos + a * sin
            else:
                a, b = part[..., : dim // 2], part[..., dim // 2 :]
                out = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
            view[:, : heads + kv_heads] = out.to(qkv.dtype)
        if cell is not None and cell.writable:
            group = batch.groups[cell.group]
            slots = group.slot_mapping.long()
            pages, offsets = slots // group.page_size, slots % group.page_size
            cell.put_key_rows(pages, offsets, view[:, heads : heads + kv_heads])  # pages are [kv, dim / w, offset, w]
            cell.put_value_rows(pages, offsets, view[:, heads + kv_heads :])  # pages are [kv, offset / v, dim, v]

    def paged_attention(self, qkv, layout, batch, cell, scale, window, *, score_slopes=None, soft_cap=None, sinks=None, keep_first=0):
        tokens = qkv.shape[0]
        heads, kv_heads, dim = layout.num_heads, layout.num_kv_heads, layout.head_dim
        queries = qkv.view(tokens, heads + 2 * kv_heads, dim)[:, :heads].float()
        group = batch.groups[cell.group]
        out = torch.zeros(tokens, heads, dim)
        row = 0
        for b, chunk in enumerate(batch.chunks):
            table = group.block_tables[b].long()
            for position in range(chunk.start, chunk.start + chunk.count):
                first = 0 if window is None else max(0, position - window + 1)
                where = torch.arange(first, position + 1)
                if keep_first and first > 0:  # the sequence's first tokens stay visible, at their own positions
                    where = torch.cat([torch.arange(0, min(keep_first, first)), where])
                pages = table[where // group.page_size]
                assert (pages >= 0).all(), "attention reads a page that was given back"
                keys = cell.key_rows(pages, where % group.page_size).float()  # [n, kv, D]
                values = cell.value_rows(pages, where % group.page_size).float()
                keys = keys.repeat_interleave(heads // kv_heads, dim=1)
                values = values.repeat_interleave(heads // kv_heads, dim=1)
                scores = torch.einsum("hd,nhd->hn", queries[row], keys) * scale
                if soft_cap is not None:
                    scores = soft_cap * torch.tanh(scores / soft_cap)
                if score_slopes is not None:
                    scores = scores - score_slopes.float().view(-1, 1) * (position - where).float()
                if sinks is not None:  # a column more in the softmax, with no value
                    scores = torch.cat([scores, sinks.float().view(-1, 1)], dim=1)
                    out[row] = torch.einsum("hn,nhd->hd", torch.softmax(scores, dim=-1)[:, :-1], values)
                else:
                    out[row] = torch.einsum("hn,nhd->hd", torch.softmax(scores, dim=-1), values)
                row += 1
        return out.reshape(tokens, heads * dim).to(self.dtype)

    def rotate_store_attend(self, qkv, layout, batch, cell, inverse_frequencies, pairing, scale, window, project=None):
        self.rotate_and_store(qkv, layout, batch, cell, inverse_frequencies, pairing)
        mixed = self.paged_attention(qkv, layout, batch, cell, scale, window)
        return mixed if project is None else self.linear(mixed, project, out_dtype=torch.float32, partial=True)

    def gather_rows(self, hidden, delta, rows):
        picked = hidden[rows.long()]
        if delta is not None and delta.ndim == 3:
            delta = delta.sum(0)
        return picked + delta[rows.long()] if delta is not None else picked.clone()

    def argmax(self, logits):
        return torch.argmax(logits, dim=-1).to(torch.int32)

    def sample(self, logits, temperatures, top_ps, uniforms, with_top_p=True):
        chosen = []
        for row in range(logits.shape[0]):
            temperature, top_p, u = float(temperatures[row]), float(top_ps[row]), float(uniforms[row])
            if temperature <= 0:
                chosen.append(int(torch.argmax(logits[row])))
                continue
            p = torch.softmax(logits[row].float() / temperature, dim=-1).double()
            if top_p < 1.0:
                values, order = torch.sort(p, descending=True, stable=True)
                before = values.cumsum(0) - values
                keep = before < top_p
                values, order = values[keep], order[keep]
            else:
                values, order = p, torch.arange(p.numel())
            running = values.cumsum(0)
            hit = torch.nonzero(running > u * running[-1])
            chosen.append(int(order[hit[0, 0]] if hit.numel() else order[-1]))
        return torch.tensor(chosen, dtype=torch.int32)

    # ------------------------------------------------------------------ layer norm, column-wise operations

    def add_layer_norm(self, hidden, delta, weight, bias, eps):
        if delta is not None:
            hidden += delta if delta.ndim == 2 else delta.sum(0)
        mean = hidden.mean(-1, keepdim=True)
        centred = hidden - mean
        variance = centred.pow(2).mean(-1, keepdim=True)
        return (centred * torch.rsqrt(variance + eps) * weight.float() + bias.float()).to(self.dtype)

    def new_rows(self, rows, width):
        return torch.zeros((rows, width), dtype=self.dtype)

    def rms_norm_columns(self, x, first, weight, eps, out=None, out_first=0, copies=1, copy_stride=0):
        width = weight.shape[0]
        part = x[:, first : first + width].float()
        normed = (part * torch.rsqrt(part.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(self.dtype)
        if out is None:
            return normed
        for copy in range(copies):
            out[:, out_first + copy * copy_stride : out_first + copy * copy_stride + width] = normed
        return out

    def rotary_table(self, batch, frequencies, magnitude=1.0):
        angles = batch.positions.float()[:, None] * frequencies.float()[None, :]
        return torch.stack([angles.cos() * magnitude, angles.sin() * magnitude], dim=-1)

    def rotate_columns(self, x, first, head_stride, heads, width, table, dims, out, out_first, out_head_stride):
        cos, sin = table[..., 0], table[..., 1]
        for head in range(heads):
            part = x[:, first + head * head_stride : first + head * head_stride + width].float()
            turned = part.clone()
            a, b = part[:, 0:dims:2], part[:, 1:dims:2]
            turned[:, 0:dims:2] = a * cos - b * sin
            turned[:, 1:dims:2] = b * cos + a * sin
            out[:, out_first + head * out_head_stride : out_first + head * out_head_stride + width] = turned.to(out.dtype)
        return out

    def prepare_headwise_linear(self, weight):
        return weight.float()

    def headwise_linear(self, x, first, head_stride, weights, out=None, out_first=0, out_head_stride=None):
        heads, outputs, inner = weights.shape
        stride = outputs if out_head_stride is None else out_head_stride
        if out is None:
            out = torch.zeros((x.shape[0], heads * outputs), dtype=self.dtype)
        for head in range(heads):
            part = x[:, first + head * head_stride : first + head * head_stride + inner].float()
            out[:, out_first + head * stride : out_first + head * stride + outputs] = (part @ weights[head].T).to(out.dtype)
        return out

    def join_rows(self, hidden, delta, embedded):
        now = hidden if delta is None else hidden + (delta if delta.ndim == 2 else delta.sum(0))
        return torch.cat([now, embedded], dim=-1).to(self.dtype)

    def activate(self, x, activation):
        acts = {"silu": torch.nn.functional.silu, "gelu": torch.nn.functional.gelu, "relu": torch.relu,
                "gelu_tanh": lambda z: torch.nn.functional.gelu(z, approximate="tanh")}
        return acts[activation](x.float()).to(x.dtype)

    def add_gated_rows(self, target, rows, gates, column, squash):
        assert squash == "sigmoid"
        target += torch.sigmoid(gates[:, column : column + 1].float()) * rows
        return target

    # ------------------------------------------------------------------ the gated delta rule

    def causal_conv(self, x, channels, taps, activation, batch, window, bias=None):
        assert activation in ("silu", "none")
        width = taps.shape[1]
        out = torch.zeros((x.shape[0], channels))
        row = 0
        for chunk in batch.chunks:
            fresh = x[row : row + chunk.count, :channels].float()
            before = window[chunk.slot] if window is not None else torch.zeros((0, channels))
            line = torch.cat([before, fresh])  # the last taps - 1 inputs, then this step's
            for j in range(width):
                out[row : row + chunk.count] += line[j : j + chunk.count] * taps[:, j]
            if window is not None:
                window[chunk.slot] = line[-(width - 1):]
            row += chunk.count
        if bias is not None:
            out = out + bias.float()
        return (torch.nn.functional.silu(out) if activation == "silu" else out).to(self.dtype)

    def gated_delta_rule(self, mixed, controls, rate, step_bias, heads, kv_heads, dim, vdim, batch, state, channel_steps=None):
        tokens = mixed.shape[0]
        q = mixed[:, : kv_heads * dim].float().view(tokens, kv_heads, dim)
        k = mixed[:, kv_heads * dim : 2 * kv_heads * dim].float().view(tokens, kv_heads, dim)
        v = mixed[:, 2 * kv_heads * dim :].float().view(tokens, heads, vdim)
        q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * dim**-0.5
        k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(controls[:, :heads].float())
        if channel_steps is None:
            decay = torch.exp(-torch.exp(rate.float()) * torch.nn.functional.softplus(controls[:, heads:].float() + step_bias.float()))
            decay = decay.view(tokens, heads, 1, 1)
        else:  # a decay for every key channel of every head
            steps = torch.nn.functional.softplus(channel_steps[:, : heads * dim].float() + step_bias.float()).view(tokens, heads, dim)
            decay = torch.exp(-torch.exp(rate.float()).view(1, heads, 1) * steps).view(tokens, heads, dim, 1)
        out = torch.zeros((tokens, heads, vdim))
        row = 0
        for chunk in batch.chunks:
            S = state[chunk.slot].transpose(1, 2)  # kept as S^T [heads, vdim, dim]; this view is S [heads, dim, vdim], updated in place
            for t in range(row, row + chunk.count):
                kt = k[t].repeat_interleave(heads // kv_heads, dim=0)
                qt = q[t].repeat_interleave(heads // kv_heads, dim=0)
                S *= decay[t]
                u = beta[t].view(heads, 1) * (v[t] - torch.einsum("hdv,hd->hv", S, kt))
                S += torch.einsum("hd,hv->hdv", kt, u)
                out[t] = torch.einsum("hdv,hd->hv", S, qt)
            row += chunk.count
        return out.reshape(tokens, heads * vdim)

    def gated_head_norm(self, read, gates, gate_first, weight, eps, heads, vdim, activation):
        squash = {"silu": torch.nn.functional.silu, "sigmoid": torch.sigmoid}[activation]
        tokens = read.shape[0]
        rows = read.view(tokens, heads, vdim)
        normed = rows * torch.rsqrt(rows.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
        gate = squash(gates[:, gate_first : gate_first + heads * vdim].float()).view(tokens, heads, vdim)
        return (normed * gate).reshape(tokens, heads * vdim).to(self.dtype)

    # ------------------------------------------------------------------ norms on results, heads put together, linear attention

    def stream_rows(self, hidden, delta):
        if delta is not None:
            hidden += delta if delta.ndim == 2 else delta.sum(0)
        return hidden if self.dtype == torch.float32 else hidden.to(self.dtype)

    def add_normed(self, hidden, update, weight, eps):
        u = update if update.ndim == 2 else update.sum(0)
        hidden += u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
        return hidden if self.dtype == torch.float32 else hidden.to(self.dtype)

    def assemble_heads(self, x, q_first, k_first, v_first, heads, kv_heads, dim, vdim, width, norm, q_weight, k_weight, eps,
                       table, rot_dims, other=None, other_first=0, blend=0.0, batch=None, cell=None, pairing="adjacent"):
        tokens = x.shape[0]
        out = torch.zeros((tokens, heads + 2 * kv_heads, width))

        def normed_turned(first, count, weight):
            part = x[:, first : first + count * dim].float()
            if norm == "row":
                part = part * torch.rsqrt(part.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
            part = part.reshape(tokens, count, dim)
            if norm == "head":
                part = part * torch.rsqrt(part.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
            if rot_dims:
                cos, sin = table[:, None, :, 0], table[:, None, :, 1]
                first, second = (slice(0, rot_dims, 2), slice(1, rot_dims, 2)) if pairing == "adjacent" else (slice(0, rot_dims // 2), slice(rot_dims // 2, rot_dims))
                a, b = part[..., first], part[..., second]
                turned = part.clone()
                turned[..., first] = a * cos - b * sin
                turned[..., second] = b * cos + a * sin
                part = turned
            return part

        out[:, :heads, :dim] = normed_turned(q_first, heads, q_weight)
        out[:, heads : heads + kv_heads, :dim] = normed_turned(k_first, kv_heads, k_weight)
        values = x[:, v_first : v_first + kv_heads * vdim].float()
        if other is not None:
            values = (1.0 - blend) * values + blend * other[:, other_first : other_first + kv_heads * vdim].float()
        out[:, heads + kv_heads :, :vdim] = values.reshape(tokens, kv_heads, vdim)
        out = out.reshape(tokens, -1).to(self.dtype)
        if cell is not None and cell.writable:
            from llmserve_amd.parts import HeadLayout

            self.rotate_and_store(out, HeadLayout(heads, kv_heads, width), batch, cell, None, "none")
        return out

    def scale_heads(self, x, heads, width, gates, gate_first, squash):
        assert squash == "sigmoid"
        gate = torch.sigmoid(gates[:, gate_first : gate_first + heads].float())
        x.copy_((x.float().view(x.shape[0], heads, width) * gate[:, :, None]).reshape(x.shape).to(x.dtype))
        return x

    def rotate_heads(self, x, first, head_stride, heads, table, dims, pairing, scale=1.0, scale_from=0):
        tokens = x.shape[0]
        for head in range(heads):
            part = x[:, first + head * head_stride : first + (head + 1) * head_stride].float()
            if dims:
                cos, sin = table[:, :, 0], table[:, :, 1]
                one, two = (slice(0, dims, 2), slice(1, dims, 2)) if pairing == "adjacent" else (slice(0, dims // 2), slice(dims // 2, dims))
                a, b = part[:, one].clone(), part[:, two].clone()
                part[:, one] = a * cos - b * sin
                part[:, two] = b * cos + a * sin
            x[:, first + head * head_stride : first + (head + 1) * head_stride] = (part * (scale if head >= scale_from else 1.0)).to(x.dtype)
        return x

    def add_normed_norm(self, hidden, update, weight, eps, next_weight, next_eps):
        self.add_normed(hidden, update, weight, eps)
        return self.add_rms_norm(hidden, None, next_weight, next_eps)

    def add_rows(self, hidden, delta, other, vector):
        if delta is not None:
            hidden += delta if delta.ndim == 2 else delta.sum(0)
        if other is not None:
            hidden += other
        if vector is not None:
            hidden += vector.float()
        return hidden

    def decay_attention(self, x, q_first, k_first, v_first, heads, dim, vdim, decays, activation, batch, state):
        assert activation in ("silu", "none")
        tokens = x.shape[0]
        act = torch.nn.functional.silu if activation == "silu" else (lambda z: z)
        q = act(x[:, q_first : q_first + heads * dim].float()).view(tokens, heads, dim)
        k = act(x[:, k_first : k_first + heads * dim].float()).view(tokens, heads, dim)
        v = act(x[:, v_first : v_first + heads * vdim].float()).view(tokens, heads, vdim)
        out = torch.zeros((tokens, heads, vdim))
        row = 0
        for chunk in batch.chunks:
            S = state[chunk.slot]  # [heads, dim, vdim], updated in place
            for t in range(row, row + chunk.count):
                S *= decays.float().view(heads, 1, 1)
                S += torch.einsum("hd,hv->hdv", k[t], v[t])
                out[t] = torch.einsum("hdv,hd->hv", S, q[t])
            row += chunk.count
        return out.reshape(tokens, heads * vdim)

    def soft_cap(self, logits, cap):
        return logits.copy_(cap * torch.tanh(logits / cap))

    # ------------------------------------------------------------------ routed experts

    def route(self, scores, experts, correction, top, scale, scoring, groups=1, keep_groups=1, renormalise=False):
        z = scores[:, :experts].float()
        squashed = torch.sigmoid(z) if scoring == "sigmoid" else torch.softmax(z, dim=-1)
        assert scoring in ("sigmoid", "softmax")
        choice = squashed + correction.float() if correction is not None else squashed.clone()
        if groups > 1:  # only experts of the best groups can be chosen; a group's score is its largest
            best = choice.view(-1, groups, experts // groups).max(-1).values
            kept = torch.sort(best, dim=-1, descending=True, stable=True).indices[:, :keep_groups]
            allowed = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True).repeat_interleave(experts // groups, dim=1)
            choice = torch.where(allowed, choice, torch.full_like(choice, -math.inf))
        chosen = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
        weights = squashed.gather(1, chosen)
        if renormalise:
            weights = weights / (weights.sum(-1, keepdim=True) + 1e-20)
        return chosen.to(torch.int32), (weights * scale).float()

    def prepare_experts(self, ups, downs, activation, gates=None, limit=None):
        stacked = torch.stack([w.float() for w in gates]) if gates is not None else None
        if activation == "limited_swish":
            if stacked is None or limit is None or not limit > 0:
                raise ValueError("experts: limited_swish gates an expert and has a positive limit")
            activation = ("limited_swish", float(limit))
        return (torch.stack([w.float() for w in ups]), torch.stack([w.float() for w in downs]), activation, stacked)

    def conv_gated_delta_rule(self, projected, channels, taps, activation, controls, rate, step_bias, heads, kv_heads, dim, vdim, batch, window, state,
                              channel_steps=None):
        mixed = self.causal_conv(projected, channels, taps, activation, batch, window)
        return self.gated_delta_rule(mixed, controls, rate, step_bias, heads, kv_heads, dim, vdim, batch, state, channel_steps=channel_steps)

    def expert_feed_forward(self, x, experts, chosen, weights, shared=None, gates=None, gate_column=0):
        ups, downs, activation, gate_weights = experts
        out = torch.zeros((x.shape[0], downs.shape[1]))
        rows = torch.zeros((x.shape[0], chosen.shape[1], downs.shape[1]))  # every (token, choice) pair's row, then added in the order of the choices
        for e in range(ups.shape[0]):
            tokens, slots = (chosen == e).nonzero(as_tuple=True)
            if tokens.numel() == 0:
                continue
            mine = x[tokens].float()
            if gate_weights is None:
                inner = self.activate((mine @ ups[e].T).to(self.dtype), activation).float()
            elif isinstance(activation, tuple):  # a function of gate and up both, rounded to the run dtype before
                gate = (mine @ gate_weights[e].T).to(self.dtype).float()
                up = (mine @ ups[e].T).to(self.dtype).float()
                inner = _limited_swish(gate, up, activation[1]).to(self.dtype).float()
            else:  # act(gate x) * (up x), both rounded to the run dtype before
                gate = self.activate((mine @ gate_weights[e].T).to(self.dtype), activation).float()
                inner = (gate * (mine @ ups[e].T).to(self.dtype).float()).to(self.dtype).float()
            rows[tokens, slots] = inner @ downs[e].T
        for slot in range(chosen.shape[1]):
            out += weights[:, slot : slot + 1] * rows[:, slot]
        if shared is not None:
            out += torch.sigmoid(gates[:, gate_column : gate_column + 1].float()) * shared if gates is not None else shared
        return out

    # ------------------------------------------------------------------ copies of the stream, a diagonal recurrence, weighted sums

    def stream_copies(self, hidden, copies, scale):
        return (hidden * scale).repeat(1, copies)

    def stream_norm(self, streams, pending, read, weight, eps, rows=None):
        copies = read.shape[0]
        now = streams if pending is None else pending.applied(streams)
        if rows is None:
            if pending is not None:
                streams.copy_(now)
        else:
            now = now[rows.long()]
        u = torch.einsum("s,nsh->nh", read.float(), now.view(now.shape[0], copies, -1))
        return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(self.dtype)

    def gated_recurrence(self, u, gates, gate_bias, rates, branch, branch_first, activation, blocks, batch, state):
        assert activation == "gelu_tanh"
        tokens, width = u.shape
        part = width // blocks
        z = gates.float().view(tokens, blocks, 2 * part) + gate_bias.float()
        r = torch.sigmoid(z[..., :part]).reshape(tokens, width)
        i = torch.sigmoid(z[..., part:]).reshape(tokens, width)
        a = torch.exp(rates.float() * r)
        push = torch.sqrt(-torch.expm1(2.0 * rates.float() * r)) * i * u.float()  # sqrt(1 - a^2), exact also where a is near one
        y = torch.nn.functional.gelu(branch[:, branch_first : branch_first + width].float(), approximate="tanh")
        out = torch.zeros((tokens, width))
        row = 0
        for chunk in batch.chunks:
            S = state[chunk.slot]
            for t in range(row, row + chunk.count):
                S.copy_(a[t] * S + push[t])
                out[t] = S * y[t]
            row += chunk.count
        return out.to(self.dtype)

    def add_scaled(self, a, a_scale, b, b_scale):
        total = a_scale * (a if a.ndim == 2 else a.sum(0))
        if b is not None:
            total = total + b_scale * (b if b.ndim == 2 else b.sum(0))
        return total
