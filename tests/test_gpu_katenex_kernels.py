"""The kernels of the Katenex parts, each alone against the same operation in elementary float32 torch (the CPU
stand-in of the kernel library), at sizes that are no powers of two and over steps that cut a request's tokens anywhere."""

from __future__ import annotations

import types

import pytest
import torch

from llmserve_amd.parts.hyper import PendingWrite
from tests.torch_kernels import TorchKernels

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
TOLERANCE = {torch.float32: dict(atol=3e-5, rtol=3e-5), torch.bfloat16: dict(atol=3e-2, rtol=3e-2)}


@pytest.fixture(scope="module")
def kernels():
    from llmserve_amd.kernels import HipKernels

    return {dtype: HipKernels(dtype) for dtype in DTYPES}


def gpu(tensor, dtype=None):
    return tensor.to("cuda", dtype) if dtype is not None else tensor.to("cuda")


def close(got, want, dtype, **more):
    torch.testing.assert_close(got.detach().cpu().float(), want.detach().float(), **{**TOLERANCE[dtype], **more})


def step_of(counts, starts, slots, device):
    chunks = [types.SimpleNamespace(request_id=str(b), slot=slot, start=start, count=count) for b, (count, start, slot) in enumerate(zip(counts, starts, slots))]
    positions = torch.cat([torch.arange(start, start + count) for count, start in zip(counts, starts)]).to(torch.int32)
    query_start = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32)
    sequence = torch.cat([torch.full((count,), b, dtype=torch.int32) for b, count in enumerate(counts)])
    return types.SimpleNamespace(
        chunks=chunks, positions=positions.to(device), query_start=query_start.to(device), max_query_length=max(counts),
        state_slots=torch.tensor(slots, dtype=torch.int32).to(device), token_sequence=sequence.to(device), computed={}, scratch={},
    )


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("copies,width", [(1, 24), (2, 30), (3, 328), (4, 1001), (8, 70), (3, 4100)])
def test_copies_of_the_stream(kernels, dtype, copies, width):
    """The copies made, a pending write done on the way to the next read (one result, partial sums), the rows picked
    behind the last layer (the copies then stay as they are)."""
    torch.manual_seed(width)
    plain, tokens = TorchKernels(dtype), 6
    embedded = torch.randn(tokens, width)
    want_streams = plain.stream_copies(embedded, copies, 2.5)
    streams = kernels[dtype].stream_copies(gpu(embedded), copies, 2.5)
    close(streams, want_streams, torch.float32)
    # the copies differ from here on
    want_streams = (want_streams + torch.randn(tokens, copies * width)).contiguous()
    streams = gpu(want_streams)
    read = 0.7 + 0.3 * torch.randn(copies)
    weight = (1 + 0.2 * torch.randn(width)).to(dtype)
    close(kernels[dtype].stream_norm(streams, None, gpu(read), gpu(weight), 1e-5), plain.stream_norm(want_streams, None, read, weight, 1e-5), dtype)
    for result in (torch.randn(tokens, width), 0.5 * torch.randn(3, tokens, width)):
        mix, out = torch.eye(copies) + 0.25 * torch.randn(copies, copies), 0.7 + 0.3 * torch.randn(copies)
        want = plain.stream_norm(want_streams, PendingWrite(result, mix, out), read, weight, 1e-5)
        got = kernels[dtype].stream_norm(streams, PendingWrite(gpu(result), gpu(mix), gpu(out)), gpu(read), gpu(weight), 1e-5)
        close(got, want, dtype)
        close(streams, want_streams, torch.float32)
    rows = torch.tensor([4, 0, 5], dtype=torch.int32)
    before = streams.clone()
    pending = PendingWrite(result, mix, out)
    want = plain.stream_norm(want_streams.clone(), pending, torch.ones(copies), weight, 1e-5, rows=rows)
    got = kernels[dtype].stream_norm(streams, PendingWrite(gpu(result), gpu(mix), gpu(out)), gpu(torch.ones(copies)), gpu(weight), 1e-5, rows=gpu(rows))
    close(got, want, dtype)
    assert torch.equal(streams, before)


def test_weighted_sums_of_results(kernels):
    torch.manual_seed(1)
    plain, library = TorchKernels(torch.float32), kernels[torch.float32]
    for a, b in ((torch.randn(5, 70), torch.randn(5, 70)), (torch.randn(3, 5, 70), torch.randn(5, 70)), (torch.randn(5, 70), torch.randn(2, 5, 70)),
                 (torch.randn(2, 5, 70), None)):
        close(library.add_scaled(gpu(a), 1.2, gpu(b) if b is not None else None, 0.5), plain.add_scaled(a, 1.2, b, 0.5), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,blocks", [(40, 5), (64, 1), (330, 3), (1280, 4)])
def test_gated_recurrence_over_steps(kernels, dtype, width, blocks):
    """Three requests in slots that are not their order; steps of single tokens, of a few, and portions long enough to be
    walked as four and as sixteen runs side by side, also shorter than the runs are many; decays near one among them."""
    torch.manual_seed(width)
    plain = TorchKernels(dtype)
    part = width // blocks
    slots = [2, 0, 3]
    state = torch.zeros(5, width)
    on_device = gpu(state)
    bias = 0.5 * torch.randn(blocks, 2 * part)
    rates = -8.0 * torch.nn.functional.softplus(torch.randn(width) * 2.0 - 4.0)
    for counts in ([1, 1, 1], [9, 1, 2], [37, 3, 64], [300, 1, 11], [2, 65, 8], [1, 1, 1]):
        tokens = sum(counts)
        u = torch.randn(tokens, width).to(dtype)
        gates = (2 * torch.randn(tokens, 2 * width)).to(dtype)
        branch = torch.randn(tokens, 7 + width + 3).to(dtype)
        want = plain.gated_recurrence(u, gates, bias, rates, branch, 7, "gelu_tanh", blocks, step_of(counts, [0] * 3, slots, "cpu"), state)
        got = kernels[dtype].gated_recurrence(gpu(u), gpu(gates), gpu(bias), gpu(rates), gpu(branch), 7, "gelu_tanh", blocks,
                                              step_of(counts, [0] * 3, slots, "cuda"), on_device)
        close(got, want, dtype, **(dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else {}))
        close(on_device, state, torch.float32, atol=1e-4, rtol=1e-4)
    assert float(on_device[1].abs().max()) == 0.0 and float(on_device[4].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 3, 4])
def test_causal_conv_with_a_bias_and_no_activation(kernels, dtype, taps):
    torch.manual_seed(taps)
    channels, extra = 70, 13
    weights, bias = torch.randn(channels, taps) / taps**0.5, 0.5 * torch.randn(channels)
    plain = TorchKernels(dtype)
    slots = [2, 0, 3]
    window = torch.zeros(5, taps - 1, channels) if taps > 1 else None
    on_device = gpu(window) if window is not None else None
    for counts in ([9, 1, 2], [1, 1, 1], [2, 5, 1]):
        x = torch.randn(sum(counts), channels + extra).to(dtype)
        want = plain.causal_conv(x, channels, weights, "none", step_of(counts, [0] * 3, slots, "cpu"), window, bias=bias)
        got = kernels[dtype].causal_conv(gpu(x), channels, gpu(weights), "none", step_of(counts, [0] * 3, slots, "cuda"), on_device, bias=gpu(bias))
        close(got, want, dtype)
        if window is not None:
            close(on_device, window, torch.float32, atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,taps", [(6, 2, 64, 32, 4), (2, 2, 16, 96, 1), (4, 1, 80, 32, 3), (3, 3, 130, 70, 2), (5, 5, 32, 48, 3), (6, 3, 24, 40, 2)])
def test_delta_rule_with_a_decay_per_key_channel(kernels, dtype, heads, kv_heads, dim, vdim, taps):
    """The rule alone and behind its convolutions, over steps of many tokens, of one and of two; the channels' steps are
    the first columns of wider rows, as the part hands them over."""
    torch.manual_seed(dim + taps)
    plain = TorchKernels(torch.float32)  # (the fused form keeps what lies between the two in float32)
    channels = 2 * kv_heads * dim + heads * vdim
    weights = torch.randn(channels, taps) / taps**0.5
    slots = [1, 3]
    rate, bias = torch.randn(heads) - 1.0, torch.randn(heads * dim)
    for fused in (False, True):
        state, window = torch.zeros(5, heads, vdim, dim), (torch.zeros(5, taps - 1, channels) if taps > 1 else None)
        on_device, window_on_device = gpu(state), (gpu(window) if window is not None else None)
        for counts in ([37, 1], [1, 1], [2, 1], [2, 19]):
            tokens = sum(counts)
            projected = torch.randn(tokens, channels + 9).to(dtype)
            controls = 2 * torch.randn(tokens, heads)
            steps = 2 * torch.randn(tokens, heads * dim + heads * vdim)
            if fused:
                want = plain.conv_gated_delta_rule(projected.float(), channels, weights, "silu", controls, rate, bias, heads, kv_heads, dim, vdim,
                                                   step_of(counts, [0, 0], slots, "cpu"), window, state, channel_steps=steps)
                got = kernels[dtype].conv_gated_delta_rule(
                    gpu(projected), channels, gpu(weights), "silu", gpu(controls), gpu(rate), gpu(bias), heads, kv_heads, dim, vdim,
                    step_of(counts, [0, 0], slots, "cuda"), window_on_device, on_device, channel_steps=gpu(steps))
            else:
                mixed = projected[:, :channels].contiguous()
                want = plain.gated_delta_rule(mixed, controls, rate, bias, heads, kv_heads, dim, vdim, step_of(counts, [0, 0], slots, "cpu"), state,
                                              channel_steps=steps)
                got = kernels[dtype].gated_delta_rule(gpu(mixed), gpu(controls), gpu(rate), gpu(bias), heads, kv_heads, dim, vdim,
                                                      step_of(counts, [0, 0], slots, "cuda"), on_device, channel_steps=gpu(steps))
            close(got, want, torch.float32, atol=3e-4, rtol=3e-4)
            close(on_device, state, torch.float32, atol=3e-4, rtol=3e-4)
        assert float(on_device[0].abs().max()) == 0.0 and float(on_device[2].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
def test_head_norm_gated_by_float32_rows(kernels, dtype):
    torch.manual_seed(3)
    heads, vdim = 3, 40
    read, gates = torch.randn(9, heads * vdim), torch.randn(9, 11 + heads * vdim)
    weight = (1 + 0.2 * torch.randn(vdim)).to(dtype)
    want = TorchKernels(dtype).gated_head_norm(read, gates, 11, weight, 1e-5, heads, vdim, "sigmoid")
    got = kernels[dtype].gated_head_norm(gpu(read), gpu(gates), 11, gpu(weight), 1e-5, heads, vdim, "sigmoid")
    assert got.dtype == dtype
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,width,rot", [(6, 2, 24, 40, 48, 10), (3, 1, 16, 16, 16, 16), (6, 3, 96, 80, 96, 32), (2, 1, 70, 6, 80, 6)])
def test_heads_turned_in_half_pairs(kernels, dtype, heads, kv_heads, dim, vdim, width, rot):
    torch.manual_seed(heads * dim)
    tokens, extra = 7, 5
    x = torch.randn(tokens, extra + (heads + kv_heads) * dim + kv_heads * vdim + 3).to(dtype)
    angles = torch.rand(tokens, rot // 2) * 6.0
    table = torch.stack([angles.cos(), angles.sin()], dim=-1).contiguous()
    first = (extra, extra + heads * dim, extra + (heads + kv_heads) * dim)
    want = TorchKernels(dtype).assemble_heads(x, *first, heads, kv_heads, dim, vdim, width, None, None, None, 1e-5, table, rot, pairing="half")
    got = kernels[dtype].assemble_heads(gpu(x), *first, heads, kv_heads, dim, vdim, width, None, None, None, 1e-5, gpu(table), rot, pairing="half")
    close(got, want, dtype)
    other = TorchKernels(dtype).assemble_heads(x, *first, heads, kv_heads, dim, vdim, width, None, None, None, 1e-5, table, rot, pairing="adjacent")
    assert rot <= 2 or float((other.float() - want.float()).abs().max()) > 0.1  # the two pairings are not the same thing


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,experts,top,groups,keep,hidden,size", [
    (1, 4, 4, 1, 1, 32, 16), (37, 8, 2, 4, 2, 96, 40), (200, 6, 3, 3, 2, 64, 72), (5, 10, 3, 5, 2, 64, 32), (300, 4, 2, 2, 2, 64, 96),
    (130, 9, 1, 3, 1, 320, 64), (700, 15, 5, 5, 3, 256, 64), (1000, 2, 1, 2, 1, 128, 64), (50, 70, 5, 7, 3, 48, 24),
])
def test_experts_chosen_within_groups_and_gated(kernels, dtype, tokens, experts, top, groups, keep, hidden, size):
    torch.manual_seed(tokens + experts)
    scores = 2 * torch.randn(tokens, experts + 2)
    plain = TorchKernels(dtype)
    want_chosen, want_weights = plain.route(scores, experts, None, top, 1.5, "softmax", groups, keep, True)
    chosen, weights = kernels[dtype].route(gpu(scores), experts, None, top, 1.5, "softmax", groups, keep, True)
    assert torch.equal(chosen.cpu(), want_chosen)
    close(weights, want_weights, torch.float32)
    if keep < groups and top > keep:  # (the `top` best experts always lie in the `top` best groups)
        free, _ = plain.route(scores, experts, None, top, 1.5, "softmax")
        assert not torch.equal(free, want_chosen)  # the groups do restrict the choice somewhere
    _, plainly = kernels[dtype].route(gpu(scores), experts, None, top, 1.5, "softmax", groups, keep, False)
    close(plainly, plain.route(scores, experts, None, top, 1.5, "softmax", groups, keep, False)[1], torch.float32)
    x = torch.randn(tokens, hidden).to(dtype)
    gates = [(torch.randn(size, hidden) / hidden**0.5).to(dtype) for _ in range(experts)]
    ups = [(torch.randn(size, hidden) / hidden**0.5).to(dtype) for _ in range(experts)]
    downs = [(torch.randn(hidden, size) / size**0.5).to(dtype) for _ in range(experts)]
    shared = torch.randn(tokens, hidden)
    want = plain.expert_feed_forward(x, plain.prepare_experts(ups, downs, "silu", gates=gates), want_chosen, want_weights, shared=shared)
    prepared = kernels[dtype].prepare_experts([gpu(w) for w in ups], [gpu(w) for w in downs], "silu", gates=[gpu(w) for w in gates])
    got = kernels[dtype].expert_feed_forward(gpu(x), prepared, chosen, weights, shared=gpu(shared))
    close(got, want, dtype)
    again = kernels[dtype].expert_feed_forward(gpu(x), prepared, chosen, weights, shared=gpu(shared))
    assert torch.equal(got, again)
