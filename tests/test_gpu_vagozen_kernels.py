"""The kernels of the Vagozen parts, each alone against the same operation in elementary float32 torch (the CPU
stand-in of the kernel library), at sizes that are no powers of two and over steps that cut a request's tokens anywhere."""

from __future__ import annotations

import types

import pytest
import torch

from tests.test_gpu_sozavik_kernels import DTYPES, close, gpu, step_of
from tests.torch_kernels import TorchKernels

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def kernels():
    from llmserve_amd.kernels import HipKernels

    return {dtype: HipKernels(dtype) for dtype in DTYPES}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [24, 30, 328, 1001, 4100, 6000])
def test_add_normed_norm_and_add_rows(kernels, dtype, width):
    torch.manual_seed(width)
    hidden = torch.randn(5, width) + 0.5
    weight = 1 + 0.2 * torch.randn(width)  # (float32: a norm's weight times a learned vector)
    next_weight = (1 + 0.2 * torch.randn(width)).to(dtype)
    plain = TorchKernels(dtype)
    for update in (0.3 * torch.randn(3, 5, width), 2.0 * torch.randn(5, width)):
        plain_hidden, on_device = hidden.clone(), gpu(hidden)
        want = plain.add_normed_norm(plain_hidden, update, weight, 1e-5, next_weight, 1e-3)
        got = kernels[dtype].add_normed_norm(on_device, gpu(update), gpu(weight), 1e-5, gpu(next_weight), 1e-3)
        close(on_device, plain_hidden, torch.float32)
        close(got, want, dtype)
        assert got.dtype == dtype and got.data_ptr() != on_device.data_ptr()
    other, vector = torch.randn(5, width), torch.randn(width)
    for delta, rows, one in ((0.3 * torch.randn(2, 5, width), other, vector), (None, other, vector), (torch.randn(5, width), None, vector),
                             (None, None, vector), (torch.randn(5, width), other, None)):
        plain_hidden, on_device = hidden.clone(), gpu(hidden)
        plain.add_rows(plain_hidden, delta, rows, one)
        result = kernels[dtype].add_rows(on_device, *(None if t is None else gpu(t) for t in (delta, rows, one)))
        assert result.data_ptr() == on_device.data_ptr()
        close(on_device, plain_hidden, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pairing", ["adjacent", "half"])
@pytest.mark.parametrize("heads,stride,dims,scale", [(3, 16, 16, 1.0), (4, 24, 10, 0.25), (1, 70, 2, 1.7), (5, 8, 0, 0.5), (2, 128, 64, 0.088)])
def test_rotate_heads(kernels, dtype, pairing, heads, stride, dims, scale):
    torch.manual_seed(heads * stride + dims)
    tokens, first = 9, 5
    angles = torch.rand(tokens, max(dims // 2, 1)) * 6.0
    table = torch.stack([angles.cos(), angles.sin()], dim=-1)[:, : dims // 2].contiguous()
    for kind in (torch.float32, dtype):  # (rows a product left in float32, and rows in the run dtype)
        x = torch.randn(tokens, first + heads * stride + 3).to(kind)
        for scale_from in (0, heads // 2):
            want = TorchKernels(dtype).rotate_heads(x.clone(), first, stride, heads, table, dims, pairing, scale, scale_from)
            got = kernels[dtype].rotate_heads(gpu(x), first, stride, heads, gpu(table) if dims else None, dims, pairing, scale, scale_from)
            close(got, want, kind)
        assert torch.equal(got.cpu()[:, :first], x[:, :first]) and torch.equal(got.cpu()[:, first + heads * stride:], x[:, first + heads * stride:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 8, 40, 300])
@pytest.mark.parametrize("hidden,size,limit", [(64, 96, 1.0), (40, 24, 2.5), (256, 512, 0.5)])
def test_the_gate_with_a_limit(kernels, dtype, rows, hidden, size, limit):
    torch.manual_seed(rows + size)
    x = torch.randn(rows, hidden).to(dtype)
    gate, up = ((1.5 * torch.randn(size, hidden) / hidden ** 0.5).to(dtype) for _ in range(2))
    want = TorchKernels(dtype).gated_linear(x, TorchKernels(dtype).prepare_gated_linear(gate, up, "limited_swish", limit=limit))
    library = kernels[dtype]
    got = library.gated_linear(gpu(x), library.prepare_gated_linear(gpu(gate), gpu(up), "limited_swish", limit=limit))
    close(got, want, dtype, **({"atol": 6e-2, "rtol": 3e-2} if dtype == torch.bfloat16 else {}))
    from llmserve_amd.kernels.hip import KernelError

    for wrong in (dict(activation="limited_swish"), dict(activation="silu", limit=1.0), dict(activation="limited_swish", limit=0.0)):
        with pytest.raises(KernelError):
            library.prepare_gated_linear(gpu(gate), gpu(up), **wrong)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,experts,top,hidden,size", [(7, 5, 2, 40, 24), (3, 4, 4, 64, 32), (200, 4, 2, 64, 64), (900, 3, 1, 128, 64)])
def test_experts_gated_with_a_limit_and_a_softmax_over_the_chosen(kernels, dtype, tokens, experts, top, hidden, size):
    """Every product kernel of the experts (a few rows an expert, tiles of 64 and of 128 rows, the plain one), the gate
    with a limit behind the first product, and weights that are the softmax over the chosen logits alone."""
    torch.manual_seed(tokens + experts)
    x = torch.randn(tokens, hidden).to(dtype)
    gates, ups = ([(1.5 * torch.randn(size, hidden) / hidden ** 0.5).to(dtype) for _ in range(experts)] for _ in range(2))
    downs = [(torch.randn(hidden, size) / size ** 0.5).to(dtype) for _ in range(experts)]
    logits = 2.0 * torch.randn(tokens, experts + 2)
    plain, library = TorchKernels(dtype), kernels[dtype]
    chosen, weights = plain.route(logits, experts, None, top, 1.0, "softmax", renormalise=True)
    best = torch.topk(logits[:, :experts], top, dim=-1)
    assert torch.equal(chosen.long().sort(-1).values, best.indices.sort(-1).values)
    torch.testing.assert_close(weights.sort(-1).values, torch.softmax(best.values, -1).sort(-1).values, atol=1e-6, rtol=1e-5)
    got_chosen, got_weights = library.route(gpu(logits), experts, None, top, 1.0, "softmax", renormalise=True)
    assert torch.equal(got_chosen.cpu(), chosen)
    close(got_weights, weights, torch.float32)
    want = plain.expert_feed_forward(x, plain.prepare_experts(ups, downs, "limited_swish", gates=gates, limit=1.25), chosen, weights)
    prepared = library.prepare_experts([gpu(w) for w in ups], [gpu(w) for w in downs], "limited_swish", gates=[gpu(w) for w in gates], limit=1.25)
    got = library.expert_feed_forward(gpu(x), prepared, got_chosen, got_weights)
    close(got, want, dtype, **({"atol": 8e-2, "rtol": 5e-2} if dtype == torch.bfloat16 else {"atol": 1e-4, "rtol": 1e-4}))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim", [(3, 32, 48), (2, 24, 40), (2, 64, 128)])
@pytest.mark.parametrize("counts", [[1, 1, 1], [37, 1, 16], [300, 2, 130]])
def test_decay_attention_of_float32_rows_without_an_activation(kernels, dtype, heads, dim, vdim, counts):
    """What a retention layer asks for: rows that the product left in float32 (in either run), no activation."""
    torch.manual_seed(dim + vdim + sum(counts))
    tokens = sum(counts)
    row = 2 * heads * dim + 2 * heads * vdim
    decays = torch.tensor([0.999, 0.6, 0.93][:heads], dtype=torch.float32)
    state = 0.5 * torch.randn(5, heads, dim, vdim)
    x = torch.randn(tokens, row)
    firsts = (0, heads * dim, 2 * heads * dim)
    batch = step_of(counts, [0] * len(counts), [3, 0, 4], "cuda")
    plain_state, device_state = state.clone(), gpu(state)
    want = TorchKernels(dtype).decay_attention(x, *firsts, heads, dim, vdim, decays, "none", batch, plain_state)
    got = kernels[dtype].decay_attention(gpu(x), *firsts, heads, dim, vdim, gpu(decays), "none", batch, device_state)
    scale = float(want.abs().max())
    close(got / scale, want / scale, torch.float32, atol=2e-5, rtol=1e-4)
    close(device_state, plain_state, torch.float32, atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,page", [(4, 2, 64, 16), (8, 1, 128, 16), (6, 1, 48, 8), (3, 3, 24, 4)])
@pytest.mark.parametrize("counts,starts", [([1, 1, 1], [700, 3, 140]), ([33, 1, 7], [0, 90, 250]), ([300], [0]), ([64, 2, 17], [100, 511, 31])])
@pytest.mark.parametrize("window,keep", [(50, 6), (7, 3), (33, 40), (20, 1), (64, 32), (16, 70), (40, 0)])
def test_attention_keeps_a_sequences_first_tokens(kernels, dtype, heads, kv_heads, dim, page, counts, starts, window, keep):
    """Behind a window the first `keep` keys stay visible, through every attention kernel, with key splits, in portions
    and single tokens.  The pages between the kept ones and the window's, which a cache gives back, hold no number here:
    a kernel that read one, even with a weight of zero, would show it."""
    from llmserve_amd.cache.cell import CacheCell
    from llmserve_amd.parts import HeadLayout, PagedKeyValue

    torch.manual_seed(dim + sum(counts) + window)
    layout = HeadLayout(heads, kv_heads, dim)
    need = PagedKeyValue(kv_heads, dim, window, keep)
    longest = max(s + c for s, c in zip(starts, counts))
    per = -(-longest // page)
    pages = per * len(counts) + 2
    fields = {name: (0.7 * torch.randn(pages, *shape)).to(dtype) for name, shape in need.page_fields(page).items()}
    for value in fields.values():
        value[pages - 1] = float("nan")  # the page that stands for every page given back
    order = torch.randperm(pages - 2) + 1
    tables = order[: per * len(counts)].reshape(len(counts), per).to(torch.int32)
    for b, start in enumerate(starts):
        tables[b, -(-keep // page): max(0, start - window + 1) // page] = pages - 1
    tokens = sum(counts)
    qkv = (0.8 * torch.randn(tokens, layout.width)).to(dtype)

    def batch_on(device):
        batch = step_of(counts, starts, list(range(len(counts))), device)
        batch.token_sequence = torch.cat([torch.full((c,), b) for b, c in enumerate(counts)]).to(torch.int32).to(device)
        batch.max_context_length = longest
        batch.context_lengths = torch.tensor([s + c for s, c in zip(starts, counts)], dtype=torch.int32).to(device)
        batch.groups = [types.SimpleNamespace(page_size=page, block_tables=tables.to(device), slot_mapping=None, width=per)]
        batch.padded_to = None
        return batch

    plain_cell = CacheCell(need, group=0, fields={name: value.clone() for name, value in fields.items()})
    device_cell = CacheCell(need, group=0, fields={name: gpu(value) for name, value in fields.items()})
    want = TorchKernels(dtype).paged_attention(qkv, layout, batch_on("cpu"), plain_cell, 0.2, window, keep_first=keep)
    assert not torch.isnan(want.float()).any()
    got = kernels[dtype].paged_attention(gpu(qkv), layout, batch_on("cuda"), device_cell, 0.2, window, keep_first=keep)
    close(got, want, dtype)
