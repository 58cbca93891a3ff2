"""The kernels of the Sozavik parts, each alone against the same operation in elementary float32 torch (the CPU
stand-in of the kernel library), at sizes that are no powers of two and over steps that cut a request's tokens anywhere."""

from __future__ import annotations

import types

import pytest
import torch

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
    return types.SimpleNamespace(
        chunks=chunks, positions=positions.to(device), query_start=query_start.to(device), max_query_length=max(counts),
        state_slots=torch.tensor(slots, dtype=torch.int32).to(device), computed={}, scratch={},
    )


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [24, 30, 328, 1001, 4100, 6000])
def test_add_normed_and_stream_rows(kernels, dtype, width):
    torch.manual_seed(width)
    hidden = torch.randn(5, width) + 0.5
    weight = (1 + 0.2 * torch.randn(width)).to(dtype)
    plain = TorchKernels(dtype)
    for update in (0.3 * torch.randn(3, 5, width), 2.0 * torch.randn(5, width)):
        plain_hidden, on_device = hidden.clone(), gpu(hidden)
        want = plain.add_normed(plain_hidden, update, weight, 1e-5)
        got = kernels[dtype].add_normed(on_device, gpu(update), gpu(weight), 1e-5)
        close(on_device, plain_hidden, torch.float32)
        close(got, want, dtype)
        assert got.dtype == dtype and (dtype != torch.float32 or got.data_ptr() == on_device.data_ptr())
    plain_hidden, on_device = hidden.clone(), gpu(hidden)
    delta = 0.3 * torch.randn(2, 5, width)
    close(kernels[dtype].stream_rows(on_device, gpu(delta)), plain.stream_rows(plain_hidden, delta), dtype)
    close(on_device, plain_hidden, torch.float32)
    close(kernels[dtype].stream_rows(on_device, None), plain.stream_rows(plain_hidden, None), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("norm,heads,kv_heads,dim,vdim,width,rot", [
    ("head", 6, 2, 24, 40, 48, 10), ("row", 5, 5, 40, 24, 48, 0), (None, 3, 1, 16, 16, 16, 16), ("head", 4, 2, 72, 72, 80, 72), ("row", 2, 1, 70, 3, 80, 6),
])
def test_assemble_heads(kernels, dtype, norm, heads, kv_heads, dim, vdim, width, rot):
    torch.manual_seed(heads * dim)
    tokens, extra = 7, 5
    row = heads * dim + kv_heads * dim + kv_heads * vdim
    x = torch.randn(tokens, extra + row + 3).to(dtype)
    other = torch.randn(tokens, 11 + kv_heads * vdim).to(dtype)
    length = {"head": (dim, dim), "row": (heads * dim, kv_heads * dim), None: (1, 1)}[norm]
    q_weight, k_weight = ((1 + 0.3 * torch.randn(n)).to(dtype) for n in length)
    angles = torch.rand(tokens, max(rot // 2, 1)) * 6.0
    table = torch.stack([angles.cos(), angles.sin()], dim=-1)[:, : rot // 2].contiguous()
    first = (extra, extra + heads * dim, extra + (heads + kv_heads) * dim)
    for given, blend in ((None, 0.0), (other, 0.37)):
        want = TorchKernels(dtype).assemble_heads(x, *first, heads, kv_heads, dim, vdim, width, norm, q_weight, k_weight, 1e-4,
                                                  table if rot else None, rot, given, 11, blend)
        got = kernels[dtype].assemble_heads(gpu(x), *first, heads, kv_heads, dim, vdim, width, norm, gpu(q_weight) if norm else None,
                                            gpu(k_weight) if norm else None, 1e-4, gpu(table) if rot else None, rot,
                                            gpu(given) if given is not None else None, 11, blend)
        close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_scale_heads_and_soft_cap(kernels, dtype):
    torch.manual_seed(3)
    x, gates = torch.randn(9, 5 * 24).to(dtype), (2 * torch.randn(9, 13)).to(dtype)
    want = TorchKernels(dtype).scale_heads(x.clone(), 5, 24, gates, 4, "sigmoid")
    close(kernels[dtype].scale_heads(gpu(x), 5, 24, gpu(gates), 4, "sigmoid"), want, dtype)
    logits = 40 * torch.randn(3, 77)
    close(kernels[dtype].soft_cap(gpu(logits), 12.5), 12.5 * torch.tanh(logits / 12.5), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim", [(16, 32, 128), (32, 16, 128), (40, 16, 64)])
def test_decay_attention_of_many_heads(kernels, dtype, heads, dim, vdim):
    """Enough (head, segment, columns) to go round the chip: a wave then owns two or four tiles of value columns."""
    torch.manual_seed(heads)
    counts = [300, 1, 530]
    tokens, row = sum(counts), 2 * heads * dim + heads * vdim
    decays = (1.0 - 2.0 ** -(1.0 + 8.0 * torch.rand(heads))).to(torch.float32)
    state = 0.5 * torch.randn(4, heads, dim, vdim)
    x = torch.randn(tokens, row).to(dtype)
    batch = step_of(counts, [0] * 3, [2, 0, 3], "cuda")
    plain_state, device_state = state.clone(), gpu(state)
    want = TorchKernels(dtype).decay_attention(x, 0, heads * dim, 2 * heads * dim, heads, dim, vdim, decays, "silu", batch, plain_state)
    got = kernels[dtype].decay_attention(gpu(x), 0, heads * dim, 2 * heads * dim, heads, dim, vdim, gpu(decays), "silu", batch, device_state)
    scale = float(want.abs().max())
    close(got / scale, want / scale, torch.float32, atol=2e-5, rtol=1e-4)
    close(device_state, plain_state, torch.float32, atol=5e-5, rtol=1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("activation", ["silu", "sigmoid"])
@pytest.mark.parametrize("heads,vdim", [(3, 40), (1, 300), (1, 1300)])
def test_gated_head_norm_wide_and_squashed(kernels, dtype, activation, heads, vdim):
    torch.manual_seed(vdim)
    read, gates = 3 * torch.randn(6, heads * vdim), torch.randn(6, 7 + heads * vdim).to(dtype)
    weight = (1 + 0.2 * torch.randn(vdim)).to(dtype)
    want = TorchKernels(dtype).gated_head_norm(read, gates, 7, weight, 1e-5, heads, vdim, activation)
    close(kernels[dtype].gated_head_norm(gpu(read), gpu(gates), 7, gpu(weight), 1e-5, heads, vdim, activation), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim", [(3, 32, 48), (2, 16, 16), (2, 24, 40), (1, 48, 70), (2, 64, 128)])
@pytest.mark.parametrize("counts", [[1, 1, 1], [37, 1, 16], [2, 3, 1], [17, 64, 5], [300, 1, 530], [256, 129, 128]])
def test_decay_attention(kernels, dtype, heads, dim, vdim, counts):
    """Steps of single tokens, of runs that end anywhere, and of both; states carried over; both kernels (sizes that
    are multiples of 16 walk runs on the matrix cores where a request brings four tokens or more, in segments side by
    side where one brings 256 or more)."""
    torch.manual_seed(dim + vdim + sum(counts))
    tokens = sum(counts)
    row = 5 + 2 * heads * dim + heads * vdim  # (the columns begin where 16-byte loads may not: the kernels decide by that)
    row += (-row) % 4
    decays = torch.tensor([0.999, 0.6, 0.93][:heads], dtype=torch.float32)
    state = 0.5 * torch.randn(5, heads, dim, vdim)
    for q_first in (4, 5):
        x = torch.randn(tokens, row).to(dtype)
        firsts = (q_first, q_first + heads * dim, q_first + 2 * heads * dim) if q_first == 4 else (heads * vdim + 1, heads * vdim + 1 + heads * dim, 0)
        if max(firsts[0], firsts[1]) + heads * dim > row:
            continue
        batch = step_of(counts, [0] * len(counts), [3, 0, 4], "cuda")
        plain_state, device_state = state.clone(), gpu(state)
        want = TorchKernels(dtype).decay_attention(x, *firsts, heads, dim, vdim, decays, "silu", batch, plain_state)
        got = kernels[dtype].decay_attention(gpu(x), *firsts, heads, dim, vdim, gpu(decays), "silu", batch, device_state)
        scale = float(want.abs().max())
        close(got / scale, want / scale, torch.float32, atol=2e-5, rtol=1e-4)
        close(device_state, plain_state, torch.float32, atol=2e-5, rtol=1e-4)
        assert torch.equal(device_state[1].cpu(), state[1]) and torch.equal(device_state[2].cpu(), state[2])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,page", [(4, 2, 64, 16), (6, 1, 48, 8), (3, 3, 24, 4)])
@pytest.mark.parametrize("counts,starts", [([1, 1, 1], [700, 3, 40]), ([33, 1, 7], [0, 90, 250]), ([300], [0])])
def test_attention_with_sinks_and_capped_scores(kernels, dtype, heads, kv_heads, dim, page, counts, starts):
    """The sink in the denominator, with and without a cap, a window and key splits, through every attention kernel."""
    from llmserve_amd.cache.cell import CacheCell
    from llmserve_amd.parts import HeadLayout, PagedKeyValue

    torch.manual_seed(dim + sum(counts))
    layout = HeadLayout(heads, kv_heads, dim)
    need = PagedKeyValue(kv_heads, dim, None)
    longest = max(s + c for s, c in zip(starts, counts))
    per = -(-longest // page)
    pages = per * len(counts) + 1
    fields = {name: (0.7 * torch.randn(pages, *shape)).to(dtype) for name, shape in need.page_fields(page).items()}
    order = torch.randperm(pages - 1) + 1
    tables = order[: per * len(counts)].reshape(len(counts), per).to(torch.int32)
    tokens = sum(counts)
    qkv = (0.8 * torch.randn(tokens, layout.width)).to(dtype)
    sinks = torch.tensor([2.5, -1.0, 0.3, 6.0, -30.0, 1.0][:heads], dtype=torch.float32)

    def batch_on(device):
        batch = step_of(counts, starts, list(range(len(counts))), device)
        batch.token_sequence = torch.cat([torch.full((c,), b) for b, c in enumerate(counts)]).to(torch.int32).to(device)
        batch.max_context_length = longest
        batch.context_lengths = torch.tensor([s + c for s, c in zip(starts, counts)], dtype=torch.int32).to(device)
        batch.groups = [types.SimpleNamespace(page_size=page, block_tables=tables.to(device), slot_mapping=None, width=per)]
        batch.padded_to = None
        return batch

    for window, cap in ((None, None), (50, 4.0), (7, None)):
        plain_cell = CacheCell(need, group=0, fields={name: value.clone() for name, value in fields.items()})
        device_cell = CacheCell(need, group=0, fields={name: gpu(value) for name, value in fields.items()})
        want = TorchKernels(dtype).paged_attention(qkv, layout, batch_on("cpu"), plain_cell, 0.2, window, soft_cap=cap, sinks=sinks)
        got = kernels[dtype].paged_attention(gpu(qkv), layout, batch_on("cuda"), device_cell, 0.2, window, soft_cap=cap, sinks=gpu(sinks))
        close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("counts", [[1, 1, 1, 1], [5, 1, 9]])
def test_assemble_heads_stores_keys_and_values(kernels, dtype, counts):
    """A step of single tokens stores in the kernel that puts the heads together, a step of portions in the kernel that
    stores portions: the pages hold the same either way, and only at the step's places."""
    from llmserve_amd.cache.cell import CacheCell
    from llmserve_amd.parts import PagedKeyValue

    torch.manual_seed(sum(counts))
    heads, kv_heads, dim, vdim, width, page = 6, 2, 24, 40, 48, 8
    need = PagedKeyValue(kv_heads, width, None)
    tokens = sum(counts)
    fields = {name: torch.randn(12, *shape).to(dtype) for name, shape in need.page_fields(page).items()}
    slots = torch.randperm(12 * page)[:tokens].to(torch.int32)
    x = torch.randn(tokens, heads * dim + kv_heads * (dim + vdim)).to(dtype)
    weight = (1 + 0.3 * torch.randn(dim)).to(dtype)

    def run(library, device):
        batch = step_of(counts, [3] * len(counts), list(range(len(counts))), device)
        batch.groups = [types.SimpleNamespace(page_size=page, block_tables=None, slot_mapping=slots.to(device), width=0)]
        cell = CacheCell(need, group=0, fields={name: value.clone().to(device) for name, value in fields.items()})
        move = (lambda t: t.to(device))
        rows = library.assemble_heads(move(x), 0, heads * dim, (heads + kv_heads) * dim, heads, kv_heads, dim, vdim, width, "head",
                                      move(weight), move(weight), 1e-5, None, 0, batch=batch, cell=cell)
        return rows, cell

    want_rows, want_cell = run(TorchKernels(dtype), "cpu")
    got_rows, got_cell = run(kernels[dtype], "cuda")
    close(got_rows, want_rows, dtype)
    for name in fields:
        close(got_cell.fields[name], want_cell.fields[name], dtype)
