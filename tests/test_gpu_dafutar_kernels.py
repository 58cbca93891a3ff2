"""The kernels of the Dafutar parts, each alone against the same operation in elementary float32 torch (the CPU
stand-in of the kernel library), at sizes that are no powers of two, with strides, and over steps that cut a
request's tokens anywhere."""

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
    """What the kernels read of a step: request b brings counts[b] tokens from position starts[b] on."""
    chunks = [types.SimpleNamespace(request_id=str(b), slot=slot, start=start, count=count) for b, (count, start, slot) in enumerate(zip(counts, starts, slots))]
    positions = torch.cat([torch.arange(start, start + count) for count, start in zip(counts, starts)]).to(torch.int32)
    sequence = torch.cat([torch.full((count,), b) for b, count in enumerate(counts)]).to(torch.int32)
    query_start = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32)
    return types.SimpleNamespace(
        chunks=chunks, positions=positions.to(device), token_sequence=sequence.to(device), query_start=query_start.to(device),
        state_slots=torch.tensor(slots, dtype=torch.int32).to(device), computed={}, scratch={},
    )


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [24, 30, 328, 1001, 2500])
def test_add_layer_norm(kernels, dtype, width):
    torch.manual_seed(width)
    hidden, delta = torch.randn(5, width) + 0.5, 0.3 * torch.randn(3, 5, width)
    weight, bias = (1 + 0.2 * torch.randn(width)).to(dtype), (0.1 * torch.randn(width)).to(dtype)
    plain_hidden = hidden.clone()
    want = TorchKernels(dtype).add_layer_norm(plain_hidden, delta, weight, bias, 1e-5)
    on_device = gpu(hidden)
    got = kernels[dtype].add_layer_norm(on_device, gpu(delta), gpu(weight), gpu(bias), 1e-5)
    close(got, want, dtype)
    close(on_device, plain_hidden, torch.float32)
    got = kernels[dtype].add_layer_norm(on_device, None, gpu(weight), gpu(bias), 1e-5)
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rms_norm_columns(kernels, dtype):
    torch.manual_seed(1)
    x = torch.randn(6, 50).to(dtype)
    weight = (1 + 0.2 * torch.randn(22)).to(dtype)
    plain = TorchKernels(dtype)
    close(kernels[dtype].rms_norm_columns(gpu(x), 9, gpu(weight), 1e-5), plain.rms_norm_columns(x, 9, weight, 1e-5), dtype)
    out, want = torch.zeros(6, 90).to(dtype), torch.zeros(6, 90).to(dtype)
    plain.rms_norm_columns(x, 28, weight, 1e-3, out=want, out_first=7, copies=3, copy_stride=25)
    got = kernels[dtype].rms_norm_columns(gpu(x), 28, gpu(weight), 1e-3, out=gpu(out), out_first=7, copies=3, copy_stride=25)
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dims,width", [(8, 8), (6, 10)])
def test_rotate_columns(kernels, dtype, dims, width):
    torch.manual_seed(2)
    batch = step_of([3, 1, 4], [0, 1000, 77], [0, 1, 2], "cuda")
    host = step_of([3, 1, 4], [0, 1000, 77], [0, 1, 2], "cpu")
    frequencies = torch.rand(dims // 2) + 0.01
    plain = TorchKernels(dtype)
    table = kernels[dtype].rotary_table(batch, gpu(frequencies), 1.25)
    want_table = plain.rotary_table(host, frequencies, 1.25)
    close(table, want_table, torch.float32, atol=2e-4, rtol=0)
    heads, stride = 3, width + 5
    x = torch.randn(8, 2 + heads * stride).to(dtype)
    out, want = torch.zeros(8, 4 + heads * 20).to(dtype), torch.zeros(8, 4 + heads * 20).to(dtype)
    plain.rotate_columns(x, 2, stride, heads, width, want_table, dims, want, 4, 20)
    got = kernels[dtype].rotate_columns(gpu(x), 2, stride, heads, width, table, dims, gpu(out), 4, 20)
    close(got, want, dtype, atol=1e-3 if dtype == torch.float32 else 3e-2, rtol=0)
    # one source for several heads (a key part that all heads share)
    plain.rotate_columns(x, 3, 0, 2, width, want_table, dims, want, 0, 11)
    got = kernels[dtype].rotate_columns(gpu(x), 3, 0, 2, width, table, dims, got, 0, 11)
    close(got, want, dtype, atol=1e-3 if dtype == torch.float32 else 3e-2, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,heads,outputs,inner,gap", [
    (1, 3, 5, 7, 3), (19, 5, 136, 64, 3), (70, 2, 70, 100, 3),
    # rows that begin at multiples of eight elements and a K in steps of 32: in bfloat16 the matrix cores
    (3, 5, 192, 128, 8), (150, 3, 40, 64, 16), (33, 2, 300, 96, 0),
])
def test_headwise_linear(kernels, dtype, rows, heads, outputs, inner, gap):
    torch.manual_seed(rows)
    stride = inner + gap
    x = torch.randn(rows, 8 + heads * stride).to(dtype)
    weight = (torch.randn(heads, outputs, inner) / inner**0.5).to(dtype)
    plain = TorchKernels(dtype)
    prepared = kernels[dtype].prepare_headwise_linear(gpu(weight))
    first = 8 if gap % 8 == 0 else 4
    close(kernels[dtype].headwise_linear(gpu(x), first, stride, prepared), plain.headwise_linear(x, first, stride, weight.float()), dtype)
    out, want = torch.zeros(rows, 2 + heads * (outputs + 6)).to(dtype), torch.zeros(rows, 2 + heads * (outputs + 6)).to(dtype)
    plain.headwise_linear(x, first, stride, weight.float(), out=want, out_first=2, out_head_stride=outputs + 6)
    got = kernels[dtype].headwise_linear(gpu(x), first, stride, prepared, out=gpu(out), out_first=2, out_head_stride=outputs + 6)
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_join_activate_and_gated_add(kernels, dtype):
    torch.manual_seed(3)
    hidden, delta, other = torch.randn(5, 40), torch.randn(2, 5, 40), torch.randn(5, 40)
    plain = TorchKernels(dtype)
    close(kernels[dtype].join_rows(gpu(hidden), gpu(delta), gpu(other)), plain.join_rows(hidden, delta, other), dtype)
    close(kernels[dtype].join_rows(gpu(hidden), None, gpu(other)), plain.join_rows(hidden, None, other), dtype)
    x = (3 * torch.randn(7, 33)).to(dtype)
    for activation in ("gelu", "gelu_tanh", "silu", "relu"):
        close(kernels[dtype].activate(gpu(x), activation), plain.activate(x, activation), dtype)
    target, rows, gates = torch.randn(5, 40), torch.randn(5, 40), torch.randn(5, 9)
    want = plain.add_gated_rows(target.clone(), rows, gates, 8, "sigmoid")
    close(kernels[dtype].add_gated_rows(gpu(target), gpu(rows), gpu(gates), 8, "sigmoid"), want, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,experts,top,hidden,size", [
    (1, 4, 4, 32, 16), (37, 8, 2, 96, 40), (200, 5, 3, 64, 72),
    # sizes in steps of 32: in bfloat16 the matrix cores, tiles of 16 rows for a few rows an expert and of 64 for many
    (5, 8, 2, 64, 32), (300, 4, 2, 64, 96), (130, 3, 1, 320, 64), (700, 3, 2, 192, 320), (1000, 2, 1, 128, 64),
])
def test_routed_experts(kernels, dtype, tokens, experts, top, hidden, size):
    torch.manual_seed(tokens)
    scores = 2 * torch.randn(tokens, experts + 1)
    correction = 0.5 * torch.randn(experts)
    plain = TorchKernels(dtype)
    want_chosen, want_weights = plain.route(scores, experts, correction, top, 1.5, "sigmoid")
    chosen, weights = kernels[dtype].route(gpu(scores), experts, gpu(correction), top, 1.5, "sigmoid")
    assert torch.equal(chosen.cpu(), want_chosen)
    close(weights, want_weights, torch.float32)
    x = torch.randn(tokens, hidden).to(dtype)
    ups = [(torch.randn(size, hidden) / hidden**0.5).to(dtype) for _ in range(experts)]
    downs = [(torch.randn(hidden, size) / size**0.5).to(dtype) for _ in range(experts)]
    want = plain.expert_feed_forward(x, plain.prepare_experts(ups, downs, "gelu"), want_chosen, want_weights)
    prepared = kernels[dtype].prepare_experts([gpu(w) for w in ups], [gpu(w) for w in downs], "gelu")
    got = kernels[dtype].expert_feed_forward(gpu(x), prepared, chosen, weights)
    close(got, want, dtype)
    again = kernels[dtype].expert_feed_forward(gpu(x), prepared, chosen, weights)
    assert torch.equal(got, again)  # whatever order the sort gave the rows of an expert
    shared = torch.randn(tokens, hidden)
    want = plain.expert_feed_forward(x, plain.prepare_experts(ups, downs, "gelu"), want_chosen, want_weights, shared=shared, gates=scores, gate_column=experts)
    got = kernels[dtype].expert_feed_forward(gpu(x), prepared, chosen, weights, shared=gpu(shared), gates=gpu(scores), gate_column=experts)
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_causal_conv_over_steps(kernels, dtype, taps):
    """Three requests in slots that are not their order, over steps of 1 to 9 tokens (fewer than taps - 1 too);
    the kept inputs carry from step to step."""
    torch.manual_seed(taps)
    channels, extra = 70, 13
    weights = torch.randn(channels, taps) / taps**0.5
    plain = TorchKernels(dtype)
    slots = [2, 0, 3]
    window = torch.zeros(5, taps - 1, channels) if taps > 1 else None
    on_device = gpu(window) if window is not None else None
    for counts in ([9, 1, 2], [1, 1, 1], [2, 5, 1], [3, 1, 8]):
        x = torch.randn(sum(counts), channels + extra).to(dtype)
        want = plain.causal_conv(x, channels, weights, "silu", step_of(counts, [0] * 3, slots, "cpu"), window)
        got = kernels[dtype].causal_conv(gpu(x), channels, gpu(weights), "silu", step_of(counts, [0] * 3, slots, "cuda"), on_device)
        close(got, want, dtype)
        if window is not None:
            close(on_device, window, torch.float32, atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim", [(6, 2, 64, 32), (2, 2, 16, 96), (4, 1, 80, 32), (3, 3, 130, 70)])
def test_gated_delta_rule_over_steps(kernels, dtype, heads, kv_heads, dim, vdim):
    torch.manual_seed(dim)
    plain = TorchKernels(dtype)
    slots = [1, 3]
    state = torch.zeros(5, heads, vdim, dim)
    on_device = gpu(state)
    rate, bias = torch.randn(heads) - 1.0, torch.randn(heads)
    for counts in ([11, 1], [1, 1], [2, 6]):
        tokens = sum(counts)
        mixed = torch.randn(tokens, 2 * kv_heads * dim + heads * vdim).to(dtype)
        controls = 2 * torch.randn(tokens, 2 * heads)
        want = plain.gated_delta_rule(mixed, controls, rate, bias, heads, kv_heads, dim, vdim, step_of(counts, [0, 0], slots, "cpu"), state)
        got = kernels[dtype].gated_delta_rule(
            gpu(mixed), gpu(controls), gpu(rate), gpu(bias), heads, kv_heads, dim, vdim, step_of(counts, [0, 0], slots, "cuda"), on_device
        )
        close(got, want, torch.float32, atol=2e-4, rtol=2e-4)
        close(on_device, state, torch.float32, atol=2e-4, rtol=2e-4)
    assert float(on_device[0].abs().max()) == 0.0 and float(on_device[2].abs().max()) == 0.0  # other requests' slots untouched


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,vdim", [(5, 64), (3, 70), (2, 200)])
def test_gated_head_norm(kernels, dtype, heads, vdim):
    torch.manual_seed(vdim)
    read = torch.randn(9, heads * vdim)
    gates = torch.randn(9, 5 + heads * vdim).to(dtype)
    weight = (1 + 0.2 * torch.randn(vdim)).to(dtype)
    want = TorchKernels(dtype).gated_head_norm(read, gates, 5, weight, 1e-5, heads, vdim, "silu")
    got = kernels[dtype].gated_head_norm(gpu(read), gpu(gates), 5, gpu(weight), 1e-5, heads, vdim, "silu")
    close(got, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,taps", [(6, 2, 64, 32, 4), (2, 2, 16, 96, 1), (4, 1, 80, 32, 3), (3, 3, 130, 70, 2), (2, 1, 32, 48, 6)])
def test_convolutions_and_delta_rule_in_one(kernels, dtype, heads, kv_heads, dim, vdim, taps):
    """The fused form against the two operations one after the other, over steps of many tokens, of one and of two."""
    torch.manual_seed(dim + taps)
    plain = TorchKernels(torch.float32)  # (the fused form keeps what lies between the two in float32)
    channels = 2 * kv_heads * dim + heads * vdim
    weights = torch.randn(channels, taps) / taps**0.5
    slots = [1, 3]
    state, window = torch.zeros(5, heads, vdim, dim), (torch.zeros(5, taps - 1, channels) if taps > 1 else None)
    on_device, window_on_device = gpu(state), (gpu(window) if window is not None else None)
    rate, bias = torch.randn(heads) - 1.0, torch.randn(heads)
    for counts in ([37, 1], [1, 1], [2, 1], [2, 19]):
        tokens = sum(counts)
        projected = torch.randn(tokens, channels + 11).to(dtype)
        controls = 2 * torch.randn(tokens, 2 * heads)
        host, device = step_of(counts, [0, 0], slots, "cpu"), step_of(counts, [0, 0], slots, "cuda")
        device.max_query_length = max(counts)
        want = plain.conv_gated_delta_rule(projected.float(), channels, weights, "silu", controls, rate, bias, heads, kv_heads, dim, vdim, host, window, state)
        got = kernels[dtype].conv_gated_delta_rule(
            gpu(projected), channels, gpu(weights), "silu", gpu(controls), gpu(rate), gpu(bias), heads, kv_heads, dim, vdim, device,
            window_on_device, on_device,
        )
        close(got, want, torch.float32, atol=3e-4, rtol=3e-4)
        close(on_device, state, torch.float32, atol=3e-4, rtol=3e-4)
        if window is not None:
            close(window_on_device, window, torch.float32, atol=0, rtol=0)
