"""GPU parity of the reference's padded grouping interface (group_with_padding / ungroup_with_padding and the padding
offsets), forward and backward, against a row-by-row restatement of what the reference's kernels write."""

import pytest
import torch

from fma.modules.moe.cuda_implementation import (
    _get_expert_padding_offset,
    build_routing_index,
    group_with_padding,
    ungroup_with_padding,
)
from oracle import moe_oracle as O
from synthetic_inputs import make_routing

from gpu_util import DEV

pytestmark = pytest.mark.gpu


def test_padding_offsets_closed_form():
    # pad[e] = p - (M_e mod p) in [1, p]: a multiple of p still gets p rows
    # (fma/modules/moe/cuda_implementation/padded_expert_frequency_kernel.py:14-24)
    freq = torch.tensor([0, 1, 7, 8, 9, 16, 1000], dtype=torch.int64).to(torch.uint32).to(DEV)
    padded, offset = _get_expert_padding_offset(freq, 7, 8)
    assert padded.cpu().to(torch.int64).tolist() == [8, 8, 8, 16, 16, 24, 1008]
    assert offset.cpu().tolist() == [0, 8, 15, 16, 24, 31, 39, 47]


@pytest.mark.parametrize("pad", [1, 8])
@pytest.mark.parametrize("T,E,k,H,kind,empty", [(37, 4, 2, 64, "uniform", 0), (200, 16, 4, 128, "zipf", 3)])
def test_group_and_ungroup_with_padding(pad, T, E, k, H, kind, empty):
    selected, _ = make_routing(T, E, k, kind, seed=3, empty_tail=empty)
    R = T * k
    freq, _, scattered, sorted_e, _ = build_routing_index(selected.to(DEV), E)
    torch.manual_seed(pad + T)
    x = torch.randn(T, H).bfloat16().to(DEV).requires_grad_()

    out, padded_freq, pad_off = group_with_padding(x, freq, sorted_e, scattered, k, pad)
    counts = freq.cpu().to(torch.int64)
    if pad == 1:
        assert pad_off is None and out.shape == (R, H) and torch.equal(padded_freq, freq)
        off = torch.zeros(E + 1, dtype=torch.int64)
    else:
        assert out.shape == ((-(-R // pad) + E) * pad, H)  # the reference's data-independent shape
        off = pad_off.cpu()
        assert torch.equal(padded_freq.cpu().to(torch.int64), counts + (pad - counts % pad))
    # row by row: grouped row i of expert e sits at i + off[e] and holds the token of its slot; the rest is zero
    expect = torch.zeros(out.shape, dtype=torch.bfloat16)
    sc, se, xc = scattered.cpu().long(), sorted_e.cpu().long(), x.detach().cpu()
    dst = torch.arange(R) + off[se]
    for i in range(R):
        expect[dst[i]] = xc[sc[i] // k]
    used = torch.zeros(out.size(0), dtype=torch.bool)
    used[dst] = True
    assert torch.equal(out.detach().cpu()[used], expect[used])
    if pad != 1:
        assert not out.detach().cpu()[~used].any()

    # backward of the grouping: every token receives the sum of its k grouped rows
    g = torch.randn(out.shape).bfloat16().to(DEV)
    out.backward(g)
    gx = torch.zeros(T, H, dtype=torch.float32)
    gc = g.cpu().float()
    for i in range(R):
        gx[sc[i] // k] += gc[dst[i]]
    assert (x.grad.cpu().float() - gx).abs().max() <= 2**-7 * gx.abs().max()

    # ungrouping returns every slot's row; its backward scatters the slot gradients back and zeroes the padding
    y = out.detach().clone().requires_grad_()
    u = ungroup_with_padding(y, pad_off, sorted_e, scattered, k, T, pad)
    assert u.shape == (T, k, H)
    assert torch.equal(u.detach().cpu().view(R, H), xc.repeat_interleave(k, dim=0))
    gu = torch.randn(T, k, H).bfloat16().to(DEV)
    u.backward(gu)
    expect_gy = torch.zeros(out.shape, dtype=torch.bfloat16)
    expect_gy[dst] = gu.cpu().view(R, H)[sc]
    assert torch.equal(y.grad.cpu()[used], expect_gy[used])
    if pad != 1:
        assert not y.grad.cpu()[~used].any()
