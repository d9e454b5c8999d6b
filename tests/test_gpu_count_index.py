"""GPU parity of continuous_count and the routing-index construction: bit-exact against the CPU oracle."""

import numpy as np
import pytest
import torch

from fma import KernelBackend, continuous_count
from fma.modules.moe.cuda_implementation import build_routing_index
from oracle import c_oracle, moe_oracle as O
from synthetic_inputs import make_ids, make_routing

from gpu_util import DEV, to_np

pytestmark = pytest.mark.gpu


def _sizes():
    sizes = set()
    for i in range(15):
        for j in range(3):
            sizes.add(2**i + j)
    rng = np.random.default_rng(0)
    sizes.update(int(s) for s in rng.integers(2000, 4001, size=10))
    return sorted(sizes)


@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_count_reference_generator(dtype):
    # randint(0, 72), seed 42, exact equality: the reference's test (tests/ops/continuous_count_test.py:20-41)
    for n in _sizes():
        torch.manual_seed(42)
        x = torch.randint(0, 72, (n,), dtype=dtype)
        got = continuous_count(x=x.to(DEV), size=72)
        assert got.dtype == torch.uint32 and got.shape == (72,)
        assert np.array_equal(to_np(got), O.continuous_count(x.numpy(), 72)), f"n={n}"


@pytest.mark.parametrize("kind", ["uniform", "zipf"])
@pytest.mark.parametrize("np_dtype,dtype", [(np.int32, torch.int32), (np.int64, torch.int64)])
def test_count_16m_ids(kind, np_dtype, dtype):
    # the histogram benchmark configuration: 16 Mi ids in [0, 64), uniform and Zipf(1.2)
    n, E = 16 << 20, 64
    ids = make_ids(n, E, kind, seed=11, dtype=np_dtype)
    x = torch.from_numpy(ids).to(DEV)
    expect = c_oracle.continuous_count(ids, E)
    for _ in range(3):  # back-to-back calls must not see each other's partial histograms
        got = to_np(continuous_count(x, E, kernel_backend=KernelBackend.cuda))
        assert np.array_equal(got, expect)
    assert int(got.astype(np.int64).sum()) == n


@pytest.mark.parametrize("E", [2, 3, 72, 129, 1000, 4096, 16384])
def test_count_bin_counts(E):
    ids = make_ids(300_007, E, "zipf", seed=E, dtype=np.int64)
    got = to_np(continuous_count(torch.from_numpy(ids).to(DEV), E))
    assert np.array_equal(got, c_oracle.continuous_count(ids, E))


def test_count_edge_cases():
    assert to_np(continuous_count(torch.zeros(0, dtype=torch.int32, device=DEV), 8)).tolist() == [0] * 8
    assert to_np(continuous_count(torch.full((5,), 3, dtype=torch.int64, device=DEV), 1)).tolist() == [5]
    x = torch.tensor([0, 7, 8, -1, 3, 3, 100, 7], dtype=torch.int32)  # ids outside [0, 8) are ignored
    assert to_np(continuous_count(x.to(DEV), 8)).tolist() == [1, 0, 0, 2, 0, 0, 0, 2]
    x = torch.full((100_001,), 5, dtype=torch.int32)  # every lane hits one bin
    assert to_np(continuous_count(x.to(DEV), 64))[5] == 100_001


@pytest.mark.parametrize(
    "T,E,k,kind,empty",
    [
        (7, 8, 2, "uniform", 0),
        (512, 8, 2, "uniform", 0),
        (1, 4, 4, "uniform", 0),
        (333, 5, 3, "uniform", 0),
        (16384, 8, 2, "uniform", 0),  # Mixtral shape
        (32768, 64, 8, "zipf", 4),  # fine-grained, ragged, four empty experts
        (8192, 128, 8, "uniform", 0),  # large expert count
        (1000, 1024, 8, "zipf", 100),
    ],
)
@pytest.mark.parametrize("dtype", [torch.int64, torch.int32])
def test_routing_index(T, E, k, kind, empty, dtype):
    selected, _ = make_routing(T, E, k, kind, seed=T + E, empty_tail=empty)
    expect = c_oracle.routing_index(selected.numpy(), E)
    counts, offsets, perm, eid, inv = build_routing_index(selected.to(dtype).to(DEV), E)
    assert np.array_equal(to_np(counts), expect["counts"])
    assert np.array_equal(to_np(offsets), expect["offsets"])
    assert np.array_equal(to_np(perm), expect["perm"])
    assert np.array_equal(to_np(eid), expect["eid"])
    assert np.array_equal(to_np(inv), expect["inv"])
    # and against the library routine the reference itself calls, made stable
    sorted_ids, sorted_slots = selected.flatten().sort(stable=True)
    assert np.array_equal(to_np(perm), sorted_slots.numpy().astype(np.int32))
    assert np.array_equal(to_np(eid), sorted_ids.numpy().astype(np.int32))
    if empty:
        assert (to_np(counts)[-empty:] == 0).all()


@pytest.mark.parametrize(
    "T,E,k,kind,empty",
    [
        (7, 8, 2, "uniform", 0),
        (1, 4, 4, "uniform", 0),
        (333, 5, 3, "uniform", 0),  # 48 slots per block of 16 tokens: chunks of 10 blocks, the last one short
        (16384, 8, 2, "uniform", 0),  # Mixtral shape
        (16384, 64, 6, "zipf", 4),  # fine-grained: 96 slots per block, chunks of 5 blocks
        (32768, 64, 8, "zipf", 4),
        (8192, 128, 8, "uniform", 0),
        (1000, 1024, 8, "zipf", 100),
        (100, 64, 64, "uniform", 0),  # 1024 slots per block: the placement's long chunk
        (530, 80, 40, "uniform", 0),  # 640 slots per block
    ],
)
def test_routing_index_from_token_block_histogram(T, E, k, kind, empty):
    # the two-launch build that starts from per-16-token histograms (as the router kernel writes them, here counted
    # with numpy): the same five arrays as the oracle's, and the histogram may be consumed
    selected, _ = make_routing(T, E, k, kind, seed=T + E, empty_tail=empty)
    expect = c_oracle.routing_index(selected.numpy(), E)
    hist = np.zeros(((T + 15) // 16, E), dtype=np.int32)
    np.add.at(hist, (np.repeat(np.arange(T) // 16, k), selected.numpy().reshape(-1)), 1)
    got = build_routing_index(
        selected.to(torch.int32).to(DEV), E, token_block_histogram=torch.from_numpy(hist).to(DEV).view(torch.uint32)
    )
    for a, key in zip(got, ("counts", "offsets", "perm", "eid", "inv")):
        assert np.array_equal(to_np(a), expect[key]), key


def test_routing_index_fixture():
    # tests/golden/routing_index_4096.npz: 4096 skewed ids, three empty experts, answers from numpy
    import os

    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "routing_index_4096.npz"))
    for dtype in (torch.int32, torch.int64):
        ids = torch.from_numpy(fx["ids"]).to(dtype).to(DEV)
        assert np.array_equal(to_np(continuous_count(x=ids, size=64)), fx["counts"])
        counts, offsets, perm, eid, inv = build_routing_index(ids.view(-1, 1), 64)
        for got, key in ((counts, "counts"), (offsets, "offsets"), (perm, "perm"), (eid, "eid"), (inv, "inv")):
            assert np.array_equal(to_np(got), fx[key]), f"{key} ({dtype})"
