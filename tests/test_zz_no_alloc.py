"""The allocation-free index build (fma_moe_build_index_static: scratch in a fixed device array of the library) against
fma_moe_build_index with a caller-supplied workspace, through the C ABI: identical outputs on two calls in a row, the
second on a smaller input (the array keeps the first call's contents), and a size beyond the array is refused."""

import pytest
import torch

from fma import _lib

pytestmark = pytest.mark.gpu


def _routing(R, E, seed):
    g = torch.Generator().manual_seed(seed)
    # skewed, with the last expert empty
    p = 1.0 / torch.arange(1, E + 1, dtype=torch.float64)
    p[-1] = 0
    return torch.multinomial(p / p.sum(), R, replacement=True, generator=g).to(torch.int32)


def _outputs(R, E, dev):
    return [
        torch.full((E,), -1, dtype=torch.int32, device=dev),
        torch.full((E,), -1, dtype=torch.int32, device=dev),
        torch.full((R,), -1, dtype=torch.int32, device=dev),
        torch.full((R,), -1, dtype=torch.int32, device=dev),
        torch.full((R,), -1, dtype=torch.int32, device=dev),
    ]


@pytest.mark.parametrize("id_dtype", [torch.int32, torch.int64])
def test_static_scratch_index_build_matches_workspace_version(lib, id_dtype):
    dev = torch.device("cuda", 0)
    stream = torch.cuda.current_stream(dev).cuda_stream
    assert lib.fma_moe_build_index_static_max_words() > 0  # (also resolves the array's address on this device)
    for R, E, seed in ((262144, 64, 1), (5000, 16, 2)):  # the second call is smaller and finds the first one's scratch
        ids = _routing(R, E, seed).to(id_dtype).to(dev)
        ws = torch.empty(lib.fma_moe_build_index_workspace_bytes(R, E), dtype=torch.uint8, device=dev)
        ref, got = _outputs(R, E, dev), _outputs(R, E, dev)
        rc = lib.fma_moe_build_index(ids.data_ptr(), ids.element_size(), R, E, *[t.data_ptr() for t in ref],
                                     ws.data_ptr(), ws.numel(), stream)
        _lib.check(rc, "fma_moe_build_index")
        torch.cuda.synchronize()
        # what defines the entry point: the call takes no device memory (neither from the driver nor from torch's pool)
        free_before, _ = torch.cuda.mem_get_info(dev)
        reserved_before = torch.cuda.memory_reserved(dev)
        rc = lib.fma_moe_build_index_static(ids.data_ptr(), ids.element_size(), R, E, *[t.data_ptr() for t in got],
                                            stream)
        _lib.check(rc, "fma_moe_build_index_static")
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info(dev)
        assert free_after == free_before and torch.cuda.memory_reserved(dev) == reserved_before, "the call allocated device memory"
        for name, a, b in zip(("counts", "offsets", "perm", "eid", "inv"), ref, got):
            assert torch.equal(a, b), f"{name} differs (R={R}, E={E})"
        assert int(ref[0].sum()) == R and sorted(got[2].tolist()) == list(range(R))


def test_static_scratch_index_build_refuses_oversized_input(lib):
    dev = torch.device("cuda", 0)
    words = lib.fma_moe_build_index_static_max_words()
    E = 1024
    R = (words // E + 1) * 512  # one chunk of 512 slots more than the array holds
    assert lib.fma_moe_build_index_workspace_bytes(R, E) > 4 * words
    ids = torch.zeros(R, dtype=torch.int32, device=dev)
    out = _outputs(R, E, dev)
    rc = lib.fma_moe_build_index_static(ids.data_ptr(), 4, R, E, *[t.data_ptr() for t in out], None)
    assert rc == -7 and "scratch" in lib.fma_last_error_string().decode()
    torch.cuda.synchronize()
    assert all(bool((t == -1).all()) for t in out), "a refused call must launch nothing"


def test_static_scratch_index_build_under_graph_capture(lib):
    """The use the entry point exists for: recorded into a HIP graph (no allocation may happen during capture) and replayed
    on new ids, each replay against the workspace version run eagerly."""
    dev = torch.device("cuda", 0)
    R, E = 40000, 32
    assert lib.fma_moe_build_index_static_max_words() * 4 >= lib.fma_moe_build_index_workspace_bytes(R, E)
    ids = _routing(R, E, 3).to(dev)
    got = _outputs(R, E, dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # one eager call first, as for any captured region
        _lib.check(lib.fma_moe_build_index_static(ids.data_ptr(), 4, R, E, *[t.data_ptr() for t in got], side.cuda_stream),
                   "fma_moe_build_index_static")
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = torch.cuda.current_stream(dev).cuda_stream
        _lib.check(lib.fma_moe_build_index_static(ids.data_ptr(), 4, R, E, *[t.data_ptr() for t in got], st),
                   "fma_moe_build_index_static (captured)")
    ws = torch.empty(lib.fma_moe_build_index_workspace_bytes(R, E), dtype=torch.uint8, device=dev)
    for seed in (4, 5, 6):
        ids.copy_(_routing(R, E, seed).to(dev))
        for t in got:
            t.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        ref = _outputs(R, E, dev)
        _lib.check(lib.fma_moe_build_index(ids.data_ptr(), 4, R, E, *[t.data_ptr() for t in ref], ws.data_ptr(), ws.numel(),
                                           torch.cuda.current_stream(dev).cuda_stream), "fma_moe_build_index")
        torch.cuda.synchronize()
        for name, a, b in zip(("counts", "offsets", "perm", "eid", "inv"), ref, got):
            assert torch.equal(a, b), f"{name} differs on the replay with seed {seed}"
