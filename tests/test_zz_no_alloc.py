"""mxp_checksum32_static (the entry point that allocates nothing) against mxp_checksum32 and the oracle.

Two calls in a row share the GPU's scratch array, the second with a smaller input: whatever the
first call left in the descriptor tables and accumulators must not leak into the second.
"""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dev(arr: np.ndarray) -> torch.Tensor:
    if arr.size == 0:
        return torch.empty(0, dtype=torch.uint8, device="cuda")
    return torch.from_numpy(arr.copy()).cuda()


def test_static_checksum_matches_allocating_entry_point(gpu_engine, oracle_c):
    rng = np.random.default_rng(77)
    first = [rng.integers(0, 256, n, dtype=np.uint8) for n in
             (0, 1, 15, 16, 17, 4096, 65537, 8192 * 3 + 5, 1 << 20, (1 << 22) + 12345, 3 << 20)]
    second = [rng.integers(0, 256, n, dtype=np.uint8) for n in (5, 70000, 4097)]
    for bufs in (first, second):
        dev = [_dev(b) for b in bufs]
        got = gpu_engine.checksum32_static(dev)
        assert got == gpu_engine.checksum32(dev)
        assert got == [oracle_c.checksum32(b) for b in bufs]
    # unaligned views take the narrow access paths
    base = rng.integers(0, 256, 70000, dtype=np.uint8)
    d = _dev(base)
    views = [d[off: off + n] for off, n in ((1, 1000), (3, 65000), (13, 16), (16, 50000))]
    assert gpu_engine.checksum32_static(views) == gpu_engine.checksum32(views)
    assert gpu_engine.checksum32_static([]) == []


def test_static_checksum_limits(gpu_engine, mxp):
    d = torch.zeros(16, dtype=torch.uint8, device="cuda")
    with pytest.raises(mxp.MxpError) as too_many:
        gpu_engine.checksum32_static([d] * 1025)
    assert too_many.value.code == mxp.ERR_ARG and "1024" in too_many.value.message
    # a claimed size beyond the scratch's workgroup table is refused before anything is launched
    with pytest.raises(mxp.MxpError) as too_big:
        gpu_engine.checksum32_static([d], nbytes=[13 << 30])
    assert too_big.value.code == mxp.ERR_ARG and "12 GiB" in too_big.value.message
    # and the scratch is still usable afterwards
    assert gpu_engine.checksum32_static([d]) == gpu_engine.checksum32([d])


def test_static_checksum_second_engine_shares_the_scratch(gpu_engine, oracle_c):
    """Another engine on the same GPU resolves the same array; calls one after the other stay correct."""
    from modelexpress_amd.engine import PlacementEngine

    rng = np.random.default_rng(78)
    a = rng.integers(0, 256, 300001, dtype=np.uint8)
    b = rng.integers(0, 256, 1234, dtype=np.uint8)
    other = PlacementEngine(0)
    try:
        assert gpu_engine.checksum32_static([_dev(a)]) == [oracle_c.checksum32(a)]
        assert other.checksum32_static([_dev(b)]) == [oracle_c.checksum32(b)]
        assert gpu_engine.checksum32_static([_dev(b), _dev(a)]) == [oracle_c.checksum32(b), oracle_c.checksum32(a)]
    finally:
        other.close()


def test_static_checksum_refuses_a_capturing_stream_and_leaves_the_capture_valid(gpu_engine, mxp):
    """The call waits for its stream and returns host results, so it cannot be recorded: a stream under capture is
    refused before anything is queued, and the caller's graph still captures and replays."""
    x = torch.zeros(1024, dtype=torch.int32, device="cuda")
    d = torch.arange(4096, dtype=torch.int32, device="cuda").view(torch.uint8)
    want = gpu_engine.checksum32([d])
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            x.add_(1)
            with pytest.raises(mxp.MxpError) as refused:
                gpu_engine.checksum32_static([d], stream=torch.cuda.current_stream().cuda_stream)
            x.add_(2)
    assert refused.value.code == mxp.ERR_STATE and "captured" in refused.value.message
    torch.cuda.synchronize()
    for replay in range(2):
        graph.replay()
        torch.cuda.synchronize()
        assert int(x[0]) == 3 * (replay + 1)
    assert gpu_engine.checksum32_static([d]) == want  # and the entry point works as before outside a capture
