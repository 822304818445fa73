"""itexhip_quantize_dynamic_static: the entry point that allocates nothing (its partial ranges live in a fixed array of
the library's own device memory) against itexhip_quantize_dynamic (caller-provided workspace), through the C ABI.
Bit-exact: the quantized bytes and the six floats of the range / parameter block.  Two calls in a row, the second on
a smaller input, so that what the first call left in the shared array must not leak into the second."""
import numpy as np
import pytest

from oracle import pyoracle as orc

pytestmark = pytest.mark.gpu


def _pair(hip, torch, dev, x, T, mode):
    n = x.size
    x_d = torch.from_numpy(x).to(dev)
    tdt = torch.int8 if T == orc.QINT8 else torch.uint8
    q_ref = torch.zeros(n, dtype=tdt, device=dev)
    q_new = torch.zeros(n, dtype=tdt, device=dev)
    state = torch.full((hip.DYNAMIC_STATE_FLOATS,), float("nan"), dtype=torch.float32, device=dev)
    rng_out = torch.full((8,), float("nan"), dtype=torch.float32, device=dev)
    hip.quantize_dynamic(x_d, q_ref, n, T, mode, 0.01, state)
    hip.quantize_dynamic_static(x_d, q_new, n, T, mode, 0.01, rng_out)
    torch.cuda.synchronize()
    return q_ref.cpu().numpy(), q_new.cpu().numpy(), state[:6].cpu().numpy(), rng_out[:6].cpu().numpy()


@pytest.mark.parametrize("T,mode", [(orc.QUINT8, orc.MIN_FIRST), (orc.QINT8, orc.SCALED), (orc.QINT8, 3)])
def test_static_scratch_entry_matches_workspace_entry(hip, dev, T, mode):
    import torch
    rng = np.random.default_rng(17)
    # first call: 512 partial ranges in use, several grid-stride rounds, a tail of 3 elements; the extremes sit in
    # different workgroups' shares
    n1 = (1 << 23) + 3
    x1 = rng.standard_normal(n1).astype(np.float32)
    x1[5_000_000] = 41.0
    x1[123] = -37.5
    q_ref, q_new, st_ref, st_new = _pair(hip, torch, dev, x1, T, mode)
    np.testing.assert_array_equal(q_new, q_ref)
    np.testing.assert_array_equal(st_new.view(np.uint32), st_ref.view(np.uint32))
    assert st_new[0] == -37.5 and st_new[1] == 41.0
    # against the oracle as well, on a window
    omode = orc.MIN_FIRST if mode == 3 else mode
    _, q_orc, omn, omx = orc.quantize_v2(x1, x1.min(), x1.max(), T, omode, classic=(mode == 3))
    np.testing.assert_array_equal(q_new, q_orc)
    assert st_new[2] == omn[0] and st_new[3] == omx[0]
    # second call, smaller (17 partial ranges; a narrower range than what the first call left behind)
    n2 = 134400
    x2 = (rng.standard_normal(n2) * 0.25).astype(np.float32)
    q_ref, q_new, st_ref, st_new = _pair(hip, torch, dev, x2, T, mode)
    np.testing.assert_array_equal(q_new, q_ref)
    np.testing.assert_array_equal(st_new.view(np.uint32), st_ref.view(np.uint32))
    assert st_new[0] == x2.min() and st_new[1] == x2.max()
    # third, tiny: one partial range
    x3 = np.array([0.5, -0.25, 0.125, 2.0, 1.0], np.float32)
    q_ref, q_new, st_ref, st_new = _pair(hip, torch, dev, x3, T, mode)
    np.testing.assert_array_equal(q_new, q_ref)
    np.testing.assert_array_equal(st_new.view(np.uint32), st_ref.view(np.uint32))


def test_static_scratch_entry_rejects_what_it_cannot_take(hip, dev):
    import torch
    x = torch.zeros(64, dtype=torch.float32, device=dev)
    q = torch.zeros(64, dtype=torch.int8, device=dev)
    r = torch.zeros(8, dtype=torch.float32, device=dev)
    with pytest.raises(hip.ItexHipError, match="2\\^36"):
        hip.quantize_dynamic_static(x, q, (1 << 36) + 4, orc.QINT8, orc.SCALED, 0.01, r)   # rejected before any launch
    with pytest.raises(hip.ItexHipError, match="at least 4"):
        hip.quantize_dynamic_static(x, q, 3, orc.QINT8, orc.SCALED, 0.01, r)
    with pytest.raises(hip.ItexHipError, match="aligned"):
        hip.quantize_dynamic_static(x[1:], q, 32, orc.QINT8, orc.SCALED, 0.01, r)
    with pytest.raises(hip.ItexHipError):
        hip.quantize_dynamic_static(x, q, 64, orc.QINT8, orc.MIN_FIRST, 0.01, r)   # MIN_FIRST quantizes to quint8


def test_static_scratch_entry_in_a_hip_graph(hip, dev):
    """After one ordinary call on the device the entry point only launches kernels, so it can be captured into a HIP
    graph.  The graph is replayed on new input contents with eager work and synchronisations between the replays,
    and every replay must leave the bytes itexhip_quantize_dynamic leaves for the same input."""
    import torch
    T, mode = orc.QUINT8, orc.MIN_FIRST
    n = (1 << 20) + 8
    x_static = torch.zeros(n, dtype=torch.float32, device=dev)
    q_graph = torch.zeros(n, dtype=torch.uint8, device=dev)
    r_graph = torch.zeros(8, dtype=torch.float32, device=dev)
    q_eager = torch.zeros(n, dtype=torch.uint8, device=dev)
    state = torch.zeros(hip.DYNAMIC_STATE_FLOATS, dtype=torch.float32, device=dev)
    hip.quantize_dynamic_static(x_static, q_graph, n, T, mode, 0.01, r_graph)   # resolves the array's address: not capturable
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        hip.quantize_dynamic_static(x_static, q_graph, n, T, mode, 0.01, r_graph, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    rng = np.random.default_rng(5)
    for rep in range(4):
        x = (rng.standard_normal(n) * (0.5 + rep)).astype(np.float32)
        x_static.copy_(torch.from_numpy(x).to(dev))
        q_graph.fill_(7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        hip.quantize_dynamic(x_static, q_eager, n, T, mode, 0.01, state)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(q_graph.cpu().numpy(), q_eager.cpu().numpy())
        np.testing.assert_array_equal(r_graph[:6].cpu().numpy().view(np.uint32), state[:6].cpu().numpy().view(np.uint32))
        _, q_orc, _, _ = orc.quantize_v2(x, x.min(), x.max(), T, mode)
        np.testing.assert_array_equal(q_graph.cpu().numpy(), q_orc)
