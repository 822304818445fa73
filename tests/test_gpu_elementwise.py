"""GPU parity: QuantizeV2 / Dequantize / RequantizePerChannel / range reductions through the C ABI
versus the CPU oracle.  Integer outputs and min/max bit-exact; fp32 outputs bit-exact (the bar is
1 ULP of the int->fp32 scale product; the kernels perform the same single fp32 multiply)."""
import numpy as np
import pytest

from oracle import pyoracle as orc

pytestmark = pytest.mark.gpu

TORCH_OF = None


def tdtype(T):
    import torch
    return {orc.QINT8: torch.int8, orc.QUINT8: torch.uint8}[T]


def scale_per_slice(shape, axis, values):
    out = np.take(values, np.remainder(np.arange(np.prod(shape)), len(values))).reshape(shape)
    if axis is not None:
        scale_shape = [1] * len(shape)
        scale_shape[axis] = shape[axis]
        out = out * np.arange(1, shape[axis] + 1).reshape(scale_shape)
    return out


def host_quant_params(T, mode, classic, mn, mx, ensure=0.01):
    """Host-side parameter math (the op kernel's job) done with the oracle's scalar helpers, returning
    what the C ABI takes: per-slice scale and addend, and the reported output range."""
    mn = np.atleast_1d(np.float32(mn))
    mx = np.atleast_1d(np.float32(mx))
    amn, amx = np.zeros_like(mn), np.zeros_like(mx)
    for i in range(mn.size):
        st, amn[i], amx[i] = orc.adjust_input_range(float(mn[i]), float(mx[i]), ensure)
        assert st == orc.OK
    if mode == orc.SCALED or classic:
        st, omn, omx, sc, zp = orc.scale_zeropoint_align(T, mode, False, amn, amx)
        add = zp.astype(np.float32) if mode == orc.MIN_FIRST else np.zeros_like(sc)
        if mode == orc.SCALED and T == orc.QUINT8:
            omn = np.zeros_like(omn)
    else:
        sc = np.array([orc.legacy_min_first_scale(T, float(a), float(b)) for a, b in zip(amn, amx)], np.float32)
        add = (-amn).astype(np.float32) * sc
        omn, omx = amn, amx
    return sc, add, omn, omx


def gpu_quantize(hip, dev, x, T, mode, mn, mx, axis=None, classic=False):
    import torch
    sc, add, omn, omx = host_quant_params(T, mode, classic, mn, mx)
    x_d = torch.from_numpy(np.ascontiguousarray(x)).to(dev)
    q_d = torch.empty(x.shape, dtype=tdtype(T), device=dev)
    if axis is None:
        hip.quantize(x_d, q_d, x.size, T, float(sc[0]), float(add[0]))
    else:
        outer = int(np.prod(x.shape[:axis], dtype=np.int64))
        inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
        sc_d = torch.from_numpy(sc).to(dev)
        add_d = torch.from_numpy(add).to(dev)
        hip.quantize_axis(x_d, q_d, outer, x.shape[axis], inner, T, sc_d, add_d)
    torch.cuda.synchronize()
    return q_d.cpu().numpy(), omn, omx


def test_quantize_golden_vectors(hip, dev, golden):
    T = {"quint8": orc.QUINT8, "qint8": orc.QINT8}
    Mo = {"MIN_FIRST": orc.MIN_FIRST, "SCALED": orc.SCALED}
    for case in golden["quantize_v2"]:
        x = np.array(case["x"], np.float32).reshape(case["shape"])
        q, omn, omx = gpu_quantize(hip, dev, x, T[case["T"]], Mo[case["mode"]], case["min_range"],
                                   case["max_range"], classic=case["classic_asymmetric_algorithm"])
        assert q.ravel().tolist() == case["expected"], case["source"]


def test_quantize_axis_golden(hip, dev, golden):
    g = golden["quantize_v2_axis"]
    shape = np.array(g["shape"])
    values = np.array(g["values"], np.float32)
    expected = scale_per_slice(shape, None, np.array(g["quant_values"], np.int32))
    for axis in g["axes"]:
        x = scale_per_slice(shape, axis, values).astype(np.float32)
        if axis is None:
            mn, mx = g["min_unit"], g["max_unit"]
        else:
            mn = [g["min_unit"] * (s + 1) for s in range(shape[axis])]
            mx = [g["max_unit"] * (s + 1) for s in range(shape[axis])]
        q, omn, omx = gpu_quantize(hip, dev, x, orc.QINT8, orc.SCALED, mn, mx, axis=axis)
        np.testing.assert_array_equal(q.astype(np.int32), expected)


def outlier_normal(rng, n, frac, mult):
    x = rng.standard_normal(n).astype(np.float32)
    k = max(1, int(n * frac))
    idx = rng.integers(0, n, k)
    x[idx] *= mult
    return x


@pytest.mark.parametrize("T,mode,classic", [
    (orc.QINT8, orc.SCALED, False), (orc.QUINT8, orc.SCALED, False),
    (orc.QUINT8, orc.MIN_FIRST, False), (orc.QINT8, orc.MIN_FIRST, False),
    (orc.QUINT8, orc.MIN_FIRST, True)])
@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 4096, (1 << 20) + 7])
def test_quantize_random_vs_oracle(hip, dev, T, mode, classic, n):
    rng = np.random.default_rng(30 + n % 97)
    x = outlier_normal(rng, n, 1e-4, 50.0)
    # ties and saturation: exact half-steps for scale 1 when the range is +-127
    mn, mx = float(x.min()), float(x.max())
    st, q_ref, omn_ref, omx_ref = orc.quantize_v2(x, mn, mx, T, mode, None, classic)
    q, omn, omx = gpu_quantize(hip, dev, x, T, mode, mn, mx, classic=classic)
    np.testing.assert_array_equal(q, q_ref)
    np.testing.assert_array_equal(omn, omn_ref)
    np.testing.assert_array_equal(omx, omx_ref)


def test_quantize_ties_and_saturation(hip, dev):
    x = np.concatenate([np.arange(-130, 131, dtype=np.float32) + 0.5,
                        np.array([300.0, -300.0, 1e30, -1e30, 0.0, -0.0], np.float32)])
    for T in (orc.QINT8, orc.QUINT8):
        st, q_ref, _, _ = orc.quantize_v2(x, -127.0, 127.0, T, orc.SCALED)
        q, _, _ = gpu_quantize(hip, dev, x, T, orc.SCALED, -127.0, 127.0)
        if T == orc.QINT8:
            np.testing.assert_array_equal(q, q_ref)
            assert q[0] == -128 and q[130 + 0] % 2 == 0
        else:
            # quint8 SCALED scale is 255/127: not all ties, still must equal the oracle
            np.testing.assert_array_equal(q, q_ref)


def test_quantize_unaligned_pointers(hip, dev):
    import torch
    rng = np.random.default_rng(1)
    x = rng.standard_normal(1000 + 3).astype(np.float32)
    x_d = torch.from_numpy(x).to(dev)
    q_d = torch.zeros(1003 + 8, dtype=torch.int8, device=dev)
    # input offset by one float (not 16-byte aligned), output offset by 1 byte
    hip.quantize(x_d.data_ptr() + 4, q_d.data_ptr() + 1, 1002, hip.QINT8, 20.0, 0.0)
    torch.cuda.synchronize()
    st, q_ref, _, _ = orc.quantize_v2(x[1:], -6.35, 6.35, orc.QINT8, orc.SCALED)
    got = q_d.cpu().numpy()
    np.testing.assert_array_equal(got[1:1003], q_ref)
    assert got[0] == 0 and np.all(got[1003:] == 0)


@pytest.mark.parametrize("seed", range(3))
def test_random_sizes_and_offsets_vs_oracle(hip, dev, seed):
    """Seeded random element counts (1 .. 3 million: vector body, grid-strided second group, scalar head and tail) and
    random element offsets of input and output inside larger buffers; QuantizeV2 in every mode, Dequantize and
    Requantize against the oracle, with guard bytes around each output that must stay untouched."""
    import torch
    rng = np.random.default_rng(4000 + seed)
    modes = [(orc.QINT8, orc.SCALED, False), (orc.QUINT8, orc.SCALED, False), (orc.QUINT8, orc.MIN_FIRST, False),
             (orc.QINT8, orc.MIN_FIRST, False), (orc.QUINT8, orc.MIN_FIRST, True)]
    for case in range(12):
        n = int(rng.choice([rng.integers(1, 300), rng.integers(300, 70000), rng.integers(70000, 3000000)]))
        xo, qo = int(rng.integers(0, 8)), int(rng.integers(0, 16))
        T, mode, classic = modes[int(rng.integers(0, 5))]
        x = outlier_normal(rng, n, 1e-4, 50.0)
        mn, mx = float(x.min()), float(x.max())
        st, q_ref, _, _ = orc.quantize_v2(x, mn, mx, T, mode, None, classic)
        sc, add, _, _ = host_quant_params(T, mode, classic, mn, mx)
        xb = torch.zeros(n + 8, dtype=torch.float32, device=dev)
        xb[xo:xo + n] = torch.from_numpy(x).to(dev)
        qb = torch.full((n + 32,), 0x55, dtype=torch.uint8, device=dev)
        hip.quantize(xb.data_ptr() + 4 * xo, qb.data_ptr() + qo, n, T, float(sc[0]), float(add[0]))
        torch.cuda.synchronize()
        got = qb.cpu().numpy()
        msg = "quantize n %d offsets %d %d type %d mode %d classic %d" % (n, xo, qo, T, mode, classic)
        np.testing.assert_array_equal(got[qo:qo + n].view(orc.NP_OF[T]), q_ref, err_msg=msg)
        assert np.all(got[:qo] == 0x55) and np.all(got[qo + n:] == 0x55), msg
        # Dequantize of those bytes
        dmode = orc.SCALED if mode == orc.SCALED else orc.MIN_FIRST
        st, y_ref = orc.dequantize(q_ref, np.float32(-3.7), np.float32(5.2), T, dmode)
        st, _, _, dsc, dzp = orc.scale_zeropoint_align(T, dmode, True, np.float32(-3.7), np.float32(5.2))
        yo = int(rng.integers(0, 8))
        yb = torch.full((n + 16,), -7.0, dtype=torch.float32, device=dev)
        hip.dequantize(qb.data_ptr() + qo, yb.data_ptr() + 4 * yo, n, T, float(dsc[0]), int(dzp[0]) if dmode == orc.MIN_FIRST else 0)
        torch.cuda.synchronize()
        goty = yb.cpu().numpy()
        np.testing.assert_array_equal(goty[yo:yo + n], y_ref, err_msg="de" + msg)
        assert np.all(goty[:yo] == -7.0) and np.all(goty[yo + n:] == -7.0), "de" + msg


def test_narrow_range_flag_is_inert(hip, dev):
    # the reference reads narrow_range and ignores it: there is no such argument at this level;
    # saturation is full-range (-128) in both cases
    q, _, _ = gpu_quantize(hip, dev, np.array([-10.0, 10.0], np.float32), orc.QINT8, orc.SCALED, -1.0, 1.0)
    assert q.tolist() == [-128, 127]


@pytest.mark.parametrize("T,mode", [(orc.QINT8, orc.SCALED), (orc.QUINT8, orc.SCALED),
                                    (orc.QUINT8, orc.MIN_FIRST), (orc.QINT8, orc.MIN_FIRST)])
@pytest.mark.parametrize("n", [1, 5, 4099, 1 << 20])
def test_dequantize_vs_oracle(hip, dev, T, mode, n):
    import torch
    rng = np.random.default_rng(n)
    info = np.iinfo(orc.NP_OF[T])
    q = rng.integers(info.min, info.max + 1, n).astype(orc.NP_OF[T])
    mn, mx = np.float32(-3.7), np.float32(5.2)
    st, y_ref = orc.dequantize(q, mn, mx, T, mode)
    st, _, _, sc, zp = orc.scale_zeropoint_align(T, mode, True, mn, mx)
    q_d = torch.from_numpy(q).to(dev)
    y_d = torch.empty(n, dtype=torch.float32, device=dev)
    hip.dequantize(q_d, y_d, n, T, float(sc[0]), int(zp[0]) if mode == orc.MIN_FIRST else 0)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(y_d.cpu().numpy(), y_ref)


def test_dequantize_golden(hip, dev, golden):
    import torch
    g = golden["dequantize_axis"]
    shape = np.array(g["shape"])
    q = scale_per_slice(shape, None, np.array(g["values"], np.int32)).astype(np.int8)
    deq = np.array(g["dequant_values"], np.float32)
    for axis in g["axes"]:
        expected = scale_per_slice(shape, axis, deq)
        if axis is None:
            mn, mx = [g["min_unit"]], [g["max_unit"]]
        else:
            mn = [g["min_unit"] * (s + 1) for s in range(shape[axis])]
            mx = [g["max_unit"] * (s + 1) for s in range(shape[axis])]
        st, _, _, sc, zp = orc.scale_zeropoint_align(orc.QINT8, orc.SCALED, True, mn, mx)
        q_d = torch.from_numpy(q).to(dev)
        y_d = torch.empty(q.shape, dtype=torch.float32, device=dev)
        if axis is None:
            hip.dequantize(q_d, y_d, q.size, orc.QINT8, float(sc[0]), 0)
        else:
            outer = int(np.prod(shape[:axis], dtype=np.int64))
            inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
            hip.dequantize_axis(q_d, y_d, outer, int(shape[axis]), inner, orc.QINT8,
                                torch.from_numpy(sc).to(dev), torch.from_numpy(zp).to(dev))
        torch.cuda.synchronize()
        y = y_d.cpu().numpy()
        np.testing.assert_allclose(y, expected, rtol=g["tolerance"], atol=g["tolerance"])
        st, y_ref = orc.dequantize(q, mn, mx, orc.QINT8, orc.SCALED, axis)
        np.testing.assert_array_equal(y, y_ref)


# Shapes for the per-axis kernels: the axis innermost with a multiple of 4 slices (one 16-byte parameter load per
# lane), inner a multiple of 4 (the lane's 4 elements share a slice), and shapes neither rule takes (element kernel).
AXIS_CASES = [((768, 3072), 1), ((3, 5, 64), 2), ((3072, 768), 0), ((6, 5, 12), 1), ((7, 16, 4), 1), ((3, 3, 16, 8), 3),
              ((5, 6), 1), ((4, 7, 3), 1), ((1, 4), 1), ((2, 1, 8), 1)]


@pytest.mark.parametrize("T,mode,classic", [(orc.QINT8, orc.SCALED, False), (orc.QUINT8, orc.MIN_FIRST, True),
                                            (orc.QUINT8, orc.MIN_FIRST, False)])
@pytest.mark.parametrize("shape,axis", AXIS_CASES)
def test_quantize_axis_vector_paths_vs_oracle(hip, dev, shape, axis, T, mode, classic):
    rng = np.random.default_rng(sum(shape) * 7 + axis)
    ns = shape[axis]
    bshape = [1] * len(shape)
    bshape[axis] = ns
    spread = (0.05 + rng.random(ns) * 3).astype(np.float32)
    x = (rng.standard_normal(shape) * spread.reshape(bshape)).astype(np.float32)
    x.flat[::97] *= 40.0  # saturating values
    x.flat[1::53] = np.rint(x.flat[1::53]) + np.float32(0.5)  # ties after scaling by powers of two
    red = tuple(d for d in range(len(shape)) if d != axis)
    mn = np.minimum(x.min(axis=red), 0).astype(np.float32) * np.float32(0.5)
    mx = np.maximum(x.max(axis=red), 0).astype(np.float32) * np.float32(0.5)
    st, q_ref, mn_ref, mx_ref = orc.quantize_v2(x, mn, mx, T, mode, axis=axis, classic=classic)
    assert st == orc.OK
    q, omn, omx = gpu_quantize(hip, dev, x, T, mode, mn, mx, axis=axis, classic=classic)
    np.testing.assert_array_equal(q.view(np.uint8), np.asarray(q_ref).view(np.uint8).reshape(shape))
    np.testing.assert_array_equal(omn, mn_ref)
    np.testing.assert_array_equal(omx, mx_ref)


@pytest.mark.parametrize("T,mode", [(orc.QINT8, orc.SCALED), (orc.QUINT8, orc.MIN_FIRST)])
@pytest.mark.parametrize("shape,axis", AXIS_CASES)
def test_dequantize_axis_vector_paths_vs_oracle(hip, dev, shape, axis, T, mode):
    import torch
    rng = np.random.default_rng(sum(shape) * 11 + axis)
    ns = shape[axis]
    q = rng.integers(0, 256, size=shape, dtype=np.uint8).view(np.int8 if T == orc.QINT8 else np.uint8)
    mn = -(0.1 + rng.random(ns) * 5).astype(np.float32)
    mx = (0.1 + rng.random(ns) * 7).astype(np.float32)
    st, y_ref = orc.dequantize(q, mn, mx, T, mode, axis)
    assert st == orc.OK
    st, _, _, sc, zp = orc.scale_zeropoint_align(T, mode, True, mn, mx)
    assert st == orc.OK
    outer = int(np.prod(shape[:axis], dtype=np.int64))
    inner = int(np.prod(shape[axis + 1:], dtype=np.int64))
    y_d = torch.empty(shape, dtype=torch.float32, device=dev)
    zp_d = torch.from_numpy(np.ascontiguousarray(zp, np.int32)).to(dev) if mode == orc.MIN_FIRST else None
    hip.dequantize_axis(torch.from_numpy(q).to(dev), y_d, outer, ns, inner, T, torch.from_numpy(sc).to(dev), zp_d)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(y_d.cpu().numpy(), np.asarray(y_ref).reshape(shape))


@pytest.mark.parametrize("out_type", [orc.QINT8, orc.QUINT8])
@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (2, 3, 5, 7), (2, 4, 8, 64), (1, 1, 4096, 1), (1, 1, 1000, 3), (4, 8, 16, 256)])
def test_requantize_per_channel_vs_oracle(hip, dev, out_type, shape):
    import torch
    rng = np.random.default_rng(sum(shape))
    x = np.rint(rng.standard_normal(shape) * (1 << 20)).astype(np.int32)
    x.flat[0] = np.iinfo(np.int32).max
    x.flat[-1] = np.iinfo(np.int32).min
    depth = shape[-1]
    in_min = -(rng.random(depth).astype(np.float32) * 8 + 0.1)
    in_max = rng.random(depth).astype(np.float32) * 8 + 0.1
    req_min, req_max = -0.004, 0.0035
    st, q_ref, omn, omx = orc.requantize_per_channel(x, in_min, in_max, req_min, req_max, out_type)
    factor = np.float32(127.0 if out_type == orc.QINT8 else 255.0)
    mm = np.maximum(np.abs(in_min), np.abs(in_max))
    scales = factor * (mm / np.maximum(np.abs(np.float32(req_min)), np.abs(np.float32(req_max))) / np.float32(2 ** 31))
    x_d = torch.from_numpy(x).to(dev)
    q_d = torch.empty(shape, dtype=tdtype(out_type), device=dev)
    hip.requantize_per_channel(x_d, q_d, x.size // depth, depth, out_type, torch.from_numpy(scales).to(dev))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(q_d.cpu().numpy(), q_ref)
    if depth == 1:
        hip.requantize(x_d, q_d.zero_(), x.size, out_type, float(scales[0]))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(q_d.cpu().numpy(), q_ref)


@pytest.mark.parametrize("shape", [(1, 1), (7, 1), (100003, 1), (1 << 20, 1), (33, 3), (1000, 64), (257, 300), (5, 1000)])
def test_minmax_i32_per_channel(hip, dev, shape):
    import torch
    rng = np.random.default_rng(shape[0])
    x = rng.integers(-2 ** 31, 2 ** 31, size=shape, dtype=np.int64).astype(np.int32)
    x_d = torch.from_numpy(x).to(dev)
    mn_d = torch.zeros(shape[1], dtype=torch.int32, device=dev)
    mx_d = torch.zeros(shape[1], dtype=torch.int32, device=dev)
    for _ in range(2):  # second call must not see the first call's result
        hip.minmax_i32_per_channel(x_d, shape[0], shape[1], mn_d, mx_d)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(mn_d.cpu().numpy(), x.min(0))
    np.testing.assert_array_equal(mx_d.cpu().numpy(), x.max(0))
    # the op's float range is host math on these integers: compare with the oracle end to end
    in_min = -(rng.random(shape[1]).astype(np.float32) + 0.5)
    in_max = rng.random(shape[1]).astype(np.float32) + 0.5
    st, omn_ref, omx_ref = orc.requantization_range_per_channel(x, in_min, in_max, 6.0)
    mn, mx = mn_d.cpu().numpy(), mx_d.cpu().numpy()
    out = np.float32(np.finfo(np.float32).tiny)
    nonneg = True
    for c in range(shape[1]):
        amax = np.int32(max(abs(int(mn[c])) if mn[c] != -2 ** 31 else -2 ** 31, abs(int(mx[c]))))
        r = np.float32(max(abs(in_min[c]), abs(in_max[c]))) * np.float32(amax) / np.float32(2 ** 31)
        out = max(out, np.float32(r))
        nonneg = nonneg and mn[c] >= 0
    out = min(out, np.float32(6.0))
    assert np.float32(out) == omx_ref and (np.float32(0.0) if nonneg else -np.float32(out)) == omn_ref


@pytest.mark.parametrize("n,offset", [(1, 0), (5, 0), (1027, 1), (1 << 20, 0), ((1 << 20) + 3, 3)])
def test_minmax_f32(hip, dev, n, offset):
    import torch
    rng = np.random.default_rng(n)
    x = outlier_normal(rng, n + offset, 1e-3, 50.0)
    if n > 100:
        x[offset + 17] = np.nan  # ignored
    x_d = torch.from_numpy(x).to(dev)
    out = torch.zeros(2, dtype=torch.float32, device=dev)
    hip.minmax_f32(x_d.data_ptr() + 4 * offset, n, out)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert got[0] == np.nanmin(x[offset:]) and got[1] == np.nanmax(x[offset:])


def test_full_size_quantize_properties(hip, dev):
    """2^28 elements (the benchmark size): oracle on a strided sample + structural properties."""
    import torch
    n = 1 << 28
    g = torch.Generator(device=dev)
    g.manual_seed(30)
    x_d = torch.randn(n, device=dev, generator=g)
    x_d[::9973] *= 50.0
    mm = torch.zeros(2, dtype=torch.float32, device=dev)
    hip.minmax_f32(x_d, n, mm)
    mn, mx = [float(v) for v in mm.cpu().numpy()]
    assert mn == float(x_d.min()) and mx == float(x_d.max())
    for T, mode in ((orc.QINT8, orc.SCALED), (orc.QUINT8, orc.MIN_FIRST)):
        sc, add, omn, omx = host_quant_params(T, mode, False, mn, mx)
        q_d = torch.empty(n, dtype=tdtype(T), device=dev)
        hip.quantize(x_d, q_d, n, T, float(sc[0]), float(add[0]))
        torch.cuda.synchronize()
        # sample: three windows (start, middle, end) checked exactly against the oracle
        for lo in (0, n // 2 - 12345, n - (1 << 20)):
            xs = x_d[lo:lo + (1 << 20)].cpu().numpy()
            st, q_ref, _, _ = orc.quantize_v2(xs, mn, mx, T, mode)
            np.testing.assert_array_equal(q_d[lo:lo + (1 << 20)].cpu().numpy(), q_ref)
        # size-independent property: dequantize(quantize(x)) is within half a step of clip(x)
        st, _, _, dsc, dzp = orc.scale_zeropoint_align(T, mode, True, omn, omx)
        y_d = torch.empty(n, dtype=torch.float32, device=dev)
        hip.dequantize(q_d, y_d, n, T, float(dsc[0]), int(dzp[0]))
        torch.cuda.synchronize()
        step = float(dsc[0])
        err = float((y_d - x_d.clamp(float(omn[0]), float(omx[0]))).abs().max())
        assert err <= step * (0.5 if mode == orc.SCALED else 1.0) * 1.001 + 1e-6
        del q_d, y_d


def _windows(n, size=1 << 20):
    return (0, n // 2 - 12345, n - size)


def test_full_size_scaled_quint8_and_dequantize_vs_oracle(hip, dev):
    """2^28 elements: QuantizeV2 SCALED -> quint8 (negatives clamp to 0, output range (0, r)) and Dequantize of both
    8-bit types in both modes against the oracle on three windows of 2^20 elements, plus a whole-tensor int64 checksum
    of the quantized bytes against torch's evaluation of the same formula."""
    import torch
    n = 1 << 28
    g = torch.Generator(device=dev)
    g.manual_seed(30)
    x_d = torch.randn(n, device=dev, generator=g)
    x_d[::9973] *= 50.0
    mn, mx = float(x_d.min()), float(x_d.max())
    sc, add, omn, omx = host_quant_params(orc.QUINT8, orc.SCALED, False, mn, mx)
    assert omn[0] == 0.0
    q_d = torch.empty(n, dtype=torch.uint8, device=dev)
    hip.quantize(x_d, q_d, n, orc.QUINT8, float(sc[0]), float(add[0]))
    torch.cuda.synchronize()
    for lo in _windows(n):
        xs = x_d[lo:lo + (1 << 20)].cpu().numpy()
        st, q_ref, _, _ = orc.quantize_v2(xs, mn, mx, orc.QUINT8, orc.SCALED)
        np.testing.assert_array_equal(q_d[lo:lo + (1 << 20)].cpu().numpy(), q_ref)
    expect_sum = 0
    for lo in range(0, n, 1 << 26):   # the same fp32 multiply, round-half-even and clamp, by torch
        part = torch.round(x_d[lo:lo + (1 << 26)] * float(sc[0])).clamp_(0, 255)
        expect_sum += int(part.sum(dtype=torch.float64).item())
    assert int(q_d.sum(dtype=torch.int64).item()) == expect_sum
    del x_d
    # Dequantize at full size: the quint8 bytes above in both modes, and the same bytes read as qint8
    y_d = torch.empty(n, dtype=torch.float32, device=dev)
    for T, mode, rmn, rmx in ((orc.QUINT8, orc.SCALED, 0.0, mx), (orc.QUINT8, orc.MIN_FIRST, mn, mx),
                              (orc.QINT8, orc.SCALED, mn, mx), (orc.QINT8, orc.MIN_FIRST, mn, mx)):
        st, _, _, dsc, dzp = orc.scale_zeropoint_align(T, mode, True, rmn, rmx)
        src = q_d if T == orc.QUINT8 else q_d.view(torch.int8)
        hip.dequantize(src, y_d, n, T, float(dsc[0]), int(dzp[0]) if mode == orc.MIN_FIRST else 0)
        torch.cuda.synchronize()
        for lo in _windows(n):
            st, y_ref = orc.dequantize(src[lo:lo + (1 << 20)].cpu().numpy(), rmn, rmx, T, mode)
            np.testing.assert_array_equal(y_d[lo:lo + (1 << 20)].cpu().numpy(), y_ref)
        # whole tensor: y is an exact function of the byte, so the histogram of q fixes the sum of y in float64
        table = orc.dequantize(np.arange(256, dtype=np.uint8).view(orc.NP_OF[T]), rmn, rmx, T, mode)[1].astype(np.float64)
        counts = torch.bincount(q_d.to(torch.int32), minlength=256).cpu().numpy()
        assert abs(float(y_d.sum(dtype=torch.float64).item()) - float((counts * table).sum())) <= 1e-6 * abs(float((counts * table).sum())) + 1e-3


def test_full_size_requantize_and_range_vs_oracle(hip, dev):
    """2^28 int32 accumulators: RequantizationRange (depth 1) is the exact min / max, its float range equals the
    oracle's on the same extremes, and Requantize int32 -> qint8 / quint8 equals the oracle on three windows; the
    whole tensor through an int64 checksum against torch's evaluation of the same fp32 multiply, rounding and clamp."""
    import torch
    n = 1 << 28
    g = torch.Generator(device=dev)
    g.manual_seed(31)
    acc = (torch.randn(n, device=dev, generator=g) * float(1 << 20)).round_().to(torch.int32)
    acc[12345] = -(1 << 27)
    acc[n - 77] = (1 << 27) + 12345
    imn = torch.zeros(1, dtype=torch.int32, device=dev)
    imx = torch.zeros(1, dtype=torch.int32, device=dev)
    hip.minmax_i32_per_channel(acc, n, 1, imn, imx)
    torch.cuda.synchronize()
    lo_i, hi_i = int(imn.item()), int(imx.item())
    assert lo_i == int(acc.min().item()) == -(1 << 27) and hi_i == int(acc.max().item()) == (1 << 27) + 12345
    # the op's float range is host math on the two integers: the oracle on a tensor holding just the extremes
    in_min, in_max = np.float32(-1.5), np.float32(2.25)
    st, omn_ref, omx_ref = orc.requantization_range_per_channel(np.array([[lo_i], [hi_i]], np.int32), [in_min], [in_max], 6.0)
    amax = np.float32(max(abs(lo_i), abs(hi_i)))
    rng_f = np.float32(max(abs(in_min), abs(in_max))) * amax / np.float32(2 ** 31)
    assert np.float32(min(rng_f, np.float32(6.0))) == omx_ref and -omx_ref == omn_ref
    for out_type, tdt in ((orc.QINT8, torch.int8), (orc.QUINT8, torch.uint8)):
        factor = np.float32(127.0 if out_type == orc.QINT8 else 255.0)
        req = np.float32(omx_ref)
        scale = factor * (np.float32(max(abs(in_min), abs(in_max))) / req / np.float32(2 ** 31))
        q_d = torch.empty(n, dtype=tdt, device=dev)
        hip.requantize(acc, q_d, n, out_type, float(scale))
        torch.cuda.synchronize()
        for lo in _windows(n):
            xs = acc[lo:lo + (1 << 20)].cpu().numpy().reshape(1, 1, -1, 1)
            st, q_ref, _, _ = orc.requantize_per_channel(xs, [in_min], [in_max], -float(req), float(req), out_type)
            np.testing.assert_array_equal(q_d[lo:lo + (1 << 20)].cpu().numpy(), q_ref.reshape(-1))
        info = np.iinfo(orc.NP_OF[out_type])
        expect_sum = 0
        for lo in range(0, n, 1 << 26):
            part = torch.round(acc[lo:lo + (1 << 26)].to(torch.float32) * float(scale)).clamp_(float(info.min), float(info.max))
            expect_sum += int(part.sum(dtype=torch.float64).item())
        assert int(q_d.sum(dtype=torch.int64).item()) == expect_sum
        del q_d


@pytest.mark.parametrize("nbytes,offset", [(1 << 20, 0), (4099, 0), (70001, 3), (15, 1), (0, 0)])
def test_device_copy_kernel(hip, dev, nbytes, offset):
    import torch
    src = torch.randint(0, 256, (nbytes + 64,), dtype=torch.uint8, device=dev)
    dst = torch.zeros(nbytes + 64, dtype=torch.uint8, device=dev)
    hip.memcpy_d2d_async(dst.data_ptr() + offset, src.data_ptr() + offset, nbytes,
                         torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    expect = torch.zeros_like(dst)
    expect[offset:offset + nbytes] = src[offset:offset + nbytes]
    assert torch.equal(dst, expect)


def test_more_than_2_31_elements(hip, dev):
    """64-bit indexing: QuantizeV2, the range pass and Dequantize over 2^31 + 4099 elements.  Checked through
    properties (no host copy of 8 GiB): the quantized tensor equals torch's own evaluation of the same
    formula on slices at the start, across the 2^31 boundary and at the ragged end, and its checksum
    over the whole tensor equals the sum of the checksums of the slices computed independently."""
    import torch
    n = (1 << 31) + 4099
    free, _ = torch.cuda.mem_get_info()
    if free < 14 * (1 << 30):
        pytest.skip("needs ~14 GiB of free device memory")
    x = torch.empty(n, dtype=torch.float32, device=dev)
    piece = torch.randn(1 << 24, device=dev)
    for off in range(0, n, 1 << 24):
        m = min(1 << 24, n - off)
        x[off:off + m] = piece[:m] * (1.0 + (off >> 24) * 0.01)
    x[n - 1] = -77.0   # extreme values behind the 2^31 boundary
    x[(1 << 31) + 5] = 91.0
    mm = torch.zeros(2, dtype=torch.float32, device=dev)
    hip.minmax_f32(x, n, mm)
    torch.cuda.synchronize()
    assert mm.cpu().tolist() == [-77.0, 91.0]
    scale = np.float32(127.0) / np.float32(91.0)
    q = torch.empty(n, dtype=torch.int8, device=dev)
    hip.quantize(x, q, n, hip.QINT8, float(scale), 0.0)
    torch.cuda.synchronize()
    total = 0
    for lo, hi in ((0, 1 << 20), ((1 << 31) - 4096, (1 << 31) + 4096), (n - 5000, n)):
        ref = torch.clamp(torch.round(x[lo:hi] * float(scale)), -128, 127).to(torch.int8)
        assert torch.equal(q[lo:hi], ref), (lo, hi)
    for off in range(0, n, 1 << 28):
        m = min(1 << 28, n - off)
        ref = torch.clamp(torch.round(x[off:off + m] * float(scale)), -128, 127)
        total += int(ref.sum(dtype=torch.float64).item())
    got = 0
    for off in range(0, n, 1 << 28):
        m = min(1 << 28, n - off)
        got += int(q[off:off + m].sum(dtype=torch.int64).item())
    assert got == total
    # Dequantize back into the same fp32 buffer (in place of x) and compare the ragged end
    inv = np.float32(91.0) / np.float32(127.0)
    q_tail = q[n - 5000:].clone()
    hip.dequantize(q, x, n, hip.QINT8, float(inv), 0)
    torch.cuda.synchronize()
    assert torch.equal(x[n - 5000:], q_tail.to(torch.float32) * float(inv))
    assert torch.equal(x[(1 << 31) - 8:(1 << 31) + 8], q[(1 << 31) - 8:(1 << 31) + 8].to(torch.float32) * float(inv))


# ------------------------------------------------------------------------------------------------
# 16-bit floating point ends: QuantizeV2 from bfloat16, Dequantize to bfloat16 / half
# ------------------------------------------------------------------------------------------------
def f32_to_bf16_bits(a):
    """fp32 -> bfloat16 bit patterns, round to nearest even (NaN kept quiet)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7fffffff) > 0x7f800000
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), rounded)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


@pytest.mark.parametrize("T,mode", [(orc.QINT8, orc.SCALED), (orc.QUINT8, orc.MIN_FIRST)])
@pytest.mark.parametrize("n,offset", [(1 << 16, 0), (4099, 0), (1001, 3), (5, 0)])
def test_quantize_from_bfloat16(hip, dev, T, mode, n, offset):
    """A bfloat16 source widens exactly to fp32; from there on it is the fp32 op (oracle on the widened values)."""
    import torch
    rng = np.random.default_rng(n + offset)
    bits = f32_to_bf16_bits(rng.standard_normal(n + offset) * 3)
    x = bf16_bits_to_f32(bits[offset:])
    mn, mx = float(x.min()), float(x.max())
    scale, addend, omn, omx = host_quant_params(T, mode, False, mn, mx)
    _, q_ref, _, _ = orc.quantize_v2(x, mn, mx, T, mode)
    x_d = torch.from_numpy(bits.view(np.int16)).to(dev)
    q_d = torch.zeros(n + 8, dtype=tdtype(T), device=dev)
    hip.quantize_bf16(x_d.data_ptr() + 2 * offset, q_d, n, T, float(scale[0]), float(addend[0]))
    torch.cuda.synchronize()
    got = q_d.cpu().numpy()
    np.testing.assert_array_equal(got[:n], q_ref)
    assert (got[n:] == 0).all()


def test_quantize_axis_from_bfloat16(hip, dev):
    import torch
    rng = np.random.default_rng(8)
    shape = (3, 5, 17)
    bits = f32_to_bf16_bits(rng.standard_normal(shape) * np.arange(1, 6).reshape(1, 5, 1))
    x = bf16_bits_to_f32(bits)
    mn, mx = x.min((0, 2)), x.max((0, 2))
    scale, addend, omn, omx = host_quant_params(orc.QINT8, orc.SCALED, False, mn, mx)
    _, q_ref, _, _ = orc.quantize_v2(x, mn, mx, orc.QINT8, orc.SCALED, axis=1)
    q_d = torch.zeros(shape, dtype=torch.int8, device=dev)
    hip.quantize_axis_bf16(torch.from_numpy(bits.view(np.int16)).to(dev), q_d, 3, 5, 17, orc.QINT8,
                           torch.from_numpy(scale).to(dev), torch.from_numpy(addend).to(dev))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(q_d.cpu().numpy(), q_ref)


@pytest.mark.parametrize("T,mode", [(orc.QINT8, orc.SCALED), (orc.QUINT8, orc.MIN_FIRST)])
@pytest.mark.parametrize("y_type", ["bf16", "f16"])
@pytest.mark.parametrize("n,offset", [(1 << 16, 0), (4099, 0), (1001, 1), (7, 0)])
def test_dequantize_to_16_bit(hip, dev, T, mode, y_type, n, offset):
    """The fp32 result of Dequantize rounded to nearest even into bfloat16 / half; the range is chosen so that
    half overflows to infinity for the largest codes."""
    import torch
    rng = np.random.default_rng(n)
    info = np.iinfo(orc.NP_OF[T])
    q = rng.integers(info.min, info.max + 1, n + offset).astype(orc.NP_OF[T])
    mn, mx = (-70000.0, 70000.0) if y_type == "f16" and T == orc.QINT8 else (-2.5, 3.25)
    _, y32 = orc.dequantize(q[offset:], mn, mx, T, mode)
    _, _, _, sc, zp = orc.scale_zeropoint_align(T, mode, True, np.float32([mn]), np.float32([mx]))
    y_d = torch.zeros(n + 8, dtype=torch.int16, device=dev)
    hip.dequantize16(torch.from_numpy(q).to(dev).data_ptr() + offset, y_d, n, T, hip.BFLOAT16 if y_type == "bf16" else hip.HALF,
                     float(sc[0]), int(zp[0]) if mode == orc.MIN_FIRST else 0)
    torch.cuda.synchronize()
    got = y_d.cpu().numpy().view(np.uint16)
    with np.errstate(over="ignore"):
        expect = f32_to_bf16_bits(y32) if y_type == "bf16" else y32.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(got[:n], expect)
    assert (got[n:] == 0).all()
    if y_type == "f16" and T == orc.QINT8 and n >= 4099:
        assert np.isinf(expect.view(np.float16)).any()


def test_dequantize_axis_to_16_bit(hip, dev):
    import torch
    rng = np.random.default_rng(9)
    shape = (4, 6, 9)
    q = rng.integers(0, 256, shape).astype(np.uint8)
    mn = -np.arange(1, 7, dtype=np.float32)
    mx = np.arange(1, 7, dtype=np.float32) * 1.5
    _, y32 = orc.dequantize(q, mn, mx, orc.QUINT8, orc.MIN_FIRST, axis=1)
    _, _, _, sc, zp = orc.scale_zeropoint_align(orc.QUINT8, orc.MIN_FIRST, True, mn.copy(), mx.copy())
    for y_type, conv in ((hip.BFLOAT16, f32_to_bf16_bits), (hip.HALF, lambda v: v.astype(np.float16).view(np.uint16))):
        y_d = torch.zeros(shape, dtype=torch.int16, device=dev)
        hip.dequantize_axis16(torch.from_numpy(q).to(dev), y_d, 4, 6, 9, orc.QUINT8, y_type, torch.from_numpy(sc).to(dev),
                              torch.from_numpy(zp).to(dev))
        torch.cuda.synchronize()
        np.testing.assert_array_equal(y_d.cpu().numpy().view(np.uint16), conv(y32))
