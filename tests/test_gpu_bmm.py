"""GPU parity of the quantized BatchMatMul (itexhip_qbatch_matmul) against the CPU oracle, through the C ABI.
Bit-exact: the accumulation is integer and the epilogue is the same sequence of separately rounded fp32
operations; 16-bit outputs compare as bit patterns."""
import numpy as np
import pytest

from oracle import pyoracle as orc

pytestmark = pytest.mark.gpu

NP16 = {orc.BFLOAT16: "bfloat16", orc.HALF: "float16"}


def to16(torch, a, T):
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(getattr(torch, NP16[T])).view(torch.int16).numpy().view(np.uint16)


def run(hip, dev, x, y, rng_x, rng_y, adj_x=False, adj_y=False, binary=(), t_out=orc.FLOAT, x_off=0, y_off=0):
    """binary: (alg, numpy array) with float32 (fp32 output) or uint16 bit patterns (16-bit outputs)."""
    import torch
    scale = float(np.float32(np.float32(rng_x) * np.float32(rng_y)) / np.float32(127 * 127))
    # operands optionally placed at a byte offset inside a larger buffer (unaligned bases)
    xb = torch.zeros(x.size + 64, dtype=torch.int8, device=dev)
    yb = torch.zeros(y.size + 64, dtype=torch.int8, device=dev)
    xb[x_off:x_off + x.size] = torch.from_numpy(x.ravel()).to(dev)
    yb[y_off:y_off + y.size] = torch.from_numpy(y.ravel()).to(dev)
    keep, bins = [], []
    for alg, arr in binary:
        t = torch.from_numpy(arr.view(np.int16) if arr.dtype == np.uint16 else arr).to(dev)
        keep.append(t)
        bins.append((alg, t, arr.shape))
    p, oshape = hip.bmm_params(x.shape, y.shape, adj_x, adj_y, t_out, scale, bins)
    n_out = int(np.prod(oshape, dtype=np.int64))
    out = torch.full((max(n_out, 1),), -1, dtype=torch.float32 if t_out == orc.FLOAT else torch.int16, device=dev)
    hip.qbatch_matmul(p, xb.data_ptr() + x_off, yb.data_ptr() + y_off, out)
    torch.cuda.synchronize()
    got = out[:n_out].cpu().numpy().reshape(oshape)
    return got.view(np.uint16) if t_out != orc.FLOAT else got


def check(hip, dev, x, y, adj_x=False, adj_y=False, binary=(), t_out=orc.FLOAT, x_off=0, y_off=0, rx=3.0, ry=1.5):
    st, ref = orc.qbatch_matmul(x, y, -rx, rx * 0.5, -ry * 0.25, ry, adj_x, adj_y, binary, t_out)
    assert st == orc.OK
    got = run(hip, dev, x, y, rx, ry, adj_x, adj_y, binary, t_out, x_off, y_off)
    np.testing.assert_array_equal(got, ref)


@pytest.mark.parametrize("adj_x", [False, True])
@pytest.mark.parametrize("adj_y", [False, True])
@pytest.mark.parametrize("B,M,K,N", [((2,), 2, 3, 2), ((3,), 70, 64, 130), ((2, 2), 64, 128, 64), ((1,), 1, 1, 1),
                                     ((5,), 33, 17, 5), ((2,), 100, 200, 36), ((), 128, 48, 96), ((2, 1, 3), 20, 32, 24)])
def test_layouts_and_ragged_shapes(hip, dev, adj_x, adj_y, B, M, K, N):
    """Every operand layout on aligned (vector loads) and ragged (byte loads) shapes, partial tiles in M, N and K."""
    rng = np.random.default_rng(M * 7 + K * 3 + N + adj_x * 2 + adj_y)
    x = rng.integers(-128, 128, B + ((K, M) if adj_x else (M, K))).astype(np.int8)
    y = rng.integers(-128, 128, B + ((N, K) if adj_y else (K, N))).astype(np.int8)
    check(hip, dev, x, y, adj_x, adj_y)


@pytest.mark.parametrize("x_off,y_off", [(1, 0), (0, 3), (4, 16), (16, 4)])
def test_unaligned_operand_bases(hip, dev, x_off, y_off):
    """Aligned shapes at unaligned addresses must leave the vector-load path."""
    rng = np.random.default_rng(x_off + y_off)
    x = rng.integers(-128, 128, (3, 64, 64)).astype(np.int8)
    y = rng.integers(-128, 128, (3, 64, 64)).astype(np.int8)
    for adj_x in (False, True):
        for adj_y in (False, True):
            check(hip, dev, x, y, adj_x, adj_y, x_off=x_off, y_off=y_off)


def test_batch_broadcast(hip, dev):
    rng = np.random.default_rng(1)
    x = rng.integers(-128, 128, (4, 1, 40, 32)).astype(np.int8)
    y = rng.integers(-128, 128, (1, 5, 32, 24)).astype(np.int8)
    check(hip, dev, x, y)
    check(hip, dev, rng.integers(-128, 128, (40, 32)).astype(np.int8), y)                  # rank-2 x
    check(hip, dev, x, rng.integers(-128, 128, (24, 32)).astype(np.int8), adj_y=True)       # rank-2 y


def test_reference_cases(hip, dev, golden):
    """The three cases of the reference's quantized_batch_matmul_test.py (plain, Mul, Mul + Add; K = 3)."""
    g = golden["batch_matmul"]
    x, y, add = (np.array(g[k], np.float32) for k in ("x", "y", "add"))
    mul = np.float32([g["mul"]])
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QINT8, orc.SCALED)
    _, yq, ymn, ymx = orc.quantize_v2(y, y.min(), y.max(), orc.QINT8, orc.SCALED)
    for binary, ref32 in (((), x @ y), (((orc.BIN_MUL, mul),), (x @ y) * mul),
                          (((orc.BIN_MUL, mul), (orc.BIN_ADD, add)), (x @ y) * mul + add)):
        st, ref = orc.qbatch_matmul(xq, yq, xmn[0], xmx[0], ymn[0], ymx[0], binary=binary)
        assert st == orc.OK
        got = run(hip, dev, xq, yq, max(abs(xmn[0]), abs(xmx[0])), max(abs(ymn[0]), abs(ymx[0])), binary=binary)
        np.testing.assert_array_equal(got, ref)
        np.testing.assert_allclose(got, ref32, rtol=g["tolerance"], atol=g["tolerance"])


@pytest.mark.parametrize("t_out", [orc.FLOAT, orc.BFLOAT16, orc.HALF])
def test_attention_shapes_with_scale_and_mask(hip, dev, t_out):
    """Q.K^T with a scalar Mul and a broadcast additive mask, then P.V: BERT-base head shapes (S = 128, d = 64)."""
    import torch
    rng = np.random.default_rng(3)
    B, H, S, D = 2, 12, 128, 64
    q = rng.integers(-128, 128, (B, H, S, D)).astype(np.int8)
    k = rng.integers(-128, 128, (B, H, S, D)).astype(np.int8)
    v = rng.integers(-128, 128, (B, H, S, D)).astype(np.int8)
    pr = rng.integers(-128, 128, (B, H, S, S)).astype(np.int8)
    mul = np.float32([0.125])
    mask = np.where(rng.random((B, 1, 1, S)) < 0.2, np.float32(-10000.0), np.float32(0.0)).astype(np.float32)
    if t_out != orc.FLOAT:
        mul, mask = to16(torch, mul, t_out), to16(torch, mask, t_out)
    check(hip, dev, q, k, adj_y=True, binary=((orc.BIN_MUL, mul), (orc.BIN_ADD, mask)), t_out=t_out)
    check(hip, dev, pr, v, t_out=t_out)
    full = rng.standard_normal((B, H, S, S)).astype(np.float32)
    if t_out != orc.FLOAT:
        full = to16(torch, full, t_out)
    check(hip, dev, q, k, adj_y=True, binary=((orc.BIN_ADD, full), (orc.BIN_MUL, mul)), t_out=t_out)   # other order


def test_binary_operand_broadcast_forms(hip, dev):
    rng = np.random.default_rng(4)
    x = rng.integers(-128, 128, (2, 3, 37, 16)).astype(np.int8)
    y = rng.integers(-128, 128, (2, 3, 16, 21)).astype(np.int8)
    for shape in [(2, 3, 37, 21), (1, 1, 1, 1), (2, 1, 37, 1), (1, 3, 1, 21), (1, 1, 37, 21), (1,)]:
        t = rng.standard_normal(shape).astype(np.float32)
        check(hip, dev, x, y, binary=((orc.BIN_ADD, t),))
        check(hip, dev, x, y, binary=((orc.BIN_MUL, t), (orc.BIN_ADD, t)))


@pytest.mark.parametrize("seed", range(4))
def test_random_shapes_layouts_and_operands(hip, dev, seed):
    """Seeded random batch shapes, matrix sizes, layouts, operand base offsets, output types and fused operands in every
    broadcast form, each case launched twice."""
    import torch
    rng = np.random.default_rng(3000 + seed)
    for case in range(25):
        B = [(), (1,), (3,), (2, 2), (2, 1, 3)][int(rng.integers(0, 5))]
        M = int(rng.choice([1, 5, 16, 31, 32, 33, 64, 70, 100, 128, 130]))
        K = int(rng.choice([1, 4, 16, 17, 32, 48, 64, 100, 128, 200]))
        N = int(rng.choice([1, 4, 8, 21, 32, 36, 64, 96, 128, 130]))
        adj_x, adj_y = bool(rng.random() < 0.3), bool(rng.random() < 0.5)
        t_out = [orc.FLOAT, orc.FLOAT, orc.BFLOAT16, orc.HALF][int(rng.integers(0, 4))]
        x = rng.integers(-128, 128, B + ((K, M) if adj_x else (M, K))).astype(np.int8)
        y = rng.integers(-128, 128, B + ((N, K) if adj_y else (K, N))).astype(np.int8)
        ones = (1,) * len(B)
        binary = []
        for _ in range(int(rng.choice([0, 0, 1, 2]))):
            shape = [(1,), B + (M, N), ones + (1, N), ones + (M, 1), ones + (M, N)][int(rng.integers(0, 5))]
            t = rng.standard_normal(shape).astype(np.float32)
            if t_out != orc.FLOAT:
                t = to16(torch, t, t_out)
            binary.append((orc.BIN_MUL if rng.random() < 0.5 else orc.BIN_ADD, t))
        x_off, y_off = [(0, 0), (16, 16), (1, 0), (4, 3)][int(rng.integers(0, 4))]
        for launch in range(2):
            check(hip, dev, x, y, adj_x, adj_y, tuple(binary), t_out, x_off, y_off)


@pytest.mark.parametrize("adj_x,adj_y", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("M,K,N", [(72, 48, 132), (128, 64, 128), (100, 80, 36), (68, 16, 64)])
def test_tiles_of_128_rows(hip, dev, adj_x, adj_y, M, K, N):
    """Calls with at least 1024 tiles of 128 rows, aligned operands and fused operands that do not depend on the row run
    tiles of 128 x 128 (N > 64) or 128 x 64 outputs, ragged at both edges here; every layout, fp32 without operands,
    bfloat16 with a scalar Mul and a mask broadcast over the rows, and with a per-row operand the 64 x 64 tiles again."""
    import torch
    rng = np.random.default_rng(M + K + N + adj_x * 2 + adj_y)
    B = (1030,)
    x = rng.integers(-128, 128, B + ((K, M) if adj_x else (M, K))).astype(np.int8)
    y = rng.integers(-128, 128, B + ((N, K) if adj_y else (K, N))).astype(np.int8)
    check(hip, dev, x, y, adj_x, adj_y)
    mul = to16(torch, np.float32([0.125]), orc.BFLOAT16)
    mask = to16(torch, np.where(rng.random((1, 1, N)) < 0.3, np.float32(-100.0), np.float32(0.0)).astype(np.float32), orc.BFLOAT16)
    check(hip, dev, x, y, adj_x, adj_y, binary=((orc.BIN_MUL, mul), (orc.BIN_ADD, mask)), t_out=orc.BFLOAT16)
    if (adj_x, adj_y) == (False, True):
        per_row = rng.standard_normal((1, M, 1)).astype(np.float32)
        check(hip, dev, x, y, adj_x, adj_y, binary=((orc.BIN_ADD, per_row),))


def test_empty_and_invalid(hip, dev):
    import torch
    z = np.zeros((2, 0, 8), np.int8)
    y = np.ones((2, 8, 4), np.int8)
    assert run(hip, dev, z, y, 1.0, 1.0).shape == (2, 0, 4)
    # K = 0: an empty sum times the scale
    got = run(hip, dev, np.zeros((2, 5, 0), np.int8), np.zeros((2, 0, 4), np.int8), 1.0, 1.0)
    np.testing.assert_array_equal(got, np.zeros((2, 5, 4), np.float32))
    p, _ = hip.bmm_params((2, 4, 8), (2, 8, 4), False, False, orc.QINT8, 1.0)
    out = torch.empty(64, dtype=torch.float32, device=dev)
    with pytest.raises(hip.ItexHipError):
        hip.qbatch_matmul(p, out, out, out)              # integer output types do not exist for this op
    p, _ = hip.bmm_params((2, 4, 8), (2, 8, 4), False, False, orc.FLOAT, 1.0)
    p.n_binary = 3
    with pytest.raises(hip.ItexHipError):
        hip.qbatch_matmul(p, out, out, out)
    p.n_binary = 0
    with pytest.raises(hip.ItexHipError):
        hip.qbatch_matmul(p, None, out, out)


def test_many_small_matrices(hip, dev):
    rng = np.random.default_rng(6)
    x = rng.integers(-128, 128, (3000, 8, 16)).astype(np.int8)
    y = rng.integers(-128, 128, (3000, 16, 8)).astype(np.int8)
    check(hip, dev, x, y)


def test_half_output_is_rounded_from_the_fp32_result(hip, dev):
    """float(acc) * scale is rounded to fp32 and only then to half.  A conversion fused with the multiply would round
    the exact product once; the two differ on a handful of elements per million, which this problem contains."""
    rng = np.random.default_rng(11)
    x = rng.integers(-128, 128, (16, 256, 32)).astype(np.int8)
    y = rng.integers(-128, 128, (16, 32, 256)).astype(np.int8)
    rx, ry = 3.0, 1.5
    acc = np.matmul(x.astype(np.int64), y.astype(np.int64)).astype(np.float64)
    scale = np.float64(np.float32(np.float32(rx) * np.float32(ry)) / np.float32(127 * 127))
    with np.errstate(over="ignore"):
        once = (acc * scale).astype(np.float16)                          # exact product, one rounding
        twice = (acc * scale).astype(np.float32).astype(np.float16)      # what the op defines
    differ = once.view(np.uint16) != twice.view(np.uint16)
    assert differ.sum() >= 3
    got = run(hip, dev, x, y, rx, ry, t_out=orc.HALF)
    np.testing.assert_array_equal(got[differ], twice.view(np.uint16)[differ])
    st, ref = orc.qbatch_matmul(x, y, -rx, rx * 0.5, -ry * 0.25, ry, t_out=orc.HALF)
    np.testing.assert_array_equal(got, ref)
