"""GPU parity of the quantized MatMul path through the C ABI versus the CPU oracle:
prepack + column sums, device-side parameter preparation, MFMA tile kernel, small-M kernel and the
shape-agnostic kernel.  int32 accumulators / int8 outputs / prepared vectors bit-exact; fp32 outputs
bit-exact as well (bar: 1 ULP of the int32->fp32 scale product)."""
import numpy as np
import pytest

from oracle import pyoracle as orc

pytestmark = pytest.mark.gpu


def tdt(T):
    import torch
    return {orc.QINT8: torch.int8, orc.QUINT8: torch.uint8, orc.QINT32: torch.int32, orc.FLOAT: torch.float32,
            orc.BFLOAT16: torch.int16, orc.HALF: torch.int16}[T]   # bfloat16 / half travel as bit patterns


def bits16(a):
    return a.view(np.uint16) if a.dtype == np.int16 else a


class Linear:
    """A quantized linear layer resident on the GPU (weights prepacked once)."""

    def __init__(self, hip, dev, wq, min_b, max_b, bias):
        import torch
        self.hip, self.dev = hip, dev
        self.K, self.N = wq.shape
        self.wq, self.min_b, self.max_b, self.bias = wq, np.atleast_1d(min_b), np.atleast_1d(max_b), bias
        self.w_d = torch.from_numpy(wq).to(dev)
        self.packed = torch.empty(hip.qgemm_packed_bytes(self.K, self.N), dtype=torch.int8, device=dev)
        self.colsum = torch.empty(self.N, dtype=torch.int32, device=dev)
        hip.qgemm_prepack_b(self.w_d, False, self.K, self.N, self.packed, self.colsum)
        self.min_b_d = torch.from_numpy(self.min_b.astype(np.float32)).to(dev)
        self.max_b_d = torch.from_numpy(self.max_b.astype(np.float32)).to(dev)
        self.bias_d = torch.from_numpy(bias).to(dev)
        self.scales_d = torch.empty(max(self.N, 1), dtype=torch.float32, device=dev)
        self.sbias_d = torch.empty(self.N, dtype=torch.float32, device=dev)

    def run(self, xq, kw, min_a, max_a, min_out=0.0, max_out=0.0, path="auto"):
        import torch
        hip = self.hip
        M = xq.shape[0]
        t_in = orc.QUINT8 if xq.dtype == np.uint8 else orc.QINT8
        p = hip.matmul_params(t_in=t_in, min_a=float(min_a), max_a=float(max_a), min_out=float(min_out),
                              max_out=float(max_out), **kw)
        nb = self.min_b.size
        ep = hip.qmatmul_epilogue_desc(p, nb)
        hip.qmatmul_prepare(p, self.min_b_d, self.max_b_d, nb, self.bias_d, self.colsum, self.N,
                            self.scales_d, self.sbias_d)
        x_d = torch.from_numpy(xq).to(self.dev)
        out = torch.empty((M, self.N), dtype=tdt(kw["t_out"]), device=self.dev)
        out.view(torch.uint8).fill_(0x55)        # an element the kernel does not write cannot pass by luck
        fn = {"auto": hip.qgemm, "tile": hip.qgemm_tile, "gemv": hip.qgemv}.get(path)
        if path == "fused":
            hip.qmatmul(p, x_d, self.packed, self.colsum, M, self.K, self.N, self.min_b_d, self.max_b_d, nb,
                        self.bias_d, out)
        elif path == "naive":
            hip.qgemm_naive(x_d, t_in, self.w_d, False, M, self.K, self.N, self.scales_d, self.sbias_d, ep,
                            kw["t_out"], out)
        else:
            fn(x_d, t_in, self.packed, self.colsum, M, self.K, self.N, self.scales_d, self.sbias_d, ep,
               kw["t_out"], out)
        torch.cuda.synchronize()
        return out.cpu().numpy()

    def oracle(self, xq, kw, min_a, max_a, min_out=0.0, max_out=0.0):
        t_in = orc.QUINT8 if xq.dtype == np.uint8 else orc.QINT8
        at = orc.matmul_attrs(t_in=t_in, **kw)
        st, y = orc.qmatmul(at, xq, self.wq, self.bias, min_a, max_a, self.min_b, self.max_b, min_out, max_out)
        assert st == orc.OK
        return y


def make_layer(hip, dev, K, N, seed, per_channel=True, wstd=0.02):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((K, N)) * wstd).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
    if per_channel:
        r = np.abs(w).max(0).astype(np.float32)
        _, wq, mn, mx = orc.quantize_v2(w, -r, r, orc.QINT8, orc.SCALED, axis=1)
    else:
        _, wq, mn, mx = orc.quantize_v2(w, w.min(), w.max(), orc.QINT8, orc.SCALED)
    return Linear(hip, dev, wq, mn, mx, bias), w, bias


def make_acts(M, K, seed, mode=orc.MIN_FIRST, outlier=0.0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K)).astype(np.float32)
    if outlier:
        idx = rng.integers(0, x.size, max(1, int(x.size * outlier)))
        x.flat[idx] *= 20.0
    T = orc.QUINT8 if mode == orc.MIN_FIRST else orc.QINT8
    _, xq, mn, mx = orc.quantize_v2(x, x.min(), x.max(), T, mode)
    return x, xq, float(mn[0]), float(mx[0])


V2_DEQ = dict(api=orc.API_V2, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST, has_dequantize=True)
V2_DEQ_RELU = dict(V2_DEQ, activation=orc.ACT_RELU)
V2_REQ_S8 = dict(api=orc.API_V2, t_out=orc.QINT8, input_mode=orc.MIN_FIRST, has_requantize=True)
V2_REQ_U8_RELU = dict(api=orc.API_V2, t_out=orc.QUINT8, input_mode=orc.MIN_FIRST, has_requantize=True,
                      activation=orc.ACT_RELU, n_fused_ops=2)
V1_S32 = dict(api=orc.API_V1, t_out=orc.QINT32, input_mode=orc.MIN_FIRST, n_fused_ops=1)


def test_prepack_colsum(hip, dev):
    import torch
    rng = np.random.default_rng(0)
    for (K, N) in [(64, 16), (3, 4), (100, 37), (4096, 1024), (130, 48)]:
        w = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
        w_d = torch.from_numpy(w).to(dev)
        nbytes = hip.qgemm_packed_bytes(K, N)
        packed = torch.full((nbytes,), 77, dtype=torch.int8, device=dev)
        colsum = torch.full((N,), 123, dtype=torch.int32, device=dev)
        hip.qgemm_prepack_b(w_d, False, K, N, packed, colsum)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(colsum.cpu().numpy(), orc.weight_colsum(w))
        # layout: chunk [n/32][k/32] (k padded to a multiple of 64), lane (n%32) + 32*((k%32)/16),
        # 16 consecutive k per lane
        KC, NT = 2 * ((K + 63) // 64), (N + 31) // 32
        wp = np.zeros((NT * 32, KC * 32), np.int8)
        wp[:N, :K] = w.T
        ref = wp.reshape(NT, 32, KC, 2, 16).transpose(0, 2, 3, 1, 4).reshape(-1)
        np.testing.assert_array_equal(packed.cpu().numpy(), ref)
        # transposed source gives the same packing
        wt_d = torch.from_numpy(np.ascontiguousarray(w.T)).to(dev)
        packed2 = torch.empty_like(packed)
        hip.qgemm_prepack_b(wt_d, True, K, N, packed2, colsum)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(packed2.cpu().numpy(), ref)


@pytest.mark.parametrize("kw", [V2_DEQ, V2_REQ_S8, V2_REQ_U8_RELU, V1_S32,
                                dict(api=orc.API_V1, t_out=orc.QINT8, input_mode=orc.MIN_FIRST, n_fused_ops=1),
                                dict(api=orc.API_V2, t_out=orc.QUINT8, input_mode=orc.MIN_FIRST, has_requantize=True,
                                     out_min_first=True, activation=orc.ACT_RELU),
                                dict(api=orc.API_V2, t_out=orc.FLOAT, input_mode=orc.SCALED, has_dequantize=True),
                                dict(api=orc.API_V2, t_out=orc.QINT32, input_mode=orc.SCALED)])
@pytest.mark.parametrize("per_channel", [True, False])
def test_prepare_vs_oracle(hip, dev, kw, per_channel):
    import torch
    N, K = 200, 64
    layer, w, bias = make_layer(hip, dev, K, N, 3, per_channel)
    t_in = orc.QUINT8 if kw["input_mode"] == orc.MIN_FIRST else orc.QINT8
    min_a, max_a, min_out, max_out = -2.3, 3.1, -1.7, 2.9
    at = orc.matmul_attrs(t_in=t_in, **kw)
    cs = orc.weight_colsum(layer.wq)
    st, sc_ref, sb_ref, ep_ref = orc.qmatmul_prepare(at, N, cs, min_a, max_a, layer.min_b, layer.max_b,
                                                     min_out, max_out, bias)
    assert st == orc.OK
    p = hip.matmul_params(t_in=t_in, min_a=min_a, max_a=max_a, min_out=min_out, max_out=max_out, **kw)
    nb = layer.min_b.size
    layer.scales_d.fill_(-7.0)
    hip.qmatmul_prepare(p, layer.min_b_d, layer.max_b_d, nb, layer.bias_d, layer.colsum, N, layer.scales_d,
                        layer.sbias_d)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(layer.sbias_d.cpu().numpy(), sb_ref)
    np.testing.assert_array_equal(layer.scales_d.cpu().numpy()[:ep_ref.n_scales], sc_ref)


def test_reference_fused_matmul_case(hip, dev, golden):
    """The 2x3 . 3x4 case of the reference's own test (K = 3 goes through the shape-agnostic kernel)."""
    g = golden["fused_matmul"]
    x = np.array(g["x"], np.float32)
    w = np.array(g["w"], np.float32)
    b = np.array(g["bias"], np.float32)
    _, xq, xmn, xmx = orc.quantize_v2(x, x.min(), x.max(), orc.QUINT8, orc.MIN_FIRST)
    for per_channel in (False, True):
        if per_channel:
            _, wq, wmn, wmx = orc.quantize_v2(w, w.min(0), w.max(0), orc.QINT8, orc.SCALED, axis=1)
        else:
            _, wq, wmn, wmx = orc.quantize_v2(w, w.min(), w.max(), orc.QINT8, orc.SCALED)
        layer = Linear(hip, dev, wq, wmn, wmx, b)
        for api in (orc.API_V1, orc.API_V2):
            kw = dict(V2_DEQ, api=api)
            y = layer.run(xq, kw, xmn[0], xmx[0], path="naive")
            np.testing.assert_allclose(y, x @ w + b, rtol=g["tolerance"], atol=g["tolerance"])
            np.testing.assert_array_equal(y, layer.oracle(xq, kw, xmn[0], xmx[0]))


SHAPES = [(17, 64, 16), (32, 128, 48), (100, 256, 200), (256, 512, 256), (300, 1024, 520), (128, 1024, 1024),
          (513, 192, 1000), (64, 4096, 64)]


@pytest.mark.parametrize("M,K,N", SHAPES)
@pytest.mark.parametrize("kw", [V2_DEQ_RELU, V2_REQ_S8, V1_S32])
def test_tile_kernel_vs_oracle(hip, dev, M, K, N, kw):
    layer, w, bias = make_layer(hip, dev, K, N, seed=K + N)
    x, xq, mn, mx = make_acts(M, K, seed=M)
    r_out = float(np.abs(x @ w + bias).max())
    ref = layer.oracle(xq, kw, mn, mx, -r_out, r_out)
    got = layer.run(xq, kw, mn, mx, -r_out, r_out, path="tile")
    np.testing.assert_array_equal(got, ref)
    np.testing.assert_array_equal(layer.run(xq, kw, mn, mx, -r_out, r_out, path="fused"), ref)


@pytest.mark.parametrize("M,K,N", [(127, 240, 8316), (100, 144, 8340)])
def test_tile_kernel_repeated_launches_equal_the_oracle(hip, dev, M, K, N):
    """fp32 outputs of the tile kernel, many workgroups, K not a multiple of 64, launched several times: every launch
    must equal the oracle (an epilogue store whose data registers were overwritten too early showed as a few wrong
    elements in some launches only)."""
    layer, w, bias = make_layer(hip, dev, K, N, seed=K + N)
    x, xq, mn, mx = make_acts(M, K, seed=M)
    ref = layer.oracle(xq, V2_DEQ_RELU, mn, mx)
    for launch in range(8):
        np.testing.assert_array_equal(layer.run(xq, V2_DEQ_RELU, mn, mx, path="tile"), ref, err_msg="launch %d" % launch)


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_on_every_path_vs_oracle(hip, dev, monkeypatch, seed):
    """Seeded random problem sizes (ragged in M, N and K), output types and forced tile shapes; the tile kernel, the
    small-M kernel where it takes the row count, the dispatching entry point and the single-launch op against the
    oracle, each launched twice into pre-filled outputs."""
    rng = np.random.default_rng(1000 + seed)
    for case in range(8):
        M = int(rng.choice([1, 3, 16, 17, 33, 64, 100, 127, 128, 129, 200, 257, 300]))
        K = 16 * int(rng.integers(1, 48))
        N = 4 * int(rng.integers(1, 500)) if case % 2 else 16 * int(rng.integers(1, 130))
        kw = [V2_DEQ, V2_DEQ_RELU, V2_REQ_S8, V2_REQ_U8_RELU, V1_S32][int(rng.integers(0, 5))]
        shape = int(rng.integers(-1, 5))
        if shape >= 0:
            hip.force_tile_shape(matmul=shape)
        else:
            hip.force_tile_shape(matmul=-1)
        layer, w, bias = make_layer(hip, dev, K, N, seed=seed * 100 + case)
        x, xq, mn, mx = make_acts(M, K, seed=seed * 100 + case + 50)
        full = x @ w + bias
        r_out = float(np.abs(np.maximum(full, 0) if kw.get("activation") else full).max())
        lo = 0.0 if kw["t_out"] == orc.QUINT8 else -r_out
        ref = layer.oracle(xq, kw, mn, mx, lo, r_out)
        for path in ("tile", "auto", "fused") + (("gemv",) if M <= 128 else ()):
            for launch in range(2):
                np.testing.assert_array_equal(layer.run(xq, kw, mn, mx, lo, r_out, path=path), ref,
                                              err_msg="case %d: M %d K %d N %d shape %d %s launch %d" % (case, M, K, N, shape, path, launch))


@pytest.mark.parametrize("M,K,N", [(17, 64, 16), (32, 4096, 1000), (33, 448, 528), (64, 1024, 100), (100, 256, 200),
                                   (128, 1024, 1024), (127, 2048, 24), (48, 80, 2051)])
@pytest.mark.parametrize("kw", [V2_DEQ_RELU, V2_REQ_S8, V2_REQ_U8_RELU, V1_S32])
def test_small_m_kernel_in_row_blocks_vs_oracle(hip, dev, M, K, N, kw):
    """17 .. 128 rows go through the small-M kernel in blocks of 16 rows (ragged last block, strips that do not fill a
    group of 8, K not a multiple of 64): forced, through the dispatching entry point and as the single-launch op."""
    layer, w, bias = make_layer(hip, dev, K, N, seed=K + N + 1)
    x, xq, mn, mx = make_acts(M, K, seed=M + 3)
    full = x @ w + bias
    r_out = float(np.abs(np.maximum(full, 0) if kw.get("activation") else full).max())
    lo = 0.0 if kw["t_out"] == orc.QUINT8 else -r_out
    ref = layer.oracle(xq, kw, mn, mx, lo, r_out)
    for path in ("gemv", "auto", "fused"):
        np.testing.assert_array_equal(layer.run(xq, kw, mn, mx, lo, r_out, path=path), ref, err_msg=path)


@pytest.mark.parametrize("kw", [V2_DEQ, V2_DEQ_RELU, V2_REQ_S8, V2_REQ_U8_RELU, V1_S32,
                                dict(api=orc.API_V1, t_out=orc.QINT8, input_mode=orc.MIN_FIRST, n_fused_ops=1),
                                dict(api=orc.API_LEGACY, t_out=orc.QUINT8, input_mode=orc.MIN_FIRST, activation=orc.ACT_RELU),
                                dict(api=orc.API_LEGACY, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST),
                                dict(api=orc.API_V2, t_out=orc.FLOAT, input_mode=orc.SCALED, has_dequantize=True)])
@pytest.mark.parametrize("per_channel", [True, False])
@pytest.mark.parametrize("M", [5, 200])
def test_single_launch_op_vs_oracle(hip, dev, kw, per_channel, M):
    """itexhip_qmatmul derives the per-channel parameters inside the MatMul kernel (GEMV and tile paths)."""
    if kw["api"] == orc.API_LEGACY and per_channel:
        pytest.skip("the legacy ops take per-tensor weight ranges")
    K, N = 320, 272
    layer, w, bias = make_layer(hip, dev, K, N, seed=77, per_channel=per_channel)
    mode = kw["input_mode"]
    x, xq, mn, mx = make_acts(M, K, seed=M, mode=mode)
    full = x @ w + bias
    r_out = float(np.abs(np.maximum(full, 0) if kw.get("activation") else full).max())
    lo = 0.0 if kw["t_out"] == orc.QUINT8 else -r_out
    ref = layer.oracle(xq, kw, mn, mx, lo, r_out)
    np.testing.assert_array_equal(layer.run(xq, kw, mn, mx, lo, r_out, path="fused"), ref)


@pytest.mark.parametrize("shape", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("M,K,N,kw", [(300, 448, 528, V2_REQ_S8), (513, 192, 400, V2_DEQ_RELU), (257, 64, 208, V1_S32),
                                      (40, 1024, 96, V2_REQ_U8_RELU), (256, 320, 200, V2_REQ_S8)])
def test_every_tile_shape_on_ragged_problems(hip, dev, monkeypatch, shape, M, K, N, kw):
    """The tile shape is normally chosen from the problem size; itexhip_test_force_tile_shape forces one, so that
    every shape (256x256, 256x192, 256x128, 128x128, 64x64) meets partial tiles in M and N, odd step
    counts, K not a multiple of 64 and the element-wise store path (N * element size not a multiple of 16)."""
    hip.force_tile_shape(matmul=shape)
    layer, w, bias = make_layer(hip, dev, K, N, seed=K + N + shape)
    x, xq, mn, mx = make_acts(M, K, seed=M)
    r_out = float(np.abs(np.maximum(x @ w + bias, 0) if kw.get("activation") else x @ w + bias).max())
    lo = 0.0 if kw["t_out"] == orc.QUINT8 else -r_out
    ref = layer.oracle(xq, kw, mn, mx, lo, r_out)
    got = layer.run(xq, kw, mn, mx, lo, r_out, path="tile")
    np.testing.assert_array_equal(got, ref)


CHAINS = {   # post-op chains of the form [activation] [linear map] that the vector epilogue resolves on the host
    "leaky_f32": dict(V2_DEQ, activation=orc.ACT_LEAKYRELU, leakyrelu_alpha=0.2),
    "relu6_f32": dict(V2_DEQ, activation=orc.ACT_RELU6),
    "leaky_req_s8": dict(V2_REQ_S8, activation=orc.ACT_LEAKYRELU, leakyrelu_alpha=0.1),
    "relu6_req_u8": dict(V2_REQ_U8_RELU, activation=orc.ACT_RELU6),
    "relu_req_minfirst_u8": dict(V2_REQ_U8_RELU, out_min_first=True),       # ReLU, then the linear map of a MIN_FIRST output
    "leaky_req_minfirst_s8": dict(V2_REQ_S8, activation=orc.ACT_LEAKYRELU, leakyrelu_alpha=0.3, out_min_first=True),
    "req_minfirst_s8": dict(V2_REQ_S8, out_min_first=True),                 # the linear map alone
    "gelu_tanh_f32": dict(V2_DEQ, activation=orc.ACT_GELU_APPROX),
    "gelu_erf_bf16": dict(V2_DEQ, activation=orc.ACT_GELU_EXACT, t_out=orc.BFLOAT16),
    "transc_tanh_f32": dict(V2_DEQ, activation=orc.ACT_TANH),
    "transc_sigmoid_f32": dict(V2_DEQ, activation=orc.ACT_SIGMOID),
    "transc_swish_f32": dict(V2_DEQ, activation=orc.ACT_SWISH),
    "transc_elu_f32": dict(V2_DEQ, activation=orc.ACT_ELU),
    "transc_mish_bf16": dict(V2_DEQ, activation=orc.ACT_MISH, t_out=orc.BFLOAT16),
}


@pytest.mark.parametrize("shape", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("chain", sorted(CHAINS))
def test_canonical_chains_every_tile_shape(hip, dev, monkeypatch, shape, chain):
    """Every tile shape with every kind of run-time post-op chain, K a multiple of 64 (uniform activation addresses)
    and not (per-lane clamped addresses), ragged M and N: bit-equal to the oracle except for the GELU and the other
    transcendental chains, where the device's exp / erf need not round like the host's (2e-6 relative, 1e-6 absolute; one unit of the
    output type where that is coarser)."""
    hip.force_tile_shape(matmul=shape)
    kw = CHAINS[chain]
    for M, K, N in [(300, 448, 528), (257, 208, 400)]:
        layer, w, bias = make_layer(hip, dev, K, N, seed=K + N + shape)
        x, xq, mn, mx = make_acts(M, K, seed=M + 1)
        r_out = float(np.abs(x @ w + bias).max())
        lo = 0.0 if kw["t_out"] == orc.QUINT8 else -r_out
        ref = layer.oracle(xq, kw, mn, mx, lo, r_out)
        for path in ("tile", "fused"):
            got = layer.run(xq, kw, mn, mx, lo, r_out, path=path)
            if "gelu" not in chain and "transc" not in chain:
                np.testing.assert_array_equal(got, ref)
            elif kw["t_out"] == orc.FLOAT:
                np.testing.assert_allclose(got, ref, rtol=2e-6, atol=1e-6)
            else:   # bfloat16 bit patterns: equal, or neighbours where the fp32 values straddle a rounding boundary
                d = np.abs(bits16(got).astype(np.int64) - bits16(ref).astype(np.int64))
                assert d.max() <= 1 and (d > 0).mean() < 1e-3


@pytest.mark.parametrize("T,mode", [(orc.QUINT8, orc.MIN_FIRST), (orc.QINT8, orc.SCALED), (orc.QUINT8, orc.SCALED)],
                         ids=["min_first_u8", "scaled_s8", "scaled_u8"])
@pytest.mark.parametrize("M,K,N", [(4, 448, 528), (300, 448, 528), (16, 1024, 96), (257, 208, 400), (1, 16, 8), (513, 64, 2051)])
def test_dynamic_quantize_then_device_range_matmul(hip, dev, T, mode, M, K, N):
    """itexhip_quantize_dynamic + itexhip_qmatmul_device_range: the range of the float tensor, the op's parameter
    math, the quantization and the MatMul's scale / bias derivation all on the device.  Bit-equal to QuantizeV2 fed
    with the tensor's min and max followed by the MatMul fed with its output range (oracle), for the small-M and the
    tile kernels, unaligned sizes included."""
    import torch
    rng = np.random.default_rng(M * 7 + K + N)
    x = (rng.standard_normal((M, K)) * 2.5 + (0.4 if T == orc.QUINT8 and mode == orc.SCALED else 0.0)).astype(np.float32)
    if T == orc.QUINT8 and mode == orc.SCALED:
        x = np.abs(x)
    layer, w, bias = make_layer(hip, dev, K, N, seed=K + N + 3)
    _, xq_ref, omn, omx = orc.quantize_v2(x, x.min(), x.max(), T, mode)
    x_d = torch.from_numpy(x).to(dev)
    xq_d = torch.empty((M, K), dtype=tdt(T), device=dev)
    state = torch.full((hip.DYNAMIC_STATE_FLOATS,), float("nan"), dtype=torch.float32, device=dev)
    for emr in (0.01,):
        hip.quantize_dynamic(x_d, xq_d, M * K, T, mode, emr, state)
    torch.cuda.synchronize()
    st = state.cpu().numpy()
    assert st[0] == x.min() and st[1] == x.max()
    assert st[2] == omn[0] and st[3] == omx[0]
    np.testing.assert_array_equal(xq_d.cpu().numpy(), xq_ref)
    r_out = float(np.abs(x @ w + bias).max())
    for kw in (dict(V2_DEQ, input_mode=mode), dict(V2_REQ_S8, input_mode=mode),
               dict(V2_DEQ, input_mode=mode, activation=orc.ACT_GELU_APPROX)):
        p = hip.matmul_params(t_in=T, min_a=123.0, max_a=-7.0, min_out=-r_out, max_out=r_out, **kw)   # min_a / max_a unused
        out = torch.empty((M, N), dtype=tdt(kw["t_out"]), device=dev)
        hip.qmatmul_device_range(p, xq_d, layer.packed, layer.colsum, M, K, N, state[2:], layer.min_b_d, layer.max_b_d,
                                 layer.min_b.size, layer.bias_d, out)
        torch.cuda.synchronize()
        ref = layer.oracle(xq_ref, kw, float(omn[0]), float(omx[0]), -r_out, r_out)
        if kw.get("activation"):
            np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=2e-6, atol=1e-6)
        else:
            np.testing.assert_array_equal(out.cpu().numpy(), ref)


@pytest.mark.parametrize("T,mode", [(orc.QUINT8, orc.MIN_FIRST), (orc.QINT8, orc.SCALED)], ids=["min_first_u8", "scaled_s8"])
@pytest.mark.parametrize("M,K,N", [(16, 1024, 96), (5, 448, 528), (3, 75 * 16, 40), (1, 16, 8)])
def test_per_token_dynamic_quantize_then_per_row_matmul(hip, dev, T, mode, M, K, N):
    """itexhip_quantize_dynamic_rows + itexhip_qmatmul_per_row: every row quantized against its own range on the device
    and multiplied with that range.  Row m equals QuantizeV2 (axis 0, the rows' min / max) and the 1 x K MatMul fed with
    row m's output range (oracle); also with an unaligned view (scalar path)."""
    import torch
    rng = np.random.default_rng(M + K)
    x = (rng.standard_normal((M, K)) * (1.0 + np.arange(M)[:, None])).astype(np.float32)
    layer, w, bias = make_layer(hip, dev, K, N, seed=K + N + 9)
    _, xq_ref, omn, omx = orc.quantize_v2(x, x.min(1), x.max(1), T, mode, axis=0)
    for shift in (0, 1):     # 1: the tensor starts 4 bytes off a 16-byte boundary
        buf = torch.zeros(M * K + 4, dtype=torch.float32, device=dev)
        x_d = buf[shift:shift + M * K].view(M, K)
        x_d.copy_(torch.from_numpy(x))
        xq_d = torch.empty((M, K), dtype=tdt(T), device=dev)
        rmn = torch.empty(M, dtype=torch.float32, device=dev)
        rmx = torch.empty(M, dtype=torch.float32, device=dev)
        hip.quantize_dynamic_rows(x_d, xq_d, M, K, T, mode, 0.01, rmn, rmx)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(xq_d.cpu().numpy(), xq_ref)
        np.testing.assert_array_equal(rmn.cpu().numpy(), omn)
        np.testing.assert_array_equal(rmx.cpu().numpy(), omx)
    kw = dict(V2_DEQ, input_mode=mode)
    p = hip.matmul_params(t_in=T, **kw)
    out = torch.empty((M, N), dtype=torch.float32, device=dev)
    hip.qmatmul_per_row(p, xq_d, layer.packed, layer.colsum, M, K, N, rmn, rmx, layer.min_b_d, layer.max_b_d, layer.min_b.size,
                        layer.bias_d, out)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    for m in range(M):
        ref = layer.oracle(xq_ref[m:m + 1], kw, float(omn[m]), float(omx[m]))
        np.testing.assert_array_equal(got[m:m + 1], ref)


def test_dynamic_quantize_range_floor_and_constant_tensors(hip, dev):
    """ensure_minimum_range widens a degenerate range exactly as the host code does (quantize_op.h:130-152): all-zero,
    constant positive, constant negative and tiny tensors, both modes."""
    import torch
    for fill, emr in ((0.0, 0.01), (3.0, 0.01), (-2.0, 0.01), (1e-6, 0.5), (0.0, 0.0 + 1e-3)):
        x = np.full(37, fill, np.float32)
        for T, mode, classic in ((orc.QUINT8, orc.MIN_FIRST, False), (orc.QINT8, orc.SCALED, False),
                                 (orc.QUINT8, orc.MIN_FIRST, True), (orc.QINT8, orc.MIN_FIRST, True)):
            _, q_ref, omn, omx = orc.quantize_v2(x, x.min(), x.max(), T, mode, ensure_minimum_range=emr, classic=classic)
            mode = 3 if classic else mode     # ITEXHIP_MIN_FIRST_CLASSIC
            x_d = torch.from_numpy(x).to(dev)
            q_d = torch.empty(37, dtype=tdt(T), device=dev)
            state = torch.zeros(hip.DYNAMIC_STATE_FLOATS, dtype=torch.float32, device=dev)
            hip.quantize_dynamic(x_d, q_d, 37, T, mode, emr, state)
            torch.cuda.synchronize()
            st = state.cpu().numpy()
            assert st[2] == omn[0] and st[3] == omx[0], (fill, emr, T, st, omn, omx)
            np.testing.assert_array_equal(q_d.cpu().numpy(), q_ref)
    # a tensor that starts 4 bytes off a 16-byte boundary takes the grid-wide reduction with atomics
    x = np.random.default_rng(1).standard_normal(70003).astype(np.float32)
    buf = torch.zeros(70004, dtype=torch.float32, device=dev)
    buf[1:].copy_(torch.from_numpy(x))
    q_d = torch.empty(70003, dtype=torch.int8, device=dev)
    hip.quantize_dynamic(buf[1:], q_d, 70003, orc.QINT8, orc.SCALED, 0.01, state)
    torch.cuda.synchronize()
    _, q_ref, omn, omx = orc.quantize_v2(x, x.min(), x.max(), orc.QINT8, orc.SCALED)
    np.testing.assert_array_equal(q_d.cpu().numpy(), q_ref)
    assert state[2].item() == omn[0] and state[3].item() == omx[0]
    x_d, q_d = buf[:37], q_d[:37]
    with pytest.raises(hip.ItexHipError):
        hip.quantize_dynamic(x_d, q_d, 0, orc.QINT8, orc.SCALED, 0.01, state)
    with pytest.raises(hip.ItexHipError):
        hip.quantize_dynamic(x_d, q_d, 37, orc.QINT8, orc.MIN_FIRST, 0.01, state)


@pytest.mark.parametrize("M", [1, 2, 4, 7, 16])
@pytest.mark.parametrize("K,N", [(64, 16), (256, 100), (4096, 512), (1024, 4096), (8192, 48), (64, 8200), (512, 16384)])
@pytest.mark.parametrize("kw", [V2_DEQ, V2_REQ_S8])
def test_gemv_kernel_vs_oracle(hip, dev, M, K, N, kw):
    layer, w, bias = make_layer(hip, dev, K, N, seed=K + N + 1)
    x, xq, mn, mx = make_acts(M, K, seed=M + 100)
    r_out = float(np.abs(x @ w + bias).max())
    ref = layer.oracle(xq, kw, mn, mx, -r_out, r_out)
    np.testing.assert_array_equal(layer.run(xq, kw, mn, mx, -r_out, r_out, path="gemv"), ref)
    np.testing.assert_array_equal(layer.run(xq, kw, mn, mx, -r_out, r_out, path="auto"), ref)
    np.testing.assert_array_equal(layer.run(xq, kw, mn, mx, -r_out, r_out, path="tile"), ref)
    np.testing.assert_array_equal(layer.run(xq, kw, mn, mx, -r_out, r_out, path="fused"), ref)


def test_signed_activations_and_extremes(hip, dev):
    rng = np.random.default_rng(5)
    K, N, M = 512, 64, 48
    wq = rng.integers(-128, 128, size=(K, N)).astype(np.int8)
    wq[:, 0] = -128
    wq[:, 1] = 127
    bias = np.zeros(N, np.float32)
    layer = Linear(hip, dev, wq, np.float32([-1.0]), np.float32([1.0]), bias)
    kw = dict(api=orc.API_V1, t_out=orc.QINT32, input_mode=orc.SCALED, n_fused_ops=1)
    for dtype in (np.int8, np.uint8):
        info = np.iinfo(dtype)
        xq = rng.integers(info.min, info.max + 1, size=(M, K)).astype(dtype)
        xq[0, :] = info.max
        xq[1, :] = info.min
        ref = layer.oracle(xq, kw, -1.0, 1.0)
        exact = xq.astype(np.int64) @ wq.astype(np.int64)
        # |acc| < 2^24 here so the fp32 round trip of the s32 output is exact
        np.testing.assert_array_equal(ref, exact)
        for path in ("tile", "naive"):
            np.testing.assert_array_equal(layer.run(xq, kw, -1.0, 1.0, path=path), exact)
        np.testing.assert_array_equal(layer.run(xq[:16], kw, -1.0, 1.0, path="gemv"), exact[:16])


def test_config1_literal(hip, dev):
    """The single quantized linear of the reference's CPU-runnable case: SCALED qint8 activations, per-channel weights, fp32 bias,
    [BiasAdd, Relu, Requantize] -> quint8, V1 and V2 spellings agree with the oracle (including the
    reference's as-written bias scaling and dropped requantize factor)."""
    M, K, N = 128, 1024, 1024
    layer, w, bias = make_layer(hip, dev, K, N, seed=0)
    x, xq, mn, mx = make_acts(M, K, seed=0, mode=orc.SCALED)
    r_out = float(np.maximum(x @ w + bias, 0).max())
    for kw in (dict(api=orc.API_V1, t_out=orc.QUINT8, input_mode=orc.SCALED, activation=orc.ACT_RELU, n_fused_ops=2),
               dict(api=orc.API_V2, t_out=orc.QUINT8, input_mode=orc.SCALED, activation=orc.ACT_RELU,
                    has_requantize=True, n_fused_ops=3)):
        ref = layer.oracle(xq, kw, mn, mx, 0.0, r_out)
        np.testing.assert_array_equal(layer.run(xq, kw, mn, mx, 0.0, r_out), ref)


@pytest.mark.parametrize("path", ["auto", "fused"])
@pytest.mark.parametrize("K,N,relu", [(768, 2304, False), (768, 768, False), (768, 3072, True), (3072, 768, False)])
def test_bert_linears_rows_sampled(hip, dev, K, N, relu, path):
    """BERT-base encoder linears at full size (M = 4096); the oracle checks 96 sampled rows exactly.  Both forms of
    the op: parameter vectors prepared by a launch of their own ("auto") and the single launch the op kernel and
    the benchmark use, which derives them inside the MatMul kernel ("fused")."""
    M = 4096
    layer, w, bias = make_layer(hip, dev, K, N, seed=K * 3 + N)
    x, xq, mn, mx = make_acts(M, K, seed=1)
    kw = V2_DEQ_RELU if relu else V2_DEQ
    got = layer.run(xq, kw, mn, mx, path=path)
    rows = np.random.default_rng(2).choice(M, 96, replace=False)
    ref = layer.oracle(xq[rows], kw, mn, mx)
    np.testing.assert_array_equal(got[rows], ref)
    full = np.maximum(x @ w + bias, 0) if relu else x @ w + bias
    assert np.abs(got - full).max() < 0.2


@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 6144), (4096, 14336), (14336, 4096)])
def test_llama_prefill_rows_sampled(hip, dev, K, N):
    """Llama-3-8B prefill linears at full size (M = 2048): int8 output bit-exact on 64 sampled rows, and the
    size-independent property sum_n acc[m, n] = a[m, :] . rowsum(w) on the s32 output of all rows.  The single-launch
    form of the op (what the op kernel and the benchmark time) must give the same bytes as the two-step form
    everywhere, not only on the sampled rows."""
    import torch
    M = 2048
    layer, w, bias = make_layer(hip, dev, K, N, seed=20 + K % 7 + N % 11)
    x, xq, mn, mx = make_acts(M, K, seed=21, outlier=1e-3)
    r_out = float(np.abs(x[:64] @ w + bias).max()) * 1.5
    got = layer.run(xq, V2_REQ_S8, mn, mx, -r_out, r_out)
    got_single = layer.run(xq, V2_REQ_S8, mn, mx, -r_out, r_out, path="fused")
    np.testing.assert_array_equal(got_single, got)
    rows = np.random.default_rng(3).choice(M, 64, replace=False)
    ref = layer.oracle(xq[rows], V2_REQ_S8, mn, mx, -r_out, r_out)
    np.testing.assert_array_equal(got[rows], ref)
    # checksum of the raw accumulators over every row (zero bias, SCALED-mode bias path keeps it zero)
    layer0 = Linear(hip, dev, layer.wq, layer.min_b, layer.max_b, np.zeros(N, np.float32))
    kw = dict(api=orc.API_V1, t_out=orc.QINT32, input_mode=orc.SCALED, n_fused_ops=1)
    acc = layer0.run(xq, kw, mn, mx).astype(np.int64)
    # the qint32 result passes through fp32 (scale 1.0), which is exact below 2^24: true for this data at every K
    # tested (|acc| stays below ~3e6), and asserted so that the identity below can never be skipped silently
    assert np.abs(acc).max() < 2 ** 24
    rowsum_w = layer.wq.astype(np.int64).sum(1)
    np.testing.assert_array_equal(acc.sum(1), xq.astype(np.int64) @ rowsum_w)


@pytest.mark.parametrize("mode", [orc.MIN_FIRST, orc.SCALED])
@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
def test_llama_decode_gemv(hip, dev, M, K, N, mode):
    """Llama-3-8B decode shapes at full size, every output checked against the oracle: MIN_FIRST quint8 and SCALED
    qint8 activations (zero bias, which also keeps the reference's as-written bias scaling of the SCALED form out of
    the result), two-step and single-launch form."""
    layer, w, bias = make_layer(hip, dev, K, N, seed=10 + M)
    layer_zero_bias = Linear(hip, dev, layer.wq, layer.min_b, layer.max_b, np.zeros(N, np.float32))
    x, xq, mn, mx = make_acts(M, K, seed=11 + M, mode=mode)
    kw = dict(V2_DEQ, input_mode=mode)
    ref = layer_zero_bias.oracle(xq, kw, mn, mx)
    np.testing.assert_array_equal(layer_zero_bias.run(xq, kw, mn, mx), ref)
    np.testing.assert_array_equal(layer_zero_bias.run(xq, kw, mn, mx, path="fused"), ref)
    assert np.abs(ref - x @ w).max() < 0.2


@pytest.mark.parametrize("M", [1, 3, 16])
@pytest.mark.parametrize("kw", [V2_DEQ, V2_REQ_S8, V2_DEQ_RELU])
@pytest.mark.parametrize("K,N", [(512, 272), (4096, 1024), (128, 8200)])  # the last one: 32-channel strips, ragged N
def test_per_token_activation_ranges(hip, dev, M, kw, K, N):
    """Rows quantized with their own range: row m of the GPU result equals the oracle's 1 x K problem
    with that row's (min, max).  The reference's MatMul ops have no per-row range; this is the decode
    configuration's per-token quantization."""
    import torch
    layer, w, bias = make_layer(hip, dev, K, N, seed=K + N + 5)
    rng = np.random.default_rng(M + K)
    x = (rng.standard_normal((M, K)) * rng.uniform(0.3, 3.0, (M, 1))).astype(np.float32)
    rows_q, mins, maxs = [], [], []
    for m in range(M):
        _, q, mn, mx = orc.quantize_v2(x[m:m + 1], x[m].min(), x[m].max(), orc.QUINT8, orc.MIN_FIRST)
        rows_q.append(q)
        mins.append(mn[0])
        maxs.append(mx[0])
    xq = np.concatenate(rows_q, 0)
    full = x @ w + bias
    r_out = float(np.abs(full).max())
    ref = np.concatenate([layer.oracle(xq[m:m + 1], kw, mins[m], maxs[m], -r_out, r_out) for m in range(M)], 0)
    p = hip.matmul_params(t_in=orc.QUINT8, min_a=0.0, max_a=0.0, min_out=-r_out, max_out=r_out, **kw)
    out = torch.empty((M, N), dtype=tdt(kw["t_out"]), device=dev)
    mins_d = torch.tensor(mins, dtype=torch.float32, device=dev)
    maxs_d = torch.tensor(maxs, dtype=torch.float32, device=dev)
    hip.qmatmul_per_row(p, torch.from_numpy(xq).to(dev), layer.packed, layer.colsum, M, K, N, mins_d, maxs_d,
                        layer.min_b_d, layer.max_b_d, layer.min_b.size, layer.bias_d, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), ref)
    with pytest.raises(hip.ItexHipError):
        hip.qmatmul_per_row(p, torch.from_numpy(xq).to(dev), layer.packed, layer.colsum, 17, K, N, mins_d, maxs_d,
                            layer.min_b_d, layer.max_b_d, layer.min_b.size, layer.bias_d, out)


@pytest.mark.parametrize("T,mode", [(orc.QUINT8, orc.MIN_FIRST), (orc.QINT8, orc.SCALED)])
@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("K,N", [(4096, 14336), (14336, 4096)])
def test_llama_decode_per_token_full_size(hip, dev, M, K, N, T, mode):
    """The decode shapes at full size with per-token activation ranges, from float activations: the per-row dynamic
    quantization (itexhip_quantize_dynamic_rows) must equal QuantizeV2 of each row against its own range, and every
    output of itexhip_qmatmul_per_row the oracle's 1 x K problem with that row's range.  MIN_FIRST quint8 and SCALED qint8
    activations."""
    import torch
    layer, w, bias = make_layer(hip, dev, K, N, seed=30 + M)
    if mode == orc.SCALED:   # as written, the reference inflates a float bias of SCALED activations: keep it zero here
        bias = np.zeros(N, np.float32)
        layer = Linear(hip, dev, layer.wq, layer.min_b, layer.max_b, bias)
    rng = np.random.default_rng(40 + M + K)
    x = (rng.standard_normal((M, K)) * rng.uniform(0.5, 2.0, (M, 1))).astype(np.float32)
    rows_q, mins, maxs = [], [], []
    for m in range(M):
        _, q, mn, mx = orc.quantize_v2(x[m:m + 1], x[m].min(), x[m].max(), T, mode)
        rows_q.append(q)
        mins.append(mn[0])
        maxs.append(mx[0])
    xq_ref = np.concatenate(rows_q, 0)
    x_d = torch.from_numpy(x).to(dev)
    xq_d = torch.empty((M, K), dtype=tdt(T), device=dev)
    rmn = torch.empty(M, dtype=torch.float32, device=dev)
    rmx = torch.empty(M, dtype=torch.float32, device=dev)
    hip.quantize_dynamic_rows(x_d, xq_d, M, K, T, mode, 0.01, rmn, rmx)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(xq_d.cpu().numpy(), xq_ref)
    np.testing.assert_array_equal(rmn.cpu().numpy(), np.array(mins, np.float32))
    np.testing.assert_array_equal(rmx.cpu().numpy(), np.array(maxs, np.float32))
    kw = dict(V2_DEQ, input_mode=mode)
    ref = np.concatenate([layer.oracle(xq_ref[m:m + 1], kw, mins[m], maxs[m]) for m in range(M)], 0)
    p = hip.matmul_params(t_in=T, min_a=0.0, max_a=0.0, **kw)
    out = torch.empty((M, N), dtype=torch.float32, device=dev)
    hip.qmatmul_per_row(p, xq_d, layer.packed, layer.colsum, M, K, N, rmn, rmx, layer.min_b_d, layer.max_b_d,
                        layer.min_b.size, layer.bias_d, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), ref)
    assert np.abs(ref - (x @ w + bias)).max() < 0.35


@pytest.mark.parametrize("T,mode", [(orc.QUINT8, orc.MIN_FIRST), (orc.QINT8, orc.SCALED)])
@pytest.mark.parametrize("n,offset_elems", [((1 << 23) + 8, 0), ((1 << 23) + 6, 0), ((1 << 24) + 1, 0)])
def test_dynamic_quantize_large_tensors(hip, dev, T, mode, n, offset_elems):
    """itexhip_quantize_dynamic above 4 M elements: the range pass takes several grid-stride rounds and all 512
    partial ranges are in use (aligned sizes, sizes with a tail of 1 .. 3 elements); bytes and ranges against
    QuantizeV2 fed with the tensor's min and max."""
    import torch
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    x[n - 2] = 9.5      # the extremes sit in the last workgroup's share and in the tail
    x[n // 3] = -7.25
    _, q_ref, omn, omx = orc.quantize_v2(x, x.min(), x.max(), T, mode)
    x_d = torch.from_numpy(x).to(dev)
    q_d = torch.empty(n, dtype=tdt(T), device=dev)
    state = torch.full((hip.DYNAMIC_STATE_FLOATS,), float("nan"), dtype=torch.float32, device=dev)
    hip.quantize_dynamic(x_d, q_d, n, T, mode, 0.01, state)
    torch.cuda.synchronize()
    st = state.cpu().numpy()
    assert st[0] == -7.25 and st[1] == 9.5 and st[2] == omn[0] and st[3] == omx[0]
    np.testing.assert_array_equal(q_d.cpu().numpy(), q_ref)


def test_hip_graph_replays_match_eager(hip, dev):
    """The op chain range pass -> QuantizeV2 -> single-launch MatMul captured once into a HIP graph and
    replayed with new input contents: every replay must equal the eager result on the same input (eager
    work and synchronisations sit between the replays)."""
    import torch
    M, K, N = 64, 512, 384
    layer, w, bias = make_layer(hip, dev, K, N, seed=3)
    kw = V2_DEQ_RELU
    x_static = torch.zeros((M, K), dtype=torch.float32, device=dev)
    xq = torch.empty((M, K), dtype=torch.uint8, device=dev)
    mm = torch.zeros(2, dtype=torch.float32, device=dev)
    out = torch.empty((M, N), dtype=torch.float32, device=dev)
    # the activation range is fixed at capture time (the host-memory min/max of the ops are call arguments)
    mn, mx = -4.0, 4.5
    _, amn, amx = orc.adjust_input_range(mn, mx)
    scale = orc.legacy_min_first_scale(orc.QUINT8, amn, amx)
    addend = float(np.float32(-amn) * scale)
    _, omn, omx, _, _ = orc.scale_zeropoint_align(orc.QUINT8, orc.MIN_FIRST, False, np.float32([amn]), np.float32([amx]))
    p = hip.matmul_params(t_in=orc.QUINT8, min_a=float(amn), max_a=float(amx), **kw)

    def chain(stream):
        hip.minmax_f32(x_static, M * K, mm, stream)
        hip.quantize(x_static, xq, M * K, hip.QUINT8, float(scale), addend, stream)
        hip.qmatmul(p, xq, layer.packed, layer.colsum, M, K, N, layer.min_b_d, layer.max_b_d, layer.min_b.size,
                    layer.bias_d, out, stream)

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        chain(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    rng = np.random.default_rng(11)
    for rep in range(4):
        x = np.clip(rng.standard_normal((M, K)) * (1.0 + 0.3 * rep), -3.9, 4.4).astype(np.float32)
        x_static.copy_(torch.from_numpy(x).to(dev))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got, got_mm = out.cpu().numpy().copy(), mm.cpu().numpy().copy()
        out.zero_()
        chain(torch.cuda.current_stream().cuda_stream)  # eager, same buffers
        torch.cuda.synchronize()
        np.testing.assert_array_equal(got, out.cpu().numpy())
        np.testing.assert_array_equal(got_mm, np.float32([x.min(), x.max()]))
        _, xq_ref, _, _ = orc.quantize_v2(x, mn, mx, orc.QUINT8, orc.MIN_FIRST)
        np.testing.assert_array_equal(got, layer.oracle(xq_ref, kw, amn, amx))


def _run_single_launch(hip, dev, layer, kw, xq, mn, mx, bias_host, addend=None, lo=0.0, hi=0.0):
    import torch
    M = xq.shape[0]
    p = hip.matmul_params(t_in=orc.QUINT8 if xq.dtype == np.uint8 else orc.QINT8, min_a=float(mn), max_a=float(mx),
                          min_out=float(lo), max_out=float(hi), **kw)
    out = torch.empty((M, layer.N), dtype=tdt(kw["t_out"]), device=dev)
    bias_d = torch.from_numpy(np.ascontiguousarray(bias_host)).to(dev)
    add_d = None if addend is None else torch.from_numpy(np.ascontiguousarray(addend)).to(dev)
    hip.qmatmul(p, torch.from_numpy(xq).to(dev), layer.packed, layer.colsum, M, layer.K, layer.N, layer.min_b_d,
                layer.max_b_d, layer.min_b.size, bias_d, out, addend=add_d)
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("M", [3, 150])
@pytest.mark.parametrize("pos,act", [(1, orc.ACT_NONE), (1, orc.ACT_RELU), (2, orc.ACT_RELU), (2, orc.ACT_LEAKYRELU)])
def test_add_fusion_vs_oracle(hip, dev, M, pos, act):
    """[BiasAdd, Add, (act), Dequantize] and [BiasAdd, act, Add, Dequantize]: the addend is added in fp32 at its
    place in the post-op chain; GEMV (M = 3) and tile (M = 150) paths, N not a multiple of 4."""
    K, N = 256, 203
    layer, w, bias = make_layer(hip, dev, K, N, seed=31)
    x, xq, mn, mx = make_acts(M, K, seed=M)
    z = (np.random.default_rng(4).standard_normal((M, N)) * 2).astype(np.float32)
    kw = dict(api=orc.API_V2, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST, has_dequantize=True, activation=act,
              add_position=pos, leakyrelu_alpha=0.3)
    st, ref = orc.qmatmul(orc.matmul_attrs(t_in=orc.QUINT8, **kw), xq, layer.wq, bias, mn, mx, layer.min_b, layer.max_b,
                          addend=z)
    assert st == orc.OK
    np.testing.assert_array_equal(_run_single_launch(hip, dev, layer, kw, xq, mn, mx, bias, z), ref)
    with pytest.raises(hip.ItexHipError):   # the addend and "Add" go together
        _run_single_launch(hip, dev, layer, kw, xq, mn, mx, bias, None)
    with pytest.raises(hip.ItexHipError):   # a quantized addend does not exist
        _run_single_launch(hip, dev, layer, dict(kw, t_out=orc.QINT8, has_requantize=True, has_dequantize=False), xq, mn, mx,
                           bias, z, -1, 1)


def _widen16(bits, T):
    """uint16 bit patterns of bfloat16 / half values -> float32 (exact)"""
    if T == orc.BFLOAT16:
        return (bits.astype(np.uint32) << 16).view(np.float32)
    return bits.view(np.float16).astype(np.float32)


@pytest.mark.parametrize("T16", [orc.BFLOAT16, orc.HALF], ids=["bf16", "f16"])
@pytest.mark.parametrize("M,N", [(3, 203), (150, 203), (150, 208), (260, 528)])
@pytest.mark.parametrize("pos,act", [(1, orc.ACT_RELU), (2, orc.ACT_LEAKYRELU)])
def test_add_fusion_with_16_bit_output(hip, dev, T16, M, N, pos, act):
    """[BiasAdd, Add / act, Dequantize] with a bfloat16 / half result: the addend has the output's type (the sum post-op
    reads the destination, quantized_matmul_common.h:341-389), is widened exactly, added in fp32, and the result is
    rounded once.  Bit patterns equal the oracle's (fed the widened addend); small-M, element-wise (N = 203) and
    vector (N = 208, 528) epilogues."""
    K = 256
    layer, w, bias = make_layer(hip, dev, K, N, seed=N)
    x, xq, mn, mx = make_acts(M, K, seed=M)
    rng = np.random.default_rng(N + M)
    zf = (rng.standard_normal((M, N)) * 2).astype(np.float32)
    zbits = ((zf.view(np.uint32) >> 16).astype(np.uint16) if T16 == orc.BFLOAT16 else zf.astype(np.float16).view(np.uint16))
    kw = dict(api=orc.API_V2, t_out=T16, input_mode=orc.MIN_FIRST, has_dequantize=True, activation=act,
              add_position=pos, leakyrelu_alpha=0.3)
    st, ref = orc.qmatmul(orc.matmul_attrs(t_in=orc.QUINT8, **kw), xq, layer.wq, bias, mn, mx, layer.min_b, layer.max_b,
                          addend=_widen16(zbits, T16))
    assert st == orc.OK and ref.dtype == np.uint16
    got = _run_single_launch(hip, dev, layer, kw, xq, mn, mx, bias, zbits.view(np.int16))
    np.testing.assert_array_equal(bits16(got), ref)


@pytest.mark.parametrize("M", [4, 130])
@pytest.mark.parametrize("act", [orc.ACT_GELU_APPROX, orc.ACT_GELU_EXACT])
def test_gelu_fusion_close_to_oracle(hip, dev, M, act):
    """GELU post-ops: the device's tanhf / erff need not round like the host's (nor like oneDNN's own
    kernels), so this is a tolerance check (2e-6 relative, 1e-6 absolute) - parity unpinned at bit level."""
    K, N = 512, 256
    layer, w, bias = make_layer(hip, dev, K, N, seed=32)
    x, xq, mn, mx = make_acts(M, K, seed=M + 9)
    kw = dict(api=orc.API_V2, t_out=orc.FLOAT, input_mode=orc.MIN_FIRST, has_dequantize=True, activation=act)
    ref = layer.oracle(xq, kw, mn, mx)
    got = _run_single_launch(hip, dev, layer, kw, xq, mn, mx, bias)
    np.testing.assert_allclose(got, ref, rtol=2e-6, atol=1e-6)
    gelu = x @ w + bias
    gelu = 0.5 * gelu * (1 + np.tanh(np.sqrt(2 / np.pi) * (gelu + 0.044715 * gelu ** 3)))
    if act == orc.ACT_GELU_APPROX:
        np.testing.assert_allclose(got, gelu, rtol=0.2, atol=0.2)   # the reference test's own bar


@pytest.mark.parametrize("act", [orc.ACT_GELU_APPROX, orc.ACT_GELU_EXACT, orc.ACT_ELU, orc.ACT_SIGMOID, orc.ACT_TANH,
                                 orc.ACT_SWISH, orc.ACT_MISH])
@pytest.mark.parametrize("path", ["tile", "gemv"])
def test_transcendental_activations_over_a_dense_range(hip, dev, act, path):
    """The device evaluates these activations with the hardware's exp2 / reciprocal and its own polynomial forms.  With
    an all-zero weight the fp32 value entering the activation is the bias itself, so the whole input range is swept, not
    only what a matrix product happens to produce: 16 K points over [-30, 30] (dense around 0), the break points of the
    device's forms and the large magnitudes where exp overflows.  Same tolerance as the other GELU tests."""
    M, K = 3, 64
    xs = np.concatenate([np.linspace(-30, 30, 8192), np.linspace(-1, 1, 4096), np.linspace(-12, -2, 4000),
                         [-0.35, -0.3500001, -0.3499999, 20.0, 20.00001, 19.99999, 0.0, -0.0, 1e-8, -1e-8, 1e-30, -1e-30,
                          88.0, -88.0, 104.0, -104.0, 1e4, -1e4, 3e38, -3e38]]).astype(np.float32)
    N = ((xs.size + 31) // 32) * 32
    bias = np.zeros(N, np.float32)
    bias[:xs.size] = xs
    wq = np.zeros((K, N), np.int8)
    one = np.ones(N, np.float32)
    layer = Linear(hip, dev, wq, -one, one, bias)
    x, xq, mn, mx = make_acts(M, K, seed=3)
    kw = dict(V2_DEQ, activation=act)
    ref = layer.oracle(xq, kw, mn, mx)
    got = layer.run(xq, kw, mn, mx, path=path)
    assert np.isfinite(ref[:, :xs.size - 2]).all()
    np.testing.assert_allclose(got, ref, rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("M", [2, 140])
@pytest.mark.parametrize("t_out,mode", [(orc.FLOAT, orc.MIN_FIRST), (orc.QINT8, orc.MIN_FIRST), (orc.QINT32, orc.MIN_FIRST),
                                        (orc.FLOAT, orc.SCALED)])
def test_qint32_bias_vs_oracle(hip, dev, M, t_out, mode):
    K, N = 320, 144
    layer, w, _ = make_layer(hip, dev, K, N, seed=33)
    x, xq, mn, mx = make_acts(M, K, seed=M + 3, mode=mode)
    b32 = np.random.default_rng(6).integers(-3000, 3000, N).astype(np.int32)
    kw = dict(api=orc.API_V2 if t_out != orc.QINT32 else orc.API_V1, t_out=t_out, input_mode=mode,
              has_dequantize=t_out == orc.FLOAT, has_requantize=t_out == orc.QINT8, t_bias=orc.QINT32)
    st, ref = orc.qmatmul(orc.matmul_attrs(t_in=orc.QUINT8 if mode == orc.MIN_FIRST else orc.QINT8, **kw), xq, layer.wq, b32,
                          mn, mx, layer.min_b, layer.max_b, -40.0, 40.0)
    assert st == orc.OK
    got = _run_single_launch(hip, dev, layer, kw, xq, mn, mx, b32, lo=-40.0, hi=40.0)
    np.testing.assert_array_equal(got, ref)
    # the two-launch form prepares the same vectors
    import torch
    p = hip.matmul_params(t_in=orc.QUINT8 if mode == orc.MIN_FIRST else orc.QINT8, min_a=float(mn), max_a=float(mx),
                          min_out=-40.0, max_out=40.0, **kw)
    ep = hip.qmatmul_epilogue_desc(p, layer.min_b.size)
    hip.qmatmul_prepare(p, layer.min_b_d, layer.max_b_d, layer.min_b.size, torch.from_numpy(b32).to(dev), layer.colsum, N,
                        layer.scales_d, layer.sbias_d)
    out = torch.empty((M, N), dtype=tdt(t_out), device=dev)
    hip.qgemm(torch.from_numpy(xq).to(dev), p.t_in, layer.packed, layer.colsum, M, K, N, layer.scales_d, layer.sbias_d, ep,
              t_out, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.cpu().numpy(), ref)


V2_DEQ_BF16 = dict(V2_DEQ, t_out=orc.BFLOAT16)
V2_DEQ_F16 = dict(V2_DEQ, t_out=orc.HALF)


@pytest.mark.parametrize("T16", [orc.BFLOAT16, orc.HALF])
@pytest.mark.parametrize("path", ["gemv", "tile", "auto", "fused", "naive"])
@pytest.mark.parametrize("M,K,N", [(3, 512, 272), (150, 256, 203), (16, 64, 8), (300, 448, 528)])
def test_bfloat16_output_vs_oracle(hip, dev, path, M, K, N, T16):
    """Tout = bfloat16 / half (_QuantizedMatMul, ...AndDequantize): bit patterns equal the oracle's on every kernel,
    with N odd / not a multiple of the 8-element vector store."""
    V2_DEQ_BF16 = dict(V2_DEQ, t_out=T16)
    if path == "gemv" and M > 128:
        pytest.skip("the small-M kernel takes M <= 128")
    layer, w, bias = make_layer(hip, dev, K, N, seed=K + N)
    x, xq, mn, mx = make_acts(M, K, seed=M + 1)
    for kw in (V2_DEQ_BF16, dict(V2_DEQ_BF16, activation=orc.ACT_RELU)):
        ref = layer.oracle(xq, kw, mn, mx)
        assert ref.dtype == np.uint16
        np.testing.assert_array_equal(bits16(layer.run(xq, kw, mn, mx, path=path)), ref)


@pytest.mark.parametrize("path", ["gemv", "tile", "naive"])
def test_bfloat16_rounding_of_special_values(hip, dev, path):
    """The bfloat16 store rounds with the GPU's conversion instruction; the oracle with the integer formula.  All-zero
    weight columns make the fp32 result of a column equal its bias exactly, so any fp32 bit pattern can be sent through the
    epilogue's conversion: ties to even in both directions, carries into the exponent, the largest finite values
    (rounding to infinity), denormals (fp32 denormals that stay bfloat16 denormals or round up to the smallest normal),
    infinities and NaNs.  Bit patterns must equal the oracle's, except that a NaN only has to be a NaN."""
    M, K, N = 40, 256, 96
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((K, N)) * 0.02).astype(np.float32)
    r = np.abs(w).max(0).astype(np.float32)
    _, wq, mn_b, mx_b = orc.quantize_v2(w, -r, r, orc.QINT8, orc.SCALED, axis=1)
    special = np.array([0x3f808000, 0x3f818000, 0x3f807fff, 0x3f808001, 0x3fffffff, 0x3fff8000, 0x7f7fffff, 0x7f7f8000,
                        0x7f7f7fff, 0xff7fffff, 0x00000001, 0x00008000, 0x00008001, 0x00018000, 0x007fffff, 0x007f8000,
                        0x807fffff, 0x00800000, 0x80000000, 0x00000000, 0x7f800000, 0xff800000, 0x7fc00000, 0xffc00000,
                        0x33333333, 0xb3333333, 0x4b7fffff, 0xcb7f8000, 0x0000ffff, 0x80010000, 0x7f000000, 0x3effffff],
                       dtype=np.uint32)
    cols = np.arange(special.size) * 3  # spread over the 32-channel tiles and their 4-channel groups
    wq[:, cols] = 0
    bias = (rng.standard_normal(N) * 0.01).astype(np.float32)
    bias[cols] = special.view(np.float32)
    layer = Linear(hip, dev, wq, mn_b, mx_b, bias)
    x, xq, mn, mx = make_acts(M, K, seed=9)
    kw = dict(V2_DEQ, t_out=orc.BFLOAT16)
    ref = layer.oracle(xq, kw, mn, mx)
    got = bits16(layer.run(xq, kw, mn, mx, path=path))
    nan = (ref & 0x7fff) > 0x7f80
    assert nan[:, cols[22]].all() and nan[:, cols[23]].all() and nan.sum() == 2 * M
    np.testing.assert_array_equal((got & 0x7fff) > 0x7f80, nan)
    np.testing.assert_array_equal(got[~nan], ref[~nan])
    # the special columns really carry the rounded bias (the fixture does what it says)
    f = special.astype(np.uint64)
    want = ((f + 0x7fff + ((f >> 16) & 1)) >> 16).astype(np.uint16)
    want[18] = 0  # a bias of -0 is added to the accumulator's +0
    finite = np.array([i for i in range(special.size) if i not in (22, 23)])
    np.testing.assert_array_equal(ref[0, cols[finite]], want[finite])


@pytest.mark.parametrize("shape", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("V2_DEQ_BF16", [V2_DEQ_BF16, V2_DEQ_F16], ids=["bf16", "f16"])
def test_bfloat16_output_every_tile_shape(hip, dev, monkeypatch, shape, V2_DEQ_BF16):
    hip.force_tile_shape(matmul=shape)
    for M, K, N in [(513, 192, 400), (260, 320, 203)]:
        layer, w, bias = make_layer(hip, dev, K, N, seed=N + shape)
        x, xq, mn, mx = make_acts(M, K, seed=M)
        ref = layer.oracle(xq, V2_DEQ_BF16, mn, mx)
        np.testing.assert_array_equal(bits16(layer.run(xq, V2_DEQ_BF16, mn, mx, path="tile")), ref)
        np.testing.assert_array_equal(bits16(layer.run(xq, V2_DEQ_BF16, mn, mx, path="fused")), ref)


@pytest.mark.parametrize("V2_DEQ_BF16", [V2_DEQ_BF16, V2_DEQ_F16], ids=["bf16", "f16"])
def test_bfloat16_output_unpacked_weight_odd_k(hip, dev, V2_DEQ_BF16):
    import torch
    M, K, N = 37, 75, 61
    layer, w, bias = make_layer(hip, dev, K, N, seed=5)
    x, xq, mn, mx = make_acts(M, K, seed=2)
    ref = layer.oracle(xq, V2_DEQ_BF16, mn, mx)
    p = hip.matmul_params(t_in=orc.QUINT8, min_a=mn, max_a=mx, **V2_DEQ_BF16)
    out = torch.empty((M, N), dtype=torch.int16, device=dev)
    hip.qmatmul_unpacked(p, torch.from_numpy(xq).to(dev), layer.w_d, False, M, K, N, layer.min_b_d, layer.max_b_d,
                         layer.min_b.size, layer.bias_d, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(bits16(out.cpu().numpy()), ref)


@pytest.mark.parametrize("M", [2, 140])
@pytest.mark.parametrize("t_out,mode", [(orc.FLOAT, orc.MIN_FIRST), (orc.BFLOAT16, orc.MIN_FIRST), (orc.HALF, orc.MIN_FIRST),
                                        (orc.QINT8, orc.MIN_FIRST),
                                        (orc.QINT32, orc.MIN_FIRST), (orc.FLOAT, orc.SCALED)])
@pytest.mark.parametrize("T16", [orc.BFLOAT16, orc.HALF])
def test_bfloat16_bias_vs_oracle(hip, dev, M, t_out, mode, T16):
    """Tbias = bfloat16 / half: the adjusted bias is rounded to that type before the epilogue adds it."""
    import torch
    K, N = 320, 144
    layer, w, _ = make_layer(hip, dev, K, N, seed=34)
    x, xq, mn, mx = make_acts(M, K, seed=M + 5, mode=mode)
    b16 = torch.from_numpy((np.random.default_rng(7).standard_normal(N) * 0.3).astype(np.float32)) \
        .to(torch.bfloat16 if T16 == orc.BFLOAT16 else torch.float16).view(torch.int16).numpy().view(np.uint16)
    isf = t_out in (orc.FLOAT, orc.BFLOAT16, orc.HALF)
    kw = dict(api=orc.API_V2 if t_out != orc.QINT32 else orc.API_V1, t_out=t_out, input_mode=mode,
              has_dequantize=isf, has_requantize=t_out == orc.QINT8, t_bias=T16)
    t_in = orc.QUINT8 if mode == orc.MIN_FIRST else orc.QINT8
    st, ref = orc.qmatmul(orc.matmul_attrs(t_in=t_in, **kw), xq, layer.wq, b16, mn, mx, layer.min_b, layer.max_b, -40.0, 40.0)
    assert st == orc.OK
    got = _run_single_launch(hip, dev, layer, kw, xq, mn, mx, b16.view(np.int16), lo=-40.0, hi=40.0)
    np.testing.assert_array_equal(bits16(got), ref)
    # the widened bias through the fp32 path differs (no rounding of the adjusted bias)
    st, ref32 = orc.qmatmul(orc.matmul_attrs(t_in=t_in, **dict(kw, t_bias=orc.FLOAT)), xq, layer.wq,
                            b16.view(np.float16).astype(np.float32) if T16 == orc.HALF else
                            (b16.astype(np.uint32) << 16).view(np.float32), mn, mx, layer.min_b, layer.max_b, -40.0, 40.0)
    assert st == orc.OK and (t_out != orc.FLOAT or not np.array_equal(ref, ref32))
    # the two-launch form prepares the same vectors
    p = hip.matmul_params(t_in=t_in, min_a=float(mn), max_a=float(mx), min_out=-40.0, max_out=40.0, **kw)
    ep = hip.qmatmul_epilogue_desc(p, layer.min_b.size)
    hip.qmatmul_prepare(p, layer.min_b_d, layer.max_b_d, layer.min_b.size, torch.from_numpy(b16.view(np.int16)).to(dev),
                        layer.colsum, N, layer.scales_d, layer.sbias_d)
    out = torch.empty((M, N), dtype=tdt(t_out), device=dev)
    hip.qgemm(torch.from_numpy(xq).to(dev), p.t_in, layer.packed, layer.colsum, M, K, N, layer.scales_d, layer.sbias_d, ep,
              t_out, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(bits16(out.cpu().numpy()), ref)


@pytest.mark.parametrize("path", ["tile", "gemv", "naive"])
def test_half_output_is_rounded_from_the_fp32_result(hip, dev, path):
    """The epilogue's fp32 result is rounded to fp32 and only then to half: elements where one rounding of the exact
    value would differ (a few per million) must follow the two-step definition."""
    M = 16 if path == "gemv" else 512
    K, N = 64, 2048 if path != "gemv" else 32768
    layer, w, bias = make_layer(hip, dev, K, N, seed=3)
    x, xq, mn, mx = make_acts(M, K, seed=8)
    ref = layer.oracle(xq, V2_DEQ_F16, mn, mx)
    ref32 = layer.oracle(xq, V2_DEQ, mn, mx)
    np.testing.assert_array_equal(ref, ref32.astype(np.float16).view(np.uint16))
    got = bits16(layer.run(xq, V2_DEQ_F16, mn, mx, path=path))
    np.testing.assert_array_equal(got, ref)
    # the sample does contain elements that tell the two roundings apart
    st, sc, sb, ep = orc.qmatmul_prepare(orc.matmul_attrs(t_in=orc.QUINT8, **V2_DEQ_F16), N, layer.wq.astype(np.int32).sum(0),
                                         mn, mx, layer.min_b, layer.max_b, 0.0, 0.0, bias)
    acc = xq.astype(np.int64) @ layer.wq.astype(np.int64)
    exact = acc.astype(np.float64) * sc.astype(np.float64) + sb.astype(np.float64)
    with np.errstate(over="ignore"):
        once = exact.astype(np.float16).view(np.uint16)
    assert (once != ref).sum() >= 3


def test_random_shapes_through_the_single_launch_op(hip, dev):
    """Seeded sweep over shapes, output types and fusions through itexhip_qmatmul (the dispatcher picks GEMV, tile shape
    and store path from the shape), every case bit-compared with the oracle."""
    rng = np.random.default_rng(2024)
    kinds = [V2_DEQ, V2_DEQ_RELU, V2_REQ_S8, V2_REQ_U8_RELU, V1_S32, V2_DEQ_BF16, V2_DEQ_F16]
    for case in range(48):
        M = int(rng.choice([1, 2, 3, 5, 8, 15, 16, 17, 31, 33, 64, 100, 129, 255, 300]))
        K = 16 * int(rng.integers(1, 96))
        N = int(rng.choice([1, 7, 16, 31, 32, 33, 100, 255, 256, 1000, 4100, 8200, 9000]))
        kw = kinds[int(rng.integers(0, len(kinds)))]
        per_channel = bool(rng.integers(0, 2))
        layer, w, bias = make_layer(hip, dev, K, N, seed=case, per_channel=per_channel)
        x, xq, mn, mx = make_acts(M, K, seed=100 + case, mode=kw["input_mode"])
        full = x @ w + bias
        r_out = float(np.abs(np.maximum(full, 0) if kw.get("activation") else full).max())
        lo = 0.0 if kw["t_out"] == orc.QUINT8 else -r_out
        ref = layer.oracle(xq, kw, mn, mx, lo, r_out)
        got = bits16(layer.run(xq, kw, mn, mx, lo, r_out, path="fused"))
        assert np.array_equal(got, ref), (case, M, K, N, kw, per_channel)
