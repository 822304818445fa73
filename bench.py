#!/usr/bin/env python3
"""Benchmark of the INT8 quantized-inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME[,NAME...]] [--no-cpu] [--tile-shape S]

Headline ("value"): the Llama-3-8B-shaped INT8 prefill linear, M=2048 K=4096 N=14336, quint8
activations x per-channel qint8 weights, fused bias + requantize to qint8 (`_QuantizedMatMul`
fused_ops=[BiasAdd, Requantize]).  One step = one launch of the op (the kernel derives the channels'
scales and biases itself), inputs resident in HBM.

Output.  The LAST line of stdout is one short JSON record (under 4 KB): the headline workload with its
`roofline` and `cpu_baseline`, plus `targets`, the worst roofline fraction of each other workload family.
The line before it, prefixed "BENCH_DETAIL ", is the same record with everything else: under "others" every
other workload (standalone quantization ops at 2^28 elements, decode GEMV, BERT linears, the remaining
prefill shapes, ...) with its own roofline fraction, and under "roofline" the power samples and notes; the
same JSON is written to gpurun_out/bench_<sections>.json.

Timing uses HIP events on the stream the kernels are launched on (PyTorch's current stream, whose
raw handle is passed through the C ABI).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0      # MI355X HBM3E, published
PEAK_INT8_TOPS = 5000.0    # MI355X dense int8 MFMA, published (tera-ops/s)


def kernel_source_sha(root):
    """sha256 over the sources of the headline kernel: ties a counter measurement to the code it was taken on."""
    import hashlib
    h = hashlib.sha256()
    for f in ("qgemm_tile.hpp", "qgemm_common.hpp", "qmatmul_params.hpp"):
        h.update(open(os.path.join(root, "intel-extension-for-tensorflow_amd", "csrc", f), "rb").read())
    return h.hexdigest()


def _setup():
    import torch
    import __graft_entry__ as entry
    hip = entry.load_package().itexhip
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU (torch.cuda.is_available() is False)")
    return torch, hip


RAMP_MS = 40.0  # sustained load before timing: the clock governor takes ~30 ms to settle under MFMA load


class Timer:
    """HIP-event timing of `fn` launched `steps` times back to back on the current stream.  Untimed
    part: `warmup` steps, then more of the same steps until RAMP_MS of wall time have passed under
    load, so that the timed steps run at the clocks of a sustained run."""

    def __init__(self, torch):
        self.torch = torch

    def run(self, fn, steps, warmup):
        torch = self.torch
        t0 = time.perf_counter()
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        i = warmup
        while (time.perf_counter() - t0) * 1e3 < RAMP_MS:
            for _ in range(32):
                fn(i)
                i += 1
            torch.cuda.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(steps):
            fn(warmup + i)
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / steps  # ms per step

    def run_graph(self, make_fn, steps, warmup):
        """The same `steps` launches captured once into a HIP graph and replayed: host launch cost
        leaves the measurement.  `make_fn(stream_handle)` returns fn(i) that launches on that stream."""
        torch = self.torch
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.graph(graph, stream=side):
            fn = make_fn(torch.cuda.current_stream().cuda_stream)
            for i in range(steps):
                fn(warmup + i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        while (time.perf_counter() - t0) * 1e3 < RAMP_MS:
            graph.replay()
            torch.cuda.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        graph.replay()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / steps


def _stream(torch):
    return torch.cuda.current_stream().cuda_stream


# ------------------------------------------------------------------------------------------------
# synthetic data
# ------------------------------------------------------------------------------------------------
def make_weights(torch, hip, K, N, seed, dev):
    """qint8 symmetric per-output-channel weights from N(0, 0.02), prepacked; returns a dict."""
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    w = torch.randn(K, N, device=dev, generator=g) * 0.02
    r = w.abs().amax(0)
    wq = torch.round(w * (127.0 / r)).clamp_(-127, 127).to(torch.int8)
    del w
    packed = torch.empty(hip.qgemm_packed_bytes(K, N), dtype=torch.int8, device=dev)
    colsum = torch.empty(N, dtype=torch.int32, device=dev)
    hip.qgemm_prepack_b(wq, False, K, N, packed, colsum, _stream(torch))
    bias = torch.randn(N, device=dev, generator=g) * 0.01
    return dict(K=K, N=N, wq=wq, packed=packed, colsum=colsum, min_b=(-r).contiguous(), max_b=r.contiguous(),
                bias=bias, scales=torch.empty(N, dtype=torch.float32, device=dev),
                sbias=torch.empty(N, dtype=torch.float32, device=dev))


def make_acts(torch, hip, M, K, seed, dev, outlier_frac=0.0, outlier_mult=1.0):
    """fp32 N(0,1) activations (+ outliers) quantized to quint8 with MIN_FIRST against their own range, all on the
    device (itexhip_quantize_dynamic); returns the op's output range as the MatMul's min_a / max_a."""
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    x = torch.randn(M, K, device=dev, generator=g)
    if outlier_frac:
        n_out = max(1, int(M * K * outlier_frac))
        idx = torch.randint(0, M * K, (n_out,), device=dev, generator=g)
        x.view(-1)[idx] *= outlier_mult
    xq = torch.empty(M, K, dtype=torch.uint8, device=dev)
    state = torch.zeros(hip.DYNAMIC_STATE_FLOATS, dtype=torch.float32, device=dev)
    hip.quantize_dynamic(x, xq, M * K, hip.QUINT8, hip.MIN_FIRST, 0.01, state, _stream(torch))
    torch.cuda.synchronize()
    amn, amx = [float(v) for v in state[2:4].cpu().numpy()]
    return x, xq, float(amn), float(amx)


# ------------------------------------------------------------------------------------------------
# workloads
# ------------------------------------------------------------------------------------------------
def bench_linear(torch, hip, timer, M, K, N, kind, steps, warmup, dev, seed, rotate=1, graph=False, per_row=False,
                 keep_out=False):
    """kind: 'requant_s8' ([BiasAdd, Requantize] -> qint8), 'deq' / 'deq_relu' / 'deq_gelu' ([.., Dequantize] -> fp32;
    GeluApproximate is what BERT's first feed-forward linear fuses), the same with '_bf16' appended -> bfloat16.
    rotate > 1 cycles through that many distinct weight copies so that the weight stream comes from
    HBM, not from the 256 MiB last-level cache."""
    layers = [make_weights(torch, hip, K, N, seed + i, dev) for i in range(rotate)]
    x, xq, min_a, max_a = make_acts(torch, hip, M, K, seed + 100, dev,
                                    outlier_frac=1e-3 if kind == "requant_s8" else 0.0, outlier_mult=20.0)
    if kind == "requant_s8":
        t_out, out_dtype = hip.QINT8, torch.int8
        r_out = float((x[:64] @ (layers[0]["wq"].float() * (layers[0]["max_b"] / 127.0))).abs().max()) * 1.5
        p = hip.matmul_params(api=hip.API_V2, t_in=hip.QUINT8, t_out=t_out, input_mode=hip.MIN_FIRST,
                              has_requantize=True, min_a=min_a, max_a=max_a, min_out=-r_out, max_out=r_out)
        out_bytes = 1
    else:
        bf16 = kind.endswith("_bf16")  # Dequantize to bfloat16: half the output bytes of the fp32 rows
        t_out, out_dtype = (hip.BFLOAT16, torch.bfloat16) if bf16 else (hip.FLOAT, torch.float32)
        act = kind[:-5] if bf16 else kind
        p = hip.matmul_params(api=hip.API_V2, t_in=hip.QUINT8, t_out=t_out, input_mode=hip.MIN_FIRST,
                              has_dequantize=True,
                              activation={"deq_relu": hip.ACT_RELU, "deq_gelu": hip.ACT_GELU_APPROX}.get(act, hip.ACT_NONE),
                              min_a=min_a, max_a=max_a, add_position=1 if act == "deq_add" else 0)
        out_bytes = 2 if bf16 else 4
    del x
    ep = hip.qmatmul_epilogue_desc(p, N)
    out = torch.empty(M, N, dtype=out_dtype, device=dev)
    st = _stream(torch)
    # [BiasAdd, Add, Dequantize]: the residual connection fused as the "Add" post-op, an fp32 tensor of the output's shape
    addend = torch.randn(M, N, dtype=out_dtype, device=dev) if kind == "deq_add" else None

    if per_row:  # per-token ranges (here: the tensor's range widened a little more for each row)
        row_min = torch.tensor([min_a * (1.0 + 0.01 * m) for m in range(M)], dtype=torch.float32, device=dev)
        row_max = torch.tensor([max_a * (1.0 + 0.01 * m) for m in range(M)], dtype=torch.float32, device=dev)

    def step(i):
        # what the op kernel runs per Compute: one launch, channel parameters derived inside the kernel
        L = layers[i % rotate]
        if per_row:
            hip.qmatmul_per_row(p, xq, L["packed"], L["colsum"], M, K, N, row_min, row_max, L["min_b"], L["max_b"], N,
                                L["bias"], out, st)
        else:
            hip.qmatmul(p, xq, L["packed"], L["colsum"], M, K, N, L["min_b"], L["max_b"], N, L["bias"], out, st, addend=addend)

    for L in layers:  # parameter vectors for the two-launch form below
        hip.qmatmul_prepare(p, L["min_b"], L["max_b"], N, L["bias"], L["colsum"], N, L["scales"], L["sbias"], st)

    def gemm_only(i):
        # the MatMul kernel alone, parameters prepared beforehand
        L = layers[i % rotate]
        if addend is not None:
            hip.qgemm_sum(xq, hip.QUINT8, L["packed"], L["colsum"], M, K, N, L["scales"], L["sbias"], ep, addend, t_out, t_out, out, st)
        else:
            hip.qgemm(xq, hip.QUINT8, L["packed"], L["colsum"], M, K, N, L["scales"], L["sbias"], ep, t_out, out, st)

    def make_graph_fn(stream):
        def fn(i):
            L = layers[i % rotate]
            hip.qmatmul(p, xq, L["packed"], L["colsum"], M, K, N, L["min_b"], L["max_b"], N, L["bias"], out, stream, addend=addend)
        return fn

    ms_step = timer.run(step, steps, warmup)
    # what the last of the timed single-launch calls left in the output buffer (it ran on layer (warmup+steps-1) % rotate)
    out_timed = out.clone() if keep_out else None
    ms_kernel = timer.run(gemm_only, steps, warmup)
    ms_graph = timer.run_graph(make_graph_fn, steps, warmup) if graph else None
    ops = 2.0 * M * N * K
    nbytes = M * K + K * N + out_bytes * M * N * (2 if addend is not None else 1) + 8 * N
    res = dict(M=M, K=K, N=N, kind=kind, ms_per_step=ms_step, us_kernel=ms_kernel * 1e3,
               tops=ops / (ms_step * 1e-3) / 1e12, tops_kernel=ops / (ms_kernel * 1e-3) / 1e12,
               gbs_kernel=nbytes / (ms_kernel * 1e-3) / 1e9, ops=ops, bytes=nbytes)
    if ms_graph is not None:
        res.update(us_kernel_graph=ms_graph * 1e3, gbs_kernel_graph=nbytes / (ms_graph * 1e-3) / 1e9,
                   tops_kernel_graph=ops / (ms_graph * 1e-3) / 1e12)
    res["_ctx"] = dict(layers=layers, xq=xq, p=p, min_a=min_a, max_a=max_a, out_timed=out_timed)
    return res


def bench_dynamic_linear(torch, hip, timer, M, K, N, steps, warmup, dev, seed):
    """A dynamically quantized linear from float activations: range of x, QuantizeV2 (MIN_FIRST quint8), MatMul
    [BiasAdd, Dequantize].  `device_range`: itexhip_quantize_dynamic + itexhip_qmatmul_device_range, nothing waits on the
    host (what _ITEXQuantizedMatMulDynamicInput enqueues).  `host_range`: the range is copied to the host between the
    reduction and the quantization, as the separate ops need for their host-memory min / max tensors."""
    import numpy as np
    L = make_weights(torch, hip, K, N, seed, dev)
    g = torch.Generator(device=dev)
    g.manual_seed(seed + 100)
    x = torch.randn(M, K, device=dev, generator=g)
    xq = torch.empty(M, K, dtype=torch.uint8, device=dev)
    out = torch.empty(M, N, dtype=torch.float32, device=dev)
    state = torch.zeros(hip.DYNAMIC_STATE_FLOATS, dtype=torch.float32, device=dev)
    st = _stream(torch)
    p = hip.matmul_params(api=hip.API_V2, t_in=hip.QUINT8, t_out=hip.FLOAT, input_mode=hip.MIN_FIRST, has_dequantize=True)

    def device_range(i):
        hip.quantize_dynamic(x, xq, M * K, hip.QUINT8, hip.MIN_FIRST, 0.01, state, st)
        hip.qmatmul_device_range(p, xq, L["packed"], L["colsum"], M, K, N, state[2:], L["min_b"], L["max_b"], N, L["bias"], out, st)

    host = np.zeros(2, np.float32)
    f32 = np.float32

    def host_range(i):
        hip.minmax_f32(x, M * K, state, st)
        hip.memcpy_d2h(host, state, 8, st)   # waits for the stream
        amn, amx = min(f32(0.0), host[0]), max(f32(0.0), host[1])
        scale = f32(255.0 / float(amx - amn))
        hip.quantize(x, xq, M * K, hip.QUINT8, float(scale), float(f32(-amn) * scale), st)
        p.min_a, p.max_a = float(amn), float(amx)
        hip.qmatmul(p, xq, L["packed"], L["colsum"], M, K, N, L["min_b"], L["max_b"], N, L["bias"], out, st)

    rmn = torch.empty(M, dtype=torch.float32, device=dev)
    rmx = torch.empty(M, dtype=torch.float32, device=dev)

    def per_token(i):   # every row against its own range (M <= 16)
        hip.quantize_dynamic_rows(x, xq, M, K, hip.QUINT8, hip.MIN_FIRST, 0.01, rmn, rmx, st)
        hip.qmatmul_per_row(p, xq, L["packed"], L["colsum"], M, K, N, rmn, rmx, L["min_b"], L["max_b"], N, L["bias"], out, st)

    ms_dev = timer.run(device_range, steps, warmup)
    ms_tok = timer.run(per_token, steps, warmup) if M <= 16 else None
    ms_host = timer.run(host_range, steps, warmup)
    return dict(name="dynamic_linear_from_float", M=M, K=K, N=N, us_device_range=ms_dev * 1e3, us_host_range=ms_host * 1e3,
                us_device_range_per_token=None if ms_tok is None else ms_tok * 1e3,
                note="range + QuantizeV2 + MatMul[BiasAdd, Dequantize] per step; device_range: no host wait; host_range: "
                     "the range crosses to the host between reduction and quantization")


def bench_elementwise(torch, hip, timer, n, steps, warmup, dev):
    import numpy as np
    g = torch.Generator(device=dev)
    g.manual_seed(30)
    x = torch.randn(n, device=dev, generator=g)
    x[::10007] *= 50.0
    st = _stream(torch)
    mm = torch.zeros(2, dtype=torch.float32, device=dev)
    hip.minmax_f32(x, n, mm, st)
    mn, mx = [float(v) for v in mm.cpu().numpy()]
    out = []

    def add(name, fn, nbytes):
        ms = timer.run(fn, steps, warmup)
        out.append(dict(name=name, n=n, us_kernel=ms * 1e3, gbs=nbytes / (ms * 1e-3) / 1e9, bytes=nbytes,
                        frac=nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS))

    q8 = torch.empty(n, dtype=torch.int8, device=dev)
    qu8 = torch.empty(n, dtype=torch.uint8, device=dev)
    # the ops' host parameter math for this range, in fp32 (range widened to hold 0; SCALED: 127 / max|.|; legacy
    # MIN_FIRST: 255 / (max - min) with the shift folded into an addend; Dequantize: the inverse scales)
    f32 = np.float32
    amn, amx = min(f32(0.0), f32(mn)), max(f32(0.0), f32(mx))
    r = max(abs(amn), abs(amx))
    add("quantize_v2_scaled_qint8", lambda i: hip.quantize(x, q8, n, hip.QINT8, float(f32(127.0) / r), 0.0, st), 5 * n)
    scale = f32(255.0 / float(amx - amn))
    addend = float(f32(-amn) * scale)
    add("quantize_v2_min_first_quint8", lambda i: hip.quantize(x, qu8, n, hip.QUINT8, float(scale), addend, st), 5 * n)
    add("minmax_f32_range_pass", lambda i: hip.minmax_f32(x, n, mm, st), 4 * n)
    y = x  # reuse the fp32 buffer as the dequantize output
    dsc = (amx - amn) / f32(255.0)
    dzp = int(np.round(f32(255.0) - amx / dsc))
    add("dequantize_min_first_quint8", lambda i: hip.dequantize(qu8, y, n, hip.QUINT8, float(dsc), dzp, st), 5 * n)
    add("dequantize_scaled_qint8", lambda i: hip.dequantize(q8, y, n, hip.QINT8, float(r / f32(127.0)), 0, st), 5 * n)
    # Requantize: int32 accumulators ~ N(0, 2^20), range pass then per-tensor requantize to qint8
    acc = (torch.randn(n, device=dev, generator=g) * float(1 << 20)).round_().to(torch.int32)
    imn = torch.zeros(1, dtype=torch.int32, device=dev)
    imx = torch.zeros(1, dtype=torch.int32, device=dev)
    add("requantization_range_int32", lambda i: hip.minmax_i32_per_channel(acc, n, 1, imn, imx, st), 4 * n)
    amax = max(abs(int(imn.cpu())), abs(int(imx.cpu())))
    # input range (-1, 1); requested range = the range the range-op reports: 1.0 * amax / 2^31
    req = np.float32(1.0) * np.float32(amax) / np.float32(2.0 ** 31)
    rscale = float(np.float32(127.0) * (np.float32(1.0) / req / np.float32(2.0 ** 31)))
    add("requantize_int32_to_qint8", lambda i: hip.requantize(acc, q8, n, hip.QINT8, rscale, st), 5 * n)
    # the same tensor as [2^20, 256] with one scale per channel (RequantizePerChannel on an NHWC tensor of 256 channels)
    depth = 256
    rsc = torch.full((depth,), rscale, dtype=torch.float32, device=dev) * (torch.rand(depth, device=dev, generator=g) * 0.5 + 0.75)
    add("requantize_per_channel_int32_to_qint8_256_channels",
        lambda i: hip.requantize_per_channel(acc, q8, n // depth, depth, hip.QINT8, rsc, st), 5 * n)
    # per-channel (per-axis) forms on a [4096, 14336] fp32 weight: the weight-quantization path; channels innermost
    # (axis 1) and outermost (axis 0 of the transposed layout)
    K, N = 4096, 14336
    nw = K * N
    if nw <= n:
        w, wq = x[:nw], q8[:nw]
        sc_n = torch.rand(N, device=dev, generator=g) * 50.0 + 10.0
        sc_k = torch.rand(K, device=dev, generator=g) * 50.0 + 10.0
        for name, fn in (("quantize_per_channel_axis1_4096x14336", lambda i: hip.quantize_axis(w, wq, K, N, 1, hip.QINT8, sc_n, None, st)),
                         ("quantize_per_channel_axis0_4096x14336", lambda i: hip.quantize_axis(w, wq, 1, K, N, hip.QINT8, sc_k, None, st)),
                         ("dequantize_per_channel_axis1_4096x14336", lambda i: hip.dequantize_axis(wq, w, K, N, 1, hip.QINT8, sc_n, None, st))):
            ms = timer.run(fn, steps, warmup)
            out.append(dict(name=name, n=nw, us_kernel=ms * 1e3, gbs=5 * nw / (ms * 1e-3) / 1e9, bytes=5 * nw,
                            frac=5 * nw / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS))
    return out


def bench_bmm(torch, hip, timer, steps, warmup, dev):
    """The two quantized BatchMatMuls of a BERT-base attention block (12 heads of 64, 128 tokens): Q.K^T with the
    1/sqrt(d) Mul and the mask Add, then P.V.  fp32 outputs, so both are bound by the output write;
    bytes = both int8 operands + the mask + the output.  Two batch sizes: 32 sequences (the token count of the
    linears above; ~30 MB per launch, where the fixed cost of a launch is about half of the time) and 128 sequences
    (the sustained rate)."""
    H, S, D = 12, 128, 64
    g = torch.Generator(device=dev)
    g.manual_seed(40)
    rnd = lambda *shape: torch.randint(-128, 128, shape, dtype=torch.int8, device=dev, generator=g)
    st = _stream(torch)
    out = []
    scale = float(6.0 * 6.0 / (127.0 * 127.0))
    for B in (32, 128):
        q, k, v, pr = rnd(B, H, S, D), rnd(B, H, S, D), rnd(B, H, S, D), rnd(B, H, S, S)
        mul = torch.tensor([0.125], dtype=torch.float32, device=dev)
        mask = torch.zeros(B, 1, 1, S, dtype=torch.float32, device=dev)
        p1, s1 = hip.bmm_params(q.shape, k.shape, False, True, hip.FLOAT, scale,
                                [(hip.BIN_MUL, mul, (1,)), (hip.BIN_ADD, mask, tuple(mask.shape))])
        o1 = torch.empty(s1, dtype=torch.float32, device=dev)
        p2, s2 = hip.bmm_params(pr.shape, v.shape, False, False, hip.FLOAT, scale)
        o2 = torch.empty(s2, dtype=torch.float32, device=dev)
        for name, p, a, b, o, nbytes, ops in (
                ("bmm_qk_t_mul_add", p1, q, k, o1, q.numel() + k.numel() + 4 * mask.numel() + 4 * o1.numel(), 2 * B * H * S * S * D),
                ("bmm_p_v", p2, pr, v, o2, pr.numel() + v.numel() + 4 * o2.numel(), 2 * B * H * S * S * D)):
            ms_eager = timer.run(lambda i: hip.qbatch_matmul(p, a, b, o, st), steps, warmup)
            # launches captured in a HIP graph: the host's launch rate leaves the measurement
            ms = timer.run_graph(lambda stream: (lambda i: hip.qbatch_matmul(p, a, b, o, stream)), steps, warmup)
            out.append(dict(name=name, batch=B * H, M=S, K=D if o is o1 else S, N=S if o is o1 else D, us_kernel=ms * 1e3,
                            us_eager=ms_eager * 1e3, bytes=nbytes, ops=ops, gbs=nbytes / (ms * 1e-3) / 1e9, bound="hbm",
                            frac=nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                            frac_mfma=ops / (ms * 1e-3) / 1e12 / PEAK_INT8_TOPS))
        del q, k, v, pr, o1, o2
    return out


def bench_conv(torch, hip, timer, steps, warmup, dev):
    """Quantized Conv2D [BiasAdd, Relu, Requantize] quint8 -> quint8 at ResNet-50 layer shapes, batch 32, as the op kernel
    runs them: the 3x3 layers as an implicit GEMM (itexhip_qconv2d) and, for comparison, as patch matrix
    (itexhip_im2col8) + GEMM; the 1x1 layer is a plain GEMM.  Algorithmic bytes = input + filter + output."""
    out = []
    g_ = torch.Generator(device=dev)
    g_.manual_seed(50)
    st = _stream(torch)
    # (the first layer of ResNet-50 has 3 input channels: the op kernel copies the input to 4 channels with the spatial
    # padding in place and gathers pixel runs from the copy; before, the patch matrix with rows padded from 147 to 160 bytes)
    for name, (B, H, W, C), (KH, KW, O), stride, patches in (
            ("conv7x7s2_224x224x3_to_64", (32, 224, 224, 3), (7, 7, 64), 2, "narrow"),
            ("conv7x7s2_224x224x3_to_64_patch_matrix", (32, 224, 224, 3), (7, 7, 64), 2, True),
            ("conv3x3_56x56x64_to_64", (32, 56, 56, 64), (3, 3, 64), 1, False),
            ("conv3x3_56x56x64_to_64_patch_matrix", (32, 56, 56, 64), (3, 3, 64), 1, True),
            ("conv3x3_28x28x128_to_128", (32, 28, 28, 128), (3, 3, 128), 1, False),
            ("conv3x3_14x14x256_to_256", (32, 14, 14, 256), (3, 3, 256), 1, False),
            ("conv1x1_56x56x256_to_64", (32, 56, 56, 256), (1, 1, 64), 1, False)):
        x = torch.randint(0, 256, (B, H, W, C), dtype=torch.uint8, device=dev, generator=g_)
        w = torch.randint(-127, 128, (KH * KW * C, O), dtype=torch.int8, device=dev, generator=g_)
        K = KH * KW * C
        Kp = (K + 15) // 16 * 16
        OH, OW = -(-H // stride), -(-W // stride)
        M = B * OH * OW
        packed = torch.empty(hip.qgemm_packed_bytes(Kp, O), dtype=torch.int8, device=dev)
        colsum = torch.empty(O, dtype=torch.int32, device=dev)
        hip.qgemm_prepack_b(w, False, K, O, packed, colsum, st)
        scales = torch.full((O,), 1e-4, dtype=torch.float32, device=dev)
        bias = torch.zeros(O, dtype=torch.float32, device=dev)
        ep = hip.Epilogue()
        ep.n_scales, ep.n_eltwise = O, 1
        ep.elt[0].alg, ep.elt[0].alpha, ep.elt[0].beta = hip.ELT_RELU, 0.0, 0.0
        y = torch.empty((M, O), dtype=torch.uint8, device=dev)
        pad = max((OH - 1) * stride + KH - H, 0) // 2       # SAME: the smaller half leads
        geo = hip.ConvGeometry(B, H, W, C, KH, KW, OH, OW, stride, stride, 1, 1, pad, pad)
        cols = torch.empty((M, Kp), dtype=torch.uint8, device=dev) if patches is True else None
        implicit = KH * KW > 1 and not patches
        assert not implicit or hip.qconv2d_implicit_ok(geo, x, O, hip.QUINT8, y)
        if patches == "narrow":   # 4 channels, window rows of 8 pixels = 32 bytes, padding written into the copy
            Cn, KWn = 4, 8
            Hn, Wn = max(pad + H, (OH - 1) * stride + KH), (max(pad + W, (OW - 1) * stride + KWn) + 3) // 4 * 4
            xn = torch.empty((B, Hn, Wn, Cn), dtype=torch.uint8, device=dev)
            wn = torch.empty((KH, KWn, Cn, O), dtype=torch.int8, device=dev)
            hip.pad_nhwc8(w, KH, KW, C, O, 0, 0, KWn, Cn, O, wn, st)
            Kn = KH * KWn * Cn
            packed_n = torch.empty(hip.qgemm_packed_bytes(Kn, O), dtype=torch.int8, device=dev)
            hip.qgemm_prepack_b(wn, False, Kn, O, packed_n, colsum, st)
            geo_n = hip.ConvGeometry(B, Hn, Wn, Cn, KH, KWn, OH, OW, stride, stride, 1, 1, 0, 0)
            assert hip.qconv2d_implicit_ok(geo_n, xn, O, hip.QUINT8, y)

        def make(stream):
            def fn(i):
                if patches == "narrow":
                    hip.pad_nhwc8(x, B, H, W, C, pad, pad, Hn, Wn, Cn, xn, stream)
                    hip.qconv2d(xn, hip.QUINT8, geo_n, packed_n, colsum, O, scales, bias, ep, hip.QUINT8, y, stream)
                    return
                if implicit:
                    hip.qconv2d(x, hip.QUINT8, geo, packed, colsum, O, scales, bias, ep, hip.QUINT8, y, stream)
                    return
                a = x
                if cols is not None:
                    hip.im2col8(x, geo, Kp, cols, stream)
                    a = cols
                hip.qgemm(a, hip.QUINT8, packed, colsum, M, Kp, O, scales, bias, ep, hip.QUINT8, y, stream)
            return fn
        ms = timer.run_graph(make, steps, warmup)
        nbytes = x.numel() + w.numel() + y.numel()
        ops = 2 * M * K * O
        t_roof = max(ops / (PEAK_INT8_TOPS * 1e12), nbytes / (PEAK_HBM_GBS * 1e9))
        out.append(dict(name=name, M=M, K=K, N=O, us_kernel=ms * 1e3, bytes=nbytes, ops=ops, bound="max(mfma,hbm)",
                        frac=t_roof / (ms * 1e-3), tops=ops / (ms * 1e-3) / 1e12, gbs=nbytes / (ms * 1e-3) / 1e9,
                        note="channel- and window-padded copy + implicit GEMM, two launches" if patches == "narrow" else
                        "implicit GEMM, one launch" if implicit else "im2col + GEMM launches" if patches else "GEMM launch only"))
        del x, w, packed, y, cols
    # the last 1x1 convolution of a ResNet-50 bottleneck block (56x56x64 -> 256) with the block's residual fused as the Sum
    # post-op: [BiasAdd, Sum, Relu, Requantize], quint8 addend of the output's shape; a plain GEMM with one more operand
    M, K, O = 32 * 56 * 56, 64, 256
    x = torch.randint(0, 256, (M, K), dtype=torch.uint8, device=dev, generator=g_)
    w = torch.randint(-127, 128, (K, O), dtype=torch.int8, device=dev, generator=g_)
    z = torch.randint(0, 256, (M, O), dtype=torch.uint8, device=dev, generator=g_)
    packed = torch.empty(hip.qgemm_packed_bytes(K, O), dtype=torch.int8, device=dev)
    colsum = torch.empty(O, dtype=torch.int32, device=dev)
    hip.qgemm_prepack_b(w, False, K, O, packed, colsum, st)
    scales = torch.full((O,), 1e-4, dtype=torch.float32, device=dev)
    bias = torch.zeros(O, dtype=torch.float32, device=dev)
    y = torch.empty((M, O), dtype=torch.uint8, device=dev)
    for with_sum in (False, True):
        ep = hip.Epilogue()
        ep.n_scales, ep.n_eltwise = O, 2 if with_sum else 1
        k = 0
        if with_sum:
            ep.elt[0].alg, ep.elt[0].alpha, ep.elt[0].beta = hip.ELT_SUM, 0.5, 0.0
            k = 1
        ep.elt[k].alg, ep.elt[k].alpha, ep.elt[k].beta = hip.ELT_RELU, 0.0, 0.0

        def make_sum(stream):
            if with_sum:
                return lambda i: hip.qgemm_sum(x, hip.QUINT8, packed, colsum, M, K, O, scales, bias, ep, z, hip.QUINT8, hip.QUINT8, y, stream)
            return lambda i: hip.qgemm(x, hip.QUINT8, packed, colsum, M, K, O, scales, bias, ep, hip.QUINT8, y, stream)
        ms = timer.run_graph(make_sum, steps, warmup)
        nbytes = x.numel() + w.numel() + y.numel() * (2 if with_sum else 1)
        ops = 2 * M * K * O
        out.append(dict(name="conv1x1_56x56x64_to_256" + ("_sum_relu" if with_sum else "_relu"), M=M, K=K, N=O, us_kernel=ms * 1e3,
                        bytes=nbytes, ops=ops, bound="hbm", frac=nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                        tops=ops / (ms * 1e-3) / 1e12, gbs=nbytes / (ms * 1e-3) / 1e9, note="GEMM launch only"))
    del x, w, z, packed, y
    # depthwise 3x3 (MobileNet shapes): no matrix product, bound by input + output bytes
    for name, (B, H, W, C) in (("dwconv3x3_112x112x32", (32, 112, 112, 32)), ("dwconv3x3_56x56x128", (32, 56, 56, 128))):
        x = torch.randint(0, 256, (B, H, W, C), dtype=torch.uint8, device=dev, generator=g_)
        w = torch.randint(-127, 128, (3, 3, C, 1), dtype=torch.int8, device=dev, generator=g_)
        scales = torch.full((C,), 2e-3, dtype=torch.float32, device=dev)
        bias = torch.zeros(C, dtype=torch.float32, device=dev)
        ep = hip.Epilogue()
        ep.n_scales, ep.n_eltwise = C, 1
        ep.elt[0].alg, ep.elt[0].alpha, ep.elt[0].beta = hip.ELT_RELU, 0.0, 0.0
        y = torch.empty((B * H * W, C), dtype=torch.uint8, device=dev)
        geo = hip.ConvGeometry(B, H, W, C, 3, 3, H, W, 1, 1, 1, 1, 1, 1)

        def make_dw(stream):
            return lambda i: hip.qdepthwise_conv2d(x, hip.QUINT8, geo, 1, w, scales, bias, ep, hip.QUINT8, y, stream)
        ms = timer.run_graph(make_dw, steps, warmup)
        nbytes = x.numel() + w.numel() + y.numel()
        out.append(dict(name=name, M=B * H * W, K=9, N=C, us_kernel=ms * 1e3, bytes=nbytes, ops=2 * 9 * y.numel(), bound="hbm",
                        frac=nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, tops=2 * 9 * y.numel() / (ms * 1e-3) / 1e12,
                        gbs=nbytes / (ms * 1e-3) / 1e9, note="depthwise kernel, one launch"))
        del x, w, y
    return out



def bench_config1_chain(torch, hip, timer, steps, warmup, dev):
    """BASELINE config 1 as a chain of three ops on one stream, 128 x 1024 x 1024: QuantizeV2 (given range) ->
    quantized MatMul [BiasAdd, Relu, Requantize] -> quint8 -> Dequantize (SCALED).  Latency-bound: reported in us per
    chain, launched eagerly and replayed from a HIP graph.  `literal`: SCALED qint8 activations as the configuration
    states it, V1 (_QuantizedFusedMatMulAndRequantize, fused_ops [BiasAdd, Relu]) and V2 (_QuantizedMatMul, fused_ops
    [BiasAdd, Relu, Requantize]) spellings, with the reference's as-written bias scaling and dropped requantize factor;
    `min_first`: the same chain with MIN_FIRST quint8 activations (the V2 spelling), where those two quirks do not
    apply."""
    import numpy as np
    M, K, N = 128, 1024, 1024
    L = make_weights(torch, hip, K, N, 0, dev)
    g = torch.Generator(device=dev)
    g.manual_seed(0)
    x = torch.randn(M, K, device=dev, generator=g)
    mn, mx = float(x.min()), float(x.max())
    r_out = float(torch.relu(x @ (L["wq"].float() * (L["max_b"] / 127.0)) + L["bias"]).max())
    f32 = np.float32
    y = torch.empty(M, N, dtype=torch.float32, device=dev)
    out = []
    for name, t_in, mode, api in (("literal_v1", hip.QINT8, hip.SCALED, hip.API_V1), ("literal_v2", hip.QINT8, hip.SCALED, hip.API_V2),
                                  ("min_first_v2", hip.QUINT8, hip.MIN_FIRST, hip.API_V2)):
        amn, amx = min(f32(0.0), f32(mn)), max(f32(0.0), f32(mx))
        if mode == hip.SCALED:
            r = max(abs(amn), abs(amx))
            q_scale, q_add, min_a, max_a = float(f32(127.0) / r), 0.0, float(-r), float(r)
        else:
            sc = f32(255.0 / float(amx - amn))
            q_scale, q_add, min_a, max_a = float(sc), float(f32(-amn) * sc), float(amn), float(amx)
        xq = torch.empty(M, K, dtype=torch.int8 if t_in == hip.QINT8 else torch.uint8, device=dev)
        q8 = torch.empty(M, N, dtype=torch.uint8, device=dev)
        kw = dict(api=api, t_in=t_in, t_out=hip.QUINT8, input_mode=mode, activation=hip.ACT_RELU, min_a=min_a, max_a=max_a,
                  min_out=0.0, max_out=r_out)
        if api == hip.API_V1:
            kw["n_fused_ops"] = 2
        else:
            kw["has_requantize"] = True
        p = hip.matmul_params(**kw)
        dq_scale = float(f32(r_out) / f32(255.0))   # Dequantize SCALED of a quint8 tensor with range (0, r_out)

        def make(stream):
            def chain(i):
                hip.quantize(x, xq, M * K, t_in, q_scale, q_add, stream)
                hip.qmatmul(p, xq, L["packed"], L["colsum"], M, K, N, L["min_b"], L["max_b"], N, L["bias"], q8, stream)
                hip.dequantize(q8, y, M * N, hip.QUINT8, dq_scale, 0, stream)
            return chain
        ms_eager = timer.run(make(_stream(torch)), steps, warmup)
        ms_graph = timer.run_graph(make, steps, warmup)
        out.append(dict(name="config1_chain_" + name, M=M, K=K, N=N, us_per_chain=ms_graph * 1e3, us_per_chain_eager=ms_eager * 1e3,
                        launches=3, ops=2.0 * M * K * N, bound="latency",
                        note="QuantizeV2 -> MatMul [BiasAdd, Relu, Requantize] -> Dequantize, three launches; graph replay / eager"))
    return out


def bench_read_floor(torch, hip, timer, nbytes, steps, warmup, dev, copies=8):
    """What one launch that only reads `nbytes` from HBM costs on this box (`copies` distinct buffers cycled): the floor
    under the decode MatMul, which has to stream as many weight bytes per launch."""
    bufs = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=dev) for _ in range(copies)]
    sink = torch.zeros(256, dtype=torch.int32, device=dev)
    st = _stream(torch)
    ms = timer.run(lambda i: hip.read_probe(bufs[i % copies], nbytes, sink, st), steps, warmup)
    ms_g = timer.run_graph(lambda stream: (lambda i: hip.read_probe(bufs[i % copies], nbytes, sink, stream)), steps, warmup)
    best = min(ms, ms_g)
    return dict(name="hbm_read_floor", bytes=nbytes, us_kernel=best * 1e3, us_eager=ms * 1e3, us_graph=ms_g * 1e3,
                gbs=nbytes / (best * 1e-3) / 1e9, frac=nbytes / (best * 1e-3) / 1e9 / PEAK_HBM_GBS, bound="hbm",
                note="itexhip_read_probe: one launch that only reads the decode weight's byte count (8 buffers cycled)")


class PowerSampler:
    """Socket power and shader clock from the amdgpu sysfs files, sampled while `fn` is launched back to back for
    `seconds`: the evidence for (or against) a power-limited kernel.  Returns None where the files are not readable."""

    def __init__(self):
        import glob
        self.power = (glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input") +
                      glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average") + [None])[0]
        self.cap = (glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap") + [None])[0]
        self.sclk = (glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk") + [None])[0]

    @staticmethod
    def _read(path):
        try:
            return open(path).read()
        except Exception:
            return None

    def _sample(self):
        pw = self._read(self.power) if self.power else None
        ck = self._read(self.sclk) if self.sclk else None
        mhz = None
        if ck:
            cur = [l for l in ck.splitlines() if "*" in l]
            if cur:
                digits = "".join(c for c in cur[0].split(":")[1] if c.isdigit())
                mhz = float(digits) if digits else None
        return (float(pw) / 1e6 if pw else None), mhz

    def run(self, torch, fn, seconds=1.5):
        import threading
        if not self.power:
            return None
        stop = [False]
        count = [0]

        def worker():
            torch.cuda.set_device(0)
            while not stop[0]:
                for _ in range(100):
                    fn()
                torch.cuda.synchronize()
                count[0] += 100
        th = threading.Thread(target=worker)
        t0 = time.perf_counter()
        th.start()
        watts, mhz = [], []
        while time.perf_counter() - t0 < seconds:
            time.sleep(0.05)
            if time.perf_counter() - t0 < 0.4:   # let the governor settle
                continue
            w, c = self._sample()
            if w is not None:
                watts.append(w)
            if c is not None:
                mhz.append(c)
        stop[0] = True
        th.join()
        dt = time.perf_counter() - t0
        cap = self._read(self.cap)
        return dict(power_w=sum(watts) / len(watts) if watts else None, sclk_mhz=sum(mhz) / len(mhz) if mhz else None,
                    power_cap_w=float(cap) / 1e6 if cap else None, us_per_launch_sustained=dt / max(count[0], 1) * 1e6,
                    samples=len(watts))


def bench_mfma_ceiling(torch, hip, timer, xq, wq, dev):
    """Matrix-pipe-only rate for operand bits like the workload's (bytes of the quantized activations,
    sign-flipped as the kernel feeds them, and of the weights) and for constant operands."""
    sink = torch.zeros(256, dtype=torch.int32, device=dev)
    st = _stream(torch)
    iters, wgs = 2000, 256
    ops = wgs * 4 * iters * 8 * 2.0 * 32 * 32 * 32
    out = {}
    a_bytes = (xq.reshape(-1)[:4096] ^ 0x80).contiguous()
    w_bytes = wq.reshape(-1)[:4096].contiguous().view(torch.uint8)
    # weights in the first operand slot, activations in the second, as the MatMul kernels feed them
    for name, buf in (("workload_data", torch.cat([w_bytes, a_bytes])),
                      ("constant_operands", torch.ones(8192, dtype=torch.uint8, device=dev))):
        ms = timer.run(lambda i: hip.mfma_probe(wgs, iters, buf, sink, st), 10, 2)
        out[name] = ops / (ms * 1e-3) / 1e12
    return out


def cpu_baseline_gemm(ctx, M_sample, K, N):
    """The oracle (a scalar-C restatement of the reference's CPU path, OpenMP over rows) on the first
    M_sample rows of the headline workload."""
    import numpy as np
    from oracle import pyoracle as orc
    L = ctx["layers"][0]
    xq = ctx["xq"][:M_sample].cpu().numpy()
    wq = L["wq"].cpu().numpy()
    bias = L["bias"].cpu().numpy()
    min_b, max_b = L["min_b"].cpu().numpy(), L["max_b"].cpu().numpy()
    p = ctx["p"]
    at = orc.matmul_attrs(api=orc.API_V2, t_in=orc.QUINT8, t_out=orc.QINT8, input_mode=orc.MIN_FIRST,
                          has_requantize=True)
    t0 = time.perf_counter()
    st, y = orc.qmatmul(at, xq, wq, bias, p.min_a, p.max_a, min_b, max_b, p.min_out, p.max_out)
    dt = time.perf_counter() - t0
    assert st == orc.OK
    return 2.0 * M_sample * K * N / dt / 1e12, dt, y


def cpu_onednn_in_torch(torch, xq_host, wq_host, w_scale, bias):
    """The closest executable stand-in for the reference's CPU path on this host: the oneDNN int8 inner product
    bundled with PyTorch (another oneDNN build than the reference pins; not ITEX).  u8 x s8 per channel, fp32 bias,
    fp32 output.  Returns (TOP/s, threads) or None when that operator is not callable."""
    try:
        M, K = xq_host.shape
        N = wq_host.shape[1]
        x = torch.from_numpy(xq_host)
        packed = torch.ops.onednn.qlinear_prepack(torch.from_numpy(wq_host.T.copy()), [M, K])
        args = (x, 1.0, 0, packed, torch.from_numpy(w_scale), torch.zeros(N, dtype=torch.int64), torch.from_numpy(bias),
                1.0, 0, torch.float32, "none", [], "")
        torch.ops.onednn.qlinear_pointwise(*args)
        best = 1e30
        for _ in range(3):
            t0 = time.perf_counter()
            torch.ops.onednn.qlinear_pointwise(*args)
            best = min(best, time.perf_counter() - t0)
        return 2.0 * M * K * N / best / 1e12, torch.get_num_threads()
    except Exception:
        return None


MAX_LINE_BYTES = 4096  # the final stdout line must stay a short record; everything else goes on an earlier line


def _best(rows, name, pred=lambda r: True, key="frac", fn=min):
    vals = [r[key] for r in rows if r.get("name") == name and pred(r) and r.get(key) is not None]
    return round(fn(vals), 4) if vals else None


def summary_line(head, steps, warmup, traffic, cpu, others):
    """The one-line record: the headline workload with its roofline and CPU baseline, plus the roofline fractions of
    the other workloads the metric names (worst row of each family)."""
    targets = {
        "prefill_gemm_other_shapes_frac_mfma_min": _best(others, "prefill_gemm"),
        "bert_linear_fp32_frac_min": _best(others, "bert_linear", lambda r: r.get("kind") in ("deq", "deq_relu")),
        "decode_gemv_m1_m4_frac_hbm_min": _best(others, "decode_gemv", lambda r: r.get("M", 99) <= 4),
        "decode_gemv_m16_frac_hbm_min": _best(others, "decode_gemv", lambda r: r.get("M") == 16),
        "quantize_v2_frac_hbm_min": _best([dict(r, name="q") for r in others
                                           if str(r.get("name", "")).startswith("quantize_v2_")], "q"),
        "dequantize_frac_hbm_min": _best([dict(r, name="d") for r in others
                                          if str(r.get("name", "")).startswith("dequantize_") and "per_channel" not in r["name"]], "d"),
        "requantize_frac_hbm": _best(others, "requantize_int32_to_qint8"),
    }
    line = {
        "metric": "int8 GEMM TOPS (% MFMA peak); quantize/GEMV GB/s (% HBM peak), 1 MI355X",
        "value": head["tops"], "unit": "TOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "s8", "data": "synthetic",
        "config": {"workload": "Llama-3-8B prefill linear M=2048 K=4096 N=14336, quint8 act x qint8 per-channel weights, "
                               "_QuantizedMatMul [BiasAdd, Requantize] -> qint8, one launch per step"},
        "roofline": {"bound": "mfma", "achieved": head["tops_kernel"], "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": head["tops_kernel"] / PEAK_INT8_TOPS, "traffic": traffic,
                     "kernel": "qgemm_tile_kernel", "us_per_launch": head["us_kernel"]},
        "cpu_baseline": cpu,
        "targets": {k: v for k, v in targets.items() if v is not None},
    }
    text = json.dumps(line)
    if len(text) >= MAX_LINE_BYTES:   # never let an optional part push the record over the limit
        line.pop("targets")
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--only", type=str, default="", help="comma list of: headline, c1, prefill, bert, bmm, conv, gemv, elementwise, copy, power")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--tile-shape", type=int, default=-1,
                    help="force the tile shape of the MatMul tile kernel (0..4) for this run; results do not depend on it")
    ap.add_argument("--cpu-rows", type=int, default=2048, help="rows of the headline workload the CPU oracle runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU only: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    only = set(s for s in args.only.split(",") if s) or {"headline", "c1", "prefill", "bert", "bmm", "conv", "gemv", "elementwise", "power"}

    torch, hip = _setup()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.tile_shape >= 0:
        hip.force_tile_shape(matmul=args.tile_shape)
    timer = Timer(torch)
    K_steps, W = args.steps, args.warmup
    # launches of 4 - 25 us (every workload below except the prefill shapes and the 2^28-element ops): the start of a
    # timed region costs a fixed 10 - 20 us, which 20 such launches do not amortise, so these rows time at least 100
    S_steps = max(K_steps, 100)
    others = []

    M, K, N = 2048, 4096, 14336
    head = bench_linear(torch, hip, timer, M, K, N, "requant_s8", K_steps, W, dev, seed=22, keep_out=True)
    ctx = head.pop("_ctx")

    ceiling = bench_mfma_ceiling(torch, hip, timer, ctx["xq"], ctx["layers"][0]["wq"], dev)

    power = None
    if "power" in only:
        # socket power and shader clock under the headline kernel, under the matrix-pipe probe on the workload's
        # operand bytes and on constant operands, and at idle: a kernel whose clock drops while the power sits at the
        # board's limit is limited by energy per operation, not by issue slots
        sampler = PowerSampler()
        L0, p0, xq0 = ctx["layers"][0], ctx["p"], ctx["xq"]
        out0 = torch.empty(M, N, dtype=torch.int8, device=dev)
        st0 = _stream(torch)
        sink = torch.zeros(256, dtype=torch.int32, device=dev)
        wl = torch.cat([L0["wq"].reshape(-1)[:4096].contiguous().view(torch.uint8), (xq0.reshape(-1)[:4096] ^ 0x80).contiguous()])
        ones = torch.ones(8192, dtype=torch.uint8, device=dev)
        time.sleep(0.5)
        idle = sampler._sample()
        power = dict(
            idle_w=idle[0],
            headline_gemm=sampler.run(torch, lambda: hip.qmatmul(p0, xq0, L0["packed"], L0["colsum"], M, K, N, L0["min_b"], L0["max_b"], N,
                                                                 L0["bias"], out0, st0)),
            mfma_probe_workload_data=sampler.run(torch, lambda: hip.mfma_probe(256, 200, wl, sink, st0)),
            mfma_probe_constant_operands=sampler.run(torch, lambda: hip.mfma_probe(256, 200, ones, sink, st0)),
            note="amdgpu sysfs (power1_input, pp_dpm_sclk) sampled every 50 ms over 1.5 s of back-to-back launches")
        # the headline kernel itself on constant operands (every activation byte 0x81, every weight 1): the same
        # instructions and memory traffic with almost no bit toggling in the matrix pipe and on the data paths, i.e. what
        # the kernel's schedule delivers when the clock is not held down by the energy of the data
        try:
            w1 = torch.ones(K, N, dtype=torch.int8, device=dev)
            packed1, colsum1 = torch.empty_like(L0["packed"]), torch.empty_like(L0["colsum"])
            hip.qgemm_prepack_b(w1, False, K, N, packed1, colsum1, st0)
            x1 = torch.full_like(xq0, 0x81)
            power["headline_gemm_constant_operands"] = sampler.run(
                torch, lambda: hip.qmatmul(p0, x1, packed1, colsum1, M, K, N, L0["min_b"], L0["max_b"], N, L0["bias"], out0, st0))
            del w1, packed1, colsum1, x1
        except Exception as exc:
            power["headline_gemm_constant_operands"] = dict(error=str(exc)[:200])
        # the vendor library on the same int8 problem (hipBLASLt behind torch._int_mm, int32 output, no epilogue), as a
        # point of comparison for rate and power: a measurement only, nothing of the product calls it
        try:
            a8 = (xq0 ^ 0x80).view(torch.int8).contiguous()
            b8 = L0["wq"].contiguous()
            torch._int_mm(a8, b8)
            power["vendor_int8_gemm_torch_int_mm"] = sampler.run(torch, lambda: torch._int_mm(a8, b8))
        except Exception as exc:  # not available in this PyTorch build
            power["vendor_int8_gemm_torch_int_mm"] = dict(error=str(exc)[:200])

    cpu, cpu_detail = None, None
    if not args.no_cpu:
        rows = min(args.cpu_rows, M)
        tops_cpu, dt, y_cpu = cpu_baseline_gemm(ctx, rows, K, N)
        # the same rows as the timed launches of itexhip_qmatmul left them in the output buffer must be identical
        same = bool((ctx["out_timed"][:rows].cpu().numpy() == y_cpu).all())
        cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        cpu = dict(value=tops_cpu, unit="TOP/s", cores=cores, kind="port",
                   sample="first %d of %d rows of the headline workload (same weights), %.1f s; output of the timed GPU "
                          "launches identical: %s" % (rows, M, dt, same))
        L = ctx["layers"][0]
        alt = cpu_onednn_in_torch(torch, ctx["xq"][:rows].cpu().numpy(), L["wq"].cpu().numpy(),
                                  (L["max_b"].cpu().numpy() / 127.0).astype("float32"), L["bias"].cpu().numpy())
        if alt:
            cpu_detail = dict(onednn_in_torch=dict(value=alt[0], unit="TOP/s", threads=alt[1],
                                          note="torch.ops.onednn.qlinear_pointwise (oneDNN bundled with PyTorch, fp32 output) "
                                               "on the same rows and weights: the nearest executable relative of the "
                                               "reference's CPU path, not ITEX itself"))
    del ctx

    if "c1" in only:
        others.extend(bench_config1_chain(torch, hip, timer, S_steps, W, dev))
    if "prefill" in only:
        others.append(bench_dynamic_linear(torch, hip, timer, 2048, 4096, 14336, max(10, K_steps // 2), max(3, W // 2), dev, seed=22))
        for (k, n, seed) in ((4096, 4096, 20), (4096, 6144, 21), (14336, 4096, 23)):
            r = bench_linear(torch, hip, timer, 2048, k, n, "requant_s8", K_steps, W, dev, seed)
            r.pop("_ctx")
            r.update(name="prefill_gemm", bound="mfma", frac=r["tops_kernel"] / PEAK_INT8_TOPS)
            others.append(r)
    if "bert" in only:
        for (k, n, kind, seed) in ((768, 2304, "deq", 1), (768, 768, "deq", 2), (768, 3072, "deq_relu", 3),
                                   (768, 3072, "deq_gelu", 3), (3072, 768, "deq", 4),
                                   (768, 2304, "deq_bf16", 1), (768, 3072, "deq_gelu_bf16", 3), (3072, 768, "deq_add", 4)):
            r = bench_linear(torch, hip, timer, 4096, k, n, kind, S_steps, W, dev, seed, graph=True)
            r.pop("_ctx")
            t_roof = max(r["ops"] / (PEAK_INT8_TOPS * 1e12), r["bytes"] / (PEAK_HBM_GBS * 1e9))
            # launches of ~15 us: the better of back-to-back launches from the host and replays of the same launches
            # from a HIP graph (a host hiccup in a region of 100 launches shows in the first, never in the second)
            best = min(r["us_kernel"], r["us_kernel_graph"])
            r.update(name="bert_linear", bound="max(mfma,hbm)", us_best=best, frac=t_roof / (best * 1e-6),
                     frac_mfma=r["ops"] / (best * 1e-6) / 1e12 / PEAK_INT8_TOPS, frac_hbm=r["bytes"] / (best * 1e-6) / 1e9 / PEAK_HBM_GBS)
            others.append(r)
    if "bmm" in only:
        others.extend(bench_bmm(torch, hip, timer, S_steps, W, dev))
    if "conv" in only:
        others.extend(bench_conv(torch, hip, timer, S_steps, W, dev))
    if "gemv" in only:
        floor = bench_read_floor(torch, hip, timer, 4096 * 14336, S_steps, W, dev)
        others.append(floor)
        for (k, n) in ((4096, 14336), (14336, 4096)):
            for m in (1, 4, 16):
                r = bench_linear(torch, hip, timer, m, k, n, "deq", S_steps, W, dev, seed=10, rotate=8, graph=True)
                r.pop("_ctx")
                best = min(r["us_kernel"], r["us_kernel_graph"])   # as for the read floor: eager or graph replay
                r.update(name="decode_gemv", bound="hbm", us_best=best, frac=r["bytes"] / (best * 1e-6) / 1e9 / PEAK_HBM_GBS,
                         frac_eager=r["gbs_kernel"] / PEAK_HBM_GBS, frac_graph=r["gbs_kernel_graph"] / PEAK_HBM_GBS,
                         read_floor_us=floor["us_kernel"], frac_of_read_floor=floor["us_kernel"] / best,
                         note="8 weight copies cycled (470 MB > last-level cache)")
                others.append(r)
            # a batched decode step of 32 rows: the small-M kernel in two blocks of 16 rows (the workgroups of a strip share
            # its weights through one L2); the tile kernel would run 64 x 64 tiles over a fraction of the CUs here
            r = bench_linear(torch, hip, timer, 32, k, n, "deq", S_steps, W, dev, seed=10, rotate=8, graph=True)
            r.pop("_ctx")
            r.update(name="decode_gemv_32_rows", bound="hbm", frac=r["gbs_kernel"] / PEAK_HBM_GBS,
                     note="8 weight copies cycled; rows in blocks of 16")
            others.append(r)
            others.append(bench_dynamic_linear(torch, hip, timer, 16, k, n, S_steps, W, dev, seed=10))
            r = bench_linear(torch, hip, timer, 16, k, n, "deq", S_steps, W, dev, seed=10, rotate=8, per_row=True)
            r.pop("_ctx")
            r.update(name="decode_gemv_per_token_ranges", bound="hbm", us_kernel=r["ms_per_step"] * 1e3,
                     gbs_kernel=r["bytes"] / (r["ms_per_step"] * 1e-3) / 1e9,
                     frac=r["bytes"] / (r["ms_per_step"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
                     note="one launch per step, each row with its own activation range")
            others.append(r)
    if "copy" in only:
        # device copy of 1 GiB: the kernel of known traffic that calibrates the memory counters
        nb = 1 << 30
        src = torch.empty(nb, dtype=torch.uint8, device=dev).random_(0, 256)
        dst = torch.empty_like(src)
        st = _stream(torch)
        ms = timer.run(lambda i: hip.memcpy_d2d_async(dst, src, nb, st), max(10, K_steps // 2), max(3, W // 2))
        others.append(dict(name="copy_d2d", n=nb, us_kernel=ms * 1e3, bytes=2 * nb, gbs=2 * nb / (ms * 1e-3) / 1e9,
                           frac=2 * nb / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, bound="hbm"))
        del src, dst
    if "elementwise" in only:
        for r in bench_elementwise(torch, hip, timer, 1 << 28, max(10, K_steps // 2), max(3, W // 2), dev):
            r.update(bound="hbm")
            others.append(r)

    # HBM bytes per launch of the headline kernel as the memory counters measured them (rocprofv3 --pmc FETCH_SIZE /
    # WRITE_SIZE, see profiles/): only reported when the kernel's source is still the one that was profiled
    traffic, traffic_note = None, "not measured for this version of the kernel source"
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        try:
            rec = json.load(open(tpath))
            if rec.get("_detail", {}).get("kernel_source_sha256") == kernel_source_sha(ROOT):
                traffic = rec.get("qgemm_tile_prefill_2048x4096x14336")
                traffic_note = "bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, see profiles/"
        except Exception:
            traffic = None

    line = summary_line(head, K_steps, W, traffic, cpu, others)
    # every other workload and the long notes: on an earlier line (and in a file next to the other run outputs), so
    # that the last line of stdout stays a short record
    full = dict(line)
    full["clock_ramp_ms"] = RAMP_MS
    full["roofline"] = dict(line["roofline"], traffic_note=traffic_note, power=power,
                            note="ops are int8 multiply-accumulates (2*M*N*K per launch); achieved and peak are tera-ops/s",
                            mfma_only_rate_measured=ceiling,
                            mfma_only_note="TOP/s of back-to-back 32x32x32 i8 MFMAs on all CUs with no other instruction, "
                                           "measured in this run: the matrix cores' sustained rate depends on operand bit "
                                           "toggling (clock under load), so 'workload_data' is the practical ceiling")
    if cpu is not None and cpu_detail:
        full["cpu_baseline"] = dict(cpu, **cpu_detail)
    full["others"] = others
    print("BENCH_DETAIL " + json.dumps(full))
    try:
        os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
        tag = "full" if not args.only else args.only.replace(",", "_")
        with open(os.path.join(ROOT, "gpurun_out", "bench_%s.json" % tag), "w") as f:
            json.dump(full, f)
    except OSError:
        pass
    sys.stdout.flush()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
