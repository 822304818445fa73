"""CPU-only checks of the C-ABI library: it loads without a GPU, exports every symbol that
include/itexhip.h declares, validates arguments before touching the device, and its host-only
epilogue descriptor agrees with the oracle's."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from oracle import pyoracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "itexhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(itexhip_\w+)\s*\(", text)))


def test_exports_every_declared_symbol(hip):
    syms = declared_symbols()
    assert len(syms) >= 18
    for s in syms:
        assert hasattr(hip.raw(), s), "missing export: " + s
    assert sorted(hip.EXPORTS) == syms


def test_build_info(hip):
    assert "gfx950" in hip.build_info()


def test_argument_validation_needs_no_gpu(hip):
    with pytest.raises(hip.ItexHipError) as e:
        hip.quantize(16, 16, 4, hip.FLOAT, 1.0)
    assert e.value.code == hip.INVALID_ARGUMENT and "qint8 or quint8" in str(e.value)
    with pytest.raises(hip.ItexHipError):
        hip.quantize(16, 16, -1, hip.QINT8, 1.0)
    # empty tensors are a no-op, no device call
    hip.quantize(None, None, 0, hip.QINT8, 1.0)
    hip.dequantize(None, None, 0, hip.QUINT8, 1.0)
    hip.requantize(None, None, 0, hip.QINT8, 1.0)
    ep = hip.Epilogue()
    hip.qgemm(None, hip.QUINT8, None, None, 0, 64, 16, None, None, ep, hip.FLOAT, None)
    with pytest.raises(hip.ItexHipError) as e:
        hip.qgemm(16, hip.QUINT8, 16, 16, 32, 3, 16, None, None, ep, hip.FLOAT, 16)
    assert "multiple of 16" in str(e.value)
    with pytest.raises(hip.ItexHipError):
        hip.qgemv(16, hip.QUINT8, 16, 16, 129, 64, 16, None, None, ep, hip.FLOAT, 16)
    assert hip.qgemm_packed_bytes(4096, 14336) == 4096 * 14336
    assert hip.qgemm_packed_bytes(3, 4) == 2048


CASES = [
    dict(api=0, t_out=orc.FLOAT, has_dequantize=True),
    dict(api=0, t_out=orc.FLOAT, has_dequantize=True, activation=orc.ACT_RELU),
    dict(api=0, t_out=orc.QINT8, has_requantize=True),
    dict(api=0, t_out=orc.QUINT8, has_requantize=True, activation=orc.ACT_RELU, n_fused_ops=2),
    dict(api=0, t_out=orc.QUINT8, has_requantize=True, out_min_first=True),
    dict(api=0, t_out=orc.QUINT8, has_requantize=True, out_min_first=True, activation=orc.ACT_RELU),
    dict(api=0, t_out=orc.FLOAT, has_dequantize=True, activation=orc.ACT_LEAKYRELU, leakyrelu_alpha=0.3),
    dict(api=0, t_out=orc.FLOAT, has_dequantize=True, activation=orc.ACT_RELU6),
    dict(api=0, t_out=orc.QINT32),
    dict(api=1, t_out=orc.QINT32, n_fused_ops=1),
    dict(api=1, t_out=orc.QINT8, n_fused_ops=1),
    dict(api=1, t_out=orc.QUINT8, n_fused_ops=2, activation=orc.ACT_RELU),
    dict(api=1, t_out=orc.FLOAT, n_fused_ops=1),
    dict(api=2, t_out=orc.QINT32),
    dict(api=2, t_out=orc.QUINT8, activation=orc.ACT_RELU),
    dict(api=2, t_out=orc.QINT8),
    dict(api=2, t_out=orc.FLOAT),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("input_mode", [orc.MIN_FIRST, orc.SCALED])
def test_epilogue_desc_matches_oracle(hip, case, input_mode):
    kw = dict(case)
    t_in = orc.QUINT8 if input_mode == orc.MIN_FIRST else orc.QINT8
    at = orc.matmul_attrs(t_in=t_in, input_mode=input_mode, **kw)
    N = 8
    nb = 1 if kw["api"] == 2 else N
    rng = np.random.default_rng(0)
    min_b = -rng.random(nb).astype(np.float32)
    max_b = rng.random(nb).astype(np.float32)
    st, sc, sb, ep_o = orc.qmatmul_prepare(at, N, np.arange(N), -1.5, 2.5, min_b, max_b, -3.0, 4.0,
                                           np.ones(N, np.float32))
    assert st == orc.OK
    p = hip.matmul_params(t_in=t_in, input_mode=input_mode, min_a=-1.5, max_a=2.5, min_out=-3.0,
                          max_out=4.0, **kw)
    ep = hip.qmatmul_epilogue_desc(p, nb)
    assert ep.n_scales == ep_o.n_scales and ep.n_eltwise == ep_o.n_eltwise
    for e in range(ep.n_eltwise):
        assert (ep.elt[e].alg, ep.elt[e].alpha, ep.elt[e].beta) == \
               (ep_o.elt[e].alg, ep_o.elt[e].alpha, ep_o.elt[e].beta)
