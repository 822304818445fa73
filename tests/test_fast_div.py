"""The multiply-shift division of the convolution kernel (FastDiv in csrc/qgemm_common.hpp): mul = ceil(2^sh / d),
sh = 31 + ceil(log2 d), n / d = (n * mul) >> sh.  The claim that this is exact for every 0 <= n < 2^31 and that mul fits
32 bits is checked here against integer division, on the divisors the kernel can meet and on the dividends where a
wrong constant shows first (multiples of d and their neighbours, the top of the range).  The device code itself is
exercised by the convolution parity tests."""
import random


def make_fast_div(d):
    s = 0
    while (1 << s) < d:
        s += 1
    sh = 31 + s
    return ((1 << sh) + d - 1) // d, sh


def test_constants_fit_and_divide_exactly():
    rnd = random.Random(7)
    divisors = list(range(1, 1200)) + [(1 << k) + o for k in range(1, 31) for o in (-1, 0, 1)] + \
               [rnd.randrange(1, 1 << 31) for _ in range(300)] + [(1 << 31) - 1]
    top = (1 << 31) - 1
    for d in divisors:
        if not 1 <= d <= top:
            continue
        mul, sh = make_fast_div(d)
        assert mul < (1 << 32) and sh < 64, d
        assert top * mul < (1 << 64), d            # the product the kernel forms in 64 bits
        ns = {0, 1, d - 1, d, d + 1, top, top - 1, top - d, (top // d) * d, (top // d) * d - 1}
        ns.update(rnd.randrange(0, top + 1) for _ in range(40))
        ns.update(q * d + r for q in (1, 2, 3, 1000, top // d - 1) for r in (-1, 0, 1))
        for n in ns:
            if 0 <= n <= top:
                assert (n * mul) >> sh == n // d, (n, d)


def test_source_states_the_same_constants():
    import os, re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = open(os.path.join(root, "intel-extension-for-tensorflow_amd", "csrc", "qgemm_common.hpp")).read()
    body = src[src.index("inline FastDiv make_fast_div"):src.index("__device__ __forceinline__ int fast_div")]
    assert re.search(r"sh = 31 \+ s;", body) and "(1ull << sh) + static_cast<uint64_t>(d) - 1) / static_cast<uint64_t>(d)" in body
    assert ">> f.sh" in src[src.index("__device__ __forceinline__ int fast_div"):][:300]
