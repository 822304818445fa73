"""Measurement builds of the MatMul tile kernel with parts compiled out (ITEXHIP_ABLATE in csrc/qgemm_tile.hpp).

    python intel-extension-for-tensorflow_amd/ablate.py [--unit qgemm_tile_f32.hip] MASK [MASK ...]

builds lib/ablate_<MASK>/libitexhip.so for each bit mask: one translation unit of the tile kernels (by default
csrc/qgemm_tile_s8.hip, the 8-bit outputs, which holds the kernel of the prefill benchmark; --unit names another, e.g.
the fp32 outputs of the BERT-base rows) compiled with -DITEXHIP_ABLATE=<MASK>, linked with the objects of the last
ordinary build (run build.py first).  Such a library computes wrong results and is
for time / power measurements only:

    ITEXHIP_LIB=$PWD/intel-extension-for-tensorflow_amd/lib/ablate_4/libitexhip.so python3 bench.py --only power --no-cpu

prints, under roofline.power.headline_gemm of the "BENCH_DETAIL" line, the board power, shader clock and time per
launch of the prefill MatMul with the K loop's operand loads compiled out.  Nothing in the product loads these
libraries.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import build as b  # noqa: E402

UNIT = "qgemm_tile_s8.hip"


def build_variant(mask):
    mask = int(mask)
    if not 0 < mask < 64:
        raise SystemExit("mask must be 1..63, got %d" % mask)
    out_dir = os.path.join(b.LIB, "ablate_%d" % mask)
    os.makedirs(out_dir, exist_ok=True)
    obj = os.path.join(b.OBJ, "ablate_%d.o" % mask)
    b._run([b.HIPCC] + b.HIP_FLAGS + ["-DITEXHIP_ABLATE=%d" % mask, "-c", os.path.join(b.CSRC, UNIT), "-o", obj])
    objs = []
    for src in sorted(glob.glob(os.path.join(b.CSRC, "*.hip"))):
        o = obj if os.path.basename(src) == UNIT else os.path.join(b.OBJ, os.path.basename(src) + ".o")
        if not os.path.exists(o):
            raise SystemExit("missing %s: run build.py first" % o)
        objs.append(o)
    lib = os.path.join(out_dir, "libitexhip.so")
    b._run([b.HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    os.remove(obj)
    return lib


if __name__ == "__main__":
    masks = sys.argv[1:]
    if len(masks) >= 2 and masks[0] == "--unit":
        UNIT = os.path.basename(masks[1])
        if not (UNIT.startswith("qgemm_tile_") and os.path.exists(os.path.join(b.CSRC, UNIT))):
            raise SystemExit("no tile unit %s under csrc/" % UNIT)
        masks = masks[2:]
    if not masks:
        raise SystemExit(__doc__)
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(masks))) as ex:
        for lib in ex.map(build_variant, masks):
            print("built", os.path.relpath(lib, b.ROOT))
