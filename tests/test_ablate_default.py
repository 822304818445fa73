"""The measurement switch of the tile kernel (ITEXHIP_ABLATE: parts of the kernel compiled out for time / power
measurements, wrong results) is off in every ordinary build, and only ablate.py turns it on, into libraries of
their own that nothing loads by default."""
import importlib.util
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "intel-extension-for-tensorflow_amd")


def _load(name):
    spec = importlib.util.spec_from_file_location(name, os.path.join(PKG, name + ".py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_switch_defaults_to_off_and_the_build_never_sets_it():
    text = open(os.path.join(PKG, "csrc", "qgemm_tile.hpp")).read()
    assert re.search(r"#ifndef ITEXHIP_ABLATE\s*\n#define ITEXHIP_ABLATE 0\s*\n#endif", text)
    build = _load("build")
    assert not any("ITEXHIP_ABLATE" in f for f in build.HIP_FLAGS)
    for name in os.listdir(PKG):
        if name.endswith(".py") and name != "ablate.py":
            assert "ITEXHIP_ABLATE" not in open(os.path.join(PKG, name)).read(), name


def test_measurement_libraries_live_apart_from_the_product_library():
    src = open(os.path.join(PKG, "ablate.py")).read()
    assert '"ablate_%d" % mask' in src                      # lib/ablate_<mask>/libitexhip.so
    binding = open(os.path.join(PKG, "itexhip.py")).read()
    assert "ablate" not in binding                          # only an explicit ITEXHIP_LIB reaches them
