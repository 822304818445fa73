"""The tile kernels issue some memory instructions as inline assembly, which the compiler neither counts in its wait
counts nor protects with hazard wait states.  The build runs csrc/check_asm_hazards.py on the compiled device assembly
and refuses to link on a finding; these tests keep that rule alive: the checker must still flag the two hazards on
hand-made assembly, and the assembly the last build left behind must be clean."""
import glob
import importlib.util
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "intel-extension-for-tensorflow_amd")


def _load(path, name):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="module")
def chk():
    return _load(os.path.join(PKG, "csrc", "check_asm_hazards.py"), "check_asm_hazards")


KERNEL = """
_Z6kernelv:
\ts_load_dwordx2 s[0:1], s[4:5], 0x0
\t;;#ASMSTART
\tglobal_load_dword v7, v[2:3], off
\t;;#ASMEND
\tglobal_load_dwordx4 v[10:13], v[4:5], off
%s
\tv_add_f32_e32 v8, v7, v7
\t;;#ASMSTART
\tglobal_store_dwordx4 v[2:3], v[10:13], off sc1
%s
\t;;#ASMEND
\ts_endpgm
"""


def _check(chk, tmp_path, wait, nop, capsys):
    f = tmp_path / "k.s"
    f.write_text(KERNEL % (wait, nop))
    flagged = chk.check_file(str(f))
    return flagged, capsys.readouterr().out


def test_checker_accepts_waited_load_and_padded_store(chk, tmp_path, capsys):
    flagged, out = _check(chk, tmp_path, "\ts_waitcnt vmcnt(1)", "\ts_nop 1", capsys)
    assert flagged == 0, out
    assert "1 early load sites" in out


def test_checker_flags_use_of_an_early_load_without_wait(chk, tmp_path, capsys):
    # vmcnt(2) still allows the early load (two newer memory instructions... only one was issued) to be in flight
    flagged, out = _check(chk, tmp_path, "\ts_waitcnt vmcnt(2)", "\ts_nop 1", capsys)
    assert flagged == 1 and "v7 is used" in out
    flagged, out = _check(chk, tmp_path, "", "\ts_nop 1", capsys)
    assert flagged == 1 and "v7 is used" in out


def test_checker_flags_assembly_store_without_wait_states(chk, tmp_path, capsys):
    flagged, out = _check(chk, tmp_path, "\ts_waitcnt vmcnt(1)", "", capsys)
    assert flagged == 1 and "without two wait states" in out
    flagged, out = _check(chk, tmp_path, "\ts_waitcnt vmcnt(1)", "\ts_nop 0", capsys)
    assert flagged == 1


def test_assembly_of_the_last_build_is_clean(chk, capsys):
    build = _load(os.path.join(PKG, "build.py"), "itex_amd_build_for_hazards")
    srcs = sorted(f for f in glob.glob(os.path.join(PKG, "csrc", "*.hip")) if build._has_untracked_asm(f))
    assert srcs, "no translation unit with inline-assembly memory instructions found: the rule names the wrong files"
    asm = [build.device_assembly_of(f) for f in srcs]
    if not all(os.path.exists(f) for f in asm):
        pytest.skip("device assembly not present (the library was not built in this tree)")
    lib = os.path.join(PKG, "lib", "libitexhip.so")
    assert os.path.exists(lib)
    for f, src in zip(asm, srcs):   # the assembly is the one the library was built from, not a stale file
        assert os.path.getmtime(f) <= os.path.getmtime(lib) + 1
    sites = 0
    for f in asm:
        assert chk.check_file(f) == 0, capsys.readouterr().out
    out = capsys.readouterr().out
    sites = sum(int(l.split(" functions, ")[1].split(" early")[0]) for l in out.splitlines() if " early load sites" in l)
    assert sites > 0, "the checker found no early load at all: its pattern no longer matches the kernels"


def test_inline_assembly_memory_instructions_only_in_checked_units():
    """Every translation unit that can contain an untracked load or an assembly store (it includes the tile kernel's
    header, calls the early parameter loads or writes such an instruction itself) is one the build checks."""
    import re
    pat = re.compile(r'asm\s+volatile\s*\(\s*"[^"]*global_(load_dword|load_ushort|store)')
    build = _load(os.path.join(PKG, "build.py"), "itex_amd_build_for_hazards2")
    headers = [f for f in glob.glob(os.path.join(PKG, "csrc", "*.hpp")) if pat.search(open(f).read())]
    assert sorted(os.path.basename(h) for h in headers) == ["qgemm_common.hpp", "qgemm_tile.hpp"]
    checked = 0
    for src in glob.glob(os.path.join(PKG, "csrc", "*.hip")):
        text = open(src).read()
        exposed = bool(pat.search(text)) or '"qgemm_tile.hpp"' in text or "load_raw_channel_early(" in text
        assert exposed == build._has_untracked_asm(src), os.path.basename(src)
        checked += exposed
    assert checked >= 6
