"""The generated ISA of the kernels that store 128 bits per lane must not write a data register of such a store within
the next two instructions: on gfx950 a `buffer_store_dwordx4 ... offen` with a scalar soffset, followed directly by a
vector instruction that rewrites one of its data registers, now and then stores the new value (the compiler inserts wait
states for this hazard only when the store has no scalar soffset). The library's stores go through
`buffer_store_b128_guarded` (csrc/common.hpp); this test compiles the sources that use it to assembly (hipcc
cross-compiles without a GPU) and scans for the pattern."""
import concurrent.futures
import glob
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "dragon-alpha-v1.0_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
WINDOW = 2


def _regs(tok):
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def hazard_sites(asm_text):
    lines = [l.strip() for l in asm_text.splitlines()]
    ins = [l for l in lines if l and not l.startswith((";", "//")) and not (l.startswith(".") and not l.startswith(".LBB"))]
    sites = []
    for k, l in enumerate(ins):
        m = re.match(r"buffer_store_dwordx[34]\s+(v\[\d+:\d+\])", l)
        if not m:
            continue
        data = _regs(m.group(1))
        for l2 in ins[k + 1:k + 1 + WINDOW]:
            if l2.startswith((".LBB", "s_cbranch", "s_branch", "s_endpgm", "s_barrier", "s_nop")) or l2.endswith(":"):
                break
            mm = re.match(r"v_\w+\s+([^,\s]+)", l2)
            if mm and (_regs(mm.group(1)) & data):
                sites.append((l, l2))
                break
    return sites


def test_scanner_sees_the_pattern():
    bad = "buffer_store_dwordx4 v[60:63], v125, s[8:11], s59 offen\nv_mov_b32_e32 v60, v57\n"
    ok = "buffer_store_dwordx4 v[60:63], v125, s[8:11], s59 offen\ns_nop 1\nv_mov_b32_e32 v60, v57\n"
    far = "buffer_store_dwordx4 v[60:63], v125, s[8:11], s59 offen\nv_mov_b32_e32 v70, v57\nv_mov_b32_e32 v71, v57\nv_mov_b32_e32 v60, v57\n"
    assert len(hazard_sites(bad)) == 1 and not hazard_sites(ok) and not hazard_sites(far)


def _sources():
    """The translation units with 96- / 128-bit buffer stores: the helper's name in the file or in a kernel header it includes."""
    out = []
    for src in sorted(glob.glob(os.path.join(CSRC, "*.hip"))):
        text = open(src).read()
        for inc in re.findall(r'#include "([^"]+_kernel\.hpp)"', text):
            text += open(os.path.join(CSRC, inc)).read()
        if "buffer_store_b128" in text or "buffer_store_guarded" in text:
            out.append(src)
    return out


def _compile(src, tmp):
    s_path = os.path.join(tmp, os.path.basename(src)[:-4] + ".s")
    subprocess.run([HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                    "-S", "--cuda-device-only", "-o", s_path, src], stderr=subprocess.DEVNULL, check=True)
    return src, open(s_path).read()


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not found")
def test_no_store_is_followed_by_a_write_to_its_data_registers(tmp_path):
    srcs = _sources()
    assert len(srcs) >= 8, srcs          # the kernels with 128-bit buffer stores, direct_conv.hip, direct_conv_narrow.hip and direct_conv_odd.hip among them
    assert all(any(s.endswith(f) for s in srcs) for f in ("direct_conv.hip", "direct_conv_narrow.hip", "direct_conv_odd.hip"))
    assert not [s for s in srcs if "__builtin_amdgcn_raw_buffer_store_b128" in open(s).read()], "a store bypasses the guarded helper"
    with concurrent.futures.ThreadPoolExecutor(max_workers=6) as ex:
        results = list(ex.map(lambda s: _compile(s, str(tmp_path)), srcs))
    for src, asm in results:
        assert "buffer_store_dwordx4" in asm or "buffer_store_dwordx3" in asm, src   # (the narrow kernels store 96, 64 or 32 bits)
        sites = hazard_sites(asm)
        assert not sites, "%s: %d sites, first: %s || %s" % (os.path.basename(src), len(sites), sites[0][0], sites[0][1])
