"""Compile-time check of the inline-asm prefetch rings of the int8 and FP6 GEMV kernels (no GPU: hipcc cross-compiles).

Those kernels request D - 1 weight tiles with asm loads before they stage the activations and wait for them with explicit
`s_waitcnt vmcnt(n)` blocks that name no registers.  The compiler does not know that the loaded registers are still being
filled; the scheme is only sound if, between a tile's request and the first explicit wait, no other instruction reads or
writes those registers (a copy or a spill there would move stale data).  This test reads the generated ISA of every
staged instantiation and checks exactly that for the prologue prefetch, and that the kernels use no scratch memory."""
import os
import re
import shutil
import subprocess

import pytest

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
          "-packed-fp32-ops", "-S", "--cuda-device-only", f"-I{_ROOT}/ao_amd/csrc", f"-I{_ROOT}/include"]

_CASES = [
    ("int8wo_linear.hip", r"_ZN2ao20int8wo_linear_kernelILi\d+ELb1ELb[01]E\w*",
     r"global_load_dwordx4 v\[(\d+):(\d+)\], v\d+, s\[.* nt", 2),
    ("fp6.hip", r"_ZN2ao15fp6_gemv_kernelILi\d+ELb[01]ELb[01]E\w*",
     r"global_load_dwordx[24] v\[(\d+):(\d+)\], v\d+, s\[.* nt", 2),
]


def _regs(text):
    out = set()
    for r in re.finditer(r"v\[(\d+):(\d+)\]|\bv(\d+)\b", text):
        if r.group(3):
            out.add(int(r.group(3)))
        else:
            out.update(range(int(r.group(1)), int(r.group(2)) + 1))
    return out


@pytest.mark.parametrize("source,kernel_pat,load_pat,loads_per_tile", _CASES)
def test_prefetched_registers_are_untouched_until_the_first_wait(tmp_path, source, kernel_pat, load_pat, loads_per_tile):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    asm = tmp_path / (source + ".s")
    subprocess.run([hipcc, *_FLAGS, "-o", str(asm), os.path.join(_ROOT, "ao_amd", "csrc", source)], check=True,
                   capture_output=True, timeout=600)
    text = asm.read_text()
    kernels = list(re.finditer(r"^(" + kernel_pat + r"): ; @.*?\n(.*?)s_endpgm(.*?)\.end_amdhsa_kernel", text, re.S | re.M))
    assert len(kernels) >= 10, f"expected the staged instantiations of {source}, found {len(kernels)}"
    for m in kernels:
        name, body, meta = m.group(1), m.group(2), m.group(3)
        dual = name.endswith("Lb1EEEvNS_8Int8ArgsE") or "Lb1EEEvNS_11Fp6GemvArgsE" in name
        n_prefetch = 3 * loads_per_tile * (2 if dual else 1)  # D - 1 = 3 tiles
        first_wait = body.find(";;#ASMSTART\n\ts_waitcnt vmcnt")
        assert first_wait > 0, name
        lines = body[:first_wait].splitlines()
        dests, seen, last = set(), 0, None
        for i, line in enumerate(lines):
            d = re.search(load_pat, line)
            if d and seen < n_prefetch:
                dests.update(range(int(d.group(1)), int(d.group(2)) + 1))
                seen, last = seen + 1, i
        assert seen == n_prefetch, (name, seen)
        touched = [l.strip() for l in lines[last + 1:]
                   if l.strip() and not l.strip().startswith((";", ".")) and _regs(l) & dests]
        assert not touched, (name, touched[:4])
        scratch = re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", meta)
        assert scratch is None or int(scratch.group(1)) == 0, (name, scratch.group(0))
