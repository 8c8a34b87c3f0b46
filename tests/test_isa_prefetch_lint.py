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


def test_gemv1_ring_registers_are_untouched_between_their_request_and_the_loop(tmp_path):
    """int4wo_gemv1_kernel requests seven weight tiles into fixed registers, stages its activations with compiler
    generated code, then enters the hand-scheduled loop with the requests possibly still in flight.  Checked on the
    generated ISA of every instantiation:
      * nothing between the first request and the loop's first instruction names a ring register, and the loop
        receives the tiles where the requests put them;
      * the activation registers are not read between their loads and the one explicit wait that covers them;
      * a wave that skips the loop waits for its requests before any other instruction of that path names a ring register;
      * every operand the compiler hands the loop lives below the loop's own register range (the loop overwrites
        its own registers, the accumulator output included, while it still reads its operands);
      * no scratch memory."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    asm = tmp_path / "gemv1.s"
    subprocess.run([hipcc, *_FLAGS, "-o", str(asm), os.path.join(_ROOT, "ao_amd", "csrc", "int4wo_gemv1.hip")], check=True,
                   capture_output=True, timeout=600)
    text = asm.read_text()
    inc = open(os.path.join(_ROOT, "ao_amd", "csrc", "int4wo_gemv1_loop.inc")).read()
    depth = int(re.search(r"#define GEMV1_RING_DEPTH (\d+)", inc).group(1))
    vbase = int(re.search(r"#define GEMV1_VBASE (\d+)", inc).group(1))
    template = [t.replace("\\n", "").replace("\\t", "").strip()
                for t in re.findall(r'"((?:[^"\\]|\\.)*)"', inc.split("#define GEMV1_LOOP_ASM", 1)[1])]
    template = [t for t in template if t]
    ring = set()
    for j in range(depth - 1):
        w = re.search(r'#define GEMV1_W%d "\{v\[(\d+):(\d+)\]\}"' % j, inc)
        ring.update(range(int(w.group(1)), int(w.group(2)) + 1))
    kernels = list(re.finditer(r"^(_ZN2ao19int4wo_gemv1_kernelILi\d+ELi\d+ELb[01]EEE\w*): ; @.*?\n(.*?)s_endpgm(.*?)\.end_amdhsa_kernel", text, re.S | re.M))
    assert len(kernels) == 10
    for m in kernels:
        name, body, meta = m.group(1), m.group(2), m.group(3)
        tp = re.match(r"_ZN2ao19int4wo_gemv1_kernelILi(\d+)ELi(\d+)ELb([01])E", name)
        xl, norm = int(tp.group(2)), tp.group(3) == "1"
        lines = [l for l in body.splitlines() if l.strip() and not re.match(r"\s*;(?!;#ASM)", l) and not l.strip().startswith(".") or re.match(r"\.LBB", l.strip())]
        code = lambda l: l.strip() and not l.strip().startswith((";", "."))
        first = next(i for i, l in enumerate(lines) if re.search(r"global_load_dwordx4 v\[\d+:\d+\], v\d+, s\[.* nt", l))
        loop = next(i for i, l in enumerate(lines) if l.strip() == template[0])
        assert first < loop, name
        requests = [l for l in lines[first:loop] if "global_load_dword" in l]
        assert len(requests) == depth - 1, (name, len(requests))
        got = set()
        for l in requests:
            got |= _regs(l.split(",")[0])
        assert got == ring, (name, sorted(got ^ ring))
        for i in range(first, loop):
            if "global_load_dword" not in lines[i]:
                continue
            dest = _regs(lines[i].split(",")[0])
            others = [l.strip() for l in lines[i + 1:loop] if code(l) and _regs(l) & dest]
            assert not others, (name, lines[i].strip(), others[:4])
        # activation loads: plain 16-byte loads before the first request, waited for by one vmcnt wait
        xloads = [i for i, l in enumerate(lines[:first]) if re.search(r"global_load_dwordx4 v\[\d+:\d+\], v\d+, s\[\d+:\d+\]$", l.strip())]
        assert len(xloads) == xl // 2 + (2 * xl + 2 if norm else xl), (name, len(xloads))
        wait = next(i for i, l in enumerate(lines) if "s_waitcnt vmcnt(%d)" % (depth - 1) in l)
        assert xloads[-1] < wait < loop
        for i in xloads:
            dest = _regs(lines[i].split(",")[0])
            early = [l.strip() for l in lines[i + 1:wait] if code(l) and _regs(l) & dest]
            assert not early, (name, lines[i].strip(), early[:4])
        # the path around the loop
        skip = [i for i, l in enumerate(lines) if l.strip() == "s_waitcnt vmcnt(0)" and not loop <= i < loop + len(template)]
        assert len(skip) == 1, (name, skip)
        j = skip[0]
        while not re.match(r"\.LBB\d+_\d+:", lines[j].strip()):
            j -= 1
        before = [l.strip() for l in lines[j + 1:skip[0]] if code(l) and _regs(l) & ring]
        assert not before, (name, before[:4])
        # operands of the loop
        actual = [l.strip() for l in lines[loop:loop + len(template)]]
        assert len(actual) == len(template)
        operands = {}
        for t, a in zip(template, actual):
            if "%[" not in t:
                assert t == a, (name, t, a)
                continue
            pat = re.escape(t)
            pat = re.sub(r"%\\\[(\w+)\\\]", lambda mm: "(?P<%s_%d>v\\[\\d+:\\d+\\]|v\\d+)" % (mm.group(1), len(operands) + id(mm) % 1000), pat)
            mm = re.fullmatch(pat, a)
            assert mm, (name, t, a)
            for key, val in mm.groupdict().items():
                operands.setdefault(key.rsplit("_", 1)[0], set()).add(val)
        assert set(operands) == {"woff", "qaddr", "xaddr", "mask", "sello", "selhi", "bc1", "bc2"}, (name, sorted(operands))
        used = set()
        for key, vals in operands.items():
            assert len(vals) == 1, (name, key, vals)
            regs = _regs(next(iter(vals)))
            assert max(regs) < vbase, (name, key, vals)
            assert not (regs & used), (name, key, vals)
            used |= regs
        scratch = re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", meta)
        assert scratch is None or int(scratch.group(1)) == 0, (name, scratch.group(0))


def test_prefill_gemm_requests_are_waited_for_before_their_registers_are_touched(tmp_path):
    """int4wo_gemm_lds_kernel issues every load of its K loop as an asm statement and waits for them with explicit
    s_waitcnt vmcnt(0) statements; the compiler neither counts those loads nor knows that their target registers are
    being filled.  Checked on the generated ISA of every instantiation:
      * between a weight load and the next vmcnt(0) wait, on every path (around the loop's back edge and out of the loop by
        either exit), no instruction reads or writes the load's target registers, so a copy of stale contents or a reuse
        of a register under a load in flight (the epilogue's, after the last, unused requests of the loop) cannot happen;
      * the K loop carries the LDS-direct activation requests (16 per two steps and wave of the 256-row kernel, 32 of the
        128-row kernel, whose waves each bring in their own slices) and the weight requests (a chunk and its scale / zero
        per 32-row block) of its two steps;
      * no scratch access inside the K loop, every matrix instruction accumulates in accumulation registers;
      * no accumulator is read before the wait that follows the loop."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    asm = tmp_path / "gemm.s"
    subprocess.run([hipcc, *_FLAGS, "-o", str(asm), os.path.join(_ROOT, "ao_amd", "csrc", "int4wo_gemm.hip")], check=True,
                   capture_output=True, timeout=900)
    text = asm.read_text()
    kernels = list(re.finditer(r"^(_ZN2ao22int4wo_gemm_lds_kernelILi(\d+)ELi([12])EEEvNS_10LinearArgsEiii): ; @.*?\n(.*?)s_endpgm(.*?)\.end_amdhsa_kernel",
                               text, re.S | re.M))
    assert len(kernels) == 8
    # the 128-row kernel whose waves split K: the same discipline, 16 activation requests per step and wave
    kwave = list(re.finditer(r"^(_ZN2ao24int4wo_gemm_kwave_kernelILi(\d+)EEEvNS_10LinearArgsEiii): ; @.*?\n(.*?)s_endpgm(.*?)\.end_amdhsa_kernel",
                             text, re.S | re.M))
    assert len(kwave) == 4
    cases = [(m.group(1), int(m.group(3)), 16, m.group(4)) for m in kernels] + [(m.group(1), 2, 32, m.group(3)) for m in kwave]
    for name, nt, dma, body in cases:
        lines = [l.strip() for l in body.splitlines()]
        lines = [l for l in lines if l and not l.startswith(";") and not (l.startswith(".") and not l.startswith(".LBB"))]
        labels = {re.match(r"(\.LBB\d+_\d+):", l).group(1): i for i, l in enumerate(lines) if re.match(r"\.LBB\d+_\d+:", l)}
        back = {}
        for i, l in enumerate(lines):
            b = re.match(r"s_c?branch\w* (\.LBB\d+_\d+)", l)
            if b and labels.get(b.group(1), i) < i:
                back[i] = labels[b.group(1)]
        assert len(set(back.values())) == 1, (name, back)   # the K loop is the only loop (its second step may be skipped
        loop_end, loop_head = max(back), min(back.values())  # at the end of K: two branches back to the one head)
        loads = [i for i, l in enumerate(lines) if re.match(r"global_load_dword(x4)? v", l)]
        assert sum(1 for i in loads if loop_head < i < loop_end) == 2 * nt * 2, name   # chunk + qparams per block, two steps
        assert sum(1 for l in lines[loop_head:loop_end] if l.startswith("global_load_lds_dwordx4")) == dma, name
        # every path from a load to its first vmcnt(0) wait: around the back edge, and out of the loop by either exit
        # (the requests of the last step are issued for a step past the end and are still in flight when the loop is
        # left; the wait behind the loop names their targets as operands, which is what keeps the epilogue's first
        # instructions, scheduled in front of that wait, out of those registers)
        for i in loads:
            dest = _regs(lines[i].split(",")[0])
            todo, seen = [i + 1], set()
            while todo:
                j = todo.pop()
                if j in seen:
                    continue
                seen.add(j)
                assert j < len(lines), (name, lines[i], "no wait before the end of the kernel")
                if lines[j].startswith("s_waitcnt vmcnt(0)"):
                    continue
                touched = not lines[j].startswith((".LBB", "s_", "global_load")) and _regs(lines[j]) & dest
                assert not touched, (name, lines[i], lines[j])
                b = re.match(r"s_(c?)branch\w* (\.LBB\d+_\d+)", lines[j])
                if b:
                    todo.append(labels[b.group(2)])
                    if b.group(1):
                        todo.append(j + 1)
                else:
                    todo.append(j + 1)
        # the accumulators are first read behind the wait that follows the loop: the matrix instructions are asm
        # statements, whose result latency the compiler does not know, so a copy placed right behind the loop would
        # read a register the last matrix instructions have not written yet
        last_mfma = max(i for i, l in enumerate(lines) if l.startswith("v_mfma"))
        nops = [i for i, l in enumerate(lines) if l == "s_nop 15" and i > last_mfma]
        assert nops, name
        assert not [l for l in lines[:nops[0]] if l.startswith(("v_accvgpr_read", "v_accvgpr_mov"))], name
        # values the epilogue needs may be parked in scratch around the loop, never inside it
        assert not [l for l in lines[loop_head:loop_end] if l.startswith("scratch_")], name
        assert len(re.findall(r"v_mfma_f32_32x32x16_bf16 a\[", body)) >= (64 * nt if dma == 16 else 64), name


def _vmcnt(line):
    m = re.search(r"vmcnt\((\d+)\)", line)
    return int(m.group(1)) if m else None


def _asm_load_violations(body):
    """Walks every path from every asm-issued global load of a kernel to the wait that covers it and returns the
    instructions on the way that read or write the load's target registers.

    The count wait `s_waitcnt vmcnt(n)` covers a load when at least n vector memory loads were issued after it (they
    return in order).  Loads the compiler issues count too; stores are ignored, which only makes the check stricter."""
    raw = [l.strip() for l in body.splitlines()]
    lines, in_asm, is_asm = [], False, []
    for l in raw:
        if l.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if l.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not l or l.startswith(";") or (l.startswith(".") and not l.startswith(".LBB")):
            continue
        lines.append(l.split(";")[0].strip())
        is_asm.append(in_asm)
    labels = {re.match(r"(\.LBB\d+_\d+):", l).group(1): i for i, l in enumerate(lines) if re.match(r"\.LBB\d+_\d+:", l)}
    is_load = [bool(re.match(r"(global|buffer|scratch|flat)_load", l)) for l in lines]
    out = []
    for i, l in enumerate(lines):
        if not (is_asm[i] and re.match(r"global_load_dword(x[234])? v", l)):
            continue
        dest = _regs(l.split(",")[0])
        todo, seen = [(i + 1, 0)], set()
        while todo:
            j, younger = todo.pop()
            if (j, younger) in seen or j >= len(lines):
                continue
            seen.add((j, younger))
            cur = lines[j]
            if cur.startswith("s_endpgm"):
                continue
            if cur.startswith("s_waitcnt"):
                n = _vmcnt(cur)
                if n is not None and younger >= n:
                    continue
            elif is_load[j]:
                younger = min(younger + 1, 63)
            elif not cur.startswith((".LBB", "s_")) and _regs(cur) & dest:
                out.append((l, cur))
                continue
            b = re.match(r"s_(c?)branch\w* (\.LBB\d+_\d+)", cur)
            if b:
                todo.append((labels[b.group(2)], younger))
                if b.group(1):
                    todo.append((j + 1, younger))
            else:
                todo.append((j + 1, younger))
    return out


def test_gemv2_loop_operands_and_ring(tmp_path):
    """int4wo_gemv2_kernel: in every instantiation the three requests of the prologue land in the ring registers the
    generated loop reads them from, every operand the compiler hands the loop lives below the loop's own register range
    (the loop overwrites its registers while it still reads its operands) and is a register of its own, the loop text is
    the generated one, and no scratch memory is used."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    asm = tmp_path / "gemv2.s"
    subprocess.run([hipcc, *_FLAGS, "-o", str(asm), os.path.join(_ROOT, "ao_amd", "csrc", "int4wo_gemv2.hip")], check=True,
                   capture_output=True, timeout=600)
    text = asm.read_text()
    inc = open(os.path.join(_ROOT, "ao_amd", "csrc", "int4wo_gemv2_loop.inc")).read()
    vbase = int(re.search(r"#define GEMV2_VBASE (\d+)", inc).group(1))
    template = [t.replace("\\n", "").replace("\\t", "").strip()
                for t in re.findall(r'"((?:[^"\\]|\\.)*)"', inc.split("#define GEMV2_LOOP_ASM", 1)[1])]
    template = [t for t in template if t]
    ring = set()
    for j in range(3):
        w = re.search(r'#define GEMV2_W%d "\{v\[(\d+):(\d+)\]\}"' % j, inc)
        ring.update(range(int(w.group(1)), int(w.group(2)) + 1))
    kernels = list(re.finditer(r"^(_ZN2ao19int4wo_gemv2_kernelILi\d+ELi\d+EEE\w*): ; @.*?\n(.*?)s_endpgm(.*?)\.end_amdhsa_kernel", text, re.S | re.M))
    assert len(kernels) == 6
    for m in kernels:
        name, body, meta = m.group(1), m.group(2), m.group(3)
        lines = [l.strip() for l in body.splitlines() if l.strip() and not l.strip().startswith(";") and
                 (not l.strip().startswith(".") or l.strip().startswith(".LBB"))]
        loop = next(i for i, l in enumerate(lines) if l == template[0])
        requests = [l for l in lines[:loop] if re.match(r"global_load_dwordx4 v\[\d+:\d+\], v\d+, s\[.* nt", l)]
        assert len(requests) == 3, (name, len(requests))
        got = set()
        for l in requests:
            got |= _regs(l.split(",")[0])
        assert got == ring, (name, sorted(got ^ ring))
        actual = lines[loop:loop + len(template)]
        operands = {}
        for t, a in zip(template, actual):
            if "%[" not in t:
                assert t == a, (name, t, a)
                continue
            keys = re.findall(r"%\[(\w+)\]", t)
            pat = re.sub(r"%\\\[\w+\\\]", lambda mm: r"(v\[\d+:\d+\]|v\d+)", re.escape(t))
            mm = re.fullmatch(pat, a)
            assert mm, (name, t, a)
            for key, val in zip(keys, mm.groups()):
                operands.setdefault(key, set()).add(val)
        assert set(operands) == {"woff", "qaddr", "xlane", "redaddr", "finv", "mask", "sello", "selhi", "bc1", "bc2"}, (name, sorted(operands))
        used = set()
        for key, vals in operands.items():
            assert len(vals) == 1, (name, key, vals)
            regs = _regs(next(iter(vals)))
            assert max(regs) < vbase, (name, key, vals)
            assert not (regs & used), (name, key, vals)
            used |= regs
        scratch = re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", meta)
        assert scratch is None or int(scratch.group(1)) == 0, (name, scratch.group(0))


@pytest.mark.parametrize("source", ["int4wo_gemm.hip", "int4wo_gemv1.hip", "int4wo_gemv2.hip"])
def test_asm_loads_are_waited_for_on_every_path_before_their_registers_are_touched(tmp_path, source):
    """Every kernel that issues global loads from asm statements (the weight streams of the GEMV rings and of the
    prefill kernels): between such a load and the wait that covers it, on every path through loops and out of them,
    nothing reads or writes the registers being filled.  The compiler knows neither that the load is outstanding nor,
    once the loaded value is dead, that the register is not free yet."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    asm = tmp_path / (source + ".s")
    subprocess.run([hipcc, *_FLAGS, "-o", str(asm), os.path.join(_ROOT, "ao_amd", "csrc", source)], check=True,
                   capture_output=True, timeout=900)
    text = asm.read_text()
    kernels = list(re.finditer(r"^(_ZN2ao\w+): ; @.*?\n(.*?)\.end_amdhsa_kernel", text, re.S | re.M))
    checked = 0
    for m in kernels:
        name, body = m.group(1), m.group(2)
        if ";;#ASMSTART\n\tglobal_load_dword" not in body:
            continue
        checked += 1
        bad = _asm_load_violations(body)
        assert not bad, (name, bad[:4])
    assert checked >= 4, (source, checked)
