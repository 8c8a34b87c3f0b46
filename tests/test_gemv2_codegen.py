"""CPU checks of the generated tile loop of int4wo_gemv2_kernel (ao_amd/csrc/int4wo_gemv2_loop.inc): the variant of
the single-row GEMV loop whose runs cross row-block / K-split boundaries, read the activation row from one shared LDS
image and park one row of partial sums per unit in LDS.  Executed by the wavefront model of tests/_gemv1_sim.py
against weights packed by the oracle, like tests/test_gemv1_codegen.py does for the first variant."""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from _gemv1_sim import HazardError, Wave
from test_gemv1_codegen import _bf16, _f32, lane_constants, stage_x

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ao_amd", "csrc")
INC = os.path.join(CSRC, "int4wo_gemv2_loop.inc")
GEN = os.path.join(CSRC, "gen_int4wo_gemv1.py")

VIN = {"woff": "v0", "qaddr": "v1", "xlane": "v2", "mask": "v3", "sello": "v4", "selhi": "v5", "bc1": "v[8:9]",
       "bc2": "v[10:11]", "redaddr": "v6", "finv": "v7"}


def _asm_lines():
    text = open(INC).read()
    body = text.split("#define GEMV2_LOOP_ASM", 1)[1]
    out = []
    for ln in re.findall(r'"((?:[^"\\]|\\.)*)"', body):
        ln = ln.replace("\\n", "").replace("\\t", "").strip()
        if not ln:
            continue
        for k, val in VIN.items():
            ln = ln.replace("%%[%s]" % k, val)
        assert "%[" not in ln, ln
        out.append(ln)
    return out


def _define(name):
    return re.search(r"#define %s (.+)" % name, open(INC).read()).group(1).strip()


def _sreg(name):
    return int(re.search(r"s\[?(\d+)", _define("GEMV2_S_" + name)).group(1))


def test_include_file_is_what_the_generator_prints():
    out = subprocess.run([sys.executable, GEN, "--v2"], capture_output=True, text=True, check=True).stdout
    assert out == open(INC).read()


def make_problem(oracle, G, KB, R, seed, one_hot=None):
    rng = np.random.default_rng(seed)
    K = KB * 128
    codes = rng.integers(0, 16, size=(16 * R, K)).astype(np.int32)
    ng = K // G
    scale = _bf16((1.0 + rng.integers(0, 128, size=(16 * R, ng)) / 128.0) * np.exp2(rng.integers(-12, -3, size=(16 * R, ng)).astype(np.float64)))
    zero = _bf16(rng.standard_normal((16 * R, ng)) * _f32(scale) * 4)
    zero[rng.random((16 * R, ng)) < 0.1] = 0
    packed, qparams = oracle.int4wo_pack(codes, scale, zero, G)
    if one_hot is None:
        x = _bf16(rng.standard_normal(K))
        x[rng.random(K) < 0.05] = 0
    else:
        x = np.zeros(K, np.uint16)
        x[one_hot] = 0x3F80
    t1 = _f32(_bf16((codes - 8).astype(np.float32) * _f32(np.repeat(scale, G, axis=1))))
    wdq = _f32(_bf16(t1 + _f32(np.repeat(zero, G, axis=1))))
    return packed, qparams, x, wdq


def run_wave(G, KB, UT, G0, nt, packed, qparams, x, check=True, lines=None):
    """one wave of int4wo_gemv2_kernel: tiles G0 .. G0 + nt - 1 of the stream of R x KB tiles"""
    R = packed.shape[0]
    depth = int(_define("GEMV2_RING_DEPTH"))
    nseg = (G0 + nt - 1) // UT - G0 // UT + 1
    x_bytes = KB * 256 + 512
    q_bytes = (nt + 2) * 128
    lds = np.zeros(x_bytes + q_bytes + nseg * 256, dtype=np.uint8)
    lds[:KB * 256] = stage_x(x, 0, KB)[:KB * 256]
    q32 = lds[x_bytes: x_bytes + q_bytes].view(np.uint32)
    qflat = qparams.reshape(-1, 16)   # [row block][group] -> global group index
    for t in range(nt):
        for h in range(2):
            g = ((G0 + t) * 128 + 64 * h) // G
            q32[t * 32 + h * 16: t * 32 + h * 16 + 16] = qflat[g]
    red = x_bytes + q_bytes
    wbase = 0x7F0000001000
    w = Wave({wbase: packed.reshape(-1).view(np.uint8)}, lds, check_hazards=check)
    c = lane_constants(G)
    lane = np.arange(64)
    w.v[0], w.v[3], w.v[4], w.v[5] = c["woff"], c["mask"], c["sello"], c["selhi"]
    w.v[1] = (x_bytes + c["qlane"]).astype(np.uint32)
    w.v[2] = (16 * (lane & 3)).astype(np.uint32)
    w.v[6] = (red + 4 * lane).astype(np.uint32)
    w.v[7] = c["inv_f"].astype(np.float32).view(np.uint32)
    w.v[8], w.v[9], w.v[10], w.v[11] = c["bc1"], 0, c["bc2"], 0
    ldi = min(nt - 1, depth - 2)
    wp = wbase + (G0 + ldi) * 1024
    w.s[_sreg("WP")], w.s[_sreg("WP") + 1] = wp & 0xFFFFFFFF, wp >> 32
    w.s[_sreg("LDI")], w.s[_sreg("NTM1")] = ldi, nt - 1
    w.s[_sreg("KTN")], w.s[_sreg("KBX")] = G0 % KB, KB
    w.s[_sreg("UREM")], w.s[_sreg("UT")] = UT - G0 % UT, UT
    flat = packed.reshape(R * KB, 64, 4)
    chunk = (lane & 3) * 16 + (lane >> 2)
    for j in range(depth - 1):
        t = G0 + min(j, nt - 1)
        wreg = int(re.search(r"v\[(\d+):", _define("GEMV2_W%d" % j)).group(1))
        for r in range(4):
            w.valid[wreg + r] = False
        w.vm_pending.append(([wreg + r for r in range(4)], [flat[t][chunk, d].copy() for d in range(4)]))
    w.run(lines if lines is not None else _asm_lines())
    got = lds[red:].view(np.float32).reshape(nseg, 64)
    return got, w


def reference(KB, UT, G0, nt, x, wdq):
    """float64 partial dot products per unit the run touches: [segment][16 rows]"""
    out = []
    u_first, u_last = G0 // UT, (G0 + nt - 1) // UT
    for u in range(u_first, u_last + 1):
        t_lo, t_hi = max(G0, u * UT), min(G0 + nt, (u + 1) * UT)
        rb = t_lo // KB
        k_lo, k_hi = (t_lo - rb * KB) * 128, (t_hi - rb * KB) * 128
        out.append(wdq[16 * rb: 16 * rb + 16, k_lo:k_hi].astype(np.float64) @ _f32(x[k_lo:k_hi]).astype(np.float64))
    return np.array(out)


CASES = [
    # G, KB, UT, rows blocks, G0, nt
    (64, 8, 8, 3, 0, 8),      # exactly one row block
    (64, 8, 8, 3, 5, 7),      # crosses one row-block boundary at a position that is no multiple of the ring depth
    (64, 8, 8, 3, 6, 14),     # two boundaries, ends inside the third row block
    (128, 8, 4, 3, 3, 9),     # K split in two: unit boundaries every 4 tiles, activation wrap every 8
    (256, 8, 4, 2, 4, 4),     # one whole unit that starts in the middle of a row block
    (64, 4, 4, 4, 3, 13),     # run longer than three units
    (64, 32, 32, 2, 28, 14),  # the gate / up launch of Llama-3-8B: 14-tile runs over 32-tile row blocks
    (64, 8, 8, 2, 7, 1),      # single tile that is the last of its unit
    (64, 8, 8, 2, 7, 2),
    (64, 8, 8, 2, 8, 3),
]


@pytest.mark.parametrize("case", CASES)
def test_partial_sums_per_unit(oracle, case):
    G, KB, UT, R, G0, nt = case
    packed, qparams, x, wdq = make_problem(oracle, G, KB, R, seed=hash(case) % 10000)
    got, w = run_wave(G, KB, UT, G0, nt, packed, qparams, x)
    want = reference(KB, UT, G0, nt, x, wdq)
    assert got.shape[0] == want.shape[0]
    scale = np.abs(want).max() + 1e-30
    # every lane of a row holds the row's sum
    for q in range(4):
        assert np.max(np.abs(got[:, q::4].astype(np.float64) - want)) / scale < 2e-6, q
    assert np.array_equal(got[:, 0::4], got[:, 1::4]) and np.array_equal(got[:, 0::4], got[:, 3::4])
    assert not w.lgkm_pending and not w.vm_pending
    assert w.counts.get("global_load_dwordx4", 0) == max(0, nt - (int(_define("GEMV2_RING_DEPTH")) - 1))
    assert w.counts.get("ds_write_b32", 0) == want.shape[0]


def test_one_hot_activation_is_bit_exact_across_a_boundary(oracle):
    G, KB, UT, R, G0, nt = 64, 8, 8, 3, 5, 14
    rng = np.random.default_rng(11)
    for trial in range(6):
        k_hot = int(rng.integers(0, KB * 128))
        packed, qparams, x, wdq = make_problem(oracle, G, KB, R, seed=trial, one_hot=k_hot)
        got, _ = run_wave(G, KB, UT, G0, nt, packed, qparams, x)
        kt = k_hot // 128
        for seg, u in enumerate(range(G0 // UT, (G0 + nt - 1) // UT + 1)):
            t_lo, t_hi = max(G0, u * UT) - u * KB, min(G0 + nt, (u + 1) * UT) - u * KB
            want = wdq[16 * u: 16 * u + 16, k_hot] if t_lo <= kt < t_hi else np.zeros(16, np.float32)
            assert np.array_equal(got[seg, 0::4].view(np.uint32), want.astype(np.float32).view(np.uint32)), (trial, seg)


def test_model_rejects_a_missing_wait(oracle):
    G, KB, UT, R, G0, nt = 64, 8, 8, 2, 2, 9
    packed, qparams, x, _ = make_problem(oracle, G, KB, R, seed=3)
    lines = [ln for ln in _asm_lines() if not ln.startswith("s_waitcnt vmcnt")]
    with pytest.raises(HazardError):
        run_wave(G, KB, UT, G0, nt, packed, qparams, x, lines=lines)
