"""CPU checks of the generated tile loop of the single-row int4 GEMV (ao_amd/csrc/int4wo_gemv1_loop.inc).

The loop is one block of hand-scheduled gfx950 assembly.  Here its text is executed by a small wavefront model
(tests/_gemv1_sim.py) against packed weights made by the oracle: the accumulated dot products must equal
x . dequantize_affine(W) computed in float64 from the doubly rounded weights, no register may be read before the wait
that covers its load, and every dependency distance the hardware leaves to software must hold on the executed path.
"""
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from _gemv1_sim import HazardError, Wave

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ao_amd", "csrc")
INC = os.path.join(CSRC, "int4wo_gemv1_loop.inc")
GEN = os.path.join(CSRC, "gen_int4wo_gemv1.py")

# physical registers the test hands the asm operands to (all below the block's own range)
VIN = {"woff": "v0", "qaddr": "v1", "xaddr": "v2", "mask": "v3", "sello": "v4", "selhi": "v5", "bc1": "v[8:9]", "bc2": "v[10:11]"}
SIN = {}


def _asm_lines():
    text = open(INC).read()
    body = text.split("#define GEMV1_LOOP_ASM", 1)[1]
    lines = re.findall(r'"((?:[^"\\]|\\.)*)"', body)
    out = []
    for ln in lines:
        ln = ln.replace("\\n", "").replace("\\t", "").strip()
        if not ln:
            continue
        for k, val in {**VIN, **SIN}.items():
            ln = ln.replace("%%[%s]" % k, val)
        assert "%[" not in ln, ln
        out.append(ln)
    return out


def _define(name):
    m = re.search(r"#define %s (.+)" % name, open(INC).read())
    return m.group(1).strip()


def test_include_file_is_what_the_generator_prints():
    out = subprocess.run([sys.executable, GEN], capture_output=True, text=True, check=True).stdout
    assert out == open(INC).read()


def _bf16(x):
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)


def _f32(bits):
    return (np.asarray(bits).astype(np.uint32) << 16).view(np.float32)


def lane_constants(G):
    """what int4wo_gemv1_kernel hands the loop, per lane"""
    lane = np.arange(64)
    b, i = lane >> 2, lane & 3
    hi = i >= 2
    c = {}
    c["woff"] = (16 * (b + 16 * i)).astype(np.uint32)
    c["qlane"] = (4 * (b + 16 * (i >> 1))).astype(np.uint32)   # byte of the lane's word inside a tile's 128 qparam bytes
    c["mask"] = np.where(hi, 0x00F000F0, 0x000F000F).astype(np.uint32)
    low, high, none = 0x0C0C0100, 0x01000C0C, 0x0C0C0C0C
    c["sello"] = np.select([i == 0, i == 1], [low, high], none).astype(np.uint32)
    c["selhi"] = np.select([i == 2, i == 3], [low, high], none).astype(np.uint32)
    c["bc1"] = np.where(hi, 0x8080, 0x8008).astype(np.uint32)   # -8 * 2^-20 / -8 * 2^-24 as fp16 subnormals
    c["bc2"] = np.where(hi, 0x35800000, 0x33800000).astype(np.uint32)  # 2^-20 / 2^-24 as bf16 in the upper half
    c["inv_f"] = np.where(hi, 2.0 ** 20, 2.0 ** 24)
    return c


def _sreg(name):
    return int(re.search(r"s\[?(\d+)", _define("GEMV1_S_" + name)).group(1))


def prepare_wave(w, G, kb0, nt, wbase, packed, q_lds_base):
    """registers as int4wo_gemv1_kernel leaves them when it enters the loop: lane constants, scalar state and the
    requests for tiles 0 .. D-2 of the run (the last tile again when the run is shorter) still in flight"""
    c = lane_constants(G)
    w.v[0], w.v[3], w.v[4], w.v[5] = c["woff"], c["mask"], c["sello"], c["selhi"]
    w.v[1] = (q_lds_base + c["qlane"]).astype(np.uint32)
    w.v[2] = (16 * (np.arange(64) & 3)).astype(np.uint32)
    w.v[8], w.v[9], w.v[10], w.v[11] = c["bc1"], 0, c["bc2"], 0
    depth = int(_define("GEMV1_RING_DEPTH"))
    ldi = min(nt - 1, depth - 2)
    wp = wbase + (kb0 + ldi) * 1024
    w.s[_sreg("WP")], w.s[_sreg("WP") + 1] = wp & 0xFFFFFFFF, wp >> 32
    w.s[_sreg("LDI")], w.s[_sreg("NTM1")] = ldi, nt - 1
    lane = np.arange(64)
    chunk = (lane & 3) * 16 + (lane >> 2)
    for j in range(depth - 1):
        t = kb0 + min(j, nt - 1)
        wreg = int(re.search(r"v\[(\d+):", _define("GEMV1_W%d" % j)).group(1))
        for r in range(4):
            w.valid[wreg + r] = False
        w.vm_pending.append(([wreg + r for r in range(4)], [packed[0, t][chunk, d].copy() for d in range(4)]))
    return c


def stage(x_bits, qparams, G, kb_first, ntiles):
    """LDS image of one wave: the activations of its run in the order the lanes consume them, then the run's
    (scale, zero) words, 128 bytes per tile as [k half][row] (see int4wo_gemv1_kernel); returns (image, byte of the
    qparam part)"""
    xbytes = (ntiles + 2) * 256
    lds = np.zeros(xbytes + (ntiles + 2) * 128, dtype=np.uint8)
    lds[:ntiles * 256] = stage_x(x_bits, kb_first, ntiles)[:ntiles * 256]
    q32 = lds[xbytes:].view(np.uint32)
    for t in range(ntiles):
        for h in range(2):
            g = ((kb_first + t) * 128 + 64 * h) // G
            q32[t * 32 + h * 16: t * 32 + h * 16 + 16] = qparams[0, g, :]
    return lds, xbytes


def stage_x(x_bits, kb_first, ntiles):
    """activation row -> LDS image in the order the lanes consume it (see int4wo_gemv1_kernel)"""
    lds = np.zeros(ntiles * 256 + 512, dtype=np.uint8)
    v16 = lds[: ntiles * 256].view(np.uint16)
    for t in range(ntiles):
        kb = kb_first + t
        for kq in range(4):
            for sl in range(4):
                k0 = 128 * kb + 32 * kq + 8 * sl
                for c in range(4):
                    j = (kq % 2) + 2 * (c % 2)
                    step = 2 * sl + c // 2
                    byte = t * 256 + (step // 2) * 64 + j * 16 + (step % 2) * 8 + (kq // 2) * 4
                    v16[byte // 2] = x_bits[k0 + 2 * c]
                    v16[byte // 2 + 1] = x_bits[k0 + 2 * c + 1]
    return lds


def run_wave(oracle, G, KB, kb0, nt, seed, scale_exp=(-12, -4), check=True):
    rng = np.random.default_rng(seed)
    K = KB * 128
    codes = rng.integers(0, 16, size=(16, K)).astype(np.int32)
    ng = K // G
    sexp = rng.integers(scale_exp[0], scale_exp[1] + 1, size=(16, ng))
    scale = _bf16((1.0 + rng.integers(0, 128, size=(16, ng)) / 128.0) * np.exp2(sexp.astype(np.float64)))
    zero = _bf16(rng.standard_normal((16, ng)) * _f32(scale) * 4)
    zero[rng.random((16, ng)) < 0.1] = 0
    packed, qparams = oracle.int4wo_pack(codes, scale, zero, G)
    x = _bf16(rng.standard_normal(K))
    x[rng.random(K) < 0.05] = 0

    wbase = 0x7F0000001000
    mem = {wbase: packed.reshape(-1).view(np.uint8)}
    lds, qoff = stage(x, qparams, G, kb0, nt)
    w = Wave(mem, lds, check_hazards=check)
    c = prepare_wave(w, G, kb0, nt, wbase, packed, qoff)

    w.run(_asm_lines())
    acc_reg = int(re.search(r"v\[(\d+):", _define("GEMV1_ACC")).group(1))
    lane = np.arange(64)
    part = w.v[acc_reg + (lane & 3), lane].view(np.float32).astype(np.float64) * c["inv_f"]
    got = part.reshape(16, 4).sum(axis=1)

    # reference: doubly rounded dequantize_affine, float64 dot product over the wave's K range
    ks = np.arange(kb0 * 128, (kb0 + nt) * 128)
    s_el = _f32(np.repeat(scale, G, axis=1)[:, ks]).astype(np.float32)
    z_el = _f32(np.repeat(zero, G, axis=1)[:, ks]).astype(np.float32)
    t1 = _f32(_bf16((codes[:, ks] - 8).astype(np.float32) * s_el))
    wdq = _f32(_bf16(t1 + z_el)).astype(np.float64)
    want = wdq @ _f32(x[ks]).astype(np.float64)
    return got, want, w


@pytest.mark.parametrize("G", [64, 128, 256])
@pytest.mark.parametrize("nt", [1, 2, 3, 5, 6, 7, 8, 13])
def test_loop_values_waits_and_distances(oracle, G, nt):
    KB = 16
    kb0 = 2 if nt <= 13 else 0
    got, want, w = run_wave(oracle, G, KB, kb0, nt, seed=100 * nt + G)
    scale = np.abs(want).max() + 1e-30
    assert np.max(np.abs(got - want)) / scale < 2e-6
    # nothing is left in flight and no tile was requested twice
    assert not w.lgkm_pending and not w.vm_pending
    assert w.counts.get("global_load_dwordx4", 0) == max(0, nt - (int(_define("GEMV1_RING_DEPTH")) - 1))


def test_one_hot_activation_is_bit_exact(oracle):
    # a single 1.0 in x picks one dequantized weight per row: the loop must return exactly that bf16 value
    G, KB, nt, kb0 = 64, 8, 8, 0
    rng = np.random.default_rng(7)
    for trial in range(6):
        K = KB * 128
        codes = rng.integers(0, 16, size=(16, K)).astype(np.int32)
        ng = K // G
        scale = _bf16((1.0 + rng.integers(0, 128, size=(16, ng)) / 128.0) * np.exp2(rng.integers(-20, 3, size=(16, ng)).astype(np.float64)))
        zero = _bf16(rng.standard_normal((16, ng)) * _f32(scale) * 3)
        packed, qparams = oracle.int4wo_pack(codes, scale, zero, G)
        k_hot = int(rng.integers(0, K))
        x = np.zeros(K, np.uint16)
        x[k_hot] = 0x3F80
        mem = {0x1000: packed.reshape(-1).view(np.uint8)}
        lds, qoff = stage(x, qparams, G, kb0, nt)
        w = Wave(mem, lds)
        c = prepare_wave(w, G, kb0, nt, 0x1000, packed, qoff)
        w.run(_asm_lines())
        acc_reg = int(re.search(r"v\[(\d+):", _define("GEMV1_ACC")).group(1))
        lane = np.arange(64)
        part = w.v[acc_reg + (lane & 3), lane].view(np.float32) * c["inv_f"].astype(np.float32)
        got = part.reshape(16, 4).sum(axis=1, dtype=np.float32)
        g_hot = k_hot // G
        t1 = _f32(_bf16((codes[:, k_hot] - 8).astype(np.float32) * _f32(scale[:, g_hot])))
        want = _f32(_bf16(t1 + _f32(zero[:, g_hot])))
        assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32)), (trial, k_hot)


def test_model_rejects_a_missing_wait():
    # the checker itself: a schedule that drops the waits must be refused
    lines = [ln for ln in _asm_lines() if not ln.startswith("s_waitcnt vmcnt")]
    import oracle as O

    O.lib()
    rng = np.random.default_rng(1)
    codes = rng.integers(0, 16, size=(16, 1024)).astype(np.int32)
    scale = np.full((16, 16), 0x3C00, np.uint16)
    zero = np.zeros((16, 16), np.uint16)
    packed, qparams = O.int4wo_pack(codes, scale, zero, 64)
    lds, qoff = stage(np.zeros(1024, np.uint16), qparams, 64, 0, 4)
    w = Wave({0x1000: packed.reshape(-1).view(np.uint8)}, lds)
    prepare_wave(w, 64, 0, 4, 0x1000, packed, qoff)
    with pytest.raises(HazardError):
        w.run(lines)
