"""A functional model of one gfx950 wavefront for the handful of instructions the generated int4 GEMV loop uses.

Test infrastructure: it executes the text of GEMV1_LOOP_ASM (ao_amd/csrc/int4wo_gemv1_loop.inc) on numpy arrays so
that the schedule can be checked without a GPU:
  * values: every instruction is evaluated for 64 lanes (the 4x4x4 matrix instructions per 4-lane block);
  * memory ordering: a load's destination registers are poisoned until an s_waitcnt retires it (loads retire in
    order), and reading a poisoned register is an error;
  * dependency distances the hardware does not interlock: a VALU result may feed a matrix instruction or a DPP read
    no sooner than 2 issue slots later, a 2-pass matrix result may be read or overwritten no sooner than 5 slots later.
"""
import re

import numpy as np

NLANES = 64


def _bf16_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def _f32_to_bf16(x):
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint32)


def _f16_to_f64(bits):
    return bits.astype(np.uint16).view(np.float16).astype(np.float64)


class HazardError(AssertionError):
    pass


class Wave:
    def __init__(self, global_mem, lds, check_hazards=True):
        self.v = np.zeros((256, NLANES), dtype=np.uint32)
        self.valid = np.ones(256, dtype=bool)
        self.s = np.zeros(128, dtype=np.uint64)
        self.scc = 0
        self.mem = global_mem          # dict base_address -> np.uint8 array ; addresses resolved by range
        self.lds = lds                 # np.uint8 array
        self.vm_pending = []           # [(regs, values)] in issue order
        self.lgkm_pending = []
        self.slot = 0
        self.last_write = {}           # vgpr -> (slot, kind)
        self.check = check_hazards
        self.executed = 0
        self.counts = {}

    # ------------------------------------------------------------------ operand helpers
    def _regs(self, tok):
        m = re.fullmatch(r"v\[(\d+):(\d+)\]", tok)
        if m:
            return list(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.fullmatch(r"v(\d+)", tok)
        if m:
            return [int(m.group(1))]
        raise ValueError("not a vgpr operand: " + tok)

    def _sregs(self, tok):
        m = re.fullmatch(r"s\[(\d+):(\d+)\]", tok)
        if m:
            return list(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.fullmatch(r"s(\d+)", tok)
        if m:
            return [int(m.group(1))]
        raise ValueError("not an sgpr operand: " + tok)

    def _read_v(self, reg, reader):
        if not self.valid[reg]:
            raise HazardError("v%d read while a load into it is outstanding (%s)" % (reg, reader))
        if self.check and reg in self.last_write:
            wslot, wkind = self.last_write[reg]
            dist = self.slot - wslot
            if wkind == "mfma" and dist < 6:
                raise HazardError("v%d: matrix result read %d slots after issue by %s" % (reg, dist, reader))
            if wkind == "valu" and reader in ("mfma", "dpp") and dist < 3:
                raise HazardError("v%d: VALU result read %d slots later by %s" % (reg, dist, reader))
        return self.v[reg]

    def _write_v(self, reg, val, kind):
        if not self.valid[reg]:
            raise HazardError("v%d written while a load into it is outstanding" % reg)
        if self.check and reg in self.last_write:
            wslot, wkind = self.last_write[reg]
            if wkind == "mfma" and self.slot - wslot < 6:
                raise HazardError("v%d overwritten %d slots after a matrix instruction wrote it" % (reg, self.slot - wslot))
        self.v[reg] = val
        self.last_write[reg] = (self.slot, kind)

    def _src(self, tok, reader="valu"):
        """vector-instruction source: vgpr, sgpr, or literal -> uint32[64]"""
        tok = tok.strip()
        if tok.startswith("v"):
            return self._read_v(self._regs(tok)[0], reader)
        if tok.startswith("s"):
            return np.full(NLANES, np.uint32(self.s[self._sregs(tok)[0]] & 0xFFFFFFFF))
        return np.full(NLANES, np.uint32(int(tok, 0) & 0xFFFFFFFF))

    def _ssrc(self, tok):
        tok = tok.strip()
        if tok.startswith("s"):
            return int(self.s[self._sregs(tok)[0]]) & 0xFFFFFFFF
        return int(tok, 0) & 0xFFFFFFFF

    def _load_bytes(self, addr, n):
        for base, arr in self.mem.items():
            if base <= addr and addr + n <= base + arr.size:
                return arr[addr - base: addr - base + n]
        raise HazardError("global load outside every buffer: 0x%x + %d" % (addr, n))

    # ------------------------------------------------------------------ execution
    def run(self, lines, max_instr=2_000_000):
        labels = {}
        prog = []
        for ln in lines:
            ln = ln.strip()
            if not ln:
                continue
            m = re.fullmatch(r"(\d+):", ln)
            if m:
                labels.setdefault(m.group(1), []).append(len(prog))
                continue
            prog.append(ln)
        pc = 0
        while pc < len(prog):
            self.executed += 1
            if self.executed > max_instr:
                raise RuntimeError("instruction budget exceeded")
            ins = prog[pc]
            op, _, rest = ins.partition(" ")
            self.counts[op] = self.counts.get(op, 0) + 1
            nxt = pc + 1
            if op in ("s_branch", "s_cbranch_scc1", "s_cbranch_scc0"):
                take = op == "s_branch" or (op == "s_cbranch_scc1" and self.scc) or (op == "s_cbranch_scc0" and not self.scc)
                if take:
                    lab, direction = rest.strip()[:-1], rest.strip()[-1]
                    cands = labels[lab]
                    if direction == "f":
                        nxt = min(c for c in cands if c > pc)
                    else:
                        nxt = max(c for c in cands if c <= pc)
                self.slot += 1
            else:
                self._exec(op, rest)
            pc = nxt

    def _exec(self, op, rest):
        args = [a.strip() for a in self._split(rest)]
        slots = 1
        if op == "s_nop":
            slots = int(args[0], 0) + 1
        elif op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", rest)
            if m:
                self._retire(self.vm_pending, int(m.group(1)))
            m = re.search(r"lgkmcnt\((\d+)\)", rest)
            if m:
                self._retire(self.lgkm_pending, int(m.group(1)))
        elif op.startswith("s_"):
            self._salu(op, args)
        elif op.startswith("v_mfma"):
            self._mfma(op, args)
        elif op.startswith("global_load"):
            self._gload(op, args)
        elif op.startswith("ds_read"):
            self._dsread(op, args)
        elif op == "ds_write_b32":
            addr = self._src(args[0]).astype(np.int64)
            data = self._src(args[1])
            for lane in range(NLANES):
                ad = int(addr[lane])
                if ad < 0 or ad + 4 > self.lds.size:
                    raise HazardError("ds_write outside the LDS image: %d" % ad)
                self.lds[ad: ad + 4] = np.frombuffer(np.uint32(data[lane]).tobytes(), dtype=np.uint8)
            self.lgkm_pending.append(([], []))
        elif op.startswith("v_"):
            self._valu(op, args, rest)
        else:
            raise ValueError("unknown instruction: " + op)
        self.slot += slots

    @staticmethod
    def _split(rest):
        out, depth, cur = [], 0, ""
        for ch in rest:
            if ch == "[":
                depth += 1
            if ch == "]":
                depth -= 1
            if ch == "," and depth == 0:
                out.append(cur)
                cur = ""
            else:
                cur += ch
        if cur.strip():
            out.append(cur)
        return out

    def _retire(self, queue, keep):
        while len(queue) > keep:
            regs, vals = queue.pop(0)
            for r, val in zip(regs, vals):
                self.valid[r] = True
                self.v[r] = val
                self.last_write[r] = (self.slot, "mem")

    def _salu(self, op, a):
        M = 0xFFFFFFFF
        if op == "s_mov_b32":
            self.s[self._sregs(a[0])[0]] = self._ssrc(a[1])
        elif op == "s_add_u32":
            r = self._ssrc(a[1]) + self._ssrc(a[2])
            self.scc = int(r > M)
            self.s[self._sregs(a[0])[0]] = r & M
        elif op == "s_addc_u32":
            r = self._ssrc(a[1]) + self._ssrc(a[2]) + self.scc
            self.scc = int(r > M)
            self.s[self._sregs(a[0])[0]] = r & M
        elif op == "s_sub_u32":
            x, y = self._ssrc(a[1]), self._ssrc(a[2])
            self.scc = int(y > x)
            self.s[self._sregs(a[0])[0]] = (x - y) & M
        elif op == "s_min_u32":
            x, y = self._ssrc(a[1]), self._ssrc(a[2])
            self.scc = int(x <= y)
            self.s[self._sregs(a[0])[0]] = min(x, y)
        elif op == "s_lshl_b32":
            r = (self._ssrc(a[1]) << (self._ssrc(a[2]) & 31)) & M
            self.scc = int(r != 0)
            self.s[self._sregs(a[0])[0]] = r
        elif op == "s_lshr_b32":
            r = self._ssrc(a[1]) >> (self._ssrc(a[2]) & 31)
            self.scc = int(r != 0)
            self.s[self._sregs(a[0])[0]] = r
        elif op == "s_cmp_lt_u32":
            self.scc = int(self._ssrc(a[0]) < self._ssrc(a[1]))
        elif op == "s_cmp_eq_u32":
            self.scc = int(self._ssrc(a[0]) == self._ssrc(a[1]))
        elif op == "s_cselect_b32":
            self.s[self._sregs(a[0])[0]] = self._ssrc(a[1]) if self.scc else self._ssrc(a[2])
        else:
            raise ValueError("unknown SALU instruction: " + op)

    def _valu(self, op, a, rest):
        d = self._regs(a[0])[0]
        if op == "v_mov_b32":
            r = self._src(a[1]).copy()
        elif op == "v_and_b32":
            r = self._src(a[1]) & self._src(a[2])
        elif op == "v_and_b32_dpp":
            last = a[2].split()
            m = re.search(r"quad_perm:\[(\d),(\d),(\d),(\d)\]", rest)
            perm = [int(m.group(i)) for i in range(1, 5)]
            src0 = self._src(a[1], "dpp")
            lanes = np.arange(NLANES)
            sel = (lanes & ~3) + np.array(perm)[lanes & 3]
            r = src0[sel] & self._src(last[0])
        elif op == "v_lshrrev_b32":
            r = self._src(a[2]) >> (self._src(a[1]) & 31)
        elif op == "v_lshl_or_b32":
            r = (self._src(a[1]) << (self._src(a[2]) & 31)) | self._src(a[3])
        elif op == "v_add_u32":
            r = self._src(a[1]) + self._src(a[2])
        elif op == "v_lshl_add_u32":
            r = (self._src(a[1]) << (self._src(a[2]) & 31)) + self._src(a[3])
        elif op == "v_cndmask_b32":
            sr = self._sregs(a[3])
            m = int(self.s[sr[0]]) | (int(self.s[sr[1]]) << 32)
            bits = np.array([(m >> i) & 1 for i in range(NLANES)], dtype=bool)
            r = np.where(bits, self._src(a[2]), self._src(a[1]))
        elif op == "v_mul_f32":
            r = (self._src(a[1]).view(np.float32) * self._src(a[2]).view(np.float32)).astype(np.float32).view(np.uint32)
        elif op == "v_add_f32_dpp":
            last = a[2].split()
            m = re.search(r"quad_perm:\[(\d),(\d),(\d),(\d)\]", rest)
            perm = [int(m.group(i)) for i in range(1, 5)]
            src0 = self._src(a[1], "dpp")
            lanes = np.arange(NLANES)
            sel = (lanes & ~3) + np.array(perm)[lanes & 3]
            r = (src0[sel].view(np.float32) + self._src(last[0]).view(np.float32)).astype(np.float32).view(np.uint32)
        elif op == "v_perm_b32":
            s0, s1, sel = self._src(a[1]), self._src(a[2]), self._src(a[3])
            pool = (s0.astype(np.uint64) << 32) | s1.astype(np.uint64)
            r = np.zeros(NLANES, dtype=np.uint32)
            for i in range(4):
                sb = (sel >> (8 * i)) & 0xFF
                byte = np.where(sb < 8, (pool >> (8 * np.minimum(sb, 7).astype(np.uint64))) & 0xFF, 0)
                byte = np.where(sb >= 13, 0xFF, byte)
                if np.any((sb >= 8) & (sb < 12)):
                    raise ValueError("v_perm_b32 sign selectors are not modelled")
                r |= (byte.astype(np.uint32) << (8 * i))
        elif op == "v_cvt_pk_bf16_f32":
            lo = _f32_to_bf16(self._src(a[1]).view(np.float32))
            hi = _f32_to_bf16(self._src(a[2]).view(np.float32))
            r = (lo | (hi << 16)).astype(np.uint32)
        else:
            raise ValueError("unknown VALU instruction: " + op)
        self._write_v(d, r.astype(np.uint32), "valu")

    def _halves(self, regs, reader, f16):
        vals = []
        for r in regs:
            w = self._read_v(r, reader)
            vals.append(w & 0xFFFF)
            vals.append(w >> 16)
        k = np.stack(vals, axis=0)  # [4][64]
        if f16:
            return _f16_to_f64(k.astype(np.uint16))
        return _bf16_to_f32(k).astype(np.float64)

    def _mfma(self, op, a):
        f16 = op.endswith("_f16")
        dst = self._regs(a[0])
        A = self._halves(self._regs(a[1]), "mfma", f16)  # [k][lane]
        B = self._halves(self._regs(a[2]), "mfma", f16)
        if a[3].strip() == "0":
            C = np.zeros((4, NLANES))
        else:
            C = np.stack([self._read_v(r, "mfma").view(np.float32).astype(np.float64) for r in self._regs(a[3])], axis=0)
        out = np.zeros((4, NLANES))
        lanes = np.arange(NLANES)
        blk = lanes & ~3
        for i in range(4):
            acc = C[i].copy()
            for k in range(4):
                acc = acc + A[k][blk + i] * B[k][lanes]
            out[i] = acc
        with np.errstate(over="ignore", invalid="ignore"):
            res = out.astype(np.float32)
        for i, r in enumerate(dst):
            self._write_v(r, res[i].view(np.uint32), "mfma")

    def _gload(self, op, a):
        n = 16 if op.endswith("x4") else 4
        dst = self._regs(a[0])
        voff = self._src(a[1])
        sb = self._sregs(a[2].split()[0])
        base = int(self.s[sb[0]]) | (int(self.s[sb[1]]) << 32)
        vals = np.zeros((len(dst), NLANES), dtype=np.uint32)
        for lane in range(NLANES):
            raw = self._load_bytes(base + int(voff[lane]), n)
            vals[:, lane] = np.frombuffer(raw.tobytes(), dtype=np.uint32)
        for r in dst:
            if not self.valid[r]:
                raise HazardError("load into v%d while an older load into it is outstanding" % r)
            self.valid[r] = False
        self.vm_pending.append((dst, list(vals)))

    def _dsread(self, op, a):
        dst = self._regs(a[0])
        m = re.match(r"(v\d+)\s+offset:(\d+)", a[1])
        addr = self._src(m.group(1)).astype(np.int64) + int(m.group(2))
        nb = 4 * len(dst)
        vals = np.zeros((len(dst), NLANES), dtype=np.uint32)
        for lane in range(NLANES):
            ad = int(addr[lane])
            raw = np.zeros(nb, dtype=np.uint8)
            if ad + nb <= self.lds.size:
                raw = self.lds[ad: ad + nb]
            vals[:, lane] = np.frombuffer(raw.tobytes(), dtype=np.uint32)
        for r in dst:
            if self.check and r in self.last_write and self.last_write[r][1] == "mfma" and self.slot - self.last_write[r][0] < 6:
                raise HazardError("ds_read into v%d right after a matrix write" % r)
            self.valid[r] = False
        self.lgkm_pending.append((dst, list(vals)))
