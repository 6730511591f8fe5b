"""A functional model of a gfx9-family wave, enough to run this library's compiled kernels on the CPU.

What it is for: a hand-written kernel that reads or writes out of bounds, or uses a register before a wait has made its
contents valid, faults or silently corrupts on the GPU, where the only evidence is a dead process.  The model runs the
assembly text that `hipcc -S --cuda-device-only` emits for a kernel, workgroup by workgroup and wave by wave, and makes such
mistakes visible and attributable:

* every global access is checked against the list of regions the test registered (`Memory`); a violation raises `Fault`
  naming wave, source line and instruction;
* memory instructions complete late: a load's destination holds a poison value until a wait (`s_waitcnt`) or a latency
  in instructions has passed, so a missing or too-weak wait changes the result;
* registers and LDS start out as garbage (`GARBAGE`), as on the device;
* the waves of a workgroup are interleaved at random (seeded) and meet at `s_barrier` as the hardware's barrier does: it
  counts arrivals, whichever barrier instruction a wave is at;
* optionally, the wait-state rules between dependent instructions that the hardware does not interlock (`HAZARDS`), and
  executed-instruction counts by source line (`COUNTS`).

Only the instructions that the compiled kernels use are modelled; an unknown one raises `Fault("instruction not
modelled")`.  Timing is not modelled at all.  `Kernel` reads a kernel's descriptor and argument layout from the same
assembly file and launches it the way the runtime does (kernarg segment, workgroup ids, lane ids)."""
import functools
import os
import random
import re
import struct
import tempfile

import numpy as np

U32 = np.uint32
MASK64 = (1 << 64) - 1


class Fault(Exception):
    pass


@functools.lru_cache(maxsize=None)
def _reg_index(kind, tok):
    """(first register, count) of `v7`, `s[4:5]`, ...; (None, 0) for anything else"""
    m = re.match(r"^%s(\d+)$" % kind, tok)
    if m:
        return int(m.group(1)), 1
    m = re.match(r"^%s\[(\d+):(\d+)\]$" % kind, tok)
    if m:
        return int(m.group(1)), int(m.group(2)) - int(m.group(1)) + 1
    return None, 0


@functools.lru_cache(maxsize=4096)
def _lanes_of(exec_mask):
    out = np.array([(exec_mask >> k) & 1 for k in range(64)], dtype=bool)
    out.flags.writeable = False
    return out


class Memory:
    def __init__(self):
        self.regions = []          # (base, np.uint8 array, name)

    def add(self, base, data, name):
        self.regions.append((base, data, name))

    def find(self, addr, size):
        for base, data, name in self.regions:
            if base <= addr and addr + size <= base + len(data):
                return data, addr - base
        return None, None

    def read(self, addr, size, who):
        data, off = self.find(addr, size)
        if data is None:
            raise Fault(f"read of {size} bytes at {addr:#x} outside every region ({who})")
        return bytes(data[off:off + size])

    def write(self, addr, payload, who):
        data, off = self.find(addr, len(payload))
        if data is None:
            raise Fault(f"write of {len(payload)} bytes at {addr:#x} outside every region ({who})")
        data[off:off + len(payload)] = np.frombuffer(payload, dtype=np.uint8)


ASM_LINES = set()


E32_ALIASES = {"v_cndmask_b32", "v_add_f32", "v_add_u32", "v_mov_b32", "v_and_b32", "v_or_b32", "v_xor_b32", "v_cvt_f16_f32", "v_sub_u32",
               "v_mul_f32", "v_lshlrev_b32", "v_lshrrev_b32"}


INT_E64_AS_E32 = {"v_add_u32", "v_sub_u32", "v_subrev_u32", "v_and_b32", "v_or_b32", "v_xor_b32", "v_lshlrev_b32", "v_lshrrev_b32",
                  "v_ashrrev_i32", "v_min_u32", "v_max_u32", "v_mul_u32_u24", "v_mul_i32_i24"}


def _arith(text):
    """`3-1`, `1*128+14+1`, `0*16384+256`, `v[96+8*1+2*3:96+8*1+2*3+1]`: constant expressions the assembler folds
    (hand-written blocks use them for offsets and register numbers that depend on a macro parameter).  Anything else is
    returned as it is."""
    m = re.fullmatch(r"([vsa])\[([0-9+* -]+):([0-9+* -]+)\]", text)
    if m:
        return "%s[%d:%d]" % (m.group(1), eval(m.group(2), {"__builtins__": {}}, {}), eval(m.group(3), {"__builtins__": {}}, {}))
    if re.fullmatch(r"[0-9a-fA-Fx+*() -]+", text) and re.search(r"[+*-]", text.lstrip("-")) and not re.fullmatch(r"-?(0x)?[0-9a-fA-F]+", text):
        return str(eval(text, {"__builtins__": {}}, {}))
    return text


def parse(path):
    insts, labels = [], {}
    local_defs = {}          # numeric local labels ("10:"): number -> instruction indices where it is defined
    in_asm = False
    for ln, raw in enumerate(open(path).read().split("\n"), 1):
        if "#ASMSTART" in raw:
            in_asm = True
        elif "#ASMEND" in raw:
            in_asm = False
        elif in_asm:
            ASM_LINES.add(ln)
        t = raw.split(";")[0].rstrip() if not raw.strip().startswith(";;#") else ""
        t = t.strip()
        if not t or t.startswith(".p2align") or t.startswith(".") and not t.startswith(".LBB"):
            continue
        m = re.match(r"^([.\w$]+):", t)
        if m:
            if m.group(1).isdigit():
                local_defs.setdefault(m.group(1), []).append(len(insts))
            else:
                labels[m.group(1)] = len(insts)
            continue
        parts = t.split(None, 1)
        op = parts[0]
        if op in E32_ALIASES:                # hand-written blocks name the 32-bit encodings without their suffix
            op += "_e32"
        if op.endswith("_e64") and op[:-4] in INT_E64_AS_E32:      # the long encoding of an integer op: other operand kinds, same result
            op = op[:-4] + "_e32"
        rest = parts[1] if len(parts) > 1 else ""
        # split operands from modifiers
        ops, mods = [], {}
        toks = [x.strip() for x in re.split(r",(?![^\[]*\])", rest)] if rest else []
        # the last operand may carry modifiers separated by spaces
        flat = []
        for tk in toks:
            sub = tk.split()
            if not sub:
                continue
            flat.append(_arith(sub[0]))
            for s in sub[1:]:
                if ":" in s:
                    k, v = s.split(":", 1)
                    mods[k] = _arith(v)
                else:
                    mods[s] = True
        insts.append((op, flat, mods, ln, t))
    # references to numeric local labels: "10b" is the nearest definition at or before the instruction, "10f" the nearest after
    for i, (op, flat, mods, ln, t) in enumerate(insts):
        if (op == "s_branch" or op.startswith("s_cbranch")) and flat and re.fullmatch(r"\d+[bf]", flat[0]):
            num, way = flat[0][:-1], flat[0][-1]
            defs = local_defs.get(num, [])
            cands = [d for d in defs if d <= i] if way == "b" else [d for d in defs if d > i]
            if not cands:
                raise Fault(f"line {ln}: no local label for {flat[0]}")
            target = max(cands) if way == "b" else min(cands)
            name = f".Llocal_{num}_{target}"
            labels[name] = target
            insts[i] = (op, [name] + flat[1:], mods, ln, t)
    return insts, labels


INLINE_FLOAT = {"0.5": 0x3F000000, "-0.5": 0xBF000000, "1.0": 0x3F800000, "-1.0": 0xBF800000, "2.0": 0x40000000,
                "-2.0": 0xC0000000, "4.0": 0x40800000, "-4.0": 0xC0800000}


def f32(a):
    return a.view(np.float32)


def f16_bits(a):
    """float array -> fp16 bit patterns in uint32 (round to nearest even; garbage lanes may overflow: no warnings)"""
    with np.errstate(all="ignore"):
        return np.asarray(a).astype(np.float16).view(np.uint16).astype(U32)


def as_u32(a):
    return np.asarray(a, dtype=np.float32).view(U32)


GARBAGE = False
COUNTS = None           # set to a dict to count executed instructions by source line
HAZARDS = None          # set to a dict to collect wait-state hazards: (rule, producer line, consumer line) -> count


def _regs(tok, letter):
    out = set()
    for a, b in re.findall(r"\b%s\[(\d+):(\d+)\]" % letter, tok):
        out.update(range(int(a), int(b) + 1))
    for a in re.findall(r"\b%s(\d+)\b" % letter, tok):
        out.add(int(a))
    return out


VCC_LO, VCC_HI, EXEC_LO, EXEC_HI, M0_REG = 106, 107, 126, 127, 124
TRANS = ("v_exp_", "v_log_", "v_rcp_", "v_rsq_", "v_sqrt_", "v_sin_", "v_cos_")
INFO_CACHE = {}


def inst_info(inst):
    op, o, mods, ln, text = inst
    key = (ln, text)
    if key in INFO_CACHE:
        return INFO_CACHE[key]
    def sregs(tok):
        r = _regs(tok, "s")
        if re.search(r"\bvcc\b|\bvcc_lo\b", tok): r |= {VCC_LO, VCC_HI}
        if re.search(r"\bexec\b", tok): r |= {EXEC_LO, EXEC_HI}
        if re.search(r"\bm0\b", tok): r.add(M0_REG)
        return r
    kind = "other"
    if op.startswith("v_"): kind = "valu"
    elif re.match(r"(global|buffer|flat|scratch)_", op): kind = "vmem"
    elif op.startswith("ds_"): kind = "lds"
    elif re.match(r"s_(load|buffer_load|store|atomic|dcache)", op): kind = "smem"
    elif op.startswith("s_") and not re.match(r"s_(nop|waitcnt|branch|cbranch|barrier|endpgm|sleep|setprio)", op): kind = "salu"
    sdef, vdef, suse, vuse = set(), set(), set(), set()
    if kind == "valu":
        ndst = 1
        if re.match(r"v_(add|sub|subrev)_co_|v_(addc|subb|subbrev)_co_|v_mad_[ui]64_[ui]32|v_div_scale", op): ndst = 2
        if op.startswith("v_cmp") and op.endswith("_e32"):
            ndst = 0; sdef |= {VCC_LO, VCC_HI}
        if op.startswith("v_cmpx"): sdef |= {EXEC_LO, EXEC_HI}
        for t in o[:ndst]:
            sdef |= sregs(t); vdef |= _regs(t, "v")
        for t in o[ndst:]:
            suse |= sregs(t); vuse |= _regs(t, "v")
        if op.endswith("_e32") and re.match(r"v_(cndmask|addc_co|subb_co|subbrev_co)", op) and len(o) == 3:
            suse |= {VCC_LO, VCC_HI}
        if op.startswith("v_div_fmas"): suse |= {VCC_LO, VCC_HI}
    elif kind == "salu":
        if o:
            sdef |= sregs(o[0])
        for t in o[1:]:
            suse |= sregs(t)
        if op.startswith("s_cmp") or op.startswith("s_bitcmp"):
            sdef = set(); suse |= sregs(o[0])
        if "saveexec" in op: sdef |= {EXEC_LO, EXEC_HI}; suse |= {EXEC_LO, EXEC_HI}
    elif kind == "vmem":
        toks = list(o)
        is_store = "store" in op
        if not is_store and "_lds_" not in op and not (op.startswith("global_load_lds")):
            vdef |= _regs(toks[0], "v"); toks = toks[1:]
        for t in toks:
            suse |= sregs(t); vuse |= _regs(t, "v")
    elif kind == "smem":
        sdef |= sregs(o[0]) if o else set()
        for t in o[1:]:
            suse |= sregs(t)
    elif kind == "lds":
        if op.startswith("ds_read") or "_rtn" in op or op.startswith("ds_bpermute") or op.startswith("ds_swizzle"):
            vdef |= _regs(o[0], "v")
            for t in o[1:]: vuse |= _regs(t, "v")
        else:
            for t in o: vuse |= _regs(t, "v")
    mfma_passes = {"v_mfma_f32_4x4x4_16b_f16": 2, "v_mfma_f32_16x16x32_f16": 5}.get(op, 0)    # (passes + 3 = the distance hipcc keeps: 5 and 8)
    info = dict(kind=kind, sdef=sdef, vdef=vdef, suse=suse, vuse=vuse, op=op, ln=ln, text=text, mfma=mfma_passes,
                srcc=(_regs(o[3], "v") if mfma_passes and len(o) > 3 else set()),
                dpp=any(k in mods for k in ("row_shr", "row_shl", "row_ror", "quad_perm", "row_bcast", "wave_shr", "wave_shl", "row_mirror", "row_half_mirror", "row_newbcast")) or "_dpp" in op,
                trans=op.startswith(TRANS), lds_dma=("_lds_" in op or (kind == "vmem" and "lds" in mods)),
                rwlane=bool(re.match(r"v_(readlane|writelane)", op)), readlane=bool(re.match(r"v_(readlane|readfirstlane)", op)),
                partial=("dst_sel" in mods and mods.get("dst_sel") != "DWORD") or bool(re.match(r"v_(mad_mixhi|mad_mixlo|fma_mixhi|fma_mixlo)", op)) or (re.search(r"op_sel:\[[01],[01],[01],1\]|op_sel:\[[01],[01],1\]$", text) is not None and not op.startswith("v_pk")),
                wide_store=(kind == "vmem" and "store" in op and re.search(r"x3|x4", op) is not None),
                asm=ln in ASM_LINES)
    INFO_CACHE[key] = info
    return info


class Wave:
    def check_hazards(self):
        cur = inst_info(self.insts[self.pc])
        hist = self.__dict__.setdefault("hist", [])
        now = self.__dict__.setdefault("wstate", 0)
        def hit(rule, prev):
            key = (rule, prev["ln"], cur["ln"])
            if key not in HAZARDS:
                HAZARDS[key] = [0, prev["text"], cur["text"], prev["asm"], cur["asm"]]
            HAZARDS[key][0] += 1
        for after, prev in reversed(hist):
            between = now - after
            if between >= 12:
                break
            # matrix instructions (what the compiler puts between such pairs on gfx950: 2 wait states between a matrix
            # instruction and one that accumulates into its result, passes + 3 before anything else reads the result, 2
            # between a vector instruction that writes a register and a matrix instruction that reads it)
            if prev["mfma"]:
                if cur["mfma"] and between < 2 and prev["vdef"] & cur["srcc"]:
                    hit("matrix result -> accumulated into by the next matrix instruction (2)", prev)
                elif not cur["mfma"] and between < prev["mfma"] + 3 and cur["kind"] in ("valu", "vmem", "lds") and prev["vdef"] & (cur["vuse"] | cur["vdef"]):
                    hit("matrix result -> read or overwritten by another instruction (passes + 3)", prev)
            elif prev["kind"] == "valu" and cur["mfma"] and between < 2 and prev["vdef"] & cur["vuse"]:
                hit("VALU writes VGPR -> matrix instruction reads it (2)", prev)
            if between >= 5:
                continue
            pv = prev["kind"] == "valu"
            if pv and cur["kind"] == "vmem" and prev["sdef"] & cur["suse"]:
                hit("VALU writes SGPR -> VMEM reads it (5)", prev)
            if pv and cur["rwlane"] and between < 4 and prev["sdef"] & cur["suse"]:
                hit("VALU writes SGPR -> lane select (4)", prev)
            if pv and cur["op"].startswith("v_div_fmas") and between < 4 and prev["sdef"] & {VCC_LO, VCC_HI}:
                hit("VALU writes VCC -> v_div_fmas (4)", prev)
            if pv and cur["dpp"] and between < 2 and prev["vdef"] & cur["vuse"]:
                hit("VALU writes VGPR -> DPP reads it (2)", prev)
            if pv and cur["dpp"] and prev["sdef"] & {EXEC_LO, EXEC_HI}:
                hit("VALU writes EXEC -> DPP (5)", prev)
            if prev["kind"] == "salu" and M0_REG in prev["sdef"] and cur["lds_dma"] and between < 1:
                hit("SALU writes M0 -> LDS-direct load (1)", prev)
            if pv and cur["kind"] == "valu" and between < 2 and prev["sdef"] & cur["suse"]:
                hit("gfx940: VALU writes SGPR/VCC -> VALU reads it (2)", prev)
            if pv and prev["trans"] and cur["kind"] == "valu" and between < 1 and prev["vdef"] & cur["vuse"]:
                hit("gfx940: trans result -> VALU reads it (1)", prev)
            if pv and prev["partial"] and cur["kind"] == "valu" and between < 1 and prev["vdef"] & cur["vuse"]:
                hit("gfx940: partial-dword write -> VALU reads it (1)", prev)
            if pv and cur["readlane"] and between < 1 and prev["vdef"] & cur["vuse"]:
                hit("gfx940: VALU writes VGPR -> readlane reads it (1)", prev)
            if pv and (cur["rwlane"] or cur["readlane"]) and between < 4 and prev["sdef"] & {EXEC_LO, EXEC_HI}:
                hit("gfx940: VALU writes EXEC -> read/writelane (4)", prev)
            if prev["wide_store"] and cur["kind"] == "valu" and between < 2 and prev["vuse"] & cur["vdef"]:
                hit("wide store data overwritten (2)", prev)
        m = re.match(r"s_nop", cur["op"])
        step = 1
        if m:
            try: step = int(self.insts[self.pc][1][0], 0) + 1
            except Exception: step = 1
        self.wstate = now + step
        hist.append((self.wstate, cur))
        if len(hist) > 16:
            del hist[0]

    def __init__(self, wg, wid, insts, labels, mem, lds, kernarg, wg_id, rng):
        self.wg, self.wid, self.insts, self.labels, self.mem, self.lds = wg, wid, insts, labels, mem, lds
        self.s = np.zeros(128, dtype=U32)
        self.v = np.zeros((256, 64), dtype=U32)
        self.vcc = 0
        self.exec = MASK64
        self.scc = 0
        self.m0 = 0
        self.pc = 0
        self.done = False
        self.at_barrier = False
        self.vmq = []          # pending vector-memory ops: (age, fn)
        self.lgq = []          # pending LDS / scalar-memory ops
        self.tick = 0
        self.rng = rng
        if GARBAGE:
            # what a wave finds in registers nobody initialised: leftovers of other waves
            g = np.random.default_rng(rng.randrange(1 << 30))
            self.s[:] = g.integers(0, 1 << 32, 128, dtype=np.uint64).astype(U32)
            self.v[:] = g.integers(0, 1 << 32, (256, 64), dtype=np.uint64).astype(U32)
            self.vcc = int(g.integers(0, 1 << 62))
            self.m0 = int(g.integers(0, 1 << 32))
            self.scc = int(g.integers(0, 2))
        self.s[0] = kernarg & 0xFFFFFFFF
        self.s[1] = kernarg >> 32
        self.s[15] = wg_id
        self.v[0] = np.arange(64, dtype=U32) + 64 * wid
        self.trace = []

    # ------------------------------------------------------------ operands
    def who(self):
        op, ops, mods, ln, t = self.insts[self.pc]
        return f"wg {self.wg} wave {self.wid} line {ln}: {t}"

    def sreg_index(self, tok):
        return _reg_index("s", tok)

    def vreg_index(self, tok):
        return _reg_index("v", tok)

    def rs(self, tok, width=1):
        """scalar source -> python int (width 1 or 2 dwords)"""
        tok = tok.strip()
        if tok == "vcc":
            return self.vcc if width == 2 else self.vcc & 0xFFFFFFFF
        if tok == "vcc_lo":
            return self.vcc & 0xFFFFFFFF
        if tok == "vcc_hi":
            return self.vcc >> 32
        if tok == "exec":
            return self.exec if width == 2 else self.exec & 0xFFFFFFFF
        if tok == "exec_lo":
            return self.exec & 0xFFFFFFFF
        if tok == "exec_hi":
            return self.exec >> 32
        if tok == "m0":
            return self.m0
        if tok == "scc":
            return self.scc
        i, n = self.sreg_index(tok)
        if i is not None:
            if width == 2 or n == 2:
                return int(self.s[i]) | (int(self.s[i + 1]) << 32)
            return int(self.s[i])
        if tok in INLINE_FLOAT:
            return INLINE_FLOAT[tok]
        if tok == "off":
            return 0
        try:
            val = int(tok, 0)
        except ValueError:
            raise Fault(f"cannot read scalar operand {tok!r} ({self.who()})")
        return val & (MASK64 if width == 2 else 0xFFFFFFFF)

    def ws(self, tok, val, width=None):
        tok = tok.strip()
        if tok == "vcc":
            self.vcc = val & MASK64
            return
        if tok == "vcc_lo":
            self.vcc = (self.vcc & ~0xFFFFFFFF & MASK64) | (val & 0xFFFFFFFF)
            return
        if tok == "vcc_hi":
            self.vcc = (self.vcc & 0xFFFFFFFF) | ((val & 0xFFFFFFFF) << 32)
            return
        if tok == "exec_lo":
            self.exec = (self.exec & ~0xFFFFFFFF & MASK64) | (val & 0xFFFFFFFF)
            return
        if tok == "exec_hi":
            self.exec = (self.exec & 0xFFFFFFFF) | ((val & 0xFFFFFFFF) << 32)
            return
        if tok == "exec":
            self.exec = val & MASK64
            return
        if tok == "m0":
            self.m0 = val & 0xFFFFFFFF
            return
        i, n = self.sreg_index(tok)
        if i is None:
            raise Fault(f"cannot write scalar operand {tok!r} ({self.who()})")
        if width is None:
            width = n
        for k in range(width):
            self.s[i + k] = (val >> (32 * k)) & 0xFFFFFFFF

    def rv(self, tok):
        """vector (or scalar / literal, broadcast) source -> uint32[64]"""
        tok = tok.strip()
        neg = ab = False
        if tok.startswith("-"):
            if re.match(r"^-\d", tok) is None or tok in INLINE_FLOAT:
                pass
            if tok[1:2] in ("v", "s", "|"):
                neg, tok = True, tok[1:]
        if tok.startswith("|") and tok.endswith("|"):
            ab, tok = True, tok[1:-1]
        i, n = self.vreg_index(tok)
        if i is not None:
            val = self.v[i].copy()
        else:
            val = np.full(64, self.rs(tok) & 0xFFFFFFFF, dtype=U32)
        if ab:
            val = val & U32(0x7FFFFFFF)
        if neg:
            val = val ^ U32(0x80000000)
        return val

    def v64(self, tok):
        i, n = self.vreg_index(tok)
        if i is not None:
            return self.v[i].astype(np.uint64) | (self.v[i + 1].astype(np.uint64) << np.uint64(32))
        j, _ = self.sreg_index(tok)
        if j is not None or tok in ("vcc", "exec"):
            return np.full(64, self.rs(tok, 2), dtype=np.uint64)
        return np.full(64, int(tok, 0) & MASK64, dtype=np.uint64)

    def wv64(self, tok, val):
        d, _ = self.vreg_index(tok)
        m = self.lanes()
        val = np.asarray(val).astype(np.uint64)
        self.v[d][m] = (val & np.uint64(0xFFFFFFFF)).astype(U32)[m]
        self.v[d + 1][m] = (val >> np.uint64(32)).astype(U32)[m]

    def lanes(self):
        return _lanes_of(self.exec)

    def wv(self, tok, val, mask=None):
        i, n = self.vreg_index(tok)
        if i is None:
            raise Fault(f"cannot write vector operand {tok!r} ({self.who()})")
        m = self.lanes() if mask is None else mask
        self.v[i][m] = np.asarray(val, dtype=U32)[m]

    def mask_to_int(self, b):
        out = 0
        for k in range(64):
            if b[k]:
                out |= 1 << k
        return out

    # ------------------------------------------------------------ memory queues
    def force_vm(self, n):
        while len(self.vmq) > n:
            self.vmq.pop(0)[1]()

    def force_lgkm(self, n):
        while len(self.lgq) > n:
            self.lgq.pop(0)[1]()

    def age_queues(self):
        self.tick += 1
        while self.vmq and self.tick - self.vmq[0][0] > self.vm_latency:
            self.vmq.pop(0)[1]()
        while self.lgq and self.tick - self.lgq[0][0] > self.lgkm_latency:
            self.lgq.pop(0)[1]()

    vm_latency = 400
    lgkm_latency = 60

    # ------------------------------------------------------------ LDS helpers
    def lds_read32(self, addr):
        if addr + 4 > len(self.lds) * 4 or addr % 4:
            raise Fault(f"LDS read at {addr:#x} beyond {len(self.lds) * 4:#x} or misaligned ({self.who()})")
        return self.lds[addr // 4]

    def lds_write32(self, addr, val, who):
        if addr + 4 > len(self.lds) * 4 or addr % 4:
            raise Fault(f"LDS write at {addr:#x} beyond {len(self.lds) * 4:#x} or misaligned ({who})")
        self.lds[addr // 4] = val

    # ------------------------------------------------------------ DPP
    def dpp_src(self, src, mods, old):
        """returns (values, valid mask) of the DPP-selected source lanes"""
        out = np.zeros(64, dtype=U32)
        valid = np.zeros(64, dtype=bool)
        bound = "bound_ctrl" in mods
        for lane in range(64):
            row, idx = lane // 16, lane % 16
            srcl = None
            if "row_shr" in mods:
                k = int(mods["row_shr"])
                if idx - k >= 0:
                    srcl = lane - k
            elif "wave_shr" in mods:
                if lane - 1 >= 0:
                    srcl = lane - 1
            elif "row_bcast" in mods:
                if int(mods["row_bcast"]) == 15 and row > 0:
                    srcl = (row - 1) * 16 + 15
                elif int(mods["row_bcast"]) == 31 and row >= 2:
                    srcl = 31
            elif "quad_perm" in mods:
                qp = [int(x) for x in mods["quad_perm"].strip("[]").split(",")]
                srcl = (lane & ~3) + qp[lane & 3]
            elif "row_mirror" in mods:
                srcl = row * 16 + (15 - idx)
            elif "row_half_mirror" in mods:
                srcl = row * 16 + (idx & 8) + (7 - (idx & 7))
            elif "row_shl" in mods:
                k = int(mods["row_shl"])
                if idx + k <= 15:
                    srcl = lane + k
            elif "row_ror" in mods:
                srcl = row * 16 + ((idx - int(mods["row_ror"])) & 15)
            else:
                raise Fault(f"DPP control not modelled: {mods} ({self.who()})")
            if srcl is not None and (self.exec >> srcl) & 1:
                out[lane], valid[lane] = src[srcl], True
            elif bound:
                out[lane], valid[lane] = 0, True
        row_mask = int(mods.get("row_mask", "0xf"), 0)
        bank_mask = int(mods.get("bank_mask", "0xf"), 0)
        for lane in range(64):
            if not (row_mask >> (lane // 16)) & 1 or not (bank_mask >> ((lane % 16) // 4)) & 1:
                valid[lane] = False
        return out, valid

    # ------------------------------------------------------------ one instruction
    def step(self):
        if self.done:
            return
        self.age_queues()
        op, o, mods, ln, text = self.insts[self.pc]
        nxt = self.pc + 1
        if HAZARDS is not None:
            self.check_hazards()
        if COUNTS is not None:
            COUNTS[ln] = COUNTS.get(ln, 0) + 1
        S, V = self.rs, self.rv

        def setscc(c):
            self.scc = 1 if c else 0

        def sx(x):     # sign-extend 32
            return x - (1 << 32) if x & 0x80000000 else x

        if op == "s_nop" or op == "s_setprio" or op == "s_sleep":
            pass
        elif op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", text)
            if m:
                self.force_vm(int(m.group(1)))
            m = re.search(r"lgkmcnt\((\d+)\)", text)
            if m:
                self.force_lgkm(int(m.group(1)))
        elif op == "s_endpgm":
            self.force_vm(0)
            self.force_lgkm(0)
            self.done = True
            return
        elif op == "s_barrier":
            self.at_barrier = True
            self.pc = nxt
            return
        elif op == "s_branch":
            nxt = self.labels[o[0]]
        elif op == "s_cbranch_scc0":
            if not self.scc: nxt = self.labels[o[0]]
        elif op == "s_cbranch_scc1":
            if self.scc: nxt = self.labels[o[0]]
        elif op == "s_cbranch_vccz":
            if self.vcc == 0: nxt = self.labels[o[0]]
        elif op == "s_cbranch_vccnz":
            if self.vcc != 0: nxt = self.labels[o[0]]
        elif op == "s_cbranch_execz":
            if self.exec == 0: nxt = self.labels[o[0]]
        elif op == "s_cbranch_execnz":
            if self.exec != 0: nxt = self.labels[o[0]]
        elif op == "s_mov_b32":
            self.ws(o[0], S(o[1]), 1)
        elif op == "s_mov_b64":
            self.ws(o[0], S(o[1], 2) if not re.match(r"^-?\d", o[1]) else (int(o[1], 0) & MASK64), 2)
        elif op in ("s_add_i32", "s_add_u32", "s_addk_i32"):
            a, b = (S(o[1]), S(o[2])) if op != "s_addk_i32" else (S(o[0]), int(o[1], 0) & 0xFFFFFFFF)
            r = a + b
            if op == "s_add_u32":
                setscc(r >> 32)
            else:
                setscc((sx(a) + sx(b)) != sx(r & 0xFFFFFFFF))
            self.ws(o[0], r & 0xFFFFFFFF, 1)
        elif op == "s_addc_u32":
            r = S(o[1]) + S(o[2]) + self.scc
            setscc(r >> 32)
            self.ws(o[0], r & 0xFFFFFFFF, 1)
        elif op == "s_sub_u32":
            a, b = S(o[1]), S(o[2])
            setscc(b > a)                         # borrow
            self.ws(o[0], (a - b) & 0xFFFFFFFF, 1)
        elif op == "s_sub_i32":
            a, b = S(o[1]), S(o[2])
            r = (a - b) & 0xFFFFFFFF
            setscc((sx(a) - sx(b)) != sx(r))
            self.ws(o[0], r, 1)
        elif op == "s_mul_i32":
            self.ws(o[0], (S(o[1]) * S(o[2])) & 0xFFFFFFFF, 1)
        elif op == "s_mul_hi_u32":
            self.ws(o[0], (S(o[1]) * S(o[2])) >> 32, 1)
        elif op == "s_mul_hi_i32":
            self.ws(o[0], ((sx(S(o[1])) * sx(S(o[2]))) >> 32) & 0xFFFFFFFF, 1)
        elif op == "s_abs_i32":
            a = S(o[1])
            r = (0x100000000 - a) & 0xFFFFFFFF if a & 0x80000000 else a
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op == "s_mulk_i32":
            v = int(o[1], 0)
            if v & 0x8000 and v > 0: v -= 0x10000
            self.ws(o[0], (S(o[0]) * v) & 0xFFFFFFFF, 1)
        elif op in ("s_and_b32", "s_or_b32", "s_xor_b32"):
            a, b = S(o[1]), S(o[2])
            r = a & b if op == "s_and_b32" else (a | b if op == "s_or_b32" else a ^ b)
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op in ("s_and_b64", "s_or_b64", "s_xor_b64", "s_andn2_b64", "s_orn2_b64"):
            a, b = S(o[1], 2), S(o[2], 2)
            r = {"s_and_b64": a & b, "s_or_b64": a | b, "s_xor_b64": a ^ b, "s_andn2_b64": a & ~b & MASK64,
                 "s_orn2_b64": (a | ~b) & MASK64}[op]
            setscc(r != 0)
            self.ws(o[0], r, 2)
        elif op == "s_and_saveexec_b64":
            old = self.exec
            self.exec = S(o[1], 2) & old
            setscc(self.exec != 0)
            self.ws(o[0], old, 2)
        elif op == "s_lshl_b32":
            r = (S(o[1]) << (S(o[2]) & 31)) & 0xFFFFFFFF
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op == "s_lshr_b32":
            r = S(o[1]) >> (S(o[2]) & 31)
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op == "s_ashr_i32":
            r = (sx(S(o[1])) >> (S(o[2]) & 31)) & 0xFFFFFFFF
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op == "s_lshr_b64":
            r = S(o[1], 2) >> (S(o[2]) & 63)
            setscc(r != 0)
            self.ws(o[0], r, 2)
        elif op in ("s_bitset0_b32", "s_bitset1_b32"):
            bit = 1 << (S(o[1]) & 31)
            self.ws(o[0], (S(o[0]) | bit) if op == "s_bitset1_b32" else (S(o[0]) & ~bit & 0xFFFFFFFF), 1)
        elif op == "s_lshl_b64":
            r = (S(o[1], 2) << (S(o[2]) & 63)) & MASK64
            setscc(r != 0)
            self.ws(o[0], r, 2)
        elif op == "s_bfe_u32":
            a, b = S(o[1]), S(o[2])
            off, wid = b & 31, (b >> 16) & 0x7F
            r = (a >> off) & ((1 << wid) - 1) if wid else 0
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op == "s_bfe_i32":
            a, b = S(o[1]), S(o[2])
            off, wid = b & 31, (b >> 16) & 0x7F
            r = (a >> off) & ((1 << wid) - 1) if wid else 0
            if wid and r & (1 << (wid - 1)):
                r |= 0xFFFFFFFF & ~((1 << wid) - 1)          # sign-extended
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op in ("s_min_i32", "s_min_u32", "s_max_u32", "s_max_i32"):
            a, b = S(o[1]), S(o[2])
            if op.endswith("i32"):
                c = sx(a) < sx(b) if "min" in op else sx(a) > sx(b)
            else:
                c = a < b if "min" in op else a > b
            setscc(c)
            self.ws(o[0], a if c else b, 1)
        elif op in ("s_cmp_eq_u64", "s_cmp_lg_u64"):
            a = S(o[0], 2)
            b = S(o[1], 2) if not re.match(r"^-?\d", o[1]) else int(o[1], 0) & MASK64
            setscc((a == b) == (op == "s_cmp_eq_u64"))
        elif op.startswith("s_cmp_") or op.startswith("s_cmpk_"):
            a = S(o[0])
            b = S(o[1]) if op.startswith("s_cmp_") else int(o[1], 0) & 0xFFFFFFFF
            kind = op.split("_")[2]
            signed = op.endswith("i32")
            if signed:
                a, b = sx(a), sx(b)
            setscc({"eq": a == b, "lg": a != b, "gt": a > b, "ge": a >= b, "lt": a < b, "le": a <= b}[kind])
        elif op == "s_bitcmp1_b32":
            setscc((S(o[0]) >> (S(o[1]) & 31)) & 1)
        elif op == "s_bitcmp0_b32":
            setscc(not (S(o[0]) >> (S(o[1]) & 31)) & 1)
        elif op == "s_cselect_b32":
            self.ws(o[0], S(o[1]) if self.scc else S(o[2]), 1)
        elif op == "s_cselect_b64":
            a = S(o[1], 2) if not re.match(r"^-?\d", o[1]) else int(o[1], 0) & MASK64
            b = S(o[2], 2) if not re.match(r"^-?\d", o[2]) else int(o[2], 0) & MASK64
            self.ws(o[0], a if self.scc else b, 2)
        elif op == "s_bcnt1_i32_b64":
            r = bin(S(o[1], 2)).count("1")
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op.startswith("s_load_dword"):
            n = {"s_load_dword": 1, "s_load_dwordx2": 2, "s_load_dwordx4": 4, "s_load_dwordx8": 8, "s_load_dwordx16": 16}[op]
            base = S(o[1], 2)
            off = S(o[2]) if len(o) > 2 else 0
            if "offset" in mods:
                off += int(mods["offset"], 0)
            addr = (base + off) & ~3
            dst = o[0]
            who = self.who()

            def fn(addr=addr, n=n, dst=dst, who=who):
                data = self.mem.read(addr, 4 * n, who)
                i, _ = self.sreg_index(dst)
                self.s[i:i + n] = np.frombuffer(data, dtype=U32)
            # poison the destination until the data arrives
            i, _ = self.sreg_index(dst)
            self.s[i:i + n] = 0xDEAD0000 + np.arange(n, dtype=U32)
            self.lgq.append((self.tick, fn))
        # ---------------------------------------------------------------- vector ALU
        elif op in ("v_mov_b32_e32", "v_mov_b32_e64"):
            self.wv(o[0], V(o[1]))
        elif op in ("v_not_b32_e32", "v_not_b32_e64"):
            self.wv(o[0], (~V(o[1]).astype(np.uint64) & np.uint64(0xFFFFFFFF)).astype(U32))
        elif op == "v_bfrev_b32_e32":
            a = V(o[1]).astype(np.uint64)
            r = np.zeros(64, dtype=np.uint64)
            for bit in range(32):
                r |= ((a >> np.uint64(bit)) & np.uint64(1)) << np.uint64(31 - bit)
            self.wv(o[0], r.astype(U32))
        elif op == "v_mov_b32_dpp":
            src, valid = self.dpp_src(V(o[1]), mods, None)
            self.wv(o[0], src, self.lanes() & valid)
        elif op == "v_readfirstlane_b32":
            lane = next((k for k in range(64) if (self.exec >> k) & 1), 0)
            self.ws(o[0], int(V(o[1])[lane]), 1)
        elif op in ("v_add_u32_e32", "v_sub_u32_e32", "v_subrev_u32_e32", "v_and_b32_e32", "v_or_b32_e32", "v_xor_b32_e32",
                    "v_lshlrev_b32_e32", "v_lshrrev_b32_e32", "v_ashrrev_i32_e32", "v_min_u32_e32", "v_max_u32_e32",
                    "v_mul_u32_u24_e32", "v_mul_i32_i24_e32"):
            a, b = V(o[1]).astype(np.uint64), V(o[2]).astype(np.uint64)
            if op == "v_add_u32_e32": r = a + b
            elif op == "v_sub_u32_e32": r = a - b
            elif op == "v_subrev_u32_e32": r = b - a
            elif op == "v_and_b32_e32": r = a & b
            elif op == "v_or_b32_e32": r = a | b
            elif op == "v_xor_b32_e32": r = a ^ b
            elif op == "v_lshlrev_b32_e32": r = b << (a & 31)
            elif op == "v_lshrrev_b32_e32": r = b >> (a & 31)
            elif op == "v_ashrrev_i32_e32": r = (b.astype(np.uint32).view(np.int32).astype(np.int64) >> (a & 31).astype(np.int64)).astype(np.uint64)
            elif op == "v_min_u32_e32": r = np.minimum(a, b)
            elif op == "v_max_u32_e32": r = np.maximum(a, b)
            elif op == "v_mul_u32_u24_e32": r = (a & 0xFFFFFF) * (b & 0xFFFFFF)
            else:
                sa = ((a & 0xFFFFFF) ^ 0x800000).astype(np.int64) - 0x800000
                sb = ((b & 0xFFFFFF) ^ 0x800000).astype(np.int64) - 0x800000
                r = (sa * sb).astype(np.uint64)
            self.wv(o[0], (r & 0xFFFFFFFF).astype(U32))
        elif op == "v_mad_i32_i24":
            a, b, c = V(o[1]).astype(np.uint64), V(o[2]).astype(np.uint64), V(o[3]).astype(np.int64)
            sa = ((a & 0xFFFFFF) ^ 0x800000).astype(np.int64) - 0x800000
            sb = ((b & 0xFFFFFF) ^ 0x800000).astype(np.int64) - 0x800000
            self.wv(o[0], ((sa * sb + c) & 0xFFFFFFFF).astype(U32))
        elif op == "v_add3_u32":
            r = V(o[1]).astype(np.uint64) + V(o[2]).astype(np.uint64) + V(o[3]).astype(np.uint64)
            self.wv(o[0], (r & 0xFFFFFFFF).astype(U32))
        elif op == "v_lshl_add_u32":
            r = (V(o[1]).astype(np.uint64) << (V(o[2]).astype(np.uint64) & 31)) + V(o[3]).astype(np.uint64)
            self.wv(o[0], (r & 0xFFFFFFFF).astype(U32))
        elif op == "v_add_lshl_u32":
            r = (V(o[1]).astype(np.uint64) + V(o[2]).astype(np.uint64)) << (V(o[3]).astype(np.uint64) & 31)
            self.wv(o[0], (r & 0xFFFFFFFF).astype(U32))
        elif op == "v_lshl_add_u64":
            i, _ = self.vreg_index(o[1])
            if i is not None:
                a = self.v[i].astype(np.uint64) | (self.v[i + 1].astype(np.uint64) << np.uint64(32))
            else:
                a = np.full(64, S(o[1], 2), dtype=np.uint64)
            sh = np.uint64(int(o[2], 0))
            j, _ = self.vreg_index(o[3])
            if j is not None:
                c = self.v[j].astype(np.uint64) | (self.v[j + 1].astype(np.uint64) << np.uint64(32))
            else:
                c = np.full(64, S(o[3], 2) if self.sreg_index(o[3])[0] is not None else int(o[3], 0) & MASK64, dtype=np.uint64)
            r = (a << sh) + c
            d, _ = self.vreg_index(o[0])
            m = self.lanes()
            self.v[d][m] = (r & np.uint64(0xFFFFFFFF)).astype(U32)[m]
            self.v[d + 1][m] = (r >> np.uint64(32)).astype(U32)[m]
        elif op in ("v_mad_u64_u32", "v_mad_i64_i32"):
            a, b = V(o[2]).astype(np.uint64), V(o[3]).astype(np.uint64)
            if op == "v_mad_i64_i32":
                # sign-extend both factors; the product and the sum wrap at 64 bits
                a = np.where(a & np.uint64(0x80000000), a | np.uint64(0xFFFFFFFF00000000), a)
                b = np.where(b & np.uint64(0x80000000), b | np.uint64(0xFFFFFFFF00000000), b)
            j, _ = self.vreg_index(o[4])
            if j is not None:
                c = self.v[j].astype(np.uint64) | (self.v[j + 1].astype(np.uint64) << np.uint64(32))
            else:
                c = np.full(64, S(o[4], 2) if self.sreg_index(o[4])[0] is not None else int(o[4], 0), dtype=np.uint64)
            r = a * b + c
            d, _ = self.vreg_index(o[0])
            m = self.lanes()
            self.v[d][m] = (r & np.uint64(0xFFFFFFFF)).astype(U32)[m]
            self.v[d + 1][m] = (r >> np.uint64(32)).astype(U32)[m]
            self.ws(o[1], 0, 2)
        elif op == "v_addc_co_u32_e32":
            a, b = V(o[2]).astype(np.uint64), V(o[3]).astype(np.uint64)
            cin = np.array([(self.vcc >> k) & 1 for k in range(64)], dtype=np.uint64)
            r = a + b + cin
            m = self.lanes()
            self.wv(o[0], (r & 0xFFFFFFFF).astype(U32))
            carry = (r >> np.uint64(32)) != 0
            newvcc = self.vcc
            for k in range(64):
                if m[k]:
                    newvcc = (newvcc & ~(1 << k)) | (int(carry[k]) << k)
            self.vcc = newvcc
        elif op == "v_bfi_b32":
            # bits of source 1 where source 0 has ones, of source 2 elsewhere
            mask = V(o[1])
            self.wv(o[0], (mask & V(o[2])) | (~mask & V(o[3])))
        elif op == "v_or3_b32":
            self.wv(o[0], V(o[1]) | V(o[2]) | V(o[3]))
        elif op in ("v_bitop3_b32", "v_bitop3_b16"):
            # every result bit is the truth table's entry for the three source bits (source 0 the most significant of the
            # index).  The 16-bit form is taken to write the low half and keep the high one; a use of the high half of
            # its result would show which the hardware does, and none is modelled.
            if "op_sel" in mods:
                raise Fault(f"operand selects of {op} not modelled ({self.who()})")
            tt = int(mods["bitop3"], 0)
            a, b, c = V(o[1]), V(o[2]), V(o[3])
            r = np.zeros(64, dtype=U32)
            for idx in range(8):
                if (tt >> idx) & 1:
                    r |= (a if idx & 4 else ~a) & (b if idx & 2 else ~b) & (c if idx & 1 else ~c)
            if op.endswith("b16"):
                i, _ = self.vreg_index(o[0])
                r = (r & U32(0xFFFF)) | (self.v[i] & U32(0xFFFF0000))
            self.wv(o[0], r)
        elif op == "v_mfma_f32_16x16x32_f16":
            # D[16 x 16] = A[16 x 32] B[32 x 16] + C, fp32.  Lane l = 16 g + i holds A[i][8 g .. 8 g + 7] (four registers of two
            # halves) and, with j for i, B[8 g .. 8 g + 7][j]; register r of lane l = 16 q + j holds C and D [4 q + r][j].
            # Every lane takes part whatever EXEC says.  The hardware's internal rounding is not modelled (sums in double).
            if mods:
                raise Fault(f"modifiers of {op} not modelled ({self.who()})")
            def halves(tok):
                i0, n = self.vreg_index(tok)
                assert n == 4, tok
                regs = np.stack([self.v[i0 + q] for q in range(4)], axis=1)                       # [lane][4]
                h = np.stack([regs & U32(0xFFFF), regs >> U32(16)], axis=2).reshape(64, 8)       # [lane][8], low half first
                return h.astype(np.uint16).view(np.float16).astype(np.float64)
            ha, hb = halves(o[1]), halves(o[2])
            A, B = np.zeros((16, 32)), np.zeros((32, 16))
            for l in range(64):
                A[l % 16, 8 * (l // 16):8 * (l // 16) + 8] = ha[l]
                B[8 * (l // 16):8 * (l // 16) + 8, l % 16] = hb[l]
            C = np.zeros((16, 16))
            if self.vreg_index(o[3])[0] is not None:
                c0, _ = self.vreg_index(o[3])
                for l in range(64):
                    for r in range(4):
                        C[4 * (l // 16) + r, l % 16] = f32(self.v[c0 + r][l:l + 1])[0]
            elif int(o[3], 0) != 0:
                raise Fault(f"constant accumulator of {op} not modelled ({self.who()})")
            with np.errstate(all="ignore"):
                D = (A @ B + C).astype(np.float32)
            d0, _ = self.vreg_index(o[0])
            for r in range(4):
                self.v[d0 + r] = as_u32(np.array([D[4 * (l // 16) + r, l % 16] for l in range(64)], dtype=np.float32))
        elif op == "v_mfma_f32_4x4x4_16b_f16":
            # Sixteen independent 4 x 4 x 4 products: block b = lanes 4 b .. 4 b + 3.  Lane 4 b + i holds A_b[i][0 .. 3] (two
            # registers of two halves) and, with j for i, B_b[0 .. 3][j]; register r of lane 4 b + j holds C and D [r][j].
            # Every lane takes part whatever EXEC says; sums in double, rounded once to fp32.
            if mods:
                raise Fault(f"modifiers of {op} not modelled ({self.who()})")
            def halves4(tok):
                i0, n = self.vreg_index(tok)
                assert n == 2, tok
                regs = np.stack([self.v[i0 + q] for q in range(2)], axis=1)                       # [lane][2]
                h = np.stack([regs & U32(0xFFFF), regs >> U32(16)], axis=2).reshape(64, 4)       # [lane][4], low half first
                return h.astype(np.uint16).view(np.float16).astype(np.float64)
            ha, hb = halves4(o[1]), halves4(o[2])
            c0 = self.vreg_index(o[3])[0]
            if c0 is None and int(o[3], 0) != 0:
                raise Fault(f"constant accumulator of {op} not modelled ({self.who()})")
            d0, nd = self.vreg_index(o[0])
            assert nd == 4, o[0]
            out = np.zeros((4, 64), dtype=np.float32)
            with np.errstate(all="ignore"):
                for l in range(64):
                    b, j = l // 4, l % 4
                    for r in range(4):
                        acc = float(f32(self.v[c0 + r][l:l + 1])[0]) if c0 is not None else 0.0
                        out[r, l] = np.float32(acc + float(np.dot(ha[4 * b + r], hb[4 * b + j])))
            for r in range(4):
                self.v[d0 + r] = as_u32(out[r])
        elif op in ("v_and_or_b32", "v_perm_b32", "v_alignbit_b32", "v_pk_mad_u16"):
            a, b, c = V(o[1]), V(o[2]), V(o[3])
            if op == "v_and_or_b32":
                r = (a & b) | c
            elif op == "v_alignbit_b32":
                r = (((a.astype(np.uint64) << np.uint64(32)) | b.astype(np.uint64)) >> (c.astype(np.uint64) & np.uint64(31))).astype(np.uint64) & np.uint64(0xFFFFFFFF)
                r = r.astype(U32)
            elif op == "v_pk_mad_u16":
                lo = ((a & 0xFFFF).astype(np.uint64) * (b & 0xFFFF).astype(np.uint64) + (c & 0xFFFF).astype(np.uint64)) & np.uint64(0xFFFF)
                hi = ((a >> 16).astype(np.uint64) * (b >> 16).astype(np.uint64) + (c >> 16).astype(np.uint64)) & np.uint64(0xFFFF)
                r = (lo | (hi << np.uint64(16))).astype(U32)
            else:
                r = np.zeros(64, dtype=U32)
                for k in range(64):
                    src = (int(a[k]) << 32) | int(b[k])
                    out = 0
                    for byte in range(4):
                        sel = (int(c[k]) >> (8 * byte)) & 0xFF
                        if sel <= 7:
                            val = (src >> (8 * sel)) & 0xFF
                        elif sel == 0x0C:
                            val = 0
                        elif sel >= 0x0D:
                            val = 0xFF
                        else:
                            val = 0xFF if (src >> (16 * (sel - 8) + 15)) & 1 else 0
                        out |= val << (8 * byte)
                    r[k] = out
            self.wv(o[0], r)
        elif op in ("v_dot2c_f32_f16", "v_dot2c_f32_f16_e32", "v_dot2_f32_f16"):
            a, b = V(o[1]), V(o[2])
            acc = f32(self.v[self.vreg_index(o[0])[0]].copy()) if op.startswith("v_dot2c_") else f32(V(o[3]))
            al, ah = (a & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32), (a >> 16).astype(np.uint16).view(np.float16).astype(np.float32)
            bl, bh = (b & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32), (b >> 16).astype(np.uint16).view(np.float16).astype(np.float32)
            with np.errstate(all="ignore"):
                r = (al * bl + ah * bh + acc).astype(np.float32)
            self.wv(o[0], as_u32(r))
        elif op in ("v_add_f32_e32", "v_mul_f32_e32", "v_sub_f32_e32"):
            a, b = f32(V(o[1])), f32(V(o[2]))
            with np.errstate(all="ignore"):
                r = a + b if op == "v_add_f32_e32" else (a * b if op == "v_mul_f32_e32" else a - b)
            self.wv(o[0], as_u32(r))
        elif op == "v_add_f32_dpp":
            src0, valid = self.dpp_src(V(o[1]), mods, None)
            with np.errstate(all="ignore"):
                r = f32(src0) + f32(V(o[2]))
            self.wv(o[0], as_u32(r), self.lanes() & valid)
        elif op == "v_cndmask_b32_dpp":
            src0, valid = self.dpp_src(V(o[1]), mods, None)
            sel = np.array([(S(o[3], 2) >> k) & 1 for k in range(64)], dtype=bool)
            r = np.where(sel, V(o[2]), src0)
            self.wv(o[0], r, self.lanes() & valid)
        elif op in ("v_max_f32_e32", "v_min_f32_e32", "v_max3_f32", "v_min3_f32", "v_max_f32_e64", "v_min_f32_e64"):
            # IEEE maxNum / minNum: a number wins over a NaN
            fn = np.fmax if "max" in op else np.fmin
            r = fn(f32(V(o[1])), f32(V(o[2])))
            if "3" in op.split("_")[1]:
                r = fn(r, f32(V(o[3])))
            self.wv(o[0], as_u32(r.astype(np.float32)))
        elif op == "v_fmac_f32_e32":
            with np.errstate(all="ignore"):
                r = (f32(V(o[1])).astype(np.float64) * f32(V(o[2])).astype(np.float64) + f32(V(o[0])).astype(np.float64)).astype(np.float32)
            self.wv(o[0], as_u32(r))
        elif op == "v_fma_f32":
            # one rounding: the product of two fp32 values is exact in double
            with np.errstate(all="ignore"):
                r = (f32(V(o[1])).astype(np.float64) * f32(V(o[2])).astype(np.float64) + f32(V(o[3])).astype(np.float64)).astype(np.float32)
            self.wv(o[0], as_u32(r))
        elif op == "v_rsq_f32_e32":
            with np.errstate(all="ignore"):
                r = (np.float32(1.0) / np.sqrt(f32(V(o[1])).astype(np.float64))).astype(np.float32)
            self.wv(o[0], as_u32(r))
        elif op == "v_cvt_f16_f32_sdwa":
            # dst_unused:UNUSED_PAD: the half that is not written becomes zero
            if mods.get("src0_sel", "DWORD") != "DWORD" or mods.get("dst_unused", "UNUSED_PAD") != "UNUSED_PAD" or "sext" in text:
                raise Fault(f"operand selects of {op} not modelled ({self.who()})")
            with np.errstate(all="ignore"):
                h = f32(V(o[1])).astype(np.float16).view(np.uint16).astype(U32)
            where = mods.get("dst_sel", "DWORD")
            if where not in ("DWORD", "WORD_0", "WORD_1"):
                raise Fault(f"operand selects of {op} not modelled ({self.who()})")
            self.wv(o[0], h << U32(16) if where == "WORD_1" else h)
        elif op in ("v_exp_f32_e32", "v_rcp_f32_e32", "v_log_f32_e32", "v_sqrt_f32_e32"):
            # the hardware's approximations are within an ulp of these; kernels that must agree bit for bit run the same
            # instruction on the same input on both sides, which the model reproduces
            with np.errstate(all="ignore"):
                x = f32(V(o[1])).astype(np.float64)
                r = {"v_exp_f32_e32": np.exp2, "v_rcp_f32_e32": lambda v: 1.0 / v, "v_log_f32_e32": np.log2, "v_sqrt_f32_e32": np.sqrt}[op](x)
                r = r.astype(np.float32)
            self.wv(o[0], as_u32(r))
        elif op == "v_div_scale_f32":
            # the operand (numerator or denominator) as it is and VCC = 0: true for operands far from the ends of the
            # exponent range, which is checked (the scaled cases are not modelled)
            src0 = f32(V(o[2]))
            mag = np.abs(np.concatenate([f32(V(o[2])), f32(V(o[3])), f32(V(o[4]))]).astype(np.float64))
            live = np.concatenate([self.lanes()] * 3)
            if ((mag[live] != 0) & ((mag[live] < 1e-30) | (mag[live] > 1e30))).any():
                raise Fault(f"{op}: operands that need scaling are not modelled ({self.who()})")
            self.wv(o[0], as_u32(src0))
            old = S(o[1], 2)
            for k in range(64):
                if self.lanes()[k]:
                    old &= ~(1 << k)
            self.ws(o[1], old, 2)
        elif op == "v_div_fmas_f32":
            with np.errstate(all="ignore"):
                r = (f32(V(o[1])).astype(np.float64) * f32(V(o[2])).astype(np.float64) + f32(V(o[3])).astype(np.float64)).astype(np.float32)
            self.wv(o[0], as_u32(r))
        elif op == "v_div_fixup_f32":
            q, den, num = f32(V(o[1])), f32(V(o[2])), f32(V(o[3]))
            with np.errstate(all="ignore"):
                exact = (num.astype(np.float64) / den.astype(np.float64)).astype(np.float32)
            special = ~np.isfinite(q) | (den == 0) | ~np.isfinite(den) | ~np.isfinite(num)
            self.wv(o[0], as_u32(np.where(special, exact, q)))
        elif op == "v_rcp_iflag_f32_e32":
            with np.errstate(all="ignore"):
                r = np.float32(1.0) / f32(V(o[1]))
            self.wv(o[0], as_u32(r))
        elif op == "v_trunc_f32_e32":
            self.wv(o[0], as_u32(np.trunc(f32(V(o[1])))))
        elif op == "v_cvt_u32_f32_e32":
            with np.errstate(all="ignore"):
                r = np.clip(np.nan_to_num(f32(V(o[1]))), 0, 4294967295.0).astype(np.uint64).astype(U32)
            self.wv(o[0], r)
        elif op == "v_cvt_f32_u32_e32":
            self.wv(o[0], as_u32(V(o[1]).astype(np.float32)))
        elif op == "v_cvt_f32_i32_e32":
            self.wv(o[0], as_u32(V(o[1]).astype(np.int32).astype(np.float32)))
        elif op == "v_cvt_f32_ubyte0_e32":
            self.wv(o[0], as_u32((V(o[1]) & 0xFF).astype(np.float32)))
        elif op == "v_bfe_u32":
            a, off, width = V(o[1]).astype(np.uint64), V(o[2]) & U32(31), V(o[3]) & U32(31)
            r = (a >> off.astype(np.uint64)) & ((np.uint64(1) << width.astype(np.uint64)) - np.uint64(1))
            self.wv(o[0], r.astype(U32))
        elif op in ("v_lshrrev_b16_e32", "v_lshlrev_b16_e32", "v_add_u16_e32", "v_sub_u16_e32", "v_subrev_u16_e32", "v_mul_lo_u16_e32",
                    "v_max_u16_e32", "v_min_u16_e32"):
            # 16-bit integer ops on the low halves; the high half of the destination becomes zero (gfx9)
            a, b = (V(o[1]) & 0xFFFF).astype(np.int64), (V(o[2]) & 0xFFFF).astype(np.int64)
            r = {"v_lshrrev_b16_e32": lambda: b >> (a & 15), "v_lshlrev_b16_e32": lambda: b << (a & 15), "v_add_u16_e32": lambda: a + b,
                 "v_sub_u16_e32": lambda: a - b, "v_subrev_u16_e32": lambda: b - a, "v_mul_lo_u16_e32": lambda: a * b,
                 "v_max_u16_e32": lambda: np.maximum(a, b), "v_min_u16_e32": lambda: np.minimum(a, b)}[op]()
            self.wv(o[0], (r & 0xFFFF).astype(U32))
        elif op in ("v_mul_f16_e32", "v_add_f16_e32", "v_sub_f16_e32", "v_subrev_f16_e32", "v_max_f16_e32", "v_min_f16_e32"):
            # the low halves; the high half of the destination becomes zero (gfx9: 16-bit vector ops clear it)
            a = (V(o[1]) & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float64)
            b = (V(o[2]) & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float64)
            with np.errstate(all="ignore"):
                r = {"v_mul_f16_e32": a * b, "v_add_f16_e32": a + b, "v_sub_f16_e32": a - b, "v_subrev_f16_e32": b - a,
                     "v_max_f16_e32": np.maximum(a, b), "v_min_f16_e32": np.minimum(a, b)}[op]
            self.wv(o[0], f16_bits(r))
        elif op in ("v_pk_mul_f16", "v_pk_add_f16", "v_pk_fma_f16"):
            # op_sel[i]: the half of source i that feeds the low result; op_sel_hi[i]: the one that feeds the high result
            nsrc = 3 if op == "v_pk_fma_f16" else 2
            if "clamp" in mods:
                raise Fault(f"modifiers of {op} not modelled ({self.who()})")
            neg_lo = [int(x) for x in mods.get("neg_lo", "[0,0,0]").strip("[]").split(",")] + [0, 0, 0]
            neg_hi = [int(x) for x in mods.get("neg_hi", "[0,0,0]").strip("[]").split(",")] + [0, 0, 0]
            sel_lo = [int(x) for x in mods.get("op_sel", "[0,0,0]").strip("[]").split(",")] + [0, 0, 0]
            sel_hi = [int(x) for x in mods.get("op_sel_hi", "[1,1,1]").strip("[]").split(",")] + [1, 1, 1]

            def halves(tok):
                raw = V(tok)
                return ((raw & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float64),
                        (raw >> U32(16)).astype(np.uint16).view(np.float16).astype(np.float64))
            src = [halves(o[1 + q]) for q in range(nsrc)]
            with np.errstate(all="ignore"):
                lo = [src[q][sel_lo[q]] * (-1.0 if neg_lo[q] else 1.0) for q in range(nsrc)]
                hi = [src[q][sel_hi[q]] * (-1.0 if neg_hi[q] else 1.0) for q in range(nsrc)]
            with np.errstate(all="ignore"):
                if op == "v_pk_mul_f16": rl, rh = lo[0] * lo[1], hi[0] * hi[1]
                elif op == "v_pk_add_f16": rl, rh = lo[0] + lo[1], hi[0] + hi[1]
                else: rl, rh = lo[0] * lo[1] + lo[2], hi[0] * hi[1] + hi[2]
            self.wv(o[0], f16_bits(rl) | (f16_bits(rh) << U32(16)))
        elif op == "v_pack_b32_f16":
            self.wv(o[0], (V(o[1]) & U32(0xFFFF)) | ((V(o[2]) & U32(0xFFFF)) << U32(16)))
        elif op == "v_cvt_pk_f16_f32":
            # two fp32 values rounded to nearest even into the halves of one register (gfx950)
            with np.errstate(all="ignore"):
                lo16 = f32(V(o[1])).astype(np.float16).view(np.uint16).astype(U32)
                hi16 = f32(V(o[2])).astype(np.float16).view(np.uint16).astype(U32)
            self.wv(o[0], lo16 | (hi16 << U32(16)))
        elif op in ("v_fma_mixlo_f16", "v_fma_mixhi_f16"):
            # as v_fma_mix_f32 (the sum rounded to fp32), that result then rounded to fp16 and written to one half of the
            # destination (the other kept): the compiler emits it for a half(a * b) with fp32 a and b, which rounds twice
            hi = [int(x) for x in mods.get("op_sel_hi", "[0,0,0]").strip("[]").split(",")]
            lo = [int(x) for x in mods.get("op_sel", "[0,0,0]").strip("[]").split(",")]
            if "neg_" in text or "clamp" in text:
                raise Fault(f"modifiers of {op} not modelled ({self.who()})")
            src = []
            for q in range(3):
                tok = o[1 + q].strip()
                negate = tok.startswith("-") and tok[1:2] in ("v", "s", "|")
                tok = tok[1:] if negate else tok
                absolute = tok.startswith("|") and tok.endswith("|")
                tok = tok[1:-1] if absolute else tok
                raw = V(tok)
                if hi[q]:
                    half = (raw >> U32(16)) if lo[q] else raw
                    val = (half & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float64)
                else:
                    val = f32(raw).astype(np.float64)
                # the modifiers act on the value the selects picked (the sign of the half, not bit 31 of the register)
                val = np.abs(val) if absolute else val
                src.append(-val if negate else val)
            with np.errstate(all="ignore"):
                h = (src[0] * src[1] + src[2]).astype(np.float32).astype(np.float16).view(np.uint16).astype(U32)
            i, _ = self.vreg_index(o[0])
            old_v = self.v[i]
            self.wv(o[0], (old_v & U32(0xFFFF0000)) | h if op == "v_fma_mixlo_f16" else (old_v & U32(0xFFFF)) | (h << U32(16)))
        elif op == "v_fma_mix_f32":
            # a source is fp32, or (its op_sel_hi bit set) the fp16 in the half of the register that op_sel names
            hi = [int(x) for x in mods.get("op_sel_hi", "[0,0,0]").strip("[]").split(",")]
            lo = [int(x) for x in mods.get("op_sel", "[0,0,0]").strip("[]").split(",")]
            if "neg_" in text or "clamp" in text:
                raise Fault(f"modifiers of {op} not modelled ({self.who()})")
            src = []
            for q in range(3):
                tok = o[1 + q].strip()
                negate = tok.startswith("-") and tok[1:2] in ("v", "s", "|")
                tok = tok[1:] if negate else tok
                absolute = tok.startswith("|") and tok.endswith("|")
                tok = tok[1:-1] if absolute else tok
                raw = V(tok)
                if hi[q]:
                    half = (raw >> U32(16)) if lo[q] else raw
                    val = (half & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float64)
                else:
                    val = f32(raw).astype(np.float64)
                # the modifiers act on the value the selects picked (the sign of the half, not bit 31 of the register)
                val = np.abs(val) if absolute else val
                src.append(-val if negate else val)
            with np.errstate(all="ignore"):
                self.wv(o[0], as_u32((src[0] * src[1] + src[2]).astype(np.float32)))
        elif op in ("v_cvt_f32_f16_e32", "v_cvt_f32_f16_sdwa", "v_cvt_f32_f16_e64"):
            tok = o[1]
            absolute, negate = "|" in tok, tok.startswith("-")
            src = V(tok.strip("-|"))
            if absolute:
                src = src & U32(0x7FFF)
            if negate:
                src = src ^ U32(0x8000)
            if op.endswith("_sdwa"):
                how = mods.get("src0_sel", "DWORD")
                if mods.get("dst_sel", "DWORD") != "DWORD" or how not in ("DWORD", "WORD_0", "WORD_1") or "sext" in text:
                    raise Fault(f"operand selects of {op} not modelled ({self.who()})")
                if how == "WORD_1":
                    src = src >> U32(16)
            self.wv(o[0], as_u32((src & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32)))
        elif op == "v_cvt_f16_f32_e32":
            with np.errstate(all="ignore"):
                h = f32(V(o[1])).astype(np.float16).view(np.uint16).astype(U32)
            self.wv(o[0], h)
        elif op in ("v_mbcnt_lo_u32_b32", "v_mbcnt_hi_u32_b32"):
            maskv = S(o[1]) if not o[1].startswith("-") else 0xFFFFFFFF
            base = V(o[2])
            r = np.zeros(64, dtype=U32)
            for k in range(64):
                if op.endswith("lo_u32_b32"):
                    bits = maskv & ((1 << min(k, 32)) - 1)
                else:
                    bits = maskv & ((1 << max(k - 32, 0)) - 1)
                r[k] = (bin(bits).count("1") + int(base[k])) & 0xFFFFFFFF
            self.wv(o[0], r)
        elif op.startswith("v_cmp_"):
            m = re.match(r"v_cmp_(\w+?)_(u32|i32|f32|i64|u64|u16|i16)_(e32|e64)", op)
            if not m:
                raise Fault(f"instruction not modelled: {op} ({self.who()})")
            kind, ty, enc = m.group(1), m.group(2), m.group(3)
            dst, a, b = (o[0], o[1], o[2])
            if ty in ("i64", "u64"):
                A, B = self.v64(a), self.v64(b)
                if ty == "i64":
                    A, B = A.view(np.int64), B.view(np.int64)
            else:
                A, B = V(a), V(b)
            if ty in ("i64", "u64"):
                pass
            elif ty == "i32":
                A, B = A.view(np.int32).astype(np.int64), B.view(np.int32).astype(np.int64)
            elif ty == "u16":
                A, B = (A & 0xFFFF).astype(np.int64), (B & 0xFFFF).astype(np.int64)
            elif ty == "i16":
                A, B = (A & 0xFFFF).astype(np.uint16).view(np.int16).astype(np.int64), (B & 0xFFFF).astype(np.uint16).view(np.int16).astype(np.int64)
            elif ty == "f32":
                A, B = f32(A), f32(B)
            else:
                A, B = A.astype(np.int64), B.astype(np.int64)
            with np.errstate(all="ignore"):
                table = {"eq": A == B, "ne": A != B, "gt": A > B, "ge": A >= B, "lt": A < B, "le": A <= B}
                if ty == "f32":
                    # the negated forms are true when an operand is not a number; lg is "less or greater"
                    table.update({"nlt": ~(A < B), "ngt": ~(A > B), "nge": ~(A >= B), "nle": ~(A <= B), "neq": ~(A == B),
                                  "lg": (A < B) | (A > B), "nlg": ~((A < B) | (A > B)), "o": ~(np.isnan(A) | np.isnan(B)),
                                  "u": np.isnan(A) | np.isnan(B)})
                c = table[kind]
            val = self.mask_to_int(c & self.lanes())
            self.ws(dst, val, 2)
        elif op in ("v_cndmask_b32_e32", "v_cndmask_b32_e64"):
            selm = S(o[3], 2)
            sel = np.array([(selm >> k) & 1 for k in range(64)], dtype=bool)
            self.wv(o[0], np.where(sel, V(o[2]), V(o[1])))
        elif op == "v_cndmask_b32_sdwa":
            # sub-dword operand selects (zero-extended); the whole destination register is written
            def pick(val, how):
                val = val.astype(np.uint64)
                if how == "DWORD":
                    return val
                kind, idx = how.split("_")
                width = 16 if kind == "WORD" else 8
                return (val >> np.uint64(width * int(idx))) & np.uint64((1 << width) - 1)
            if mods.get("dst_sel", "DWORD") != "DWORD" or "sext" in text:
                raise Fault(f"operand selects of {op} not modelled ({self.who()})")
            selm = S(o[3], 2)
            sel = np.array([(selm >> k) & 1 for k in range(64)], dtype=bool)
            a, b = pick(V(o[1]), mods.get("src0_sel", "DWORD")), pick(V(o[2]), mods.get("src1_sel", "DWORD"))
            self.wv(o[0], np.where(sel, b, a).astype(U32))
        elif op in ("v_lshlrev_b32_sdwa", "v_lshrrev_b32_sdwa", "v_or_b32_sdwa", "v_and_b32_sdwa", "v_xor_b32_sdwa", "v_add_u32_sdwa",
                    "v_mul_u32_u24_sdwa", "v_mul_f16_sdwa", "v_add_f16_sdwa", "v_sub_f16_sdwa"):
            # a two-operand op whose sources go through a sub-dword select first (zero-extended) and whose result goes to
            # the selected part of the destination, the rest zero (UNUSED_PAD) or kept (UNUSED_PRESERVE)
            def pick(val, how):
                if how == "DWORD":
                    return val.astype(np.uint64)
                kind, idx = how.split("_")
                width = 16 if kind == "WORD" else 8
                return (val.astype(np.uint64) >> np.uint64(width * int(idx))) & np.uint64((1 << width) - 1)
            unused = mods.get("dst_unused", "UNUSED_PAD")
            if unused not in ("UNUSED_PAD", "UNUSED_PRESERVE") or "sext" in text:
                raise Fault(f"operand selects of {op} not modelled ({self.who()})")
            x, y = pick(V(o[1]), mods.get("src0_sel", "DWORD")), pick(V(o[2]), mods.get("src1_sel", "DWORD"))
            base = op[:-5]
            if base == "v_lshlrev_b32": r = y << (x & np.uint64(31))          # the count is source 0
            elif base == "v_lshrrev_b32": r = y >> (x & np.uint64(31))
            elif base == "v_or_b32": r = x | y
            elif base == "v_and_b32": r = x & y
            elif base == "v_xor_b32": r = x ^ y
            elif base == "v_mul_u32_u24": r = (x & np.uint64(0xFFFFFF)) * (y & np.uint64(0xFFFFFF))
            elif base in ("v_mul_f16", "v_add_f16", "v_sub_f16"):
                hx = (x & np.uint64(0xFFFF)).astype(np.uint16).view(np.float16).astype(np.float64)
                hy = (y & np.uint64(0xFFFF)).astype(np.uint16).view(np.float16).astype(np.float64)
                with np.errstate(all="ignore"):
                    hr = hx * hy if base == "v_mul_f16" else hx + hy if base == "v_add_f16" else hx - hy
                r = f16_bits(hr).astype(np.uint64)
            else: r = x + y
            r = r & np.uint64(0xFFFFFFFF)
            where = mods.get("dst_sel", "DWORD")
            if where != "DWORD":
                kind, idx = where.split("_")
                width = 16 if kind == "WORD" else 8
                field = np.uint64(((1 << width) - 1) << (width * int(idx)))
                r = (r << np.uint64(width * int(idx))) & field
                if unused == "UNUSED_PRESERVE":
                    i, _ = self.vreg_index(o[0])
                    r = r | (self.v[i].astype(np.uint64) & ~field & np.uint64(0xFFFFFFFF))
            self.wv(o[0], r.astype(U32))
        # ---------------------------------------------------------------- LDS
        elif op == "ds_read_b32":
            addr = V(o[1]).astype(np.int64) + int(mods.get("offset", "0"), 0)
            dst, m, who = o[0], self.lanes().copy(), self.who()

            def fn(addr=addr, dst=dst, m=m, who=who):
                i, _ = self.vreg_index(dst)
                for k in range(64):
                    if m[k]:
                        a = int(addr[k])
                        if a + 4 > len(self.lds) * 4 or a % 4:
                            raise Fault(f"LDS read at {a:#x} ({who})")
                        self.v[i][k] = self.lds[a // 4]
            i, _ = self.vreg_index(dst)
            self.v[i][m] = 0xDEADBEEF
            self.lgq.append((self.tick, fn))
        elif op == "ds_bpermute_b32":
            # lane k receives the data register of lane (address / 4) mod 64, or zero when that lane is switched off; the
            # result arrives like an LDS read's (no LDS memory is touched)
            src = (V(o[1]) >> U32(2)) & U32(63)
            data, m, who, dst = V(o[2]).copy(), self.lanes().copy(), self.who(), o[0]

            def fn(src=src, data=data, m=m, dst=dst):
                i, _ = self.vreg_index(dst)
                for k in range(64):
                    if m[k]:
                        self.v[i][k] = data[src[k]] if m[src[k]] else 0
            i, _ = self.vreg_index(dst)
            self.v[i][m] = 0xDEADBEEF
            self.lgq.append((self.tick, fn))
        elif op in ("ds_read_u16", "ds_read_u8"):
            size = 2 if op == "ds_read_u16" else 1
            addr = V(o[1]).astype(np.int64) + int(mods.get("offset", "0"), 0)
            dst, m, who = o[0], self.lanes().copy(), self.who()

            def fn(addr=addr, dst=dst, m=m, who=who, size=size):
                i, _ = self.vreg_index(dst)
                for k in range(64):
                    if m[k]:
                        a = int(addr[k])
                        if a + size > len(self.lds) * 4 or a % size:
                            raise Fault(f"LDS read at {a:#x} ({who})")
                        self.v[i][k] = (int(self.lds[a // 4]) >> (8 * (a % 4))) & ((1 << (8 * size)) - 1)
            i, _ = self.vreg_index(dst)
            self.v[i][m] = 0xDEADBEEF
            self.lgq.append((self.tick, fn))
        elif op in ("ds_write_b32", "ds_add_u32"):
            addr = V(o[0]).astype(np.int64) + int(mods.get("offset", "0"), 0)
            data, m, who = V(o[1]), self.lanes().copy(), self.who()

            def fn(addr=addr, data=data, m=m, who=who, add=(op == "ds_add_u32")):
                for k in range(64):
                    if m[k]:
                        a = int(addr[k])
                        cur = int(self.lds_read32(a)) if add else 0
                        self.lds_write32(a, (cur + int(data[k])) & 0xFFFFFFFF, who)
            self.lgq.append((self.tick, fn))
        elif op == "ds_write2st64_b32":
            addr = V(o[0]).astype(np.int64)
            d0, d1, m, who = V(o[1]), V(o[2]), self.lanes().copy(), self.who()
            o0, o1 = int(mods.get("offset0", "0"), 0) * 256, int(mods.get("offset1", "0"), 0) * 256

            def fn(addr=addr, d0=d0, d1=d1, m=m, who=who, o0=o0, o1=o1):
                for k in range(64):
                    if m[k]:
                        self.lds_write32(int(addr[k]) + o0, int(d0[k]), who)
                        self.lds_write32(int(addr[k]) + o1, int(d1[k]), who)
            self.lgq.append((self.tick, fn))
        # ---------------------------------------------------------------- global memory
        elif op in ("global_load_dwordx4", "global_load_dword", "global_load_dwordx2", "global_load_dwordx3",
                    "flat_load_dwordx4", "flat_load_dword", "flat_load_dwordx2", "flat_load_dwordx3"):
            # a flat load whose address is in global memory is a global load that counts in both counters
            if op.startswith("flat_"):
                self.lgq.append((self.tick, lambda: None))
            n = {"4": 4, "2": 2, "3": 3}.get(op[-1], 1)
            addr = self.global_addr(o[1], o[2] if len(o) > 2 else "off", mods)
            dst, m, who = o[0], self.lanes().copy(), self.who()

            def fn(addr=addr, dst=dst, m=m, who=who, n=n):
                i, _ = self.vreg_index(dst)
                for k in range(64):
                    if m[k]:
                        data = np.frombuffer(self.mem.read(int(addr[k]), 4 * n, who), dtype=U32)
                        for q in range(n):
                            self.v[i + q][k] = data[q]
            # the registers hold garbage until the load lands
            i, _ = self.vreg_index(dst)
            for q in range(n):
                self.v[i + q][m] = 0xBAD00000 + q
            # addresses are checked when the instruction issues
            for k in range(64):
                if m[k]:
                    self.mem.read(int(addr[k]), 4 * n, who)
            self.vmq.append((self.tick, fn))
        elif op in ("global_load_ushort", "global_load_ubyte"):
            size = 2 if op == "global_load_ushort" else 1
            addr = self.global_addr(o[1], o[2] if len(o) > 2 else "off", mods)
            dst, m, who = o[0], self.lanes().copy(), self.who()

            def fn(addr=addr, dst=dst, m=m, who=who, size=size):
                i, _ = self.vreg_index(dst)
                for k in range(64):
                    if m[k]:
                        self.v[i][k] = int.from_bytes(self.mem.read(int(addr[k]), size, who), "little")
            i, _ = self.vreg_index(dst)
            self.v[i][m] = 0xBAD00000
            for k in range(64):
                if m[k]:
                    self.mem.read(int(addr[k]), size, who)
            self.vmq.append((self.tick, fn))
        elif op == "global_load_lds_dword":
            addr = self.global_addr(o[0], o[1] if len(o) > 1 else "off", mods)
            m, who, m0 = self.lanes().copy(), self.who(), self.m0

            def fn(addr=addr, m=m, who=who, m0=m0):
                for k in range(64):
                    if m[k]:
                        val = np.frombuffer(self.mem.read(int(addr[k]), 4, who), dtype=U32)[0]
                        self.lds_write32((m0 & 0x3FFFF) + 4 * k, int(val), who)
            for k in range(64):
                if m[k]:
                    self.mem.read(int(addr[k]), 4, who)
            self.vmq.append((self.tick, fn))
        elif op in ("global_store_dwordx2", "global_store_dwordx3", "global_store_dwordx4"):
            n = int(op[-1])
            addr = self.global_addr(o[0], o[2] if len(o) > 2 else "off", mods)
            i, _ = self.vreg_index(o[1])
            data = np.stack([self.v[i + q].copy() for q in range(n)])
            m, who = self.lanes().copy(), self.who()

            def fn(addr=addr, data=data, m=m, who=who, n=n):
                for k in range(64):
                    if m[k]:
                        self.mem.write(int(addr[k]), b"".join(struct.pack("<I", int(data[q][k])) for q in range(n)), who)
            for k in range(64):
                if m[k]:
                    self.mem.read(int(addr[k]), 4 * n, who)
            self.vmq.append((self.tick, fn))
        elif op in ("global_store_dword", "global_store_short", "global_store_byte"):
            addr = self.global_addr(o[0], o[2] if len(o) > 2 else "off", mods)
            data, m, who = V(o[1]), self.lanes().copy(), self.who()
            size = 4 if op.endswith("dword") else 2 if op.endswith("short") else 1

            def fn(addr=addr, data=data, m=m, who=who, size=size):
                for k in range(64):
                    if m[k]:
                        self.mem.write(int(addr[k]), struct.pack("<I", int(data[k]))[:size], who)
            for k in range(64):
                if m[k]:
                    self.mem.read(int(addr[k]), size, who)
            self.vmq.append((self.tick, fn))
        elif op == "global_atomic_add":
            ret = "sc0" in mods
            if ret:
                dst, a_tok, d_tok, s_tok = o[0], o[1], o[2], o[3] if len(o) > 3 else "off"
            else:
                dst, a_tok, d_tok, s_tok = None, o[0], o[1], o[2] if len(o) > 2 else "off"
            addr = self.global_addr(a_tok, s_tok, mods)
            data, m, who = V(d_tok), self.lanes().copy(), self.who()

            def fn(addr=addr, data=data, m=m, who=who, dst=dst):
                for k in range(64):
                    if m[k]:
                        cur = np.frombuffer(self.mem.read(int(addr[k]), 4, who), dtype=U32)[0]
                        self.mem.write(int(addr[k]), struct.pack("<I", (int(cur) + int(data[k])) & 0xFFFFFFFF), who)
                        if dst is not None:
                            self.v[self.vreg_index(dst)[0]][k] = cur
            self.vmq.append((self.tick, fn))
        elif op in ("buffer_inv", "buffer_wbl2"):
            pass
        elif op in ("ds_read_b64", "ds_read_b128", "ds_read2_b32", "ds_read2_b64", "ds_read2st64_b32"):
            base = V(o[1]).astype(np.int64)
            if op.startswith("ds_read2"):
                unit = (8 if op.endswith("b64") else 4) * (64 if "st64" in op else 1)
                offs = [int(mods.get("offset0", "0"), 0) * unit, int(mods.get("offset1", "0"), 0) * unit]
                words = 2 if op.endswith("b64") else 1
            else:
                offs = [int(mods.get("offset", "0"), 0)]
                words = 2 if op.endswith("b64") else 4
            dst, m, who = o[0], self.lanes().copy(), self.who()
            i, _ = self.vreg_index(dst)
            total = words * len(offs)

            def fn(base=base, i=i, m=m, who=who, offs=offs, words=words):
                for k in range(64):
                    if m[k]:
                        q = 0
                        for off in offs:
                            a = int(base[k]) + off
                            if a + 4 * words > len(self.lds) * 4 or a % (4 * words):
                                raise Fault(f"LDS read at {a:#x} beyond the allocation or misaligned ({who})")
                            for w in range(words):
                                self.v[i + q][k] = self.lds[a // 4 + w]
                                q += 1
            for q in range(total):
                self.v[i + q][m] = 0xDEADBEEF
            self.lgq.append((self.tick, fn))
        elif op in ("ds_write_b64", "ds_write_b128", "ds_write2_b32", "ds_write2_b64"):
            base = V(o[0]).astype(np.int64)
            m, who = self.lanes().copy(), self.who()
            if op.startswith("ds_write2"):
                unit = 8 if op.endswith("b64") else 4
                words = unit // 4
                parts = []
                for tok, key in ((o[1], "offset0"), (o[2], "offset1")):
                    j, _ = self.vreg_index(tok)
                    parts.append((int(mods.get(key, "0"), 0) * unit, [self.v[j + w].copy() for w in range(words)]))
            else:
                words = 2 if op.endswith("b64") else 4
                j, _ = self.vreg_index(o[1])
                parts = [(int(mods.get("offset", "0"), 0), [self.v[j + w].copy() for w in range(words)])]

            def fn(base=base, m=m, who=who, parts=parts):
                for k in range(64):
                    if m[k]:
                        for off, data in parts:
                            if (int(base[k]) + off) % (4 * len(data)):
                                raise Fault(f"LDS write at {int(base[k]) + off:#x} misaligned ({who})")
                            for w, d in enumerate(data):
                                self.lds_write32(int(base[k]) + off + 4 * w, int(d[k]), who)
            self.lgq.append((self.tick, fn))
        elif op in ("s_andn2_b32", "s_orn2_b32", "s_nand_b32", "s_nor_b32"):
            a, b = S(o[1]), S(o[2])
            r = {"s_andn2_b32": a & ~b, "s_orn2_b32": a | ~b, "s_nand_b32": ~(a & b), "s_nor_b32": ~(a | b)}[op] & 0xFFFFFFFF
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op == "v_writelane_b32":
            # one lane of a vector register, whatever the execution mask says
            i, _ = self.vreg_index(o[0])
            self.v[i][S(o[2]) & 63] = S(o[1]) & 0xFFFFFFFF
        elif op == "v_readlane_b32":
            i, _ = self.vreg_index(o[1])
            self.ws(o[0], int(self.v[i][S(o[2]) & 63]), 1)
        elif op == "s_not_b64":
            r = ~S(o[1], 2) & MASK64
            setscc(r != 0)
            self.ws(o[0], r, 2)
        elif op == "s_not_b32":
            r = ~S(o[1]) & 0xFFFFFFFF
            setscc(r != 0)
            self.ws(o[0], r, 1)
        elif op == "s_brev_b32":
            self.ws(o[0], int(format(S(o[1]) & 0xFFFFFFFF, "032b")[::-1], 2), 1)
        elif op == "s_movk_i32":
            v = int(o[1], 0)
            if v & 0x8000 and v > 0: v -= 0x10000
            self.ws(o[0], v & 0xFFFFFFFF, 1)
        elif op == "s_andn2_saveexec_b64":
            old = self.exec
            self.exec = S(o[1], 2) & ~old & MASK64
            setscc(self.exec != 0)
            self.ws(o[0], old, 2)
        elif op == "s_or_saveexec_b64":
            old = self.exec
            self.exec = (S(o[1], 2) | old) & MASK64
            setscc(self.exec != 0)
            self.ws(o[0], old, 2)
        elif op == "v_lshl_or_b32":
            r = (V(o[1]).astype(np.uint64) << (V(o[2]).astype(np.uint64) & np.uint64(31))) | V(o[3]).astype(np.uint64)
            self.wv(o[0], (r & np.uint64(0xFFFFFFFF)).astype(U32))
        elif op == "v_bitop3_b32":
            a, b, c = V(o[1]), V(o[2]), V(o[3])
            tt = int(mods["bitop3"], 0)
            r = np.zeros(64, dtype=U32)
            for idx in range(8):
                if (tt >> idx) & 1:
                    ta = a if idx & 4 else ~a
                    tb = b if idx & 2 else ~b
                    tc = c if idx & 1 else ~c
                    r |= ta & tb & tc
            self.wv(o[0], r)
        elif op == "v_mov_b64_e32":
            self.wv64(o[0], self.v64(o[1]))
        elif op == "v_lshlrev_b64":
            self.wv64(o[0], self.v64(o[2]) << (V(o[1]).astype(np.uint64) & np.uint64(63)))
        elif op in ("v_lshrrev_b64", "v_ashrrev_i64"):
            x = self.v64(o[2])
            sh = V(o[1]).astype(np.uint64) & np.uint64(63)
            self.wv64(o[0], (x >> sh) if op == "v_lshrrev_b64" else (x.view(np.int64) >> sh.astype(np.int64)).view(np.uint64))
        elif op == "v_mad_u32_u24":
            r = (V(o[1]).astype(np.uint64) & np.uint64(0xFFFFFF)) * (V(o[2]).astype(np.uint64) & np.uint64(0xFFFFFF)) + V(o[3]).astype(np.uint64)
            self.wv(o[0], (r & np.uint64(0xFFFFFFFF)).astype(U32))
        elif op == "v_mul_lo_u32":
            self.wv(o[0], ((V(o[1]).astype(np.uint64) * V(o[2]).astype(np.uint64)) & np.uint64(0xFFFFFFFF)).astype(U32))
        elif op == "v_mul_hi_u32":
            self.wv(o[0], ((V(o[1]).astype(np.uint64) * V(o[2]).astype(np.uint64)) >> np.uint64(32)).astype(U32))
        elif op in ("v_min_i32_e32", "v_max_i32_e32"):
            a, b = V(o[1]).view(np.int32), V(o[2]).view(np.int32)
            self.wv(o[0], (np.minimum(a, b) if "min" in op else np.maximum(a, b)).view(U32))
        elif re.match(r"v_(add|sub|subrev)_co_u32_e(32|64)$", op) or re.match(r"v_(addc|subb|subbrev)_co_u32_e(64)$", op) or op in ("v_subb_co_u32_e32", "v_subbrev_co_u32_e32"):
            # D, carry-out, a, b [, carry-in]
            a, b = V(o[2]).astype(np.int64), V(o[3]).astype(np.int64)
            cin = np.zeros(64, dtype=np.int64)
            if len(o) > 4:
                cm = S(o[4], 2)
                cin = np.array([(cm >> k) & 1 for k in range(64)], dtype=np.int64)
            kind = op.split("_")[1]
            if kind in ("add", "addc"):
                r = a + b + cin
                carry = r >> 32 != 0
            elif kind in ("sub", "subb"):
                r = a - b - cin
                carry = r < 0
            else:
                r = b - a - cin
                carry = r < 0
            lanes = self.lanes()
            self.wv(o[0], (r & 0xFFFFFFFF).astype(U32))
            old = S(o[1], 2)
            new = old
            for k in range(64):
                if lanes[k]:
                    new = (new & ~(1 << k)) | (int(carry[k]) << k)
            self.ws(o[1], new, 2)
        else:
            raise Fault(f"instruction not modelled: {op} ({self.who()})")
        self.pc = nxt

    def global_addr(self, v_tok, s_tok, mods):
        off = int(mods.get("offset", "0"), 0)
        i, n = self.vreg_index(v_tok)
        if s_tok != "off" and self.sreg_index(s_tok)[0] is not None:
            base = self.rs(s_tok, 2)
            return (np.uint64(base) + self.v[i].astype(np.uint64) + np.uint64(off & MASK64)) & np.uint64(MASK64)
        a = self.v[i].astype(np.uint64) | (self.v[i + 1].astype(np.uint64) << np.uint64(32))
        return (a + np.uint64(off & MASK64)) & np.uint64(MASK64)


class Kernel:
    """One kernel of an assembly file written by `hipcc -S --cuda-device-only`: its instructions, its descriptor
    (`.amdhsa_*`) and the layout of its arguments (the YAML metadata at the end of the file).

        k = Kernel("matvec.s", "_ZN4rptc18matvec_loop_kernelILi8ELi0ELi3E")
        mem = Memory(); mem.add(address, numpy_uint8_array, "name") ...
        k.launch(mem, grid=(256,), block=1024, args=[("ptr", address), ("i32", 3), ...], lds_bytes=98304, groups=[(0, 0, 0)])
    """

    _files = {}          # path -> (mtime, lines, parsed metadata): an assembly file is read and its metadata parsed once

    @classmethod
    def _file(cls, path):
        import yaml
        mtime = os.path.getmtime(path)
        hit = cls._files.get(path)
        if hit is None or hit[0] != mtime:
            text = open(path).read().split("\n")
            y0 = next(i for i, l in enumerate(text) if l.strip() == ".amdgpu_metadata")
            y1 = next(i for i, l in enumerate(text) if l.strip() == ".end_amdgpu_metadata")
            loader = getattr(yaml, "CSafeLoader", yaml.SafeLoader)
            hit = (mtime, text, yaml.load("\n".join(text[y0 + 1:y1]), Loader=loader))
            cls._files[path] = hit
        return hit[1], hit[2]

    def __init__(self, path, symbol_prefix):
        text, meta = self._file(path)
        start = next(i for i, l in enumerate(text) if l.startswith(symbol_prefix) and re.match(r"^[\w$.]+:", l))
        self.symbol = text[start].split(":")[0]
        end = next(i for i in range(start, len(text)) if text[i].startswith(".Lfunc_end"))
        with tempfile.NamedTemporaryFile("w", suffix=".s", delete=False) as f:
            f.write("\n".join(text[start + 1:end]))
            body = f.name
        ASM_LINES.clear()
        INFO_CACHE.clear()
        try:
            self.insts, self.labels = parse(body)
        finally:
            os.unlink(body)
        # kernel descriptor
        d0 = next(i for i, l in enumerate(text) if l.strip() == ".amdhsa_kernel " + self.symbol)
        self.desc = {}
        for l in text[d0 + 1:]:
            if ".end_amdhsa_kernel" in l:
                break
            k, v = l.split()
            self.desc[k[len(".amdhsa_"):]] = int(v, 0)
        # argument offsets from the metadata
        entry = next(k for k in meta["amdhsa.kernels"] if k[".name"] == self.symbol)
        self.args = [{k[1:]: str(v) for k, v in a.items()} for a in entry[".args"]]
        self.kernarg_size = self.desc["kernarg_size"]

    def kernarg(self, args, grid, block):
        buf = bytearray(max(self.kernarg_size, 8) + 64)
        explicit = [a for a in self.args if not a["value_kind"].startswith("hidden")]
        assert len(explicit) == len(args), (len(explicit), len(args))
        for meta, (kind, val) in zip(explicit, args):
            off, size = int(meta["offset"]), int(meta["size"])
            fmt = {"ptr": "<Q", "i64": "<q", "u64": "<Q", "i32": "<i", "u32": "<I", "f32": "<f"}[kind]
            assert struct.calcsize(fmt) == size, (meta, kind)
            struct.pack_into(fmt, buf, off, val)
        for meta in self.args:
            kind, off = meta["value_kind"], int(meta["offset"])
            if kind.startswith("hidden_block_count_"):
                struct.pack_into("<I", buf, off, grid["xyz".index(kind[-1])])
            elif kind.startswith("hidden_group_size_"):
                struct.pack_into("<H", buf, off, block if kind[-1] == "x" else 1)
            elif kind.startswith("hidden_remainder_"):
                struct.pack_into("<H", buf, off, 0)
            elif kind == "hidden_grid_dims":
                struct.pack_into("<H", buf, off, 3 if grid[2] > 1 else 2 if grid[1] > 1 else 1)
        return bytes(buf)

    def launch(self, mem, grid, block, args, lds_bytes=0, seed=1, groups=None, max_steps=50_000_000, garbage=True,
               kernarg_at=0x7e0000001000, burst=8, barrier_orders_memory=False):
        """Runs the workgroups `groups` (default: the whole grid) one after the other; `args` is a list of (kind, value)
        with kind in ptr, i64, u64, i32, u32, f32; `burst` bounds how many instructions a wave runs before another
        is picked (a large value lets every wave run until it blocks).  Returns the number of instructions executed.

        `barrier_orders_memory`: the vector memory operations of a workgroup's waves pass through their compute unit's
        one memory pipeline in the order they were issued, so a load issued behind a barrier sees a store issued in front
        of it by another wave of the workgroup without any wait for the store; the compiler's workgroup-scope fence
        (`__syncthreads()`) relies on that and emits no `vmcnt` wait.  The model's memory operations complete late and
        wave by wave, which is stricter; with this flag every queued operation of the workgroup completes when a barrier
        opens.  For kernels whose waves hand data to each other through global memory; not for hand-overs between
        workgroups, which need the wait."""
        grid = tuple(grid) + (1,) * (3 - len(grid))
        ka = self.kernarg(args, grid, block)
        mem.add(kernarg_at, np.frombuffer(ka, dtype=np.uint8).copy(), "kernarg")
        d = self.desc
        assert not d.get("user_sgpr_dispatch_ptr") and not d.get("user_sgpr_queue_ptr") and not d.get("user_sgpr_dispatch_id")
        assert d.get("user_sgpr_kernarg_segment_ptr") == 1
        user = d["user_sgpr_count"]
        global GARBAGE
        GARBAGE = garbage
        rng = random.Random(seed)
        total = 0
        # the kernel's static LDS (its `__shared__` variables) comes first, the launch's dynamic LDS behind it
        lds_words = max((self.desc.get("group_segment_fixed_size", 0) + lds_bytes) // 4, 16)
        waves = (block + 63) // 64
        todo = groups if groups is not None else [(x, y, z) for z in range(grid[2]) for y in range(grid[1]) for x in range(grid[0])]
        for (gx, gy, gz) in todo:
            lds = np.zeros(lds_words, dtype=U32)
            if garbage:
                lds[:] = np.random.default_rng(rng.randrange(1 << 30)).integers(0, 1 << 32, lds_words, dtype=np.uint64).astype(U32)
            ws = []
            for w in range(waves):
                wave = Wave((gx, gy, gz), w, self.insts, self.labels, mem, lds, kernarg_at, 0, rng)
                if not garbage:
                    wave.s[15] = 0
                s = user
                for flag, val in (("system_sgpr_workgroup_id_x", gx), ("system_sgpr_workgroup_id_y", gy), ("system_sgpr_workgroup_id_z", gz)):
                    if d.get(flag):
                        wave.s[s] = val
                        s += 1
                wave.s[0], wave.s[1] = kernarg_at & 0xFFFFFFFF, kernarg_at >> 32
                lanes = np.arange(64, dtype=U32) + 64 * w
                wave.v[0] = lanes
                n_active = min(64, block - 64 * w)
                wave.exec = (1 << n_active) - 1
                ws.append(wave)
            steps = 0
            while True:
                live = [w for w in ws if not w.done and not w.at_barrier]
                if not live:
                    if all(w.done for w in ws):
                        break
                    for w in ws:
                        w.at_barrier = False
                        if barrier_orders_memory:
                            w.force_vm(0)
                    continue
                w = rng.choice(live)
                for _ in range(rng.randint(1, burst)):
                    if w.done or w.at_barrier:
                        break
                    with np.errstate(all="ignore"):          # lanes that hold garbage overflow and divide by zero
                        w.step()
                    steps += 1
                if steps > max_steps:
                    raise Fault("step limit: " + "; ".join(f"w{x.wid}@{x.insts[x.pc][3]}" for x in ws if not x.done))
            total += steps
        return total
