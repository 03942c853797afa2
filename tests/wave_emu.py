"""Test infrastructure: an emulator of the part of the gfx950 instruction set the generated wave programs
(jittorinfer_amd/csrc/mla_decode_*.inc) are written in, with the bookkeeping of a hazard checker.

It runs the instruction stream of an inline-asm block for all waves of one workgroup -- scalar and vector ALU, the matrix
instructions, LDS and global memory, the two wait counters and the workgroup barrier -- and while it does so it keeps, per wave,
the queue of memory operations in flight and, per 32-bit word of LDS, who wrote it last and who read it since.  What it reports:

  * a register read (or overwritten) while a load into it is still in flight: the wait in front of the use is missing or counts
    too few operations;
  * an LDS word read by one wave that another wave wrote, without "writer waits for its write, barrier" in between; the mirror
    image for a write over a word another wave has read or written (read -> wait -> barrier -> overwrite); LDS written by a
    tile copy (global_load_lds) counts as written by the wave that issued the copy, complete when that wave's vmcnt wait says so;
  * counted vmcnt waits (vmcnt(N), N > 0) that are only right if vector-memory operations of different kinds (loads into
    registers, copies into LDS, stores) complete in the order they were issued -- which the hardware's counter promises and the
    compiler's own wait insertion relies on, listed so that a reader knows where the programs lean on it;
  * global accesses outside the buffers the scenario handed in.

Values are computed for real (the programs' own outputs can be compared with a float64 attention), so scalar branches follow the
data.  Nothing here is product code: only tests import it."""
import re

import numpy as np

LDS_BYTES = 163840
U32 = np.uint32
F32 = np.float32


class Finding:
    def __init__(self, kind, wave, pc, text, detail):
        self.kind, self.wave, self.pc, self.text, self.detail = kind, wave, pc, text, detail

    def __repr__(self):
        return "%s: wave %d, instruction %d `%s`: %s" % (self.kind, self.wave, self.pc, self.text, self.detail)


# ------------------------------------------------------------------------------------------------------------ parsing
def parse_program(text):
    """The lines of a generated .inc file -> (instructions, labels).  An instruction is (mnemonic, operands, modifiers, text)."""
    instrs, labels = [], {}
    for raw in text.splitlines():
        raw = raw.strip()
        if not raw.startswith('"'):
            continue
        body = raw[1:raw.rindex('"')]
        for ln in body.split("\\n\\t"):
            ln = ln.strip()
            if not ln or ln.startswith(";"):
                continue
            if ln.endswith(":"):
                labels[ln[:-1]] = len(instrs)
                continue
            instrs.append(_parse_instr(ln))
    return instrs, labels


_MOD = re.compile(r"\b(offset|offset0|offset1|dst_sel|dst_unused|src0_sel|src1_sel|op_sel|op_sel_hi):(\[[^\]]*\]|\S+)")
_WAIT = re.compile(r"(vmcnt|lgkmcnt)\((\d+)\)")


def _parse_instr(ln):
    mn, _, rest = ln.partition(" ")
    if mn == "s_waitcnt":
        return (mn, [], {k: int(n) for k, n in _WAIT.findall(rest)}, ln)
    mods = {}
    for k, val in _MOD.findall(rest):
        mods[k] = [int(x) for x in val[1:-1].split(",")] if val.startswith("[") else (int(val, 0) if re.fullmatch(r"-?(0x[0-9a-f]+|\d+)", val) else val)
    rest = _MOD.sub("", rest)
    rest = re.sub(r"\s+(nt|sc0|sc1)\b", "", rest)       # cache-policy hints of loads and stores: nothing the emulator models
    ops = [_parse_operand(x.strip()) for x in _split_operands(rest) if x.strip()]
    return (mn, ops, mods, ln)


def _split_operands(s):
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "[(":
            depth += 1
        elif ch in "])":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    out.append(cur)
    return out


def _parse_operand(x):
    neg = sext = False
    if x.startswith("sext(") and x.endswith(")"):
        sext, x = True, x[5:-1]
    if x.startswith("-") and not re.fullmatch(r"-(\d+|0x[0-9a-f]+|\d+\.\d+)", x):
        neg, x = True, x[1:]
    m = re.fullmatch(r"([vas])(\d+)", x)
    if m:
        return (m.group(1), int(m.group(2)), 1, neg, sext)
    m = re.fullmatch(r"([vas])\[(\d+):(\d+)\]", x)
    if m:
        return (m.group(1), int(m.group(2)), int(m.group(3)) - int(m.group(2)) + 1, neg, sext)
    if x in ("vcc", "exec", "m0", "exec_hi", "exec_lo", "vcc_lo", "vcc_hi", "scc"):
        return (x, 0, 1, neg, sext)
    m = re.fullmatch(r"%\[(\w+)\]", x)
    if m:
        return ("in", m.group(1), 1, neg, sext)
    if re.fullmatch(r"-?\d+\.\d+", x):
        return ("lit", int(np.array([float(x)], dtype=F32).view(U32)[0]), 1, neg, sext)
    if re.fullmatch(r"-?(0x[0-9a-fA-F]+|\d+)", x):
        return ("lit", int(x, 0) & 0xffffffffffffffff, 1, neg, sext)
    return ("label", x, 1, neg, sext)


# ------------------------------------------------------------------------------------------------------------ numerics
def f16_to_f32(h):
    return h.astype(np.uint16).view(np.float16).astype(F32)


def f32_to_f16_rne(x):
    with np.errstate(over="ignore", invalid="ignore"):
        return x.astype(np.float16).view(np.uint16)


def f32_to_f16_rtz(x):
    with np.errstate(over="ignore", invalid="ignore"):
        h = x.astype(np.float16)
        back = h.astype(F32)
        over = np.abs(back) > np.abs(x)                      # rounded away from zero (an overflow to infinity included)
        bits = h.view(np.uint16).copy()
        fix = over & ~np.isnan(x)
        bits[fix] = bits[fix] - 1                            # one step towards zero (inf -> 65504)
        return bits


def f32_to_bf16_rne(x):
    b = x.view(U32).astype(np.uint64)
    r = ((b + 0x7fff + ((b >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    r[nan] = ((b[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_to_f32(h):
    return (h.astype(U32) << 16).view(F32)


# ------------------------------------------------------------------------------------------------------------ memory
class GlobalMemory:
    """Named buffers at addresses of the scenario's choosing; an access outside them is reported and reads as zero."""

    def __init__(self):
        self.bufs = []          # (base, array of uint8, name, writable)

    def add(self, name, arr, base=None, writable=False):
        data = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
        if base is None:
            base = (self.bufs[-1][0] + len(self.bufs[-1][1]) + 0xfffff) & ~0xfffff if self.bufs else 0x7f0000100000
        if writable:
            data = data.copy()
        self.bufs.append((base, data, name, writable))
        return base

    def array(self, name):
        return next(b[1] for b in self.bufs if b[2] == name)

    def _locate(self, addrs, nbytes):
        idx = np.full(len(addrs), -1)
        for k, (base, data, _, _) in enumerate(self.bufs):
            inside = (addrs >= base) & (addrs + nbytes <= base + len(data))
            idx[inside] = k
        return idx

    def read(self, addrs, nbytes, active):
        out = np.zeros((len(addrs), nbytes), np.uint8)
        idx = self._locate(addrs, nbytes)
        bad = active & (idx < 0)
        for k in np.unique(idx[active & (idx >= 0)]):
            base, data = self.bufs[k][0], self.bufs[k][1]
            sel = active & (idx == k)
            off = (addrs[sel] - base).astype(np.int64)
            out[sel] = data[off[:, None] + np.arange(nbytes)]
        return out, bad

    def write(self, addrs, payload, active):
        nbytes = payload.shape[1]
        idx = self._locate(addrs, nbytes)
        bad = active & (idx < 0)
        for k in np.unique(idx[active & (idx >= 0)]):
            base, data, _, writable = self.bufs[k]
            sel = active & (idx == k)
            if not writable:
                bad = bad | sel
                continue
            off = (addrs[sel] - base).astype(np.int64)
            data[off[:, None] + np.arange(nbytes)] = payload[sel]
        return bad


class MemOp:
    __slots__ = ("wave", "kind", "epoch", "done", "pc", "text", "regs", "data", "mask", "mixed")

    def __init__(self, wave, kind, epoch, pc, text):
        self.wave, self.kind, self.epoch, self.pc, self.text = wave, kind, epoch, pc, text
        self.done = None        # the epoch (barriers passed by its wave) in which a wait covered it
        self.regs = None
        self.data = None
        self.mask = None
        self.mixed = False


class Workgroup:
    """The waves of one workgroup, their LDS, and the access history the hazard checks need."""

    def __init__(self, text, n_waves, gmem, inputs, lds_init=None, max_steps=2_000_000):
        self.instrs, self.labels = parse_program(text)
        self.gmem = gmem
        self.lds = np.zeros(LDS_BYTES, np.uint8)
        self.w_op = np.full(LDS_BYTES // 4, -1, np.int64)              # last write of each word: index into self.ops (-2: before the program)
        self.r_op = np.full((LDS_BYTES // 4, n_waves), -1, np.int64)   # last read of each word by each wave
        if lds_init:
            for off, arr in lds_init:
                b = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
                self.lds[off:off + len(b)] = b
                self.w_op[off // 4:(off + len(b) + 3) // 4] = -2
        self.ops = []
        self.findings = []
        self.mixed_waits = {}
        self.waves = [Wave(self, w, inputs(w) if callable(inputs) else inputs) for w in range(n_waves)]
        self.max_steps = max_steps
        self.barriers = 0
        self.branch_handlers = {}       # a test may wrap the conditional branches (coverage)

    def report(self, kind, wave, pc, detail):
        if len(self.findings) < 200:
            self.findings.append(Finding(kind, wave, pc, self.instrs[pc][3], detail))

    def run(self):
        steps = 0
        while True:
            live = [w for w in self.waves if not w.ended]
            if not live:
                break
            for w in live:
                steps += w.run_to_barrier(self.max_steps - steps)
                if steps >= self.max_steps:
                    raise RuntimeError("step limit reached (a loop that does not end?) at pc %d of wave %d" % (w.pc, w.index))
            ended = [w.ended for w in self.waves]
            if any(ended) and not all(ended):
                waiting = [w.index for w in self.waves if not w.ended]
                self.report("barrier", waiting[0], self.waves[waiting[0]].pc - 1, "waves %s wait at a barrier the others never reach" % waiting)
                break
            for w in self.waves:
                w.epoch += 1
            self.barriers += 1
        for w in self.waves:
            if w.vmq or w.lgq:
                self.report("in-flight", w.index, len(self.instrs) - 1, "%d vector-memory and %d LDS operations in flight at the end" % (len(w.vmq), len(w.lgq)))
        return self.findings

    # ---- LDS history
    def lds_read_check(self, wave, words, pc):
        wv = self.waves[wave]
        for oid in np.unique(self.w_op[words]):
            if oid < 0:
                continue
            x = self.ops[oid]
            if x.wave == wave:
                if x.kind == "dma" and x.done is None:
                    self.report("lds-raw", wave, pc, "reads LDS its own tile copy (instruction %d) may not have filled yet: no vmcnt wait in between" % x.pc)
            elif x.done is None or x.done >= wv.epoch:
                self.report("lds-raw", wave, pc, "reads LDS that wave %d writes (instruction %d `%s`, %s) without wait + barrier in between"
                            % (x.wave, x.pc, x.text, "never waited for" if x.done is None else "waited for after the last barrier"))

    def lds_write_check(self, wave, words, pc, kind):
        wv = self.waves[wave]
        for oid in np.unique(self.w_op[words]):
            if oid < 0:
                continue
            x = self.ops[oid]
            if x.wave == wave:
                if x.kind != kind and x.done is None:
                    self.report("lds-waw", wave, pc, "overwrites LDS its own %s (instruction %d) may not have written yet" % (x.kind, x.pc))
            elif x.done is None or x.done >= wv.epoch:
                self.report("lds-waw", wave, pc, "overwrites LDS that wave %d writes (instruction %d) without wait + barrier in between" % (x.wave, x.pc))
        for u in range(len(self.waves)):
            for oid in np.unique(self.r_op[words, u]):
                if oid < 0:
                    continue
                x = self.ops[oid]
                if u == wave:
                    if kind == "dma" and x.done is None:
                        self.report("lds-war", wave, pc, "a tile copy overwrites LDS the wave's own read (instruction %d) has not been waited for" % x.pc)
                elif x.done is None or x.done >= wv.epoch:
                    self.report("lds-war", wave, pc, "overwrites LDS that wave %d reads (instruction %d `%s`, %s) without wait + barrier in between"
                                % (u, x.pc, x.text, "never waited for" if x.done is None else "waited for after the last barrier"))


def _bits(mask):
    return np.array([(mask >> i) & 1 for i in range(64)], dtype=bool)


LANES = np.arange(64)


class Wave:
    def __init__(self, wg, index, inputs):
        self.wg, self.index, self.inputs = wg, index, inputs
        self.v = np.zeros((256, 64), U32)
        self.a = np.zeros((256, 64), U32)
        self.s = np.zeros(128, U32)
        self.v_pending = np.full(256, -1, np.int64)     # the memory operation that will write the register
        self.a_pending = np.full(256, -1, np.int64)
        self.vcc = 0
        self.exec = (1 << 64) - 1
        self.em = _bits(self.exec)
        self.scc = 0
        self.m0 = 0
        self.pc = 0
        self.epoch = 0
        self.ended = False
        self.vmq, self.lgq = [], []
        self.executed = 0
        self.s_poison = {}      # scalar registers that hold a lane of a vector register whose load was still in flight

    # ---- operand access
    def set_exec(self, val):
        self.exec = val & ((1 << 64) - 1)
        self.em = _bits(self.exec)

    def _use_v(self, file, idx, n, write):
        pend = self.v_pending if file == "v" else self.a_pending
        for r in range(idx, idx + n):
            oid = pend[r]
            if oid >= 0:
                x = self.wg.ops[oid]
                self.wg.report("reg-waw" if write else "reg-raw", self.index, self.pc,
                               "%s%d is %s while the load of instruction %d `%s` into it is in flight" % (file, r, "written" if write else "read", x.pc, x.text))
                self._deliver(x)

    def rs(self, op, width=1):
        """Scalar source as a Python integer (width 2: 64 bits)."""
        k = op[0]
        if k == "s":
            for r in range(op[1], op[1] + width):
                if r in self.s_poison:
                    self.wg.report("reg-raw", self.index, self.pc, "s%d holds a lane of a register read while its load was in flight (%s)" % (r, self.s_poison.pop(r)))
            return int(self.s[op[1]]) | (int(self.s[op[1] + 1]) << 32 if width == 2 else 0)
        if k == "lit":
            return op[1] & (0xffffffff if width == 1 else 0xffffffffffffffff)   # (negative literals were sign-extended to 64 bits when parsed)
        if k == "vcc":
            return self.vcc if width == 2 else self.vcc & 0xffffffff
        if k == "exec":
            return self.exec if width == 2 else self.exec & 0xffffffff
        if k == "m0":
            return self.m0
        if k == "in":
            val = self.inputs[op[1]]
            return int(val) & (0xffffffffffffffff if width == 2 else 0xffffffff)
        raise ValueError("scalar source %r" % (op,))

    def ws(self, op, val, width=1):
        k = op[0]
        if k == "s":
            self.s[op[1]] = val & 0xffffffff
            self.s_poison.pop(op[1], None)
            if width == 2:
                self.s[op[1] + 1] = (val >> 32) & 0xffffffff
                self.s_poison.pop(op[1] + 1, None)
        elif k == "vcc":
            self.vcc = val & ((1 << 64) - 1)
        elif k == "exec":
            self.set_exec(val)
        elif k == "exec_hi":
            self.set_exec((self.exec & 0xffffffff) | ((val & 0xffffffff) << 32))
        elif k == "exec_lo":
            self.set_exec((self.exec & ~0xffffffff) | (val & 0xffffffff))
        elif k == "m0":
            self.m0 = val & 0xffffffff
        else:
            raise ValueError("scalar destination %r" % (op,))

    def rv(self, op, word=0):
        """Vector source as uint32[64] (register `word` of a register group)."""
        k = op[0]
        if k in ("v", "a"):
            self._use_v(k, op[1] + word, 1, False)
            val = (self.v if k == "v" else self.a)[op[1] + word]
        elif k == "in":
            val = np.asarray(self.inputs[op[1]])
            val = np.broadcast_to(val.astype(np.int64).astype(U32) if val.ndim else U32(int(val) & 0xffffffff), (64,))
        else:
            val = np.full(64, self.rs(op) & 0xffffffff, U32)
        return val

    def rvf(self, op):
        x = self.rv(op).view(F32)        # (an integer inline constant in a float instruction is its bit pattern)
        return -x if op[3] else x

    def wv(self, op, val, word=0):
        self._use_v(op[0], op[1] + word, 1, True)
        reg = (self.v if op[0] == "v" else self.a)[op[1] + word]
        val = np.asarray(val)
        assert val.dtype == U32 and val.shape == (64,), (val.dtype, val.shape)
        reg[self.em] = val[self.em]

    def wvcc(self, cond):
        bits = cond & self.em
        self.vcc = int(sum(1 << int(i) for i in np.nonzero(bits)[0]))

    # ---- memory operations in flight
    def _issue(self, kind, queue, regs=None, data=None, mask=None):
        op = MemOp(self.index, kind, self.epoch, self.pc, self.wg.instrs[self.pc][3])
        op.regs, op.data, op.mask = regs, data, mask
        self.wg.ops.append(op)
        oid = len(self.wg.ops) - 1
        if regs:
            file, idx, n = regs
            self._use_v(file, idx, n, True)
            (self.v_pending if file == "v" else self.a_pending)[idx:idx + n] = oid
        queue.append(oid)
        return oid

    def _deliver(self, x):
        if x.regs and x.data is not None:
            file, idx, n = x.regs
            pend = self.v_pending if file == "v" else self.a_pending
            regs = self.v if file == "v" else self.a
            for k in range(n):
                regs[idx + k][x.mask] = x.data[k][x.mask]
            pend[idx:idx + n] = -1
            x.data = None

    def _wait(self, queue, n):
        if len(queue) <= n:
            return
        done, keep = queue[:len(queue) - n], queue[len(queue) - n:]
        if queue is self.vmq and n > 0:
            kinds_after = [self.wg.ops[o].kind for o in queue]
            for i, oid in enumerate(done):
                kind = self.wg.ops[oid].kind
                if sum(1 for k in kinds_after[i:] if k == kind) <= n:
                    self.wg.mixed_waits.setdefault(self.pc, set()).add((kind, tuple(sorted(set(kinds_after[len(done):])))))
                    self.wg.ops[oid].mixed = True
        for oid in done:
            x = self.wg.ops[oid]
            x.done = self.epoch
            self._deliver(x)
        del queue[:len(queue) - n]

    # ---- execution
    def run_to_barrier(self, budget):
        n = 0
        instrs = self.wg.instrs
        while not self.ended and n < budget:
            if self.pc >= len(instrs):
                self.ended = True
                break
            mn, ops, mods, text = instrs[self.pc]
            n += 1
            if mn == "s_barrier":
                self.pc += 1
                break
            h = self.wg.branch_handlers.get(mn) or HANDLERS.get(mn)
            if h is None:
                raise NotImplementedError("instruction %d: %s" % (self.pc, text))
            jump = h(self, ops, mods)
            if jump is None:
                self.pc += 1
            else:
                self.pc = jump
        self.executed += n
        return n


HANDLERS = {}


def op(*names):
    def deco(fn):
        for nm in names:
            HANDLERS[nm] = fn
        return fn
    return deco


def _s32(x):
    x &= 0xffffffff
    return x - (1 << 32) if x >> 31 else x


# ---- scalar ALU
@op("s_nop", "s_memtime")
def _(w, o, m):
    return None


@op("s_waitcnt")
def _(w, o, m):
    if "vmcnt" in m:
        w._wait(w.vmq, m["vmcnt"])
    if "lgkmcnt" in m:
        w._wait(w.lgq, m["lgkmcnt"])


@op("s_mov_b32")
def _(w, o, m):
    w.ws(o[0], w.rs(o[1]))


@op("s_mov_b64")
def _(w, o, m):
    w.ws(o[0], w.rs(o[1], 2), 2)


@op("s_add_u32")
def _(w, o, m):
    r = w.rs(o[1]) + w.rs(o[2])
    w.scc = r >> 32
    w.ws(o[0], r)


@op("s_addc_u32")
def _(w, o, m):
    r = w.rs(o[1]) + w.rs(o[2]) + w.scc
    w.scc = r >> 32
    w.ws(o[0], r)


@op("s_sub_u32")
def _(w, o, m):
    x, y = w.rs(o[1]), w.rs(o[2])
    w.scc = 1 if y > x else 0
    w.ws(o[0], x - y)


@op("s_subb_u32")
def _(w, o, m):
    x, y = w.rs(o[1]), w.rs(o[2]) + w.scc
    w.scc = 1 if y > x else 0
    w.ws(o[0], x - y)


@op("s_sub_i32")
def _(w, o, m):
    r = _s32(w.rs(o[1])) - _s32(w.rs(o[2]))
    w.scc = 1 if not -(1 << 31) <= r < (1 << 31) else 0
    w.ws(o[0], r)


@op("s_mul_i32")
def _(w, o, m):
    w.ws(o[0], w.rs(o[1]) * w.rs(o[2]))


@op("s_mul_hi_u32")
def _(w, o, m):
    w.ws(o[0], (w.rs(o[1]) * w.rs(o[2])) >> 32)


def _logic(fn, width=1):
    def h(w, o, m):
        r = fn(w.rs(o[1], width), w.rs(o[2], width)) & ((1 << (32 * width)) - 1)
        w.scc = 1 if r else 0
        w.ws(o[0], r, width)
    return h


HANDLERS["s_lshl_b32"] = _logic(lambda x, y: x << (y & 31))
HANDLERS["s_lshr_b32"] = _logic(lambda x, y: x >> (y & 31))
HANDLERS["s_and_b32"] = _logic(lambda x, y: x & y)
HANDLERS["s_and_b64"] = _logic(lambda x, y: x & y, 2)


def _minmax(pick, signed):
    def h(w, o, m):
        x, y = w.rs(o[1]), w.rs(o[2])
        kx, ky = (_s32(x), _s32(y)) if signed else (x, y)
        first = pick(kx, ky) == kx
        w.scc = 1 if first else 0
        w.ws(o[0], x if first else y)
    return h


HANDLERS["s_min_u32"] = _minmax(min, False)
HANDLERS["s_min_i32"] = _minmax(min, True)
HANDLERS["s_max_i32"] = _minmax(max, True)


@op("s_cselect_b32")
def _(w, o, m):
    w.ws(o[0], w.rs(o[1]) if w.scc else w.rs(o[2]))     # (only the operand taken is read)


def _scmp(fn, width=1, signed=False):
    def h(w, o, m):
        x, y = w.rs(o[0], width), w.rs(o[1], width)
        if signed:
            x, y = _s32(x), _s32(y)
        w.scc = 1 if fn(x, y) else 0
    return h


HANDLERS["s_cmp_eq_u32"] = _scmp(lambda x, y: x == y)
HANDLERS["s_cmp_lg_u32"] = _scmp(lambda x, y: x != y)
HANDLERS["s_cmp_ge_u32"] = _scmp(lambda x, y: x >= y)
HANDLERS["s_cmp_lt_u32"] = _scmp(lambda x, y: x < y)
HANDLERS["s_cmp_eq_u64"] = _scmp(lambda x, y: x == y, 2)
HANDLERS["s_cmp_lg_u64"] = _scmp(lambda x, y: x != y, 2)


@op("s_bitcmp1_b32")
def _(w, o, m):
    w.scc = (w.rs(o[0]) >> (w.rs(o[1]) & 31)) & 1


@op("s_branch")
def _(w, o, m):
    return w.wg.labels[o[0][1]]


@op("s_cbranch_scc1")
def _(w, o, m):
    return w.wg.labels[o[0][1]] if w.scc else None


@op("s_cbranch_scc0")
def _(w, o, m):
    return None if w.scc else w.wg.labels[o[0][1]]


# ---- vector ALU, integer
def _vbin(fn):
    def h(w, o, m):
        with np.errstate(over="ignore"):
            w.wv(o[0], fn(w.rv(o[1]), w.rv(o[2])).astype(U32))
    return h


HANDLERS["v_add_u32"] = _vbin(lambda x, y: x + y)
HANDLERS["v_sub_u32"] = _vbin(lambda x, y: x - y)
HANDLERS["v_subrev_u32"] = _vbin(lambda x, y: y - x)
HANDLERS["v_and_b32"] = _vbin(lambda x, y: x & y)
HANDLERS["v_or_b32"] = _vbin(lambda x, y: x | y)
HANDLERS["v_lshlrev_b32"] = _vbin(lambda x, y: y << (x & 31))
HANDLERS["v_lshrrev_b32"] = _vbin(lambda x, y: y >> (x & 31))
HANDLERS["v_min_u32"] = _vbin(np.minimum)
HANDLERS["v_max_i32"] = _vbin(lambda x, y: np.maximum(x.view(np.int32), y.view(np.int32)).view(U32))
HANDLERS["v_min_i32"] = _vbin(lambda x, y: np.minimum(x.view(np.int32), y.view(np.int32)).view(U32))
HANDLERS["v_mul_lo_u32"] = _vbin(lambda x, y: (x.astype(np.uint64) * y.astype(np.uint64)).astype(U32))


@op("v_mov_b32")
def _(w, o, m):
    w.wv(o[0], w.rv(o[1]).copy())


@op("v_accvgpr_read_b32", "v_accvgpr_write_b32")
def _(w, o, m):
    w.wv(o[0], w.rv(o[1]).copy())


@op("v_mad_u32_u24")
def _(w, o, m):
    x, y, z = (w.rv(o[k]).astype(np.uint64) for k in (1, 2, 3))
    w.wv(o[0], ((x & 0xffffff) * (y & 0xffffff) + z).astype(U32))


@op("v_bfe_u32")
def _(w, o, m):
    x, off, width = w.rv(o[1]), w.rv(o[2]) & 31, w.rv(o[3]) & 31
    w.wv(o[0], ((x >> off) & ((U32(1) << width) - U32(1))).astype(U32))


@op("v_lshl_or_b32")
def _(w, o, m):
    w.wv(o[0], ((w.rv(o[1]) << (w.rv(o[2]) & 31)) | w.rv(o[3])).astype(U32))


@op("v_or3_b32")
def _(w, o, m):
    w.wv(o[0], w.rv(o[1]) | w.rv(o[2]) | w.rv(o[3]))


@op("v_perm_b32")
def _(w, o, m):
    src = np.concatenate([w.rv(o[2]).view(np.uint8).reshape(64, 4), w.rv(o[1]).view(np.uint8).reshape(64, 4)], axis=1)   # bytes 0-3: src1, 4-7: src0
    sel = w.rv(o[3]).view(np.uint8).reshape(64, 4)
    assert (sel < 8).all(), "v_perm_b32 selector beyond the plain byte picks"
    w.wv(o[0], np.take_along_axis(src, sel.astype(np.int64), axis=1).copy().view(U32).reshape(64))


@op("v_alignbyte_b32")
def _(w, o, m):
    wide = (w.rv(o[1]).astype(np.uint64) << 32) | w.rv(o[2]).astype(np.uint64)
    w.wv(o[0], (wide >> ((w.rv(o[3]).astype(np.uint64) & 3) * 8)).astype(U32))


def _sel(x, sel, sext=False):
    if sel == "DWORD":
        return x
    kind, n = sel.split("_")
    n = int(n)
    if kind == "WORD":
        r = (x >> (16 * n)) & 0xffff
        return ((r ^ 0x8000) - 0x8000).astype(np.int64) if sext else r
    r = (x >> (8 * n)) & 0xff
    return ((r.astype(np.int64) ^ 0x80) - 0x80) if sext else r


def _sdwa_dst(w, o, m, val16):
    k = int(m["dst_sel"].split("_")[1])
    old = w.rv(o[0]) if m["dst_unused"] == "UNUSED_PRESERVE" else np.zeros(64, U32)
    keep = U32(0xffff0000) if k == 0 else U32(0x0000ffff)
    w.wv(o[0], ((old & keep) | (val16.astype(U32) << (16 * k))).astype(U32))


@op("v_min_u32_sdwa")
def _(w, o, m):
    w.wv(o[0], np.minimum(_sel(w.rv(o[1]), m["src0_sel"]), _sel(w.rv(o[2]), m["src1_sel"])).astype(U32))


@op("v_cvt_f16_i16_sdwa")
def _(w, o, m):
    x = _sel(w.rv(o[1]), m["src0_sel"], sext=o[1][4])
    _sdwa_dst(w, o, m, x.astype(np.float16).view(np.uint16))


@op("v_cvt_f32_f16_sdwa")
def _(w, o, m):
    w.wv(o[0], f16_to_f32(_sel(w.rv(o[1]), m["src0_sel"])).view(U32))


@op("v_mbcnt_lo_u32_b32")
def _(w, o, m):
    mask = w.rs(o[1]) & 0xffffffff if o[1][0] != "lit" else o[1][1] & 0xffffffff
    cnt = np.array([bin(mask & ((1 << min(l, 32)) - 1)).count("1") for l in range(64)], U32)
    w.wv(o[0], cnt + w.rv(o[2]))


@op("v_mbcnt_hi_u32_b32")
def _(w, o, m):
    mask = w.rs(o[1]) & 0xffffffff if o[1][0] != "lit" else o[1][1] & 0xffffffff
    cnt = np.array([bin(mask & ((1 << max(l - 32, 0)) - 1)).count("1") for l in range(64)], U32)
    w.wv(o[0], cnt + w.rv(o[2]))


@op("v_readlane_b32")
def _(w, o, m):
    oid = w.v_pending[o[1][1]] if o[1][0] == "v" else -1
    if oid >= 0:            # the value is unknown; the program may still throw it away (a select that takes the other operand)
        w.ws(o[0], 0xdeadbeef)
        w.s_poison[o[0][1]] = "instruction %d `%s`" % (w.pc, w.wg.instrs[w.pc][3])
        return
    w.ws(o[0], int(w.rv(o[1])[w.rs(o[2]) & 63]))


@op("v_readfirstlane_b32")
def _(w, o, m):
    lane = int(np.nonzero(w.em)[0][0]) if w.exec else 0
    w.ws(o[0], int(w.rv(o[1])[lane]))


@op("v_permlane32_swap_b32")
def _(w, o, m):
    x, y = w.rv(o[0]).copy(), w.rv(o[1]).copy()
    x2, y2 = x.copy(), y.copy()
    x2[32:], y2[:32] = y[:32], x[32:]
    w.wv(o[0], x2)
    w.wv(o[1], y2)


def _vcmp(fn, view=None):
    def h(w, o, m):
        x, y = w.rv(o[1]), w.rv(o[2])
        if view is not None:
            x, y = x.view(view), y.view(view)
        with np.errstate(invalid="ignore"):
            w.wvcc(fn(x, y))
    return h


HANDLERS["v_cmp_gt_u32"] = _vcmp(lambda x, y: x > y)
HANDLERS["v_cmp_le_u32"] = _vcmp(lambda x, y: x <= y)
HANDLERS["v_cmp_ne_u32"] = _vcmp(lambda x, y: x != y)
HANDLERS["v_cmp_gt_i32"] = _vcmp(lambda x, y: x > y, np.int32)
HANDLERS["v_cmp_gt_f32"] = _vcmp(lambda x, y: x > y, F32)
HANDLERS["v_cmp_eq_f32"] = _vcmp(lambda x, y: x == y, F32)


@op("v_cmp_ne_u64")
def _(w, o, m):
    lo, hi = w.rv(o[2], 0), w.rv(o[2], 1)
    w.wvcc(((lo.astype(np.uint64) | (hi.astype(np.uint64) << 32)) != np.uint64(w.rs(o[1], 2))))


@op("v_cmp_class_f32")
def _(w, o, m):
    x = w.rv(o[1]).view(F32)
    mask = w.rs(o[2])
    sign = np.signbit(x)
    with np.errstate(invalid="ignore"):
        cls = np.where(np.isnan(x), 1, np.where(np.isinf(x), np.where(sign, 2, 9), np.where(x == 0, np.where(sign, 5, 6),
                       np.where(np.abs(x) < np.finfo(F32).tiny, np.where(sign, 4, 7), np.where(sign, 3, 8)))))
    w.wvcc(((mask >> cls) & 1).astype(bool))


@op("v_cndmask_b32", "v_cndmask_b32_e64")
def _(w, o, m):
    sel = _bits(w.rs(o[3], 2))
    a0 = w.rv(o[1]) if o[1][0] != "lit" else np.full(64, o[1][1] & 0xffffffff, U32)
    a1 = w.rv(o[2]) if o[2][0] != "lit" else np.full(64, o[2][1] & 0xffffffff, U32)
    w.wv(o[0], np.where(sel, a1, a0).astype(U32))


@op("v_add_co_u32")
def _(w, o, m):
    r = w.rv(o[2]).astype(np.uint64) + w.rv(o[3]).astype(np.uint64)
    w.wvcc((r >> 32).astype(bool))
    w.wv(o[0], r.astype(U32))


@op("v_addc_co_u32")
def _(w, o, m):
    r = w.rv(o[2]).astype(np.uint64) + w.rv(o[3]).astype(np.uint64) + _bits(w.rs(o[4], 2)).astype(np.uint64)
    w.wvcc((r >> 32).astype(bool))
    w.wv(o[0], r.astype(U32))


# ---- vector ALU, floating point
def _fbin(fn):
    def h(w, o, m):
        with np.errstate(all="ignore"):
            w.wv(o[0], fn(w.rvf(o[1]), w.rvf(o[2])).astype(F32).view(U32))
    return h


HANDLERS["v_mul_f32"] = _fbin(lambda x, y: x * y)
HANDLERS["v_add_f32"] = _fbin(lambda x, y: x + y)
HANDLERS["v_sub_f32"] = _fbin(lambda x, y: x - y)
HANDLERS["v_max_f32"] = _fbin(np.fmax)


@op("v_max3_f32")
def _(w, o, m):
    w.wv(o[0], np.fmax(np.fmax(w.rvf(o[1]), w.rvf(o[2])), w.rvf(o[3])).view(U32))


@op("v_fma_f32")
def _(w, o, m):
    with np.errstate(all="ignore"):
        r = w.rvf(o[1]).astype(np.float64) * w.rvf(o[2]).astype(np.float64) + w.rvf(o[3]).astype(np.float64)
        w.wv(o[0], r.astype(F32).view(U32))


@op("v_exp_f32")
def _(w, o, m):
    with np.errstate(all="ignore"):
        w.wv(o[0], np.exp2(w.rvf(o[1]).astype(np.float64)).astype(F32).view(U32))


@op("v_rcp_f32")
def _(w, o, m):
    with np.errstate(all="ignore"):
        w.wv(o[0], (1.0 / w.rvf(o[1]).astype(np.float64)).astype(F32).view(U32))


@op("v_cvt_pk_f16_f32")
def _(w, o, m):
    w.wv(o[0], f32_to_f16_rne(w.rvf(o[1])).astype(U32) | (f32_to_f16_rne(w.rvf(o[2])).astype(U32) << 16))


@op("v_cvt_pkrtz_f16_f32")
def _(w, o, m):
    w.wv(o[0], f32_to_f16_rtz(w.rvf(o[1])).astype(U32) | (f32_to_f16_rtz(w.rvf(o[2])).astype(U32) << 16))


@op("v_cvt_pk_bf16_f32")
def _(w, o, m):
    w.wv(o[0], f32_to_bf16_rne(w.rvf(o[1])).astype(U32) | (f32_to_bf16_rne(w.rvf(o[2])).astype(U32) << 16))


@op("v_dot2_f32_f16")
def _(w, o, m):
    x, y = w.rv(o[1]), w.rv(o[2])
    acc = w.rvf(o[3]).astype(np.float64)
    r = acc + f16_to_f32(x & 0xffff).astype(np.float64) * f16_to_f32(y & 0xffff) + f16_to_f32(x >> 16).astype(np.float64) * f16_to_f32(y >> 16)
    w.wv(o[0], r.astype(F32).view(U32))


@op("v_fma_mix_f32")
def _(w, o, m):
    src = []
    for k in range(3):
        x = w.rv(o[1 + k])
        if m["op_sel_hi"][k]:
            x = f16_to_f32((x >> 16) if m["op_sel"][k] else (x & 0xffff))
        else:
            x = x.view(F32)
        src.append(x.astype(np.float64))
    with np.errstate(all="ignore"):
        w.wv(o[0], (src[0] * src[1] + src[2]).astype(F32).view(U32))


@op("v_pk_mul_f16")
def _(w, o, m):
    x, y = w.rv(o[1]), w.rv(o[2])
    with np.errstate(all="ignore"):
        lo = (f16_to_f32(x & 0xffff) * f16_to_f32(y & 0xffff)).astype(np.float16).view(np.uint16)
        hi = (f16_to_f32(x >> 16) * f16_to_f32(y >> 16)).astype(np.float16).view(np.uint16)
    w.wv(o[0], lo.astype(U32) | (hi.astype(U32) << 16))


# ---- matrix instructions: D[i][j] = C[i][j] + sum over (g, e) of A[lane (i, g)][e] * B[lane (j, g)][e];
# lane l = 32 g + i (or j) holds eight 16-bit elements in four registers; D register r of lane l is row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32
def _mfma(to_f32):
    rows = (8 * (np.arange(16)[:, None] // 4) + 4 * (LANES[None, :] // 32) + np.arange(16)[:, None] % 4)     # [r][lane]
    cols = np.broadcast_to(LANES[None, :] % 32, (16, 64))

    def h(w, o, m):
        def operand(opd):
            regs = np.stack([w.rv(opd, k) for k in range(4)], axis=1)                  # [lane][4]
            halves = np.stack([regs & 0xffff, regs >> 16], axis=2).reshape(64, 8)       # [lane][8]
            return to_f32(halves.astype(np.uint16)).astype(np.float64).reshape(2, 32, 8)   # [g][i][e]
        A, B = operand(o[1]), operand(o[2])
        prod = np.einsum("gie,gje->ij", A, B)
        if o[3][0] == "lit":
            C = np.zeros((16, 64))
        else:
            C = np.stack([w.rv(o[3], r).view(F32) for r in range(16)]).astype(np.float64)
        with np.errstate(all="ignore"):
            D = (C + prod[rows, cols]).astype(F32)
        for r in range(16):
            w.wv(o[0], D[r].view(U32), r)
    return h


HANDLERS["v_mfma_f32_32x32x16_f16"] = _mfma(f16_to_f32)
HANDLERS["v_mfma_f32_32x32x16_bf16"] = _mfma(bf16_to_f32)


# ---- LDS
def _lds_words(addr, nbytes, active):
    a = addr[active].astype(np.int64)
    return np.unique(((a[:, None] + np.arange(0, nbytes, 4)) // 4).reshape(-1))


def _lds_read(w, o, nbytes, offsets, transform=None):
    wg = w.wg
    base = w.rv(o[1]).astype(np.int64)
    n_regs = (nbytes * len(offsets) + 3) // 4
    chunks = []
    for off in offsets:
        addr = base + off
        if (addr[w.em] + nbytes > LDS_BYTES).any():
            wg.report("lds-oob", w.index, w.pc, "LDS read beyond %d bytes" % LDS_BYTES)
            addr = np.minimum(addr, LDS_BYTES - nbytes)
        words = _lds_words(addr, nbytes, w.em)
        wg.lds_read_check(w.index, words, w.pc)
        chunks.append((addr, words, wg.lds[addr[:, None] + np.arange(nbytes)]))
    raw = np.concatenate([c[2] for c in chunks], axis=1)
    if raw.shape[1] % 4:
        raw = np.concatenate([raw, np.zeros((64, 4 - raw.shape[1] % 4), np.uint8)], axis=1)
    regs = np.ascontiguousarray(raw).view(U32).reshape(64, n_regs)
    if transform:
        regs = transform(regs, w.em)
    oid = w._issue("ds_read", w.lgq, regs=(o[0][0], o[0][1], n_regs), data=[regs[:, k].copy() for k in range(n_regs)], mask=w.em.copy())
    for _, words, _ in chunks:
        wg.r_op[words, w.index] = oid


def _tr_b16(regs, em):
    """ds_read_b64_tr_b16: inside each block of 16 lanes, lane i receives element i % 4 of the four lanes 4 e + i / 4, e = 0..3."""
    halves = np.stack([regs & 0xffff, regs >> 16], axis=2).reshape(64, 4)
    out = np.zeros_like(halves)
    for blk in range(4):
        h = halves[16 * blk:16 * blk + 16]
        i = np.arange(16)
        for e_ in range(4):
            out[16 * blk + i, e_] = h[4 * e_ + i // 4, i % 4]
    return (out[:, 0::2] | (out[:, 1::2] << 16)).astype(U32)


@op("ds_read_b128")
def _(w, o, m):
    _lds_read(w, o, 16, [m.get("offset", 0)])


@op("ds_read_b64")
def _(w, o, m):
    _lds_read(w, o, 8, [m.get("offset", 0)])


@op("ds_read_b32")
def _(w, o, m):
    _lds_read(w, o, 4, [m.get("offset", 0)])


@op("ds_read_u16")
def _(w, o, m):
    _lds_read(w, o, 2, [m.get("offset", 0)])


@op("ds_read2_b32")
def _(w, o, m):
    _lds_read(w, o, 4, [4 * m.get("offset0", 0), 4 * m.get("offset1", 0)])


@op("ds_read_b64_tr_b16")
def _(w, o, m):
    _lds_read(w, o, 8, [m.get("offset", 0)], transform=_tr_b16)


def _lds_write(w, o, n_regs, m):
    wg = w.wg
    addr = w.rv(o[0]).astype(np.int64) + m.get("offset", 0)
    nbytes = 4 * n_regs
    if (addr[w.em] + nbytes > LDS_BYTES).any():
        wg.report("lds-oob", w.index, w.pc, "LDS write beyond %d bytes" % LDS_BYTES)
        return
    data = np.stack([w.rv(o[1], k) for k in range(n_regs)], axis=1)
    words = _lds_words(addr, nbytes, w.em)
    wg.lds_write_check(w.index, words, w.pc, "ds_write")
    oid = w._issue("ds_write", w.lgq)
    act = np.nonzero(w.em)[0]
    wg.lds[addr[act, None] + np.arange(nbytes)] = np.ascontiguousarray(data[act]).view(np.uint8).reshape(len(act), nbytes)
    wg.w_op[words] = oid
    wg.r_op[words, :] = -1


@op("ds_write_b128")
def _(w, o, m):
    _lds_write(w, o, 4, m)


@op("ds_write_b64")
def _(w, o, m):
    _lds_write(w, o, 2, m)


@op("ds_write_b32")
def _(w, o, m):
    _lds_write(w, o, 1, m)


# ---- global memory
def _gaddr(w, voff, sbase, m):
    if sbase[0] == "label" and sbase[1] == "off":       # no scalar base: the address is a register pair
        return (w.rv(voff, 0).astype(np.uint64) | (w.rv(voff, 1).astype(np.uint64) << np.uint64(32))) + np.uint64(m.get("offset", 0))
    return (np.uint64(w.rs(sbase, 2)) + w.rv(voff).astype(np.uint64) + np.uint64(m.get("offset", 0))).astype(np.uint64)


def _gload(n_regs):
    def h(w, o, m):
        addr = _gaddr(w, o[1], o[2], m)
        data, bad = w.wg.gmem.read(addr, 4 * n_regs, w.em)
        if bad.any():
            w.wg.report("global-oob", w.index, w.pc, "load outside the scenario's buffers, lanes %s, e.g. 0x%x" % (np.nonzero(bad)[0][:4], int(addr[bad][0])))
        regs = np.ascontiguousarray(data).view(U32).reshape(64, n_regs)
        w._issue("vload", w.vmq, regs=(o[0][0], o[0][1], n_regs), data=[regs[:, k].copy() for k in range(n_regs)], mask=w.em.copy())
    return h


HANDLERS["global_load_dword"] = _gload(1)
HANDLERS["global_load_dwordx2"] = _gload(2)
HANDLERS["global_load_dwordx4"] = _gload(4)


@op("global_load_lds_dwordx4")
def _(w, o, m):
    wg = w.wg
    addr = _gaddr(w, o[0], o[1], m)       # (the instruction offset moves the LDS address as well as the global one)
    data, bad = wg.gmem.read(addr, 16, w.em)
    if bad.any():
        wg.report("global-oob", w.index, w.pc, "tile copy reads outside the scenario's buffers, lanes %s, e.g. 0x%x" % (np.nonzero(bad)[0][:4], int(addr[bad][0])))
    dst = w.m0 + m.get("offset", 0) + 16 * LANES.astype(np.int64)
    if (dst[w.em] + 16 > LDS_BYTES).any():
        wg.report("lds-oob", w.index, w.pc, "tile copy writes beyond %d bytes of LDS" % LDS_BYTES)
        return
    words = _lds_words(dst, 16, w.em)
    wg.lds_write_check(w.index, words, w.pc, "dma")
    oid = w._issue("dma", w.vmq)
    act = np.nonzero(w.em)[0]
    wg.lds[dst[act, None] + np.arange(16)] = data[act]
    wg.w_op[words] = oid
    wg.r_op[words, :] = -1


def _gstore(n_regs):
    def h(w, o, m):
        addr = _gaddr(w, o[0], o[2], m)
        data = np.stack([w.rv(o[1], k) for k in range(n_regs)], axis=1)
        bad = w.wg.gmem.write(addr, np.ascontiguousarray(data).view(np.uint8).reshape(64, 4 * n_regs), w.em)
        if bad.any():
            w.wg.report("global-oob", w.index, w.pc, "store outside the scenario's output buffers, lanes %s, e.g. 0x%x" % (np.nonzero(bad)[0][:4], int(addr[bad][0])))
        w._issue("store", w.vmq)
    return h


HANDLERS["global_store_dwordx2"] = _gstore(2)
HANDLERS["global_store_dwordx4"] = _gstore(4)
