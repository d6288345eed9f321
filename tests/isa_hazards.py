"""Wait states of gfx950 machine code, checked on the CPU (test infrastructure).

Some dependencies between instructions are not interlocked by the hardware: the program has to leave a number of
wait states (instructions issued; `s_nop k` counts k + 1) between the producer and the consumer.  The compiler
leaves them for the instructions it schedules itself, but a hand-written assembly statement is opaque to it: it does
not see a producer at the end of a statement, a consumer at its start, or either inside.  This module reads the
disassembly of a code object (`llvm-objdump -d` of the library's own kernels), rebuilds the control flow of every
kernel and checks each rule below along every path, so that what is checked is the shipped machine code, statements
and compiler output together.

The rules (CDNA3 instruction set guide, "manually inserted wait states", and what the compiler itself leaves after
the same instructions in these kernels):

  sgpr_vmem      VALU writes an SGPR / VCC         -> VMEM instruction reads it                        5
  sgpr_lane      VALU writes an SGPR / VCC         -> v_readlane / v_writelane use it as lane select   4
  exec_dpp       VALU writes EXEC                  -> DPP instruction                                  5
  vgpr_dpp       VALU writes a VGPR                -> DPP instruction reads it                         2
  sgpr_valu      VALU writes an SGPR / VCC         -> VALU reads it                                    2
  vgpr_readlane  VALU writes a VGPR                -> v_readlane / v_readfirstlane read it             1
  exec_lane      VALU writes EXEC                  -> v_readlane / v_readfirstlane / v_writelane       4
  trans_use      transcendental VALU writes a VGPR -> other VALU reads it                              1
  dst_sel        VALU writes part of a VGPR (SDWA dst_sel, op_sel high half) -> VALU reads it          1
  vgpr_mfma      VALU writes a VGPR                -> matrix instruction reads it                      2
  vgpr_permlane  VALU writes a VGPR                -> v_permlane16/32_swap reads it                    2
  mfma_result    matrix instruction writes VGPRs   -> VALU / VMEM / LDS reads or writes one of them    MFMA_RESULT
                 (a matrix instruction that accumulates into exactly the same registers may follow at once)
"""
from __future__ import annotations

import re
from dataclasses import dataclass, field

# v_mfma_f32_32x32x16_bf16: the compiler leaves `s_nop 11` between this instruction and a VALU read of its result
MFMA_RESULT = 12

NO_DEST = re.compile(
    r"^(s_cmpk?_\w+|s_bitcmp\w+|s_cbranch_\w+|s_branch|s_waitcnt\w*|s_nop|s_barrier|s_sleep|s_endpgm|s_setprio|s_sethalt|"
    r"s_trap|s_setpc_b64|s_sendmsg\w*|s_setreg\w*|"
    r"(global|scratch|buffer|flat)_store_\w+|ds_write\w*)$")
TRANS = re.compile(r"^v_(rcp|rsq|sqrt|exp|log|sin|cos)_")
TWO_DESTS = re.compile(r"^(v_(add|sub|subrev|addc|subb|subbrev)_co_|v_mad_[ui]64_|v_div_scale_|v_permlane(16|32)_swap)")
READS_DEST = re.compile(r"^(v_fmac_|v_mac_|v_writelane_|v_permlane(16|32)_swap|v_dot\w+c_)")


def regs_of(tok: str) -> list:
    """Registers one operand names: ('v', n), ('s', n), 'vcc', 'exec', 'm0'."""
    tok = tok.strip().lstrip("-").strip("|")
    m = re.fullmatch(r"(?:neg|abs)\((.*)\)", tok)
    if m:
        tok = m.group(1)
    m = re.fullmatch(r"([vsa])(\d+)", tok)
    if m:
        return [(m.group(1), int(m.group(2)))]
    m = re.fullmatch(r"([vsa])\[(\d+):(\d+)\]", tok)
    if m:
        return [(m.group(1), r) for r in range(int(m.group(2)), int(m.group(3)) + 1)]
    if tok in ("vcc", "vcc_lo", "vcc_hi"):
        return ["vcc"]
    if tok in ("exec", "exec_lo", "exec_hi"):
        return ["exec"]
    if tok == "m0":
        return ["m0"]
    return []


def split_operands(text: str) -> list:
    out, cur, depth = [], [], 0
    for ch in text:
        if ch == "[":
            depth += 1
        elif ch == "]":
            depth -= 1
        if ch == "," and depth == 0:
            out.append("".join(cur))
            cur = []
        else:
            cur.append(ch)
    if "".join(cur).strip():
        out.append("".join(cur))
    return [o.strip() for o in out]


@dataclass
class Ins:
    addr: int
    mn: str            # mnemonic without _e32 / _e64
    text: str          # as disassembled
    ops: list          # operand tokens (modifiers stripped)
    mods: str          # modifiers of the last operand (dst_sel:..., quad_perm:..., offset:...)
    word: int = 0      # first dword of the encoding
    defs: list = field(default_factory=list)
    uses: list = field(default_factory=list)
    succ: list = field(default_factory=list)
    pred: list = field(default_factory=list)

    @property
    def valu(self):
        return self.mn.startswith("v_")

    @property
    def mfma(self):
        return self.mn.startswith("v_mfma") or self.mn.startswith("v_smfma")

    @property
    def vmem(self):
        return self.mn.startswith(("global_", "scratch_", "buffer_", "flat_"))

    @property
    def lds(self):
        return self.mn.startswith("ds_")

    @property
    def dpp(self):
        return "_dpp" in self.mn

    @property
    def wait_states(self):
        if self.mn == "s_nop":
            return int(self.ops[0], 0) + 1
        return 1


def decode(mn_raw: str, operand_text: str, addr: int, text: str) -> Ins:
    mn = re.sub(r"_e(32|64)$", "", mn_raw)
    toks = split_operands(operand_text)
    ops, mods = [], ""
    for t in toks:
        parts = t.split(None, 1)
        ops.append(parts[0] if parts else "")
        if len(parts) > 1:
            mods += " " + parts[1]
    ins = Ins(addr, mn, text, ops, mods)
    n_dst = 0
    if not NO_DEST.match(mn) and ops:
        n_dst = 2 if TWO_DESTS.match(mn) else 1
        if re.match(r"^(global|flat|buffer)_atomic_", mn) and "sc0" not in (mods + " " + " ".join(ops)):
            n_dst = 0  # no value returned
        if re.match(r"^ds_(add|sub|min|max|and|or|xor|inc|dec)_[uif]\d+$", mn):
            n_dst = 0
    for t in ops[:n_dst]:
        ins.defs += regs_of(t)
    if mn.startswith("v_cmpx") or "saveexec" in mn:
        ins.defs.append("exec")
    for t in ops[n_dst:]:
        ins.uses += regs_of(t)
    if n_dst and (READS_DEST.match(mn) or ins.dpp):  # accumulators, and the `old` value of a DPP result
        for t in ops[:n_dst]:
            ins.uses += [r for r in regs_of(t) if r[0] == "v"]
    return ins


LINE = re.compile(r"^\s+(\S+)\s*(.*?)\s*//\s*([0-9A-Fa-f]+):\s*([0-9A-Fa-f]{8})")
SYMBOL = re.compile(r"^([0-9a-f]+) <(.+)>:$")


def kernels_of(disassembly: str, is_kernel=lambda name: name.startswith("_Z")) -> dict:
    """{kernel symbol: [Ins, ...]}: the instructions a kernel can reach from its entry, in address order, with
    successors and predecessors (as indices into that list) filled in.  A kernel is not a contiguous range: the
    out-of-line pieces of assembly statements (`.subsection 1`) lie behind the last kernel of the section."""
    program, entries = [], {}
    for line in disassembly.splitlines():
        m = SYMBOL.match(line)
        if m:
            if is_kernel(m.group(2)):
                entries[m.group(2)] = int(m.group(1), 16)
            continue
        m = LINE.match(line)
        if m:
            program.append(decode(m.group(1), m.group(2), int(m.group(3), 16), line.split("//")[0].strip()))
            program[-1].word = int(m.group(4), 16)
    at = {ins.addr: i for i, ins in enumerate(program)}
    succ = []
    for i, ins in enumerate(program):
        nxt = [i + 1] if i + 1 < len(program) else []
        if ins.mn == "s_branch" or ins.mn.startswith("s_cbranch_"):
            simm = ins.word & 0xFFFF  # (the operand is printed as a number or as a label; the encoding is always there)
            if simm >= 0x8000:
                simm -= 0x10000
            target = at.get(ins.addr + 4 + 4 * simm)
            if target is None:
                raise ValueError(f"branch at {ins.addr:#x} to no instruction: {ins.text}")
            succ.append([target] if ins.mn == "s_branch" else nxt + [target])
        elif ins.mn in ("s_endpgm", "s_setpc_b64"):
            succ.append([])
        else:
            succ.append(nxt)
    out = {}
    for name, entry in entries.items():
        reach, stack = set(), [at[entry]]
        while stack:
            i = stack.pop()
            if i not in reach:
                reach.add(i)
                stack += succ[i]
        order = sorted(reach)
        local = {g: k for k, g in enumerate(order)}
        body = []
        for g in order:
            src = program[g]
            ins = Ins(src.addr, src.mn, src.text, src.ops, src.mods, src.word, src.defs, src.uses)
            ins.succ = [local[t] for t in succ[g]]
            body.append(ins)
        for k, ins in enumerate(body):
            for t in ins.succ:
                body[t].pred.append(k)
        out[name] = body
    return out


def labels_of(disassembly: str) -> dict:
    """{symbol: address} of everything the disassembly names: kernels and the named labels of assembly statements."""
    return {m.group(2): int(m.group(1), 16) for m in map(SYMBOL.match, disassembly.splitlines()) if m}


def kind_of(ins: Ins) -> str:
    """The issue class of an instruction, for counting what a loop costs."""
    if ins.mfma:
        return "mfma"
    if ins.valu:
        return "valu"
    if ins.lds:
        return "lds"
    if ins.vmem:
        return "vmem"
    if ins.mn in ("s_waitcnt", "s_nop"):
        return "wait"
    if ins.mn == "s_branch" or ins.mn.startswith("s_cbranch_"):
        return "branch"
    return "salu"


def nearest_producer(body: list, start: int, limit: int, is_producer):
    """(wait states, index) of the producer from which `start` is reached with the fewest wait states in between,
    along any path, looking back at most `limit` wait states; None if there is none."""
    best, seen = None, {}
    stack = [(p, 0) for p in body[start].pred]
    while stack:
        i, waited = stack.pop()
        if waited >= limit or seen.get(i, limit) <= waited:
            continue
        seen[i] = waited
        if is_producer(body[i]):
            if best is None or waited < best[0]:
                best = (waited, i)
            continue
        waited += body[i].wait_states
        stack += [(p, waited) for p in body[i].pred]
    return best


def is_sgpr(r):
    return r == "vcc" or (isinstance(r, tuple) and r[0] == "s")


def is_vgpr(r):
    return isinstance(r, tuple) and r[0] == "v"


def writes_part_of_a_register(ins: Ins) -> bool:
    m = re.search(r"dst_sel:(\w+)", ins.mods)
    if m and m.group(1) != "DWORD":
        return True
    m = re.search(r"op_sel:\[([01,]+)\]", ins.mods)
    return bool(m and m.group(1).split(",")[-1] == "1" and len(m.group(1).split(",")) == len(ins.ops))


def plain_valu(ins: Ins) -> bool:
    return ins.valu and not ins.mfma


def dependencies(ins: Ins):
    """(rule, wait states needed, registers, kind of producer) for everything `ins` consumes under the table."""
    sg = [r for r in ins.uses if is_sgpr(r)]
    vg = [r for r in ins.uses if is_vgpr(r)]
    lane_op = ins.mn.startswith(("v_readlane", "v_writelane"))
    if ins.vmem:
        yield "sgpr_vmem", 5, sg, plain_valu
    if lane_op and len(ins.ops) > 2:
        yield "sgpr_lane", 4, [r for r in regs_of(ins.ops[2]) if is_sgpr(r)], plain_valu
    if ins.dpp:
        yield "exec_dpp", 5, ["exec"], plain_valu
        yield "vgpr_dpp", 2, vg, plain_valu
    if ins.valu:
        yield "sgpr_valu", 2, sg, plain_valu
        if not TRANS.match(ins.mn):
            yield "trans_use", 1, vg, lambda p: p.valu and bool(TRANS.match(p.mn))
        yield "dst_sel", 1, vg, lambda p: p.valu and writes_part_of_a_register(p)
    if ins.mn.startswith(("v_readlane", "v_readfirstlane")):
        yield "vgpr_readlane", 1, [r for r in regs_of(ins.ops[1]) if is_vgpr(r)], plain_valu
    if lane_op or ins.mn.startswith("v_readfirstlane"):
        yield "exec_lane", 4, ["exec"], plain_valu
    if ins.mfma:
        yield "vgpr_mfma", 2, vg, plain_valu
    if ins.mn.startswith("v_permlane"):
        yield "vgpr_permlane", 2, vg, plain_valu
    if ins.valu or ins.vmem or ins.lds:
        touched = [r for r in ins.uses + ins.defs if is_vgpr(r)]
        if ins.mfma:
            # accumulating into exactly the registers the earlier instruction wrote needs no wait
            acc = set(regs_of(ins.ops[3])) if len(ins.ops) > 3 else set()
            yield "mfma_result", MFMA_RESULT, touched, lambda p: p.mfma and not set(p.defs) == acc == set(ins.defs)
        else:
            yield "mfma_result", MFMA_RESULT, touched, lambda p: p.mfma


def check(body: list, closest: dict | None = None) -> list:
    """[(rule, producer Ins, consumer Ins, wait states found)] for every dependency of the table with too few wait
    states.  `closest`, if given, collects per rule the smallest number of wait states seen at all (looking back
    twice as far as the rule asks): where the compiler had to pad with s_nop, that is the rule's own figure."""
    bad = []
    for c, ins in enumerate(body):
        for rule, need, regs, kind in dependencies(ins):
            if not regs:
                continue
            wanted = set(regs)
            hit = nearest_producer(body, c, 2 * need if closest is not None else need,
                                   lambda p: kind(p) and bool(wanted & set(p.defs)))
            if hit is None:
                continue
            if closest is not None:
                closest[rule] = min(closest.get(rule, hit[0]), hit[0])
            if hit[0] < need:
                bad.append((rule, body[hit[1]], ins, hit[0]))
    return bad
