"""Every hand-written assembly statement of the HIP sources tells the compiler what it changes.

The sources are preprocessed for the device (`hipcc -E`), every `asm volatile(...)` statement is cut into its
template, outputs, inputs and clobbers, the template is read instruction by instruction, and every register an
instruction writes -- a named operand, a literal VGPR / SGPR, `vcc`, `scc`, `exec` -- must be an output operand, a
listed clobber or, for `exec`, restored from the saved copy inside the statement.  A statement that leaves one
out lets the compiler keep a live value (a loop compare in SCC, say) across it.  A statement with a memory
instruction must list "memory": the bytes it reads were stored by C++ code the compiler is otherwise free to move.
"""
from __future__ import annotations

import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "comp_inference_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
SOURCES = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))

pytestmark = pytest.mark.skipif(shutil.which(HIPCC) is None and not os.path.exists(HIPCC), reason="hipcc not found")


def preprocess(src: str) -> str:
    return subprocess.run([HIPCC, "-E", "--cuda-device-only", "--offload-arch=gfx950", "-std=c++17",
                           os.path.join(CSRC, src), "-o", "-"], check=True, capture_output=True, text=True).stdout


def asm_statements(text: str):
    """Yield the argument text of every `asm volatile( ... )` of our own code (system headers have none)."""
    for m in re.finditer(r"\basm\s+volatile\s*\(", text):
        i, depth, in_str = m.end(), 1, False
        while depth:
            c = text[i]
            if in_str:
                if c == "\\":
                    i += 1
                elif c == '"':
                    in_str = False
            elif c == '"':
                in_str = True
            elif c == "(":
                depth += 1
            elif c == ")":
                depth -= 1
            i += 1
        yield text[m.end():i - 1]


def split_sections(body: str):
    """template : outputs : inputs : clobbers, split at colons outside strings and parentheses."""
    parts, cur, depth, in_str, i = [], [], 0, False, 0
    while i < len(body):
        c = body[i]
        if in_str:
            cur.append(c)
            if c == "\\":
                cur.append(body[i + 1])
                i += 1
            elif c == '"':
                in_str = False
        elif c == '"':
            in_str = True
            cur.append(c)
        elif c in "([":
            depth += 1
            cur.append(c)
        elif c in ")]":
            depth -= 1
            cur.append(c)
        elif c == ":" and depth == 0:
            parts.append("".join(cur))
            cur = []
        else:
            cur.append(c)
        i += 1
    parts.append("".join(cur))
    while len(parts) < 4:
        parts.append("")
    return parts


def string_literals(s: str) -> str:
    out = []
    for m in re.finditer(r'"((?:[^"\\]|\\.)*)"', s):
        out.append(m.group(1).replace("\\n", "\n").replace("\\t", " "))
    return "".join(out)


def operands(section: str):
    """{name: constraint} of a list like  [X] "+v"(st.X), [e] "=&v"(e)  (unnamed operands get their position)."""
    ops = {}
    for n, m in enumerate(re.finditer(r'(?:\[(\w+)\]\s*)?"([^"]*)"\s*\(', section)):
        ops[m.group(1) or str(n)] = m.group(2)
    return ops


NO_DEST = re.compile(r"^(s_waitcnt|s_nop|s_branch|s_cbranch_\w+|s_barrier|s_sleep|s_setprio|global_store_\w+|"
                     r"ds_write\w*|buffer_store_\w+|s_endpgm)$")
SCC_WRITERS = re.compile(r"^s_(add|sub|addc|subb|and|or|xor|andn2|orn2|nand|nor|xnor|lshl|lshr|ashr|bfe|min|max|abs|not|"
                         r"cmp|bitcmp)\w*$")
SCC_READERS = re.compile(r"^s_(cselect|cbranch_scc\d|addc|subb|cmov)\w*$")


def regs_of(tok: str):
    """Registers named by one operand token: ('v', 72), ('s', 20), 'vcc', 'exec', or ('%', name)."""
    tok = tok.strip()
    m = re.fullmatch(r"%\[(\w+)\]", tok)
    if m:
        return [("%", m.group(1))]
    m = re.fullmatch(r"%(\d+)", tok)
    if m:
        return [("%", m.group(1))]
    m = re.fullmatch(r"([vs])(\d+)", tok)
    if m:
        return [(m.group(1), int(m.group(2)))]
    m = re.fullmatch(r"([vs])\[(\d+):(\d+)\]", tok)
    if m:
        return [(m.group(1), r) for r in range(int(m.group(2)), int(m.group(3)) + 1)]
    if tok in ("vcc", "vcc_lo", "vcc_hi"):
        return ["vcc"]
    if tok in ("exec", "exec_lo", "exec_hi"):
        return ["exec"]
    return []


def written_by(line: str):
    """(registers written, writes scc, reads scc) for one instruction line."""
    parts = line.split(None, 1)
    mn = parts[0]
    ops = [o for o in (parts[1].split(",") if len(parts) > 1 else [])]
    # operands like "offset:32" ride on the last comma-separated piece; keep the register part
    ops = [o.strip().split()[0] if o.strip() else "" for o in ops]
    writes, w_scc, r_scc = [], bool(SCC_WRITERS.match(mn)), bool(SCC_READERS.match(mn))
    if NO_DEST.match(mn):
        return writes, w_scc, r_scc
    if mn.startswith("s_cmp") or mn.startswith("s_bitcmp"):
        return writes, True, r_scc
    if mn.startswith("v_cmpx"):
        writes.append("exec")
        if ops:
            writes += regs_of(ops[0])  # the explicit sdst of the VOP3 form / vcc of the VOPC form
        return writes, w_scc, r_scc
    if ops:
        writes += regs_of(ops[0])
    if re.match(r"^v_(add|sub|subrev)_co_|^v_(addc|subb|subbrev)_co_|^v_div_scale|^v_mad_[ui]64", mn) and len(ops) > 1:
        writes += regs_of(ops[1])
    if "saveexec" in mn:
        writes.append("exec")
    return writes, w_scc, r_scc


def check_statement(body: str):
    template_src, outs_src, ins_src, clob_src = split_sections(body)[:4]
    template = string_literals(template_src)
    outs, ins = operands(outs_src), operands(ins_src)
    clobbers = set(re.findall(r'"([^"]+)"', clob_src))
    problems = []
    lines = []
    for raw in template.split("\n"):
        line = raw.split("//")[0].split(";")[0].strip()
        if not line or line.endswith(":") or line.startswith("."):
            continue
        lines.append(line)
    saves, restores = 0, 0
    scc_written = False
    for line in lines:
        writes, w_scc, _ = written_by(line)
        scc_written |= w_scc
        if re.match(r"s_\w+_saveexec", line):
            saves += 1
        if re.match(r"s_mov_b64\s+exec\s*,\s*s\[", line):
            restores += 1
            writes = [w for w in writes if w != "exec"]
        for w in writes:
            if w == "exec":
                continue  # judged below: saved and restored inside the statement
            if w == "vcc":
                if "vcc" not in clobbers:
                    problems.append(f"`{line}` writes vcc, not a clobber")
            elif w[0] == "%":
                name = w[1]
                if name in ins and name not in outs:
                    problems.append(f"`{line}` writes input operand %[{name}]")
                elif name not in outs:
                    problems.append(f"`{line}` writes unknown operand %[{name}]")
            else:
                reg = f"{w[0]}{w[1]}"
                if reg not in clobbers:
                    problems.append(f"`{line}` writes {reg}, not a clobber")
    if scc_written and "scc" not in clobbers:
        problems.append("an instruction writes SCC and \"scc\" is not a clobber")
    if saves and restores < 1:
        problems.append("exec is masked and never restored")
    writes_exec = any("exec" in written_by(l)[0] for l in lines)
    if writes_exec and not saves:
        problems.append("exec is written without a saved copy")
    # a pure output written before the statement's last read of its inputs must be early-clobber
    if len(lines) > 1:
        for name, cons in outs.items():
            if cons.startswith("=") and "&" not in cons:
                problems.append(f"output %[{name}] of a multi-instruction statement is not early-clobber (\"=&\")")
    # a statement that reads or writes memory says so: without "memory" among the clobbers the compiler may move the C++
    # stores that stage bytes in the LDS behind the statement that reads them, or drop them (nothing it can see reads them)
    touches_memory = any(re.match(r"(ds_|global_|buffer_|flat_|scratch_|s_load|s_buffer_load)", line.split()[0]) for line in lines)
    if touches_memory and "memory" not in clobbers:
        problems.append("an instruction reads or writes memory and \"memory\" is not a clobber")
    # loads issued inside the statement are drained before it ends (the compiler knows nothing of them)
    issued_lgkm = issued_vm = False
    for line in lines:
        mn = line.split()[0]
        if mn.startswith("ds_read") or mn.startswith("s_load"):
            issued_lgkm = True
        if mn.startswith("global_load") or mn.startswith("buffer_load"):
            issued_vm = True
        if mn == "s_waitcnt":
            if "lgkmcnt(0)" in line:
                issued_lgkm = False
            if "vmcnt(0)" in line:
                issued_vm = False
    if issued_lgkm:
        problems.append("an LDS read may still be in flight when the statement ends")
    if issued_vm:
        problems.append("a global load may still be in flight when the statement ends")
    return problems, len(lines)


@pytest.mark.parametrize("src", SOURCES)
def test_every_asm_statement_declares_what_it_writes(src):
    text = preprocess(src)
    n_statements = n_instructions = 0
    failures = []
    for body in asm_statements(text):
        problems, n = check_statement(body)
        n_statements += 1
        n_instructions += n
        if problems:
            head = string_literals(split_sections(body)[0])[:60].replace("\n", " | ")
            failures.append(f"{src}: asm starting `{head}`: " + "; ".join(sorted(set(problems))))
    assert not failures, "\n".join(failures)
    if src in ("linear.hip", "decode.hip", "transposed.hip", "embedding.hip"):
        assert n_statements >= 3 and n_instructions > 100, "the hand-scheduled loops were not found: the parser is blind"


def test_the_checker_sees_a_missing_scc_clobber():
    ok = r'''"s_sub_u32 s22, s22, 1\n" "s_and_saveexec_b64 s[20:21], vcc\n" "s_mov_b64 exec, s[20:21]\n"
             : [X] "+v"(x) : [n] "s"(n) : "vcc", "scc", "s20", "s21", "s22"'''
    assert check_statement(ok)[0] == []
    for drop, what in (('"scc", ', "SCC"), ('"s22"', "s22"), ('"s20", ', "s20")):
        bad = ok.replace(drop, '"s99"' if drop == '"s22"' else "")
        assert any(what in p for p in check_statement(bad)[0]), (drop, check_statement(bad)[0])
    # an unrestored execution mask, a written input, a late-bound output, a load left in flight
    assert any("restored" in p for p in check_statement(
        r'"s_and_saveexec_b64 s[20:21], vcc\n" "s_nop 0\n" : : : "scc", "s20", "s21"')[0])
    assert any("input operand" in p for p in check_statement(r'"v_mov_b32 %[n], 0\n" "s_nop 0\n" : : [n] "v"(n) :')[0])
    assert any("early-clobber" in p for p in check_statement(
        r'"v_mov_b32 %[e], %[n]\n" "v_mov_b32 v3, %[n]\n" : [e] "=v"(e) : [n] "v"(n) : "v3"')[0])
    assert any("in flight" in p for p in check_statement(r'"ds_read_b32 %[e], %[n]\n" : [e] "=&v"(e) : [n] "v"(n) :')[0])
    # a memory instruction without "memory" among the clobbers
    load = r'"ds_read_b32 %[e], %[n]\n" "s_waitcnt lgkmcnt(0)\n" : [e] "=&v"(e) : [n] "v"(n) : '
    assert any('"memory" is not a clobber' in p for p in check_statement(load)[0])
    assert check_statement(load + '"memory"')[0] == []
