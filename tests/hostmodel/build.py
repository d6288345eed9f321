"""Builds the library's HIP sources for the host model (sim.h): libci_hostmodel.so beside this file.

    python tests/hostmodel/build.py [--force]

Every source is preprocessed as plain C++ against the stand-in hip/hip_runtime.h of this directory, then three
things are rewritten in the preprocessed text before it is compiled for x86-64:

  * `asm volatile(template : outputs : inputs : clobbers)` becomes a call of the model's interpreter with the same
    template string and a pointer to every operand;
  * the dynamic LDS declaration becomes a pointer to the model's LDS area, other `__shared__` arrays statics;
  * the helpers that stage bytes into LDS for other lanes of the same wavefront to read get a meeting point of the
    wavefront before and after: on the GPU a wavefront's LDS operations complete in order, in the model the lanes are
    fibres that run one after the other between meeting points.

A second library, libci_hostmodel_order.so (`build(order=True)`, `--order`), is the same with the kernel sources
compiled under the compiler's thread-sanitizer instrumentation and no sanitizer runtime: the model itself (sim.cpp,
"ordering between wavefronts") takes the calls the instrumentation makes at every plain memory access, and reports
two wavefronts that touch the same byte with no barrier or release/acquire pair between them -- what fibres that run
one after the other would never show.  A third, libci_hostmodel_undefined.so (`build(undefined=True)`, `--undefined`),
compiles them with the compiler's undefined-behaviour checks (array bounds, shift amounts, alignment, null, signed
overflow, pointer arithmetic), again without a runtime: the checks' calls become violations of the model.

Test infrastructure: nothing of the product is built from, or loads, what this makes.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "comp_inference_amd", "csrc")
OUT_DIR = os.path.join(HERE, "_build")
LIB_PATH = os.path.join(HERE, "libci_hostmodel.so")
ORDER_LIB_PATH = os.path.join(HERE, "libci_hostmodel_order.so")
ORDER_FLAGS = ["-fsanitize=thread", "-mllvm", "-tsan-instrument-func-entry-exit=0"]
UNDEFINED_LIB_PATH = os.path.join(HERE, "libci_hostmodel_undefined.so")
UNDEFINED_FLAGS = ["-fsanitize=bounds,shift,alignment,integer-divide-by-zero,null,unreachable,signed-integer-overflow,pointer-overflow"]
CXX = os.environ.get("CI_HOSTMODEL_CXX", "/opt/rocm/llvm/bin/clang++")
SOURCES = ["api.hip", "encode.hip", "decode.hip", "linear.hip", "embedding.hip", "transposed.hip", "legacy.hip"]
CXXFLAGS = ["-std=c++17", "-O1", "-g", "-fPIC", "-fno-strict-aliasing", "-Wno-unused-value", "-Wno-unknown-attributes",
            "-Wno-ignored-attributes", "-Wno-pass-failed", "-Wno-psabi"]

# Functions after (and before) which the lanes of a wavefront read LDS bytes that other lanes wrote.
LDS_HANDOVER = ["stage_commit", "stage_window_pair", "stage_window"]


def _balanced(text: str, i: int, open_c: str = "(", close_c: str = ")") -> int:
    """Index just past the bracket that closes the one at text[i]."""
    assert text[i] == open_c
    depth, in_str = 0, False
    while True:
        c = text[i]
        if in_str:
            if c == "\\":
                i += 1
            elif c == '"':
                in_str = False
        elif c == '"':
            in_str = True
        elif c == open_c:
            depth += 1
        elif c == close_c:
            depth -= 1
            if depth == 0:
                return i + 1
        i += 1


def _split_top(body: str, sep: str) -> list[str]:
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
        elif c in "([{":
            depth += 1
            cur.append(c)
        elif c in ")]}":
            depth -= 1
            cur.append(c)
        elif c == sep and depth == 0:
            parts.append("".join(cur))
            cur = []
        else:
            cur.append(c)
        i += 1
    parts.append("".join(cur))
    return parts


def _operands(section: str) -> list[tuple[str, str, str]]:
    """[(name, constraint, expression)] of an operand list."""
    out = []
    for item in _split_top(section, ","):
        item = item.strip()
        if not item:
            continue
        m = re.match(r'(?:\[(\w+)\]\s*)?"([^"]*)"\s*\(', item, re.S)
        assert m, f"operand not understood: {item!r}"
        expr = item[m.end():item.rindex(")")]
        out.append((m.group(1) or "", m.group(2), expr.strip()))
    return out


_counter = [0]


def rewrite_asm(text: str) -> str:
    out, at = [], 0
    for m in re.finditer(r"\basm\s+volatile\s*\(", text):
        if m.start() < at:
            continue
        end = _balanced(text, m.end() - 1)
        body = text[m.end():end - 1]
        semi = text.index(";", end)
        sections = _split_top(body, ":")
        template = sections[0].strip()
        outs = _operands(sections[1]) if len(sections) > 1 else []
        ins = _operands(sections[2]) if len(sections) > 2 else []
        _counter[0] += 1
        k = _counter[0]
        lines, ops = ["{"], []
        for name, cons, expr in outs:
            ops.append(f'{{"{name}", "{cons}", (void *)&({expr}), (uint32_t)sizeof({expr})}}')
        for j, (name, cons, expr) in enumerate(ins):
            lines.append(f"auto asm_in_{k}_{j} = ({expr});")
            ops.append(f'{{"{name}", "{cons}", (void *)&asm_in_{k}_{j}, (uint32_t)sizeof(asm_in_{k}_{j})}}')
        if ops:
            lines.append(f"sim::AsmOperand asm_ops_{k}[] = {{{', '.join(ops)}}};")
            lines.append(f"sim::run_asm({template}, asm_ops_{k}, {len(ops)});")
        else:
            lines.append(f"sim::run_asm({template}, nullptr, 0);")
        lines.append("}")
        out.append(text[at:m.start()])
        out.append(" ".join(lines))
        at = semi + 1
    out.append(text[at:])
    return "".join(out)


def rewrite_lds(text: str) -> str:
    text, n = re.subn(r"extern\s+__shared__\s+__attribute__\(\(aligned\(16\)\)\)\s+uint8_t\s+lds\[\]\s*;",
                      "uint8_t *const lds = sim::lds_base();", text)
    # a `__shared__` array is a static here; the ordering check is told that it is shared memory of the workgroup
    text = re.sub(r"\b__shared__\s+([\w:]+)\s+(\w+)\s*\[([^\]]+)\]\s*;",
                  r"static \1 \2[\3]; sim::shared_static(\2, sizeof(\2));", text)
    return re.sub(r"\b__shared__\b", "static", text)


def fence_handover(text: str) -> str:
    for name in LDS_HANDOVER:
        for m in list(re.finditer(r"\b%s\s*\(" % name, text))[::-1]:
            close = _balanced(text, m.end() - 1)
            rest = text[close:close + 8].lstrip()
            if not rest.startswith("{"):
                continue  # a call, not the definition
            brace = text.index("{", close)
            end = _balanced(text, brace, "{", "}")
            text = text[:brace + 1] + " sim::wave_sync(); " + text[brace + 1:end - 1] + " sim::wave_sync(); " + text[end - 1:]
    return text


def rewrite(text: str) -> str:
    return fence_handover(rewrite_lds(rewrite_asm(text)))


def needs_build(lib_path: str = LIB_PATH) -> bool:
    if not os.path.exists(lib_path):
        return True
    built = os.path.getmtime(lib_path)
    deps = [os.path.join(CSRC, f) for f in os.listdir(CSRC)] + [os.path.join(HERE, f) for f in ("sim.cpp", "sim.h", "build.py", "selftest.hip")]
    deps += [os.path.join(HERE, "hip", "hip_runtime.h"), os.path.join(ROOT, "include", "comp_inference_hip.h")]
    return any(os.path.getmtime(d) > built for d in deps)


def build(force: bool = False, verbose: bool = False, order: bool = False, undefined: bool = False) -> str:
    lib_path = ORDER_LIB_PATH if order else UNDEFINED_LIB_PATH if undefined else LIB_PATH
    if not force and not needs_build(lib_path):
        return lib_path
    out_dir = os.path.join(OUT_DIR, "order") if order else os.path.join(OUT_DIR, "undefined") if undefined else OUT_DIR
    os.makedirs(out_dir, exist_ok=True)
    flags = CXXFLAGS + (ORDER_FLAGS if order else UNDEFINED_FLAGS if undefined else [])
    procs, objs = [], []
    for src in SOURCES + ["selftest.hip"]:
        path = os.path.join(HERE if src == "selftest.hip" else CSRC, src)
        pre = subprocess.run([CXX, "-E", "-x", "c++", "-std=c++17", "-I", HERE, "-I", CSRC, path, "-o", "-"],
                             check=True, capture_output=True, text=True).stdout
        ii = os.path.join(out_dir, src + ".ii")
        with open(ii, "w") as f:
            f.write(rewrite(pre))
        obj = os.path.join(out_dir, src + ".o")
        procs.append((src, subprocess.Popen([CXX, "-x", "c++-cpp-output", *flags, "-c", ii, "-o", obj],
                                            stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    obj = os.path.join(out_dir, "sim.o")  # (the model itself is never instrumented)
    procs.append(("sim.cpp", subprocess.Popen([CXX, *CXXFLAGS, "-O2", "-c", os.path.join(HERE, "sim.cpp"), "-o", obj],
                                              stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            failed = True
            print(f"host-model build failed on {src}:\n{out[-6000:]}", file=sys.stderr)
        elif verbose and out.strip():
            print(out[-3000:])
    if failed:
        raise RuntimeError("host-model build failed")
    subprocess.check_call([CXX, "-shared", "-fPIC", "-o", lib_path, *objs])
    return lib_path


def build_mutant(tag: str, edits: list, rebuild: list, order: bool = False) -> str:
    """The host-model library with a deliberate mistake in the kernels: `edits` = [(file under csrc, old text, new text[, occurrences])],
    the first occurrence of each old text replaced (of one, unless stated); `rebuild` = the .hip sources to compile again from the edited copy (the other
    objects are the intact build's).  Returns the path of the mutant library, under _build/mutants/<tag>/.  For the
    tests that show that a mistake of a given kind in the real kernels is noticed.  `order`: the build that checks the
    ordering between wavefronts."""
    import shutil

    build(order=order)
    intact = os.path.join(OUT_DIR, "order") if order else OUT_DIR
    flags = CXXFLAGS + (ORDER_FLAGS if order else [])
    base = os.path.join(OUT_DIR, "mutants", tag + ("_order" if order else ""))
    src_dir = os.path.join(base, "csrc")
    shutil.rmtree(base, ignore_errors=True)
    shutil.copytree(CSRC, src_dir, ignore=shutil.ignore_patterns("*.o", "*.so"))
    for name, old_text, new_text, *occurrences in edits:
        path = os.path.join(src_dir, name)
        text = open(path).read()
        want = occurrences[0] if occurrences else 1  # how often the text occurs; the first occurrence is replaced
        assert text.count(old_text) == want, f"{name}: {text.count(old_text)} occurrences of {old_text!r}"
        with open(path, "w") as f:
            f.write(text.replace(old_text, new_text, 1))
    procs, objs = [], []
    for src in SOURCES + ["selftest.hip"]:
        if src not in rebuild:
            objs.append(os.path.join(intact, src + ".o"))
            continue
        pre = subprocess.run([CXX, "-E", "-x", "c++", "-std=c++17", "-I", HERE, "-I", src_dir, os.path.join(src_dir, src), "-o", "-"],
                             check=True, capture_output=True, text=True).stdout
        ii, obj = os.path.join(base, src + ".ii"), os.path.join(base, src + ".o")
        with open(ii, "w") as f:
            f.write(rewrite(pre))
        procs.append((src, subprocess.Popen([CXX, "-x", "c++-cpp-output", *flags, "-c", ii, "-o", obj],
                                            stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    objs.append(os.path.join(intact, "sim.o"))
    for src, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError(f"mutant {tag}: build failed on {src}:\n{out[-3000:]}")
    lib = os.path.join(base, "libci_hostmodel.so")
    subprocess.check_call([CXX, "-shared", "-fPIC", "-o", lib, *objs])
    return lib


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True, order="--order" in sys.argv, undefined="--undefined" in sys.argv))
