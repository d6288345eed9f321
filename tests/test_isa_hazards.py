"""The wait states the hardware does not enforce, checked in the machine code of every kernel of the built library
(tests/isa_hazards.py).  The compiler pads its own instructions; what it cannot see is a hand-written assembly
statement -- a scalar address computed by a VALU instruction right before a statement that loads through it, a
register written by the statement's last instruction and fed to a matrix instruction or a lane exchange right
after it, the matrix instruction's result read too early.  This is where such a mistake shows without a GPU."""
import os
import shutil
import subprocess

import pytest

import isa_hazards as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "comp_inference_amd", "libcomp_inference_hip.so")
OBJDUMP = "/opt/rocm/llvm/bin/llvm-objdump"


def listing(lines):
    """Disassembly text of a made-up kernel: (mnemonic and operands) or ("label:",); branches name labels."""
    addr, where, rows = 0, {}, []
    for ln in lines:
        if ln.endswith(":"):
            where[ln[:-1]] = addr
        else:
            rows.append((addr, ln))
            addr += 4
    out = ["0000000000000000 <_Zkernel>:"]
    for a, ln in rows:
        word = 0
        parts = ln.split()
        if parts[0] == "s_branch" or parts[0].startswith("s_cbranch"):
            word = ((where[parts[1]] - (a + 4)) // 4) & 0xFFFF
        out.append(f"\t{ln}    // {a:012X}: {word:08X}")
    return "\n".join(out) + "\n"


def found(lines):
    (body,) = H.kernels_of(listing(lines + ["s_endpgm"])).values()
    return sorted({b[0] for b in H.check(body)})


CASES = {
    # rule: (producer, instructions that make up the wait states, consumer, wait states needed)
    "sgpr_vmem": ("v_readfirstlane_b32 s22, v62", "global_load_dword v1, v2, s[22:23]", 5),
    "sgpr_lane": ("v_readfirstlane_b32 s4, v1", "v_readlane_b32 s5, v9, s4", 4),
    "exec_dpp": ("v_cmpx_gt_u32_e32 vcc, s9, v7", "v_mov_b32_dpp v3, v4 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf", 5),
    "vgpr_dpp": ("v_add_u32_e32 v4, v5, v6", "v_mov_b32_dpp v3, v4 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf", 2),
    "sgpr_valu": ("v_cmp_lt_u32_e64 s[20:21], v1, v2", "v_cndmask_b32_e64 v16, 0, v71, s[20:21]", 2),
    "vgpr_readlane": ("v_add_u32_e32 v4, v5, v6", "v_readfirstlane_b32 s10, v4", 1),
    "exec_lane": ("v_cmpx_gt_u32_e32 vcc, s9, v7", "v_readfirstlane_b32 s10, v40", 4),
    "trans_use": ("v_rcp_f32_e32 v2, v3", "v_mul_f32_e32 v5, v2, v2", 1),
    "dst_sel": ("v_or_b32_sdwa v9, v1, v2 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD",
                "v_add_u32_e32 v8, v9, v9", 1),
    "vgpr_mfma": ("v_and_or_b32 v111, v112, s5, v83", "v_mfma_f32_32x32x16_bf16 v[0:15], v[108:111], v[100:103], v[0:15]", 2),
    "vgpr_permlane": ("v_add_f32_e32 v84, v1, v2", "v_permlane32_swap_b32_e32 v84, v85", 2),
    "mfma_result": ("v_mfma_f32_32x32x16_bf16 v[0:15], v[108:111], v[100:103], v[0:15]", "v_mul_f32_e32 v20, v3, v3", H.MFMA_RESULT),
}


@pytest.mark.parametrize("rule", sorted(CASES))
def test_each_rule_on_a_made_up_kernel(rule):
    producer, consumer, need = CASES[rule]
    pad = ["s_mov_b32 s99, 0"]
    assert found([producer] + pad * (need - 1) + [consumer]) == [rule]
    assert found([producer] + pad * need + [consumer]) == []
    assert found([producer, f"s_nop {need - 1}", consumer]) == []
    if need > 1:
        assert found([producer, f"s_nop {need - 2}", consumer]) == [rule]


def test_paths_not_address_order_decide():
    # the producer sits at the end of a loop body, the consumer at its head; and out of line behind the kernel's end
    loop = ["s_mov_b32 s3, 4", "head:", "global_load_dword v1, v2, s[22:23]", "s_nop 7", "v_readfirstlane_b32 s22, v62",
            "s_sub_u32 s3, s3, 1", "s_cmp_lg_u32 s3, 0", "s_cbranch_scc1 head"]
    assert found(loop) == ["sgpr_vmem"]
    assert found(loop[:5] + ["s_nop 1"] + loop[5:]) == []
    far = ["v_cmpx_gt_u32_e32 vcc, s9, v7", "s_cbranch_execnz far", "back:", "v_readfirstlane_b32 s10, v40", "s_endpgm",
           "far:", "s_nop 0", "s_branch back"]
    (body,) = H.kernels_of(listing(far)).values()
    assert [b[0] for b in H.check(body)] == ["exec_lane"] and len(body) == 6
    # an accumulating matrix instruction may follow the one that wrote its accumulator; any other reader may not
    mm = "v_mfma_f32_32x32x16_bf16 v[0:15], v[108:111], v[100:103], v[0:15]"
    assert found([mm, mm]) == []
    assert found([mm, "v_mfma_f32_32x32x16_bf16 v[16:31], v[0:3], v[100:103], v[16:31]"]) == ["mfma_result"]
    assert found([mm, "global_store_dword v40, v3, s[4:5]"]) == ["mfma_result"]


@pytest.mark.skipif(not (os.path.exists(OBJDUMP) and os.path.exists(LIB)), reason="needs the built library and llvm-objdump")
def test_the_built_library_leaves_every_wait_state(tmp_path):
    shutil.copy(LIB, tmp_path / "lib.so")
    subprocess.run([OBJDUMP, "--offloading", "lib.so"], cwd=tmp_path, check=True, capture_output=True)
    kernels, instructions, closest, bad = 0, 0, {}, []
    for f in sorted(os.listdir(tmp_path)):
        if "gfx950" not in f:
            continue
        text = subprocess.run([OBJDUMP, "-d", str(tmp_path / f)], check=True, capture_output=True, text=True).stdout
        for name, body in H.kernels_of(text).items():
            kernels += 1
            instructions += len(body)
            for rule, p, c, got in H.check(body, closest):
                bad.append(f"{name}: {rule}: `{p.text}` at {p.addr:#x} -> `{c.text}` at {c.addr:#x}: {got} wait states")
    assert kernels >= 50 and instructions >= 100000, (kernels, instructions)
    assert not bad, "\n".join(bad[:20])
    # The rules are neither looser nor stricter than the compiler's own: where it had to pad its own instructions
    # with s_nop, what it left is exactly the figure of the rule.
    for rule in ("sgpr_vmem", "sgpr_valu", "vgpr_dpp", "vgpr_readlane", "trans_use", "dst_sel", "vgpr_mfma", "vgpr_permlane",
                 "mfma_result"):
        assert closest.get(rule) == CASES[rule][2], (rule, closest.get(rule))


# What one pass of each hand-scheduled loop issues, by class, in the built library (steps = decode steps of the
# 64 streams of a wavefront).  The loops are assembly text, so these are exact, and a change to the step shows up here:
# ten vector instructions and two LDS reads per step are what bounds every kernel built on it.  The two-byte
# renormalisation (about one step in a thousand) runs out of line and is not part of the loop body.
LOOPS = {
    # stand-alone decode: a pair of steps and the two exponent bytes they store
    "ci_dec_loop": dict(steps=2, valu=20, lds=4, salu=6, vmem=2, branch=4, wait=4, mfma=0),
    # fused linear, up to 32 rows of x: two blocks of eight steps, their sign|mantissa and x loads, two matrix instructions
    "ci_lin_loop": dict(steps=16, valu=164, lds=32, salu=42, vmem=18, branch=18, wait=36, mfma=2),
    # the same for 33 to 64 rows: a second x fragment per block and a second matrix instruction
    "ci_lin2_loop": dict(steps=16, valu=166, lds=32, salu=42, vmem=20, branch=18, wait=36, mfma=4),
}


@pytest.mark.skipif(not (os.path.exists(OBJDUMP) and os.path.exists(LIB)), reason="needs the built library and llvm-objdump")
def test_what_the_hand_scheduled_loops_issue_per_step(tmp_path):
    import collections
    import re

    shutil.copy(LIB, tmp_path / "lib.so")
    subprocess.run([OBJDUMP, "--offloading", "lib.so"], cwd=tmp_path, check=True, capture_output=True)
    seen = collections.Counter()
    for f in sorted(os.listdir(tmp_path)):
        if "gfx950" not in f:
            continue
        text = subprocess.run([OBJDUMP, "-d", str(tmp_path / f)], check=True, capture_output=True, text=True).stdout
        labels = {a: n for n, a in H.labels_of(text).items() if re.fullmatch(r"ci_(dec|lin|lin2)_loop\d+", n)}
        for body in H.kernels_of(text).values():
            for i, ins in enumerate(body):
                if ins.addr not in labels:
                    continue
                family = re.sub(r"\d+$", "", labels[ins.addr])
                end = next(j for j in range(i, len(body)) if body[j].mn == "s_branch" and body[j].succ == [i])
                loop = body[i:end + 1]
                count = collections.Counter(H.kind_of(k) for k in loop)
                count["steps"] = sum(1 for k in loop if k.mn == "v_mad_u32_u24")
                want = LOOPS[family]
                assert {k: count.get(k, 0) for k in want} == want, (labels[ins.addr], dict(count))
                seen[family] += 1
    # every kernel that contains a statement has its own copy of the loop
    assert seen["ci_dec_loop"] >= 2 and seen["ci_lin_loop"] >= 4 and seen["ci_lin2_loop"] >= 4, seen


@pytest.mark.skipif(not (os.path.exists(OBJDUMP) and os.path.exists(LIB)), reason="needs the built library and llvm-objdump")
def test_kernels_that_read_staged_bytes_also_stage_them(tmp_path):
    """The decode step reads its stream bytes from the LDS inside assembly statements; the bytes get there by plain
    C++ stores that nothing the compiler can see ever reads.  The statements list "memory" so that the stores stay
    where they are (tests/test_asm_clobbers.py); here the machine code itself is looked at: every kernel with the
    step's byte reads also stores to the LDS, and the sixteen-wavefront kernels, which stage a window as it lies in
    memory, sixteen bytes a lane and piece, hold those 16-byte stores."""
    shutil.copy(LIB, tmp_path / "lib.so")
    subprocess.run([OBJDUMP, "--offloading", "lib.so"], cwd=tmp_path, check=True, capture_output=True)
    seen, flat = {}, []
    for f in sorted(os.listdir(tmp_path)):
        if "gfx950" not in f:
            continue
        text = subprocess.run([OBJDUMP, "-d", str(tmp_path / f)], check=True, capture_output=True, text=True).stdout
        for name, body in H.kernels_of(text).items():
            mn = [i.text.split()[0] for i in body]
            flat += [f"{name}: {m}" for m in mn if m.startswith("flat_")]
            if "ds_read_u8" in mn:
                seen[name] = (sum(m.startswith("ds_write") for m in mn), mn.count("ds_write_b128"))
    assert len(seen) >= 20, sorted(seen)
    # (and no kernel holds a flat memory instruction: a flat load counts against the LDS counter too, which every
    # `s_waitcnt lgkmcnt` of the step would then wait for -- what a `volatile` access compiles to)
    assert flat == [], flat
    for name, (stores, wide) in seen.items():
        assert stores >= 9, (name, stores)
        if "_seg_kernel" in name:
            assert wide >= 7, (name, wide)  # one per piece of a window, at least
