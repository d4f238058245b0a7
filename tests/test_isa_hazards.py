"""Register hazards around hand-written MFMAs, checked on the compiler's assembly output (CPU test, no GPU).

The GEMM and attention kernels issue their MFMAs through inline assembly so that accumulators stay in the register
file they were put in. The compiler does not know that those statements are matrix instructions, so it neither inserts
the idle cycles the hardware wants around them nor keeps its own register copies away from them:
  * a vector instruction that writes a register an MFMA reads needs two issue slots in between;
  * a vector, LDS or memory instruction that touches an MFMA's result register needs the MFMA to have finished
    (passes + 4 issue slots for this 4-pass instruction; the kernels place sixteen idle cycles, and this test asks for 8);
  * the attention kernel also writes its exponentials as inline assembly: a transcendental's result must not be read
    by the very next instruction.
The kernels keep these apart by construction; this test compiles the files the way the Makefile does and checks every
MFMA in the inline-assembly kernels, so that a register copy the allocator slips in front of an MFMA fails here
instead of giving wrong numbers on the GPU. Instructions are taken in layout order (branches are not followed), which
is how the straight-line loops of these kernels run.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "flux2.c_amd", "csrc")
MAKEFILE = os.path.join(ROOT, "flux2.c_amd", "Makefile")


def makefile_flags(src):
    """The device-side compile flags the Makefile uses for csrc/<src>: HIPFLAGS with $(ARCH) expanded, plus the
    file's own FLAGS_<name> if it has one. Read from the Makefile so that this test compiles what ships."""
    text = open(MAKEFILE).read()

    def var(name):
        m = re.search(r"^%s\s*\??=\s*(.*)$" % re.escape(name), text, flags=re.M)
        return m.group(1).strip() if m else ""

    flags = var("HIPFLAGS").replace("$(ARCH)", var("ARCH")).split()
    assert any(f.startswith("--offload-arch=gfx") for f in flags) and "-packed-fp32-ops" in flags, flags
    return flags + var("FLAGS_" + os.path.splitext(src)[0]).split()


def compile_device(src, out, extra):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc is not installed")
    r = subprocess.run([hipcc] + makefile_flags(src) + ["--cuda-device-only"] + extra + [os.path.join(CSRC, src), "-o", str(out)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return r

VALU_TO_MFMA_SLOTS = 2
TRANS = ("v_exp_", "v_log_", "v_rcp_", "v_rsq_", "v_sqrt_", "v_sin_", "v_cos_")
MFMA_RESULT_SLOTS = 8


def regs(tok):
    """'v[4:7]' -> {('v',4..7)}, 'a12' -> {('a',12)}; anything else -> empty."""
    m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.fullmatch(r"([va])(\d+)", tok)
    if m:
        return {(m.group(1), int(m.group(2)))}
    return set()


def parse(line):
    line = line.split(";")[0].strip()
    if not line or line.endswith(":") or line.startswith("."):
        return None
    parts = line.split(None, 1)
    op = parts[0]
    ops = [t.strip() for t in re.split(r",\s*", parts[1])] if len(parts) > 1 else []
    ops = [t.split()[0] if t else t for t in ops]          # drop modifiers such as 'offset:16'
    return op, ops


def kernel_bodies(asm):
    out, name, body = {}, None, []
    for line in asm.splitlines():
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, body = m.group(1), []
            continue
        if name:
            if re.match(r"^\.Lfunc_end\d+:", line):     # the end of the function (a kernel may hold several s_endpgm)
                out[name] = body
                name = None
            else:
                body.append(line)
    return out


def lint(body):
    """Returns a list of (line number in the kernel, message)."""
    problems = []
    recent_valu = []      # (slots ago, registers written, text)
    recent_mfma = []      # (slots ago, result registers, text)
    for ln, line in enumerate(body):
        p = parse(line)
        if not p:
            continue
        op, ops = p
        slots = 1
        if op == "s_nop":
            slots = int(ops[0]) + 1
        is_mfma = op.startswith("v_mfma")
        written, read = set(), set()
        if is_mfma:
            written = regs(ops[0])
            for t in ops[1:4]:
                read |= regs(t)
        elif op.startswith("v_") and not op.startswith("v_cmp"):
            written = regs(ops[0]) if ops else set()
            for t in ops[1:]:
                read |= regs(t)
        elif op.startswith(("ds_read", "global_load", "buffer_load", "scratch_load")):
            written = regs(ops[0]) if ops and not op.startswith("global_load_lds") else set()
            for t in ops[1:] if written else ops:
                read |= regs(t)
        else:
            for t in ops:
                read |= regs(t)
        for ago, w, text in recent_valu:
            if ago == 0 and text.startswith(TRANS) and w & read:
                problems.append((ln, f"'{line.strip()}' reads the result of '{text}' in the next slot"))
        if is_mfma:
            for ago, w, text in recent_valu:
                if ago < VALU_TO_MFMA_SLOTS and w & read:
                    problems.append((ln, f"MFMA reads a register {ago} slot(s) after '{text}' wrote it: {line.strip()}"))
        else:
            for ago, w, text in recent_mfma:
                if ago < MFMA_RESULT_SLOTS and w & (read | written):
                    problems.append((ln, f"'{line.strip()}' touches the result of '{text}' {ago} slot(s) after it was issued"))
        recent_valu = [(a + slots, w, t) for a, w, t in recent_valu if a + slots < 4]
        recent_mfma = [(a + slots, w, t) for a, w, t in recent_mfma if a + slots < MFMA_RESULT_SLOTS + 2]
        if is_mfma:
            recent_mfma.append((0, written, line.strip()))
        elif op.startswith("v_") and written:
            recent_valu.append((0, written, line.strip()))
    return problems


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    """Assembly text and resource-usage remarks of gemm.hip and attention.hip, compiled once per test run."""
    out = {}
    for src in ("gemm.hip", "attention.hip"):
        path = tmp_path_factory.mktemp("asm") / (src + ".s")
        r = compile_device(src, path, ["-S", "-Rpass-analysis=kernel-resource-usage"])
        out[src] = (path.read_text(), r.stderr)
    return out


@pytest.mark.parametrize("src,pattern", [("attention.hip", "attention_wide_kernel"), ("gemm.hip", "gemm4w_kernel"), ("gemm.hip", "gemm4d_kernel")])
def test_inline_asm_mfma_hazards(src, pattern, assembly):
    kernels = {k: v for k, v in kernel_bodies(assembly[src][0]).items() if pattern in k}
    assert kernels, f"no kernel named *{pattern}* in {src}"
    report = []
    for name, body in sorted(kernels.items()):
        assert any("v_mfma" in l for l in body), name
        for ln, msg in lint(body):
            report.append(f"{name} +{ln}: {msg}")
    assert not report, "\n".join(report[:40]) + f"\n({len(report)} in all)"


def test_the_lint_sees_a_planted_hazard():
    body = ["\tv_mov_b32_e32 v5, v9", "\tv_mfma_f32_16x16x32_bf16 v[0:3], v[4:7], v[8:11], v[0:3]", "\tv_add_f32_e32 v20, v1, v1",
            "\ts_nop 7", "\tv_add_f32_e32 v21, v2, v2", "\ts_endpgm"]
    found = lint(body)
    assert len(found) == 2 and "MFMA reads" in found[0][1] and "touches the result" in found[1][1]
    assert len(lint(["\tv_exp_f32_e32 v1, v1", "\tv_cvt_pk_bf16_f32 v2, v1, v3", "\ts_endpgm"])) == 1
    assert not lint(["\tv_exp_f32_e32 v1, v1", "\tv_exp_f32_e32 v3, v3", "\tv_cvt_pk_bf16_f32 v2, v1, v4", "\ts_endpgm"])
    clean = ["\tv_mov_b32_e32 v5, v9", "\ts_nop 1", "\tv_mfma_f32_16x16x32_bf16 v[0:3], v[4:7], v[8:11], v[0:3]", "\ts_nop 7",
             "\tv_add_f32_e32 v20, v1, v1", "\ts_endpgm"]
    assert not lint(clean)


def resource_usage(remarks):
    """{mangled kernel name: {field: int}} from the compiler's -Rpass-analysis=kernel-resource-usage remarks."""
    out, name = {}, None
    for line in remarks.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            out[name] = {}
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+) \[-Rpass", line)
        if m and name:
            out[name][m.group(1).strip()] = int(m.group(2))
    return out


def innermost_loops(body):
    """(first line, last line) of every loop of the kernel that holds no other loop: label ... backward branch to it."""
    labels = {}
    for ln, line in enumerate(body):
        m = re.match(r"^(\.LBB\d+_\d+):", line)
        if m:
            labels[m.group(1)] = ln
    loops = []
    for ln, line in enumerate(body):
        m = re.search(r"\bs_c?branch\w*\s+(\.LBB\d+_\d+)", line)
        if m and labels.get(m.group(1), len(body)) < ln:
            loops.append((labels[m.group(1)], ln))
    return [(a, b) for a, b in loops if not any((c, d) != (a, b) and a <= c and d <= b for c, d in loops)]


def test_gemm_kernels_fit_the_register_file(assembly):
    """No GEMM kernel may spill: a spilled register is a scratch store next to the next tile's primed loads (the
    compiler waits for all of them first), and the fused [Q|K|V|gate|up] epilogue went over the ceiling that way
    before its two store bodies were kept apart. Every kernel of gemm.hip: no scratch frame, no spilled VGPR or SGPR.
    The 4-wave kernels keep their accumulators in AGPRs and nothing else (AGPRs == 16 TM TN / 4 means that no vector
    register was parked there either), and their K loops free of copies between the two register files. The residual
    epilogue keeps two row blocks of the residual in flight and may use the whole VGPR file; the other transformer
    epilogues stay under 200 VGPRs."""
    usage = resource_usage(assembly["gemm.hip"][1])
    big = {k: v for k, v in usage.items() if "gemm4d_kernel" in k or "gemm4w_kernel" in k}
    assert len(big) >= 60 and len(usage) >= 100, (len(big), len(usage))
    bad = []
    for name, u in sorted(usage.items()):
        if u["ScratchSize"] or u["VGPRs Spill"] or u["SGPRs Spill"]:
            bad.append((name, u))
    assert not bad, bad
    bodies = kernel_bodies(assembly["gemm.hip"][0])
    for name, u in sorted(big.items()):
        tm, tn, epi = map(int, re.search(r"kernelILi(\d+)ELi(\d+)ELi(\d+)E", name).groups())
        assert u["AGPRs"] == 4 * tm * tn, (name, u)
        if epi not in (3, 6, 7):                 # (the convolution epilogues sit at 252-256, unspilled; the residual one at up to 256)
            assert u["VGPRs"] <= 200, (name, u)  # room to spare: 180 at most when this was written
        body = bodies[name]
        k_loops = [(a, b) for a, b in innermost_loops(body) if sum("v_mfma" in l for l in body[a:b]) >= 2 * tm * tn]
        assert k_loops, name
        for a, b in k_loops:
            copies = [l.strip() for l in body[a:b] if "v_accvgpr" in l or "scratch_" in l]
            assert not copies, (name, copies[:4])


def test_the_loop_finder_sees_a_planted_copy():
    body = [".LBB0_1:", "\tv_mfma_f32_16x16x32_bf16 a[0:3], v[4:7], v[8:11], a[0:3]", ".LBB0_2:", "\tv_accvgpr_read_b32 v1, a9",
            "\tv_mfma_f32_16x16x32_bf16 a[0:3], v[4:7], v[8:11], a[0:3]", "\ts_cbranch_scc1 .LBB0_2", "\ts_cbranch_vccnz .LBB0_1", "\ts_endpgm"]
    assert innermost_loops(body) == [(2, 5)]
    assert any("v_accvgpr" in l for l in body[2:5])


def test_attention_kernels_need_no_scratch_memory(assembly):
    """The flash kernels keep everything in registers: no scratch frame (a frame would have to be backed for every
    launch, and an out-of-line way out once gave the wide kernels one that only a rare path touched), nothing spilled
    to memory."""
    usage = {k: v for k, v in resource_usage(assembly["attention.hip"][1]).items() if "attention" in k}
    assert len(usage) >= 5, sorted(usage)
    for name, u in sorted(usage.items()):
        assert u["ScratchSize"] == 0 and u["VGPRs Spill"] == 0, (name, u)      # (spilled SGPRs go to lanes of a VGPR, not to memory)


def test_the_remark_parser_reads_the_fields_the_test_uses():
    text = ("x.hip:1:1: remark: Function Name: _Z1kv [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:1:1: remark:     VGPRs: 12 [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:1:1: remark:     AGPRs: 4 [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 8 [-Rpass-analysis=kernel-resource-usage]\n"
            "x.hip:1:1: remark:     VGPRs Spill: 1 [-Rpass-analysis=kernel-resource-usage]\n")
    assert resource_usage(text) == {"_Z1kv": {"VGPRs": 12, "AGPRs": 4, "ScratchSize": 8, "VGPRs Spill": 1}}
