"""Rules that the kernel sources keep, checked on their text (no compiler, no GPU)."""
import glob
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "hf.cpu_amd", "csrc")


def asm_statements(text):
    """Every ``asm volatile( ... );`` of a source as (line number, text of the statement)."""
    out = []
    for m in re.finditer(r"asm\s+volatile\s*\(", text):
        depth, i = 0, m.end() - 1
        while True:
            c = text[i]
            if c == "(":
                depth += 1
            elif c == ")":
                depth -= 1
                if depth == 0:
                    break
            i += 1
        out.append((text.count("\n", 0, m.start()) + 1, text[m.start():i + 1]))
    return out


def test_no_memory_instruction_in_assembly_reads_a_scalar_operand_of_its_statement():
    """A memory instruction may read a scalar register no sooner than five wait states after a vector instruction
    wrote it (v_readlane when the compiler brings back a scalar that it had put aside, v_readfirstlane), and the
    compiler keeps no such distance from assembly that it cannot read: a kernel with many live scalars once loaded
    weights from stale addresses. The rule since then: a statement that asks memory for something names its
    address in scalar registers that a scalar move INSIDE the statement has written (an "=&s" temporary), never
    in an "s" input directly."""
    seen = 0
    for path in sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.h"))):
        text = open(path).read()
        for line, stmt in asm_statements(text):
            body = " ".join(re.findall(r'"((?:[^"\\]|\\.)*)"', stmt.split("::")[0].split(" : ")[0]))
            loads = re.findall(r"(?:global|buffer|flat)_(?:load|store|atomic)\w*[^\\]*", body)
            if not loads:
                continue
            seen += 1
            # operands in order: outputs first, then inputs; find which numbers are "s" inputs
            constraints = re.findall(r'"([=&+]*[a-zA-Z]+)"\s*\(', stmt)
            scalar_inputs = {i for i, c in enumerate(constraints) if c == "s"}
            for ins in loads:
                used = {int(n) for n in re.findall(r"%(\d+)", ins)}
                direct = used & scalar_inputs
                assert not direct, (f"{os.path.relpath(path, ROOT)}:{line}: '{ins.strip()}' reads scalar input operand(s) "
                                    f"{sorted(direct)} directly; copy them with s_mov inside the statement first")
    assert seen >= 4, "the kernels with direct loads into LDS were meant to be looked at"


def test_hip_is_compiled_without_packed_fp32_operations():
    from hf_cpu_amd.kernels import build
    flags = " ".join(build.FLAGS)
    assert "-target-feature" in flags and "-packed-fp32-ops" in flags
