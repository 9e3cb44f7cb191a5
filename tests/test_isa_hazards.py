"""Static check of the compiled matrix-core kernels: no vector instruction may read the destination of a matrix
instruction within a few issue slots of it on ANY control-flow path.

One build of the backward kernel had a branch between the last matrix instruction of a score tile and the first read
of its result; the compiler's wait states covered the fall-through path only, and the taken path read half-finished
sums (wrong gradients for some shapes, no error).  The kernels avoid such branches; this test compiles them to
assembly (no GPU needed) and walks every path behind every matrix instruction."""
import os
import re
import subprocess
import tempfile

import pytest

from vig_amd import build as B

SOURCES = ["gla_tiles.hip", "gla_mfma.hip", "gla_backward_mfma.hip", "gates.hip", "patch_conv.hip", "linear.hip"]
WINDOW = 8  # issue slots behind a 32x32x16 matrix instruction in which its destination must not be read


def _regs(text):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]", text):
        out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\bv(\d+)\b", text):
        out.add(int(m.group(1)))
    return out


def early_reads(asm: str, window: int = WINDOW):
    lines = asm.split("\n")
    labels = {m.group(1): i for i, l in enumerate(lines) if (m := re.match(r"^(\.LBB\w+):", l))}
    mfma = re.compile(r"v_mfma_\w+\s+v\[(\d+):(\d+)\]")
    found = []
    for i, l in enumerate(lines):
        m = mfma.search(l)
        if not m:
            continue
        dst = set(range(int(m.group(1)), int(m.group(2)) + 1))
        stack, seen = [(i + 1, 0)], set()
        while stack:
            k, slots = stack.pop()
            while k < len(lines) and slots < window and k not in seen:
                seen.add(k)
                t = lines[k].strip()
                k += 1
                if not t or t.startswith(";") or t.startswith(".") or t.endswith(":"):
                    continue
                op = t.split()[0]
                if op == "s_nop":
                    slots += int(t.split()[1]) + 1
                elif op.startswith("s_cbranch"):
                    if t.split()[1] in labels:
                        stack.append((labels[t.split()[1]], slots + 1))
                    slots += 1
                elif op == "s_branch":
                    k = labels.get(t.split()[1], len(lines))
                    slots += 1
                elif op == "s_endpgm":
                    break
                elif op.startswith("v_mfma"):
                    if _regs(t.split(",")[0]) & dst:
                        break  # accumulates into / overwrites the same registers: interlocked by hardware
                    slots += 8
                else:
                    stores = ("ds_write", "buffer_store", "global_store", "scratch_store")
                    srcs = t if op.startswith(stores) else (",".join(t.split(",")[1:]) if "," in t else "")
                    if _regs(srcs) & dst:
                        found.append((i + 1, l.strip(), k, slots, t))
                        break
                    slots += 1
    return found


def test_checker_sees_the_pattern():
    asm = """
.LBB0_1:
\tv_mfma_f32_32x32x16_bf16 v[0:15], v[70:73], v[28:31], v[0:15]
\ts_cbranch_scc1 .LBB0_3
\ts_nop 10
\tv_cndmask_b32_e64 v0, v0, 0, s[44:45]
.LBB0_3:
\tv_cvt_pk_bf16_f32 v71, v2, v3
\ts_endpgm
"""
    hits = early_reads(asm)
    assert len(hits) == 1 and "v_cvt_pk_bf16_f32" in hits[0][4]
    assert early_reads(asm.replace("\ts_cbranch_scc1 .LBB0_3\n", "")) == []


@pytest.mark.parametrize("src", SOURCES)
def test_no_early_read_of_matrix_results(src):
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, src + ".s")
        cmd = [B.HIPCC, *[f for f in B.FLAGS if f != "-fPIC"], "-S", "--cuda-device-only", "-I", B.CSRC,
               os.path.join(B.CSRC, src), "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        hits = early_reads(open(out).read())
    assert hits == [], "\n".join(f"line {a}: {b}  ->  line {c} after {d} slots: {e}" for a, b, c, d, e in hits[:10])
