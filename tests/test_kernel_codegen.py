"""What the compiler made of the dense tile kernel's K loop, checked on the assembly (no GPU needed: hipcc cross-compiles).

The four-wavefront dense kernel runs one wavefront per SIMD, so its speed rests on properties of the generated loop that
no numerical test sees: all 256 accumulators stay in their accumulation registers across the loop (small changes to the
source have made the register allocator move them through vector registers every iteration, 14 % slower with identical
results), the loop is fully unrolled (128 matrix instructions per K step, two steps per iteration), and nothing spills.

The counts below are those of ROCm 7.2's hipcc on the source as committed.  Another compiler version may schedule or
allocate differently without anything being wrong with the kernel: a failure here after a toolchain change alone means
"measure the dense kernel again" (bench.py, gemm.roofline), not "the kernel is broken".
"""
import os
import re
import shutil
import subprocess

import pytest

from sensenova_u1_amd import build


def _assembly(tmp_path, src):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    out = tmp_path / (os.path.splitext(src)[0] + ".s")
    cmd = [hipcc, *build.HIP_FLAGS, *build.SOURCE_FLAGS.get(src, []), "-x", "hip", "-S", "--cuda-device-only",
           os.path.join(build.CSRC, src), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return out.read_text()


def test_dense_kernel_loop_keeps_its_accumulators_in_place(tmp_path):
    text = _assembly(tmp_path, "gemm_dense4.hip")
    lines = text.splitlines()
    starts = [i for i, l in enumerate(lines) if re.match(r"^_ZN6sngguf.*gemm_dense4_kernelILi\dEEE.*:", l)]
    assert len(starts) == 4, "one kernel instance per epilogue"
    for s in starts:
        name = lines[s].split(":")[0]
        end = next(i for i in range(s, len(lines)) if lines[i].startswith(".Lfunc_end"))
        # basic blocks of the function: the K loop is the one with the most matrix instructions
        blocks, cur = [], []
        for l in lines[s:end]:
            if re.match(r"^\.LBB\d+_\d+:", l):
                blocks.append(cur)
                cur = []
            cur.append(l)
        blocks.append(cur)
        loop = max(blocks, key=lambda b: sum("v_mfma_f32_16x16x32_bf16" in l for l in b))
        count = lambda pat: sum(bool(re.search(pat, l)) for l in loop)
        assert count(r"v_mfma_f32_16x16x32_bf16") == 256, name          # two K steps of 128, fully unrolled
        assert count(r"v_accvgpr_(read|write|mov)") == 0, name           # accumulators stay where they are
        assert count(r"\bds_read_b128\b") == 64, name                    # 16 fragments per half step
        assert count(r"global_load_lds_dwordx4") == 32, name             # 16 copies per step
        assert count(r"scratch_(load|store)") == 0, name
    for field in ("vgpr_spill_count", "sgpr_spill_count", "private_segment_fixed_size"):
        vals = re.findall(rf"\.{field}:\s+(\d+)", text)
        assert vals and all(v == "0" for v in vals), (field, vals)
