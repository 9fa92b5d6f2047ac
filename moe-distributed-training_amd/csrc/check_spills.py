#!/usr/bin/env python3
"""Compiles grouped_gemm.hip with the compiler's resource-usage remarks and fails if a kernel variant of the usual shapes
spills registers: the main loop of those variants sits at the edge of the scalar and vector register budgets, and a
variant that spills a few scalar registers runs 1.5-2.5 % slower.  The general-shape variants (last template argument
true) may spill scalar registers; no variant may spill vector registers.  Usage: make -C csrc check-spills"""
import re
import subprocess
import sys

cmd = sys.argv[1:]
out = subprocess.run(cmd, capture_output=True, text=True)
text = out.stdout + out.stderr
name, bad, seen = None, [], 0
for line in text.splitlines():
    m = re.search(r"Function Name: (\S+)", line)
    if m:
        name = m.group(1)
        continue
    m = re.search(r"(SGPRs|VGPRs) Spill: (\d+)", line)
    if m and name and "grouped_gemm_mfma_kernel" in name:
        seen += 1
        general = name.endswith("Lb1EEEv13MoeGemmParams")
        if int(m.group(2)) > 0 and (m.group(1) == "VGPRs" or not general):
            bad.append(f"{name}: {m.group(1)} spill {m.group(2)}")
if out.returncode != 0 or seen == 0:
    sys.stderr.write(text[-2000:])
    sys.exit("check-spills: the compile failed or printed no resource usage")
if bad:
    sys.exit("check-spills: register spills in hot kernel variants:\n  " + "\n  ".join(bad))
print(f"check-spills: {seen // 2} grouped GEMM variants, no spills in the variants of the usual shapes")
