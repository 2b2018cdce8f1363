"""The decode kernels' register / LDS budget, read from the compiler's resource report (no GPU needed: hipcc cross-compiles).
The design leans on it: a spill reload inside the key loop is a vector load that drains the whole tile queue, any scratch
at all costs a launch about 0.7 us, and the single-buffered build only pays if two of its workgroups fit a CU (half the
register file, 80 KB of LDS)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "p100e-engine_amd", "csrc")


def resource_report(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc here")
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + SRC,
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-inline-asm",
           "-Rpass-analysis=kernel-resource-usage", "--cuda-device-only", "-c", os.path.join(SRC, "p1a_decode.hip"),
           "-o", str(tmp_path / "dec.o")]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    kernels, cur = {}, None
    for line in r.stderr.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            cur = kernels.setdefault(m.group(1), {})
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+)", line)
        if m and cur is not None:
            cur[m.group(1).strip()] = int(m.group(2))
    return kernels


def test_decode_kernels_fit_their_budget(tmp_path):
    ks = {k: v for k, v in resource_report(tmp_path).items() if "dec_mfma_k" in k}
    assert len(ks) >= 12, sorted(ks)
    for name, r in ks.items():
        assert r.get("VGPRs Spill", 0) == 0 and r.get("SGPRs Spill", 0) == 0, (name, r)
        assert r.get("ScratchSize", 0) == 0, (name, r)
    # dec_mfma_k<KT, D, NT, NW, SB, KS>: the mangled name ends ...ELi<NW>ELb<SB>ELj<KS>EEEv...
    sb = {k: v for k, v in ks.items() if re.search(r"ELb1ELj\d+EEEv", k)}
    assert len(sb) >= 5, sorted(ks)
    # the staged builds (KS != KT: q8_0 / q4_0 at D = 64, 128 converted to f16 tiles) are there, one workgroup per CU
    staged = {k: v for k, v in ks.items() if re.search(r"ILj1ELi(64|128)ELi[12]ELi8ELb0ELj[28]EEEv", k)}
    assert len(staged) == 8, sorted(ks)
    for name, r in staged.items():
        assert r["LDS Size"] <= 160 * 1024, (name, r)
    for name, r in sb.items():
        waves = int(re.search(r"ELi(\d+)ELb1ELj\d+EEEv", name).group(1))
        assert r["LDS Size"] <= 80 * 1024, (name, r)                       # two workgroups in 160 KB
        assert r["Occupancy"] * 4 >= 2 * waves, (name, r)                   # two workgroups' waves on the 4 SIMDs
