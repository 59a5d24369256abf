"""Register budget of the two headline kernels, read from the compiler's own
resource report (no GPU needed).  Both ZFP fp32 kernels are held to five
wavefronts per SIMD, i.e. at most 96 vector registers, and must reach that
without scratch memory: a spill costs more HBM traffic than the occupancy wins.
Register allocation at this limit is sensitive to small source changes, so the
check runs with the other CPU tests."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

from conftest import ROOT

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not available")
def test_zfp_fp32_kernels_fit_five_waves_without_scratch():
    src = os.path.join(ROOT, "cswap_amd", "csrc", "zfp_kernels.hip")
    with tempfile.TemporaryDirectory() as d:
        from cswap_amd.build import HIPCC_FLAGS      # the flags the shipped library is built with

        out = subprocess.run(
            [HIPCC, *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage", "--cuda-device-only", "-x", "hip",
             "-c", src, "-o", os.path.join(d, "k.o")],
            capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    kernels = {}
    name = None
    for line in out.stderr.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            kernels[name] = {}
            continue
        m = re.search(r"\s(VGPRs|ScratchSize \[bytes/lane\]|Occupancy \[waves/SIMD\]): (\d+)", line)
        if m and name:
            kernels[name][m.group(1).split()[0]] = int(m.group(2))
    f32 = {k: v for k, v in kernels.items() if "zfp_encode3_f32_kernel" in k or "zfp_decode3_f32_kernel" in k}
    # 4 decoders, 4 encoders, 2 encoders that load with the nontemporal hint, all for five wavefronts per SIMD;
    # for 16 bits per value and more, 4 encoders built for three and 2 decoders built for four
    assert len(f32) == 16, sorted(kernels)
    fewer = {"Li3E": 0, "Li4E": 0}
    for k, v in f32.items():
        assert v["ScratchSize"] == 0, (k, v)
        if "Li3E" in k:
            fewer["Li3E"] += 1
            assert "encode" in k and v["VGPRs"] <= 168 and v["Occupancy"] >= 3, (k, v)
        elif "Li4E" in k:
            fewer["Li4E"] += 1
            assert "decode" in k and v["VGPRs"] <= 128 and v["Occupancy"] >= 4, (k, v)
        else:
            assert v["VGPRs"] <= 96 and v["Occupancy"] >= 5, (k, v)
    assert fewer == {"Li3E": 4, "Li4E": 2}, fewer
    # the pair forms for small fields (two wavefronts per 64 blocks): small enough in registers that
    # the LDS of their workgroups, not the register file, bounds how many are resident
    pair = {k: v for k, v in kernels.items() if "pair_kernel" in k}
    assert len(pair) == 2, sorted(kernels)
    for k, v in pair.items():
        assert v["ScratchSize"] == 0 and v["VGPRs"] <= 72 and v["Occupancy"] >= 7, (k, v)
    for k, v in kernels.items():                       # the other kernels: no scratch either
        assert v["ScratchSize"] == 0, (k, v)
