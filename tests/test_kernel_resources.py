"""Static check of the kernels that count their own outstanding vector-memory operations (inline-asm loads,
stores and DMAs waited for with hand-written s_waitcnt vmcnt(N)): a register spill would add scratch
loads and stores that those counts do not know about, so these kernels must compile without scratch.
Cross-compiles every GEMM translation unit for gfx950 (no GPU needed; the units compile in parallel)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "mase-triton_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


COUNTED = ("gemm_tall_kernel", "gemm_skinny_kernel", "gemm_mid_kernel", "gemm_wide_kernel", "gemm_rows16_kernel", "gemm_scaled_kernel")
UNITS = {"gemm_w_e4m3": 6, "gemm_w_e5m2": 6, "gemm_w_e2m3": 6, "gemm_w_e3m2": 6, "gemm_w_e2m1": 6, "gemm_scaled": 3}  # unit -> least number of such kernels


def _assembly(unit, folder):
    out = os.path.join(folder, unit + ".s")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "--cuda-device-only", "-S", os.path.join(CSRC, unit + ".hip"), "-o", out]
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, timeout=900)
    with open(out) as f:
        return f.read()


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not available")
def test_counted_wait_kernels_use_no_scratch(tmp_path):
    from concurrent.futures import ThreadPoolExecutor

    with ThreadPoolExecutor(max_workers=6) as ex:
        texts = dict(zip(UNITS, ex.map(lambda u: _assembly(u, str(tmp_path)), UNITS)))
    for unit, text in texts.items():
        names = re.findall(r"^(_ZN4mase\w+):\s*; @", text, re.M)
        scratch = re.findall(r"; ScratchSize: (\d+)", text)
        assert len(names) == len(scratch) > 0, unit
        checked = 0
        for name, size in zip(names, scratch):
            if any(tag in name for tag in COUNTED):
                assert int(size) == 0, f"{unit}: {name} spills ({size} bytes of scratch): its s_waitcnt counts would be wrong"
                checked += 1
        assert checked >= UNITS[unit], f"{unit}: {checked} kernels with counted waits found"
        # M0 carries the LDS address of the DMAs between inline-asm statements: nothing else may write it
        m0_writes = [ln for ln in text.splitlines() if re.search(r"\bm0\b", ln) and not ln.strip().startswith(";")]
        assert all(re.match(r"\s*s_mov_b32 m0, s\d+", ln) for ln in m0_writes), (unit, m0_writes[:5])
