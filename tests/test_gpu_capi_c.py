"""The C-ABI from plain C: tests/capi_smoke.c (built by flux_amd.build into flux_amd/lib/capi_smoke) links
libfluxmi_kernels.so and the HIP runtime only, runs routing, the gathered grouped GEMM, the top-k gather-reduce and
the row quantisation on small inputs and checks them against loops of its own."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu


def test_c_host_program_runs_the_path():
    from flux_amd import build
    exe = build.CAPI_SMOKE
    assert os.path.exists(exe), f"{exe} is missing: build it with `python -m flux_amd.build`"
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    print(proc.stdout, flush=True)
    assert proc.returncode == 0, proc.stdout
    for part in ("routing ok", "grouped gemm ok", "gather-reduce ok", "quant ok", "all checks passed"):
        assert part in proc.stdout
