"""A compiled C++ host program over include/dgpp_amd.hpp (tests/cpp/host_program.cpp, built by dgpp_amd/build.py)
runs on the GPU: the reference's geometry-rejection tests through the dgpp::launch_* names and the reference's
decode call order stitched from the shim's launchers, bit for bit the layer driver."""
import subprocess
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

PROGRAM = Path(__file__).resolve().parents[1] / "dgpp_amd" / "lib" / "dgpp_host_program"


def test_host_program_passes_on_the_gpu():
    assert PROGRAM.exists(), f"{PROGRAM} is missing: build it with `python -m dgpp_amd.build`"
    print("running the compiled host program", flush=True)
    run = subprocess.run([str(PROGRAM)], capture_output=True, text=True, timeout=300)
    print(run.stdout)
    print(run.stderr)
    assert run.returncode == 0, f"host program failed ({run.returncode}):\n{run.stdout}\n{run.stderr}"
    assert "all checks passed" in run.stdout
    assert run.stdout.count("[ OK ]") >= 4
