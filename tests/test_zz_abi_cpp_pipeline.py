"""The C-ABI driven from plain C++ with hipMalloc'd buffers, no Python and no
torch in the process: tests/abi_pipeline.cpp walks grid set-up, keys, sort,
gathers, grid table, neighbour search, densities and basis projection on a seeded
cloud and compares every stage with the CPU oracle (integers bit-exact, floats
within 1e-5).  The program is built beforehand (tests/Makefile, from
__graft_entry__.build()); this test only runs it, as a child process."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_host_program_matches_oracle():
    exe = os.path.join(HERE, "abi_pipeline")
    if not os.path.exists(exe):
        pytest.fail("tests/abi_pipeline is not built; run __graft_entry__.build()")
    done = subprocess.run([exe], capture_output=True, text=True, timeout=150)
    print(done.stdout)
    print(done.stderr)
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
    assert "abi_pipeline ok" in done.stdout
    for stage in ("compute_keys", "sorted_indices", "build_grid_ds", "neighbour pairs",
                  "compute_pdf", "basis_proj"):
        assert stage in done.stdout
