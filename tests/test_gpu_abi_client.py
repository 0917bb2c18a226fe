"""The C ABI from a process without Python or PyTorch: ``tests/abi_client.c`` (built by ``relax_amd/build.py`` next to
the library's objects) allocates with hipMalloc, calls the entry points declared in ``include/relax_amd.h`` with plain
pointers and checks log-probs, entropy, dlogits and the reverse KL of a three-row literal against closed forms."""

import os
import subprocess

import pytest

from tests.gpu_util import announce, require_gpu

pytestmark = pytest.mark.gpu


def test_c_client_runs_the_library_without_python_or_torch():
    require_gpu()
    announce("C client of the ABI")
    from relax_amd.build import ABI_CLIENT

    assert os.path.exists(ABI_CLIENT), f"{ABI_CLIENT} is missing: run python relax_amd/build.py"
    r = subprocess.run([ABI_CLIENT], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert "abi_client ok" in r.stdout
