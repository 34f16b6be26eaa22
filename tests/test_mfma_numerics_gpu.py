"""What the kernels assume of the matrix cores, checked on the part itself.

The product kernels run e4m3 / e5m2 widened to f16 on the f16 MFMA because the fp8 MFMA forms of gfx950 align the
products inside one lane's group to the largest of them and drop the low bits, while the f16 and bf16 forms add exact
products without loss inside an instruction. `tests/probes/mfma_probes numerics --check` (source:
tests/probes/mfma_probes.hip) measures both and fails if the f16 / bf16 forms lose bits or the f16 route is
not the more accurate one on a depth-8192 e4m3 dot product."""
import os
import subprocess

import pytest

from tests import support

pytestmark = pytest.mark.gpu
PROBE = os.path.join(support.ROOT, "tests", "probes", "mfma_probes")


def test_matrix_core_numerics(capsys):
    assert os.path.exists(PROBE), "build tests/probes/mfma_probes with `make -C tests/probes`"
    done = subprocess.run([PROBE, "numerics", "--check"], capture_output=True, text=True, timeout=120)
    with capsys.disabled():
        print("\n" + done.stdout)
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
