"""The C ABI called from compiled code: tests/cabi_host/conv_host.cpp, built next to the library by
`python -m flexgemm_amd.build`, runs one convolution (cache, forward, both gradients) with no Python and no torch in its
process and checks it against host loops written from the operator's definition.  Channel counts are whole 16-byte
chunks (four fp32 values): the entry points refuse other rows, which the Python layer pads before it calls them."""
import os
import subprocess

import pytest

from flexgemm_amd import build

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("res,ci,co", [(14, 24, 40), (20, 64, 64), (9, 4, 12), (24, 8, 136)])
def test_convolution_from_a_host_program_without_torch(gpu_device, res, ci, co):
    assert os.path.exists(build.HOST_CHECK), "the host program is not built: run python -m flexgemm_amd.build"
    print(f"[case] host program res={res} ci={ci} co={co}", flush=True)
    done = subprocess.run([build.HOST_CHECK, str(res), str(ci), str(co)], capture_output=True, text=True, timeout=100)
    print(done.stdout, done.stderr, flush=True)
    assert done.returncode == 0 and done.stdout.strip().endswith("ok"), done.stderr
