"""The C ABI from a process with no Python and no PyTorch in it: tests/c_abi/decode_from_c (built with the library by
`python -m loongserve_amd.build`) allocates with the HIP runtime, calls lsattn_decode_attention and
lsattn_decode_attention_static, and checks both against a double-precision loop on the host."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi", "decode_from_c")


@pytest.mark.parametrize("Hq,Hkv", [(32, 8), (8, 1), (16, 16)])
def test_decode_through_the_c_abi_from_a_c_program(Hq, Hkv):
    assert os.path.exists(BIN), "run `python -m loongserve_amd.build` first"
    r = subprocess.run([BIN, str(Hq), str(Hkv)], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok" in r.stdout.splitlines()[-1]
