"""The C ABI from processes with no Python and no PyTorch in them (built with the library by
`python -m loongserve_amd.build`): tests/c_abi/decode_from_c allocates with the HIP runtime, calls lsattn_decode_attention
and lsattn_decode_attention_static, and checks both against a double-precision loop on the host; tests/c_abi/prefill_from_c
does the same for lsattn_prefill_step and lsattn_prefill_step_accumulate on a striped, ragged ring step."""
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


def test_prefill_through_the_c_abi_from_a_c_program():
    exe = os.path.join(os.path.dirname(BIN), "prefill_from_c")
    assert os.path.exists(exe), "run `python -m loongserve_amd.build` first"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok" in r.stdout.splitlines()[-1]
