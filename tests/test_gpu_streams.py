"""The library keeps no state: calls on different streams, from different host threads, do not disturb each other.
Prefill steps and decode steps are issued concurrently on two streams (default priority) from two threads and compared
with the same calls made one after the other."""
import threading

import pytest
import torch

from tests.helpers import decode_case, meta, rand_t

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_two_threads_two_streams(lsa):
    Hq, Hkv, D, BS = 8, 2, 128, 64
    lens = [900, 300]
    T = sum(lens)
    q, k, v = [rand_t(s, i).to(DEV) for i, s in enumerate(((T, Hq, D), (T, Hkv, D), (T, Hkv, D)))]
    m = [t.to(DEV) for t in meta(lens)]
    dl = [700, 33, 1025]
    dq, dkv, table, b_req, b_len = [t.to(DEV) for t in decode_case(77, 3, Hq, Hkv, D, dl, 3000)]
    nblk = (max(dl) + BS - 1) // BS

    def prefill(out, lse):
        lsa.prefill_attention_step(q, k, v, *m, *m, 1, max(lens), out, lse)

    def decode(mo, ml, o, l):
        lsa.longserve_token_decode_attention_flash_decoding(dq, table, b_req, b_len, mo, ml, 3, max(dl), Hq, D, dkv[:, :Hkv],
                                                            dkv[:, Hkv:], BS, o, l)

    def bufs():
        return (torch.empty(T, Hq, D, device=DEV), torch.empty(T, Hq, device=DEV), torch.empty(nblk, 3, Hq, D, device=DEV),
                torch.empty(nblk, 3, Hq, device=DEV), torch.empty(3, Hq, D, device=DEV), torch.empty(3, Hq, device=DEV))

    ref = bufs()
    prefill(ref[0], ref[1]); decode(*ref[2:])
    torch.cuda.synchronize()

    got = [bufs() for _ in range(8)]
    errors = []

    def worker(kind):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                for b in got:
                    if kind == 0:
                        prefill(b[0], b[1])
                    else:
                        decode(*b[2:])
            s.synchronize()
        except Exception as e:  # surfaced below: an exception in a thread would otherwise be lost
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(kind,)) for kind in (0, 1)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for b in got:
        assert torch.equal(b[0], ref[0]) and torch.equal(b[1], ref[1])
        assert torch.equal(b[4], ref[4]) and torch.equal(b[5], ref[5])


def test_an_error_left_behind_by_the_host_program_is_not_reported_as_a_launch_failure(lsa):
    """The runtime keeps the last error of a host thread until somebody asks for it, harmless ones included (a framework's
    copy engine polls events and gets "not ready"; here: a device number that does not exist).  The library's launches
    report their own outcome, not what was there before them."""
    import ctypes
    # (the runtime this process already runs on, by the path it was loaded from: a bare library name could bring in a second one)
    loaded = sorted({ln.split()[-1] for ln in open("/proc/self/maps") if "libamdhip64" in ln})
    assert len(loaded) == 1, loaded
    hip = ctypes.CDLL(loaded[0])
    hip.hipSetDevice.argtypes = [ctypes.c_int]
    hip.hipPeekAtLastError.restype = ctypes.c_int
    Hq, Hkv, D, BS = 8, 2, 128, 64
    lens = [300]
    q, k, v = [rand_t(s, 40 + i).to(DEV) for i, s in enumerate(((300, Hq, D), (300, Hkv, D), (300, Hkv, D)))]
    m = [t.to(DEV) for t in meta(lens)]
    o_ok, lse_ok = lsa.prefill_attention_step(q, k, v, *m, *m, 1, 300)
    dq, dkv, table, b_req, b_len = [t.to(DEV) for t in decode_case(78, 2, Hq, Hkv, D, [500, 70], 2000)]
    mo = torch.empty(8, 2, Hq, D, device=DEV)
    ml = torch.empty(8, 2, Hq, device=DEV)
    d_ok = lsa.longserve_token_decode_attention_flash_decoding(dq, table, b_req, b_len, mo, ml, 2, 500, Hq, D, dkv[:, :Hkv], dkv[:, Hkv:], BS)
    torch.cuda.synchronize()
    for call in ("prefill", "decode"):
        assert hip.hipSetDevice(12345) != 0      # fails, changes nothing, and stays behind as the thread's last error
        assert hip.hipPeekAtLastError() != 0
        if call == "prefill":
            o, lse = lsa.prefill_attention_step(q, k, v, *m, *m, 1, 300)
            torch.cuda.synchronize()
            assert torch.equal(o, o_ok) and torch.equal(lse, lse_ok)
        else:
            d = lsa.longserve_token_decode_attention_flash_decoding(dq, table, b_req, b_len, mo, ml, 2, 500, Hq, D, dkv[:, :Hkv], dkv[:, Hkv:], BS)
            torch.cuda.synchronize()
            assert torch.equal(d[0], d_ok[0]) and torch.equal(d[1], d_ok[1])
