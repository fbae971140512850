"""GPU parity of the KV-pool slot allocator against the numpy oracle (integer work: bit-exact), through the C ABI
and through the reference-named manager classes."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle.pool_oracle import MemoryManagerOracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _manager(lsa, size, **kw):
    return lsa.LongServeMemoryManager(size, torch.float16, 1, 16, 1, **kw)


def _pair(lsa, state):
    """A device manager and an oracle, both holding `state` (reference counts per slot)."""
    state = np.asarray(state, dtype=np.int32)
    m = _manager(lsa, len(state))
    m.mem_state.copy_(torch.from_numpy(state))
    m.can_use_mem_size = int((state == 0).sum())
    o = MemoryManagerOracle(len(state))
    o.mem_state[:] = state
    o.can_use_mem_size = m.can_use_mem_size
    return m, o


def _same(m, o):
    assert torch.equal(m.mem_state.cpu(), torch.from_numpy(o.mem_state))
    assert m.can_use_mem_size == o.can_use_mem_size


@pytest.mark.parametrize("size", [1, 5, 255, 1024, 4095, 4096, 4097, 10000, 70001])
def test_alloc_takes_the_first_free_slots(lsa, size):
    rng = np.random.default_rng(size)
    for frac in (0.0, 0.2, 0.9):
        state = (rng.random(size) < frac).astype(np.int32) * rng.integers(1, 4, size).astype(np.int32)
        m, o = _pair(lsa, state)
        for need in sorted({0, 1, min(3, o.can_use_mem_size), o.can_use_mem_size // 2, o.can_use_mem_size}):
            if need > o.can_use_mem_size:
                continue
            got, want = m.alloc(need), o.alloc(need)
            assert got.dtype == torch.int64 and got.device.type == "cuda"
            assert got.cpu().tolist() == want.tolist()
            _same(m, o)
    with pytest.raises(AssertionError):
        m.alloc(m.can_use_mem_size + 1)
    _same(m, o)


def test_alloc_through_the_c_abi_pads_with_minus_one_when_the_pool_runs_out(lsa):
    from loongserve_amd import _lib
    lib = _lib.load()
    size = 9000
    state = torch.ones(size, dtype=torch.int32)
    free = [0, 4095, 4096, 8999]
    state[free] = 0
    state = state.to(DEV)
    ws_bytes = lib.lsattn_pool_search_workspace_bytes(size)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    out = torch.full((7,), 123, dtype=torch.int64, device=DEV)
    rc = lib.lsattn_pool_alloc(state.data_ptr(), size, 7, out.data_ptr(), ws.data_ptr(), ws_bytes,
                               torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert out.cpu().tolist() == free + [-1, -1, -1]
    assert int(state.sum().item()) == size          # the four free slots were taken
    assert ws[:8].view(torch.int64).item() == 4      # first workspace cell: free slots found by this call


def test_alloc_contiguous_finds_the_first_run(lsa):
    rng = np.random.default_rng(99)
    size = 3 * 4096 + 500
    cases = []
    # runs placed across every kind of boundary the kernel has: lane, wave (256 slots), piece (1024), workgroup (4096)
    for start, length in ((0, 3), (3, 1), (253, 7), (1020, 9), (4090, 12), (4096, 5), (8190, 4), (size - 6, 6), (2000, 5000),
                          (4096, 4096), (1, size - 1)):
        state = np.ones(size, dtype=np.int32)
        state[start:start + length] = 0
        cases.append((state, length))
        cases.append((state, length + 1))      # one slot too long: no run
        noisy = state.copy()                   # shorter decoy runs before the real one
        for p in range(0, start - 1, 7):
            noisy[p:p + min(length - 1, 3)] = 0
            noisy[p + min(length - 1, 3)] = 1
        cases.append((noisy, length))
    for _ in range(20):
        state = (rng.random(size) < rng.choice([0.02, 0.2, 0.6])).astype(np.int32)
        cases.append((state, int(rng.integers(1, 40))))
    cases.append((np.zeros(size, dtype=np.int32), size))
    cases.append((np.zeros(size, dtype=np.int32), 1))
    for state, need in cases:
        m, o = _pair(lsa, state)
        got, want = m.alloc_contiguous(need), o.alloc_contiguous(need)
        if want is None:
            assert got is None
        else:
            assert got is not None, (need, want[1])
            assert (got[1], got[2]) == (want[1], want[2])
            assert got[0].cpu().tolist() == want[0].tolist()
        _same(m, o)
    assert _manager(lsa, 64, always_copy=True).alloc_contiguous(4) is None


def test_reference_counts_follow_torch_indexing(lsa):
    m, o = _pair(lsa, [0, 2, 0, 1, 0, 0, 0, 0, 3, 0])
    idx = [1, 1, 4, 9, 4, 2]                       # duplicates change a slot once and count once per entry
    m.add_refs(torch.tensor(idx, device=DEV)); o.add_refs(np.array(idx)); _same(m, o)
    idx = [-1, 3, 3, 8]                            # a negative entry names a slot from the end
    m.add_refs(torch.tensor(idx, dtype=torch.int32, device=DEV)); o.add_refs(np.array(idx)); _same(m, o)
    idx = [3, 9, 9, 4, 2, 1]
    m.free(torch.tensor(idx, dtype=torch.int32, device=DEV)); o.free(np.array(idx)); _same(m, o)
    m.decrease_refs(torch.tensor([8], device=DEV)); o.decrease_refs(np.array([8])); _same(m, o)
    m.add_refs(torch.empty(0, dtype=torch.int64, device=DEV)); _same(m, o)
    with pytest.raises(IndexError):
        m.add_refs(torch.tensor([10], device=DEV))
    # many entries: more than one workgroup, all slots distinct, then a heavily duplicated list
    size = 50000
    m, o = _pair(lsa, np.zeros(size, dtype=np.int32))
    rng = np.random.default_rng(2)
    idx = rng.permutation(size)[:30000]
    m.add_refs(torch.from_numpy(idx).to(DEV)); o.add_refs(idx); _same(m, o)
    idx = rng.integers(0, size, 20000)
    m.add_refs(torch.from_numpy(idx).to(DEV)); o.add_refs(idx); _same(m, o)
    m.decrease_refs(torch.from_numpy(idx).to(DEV)); o.decrease_refs(idx); _same(m, o)
    m.free_all(); o.free_all(); _same(m, o)


def test_random_trace_of_allocations_and_frees(lsa):
    rng = np.random.default_rng(7)
    size = 20000
    m, o = _pair(lsa, np.zeros(size, dtype=np.int32))
    held = []
    for step in range(120):
        if held and rng.random() < 0.45:
            g_idx, o_idx = held.pop(int(rng.integers(len(held))))
            m.free(g_idx); o.free(o_idx)
        else:
            need = int(rng.integers(1, 1500))
            if need > o.can_use_mem_size:
                continue
            if rng.random() < 0.5:
                got, want = m.alloc_contiguous(need), o.alloc_contiguous(need)
                assert (got is None) == (want is None)
                if got is None:
                    got, want = m.alloc(need), o.alloc(need)
                else:
                    assert got[1:] == want[1:]
                    got, want = got[0], want[0]
            else:
                got, want = m.alloc(need), o.alloc(need)
            assert got.cpu().tolist() == want.tolist()
            held.append((got.clone(), want.copy()))
        _same(m, o)
    assert o.can_use_mem_size == int((o.mem_state == 0).sum())


def test_pool_of_the_decode_benchmark_size(lsa):
    """2.5 M slots: allocate, check sortedness / uniqueness / conservation rather than a slot-by-slot oracle."""
    size = 2_500_000
    m = _manager(lsa, size)
    g = torch.Generator().manual_seed(4)
    busy = torch.randperm(size, generator=g)[:1_200_000].to(DEV)
    m.add_refs(busy)
    assert m.can_use_mem_size == size - 1_200_000
    got = m.alloc(500_000)
    assert bool((got[1:] > got[:-1]).all())                     # ascending, hence unique
    assert int(m.mem_state[got].sum().item()) == 500_000        # each was free and is now held once
    free_mask = torch.ones(size, dtype=torch.bool, device=DEV)
    free_mask[busy] = False
    assert torch.equal(got, torch.nonzero(free_mask).view(-1)[:500_000])
    assert m.can_use_mem_size == int((m.mem_state == 0).sum().item())
    m.free(got[:1000]); m.free(busy[:5])
    assert m.can_use_mem_size == int((m.mem_state == 0).sum().item())
    res = m.alloc_contiguous(64)                                # a decode step's batch of new slots
    state = m.mem_state.cpu().numpy()
    if res is not None:
        assert res[2] - res[1] == 64 and (state[res[1]:res[2]] == 1).all()


def test_request_manager_and_int64_slots_in_the_kv_operators(lsa):
    mm = lsa.LongServeMemoryManager(4096, torch.float16, 2, 128, 1)
    rm = lsa.LongServeReqManager(8, 64, mm)
    assert rm.req_to_token_indexs.shape == (8, 64) and int(rm.req_to_token_indexs[0, 0]) == 2147483647
    reqs = rm.alloc(3)
    assert reqs.cpu().tolist() == [0, 1, 2] and rm.can_use_req_size == 5
    assert rm.alloc(6) is None
    rm.free_req(1)
    assert rm.alloc(2).cpu().tolist() == [1, 3]
    # slots from the allocator are int64, as in the reference; the KV operators take them as they are
    mm.add_refs(torch.tensor([0, 2], device=DEV))
    slots = mm.alloc(5)
    assert slots.cpu().tolist() == [1, 3, 4, 5, 6]
    src = torch.randn(5, 4, 128, dtype=torch.float16, device=DEV)
    lsa.kv_scatter(src, slots, mm.kv_buffer[0])
    assert torch.equal(mm.kv_buffer[0][slots], src)
    b_req = torch.tensor([3], dtype=torch.int32, device=DEV)
    b_len = torch.tensor([5], dtype=torch.int32, device=DEV)
    lsa.init_req_to_token_indexes(rm.req_to_token_indexs, b_req, b_len, slots)
    assert rm.req_to_token_indexs[3, :5].cpu().tolist() == [1, 3, 4, 5, 6]
    rm.free(reqs, slots)
    assert mm.can_use_mem_size == 4096 - 2 and rm.can_use_req_size == 8 - 4 + 3
    rm.free_all(); mm.free_all()
    assert rm.can_use_req_size == 8 and mm.can_use_mem_size == 4096
    mm.resize_mem(100)
    assert mm.mem_state.numel() == 100 and mm.kv_buffer.shape[1] == 100 and mm.alloc(100).cpu().tolist() == list(range(100))
