"""CPU restatement of the KV-pool slot allocator.  TEST INFRASTRUCTURE ONLY: imported by tests/ and by the CPU
baseline leg of bench.py, never by the product package.

Follows loongserve/common/longserve_mem_manager.py of the reference line by line, with numpy in place of torch:
  alloc             :32-40   nonzero(mem_state == 0)[0:need] then add_refs
  alloc_contiguous  :42-59   nonzero, shifted difference == need - 1, first hit, indexes[start:end], add_refs
  add_refs          :73-79   gather, count_nonzero, `mem_state[index] += 1` (a slot listed twice still gains 1)
  decrease_refs     :82-88   `mem_state[index] -= 1`, gather, count_nonzero
  free              :61-70   decrease_refs on index.long()
  free_all          :92-94

Pins (tests/test_oracle_pins.py): a slot-by-slot Python scan for the first-N-free and first-fit searches on random
and adversarial states (runs that straddle every boundary, no run, run at the very end), the conservation law
can_use_mem_size == count(mem_state == 0) after every operation of a random trace, and the duplicate-index
behaviour against numpy fancy-index assignment, which has torch's gather-then-write semantics.
"""
import numpy as np


class MemoryManagerOracle:
    def __init__(self, size, always_copy=False):
        self.mem_state = np.zeros((size,), dtype=np.int32)
        self.indexes = np.arange(0, size, dtype=np.int64)
        self.can_use_mem_size = size
        self.always_copy = always_copy

    def alloc(self, need_size):
        if need_size > self.can_use_mem_size:
            raise AssertionError("not enough free slots")  # :33-35
        can_use_index = np.nonzero(self.mem_state == 0)[0]  # :37
        select_index = can_use_index[0:need_size]  # :38
        self.add_refs(select_index)  # :39
        return select_index

    def alloc_contiguous(self, need_size):
        if self.always_copy:  # :44-45
            return None
        if need_size > self.can_use_mem_size:  # :46-48
            return None
        can_use_index = np.nonzero(self.mem_state == 0)[0]  # :50
        n = len(can_use_index)
        head = can_use_index[0:n - need_size + 1]
        hit = head[(can_use_index[need_size - 1:] - head) == need_size - 1]  # :52
        if hit.shape[0] == 0:  # :53-54
            return None
        start = int(hit[0])  # :55
        end = start + need_size
        select_index = self.indexes[start:end]  # :57
        self.add_refs(select_index)  # :58
        return select_index, start, end

    def free(self, free_index):
        self.decrease_refs(np.asarray(free_index).astype(np.int64))  # :68-69

    def add_refs(self, token_index):
        token_index = np.asarray(token_index)
        state = self.mem_state[token_index]  # :74
        has_used_tokens = int(np.count_nonzero(state))  # :75
        self.can_use_mem_size -= len(state) - has_used_tokens  # :77
        self.mem_state[token_index] = state + 1  # :78, `x[i] += 1` is gather, add, write back

    def decrease_refs(self, token_index):
        token_index = np.asarray(token_index)
        self.mem_state[token_index] = self.mem_state[token_index] - 1  # :83
        state = self.mem_state[token_index]  # :84
        used_tokens = int(np.count_nonzero(state))  # :85
        self.can_use_mem_size += len(state) - used_tokens  # :87

    def free_all(self):
        self.can_use_mem_size = len(self.mem_state)  # :93
        self.mem_state[:] = 0  # :94
