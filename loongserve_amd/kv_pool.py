"""Slot allocator of the token-indexed KV pool and the request table, with the reference's classes and methods.

LongServeMemoryManager mirrors loongserve/common/longserve_mem_manager.py:7-113 and LongServeReqManager mirrors
loongserve/common/longserve_req_manager.py:7-48: same constructor arguments, attributes (`mem_state`, `indexes`,
`can_use_mem_size`, `kv_buffer`; `req_state`, `req_to_token_indexs`, `can_use_req_size`), return values and
failure behaviour.  Where the reference searches the pool with torch.nonzero and slices on every call, these
classes call the slot-search and reference-count kernels of liblsattn.so; there is no other implementation
behind them.
"""
from __future__ import annotations

import logging

import torch

from . import _lib

logger = logging.getLogger(__name__)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


class _SlotStates:
    """An int32 state vector on the device (0 = free) plus the workspace the searches need."""

    def __init__(self, size: int):
        self.size = int(size)
        self.state = torch.zeros((self.size,), dtype=torch.int32, device="cuda")
        lib = _lib.load()
        self._search_bytes = int(lib.lsattn_pool_search_workspace_bytes(self.size))
        self._search_ws = torch.empty((max(self._search_bytes, 16),), dtype=torch.uint8, device="cuda")
        self._refs_ws = torch.empty((4096,), dtype=torch.uint8, device="cuda")
        self._cells = torch.empty((4,), dtype=torch.int64, device="cuda")

    def take_first_free(self, need: int) -> torch.Tensor:
        out = torch.empty((need,), dtype=torch.int64, device="cuda")
        rc = _lib.load().lsattn_pool_alloc(self.state.data_ptr(), self.size, need, out.data_ptr(), self._search_ws.data_ptr(),
                                           self._search_bytes, _stream())
        _lib.check(rc, "lsattn_pool_alloc")
        return out

    def first_fit(self, need: int) -> int:
        rc = _lib.load().lsattn_pool_find_contiguous(self.state.data_ptr(), self.size, need, self._cells.data_ptr(),
                                                     self._search_ws.data_ptr(), self._search_bytes, _stream())
        _lib.check(rc, "lsattn_pool_find_contiguous")
        return int(self._cells[0].item())  # the reference reads the start back as well (longserve_mem_manager.py:55)

    def update_refs(self, index: torch.Tensor, delta: int) -> int:
        """state[index] += delta with torch's gather-then-write semantics; returns the count of listed slots that
        are non-zero before (+1) or after (-1) the update."""
        index = index.reshape(-1)
        if index.dtype != torch.int64 or not index.is_contiguous():
            index = index.long().contiguous()
        n = index.numel()
        lib = _lib.load()
        need_bytes = int(lib.lsattn_pool_refs_workspace_bytes(n))
        if need_bytes > self._refs_ws.numel():
            self._refs_ws = torch.empty((need_bytes,), dtype=torch.uint8, device="cuda")
        rc = lib.lsattn_pool_update_refs(self.state.data_ptr(), self.size, index.data_ptr() if n else None, n, delta,
                                         self._cells.data_ptr() + 16, self._refs_ws.data_ptr(), self._refs_ws.numel(), _stream())
        _lib.check(rc, "lsattn_pool_update_refs")
        counted, outside = self._cells[2:4].tolist()
        if outside:
            raise IndexError("%d slot indices are outside the pool of %d slots" % (outside, self.size))
        return int(counted)


class LongServeMemoryManager:
    """Free-slot bookkeeping of the K/V pool: one int32 reference count per slot on the device."""

    def __init__(self, size, dtype, head_num, head_dim, layer_num, num_idle_slots=0, always_copy=False):
        self.size = size
        self.dtype = dtype
        self.head_num = head_num
        self.head_dim = head_dim
        self.layer_num = layer_num
        self.num_idle_slots = num_idle_slots
        self.always_copy = always_copy
        self._reset_states(size)
        self._init_buffers(size, dtype, head_num, head_dim, layer_num, num_idle_slots)

    def _reset_states(self, size):
        self._slots = _SlotStates(size)
        self.mem_state = self._slots.state
        self.indexes = torch.arange(0, size, dtype=torch.long, device="cuda")
        self.can_use_mem_size = size

    def _init_buffers(self, size, dtype, head_num, head_dim, layer_num, num_idle_slots=0):
        # K heads then V heads per slot (longserve_mem_manager.py:26)
        self.kv_buffer = torch.empty((layer_num, size + num_idle_slots, 2 * head_num, head_dim), dtype=dtype, device="cuda")

    def _free_buffers(self):
        self.kv_buffer = None

    @torch.inference_mode()
    def alloc(self, need_size):
        """The first need_size free slots, ascending, as an int64 vector; they are marked in use
        (longserve_mem_manager.py:32-40)."""
        if need_size > self.can_use_mem_size:
            msg = "KV pool exhausted: %d slots asked for, %d free" % (need_size, self.can_use_mem_size)
            logger.warning(msg)
            raise AssertionError(msg)  # the reference asserts here (longserve_mem_manager.py:35)
        select_index = self._slots.take_first_free(int(need_size))
        self.can_use_mem_size -= int(need_size)  # every slot taken was free: add_refs would count none as used
        return select_index

    @torch.inference_mode()
    def alloc_contiguous(self, need_size):
        """(indexes[start:end], start, end) for the first run of need_size consecutive free slots, marked in use;
        None if there is none (longserve_mem_manager.py:42-59)."""
        if self.always_copy:
            return None
        if need_size > self.can_use_mem_size:
            logger.warning("KV pool: no room for a run of %d slots, %d free", need_size, self.can_use_mem_size)
            return None
        if need_size < 1:
            raise ValueError("alloc_contiguous needs a positive size")
        start = self._slots.first_fit(int(need_size))
        if start < 0:
            return None
        end = start + need_size
        select_index = self.indexes[start:end]
        self.add_refs(select_index)
        return select_index, start, end

    @torch.inference_mode()
    def free(self, free_index):
        """Drop one reference on every listed slot (longserve_mem_manager.py:61-70)."""
        free_index = free_index.long()
        self.decrease_refs(free_index)
        return

    @torch.inference_mode()
    def add_refs(self, token_index: torch.Tensor):
        all_tokens = token_index.numel()
        has_used_tokens = self._slots.update_refs(token_index, +1)
        self.can_use_mem_size -= all_tokens - has_used_tokens
        return

    @torch.inference_mode()
    def decrease_refs(self, token_index: torch.Tensor):
        all_tokens = token_index.numel()
        used_tokens = self._slots.update_refs(token_index, -1)
        self.can_use_mem_size += all_tokens - used_tokens
        return

    @torch.inference_mode()
    def free_all(self):
        self.can_use_mem_size = len(self.mem_state)
        self.mem_state[:] = 0

    @torch.inference_mode()
    def resize_mem(self, new_size):
        """Start over with an empty pool of new_size slots (the reference keeps this for its tests, :97-113)."""
        self.size = new_size
        self._reset_states(new_size)
        self._free_buffers()
        self._init_buffers(new_size, self.dtype, self.head_num, self.head_dim, self.layer_num)
        return


class LongServeReqManager:
    """
    ReqManager - the mapping between request index and token slot index: req_to_token_indexs[req, pos] is the pool
    slot of that request's token, 2147483647 where unused (longserve_req_manager.py:17-21).
    """

    def __init__(self, max_request_num, max_sequence_length, mem_manager):
        self._reqs = _SlotStates(max_request_num)
        # the reference keeps a bool vector; int32 0/1 here, which is what the slot-search kernels read
        self.req_state = self._reqs.state
        self.req_to_token_indexs = torch.full((max_request_num, max_sequence_length), fill_value=2147483647,
                                              dtype=torch.int32, device="cuda")
        self.can_use_req_size = max_request_num
        self.mem_manager: LongServeMemoryManager = mem_manager

    def alloc(self, need_size):
        if need_size > self.can_use_req_size:
            logger.error("request table full: %d asked for, %d free", need_size, self.can_use_req_size)
            return None
        select_index = self._reqs.take_first_free(int(need_size))
        self.can_use_req_size -= int(need_size)
        return select_index

    def free(self, free_req_index, free_token_index):
        self.can_use_req_size += len(free_req_index)
        self.req_state[free_req_index] = 0
        if free_token_index is not None:
            self.mem_manager.free(free_token_index)

    def free_req(self, free_req_index):
        self.can_use_req_size += 1
        self.req_state[free_req_index] = 0
        return

    def free_token(self, free_token_index):
        self.mem_manager.free(free_token_index)

    def free_all(self):
        self.can_use_req_size = len(self.req_state)
        self.req_state[:] = 0
