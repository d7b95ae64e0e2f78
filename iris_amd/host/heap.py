"""Single-GPU symmetric heap.

The reference gives every rank one heap and maps the peers' heaps into each process
(iris/host/memory/symmetric_heap.py:34-172, allocators/torch_allocator.py:33-132).  Here one GPU
plays all W ranks: a single hipMalloc'd pool is cut into W equal slots, slot r standing for rank
r's heap, and heap_bases[r] is the device address of slot r.  Allocation is the reference's bump
allocator (sizes rounded up to `alignment` bytes, default 1024); because one bump pointer serves all
slots, an allocation has the same offset in every slot, which is what "symmetric" means.
"""

import logging
import math

import numpy as np
import torch

from . import hip
from .logging import log_rank


class _DeviceSpan:
    """Expose raw device memory to torch through the CUDA array interface
    (the reference's CUDAArrayInterface / tensor_from_ptr, iris/host/memory/tensor_utils.py:60-135).

    The span owns the allocation: torch keeps a reference to this object for as long as any tensor
    made from it (or any view of one) is alive, so the memory is released when the last such tensor
    goes away and never earlier - a tensor from ctx.zeros() may outlive its context, as it may in the
    reference, whose torch allocator keeps the heap alive through the tensors' storage.
    """

    def __init__(self, ptr, nbytes, release=None):
        self._ptr, self._release = ptr, release
        self.__cuda_array_interface__ = {
            "shape": (nbytes,),
            "typestr": "|u1",
            "data": (ptr, False),
            "version": 3,
        }

    def __del__(self):
        release, self._release = self._release, None
        if release is not None and self._ptr:
            try:
                release(self._ptr)
            except Exception:  # interpreter shutdown: the runtime may be gone already
                pass


class SymmetricHeap:
    """W slots of `heap_size` bytes in one allocation.

    Args:
        heap_size: bytes per slot (the reference's per-rank heap size).
        device_id: GPU index; ignored for the host backing.
        cur_rank: the slot tensors are handed out from.
        num_ranks: W.
        backing: "hip" (hipMalloc on the GPU) or "host" (pageable host memory; lets the allocator
            and address arithmetic be exercised without a GPU - kernels never run on it).
    """

    def __init__(self, heap_size, device_id, cur_rank, num_ranks, backing="hip"):
        if heap_size <= 0:
            raise ValueError(f"heap_size must be positive, got {heap_size}")
        if not (0 <= cur_rank < num_ranks):
            raise ValueError(f"cur_rank {cur_rank} outside [0, {num_ranks})")
        self.heap_size = int(heap_size)
        self.device_id = device_id
        self.cur_rank = cur_rank
        self.num_ranks = num_ranks
        self.backing = backing
        # Slots start on 4 KiB boundaries whatever heap_size is.
        self.slot_stride = (self.heap_size + 4095) // 4096 * 4096
        total = self.slot_stride * num_ranks
        self.heap_offset = 0
        self._raw_ptr = 0
        log_rank(logging.DEBUG, "SymmetricHeap: %d slots x %.2f GiB, backing=%s", num_ranks,
                 self.heap_size / (1 << 30), backing, rank=cur_rank, num_ranks=num_ranks)
        if backing == "hip":
            hip.set_device(device_id)
            self._raw_ptr = hip.hip_malloc(total)
            self.device = torch.device(f"cuda:{device_id}")
            self._pool = torch.as_tensor(_DeviceSpan(self._raw_ptr, total, hip.hip_free), device=self.device)
            base = self._raw_ptr
        elif backing == "host":
            self.device = torch.device("cpu")
            self._pool = torch.empty(total + 4096, dtype=torch.uint8)
            base = (self._pool.data_ptr() + 4095) // 4096 * 4096
            self._pool = self._pool[base - self._pool.data_ptr():][:total]
        else:
            raise ValueError(f"unknown backing {backing!r}")
        assert self._pool.data_ptr() == base
        self.base_address = base
        bases = np.array([base + r * self.slot_stride for r in range(num_ranks)], dtype=np.int64)
        # int64 like the reference (symmetric_heap.py:83-91)
        self.heap_bases = torch.tensor(bases, dtype=torch.int64).to(self.device)
        self._bases_host = [int(b) for b in bases]

    # -- allocation ---------------------------------------------------------------------------
    def allocate(self, num_elements, dtype, alignment=1024):
        """Bump-allocate `num_elements` of `dtype` in slot cur_rank (and, implicitly, at the same
        offset in every other slot).  Raises MemoryError("Heap out of memory") like the reference."""
        element_size = torch.empty((), dtype=dtype).element_size()
        size_in_bytes = num_elements * element_size
        aligned_size = math.ceil(size_in_bytes / alignment) * alignment
        if self.heap_offset + aligned_size > self.heap_size:
            log_rank(logging.ERROR, "SymmetricHeap: OOM requested=%d available=%d", aligned_size,
                     self.heap_size - self.heap_offset, rank=self.cur_rank, num_ranks=self.num_ranks)
            raise MemoryError("Heap out of memory")
        start = self.heap_offset
        self.heap_offset += aligned_size
        return self._view(self.cur_rank, start, size_in_bytes, dtype).reshape((num_elements,))

    def _view(self, slot, offset, nbytes, dtype):
        begin = slot * self.slot_stride + offset
        return self._pool[begin:begin + nbytes].view(dtype)

    # -- queries ------------------------------------------------------------------------------
    def get_heap_bases(self):
        return self.heap_bases

    def slot_base(self, rank):
        return self._bases_host[rank]

    def offset_of(self, tensor):
        """Byte offset of `tensor` inside the slot that holds it."""
        ptr = int(tensor.data_ptr())
        if not self._in_pool(ptr):
            raise RuntimeError("The tensor is not on the symmetric heap")
        return (ptr - self.base_address) % self.slot_stride

    def slot_of(self, tensor):
        ptr = int(tensor.data_ptr())
        if not self._in_pool(ptr):
            raise RuntimeError("The tensor is not on the symmetric heap")
        return (ptr - self.base_address) // self.slot_stride

    def _in_pool(self, ptr):
        return self.base_address <= ptr < self.base_address + self.slot_stride * self.num_ranks

    def is_symmetric(self, tensor):
        """True for tensors inside slot cur_rank (empty tensors count, as in the reference's
        owns_tensor, torch_allocator.py:230-245)."""
        if tensor.numel() == 0:
            return True
        if tensor.device.type != self.device.type:
            return False
        ptr = int(tensor.data_ptr())
        own = self._bases_host[self.cur_rank]
        return own <= ptr < own + self.heap_size

    def peer_view(self, tensor, rank):
        """The tensor that occupies, in slot `rank`, the bytes `tensor` occupies in its own slot:
        what rank `rank` would see as its copy of this symmetric allocation."""
        if not (0 <= rank < self.num_ranks):
            raise ValueError(f"rank {rank} outside [0, {self.num_ranks})")
        if not tensor.is_contiguous():
            raise ValueError("peer_view needs a contiguous tensor")
        offset = self.offset_of(tensor)
        nbytes = tensor.numel() * tensor.element_size()
        return self._view(rank, offset, nbytes, tensor.dtype).reshape(tensor.shape)

    def close(self):
        """Drop this object's references.  The device memory itself is released by the span object
        that torch holds, once the last tensor on the heap is gone."""
        self._raw_ptr = 0
        self._pool = None

    def __del__(self):
        self.close()
