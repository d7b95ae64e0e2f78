"""The Iris context for one MI355X standing in for W ranks.

Public surface of iris/host/iris.py (reference) that the fused operators and their callers touch:
`iris(heap_size)`, tensor factories, `get_heap_bases`, `get_device_context`, `barrier`, rank getters,
`is_symmetric`, `ops`, rank-tagged logging.  The reference takes rank and world size from
torch.distributed (iris/host/distributed/helpers.py:420-433); here they come from keyword arguments
or the environment (IRIS_NUM_RANKS, IRIS_RANK), falling back to torch.distributed when that is
initialised, else to a world of one.  All W heaps are slots of one GPU allocation.
"""

import ctypes
import logging
import os
import weakref

import torch
import torch.distributed as _dist

from . import tensors as tensor_creation
from .heap import SymmetricHeap
from .logging import logger

# int64 words the reference appends for device-side tracing (iris/host/iris.py:916-958); kept as
# zeros so the context tensor has the reference's length.
_TRACE_WORDS = 17


def _unregister_context(ptr):
    """Drop the kernel library's record of the context tensor that lived at address `ptr`."""
    try:
        from .. import _lib

        _lib.library().iris_hip_unregister_context(ctypes.c_void_p(ptr))
    except Exception:  # interpreter shutdown: the library may be gone already
        pass


def _world_from_environment(num_ranks, rank):
    if num_ranks is None and "IRIS_NUM_RANKS" in os.environ:
        num_ranks = int(os.environ["IRIS_NUM_RANKS"])
    if rank is None and "IRIS_RANK" in os.environ:
        rank = int(os.environ["IRIS_RANK"])
    if num_ranks is None or rank is None:
        import torch.distributed as dist

        if dist.is_available() and dist.is_initialized():
            num_ranks = dist.get_world_size() if num_ranks is None else num_ranks
            rank = dist.get_rank() if rank is None else rank
    num_ranks = 1 if num_ranks is None else int(num_ranks)
    rank = 0 if rank is None else int(rank)
    if num_ranks < 1 or not (0 <= rank < num_ranks):
        raise ValueError(f"invalid rank/world size {rank}/{num_ranks}")
    return num_ranks, rank


class Iris:
    """Context object: symmetric heap + rank identity + operator namespace.

    Args:
        heap_size: bytes per rank slot (default 1 GiB, as in the reference).
        allocator_type: accepted for signature parity; only the bump ("torch") allocator exists.
        num_ranks, rank: world size W and the rank this process plays (keyword-only additions).
        device: "cuda" / "cuda:i" (default: current CUDA device) or "cpu".  A "cpu" context backs
            the heap with host memory so that allocation and addressing can be tested without a
            GPU; the operators refuse to run on it.
    """

    def __init__(self, heap_size=1 << 30, allocator_type="torch", *, num_ranks=None, rank=None, device=None):
        allocator_type = os.environ.get("IRIS_ALLOCATOR", allocator_type)
        if allocator_type != "torch":
            raise ValueError(f"allocator_type {allocator_type!r} is not available: only 'torch' (bump allocator)")
        self.num_ranks, self.cur_rank = _world_from_environment(num_ranks, rank)
        self.heap_size = heap_size
        dev = torch.device(device) if device is not None else torch.device("cuda")
        if dev.type == "cuda":
            if not torch.cuda.is_available():
                raise RuntimeError("Iris needs a GPU: no CUDA/HIP device is available")
            self.gpu_id = dev.index if dev.index is not None else torch.cuda.current_device()
            torch.cuda.set_device(self.gpu_id)
            backing = "hip"
        elif dev.type == "cpu":
            self.gpu_id = -1
            backing = "host"
        else:
            raise ValueError(f"unsupported device {device!r}")
        if logger.isEnabledFor(logging.INFO):
            self._log_with_rank(
                logging.INFO,
                f"init: heap_size={heap_size / (1 << 30):.1f}GB rank={self.cur_rank}/{self.num_ranks} "
                f"allocator={allocator_type}",
            )
        self.heap = SymmetricHeap(heap_size, self.gpu_id, self.cur_rank, self.num_ranks, backing=backing)
        self.device = str(self.heap.device) if backing == "host" else f"cuda:{self.gpu_id}"
        self.heap_bases = self.heap.get_heap_bases()
        self._ops = None
        self._ccl = None
        self._cu_count = None
        # Flag-wait bound handed to the kernels (polls per flag; <= 0 waits forever as the reference).
        self.spin_limit = int(os.environ.get("IRIS_SPIN_LIMIT", str(1 << 22)))
        # Status word the kernels write on a flag-wait timeout.  With a GPU it lives in pinned host
        # memory (device-visible at the same address), so that every barrier can read it without a
        # device-to-host copy.
        if self.heap.device.type == "cuda":
            self._status = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        else:
            self._status = torch.zeros(1, dtype=torch.int32, device=self.heap.device)
        # The same word as a numpy view: reading one element of a tensor costs microseconds, and every
        # synchronous operator call ends with such a read.
        self._status_view = self._status.numpy() if self._status.device.type == "cpu" else None
        # One GPU standing in for all ranks: when set, the fused operators' preambles mark the other
        # ranks as finished (flags raised, aux zeroed) so that a launch does not wait for them.
        self.stand_in_peers = os.environ.get("IRIS_STAND_IN_PEERS", "0") not in ("", "0")
        self._build_device_context()

    def __del__(self):
        try:
            self._forget_device_context()
            if hasattr(self, "heap"):
                self.heap.close()
        except Exception:
            pass

    # -- logging ---------------------------------------------------------------------------------
    def _log_with_rank(self, level, message):
        if logger.isEnabledFor(level):
            logger.log(level, message, extra={"iris_rank": self.cur_rank, "iris_num_ranks": self.num_ranks})

    def debug(self, message):
        self._log_with_rank(logging.DEBUG, message)

    def info(self, message):
        self._log_with_rank(logging.INFO, message)

    def warning(self, message):
        self._log_with_rank(logging.WARNING, message)

    def error(self, message):
        self._log_with_rank(logging.ERROR, message)

    # -- operators ---------------------------------------------------------------------------------
    @property
    def ops(self):
        """Fused GEMM+collective operators bound to this context (`ctx.ops.matmul_all_reduce(...)`)."""
        if self._ops is None:
            from ..ops import OpsNamespace

            self._ops = OpsNamespace(self)
        return self._ops

    @property
    def ccl(self):
        """Stand-alone collectives bound to this context (`ctx.ccl.all_reduce(output, input)`)."""
        if self._ccl is None:
            self._ccl = Iris.CCL(self)
        return self._ccl

    class CCL:
        """The `ctx.ccl` namespace of the reference (iris/host/iris.py:1104-1311), for the collectives
        that have HIP kernels here: all_reduce (+ preamble) and reduce_scatter."""

        def __init__(self, iris_instance):
            # (imported here: the collectives import this module's package)
            from ..ccl.all_reduce import all_reduce, all_reduce_preamble
            from ..ccl.reduce_scatter import reduce_scatter

            self._iris = iris_instance
            self._all_reduce, self._all_reduce_preamble, self._reduce_scatter = all_reduce, all_reduce_preamble, reduce_scatter

        def all_reduce_preamble(self, output_tensor, input_tensor, config=None, workspace=None):
            return self._all_reduce_preamble(output_tensor, input_tensor, self._iris, config=config, workspace=workspace)

        def all_reduce(self, output_tensor, input_tensor, op=None, group=None, async_op=False, config=None,
                       workspace=None):
            return self._all_reduce(output_tensor, input_tensor, self._iris, op=op, group=group, async_op=async_op,
                                    config=config, workspace=workspace)

        def reduce_scatter(self, output_tensor, input_tensor, op=None, group=None, async_op=False, config=None):
            self._reduce_scatter(output_tensor, input_tensor, self._iris, op=op, group=group, async_op=async_op,
                                 config=config)

        def __getattr__(self, name):
            if name in ("all_to_all", "all_gather"):
                raise NotImplementedError(f"ccl.{name} has no HIP kernel in this package")
            raise AttributeError(name)

    # -- tensor factories --------------------------------------------------------------------------
    def _dev(self):
        return self.heap.device

    def zeros(self, *size, out=None, dtype=None, layout=torch.strided, device=None, requires_grad=False):
        return tensor_creation.zeros(self.heap, self._dev(), size, out=out, dtype=dtype, layout=layout,
                                     device=device, requires_grad=requires_grad)

    def ones(self, *size, out=None, dtype=None, layout=torch.strided, device=None, requires_grad=False):
        return tensor_creation.ones(self.heap, self._dev(), size, out=out, dtype=dtype, layout=layout,
                                    device=device, requires_grad=requires_grad)

    def full(self, size, fill_value, *, out=None, dtype=None, layout=torch.strided, device=None,
             requires_grad=False):
        return tensor_creation.full(self.heap, self._dev(), (size,), fill_value, out=out, dtype=dtype,
                                    layout=layout, device=device, requires_grad=requires_grad)

    def empty(self, *size, out=None, dtype=None, layout=torch.strided, device=None, requires_grad=False):
        return tensor_creation.empty(self.heap, self._dev(), size, out=out, dtype=dtype, layout=layout,
                                     device=device, requires_grad=requires_grad)

    def zeros_like(self, input, *, dtype=None, layout=None, device=None, requires_grad=False):
        return tensor_creation.zeros_like(self.heap, self._dev(), input, dtype=dtype, layout=layout,
                                          device=device, requires_grad=requires_grad)

    def randn(self, *size, generator=None, out=None, dtype=None, layout=torch.strided, device=None,
              requires_grad=False):
        return tensor_creation.randn(self.heap, self._dev(), size, generator=generator, out=out, dtype=dtype,
                                     layout=layout, device=device, requires_grad=requires_grad)

    def rand(self, *size, generator=None, out=None, dtype=None, layout=torch.strided, device=None,
             requires_grad=False):
        return tensor_creation.rand(self.heap, self._dev(), size, generator=generator, out=out, dtype=dtype,
                                    layout=layout, device=device, requires_grad=requires_grad)

    def uniform(self, size, low=0.0, high=1.0, dtype=torch.float):
        return tensor_creation.uniform(self.heap, self._dev(), (size,), low, high, dtype)

    def randint(self, *args, generator=None, out=None, dtype=None, layout=torch.strided, device=None,
                requires_grad=False):
        if len(args) == 2:
            low, (high, size) = 0, args
        elif len(args) == 3:
            low, high, size = args
        else:
            raise ValueError(f"randint expects (high, size) or (low, high, size), got {len(args)} arguments")
        return tensor_creation.randint(self.heap, self._dev(), low, high, size, generator=generator, out=out,
                                       dtype=dtype, layout=layout, device=device, requires_grad=requires_grad)

    def arange(self, start=0, end=None, step=1, *, out=None, dtype=None, layout=torch.strided, device=None,
               requires_grad=False):
        if end is None:
            start, end = 0, start
        return tensor_creation.arange(self.heap, self._dev(), start, end, step, out=out, dtype=dtype,
                                      layout=layout, device=device, requires_grad=requires_grad)

    def linspace(self, start, end, steps, *, out=None, dtype=None, layout=torch.strided, device=None,
                 requires_grad=False):
        return tensor_creation.linspace(self.heap, self._dev(), start, end, steps, out=out, dtype=dtype,
                                        layout=layout, device=device, requires_grad=requires_grad)

    # -- heap ------------------------------------------------------------------------------------
    def get_heap_bases(self):
        """int64 tensor [W] on the Iris device: base address of every rank's heap slot."""
        return self.heap_bases

    def _build_device_context(self):
        self._forget_device_context()  # a context rebuilt in place drops its old entry first
        data = [self.cur_rank, self.num_ranks] + self.heap_bases.tolist() + [0] * _TRACE_WORDS
        host = torch.tensor(data, dtype=torch.int64)
        self._device_context = host.to(self.heap.device)
        self._context_registered = False
        if self.heap.device.type == "cuda" and os.environ.get("IRIS_REGISTER_CONTEXT", "1") != "0":
            # The kernel library takes the heap bases as kernel arguments when it knows what the
            # context tensor holds (one dependent load less on the way to the peers' flags).
            from .. import _lib

            ptr = self._device_context.data_ptr()
            err = _lib.library().iris_hip_register_context(ctypes.c_void_p(ptr), ctypes.c_void_p(host.data_ptr()),
                                                           host.numel())
            if err == 0:
                # The registry is keyed by the tensor's address, and torch hands freed addresses out
                # again: the entry goes away with the tensor (also at interpreter exit, also when
                # __del__ never runs), so that no later tensor at this address inherits these bases.
                self._context_finalizer = weakref.finalize(self._device_context, _unregister_context, ptr)
                self._context_registered = True

    def _forget_device_context(self):
        finalizer = getattr(self, "_context_finalizer", None)
        if finalizer is not None:
            finalizer()  # idempotent: unregisters once
        self._context_registered = False

    def get_device_context(self):
        """int64 tensor [cur_rank, W, heap_base_0..heap_base_{W-1}, 0 x 17] on the Iris device."""
        return self._device_context

    def is_symmetric(self, tensor):
        return self.heap.is_symmetric(tensor)

    def peer_view(self, tensor, rank):
        """The copy of symmetric tensor `tensor` that lives in rank `rank`'s slot.  The reference has
        no such accessor (peers are other processes); a single GPU needs one to stage peer data."""
        return self.heap.peer_view(tensor, rank)

    # -- synchronisation ---------------------------------------------------------------------------
    def barrier(self, stream=None, group=None):
        """Wait for the GPU (or `stream`), then for the other ranks when torch.distributed is
        initialised; raise if a kernel reported a flag-wait timeout."""
        self._log_with_rank(logging.DEBUG, "barrier: start")
        if self.heap.device.type == "cuda":
            if stream is None:
                torch.cuda.synchronize()
            else:
                stream.synchronize()
        if _dist.is_available() and _dist.is_initialized():
            _dist.barrier(group=group)
        self.check_status()

    def check_status(self):
        """Raise RuntimeError if a kernel set a status bit since the last check (needs a sync first)."""
        status = int(self._status_view[0]) if self._status_view is not None else int(self._status[0])
        if status:
            self._status.zero_()
            raise RuntimeError(
                f"a fused kernel gave up waiting for a peer flag (status {status:#x}): "
                f"the peer's locks were not staged/written within {self.spin_limit} polls"
            )

    # -- getters -----------------------------------------------------------------------------------
    def get_device(self):
        return self.heap.device

    def get_device_id(self):
        return self.gpu_id

    def get_rank(self):
        return self.cur_rank

    def get_num_ranks(self):
        return self.num_ranks

    def get_cu_count(self):
        if self._cu_count is None:
            self._cu_count = torch.cuda.get_device_properties(self.gpu_id).multi_processor_count
        return self._cu_count


def iris(heap_size=1 << 30, allocator_type="torch", **kwargs):
    """Create an Iris context with `heap_size` bytes of symmetric heap per rank."""
    return Iris(heap_size, allocator_type, **kwargs)
