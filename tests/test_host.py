"""Host-side logic that runs without a GPU: the symmetric heap and tensor factories, the operator
wrappers' argument checking and workspace rules (reference error classes and messages), the C-ABI
library's exported symbols, and the CPU replay of the kernels' index math."""

import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

import iris_amd as iris
from iris_amd import _lib, ops
from helpers import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def cpu_ctx(heap=1 << 22, world=4, rank=1):
    return iris.iris(heap, num_ranks=world, rank=rank, device="cpu")


# -- heap ----------------------------------------------------------------------------------------------
def test_allocation_offsets_follow_the_bump_allocator():
    ctx = cpu_ctx()
    requests = [(10, torch.float32), (300, torch.bfloat16), (1024, torch.int32), (1, torch.int8), (0, torch.float32),
                (1025, torch.uint8), (7, torch.float64)]
    tensors = [ctx.zeros(n, dtype=dt) for n, dt in requests]
    expected, end = oracle.bump_offsets([(n, torch.empty((), dtype=dt).element_size()) for n, dt in requests])
    assert [ctx.heap.offset_of(t) if t.numel() else o for t, o in zip(tensors, expected)] == expected
    assert ctx.heap.heap_offset == end
    for t in tensors:
        assert ctx.is_symmetric(t) and ctx.heap.slot_of(t) == 1 if t.numel() else True


def test_heap_bases_and_device_context_layout():
    ctx = cpu_ctx(world=4, rank=2)
    bases = ctx.get_heap_bases()
    assert bases.dtype == torch.int64 and bases.shape == (4,)
    diffs = (bases[1:] - bases[:-1]).tolist()
    assert len(set(diffs)) == 1 and diffs[0] >= ctx.heap_size and diffs[0] % 4096 == 0
    dc = ctx.get_device_context()
    assert dc.dtype == torch.int64
    assert dc.tolist() == oracle.context_tensor(2, 4, bases.tolist()).tolist()
    assert dc.shape[0] >= 2 + 4 and dc[0].item() == 2 and dc[1].item() == 4  # reference test_device_context.py:478-492


def test_peer_view_is_the_translated_address():
    ctx = cpu_ctx(world=4, rank=1)
    ctx.zeros(5, dtype=torch.float32)
    t = ctx.zeros((6, 10), dtype=torch.bfloat16)
    bases = ctx.get_heap_bases().tolist()
    for r in range(4):
        v = ctx.peer_view(t, r)
        assert v.shape == t.shape and v.dtype == t.dtype
        assert v.data_ptr() == oracle.translate(t.data_ptr(), 1, r, bases)
    assert ctx.peer_view(t, 1).data_ptr() == t.data_ptr()
    ctx.peer_view(t, 3).fill_(7)
    assert torch.all(t == 0) and torch.all(ctx.peer_view(t, 3) == 7)
    with pytest.raises(RuntimeError, match="not on the symmetric heap"):
        ctx.peer_view(torch.zeros(4), 0)


@pytest.mark.parametrize("dtype", [torch.int8, torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("size", [(1,), (5,), (2, 3), (3, 4, 5), (1, 1, 1), (10, 20)])
def test_zeros_like_the_reference(dtype, size):
    """tests/unittests/test_zeros.py:31-46 of the reference: shape, dtype, zeros, on the heap."""
    ctx = cpu_ctx()
    for result in (ctx.zeros(*size, dtype=dtype), ctx.zeros(size, dtype=dtype), ctx.zeros(list(size), dtype=dtype)):
        assert result.shape == size and result.dtype == dtype
        assert torch.all(result == 0) and ctx.is_symmetric(result)
    assert not ctx.is_symmetric(torch.zeros(1000))
    assert ctx.is_symmetric(torch.zeros(0))


def test_factories_and_their_errors():
    ctx = cpu_ctx()
    assert ctx.zeros(3).dtype == torch.get_default_dtype()
    assert torch.all(ctx.ones(2, 2) == 1) and torch.all(ctx.full((2, 3), 7, dtype=torch.int32) == 7)
    assert ctx.empty(4, 4, dtype=torch.float16).shape == (4, 4)
    assert ctx.arange(5).tolist() == [0, 1, 2, 3, 4] and ctx.arange(1, 7, 2).tolist() == [1, 3, 5]
    assert ctx.linspace(0, 1, 5).tolist() == [0.0, 0.25, 0.5, 0.75, 1.0]
    assert ctx.randn(4, 4).shape == (4, 4) and ctx.rand(3).shape == (3,) and ctx.randint(0, 5, (7,)).shape == (7,)
    assert ctx.zeros_like(torch.ones(2, 5, dtype=torch.int16)).dtype == torch.int16
    buf = ctx.zeros(6, dtype=torch.float32)
    out = ctx.ones(2, 3, out=buf, dtype=torch.float32)
    assert out.data_ptr() == buf.data_ptr() and torch.all(buf == 1)
    with pytest.raises(RuntimeError, match="elements"):
        ctx.zeros(5, out=buf, dtype=torch.float32)
    with pytest.raises(RuntimeError, match="dtype"):
        ctx.zeros(6, out=buf, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="not on the symmetric heap"):
        ctx.zeros(6, out=torch.zeros(6), dtype=torch.float32)
    with pytest.raises(RuntimeError, match="Device mismatch"):
        ctx.zeros(4, device="cuda:0")
    with pytest.raises(ValueError, match="Layout"):
        ctx.zeros(4, layout=torch.sparse_coo)


def test_heap_out_of_memory():
    ctx = cpu_ctx(heap=4096)
    ctx.zeros(512, dtype=torch.float32)
    ctx.zeros(512, dtype=torch.float32)
    with pytest.raises(MemoryError, match="Heap out of memory"):
        ctx.zeros(1, dtype=torch.float32)


def test_world_from_environment(monkeypatch):
    monkeypatch.setenv("IRIS_NUM_RANKS", "8")
    monkeypatch.setenv("IRIS_RANK", "5")
    ctx = iris.iris(1 << 16, device="cpu")
    assert (ctx.get_rank(), ctx.get_num_ranks()) == (5, 8)
    monkeypatch.delenv("IRIS_NUM_RANKS")
    monkeypatch.delenv("IRIS_RANK")
    ctx = iris.iris(1 << 16, device="cpu")
    assert (ctx.get_rank(), ctx.get_num_ranks()) == (0, 1)
    with pytest.raises(ValueError):
        iris.iris(1 << 16, num_ranks=2, rank=2, device="cpu")
    with pytest.raises(ValueError, match="allocator_type"):
        iris.iris(1 << 16, "vmem", device="cpu")


# -- FusedConfig / FusedWorkspace ----------------------------------------------------------------------------
def test_fused_config_defaults_and_validation():
    c = iris.FusedConfig()
    assert (c.block_size_m, c.block_size_n, c.block_size_k, c.group_size_m, c.num_sms, c.num_xcds, c.chunk_size) == (
        256, 64, 64, 1, None, 1, 1)
    assert (c.cache_modifier_a, c.cache_modifier_b, c.allow_tf32, c.all_reduce_variant, c.all_reduce_num_rings) == (
        ".ca", ".ca", True, "two_shot", 1)
    c.validate(world_size=8)
    for field, match in [("block_size_m", "block_size_m must be positive"), ("block_size_n", "block_size_n must be positive"),
                         ("block_size_k", "block_size_k must be positive"), ("group_size_m", "group_size_m must be positive"),
                         ("num_sms", "num_sms must be positive"), ("num_xcds", "num_xcds must be positive"),
                         ("chunk_size", "chunk_size must be positive"), ("all_reduce_num_rings", "all_reduce_num_rings must be positive")]:
        with pytest.raises(ValueError, match=match):
            iris.FusedConfig(**{field: 0}).validate()
    with pytest.raises(ValueError, match="all_reduce_variant must be one of"):
        iris.FusedConfig(all_reduce_variant="tree").validate()
    with pytest.raises(ValueError, match="divisible by world_size"):
        iris.FusedConfig(all_reduce_variant="ring", block_size_n=64).validate(world_size=3)


def test_workspace_reuse_rule():
    ws = iris.FusedWorkspace(operation="matmul_all_reduce", shape=(4, 5, 6), dtype=torch.float16, world_size=2,
                             variant="one_shot", prepared=True)
    assert ws.matches("matmul_all_reduce", (4, 5, 6), torch.float16, 2, "one_shot")
    assert not ws.matches("matmul_all_reduce", (4, 5, 7), torch.float16, 2, "one_shot")
    assert not ws.matches("matmul_all_reduce", (4, 5, 6), torch.float16, 2, "two_shot")
    ws.reset()
    assert not ws.matches("matmul_all_reduce", (4, 5, 6), torch.float16, 2, "one_shot")
    ws.aux_buffer = torch.zeros(1)
    ws.clear()
    assert ws.aux_buffer is None and ws.locks is None and not ws.prepared


# -- operator wrappers: everything up to the launch --------------------------------------------------------------
def _abc(ctx, M, N, K, dtype=torch.float16):
    return ctx.zeros((M, K), dtype=dtype), ctx.zeros((K, N), dtype=dtype), ctx.zeros((M, N), dtype=dtype)


def test_matmul_all_reduce_preamble_allocates_flags_and_aux():
    ctx = cpu_ctx(heap=1 << 24)
    A, B, C = _abc(ctx, 512, 512, 64)
    C.fill_(3)
    cfg = iris.FusedConfig(block_size_m=128, block_size_n=128, block_size_k=32, all_reduce_variant="one_shot")
    ws = ops.matmul_all_reduce_preamble(ctx, C, A, B, config=cfg)
    assert ws.locks.dtype == torch.int32 and ws.locks.numel() == 16 and torch.all(ws.locks == 0)
    assert ws.aux_buffer.shape == (512, 512) and ws.aux_buffer.dtype == C.dtype
    assert ctx.is_symmetric(ws.locks) and ctx.is_symmetric(ws.aux_buffer)
    assert torch.all(C == 0) and ws.prepared and ws.variant == "one_shot" and ws.shape == (512, 512, 64)
    locks_ptr = ws.locks.data_ptr()
    ws2 = ops.matmul_all_reduce_preamble(ctx, C, A, B, config=cfg, workspace=ws)
    assert ws2 is ws and ws.locks.data_ptr() == locks_ptr  # buffers reused, not reallocated


def test_matmul_all_reduce_lock_array_too_small():
    """tests/ops/test_matmul_all_reduce.py:153-191 of the reference."""
    ctx = cpu_ctx(heap=1 << 24)
    A, B, C = _abc(ctx, 512, 512, 64)
    large = iris.FusedConfig(block_size_m=128, block_size_n=128, block_size_k=32, all_reduce_variant="one_shot")
    ws = ops.matmul_all_reduce_preamble(ctx, C, A, B, config=large)
    ws.prepared = True
    small = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="one_shot")
    with pytest.raises(ValueError, match="Lock array too small"):
        ops.matmul_all_reduce(ctx, C, A, B, config=small, workspace=ws)


def test_matmul_reduce_scatter_lock_array_too_small():
    """tests/ops/test_matmul_reduce_scatter.py:180-213 of the reference."""
    ctx = cpu_ctx(heap=1 << 24)
    A, B, C = _abc(ctx, 512, 512, 64)
    ws = ops.matmul_reduce_scatter_preamble(ctx, C, A, B, config=iris.FusedConfig(block_size_m=128, block_size_n=128, block_size_k=32))
    assert ws.variant == "two_shot" and ws.locks.numel() == 16
    with pytest.raises(ValueError, match="Lock array too small"):
        ops.matmul_reduce_scatter_preamble(ctx, C, A, B, config=iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32), workspace=ws)


def test_matmul_all_reduce_argument_errors():
    ctx = cpu_ctx(heap=1 << 24)
    A, B, C = _abc(ctx, 256, 128, 64)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="one_shot")
    with pytest.raises(ValueError, match="must be 2D"):
        ops.matmul_all_reduce(ctx, C, A[0], B, config=cfg)
    with pytest.raises(ValueError, match="Inner dimensions must match"):
        ops.matmul_all_reduce(ctx, C, A, ctx.zeros((32, 128), dtype=A.dtype), config=cfg)
    with pytest.raises(ValueError, match="doesn't match expected"):
        ops.matmul_all_reduce(ctx, ctx.zeros((256, 64), dtype=A.dtype), A, B, config=cfg)
    with pytest.raises(ValueError, match="same dtype"):
        ops.matmul_all_reduce(ctx, ctx.zeros((256, 128), dtype=torch.float32), A, B, config=cfg)
    with pytest.raises(AssertionError, match="too small for block_size_m"):
        ops.matmul_all_reduce(ctx, C, A, B, config=iris.FusedConfig(block_size_m=512, block_size_n=64, block_size_k=32))
    with pytest.raises(AssertionError, match="too small for block_size_k"):
        ops.matmul_all_reduce(ctx, C, A, B, config=iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=128))
    with pytest.raises(NotImplementedError, match="ring"):
        ops.matmul_all_reduce(ctx, C, A, B, config=iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="ring"))
    atomic = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32, all_reduce_variant="atomic")
    ws = ops.matmul_all_reduce_preamble(ctx, C, A, B, config=atomic)
    assert ws.locks is None and ws.aux_buffer is None  # reference: no buffers for the atomic variant
    with pytest.raises(ValueError, match="slot_sum"):
        ops.matmul_all_reduce(ctx, C, A, B, config=cfg, slot_sum="fp64")
    # a well-formed call reaches the launch and is refused there: the heap is host memory
    with pytest.raises(RuntimeError, match="need a GPU context"):
        ops.matmul_all_reduce(ctx, C, A, B, config=cfg)
    with pytest.raises(RuntimeError, match="need a GPU context"):
        ctx.ops.matmul_reduce_scatter(C, A, B, config=cfg)


def test_matmul_all_gather_argument_errors():
    ctx = cpu_ctx(heap=1 << 24, world=4)
    A = ctx.zeros((64, 32), dtype=torch.float16)
    B = ctx.zeros((32, 64), dtype=torch.float16)
    out = ctx.zeros((256, 64), dtype=torch.float16)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32)
    ws = ops.matmul_all_gather_preamble(ctx, A, B, cfg)
    assert ws.prepared and ws.shape == (256, 64, 32) and ws.operation == "matmul_all_gather"
    with pytest.raises(AssertionError, match="Inner dimensions must match"):
        ops.matmul_all_gather(ctx, out, A, ctx.zeros((16, 64), dtype=torch.float16), config=cfg)
    with pytest.raises(AssertionError, match="Output must be"):
        ops.matmul_all_gather(ctx, ctx.zeros((64, 64), dtype=torch.float16), A, B, config=cfg)
    with pytest.raises(AssertionError, match="M_local"):
        ops.matmul_all_gather(ctx, out, A, B, config=iris.FusedConfig(block_size_m=128, block_size_n=64, block_size_k=32))
    with pytest.raises(RuntimeError, match="symmetric heap"):
        ops.matmul_all_gather(ctx, torch.zeros((256, 64), dtype=torch.float16), A, B, config=cfg)
    with pytest.raises(RuntimeError, match="need a GPU context"):
        ctx.ops.matmul_all_gather(out, A, B, config=cfg)


def test_all_gather_matmul_argument_errors():
    ctx = cpu_ctx(heap=1 << 24, world=4)
    A = ctx.zeros((128, 32), dtype=torch.float16)
    B = ctx.zeros((128, 64), dtype=torch.float16)
    out = ctx.zeros((128, 64), dtype=torch.float16)
    cfg = iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=32)
    ws = ops.all_gather_matmul_preamble(ctx, A, B, cfg)
    assert ws.prepared and ws.shape == (128, 64, 128) and ws.operation == "all_gather_matmul"
    with pytest.raises(AssertionError, match="must equal world_size"):
        ops.all_gather_matmul(ctx, out, A, ctx.zeros((96, 64), dtype=torch.float16), config=cfg)
    with pytest.raises(AssertionError, match="Output must be"):
        ops.all_gather_matmul(ctx, ctx.zeros((64, 64), dtype=torch.float16), A, B, config=cfg)
    with pytest.raises(AssertionError, match="K_local"):
        ops.all_gather_matmul(ctx, out, A, B, config=iris.FusedConfig(block_size_m=64, block_size_n=64, block_size_k=64))
    with pytest.raises(AssertionError):
        ops.all_gather_matmul(ctx, out, A, B, bias=ctx.zeros(64, dtype=torch.float16), config=cfg)
    with pytest.raises(ValueError, match="gather_dim"):
        ops.all_gather_matmul(ctx, out, A, B, config=cfg, gather_dim=2)
    with pytest.raises(RuntimeError, match="need a GPU context"):
        ops.all_gather_matmul(ctx, out, A, B, config=cfg)


# -- the C-ABI library ------------------------------------------------------------------------------------------
def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "iris_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(iris_hip_[a-z_]+)\s*\(", header)))
    assert declared == sorted(_lib.PROTOTYPES), "ctypes prototypes and header disagree"
    lib = ctypes.CDLL(_lib.LIBRARY_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} is not exported by {_lib.LIBRARY_PATH}"
    assert _lib.library().iris_hip_abi_version() == _lib.ABI_VERSION
    assert _lib.last_error() == ""


def test_null_context_tensor_is_rejected_before_any_launch():
    """Every kernel translates addresses through the heap bases, so a NULL context tensor is an
    argument error for every fused entry point, whatever the world size; the check comes before the
    first HIP call (the pointers below are never dereferenced)."""
    lib = _lib.library()
    null, p = ctypes.c_void_p(0), ctypes.c_void_p(0x10000)
    for W in (1, 4):
        rc = lib.iris_hip_matmul_all_reduce(p, p, p, p, p, 64, 64, 64, 64, 1, 64, 1, 64, 1, null, 0, W, 64, 64, 32,
                                            _lib.VARIANT_ONE_SHOT, _lib.FP32, _lib.FP32, 1.0, 0, 0, null,
                                            _lib.PATH_GENERIC, null)
        assert rc == 1 and "context_tensor" in _lib.last_error()
        rc = lib.iris_hip_matmul_all_reduce(p, p, p, null, null, 64, 64, 64, 64, 1, 64, 1, 64, 1, null, 0, W, 64, 64, 32,
                                            _lib.VARIANT_ATOMIC, _lib.BF16, _lib.BF16, 1.0, 0, 0, null, 0, null)
        assert rc == 1 and "context_tensor" in _lib.last_error()
        rc = lib.iris_hip_matmul_reduce_scatter(p, p, p, p, p, 64, 64, 64, 64, 1, 64, 1, 64, 1, null, 0, W, 64, 64, 32,
                                                0, 1, _lib.BF16, _lib.BF16, 1.0, 0, 0, null, 0, null)
        assert rc == 1 and "context_tensor" in _lib.last_error()
        rc = lib.iris_hip_all_gather_matmul(p, p, p, null, 64, 64, 64 * W, 64, 64, 1, 64, 1, 64, 1, 1, null, 0, W,
                                            64, 64, 32, _lib.GATHER_K, _lib.BF16, _lib.BF16, _lib.BF16, 1.0, 0, null)
        assert rc == 1 and "context_tensor" in _lib.last_error()
        rc = lib.iris_hip_matmul_all_gather(p, p, p, null, 64, 64 * W, 64, 64, 64, 1, 64, 1, 64, 1, 1, null, 0, W,
                                            64, 64, 32, _lib.BF16, _lib.BF16, _lib.BF16, 1.0, 0, null)
        assert rc == 1 and "context_tensor" in _lib.last_error()


def test_context_registration_checks_its_arguments():
    """Registering what a context tensor holds touches no device memory: the host copy is read, the
    device pointer only remembered.  Bad contents are argument errors; unregistering an unknown
    pointer is not."""
    lib = _lib.library()
    words = (ctypes.c_int64 * 27)(3, 8, *[0x7000_0000_0000 + (r << 30) for r in range(8)])
    host, dev, null = ctypes.cast(words, ctypes.c_void_p), ctypes.c_void_p(0x20000), ctypes.c_void_p(0)
    assert lib.iris_hip_register_context(dev, host, 27) == 0 and _lib.last_error() == ""
    assert lib.iris_hip_register_context(dev, host, 27) == 0        # again: replaces the entry
    assert lib.iris_hip_register_context(null, host, 27) == 1 and "must not be NULL" in _lib.last_error()
    assert lib.iris_hip_register_context(dev, null, 27) == 1 and "must not be NULL" in _lib.last_error()
    assert lib.iris_hip_register_context(dev, host, 2) == 1 and "at least 3 words" in _lib.last_error()
    assert lib.iris_hip_register_context(dev, host, 9) == 1 and "bad context contents" in _lib.last_error()  # 8 bases need 10 words
    bad_rank = (ctypes.c_int64 * 10)(8, 8, *([0] * 8))
    assert lib.iris_hip_register_context(dev, ctypes.cast(bad_rank, ctypes.c_void_p), 10) == 1
    assert "bad context contents" in _lib.last_error()
    assert lib.iris_hip_unregister_context(dev) == 0
    assert lib.iris_hip_unregister_context(dev) == 0                # unknown by now: still fine
    assert lib.iris_hip_unregister_context(null) == 0


def test_device_span_releases_its_memory_exactly_once():
    """The object torch keeps alive for the heap's tensors owns the allocation."""
    from iris_amd.host.heap import _DeviceSpan

    freed = []
    span = _DeviceSpan(0x7000, 64, freed.append)
    assert span.__cuda_array_interface__["data"] == (0x7000, False)
    keeper = span  # a second reference, as torch's tensor storage holds one
    del span
    assert freed == []
    del keeper
    assert freed == [0x7000]
    _DeviceSpan(0x7000, 64)  # no release callback: nothing to do
    assert freed == [0x7000]


def test_host_heap_tensors_outlive_their_context():
    ctx = cpu_ctx()
    t = ctx.zeros((8, 8), dtype=torch.float32)
    t.fill_(3.0)
    del ctx
    assert float(t.sum()) == 192.0


def test_header_enumerations_match_python():
    header = open(os.path.join(ROOT, "include", "iris_hip.h")).read()
    values = {k: int(v) for k, v in re.findall(r"(IRIS_HIP_[A-Z0-9_]+)\s*=\s*(\d+)", header)}
    assert (values["IRIS_HIP_BF16"], values["IRIS_HIP_FP16"], values["IRIS_HIP_FP32"], values["IRIS_HIP_FP8_E4M3"]) == (
        _lib.BF16, _lib.FP16, _lib.FP32, _lib.FP8_E4M3)
    assert (values["IRIS_HIP_VARIANT_ONE_SHOT"], values["IRIS_HIP_VARIANT_TWO_SHOT"]) == (_lib.VARIANT_ONE_SHOT, _lib.VARIANT_TWO_SHOT)
    assert (values["IRIS_HIP_GATHER_K"], values["IRIS_HIP_GATHER_M"]) == (_lib.GATHER_K, _lib.GATHER_M)
    assert (values["IRIS_HIP_ACC_FP32"], values["IRIS_HIP_ACC_REFERENCE"]) == (_lib.ACC_FP32, _lib.ACC_REFERENCE)
    assert (values["IRIS_HIP_PATH_AUTO"], values["IRIS_HIP_PATH_MFMA"], values["IRIS_HIP_PATH_GENERIC"]) == (0, 1, 2)


def test_no_product_code_touches_the_oracle():
    """The oracle is the checker; the package must not import it (there is no CPU compute path)."""
    for dirpath, _, files in os.walk(os.path.join(ROOT, "iris_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("There is no fallback", ""), f"{f} mentions the oracle"


# -- index math of the kernels, replayed on the CPU ------------------------------------------------------------------
def test_layout_simulation(tmp_path):
    exe = tmp_path / "layout_sim"
    src = os.path.join(ROOT, "tests", "host_sim", "layout_sim.cpp")
    subprocess.run(["g++", "-O1", "-std=c++17", "-I" + os.path.join(ROOT, "iris_amd", "csrc"), "-o", str(exe), src], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout[-2000:]
    assert "all checks passed" in out.stdout
