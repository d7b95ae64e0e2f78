"""Helpers shared by the GPU parity tests: seeded inputs, peer staging, comparisons."""

import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import iris_oracle as oracle  # noqa: E402  (the checker; tests only)


def randn_cpu(shape, seed, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def randint_cpu(shape, seed, dtype, lo=-3, hi=4):
    """Small integers: products and sums of a few hundred of them are exact in fp32."""
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi, shape, generator=g).to(dtype)


def heap_tensor(ctx, cpu_tensor):
    t = ctx.zeros(tuple(cpu_tensor.shape), dtype=cpu_tensor.dtype)
    t.copy_(cpu_tensor)
    return t


def stage_peers(ctx, workspace, peer_aux):
    """Write the peers' aux buffers and raise their flags in the other slots of the heap."""
    for r in range(ctx.get_num_ranks()):
        if r == ctx.get_rank():
            continue
        ctx.peer_view(workspace.aux_buffer, r).copy_(peer_aux[r])
        ctx.peer_view(workspace.locks, r).fill_(1)


def slot_copies(ctx, tensor):
    """CPU copies of a symmetric tensor as every slot holds it."""
    return [ctx.peer_view(tensor, r).cpu() for r in range(ctx.get_num_ranks())]


def assert_bits_equal(x, ref, what):
    assert x.dtype == ref.dtype and x.shape == ref.shape, f"{what}: {x.dtype}{tuple(x.shape)} vs {ref.dtype}{tuple(ref.shape)}"
    xi = x.contiguous().view(torch.int16 if x.element_size() == 2 else torch.int32)
    ri = ref.contiguous().view(torch.int16 if ref.element_size() == 2 else torch.int32)
    bad = (xi != ri).nonzero()
    assert bad.numel() == 0, f"{what}: {bad.shape[0]} elements differ, first at {bad[0].tolist()}: {x[tuple(bad[0])]} vs {ref[tuple(bad[0])]}"
