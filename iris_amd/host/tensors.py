"""torch-like tensor factories on the symmetric heap.

Same contract as iris/host/memory/tensors.py:43-881 of the reference: sizes as varargs or one
tuple/list, default dtype from torch, a device argument that must name the heap's device
(RuntimeError otherwise), an optional `out=` that must live on the heap with the right element count
and dtype, torch.strided layout only.  Every factory allocates flat, fills, then reshapes.
"""

import math

import torch


def parse_size(size):
    """`(2, 3)`, `((2, 3),)` and `([2, 3],)` all mean shape (2, 3).  Returns (shape, numel)."""
    while len(size) == 1 and isinstance(size[0], (tuple, list)):
        size = size[0]
    return tuple(size), math.prod(size)


def is_valid_device(device, iris_device):
    if device is None:
        return True
    requested = torch.device(device) if isinstance(device, str) else device
    if requested.type != iris_device.type:
        return False
    if requested.type == "cuda":
        return requested.index is None or requested.index == iris_device.index
    return True


def throw_if_invalid_device(device, iris_device):
    if not is_valid_device(device, iris_device):
        raise RuntimeError(
            f"Device mismatch: requested device {device} but Iris instance is on device {iris_device}. "
            f"Iris only supports tensors on its own device."
        )


def throw_if_invalid_output_tensor(heap, tensor, num_elements, dtype):
    if tensor.numel() != num_elements:
        raise RuntimeError(f"The output tensor has {tensor.numel()} elements, but {num_elements} are required")
    if tensor.dtype != dtype:
        raise RuntimeError(f"The output tensor has dtype {tensor.dtype}, but {dtype} is required")
    if not heap.is_symmetric(tensor):
        raise RuntimeError("The output tensor is not on the symmetric heap")


def apply_layout(tensor, layout):
    if layout == torch.strided:
        return tensor
    raise ValueError(f"Layout {layout} not supported. Only torch.strided is currently supported.")


def _make(heap, iris_device, size, fill, *, out, dtype, layout, device, requires_grad):
    if dtype is None:
        dtype = torch.get_default_dtype()
    throw_if_invalid_device(device, iris_device)
    size, num_elements = parse_size(size)
    if out is not None:
        throw_if_invalid_output_tensor(heap, out, num_elements, dtype)
        flat = out.view(num_elements)
    else:
        flat = heap.allocate(num_elements, dtype)
    if fill is not None:
        fill(flat)
    tensor = apply_layout(flat.view(size) if out is not None else flat.reshape(size), layout)
    if requires_grad:
        tensor.requires_grad_()
    return tensor


def zeros(heap, iris_device, size, *, out=None, dtype=None, layout=torch.strided, device=None, requires_grad=False):
    return _make(heap, iris_device, size, lambda t: t.zero_(), out=out, dtype=dtype, layout=layout,
                 device=device, requires_grad=requires_grad)


def ones(heap, iris_device, size, *, out=None, dtype=None, layout=torch.strided, device=None, requires_grad=False):
    return _make(heap, iris_device, size, lambda t: t.fill_(1), out=out, dtype=dtype, layout=layout,
                 device=device, requires_grad=requires_grad)


def full(heap, iris_device, size, fill_value, *, out=None, dtype=None, layout=torch.strided, device=None,
         requires_grad=False):
    if dtype is None:
        if isinstance(fill_value, bool):
            dtype = torch.bool
        elif isinstance(fill_value, int):
            dtype = torch.int64
        else:
            dtype = torch.get_default_dtype()
    return _make(heap, iris_device, size, lambda t: t.fill_(fill_value), out=out, dtype=dtype, layout=layout,
                 device=device, requires_grad=requires_grad)


def empty(heap, iris_device, size, *, out=None, dtype=None, layout=torch.strided, device=None, requires_grad=False):
    return _make(heap, iris_device, size, None, out=out, dtype=dtype, layout=layout, device=device,
                 requires_grad=requires_grad)


def zeros_like(heap, iris_device, input, *, dtype=None, layout=None, device=None, requires_grad=False):
    return zeros(heap, iris_device, tuple(input.shape), dtype=dtype or input.dtype,
                 layout=layout or torch.strided, device=device, requires_grad=requires_grad)


def randn(heap, iris_device, size, *, generator=None, out=None, dtype=None, layout=torch.strided, device=None,
          requires_grad=False):
    def fill(t):
        if t.dtype in (torch.float32, torch.float64, torch.float16, torch.bfloat16):
            t.normal_(generator=generator)
        else:  # 8-bit float types: draw in fp32, then cast
            t.copy_(torch.randn(t.shape, generator=generator, device=t.device, dtype=torch.float32))
    return _make(heap, iris_device, size, fill, out=out, dtype=dtype, layout=layout, device=device,
                 requires_grad=requires_grad)


def rand(heap, iris_device, size, *, generator=None, out=None, dtype=None, layout=torch.strided, device=None,
         requires_grad=False):
    return _make(heap, iris_device, size, lambda t: t.uniform_(0, 1, generator=generator), out=out, dtype=dtype,
                 layout=layout, device=device, requires_grad=requires_grad)


def uniform(heap, iris_device, size, low=0.0, high=1.0, dtype=torch.float):
    return _make(heap, iris_device, size, lambda t: t.uniform_(low, high), out=None, dtype=dtype,
                 layout=torch.strided, device=None, requires_grad=False)


def randint(heap, iris_device, low, high, size, *, generator=None, out=None, dtype=None, layout=torch.strided,
            device=None, requires_grad=False):
    if dtype is None:
        dtype = torch.int64
    return _make(heap, iris_device, (size,), lambda t: t.random_(low, high, generator=generator), out=out,
                 dtype=dtype, layout=layout, device=device, requires_grad=requires_grad)


def arange(heap, iris_device, start, end, step, *, out=None, dtype=None, layout=torch.strided, device=None,
           requires_grad=False):
    if step == 0:
        raise ValueError("step must be non-zero")
    if (step > 0 and start >= end) or (step < 0 and start <= end):
        raise ValueError(f"Invalid range: start={start}, end={end}, step={step}")
    num_elements = math.ceil((end - start) / step)
    if dtype is None:
        if any(isinstance(x, float) for x in (start, end, step)):
            dtype = torch.get_default_dtype()
        else:
            dtype = torch.int64

    def fill(t):
        t.copy_(torch.arange(start, end, step, dtype=dtype, device=t.device))
    return _make(heap, iris_device, (num_elements,), fill, out=out, dtype=dtype, layout=layout, device=device,
                 requires_grad=requires_grad)


def linspace(heap, iris_device, start, end, steps, *, out=None, dtype=None, layout=torch.strided, device=None,
             requires_grad=False):
    steps = int(steps[0]) if isinstance(steps, (tuple, list)) else int(steps)
    if dtype is None:
        dtype = torch.get_default_dtype()

    def fill(t):
        t.copy_(torch.linspace(start, end, steps, dtype=dtype, device=t.device))
    return _make(heap, iris_device, (steps,), fill, out=out, dtype=dtype, layout=layout, device=device,
                 requires_grad=requires_grad)
