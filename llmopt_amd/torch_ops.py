"""`torch.ops.llmopt.w4a16_linear` on MI355X.

The reference registers
`w4a16_linear(Tensor input, Tensor packed_weight, Tensor scale, Tensor? bias) -> Tensor`
in the `llmopt` namespace (python/llmopt_backend/quantization.py:174-185) and
backs it with its native runtime (native/metal_runtime.cpp:139-147).  This
module registers the same schema for ROCm tensors: the tensors' device memory
is wrapped as buffers of the HIP backend (no copies), the kernel is recorded
on torch's current stream and nothing waits for it.

    import llmopt_amd.torch_ops            # registers the operator
    y = torch.ops.llmopt.w4a16_linear(x, packed, scale, bias)

Same argument checks as the reference (quantization.py:104-118,144-147): fp16
activations and bias, uint8 `[N, K/2]` weights, fp16 `[N, K/64]` scales.
"""
from __future__ import annotations

import struct
import threading
from typing import Optional

import torch

from .native import Runtime

GROUP_SIZE = 64
_library: Optional[torch.library.Library] = None
_runtimes: dict[int, Runtime] = {}
_lock = threading.Lock()


def _runtime(device_index: int) -> Runtime:
    with _lock:
        runtime = _runtimes.get(device_index)
        if runtime is None:
            runtime = Runtime(device=device_index)
            _runtimes[device_index] = runtime
        return runtime


def _check_arguments(input, packed_weight, scale, bias):
    if packed_weight.dim() != 2:
        raise ValueError(f"packed W4 weight must be 2-D, got shape {tuple(packed_weight.shape)}")
    output_features, packed_k = packed_weight.shape
    logical_k = packed_k * 2
    if logical_k % GROUP_SIZE != 0:
        raise ValueError(f"W4 K dimension {logical_k} is not a multiple of the group size {GROUP_SIZE}")
    groups = logical_k // GROUP_SIZE
    if packed_weight.dtype != torch.uint8:
        raise TypeError(f"packed W4 weight storage must be torch.uint8, got {packed_weight.dtype}")
    if scale.dtype != torch.float16:
        raise TypeError(f"W4 scales must be torch.float16, got {scale.dtype}")
    if tuple(scale.shape) != (output_features, groups):
        raise ValueError(f"W4 scales must have shape [{output_features}, {groups}], got {tuple(scale.shape)}")
    if input.dtype != torch.float16:
        raise TypeError(f"W4A16 activations must be torch.float16, got {input.dtype}")
    if bias is not None and bias.dtype != torch.float16:
        raise TypeError(f"W4A16 bias must be torch.float16, got {bias.dtype}")
    if input.shape[-1] != logical_k:
        raise ValueError(f"W4A16 input has {input.shape[-1]} features, the weight expects {logical_k}")
    if bias is not None and bias.numel() != output_features:
        raise ValueError(f"W4A16 bias must have {output_features} elements, got {bias.numel()}")
    return output_features, logical_k


def _w4a16_linear_hip(input, packed_weight, scale, bias=None):
    n, k = _check_arguments(input, packed_weight, scale, bias)
    x = input.contiguous().view(-1, k)
    m = x.shape[0]
    output = torch.empty((m, n), dtype=torch.float16, device=input.device)
    if m == 0:
        return output.view(*input.shape[:-1], n)
    packed_weight, scale = packed_weight.contiguous(), scale.contiguous()
    bias = bias.contiguous() if bias is not None else None
    runtime = _runtime(input.device.index if input.device.index is not None else torch.cuda.current_device())
    runtime.set_stream(torch.cuda.current_stream(input.device).cuda_stream)
    wrap = lambda t: runtime.wrap(t.data_ptr(), t.numel() * t.element_size())
    b_scale = wrap(scale)
    buffers = [wrap(x), wrap(packed_weight), b_scale, wrap(bias) if bias is not None else b_scale, wrap(output)]
    name = "llmopt_w4a16_linear_f16_g64" if m == 1 else "llmopt_w4a16_linear_f16_g64_m4"
    columns = m * n if m == 1 else ((m + 3) // 4) * n
    batch = runtime.begin_batch()
    batch.dispatch(name, buffers, struct.pack("<5I", m, n, k, 1 if bias is not None else 0, 0),
                   grid=(((columns + 7) // 8) * 256, 1, 1), group=(256, 1, 1))
    batch.commit_async()  # ordered on torch's stream; the tensors above outlive the launch call
    return output.view(*input.shape[:-1], n)


def _w4a16_linear_meta(input, packed_weight, scale, bias=None):
    del scale, bias
    return torch.empty((*input.shape[:-1], packed_weight.shape[0]), dtype=torch.float16, device="meta")


def register() -> None:
    """Defines `llmopt::w4a16_linear` (once) with a ROCm implementation and a meta kernel."""
    global _library
    if _library is not None:
        return
    library = torch.library.Library("llmopt", "DEF")
    library.define("w4a16_linear(Tensor input, Tensor packed_weight, Tensor scale, Tensor? bias) -> Tensor")
    library.impl("w4a16_linear", _w4a16_linear_hip, "CUDA")  # ROCm tensors carry the CUDA dispatch key
    library.impl("w4a16_linear", _w4a16_linear_meta, "Meta")
    _library = library


register()
