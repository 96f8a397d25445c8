"""relu / leaky_relu / tanh / gelu -- the four element-wise names the reference's kernel package exports
(lite_llama/kernels/activations.py:19-57: ``@triton.jit`` device helpers, no caller in its models).  Here: one HIP
kernel behind the C ABI (``ll_activation``, csrc/norm_act.hip) -- fp32 arithmetic, one rounding to the storage dtype; like
every other entry of this package there is no eager / CPU path (CPU tensors raise)."""

from __future__ import annotations

import torch

from .. import _lib as L


def _apply(x: torch.Tensor, kind: int, what: str) -> torch.Tensor:
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError(f"{what}: fp16 / bf16 tensors only, got {x.dtype}")
    L.require_cuda(x)
    xc = x.contiguous()
    y = torch.empty_like(xc)
    L.check(L.lib().ll_activation(y.data_ptr(), xc.data_ptr(), xc.numel(), kind, L.dtype_code(x.dtype), L.stream_ptr()), what)
    return y.view(x.shape)


@torch.no_grad()
def relu(x):
    return _apply(x, 0, "relu")


@torch.no_grad()
def leaky_relu(x):
    return _apply(x, 1, "leaky_relu")


@torch.no_grad()
def tanh(x):
    return _apply(x, 2, "tanh")


@torch.no_grad()
def gelu(x):
    return _apply(x, 3, "gelu")


@torch.no_grad()
def xielu(z: torch.Tensor, pq: torch.Tensor) -> torch.Tensor:
    """xIELU with its two learned numbers ``pq = (p, q)``: ``softplus(p) z^2 + z / 2`` for ``z > 0``, else
    ``(1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2``; fp32 arithmetic, one rounding to the storage dtype (fp16 / bf16 / fp32)."""
    L.require_cuda(z, pq)
    if pq.dtype != z.dtype or pq.numel() != 2:
        raise ValueError("xielu: pq holds the two numbers (p, q) in the activations' dtype")
    zc = z.contiguous()
    y = torch.empty_like(zc)
    L.check(L.lib().ll_xielu(y.data_ptr(), zc.data_ptr(), pq.contiguous().data_ptr(), zc.numel(), L.dtype_code(z.dtype),
                             L.stream_ptr()), "xielu")
    return y.view(z.shape)
