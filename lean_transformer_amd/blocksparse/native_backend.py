"""Block-sparse matmul in the reference's "native" weight format, on the HIP kernels.

Same functions and argument meaning as lean_transformer/blocksparse/native_backend.py:9-76; the reference's per-block batched
matmul + embedding_bag / embedding gather is replaced by one kernel launch that walks the index tables.
"""
from typing import Optional, Tuple

import torch

from .. import _native as nat


def _sparse_desc(weight: torch.Tensor, forward_indices: Optional[torch.Tensor], backward_indices: Optional[torch.Tensor],
                 out_features: int) -> "nat.LtLinear":
    in_features, blocks_per_in, block = weight.shape
    desc = nat.LtLinear()
    desc.weight = nat.ptr(weight)
    desc.in_features, desc.out_features = in_features, out_features
    desc.block, desc.blocks_per_in = block, blocks_per_in
    desc.blocks_per_out = (in_features // block) * blocks_per_in // (out_features // block)
    # each direction reads one table (forward: forward_indices, gradients: backward_indices); the other stays NULL
    desc.forward_indices, desc.backward_indices = nat.ptr(forward_indices), nat.ptr(backward_indices)
    return desc


def blocksparse_matmul(input: torch.Tensor, weight: torch.Tensor, forward_indices: torch.Tensor) -> torch.Tensor:
    """input [..., in_features] times a block-sparse weight -> [..., out_features].

    weight: the active blocks in the native order [in_features, blocks per input block, block]; forward_indices: the int32
    table [output blocks, K] that get_indices_from_layout returns first (entry = input block * blocks per input block +
    position of the weight block under that input block).  out_features = output blocks * block."""
    if input.shape[-1] != weight.shape[0]:
        raise AssertionError(f"input has {input.shape[-1]} features, the weight takes {weight.shape[0]}")
    device = nat.require_gpu(input, weight, forward_indices)
    block = weight.shape[2]
    out_features = forward_indices.shape[0] * block
    x = input.reshape(-1, input.shape[-1]).contiguous()
    w = weight.contiguous()
    if w.dtype != x.dtype:
        w = w.to(x.dtype)
    fwd = forward_indices.to(torch.int32).contiguous()
    y = torch.empty(x.shape[0], out_features, dtype=x.dtype, device=device)
    if x.shape[0] > 0:
        desc = _sparse_desc(w, fwd, None, out_features)
        lib = nat.lib(x.dtype)
        nat.check(lib.lt_blocksparse_forward(desc, x.shape[0], nat.dtype_code(x.dtype), nat.ptr(x), nat.ptr(y),
                                             nat.current_stream(device)), "lt_blocksparse_forward", lib)
    return y.view(*input.shape[:-1], out_features)


def blocksparse_matmul_backward(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                backward_indices: torch.Tensor, input_requires_grad: bool = True,
                                weight_requires_grad: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gradients of blocksparse_matmul w.r.t. input and/or weight; a gradient that is not requested comes back empty."""
    if not (input_requires_grad or weight_requires_grad):
        raise AssertionError("backward was asked for neither the input's nor the weight's gradient")
    device = nat.require_gpu(grad_output, input, weight, backward_indices)
    x = input.reshape(-1, input.shape[-1]).contiguous()
    dy = grad_output.reshape(x.shape[0], -1).contiguous()
    if dy.dtype != x.dtype:
        dy = dy.to(x.dtype)
    w = weight.contiguous()
    if w.dtype != x.dtype:
        w = w.to(x.dtype)
    bwd = backward_indices.to(torch.int64).contiguous()
    grad_input = torch.empty_like(x) if input_requires_grad else None
    grad_weight = torch.empty_like(w) if weight_requires_grad else None
    if x.shape[0] > 0:
        desc = _sparse_desc(w, None, bwd, dy.shape[1])
        lib = nat.lib(x.dtype)
        nat.check(lib.lt_blocksparse_backward(desc, x.shape[0], nat.dtype_code(x.dtype), nat.ptr(x), nat.ptr(dy),
                                              nat.ptr(grad_input), nat.ptr(grad_weight), nat.current_stream(device)),
                  "lt_blocksparse_backward", lib)
    else:
        if grad_weight is not None:
            grad_weight.zero_()
    empty = torch.empty(0, device=device, dtype=x.dtype)
    return (grad_input.view(*grad_output.shape[:-1], input.shape[-1]) if grad_input is not None else empty,
            grad_weight.to(weight.dtype) if grad_weight is not None else empty)
