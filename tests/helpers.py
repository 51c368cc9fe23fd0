"""Shared helpers of the GPU parity tests: turn a LeanFFN module into oracle parameters, run the oracle, collect gradients."""
from typing import Optional

import torch

import lean_transformer_amd as lt
from lean_transformer_amd import _native as nat
from lean_transformer_amd.utils import activation_kind
from oracle import ffn as offn


def oracle_linear(proj, device, dtype) -> offn.LinearParams:
    def leaf(t):
        return None if t is None else t.detach().to(device=device, dtype=dtype).clone().requires_grad_(True)

    if isinstance(proj, lt.GeneralizedLinear):
        first, second = proj.get_combined_lowrank_components()
        fwd, bwd = proj.matrix.forward_indices, proj.matrix.backward_indices
        return offn.LinearParams(leaf(proj.weight), leaf(proj.bias), leaf(first), leaf(second),
                                 None if fwd is None else fwd.cpu(), None if bwd is None else bwd.cpu(),
                                 out_features=proj.out_features)
    return offn.LinearParams(leaf(proj.weight), leaf(proj.bias), out_features=proj.out_features)


def oracle_params(ffn: "lt.LeanFFN", device="cpu", dtype=torch.float32, bf16_rounding=False) -> offn.FFNParams:
    """fp32 (or fp64) leaf copies of a module's parameters, in the oracle's container"""
    def leaf(t):
        return None if t is None else t.detach().to(device=device, dtype=dtype).clone().requires_grad_(True)

    post = ffn.post_layer_norm
    return offn.FFNParams(
        leaf(ffn.pre_layer_norm.weight), leaf(ffn.pre_layer_norm.bias),
        oracle_linear(ffn.i2h_proj, device, dtype), oracle_linear(ffn.h2o_proj, device, dtype),
        leaf(post.weight) if post is not None else None, leaf(post.bias) if post is not None else None,
        offn.FFNConfig(gated=ffn.gated, act=activation_kind(ffn.activation), ln_eps=ffn.pre_layer_norm.eps,
                       residual=ffn.residual, dropout=ffn.dropout if ffn.training else 0.0,
                       bf16_rounding=bf16_rounding))


def module_tensors(ffn: "lt.LeanFFN"):
    """module parameters in the order of FFNParams.tensors() (combined low-rank factors are not leaves: callers that use
    adapters compare those through named_parameters instead)"""
    out = [ffn.pre_layer_norm.weight, ffn.pre_layer_norm.bias]
    for proj in (ffn.i2h_proj, ffn.h2o_proj):
        out.append(proj.weight)
        if proj.bias is not None:
            out.append(proj.bias)
        if isinstance(proj, lt.GeneralizedLinear) and proj.matrix.lowrank_first is not None and proj.adapter_first is None:
            out += [proj.matrix.lowrank_first, proj.matrix.lowrank_second]
        elif isinstance(proj, lt.GeneralizedLinear) and proj.adapter_first is not None and proj.matrix.lowrank_first is None:
            out += [proj.adapter_first, proj.adapter_second]
    if ffn.post_layer_norm is not None:
        out += [ffn.post_layer_norm.weight, ffn.post_layer_norm.bias]
    return out


def dropout_mask(tokens: int, hidden: int, p: float, seed: int, offset: int, device) -> torch.Tensor:
    """the keep-mask the fused kernels apply for this Philox (seed, offset), as a bool tensor [tokens, hidden]"""
    keep = torch.empty(tokens, hidden, dtype=torch.uint8, device=device)
    nat.check(nat.lib().lt_dropout_mask(tokens, hidden, p, seed, offset, nat.ptr(keep), nat.current_stream(keep.device)),
              "lt_dropout_mask")
    return keep.bool()


def generator_position(device):
    gen = torch.cuda.default_generators[torch.device(device).index or 0]
    return gen.initial_seed(), gen.get_offset()


def run_oracle(p: offn.FFNParams, x: torch.Tensor, dy: torch.Tensor, mask: Optional[torch.Tensor] = None):
    """(y, dx, [param grads in p.tensors() order]) of the plain-autograd oracle"""
    x = x.detach().clone().requires_grad_(True)
    y = offn.plain_ffn(x, p, mask)
    grads = torch.autograd.grad(y, [x, *p.tensors()], dy)
    return y.detach(), grads[0], list(grads[1:])
