"""LeanFFN: the memory-efficient transformer feed-forward block, on hand-written gfx950 kernels.

Drop-in for lean_transformer/ffn.py: same constructor (ffn.py:35-48), attributes, state_dict keys, and the same
``_LeanFFN.apply`` argument order (ffn.py:148-175).  The forward keeps only the layer input and the pre-activation (plus
8 bytes of LayerNorm statistics per token) for backward; LayerNorm output and the (gated) activation are recomputed inside
the backward kernels.  All arithmetic of the custom-gradient path happens in csrc/libleanffn.so; nothing here falls back to
PyTorch ops.  ``ffn_custom_grad=False`` selects the plain-autograd composition, as in the reference (ffn.py:69-85).
"""
import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _native as nat
from .blocksparse.linear import GeneralizedLinear, _as, compute_dtype_for, linear_desc
from .utils import ACT2FN, ACT_KINDS, activation_kind


class LeanFFN(nn.Module):
    """
    A transformer FFN module that doesn't hog your GPU memory. Uses a manually optimized differentiation algorithm.

    :param hidden_size: base hidden size of the transformer
    :param intermediate_size: a (typically larger) hidden dimension where activation is applied
    :param activation: a pytorch nonlinearity to use in the intermediate layer
    :param gated: use gated activations based on https://arxiv.org/abs/2002.05202 and https://arxiv.org/abs/2102.11972
      note: gated activations require 1.5x more parameters compared to their non-gated variants.
    :param layer_norm_eps: see torch.nn.functional.layer_norm
    :param post_layer_norm: if set, applies an additional layer norm to projected attention outputs before residuals
    :param dropout: hidden dropout probability, applied to the output projection (before adding residual)
    :param residual: if True, adds the original layer input to the final layer output
    :param ffn_custom_grad: if True (default), use the fused HIP forward/backward that saves memory
    :param i2h_proj: custom *first* linear layer (hidden_size -> intermediate_size or 2x indermediate_size)
    :param h2o_proj: custom *second* linear layer (intermediate_size -> hidden_size)
    """

    def __init__(
        self,
        hidden_size: int,
        intermediate_size: int,
        activation=ACT2FN["gelu_fused"],
        gated: bool = False,
        layer_norm_eps: float = 1e-12,
        dropout: float = 0.0,
        post_layer_norm: bool = False,
        i2h_proj: Optional[nn.Linear] = None,
        h2o_proj: Optional[nn.Linear] = None,
        residual: bool = True,
        ffn_custom_grad: bool = True,
    ):
        super().__init__()
        i2h_out_features = intermediate_size * 2 if gated else intermediate_size
        self.i2h_proj = nn.Linear(hidden_size, i2h_out_features) if i2h_proj is None else i2h_proj
        self.h2o_proj = nn.Linear(intermediate_size, hidden_size) if h2o_proj is None else h2o_proj
        if ffn_custom_grad:
            assert type(self.i2h_proj) in (nn.Linear, GeneralizedLinear), "custom grad supports only nn.Linear and GeneralizedLinear"
            assert type(self.h2o_proj) in (nn.Linear, GeneralizedLinear), "custom grad supports only nn.Linear and GeneralizedLinear"
        assert self.i2h_proj.in_features == self.h2o_proj.out_features == hidden_size
        assert self.i2h_proj.out_features == i2h_out_features and self.h2o_proj.in_features == intermediate_size
        self.pre_layer_norm = nn.LayerNorm(hidden_size, eps=layer_norm_eps)
        self.post_layer_norm = nn.LayerNorm(hidden_size, eps=layer_norm_eps) if post_layer_norm else None
        self.activation = activation
        self.gated = gated
        self.dropout = dropout
        self.residual = residual
        self.ffn_custom_grad = ffn_custom_grad

    def forward(self, input):
        return self._forward_custom(input) if self.ffn_custom_grad else self._forward_pytorch(input)

    def _forward_pytorch(self, input):
        input_2d = input.view(-1, input.shape[-1])
        input_ln = F.layer_norm(
            input_2d, input.shape[-1:], self.pre_layer_norm.weight, self.pre_layer_norm.bias, self.pre_layer_norm.eps
        )
        pre_activation = self.i2h_proj(input_ln)
        hid_act = _LeanFFN._apply_activation(pre_activation, self.activation, gated=self.gated)

        out = self.h2o_proj(hid_act)
        if self.post_layer_norm:
            out = self.post_layer_norm(out)

        if self.dropout and self.training:
            out = torch.dropout(out, self.dropout, self.training)
        if self.residual:
            out = out + input_2d
        return out.view(*input.shape)

    def _forward_custom(self, input):
        post_ln_weight = post_ln_bias = None
        if self.post_layer_norm is not None:
            post_ln_weight, post_ln_bias = self.post_layer_norm.weight, self.post_layer_norm.bias
        i2h_lowrank_first = i2h_lowrank_second = h2o_lowrank_first = h2o_lowrank_second = None
        i2h_forward_indices = i2h_backward_indices = h2o_forward_indices = h2o_backward_indices = None
        i2h_matmul_op = h2o_matmul_op = None
        if isinstance(self.i2h_proj, GeneralizedLinear):
            i2h_lowrank_first, i2h_lowrank_second = self.i2h_proj.get_combined_lowrank_components()
            i2h_forward_indices = self.i2h_proj.matrix.forward_indices
            i2h_backward_indices = self.i2h_proj.matrix.backward_indices
            i2h_matmul_op = self.i2h_proj.matrix.matmul_op
        if isinstance(self.h2o_proj, GeneralizedLinear):
            h2o_lowrank_first, h2o_lowrank_second = self.h2o_proj.get_combined_lowrank_components()
            h2o_forward_indices = self.h2o_proj.matrix.forward_indices
            h2o_backward_indices = self.h2o_proj.matrix.backward_indices
            h2o_matmul_op = self.h2o_proj.matrix.matmul_op

        return _LeanFFN.apply(
            input,
            self.pre_layer_norm.weight, self.pre_layer_norm.bias,
            self.i2h_proj.weight, self.i2h_proj.bias, i2h_lowrank_first, i2h_lowrank_second,
            i2h_forward_indices, i2h_backward_indices, i2h_matmul_op,
            self.h2o_proj.weight, self.h2o_proj.bias, h2o_lowrank_first, h2o_lowrank_second,
            h2o_forward_indices, h2o_backward_indices, h2o_matmul_op,
            post_ln_weight, post_ln_bias,
            self.activation, self.gated, self.dropout, self.training, self.pre_layer_norm.eps, self.residual,
        )


def _draw_dropout_stream(device: torch.device, numel: int):
    """(seed, offset) of a fresh Philox sub-stream of the device's default generator, advancing it like a dropout op would.
    Goes through the generator state only (no device sync), so seeding / checkpoint replay of the RNG state reproduce it."""
    gen = torch.cuda.default_generators[device.index if device.index is not None else torch.cuda.current_device()]
    seed, offset = gen.initial_seed(), gen.get_offset()
    gen.set_offset(offset + 4 * math.ceil(numel / 4))
    return seed, offset


class _LeanFFN(torch.autograd.Function):
    """Autograd function for transformer FFN: one library call forward, one backward."""

    @staticmethod
    def _apply_activation(pre_activation: torch.Tensor, activation: callable, gated: bool):
        if not gated:
            return activation(pre_activation)
        else:
            pre_gate, lin = pre_activation.split(pre_activation.shape[-1] // 2, dim=-1)
            return activation(pre_gate).mul_(lin)

    @staticmethod
    def forward(
        ctx,
        input: torch.Tensor,
        ln_weight: torch.Tensor,
        ln_bias: torch.Tensor,
        i2h_weight: torch.Tensor,
        i2h_bias: Optional[torch.Tensor],
        i2h_lowrank_first: Optional[torch.Tensor],
        i2h_lowrank_second: Optional[torch.Tensor],
        i2h_forward_indices: Optional[torch.IntTensor],
        i2h_backward_indices: Optional[torch.IntTensor],
        i2h_matmul_op,
        h2o_weight: torch.Tensor,
        h2o_bias: Optional[torch.Tensor],
        h2o_lowrank_first: Optional[torch.Tensor],
        h2o_lowrank_second: Optional[torch.Tensor],
        h2o_forward_indices: Optional[torch.IntTensor],
        h2o_backward_indices: Optional[torch.IntTensor],
        h2o_matmul_op,
        post_ln_weight: Optional[torch.Tensor],
        post_ln_bias: Optional[torch.Tensor],
        activation: callable,
        gated: bool,
        dropout: float,
        training: bool,
        ln_eps: float,
        residual: bool,
    ):
        if i2h_matmul_op is not None or h2o_matmul_op is not None:
            raise NotImplementedError("matmul_op plug-ins (Triton) are not supported; the block-sparse matmul is built in")
        device = nat.require_gpu(input, ln_weight, ln_bias, i2h_weight, i2h_bias, i2h_lowrank_first, i2h_lowrank_second,
                                 h2o_weight, h2o_bias, h2o_lowrank_first, h2o_lowrank_second, post_ln_weight, post_ln_bias)
        act = ACT_KINDS[activation_kind(activation)]
        cdt = compute_dtype_for(i2h_weight)
        io = input.dtype
        if io not in (torch.float32, torch.bfloat16) or (io == torch.bfloat16 and cdt != torch.bfloat16):
            raise TypeError(f"LeanFFN: input dtype {io} with compute dtype {cdt} is not supported "
                            "(float32 input with float32/bfloat16 weights, or bfloat16 input with bfloat16 weights)")
        hidden = input.shape[-1]
        x = input.detach().reshape(-1, hidden).contiguous()
        tokens = x.shape[0]

        ctx._cfg = (act, bool(gated), float(ln_eps), bool(residual), cdt)
        ctx._dropout = (0.0, 0, 0)
        if training and dropout:
            ctx._dropout = (float(dropout), *_draw_dropout_stream(device, tokens * hidden))

        desc, keep = _LeanFFN._describe(
            ctx, tokens, hidden, ln_weight, ln_bias, i2h_weight, i2h_bias, i2h_lowrank_first, i2h_lowrank_second,
            i2h_forward_indices, i2h_backward_indices, h2o_weight, h2o_bias, h2o_lowrank_first, h2o_lowrank_second,
            h2o_forward_indices, h2o_backward_indices, post_ln_weight, post_ln_bias, io)
        # fp32 copies of the small vectors (LayerNorm parameters, biases): backward reuses them instead of converting again
        ctx._small_fp32 = (keep[0], keep[1], keep[2], keep[3], keep[4][1], keep[5][1])
        n1 = desc.i2h.out_features
        y = torch.empty_like(x)
        pre_activation = torch.empty(tokens, n1, dtype=cdt, device=device)
        ln_stats = torch.empty(tokens, 2, dtype=torch.float32, device=device)
        post_ln_input = torch.empty(tokens, hidden, dtype=cdt, device=device) if post_ln_weight is not None else None
        i2h_hid = torch.empty(tokens, desc.i2h.lowrank, dtype=cdt, device=device) if desc.i2h.lowrank else None
        h2o_hid = torch.empty(tokens, desc.h2o.lowrank, dtype=cdt, device=device) if desc.h2o.lowrank else None
        if tokens > 0:
            saved = nat.LtFfnSaved(nat.ptr(pre_activation), nat.ptr(ln_stats), nat.ptr(post_ln_input), nat.ptr(i2h_hid),
                                   nat.ptr(h2o_hid))
            lib = nat.lib()
            ws = nat.workspace(lib.lt_ffn_forward_workspace_bytes(desc), device)
            nat.check(lib.lt_ffn_forward(desc, nat.ptr(x), nat.ptr(y), saved, nat.ptr(ws), ws.numel(),
                                         nat.current_stream(device)), "lt_ffn_forward")
            del ws, keep
        ctx.save_for_backward(
            input, pre_activation, ln_stats, post_ln_input, i2h_hid, h2o_hid, ln_weight, ln_bias,
            i2h_weight, i2h_bias, i2h_lowrank_first, i2h_lowrank_second, i2h_forward_indices, i2h_backward_indices,
            h2o_weight, h2o_bias, h2o_lowrank_first, h2o_lowrank_second, h2o_forward_indices, h2o_backward_indices,
            post_ln_weight, post_ln_bias)
        return y.view(*input.shape)

    @staticmethod
    def _describe(ctx, tokens, hidden, ln_weight, ln_bias, i2h_weight, i2h_bias, i2h_l1, i2h_l2, i2h_fwd, i2h_bwd,
                  h2o_weight, h2o_bias, h2o_l1, h2o_l2, h2o_fwd, h2o_bwd, post_ln_weight, post_ln_bias, io):
        """ctypes descriptor + the converted tensors it points into (which must outlive the call)"""
        act, gated, ln_eps, residual, cdt = ctx._cfg
        p, seed, offset = ctx._dropout
        keep = [_as(ln_weight, torch.float32), _as(ln_bias, torch.float32), _as(post_ln_weight, torch.float32),
                _as(post_ln_bias, torch.float32)]
        projections = []
        for w, b, l1, l2, fwd, bwd in ((i2h_weight, i2h_bias, i2h_l1, i2h_l2, i2h_fwd, i2h_bwd),
                                       (h2o_weight, h2o_bias, h2o_l1, h2o_l2, h2o_fwd, h2o_bwd)):
            tensors = (_as(w, cdt), _as(b, torch.float32), _as(l1, cdt), _as(l2, cdt),
                       None if fwd is None else fwd.to(torch.int32).contiguous(),
                       None if bwd is None else bwd.to(torch.int64).contiguous())
            keep.append(tensors)
            projections.append(linear_desc(*tensors))
        desc = nat.LtFfnDesc()
        desc.tokens, desc.hidden = tokens, hidden
        desc.intermediate = projections[1].in_features
        desc.gated, desc.act, desc.residual = int(gated), act, int(residual)
        desc.io_dtype, desc.compute_dtype = nat.dtype_code(io), nat.dtype_code(cdt)
        desc.ln_eps, desc.dropout_p, desc.dropout_seed, desc.dropout_offset = ln_eps, p, seed, offset
        desc.ln_weight, desc.ln_bias = nat.ptr(keep[0]), nat.ptr(keep[1])
        desc.post_ln_weight, desc.post_ln_bias = nat.ptr(keep[2]), nat.ptr(keep[3])
        desc.i2h, desc.h2o = projections
        return desc, keep

    @staticmethod
    def backward(ctx, grad_output):
        (input, pre_activation, ln_stats, post_ln_input, i2h_hid, h2o_hid, ln_weight, ln_bias,
         i2h_weight, i2h_bias, i2h_l1, i2h_l2, i2h_fwd, i2h_bwd,
         h2o_weight, h2o_bias, h2o_l1, h2o_l2, h2o_fwd, h2o_bwd, post_ln_weight, post_ln_bias) = ctx.saved_tensors
        cdt = ctx._cfg[4]
        device = input.device
        hidden = input.shape[-1]
        x = input.detach().reshape(-1, hidden).contiguous()
        tokens = x.shape[0]
        io = x.dtype
        dy = grad_output.detach().reshape(-1, hidden)
        if dy.dtype != io:
            dy = dy.to(io)
        dy = dy.contiguous()
        ln_w32, ln_b32, post_w32, post_b32, i2h_b32, h2o_b32 = ctx._small_fp32
        desc, keep = _LeanFFN._describe(
            ctx, tokens, hidden, ln_w32, ln_b32, i2h_weight, i2h_b32, i2h_l1, i2h_l2, i2h_fwd, i2h_bwd,
            h2o_weight, h2o_b32, h2o_l1, h2o_l2, h2o_fwd, h2o_bwd, post_w32, post_b32, io)
        need = ctx.needs_input_grad

        def new(like_shape, dtype, wanted):
            return torch.empty(like_shape, dtype=dtype, device=device) if wanted else None

        need_ln = need[1] or need[2]
        need_post = post_ln_weight is not None and (need[17] or need[18])
        dx = new(x.shape, io, need[0])
        # the kernels write the gradients of the small vectors in fp32: they share one buffer (256-byte aligned pieces) so
        # that a single conversion brings them to the parameters' dtype afterwards
        small_sizes = [hidden if need_ln else 0, hidden if need_ln else 0, hidden if need_post else 0,
                       hidden if need_post else 0, desc.i2h.out_features if i2h_bias is not None and need[4] else 0,
                       hidden if h2o_bias is not None and need[11] else 0]
        small_offsets, total = [], 0
        for n in small_sizes:
            small_offsets.append(total)
            total += -(-n // 64) * 64
        small = torch.empty(total, dtype=torch.float32, device=device)

        def piece(buffer, i):
            return buffer[small_offsets[i]:small_offsets[i] + small_sizes[i]] if small_sizes[i] else None

        d_ln_w, d_ln_b, d_post_w, d_post_b, d_i2h_b, d_h2o_b = (piece(small, i) for i in range(6))
        d_i2h_w = new(i2h_weight.shape, cdt, need[3])
        d_i2h_l1 = new(i2h_l1.shape, cdt, need[5]) if i2h_l1 is not None else None
        d_i2h_l2 = new(i2h_l2.shape, cdt, need[6]) if i2h_l2 is not None else None
        d_h2o_w = new(h2o_weight.shape, cdt, need[10])
        d_h2o_l1 = new(h2o_l1.shape, cdt, need[12]) if h2o_l1 is not None else None
        d_h2o_l2 = new(h2o_l2.shape, cdt, need[13]) if h2o_l2 is not None else None
        outputs = (dx, d_ln_w, d_ln_b, d_post_w, d_post_b, d_i2h_w, d_i2h_b, d_i2h_l1, d_i2h_l2, d_h2o_w, d_h2o_b,
                   d_h2o_l1, d_h2o_l2)
        if tokens > 0:
            grads = nat.LtFfnGrads()
            grads.dx, grads.ln_weight, grads.ln_bias = nat.ptr(dx), nat.ptr(d_ln_w), nat.ptr(d_ln_b)
            grads.post_ln_weight, grads.post_ln_bias = nat.ptr(d_post_w), nat.ptr(d_post_b)
            grads.i2h = nat.LtLinearGrads(nat.ptr(d_i2h_w), nat.ptr(d_i2h_b), nat.ptr(d_i2h_l1), nat.ptr(d_i2h_l2))
            grads.h2o = nat.LtLinearGrads(nat.ptr(d_h2o_w), nat.ptr(d_h2o_b), nat.ptr(d_h2o_l1), nat.ptr(d_h2o_l2))
            saved = nat.LtFfnSaved(nat.ptr(pre_activation), nat.ptr(ln_stats), nat.ptr(post_ln_input), nat.ptr(i2h_hid),
                                   nat.ptr(h2o_hid))
            lib = nat.lib()
            ws = nat.workspace(lib.lt_ffn_backward_workspace_bytes(desc), device)
            nat.check(lib.lt_ffn_backward(desc, nat.ptr(x), nat.ptr(dy), saved, grads, nat.ptr(ws), ws.numel(),
                                          nat.current_stream(device)), "lt_ffn_backward")
            del ws, keep
        else:
            for g in outputs[1:]:
                if g is not None:
                    g.zero_()
        small_params = (ln_weight, ln_bias, post_ln_weight, post_ln_bias, i2h_bias, h2o_bias)
        wanted = {t.dtype for t, n in zip(small_params, small_sizes) if n}
        if len(wanted) == 1 and wanted != {torch.float32} and total:
            converted = small.to(wanted.pop())
            d_ln_w, d_ln_b, d_post_w, d_post_b, d_i2h_b, d_h2o_b = (piece(converted, i) for i in range(6))
        grad_input = None if dx is None else dx.view(*input.shape)
        return (grad_input, d_ln_w if need[1] else None, d_ln_b if need[2] else None,
                d_i2h_w, d_i2h_b, d_i2h_l1, d_i2h_l2, None, None, None,
                d_h2o_w, d_h2o_b, d_h2o_l1, d_h2o_l2, None, None, None,
                d_post_w if need_post and need[17] else None, d_post_b if need_post and need[18] else None,
                None, None, None, None, None, None)
