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
    """Pre-LayerNorm feed-forward block  y = [x +] dropout([postLN](act(LN(x) W1^T + b1) W2^T + b2))  whose backward keeps
    only x and the pre-activation alive and rebuilds everything else inside the HIP kernels.

    The constructor, the attribute names and the parameter names follow lean_transformer/ffn.py:35-64 so that models and
    checkpoints written for that class work with this one.

    hidden_size        width of the residual stream (input and output)
    intermediate_size  width of the activation; the first projection is twice as wide when ``gated``
    activation         element-wise nonlinearity; on the kernel path it must be one that ``utils.activation_kind`` knows
    gated              GLU variant: the first half of the up-projection passes through ``activation`` and multiplies the
                       second half (arXiv:2002.05202); costs 1.5x the parameters of the plain block
    layer_norm_eps     epsilon of both LayerNorms
    dropout            drop probability on the block's output, before the residual is added; training mode only
    post_layer_norm    second LayerNorm right after the down-projection (CogView / NormFormer style)
    i2h_proj, h2o_proj projections to use instead of fresh ``nn.Linear`` layers (hidden -> intermediate[*2] and
                       intermediate -> hidden); the kernel path takes ``nn.Linear`` and ``GeneralizedLinear`` exactly
    residual           add the input to the output
    ffn_custom_grad    True: one fused library call forward and one backward (memory-lean).  False: the same maths as a
                       chain of stock PyTorch ops differentiated by autograd.  May be flipped at any time.
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
        up_width = 2 * intermediate_size if gated else intermediate_size
        self.i2h_proj = i2h_proj if i2h_proj is not None else nn.Linear(hidden_size, up_width)
        self.h2o_proj = h2o_proj if h2o_proj is not None else nn.Linear(intermediate_size, hidden_size)
        for name, proj, fan_in, fan_out in (("i2h_proj", self.i2h_proj, hidden_size, up_width),
                                            ("h2o_proj", self.h2o_proj, intermediate_size, hidden_size)):
            if ffn_custom_grad and type(proj) not in (nn.Linear, GeneralizedLinear):
                raise AssertionError(f"{name} is a {type(proj).__name__}: the fused path runs nn.Linear and GeneralizedLinear "
                                     "projections only (pass ffn_custom_grad=False for other layer types)")
            if (proj.in_features, proj.out_features) != (fan_in, fan_out):
                raise AssertionError(f"{name} maps {proj.in_features} -> {proj.out_features} features, "
                                     f"this block needs {fan_in} -> {fan_out}")
        self.pre_layer_norm = nn.LayerNorm(hidden_size, eps=layer_norm_eps)
        self.post_layer_norm = nn.LayerNorm(hidden_size, eps=layer_norm_eps) if post_layer_norm else None
        self.activation, self.gated = activation, gated
        self.dropout, self.residual = dropout, residual
        self.ffn_custom_grad = ffn_custom_grad

    def forward(self, input):
        if self.ffn_custom_grad:
            return self._forward_custom(input)
        return self._forward_pytorch(input)

    def _forward_pytorch(self, input):
        """The block as stock PyTorch ops under autograd (lean_transformer/ffn.py:69-85).  On a GPU the dropout mask is
        the Philox stream the fused path would draw from the same generator state, so both settings of ``ffn_custom_grad``
        drop the same elements under one seed."""
        width = input.shape[-1]
        rows = input.view(-1, width)
        ln = self.pre_layer_norm
        normed = F.layer_norm(rows, (width,), ln.weight, ln.bias, ln.eps)
        hidden_act = _LeanFFN._apply_activation(self.i2h_proj(normed), self.activation, gated=self.gated)
        out = self.h2o_proj(hidden_act)
        if self.post_layer_norm is not None:
            out = self.post_layer_norm(out)
        if self.training and self.dropout:
            if float(self.dropout) >= 1.0:
                out = torch.zeros_like(out)  # what torch.dropout returns for p = 1 (no 1 / (1 - p) to form)
            elif out.is_cuda and nat.available():
                keep = philox_keep_mask(out.shape[0], width, float(self.dropout), out.device)
                out = out * (keep.to(out.dtype) * (1.0 / (1.0 - float(self.dropout))))
            else:  # CPU tensors, or no built library: the stock op, as at lean_transformer/ffn.py:80
                out = torch.dropout(out, self.dropout, True)
        if self.residual:
            out = out + rows
        return out.view(*input.shape)

    @staticmethod
    def _projection_extras(proj):
        """(lowrank_first, lowrank_second, forward_indices, backward_indices, matmul_op) of a projection; a plain
        ``nn.Linear`` has none of them"""
        if not isinstance(proj, GeneralizedLinear):
            return None, None, None, None, None
        first, second = proj.get_combined_lowrank_components()
        return first, second, proj.matrix.forward_indices, proj.matrix.backward_indices, proj.matrix.matmul_op

    def _forward_custom(self, input):
        """Flattens the module state into the 25 positional arguments of ``_LeanFFN.apply`` (order of
        lean_transformer/ffn.py:105-131)."""
        post = self.post_layer_norm
        return _LeanFFN.apply(
            input, self.pre_layer_norm.weight, self.pre_layer_norm.bias,
            self.i2h_proj.weight, self.i2h_proj.bias, *self._projection_extras(self.i2h_proj),
            self.h2o_proj.weight, self.h2o_proj.bias, *self._projection_extras(self.h2o_proj),
            None if post is None else post.weight, None if post is None else post.bias,
            self.activation, self.gated, self.dropout, self.training, self.pre_layer_norm.eps, self.residual)


def _draw_dropout_stream(device: torch.device, numel: int):
    """(seed, offset) of a fresh Philox sub-stream of the device's default generator, advancing it like a dropout op would.
    Goes through the generator state only (no device sync), so seeding / checkpoint replay of the RNG state reproduce it."""
    gen = torch.cuda.default_generators[device.index if device.index is not None else torch.cuda.current_device()]
    seed, offset = gen.initial_seed(), gen.get_offset()
    gen.set_offset(offset + 4 * math.ceil(numel / 4))
    return seed, offset


def philox_keep_mask(tokens: int, hidden: int, p: float, device: torch.device) -> torch.Tensor:
    """uint8 keep-mask [tokens, hidden] of the next dropout sub-stream of ``device``'s generator (which it advances): the
    elements the fused forward epilogue would keep had it drawn that sub-stream"""
    seed, offset = _draw_dropout_stream(device, tokens * hidden)
    keep = torch.empty(tokens, hidden, dtype=torch.uint8, device=device)
    if tokens > 0:
        nat.check(nat.lib().lt_dropout_mask(tokens, hidden, p, seed, offset, nat.ptr(keep), nat.current_stream(device)),
                  "lt_dropout_mask")
    return keep


class _LeanFFN(torch.autograd.Function):
    """Autograd function for transformer FFN: one library call forward, one backward."""

    @staticmethod
    def _apply_activation(pre_activation: torch.Tensor, activation: callable, gated: bool):
        """stock-op activation of the up-projection's output; gated: act(first half) * second half (ffn.py:138-144)"""
        if gated:
            gate, linear = pre_activation.chunk(2, dim=-1)
            return activation(gate) * linear
        return activation(pre_activation)

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
        if io not in (torch.float32, torch.bfloat16, torch.float16) or (io != torch.float32 and cdt != io):
            raise TypeError(f"LeanFFN: input dtype {io} with compute dtype {cdt} is not supported (float32 input with "
                            "float32/bfloat16/float16 weights, or bfloat16/float16 input with weights of the same dtype)")
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
        # fp32 copies of the small vectors (LayerNorm parameters, biases): backward reuses them instead of converting again.
        # The parameters themselves go through save_for_backward below, so an in-place update between forward and backward
        # makes ctx.saved_tensors raise (autograd's version check) before these copies could be used stale.
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
            lib = nat.lib(cdt)
            ws = nat.workspace(lib.lt_ffn_forward_workspace_bytes(desc), device)
            nat.check(lib.lt_ffn_forward(desc, nat.ptr(x), nat.ptr(y), saved, nat.ptr(ws), ws.numel(),
                                         nat.current_stream(device)), "lt_ffn_forward", lib)
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
            projections.append(linear_desc(*tensors, index_owner=fwd, backward_owner=bwd))
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
            lib = nat.lib(cdt)
            ws = nat.workspace(lib.lt_ffn_backward_workspace_bytes(desc), device)
            nat.check(lib.lt_ffn_backward(desc, nat.ptr(x), nat.ptr(dy), saved, grads, nat.ptr(ws), ws.numel(),
                                          nat.current_stream(device)), "lt_ffn_backward", lib)
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
