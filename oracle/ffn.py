"""CPU oracle (test infrastructure only): the LeanFFN forward / backward in stock PyTorch.

Two restatements of lean_transformer/ffn.py:

  * ``plain_ffn``        every step a library routine, differentiated by autograd.  This is the ground truth the
                         reference's own tests compare ``_LeanFFN`` with (tests/test_ffn.py:89-147 "ReferenceFFN").
  * ``LeanFFNFunction``  an autograd.Function with the reference's save-set (input, pre-activation, LN parameters and the
                         linear layers' small tensors; ffn.py:210-216) and a closed-form backward that re-materialises the
                         LayerNorm output and the activation (ffn.py:233-306).  This one is timed as the CPU baseline.

Dropout takes an explicit keep-mask so that a device kernel's counter-based mask can be handed in.
"""
from dataclasses import dataclass, field
from typing import Optional

import torch
import torch.nn.functional as F

from . import blocksparse as bs

SQRT_2_OVER_PI = 0.79788456  # reference constant, utils.py:30
GELU_CUBIC = 0.044715


def gelu_fused(x: torch.Tensor) -> torch.Tensor:
    """reference: gelu_fused, utils.py:24-30 (tanh approximation)."""
    return x * 0.5 * (1.0 + torch.tanh(SQRT_2_OVER_PI * x * (1 + GELU_CUBIC * x * x)))


def gelu_fused_grad(grad_output: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """reference: gelu_fused_grad, utils.py:33-38.  0.1070322243 = 3 * 0.044715 * 0.79788456."""
    t = torch.tanh(SQRT_2_OVER_PI * x * (1 + GELU_CUBIC * x * x))
    jac = 0.5 * x * ((1 - t * t) * (SQRT_2_OVER_PI + 0.1070322243 * x * x)) + 0.5 * (1 + t)
    return jac * grad_output


# The closed-form entries of transformers.activations.ACT2FN (the table the reference extends at utils.py:80; transformers
# is a third-party dependency of the reference, not part of its checkout).  Restated from the published definitions of each
# function; tests/test_oracle.py pins every value against the installed transformers table and every derivative against
# fp64 autograd of the value.
LAPLACE_MU, LAPLACE_SIGMA = 0.707107, 0.282095
ACT_NAMES = ("gelu_fused", "gelu", "relu", "silu", "quick_gelu", "gelu_10", "relu6", "relu2", "leaky_relu", "mish", "sigmoid",
             "tanh", "linear", "hardswish", "laplace", "sqrtsoftplus")


def act_forward(kind: str, x: torch.Tensor) -> torch.Tensor:
    if kind == "gelu_fused":
        return gelu_fused(x)
    if kind == "gelu":
        return F.gelu(x)
    if kind == "relu":
        return F.relu(x)
    if kind == "silu":
        return F.silu(x)
    if kind == "quick_gelu":
        return x * torch.sigmoid(1.702 * x)
    if kind == "gelu_10":
        return torch.clip(F.gelu(x), -10, 10)
    if kind == "relu6":
        return F.relu6(x)  # (autograd of relu6 is 0 at both kinks; of clamp(x, 0, 6) it would be 1)
    if kind == "relu2":
        return torch.square(F.relu(x))
    if kind == "leaky_relu":
        return torch.where(x > 0, x, 0.01 * x)
    if kind == "mish":
        return x * torch.tanh(F.softplus(x))
    if kind == "sigmoid":
        return torch.sigmoid(x)
    if kind == "tanh":
        return torch.tanh(x)
    if kind == "linear":
        return x
    if kind == "hardswish":
        return x * torch.clamp(x + 3, 0, 6) / 6
    if kind == "laplace":
        return 0.5 * (1.0 + torch.erf((x - LAPLACE_MU) / (LAPLACE_SIGMA * 2.0 ** 0.5)))
    if kind == "sqrtsoftplus":
        return torch.sqrt(F.softplus(x))
    raise ValueError(kind)


def act_derivative(kind: str, x: torch.Tensor) -> torch.Tensor:
    """d act(x) / dx, element-wise, written out by hand (at a kink: the one-sided value autograd takes)"""
    one, zero = torch.ones_like(x), torch.zeros_like(x)
    if kind == "gelu_fused":
        return gelu_fused_grad(one, x)
    if kind in ("gelu", "gelu_10"):
        cdf = 0.5 * (1 + torch.erf(x * 0.7071067811865476))
        pdf = torch.exp(-0.5 * x * x) * 0.3989422804014327
        jac = cdf + x * pdf
        if kind == "gelu_10":  # the clip passes gradients where its input lies inside [-10, 10]
            g = x * cdf
            jac = torch.where((g >= -10) & (g <= 10), jac, zero)
        return jac
    if kind == "relu":
        return (x > 0).to(x.dtype)
    if kind == "silu":
        s = torch.sigmoid(x)
        return s * (1 + x * (1 - s))
    if kind == "quick_gelu":
        s = torch.sigmoid(1.702 * x)
        return s + 1.702 * x * s * (1 - s)
    if kind == "relu6":
        return ((x > 0) & (x < 6)).to(x.dtype)
    if kind == "relu2":
        return 2 * F.relu(x)
    if kind == "leaky_relu":
        return torch.where(x > 0, one, 0.01 * one)
    if kind == "mish":
        t = torch.tanh(F.softplus(x))
        return t + x * (1 - t * t) * torch.sigmoid(x)
    if kind == "sigmoid":
        s = torch.sigmoid(x)
        return s * (1 - s)
    if kind == "tanh":
        t = torch.tanh(x)
        return 1 - t * t
    if kind == "linear":
        return one
    if kind == "hardswish":
        return torch.where(x < -3, zero, torch.where(x <= 3, x / 3 + 0.5, one))
    if kind == "laplace":
        scale = LAPLACE_SIGMA * 2.0 ** 0.5
        z = (x - LAPLACE_MU) / scale
        return torch.exp(-z * z) / (scale * 3.141592653589793 ** 0.5)
    if kind == "sqrtsoftplus":
        return torch.sigmoid(x) / (2 * torch.sqrt(F.softplus(x)))
    raise ValueError(kind)


def act_backward(kind: str, grad: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    return grad * act_derivative(kind, x)


@dataclass
class LinearParams:
    """One projection in the reference's "generalized linear" form (linear.py:161-230): dense or native block-sparse main
    weight, optional bias, optional low-rank pair (first [r, in], second [out, r])."""
    weight: torch.Tensor
    bias: Optional[torch.Tensor] = None
    lowrank_first: Optional[torch.Tensor] = None
    lowrank_second: Optional[torch.Tensor] = None
    forward_indices: Optional[torch.Tensor] = None
    backward_indices: Optional[torch.Tensor] = None
    out_features: int = 0

    def tensors(self):
        return [t for t in (self.weight, self.bias, self.lowrank_first, self.lowrank_second) if t is not None]

    def dense_weight(self) -> torch.Tensor:
        if self.backward_indices is None:
            return self.weight
        # differentiable dense expansion of the sparse weight (used by plain_ffn only)
        in_features, A, b = self.weight.shape
        n_in = in_features // b
        w4 = self.weight.reshape(n_in, A, b, b)
        rows = []
        bwd = self.backward_indices.tolist()
        n_out = self.out_features // b
        blocks = [[None] * n_in for _ in range(n_out)]
        for ib in range(n_in):
            for a in range(A):
                blocks[bwd[ib][a]][ib] = w4[ib, a]
        zero = torch.zeros(b, b, dtype=self.weight.dtype, device=self.weight.device)
        for ob in range(n_out):
            rows.append(torch.cat([blk if blk is not None else zero for blk in blocks[ob]], dim=1))
        return torch.cat(rows, dim=0)


def linear_forward(x2d: torch.Tensor, lin: LinearParams) -> torch.Tensor:
    """main matmul + bias + low-rank term; reference: _forward_jit, linear.py:197-230."""
    out = F.linear(x2d, lin.dense_weight(), lin.bias)
    if lin.lowrank_first is not None:
        out = out + F.linear(F.linear(x2d, lin.lowrank_first), lin.lowrank_second)
    return out


@dataclass
class FFNConfig:
    gated: bool = False
    act: str = "gelu_fused"
    ln_eps: float = 1e-12
    residual: bool = True
    dropout: float = 0.0  # probability; the mask is passed separately
    # Round the LayerNorm output, the pre-activation and the activation output to bfloat16 (straight-through for autograd):
    # the three places where the reference stores a bf16 tensor under torch.autocast(bfloat16) -- layer_norm runs in fp32 and
    # its result is cast at the linear's input, the linear's output P is bf16, the activation's output is bf16 (ffn.py:184-191
    # under autocast).  Off: everything in the dtype of the inputs.  Needed to compare a bf16 run where the activation's
    # derivative jumps (relu): there the derivative depends on the sign of the *stored* P, not of its exact value.
    bf16_rounding: bool = False


@dataclass
class FFNParams:
    ln_weight: torch.Tensor
    ln_bias: torch.Tensor
    i2h: LinearParams
    h2o: LinearParams
    post_ln_weight: Optional[torch.Tensor] = None
    post_ln_bias: Optional[torch.Tensor] = None
    cfg: FFNConfig = field(default_factory=FFNConfig)

    def tensors(self):
        out = [self.ln_weight, self.ln_bias, *self.i2h.tensors(), *self.h2o.tensors()]
        if self.post_ln_weight is not None:
            out += [self.post_ln_weight, self.post_ln_bias]
        return out


def round_bf16_straight_through(t: torch.Tensor) -> torch.Tensor:
    """value of t rounded to bfloat16 (round-to-nearest-even, as a cast does), gradient of the identity"""
    return t + (t.to(torch.bfloat16).to(t.dtype) - t).detach()


def apply_activation(pre_activation: torch.Tensor, act: str, gated: bool) -> torch.Tensor:
    """reference: _LeanFFN._apply_activation, ffn.py:138-144 -- the FIRST half of the features is the gate."""
    if not gated:
        return act_forward(act, pre_activation)
    gate, lin = pre_activation.split(pre_activation.shape[-1] // 2, dim=-1)
    return act_forward(act, gate) * lin


def plain_ffn(x: torch.Tensor, p: FFNParams, keep_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """LN -> up-projection -> (gated) activation -> down-projection -> [post-LN] -> dropout -> [+ residual].

    reference: _LeanFFN.forward, ffn.py:182-207 (same order as LeanFFN._forward_pytorch, ffn.py:69-85).
    ``keep_mask`` (bool, shape of x flattened to 2-D) selects kept outputs; kept values are scaled by 1/(1-dropout).
    """
    cfg = p.cfg
    x2d = x.reshape(-1, x.shape[-1])
    rnd = round_bf16_straight_through if cfg.bf16_rounding else (lambda t: t)
    u = rnd(F.layer_norm(x2d, x2d.shape[-1:], p.ln_weight, p.ln_bias, cfg.ln_eps))
    pre = rnd(linear_forward(u, p.i2h))
    h = rnd(apply_activation(pre, cfg.act, cfg.gated))
    out = linear_forward(h, p.h2o)
    if p.post_ln_weight is not None:
        out = F.layer_norm(out, out.shape[-1:], p.post_ln_weight, p.post_ln_bias, cfg.ln_eps)
    if keep_mask is not None and cfg.dropout > 0:
        out = out * keep_mask.reshape(out.shape).to(out.dtype) / (1.0 - cfg.dropout)
    if cfg.residual:
        out = out + x2d
    return out.reshape(x.shape)


def layer_norm_backward(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float):
    """Closed-form LayerNorm backward (biased variance, eps inside the root): returns (dx, dweight, dbias)."""
    mean = x.mean(-1, keepdim=True)
    rstd = torch.rsqrt(x.var(-1, unbiased=False, keepdim=True) + eps)
    xhat = (x - mean) * rstd
    dxhat = dy * weight
    dx = rstd * (dxhat - dxhat.mean(-1, keepdim=True) - xhat * (dxhat * xhat).mean(-1, keepdim=True))
    return dx, (dy * xhat).sum(0), dy.sum(0)


def _linear_backward(dy: torch.Tensor, x: torch.Tensor, lowrank_hid: Optional[torch.Tensor], lin: LinearParams):
    """(dx, dweight, dbias, dlowrank_first, dlowrank_second); reference: _backward_jit, linear.py:262-328."""
    d_first = d_second = d_bias = None
    if lin.bias is not None:
        d_bias = dy.sum(0)
    if lin.backward_indices is None:
        d_weight = dy.t() @ x
        dx = dy @ lin.weight
    else:
        dx, d_weight = bs.blocksparse_matmul_backward(dy, x, lin.weight, lin.backward_indices.numpy())
    if lin.lowrank_first is not None:
        g_hid = dy @ lin.lowrank_second
        d_second = dy.t() @ lowrank_hid
        d_first = g_hid.t() @ x
        dx = dx + g_hid @ lin.lowrank_first
    return dx, d_weight, d_bias, d_first, d_second


class LeanFFNFunction(torch.autograd.Function):
    """Memory-lean FFN: saves x and the pre-activation only, recomputes LayerNorm and activation in backward.

    Argument order: x, keep_mask, params (FFNParams, non-tensor), then every parameter tensor in ``params.tensors()`` order so
    that autograd routes their gradients.
    """

    # custom_fwd / custom_bwd as on the reference's _LeanFFN (ffn.py:146-147,232-233): backward runs under the autocast state
    # of the forward, so that under torch.autocast(bfloat16) its matmuls take bf16 operands as the forward's did
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, x, keep_mask, params: FFNParams, *param_tensors):
        cfg = params.cfg
        x2d = x.reshape(-1, x.shape[-1])
        u = F.layer_norm(x2d, x2d.shape[-1:], params.ln_weight, params.ln_bias, cfg.ln_eps)
        pre = linear_forward(u, params.i2h)
        i2h_hid = F.linear(u, params.i2h.lowrank_first) if params.i2h.lowrank_first is not None else None
        h = apply_activation(pre, cfg.act, cfg.gated)
        out = linear_forward(h, params.h2o)
        h2o_hid = F.linear(h, params.h2o.lowrank_first) if params.h2o.lowrank_first is not None else None
        post_ln_input = None
        if params.post_ln_weight is not None:
            post_ln_input = out
            out = F.layer_norm(out, out.shape[-1:], params.post_ln_weight, params.post_ln_bias, cfg.ln_eps)
        if keep_mask is not None and cfg.dropout > 0:
            out = out * keep_mask.reshape(out.shape).to(out.dtype) / (1.0 - cfg.dropout)
        if cfg.residual:
            out = out + x2d
        ctx.params = params
        ctx.save_for_backward(x, pre, keep_mask, post_ln_input, i2h_hid, h2o_hid)
        return out.reshape(x.shape)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        params: FFNParams = ctx.params
        cfg = params.cfg
        x, pre, keep_mask, post_ln_input, i2h_hid, h2o_hid = ctx.saved_tensors
        x2d = x.reshape(-1, x.shape[-1])
        dy = grad_output.reshape(x2d.shape)
        g = dy
        if keep_mask is not None and cfg.dropout > 0:
            g = g * keep_mask.reshape(g.shape).to(g.dtype) / (1.0 - cfg.dropout)
        d_post_w = d_post_b = None
        if post_ln_input is not None:
            g, d_post_w, d_post_b = layer_norm_backward(g, post_ln_input, params.post_ln_weight, cfg.ln_eps)
        # re-materialise the activation, then backward through the down-projection
        h = apply_activation(pre, cfg.act, cfg.gated)
        d_h, d_w2, d_b2, d_h2o_first, d_h2o_second = _linear_backward(g, h, h2o_hid, params.h2o)
        del h
        if cfg.gated:
            gate, lin = pre.split(pre.shape[-1] // 2, dim=-1)
            d_pre = torch.cat([act_backward(cfg.act, d_h * lin, gate), d_h * act_forward(cfg.act, gate)], dim=-1)
        else:
            d_pre = act_backward(cfg.act, d_h, pre)
        # re-materialise LayerNorm, then backward through the up-projection
        u = F.layer_norm(x2d, x2d.shape[-1:], params.ln_weight, params.ln_bias, cfg.ln_eps)
        d_u, d_w1, d_b1, d_i2h_first, d_i2h_second = _linear_backward(d_pre, u, i2h_hid, params.i2h)
        del u
        dx, d_ln_w, d_ln_b = layer_norm_backward(d_u, x2d, params.ln_weight, cfg.ln_eps)
        if cfg.residual:
            dx = dx + dy
        grads = [d_ln_w, d_ln_b, d_w1]
        for present, grad in ((params.i2h.bias, d_b1), (params.i2h.lowrank_first, d_i2h_first),
                              (params.i2h.lowrank_second, d_i2h_second)):
            if present is not None:
                grads.append(grad)
        grads.append(d_w2)
        for present, grad in ((params.h2o.bias, d_b2), (params.h2o.lowrank_first, d_h2o_first),
                              (params.h2o.lowrank_second, d_h2o_second)):
            if present is not None:
                grads.append(grad)
        if params.post_ln_weight is not None:
            grads += [d_post_w, d_post_b]
        return (dx.reshape(x.shape), None, None, *grads)


def lean_ffn(x: torch.Tensor, p: FFNParams, keep_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    return LeanFFNFunction.apply(x, keep_mask, p, *p.tensors())


def make_dense_params(hidden: int, intermediate: int, *, gated: bool, std: float = 0.02, generator=None,
                      dtype=torch.float32, **cfg) -> FFNParams:
    """Synthetic dense parameters: weights ~ N(0, std), biases 0, LN weight 1 / bias 0; draws W1 then W2."""
    n1 = 2 * intermediate if gated else intermediate
    w1 = torch.randn(n1, hidden, generator=generator, dtype=dtype) * std
    w2 = torch.randn(hidden, intermediate, generator=generator, dtype=dtype) * std
    return FFNParams(
        ln_weight=torch.ones(hidden, dtype=dtype), ln_bias=torch.zeros(hidden, dtype=dtype),
        i2h=LinearParams(w1, torch.zeros(n1, dtype=dtype), out_features=n1),
        h2o=LinearParams(w2, torch.zeros(hidden, dtype=dtype), out_features=hidden),
        cfg=FFNConfig(gated=gated, **cfg))
