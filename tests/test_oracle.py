"""Pins the CPU oracle (oracle/) against the reference's golden vectors, its tests' known answers, and what the mathematics
fixes.  No GPU, no reference checkout needed (tests/golden/*.npz was written from the reference by make_golden.py)."""
import ast
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import blocksparse as obs
from oracle import ffn as offn

GOLDEN = np.load(os.path.join(os.path.dirname(__file__), "golden", "blocksparse_golden.npz"))
CASES = [str(n) for n in GOLDEN["names"]]


def _layout_from_desc(name):
    out_f, in_f, _ = (int(v) for v in GOLDEN[f"{name}/shape"])
    call = ast.parse(str(GOLDEN[f"{name}/desc"])).body[0].value
    args = [ast.literal_eval(a) for a in call.args]
    kwargs = {k.arg: ast.literal_eval(k.value) for k in call.keywords}
    fn = {"pixelfly": obs.pixelfly_layout, "hypercube": obs.hypercube_layout}[call.func.id]
    return fn(out_f, in_f, *args, **kwargs)


@pytest.mark.parametrize("name", CASES)
def test_layout_and_indices_match_reference_golden(name):
    layout = _layout_from_desc(name)
    assert np.array_equal(layout, GOLDEN[f"{name}/layout"])
    fwd, bwd = obs.indices_from_layout(layout)
    assert fwd.dtype == np.int32 and bwd.dtype == np.int64
    assert np.array_equal(fwd, GOLDEN[f"{name}/forward_indices"])
    assert np.array_equal(bwd, GOLDEN[f"{name}/backward_indices"])
    # invariant the reference asserts in tests/test_butterfly.py:33
    assert fwd.max() == fwd.shape[1] * layout.shape[0] - 1


@pytest.mark.parametrize("name", CASES)
def test_blocksparse_matmul_matches_reference_golden(name):
    x, w, dy = (torch.from_numpy(GOLDEN[f"{name}/{k}"]) for k in ("x", "w", "dy"))
    fwd, bwd = GOLDEN[f"{name}/forward_indices"], GOLDEN[f"{name}/backward_indices"]
    y = obs.blocksparse_matmul(x, w, fwd)
    dx, dw = obs.blocksparse_matmul_backward(dy, x, w, bwd)
    for got, key in ((y, "y"), (dx, "dx"), (dw, "dw")):
        assert torch.allclose(got, torch.from_numpy(GOLDEN[f"{name}/{key}"]), rtol=1e-4, atol=1e-5), key
    # the dense expansion is the same linear map
    dense = obs.sparse_to_dense(w, bwd, int(GOLDEN[f"{name}/shape"][0]))
    assert torch.allclose(x @ dense.t(), y, rtol=1e-4, atol=1e-5)


def test_blocksparse_brute_force_tiny():
    """triple loop over (token, output element, input element) on a 8 x 8 matrix of 2 x 2 blocks"""
    layout = obs.pixelfly_layout(8, 8, block_size=2)
    fwd, bwd = obs.indices_from_layout(layout)
    g = torch.Generator().manual_seed(5)
    A = bwd.shape[1]
    w = torch.randn(8, A, 2, generator=g)
    x = torch.randn(3, 8, generator=g)
    w4 = w.reshape(4, A, 2, 2)
    ref = torch.zeros(3, 8)
    for t in range(3):
        for ib in range(4):
            for a in range(A):
                ob = int(bwd[ib, a])
                for r in range(2):
                    for c in range(2):
                        ref[t, ob * 2 + r] += w4[ib, a, r, c] * x[t, ib * 2 + c]
    assert torch.allclose(obs.blocksparse_matmul(x, w, fwd), ref, atol=1e-6)


def test_blocksparse_backward_is_autograd_of_forward():
    """what reference tests/test_butterfly.py:114-142 asserts of the reference, on a smaller non-square tiled layout"""
    layout = obs.pixelfly_layout(96 * 8, 96 * 2, block_size=96)
    fwd, bwd = obs.indices_from_layout(layout)
    g = torch.Generator().manual_seed(42)
    x = torch.randn(3, 2, 96 * 2, generator=g, requires_grad=True)
    w = torch.randn(96 * 2, bwd.shape[1], 96, generator=g, requires_grad=True)
    dy = torch.randn(3, 2, 96 * 8, generator=g)
    dense = offn.LinearParams(w, backward_indices=torch.from_numpy(bwd), out_features=96 * 8).dense_weight()
    (x.reshape(-1, 96 * 2) @ dense.t()).backward(dy.reshape(-1, 96 * 8))
    dx, dw = obs.blocksparse_matmul_backward(dy, x.detach(), w.detach(), bwd)
    assert torch.allclose(dx, x.grad, rtol=1e-4, atol=1e-4)
    assert torch.allclose(dw, w.grad, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("desc,density", [
    # known answers of reference tests/test_layout.py:10-13, measured there over every GeneralizedLinear of a hidden-32
    # model (32x32, 96x32, 128x32 and 32x128 matrices): each of those shapes has the stated density
    (dict(block_size=4), 0.5), (dict(block_size=2), 0.3125), (dict(block_size=2, stretch=True), 0.3125)])
def test_pixelfly_density_known_answers(desc, density):
    for out_f, in_f in ((32, 32), (96, 32), (128, 32), (32, 128)):
        assert np.isclose(obs.pixelfly_layout(out_f, in_f, **desc).mean(), density), (out_f, in_f)


def test_hypercube_density_known_answers():
    assert np.isclose(obs.hypercube_layout(32, 32, 2, folded=False).mean(), 0.3125)
    assert np.isclose(obs.hypercube_layout(32, 32, 2, folded=True).mean(), 0.375)


def test_butterfly_mask_is_sum_of_factor_matrices():
    """brute force: factor k of a size-n butterfly is block-diagonal with 2^(k+1)-sized blocks [[D, D], [D, D]]"""
    n = 16
    total = np.zeros((n, n), dtype=bool)
    for k in range(4):
        stride = 1 << k
        fac = np.zeros((n, n), dtype=bool)
        for i in range(n):
            fac[i, i] = True
            fac[i, i ^ stride] = True
        total |= fac
    assert np.array_equal(obs.butterfly_mask(n, 4), total)
    assert obs.butterfly_mask(n, 4).sum(1).tolist() == [5] * n


def test_gelu_fused_close_to_erf_gelu():
    """reference tests/test_utils.py:25-29"""
    x = torch.linspace(-5, 5, 1000)
    assert (offn.gelu_fused(x) - F.gelu(x)).abs().max().item() <= 5e-4


@pytest.mark.parametrize("kind", offn.ACT_NAMES)
def test_activation_grad_is_autograd_of_forward(kind):
    # an even count of points over (-12, 12) misses the kinks at 0, +-3 and 6; gelu_10's clip at gelu(x) = 10 lies inside
    x = torch.linspace(-12, 12, 4001, dtype=torch.float64)[1:-1:2].clone().requires_grad_(True)
    g = torch.randn(x.shape, dtype=torch.float64, generator=torch.Generator().manual_seed(0))
    (auto,) = torch.autograd.grad(offn.act_forward(kind, x), x, g)
    assert torch.allclose(offn.act_backward(kind, g, x.detach()), auto, rtol=1e-6, atol=1e-7)
    if kind == "gelu_10":
        assert (offn.act_derivative(kind, x.detach())[x.detach() > 10.5] == 0).all()  # the clip is exercised


HF_NAMES = {  # entry of transformers.activations.ACT2FN -> the oracle's (and the kernels') activation
    "gelu": "gelu", "gelu_python": "gelu", "gelu_new": "gelu_fused", "gelu_fast": "gelu_fused", "gelu_pytorch_tanh": "gelu_fused",
    "gelu_python_tanh": "gelu_fused", "gelu_accurate": "gelu_fused", "relu": "relu", "silu": "silu", "swish": "silu",
    "quick_gelu": "quick_gelu", "gelu_10": "gelu_10", "relu6": "relu6", "relu2": "relu2", "leaky_relu": "leaky_relu",
    "mish": "mish", "sigmoid": "sigmoid", "tanh": "tanh", "linear": "linear", "hardswish": "hardswish", "laplace": "laplace",
    "sqrtsoftplus": "sqrtsoftplus"}


@pytest.mark.parametrize("name", sorted(HF_NAMES))
def test_activation_values_match_the_huggingface_table(name):
    """The reference's ACT2FN is transformers' table plus gelu_fused (utils.py:80): every closed-form entry the installed
    transformers has must equal the oracle's restatement (the tanh-form GELUs up to the digits of sqrt(2 / pi) the reference
    truncates: 3e-10), and the package's own table must name the same kernel-side activation for it."""
    hf = pytest.importorskip("transformers.activations").ACT2FN
    if name not in hf:
        pytest.skip(f"this transformers has no {name}")
    from lean_transformer_amd.utils import ACT2FN, activation_kind
    kind = HF_NAMES[name]
    x = torch.linspace(-12, 12, 4001, dtype=torch.float64)
    assert (offn.act_forward(kind, x) - hf[name](x)).abs().max().item() <= (1e-9 if kind == "gelu_fused" else 1e-14)
    assert activation_kind(hf[name]) == kind and activation_kind(ACT2FN[name]) == kind
    assert (ACT2FN[name](x) - hf[name](x)).abs().max().item() <= 1e-9


def test_activations_with_learned_parameters_are_refused():
    hf = pytest.importorskip("transformers.activations").ACT2FN
    from lean_transformer_amd.utils import activation_kind
    for name in ("prelu", "xielu"):
        if name in hf:
            with pytest.raises(NotImplementedError):
                activation_kind(hf[name])
    with pytest.raises(NotImplementedError):
        activation_kind(torch.nn.LeakyReLU(0.2))  # only the table's slope, 0.01, has a kernel
    with pytest.raises(NotImplementedError):
        activation_kind(lambda x: x * x)


def _random_params(hidden, inter, gated, post_ln, lowrank, sparse, dtype, seed, **cfg):
    g = torch.Generator().manual_seed(seed)
    n1 = 2 * inter if gated else inter

    def rnd(*shape, std=0.3):
        return (torch.randn(*shape, generator=g, dtype=torch.float64) * std).to(dtype)

    def lin(in_f, out_f):
        kw = {}
        if sparse:
            lay = obs.pixelfly_layout(out_f, in_f, block_size=4)
            fwd, bwd = obs.indices_from_layout(lay)
            kw = dict(forward_indices=torch.from_numpy(fwd), backward_indices=torch.from_numpy(bwd))
            w = rnd(in_f, bwd.shape[1], 4)
        else:
            w = rnd(out_f, in_f)
        if lowrank:
            kw.update(lowrank_first=rnd(lowrank, in_f), lowrank_second=rnd(out_f, lowrank))
        return offn.LinearParams(w, rnd(out_f), out_features=out_f, **kw)

    return offn.FFNParams(
        ln_weight=1 + rnd(hidden), ln_bias=rnd(hidden), i2h=lin(hidden, n1), h2o=lin(inter, hidden),
        post_ln_weight=(1 + rnd(hidden)) if post_ln else None, post_ln_bias=rnd(hidden) if post_ln else None,
        cfg=offn.FFNConfig(gated=gated, **cfg))


@pytest.mark.parametrize("gated,post_ln,lowrank,sparse,residual,dropout", [
    (False, False, 0, False, True, 0.0),
    (True, False, 0, False, True, 0.0),
    (True, True, 3, False, False, 0.25),
    (True, True, 2, True, True, 0.0),
    (False, False, 2, True, True, 0.5),
])
@pytest.mark.parametrize("act", ["gelu_fused", "silu"])
def test_lean_function_equals_plain_autograd(gated, post_ln, lowrank, sparse, residual, dropout, act):
    """the manual backward with the reference's save-set equals autograd of the plain composition (the property
    reference tests/test_ffn.py:58-86 and :212-241 assert of _LeanFFN), in fp64"""
    p = _random_params(16, 32, gated, post_ln, lowrank, sparse, torch.float64, seed=3, act=act, ln_eps=1e-5,
                       residual=residual, dropout=dropout)
    for t in p.tensors():
        t.requires_grad_(True)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(2, 5, 16, generator=g, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(2, 5, 16, generator=g, dtype=torch.float64)
    mask = (torch.rand(10, 16, generator=g) >= dropout) if dropout > 0 else None
    y_plain = offn.plain_ffn(x, p, mask)
    grads_plain = torch.autograd.grad(y_plain, [x, *p.tensors()], dy)
    y_lean = offn.lean_ffn(x, p, mask)
    grads_lean = torch.autograd.grad(y_lean, [x, *p.tensors()], dy)
    assert torch.allclose(y_plain, y_lean, rtol=1e-10, atol=1e-12)
    for a, b in zip(grads_plain, grads_lean):
        assert torch.allclose(a, b, rtol=1e-9, atol=1e-11)


def test_lean_function_gradcheck():
    p = _random_params(8, 12, True, True, 2, False, torch.float64, seed=11, act="gelu_fused", ln_eps=1e-5, residual=True)
    for t in p.tensors():
        t.requires_grad_(True)
    x = torch.randn(3, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(1), requires_grad=True)
    tensors = p.tensors()

    def fn(x_, *params):
        return offn.LeanFFNFunction.apply(x_, None, p, *params)

    assert torch.autograd.gradcheck(fn, (x, *tensors), eps=1e-6, atol=1e-5, rtol=1e-4)


def test_plain_ffn_is_the_textbook_composition():
    """half order of the gate (first half gates, reference ffn.py:143-144) and op order post-LN -> dropout -> residual
    (ffn.py:198-207), written out with explicit formulas on a tiny case"""
    p = _random_params(4, 6, True, True, 0, False, torch.float64, seed=2, act="gelu_fused", ln_eps=1e-3, residual=True,
                       dropout=0.5)
    x = torch.randn(3, 4, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    mask = torch.tensor([[1, 0, 1, 1], [0, 0, 1, 1], [1, 1, 1, 0]], dtype=torch.bool)
    mu, var = x.mean(-1, keepdim=True), ((x - x.mean(-1, keepdim=True)) ** 2).mean(-1, keepdim=True)
    u = (x - mu) / torch.sqrt(var + 1e-3) * p.ln_weight + p.ln_bias
    pre = u @ p.i2h.weight.t() + p.i2h.bias
    gate, lin = pre[:, :6], pre[:, 6:]
    h = 0.5 * gate * (1 + torch.tanh(0.79788456 * gate * (1 + 0.044715 * gate ** 2))) * lin
    o = h @ p.h2o.weight.t() + p.h2o.bias
    mu2, var2 = o.mean(-1, keepdim=True), ((o - o.mean(-1, keepdim=True)) ** 2).mean(-1, keepdim=True)
    o = (o - mu2) / torch.sqrt(var2 + 1e-3) * p.post_ln_weight + p.post_ln_bias
    ref = o * mask / 0.5 + x
    assert torch.allclose(offn.plain_ffn(x, p, mask), ref, rtol=1e-12, atol=1e-12)


def test_bf16_rounding_points_are_straight_through_and_representable():
    """FFNConfig.bf16_rounding: values land on bfloat16's grid (8 significant bits, round to nearest even: known answers),
    gradients pass unchanged, and with smooth activations the rounded forward stays within bf16 noise of the exact one"""
    from oracle.ffn import round_bf16_straight_through as rnd
    t = torch.tensor([1.0, 1.00390625, 1.01171875, -3.0e-5, 257.0, 258.0, 259.0], requires_grad=True)
    r = rnd(t)
    # 1 + 2^-8 is a tie between 1 and 1 + 2^-7 -> even (1.0); 1 + 3 * 2^-8 ties to 1 + 2^-6; 257 ties to 256, 259 to 260
    assert torch.equal(r.detach()[:3], torch.tensor([1.0, 1.0, 1.015625]))
    assert torch.equal(r.detach()[4:], torch.tensor([256.0, 258.0, 260.0]))
    assert torch.equal(r.detach(), r.detach().to(torch.bfloat16).float())
    (g,) = torch.autograd.grad(r.sum(), t)
    assert torch.equal(g, torch.ones_like(t))
    gen = torch.Generator().manual_seed(0)
    x, dy = torch.randn(64, 32, generator=gen), torch.randn(64, 32, generator=gen)
    exact = offn.make_dense_params(32, 64, gated=True, generator=gen, ln_eps=1e-5)
    rounded = offn.FFNParams(exact.ln_weight, exact.ln_bias, exact.i2h, exact.h2o,
                             cfg=offn.FFNConfig(gated=True, ln_eps=1e-5, bf16_rounding=True))
    y0, y1 = offn.plain_ffn(x, exact), offn.plain_ffn(x, rounded)
    assert 0 < (y0 - y1).abs().max() / y0.abs().max() < 2e-2
