"""GPU parity of the individual kernels, called through the C ABI (ctypes): GEMM cores in every operand layout, LayerNorm
forward / backward, activations, dropout mask, block-sparse matmul (against the reference's golden vectors) and the
generalized linear layer.  Bars: fp32 max relative error <= 1e-4; bf16 <= 2e-2 with cosine >= 0.9999."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import lean_transformer_amd as lt
from conftest import assert_close, rel_err
from helpers import dropout_mask
from lean_transformer_amd import _native as nat
from oracle import blocksparse as obs
from oracle import ffn as offn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLDEN = np.load(os.path.join(os.path.dirname(__file__), "golden", "blocksparse_golden.npz"))


def _gemm(a, b, a_kmajor, b_kmajor, m, n, k, c_dtype, force_generic):
    c = torch.empty(m, n, dtype=c_dtype, device=DEV)
    lib = nat.lib(a.dtype, c_dtype)
    nat.check(lib.lt_gemm(nat.dtype_code(a.dtype), m, n, k, nat.ptr(a), int(a_kmajor), nat.ptr(b), int(b_kmajor),
                          nat.dtype_code(c_dtype), nat.ptr(c), int(force_generic), nat.current_stream(c.device)),
              "lt_gemm", lib)
    return c


def _operands(m, n, k, a_kmajor, b_kmajor, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=g).to(dtype)
    b = torch.randn(n, k, generator=g).to(dtype)
    ref = a.double() @ b.double().t()
    a_dev = (a if a_kmajor else a.t().contiguous()).to(DEV)
    b_dev = (b if b_kmajor else b.t().contiguous()).to(DEV)
    return a_dev, b_dev, ref


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("a_kmajor,b_kmajor", [(True, True), (True, False), (False, False), (False, True)])
@pytest.mark.parametrize("m,n,k", [(70, 45, 33), (300, 260, 130), (1, 1, 1), (128, 128, 16)])
def test_gemm_any_shape_kernel(dtype, a_kmajor, b_kmajor, m, n, k):
    a, b, ref = _operands(m, n, k, a_kmajor, b_kmajor, dtype, seed=m + n + k)
    c = _gemm(a, b, a_kmajor, b_kmajor, m, n, k, torch.float32, force_generic=True)
    assert rel_err(c, ref) <= 1e-5  # fp32 MFMA on exactly representable inputs


@pytest.mark.parametrize("a_kmajor,b_kmajor", [(True, True), (True, False), (False, False)])
@pytest.mark.parametrize("m,n,k", [(512, 512, 256), (256, 768, 64), (1024, 256, 1024)])
@pytest.mark.parametrize("c_dtype", [torch.float32, torch.bfloat16])
def test_gemm_tiled_bf16_kernel(a_kmajor, b_kmajor, m, n, k, c_dtype):
    a, b, ref = _operands(m, n, k, a_kmajor, b_kmajor, torch.bfloat16, seed=m + 2 * n + 3 * k)
    c = _gemm(a, b, a_kmajor, b_kmajor, m, n, k, c_dtype, force_generic=False)
    if c_dtype == torch.float32:
        assert rel_err(c, ref) <= 1e-5
    else:
        assert_close(c, ref.float(), torch.bfloat16, "c")
    # and it agrees with the any-shape kernel to fp32 summation-order noise
    c2 = _gemm(a, b, a_kmajor, b_kmajor, m, n, k, torch.float32, force_generic=True)
    assert rel_err(c.float(), c2) <= (1e-5 if c_dtype == torch.float32 else 1e-2)


def test_gemm_tiled_bf16_ragged_rows_and_reduction():
    # k-major A with a ragged row count (rows past M are clamped on load, never stored)
    a, b, ref = _operands(300, 256, 128, True, True, torch.bfloat16, seed=1)
    assert rel_err(_gemm(a, b, True, True, 300, 256, 128, torch.float32, False), ref) <= 1e-5
    a, b, ref = _operands(777, 512, 192, True, False, torch.bfloat16, seed=2)
    assert rel_err(_gemm(a, b, True, False, 777, 512, 192, torch.float32, False), ref) <= 1e-5
    # both operands mn-major with a reduction length that is not a multiple of the 64-wide k-step (zero-filled tail)
    a, b, ref = _operands(256, 512, 200, False, False, torch.bfloat16, seed=3)
    assert rel_err(_gemm(a, b, False, False, 256, 512, 200, torch.float32, False), ref) <= 1e-5
    a, b, ref = _operands(512, 256, 1000, False, False, torch.bfloat16, seed=4)
    assert rel_err(_gemm(a, b, False, False, 512, 256, 1000, torch.float32, False), ref) <= 1e-5


def _kernel_tags(fn):
    """runs fn with the library's kernel timing on and returns the tags of the kernels it launched"""
    lib = nat.lib()
    lib.lt_profile_reset()
    lib.lt_profile_enable(1)
    try:
        out = fn()
        torch.cuda.synchronize()
    finally:
        lib.lt_profile_enable(0)
    tags = {entry[0] for entry in nat.profile_read()}
    lib.lt_profile_reset()
    return out, tags


TILE_LOOP_CASES = [(a, b, m, n, k) for a, b in ((True, True), (True, False), (False, False))
                   for m, n, k in ((4352, 4096, 192), (4360, 4104, 320), (8192, 8192, 64))] + [(False, False, 4352, 4096, 200)]


@pytest.mark.parametrize("a_kmajor,b_kmajor,m,n,k", TILE_LOOP_CASES)
def test_gemm_tile_loop_gives_the_same_bits_as_one_workgroup_per_tile(a_kmajor, b_kmajor, m, n, k):
    """more tiles than compute units: by default one workgroup per compute unit loops over its tiles and issues the first
    copies of its next tile before the epilogue of the current one; flag bit 8 launches one workgroup per tile instead.
    Same arithmetic in the same order: the results must be identical, whole tiles, tiles past the edge and a ragged
    reduction (mn-major operands) alike, and right."""
    g = torch.Generator(device=DEV).manual_seed(m + n + k)
    a = torch.randn((m, k) if a_kmajor else (k, m), generator=g, device=DEV).to(torch.bfloat16)
    b = torch.randn((n, k) if b_kmajor else (k, n), generator=g, device=DEV).to(torch.bfloat16)
    ref = (a.float() if a_kmajor else a.float().t()) @ (b.float().t() if b_kmajor else b.float())
    for c_dtype in (torch.float32, torch.bfloat16):
        flat = torch.full((2, m * n + 4096), 7.0, dtype=c_dtype, device=DEV)  # two results, each with a guard behind it
        for i, force in enumerate((0, 1 << 8)):
            c = flat[i, :m * n].view(m, n)
            _, tags = _kernel_tags(lambda: nat.check(
                nat.lib().lt_gemm(nat.dtype_code(a.dtype), m, n, k, nat.ptr(a), int(a_kmajor), nat.ptr(b), int(b_kmajor),
                                  nat.dtype_code(c_dtype), nat.ptr(c), force, nat.current_stream(c.device)), "lt_gemm"))
            assert any(t.startswith("gemm_bf16_") and t.endswith("_store") for t in tags), tags
        assert torch.equal(flat[0], flat[1])
        assert bool((flat[:, m * n:] == 7.0).all())
        assert rel_err(flat[0, :m * n].view(m, n).float(), ref) <= (1e-5 if c_dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("a_kmajor,b_kmajor,tag", [(True, True, "gemm_bf16_nt_store"), (True, False, "gemm_bf16_nn_store"),
                                                   (False, False, "gemm_bf16_tn_store")])
@pytest.mark.parametrize("m,n,k", [(512, 320, 128), (256, 8, 64), (328, 200, 192), (1600, 1608, 320), (264, 776, 448)])
@pytest.mark.parametrize("c_dtype", [torch.float32, torch.bfloat16])
def test_gemm_tiled_bf16_tiles_past_the_edge(a_kmajor, b_kmajor, tag, m, n, k, c_dtype):
    """N (and, for an mn-major A, M) a multiple of 8 but not of the 256-wide tile: the tiled kernel still takes the problem,
    re-reads the last row / last 8 columns for the part of the tile that sticks out and writes nothing there"""
    a, b, ref = _operands(m, n, k, a_kmajor, b_kmajor, torch.bfloat16, seed=m + 2 * n + 3 * k)
    flat = torch.full((m * n + 4096,), 7.0, dtype=c_dtype, device=DEV)  # the result, then a guard nothing may write
    c = flat[:m * n].view(m, n)
    _, tags = _kernel_tags(lambda: nat.check(
        nat.lib().lt_gemm(nat.dtype_code(a.dtype), m, n, k, nat.ptr(a), int(a_kmajor), nat.ptr(b), int(b_kmajor),
                          nat.dtype_code(c_dtype), nat.ptr(c), 0, nat.current_stream(c.device)), "lt_gemm"))
    assert tag in tags, tags
    assert bool((flat[m * n:] == 7.0).all())
    if c_dtype == torch.float32:
        assert rel_err(c, ref) <= 1e-5
    else:
        assert_close(c, ref.float(), torch.bfloat16, "c")


@pytest.mark.parametrize("tokens,hidden", [(37, 32), (64, 768), (9, 4096), (3, 10), (5, 8192), (2, 8200)])
@pytest.mark.parametrize("x_dtype,y_dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16),
                                             (torch.bfloat16, torch.bfloat16)])
def test_layernorm_forward(tokens, hidden, x_dtype, y_dtype):
    g = torch.Generator().manual_seed(tokens * hidden)
    x = (torch.randn(tokens, hidden, generator=g) * 2 + 0.5).to(x_dtype)
    w, b = torch.rand(hidden, generator=g) + 0.5, torch.randn(hidden, generator=g)
    ref = F.layer_norm(x.float(), (hidden,), w, b, 1e-5)
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    y = torch.empty(tokens, hidden, dtype=y_dtype, device=DEV)
    stats = torch.empty(tokens, 2, device=DEV)
    nat.check(nat.lib().lt_layernorm_forward(tokens, hidden, 1e-5, nat.dtype_code(x_dtype), nat.ptr(xd), nat.ptr(wd),
                                             nat.ptr(bd), nat.dtype_code(y_dtype), nat.ptr(y), nat.ptr(stats),
                                             nat.current_stream(y.device)), "lt_layernorm_forward")
    assert_close(y, ref, y_dtype, "y")
    assert torch.allclose(stats[:, 0].cpu(), x.float().mean(-1), rtol=1e-4, atol=1e-5)
    assert torch.allclose(stats[:, 1].cpu(), torch.rsqrt(x.float().var(-1, unbiased=False) + 1e-5), rtol=1e-4)


@pytest.mark.parametrize("tokens,hidden", [(37, 32), (300, 768), (2100, 256), (3, 10), (4, 8192), (3, 12288), (70, 8200), (5, 8202)])
@pytest.mark.parametrize("x_dtype,dy_dtype,dx_dtype", [(torch.float32, torch.float32, torch.float32),
                                                       (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                                       (torch.float32, torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("with_residual", [False, True])
def test_layernorm_backward(tokens, hidden, x_dtype, dy_dtype, dx_dtype, with_residual):
    g = torch.Generator().manual_seed(tokens + hidden)
    x = (torch.randn(tokens, hidden, generator=g) * 2 + 0.5).to(x_dtype)
    dy = torch.randn(tokens, hidden, generator=g).to(dy_dtype)
    res = torch.randn(tokens, hidden, generator=g).to(dx_dtype)
    w = torch.rand(hidden, generator=g) + 0.5
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    br = torch.zeros(hidden, dtype=torch.float64, requires_grad=True)
    F.layer_norm(xr, (hidden,), wr, br, 1e-5).backward(dy.double())
    ref_dx = xr.grad + (res.double() if with_residual else 0)
    xd, dyd, wd, resd = x.to(DEV), dy.to(DEV), w.to(DEV), res.to(DEV)
    stats = torch.stack([x.float().mean(-1), torch.rsqrt(x.float().var(-1, unbiased=False) + 1e-5)], 1).to(DEV)
    dx = torch.empty(tokens, hidden, dtype=dx_dtype, device=DEV)
    dw, db = torch.empty(hidden, device=DEV), torch.empty(hidden, device=DEV)
    lib = nat.lib()
    ws = nat.workspace(lib.lt_layernorm_backward_workspace_bytes(tokens, hidden), torch.device(DEV))
    nat.check(lib.lt_layernorm_backward(tokens, hidden, nat.dtype_code(x_dtype), nat.ptr(xd), nat.ptr(stats), nat.ptr(wd),
                                        nat.dtype_code(dy_dtype), nat.ptr(dyd), nat.dtype_code(dx_dtype),
                                        nat.ptr(resd) if with_residual else None, nat.ptr(dx), nat.ptr(dw), nat.ptr(db),
                                        nat.ptr(ws), ws.numel(), nat.current_stream(dx.device)), "lt_layernorm_backward")
    assert_close(dx, ref_dx.float(), dx_dtype, "dx")
    assert_close(dw, wr.grad.float(), torch.float32, "dweight")
    assert_close(db, br.grad.float(), torch.float32, "dbias")


@pytest.mark.parametrize("act", offn.ACT_NAMES)
@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_activation_forward_backward(act, gated, dtype):
    """every kernel-side activation, value and derivative, against fp64 autograd of the oracle's value on the same stored
    pre-activations (so the kinks of the piecewise ones fall on the same side)"""
    from lean_transformer_amd.utils import ACT_KINDS
    tokens, inter = 33, 70
    g = torch.Generator().manual_seed(5)
    pre = (torch.randn(tokens, 2 * inter if gated else inter, generator=g) * 3).to(dtype)
    pre[0, :6] = torch.tensor([11.0, -11.0, 25.0, -25.0, 6.5, -3.5]).to(dtype)  # beyond gelu_10's clip, softplus' switch, the kinks
    dh = torch.randn(tokens, inter, generator=g).to(dtype)
    pr = pre.double().requires_grad_(True)
    href = offn.apply_activation(pr, act, gated)
    (dpre_ref,) = torch.autograd.grad(href, pr, dh.double())
    pd, dhd = pre.to(DEV), dh.to(DEV)
    hid, dpre = torch.empty_like(dhd), torch.empty_like(pd)
    lib = nat.lib()
    nat.check(lib.lt_activation_forward(tokens, inter, int(gated), ACT_KINDS[act], nat.dtype_code(dtype), nat.ptr(pd),
                                        nat.ptr(hid), nat.current_stream(pd.device)), "lt_activation_forward")
    nat.check(lib.lt_activation_backward(tokens, inter, int(gated), ACT_KINDS[act], nat.dtype_code(dtype), nat.ptr(pd),
                                         nat.ptr(dhd), nat.ptr(dpre), nat.current_stream(pd.device)), "lt_activation_backward")
    assert_close(hid, href.detach().float(), dtype, "hid")
    assert_close(dpre, dpre_ref.float(), dtype, "dpre")


def test_tanh_gelu_saturates_cleanly_in_the_bf16_kernels():
    """the bf16 kernels evaluate the tanh GELU through a sigmoid with fast exp2 / rcp: far in the tails (e^{-2u} over- or
    underflowing) value and derivative must come out as the limits x / 0 and 1 / 0, never NaN or inf, and in between they
    must follow the closed forms of the reference (utils.py:24-38)"""
    from lean_transformer_amd.utils import ACT_KINDS
    x = torch.tensor([-3.0e4, -1.0e3, -100.0, -30.0, -12.0, -6.0, -3.0, -1.0, -0.25, -1e-3, 0.0, 1e-3, 0.25, 1.0, 3.0, 6.0,
                      12.0, 30.0, 100.0, 1.0e3, 3.0e4] + [0.0] * 11).view(4, 8)
    tokens, inter = x.shape
    pre = x.to(torch.bfloat16).to(DEV)
    dh = torch.ones_like(pre)
    hid, dpre = torch.empty_like(pre), torch.empty_like(pre)
    lib = nat.lib()
    nat.check(lib.lt_activation_forward(tokens, inter, 0, ACT_KINDS["gelu_fused"], nat.dtype_code(torch.bfloat16),
                                        nat.ptr(pre), nat.ptr(hid), nat.current_stream(pre.device)), "lt_activation_forward")
    nat.check(lib.lt_activation_backward(tokens, inter, 0, ACT_KINDS["gelu_fused"], nat.dtype_code(torch.bfloat16),
                                         nat.ptr(pre), nat.ptr(dh), nat.ptr(dpre), nat.current_stream(pre.device)),
              "lt_activation_backward")
    xf = pre.float().cpu().double()
    value = offn.gelu_fused(xf)
    grad = offn.gelu_fused_grad(torch.ones_like(xf), xf)
    hid, dpre = hid.float().cpu().double(), dpre.float().cpu().double()
    assert torch.isfinite(hid).all() and torch.isfinite(dpre).all()
    assert torch.allclose(hid, value, rtol=1e-2, atol=1e-6), (hid - value).abs().max()
    assert torch.allclose(dpre, grad, rtol=1e-2, atol=1e-6), (dpre - grad).abs().max()
    assert hid.view(-1)[0] == 0 and dpre.view(-1)[0] == 0
    assert hid.view(-1)[20] == float(pre.view(-1)[20]) and dpre.view(-1)[20] == 1


def test_dropout_mask_properties():
    dev = torch.device(DEV)
    m1 = dropout_mask(512, 768, 0.1, seed=1234, offset=0, device=dev)
    assert abs(m1.float().mean().item() - 0.9) < 5e-3
    assert torch.equal(m1, dropout_mask(512, 768, 0.1, 1234, 0, dev))          # a pure function of (seed, offset, index)
    assert not torch.equal(m1, dropout_mask(512, 768, 0.1, 1234, 4, dev))      # another stream offset
    assert not torch.equal(m1, dropout_mask(512, 768, 0.1, 1235, 0, dev))      # another seed
    assert dropout_mask(16, 32, 0.0, 1, 0, dev).all()
    # a higher drop probability drops a superset (same random words against a higher threshold)
    m5 = dropout_mask(512, 768, 0.5, 1234, 0, dev)
    assert abs(m5.float().mean().item() - 0.5) < 5e-3 and not (m5 & ~m1).any()


@pytest.mark.parametrize("name", [str(n) for n in GOLDEN["names"]])
def test_blocksparse_matmul_against_reference_golden(name):
    x, w, dy = (torch.from_numpy(GOLDEN[f"{name}/{k}"]).to(DEV) for k in ("x", "w", "dy"))
    fwd = torch.from_numpy(GOLDEN[f"{name}/forward_indices"]).to(DEV)
    bwd = torch.from_numpy(GOLDEN[f"{name}/backward_indices"]).to(DEV)
    y = lt.blocksparse_matmul(x, w, fwd)
    dx, dw = lt.blocksparse_matmul_backward(dy, x, w, bwd)
    assert_close(y, torch.from_numpy(GOLDEN[f"{name}/y"]), torch.float32, "y")
    assert_close(dx, torch.from_numpy(GOLDEN[f"{name}/dx"]), torch.float32, "dx")
    assert_close(dw, torch.from_numpy(GOLDEN[f"{name}/dw"]), torch.float32, "dw")
    dx_only, empty = lt.blocksparse_matmul_backward(dy, x, w, bwd, weight_requires_grad=False)
    assert empty.numel() == 0 and torch.equal(dx_only, dx)


@pytest.mark.parametrize("out_f,in_f,block,stretch,dtype", [
    (1024, 256, 64, True, torch.bfloat16), (256, 1024, 64, False, torch.bfloat16), (384, 96, 96 // 4, False, torch.float32),
    (8192 // 4, 4096 // 4, 256, True, torch.float32)])
def test_blocksparse_matmul_against_oracle(out_f, in_f, block, stretch, dtype):
    """larger blocks than the golden vectors hold (64: the headline block size; 256: reference tests/test_butterfly.py)"""
    layout = obs.pixelfly_layout(out_f, in_f, block_size=block, stretch=stretch)
    fwd, bwd = obs.indices_from_layout(layout)
    g = torch.Generator().manual_seed(42)
    x = torch.randn(3, 50, in_f, generator=g).to(dtype)
    w = (torch.randn(in_f, bwd.shape[1], block, generator=g) * 0.1).to(dtype)
    dy = torch.randn(3, 50, out_f, generator=g).to(dtype)
    y_ref = obs.blocksparse_matmul(x.float(), w.float(), fwd)
    dx_ref, dw_ref = obs.blocksparse_matmul_backward(dy.float(), x.float(), w.float(), bwd)
    y = lt.blocksparse_matmul(x.to(DEV), w.to(DEV), torch.from_numpy(fwd).to(DEV))
    dx, dw = lt.blocksparse_matmul_backward(dy.to(DEV), x.to(DEV), w.to(DEV), torch.from_numpy(bwd).to(DEV))
    assert_close(y, y_ref, dtype, "y")
    assert_close(dx, dx_ref, dtype, "dx")
    assert_close(dw, dw_ref, dtype, "dw")


@pytest.mark.parametrize("block_size,lowrank_dim,adapter_dim", [(0, 0, 0), (0, 60, 0), (0, 0, 4), (0, 60, 4), (8, 0, 0),
                                                                (8, 60, 4)])
@pytest.mark.parametrize("bias", [True, False])
def test_generalized_linear_against_oracle(block_size, lowrank_dim, adapter_dim, bias):
    """the cases of reference tests/test_linear.py:79-137 (dim 128, pixelfly block 8, low-rank 60, adapter 4)"""
    torch.manual_seed(1337)
    dim = 128
    layout = f"pixelfly(block_size={block_size})" if block_size else None
    layer = lt.GeneralizedLinear(lt.GeneralizedMatrix(dim, dim, layout, lowrank_dim), adapter_dim, bias=bias)
    with torch.no_grad():
        if adapter_dim:
            layer.adapter_second.normal_(std=0.1)
        if bias:
            layer.bias.normal_()
    x = torch.rand(4, 5, dim)
    dy = torch.randn(4, 5, dim)
    from helpers import oracle_linear
    p = oracle_linear(layer, "cpu", torch.float32)
    xr = x.clone().requires_grad_(True)
    y_ref = offn.linear_forward(xr.reshape(-1, dim), p).reshape(4, 5, dim)
    ref_grads = torch.autograd.grad(y_ref, [xr, *p.tensors()], dy)
    layer = layer.to(DEV)
    xd = x.to(DEV).requires_grad_(True)
    y = layer(xd)
    names = [n for n, _ in layer.named_parameters()]
    grads = torch.autograd.grad(y, [xd, *layer.parameters()], dy.to(DEV))
    assert_close(y, y_ref.detach(), torch.float32, "y")
    assert_close(grads[0], ref_grads[0], torch.float32, "dx")
    got = dict(zip(names, grads[1:]))
    ref = dict(zip(["weight"] + (["bias"] if bias else []) + (["first", "second"] if (lowrank_dim or adapter_dim) else []),
                   ref_grads[1:]))
    assert_close(got["matrix.weight"], ref["weight"], torch.float32, "dweight")
    if bias:
        assert_close(got["bias"], ref["bias"], torch.float32, "dbias")
    if lowrank_dim and adapter_dim:  # combined factors: shared low-rank rows first, adapter rows after (linear.py:131-136)
        assert_close(got["matrix.lowrank_first"], ref["first"][:lowrank_dim], torch.float32, "dlowrank_first")
        assert_close(got["adapter_first"], ref["first"][lowrank_dim:], torch.float32, "dadapter_first")
        assert_close(got["matrix.lowrank_second"], ref["second"][:, :lowrank_dim], torch.float32, "dlowrank_second")
        assert_close(got["adapter_second"], ref["second"][:, lowrank_dim:], torch.float32, "dadapter_second")
    elif lowrank_dim:
        assert_close(got["matrix.lowrank_first"], ref["first"], torch.float32, "dlowrank_first")
        assert_close(got["matrix.lowrank_second"], ref["second"], torch.float32, "dlowrank_second")
    elif adapter_dim:
        assert_close(got["adapter_first"], ref["first"], torch.float32, "dadapter_first")
        assert_close(got["adapter_second"], ref["second"], torch.float32, "dadapter_second")


def test_empty_batch():
    layer = lt.GeneralizedLinear(lt.GeneralizedMatrix(32, 64)).to(DEV)
    assert layer(torch.empty(0, 32, device=DEV)).shape == (0, 64)
    ffn = lt.LeanFFN(32, 64).to(DEV)
    assert ffn(torch.empty(2, 0, 32, device=DEV)).shape == (2, 0, 32)


def test_out_group_promise_is_checked_on_the_device_and_a_false_one_stays_inside_the_weight():
    """lt_linear.out_group is a caller's promise about the index tables.  lt_linear_check_out_group tests it on the device;
    a value that does not divide the number of output blocks is refused; and a false promise that passes that test makes the
    forward kernel compute with the wrong blocks but never read outside the weight (NaNs sit right behind it here: the
    results stay finite)."""
    from lean_transformer_amd.blocksparse.linear import linear_desc
    torch.manual_seed(3)
    m = lt.GeneralizedMatrix(1024, 4096, "pixelfly(block_size=64, stretch=True)", 0).to(DEV).to(torch.bfloat16)
    run = 4096 // 1024
    fwd, bwd = m.forward_indices, m.backward_indices
    lib = nat.lib()
    flag = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    stream = nat.current_stream(flag.device)

    def checked(group):
        desc = linear_desc(m.weight.detach(), None, None, None, fwd, bwd)
        desc.out_group = group
        status = lib.lt_linear_check_out_group(desc, nat.ptr(flag), stream)
        return status, (int(flag.item()) if status == 0 else None)

    assert linear_desc(m.weight.detach(), None, None, None, fwd, bwd).out_group == run
    assert checked(run) == (0, 1) and checked(2) == (0, 1) and checked(1) == (0, 1) and checked(0) == (0, 1)
    assert checked(8) == (0, 0) and checked(16) == (0, 0)  # longer runs than the layout has
    assert checked(3)[0] != 0 and "out_group" in lib.lt_last_error().decode()  # 64 output blocks are not a multiple of 3
    # a false promise on the forward kernel (a square layout has no runs; runs of 4 are claimed): in bounds, finite, wrong
    sq = lt.GeneralizedMatrix(2048, 2048, "pixelfly(block_size=64)", 0).to(DEV).to(torch.bfloat16)
    assert linear_desc(sq.weight.detach(), None, None, None, sq.forward_indices, sq.backward_indices).out_group == 1
    x = torch.randn(512, 2048, device=DEV).to(torch.bfloat16)
    weight = torch.full((sq.weight.numel() + 65536,), float("nan"), dtype=torch.bfloat16, device=DEV)  # NaNs behind the weight
    weight[:sq.weight.numel()] = sq.weight.detach().flatten()
    w3 = weight[:sq.weight.numel()].view_as(sq.weight)
    outs = []
    for group in (1, 4):
        desc = linear_desc(w3, None, None, None, sq.forward_indices, sq.backward_indices)
        desc.out_group = group
        y = torch.empty(512, 2048, dtype=torch.bfloat16, device=DEV)
        nat.check(lib.lt_linear_forward(desc, 512, nat.dtype_code(torch.bfloat16), nat.ptr(x), nat.ptr(y), None, stream),
                  "lt_linear_forward")
        assert torch.isfinite(y.float()).all()
        outs.append(y)
    ref = obs.blocksparse_matmul(x.float().cpu(), sq.weight.detach().float().cpu(), sq.forward_indices.cpu().numpy())
    assert_close(outs[0], ref, torch.bfloat16, "y without the promise")
    assert not torch.equal(outs[0], outs[1])


def test_in_group_promise_is_checked_on_the_device_and_a_false_one_stays_inside_the_gradient():
    """lt_linear.in_group: the same promise on the input side (runs of input blocks with one list of output blocks).
    lt_linear_check_in_group tests it on the device; a value that does not divide the number of input blocks is refused; a
    false promise writes wrong values into the weight gradient, all of them inside it (a guard band behind it stays intact)."""
    from lean_transformer_amd.blocksparse.linear import linear_desc
    torch.manual_seed(4)
    m = lt.GeneralizedMatrix(4096, 1024, "pixelfly(block_size=64, stretch=True)", 0).to(DEV).to(torch.bfloat16)
    run = 4096 // 1024
    fwd, bwd = m.forward_indices, m.backward_indices
    lib = nat.lib()
    flag = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    stream = nat.current_stream(flag.device)

    def checked(group):
        desc = linear_desc(m.weight.detach(), None, None, None, fwd, bwd)
        desc.in_group = group
        status = lib.lt_linear_check_in_group(desc, nat.ptr(flag), stream)
        return status, (int(flag.item()) if status == 0 else None)

    desc = linear_desc(m.weight.detach(), None, None, None, fwd, bwd)
    assert desc.in_group == run and desc.out_group == 1
    assert checked(run) == (0, 1) and checked(2) == (0, 1) and checked(1) == (0, 1) and checked(0) == (0, 1)
    assert checked(8) == (0, 0) and checked(16) == (0, 0)
    assert checked(3)[0] != 0 and "in_group" in lib.lt_last_error().decode()  # 64 input blocks are not a multiple of 3
    # weight gradient with the true promise, without one, and with a false one (a square layout claimed to have runs of 4)
    tokens = 1024
    sq = lt.GeneralizedMatrix(2048, 2048, "pixelfly(block_size=64)", 0).to(DEV).to(torch.bfloat16)
    grads_of = {}
    for name, matrix, groups in (("wide", m, (0, run)), ("square", sq, (0, 4))):
        in_f, out_f = matrix.weight.shape[0], matrix.forward_indices.shape[0] * 64
        x = torch.randn(tokens, in_f, device=DEV).to(torch.bfloat16)
        dy = torch.randn(tokens, out_f, device=DEV).to(torch.bfloat16)
        for group in groups:
            desc = linear_desc(matrix.weight.detach(), None, None, None, matrix.forward_indices, matrix.backward_indices)
            desc.in_group = group
            room = torch.full((matrix.weight.numel() + 65536,), 7.0, dtype=torch.bfloat16, device=DEV)
            grads = nat.LtLinearGrads()
            grads.weight = nat.ptr(room)
            need = lib.lt_linear_backward_workspace_bytes(desc, tokens, nat.dtype_code(torch.bfloat16))
            ws = torch.empty(max(int(need), 1), dtype=torch.uint8, device=DEV)
            nat.check(lib.lt_linear_backward(desc, tokens, nat.dtype_code(torch.bfloat16), nat.ptr(x), nat.ptr(dy), None, None,
                                             grads, nat.ptr(ws), ws.numel(), stream), "lt_linear_backward")
            assert bool((room[matrix.weight.numel():] == 7.0).all()), (name, group)
            assert torch.isfinite(room.float()).all()
            grads_of[name, group] = room[:matrix.weight.numel()].clone()
        ref = obs.blocksparse_matmul_backward(dy.float().cpu(), x.float().cpu(), matrix.weight.detach().float().cpu(),
                                              matrix.backward_indices.cpu().numpy())[1]
        assert_close(grads_of[name, 0].view_as(matrix.weight), ref, torch.bfloat16, name + " without the promise")
    assert_close(grads_of["wide", run].view_as(m.weight), grads_of["wide", 0].float().view_as(m.weight), torch.bfloat16, "wide")
    assert not torch.equal(grads_of["square", 0], grads_of["square", 4])


def test_strided_run_promises_of_tiled_layouts_are_checked_on_the_device():
    """tiled PixelFly layouts: the runs are blocks a square width apart; the check entries accept the true (length, distance)
    pair, raise the flag's 0 for a wrong distance, and refuse a pair that does not tile the blocks"""
    from lean_transformer_amd.blocksparse.linear import linear_desc
    lib = nat.lib()
    flag = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    stream = nat.current_stream(flag.device)
    tall = lt.GeneralizedMatrix(1024, 4096, "pixelfly(block_size=64, stretch=False)", 0).to(DEV).to(torch.bfloat16)
    wide = lt.GeneralizedMatrix(4096, 1024, "pixelfly(block_size=64, stretch=False)", 0).to(DEV).to(torch.bfloat16)
    for m, field, entry in ((tall, "out_group", lib.lt_linear_check_out_group), (wide, "in_group", lib.lt_linear_check_in_group)):
        desc = linear_desc(m.weight.detach(), None, None, None, m.forward_indices, m.backward_indices)
        assert getattr(desc, field) == 4 | (16 << 16)

        def checked(value):
            setattr(desc, field, value)
            status = entry(desc, nat.ptr(flag), stream)
            return status, (int(flag.item()) if status == 0 else None)

        assert checked(4 | (16 << 16)) == (0, 1)
        assert checked(2 | (32 << 16)) == (0, 1)   # (blocks two square widths apart share their lists too)
        assert checked(8 | (8 << 16)) == (0, 0)    # blocks half a square width apart do not
        assert checked(4 | (8 << 16))[0] != 0      # 4 x 8 is not the 64 blocks

