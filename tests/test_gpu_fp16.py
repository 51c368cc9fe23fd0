"""float16 on the twin library (libleanffn_f16.so: the same kernels compiled with IEEE binary16 as their 16-bit type).  One
case per kernel family the bfloat16 tests cover in depth -- copy-based and register-staged GEMMs in every operand layout,
LayerNorm, the LeanFFN block dense / gated / with post-LayerNorm, dropout, low-rank terms, PixelFly projections on the
walks and on the dense products over runs, the any-shape kernels of small layers -- against the fp32 CPU oracle (the block)
or fp32 stock ops on the same rounded operands (layers, GEMMs).  Bars: max relative error 4e-3, cosine 0.999996 (the bf16
bars scaled to fp16's three extra significant bits); GEMMs with fp32 output 1e-5."""
import pytest
import torch

import lean_transformer_amd as lt
from conftest import assert_close, rel_err
from helpers import dropout_mask, generator_position
from lean_transformer_amd import _native as nat
from lean_transformer_amd.utils import ACT2FN
from test_gpu_ffn import _compare, _full_size_checks, _headline
from test_gpu_ffn_bf16_paths import _dense_from_native, _randomise_small_vectors
from test_gpu_kernels import _gemm, _operands

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F16 = torch.float16


def test_each_library_names_its_16_bit_type_and_refuses_the_other_one():
    assert b"bf16" in nat.lib(torch.bfloat16).lt_version() and b"fp16" in nat.lib(F16).lt_version()
    a = torch.zeros(64, 64, dtype=F16, device=DEV)
    c = torch.zeros(64, 64, dtype=torch.float32, device=DEV)
    for lib, code in ((nat.lib(torch.bfloat16), nat.LT_F16), (nat.lib(F16), nat.LT_BF16)):
        status = lib.lt_gemm(code, 64, 64, 64, nat.ptr(a), 1, nat.ptr(a), 1, nat.LT_F32, nat.ptr(c), 0,
                             nat.current_stream(c.device))
        assert status == 1 and b"dtype code" in lib.lt_last_error()
    with pytest.raises(TypeError, match="one 16-bit type"):
        nat.lib(F16, torch.bfloat16)


@pytest.mark.parametrize("a_kmajor,b_kmajor", [(True, True), (True, False), (False, False), (False, True)])
@pytest.mark.parametrize("m,n,k,force_generic", [(512, 512, 256, False), (256, 768, 64, False), (1024, 256, 1024, False),
                                                 (300, 260, 130, False), (4096, 1024, 512, False), (70, 45, 33, True)])
@pytest.mark.parametrize("c_dtype", [torch.float32, F16])
def test_fp16_gemm(a_kmajor, b_kmajor, m, n, k, force_generic, c_dtype):
    a, b, ref = _operands(m, n, k, a_kmajor, b_kmajor, F16, seed=m + 2 * n + 3 * k)
    c = _gemm(a, b, a_kmajor, b_kmajor, m, n, k, c_dtype, force_generic=force_generic)
    if c_dtype == torch.float32:
        assert rel_err(c, ref) <= 1e-5  # fp32 accumulation of exactly representable products
    else:
        assert rel_err(c, ref) <= 2.0 ** -11  # one rounding of the result


@pytest.mark.parametrize("tokens,hidden", [(300, 512), (64, 1000), (5, 8200)])
def test_fp16_layernorm_forward_and_backward(tokens, hidden):
    torch.manual_seed(tokens + hidden)
    x = torch.randn(tokens, hidden).to(F16)
    dy = torch.randn(tokens, hidden).to(F16)
    w, b = torch.rand(hidden) + 0.5, torch.randn(hidden) * 0.2
    xr = x.float().requires_grad_(True)
    wr, br = w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    y_ref = torch.nn.functional.layer_norm(xr, (hidden,), wr, br, 1e-5)
    dx_ref, dw_ref, db_ref = torch.autograd.grad(y_ref, [xr, wr, br], dy.float())
    lib = nat.lib(F16)
    xd, dyd, wd, bd = x.to(DEV), dy.to(DEV), w.to(DEV), b.to(DEV)
    y = torch.empty_like(xd)
    stats = torch.empty(tokens, 2, dtype=torch.float32, device=DEV)
    stream = nat.current_stream(xd.device)
    nat.check(lib.lt_layernorm_forward(tokens, hidden, 1e-5, nat.LT_F16, nat.ptr(xd), nat.ptr(wd), nat.ptr(bd), nat.LT_F16,
                                       nat.ptr(y), nat.ptr(stats), stream), "lt_layernorm_forward", lib)
    assert_close(y, y_ref.detach(), F16, "y")
    dx = torch.empty_like(xd)
    dw, db = torch.empty(hidden, device=DEV), torch.empty(hidden, device=DEV)
    ws = nat.workspace(lib.lt_layernorm_backward_workspace_bytes(tokens, hidden), xd.device)
    nat.check(lib.lt_layernorm_backward(tokens, hidden, nat.LT_F16, nat.ptr(xd), nat.ptr(stats), nat.ptr(wd), nat.LT_F16,
                                        nat.ptr(dyd), nat.LT_F16, None, nat.ptr(dx), nat.ptr(dw), nat.ptr(db), nat.ptr(ws),
                                        ws.numel(), stream), "lt_layernorm_backward", lib)
    assert_close(dx, dx_ref, F16, "dx")
    assert_close(dw, dw_ref, torch.float32, "dweight")
    assert_close(db, db_ref, torch.float32, "dbias")


@pytest.mark.parametrize("io_dtype", [torch.float32, F16])
@pytest.mark.parametrize("act,gated,tokens", [("gelu_fused", True, 512), ("gelu_fused", False, 300), ("silu", True, 300),
                                              ("gelu", False, 512), ("tanh", True, 512)])
def test_fp16_ffn_dense(io_dtype, act, gated, tokens):
    torch.manual_seed(41)
    ffn = lt.LeanFFN(512, 1024, activation=ACT2FN[act], gated=gated, layer_norm_eps=1e-5)
    _randomise_small_vectors(ffn)
    ffn = ffn.to(DEV).to(F16)
    _compare(ffn, torch.randn(tokens, 512).to(io_dtype), torch.randn(tokens, 512).to(io_dtype), F16)


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("residual", [False, True])
def test_fp16_ffn_post_layer_norm_dropout_and_low_rank_terms(gated, residual):
    torch.manual_seed(43)
    tokens, hidden = 384, 1024
    ffn = lt.LeanFFN(hidden, 2048, gated=gated, post_layer_norm=True, dropout=0.1, residual=residual, layer_norm_eps=1e-5,
                     i2h_proj=lt.GeneralizedLinear(lt.GeneralizedMatrix(hidden, 4096 if gated else 2048, None, 16), 0),
                     h2o_proj=lt.GeneralizedLinear(lt.GeneralizedMatrix(2048, hidden, None, 0), 8))
    _randomise_small_vectors(ffn)
    with torch.no_grad():
        for proj in (ffn.i2h_proj, ffn.h2o_proj):
            for t in (proj.matrix.lowrank_first, proj.matrix.lowrank_second, proj.adapter_first, proj.adapter_second):
                if t is not None:
                    t.normal_(std=0.05)
    ffn = ffn.to(DEV).to(F16)
    x, dy = torch.randn(tokens, hidden), torch.randn(tokens, hidden)
    torch.cuda.manual_seed(7)
    seed, offset = generator_position(DEV)
    mask = dropout_mask(tokens, hidden, 0.1, seed, offset, torch.device(DEV)).cpu()
    _compare(ffn, x, dy, F16, mask=mask)


@pytest.mark.parametrize("tokens", [300, 2048])
@pytest.mark.parametrize("fan_in,fan_out,stretch", [(1024, 4096, True), (4096, 1024, True), (4096, 1024, False),
                                                    (1024, 4096, False)])
@pytest.mark.parametrize("lowrank_dim", [0, 64])
def test_fp16_blocksparse_wide_layers(tokens, fan_in, fan_out, stretch, lowrank_dim):
    """PixelFly with 64-wide blocks: the tiled walks forward and for dX, the weight gradient as dense products over the
    runs of blocks that share a list (stretched layouts: runs of neighbours; tiled: strided runs) or as a walk (300 tokens)"""
    torch.manual_seed(tokens + fan_out + lowrank_dim)
    layout = f"pixelfly(block_size=64, stretch={stretch})"
    layer = lt.GeneralizedLinear(lt.GeneralizedMatrix(fan_in, fan_out, layout, lowrank_dim), bias=True)
    with torch.no_grad():
        layer.bias.normal_(std=0.1)
        layer.weight.normal_(std=0.05)
        if lowrank_dim:
            layer.matrix.lowrank_first.normal_(std=0.05)
            layer.matrix.lowrank_second.normal_(std=0.05)
    layer = layer.to(DEV).to(F16)
    matrix = layer.matrix
    x, dy = torch.randn(tokens, fan_in), torch.randn(tokens, fan_out)
    xd = x.to(DEV).to(F16).requires_grad_(True)
    y = layer(xd)
    names, params = zip(*layer.named_parameters())
    grads = torch.autograd.grad(y, [xd, *params], dy.to(DEV).to(F16))
    leaves = {n: p.detach().float().requires_grad_(True) for n, p in layer.named_parameters()}
    xr = x.to(DEV).to(F16).float().requires_grad_(True)
    y_ref = xr @ _dense_from_native(leaves["matrix.weight"], matrix.backward_indices, fan_out).t() + leaves["bias"]
    if lowrank_dim:
        y_ref = y_ref + (xr @ leaves["matrix.lowrank_first"].t()) @ leaves["matrix.lowrank_second"].t()
    ref = torch.autograd.grad(y_ref, [xr, *[leaves[n] for n in names]], dy.to(DEV).to(F16).float())
    assert_close(y, y_ref.detach(), F16, "y")
    assert_close(grads[0], ref[0], F16, "dx")
    for name, a, b in zip(names, grads[1:], ref[1:]):
        assert_close(a, b, F16, name)


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("hidden,inter,block,tokens", [(1024, 4096, 64, 512), (1024, 4096, 64, 300), (32, 128, 16, 70)])
def test_fp16_ffn_with_blocksparse_projections(gated, hidden, inter, block, tokens):
    """PixelFly projections inside the block: 64-wide blocks on the tiled kernels, 16-wide blocks of a small layer on the
    any-shape kernels"""
    torch.manual_seed(47 + hidden + tokens)
    layout = f"pixelfly(block_size={block})"
    ffn = lt.LeanFFN(hidden, inter, gated=gated, layer_norm_eps=1e-5,
                     i2h_proj=lt.GeneralizedLinear(lt.GeneralizedMatrix(hidden, 2 * inter if gated else inter, layout, 4), 0),
                     h2o_proj=lt.GeneralizedLinear(lt.GeneralizedMatrix(inter, hidden, layout, 4), 0))
    _randomise_small_vectors(ffn)
    ffn = ffn.to(DEV).to(F16)
    _compare(ffn, torch.randn(tokens, hidden), torch.randn(tokens, hidden), F16)


def test_fp16_autocast_with_fp32_master_weights():
    """torch.autocast(float16) over an fp32 module: operands are cast per call, gradients come back in the parameters' dtype"""
    torch.manual_seed(53)
    tokens, hidden = 512, 512
    ffn = lt.LeanFFN(hidden, 1024, gated=True, layer_norm_eps=1e-5)
    _randomise_small_vectors(ffn)
    ffn = ffn.to(DEV)
    x, dy = torch.randn(tokens, hidden), torch.randn(tokens, hidden)
    xd = x.to(DEV).requires_grad_(True)
    with torch.autocast("cuda", dtype=F16):
        y = ffn(xd)
    params = [p for p in ffn.parameters()]
    grads = torch.autograd.grad(y, [xd, *params], dy.to(DEV))
    assert y.dtype == torch.float32 and all(g.dtype == torch.float32 for g in grads)
    half = lt.LeanFFN(hidden, 1024, gated=True, layer_norm_eps=1e-5).to(DEV)
    half.load_state_dict(ffn.state_dict())
    half = half.to(F16)
    xh = x.to(DEV).requires_grad_(True)
    yh = half(xh)
    gh = torch.autograd.grad(yh, [xh, *half.parameters()], dy.to(DEV))
    assert_close(y, yh.float(), F16, "y against the fp16 module")
    for i, (a, b) in enumerate(zip(grads, gh)):
        assert_close(a, b.float(), F16, f"grad {i} against the fp16 module")


def test_config3_fp16_full_size():
    """benchmark config 3 in float16: hidden 4096, intermediate 16384, GeGLU, x [2, 2048, 4096], weights ~N(0, 0.01); the
    oracle in fp32 on the GPU, 128 rows through the CPU oracle, weight gradients additive over token halves"""
    ffn, x, dy = _headline(4096, 16384, True, 0.01, 0.0, (2, 2048), dtype=F16)
    _full_size_checks(ffn, x, dy, 0.0, dtype=F16)
