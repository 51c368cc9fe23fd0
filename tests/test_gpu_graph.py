"""The LeanFFN forward + backward recorded into a HIP graph (torch.cuda.CUDAGraph) and replayed: the library launches
kernels on the caller's stream only -- no allocation, no host synchronisation, no memset nodes -- so a step can be captured
once and replayed.  Every replay is checked bit for bit against the eager result on the same inputs, with eager work and
synchronisations between the replays."""
import pytest
import torch

import lean_transformer_amd as lt

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _step(ffn, x, dy, params):
    y = ffn(x)
    return (y, *torch.autograd.grad(y, [x, *params], dy))


@pytest.mark.parametrize("hidden,inter,tokens,dtype,layout", [
    (512, 1024, 300, torch.bfloat16, None), (256, 4096, 200, torch.bfloat16, None), (192, 320, 130, torch.float32, None),
    # block-sparse projections: the walks, and (stretched PixelFly) the dense products over gathered blocks with their split
    # rank-64 GEMMs; the warm-up steps settle the once-per-index-tensor host check of the layout's structure before capture
    (512, 2048, 512, torch.bfloat16, "pixelfly(block_size=64, stretch=True)"),
    (512, 2048, 300, torch.bfloat16, "pixelfly(block_size=64, stretch=False)")])
def test_ffn_step_replays_from_a_graph(hidden, inter, tokens, dtype, layout):
    torch.manual_seed(hidden + tokens)
    if layout is None:
        ffn = lt.LeanFFN(hidden, inter, gated=True, layer_norm_eps=1e-5)
    else:
        up = lt.GeneralizedLinear(lt.GeneralizedMatrix(hidden, 2 * inter, layout, 64))
        down = lt.GeneralizedLinear(lt.GeneralizedMatrix(inter, hidden, layout, 64))
        ffn = lt.LeanFFN(hidden, inter, gated=True, layer_norm_eps=1e-5, i2h_proj=up, h2o_proj=down)
    with torch.no_grad():
        ffn.i2h_proj.bias.normal_(std=0.1)
        ffn.h2o_proj.bias.normal_(std=0.1)
    ffn = ffn.to(DEV).to(dtype)
    params = list(ffn.parameters())
    static_x = torch.randn(tokens, hidden, device=DEV, requires_grad=True)
    static_dy = torch.randn(tokens, hidden, device=DEV)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            _step(ffn, static_x, static_dy, params)
    torch.cuda.current_stream().wait_stream(side)

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        recorded = _step(ffn, static_x, static_dy, params)

    for trial in range(3):
        x = torch.randn(tokens, hidden, device=DEV) * (1.0 + trial)
        dy = torch.randn(tokens, hidden, device=DEV)
        with torch.no_grad():
            static_x.copy_(x)
            static_dy.copy_(dy)
        graph.replay()
        torch.cuda.synchronize()
        eager = _step(ffn, x.clone().requires_grad_(True), dy, params)
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(recorded, eager)):
            assert torch.equal(a, b), f"replay {trial}: tensor {i} differs from the eager step"
