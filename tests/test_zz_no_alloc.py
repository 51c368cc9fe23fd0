"""lt_layernorm_backward_static: the LayerNorm backward entry point that allocates nothing (its partial parameter-gradient
rows live in static device memory) against lt_layernorm_backward, which takes a caller workspace.  Both run the same
kernels in the same order, so results must be bit-identical.  Two calls in a row, the second on a smaller input: the
static buffer keeps the first call's contents, which the second must not see."""
import pytest
import torch

from lean_transformer_amd import _native as nat

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(tokens, hidden, x_dtype, dy_dtype, dx_dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(tokens, hidden, generator=g) * 2 + 0.5).to(x_dtype).to(DEV)
    dy = torch.randn(tokens, hidden, generator=g).to(dy_dtype).to(DEV)
    res = torch.randn(tokens, hidden, generator=g).to(dx_dtype).to(DEV)
    w = (torch.rand(hidden, generator=g) + 0.5).to(DEV)
    xf = x.float()
    stats = torch.stack([xf.mean(-1), torch.rsqrt(xf.var(-1, unbiased=False) + 1e-5)], 1).contiguous()
    return x, dy, res, w, stats


def _run(entry, tokens, hidden, x_dtype, dy_dtype, dx_dtype, tensors, want_params=True):
    x, dy, res, w, stats = tensors
    lib = nat.lib()
    dx = torch.full((tokens, hidden), float("nan"), dtype=dx_dtype, device=DEV)
    dw = torch.full((hidden,), float("nan"), device=DEV) if want_params else None
    db = torch.full((hidden,), float("nan"), device=DEV) if want_params else None
    stream = nat.current_stream(dx.device)
    common = (tokens, hidden, nat.dtype_code(x_dtype), nat.ptr(x), nat.ptr(stats), nat.ptr(w), nat.dtype_code(dy_dtype),
              nat.ptr(dy), nat.dtype_code(dx_dtype), nat.ptr(res), nat.ptr(dx), nat.ptr(dw), nat.ptr(db))
    if entry == "static":
        nat.check(lib.lt_layernorm_backward_static(*common, stream), "lt_layernorm_backward_static")
    else:
        ws = nat.workspace(lib.lt_layernorm_backward_workspace_bytes(tokens, hidden), torch.device(DEV))
        ws.fill_(0xFF)
        nat.check(lib.lt_layernorm_backward(*common, nat.ptr(ws), ws.numel(), stream), "lt_layernorm_backward")
    torch.cuda.synchronize()
    return dx, dw, db


@pytest.mark.parametrize("dtypes", [(torch.float32, torch.float32, torch.float32),
                                    (torch.float32, torch.bfloat16, torch.float32),
                                    (torch.bfloat16, torch.bfloat16, torch.bfloat16)])
def test_static_scratch_entry_matches_the_workspace_entry_twice_in_a_row(dtypes):
    # first call: 128 row slices of 4096 columns fill 4 MiB of the static buffer; second call: a smaller input whose
    # partial rows overlap the start of what the first call left there; third: the any-shape kernel (rows of 10 elements)
    for tokens, hidden in ((8200, 4096), (300, 768), (37, 10)):
        tensors = _case(tokens, hidden, *dtypes, seed=tokens + hidden)
        got = _run("static", tokens, hidden, *dtypes, tensors)
        ref = _run("workspace", tokens, hidden, *dtypes, tensors)
        for name, a, b in zip(("dx", "dweight", "dbias"), got, ref):
            assert torch.isfinite(a.float()).all(), name
            assert torch.equal(a, b), f"{name} differs at tokens={tokens} hidden={hidden}"


def test_static_scratch_entry_allocates_nothing_and_refuses_what_does_not_fit():
    lib = nat.lib()
    assert lib.lt_layernorm_backward_static_scratch_bytes() == 8 << 20
    dtypes = (torch.float32, torch.float32, torch.float32)
    tensors = _case(512, 1024, *dtypes, seed=1)
    _run("static", 512, 1024, *dtypes, tensors)  # the first call on the device looks the buffer up
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    _run_static_only = lib.lt_layernorm_backward_static
    x, dy, res, w, stats = tensors
    dx = torch.empty(512, 1024, device=DEV)
    dw, db = torch.empty(1024, device=DEV), torch.empty(1024, device=DEV)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        nat.check(_run_static_only(512, 1024, 0, nat.ptr(x), nat.ptr(stats), nat.ptr(w), 0, nat.ptr(dy), 0, nat.ptr(res),
                                   nat.ptr(dx), nat.ptr(dw), nat.ptr(db), nat.current_stream(dx.device)), "static")
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before  # the device's free memory did not move
    # rows of 1030 elements take the any-shape kernel: one partial row pair per workgroup, 1024 of them = 8.44 MB > 8 MiB
    tokens, hidden = 2048, 1030
    big = _case(tokens, hidden, *dtypes, seed=2)
    x, dy, res, w, stats = big
    dx = torch.empty(tokens, hidden, device=DEV)
    dw, db = torch.empty(hidden, device=DEV), torch.empty(hidden, device=DEV)
    status = _run_static_only(tokens, hidden, 0, nat.ptr(x), nat.ptr(stats), nat.ptr(w), 0, nat.ptr(dy), 0, nat.ptr(res),
                              nat.ptr(dx), nat.ptr(dw), nat.ptr(db), nat.current_stream(dx.device))
    assert status == 2, status  # LT_ERR_UNSUPPORTED
    assert b"static buffer" in lib.lt_last_error()
    # without parameter gradients nothing is staged, so the same shape runs
    nat.check(_run_static_only(tokens, hidden, 0, nat.ptr(x), nat.ptr(stats), nat.ptr(w), 0, nat.ptr(dy), 0, nat.ptr(res),
                               nat.ptr(dx), None, None, nat.current_stream(dx.device)), "static without parameter gradients")
    torch.cuda.synchronize()
    assert torch.isfinite(dx).all()


_FIRST_CALL_UNDER_CAPTURE = r"""
import sys, torch
sys.path.insert(0, sys.argv[1])
from lean_transformer_amd import _native as nat
dev = torch.device("cuda:0")
tokens, hidden = 64, 256
x = torch.randn(tokens, hidden, device=dev); dy = torch.randn(tokens, hidden, device=dev)
w = torch.ones(hidden, device=dev); dx = torch.empty_like(x); dw = torch.empty(hidden, device=dev); db = torch.empty(hidden, device=dev)
stats = torch.stack([x.mean(-1), torch.rsqrt(x.var(-1, unbiased=False) + 1e-5)], 1).contiguous()
lib = nat.lib()
def call(stream):
    return lib.lt_layernorm_backward_static(tokens, hidden, 0, nat.ptr(x), nat.ptr(stats), nat.ptr(w), 0, nat.ptr(dy), 0, None,
                                            nat.ptr(dx), nat.ptr(dw), nat.ptr(db), stream)
side = torch.cuda.Stream()
side.wait_stream(torch.cuda.current_stream())
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph, stream=side):
    status = call(side.cuda_stream)          # first call on this device, on a capturing stream: refused, capture intact
    dx.zero_()                               # (something for the graph to hold)
assert status == 2 and b"outside stream capture" in lib.lt_last_error(), (status, lib.lt_last_error())
graph.replay(); torch.cuda.synchronize()
assert call(torch.cuda.current_stream().cuda_stream) == 0   # the warm-up call outside capture
torch.cuda.synchronize()
ref_dw = dw.clone()
graph2 = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph2, stream=side):
    assert call(side.cuda_stream) == 0       # now capturable
dw.zero_(); graph2.replay(); torch.cuda.synchronize()
assert torch.equal(dw, ref_dw)
print("ok")
"""


def test_first_call_under_stream_capture_is_refused_and_later_calls_capture():
    """the buffer's address is looked up on the first call on a device, which is not a stream operation: on a capturing stream
    that first call is refused (and the capture survives); after one warm-up call the entry point captures and replays.
    Needs a process in which the library has not been called yet: a child process."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", _FIRST_CALL_UNDER_CAPTURE, root], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "ok" in out.stdout, out.stdout + out.stderr
