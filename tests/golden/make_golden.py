"""Writes tests/golden/blocksparse_golden.npz: input/output vectors of the reference's native block-sparse
backend and index builder, for the two things that reading the source and the reference's own tests leave open:

  * how the native sparse weight ``[in_features, A, block]`` is laid out in memory
    (reference: lean_transformer/blocksparse/native_backend.py:9-35, :38-76), and
  * forward/backward indices of non-square layouts, stretched and tiled
    (reference: lean_transformer/blocksparse/layout.py:56-117, :177-211).

Runs only where the reference checkout is mounted at /root/reference (it is not present on a GPU box; tests
read the committed .npz only). The reference package's __init__ pulls in an optional dependency that is not
installed, so the three source files needed are loaded as submodules of a bare namespace package instead of
through ``import lean_transformer``; nothing else of the reference is executed.

    LEAN_USE_JIT=0 python tests/golden/make_golden.py
"""
import importlib
import os
import sys
import types

import numpy as np
import torch

REF = "/root/reference/lean_transformer"


def _load_reference():
    os.environ.setdefault("LEAN_USE_JIT", "0")
    pkg = types.ModuleType("lean_transformer")
    pkg.__path__ = [REF]
    sys.modules["lean_transformer"] = pkg
    sub = types.ModuleType("lean_transformer.blocksparse")
    sub.__path__ = [os.path.join(REF, "blocksparse")]
    sys.modules["lean_transformer.blocksparse"] = sub
    layout = importlib.import_module("lean_transformer.blocksparse.layout")
    native = importlib.import_module("lean_transformer.blocksparse.native_backend")
    return layout, native


def main():
    layout_mod, native = _load_reference()
    out = {}
    cases = [
        # name, out_features, in_features, layout string
        ("sq64_b4", 64, 64, "pixelfly(block_size=4)"),
        ("up256x32_b16", 256, 32, "pixelfly(16)"),
        ("down32x128_b16", 32, 128, "pixelfly(16)"),
        ("up128x32_b4", 128, 32, "pixelfly(block_size=4)"),
        ("up128x32_b4_stretch", 128, 32, "pixelfly(block_size=4, stretch=True)"),
        ("down32x128_b4", 32, 128, "pixelfly(block_size=4)"),
        ("down32x128_b4_stretch", 32, 128, "pixelfly(block_size=4, stretch=True)"),
        ("sq64_b4_nf2", 64, 64, "pixelfly(block_size=4, butterfly_size=8, n_factors=2)"),
        ("hyper64_b4", 64, 64, "hypercube(block_size=4, folded=False)"),
        ("hyper64_b4_folded", 64, 64, "hypercube(block_size=4, folded=True)"),
        ("hyper128x32_b4_folded_stretch", 128, 32, "hypercube(block_size=4, folded=True, stretch=True)"),
    ]
    names = []
    for name, out_f, in_f, desc in cases:
        lay = layout_mod.get_blocksparse_layout(out_f, in_f, desc)
        fwd, bwd = layout_mod.get_indices_from_layout(lay)
        block = in_f // lay.shape[1]
        gen = torch.Generator().manual_seed(1234 + len(names))
        a_per_in = fwd.numel() // (in_f // block)
        x = torch.randn(2, 3, in_f, generator=gen)
        w = torch.randn(in_f, a_per_in, block, generator=gen)
        dy = torch.randn(2, 3, out_f, generator=gen)
        y = native.blocksparse_matmul(x, w, fwd)
        dx, dw = native.blocksparse_matmul_backward(dy, x, w, bwd)
        names.append(name)
        out[f"{name}/desc"] = np.array(desc)
        out[f"{name}/shape"] = np.array([out_f, in_f, block], dtype=np.int64)
        out[f"{name}/layout"] = lay.numpy().astype(np.bool_)
        out[f"{name}/forward_indices"] = fwd.numpy()
        out[f"{name}/backward_indices"] = bwd.numpy()
        out[f"{name}/x"] = x.numpy()
        out[f"{name}/w"] = w.numpy()
        out[f"{name}/dy"] = dy.numpy()
        out[f"{name}/y"] = y.numpy()
        out[f"{name}/dx"] = dx.numpy()
        out[f"{name}/dw"] = dw.numpy()
    out["names"] = np.array(names)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "blocksparse_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes;", len(names), "cases")


if __name__ == "__main__":
    main()
