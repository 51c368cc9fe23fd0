"""Where the cycles of each GEMM launch of a LeanFFN step go: prologue, main loop, epilogue, per workgroup (= per tile).

    python -m lean_transformer_amd._build --tile-timing      (once: builds csrc/libleanffn_tile_timing.so)
    python -m lean_transformer_amd.tile_timing --config c3    (on the GPU)

Runs fwd+bwd steps of a benchmark configuration (bench.py's) on the instrumented library, in which thread 0 of every
workgroup of the copy-based GEMM kernel stamps the shader clock (s_memtime) at its phase boundaries and the 100 MHz
real-time counter at both ends.  Prints, per launch of a step: tiles, wall-clock span, shader-clock ticks per tile split
into prologue (launch to first matrix instruction), main loop (with the first 16 k-steps apart) and epilogue, the ideal
(1 024 ticks per 32-wide k-step: 32 matrix instructions of 32 cycles per SIMD) and the shader clock while tiles run.
A measurement tool: nothing in the package imports it.
"""
import argparse
import os
import sys


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="c3", choices=["c2", "c3"], help="dense bf16 benchmark configuration of bench.py")
    ap.add_argument("--warmup", type=int, default=20)
    args = ap.parse_args()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.path.insert(0, root)
    import torch

    from lean_transformer_amd import _build, _native as nat

    if not os.path.exists(_build.TILE_TIMING_LIB_PATH):
        sys.exit(f"{_build.TILE_TIMING_LIB_PATH} is missing: run `python -m lean_transformer_amd._build --tile-timing`")
    nat.LIB_PATH = _build.TILE_TIMING_LIB_PATH  # before the first nat.lib() call
    import bench
    import lean_transformer_amd as lt

    dev = torch.device("cuda:0")
    cfg = bench.CONFIGS[args.config]
    ffn, x, dy = bench.build_workload(torch, lt, cfg, dev)
    params = list(ffn.parameters())
    regions, slots = 6, 4096
    stamps = torch.zeros(regions * slots * 8, dtype=torch.int64, device=dev)
    os.environ["LT_TILE_TIMING_BUFFER"] = hex(stamps.data_ptr())

    def step():
        y = ffn(x)
        torch.autograd.grad(y, [x, *params], dy)

    for _ in range(args.warmup):  # a step is six copy-based launches: region i always holds launch i of a step
        step()
    torch.cuda.synchronize()
    stamps.zero_()
    step()
    torch.cuda.synchronize()
    tokens, hidden, inter = cfg["batch"] * cfg["seq"], cfg["hidden"], cfg["inter"]
    n1 = 2 * inter if cfg["gated"] else inter
    launches = [("up-projection + activation", hidden), ("down-projection + residual", inter), ("dh + d-activation", hidden),
                ("dW2", tokens), ("du", n1), ("dW1", tokens)]
    data = stamps.cpu().numpy().reshape(regions, slots, 8)
    print(f"{cfg['name']}\nticks = shader clock cycles per 256 x 256 tile; ideal = 1024 per k-step of 32")
    total_ticks = total_ideal = 0.0
    for (label, k), d in zip(launches, data):
        d = d[d[:, 0] != 0]
        ksteps = k // 32
        prologue, loop, epilogue = d[:, 1] - d[:, 0], d[:, 2] - d[:, 1], d[:, 3] - d[:, 2]
        first16 = (d[:, 7] - d[:, 1]).mean()
        clock = ((d[:, 3] - d[:, 0]) / ((d[:, 5] - d[:, 4]) * 10.0)).mean()
        span = (d[:, 5].max() - d[:, 4].min()) / 100.0
        per_tile = (prologue + loop + epilogue).mean()
        total_ticks += per_tile * len(d)
        total_ideal += ksteps * 1024.0 * len(d)
        print(f"{label:28s} tiles {len(d):5d}  span {span:7.1f} us  ticks/tile {per_tile:9.0f}  ideal {ksteps * 1024:8d} "
              f"({ksteps * 1024 / per_tile:.3f})  prologue {prologue.mean():6.0f}  loop {loop.mean():9.0f} = "
              f"{loop.mean() / ksteps:6.1f}/k-step (first 16: {first16 / 16:6.1f}, rest: "
              f"{(loop.mean() - first16) / (ksteps - 16):6.1f})  epilogue {epilogue.mean():6.0f} (max {epilogue.max():6d})  "
              f"clock {clock:.3f} GHz")
    print(f"all six launches: matrix-core-ideal ticks / measured ticks = {total_ideal / total_ticks:.3f}")


if __name__ == "__main__":
    main()
