"""Where the cycles of each GEMM launch of a LeanFFN step go: prologue, main loop, epilogue, per workgroup (= per tile).

    python tile_timing.py --build          (once, no GPU needed: builds lean_transformer_amd/csrc/libleanffn_tile_timing.so)
    python tile_timing.py --config c3      (on the GPU; c2: the other dense configuration; c4: the block-sparse one)

Runs fwd+bwd steps of a benchmark configuration (bench.py's) on the instrumented library, in which thread 0 of every
workgroup of the copy-based GEMM kernel stamps the shader clock (s_memtime) at its phase boundaries and the 100 MHz
real-time counter at both ends.  Prints, per launch of a step: tiles, wall-clock span, shader-clock ticks per tile split
into prologue (launch to first matrix instruction), main loop (with the first 16 k-steps apart) and epilogue, the ideal
(1 024 ticks per 32-wide k-step: 32 matrix instructions of 32 cycles per SIMD) and the shader clock while tiles run.
With --config c4 the stamped kernels are the block-sparse forward / input-gradient walks (256 x 64 tiles, two workgroups per
CU): start, before the first operand loads, after the main loop, after the epilogue.
A measurement tool beside bench.py, whose workloads it runs: not part of the package, and the package never loads the
instrumented library.
"""
import argparse
import os
import sys


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", default="c3", choices=["c2", "c3", "c4"], help="bf16 benchmark configuration of bench.py")
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--build", action="store_true", help="compile the instrumented library (hipcc, no GPU needed) and exit")
    ap.add_argument("--distribution", action="store_true", help="dense configurations: also print how tile durations and "
                    "end times spread over the tiles of each launch and over the eight XCDs (100 MHz real-time stamps)")
    args = ap.parse_args()
    root = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, root)
    from lean_transformer_amd import _build

    if args.build:
        print(_build.build(tile_timing=True))
        return
    import torch

    from lean_transformer_amd import _native as nat

    if not os.path.exists(_build.TILE_TIMING_LIB_PATH):
        sys.exit(f"{_build.TILE_TIMING_LIB_PATH} is missing: run `python tile_timing.py --build`")
    nat.LIB_PATH = _build.TILE_TIMING_LIB_PATH  # before the first nat.lib() call
    import bench
    import lean_transformer_amd as lt

    dev = torch.device("cuda:0")
    cfg = bench.CONFIGS[args.config]
    ffn, x, dy = bench.build_workload(torch, lt, cfg, dev)
    params = list(ffn.parameters())
    if cfg["sparse"]:
        return sparse_walks(torch, ffn, x, dy, params, cfg, dev)
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
        setup = (d[:, 6] - d[:, 0]).mean()  # launch to the first copy instruction: index arithmetic, bias loads
        clock = ((d[:, 3] - d[:, 0]) / ((d[:, 5] - d[:, 4]) * 10.0)).mean()
        span = (d[:, 5].max() - d[:, 4].min()) / 100.0
        per_tile = (prologue + loop + epilogue).mean()
        total_ticks += per_tile * len(d)
        total_ideal += ksteps * 1024.0 * len(d)
        print(f"{label:28s} tiles {len(d):5d}  span {span:7.1f} us  ticks/tile {per_tile:9.0f}  ideal {ksteps * 1024:8d} "
              f"({ksteps * 1024 / per_tile:.3f})  prologue {prologue.mean():6.0f} (of which before the first copy {setup:5.0f})  loop {loop.mean():9.0f} = "
              f"{loop.mean() / ksteps:6.1f}/k-step (first 16: {first16 / 16:6.1f}, rest: "
              f"{(loop.mean() - first16) / (ksteps - 16):6.1f})  epilogue {epilogue.mean():6.0f} (max {epilogue.max():6d})  "
              f"clock {clock:.3f} GHz")
    print(f"all six launches: matrix-core-ideal ticks / measured ticks = {total_ideal / total_ticks:.3f}")
    if args.distribution:
        import numpy as np
        print("tile durations by the real-time counter (us); tile i of the launch order runs on XCD i % 8")
        for (label, _), d in zip(launches, data):
            idx = np.nonzero(d[:, 0])[0]
            d = d[idx]
            t0 = d[:, 4].min()
            start, end = (d[:, 4] - t0) / 100.0, (d[:, 5] - t0) / 100.0
            dur = end - start
            last = idx >= len(idx) - min(256, len(idx))
            per_xcd = " ".join(f"{dur[(idx & 7) == xcd].mean():6.1f}" for xcd in range(8))
            print(f"{label:28s} duration min {dur.min():6.1f} p50 {np.median(dur):6.1f} p90 {np.percentile(dur, 90):6.1f} max {dur.max():6.1f}"
                  f"  mean per XCD {per_xcd}  end of the last {int(last.sum())} tiles: min {end[last].min():6.1f} p50 "
                  f"{np.median(end[last]):6.1f} max {end[last].max():6.1f}")


def sparse_walks(torch, ffn, x, dy, params, cfg, dev):
    """the four block-sparse FWD / DX launches of a step: launch i of the process writes region i % 4 (8192 workgroups each)"""
    regions, slots = 4, 8192
    stamps = torch.zeros(regions * slots * 8, dtype=torch.int64, device=dev)
    os.environ["LT_TILE_TIMING_BUFFER_SPARSE"] = hex(stamps.data_ptr())

    def step():
        y = ffn(x)
        torch.autograd.grad(y, [x, *params], dy)

    for _ in range(20):
        step()
    torch.cuda.synchronize()
    stamps.zero_()
    step()
    torch.cuda.synchronize()
    data = stamps.cpu().numpy().reshape(regions, slots, 8)
    hidden, inter = cfg["hidden"], cfg["inter"]
    n1 = 2 * inter if cfg["gated"] else inter
    per_out_up, per_out_down = ffn.i2h_proj.matrix.forward_indices.shape[1], ffn.h2o_proj.matrix.forward_indices.shape[1]
    per_in_up, per_in_down = ffn.i2h_proj.matrix.backward_indices.shape[1], ffn.h2o_proj.matrix.backward_indices.shape[1]
    rank_steps = ffn.i2h_proj.matrix.lowrank_first.shape[0] // 64 if ffn.i2h_proj.matrix.lowrank_first is not None else 0
    gated = 2 if cfg["gated"] else 1  # the gated up-projection walks the gate block's and the linear block's list
    launches = [("up-projection + activation", gated * (per_out_up + rank_steps)), ("down-projection + residual", per_out_down + rank_steps),
                ("dh + d-activation", per_in_down + rank_steps), ("du", per_in_up + rank_steps)]
    print(f"{cfg['name']}\nticks = shader clock cycles per 256 x 64 tile (two workgroups share a CU); k-step = one 64 x 64 weight block; "
          "a workgroup's matrix instructions of a k-step take 512 ticks of its SIMDs")
    # Launch i of the process writes region i % 4.  A projection whose layout lets it run as a dense product over gathered
    # blocks (runs of output blocks with one list) is not a walk and leaves no stamps: with three stamped launches per step one
    # region stays empty and the filled ones follow it cyclically, in launch order.
    filled = [bool((r[:, 3] != 0).any()) for r in data]
    if not all(filled):
        first = (filled.index(False) + 1) % regions
        data = [data[(first + i) % regions] for i in range(sum(filled))]
        launches = launches[len(launches) - len(data):]
        print(f"({regions - len(data)} launch of the step is not a block-sparse walk)")
    for (label, ksteps), d in zip(launches, data):
        d = d[d[:, 3] != 0]
        prologue, loop, epilogue = d[:, 1] - d[:, 0], d[:, 2] - d[:, 1], d[:, 3] - d[:, 2]
        clock = ((d[:, 3] - d[:, 0]) / ((d[:, 5] - d[:, 4]) * 10.0)).mean()
        span = (d[:, 5].max() - d[:, 4].min()) / 100.0
        print(f"{label:28s} tiles {len(d):5d}  span {span:7.1f} us  ticks/tile {(d[:, 3] - d[:, 0]).mean():9.0f}  before the loop "
              f"{prologue.mean():6.0f}  loop {loop.mean():9.0f} = {loop.mean() / ksteps:6.1f}/k-step ({ksteps} k-steps)  "
              f"epilogue {epilogue.mean():6.0f}  clock {clock:.3f} GHz")


if __name__ == "__main__":
    main()
