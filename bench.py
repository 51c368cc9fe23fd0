"""LeanFFN fwd+bwd throughput on one MI355X: benchmark config 3 (hidden 4096, intermediate 16384, GeGLU, bf16 weights, fp32
residual stream, x [2, 2048, 4096]).  Prints one JSON line.

    python bench.py --gpus 1 --steps 20 --warmup 5

A step is one forward + backward of the module on a resident synthetic batch (parameter gradients produced, no optimizer).
K steps are timed by wall clock; the same K steps are then repeated with a HIP event pair around every kernel launch
(recorded by the library on the launch stream) and `roofline` is computed from the GEMM launches of that pass;
`cpu_baseline` times the CPU oracle (tests' checker, not the product) on a bounded sample of the same workload.
The default run also measures configurations 2, 4 and 4 with the reference's default layout (c4t: stretch=False), about a
second of GPU time each, and reports them under `extra_configs` of the same line; `--config c3h` is configuration 3 in
float16 on the library's float16 build;
`--config c5` times the full GPT train step of configuration 5 (the stock-PyTorch model of tests/gpt_harness.py around the
FFN kernels).
"""
import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "LeanFFN fwd+bwd tokens/s + MFMA util % at h4096 bf16; peak activation MB"
PEAK_BF16_TFLOPS = 2516.6  # 256 CU x 4096 flop/clk/CU x 2.4 GHz, dense
PEAK_FP32_TFLOPS = 157.3   # fp32 matrix cores: the fp32 path computes there


# benchmark configurations that fit one GPU; the default (and the only one the metric is quoted on) is config 3
CONFIGS = {
    "c1": dict(batch=8, seq=512, hidden=768, inter=3072, gated=True, std=0.02, dropout=0.0, dtype="fp32", sparse=False,
               name="config1: LeanFFN dense GeGLU fwd+bwd, hidden 768, intermediate 3072, x [8,512,768], fp32"),
    "c2": dict(batch=4, seq=2048, hidden=2048, inter=8192, gated=False, std=0.02, dropout=0.1, dtype="bf16", sparse=False,
               name="config2: LeanFFN dense GELU fwd+bwd, hidden 2048, intermediate 8192, x [4,2048,2048] fp32 residual "
                    "stream, bf16 weights/activations, dropout 0.1 (Philox)"),
    "c3": dict(batch=2, seq=2048, hidden=4096, inter=16384, gated=True, std=0.01, dropout=0.0, dtype="bf16", sparse=False,
               name="config3: LeanFFN dense GeGLU fwd+bwd, hidden 4096, intermediate 16384, x [2,2048,4096] fp32 residual "
                    "stream, bf16 weights/activations, fp32 accumulation, dropout 0"),
    "c4": dict(batch=2, seq=2048, hidden=4096, inter=16384, gated=True, std=0.02, dropout=0.0, dtype="bf16", sparse=True,
               name="config4: LeanFFN PixelFly (64x64 blocks, stretch, density 7/64) + rank-128 low-rank GeGLU fwd+bwd, "
                    "hidden 4096, intermediate 16384, x [2,2048,4096], bf16"),
    # config 3 on the float16 twin of the library (same kernels, IEEE binary16 operands on the f16 matrix instruction)
    "c3h": dict(batch=2, seq=2048, hidden=4096, inter=16384, gated=True, std=0.01, dropout=0.0, dtype="fp16", sparse=False,
                name="config3 in float16: LeanFFN dense GeGLU fwd+bwd, hidden 4096, intermediate 16384, x [2,2048,4096] fp32 "
                     "residual stream, fp16 weights/activations, fp32 accumulation, dropout 0"),
    # config 4 with the reference's default layout (pixelfly tiles the square butterfly instead of stretching it: no runs of
    # blocks with one list, every product is a walk over the index tables)
    "c4t": dict(batch=2, seq=2048, hidden=4096, inter=16384, gated=True, std=0.02, dropout=0.0, dtype="bf16", sparse=True,
                stretch=False,
                name="config4, default layout: LeanFFN PixelFly (64x64 blocks, stretch=False, density 7/64) + rank-128 "
                     "low-rank GeGLU fwd+bwd, hidden 4096, intermediate 16384, x [2,2048,4096], bf16"),
}


def build_workload(torch, lt, cfg, device):
    g = torch.Generator().manual_seed(0)
    hidden, inter, std = cfg["hidden"], cfg["inter"], cfg["std"]
    n1 = 2 * inter if cfg["gated"] else inter
    x = torch.randn(cfg["batch"], cfg["seq"], hidden, generator=g)
    if cfg["sparse"]:
        layout = f"pixelfly(block_size=64, stretch={cfg.get('stretch', True)})"
        up = lt.GeneralizedLinear(lt.GeneralizedMatrix(hidden, n1, layout, 128))
        down = lt.GeneralizedLinear(lt.GeneralizedMatrix(inter, hidden, layout, 128))
        ffn = lt.LeanFFN(hidden, inter, gated=cfg["gated"], layer_norm_eps=1e-5, dropout=cfg["dropout"], i2h_proj=up,
                         h2o_proj=down)
        with torch.no_grad():
            for t in (up.weight, down.weight, up.matrix.lowrank_first, up.matrix.lowrank_second,
                      down.matrix.lowrank_first, down.matrix.lowrank_second):
                t.copy_(torch.randn(t.shape, generator=g) * std)
    else:
        ffn = lt.LeanFFN(hidden, inter, gated=cfg["gated"], layer_norm_eps=1e-5, dropout=cfg["dropout"])
        with torch.no_grad():
            ffn.i2h_proj.weight.copy_(torch.randn(n1, hidden, generator=g) * std)
            ffn.h2o_proj.weight.copy_(torch.randn(hidden, inter, generator=g) * std)
            ffn.i2h_proj.bias.zero_()
            ffn.h2o_proj.bias.zero_()
    dy = torch.randn(cfg["batch"], cfg["seq"], hidden, generator=g)
    ffn = ffn.to(device)
    if cfg["dtype"] != "fp32":
        ffn = ffn.to(torch.bfloat16 if cfg["dtype"] == "bf16" else torch.float16)
    return ffn, x.to(device).requires_grad_(True), dy.to(device)


def algorithmic_flops(cfg):
    """fwd+bwd flops with no recompute counted: 3 x the forward GEMM flops"""
    tokens = cfg["batch"] * cfg["seq"]
    hidden, inter = cfg["hidden"], cfg["inter"]
    n1 = 2 * inter if cfg["gated"] else inter
    if not cfg["sparse"]:
        return 6.0 * tokens * hidden * (n1 + inter)
    density, rank = 7.0 / 64.0, 128
    fwd = 2 * density * hidden * n1 + 2 * density * inter * hidden + 2 * rank * (hidden + n1) + 2 * rank * (inter + hidden)
    return 3.0 * tokens * fwd


def oracle_params_of(torch, ffn, device, dtype):
    """the module's parameters as the oracle's containers (copies in `dtype` on `device`, requiring grad)"""
    from oracle import ffn as offn

    def leaf(t):
        return None if t is None else t.detach().to(device=device, dtype=dtype).clone().requires_grad_(True)

    def lin(proj):
        matrix = getattr(proj, "matrix", None)
        if matrix is None:
            return offn.LinearParams(leaf(proj.weight), leaf(proj.bias), out_features=proj.out_features)
        first, second = proj.get_combined_lowrank_components()
        fwd, bwd = matrix.forward_indices, matrix.backward_indices
        return offn.LinearParams(leaf(proj.weight), leaf(proj.bias), leaf(first), leaf(second),
                                 None if fwd is None else fwd.cpu(), None if bwd is None else bwd.cpu(),
                                 out_features=proj.out_features)

    return offn.FFNParams(leaf(ffn.pre_layer_norm.weight), leaf(ffn.pre_layer_norm.bias), lin(ffn.i2h_proj),
                          lin(ffn.h2o_proj),
                          cfg=offn.FFNConfig(gated=ffn.gated, ln_eps=ffn.pre_layer_norm.eps, residual=ffn.residual))


def cpu_baseline(torch, ffn, x, dy, sample_tokens, warmup, iters):
    """the oracle's memory-lean autograd.Function (same save-set and recompute schedule as the reference's _LeanFFN) in fp32
    on the host cores, on the first `sample_tokens` tokens of the selected workload (dropout off: it draws no time)"""
    from oracle import ffn as offn

    hidden = x.shape[-1]
    p = oracle_params_of(torch, ffn, "cpu", torch.float32)
    xs = x.detach().reshape(-1, hidden)[:sample_tokens].float().cpu().clone().requires_grad_(True)
    dys = dy.detach().reshape(-1, hidden)[:sample_tokens].float().cpu()
    times = []
    for i in range(warmup + iters):
        t0 = time.perf_counter()
        y = offn.lean_ffn(xs, p)
        torch.autograd.grad(y, [xs, *p.tensors()], dys)
        times.append(time.perf_counter() - t0)
    timed = sorted(times[warmup:])
    median = timed[len(timed) // 2]
    return sample_tokens / median, median


def reference_activation_memory(torch, ffn, x, dy):
    """(saved MiB, peak MiB) of one fwd+bwd of the oracle's LeanFFNFunction -- the reference's schedule: keep x and the
    pre-activation, recompute LayerNorm output and activation in backward -- on the GPU under bf16 autocast with the same
    weights, input and upstream gradient, measured the way the build's own figures are.  Outside every timed region."""
    from oracle import ffn as offn

    p = oracle_params_of(torch, ffn, x.device, next(ffn.parameters()).dtype)
    xr = x.detach().clone().requires_grad_(True)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = offn.lean_ffn(xr, p)
    torch.cuda.synchronize()
    saved = (torch.cuda.memory_allocated() - base - y.numel() * y.element_size()) / 2**20
    torch.autograd.grad(y, [xr, *p.tensors()], dy.to(y.dtype))
    torch.cuda.synchronize()
    peak = (torch.cuda.max_memory_allocated() - base) / 2**20
    return saved, peak


def csrc_sha16():
    """hash of the kernel sources in the tree: ties a counter summary under profiles/ to the kernels it was taken from"""
    csrc = os.path.join(ROOT, "lean_transformer_amd", "csrc")
    h = hashlib.sha256()
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".h")):
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def measured_traffic(config):
    """L2 <-> memory bytes per GEMM launch from the rocprofv3 FETCH_SIZE / WRITE_SIZE summary kept under profiles/ for this
    configuration (written when that summary is refreshed), with the algorithmic bytes of the same launches and where the
    figure comes from: the summary records the hash of the kernel sources it was measured on, and `stale` says whether the
    tree's kernels still are those.  (None, None, None) when the configuration has no such summary."""
    # the default-layout variant of config 4 and the float16 variant of config 3 have their base configuration's
    # algorithmic bytes and no counter run of their own
    counted = config not in ("c4t", "c3h")
    path = os.path.join(ROOT, "profiles", f"leanffn_config{config[1:2]}_gemm_hbm_traffic.json")
    if not os.path.exists(path):
        return None, None, None
    with open(path) as f:
        d = json.load(f)
    if not counted:
        return None, float(d["algorithmic_bytes_per_gemm_launch"]), None
    tree = csrc_sha16()
    source = {"file": os.path.relpath(path, ROOT), "measured_on_csrc_sha16": d.get("csrc_sha16"), "tree_csrc_sha16": tree,
              "stale": d.get("csrc_sha16") != tree}
    return float(d["bytes_per_gemm_launch"]), float(d["algorithmic_bytes_per_gemm_launch"]), source


def library_gemm_yardstick(torch, cfg, device, iters=10):
    """torch.matmul (the vendor GEMM library) in bf16 on the six GEMM shapes of a dense step, each in the operand layout the
    step has it in, with no epilogue work: what a plain library GEMM reaches on the same box in the same run.  Not part of
    the product path; reported next to the library's own per-kernel figures."""
    tokens, hidden, inter = cfg["batch"] * cfg["seq"], cfg["hidden"], cfg["inter"]
    n1 = 2 * inter if cfg["gated"] else inter
    # name: (M, N, K, layout); nt: A [M,K], B [N,K]; nn: A [M,K], B [K,N]; tn: A [K,M], B [K,N]
    shapes = {"up": (tokens, n1, hidden, "nt"), "down": (tokens, hidden, inter, "nt"), "dh": (tokens, inter, hidden, "nn"),
              "dW2": (hidden, inter, tokens, "tn"), "du": (tokens, hidden, n1, "nn"), "dW1": (n1, hidden, tokens, "tn")}
    out, total_us, total_flops = {}, 0.0, 0.0
    for name, (m, n, k, layout) in shapes.items():
        a = torch.randn((k, m) if layout == "tn" else (m, k), device=device, dtype=torch.bfloat16)
        b = torch.randn((n, k) if layout == "nt" else (k, n), device=device, dtype=torch.bfloat16)
        fn = {"nt": lambda: a @ b.t(), "nn": lambda: a @ b, "tn": lambda: a.t() @ b}[layout]
        for _ in range(3):
            fn()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        for _ in range(iters):
            fn()
        stop.record()
        torch.cuda.synchronize()
        us = start.elapsed_time(stop) / iters * 1e3
        out[name] = {"m": m, "n": n, "k": k, "layout": layout, "avg_us": us, "tflops": 2.0 * m * n * k / us / 1e6}
        total_us += us
        total_flops += 2.0 * m * n * k
        del a, b
    out["all"] = {"avg_us": total_us / len(shapes), "tflops": total_flops / total_us / 1e6}
    return out


def operand_path_yardstick(torch, nat, cfg, device, iters=10):
    """The library's own plain-store GEMM (lt_gemm) on the up-projection and dW2 shapes with its two operand paths: tiles
    copied HBM -> LDS without passing through registers (the product path) and tiles staged through registers (the only
    place where a LayerNorm or an activation could be applied to an operand on its way in).  What fusing LayerNorm into the
    up-projection's prologue, or recomputing the activation in the weight-gradient GEMM's prologue, would cost in GEMM time
    before any of the extra arithmetic."""
    tokens, hidden, inter = cfg["batch"] * cfg["seq"], cfg["hidden"], cfg["inter"]
    n1 = 2 * inter if cfg["gated"] else inter
    lib = nat.lib()
    out = {}
    for name, (m, n, k, a_km, b_km) in {"up": (tokens, n1, hidden, 1, 1), "dW2": (hidden, inter, tokens, 0, 0)}.items():
        a = (torch.randn(m * k, device=device) * 0.5).to(torch.bfloat16)
        b = (torch.randn(n * k, device=device) * 0.02).to(torch.bfloat16)
        c = torch.empty(m, n, dtype=torch.bfloat16, device=device)
        row = {"m": m, "n": n, "k": k}
        for label, force in (("copied_to_lds", 0), ("staged_through_registers", 2)):
            def run():
                nat.check(lib.lt_gemm(1, m, n, k, a.data_ptr(), a_km, b.data_ptr(), b_km, 1, c.data_ptr(), force,
                                      torch.cuda.current_stream().cuda_stream), "lt_gemm")
            for _ in range(3):
                run()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record()
            for _ in range(iters):
                run()
            stop.record()
            torch.cuda.synchronize()
            us = start.elapsed_time(stop) / iters * 1e3
            row[label] = {"avg_us": us, "tflops": 2.0 * m * n * k / us / 1e6}
        out[name] = row
        del a, b, c
    return out


def run_ffn_config(torch, lt, nat, name, steps, warmup, device):
    """K timed fwd+bwd steps of one LeanFFN configuration (wall clock between synchronisations, no per-kernel events), the
    same K steps again with a HIP event pair around every kernel launch, and the activation memory of one step"""
    cfg = CONFIGS[name]
    tokens = cfg["batch"] * cfg["seq"]
    ffn, x, dy = build_workload(torch, lt, cfg, device)
    params = list(ffn.parameters())

    def step():
        y = ffn(x)
        torch.autograd.grad(y, [x, *params], dy)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # peak activation memory of one fwd+bwd, relative to what is resident before it (parameters, x, dy)
    torch.cuda.reset_peak_memory_stats()
    base = torch.cuda.memory_allocated()
    y = ffn(x)
    torch.cuda.synchronize()
    saved_mb = (torch.cuda.memory_allocated() - base - y.numel() * y.element_size()) / 2**20
    torch.autograd.grad(y, [x, *params], dy)
    torch.cuda.synchronize()
    peak_mb = (torch.cuda.max_memory_allocated() - base) / 2**20
    del y

    lib = nat.lib(torch.float16 if cfg["dtype"] == "fp16" else None)
    lib.lt_profile_enable(0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    # the same K steps again with a HIP event pair around every kernel launch (recorded on the launch stream by the
    # library): per-kernel durations for the roofline.  The event packets cost about a percent, so `value` comes from the
    # run above.
    lib.lt_profile_reset()
    lib.lt_profile_enable(1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed_events = time.perf_counter() - t0
    lib.lt_profile_enable(0)
    kernels = nat.profile_read(lib)
    lib.lt_profile_reset()
    return dict(cfg=cfg, name=name, tokens=tokens, ffn=ffn, x=x, dy=dy, ms_per_step=elapsed / steps * 1e3,
                ms_events=elapsed_events / steps * 1e3, kernels=kernels, saved_mb=saved_mb, peak_mb=peak_mb)


def summarise(run, config_name):
    """throughput, kernel table and roofline object of one run_ffn_config result"""
    cfg, kernels, tokens, ms_per_step = run["cfg"], run["kernels"], run["tokens"], run["ms_per_step"]
    peak = PEAK_FP32_TFLOPS if cfg["dtype"] == "fp32" else PEAK_BF16_TFLOPS  # bf16 and fp16 share one dense peak
    tflops = algorithmic_flops(cfg) / (ms_per_step * 1e-3) / 1e12
    gemm = [k for k in kernels if k[0].startswith(("gemm_", "blocksparse_"))]
    gemm_flops, gemm_ms, gemm_launches = sum(k[3] for k in gemm), sum(k[2] for k in gemm), sum(k[1] for k in gemm)
    achieved = gemm_flops / (gemm_ms * 1e-3) / 1e12 if gemm_ms > 0 else 0.0
    kernel_table = [{"kernel": name, "launches": n, "avg_us": ms / n * 1e3,
                     **({"tflops": fl / (ms * 1e-3) / 1e12} if fl > 0 else {}),
                     **({"gbps": by / (ms * 1e-3) / 1e9} if by > 0 else {})} for name, n, ms, fl, by in kernels]
    # L2 <-> memory bytes per GEMM launch (fetch + write, averaged over the GEMM launches of a step), from the FETCH_SIZE
    # and WRITE_SIZE counter runs of this command summarised under profiles/ (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0 after
    # calibration on the dy cast kernel, a plain copy of known size)
    traffic, traffic_algorithmic, traffic_source = measured_traffic(config_name)
    roofline = {"bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s", "frac": achieved / peak,
                "traffic": traffic, "traffic_over_algorithmic": (traffic / traffic_algorithmic) if traffic else None,
                "traffic_source": traffic_source,
                "kernel": "all GEMM launches of a step: " + ", ".join(sorted({k[0] for k in gemm})),
                "flops_per_launch": gemm_flops / max(gemm_launches, 1),
                "avg_launch_us": gemm_ms / max(gemm_launches, 1) * 1e3}
    if cfg["sparse"] and traffic_algorithmic:
        # The block-sparse configuration is bound by memory traffic (its GEMM launches move 5 TB/s through the L2 boundary with
        # the matrix cores a quarter busy): priced against HBM with the launches' algorithmic bytes (every operand and result
        # once, from the same counter summary) over their measured duration.
        avg_launch_s = gemm_ms / max(gemm_launches, 1) * 1e-3
        roofline.update({"bound": "hbm", "achieved": traffic_algorithmic / avg_launch_s / 1e9, "peak": 8000.0,
                         "unit": "GB/s", "frac": traffic_algorithmic / avg_launch_s / 1e9 / 8000.0,
                         "mfma_tflops": achieved, "algorithmic_bytes_per_launch": traffic_algorithmic})
    return {"value": tokens / (ms_per_step * 1e-3), "ms_per_step": ms_per_step, "ms_per_step_with_kernel_events": run["ms_events"],
            "tflops": tflops, "mfma_util_pct": 100.0 * tflops / peak, "peak_activation_mb": run["peak_mb"],
            "saved_activation_mb": run["saved_mb"], "roofline": roofline, "kernels": kernel_table}


def run_c5(torch, nat, steps, warmup, device):
    """Configuration 5: a full GPT train step (vocab 10000, hidden 768, 12 layers, 16 heads, rotary, GeGLU 3072, tied
    embeddings, ids [16, 1024], labels = ids) under bf16 autocast with every FFN on the HIP kernels; the model around the
    FFN is the stock-PyTorch harness of the tests.  Reports the step time, what the FFN kernels take of it (the library's
    per-kernel events) and, outside the timed region, the same step with the oracle's stock-op FFN."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from gpt_harness import GPTConfig, MiniLeanGPT, copy_parameters

    cfg = GPTConfig()
    ids = torch.randint(0, cfg.vocab_size, (16, 1024), generator=torch.Generator().manual_seed(0)).to(device)
    model = MiniLeanGPT(cfg, "hip").to(device)

    def step(m):
        m.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            loss, _ = m(ids, labels=ids)
        loss.backward()

    def timed(m, n):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            step(m)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e3

    for _ in range(warmup):
        step(model)
    torch.cuda.reset_peak_memory_stats()
    step(model)
    torch.cuda.synchronize()
    peak_gib = torch.cuda.max_memory_allocated() / 2**30
    lib = nat.lib()
    lib.lt_profile_enable(0)
    ms_per_step = timed(model, steps)
    lib.lt_profile_reset()
    lib.lt_profile_enable(1)
    ms_events = timed(model, steps)
    lib.lt_profile_enable(0)
    kernels = nat.profile_read()
    lib.lt_profile_reset()
    # the same step with the oracle's stock-op FFN (same weights), outside the timed region
    stock = MiniLeanGPT(cfg, "oracle").to(device)
    copy_parameters(model, stock)
    for _ in range(2):
        step(stock)
    torch.cuda.reset_peak_memory_stats()
    stock_ms = timed(stock, max(2, steps // 4))
    stock_peak_gib = torch.cuda.max_memory_allocated() / 2**30
    tokens = ids.numel()
    H, I, L = cfg.hidden_size, cfg.intermediate_size, cfg.num_layers
    ffn_flops = 6.0 * tokens * H * (2 * I + I) * L  # fwd+bwd of the twelve GeGLU FFN blocks, no recompute counted
    gemm = [k for k in kernels if k[0].startswith(("gemm_", "blocksparse_"))]
    gemm_flops, gemm_ms, gemm_launches = sum(k[3] for k in gemm), sum(k[2] for k in gemm), sum(k[1] for k in gemm)
    ffn_kernel_ms = sum(k[2] for k in kernels) / steps
    achieved = gemm_flops / (gemm_ms * 1e-3) / 1e12
    kernel_table = [{"kernel": name, "launches": n, "avg_us": ms / n * 1e3,
                     **({"tflops": fl / (ms * 1e-3) / 1e12} if fl > 0 else {}),
                     **({"gbps": by / (ms * 1e-3) / 1e9} if by > 0 else {})} for name, n, ms, fl, by in kernels]
    return {
        "metric": METRIC, "value": tokens / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": ms_per_step, "ms_per_step_with_kernel_events": ms_events, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "config5: full GPT train step (fwd+bwd), vocab 10000, hidden 768, 12 layers, 16 heads, rotary, "
                               "GeGLU 3072, tied embeddings, ids [16,1024], bf16 autocast over fp32 parameters; FFN blocks on "
                               "the HIP kernels, the rest of the model stock PyTorch", "tokens": tokens, "hidden": H,
                   "intermediate": I, "layers": L},
        "ffn_kernel_ms_per_step": ffn_kernel_ms, "ffn_tflops_over_ffn_kernel_time": ffn_flops / (ffn_kernel_ms * 1e-3) / 1e12,
        "ffn_share_of_step": ffn_kernel_ms / ms_events, "peak_memory_gib": peak_gib,
        "same_step_with_stock_op_ffn": {"ms_per_step": stock_ms, "peak_memory_gib": stock_peak_gib},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": None,
                     "kernel": "all GEMM launches of the FFN blocks: " + ", ".join(sorted({k[0] for k in gemm})),
                     "flops_per_launch": gemm_flops / max(gemm_launches, 1), "avg_launch_us": gemm_ms / max(gemm_launches, 1) * 1e3},
        "kernels": kernel_table,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timing (profiling runs)")
    ap.add_argument("--no-reference-memory", action="store_true", help="skip the reference-schedule activation memory "
                    "measurement (the oracle's LeanFFNFunction under bf16 autocast on the GPU; profiling runs)")
    ap.add_argument("--no-extra-configs", action="store_true", help="skip configurations 2 and 4 (profiling runs)")
    ap.add_argument("--config", default="c3", choices=sorted(CONFIGS) + ["c5"], help="benchmark configuration (default: the "
                    "headline config 3; the others are reported for reference)")
    ap.add_argument("--yardstick", action="store_true", help="also time torch.matmul (vendor GEMM library, no epilogue) on "
                    "the six GEMM shapes of the step, for comparison (dense configurations)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no collectives and every box has one GPU (use --gpus 1)")

    import torch

    import lean_transformer_amd as lt
    from lean_transformer_amd import _native as nat

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    device = torch.device("cuda:0")
    if args.config == "c5":
        print(json.dumps(run_c5(torch, nat, args.steps, args.warmup, device)))
        return
    run = run_ffn_config(torch, lt, nat, args.config, args.steps, args.warmup, device)
    cfg, ffn, x, dy, tokens = run["cfg"], run["ffn"], run["x"], run["dy"], run["tokens"]
    hidden, inter = cfg["hidden"], cfg["inter"]
    flops_per_step = algorithmic_flops(cfg)
    summary = summarise(run, args.config)
    result = {
        "metric": METRIC, "value": summary["value"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": summary["ms_per_step"],
        "ms_per_step_with_kernel_events": summary["ms_per_step_with_kernel_events"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": {"bf16": "bf16", "fp16": "f16", "fp32": "f32"}[cfg["dtype"]], "data": "synthetic",
        "config": {"workload": cfg["name"], "tokens": tokens, "hidden": hidden, "intermediate": inter},
        "tflops": summary["tflops"], "mfma_util_pct": summary["mfma_util_pct"],
        "peak_activation_mb": summary["peak_activation_mb"], "saved_activation_mb": summary["saved_activation_mb"],
        "roofline": summary["roofline"], "kernels": summary["kernels"],
    }
    if cfg["sparse"]:
        # the oracle multiplies a dense expansion of the block-sparse weights: its memory says nothing about the reference's
        result["reference_saved_activation_mb"] = result["reference_peak_activation_mb"] = None
    elif not args.no_reference_memory:
        ref_saved, ref_peak = reference_activation_memory(torch, ffn, x, dy)
        result["reference_saved_activation_mb"] = ref_saved
        result["reference_peak_activation_mb"] = ref_peak
    if not args.no_cpu_baseline:
        torch.set_num_threads(min(os.cpu_count() or 1, 16))
        # bounded sample: about 25 s of host work (12 fwd+bwd) whatever the configuration
        per_token = flops_per_step / tokens if not cfg["sparse"] else 6.0 * hidden * (
            (2 * inter if cfg["gated"] else inter) + inter)  # the oracle multiplies the dense expansion of a sparse weight
        sample = int(min(tokens, max(256, 2048 * 1.208e9 / per_token)))
        value, sec = cpu_baseline(torch, ffn, x, dy, sample, warmup=2, iters=10)
        result["cpu_baseline"] = {
            "value": value, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle LeanFFNFunction (stock PyTorch fp32, reference save-set) on the first {sample} of {tokens} "
                      f"tokens of {args.config}, median of 10 fwd+bwd after 2 warm-ups, {sec:.2f} s each"}
    if args.yardstick and not cfg["sparse"] and cfg["dtype"] == "bf16":
        result["library_gemm_yardstick"] = library_gemm_yardstick(torch, cfg, device)
        result["operand_path_yardstick"] = operand_path_yardstick(torch, nat, cfg, device)
    if args.config == "c3" and not args.no_extra_configs:
        # the other single-GPU LeanFFN configurations, measured the same way in the same process (parity-test cases of their
        # own; `value` and `config` of this line stay configuration 3's)
        del run, ffn, x, dy
        torch.cuda.empty_cache()
        extra = {}
        for name in ("c2", "c4", "c4t"):
            other = run_ffn_config(torch, lt, nat, name, args.steps, args.warmup, device)
            entry = summarise(other, name)
            entry["config"] = {"workload": other["cfg"]["name"], "tokens": other["tokens"], "hidden": other["cfg"]["hidden"],
                               "intermediate": other["cfg"]["inter"]}
            entry["unit"] = "tokens/s"
            extra[name] = entry
            del other
            torch.cuda.empty_cache()
        result["extra_configs"] = extra
    print(json.dumps(result))


if __name__ == "__main__":
    main()
