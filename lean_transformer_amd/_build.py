"""Builds lean_transformer_amd/csrc/libleanffn.so and libleanffn_f16.so from the HIP sources with hipcc for gfx950
(cross-compiles without a GPU).  The two libraries are the same sources with the 16-bit element type fixed at compile time:
bfloat16 in the first, IEEE binary16 (-DLT_HALF_IS_FP16) in the second.

    python -m lean_transformer_amd._build            # both
    python -m lean_transformer_amd._build --bf16     # libleanffn.so only
    python -m lean_transformer_amd._build --f16      # libleanffn_f16.so only
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(CSRC, "libleanffn.so")
# the tiled GEMM kernels are instantiated per epilogue kind in four translation units so that they compile in parallel
SOURCES = ["gemm_mfma_kind0.hip", "gemm_mfma_kind1.hip", "gemm_mfma_kind2.hip", "gemm_mfma_kind3.hip", "gemm_generic.hip",
           "elementwise.hip", "ffn.hip", "gemm_mfma_bf16.hip", "profile.hip"]
# -packed-fp32-ops is switched off: the compiler must not form v_pk_{add,mul,fma}_f32 from scalar float code
# -pragma-unroll-threshold: the fused GEMM epilogues index the accumulator registers from fully unrolled loops; left rolled
# (the default threshold is too small for them) the accumulators would be demoted to scratch memory
FLAGS = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-mllvm", "-pragma-unroll-threshold=100000", "-Wno-unused-command-line-argument",
         "-Wno-unknown-warning-option"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + proc.stdout)
    return proc.stdout


F16_LIB_PATH = os.path.join(CSRC, "libleanffn_f16.so")
TILE_TIMING_LIB_PATH = os.path.join(CSRC, "libleanffn_tile_timing.so")


def build_all(verbose: bool = False) -> list:
    """Both libraries, their translation units compiled side by side; returns their paths."""
    with ThreadPoolExecutor(max_workers=2) as pool:
        futures = [pool.submit(build, verbose=verbose, f16=f16, workers=4) for f16 in (False, True)]
        return [f.result() for f in futures]


def build(verbose: bool = False, extra_flags=(), tile_timing: bool = False, f16: bool = False, workers: int = 8) -> str:
    """Compile every translation unit (in parallel) and link the shared library; returns its path.

    f16: build libleanffn_f16.so, whose 16-bit element type is IEEE binary16, instead of the bfloat16 library.

    tile_timing: build the instrumented library instead (csrc/libleanffn_tile_timing.so, -DLT_TILE_TIMING: the copy-based
    GEMM kernels record per-workgroup phase timestamps; read by tile_timing.py at the repository root).  Never loaded by the
    package itself."""
    hipcc = _hipcc()
    if tile_timing and f16:
        raise ValueError("the instrumented library is built for bfloat16 only")
    suffix = ".tile_timing.o" if tile_timing else ".f16.o" if f16 else ".o"
    lib_path = TILE_TIMING_LIB_PATH if tile_timing else F16_LIB_PATH if f16 else LIB_PATH
    if tile_timing:
        extra_flags = (*extra_flags, "-DLT_TILE_TIMING")
    if f16:
        extra_flags = (*extra_flags, "-DLT_HALF_IS_FP16")
    objects = [os.path.join(CSRC, src.replace(".hip", suffix)) for src in SOURCES]

    def compile_one(pair):
        src, obj = pair
        out = _run([hipcc, *FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)

    with ThreadPoolExecutor(max_workers=min(os.cpu_count() or 4, workers, len(SOURCES))) as pool:
        list(pool.map(compile_one, zip(SOURCES, objects)))
    _run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *objects, "-o", lib_path])
    return lib_path


if __name__ == "__main__":
    if "--tile-timing" in sys.argv:
        print(build(verbose="-v" in sys.argv, tile_timing=True))
    elif "--bf16" in sys.argv or "--f16" in sys.argv:
        print(build(verbose="-v" in sys.argv, f16="--f16" in sys.argv))
    else:
        print(*build_all(verbose="-v" in sys.argv), sep="\n")
