"""Build libllmq_gfx950.so (gfx950 only) from the HIP sources in this directory.

    python -m llmqrt_amd.csrc.build          # or: python llmqrt_amd/csrc/build.py

hipcc cross-compiles without a GPU.  Each translation unit is compiled to an object in
parallel, then linked into llmqrt_amd/lib/libllmq_gfx950.so.
"""
import concurrent.futures
import pathlib
import subprocess
import sys

HERE = pathlib.Path(__file__).resolve().parent
ROOT = HERE.parent.parent
OUT_DIR = HERE.parent / "lib"
OBJ_DIR = OUT_DIR / "obj"
LIB = OUT_DIR / "libllmq_gfx950.so"
MICROBENCH_LIB = OUT_DIR / "libllmq_microbench_gfx950.so"  # hardware microbenchmarks for `bench.py --micro`; not the product
# the tile GEMM is instantiated per operand format in four translation units (the long poles of the build), listed first
SOURCES = ["gemm_tile_i8.hip", "gemm_tile_fp8.hip", "gemm_tile_fp8_e5m2.hip", "gemm_tile_f16.hip", "gemm_mfma.hip", "abi.hip",
           "quant.hip", "gemm_skinny.hip", "linear_fused.hip", "awq.hip", "awq_decode.hip", "awq_tile.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-fp32 VALU ops are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",  # the LDS-DMA asm names m0 as clobbered on purpose
    f"-I{ROOT / 'include'}", f"-I{HERE}",
]


def _compile(src: str) -> pathlib.Path:
    obj = OBJ_DIR / (src.replace(".hip", ".o"))
    cmd = ["hipcc", *HIPCC_FLAGS, "-c", str(HERE / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warn:
        sys.stderr.write(warn + "\n")
    return obj


def _link(lib: pathlib.Path, objs) -> None:
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(lib), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")


def build(verbose: bool = True) -> pathlib.Path:
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=6) as ex:
        objs = list(ex.map(_compile, SOURCES + ["microbench.hip"]))
    _link(LIB, objs[:-1])
    _link(MICROBENCH_LIB, objs[-1:])
    if verbose:
        print(f"built {LIB}\nbuilt {MICROBENCH_LIB}")
    return LIB


if __name__ == "__main__":
    build()
