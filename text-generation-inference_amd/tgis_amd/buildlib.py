"""Compiles csrc/*.hip into the C-ABI library with hipcc (gfx950; cross-compiles without a GPU).

`compile_library()` builds everything into lib/libtgis_hip.so.  `compile_library(units=FAMILY_UNITS[family])` builds only the
translation units one model family's path calls, into lib/libtgis_hip.<family>.so: what a fresh checkout compiles when it is
asked to serve that family before anything else was built (`native.load_library` binds the symbols such a library has and
reports a missing one when it is called)."""
import glob
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor
from typing import Optional, Sequence

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# translation units per family (api.hip: error state / version; elementwise.hip: decode bookkeeping, argmax)
FAMILY_UNITS = {
    "lenisun": ["api", "elementwise", "gemm_dense", "residual_f32", "attn_varlen", "wkv", "moe", "sampler"],
    "senadra": ["api", "elementwise", "gemm_dense", "residual_f32", "attn_varlen", "delta_rule", "sampler"],
    "mananex": ["api", "elementwise", "gemm_dense", "residual_f32", "attn_varlen", "gated_linear_scan", "moe", "sampler"],
    "tatevik": ["api", "elementwise", "gemm_dense", "residual_f32", "norm_f32", "attn_varlen", "attn_mixed_heads", "gated_linear_scan",
                "selective_scan", "causal_conv", "moe", "sampler"],
}


def library_path(family: Optional[str] = None) -> str:
    return os.path.join(LIB_DIR, f"libtgis_hip.{family}.so" if family else "libtgis_hip.so")


def compile_library(units: Optional[Sequence[str]] = None, out: Optional[str] = None, jobs: Optional[int] = None) -> str:
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip"))) if units is None else [os.path.join(CSRC, u + ".hip") for u in units]
    out = out or library_path()
    objdir = os.path.join(LIB_DIR, "obj")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, os.path.basename(src)[:-4] + ".o")
        subprocess.run(["hipcc", *FLAGS, "-c", src, "-o", obj], check=True, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE)
        return obj

    workers = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", 0)) or os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=workers) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp = out + f".{os.getpid()}.tmp"
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs], check=True)
    os.replace(tmp, out)  # a reader never sees a half-written library
    return out
