"""Builds libflexattn.so (gfx950) in-tree with hipcc.  Usage: python -m flex_attention_tpu_amd.build"""
from __future__ import annotations

import concurrent.futures
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(os.path.dirname(PKG_DIR), "include")
BUILD_DIR = os.path.join(CSRC, "_build")
LIB_PATH = os.path.join(PKG_DIR, "libflexattn.so")

SOURCES = [
    "api.hip",
    "block_mask.hip",
    "delta.hip",
    "attn_f32.hip",
    "attn_f32_mfma.hip",
    "fwd_bf16.hip",
    "bwd_dq_bf16.hip",
    "bwd_dkv_bf16.hip",
    "bwd_dq_ds.hip",
]

# instruction streams generated before compiling: (generator script, output it writes next to itself)
GENERATED = [("gen_dkv_tile.py", "bwd_dkv_tile.inc"), ("gen_dq_tile.py", "bwd_dq_tile.inc"),
             ("gen_fwd_tile.py", "fwd_tile.inc")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffast-math",
    "-fno-finite-math-only",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def _compile(src: str, force: bool, build_dir: str = BUILD_DIR, extra_flags=()) -> str:
    obj = os.path.join(build_dir, os.path.splitext(src)[0] + ".o")
    src_path = os.path.join(CSRC, src)
    if not force and os.path.exists(obj):
        deps = [src_path] + [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hpp", ".inc"))]
        deps.append(os.path.join(INCLUDE, "flexattn.h"))
        if all(os.path.getmtime(d) <= os.path.getmtime(obj) for d in deps):
            return obj
    cmd = [HIPCC, *FLAGS, *extra_flags, "-c", src_path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if warn:
        sys.stderr.write(warn + "\n")
    return obj


def generate_streams(out_dir: str = CSRC) -> None:
    """Runs the stream generators; each writes its include file into `out_dir` (written under a temporary name
    and moved into place, so that a compiler running in another process never reads half a file)."""
    for gen, out in GENERATED:
        final = os.path.join(out_dir, out)
        tmp = f"{final}.{os.getpid()}.tmp"
        r = subprocess.run([sys.executable, os.path.join(CSRC, gen), tmp], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"{gen} failed:\n{r.stdout}\n{r.stderr}")
        os.replace(tmp, final)


def build_library(force: bool = True, jobs: int = 8, out_path: str = LIB_PATH, build_dir: str = BUILD_DIR,
                  extra_flags=(), include_dir: str = CSRC) -> str:
    """Compiles every HIP source for gfx950 and links libflexattn.so next to the package (or, with
    `out_path` / `build_dir` / `extra_flags`, a functor library of compiler.py against its generated header).
    `include_dir`: where the generated streams go (a functor library writes its copy into its own build
    directory and nothing into the package; the compiler takes the package's copy, the same text, where one
    lies next to the sources, and this one otherwise).  The library is linked under a temporary name
    and moved into place: a process that finds the file finds a complete one."""
    os.makedirs(build_dir, exist_ok=True)
    generate_streams(include_dir)
    inc = (f"-I{include_dir}",) if include_dir != CSRC else ()
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force, build_dir, inc + tuple(extra_flags)), SOURCES))
    tmp = f"{out_path}.{os.getpid()}.tmp"
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, out_path)
    return out_path


if __name__ == "__main__":
    print(build_library(force="--incremental" not in sys.argv))
