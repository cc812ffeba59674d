"""Builds libvqattn_gfx950.so in-tree with hipcc (cross-compiles for gfx950; no GPU needed)."""
import glob
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libvqattn_gfx950.so")

HIPCC_FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Wall",
    "-Wno-unused-function",
    "-Wno-inline-asm",
    # packed fp32 VALU ops stay off for device code
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC_DIR, "*.hip")))


def _compile(cmd):
    # communicate() drains the compiler's output while it runs, so a long warning log cannot block the child
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return proc.returncode, proc.stdout


def build(verbose: bool = True, jobs: int = 8) -> str:
    """Compile every csrc/*.hip into objects (in parallel) and link the shared library.  Always recompiles."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)
    flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    srcs = sources()
    objs = [os.path.join(obj_dir, os.path.basename(src) + ".o") for src in srcs]
    cmds = [[hipcc, *flags, "-c", src, "-o", obj] for src, obj in zip(srcs, objs)]
    if verbose:
        for cmd in cmds:
            print(" ".join(cmd), flush=True)
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        results = list(pool.map(_compile, cmds))
    failed = False
    for src, (rc, out) in zip(srcs, results):
        lines = [l for l in out.splitlines() if "is not a recognized feature for this target" not in l]
        if rc != 0:
            failed = True
            print(f"FAILED: {src}\n" + "\n".join(lines), file=sys.stderr)
        elif verbose and lines:
            print("\n".join(lines))
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


if __name__ == "__main__":
    build()
