"""Builds libturbogpt.so (HIP kernels + engine, gfx950 only) in-tree with hipcc.

    python -m turbogpt_amd.build          # compile what changed, link
    python -m turbogpt_amd.build --force  # recompile everything
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
OBJ = CSRC / "_obj"
LIBRARY = HERE / "libturbogpt.so"
HOST_SOURCE = HERE / "host" / "train_bytes.cpp"
HOST_PROGRAM = HERE / "host" / "train_bytes"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-I", str(HERE.parent / "include")]


def _sources():
    return sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.cpp")))


def _headers_mtime():
    headers = list(CSRC.glob("*.h")) + list((HERE.parent / "include").glob("*.h"))
    return max((h.stat().st_mtime for h in headers), default=0)


def _compile(source, force):
    obj = OBJ / (source.name + ".o")
    newest = max(source.stat().st_mtime, _headers_mtime())
    if not force and obj.exists() and obj.stat().st_mtime >= newest:
        return obj
    cmd = [HIPCC, *FLAGS, "-c", str(source), "-o", str(obj)]
    if source.suffix == ".cpp":
        cmd.insert(1, "-x")
        cmd.insert(2, "hip")
    result = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    errors = "\n".join(line for line in result.stderr.splitlines() if noise not in line)
    if result.returncode:
        raise RuntimeError(f"hipcc failed on {source.name}:\n{errors}")
    if errors.strip():
        print(errors, file=sys.stderr)
    return obj


def build_host():
    """The host program over the C ABI (host/train_bytes.cpp), with plain g++ against the library."""
    cmd = [os.environ.get("CXX", "g++"), "-std=c++17", "-O2", "-Wall", "-Wextra", "-I", str(HERE.parent / "include"),
           str(HOST_SOURCE), "-L", str(HERE), "-lturbogpt", "-Wl,-rpath,$ORIGIN/..", "-Wl,-rpath-link,/opt/rocm/lib",
           "-o", str(HOST_PROGRAM)]
    result = subprocess.run(cmd, capture_output=True, text=True)
    if result.returncode:
        raise RuntimeError(f"g++ failed on {HOST_SOURCE.name}:\n{result.stderr}")
    return HOST_PROGRAM


def build(force=False, jobs=8):
    OBJ.mkdir(exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = list(pool.map(lambda s: _compile(s, force), _sources()))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIBRARY), *map(str, objects)]
    subprocess.run(cmd, check=True)
    build_host()
    return LIBRARY


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
