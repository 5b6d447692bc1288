"""hipcc build of libnq_gfx950.so (the only native artefact of the package)."""
from __future__ import annotations

import os
import shutil
import subprocess
import tempfile
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libnq_gfx950.so")
SOURCES = ("nq_gemv.hip", "nq_stream.hip", "nq_gemm.hip", "nq_panel.hip", "nq_util.hip", "nq_api.hip")
# -packed-fp32-ops off: hipcc may otherwise fuse scalar float code into packed-fp32 instructions.
FLAGS = ("--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-munsafe-fp-atomics",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops")


def build(verbose: bool = False, extra_flags=(), out_path: str = LIB_PATH) -> str:
    """Compile every HIP source for gfx950 (one hipcc per source, side by side) and link the shared library
    in-tree.  Always recompiles."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    srcs = [os.path.join(CSRC, s) for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with tempfile.TemporaryDirectory(prefix="nq_build_") as tmpdir:
        def compile_one(src):
            obj = os.path.join(tmpdir, os.path.basename(src) + ".o")
            cmd = [hipcc, *FLAGS, *extra_flags, "-c", src, "-o", obj]
            res = subprocess.run(cmd, capture_output=True, text=True)
            if res.returncode != 0:
                raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
            if verbose and res.stderr:
                print(res.stderr)
            return obj

        with ThreadPoolExecutor(max_workers=min(len(srcs), os.cpu_count() or 1)) as pool:
            objs = list(pool.map(compile_one, srcs))
        tmp = out_path + ".tmp"
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("hipcc link failed:\n" + " ".join(cmd) + "\n" + res.stdout + res.stderr)
        os.replace(tmp, out_path)
    return out_path


if __name__ == "__main__":
    print(build(verbose=True))
