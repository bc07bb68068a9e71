"""Builds the gfx950 kernel library in-tree with hipcc.

    python -m logismos_amd.build

produces ``logismos_amd/lib/liblogismos_kernels.so`` (the C-ABI declared in
``include/logismos_decode.h``) and ``liblogismos_kernels.a`` (the static
archive a Rust `kernels` build script would link, mirroring
crates/kernels/build.rs:71-124 of the reference with
``--offload-arch=gfx950`` and wave64).
"""
from __future__ import annotations

import glob
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
SO_PATH = os.path.join(LIBDIR, "liblogismos_kernels.so")
A_PATH = os.path.join(LIBDIR, "liblogismos_kernels.a")

OFFLOAD_ARCH = os.environ.get("LOGISMOS_OFFLOAD_ARCH", "gfx950")

# -packed-fp32-ops is switched off: the compiler must not form v_pk_*_f32.
HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=fast",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]


# Per-source additions.  paged_attn.hip: MFMA results stay in ordinary VGPRs (the
# kernels fit in 256 registers; the default accumulation-register form costs the
# prefill kernel ~50 register-to-register moves per key tile around its softmax).
EXTRA_FLAGS = {
    "paged_attn.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "qgemm_q4_splitk.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "qgemm_q4_stream.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "qgemm_q4_greedy.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "qgemm_q4g32.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def hipcc() -> str:
    exe = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe) and not shutil.which(exe):
        raise RuntimeError("hipcc not found (set HIPCC); the kernels cannot be built")
    return exe


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))


def _compile(src: str) -> str:
    obj = os.path.join(OBJDIR, os.path.basename(src) + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(os.path.basename(src), []), "-x", "hip", "-c",
           src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stderr}")
    noise = ("packed-fp32-ops", "is not a recognized feature")
    warn = [ln for ln in r.stderr.splitlines() if ln.strip() and not any(n in ln for n in noise)]
    if warn:
        sys.stderr.write("\n".join(warn) + "\n")
    return obj


def build(verbose: bool = True) -> str:
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        objs = list(ex.map(_compile, srcs))
    r = subprocess.run([hipcc(), f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC", "-o",
                        SO_PATH, *objs], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    if os.path.exists(A_PATH):
        os.remove(A_PATH)
    subprocess.run(["ar", "crs", A_PATH, *objs], check=True)
    if verbose:
        print(f"built {SO_PATH} from {len(srcs)} sources for {OFFLOAD_ARCH}")
    return SO_PATH


if __name__ == "__main__":
    build()
