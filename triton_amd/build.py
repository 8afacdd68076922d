"""Build the gfx950 kernel library (`csrc/*.hip` -> `csrc/libmi355_kernels.so`) with hipcc.

Plain ahead-of-time compilation: the reference compiles its kernels at first launch through a
JIT (python/triton/runtime/jit.py:642-648); here every kernel is a fixed HIP source, so the
"compiler" is one hipcc invocation per file and a link.  Run as `python -m triton_amd.build`.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent / "csrc"
LIB_NAME = "libmi355_kernels.so"
ARCH = "gfx950"

# -packed-fp32-ops off: packed fp32 VALU forms are not used by these kernels.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-ignored-attributes",
    # keeps the device assembly (<stem>-hip-amdgcn-amd-amdhsa-gfx950.s) next to the object files: the kernels issue
    # MFMAs, LDS reads and direct global->LDS loads as inline assembly, which the compiler's hazard recogniser cannot
    # see into, so tests/test_isa_hazards.py checks the generated code of every kernel instead
    "-save-temps=obj",
]

# Per-file additions.  The attention kernels rescale their MFMA accumulators with VALU code every
# key/value block, so the accumulators must live in architectural VGPRs: left to itself the
# register allocator parks them in AGPRs and spends more VALU issue slots on
# v_accvgpr_read/write pairs than on the softmax.
EXTRA_FLAGS = {
    "attn_fwd.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "attn_bwd.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm)")


def lib_path() -> Path:
    return CSRC / LIB_NAME


def _compile(hipcc: str, src: Path, obj: Path, verbose: bool) -> None:
    cmd = [hipcc, *HIPCC_FLAGS, *EXTRA_FLAGS.get(src.name, []), "-c", str(src), "-o", str(obj)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass prints a harmless note about the device-only target feature
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{err}")
    if verbose and err.strip():
        print(err, flush=True)


def build(verbose: bool = False, jobs: int | None = None) -> Path:
    """Compile every csrc/*.hip and link the shared library; always recompiles."""
    hipcc = hipcc_path()
    objdir = CSRC / "_build"
    objdir.mkdir(exist_ok=True)
    srcs = sorted(CSRC.glob("*.hip"))
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    objs = [objdir / (s.stem + ".o") for s in srcs]
    jobs = jobs or min(8, len(srcs), os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda so: _compile(hipcc, so[0], so[1], verbose), zip(srcs, objs)))
    out = lib_path()
    tmp = out.with_suffix(".so.tmp")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, out)
    try:
        build_torch_extension(verbose)
    except Exception as e:   # the operators then bind the C ABI through ctypes (_lib.ext() returns None)
        import warnings

        ext_path().unlink(missing_ok=True)   # never leave an extension of an older build next to a new library
        warnings.warn(f"PyTorch-ROCm extension not built, the operators will use the ctypes binding: {e}")
    return out


EXT_SRC = Path(__file__).resolve().parent / "csrc_ext" / "torch_ext.cpp"
EXT_NAME = "_mi355_torch"


def ext_path() -> Path:
    return Path(__file__).resolve().parent / (EXT_NAME + ".so")


def build_torch_extension(verbose: bool = False) -> Path:
    """Compile the PyTorch-ROCm extension (host C++ only: tensor checks, current stream, one C-ABI call per
    operator) with g++ against the installed torch and link it to the kernel library next to it."""
    import sysconfig

    from torch.utils import cpp_extension as ce

    out = ext_path()
    tmp = out.with_suffix(".so.tmp")
    inc = [sysconfig.get_paths()["include"], *ce.include_paths("cuda"), "/opt/rocm/include"]
    libdirs = ce.library_paths("cuda")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-DTORCH_EXTENSION_NAME={EXT_NAME}", "-DTORCH_API_INCLUDE_EXTENSION_H", "-Wno-deprecated-declarations",
           *[f"-I{i}" for i in inc], str(EXT_SRC), "-o", str(tmp),
           *[f"-L{d}" for d in libdirs], f"-L{CSRC}", "-lc10", "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10_hip", "-ltorch_hip",
           "-l:" + LIB_NAME, "-Wl,-rpath,$ORIGIN/csrc", *[f"-Wl,-rpath,{d}" for d in libdirs]]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"torch extension build failed:\n{res.stderr[-4000:]}")
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    p = build(verbose="-v" in sys.argv)
    print(p)
