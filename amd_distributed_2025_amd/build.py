"""Build the native code in-tree for gfx950.

`python -m amd_distributed_2025_amd.build` runs both steps:

`build_library()` runs hipcc on `csrc/moe_a2a.hip` and leaves `libmoe_a2a.so`
(the C ABI of include/moe_a2a.h) next to this file. hipcc cross-compiles, so no
GPU is needed to build.

`build_extension()` compiles the torch::Tensor wrappers of
`csrc/moe_a2a_torch.cpp` with `torch.utils.cpp_extension.load_inline`, the way
the reference's submissions build their kernels (all2all/hipv8.py:241-252), into
`_ext/moe_a2a_torch.so`, linked against `libmoe_a2a.so`. The build directory is
in the package so that the module travels with the tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
REPO_DIR = PKG_DIR.parent
SOURCE = PKG_DIR / "csrc" / "moe_a2a.hip"
LIBRARY = PKG_DIR / "libmoe_a2a.so"
EXT_SOURCE = PKG_DIR / "csrc" / "moe_a2a_torch.cpp"
EXT_DIR = PKG_DIR / "_ext"
EXT_NAME = "moe_a2a_torch"
# the wrappers load_inline binds, one per entry point of the C ABI
EXT_FUNCTIONS = ["a2a_version", "a2a_dispatch_send", "a2a_plan_send", "a2a_dispatch_recv", "a2a_combine_send",
                 "a2a_combine_recv", "a2a_expert_scale", "a2a_expert_gemm", "a2a_linear", "a2a_exchange_local",
                 "a2a_exchange_gather_local", "a2a_dispatch_recv_compact", "a2a_expert_scale_compact",
                 "a2a_expert_gemm_compact", "a2a_combine_send_compact"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # a soname lets the dynamic loader match an already loaded copy when the extension asks for it
    "-Wl,-soname,libmoe_a2a.so",
    # parity with torch's separate multiply and add needs un-fused arithmetic
    "-ffp-contract=off",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def source_id() -> str:
    """What `moe_a2a_build_id()` of a library built from the present sources returns."""
    import hashlib

    h = hashlib.sha256(SOURCE.read_bytes())
    h.update((REPO_DIR / "include" / "moe_a2a.h").read_bytes())
    return h.hexdigest()[:16]


def build_library(verbose: bool = False) -> Path:
    """Compile unconditionally and return the path of the shared library."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, f'-DMOE_A2A_BUILD_ID="{source_id()}"', f"-I{REPO_DIR / 'include'}",
           str(SOURCE), "-o", str(LIBRARY)]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the gfx feature named above and says so; drop that line
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, flush=True)
    return LIBRARY


def build_extension(verbose: bool = False) -> Path:
    """Compile the torch::Tensor wrappers with load_inline and return the path of the module.
    Needs `libmoe_a2a.so` (it is linked in by name and found next to the package at run time)."""
    if not LIBRARY.exists():
        raise RuntimeError(f"{LIBRARY} is missing: build_library() first")
    from torch.utils.cpp_extension import load_inline

    EXT_DIR.mkdir(exist_ok=True)
    load_inline(
        name=EXT_NAME,
        cpp_sources=[EXT_SOURCE.read_text()],
        functions=EXT_FUNCTIONS,
        extra_cflags=["-O2", "-std=c++17"],
        extra_include_paths=[str(REPO_DIR / "include")],
        # $ORIGIN/.. is the package directory as seen from _ext/ ($$ is ninja's escape for $)
        extra_ldflags=[f"-L{PKG_DIR}", "-l:libmoe_a2a.so", "-Wl,-rpath,'$$ORIGIN/..'"],
        build_directory=str(EXT_DIR),
        with_cuda=False,
        is_python_module=True,
        verbose=verbose,
    )
    built = EXT_DIR / f"{EXT_NAME}.so"
    if not built.exists():
        raise RuntimeError(f"load_inline did not leave {built}")
    return built


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_extension(verbose=True))
