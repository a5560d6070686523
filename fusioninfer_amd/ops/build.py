"""In-tree build of the CDNA4 HIP extension (gfx950 only, no hipify).

Drives hipcc directly — no CUDA compatibility layer, no JIT cache: the
resulting ``_C.so`` lives next to this file so the gpurun snapshot carries it.

Two extensions, so that a model family compiles only what it runs:

  core    -> _C.so         transformer kernels
  seqmix  -> _C_seqmix.so  sequence-mixer kernels (ops/seqmix.py)
  moe     -> _C_moe.so     expert-routing kernels (ops.moe_*)

Usage:  python -m fusioninfer_amd.ops.build [core|seqmix|moe|all] [--force]
"""

from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

OPS_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(OPS_DIR, "csrc")
SO_PATH = os.path.join(OPS_DIR, "_C.so")

SOURCES = [
    "ops.hip",
    "norm.hip",
    "activation.hip",
    "quant.hip",
    "rope.hip",
    "cache.hip",
    "paged_attention.hip",
    "prefill_attention.hip",
]

MOE_SOURCES = [
    "moe_bindings.hip",
    "moe_gemm.hip",
    "moe_plain.hip",
]


SEQMIX_SOURCES = [
    "seqmix_bindings.hip",
    "seqmix_norm.hip",
    "seqmix_attention.hip",
    "seqmix_delta.hip",
    "seqmix_stream.hip",
    "seqmix_linear.hip",
    "seqmix_window.hip",
    "seqmix_parallel.hip",
    "seqmix_sink.hip",
    "seqmix_postnorm.hip",
]

EXTENSIONS = {
    "core": ("_C", SOURCES, ["common.h"]),
    "seqmix": ("_C_seqmix", SEQMIX_SOURCES, ["common.h", "seqmix.h"]),
    "moe": ("_C_moe", MOE_SOURCES, ["common.h", "seqmix.h"]),
}


def extension_path(ext: str) -> str:
    return os.path.join(OPS_DIR, EXTENSIONS[ext][0] + ".so")


def build(verbose: bool = True, force: bool = False) -> str:
    """The core extension (kept as the historical entry point)."""
    return build_extension("core", verbose=verbose, force=force)


def build_extension(ext: str, verbose: bool = True,
                    force: bool = False) -> str:
    import torch
    from torch.utils import cpp_extension as ce

    mod_name, sources, headers = EXTENSIONS[ext]
    SO_PATH = extension_path(ext)
    srcs = [os.path.join(CSRC, s) for s in sources]
    hdrs = [os.path.join(CSRC, h) for h in headers]
    if not force and os.path.exists(SO_PATH):
        so_mtime = os.path.getmtime(SO_PATH)
        if all(os.path.getmtime(f) < so_mtime for f in srcs + hdrs):
            return SO_PATH
    # build next to the target and rename: a concurrent reader never sees
    # a half-written library
    final_path, SO_PATH = SO_PATH, SO_PATH + ".%d.tmp" % os.getpid()

    hipcc = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")
    torch_lib = ce.library_paths()[0]
    cmd = [
        hipcc,
        "--offload-arch=gfx950",
        "-O3",
        "-std=c++17",
        "-shared",
        "-fPIC",
        f"-DTORCH_EXTENSION_NAME={mod_name}",
        # packed-fp32 VALU forms are kept out of generated code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-DTORCH_API_INCLUDE_EXTENSION_H",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        *getattr(ce, "COMMON_HIP_FLAGS", ["-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1"]),
        "-DHIP_ENABLE_WARP_SYNC_BUILTINS",
        *[f"-I{p}" for p in ce.include_paths()],
        f"-I{sysconfig.get_paths()['include']}",
        f"-I{CSRC}",
        *srcs,
        f"-L{torch_lib}",
        f"-Wl,-rpath,{torch_lib}",
        "-ltorch",
        "-ltorch_python",
        "-lc10",
        "-ltorch_hip",
        "-lc10_hip",
        "-lamdhip64",
        "-o",
        SO_PATH,
    ]
    if verbose:
        print("[fusioninfer build]", " ".join(cmd), file=sys.stderr)
    subprocess.run(cmd, check=True,
                   stdout=None if verbose else subprocess.DEVNULL,
                   stderr=None if verbose else subprocess.DEVNULL)
    os.replace(SO_PATH, final_path)
    return final_path


if __name__ == "__main__":
    which = [a for a in sys.argv[1:] if not a.startswith("-")] or ["all"]
    names = list(EXTENSIONS) if "all" in which else which
    for name in names:
        print(build_extension(name, force="--force" in sys.argv))
