#!/usr/bin/env python3
"""Build the kserve_amd_C native extension in-tree for gfx950.

Kernels (.hip) are compiled by hipcc directly (pure CDNA4 HIP, no torch
coupling, no hipify); bindings.cpp compiles against torch's ROCm headers and
links the objects into kserve_amd_C.so at the repo root — the .so travels to
GPU boxes with the source snapshot.

Usage: python build_hip.py [--force] [module ...]
"""

import os
import subprocess
import sys

REPO = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(REPO, "kserve_amd", "ops", "csrc")
BUILD = os.path.join(REPO, "build", "hip")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = os.environ.get("PYTORCH_ROCM_ARCH", "gfx950")

# Extension modules. Each is one .so at the repo root, linked from its own
# kernel objects and bindings file, so a model family compiles only the module
# whose mechanisms it uses. `fast_math` stays off where kernels sit on a
# model's 32-bit path (exact exp/log/sqrt/division).
MODULES = {
    "kserve_amd_C": {
        "sources": [
            "rmsnorm.hip",
            "layernorm.hip",
            "activation.hip",
            "rope.hip",
            "kv_cache.hip",
            "attention_decode.hip",
            "attention_prefill.hip",
            "sampling.hip",
            "skinny_gemm.hip",
            "gemm8.hip",
            "mfma_probe.hip",
        ],
        "bindings": "bindings.cpp",
        "fast_math": True,
    },
    "kserve_amd_seq_C": {
        "sources": [
            "residual_norm_f32.hip",
            "ssm_scan.hip",
            "linear_scan.hip",
            "attention_f32.hip",
            "latent_attention.hip",
            "moe_route.hip",
            "activation.hip",
            "sampling.hip",
        ],
        "bindings": "bindings_seq.cpp",
        "fast_math": False,
    },
}

HEADERS = ["common.h", "mfma_layouts.h", "dtype_io.h"]
# hipcc makes packed-fp32 instructions on its own from plain float code; keep
# them off for every kernel of this package
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def newer(src, dst):
    return not os.path.exists(dst) or os.path.getmtime(src) > os.path.getmtime(dst)


def so_path(module: str) -> str:
    return os.path.join(REPO, module + ".so")


def build_module(module: str, force: bool = False, jobs: int = 8) -> str:
    import sysconfig
    from concurrent.futures import ThreadPoolExecutor

    import torch

    spec = MODULES[module]
    out_so = so_path(module)
    bdir = os.path.join(BUILD, module)
    os.makedirs(bdir, exist_ok=True)
    torch_dir = os.path.dirname(torch.__file__)
    torch_inc = [
        os.path.join(torch_dir, "include"),
        os.path.join(torch_dir, "include", "torch", "csrc", "api", "include"),
    ]
    py_inc = sysconfig.get_paths()["include"]
    headers = [os.path.join(CSRC, h) for h in HEADERS]

    cmds = []
    objs = []
    for src in spec["sources"]:
        src_path = os.path.join(CSRC, src)
        obj = os.path.join(bdir, src.replace(".hip", ".o"))
        objs.append(obj)
        if force or newer(src_path, obj) or any(newer(h, obj) for h in headers):
            cmd = [
                HIPCC, "-c", src_path, "-o", obj,
                f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC",
            ] + DEVICE_FLAGS
            if spec["fast_math"]:
                cmd.append("-ffast-math")
            cmds.append(cmd)

    bind_src = os.path.join(CSRC, spec["bindings"])
    bind_obj = os.path.join(bdir, "bindings.o")
    bind_hdr = os.path.join(CSRC, "bindings_common.h")
    if force or newer(bind_src, bind_obj) or newer(bind_hdr, bind_obj):
        cmd = [
            HIPCC, "-c", bind_src, "-o", bind_obj,
            "-O2", "-std=c++17", "-fPIC",
            "-D_GLIBCXX_USE_CXX11_ABI=1",
            f"-DTORCH_EXTENSION_NAME={module}",
            "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__",
            "-DTORCH_API_INCLUDE_EXTENSION_H",
            f"-I{py_inc}",
        ]
        cmd += [f"-I{d}" for d in torch_inc]
        cmds.append(cmd)
    objs.append(bind_obj)

    # translation units are independent: compile them side by side
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        list(pool.map(run, cmds))

    if force or any(newer(o, out_so) for o in objs):
        tmp = out_so + f".tmp{os.getpid()}"
        run([
            HIPCC, "-shared", "-o", tmp, *objs,
            f"-L{os.path.join(torch_dir, 'lib')}",
            "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10",
            "-ltorch_hip", "-lc10_hip", "-lamdhip64",
            f"-Wl,-rpath,{os.path.join(torch_dir, 'lib')}",
        ])
        os.replace(tmp, out_so)  # never expose a half-written library
    print(f"built {out_so}", flush=True)
    return out_so


def build(force: bool = False, modules=None) -> str:
    out = None
    for module in modules or list(MODULES):
        out = build_module(module, force=force)
    return out


def ensure_built(modules) -> None:
    """Build the named modules if their libraries are absent (first use in a
    fresh checkout). Serialised across processes by a lock file."""
    missing = [m for m in modules if not os.path.exists(so_path(m))]
    if not missing:
        return
    import fcntl

    os.makedirs(BUILD, exist_ok=True)
    with open(os.path.join(BUILD, ".lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        for m in missing:
            if not os.path.exists(so_path(m)):
                build_module(m)


if __name__ == "__main__":
    names = [a for a in sys.argv[1:] if not a.startswith("-")]
    build(force="--force" in sys.argv, modules=names or None)
