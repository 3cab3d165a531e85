"""On-demand, in-tree build of one HIP extension.

The full extension set is built ahead of time by ``setup.py build_ext
--inplace``; this module covers the case of a checkout with nothing built
(a fresh clone on a GPU box): the first use of a kernel family compiles just
that family's sources with hipcc for gfx950 and drops the module next to the
package, so later processes import it directly. A digest of the sources is
kept beside the module; a module whose digest no longer matches its sources
is rebuilt instead of being loaded stale.
"""

from __future__ import annotations

import fcntl
import hashlib
import importlib
import importlib.util
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from typing import List

PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REPO_DIR = os.path.dirname(PKG_DIR)
HIP_DIR = os.path.join(PKG_DIR, "ops", "hip")

# every HIP translation unit is compiled with packed-fp32 instruction
# selection switched off
HIP_FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

EXTENSIONS = {
    "_C_seq": {
        "dir": os.path.join(HIP_DIR, "seq"),
        # the dense MFMA prefill kernel is shared with _C (one source, two modules)
        "kernels": ["seq_norm.hip", "seq_attn.hip", "seq_recurrent.hip", "seq_parallel.hip", "seq_gated.hip",
                    "seq_latent.hip", "seq_stream.hip", "../attn_prefill.hip"],
        "bindings": ["seq_bindings.hip"],
        "headers": ["seq_common.h"],
    },
}


def _hipcc() -> str:
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cand = os.path.join(rocm, "bin", "hipcc")
    return cand if os.path.exists(cand) else "hipcc"


def module_path(name: str) -> str:
    return os.path.join(PKG_DIR, name + sysconfig.get_config_var("EXT_SUFFIX"))


def source_digest(name: str) -> str:
    ext = EXTENSIONS[name]
    h = hashlib.sha256(" ".join(HIP_FLAGS).encode())
    shared = ["../common.h"] if any(f.startswith("../") for f in ext["kernels"]) else []
    for f in ext["headers"] + shared + ext["kernels"] + ext["bindings"]:
        with open(os.path.join(ext["dir"], f), "rb") as fh:
            h.update(f.encode() + b"\0" + fh.read())
    return h.hexdigest()


def is_current(name: str) -> bool:
    so = module_path(name)
    try:
        with open(so + ".digest") as f:
            return os.path.exists(so) and f.read().strip() == source_digest(name)
    except OSError:
        return False


def build(name: str, verbose: bool = False) -> str:
    """Compile extension ``name`` in-tree (always compiles); returns the
    module's path."""
    from torch.utils import cpp_extension as ce

    ext = EXTENSIONS[name]
    obj_dir = os.path.join(REPO_DIR, "build", "jit", name)
    os.makedirs(obj_dir, exist_ok=True)
    so = module_path(name)
    with open(os.path.join(obj_dir, ".lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        digest = source_digest(name)
        torch_inc = [f"-I{p}" for p in ce.include_paths("cuda")] + [f"-I{sysconfig.get_paths()['include']}"]
        torch_def = ["-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DHIPBLAS_V2",
                     "-D__HIP_NO_HALF_OPERATORS__=1", "-D__HIP_NO_HALF_CONVERSIONS__=1",
                     "-DTORCH_API_INCLUDE_EXTENSION_H", f"-DTORCH_EXTENSION_NAME={name}"]
        jobs: List[List[str]] = []
        objs: List[str] = []
        for f in ext["kernels"] + ext["bindings"]:
            o = os.path.join(obj_dir, os.path.basename(f) + ".o")
            cmd = [_hipcc(), "-c", os.path.join(ext["dir"], f), "-o", o] + HIP_FLAGS
            if f in ext["bindings"]:
                cmd += torch_inc + torch_def
            jobs.append(cmd)
            objs.append(o)

        def run(cmd):
            r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
            if r.returncode != 0:
                raise RuntimeError(f"hipcc failed: {' '.join(cmd)}\n{r.stdout}")
            if verbose and r.stdout.strip():
                print(r.stdout, file=sys.stderr)

        with ThreadPoolExecutor(max_workers=min(len(jobs), 8)) as pool:
            list(pool.map(run, jobs))
        lib_dirs = ce.library_paths("cuda")
        link = ([os.environ.get("CXX", "g++"), "-shared"] + objs + [f"-L{d}" for d in lib_dirs] +
                ["-lc10", "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lamdhip64", "-lc10_hip", "-ltorch_hip",
                 "-o", so + ".tmp"])
        run(link)
        os.replace(so + ".tmp", so)
        with open(so + ".digest", "w") as f:
            f.write(digest + "\n")
    return so


def load(name: str):
    """Import extension ``name``, compiling it first when it is missing or
    older than its sources."""
    if not is_current(name):
        print(f"[kllms_amd] compiling {name} for gfx950 ...", file=sys.stderr, flush=True)
        build(name)
    import torch  # noqa: F401  (the module links against libtorch)

    spec = importlib.util.spec_from_file_location(f"kllms_amd.{name}", module_path(name))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    sys.modules[f"kllms_amd.{name}"] = mod
    return mod
