"""Build recipe of libtorchgt_hip.so: plain hipcc, gfx950 only, in-tree output.

``python -m torchgt_amd.build`` (or ``__graft_entry__.build()``) compiles every
``csrc/*.hip`` to an object file and links ``torchgt_amd/libtorchgt_hip.so``.
hipcc cross-compiles without a GPU.
"""
import os
import subprocess
import sys
import time
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libtorchgt_hip.so")
EXT_SRC = os.path.join(CSRC, "torch_binding.cpp")
EXT_PATH = os.path.join(HERE, "_torchgt_ext.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed-fp32 instructions are switched off on purpose: the compiler otherwise
# forms v_pk_*_f32 from scalar float code
FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


# sources compiled as several translation units (-D<macro>=k, k < parts), in parallel: their
# kernels take minutes to compile in one piece
SPLIT = {"sparse_attn.hip": ("TGT_SPARSE_PART", 4), "dense_attn.hip": ("TGT_DENSE_PART", 2)}


def _jobs():
    jobs = []
    for src in sources():
        if src in SPLIT:
            macro, parts = SPLIT[src]
            jobs += [(src, f"{src[:-4]}_p{k}.o", [f"-D{macro}={k}"]) for k in range(parts)]
        else:
            jobs.append((src, src[:-4] + ".o", []))
    return jobs


def _compile(job):
    src, obj_name, extra = job
    obj = os.path.join(OBJ_DIR, obj_name)
    cmd = [HIPCC] + FLAGS + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
    t0 = time.time()
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src + (" " + " ".join(extra) if extra else ""), obj, r.returncode, r.stdout + r.stderr, time.time() - t0


def build(verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = sorted(_jobs(), key=lambda j: j[0] not in SPLIT)      # the long ones first
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        results = list(ex.map(_compile, jobs))
    objs = []
    for src, obj, rc, log, dt in results:
        noise = "unknown target feature"   # harmless host-pass note about -packed-fp32-ops
        shown = "\n".join(l for l in log.splitlines() if noise not in l and "-packed-fp32-ops" not in l)
        if verbose:
            print(f"[torchgt_amd.build] {src}: {dt:.1f}s rc={rc}")
            if shown.strip():
                print(shown)
        if rc != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{log}")
        objs.append(obj)
    tmp = LIB_PATH + ".tmp"
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", tmp] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[torchgt_amd.build] linked {LIB_PATH}")
    build_extension(verbose)
    return LIB_PATH


def build_extension(verbose=True):
    """The PyTorch-ROCm extension: host code only (g++), torch's headers, linked against libtorchgt_hip.so
    next to it (rpath $ORIGIN) and torch's libraries."""
    import torch
    from torch.utils import cpp_extension
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    cmd += [f"-I{p}" for p in cpp_extension.include_paths()] + ["-I/opt/rocm/include", EXT_SRC, "-o", EXT_PATH + ".tmp",
            f"-L{tlib}", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip", f"-L{HERE}", "-ltorchgt_hip",
            "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}"]
    t0 = time.time()
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the torch extension failed:\n" + r.stdout + r.stderr)
    os.replace(EXT_PATH + ".tmp", EXT_PATH)
    if verbose:
        print(f"[torchgt_amd.build] torch_binding.cpp: {time.time() - t0:.1f}s -> {EXT_PATH}")
    return EXT_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
