"""Builds libmor_hip.so (hipcc, gfx950) and libmor_torch.so (g++) in-tree.

Each HIP source file is compiled to an object of its own, in parallel, and the objects are linked into one shared
library.  Objects and libraries are keyed by a hash of the text of their sources and headers (file times do not
survive a copy of the tree): the library reports the hash through mor_version(), ensure_built() rebuilds whatever
does not match, and mor_amd._cabi refuses to load a library built from other sources, so tests, the smoke check and
the benchmark never run a library that lags behind the sources.
"""
import glob
import hashlib
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_HERE, "csrc")
_ROOT = os.path.dirname(_HERE)
SOURCES = [os.path.join(_CSRC, n) for n in ("mor_kernels.hip", "mor_wgblock.hip", "mor_subblock.hip", "mor_scaling.hip", "mor_wire.hip", "mor_batch.hip", "mor_dual.hip", "mor_morwire.hip", "mor_mfma_check.hip")]
SOURCES = [s for s in SOURCES if os.path.exists(s)]
HEADERS = [os.path.join(_CSRC, n) for n in ("mor_device.h", "mor_common.h", "mor_quant.h", "mor_wgblock.h", "mor_wirefmt.h", "mor_host.h")] + [os.path.join(_ROOT, "include", "mor_hip.h")]
VERSION_SRC = os.path.join(_CSRC, "mor_version.cpp")
OUT = os.path.join(_HERE, "lib", "libmor_hip.so")
HASH_FILE = os.path.join(_HERE, "lib", "libmor_hip.srchash")           # the source hash libmor_hip.so was built from
TORCH_HASH_FILE = os.path.join(_HERE, "lib", "libmor_torch.srchash")
OBJ_DIR = os.path.join(_HERE, "lib", "obj")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # keep packed fp32 instructions out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is harmless
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError(f"{cmd[0]} failed:\n{out}")
    if verbose and out:
        print(out, flush=True)


def _digest(paths, extra=""):
    h = hashlib.sha256(extra.encode())
    for p in sorted(paths):
        h.update(os.path.basename(p).encode())
        with open(p, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:12]


def source_hash():
    """Hash of everything libmor_hip.so is built from (sources, headers, compiler flags)."""
    return _digest(SOURCES + HEADERS + [VERSION_SRC], " ".join(HIPCC_FLAGS))


def _read(path):
    try:
        with open(path) as f:
            return f.read().strip()
    except OSError:
        return ""


def _obj_of(src):
    return os.path.join(OBJ_DIR, f"{os.path.basename(src)}.{_digest([src] + HEADERS, ' '.join(HIPCC_FLAGS))}.o")


def build_hip(verbose=False, force=True):
    """Compiles the HIP sources (all of them when `force`, else those whose text or headers changed) and links."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    todo = [s for s in SOURCES if force or not os.path.exists(_obj_of(s))]
    with ThreadPoolExecutor(max_workers=max(1, min(len(todo), os.cpu_count() or 1, 8))) as pool:
        list(pool.map(lambda s: _run([hipcc] + HIPCC_FLAGS + ["-c", s, "-o", _obj_of(s)], verbose), todo))
    objs = [_obj_of(s) for s in SOURCES]
    for old in glob.glob(os.path.join(OBJ_DIR, "*.o")):
        if old not in objs:
            os.remove(old)
    sh = source_hash()
    vobj = os.path.join(OBJ_DIR, "mor_version.o")
    _run([os.environ.get("CXX", "g++"), "-O2", "-fPIC", "-fvisibility=hidden", f'-DMOR_SRC_HASH="{sh}"', "-c", VERSION_SRC, "-o", vobj], verbose)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT] + objs + [vobj], verbose)
    with open(HASH_FILE, "w") as f:
        f.write(sh + "\n")
    return OUT


TORCH_BINDING_SRC = os.path.join(_HERE, "csrc", "torch_binding.cpp")
TORCH_BINDING_OUT = os.path.join(_HERE, "lib", "libmor_torch.so")


def build_torch_binding(verbose=False):
    """The C++ operator registrations (no kernels): plain g++ against torch's headers and libmor_hip.so."""
    import torch
    from torch.utils import cpp_extension as ce
    tlib = ce.library_paths()[0]
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    cmd += [f"-I{p}" for p in ce.include_paths()] + ["-I/opt/rocm/include", TORCH_BINDING_SRC, "-o", TORCH_BINDING_OUT,
            f"-L{tlib}", "-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip",
            f"-L{os.path.dirname(OUT)}", "-lmor_hip", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}"]
    _run(cmd, verbose)
    with open(TORCH_HASH_FILE, "w") as f:
        f.write(_torch_hash() + "\n")
    return TORCH_BINDING_OUT


def _torch_hash():
    return _digest([TORCH_BINDING_SRC, HEADERS[-1]])


def ensure_built(verbose=False):
    """Brings both libraries up to date with the text of their sources (used by the tests, the smoke check and the
    benchmark; build() always rebuilds everything)."""
    if not os.path.exists(OUT) or _read(HASH_FILE) != source_hash():
        build_hip(verbose, force=False)
    if not os.path.exists(TORCH_BINDING_OUT) or _read(TORCH_HASH_FILE) != _torch_hash():
        build_torch_binding(verbose)


if __name__ == "__main__":
    print(build_hip(verbose=True))
    print(build_torch_binding(verbose=True))
