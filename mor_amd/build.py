"""Builds libmor_hip.so in-tree with hipcc for gfx950."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = [os.path.join(_HERE, "csrc", "mor_kernels.hip"), os.path.join(_HERE, "csrc", "mor_wire.hip")]
OUT = os.path.join(_HERE, "lib", "libmor_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    # keep packed fp32 instructions out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build_hip(verbose=False):
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", OUT] + SOURCES
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is harmless
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{out}")
    if verbose and out:
        print(out, flush=True)
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
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"g++ failed:\n{res.stdout}")
    return TORCH_BINDING_OUT


def ensure_built(verbose=False):
    """Builds what is missing (used by the tests, the smoke check and the benchmark; build() always rebuilds)."""
    if not os.path.exists(OUT):
        build_hip(verbose)
    if not os.path.exists(TORCH_BINDING_OUT):
        build_torch_binding(verbose)


if __name__ == "__main__":
    print(build_hip(verbose=True))
    print(build_torch_binding(verbose=True))
