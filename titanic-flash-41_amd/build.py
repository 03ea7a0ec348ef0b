"""Builds the package's native code in-tree with hipcc for gfx950.

  libtitanic_moe_hip.so      kernels + the C ABI of include/titanic_moe.h
  titanic_moe_gfx950.hsaco   the same kernels as a code object for hosts that load modules by name
  libtitanic_ffn_host.so     the C++ host mirror of the reference's Rust FFN operators (needs only the HIP runtime)
  tf_layer_probe             stand-alone driver of the layer for profilers (no Python in the process)
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
KERNEL_LIB = os.path.join(HERE, "libtitanic_moe_hip.so")
CODE_OBJECT = os.path.join(HERE, "titanic_moe_gfx950.hsaco")
HOST_LIB = os.path.join(HERE, "libtitanic_ffn_host.so")
PROBE = os.path.join(HERE, "tf_layer_probe")

# -ffp-contract=off: bit-exact steps are written as explicit fma / mul / add.  Packed FP32 instructions stay off.
DEVICE_FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
                "-packed-fp32-ops", "-Wno-unused-command-line-argument"]


def _run(cmd):
    result = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = ("packed-fp32-ops", "1 warning generated", "^~", "is not a recognized feature")
    lines = [l for l in result.stdout.splitlines() if l.strip() and not any(n in l for n in noise)]
    if result.returncode != 0:
        raise RuntimeError("build failed: %s\n%s" % (" ".join(cmd), "\n".join(lines)))
    return lines


def build_kernels():
    src = os.path.join(CSRC, "abi.hip")
    _run(["hipcc", *DEVICE_FLAGS, "-fPIC", "-shared", src, "-o", KERNEL_LIB])
    _run(["hipcc", *DEVICE_FLAGS, "--genco", src, "-o", CODE_OBJECT])
    return KERNEL_LIB


def build_host():
    sources = sorted(os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".cpp")) if os.path.isdir(HOST) else []
    if not sources:
        return None
    _run(["hipcc", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(ROOT, "include"), *sources,
          "-o", HOST_LIB, "-ldl"])
    return HOST_LIB


def build_probe():
    src = os.path.join(HOST, "probe", "layer_probe.hip")
    _run(["hipcc", *DEVICE_FLAGS, src, "-o", PROBE, "-L", HERE, "-ltitanic_ffn_host", "-Wl,-rpath,$ORIGIN"])
    return PROBE


def build():
    return build_kernels(), build_host(), build_probe()


if __name__ == "__main__":
    print(build())
