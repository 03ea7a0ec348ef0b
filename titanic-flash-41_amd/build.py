"""Builds the package's native code in-tree with hipcc for gfx950.

  libtitanic_moe_hip.so      kernels + the C ABI of include/titanic_moe.h
  titanic_moe_gfx950.hsaco   the same kernels as a code object for hosts that load modules by name
  libtitanic_ffn_host.so     the C++ host mirror of the reference's Rust FFN operators (needs only the HIP runtime)
  tf_layer_probe             stand-alone driver of the layer for profilers (no Python in the process)
  manifest.json              SHA-256 of the libraries just built; the host mirror refuses a kernel library that differs from it
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
KERNEL_LIB = os.path.join(HERE, "libtitanic_moe_hip.so")
CODE_OBJECT = os.path.join(HERE, "titanic_moe_gfx950.hsaco")
REFERENCE_LAYER_OBJECT = os.path.join(HERE, "titanic_moe_gfx950_reference_layer.hsaco")
HOST_LIB = os.path.join(HERE, "libtitanic_ffn_host.so")
PROBE = os.path.join(HERE, "tf_layer_probe")
MANIFEST = os.path.join(HERE, "manifest.json")

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
    # the kernels the reference launches by name with fixed argument lists, for its own layer's dimensions
    _run(["hipcc", *DEVICE_FLAGS, "--genco", os.path.join(CSRC, "reference_layer.hip"), "-o", REFERENCE_LAYER_OBJECT])
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


def write_manifest():
    """manifest.json beside the libraries: what the host mirror pins the kernel library with (the reference pins every native
    artifact by SHA-256 in its manifests and refuses another: src/ffn.rs:70-74, src/primitives.rs:75-79)."""
    import hashlib
    import json

    def digest(path):
        return hashlib.sha256(open(path, "rb").read()).hexdigest() if os.path.exists(path) else None
    manifest = {"schema": 1, "architecture": "gfx950", "abi": 1, "library": os.path.basename(KERNEL_LIB), "library_sha256": digest(KERNEL_LIB),
                "code_object": os.path.basename(CODE_OBJECT), "code_object_sha256": digest(CODE_OBJECT),
                "reference_layer_object": os.path.basename(REFERENCE_LAYER_OBJECT), "reference_layer_object_sha256": digest(REFERENCE_LAYER_OBJECT),
                "host_library": os.path.basename(HOST_LIB), "host_library_sha256": digest(HOST_LIB)}
    with open(MANIFEST, "w") as f:
        json.dump(manifest, f, indent=1)
        f.write("\n")
    return MANIFEST


def write_pinned_contracts():
    """The operator contracts with the hash of the library just built (contracts/pinned/, beside the committed ones, whose
    hash fields are null because no library is committed)."""
    import importlib
    contracts = importlib.import_module("titanic-flash-41_amd.contracts")
    contracts.main(os.path.join(HERE, "contracts", "pinned"), KERNEL_LIB)


def build():
    built = build_kernels(), build_host(), build_probe()
    write_manifest()
    write_pinned_contracts()
    return built


if __name__ == "__main__":
    print(build())
