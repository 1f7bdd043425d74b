"""Builds the native pieces in-tree (no JIT, no caches outside the repository):

  lib/mtrt_kernels.hsaco        gfx950 code object with every cluster kernel
  lib/mtrt_test_fixtures.hsaco  the two launch-ABI test kernels, as a separate module
  lib/libmtrt_hip.so            C ABI (launch layer + cluster layer) with the kernel
                                module embedded as read-only data
  lib/mtrt_standalone_selftest  host program in the style of EmitC-generated C++ that calls the
                                `namespace mtrt` flavour of the launch layer (run by the tests)

hipcc cross-compiles for gfx950 without a GPU present.  Run as
`python tensorrt-incubator_amd/build.py` or through `__graft_entry__.build()`.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

# Packed-FP32 instructions are switched off for all device code: the compiler is
# not to form v_pk_{add,mul,fma}_f32 from scalar float code.
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
# Quantize / reduce clusters must round like the host program: no FMA contraction.
EXACT_FLAGS = ["-ffp-contract=off"]


def _run(cmd):
    print("+ " + " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if out.strip():
        print(out, flush=True)
    if res.returncode != 0:
        raise RuntimeError("command failed (%d): %s" % (res.returncode, " ".join(cmd)))


def hipcc():
    exe = shutil.which("hipcc") or os.path.join(ROCM, "bin", "hipcc")
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build_kernels():
    os.makedirs(LIB, exist_ok=True)
    kdir = os.path.join(CSRC, "kernels")
    _run([hipcc(), "--genco"] + DEVICE_FLAGS + EXACT_FLAGS +
         [os.path.join(kdir, "builtin_module.hip"), "-o", os.path.join(LIB, "mtrt_kernels.hsaco")])
    _run([hipcc(), "--genco"] + DEVICE_FLAGS +
         [os.path.join(kdir, "fixtures.hip"), "-o", os.path.join(LIB, "mtrt_test_fixtures.hsaco")])


def build_runtime():
    rdir = os.path.join(CSRC, "runtime")
    srcs = sorted(os.path.join(rdir, f) for f in os.listdir(rdir) if f.endswith(".cpp"))
    hsaco = os.path.join(LIB, "mtrt_kernels.hsaco")
    # Host files that own device-side objects (a device array whose address the host looks up) are
    # compiled by hipcc as ordinary HIP translation units and linked in as objects.
    for f in sorted(os.listdir(rdir)):
        if f.endswith(".hip"):
            obj = os.path.join(LIB, f[:-4] + ".o")
            _run([hipcc(), "-c", "-fPIC", "-fvisibility=hidden"] + DEVICE_FLAGS + EXACT_FLAGS +
                 ["-I" + os.path.join(ROOT, "include"), os.path.join(rdir, f), "-o", obj])
            srcs.append(obj)
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall", "-Wextra",
          "-D__HIP_PLATFORM_AMD__", '-DMTRT_HSACO_PATH="%s"' % hsaco,
          "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROCM, "include")] + srcs +
         ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(ROCM, "lib"),
          "-o", os.path.join(LIB, "libmtrt_hip.so")])


def build_selftest():
    src = os.path.join(CSRC, "selftest", "standalone_selftest.cpp")
    # include/standalone holds the reference's header NAMES (MTRTRuntimeCuda.h ...), as generated code includes them
    _run(["g++", "-O1", "-std=c++17", "-Wall", "-Wextra", "-I" + os.path.join(ROOT, "include", "standalone"), src,
          "-L" + LIB, "-lmtrt_hip", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + os.path.join(ROCM, "lib"),
          "-o", os.path.join(LIB, "mtrt_standalone_selftest")])


def build_oracle():
    """The CPU oracle is test infrastructure; building it here keeps one build entry point."""
    _run(["make", "-C", os.path.join(ROOT, "oracle")])


def build_all():
    build_kernels()
    build_runtime()
    build_selftest()
    build_oracle()


if __name__ == "__main__":
    build_all()
    print("built:", ", ".join(sorted(os.listdir(LIB))))
    sys.exit(0)
